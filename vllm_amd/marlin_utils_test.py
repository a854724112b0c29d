"""Synthetic Marlin-layout layers for tests and benchmarks, produced on the device.

Same names and return lists as the reference's test helpers `marlin_quantize` / `awq_marlin_quantize`
(vllm/model_executor/layers/quantization/utils/marlin_utils_test.py:96-161) and `quantize_weights`
(quant_utils.py:376-468), but nothing leaves the GPU: the round-to-nearest quantizer runs as torch ops in the
weight's own dtype, the integers are packed into the GPTQ / AWQ checkpoint layouts and go through the library's
repack kernels, scales and zero points through the load-time conversions of `marlin_utils`.  A layer of
4096 x 28672 takes milliseconds instead of the minutes a host quantizer needs.

`rule` selects the scale rule: "reference" is the reference helper's (symmetric: max(|max / qmax|, |min / qmin|);
asymmetric: (max - min).clamp(1e-5) / qmax, zp = round(|min / s|)); "absmax" is absmax / 7 for symmetric 4-bit types
and (max - min) / 15 clamped to >= 1e-5 with zp = round(-min / s) for asymmetric ones, the rules the benchmark
configurations are stated with.
"""
import torch

from . import _custom_ops as ops
from .marlin_utils import marlin_permute_scales, marlin_zero_points
from .quant_utils import awq_pack, gptq_pack
from .scalar_type import ScalarType


def quantize_weights(w: torch.Tensor, quant_type: ScalarType, group_size: int | None, zero_points: bool = False,
                     rule: str = "reference"):
    """w [K, N] (fp16 / bf16, any device) -> (w_ref [K, N], stored integers int32 [K, N], scales [G, N],
    zero points int32 [G, N] or None).  All arithmetic in w's dtype, as the reference helper does."""
    assert w.is_floating_point() and w.dim() == 2 and quant_type.is_integer()
    size_k, size_n = w.shape
    gs = size_k if group_size in (-1, None) else group_size
    assert size_k % gs == 0
    wg = w.reshape(size_k // gs, gs, size_n)
    hi = wg.amax(dim=1, keepdim=True)
    lo = wg.amin(dim=1, keepdim=True)
    qmax, qmin = quant_type.max(), quant_type.min()
    zp = None
    if zero_points:
        assert not quant_type.is_signed() and not quant_type.has_bias()
        if rule == "reference":
            s = (hi - lo).clamp(min=1e-5) / qmax
            zp = torch.round(torch.abs(lo / s)).clamp(qmin, qmax).int()
        else:
            s = ((hi - lo) / qmax).clamp(min=1e-5)
            zp = torch.clamp(torch.round(-lo / s), qmin, qmax).int()
        q = torch.clamp(torch.round(wg / s).int() + zp, qmin, qmax)
        w_ref = (q - zp).to(w.dtype) * s
    else:
        if rule == "reference":
            s = torch.maximum(torch.abs(hi / qmax), torch.abs(lo / qmin))
        else:
            s = (wg.abs().amax(dim=1, keepdim=True) / qmax).clamp(min=1e-5)
        q = torch.clamp(torch.round(wg / s).int(), qmin, qmax)
        w_ref = q.to(w.dtype) * s
    if quant_type.has_bias():
        q = q + quant_type.bias
    groups = size_k // gs
    return (w_ref.reshape(size_k, size_n), q.reshape(size_k, size_n).int(), s.reshape(groups, size_n).contiguous(),
            None if zp is None else zp.reshape(groups, size_n).contiguous())


def marlin_quantize(w: torch.Tensor, quant_type: ScalarType, group_size: int, act_order: bool,
                    test_perm: torch.Tensor | None = None, rule: str = "reference"):
    """Returns [w_ref, marlin_q_w, marlin_s, g_idx, sort_indices, rand_perm].  With act_order the rows of w_ref are in
    arrival order (row i of the activations meets w_ref[i]), g_idx is sorted and sort_indices is the column gather
    for the activations, exactly what `gptq_marlin_gemm` takes."""
    size_k, size_n = w.shape
    bits = quant_type.size_bits
    gs = size_k if group_size == -1 else group_size
    w_ref, q, s, _ = quantize_weights(w, quant_type, gs, rule=rule)
    dev = w.device
    g_idx = torch.empty(0, dtype=torch.int32, device=dev)
    sort_indices = torch.empty(0, dtype=torch.int32, device=dev)
    rand_perm = torch.empty(0, dtype=torch.int64, device=dev)
    if act_order:
        assert gs < size_k, "act-order needs more than one group"
        rand_perm = (torch.randperm(size_k) if test_perm is None else test_perm).to(dev).long()
        w_ref = w_ref[rand_perm].contiguous()
        q = q[rand_perm].contiguous()
        g_arrival = (rand_perm // gs).to(torch.int32)
        sort_indices = torch.argsort(g_arrival, stable=True).to(torch.int32)
        g_idx = g_arrival[sort_indices.long()].contiguous()
    marlin_q_w = ops.gptq_marlin_repack(gptq_pack(q, bits, size_k, size_n), sort_indices, size_k, size_n, bits)
    marlin_s = marlin_permute_scales(s, size_k, size_n, gs)
    return [w_ref, marlin_q_w, marlin_s, g_idx, sort_indices, rand_perm]


def awq_marlin_quantize(w: torch.Tensor, quant_type: ScalarType, group_size: int, rule: str = "reference"):
    """Returns [w_ref, marlin_q_w, marlin_s, marlin_zp]."""
    size_k, size_n = w.shape
    bits = quant_type.size_bits
    gs = size_k if group_size == -1 else group_size
    w_ref, q, s, zp = quantize_weights(w, quant_type, gs, zero_points=True, rule=rule)
    marlin_q_w = ops.awq_marlin_repack(awq_pack(q, bits, size_k, size_n), size_k, size_n, bits)
    marlin_s = marlin_permute_scales(s, size_k, size_n, gs)
    marlin_zp = marlin_zero_points(zp, size_k // gs, size_n, bits)
    return [w_ref, marlin_q_w, marlin_s, marlin_zp]
