"""Shared builders for the parity tests: seeded synthetic layers quantized with the CPU oracle."""
from dataclasses import dataclass

import torch

from oracle import gemm_ref as gr
from oracle import marlin_layout as ml
from oracle import quant_utils as qu
from oracle import scalar_types as st


@dataclass
class Layer:
    size_k: int
    size_n: int
    group_size: int
    dtype: torch.dtype
    has_zp: bool
    act_order: bool
    w_ref: torch.Tensor          # [K, N] dequantised, rows in the order activations arrive
    q: torch.Tensor              # [K, N] stored nibbles, checkpoint row order
    scales: torch.Tensor         # [G, N] unpermuted
    zp: torch.Tensor | None      # [G, N] unpacked
    g_idx: torch.Tensor          # checkpoint g_idx (act-order) or empty
    marlin_q: torch.Tensor       # int32 [K/16, 2N]
    marlin_s: torch.Tensor       # [G, N] permuted
    marlin_zp: torch.Tensor      # int32 [G, N/8] or empty
    g_idx_sorted: torch.Tensor   # int32 [K] or empty
    sort_indices: torch.Tensor   # int32 [K] or empty
    bits: int = 4

    @property
    def type_id(self):
        return (st.uint4 if self.has_zp else st.uint4b8 if self.bits == 4 else st.uint8b128).id


def make_layer(size_k, size_n, group_size, dtype=torch.float16, has_zp=False, act_order=False, seed=0,
               w_std=1.0, rule="reference", bits=4) -> Layer:
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(size_k, size_n, generator=g) * w_std).to(dtype)
    empty_i = torch.empty(0, dtype=torch.int32)
    gs = size_k if group_size == -1 else group_size
    if has_zp:
        assert not act_order
        if rule == "reference":
            w_ref, q, s, zp = qu.quantize_weights(w, st.uint4, group_size, zero_points=True)
        else:
            w_ref, q, s, zp = qu.quantize_minmax_zp(w, group_size)
        marlin_q = ml.marlin_weights_closed_form(q)
        marlin_zp = ml.marlin_zero_points(zp, zp.shape[0], size_n)
        return Layer(size_k, size_n, group_size, dtype, True, False, w_ref, q, s, zp, empty_i, marlin_q,
                     ml.marlin_permute_scales(s, size_k, size_n, gs), marlin_zp, empty_i, empty_i)
    if rule == "reference":
        perm = torch.randperm(size_k, generator=g) if act_order else None
        w_ref, q, s, g_idx, _ = qu.gptq_quantize_weights(w, st.uint4b8 if bits == 4 else st.uint8b128, group_size,
                                                         act_order, perm)
    else:
        assert not act_order
        w_ref, q, s = qu.quantize_absmax7(w, group_size)
        g_idx = empty_i
    sort_indices, g_idx_sorted, q_sorted = empty_i, empty_i, q
    if act_order:
        q_sorted, g_idx_sorted, sort_indices = qu.sort_weights(q, g_idx)
    marlin_q = ml.marlin_weights_closed_form(q_sorted) if bits == 4 else ml.marlin_weights_closed_form8(q_sorted)
    return Layer(size_k, size_n, group_size, dtype, False, act_order, w_ref, q, s, None, g_idx, marlin_q,
                 ml.marlin_permute_scales(s, size_k, size_n, gs), empty_i, g_idx_sorted, sort_indices, bits)


def run_gemm(ops, layer: Layer, a, dev, workspace, is_k_full=True, bias=None, use_atomic_add=False, c=None):
    """Call the op the way the reference's kernel test does (test_marlin_gemm.py:330-349)."""
    import vllm_amd.scalar_type as vst
    wtype = (vst.scalar_types.uint4 if layer.has_zp else
             vst.scalar_types.uint4b8 if layer.bits == 4 else vst.scalar_types.uint8b128)
    return ops.gptq_marlin_gemm(
        a, c, layer.marlin_q.to(dev), None if bias is None else bias, layer.marlin_s.to(dev), None,
        layer.marlin_zp.to(dev), layer.g_idx_sorted.to(dev), layer.sort_indices.to(dev), workspace, wtype,
        a.shape[0], layer.size_n, layer.size_k, is_k_full=is_k_full, use_atomic_add=use_atomic_add,
        use_fp32_reduce=True, is_zp_float=False)


def tol_for(dtype):
    """Stated gate: max|out-ref|/max|ref| <= 2e-2 (fp16) / 4e-2 (bf16)."""
    return 2e-2 if dtype == torch.float16 else 4e-2


def check_close(out, a, layer: Layer, bias=None):
    ref = gr.gemm_ref(a.cpu(), layer.w_ref, None if bias is None else bias.cpu())
    m = gr.error_metrics(out, ref)
    assert m["max_rel"] <= tol_for(layer.dtype), m
    assert m["mean_rel"] < 0.04, m   # the reference test's own gate (test_marlin_gemm.py:359-361)
    return m
