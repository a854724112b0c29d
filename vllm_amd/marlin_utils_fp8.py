"""FP8 (float8_e4m3fn) weight-only path on the Marlin operator surface; host mirror of the reference's
vllm/model_executor/layers/quantization/utils/marlin_utils_fp8.py (same names, arguments and tensor contracts).

The weights travel as fp8 bytes in the 8-bit Marlin layout (`gptq_marlin_repack(num_bits=8)`), the scales are
permuted like every other Marlin scale tensor and multiplied by the exponent offset between fp8 and the
activation type (2^8 for fp16, 2^120 for bf16), because the reference's kernel re-uses the fp8 bits without
re-biasing the exponent; the gfx950 kernel takes that factor out again, so tensors prepared by either side work."""
import torch

from . import _custom_ops as ops
from .marlin_utils import (USE_FP32_REDUCE_DEFAULT, marlin_make_workspace_new, marlin_permute_bias,
                           marlin_permute_scales, should_use_atomic_add_reduce)
from .scalar_type import scalar_types


def is_fp8_marlin_supported() -> bool:
    return torch.cuda.is_available()


def fp8_fused_exponent_bias_into_scales(scales: torch.Tensor) -> torch.Tensor:
    """scales * 2^(bias(dtype) - bias(e4m3)): 2^(15-7) for fp16, 2^(127-7) for bf16 (marlin_utils_fp8.py:25-37)."""
    if scales.dtype == torch.half:
        shift = 15 - 7
    elif scales.dtype == torch.bfloat16:
        shift = 127 - 7
    else:
        raise ValueError(f"unsupported scale dtype {scales.dtype}")
    return scales * torch.full_like(scales, 2.0) ** shift


def pack_fp8_to_int32(fp8_tensor: torch.Tensor, size_k_first: bool = True) -> torch.Tensor:
    """fp8 [K, N] (size_k_first) or [N, K] -> int32 with four consecutive K bytes per word:
    [K/4, N] when size_k_first else [N, K/4] (marlin_utils_fp8.py:296-310)."""
    assert fp8_tensor.dtype == torch.float8_e4m3fn and fp8_tensor.ndim == 2
    nk = (fp8_tensor.T if size_k_first else fp8_tensor).contiguous()
    words = nk.view(torch.int32)
    return words.T.contiguous() if size_k_first else words


def apply_fp8_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                            workspace: torch.Tensor, size_n: int, size_k: int, bias: torch.Tensor | None,
                            use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    x = input.reshape(-1, input.shape[-1])
    use_atomic_add = should_use_atomic_add_reduce(m=x.size(0), n=size_n, k=size_k, device=input.device,
                                                  dtype=input.dtype)
    out = ops.gptq_marlin_gemm(a=x, c=None, b_q_weight=weight, b_bias=bias, b_scales=weight_scale, global_scale=None,
                               b_zeros=None, g_idx=None, perm=None, workspace=workspace,
                               b_q_type=scalar_types.float8_e4m3fn, size_m=x.size(0), size_n=size_n, size_k=size_k,
                               use_atomic_add=use_atomic_add, use_fp32_reduce=use_fp32_reduce)
    return out.reshape(input.shape[:-1] + (size_n,))


def _channel_or_group_scales(scales: torch.Tensor, size_n: int, weight_block_size, size_k_first: bool) -> torch.Tensor:
    """Per-tensor / per-shard / per-channel / block-wise checkpoint scales -> [1, N] or [K/block_k, N]."""
    if weight_block_size is None:
        count = scales.nelement()
        if count == 1:
            return scales.view(1, 1).repeat_interleave(size_n, 1)
        if count != size_n:                        # one scale per fused shard (e.g. gate | up)
            assert size_n % count == 0
            return scales.view(1, count).repeat_interleave(size_n // count, 1)
        return scales.view(1, size_n)
    if not size_k_first:
        scales = scales.T.contiguous()
    return scales.repeat_interleave(weight_block_size[0], 1)[:, :size_n]


def prepare_fp8_layer_for_marlin(layer: torch.nn.Module, size_k_first: bool = True) -> None:
    """layer.weight fp8 [K, N] (or [N, K]) + weight_scale / weight_scale_inv -> Marlin-layout weight, permuted and
    offset scales, workspace, permuted bias (marlin_utils_fp8.py:84-171)."""
    size_n, size_k = layer.output_size_per_partition, layer.input_size_per_partition
    block = getattr(layer, "weight_block_size", None)
    assert layer.weight.shape == ((size_k, size_n) if size_k_first else (size_n, size_k))
    device = layer.weight.device
    layer.workspace = marlin_make_workspace_new(device)
    packed = pack_fp8_to_int32(layer.weight, size_k_first)
    if not size_k_first:
        packed = packed.T.contiguous()
    layer.weight = torch.nn.Parameter(
        ops.gptq_marlin_repack(b_q_weight=packed, perm=torch.empty(0, dtype=torch.int, device=device), size_k=size_k,
                               size_n=size_n, num_bits=8), requires_grad=False)
    if hasattr(layer, "weight_scale_inv") and not hasattr(layer, "weight_scale"):
        scales = layer.weight_scale_inv.to(layer.orig_dtype)
        del layer.weight_scale_inv
    else:
        scales = layer.weight_scale.to(layer.orig_dtype)
    scales = _channel_or_group_scales(scales, size_n, block, size_k_first)
    marlin_scales = marlin_permute_scales(s=scales, size_k=size_k, size_n=size_n,
                                          group_size=-1 if block is None else block[1])
    layer.weight_scale = torch.nn.Parameter(fp8_fused_exponent_bias_into_scales(marlin_scales), requires_grad=False)
    if getattr(layer, "bias", None) is not None:
        assert layer.bias.shape == (size_n,)
        layer.bias = torch.nn.Parameter(marlin_permute_bias(layer.bias), requires_grad=False)


def marlin_quant_fp8_torch(weight: torch.Tensor, group_size: int):
    """Test helper with the reference's contract (marlin_utils_fp8.py:313-351): weight [N, K] ->
    (w_ref [K, N], Marlin weight, Marlin scales with the exponent offset folded in); scale = absmax / 448."""
    size_n, size_k = weight.shape
    gs = size_k if group_size == -1 else group_size
    scales = weight.view(size_n, -1, gs).abs().amax(-1) / 448
    rep = scales.repeat_interleave(gs, 1)
    fp8_weight = (weight / rep).to(torch.float8_e4m3fn)
    w_ref = fp8_weight.to(weight.dtype) * rep
    packed = pack_fp8_to_int32(fp8_weight, False).T.contiguous()
    marlin_q = ops.gptq_marlin_repack(b_q_weight=packed, perm=torch.empty(0, dtype=torch.int, device=weight.device),
                                      size_k=size_k, size_n=size_n, num_bits=8)
    marlin_s = marlin_permute_scales(s=scales.T, size_k=size_k, size_n=size_n, group_size=group_size)
    return w_ref.T, marlin_q, fp8_fused_exponent_bias_into_scales(marlin_s)
