"""FP4 (float4_e2m1f) weight-only path on the Marlin operator surface: NVFP4 (group 16, float8_e4m3fn scales and a
global scale) and MXFP4 (group 32, E8M0 scales, bf16).  Host mirror of the reference's
vllm/model_executor/layers/quantization/utils/marlin_utils_fp4.py: same names, arguments and tensor contracts, so
tensors prepared by either side feed either GEMM.

Scale bytes: the Marlin-permuted [G, N] scale matrix is regrouped so that a lane's 8 scales of two consecutive groups
(the two k-tiles of a k-step for NVFP4, two k-steps for MXFP4) are adjacent, each 4 swapped to (0, 2, 1, 3), and
stored one byte per scale: NVFP4 as the high byte of half(s * 2^7) << 1 (unsigned E5M3 — scales are taken to be
non-negative), MXFP4 as E8M0."""
import torch

from . import _custom_ops as ops
from .marlin_utils import (USE_FP32_REDUCE_DEFAULT, marlin_make_workspace_new, marlin_permute_bias,
                           marlin_permute_scales, should_use_atomic_add_reduce)
from .scalar_type import scalar_types

FP4_MARLIN_SUPPORTED_GROUP_SIZES = [16]


def is_fp4_marlin_supported() -> bool:
    return torch.cuda.is_available()


def _pair_rows_and_swap(marlin_scales: torch.Tensor) -> torch.Tensor:
    """[G, N] -> [G, N] with, for every row pair (2i, 2i+1) and 8-column chunk j, the 16 values
    (row 2i chunk j, row 2i+1 chunk j) adjacent, and every run of 4 reordered to (0, 2, 1, 3)
    (marlin_utils_fp4.py:38-47, 66-73)."""
    g, n = marlin_scales.shape
    assert g % 2 == 0 and n % 8 == 0
    paired = marlin_scales.view(g // 2, 2, n // 8, 8).permute(0, 2, 1, 3).reshape(g, n)
    return paired.reshape(-1, 4)[:, [0, 2, 1, 3]].reshape(g, n)


def nvfp4_marlin_process_scales(marlin_scales: torch.Tensor) -> torch.Tensor:
    s = _pair_rows_and_swap(marlin_scales.to(torch.half))
    # half(s * 2^7) << 1 drops the (zero) sign bit; its high byte is 5 exponent and 3 mantissa bits
    as_bytes = ((s * (2 ** 7)).view(torch.int16) << 1).view(torch.float8_e4m3fn)
    return as_bytes[:, 1::2].contiguous()


def mxfp4_marlin_process_scales(marlin_scales: torch.Tensor) -> torch.Tensor:
    return _pair_rows_and_swap(marlin_scales).to(torch.float8_e8m0fnu)


def nvfp4_marlin_process_global_scale(global_scale: torch.Tensor) -> torch.Tensor:
    """global_scale * 2^(bias(dtype) - bias(e2m1) - 7): 2^7 for fp16, 2^119 for bf16 (marlin_utils_fp4.py:82-93)."""
    assert global_scale.dtype in (torch.half, torch.bfloat16)
    target_exponent_bits = 5 if global_scale.dtype == torch.half else 8
    exponent_bias = 2 ** (target_exponent_bits - 1) - 2 ** (2 - 1)
    return global_scale * (2.0 ** (exponent_bias - 7))


def apply_fp4_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                            weight_scale_2: torch.Tensor | None, workspace: torch.Tensor, size_n: int, size_k: int,
                            bias: torch.Tensor | None = None,
                            use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    x = input.reshape(-1, input.shape[-1])
    use_atomic_add = should_use_atomic_add_reduce(m=x.size(0), n=size_n, k=size_k, device=input.device,
                                                  dtype=input.dtype)
    out = ops.gptq_marlin_gemm(a=x, c=None, b_q_weight=weight, b_bias=bias, b_scales=weight_scale,
                               global_scale=weight_scale_2, b_zeros=None, g_idx=None, perm=None, workspace=workspace,
                               b_q_type=scalar_types.float4_e2m1f, size_m=x.size(0), size_n=size_n, size_k=size_k,
                               use_atomic_add=use_atomic_add, use_fp32_reduce=use_fp32_reduce)
    return out.reshape(input.shape[:-1] + (size_n,))


def prepare_fp4_layer_for_marlin(layer: torch.nn.Module) -> None:
    """layer.weight uint8 [N, K/2] (two codes per byte, low nibble first), weight_scale [N, K/group] and, for NVFP4,
    weight_scale_2 -> Marlin-layout weight, processed scales, workspace, permuted bias
    (marlin_utils_fp4.py:135-199)."""
    is_nvfp4 = hasattr(layer, "weight_scale_2")
    group_size = 16 if is_nvfp4 else 32
    size_n, size_k = layer.output_size_per_partition, layer.input_size_per_partition
    dtype = layer.params_dtype
    assert layer.weight.shape == (size_n, size_k // 2)
    device = layer.weight.device
    layer.workspace = marlin_make_workspace_new(device)
    packed = layer.weight.view(torch.int32).T.contiguous()
    layer.weight = torch.nn.Parameter(
        ops.gptq_marlin_repack(b_q_weight=packed, perm=torch.empty(0, dtype=torch.int, device=device), size_k=size_k,
                               size_n=size_n, num_bits=4), requires_grad=False)
    scales = layer.weight_scale.T.contiguous()
    if not is_nvfp4:
        scales = scales.view(torch.float8_e8m0fnu)
    scales = marlin_permute_scales(s=scales.to(dtype), size_k=size_k, size_n=size_n, group_size=group_size)
    if is_nvfp4:
        layer.weight_scale = torch.nn.Parameter(nvfp4_marlin_process_scales(scales), requires_grad=False)
        layer.weight_scale_2 = torch.nn.Parameter(
            nvfp4_marlin_process_global_scale(layer.weight_scale_2.to(dtype)), requires_grad=False)
    else:
        layer.weight_scale = torch.nn.Parameter(mxfp4_marlin_process_scales(scales), requires_grad=False)
    if getattr(layer, "bias", None) is not None:
        assert layer.bias.shape == (size_n,)
        layer.bias = torch.nn.Parameter(marlin_permute_bias(layer.bias), requires_grad=False)


def _fp4_bytes_to_values(codes: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """uint8 [N, K/2] -> [N, K] values: the low nibble of byte i is element 2i."""
    table = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
                         dtype=dtype, device=codes.device)
    lo, hi = table[(codes & 0xF).long()], table[(codes >> 4).long()]
    return torch.stack([lo, hi], dim=2).reshape(codes.shape[0], -1)


def rand_marlin_weight_nvfp4_like(weight: torch.Tensor, group_size: int):
    """Test helper with the reference's contract (marlin_utils_fp4.py:303-346): weight [N, K] only sets the scale
    magnitudes; the fp4 codes are random bytes.  Returns (w_ref [K, N], Marlin weight, processed scales, processed
    global scale)."""
    assert group_size > 0
    size_n, size_k = weight.shape
    dev = weight.device
    scales = weight.view(size_n, -1, group_size).abs().amax(-1) / 6
    global_scale = scales.max() / 448
    scales = (scales / global_scale).to(torch.float8_e4m3fn)
    codes = torch.randint(0, 256, (size_n, size_k // 2), dtype=torch.uint8, device=dev)
    w_ref = (_fp4_bytes_to_values(codes, weight.dtype) * global_scale.to(weight.dtype)
             * scales.repeat_interleave(group_size, 1).to(weight.dtype))
    marlin_q = ops.gptq_marlin_repack(b_q_weight=codes.view(torch.int32).T.contiguous(),
                                      perm=torch.empty(0, dtype=torch.int, device=dev), size_k=size_k, size_n=size_n,
                                      num_bits=4)
    marlin_s = marlin_permute_scales(s=scales.T.to(weight.dtype), size_k=size_k, size_n=size_n, group_size=group_size)
    return (w_ref.T, marlin_q, nvfp4_marlin_process_scales(marlin_s),
            nvfp4_marlin_process_global_scale(global_scale.to(weight.dtype)))


def rand_marlin_weight_mxfp4_like(weight: torch.Tensor, group_size: int):
    """As above for MXFP4 (marlin_utils_fp4.py:349-397): E8M0 scale bytes drawn from [100, 125)."""
    assert group_size > 0
    size_n, size_k = weight.shape
    dev = weight.device
    scales = torch.randint(100, 125, (size_n, size_k // group_size), dtype=torch.uint8, device=dev).view(
        torch.float8_e8m0fnu)
    codes = torch.randint(0, 256, (size_n, size_k // 2), dtype=torch.uint8, device=dev)
    w_ref = _fp4_bytes_to_values(codes, weight.dtype) * scales.repeat_interleave(group_size, 1).to(weight.dtype)
    marlin_q = ops.gptq_marlin_repack(b_q_weight=codes.view(torch.int32).T.contiguous(),
                                      perm=torch.empty(0, dtype=torch.int, device=dev), size_k=size_k, size_n=size_n,
                                      num_bits=4)
    marlin_s = marlin_permute_scales(s=scales.T.to(weight.dtype), size_k=size_k, size_n=size_n, group_size=group_size)
    return w_ref.T, marlin_q, mxfp4_marlin_process_scales(marlin_s)
