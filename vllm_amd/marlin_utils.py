"""Host-side helpers of the Marlin linear path, mirroring the reference's
vllm/model_executor/layers/quantization/utils/marlin_utils.py (names, arguments and results),
restricted to what the 4-bit GPTQ / AWQ path needs.  All tensor work runs on the tensor's device.
"""
import torch

from . import _custom_ops as ops
from . import _lib
from .quant_utils import pack_cols, unpack_cols
from .scalar_type import ScalarType, scalar_types

GPTQ_MARLIN_TILE = 16
GPTQ_MARLIN_MIN_THREAD_N = 64
GPTQ_MARLIN_MIN_THREAD_K = 128
GPTQ_MARLIN_MAX_PARALLEL = 16

MARLIN_SUPPORTED_GROUP_SIZES = [-1, 32, 64, 128]
USE_FP32_REDUCE_DEFAULT = True

_INTERLEAVE_4BIT = (0, 2, 4, 6, 1, 3, 5, 7)


def query_marlin_supported_quant_types(has_zp: bool | None = None, include_fp_type: bool = True,
                                       device_capability: int | None = None) -> list[ScalarType]:
    """marlin_utils.py:35-78, narrowed to the types this library implements."""
    if has_zp is None:
        return (query_marlin_supported_quant_types(False, include_fp_type, device_capability) +
                query_marlin_supported_quant_types(True, include_fp_type, device_capability))
    if has_zp:
        return [scalar_types.uint4]
    res = [scalar_types.uint4b8, scalar_types.uint8b128]
    return res + [scalar_types.float8_e4m3fn, scalar_types.float4_e2m1f] if include_fp_type else res


def check_marlin_supports_shape(output_size_per_partition: int, input_size_per_partition: int,
                                input_size: int, group_size: int) -> tuple[bool, str | None]:
    """marlin_utils.py:126-175 (same gates, same messages)."""
    try:
        verify_marlin_supports_shape(output_size_per_partition, input_size_per_partition, input_size, group_size)
    except ValueError as e:
        return False, str(e)
    return True, None


def verify_marlin_supports_shape(output_size_per_partition: int, input_size_per_partition: int,
                                 input_size: int, group_size: int) -> None:
    if output_size_per_partition % GPTQ_MARLIN_MIN_THREAD_N != 0:
        raise ValueError(f"Weight output_size_per_partition = {output_size_per_partition} is not divisible by "
                         f" min_thread_n = {GPTQ_MARLIN_MIN_THREAD_N}. Consider reducing tensor_parallel_size or "
                         "running with --quantization gptq.")
    if input_size_per_partition % GPTQ_MARLIN_MIN_THREAD_K != 0:
        raise ValueError(f"Weight input_size_per_partition = {input_size_per_partition} is not divisible by "
                         f"min_thread_k = {GPTQ_MARLIN_MIN_THREAD_K}. Consider reducing tensor_parallel_size or "
                         "running with --quantization gptq.")
    if group_size < input_size and input_size_per_partition % group_size != 0:
        raise ValueError(f"Weight input_size_per_partition = {input_size_per_partition} is not divisible by "
                         f"group_size = {group_size}. Consider reducing tensor_parallel_size or running with "
                         "--quantization gptq.")


def _check_marlin_supported(quant_type: ScalarType, group_size: int | None, has_zp: bool,
                            device_capability: int | None = None) -> tuple[bool, str | None]:
    """Type and group-size gate with the reference's messages (marlin_utils.py:72-104)."""
    supported_types = query_marlin_supported_quant_types(has_zp, True, device_capability)
    if quant_type not in supported_types:
        return False, (f"Marlin does not support weight_bits = {quant_type}. Only types = "
                       f"{[str(t) for t in supported_types]} are supported (for group_size = {group_size}, "
                       f"device_capability = {device_capability}, zp = {has_zp}).")
    if group_size is None or group_size not in MARLIN_SUPPORTED_GROUP_SIZES:
        return False, (f"Marlin does not support group_size = {group_size}. Only group_sizes = "
                       f"{MARLIN_SUPPORTED_GROUP_SIZES} are supported.")
    return True, None


def check_marlin_supported(quant_type: ScalarType, group_size: int, has_zp: bool = False,
                           device_capability: int | None = None) -> bool:
    return _check_marlin_supported(quant_type, group_size, has_zp, device_capability)[0]


def verify_marlin_supported(quant_type: ScalarType, group_size: int, has_zp: bool = False) -> None:
    ok, msg = _check_marlin_supported(quant_type, group_size, has_zp)
    if not ok:
        raise ValueError(msg)


def check_marlin_supports_layer(layer, group_size: int) -> bool:
    """marlin_utils.py:176-189: the layer's partition sizes (or its full sizes) against the shape gates."""
    out_size = getattr(layer, "output_size_per_partition", None) or layer.output_size
    in_size = getattr(layer, "input_size_per_partition", None) or layer.input_size
    return check_marlin_supports_shape(out_size, in_size, layer.input_size, group_size)[0]


def check_moe_marlin_supports_layer(layer, group_size: int) -> bool:
    """marlin_utils.py:192-213: hidden % 128, intermediate % max(64, group), SiLU, router weight on the output."""
    shape_ok = layer.hidden_size % 128 == 0 and layer.intermediate_size_per_partition % max(64, group_size) == 0
    return (shape_ok and group_size in (-1, 32, 64, 128) and not layer.apply_router_weight_on_input and
            layer.activation == "silu")


def marlin_moe_intermediate_size(w1_packed: torch.Tensor, w2_packed: torch.Tensor) -> int:
    """w2 is [E, N/16, ...]: rows are 16-row k-tiles of the intermediate size N (marlin_utils.py:216-222)."""
    return w2_packed.size(1) * GPTQ_MARLIN_TILE


def marlin_make_workspace(output_size_per_partition: int, device: torch.device) -> torch.Tensor:
    """The older sizing rule, (N / 64) * 16 zeroed ints (marlin_utils.py:225-234); any all-zero int32 tensor works."""
    size = (output_size_per_partition // GPTQ_MARLIN_MIN_THREAD_N) * GPTQ_MARLIN_MAX_PARALLEL
    return torch.zeros(size, dtype=torch.int, device=device, requires_grad=False)


def marlin_make_workspace_new(device: torch.device, max_blocks_per_sm: int = 1) -> torch.Tensor:
    """int32 zeros, four counters per compute unit (x max_blocks_per_sm); the reference's function
    (marlin_utils.py:237-245) allocates one per SM, which the GEMM also accepts: the extra length only lets it place
    the counters of neighbouring tiles 16 bytes apart.  The GEMM keeps the all-zero-on-exit invariant, so one
    workspace serves any number of calls."""
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    return torch.zeros(4 * cus * max_blocks_per_sm, dtype=torch.int, device=device, requires_grad=False)


def marlin_is_k_full(act_order: bool, is_row_parallel: bool) -> bool:
    return (not act_order) or (act_order and not is_row_parallel)


def marlin_repeat_scales_on_all_ranks(act_order: bool, group_size: int, is_row_parallel: bool) -> bool:
    return act_order or (group_size == -1 and is_row_parallel)


def marlin_make_empty_g_idx(device: torch.device) -> torch.Tensor:
    return torch.nn.Parameter(torch.empty(0, dtype=torch.int, device=device), requires_grad=False)


def marlin_make_empty_zp(device: torch.device) -> torch.Tensor:
    return torch.nn.Parameter(torch.empty(0, dtype=torch.int, device=device), requires_grad=False)


def marlin_sort_g_idx(g_idx: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    g_idx_sort_indices = torch.argsort(g_idx).to(torch.int)
    return g_idx[g_idx_sort_indices.long()], g_idx_sort_indices


def get_scale_perms() -> tuple[list[int], list[int]]:
    scale_perm = [i + 8 * j for i in range(8) for j in range(8)]
    scale_perm_single = [2 * i + j for i in range(4) for j in (0, 1, 8, 9, 16, 17, 24, 25)]
    return scale_perm, scale_perm_single


def _device_permute(s: torch.Tensor, grouped: bool) -> torch.Tensor:
    """One launch of the library's permutation kernel over rows of s.shape[-1] elements."""
    src = s.contiguous()
    out = torch.empty_like(src)
    if src.numel():
        with torch.cuda.device(src.device):
            _lib.check(_lib.load().w4a16_marlin_permute_scales(
                src.data_ptr(), out.data_ptr(), src.numel() // src.shape[-1], src.shape[-1], int(grouped),
                torch.cuda.current_stream(src.device).cuda_stream))
    return out


def _torch_permute(s: torch.Tensor, perm: list[int], shape) -> torch.Tensor:
    idx = torch.tensor(perm, device=s.device)
    return s.reshape((-1, len(perm)))[:, idx].reshape(shape).contiguous()


def marlin_permute_scales(s: torch.Tensor, size_k: int, size_n: int, group_size: int) -> torch.Tensor:
    """[G, size_n] scales -> Marlin order (reference marlin_utils.py:288-298).  16-bit tensors on the GPU go through
    one kernel launch; anything else (byte-sized fp4 scales, host tensors) through torch indexing."""
    grouped = group_size < size_k and group_size != -1
    if s.is_cuda and s.element_size() == 2 and size_n % 64 == 0:
        return _device_permute(s.reshape(-1, size_n), grouped)
    scale_perm, scale_perm_single = get_scale_perms()
    return _torch_permute(s, scale_perm if grouped else scale_perm_single, (-1, size_n))


def marlin_permute_bias(s: torch.Tensor) -> torch.Tensor:
    if s.is_cuda and s.element_size() == 2 and s.shape[-1] % 64 == 0:
        return _device_permute(s, False)
    return _torch_permute(s, get_scale_perms()[1], s.shape)


def marlin_moe_permute_scales(s: torch.Tensor, size_k: int, size_n: int, group_size: int) -> torch.Tensor:
    """All experts in one launch: the permutation works on rows, whichever expert they belong to."""
    return marlin_permute_scales(s.reshape(-1, size_n), size_k, size_n, group_size).reshape(s.shape)


def _device_zero_points(zp: torch.Tensor, num_groups: int, size_n: int, fmt: int) -> torch.Tensor:
    src = zp.contiguous()
    out = torch.empty((num_groups, size_n // 8), dtype=torch.int32, device=src.device)
    if out.numel():
        with torch.cuda.device(src.device):
            _lib.check(_lib.load().w4a16_marlin_zero_points(src.data_ptr(), out.data_ptr(), num_groups, size_n, fmt,
                                                            torch.cuda.current_stream(src.device).cuda_stream))
    return out


def marlin_zero_points(zp: torch.Tensor, size_k: int, size_n: int, num_bits: int) -> torch.Tensor:
    """Unpacked zero points [size_k(=groups), size_n] -> Marlin-packed int32 [groups, size_n/8]
    (marlin_utils.py:326-346)."""
    assert num_bits == 4, "only 4-bit zero points are implemented"
    if zp.is_cuda and size_n % 64 == 0:
        return _device_zero_points(zp.reshape(size_k, size_n).to(torch.int32), size_k, size_n, 2)
    scale_perm, _ = get_scale_perms()
    zp = zp.reshape((-1, len(scale_perm)))[:, torch.tensor(scale_perm, device=zp.device)]
    inter = torch.tensor(_INTERLEAVE_4BIT, device=zp.device)
    zp = zp.reshape((-1, len(_INTERLEAVE_4BIT)))[:, inter].reshape((-1, size_n)).contiguous()
    return pack_cols(zp, num_bits, size_k, size_n)


def marlin_zero_points_from_packed(zp_packed: torch.Tensor, num_groups: int, size_n: int, num_bits: int) -> torch.Tensor:
    """Column-packed zero points int32 [groups, size_n/8] (nibble j of word c = column 8c + j) -> Marlin packing.
    Same result as marlin_zero_points(unpack_cols(zp_packed, ...), ...) without the unpacked intermediate."""
    assert num_bits == 4, "only 4-bit zero points are implemented"
    if zp_packed.is_cuda and size_n % 64 == 0:
        return _device_zero_points(zp_packed, num_groups, size_n, 0)
    return marlin_zero_points(unpack_cols(zp_packed, num_bits, num_groups, size_n), num_groups, size_n, num_bits)


def awq_to_marlin_zero_points(q_zp_packed: torch.Tensor, size_k: int, size_n: int, num_bits: int) -> torch.Tensor:
    """AWQ-packed zero points -> Marlin-packed (marlin_utils.py:349-370)."""
    assert num_bits == 4, "only 4-bit zero points are implemented"
    if q_zp_packed.is_cuda and size_n % 64 == 0:
        return _device_zero_points(q_zp_packed, size_k, size_n, 1)
    q_zp = unpack_cols(q_zp_packed, num_bits, size_k, size_n)
    undo = torch.argsort(torch.tensor(_INTERLEAVE_4BIT, device=q_zp.device))
    q_zp = q_zp.reshape((-1, len(_INTERLEAVE_4BIT)))[:, undo].reshape((-1, size_n)).contiguous()
    return marlin_zero_points(q_zp, size_k, size_n, num_bits)


def moe_awq_to_marlin_zero_points(q_zp_packed: torch.Tensor, size_k: int, size_n: int, num_bits: int):
    """All experts in one launch ([E, groups, size_n/8] is [E * groups, size_n/8] to the kernel)."""
    e = q_zp_packed.shape[0]
    return awq_to_marlin_zero_points(q_zp_packed.reshape(e * size_k, -1), e * size_k, size_n, num_bits).reshape(
        q_zp_packed.shape)


def should_use_atomic_add_reduce(m: int, n: int, k: int, device: torch.device, dtype: torch.dtype) -> bool:
    """Kept for callers that import it (reference marlin_utils.py:412-432).  The gfx950 kernels sum split-K partials in
    fp32 in a fixed order and have no atomic-add reduction to switch on, so the answer is always False."""
    return False


def _marlin_linear(x: torch.Tensor, weight, scales, zeros, g_idx, sort_indices, workspace, wtype: ScalarType,
                   size_n: int, size_k: int, is_k_full: bool, bias, use_fp32_reduce: bool) -> torch.Tensor:
    """[..., size_k] activations through one gptq_marlin_gemm call; leading dimensions are kept."""
    x2d = x.reshape(-1, x.shape[-1])
    y = ops.gptq_marlin_gemm(x2d, None, weight, bias, scales, None, zeros, g_idx, sort_indices, workspace, wtype,
                             x2d.shape[0], size_n, size_k, is_k_full, False, use_fp32_reduce, False)
    return y.reshape(*x.shape[:-1], size_n)


def apply_gptq_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                             weight_zp: torch.Tensor, g_idx: torch.Tensor, g_idx_sort_indices: torch.Tensor,
                             workspace: torch.Tensor, wtype: ScalarType, output_size_per_partition: int,
                             input_size_per_partition: int, is_k_full: bool, bias: torch.Tensor | None = None,
                             use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    """Argument list of the reference's function of this name (marlin_utils.py:435-480)."""
    return _marlin_linear(input, weight, weight_scale, weight_zp, g_idx, g_idx_sort_indices, workspace, wtype,
                          output_size_per_partition, input_size_per_partition, is_k_full, bias, use_fp32_reduce)


def apply_awq_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                            weight_zp: torch.Tensor, g_idx: torch.Tensor, g_idx_sort_indices: torch.Tensor,
                            workspace: torch.Tensor, quant_type: ScalarType, output_size_per_partition: int,
                            input_size_per_partition: int, bias: torch.Tensor | None = None,
                            use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    """Argument list of the reference's function of this name (marlin_utils.py:483-530); AWQ has no act-order."""
    return _marlin_linear(input, weight, weight_scale, weight_zp, g_idx, g_idx_sort_indices, workspace, quant_type,
                          output_size_per_partition, input_size_per_partition, True, bias, use_fp32_reduce)


def apply_rtn_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                            workspace: torch.Tensor, quant_type: ScalarType, output_size_per_partition: int,
                            input_size_per_partition: int, bias: torch.Tensor | None = None,
                            use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    """Round-to-nearest checkpoints: symmetric weights, no zero points, no act-order (marlin_utils.py:533-577)."""
    return _marlin_linear(input, weight, weight_scale, None, None, None, workspace, quant_type,
                          output_size_per_partition, input_size_per_partition, True, bias, use_fp32_reduce)
