"""PyTorch operator surface of the gfx950 W4A16 library.

Defines (when nothing else has) and implements, for the CUDA dispatch key (= HIP tensors on
PyTorch-ROCm), the operators the reference reaches through `vllm/_custom_ops.py`:

  _C::gptq_marlin_repack, _C::awq_marlin_repack, _C::gptq_marlin_gemm, _C::permute_cols,
  _C::silu_and_mul, _moe_C::moe_wna16_marlin_gemm, _moe_C::moe_align_block_size, _moe_C::moe_sum,
  _moe_C::topk_softmax, _moe_C::batched_moe_align_block_size

with the reference's schemas (csrc/torch_bindings.cpp:118, 312-336; csrc/moe/torch_bindings.cpp:13-23, 63-75),
plus fake (meta) implementations for tracing (reference vllm/_custom_ops.py:553-576, 1179-1218,
2089-2120).  On ROCm builds of the reference these operator definitions are compiled out
(csrc/torch_bindings.cpp:240, csrc/moe/torch_bindings.cpp:52), which is why they are defined here.

The Python wrappers below keep the names and argument order of the reference's wrappers
(vllm/_custom_ops.py:1167-1303, 2004-2060).  Every implementation calls the HIP library through
its C ABI; there is no fallback.
"""
import ctypes

import torch

from . import _lib
from .scalar_type import ScalarType, scalar_types

_GEMM_SCHEMA = (
    "gptq_marlin_gemm(Tensor a, Tensor? c_or_none, Tensor b_q_weight, Tensor? b_bias_or_none, "
    "Tensor b_scales, Tensor? global_scale, Tensor? b_zeros_or_none, Tensor? g_idx_or_none, "
    "Tensor? perm_or_none, Tensor workspace, int b_q_type, SymInt size_m, SymInt size_n, "
    "SymInt size_k, bool is_k_full, bool use_atomic_add, bool use_fp32_reduce, "
    "bool is_zp_float) -> Tensor")
_MOE_GEMM_SCHEMA = (
    "moe_wna16_marlin_gemm(Tensor! a, Tensor? c_or_none, Tensor! b_q_weight, Tensor? b_bias_or_none, "
    "Tensor! b_scales, Tensor? global_scale, Tensor? b_zeros_or_none, Tensor? g_idx_or_none, "
    "Tensor? perm_or_none, Tensor! workspace, Tensor sorted_token_ids, Tensor! expert_ids, "
    "Tensor! num_tokens_past_padded, Tensor! topk_weights, int moe_block_size, int top_k, "
    "bool mul_topk_weights, bool is_ep, int b_q_type_id, int size_m, int size_n, int size_k, "
    "bool is_full_k, bool use_atomic_add, bool use_fp32_reduce, bool is_zp_float) -> Tensor")

_C_SCHEMAS = {
    "gptq_marlin_gemm": _GEMM_SCHEMA,
    "gptq_marlin_repack": "gptq_marlin_repack(Tensor b_q_weight, Tensor perm, SymInt size_k, SymInt size_n, "
                          "int num_bits) -> Tensor",
    "awq_marlin_repack": "awq_marlin_repack(Tensor b_q_weight, SymInt size_k, SymInt size_n, int num_bits) -> Tensor",
    "permute_cols": "permute_cols(Tensor A, Tensor perm) -> Tensor",
    "silu_and_mul": "silu_and_mul(Tensor! result, Tensor input) -> ()",
}
_MOE_SCHEMAS = {
    "moe_wna16_marlin_gemm": _MOE_GEMM_SCHEMA,
    "moe_align_block_size": "moe_align_block_size(Tensor topk_ids, int num_experts, int block_size, "
                            "Tensor! sorted_token_ids, Tensor! experts_ids, Tensor! num_tokens_post_pad) -> ()",
    "batched_moe_align_block_size": "batched_moe_align_block_size(int max_tokens_per_batch, int block_size, "
                                    "Tensor expert_num_tokens, Tensor! sorted_token_ids, Tensor! experts_ids, "
                                    "Tensor! num_tokens_post_pad) -> ()",
    "moe_sum": "moe_sum(Tensor input, Tensor! output) -> ()",
    "topk_softmax": "topk_softmax(Tensor! topk_weights, Tensor! topk_indices, Tensor! token_expert_indices, "
                    "Tensor gating_output, bool renormalize) -> ()",
}


def _ptr(t: torch.Tensor | None):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _opt(t: torch.Tensor | None) -> torch.Tensor | None:
    """`Tensor?` arguments arrive as None or as zero-length tensors; both mean absent."""
    return None if t is None or t.numel() == 0 else t


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float16:
        return _lib.DTYPE_F16
    if dt == torch.bfloat16:
        return _lib.DTYPE_BF16
    raise RuntimeError("gpt_marlin_gemm only supports bfloat16 and float16")


def _wtype_code(type_id: int, has_zp: bool) -> int:
    if type_id == scalar_types.uint4b8.id:
        _check(not has_zp, "b_q_type must be uint4 or uint8 when has_zp = True. Got = uint4b8")
        return _lib.WTYPE_U4B8
    if type_id == scalar_types.uint8b128.id:
        _check(not has_zp, "b_q_type must be uint4 or uint8 when has_zp = True. Got = uint8b128")
        return _lib.WTYPE_U8B128
    if type_id == scalar_types.uint4.id:
        _check(has_zp, "b_q_type must be uint4b8 or uint8b128 when has_zp = False. Got = uint4")
        return _lib.WTYPE_U4
    if type_id == scalar_types.float8_e4m3fn.id:
        _check(not has_zp, "b_q_type must be uint4 or uint8 when has_zp = True. Got = float8_e4m3fn")
        return _lib.WTYPE_FE4M3
    if type_id == scalar_types.float4_e2m1f.id:
        _check(not has_zp, "b_q_type must be uint4 or uint8 when has_zp = True. Got = float4_e2m1f")
        return _lib.WTYPE_FE2M1
    raise NotImplementedError(
        f"weight type {ScalarType.from_id(type_id)} is not implemented by the gfx950 W4A16 library "
        "(supported: uint4b8, uint8b128, float8_e4m3fn, float4_e2m1f, uint4 with zero points)")


def _pack_factor(type_id: int) -> int:
    return 32 // ScalarType.from_id(int(type_id)).size_bits


# ------------------------------------------------------------------------------- implementations
def _gptq_marlin_repack_impl(b_q_weight, perm, size_k, size_n, num_bits):
    size_k, size_n = int(size_k), int(size_n)
    _check(num_bits in (4, 8), f"num_bits must be 4 or 8. Got = {num_bits}")
    pack = 32 // num_bits
    _check(size_k % 16 == 0, f"size_k = {size_k} is not divisible by tile_k_size = 16")
    _check(size_n % 64 == 0, f"size_n = {size_n} is not divisible by tile_n_size = 64")
    _check(b_q_weight.is_cuda and b_q_weight.is_contiguous(), "b_q_weight is not a contiguous GPU tensor")
    _check(b_q_weight.dtype == torch.int32, "b_q_weight type is not kInt")
    _check(tuple(b_q_weight.shape) == (size_k // pack, size_n),
           f"Shape mismatch: b_q_weight = {tuple(b_q_weight.shape)}, size_k = {size_k}, size_n = {size_n}")
    _check(perm.dtype == torch.int32, "perm type is not at::kInt")
    has_perm = perm.numel() != 0
    if has_perm:
        _check(perm.is_cuda and perm.is_contiguous() and perm.numel() == size_k, "perm must be a contiguous [size_k] GPU tensor")
    out = torch.empty((size_k // 16, size_n * 16 // pack), dtype=torch.int32, device=b_q_weight.device)
    if out.numel():
        with torch.cuda.device(b_q_weight.device):
            _lib.check(_lib.load().w4a16_gptq_marlin_repack(
                _ptr(b_q_weight), _ptr(perm) if has_perm else None, _ptr(out), size_k, size_n, num_bits,
                _stream(b_q_weight.device)))
    return out


def _awq_marlin_repack_impl(b_q_weight, size_k, size_n, num_bits):
    size_k, size_n = int(size_k), int(size_n)
    _check(num_bits in (4, 8), f"num_bits must be 4 or 8. Got = {num_bits}")
    pack = 32 // num_bits
    _check(size_k % 16 == 0, f"size_k = {size_k} is not divisible by tile_k_size = 16")
    _check(size_n % 64 == 0, f"size_n = {size_n} is not divisible by tile_n_size = 64")
    _check(b_q_weight.is_cuda and b_q_weight.is_contiguous(), "b_q_weight is not a contiguous GPU tensor")
    _check(b_q_weight.dtype == torch.int32, "b_q_weight type is not kInt")
    _check(tuple(b_q_weight.shape) == (size_k, size_n // pack),
           f"Shape mismatch: b_q_weight = {tuple(b_q_weight.shape)}, size_k = {size_k}, size_n = {size_n}")
    out = torch.empty((size_k // 16, size_n * 16 // pack), dtype=torch.int32, device=b_q_weight.device)
    if out.numel():
        with torch.cuda.device(b_q_weight.device):
            _lib.check(_lib.load().w4a16_awq_marlin_repack(_ptr(b_q_weight), _ptr(out), size_k, size_n, num_bits,
                                                            _stream(b_q_weight.device)))
    return out


def _permute_cols_impl(A, perm):
    _check(A.is_cuda and A.dim() == 2 and A.stride(1) == 1, "A must be a 2-D GPU tensor with unit column stride")
    _check(A.dtype in (torch.float16, torch.bfloat16), "A must be fp16 or bf16")
    _check(perm.dtype == torch.int32 and perm.is_contiguous() and perm.numel() == A.shape[1], "bad perm")
    out = torch.empty((A.shape[0], A.shape[1]), dtype=A.dtype, device=A.device)
    if out.numel():
        with torch.cuda.device(A.device):
            _lib.check(_lib.load().w4a16_permute_cols(_ptr(A), _ptr(perm), _ptr(out), A.shape[0], A.shape[1],
                                                       A.stride(0), _stream(A.device)))
    return out


def _fill_common(args, a, c, b_q_weight, b_bias, b_scales, b_zeros, g_idx, perm, workspace, wtype,
                 size_m, size_n, size_k, num_groups, flags):
    args.struct_size = ctypes.sizeof(_lib.GemmArgs)
    args.dtype = _dtype_code(a.dtype)
    args.wtype = wtype
    args.flags = flags
    args.a = a.data_ptr()
    args.lda = a.stride(0)
    args.c = c.data_ptr()
    args.b_q_weight = b_q_weight.data_ptr()
    args.b_scales = b_scales.data_ptr()
    args.b_zeros = None if b_zeros is None else b_zeros.data_ptr()
    args.g_idx = None if g_idx is None else g_idx.data_ptr()
    args.perm = None if perm is None else perm.data_ptr()
    args.b_bias = None if b_bias is None else b_bias.data_ptr()
    args.workspace = workspace.data_ptr()
    args.workspace_len = workspace.numel()
    args.size_m, args.size_n, args.size_k = size_m, size_n, size_k
    args.num_groups = num_groups


def _run_gemm(args, device) -> None:
    lib = _lib.load()
    with torch.cuda.device(device):
        need = lib.w4a16_gemm_scratch_bytes(ctypes.byref(args))
        if need < 0:
            _lib.check(int(need))
        c_tmp = None
        if need > 0:
            c_tmp = torch.empty(need // 4, dtype=torch.float32, device=device)
            args.c_tmp = c_tmp.data_ptr()
        _lib.check(lib.w4a16_marlin_gemm(ctypes.byref(args), _stream(device)))


def _gptq_marlin_gemm_impl(a, c_or_none, b_q_weight, b_bias_or_none, b_scales, global_scale,
                           b_zeros_or_none, g_idx_or_none, perm_or_none, workspace, b_q_type,
                           size_m, size_n, size_k, is_k_full, use_atomic_add, use_fp32_reduce, is_zp_float):
    size_m, size_n, size_k = int(size_m), int(size_n), int(size_k)
    _check(a.dim() == 2 and a.size(0) == size_m, f"Shape mismatch: a.size(0) = {a.size(0)}, size_m = {size_m}")
    _check(a.size(1) == size_k, f"Shape mismatch: a.size(1) = {a.size(1)}, size_k = {size_k}")
    _check(size_k % 16 == 0, f"size_k = {size_k} is not divisible by tile_size = 16")
    _check(b_q_weight.dim() == 2 and size_k // 16 == b_q_weight.size(0),
           f"Shape mismatch: b_q_weight.size(0) = {b_q_weight.size(0)}, size_k = {size_k}, tile_size = 16")
    _check(b_q_weight.size(1) % 16 == 0, f"b_q_weight.size(1) = {b_q_weight.size(1)} is not divisible by tile_size = 16")
    pf = _pack_factor(b_q_type)
    _check(size_n == b_q_weight.size(1) // 16 * pf,
           f"Shape mismatch: b_q_weight.size(1) = {b_q_weight.size(1)}, size_n = {size_n}, pack_factor = {pf}")
    _check(a.is_cuda, "A is not on GPU")
    _check(a.stride(1) == 1, "A.stride(1) is not 1")
    _check(a.stride(0) % 8 == 0, "A.stride(0) must divisible by 8")
    _check(a.data_ptr() % 16 == 0, "A must aligned to 16 bytes")
    _check(b_q_weight.is_cuda and b_q_weight.is_contiguous(), "b_q_weight is not a contiguous GPU tensor")
    _check(b_q_weight.dtype == torch.int32, "b_q_weight type is not kInt")
    _check(b_scales.is_cuda and b_scales.is_contiguous(), "b_scales is not a contiguous GPU tensor")
    _check(b_scales.dim() == 2 and b_scales.size(1) == size_n,
           f"b_scales dim 1 = {b_scales.size(-1)} is not size_n = {size_n}")
    num_groups = b_scales.size(0)
    is_fp4 = int(b_q_type) == scalar_types.float4_e2m1f.id
    gscale = _opt(global_scale)
    if is_fp4:
        # one byte per (group, column): NVFP4 (group 16) float8_e4m3fn + global_scale, MXFP4 (group 32) float8_e8m0fnu
        group_size = size_k // num_groups if num_groups > 0 and size_k % num_groups == 0 else 0
        _check(group_size in (16, 32),
               "float4_e2m1f only supports group_size == 16 (NVFP4) and group_size == 32 (MXFP4)")
        want = torch.float8_e4m3fn if group_size == 16 else torch.float8_e8m0fnu
        _check(b_scales.dtype == want, f"b_scales must be {want} for float4_e2m1f with group_size = {group_size}")
        if group_size == 16:
            _check(gscale is not None, "the global_scale parameter must be passed for nvfp4 format.")
            _check(gscale.is_cuda and gscale.numel() == 1 and gscale.dtype == a.dtype,
                   "global_scale must be one element of the activation type on the GPU")
        else:
            _check(gscale is None, "global_scale can only be used for nvfp4 format.")
    else:
        _check(b_scales.dtype == a.dtype, "scalar type of a and b_scales must match")
        _check(gscale is None, "global_scale can only be used for nvfp4 format.")
    _check(workspace.is_cuda and workspace.dtype == torch.int32, "workspace must be an int32 GPU tensor")

    g_idx, perm = _opt(g_idx_or_none), _opt(perm_or_none)
    _check((g_idx is None) == (perm is None),
           f"Unexpected g_idx.size(-1) = {0 if g_idx is None else g_idx.numel()} and "
           f"perm.size(-1) = {0 if perm is None else perm.numel()}")
    for name, t in (("g_idx", g_idx), ("perm", perm)):
        if t is not None:
            _check(t.is_cuda and t.is_contiguous() and t.dtype == torch.int32 and t.numel() == size_k,
                   f"{name} must be a contiguous int32 [size_k] GPU tensor")

    b_zeros = None
    if b_zeros_or_none is not None and b_zeros_or_none.size(-1) > 0:
        b_zeros = b_zeros_or_none
        _check(b_zeros.is_cuda and b_zeros.is_contiguous(), "b_zeros is not a contiguous GPU tensor")
        _check(b_zeros.dim() == 2, f"b_zeros rank = {b_zeros.dim()} is not 2")
        _check(b_zeros.size(0) == num_groups, f"b_zeros dim 0 = {b_zeros.size(0)} is not num_groups = {num_groups}")
        if is_zp_float:  # HQQ: fp16 zero points shaped and permuted like the scales (gptq_marlin.cu:866-887)
            _check(a.dtype == torch.float16, "Computation type must be float16 (half) when using float zero points.")
            _check(b_zeros.dtype == a.dtype, "b_zeros type is not the type of a")
            _check(b_zeros.size(1) == size_n, f"b_zeros dim 1 = {b_zeros.size(1)} is not size_n = {size_n}")
        else:
            _check(b_zeros.dtype == torch.int32, "b_zeros type is not kInt")
            _check(b_zeros.size(1) == size_n // 8,
                   f"b_zeros dim 1 = {b_zeros.size(1)} is not size_n / pack_factor = {size_n // 8}")
    _check(not is_zp_float or b_zeros is not None, "is_zp_float = True needs b_zeros")
    wtype = _wtype_code(int(b_q_type), b_zeros is not None)

    b_bias = _opt(b_bias_or_none)
    if b_bias is not None:
        _check(b_bias.is_cuda and b_bias.numel() == size_n and b_bias.stride(-1) == 1 and b_bias.dtype == a.dtype,
               "b_bias.size(0) must be size_n, stride 1, dtype of a")

    if c_or_none is not None:
        c = c_or_none
        _check(c.is_cuda and c.is_contiguous(), "c is not a contiguous GPU tensor")
        _check(c.size(0) == size_m and c.size(1) == size_n and c.dtype == a.dtype, "Shape mismatch: c")
    else:
        c = torch.empty((size_m, size_n), dtype=a.dtype, device=a.device)
    if size_m == 0:
        return c

    flags = _lib.F_USE_FP32_REDUCE if use_fp32_reduce else 0
    if is_k_full:
        flags |= _lib.F_IS_K_FULL
    if use_atomic_add:
        flags |= _lib.F_USE_ATOMIC_ADD
    if is_zp_float:
        flags |= _lib.F_ZP_FLOAT
    args = _lib.GemmArgs()
    _fill_common(args, a, c, b_q_weight, b_bias, b_scales, b_zeros, g_idx, perm, workspace, wtype,
                 size_m, size_n, size_k, num_groups, flags)
    args.global_scale = None if gscale is None else gscale.data_ptr()
    _run_gemm(args, a.device)
    return c


def _moe_wna16_marlin_gemm_impl(a, c_or_none, b_q_weight, b_bias_or_none, b_scales, global_scale,
                                b_zeros_or_none, g_idx_or_none, perm_or_none, workspace, sorted_token_ids,
                                expert_ids, num_tokens_past_padded, topk_weights, moe_block_size, top_k,
                                mul_topk_weights, is_ep, b_q_type_id, size_m, size_n, size_k, is_full_k,
                                use_atomic_add, use_fp32_reduce, is_zp_float):
    return _moe_gemm(a, c_or_none, b_q_weight, b_bias_or_none, b_scales, global_scale, b_zeros_or_none, g_idx_or_none,
                     perm_or_none, workspace, sorted_token_ids, expert_ids, num_tokens_past_padded, topk_weights,
                     moe_block_size, top_k, mul_topk_weights, b_q_type_id, size_m, size_n, size_k, is_full_k,
                     use_atomic_add, use_fp32_reduce, is_zp_float)


def _moe_marlin_gemm_fused_impl(a, c, b_q_weight, b_bias_or_none, b_scales, global_scale, b_zeros_or_none,
                                g_idx_or_none, perm_or_none, workspace, sorted_token_ids, expert_ids,
                                num_tokens_past_padded, topk_weights, moe_block_size, top_k, mul_topk_weights,
                                b_q_type_id, size_m, size_n, size_k, is_full_k, silu_and_mul, sum_top_k, zero_fill):
    _moe_gemm(a, c, b_q_weight, b_bias_or_none, b_scales, global_scale, b_zeros_or_none, g_idx_or_none, perm_or_none,
              workspace, sorted_token_ids, expert_ids, num_tokens_past_padded, topk_weights, moe_block_size, top_k,
              mul_topk_weights, b_q_type_id, size_m, size_n, size_k, is_full_k, False, True, False,
              silu_and_mul=silu_and_mul, sum_top_k=sum_top_k, zero_fill=zero_fill)


def _moe_gemm(a, c_or_none, b_q_weight, b_bias_or_none, b_scales, global_scale, b_zeros_or_none, g_idx_or_none,
              perm_or_none, workspace, sorted_token_ids, expert_ids, num_tokens_past_padded, topk_weights,
              moe_block_size, top_k, mul_topk_weights, b_q_type_id, size_m, size_n, size_k, is_full_k,
              use_atomic_add, use_fp32_reduce, is_zp_float, silu_and_mul=False, sum_top_k=0, zero_fill=None):
    """One launch of the MoE GEMM.  silu_and_mul: c is [size_m * top_k, size_n / 2] = silu(gate) * up;
    sum_top_k > 0: c is [size_m * top_k / sum_top_k, size_n], already zero, and receives the sum of each token's rows;
    zero_fill: a tensor the launch clears on the side (the output of a later sum_top_k launch)."""
    _check(a.is_cuda and a.is_contiguous() and a.dim() == 2, "A is not a contiguous 2-D GPU tensor")
    _check(a.size(0) == size_m, f"Shape mismatch: a.size(0) = {a.size(0)}, size_m = {size_m}")
    _check(a.size(1) == size_k, f"Shape mismatch: a.size(1) = {a.size(1)}, size_k = {size_k}")
    _check(moe_block_size == 8 or (moe_block_size % 16 == 0 and 16 <= moe_block_size <= 64),
           f"unsupported moe_block_size={moe_block_size}")
    _check(b_q_weight.is_cuda and b_q_weight.is_contiguous() and b_q_weight.dim() == 3 and b_q_weight.dtype == torch.int32,
           "b_q_weight is not a contiguous 3-D int32 GPU tensor")
    num_experts = b_q_weight.size(0)
    _check(size_k % 16 == 0 and b_q_weight.size(1) == size_k // 16,
           f"Shape mismatch: b_q_weight.size(1) = {b_q_weight.size(1)}, size_k = {size_k}, tile_size = 16")
    pf = _pack_factor(b_q_type_id)
    _check(b_q_weight.size(2) % 16 == 0 and size_n == b_q_weight.size(2) // 16 * pf,
           f"Shape mismatch: b_q_weight.size(2) = {b_q_weight.size(2)}, size_n = {size_n}, pack_factor = {pf}")
    _check(b_scales.is_cuda and b_scales.is_contiguous() and b_scales.dim() == 3, "b_scales rank is not 3")
    _check(b_scales.size(0) == num_experts and b_scales.size(2) == size_n,
           f"b_scales dim 2 = {b_scales.size(2)} is not size_n = {size_n}")
    _check(not is_zp_float, "float zero points (HQQ) are not implemented for the MoE op by the gfx950 W4A16 library")
    num_groups = b_scales.size(1)
    gscale = _opt(global_scale)
    if int(b_q_type_id) == scalar_types.float4_e2m1f.id:
        group_size = size_k // num_groups if num_groups > 0 and size_k % num_groups == 0 else 0
        _check(group_size in (16, 32),
               "float4_e2m1f only supports group_size == 16 (NVFP4) and group_size == 32 (MXFP4)")
        want = torch.float8_e4m3fn if group_size == 16 else torch.float8_e8m0fnu
        _check(b_scales.dtype == want, f"b_scales must be {want} for float4_e2m1f with group_size = {group_size}")
        if group_size == 16:
            _check(gscale is not None, "the global_scale parameter must be passed for nvfp4 format.")
            _check(gscale.is_cuda and gscale.is_contiguous() and gscale.numel() == num_experts and
                   gscale.dtype == a.dtype, "global_scale must hold one element of the activation type per expert")
        else:
            _check(gscale is None, "global_scale can only be used for nvfp4 format.")
    else:
        _check(b_scales.dtype == a.dtype, "scalar type of a and b_scales must match")
        _check(gscale is None, "global_scale can only be used for nvfp4 format.")
    g_idx, perm = _opt(g_idx_or_none), _opt(perm_or_none)
    _check((g_idx is None) == (perm is None), "g_idx and perm must both be given or both be empty")
    for name, t in (("g_idx", g_idx), ("perm", perm)):
        if t is not None:
            _check(t.is_cuda and t.is_contiguous() and t.dtype == torch.int32 and tuple(t.shape) == (num_experts, size_k),
                   f"{name} must be a contiguous int32 [E, size_k] GPU tensor")
    b_zeros = None
    if b_zeros_or_none is not None and b_zeros_or_none.size(-1) > 0:
        b_zeros = b_zeros_or_none
        _check(b_zeros.is_cuda and b_zeros.is_contiguous() and b_zeros.dtype == torch.int32 and b_zeros.dim() == 3,
               f"b_zeros rank = {b_zeros.dim()} is not 3")
        _check(b_zeros.size(1) == num_groups and b_zeros.size(2) == size_n // 8, "b_zeros shape mismatch")
    wtype = _wtype_code(int(b_q_type_id), b_zeros is not None)
    b_bias = _opt(b_bias_or_none)
    if b_bias is not None:
        _check(b_bias.is_cuda and b_bias.is_contiguous() and tuple(b_bias.shape) == (num_experts, size_n) and
               b_bias.dtype == a.dtype, "b_bias must be [E, size_n]")
    for name, t in (("sorted_token_ids", sorted_token_ids), ("expert_ids", expert_ids),
                    ("num_tokens_past_padded", num_tokens_past_padded)):
        _check(t.is_cuda and t.is_contiguous() and t.dtype == torch.int32, f"{name} must be a contiguous int32 GPU tensor")
    _check(expert_ids.numel() * moe_block_size >= sorted_token_ids.numel() - moe_block_size + 1,
           "expert_ids is too short for sorted_token_ids")
    _check(topk_weights.is_cuda and topk_weights.dtype == torch.float32 and topk_weights.is_contiguous(),
           "topk_weights must be a contiguous fp32 GPU tensor")
    c_shape = (size_m * top_k // max(sum_top_k, 1), size_n // 2 if silu_and_mul else size_n)
    if silu_and_mul:
        _check(size_n % 128 == 0, f"fused SiLU-and-mul: size_n = {size_n} must be 2 * d with d a multiple of 64")
    if sum_top_k:
        _check(sum_top_k in (1, 2) and (size_m * top_k) % sum_top_k == 0, f"unsupported sum_top_k = {sum_top_k}")
    if c_or_none is not None:
        c = c_or_none
        _check(c.is_cuda and c.is_contiguous() and c.dtype == a.dtype, "c is not a contiguous GPU tensor")
        _check(tuple(c.shape) == c_shape, "Shape mismatch: c")
    else:
        _check(not sum_top_k, "the fused top-k sum accumulates into a caller-provided, zeroed c")
        c = torch.empty(c_shape, dtype=a.dtype, device=a.device)
    if zero_fill is not None:
        _check(zero_fill.is_cuda and zero_fill.is_contiguous() and zero_fill.data_ptr() % 16 == 0 and
               (zero_fill.numel() * zero_fill.element_size()) % 16 == 0,
               "zero_fill must be a contiguous, 16-byte aligned GPU tensor of a multiple of 16 bytes")
    if size_m == 0:
        if zero_fill is not None:
            zero_fill.zero_()
        return c

    flags = _lib.F_MOE | (_lib.F_USE_FP32_REDUCE if use_fp32_reduce else 0)
    if silu_and_mul:
        flags |= _lib.F_SILU_AND_MUL
    if sum_top_k:
        flags |= _lib.F_SUM_TOPK
    if is_full_k:
        flags |= _lib.F_IS_K_FULL
    if use_atomic_add:
        flags |= _lib.F_USE_ATOMIC_ADD
    if mul_topk_weights:
        flags |= _lib.F_MUL_TOPK_WEIGHTS
    args = _lib.GemmArgs()
    _fill_common(args, a, c, b_q_weight, b_bias, b_scales, b_zeros, g_idx, perm, workspace, wtype,
                 size_m, size_n, size_k, num_groups, flags)
    args.sorted_token_ids = sorted_token_ids.data_ptr()
    args.expert_ids = expert_ids.data_ptr()
    args.num_tokens_past_padded = num_tokens_past_padded.data_ptr()
    args.topk_weights = topk_weights.data_ptr()
    args.n_sorted = min(sorted_token_ids.numel(), expert_ids.numel() * moe_block_size)
    args.moe_block_size = moe_block_size
    args.top_k = top_k
    args.num_experts = num_experts
    args.global_scale = None if gscale is None else gscale.data_ptr()
    args.sum_top_k = sum_top_k
    if zero_fill is not None:
        args.zero_fill = zero_fill.data_ptr()
        args.zero_fill_bytes = zero_fill.numel() * zero_fill.element_size()
    _run_gemm(args, a.device)
    return c


def _moe_align_block_size_impl(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad):
    _check(topk_ids.is_cuda and topk_ids.is_contiguous(), "topk_ids must be a contiguous GPU tensor")
    ids = topk_ids if topk_ids.dtype == torch.int32 else topk_ids.to(torch.int32)
    for t in (sorted_token_ids, experts_ids, num_tokens_post_pad):
        _check(t.is_cuda and t.is_contiguous() and t.dtype == torch.int32, "outputs must be contiguous int32 GPU tensors")
    with torch.cuda.device(topk_ids.device):
        _lib.check(_lib.load().w4a16_moe_align_block_size(
            _ptr(ids), ids.numel(), num_experts, block_size, _ptr(sorted_token_ids), sorted_token_ids.numel(),
            _ptr(experts_ids), experts_ids.numel(), _ptr(num_tokens_post_pad), _stream(topk_ids.device)))


def _batched_moe_align_block_size_impl(max_tokens_per_batch, block_size, expert_num_tokens, sorted_token_ids,
                                       experts_ids, num_tokens_post_pad):
    _check(expert_num_tokens.is_cuda and expert_num_tokens.is_contiguous() and expert_num_tokens.dim() == 1,
           "expert_num_tokens must be a contiguous 1-D GPU tensor")
    n = expert_num_tokens if expert_num_tokens.dtype == torch.int32 else expert_num_tokens.to(torch.int32)
    for t in (sorted_token_ids, experts_ids, num_tokens_post_pad):
        _check(t.is_cuda and t.is_contiguous() and t.dtype == torch.int32, "outputs must be contiguous int32 GPU tensors")
    with torch.cuda.device(n.device):
        _lib.check(_lib.load().w4a16_batched_moe_align_block_size(
            max_tokens_per_batch, block_size, _ptr(n), n.numel(), _ptr(sorted_token_ids), sorted_token_ids.numel(),
            _ptr(experts_ids), experts_ids.numel(), _ptr(num_tokens_post_pad), _stream(n.device)))


def _moe_sum_impl(input, output):
    _check(input.is_cuda and input.is_contiguous() and input.dim() == 3, "input must be a contiguous [T, topk, d] GPU tensor")
    _check(output.is_contiguous() and output.dtype == input.dtype and
           tuple(output.shape) == (input.size(0), input.size(2)), "output must be [T, d]")
    with torch.cuda.device(input.device):
        _lib.check(_lib.load().w4a16_moe_sum(_ptr(input), _ptr(output), input.size(0), input.size(1), input.size(2),
                                              _dtype_code(input.dtype), _stream(input.device)))


def _silu_and_mul_impl(result, input):
    d = input.size(-1) // 2
    _check(input.is_cuda and input.is_contiguous() and result.is_contiguous(), "tensors must be contiguous GPU tensors")
    _check(result.size(-1) == d and result.numel() * 2 == input.numel() and result.dtype == input.dtype, "shape mismatch")
    with torch.cuda.device(input.device):
        _lib.check(_lib.load().w4a16_silu_and_mul(_ptr(input), _ptr(result), input.numel() // (2 * d), d,
                                                   _dtype_code(input.dtype), _stream(input.device)))


def _topk_softmax_impl(topk_weights, topk_indices, token_expert_indices, gating_output, renormalize):
    _check(gating_output.is_cuda and gating_output.is_contiguous() and gating_output.dim() == 2,
           "gating_output must be a contiguous [num_tokens, num_experts] GPU tensor")
    num_tokens, num_experts = gating_output.shape
    topk = topk_weights.size(-1)
    _check(topk_weights.dtype == torch.float32 and topk_weights.is_contiguous() and
           tuple(topk_weights.shape) == (num_tokens, topk), "topk_weights must be fp32 [num_tokens, topk]")
    _check(token_expert_indices.dtype == torch.int32 and token_expert_indices.is_contiguous() and
           tuple(token_expert_indices.shape) == (num_tokens, topk), "token_expert_indices must be int32 [num_tokens, topk]")
    _check(tuple(topk_indices.shape) == (num_tokens, topk) and topk_indices.is_contiguous(), "topk_indices shape mismatch")
    code = {torch.float16: _lib.DTYPE_F16, torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_F32}.get(
        gating_output.dtype)
    _check(code is not None, "gating_output must be fp16, bf16 or fp32")
    ids = topk_indices if topk_indices.dtype == torch.int32 else torch.empty_like(topk_indices, dtype=torch.int32)
    with torch.cuda.device(gating_output.device):
        _lib.check(_lib.load().w4a16_topk_softmax(
            _ptr(gating_output), code, _ptr(topk_weights), _ptr(ids), _ptr(token_expert_indices), num_tokens,
            num_experts, topk, int(bool(renormalize)), _stream(gating_output.device)))
    if ids is not topk_indices:
        topk_indices.copy_(ids)


# ------------------------------------------------------------------------------------- fakes
def _gemm_fake(a, c_or_none, b_q_weight, b_bias_or_none, b_scales, global_scale, b_zeros_or_none,
               g_idx_or_none, perm_or_none, workspace, b_q_type, size_m, size_n, size_k,
               is_k_full=True, use_atomic_add=False, use_fp32_reduce=False, is_zp_float=False):
    return torch.empty((size_m, size_n), device=a.device, dtype=a.dtype)


def _repack_fake(b_q_weight, perm, size_k, size_n, num_bits):
    return torch.empty((size_k // 16, size_n * 16 // (32 // num_bits)), dtype=b_q_weight.dtype, device=b_q_weight.device)


def _awq_repack_fake(b_q_weight, size_k, size_n, num_bits):
    return torch.empty((size_k // 16, size_n * 16 // (32 // num_bits)), dtype=b_q_weight.dtype, device=b_q_weight.device)


def _moe_gemm_fake(a, c_or_none, b_q_weight, b_bias_or_none, b_scales, global_scale, b_zeros_or_none,
                   g_idx_or_none, perm_or_none, workspace, sorted_token_ids, expert_ids, num_tokens_past_padded,
                   topk_weights, moe_block_size, top_k, mul_topk_weights, is_ep, b_q_type_id, size_m, size_n,
                   size_k, is_full_k, use_atomic_add, use_fp32_reduce, is_zp_float):
    return torch.empty((size_m * top_k, size_n), dtype=a.dtype, device=a.device)


_IMPLS = {
    "_C": {
        "gptq_marlin_gemm": (_gptq_marlin_gemm_impl, _gemm_fake),
        "gptq_marlin_repack": (_gptq_marlin_repack_impl, _repack_fake),
        "awq_marlin_repack": (_awq_marlin_repack_impl, _awq_repack_fake),
        "permute_cols": (_permute_cols_impl, lambda A, perm: torch.empty_like(A, memory_format=torch.contiguous_format)),
        "silu_and_mul": (_silu_and_mul_impl, lambda result, input: None),
    },
    "_moe_C": {
        "moe_wna16_marlin_gemm": (_moe_wna16_marlin_gemm_impl, _moe_gemm_fake),
        "moe_align_block_size": (_moe_align_block_size_impl, lambda *a: None),
        "batched_moe_align_block_size": (_batched_moe_align_block_size_impl, lambda *a: None),
        "moe_sum": (_moe_sum_impl, lambda input, output: None),
        "topk_softmax": (_topk_softmax_impl, lambda *a: None),
    },
}
# Operators of this library's own: the MoE GEMM with a fused epilogue (no counterpart in the reference, which runs
# silu_and_mul and moe_sum as separate launches).  c, workspace and zero_fill are written.
_OWN_SCHEMAS = {
    "moe_marlin_gemm_fused": (
        "moe_marlin_gemm_fused(Tensor a, Tensor(a!) c, Tensor b_q_weight, Tensor? b_bias_or_none, Tensor b_scales, "
        "Tensor? global_scale, Tensor? b_zeros_or_none, Tensor? g_idx_or_none, Tensor? perm_or_none, "
        "Tensor(b!) workspace, Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_past_padded, "
        "Tensor topk_weights, int moe_block_size, int top_k, bool mul_topk_weights, int b_q_type_id, int size_m, "
        "int size_n, int size_k, bool is_full_k, bool silu_and_mul, int sum_top_k, Tensor(c!)? zero_fill) -> ()"),
}
_IMPLS["w4a16"] = {"moe_marlin_gemm_fused": (_moe_marlin_gemm_fused_impl, lambda *a: None)}
_SCHEMAS = {"_C": _C_SCHEMAS, "_moe_C": _MOE_SCHEMAS, "w4a16": _OWN_SCHEMAS}
_libs: list = []          # keep torch.library.Library objects alive
REGISTERED: list[str] = []  # "ns::op" names this module defined and implemented


def _has_op(ns: str, name: str) -> bool:
    try:
        return hasattr(getattr(torch.ops, ns), name)
    except (AttributeError, RuntimeError):
        return False


def _register() -> None:
    _lib.load()  # fail loudly at import if the HIP library is missing
    for ns, ops_ in _IMPLS.items():
        frag = torch.library.Library(ns, "FRAGMENT")
        _libs.append(frag)
        for name, (impl, fake) in ops_.items():
            if _has_op(ns, name):
                continue  # somebody else (a CUDA build of the reference) already provides it
            frag.define(_SCHEMAS[ns][name], tags=(torch.Tag.needs_fixed_stride_order,))
            frag.impl(name, impl, "CUDA")
            torch.library.register_fake(f"{ns}::{name}", fake, lib=frag)
            REGISTERED.append(f"{ns}::{name}")


_register()


# ----------------------------------------------------------------- wrappers (reference names)
def gptq_marlin_repack(b_q_weight: torch.Tensor, perm: torch.Tensor, size_k: int, size_n: int,
                       num_bits: int) -> torch.Tensor:
    return torch.ops._C.gptq_marlin_repack(b_q_weight, perm, size_k, size_n, num_bits)


def awq_marlin_repack(b_q_weight: torch.Tensor, size_k: int, size_n: int, num_bits: int) -> torch.Tensor:
    return torch.ops._C.awq_marlin_repack(b_q_weight, size_k, size_n, num_bits)


def gptq_marlin_moe_repack(b_q_weight: torch.Tensor, perm: torch.Tensor, size_k: int, size_n: int,
                           num_bits: int) -> torch.Tensor:
    """Per-expert repack, as vllm/_custom_ops.py:1221-1239."""
    num_experts = b_q_weight.shape[0]
    assert size_k % 16 == 0
    output = torch.empty((num_experts, size_k // 16, size_n * (num_bits // 2)), device=b_q_weight.device,
                         dtype=b_q_weight.dtype)
    for e in range(num_experts):
        output[e] = torch.ops._C.gptq_marlin_repack(b_q_weight[e], perm[e], size_k, size_n, num_bits)
    return output


def awq_marlin_moe_repack(b_q_weight: torch.Tensor, perm: torch.Tensor, size_k: int, size_n: int,
                          num_bits: int) -> torch.Tensor:
    """Per-expert repack, as vllm/_custom_ops.py:1242-1260 (`perm` is unused there too)."""
    num_experts = b_q_weight.shape[0]
    assert size_k % 16 == 0
    output = torch.empty((num_experts, size_k // 16, size_n * (num_bits // 2)), device=b_q_weight.device,
                         dtype=b_q_weight.dtype)
    for e in range(num_experts):
        output[e] = torch.ops._C.awq_marlin_repack(b_q_weight[e], size_k, size_n, num_bits)
    return output


def gptq_marlin_gemm(a, c, b_q_weight, b_bias, b_scales, global_scale, b_zeros, g_idx, perm, workspace,
                     b_q_type: ScalarType, size_m: int, size_n: int, size_k: int, is_k_full: bool = True,
                     use_atomic_add: bool = False, use_fp32_reduce: bool = False,
                     is_zp_float: bool = False) -> torch.Tensor:
    return torch.ops._C.gptq_marlin_gemm(a, c, b_q_weight, b_bias, b_scales, global_scale, b_zeros, g_idx, perm,
                                         workspace, b_q_type.id, size_m, size_n, size_k, is_k_full,
                                         use_atomic_add, use_fp32_reduce, is_zp_float)


def moe_wna16_marlin_gemm(input, output, b_qweight, b_bias, b_scales, global_scale, b_qzeros, g_idx, perm,
                          workspace, sorted_token_ids, expert_ids, num_tokens_past_padded, topk_weights,
                          moe_block_size: int, top_k: int, mul_topk_weights: bool, is_ep: bool,
                          b_q_type: ScalarType, size_m: int, size_n: int, size_k: int, is_k_full: bool,
                          use_atomic_add: bool, use_fp32_reduce: bool, is_zp_float: bool) -> torch.Tensor:
    return torch.ops._moe_C.moe_wna16_marlin_gemm(
        input, output, b_qweight, b_bias, b_scales, global_scale, b_qzeros, g_idx, perm, workspace,
        sorted_token_ids, expert_ids, num_tokens_past_padded, topk_weights, moe_block_size, top_k,
        mul_topk_weights, is_ep, b_q_type.id, size_m, size_n, size_k, is_k_full, use_atomic_add,
        use_fp32_reduce, is_zp_float)


def moe_marlin_gemm_fused(a, c, b_qweight, b_bias, b_scales, global_scale, b_qzeros, g_idx, perm, workspace,
                          sorted_token_ids, expert_ids, num_tokens_past_padded, topk_weights, moe_block_size: int,
                          top_k: int, mul_topk_weights: bool, b_q_type: ScalarType, size_m: int, size_n: int,
                          size_k: int, is_k_full: bool, silu_and_mul: bool = False, sum_top_k: int = 0,
                          zero_fill: torch.Tensor | None = None) -> None:
    """The MoE GEMM writing through a fused epilogue into `c`: silu_and_mul -> c [size_m * top_k, size_n / 2];
    sum_top_k = 2 -> c [size_m * top_k / 2, size_n] (zero on entry) receives each token's two rows added up;
    zero_fill: a tensor this launch also clears."""
    torch.ops.w4a16.moe_marlin_gemm_fused(
        a, c, b_qweight, b_bias, b_scales, global_scale, b_qzeros, g_idx, perm, workspace, sorted_token_ids,
        expert_ids, num_tokens_past_padded, topk_weights, moe_block_size, top_k, mul_topk_weights, b_q_type.id,
        size_m, size_n, size_k, is_k_full, silu_and_mul, sum_top_k, zero_fill)


def batched_moe_align_block_size(max_tokens_per_batch: int, block_size: int, expert_num_tokens: torch.Tensor,
                                 sorted_ids: torch.Tensor, expert_ids: torch.Tensor,
                                 num_tokens_post_pad: torch.Tensor) -> None:
    torch.ops._moe_C.batched_moe_align_block_size(max_tokens_per_batch, block_size, expert_num_tokens, sorted_ids,
                                                  expert_ids, num_tokens_post_pad)


def permute_cols(a: torch.Tensor, perm: torch.Tensor) -> torch.Tensor:
    return torch.ops._C.permute_cols(a, perm)


def silu_and_mul(out: torch.Tensor, x: torch.Tensor) -> None:
    torch.ops._C.silu_and_mul(out, x)


def moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                         num_tokens_post_pad) -> None:
    torch.ops._moe_C.moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                                          num_tokens_post_pad)


def moe_sum(input: torch.Tensor, output: torch.Tensor) -> None:
    torch.ops._moe_C.moe_sum(input, output)


def topk_softmax(topk_weights: torch.Tensor, topk_ids: torch.Tensor, token_expert_indices: torch.Tensor,
                 gating_output: torch.Tensor, renormalize: bool = False) -> None:
    torch.ops._moe_C.topk_softmax(topk_weights, topk_ids, token_expert_indices, gating_output, renormalize)
