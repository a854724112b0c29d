"""ctypes binding of the C ABI declared in include/w4a16_gfx950.h.

The shared library is the product: if it is missing or does not load, importing the ops fails
loudly — there is no CPU or PyTorch fallback behind these calls.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libw4a16_gfx950.so")

W4A16_OK = 0
STATIC_SCRATCH_BYTES = 64 << 20  # W4A16_STATIC_SCRATCH_BYTES
WTYPE_U4B8, WTYPE_U4, WTYPE_U8B128, WTYPE_FE4M3, WTYPE_FE2M1 = 0, 1, 2, 3, 4
DTYPE_F16, DTYPE_BF16, DTYPE_F32 = 0, 1, 2
ABI_VERSION = 3  # W4A16_ABI_VERSION of include/w4a16_gfx950.h this mirror was written against
F_IS_K_FULL, F_USE_ATOMIC_ADD, F_USE_FP32_REDUCE, F_MUL_TOPK_WEIGHTS, F_MOE, F_ZP_FLOAT = 1, 2, 4, 8, 16, 32
F_SILU_AND_MUL, F_SUM_TOPK = 64, 128

c_void_p, c_i64, c_i32, c_u32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_uint32


class GemmArgs(ctypes.Structure):
    """Mirror of `struct w4a16_gemm_args`."""
    _fields_ = [
        ("struct_size", c_u32), ("dtype", c_i32), ("wtype", c_i32), ("flags", c_i32),
        ("a", c_void_p), ("lda", c_i64), ("c", c_void_p),
        ("b_q_weight", c_void_p), ("b_scales", c_void_p), ("b_zeros", c_void_p),
        ("g_idx", c_void_p), ("perm", c_void_p), ("b_bias", c_void_p),
        ("c_tmp", c_void_p), ("workspace", c_void_p), ("workspace_len", c_i64),
        ("size_m", c_i64), ("size_n", c_i64), ("size_k", c_i64), ("num_groups", c_i64),
        ("sorted_token_ids", c_void_p), ("expert_ids", c_void_p),
        ("num_tokens_past_padded", c_void_p), ("topk_weights", c_void_p),
        ("n_sorted", c_i64), ("moe_block_size", c_i32), ("top_k", c_i32),
        ("num_experts", c_i32), ("reserved", c_i32), ("global_scale", c_void_p),
        ("zero_fill", c_void_p), ("zero_fill_bytes", c_i64), ("sum_top_k", c_i32), ("reserved2", c_i32),
    ]


EXPORTS = {
    "w4a16_abi_version": (ctypes.c_int, []),
    "w4a16_last_error": (ctypes.c_char_p, []),
    "w4a16_gptq_marlin_repack": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_i64, ctypes.c_int, c_void_p]),
    "w4a16_awq_marlin_repack": (ctypes.c_int, [c_void_p, c_void_p, c_i64, c_i64, ctypes.c_int, c_void_p]),
    "w4a16_permute_cols": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_i64, c_void_p]),
    "w4a16_marlin_permute_scales": (ctypes.c_int, [c_void_p, c_void_p, c_i64, c_i64, ctypes.c_int, c_void_p]),
    "w4a16_marlin_zero_points": (ctypes.c_int, [c_void_p, c_void_p, c_i64, c_i64, ctypes.c_int, c_void_p]),
    "w4a16_gemm_scratch_bytes": (c_i64, [ctypes.POINTER(GemmArgs)]),
    "w4a16_marlin_gemm": (ctypes.c_int, [ctypes.POINTER(GemmArgs), c_void_p]),
    "w4a16_marlin_gemm_static": (ctypes.c_int, [ctypes.POINTER(GemmArgs), c_void_p]),
    "w4a16_moe_align_block_size": (ctypes.c_int, [c_void_p, c_i64, c_i32, c_i32, c_void_p, c_i64, c_void_p,
                                                  c_i64, c_void_p, c_void_p]),
    "w4a16_batched_moe_align_block_size": (ctypes.c_int, [c_i64, c_i32, c_void_p, c_i32, c_void_p, c_i64, c_void_p,
                                                          c_i64, c_void_p, c_void_p]),
    "w4a16_moe_sum": (ctypes.c_int, [c_void_p, c_void_p, c_i64, c_i32, c_i64, c_i32, c_void_p]),
    "w4a16_silu_and_mul": (ctypes.c_int, [c_void_p, c_void_p, c_i64, c_i64, c_i32, c_void_p]),
    "w4a16_topk_softmax": (ctypes.c_int, [c_void_p, c_i32, c_void_p, c_void_p, c_void_p, c_i64, c_i32, c_i32, c_i32,
                                          c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: build it with `python -m vllm_amd.build` (hipcc, gfx950). "
                "There is no fallback implementation.")
        # torch first: it brings its own HIP runtime, and this library must bind to that same instance (loaded the
        # other way round the process holds two runtimes, and launches here fail with "no ROCm-capable device")
        import torch  # noqa: F401
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        if lib.w4a16_abi_version() != ABI_VERSION:
            raise ImportError("w4a16 ABI version mismatch")
        _lib = lib
    return _lib


def check(rc: int) -> None:
    if rc != W4A16_OK:
        msg = load().w4a16_last_error().decode("utf-8", "replace")
        if rc == -2:
            raise NotImplementedError(msg)
        raise RuntimeError(msg)
