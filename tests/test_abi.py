"""The shared library loads and exports exactly what include/w4a16_gfx950.h declares (no GPU needed)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "w4a16_gfx950.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(w4a16_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = declared_functions()
    for must in ("w4a16_gptq_marlin_repack", "w4a16_awq_marlin_repack", "w4a16_marlin_gemm",
                 "w4a16_gemm_scratch_bytes", "w4a16_moe_align_block_size", "w4a16_moe_sum", "w4a16_silu_and_mul",
                 "w4a16_permute_cols", "w4a16_abi_version", "w4a16_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from vllm_amd import _lib
    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.EXPORTS) == declared_functions()          # the ctypes table covers the header exactly
    assert lib.w4a16_abi_version() == _lib.ABI_VERSION == 3


def test_args_struct_matches_header_layout():
    """Field order and size of the ctypes mirror follow `struct w4a16_gemm_args`."""
    from vllm_amd import _lib
    text = open(HEADER).read()
    body = re.search(r"typedef struct w4a16_gemm_args \{(.*?)\} w4a16_gemm_args;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for decl in body.split(";"):
        if decl.strip():  # "int64_t size_m, size_n" declares several fields
            fields += [re.search(r"(\w+)\s*$", part.strip()).group(1) for part in decl.split(",")]
    assert fields == [f[0] for f in _lib.GemmArgs._fields_]
    assert ctypes.sizeof(_lib.GemmArgs) % 8 == 0


def test_argument_errors_are_reported_without_a_gpu():
    """Validation runs on the host before any HIP call: bad shapes come back as W4A16_EINVAL with a message."""
    from vllm_amd import _lib
    lib = _lib.load()
    rc = lib.w4a16_gptq_marlin_repack(None, None, None, 24, 64, 4, None)
    assert rc == -1 and b"size_k" in lib.w4a16_last_error()
    rc = lib.w4a16_awq_marlin_repack(None, None, 16, 96, 4, None)
    assert rc == -1 and b"size_n" in lib.w4a16_last_error()
    args = _lib.GemmArgs()
    args.struct_size = 4
    assert lib.w4a16_marlin_gemm(ctypes.byref(args), None) == -1
