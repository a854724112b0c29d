"""Compiler-output check for the kernels that issue MFMAs through inline assembly (gemm_fat.hip, gemm_mid.hip,
gemm_kq.hip): no MFMA operand (A, B or the accumulator) may be written by a VALU instruction fewer than two wait states
before the MFMA reads it.  The scan itself lives in vllm_amd/build.py and also runs in the build step; here it runs on
the real compiler output and on hand-written snippets that must (not) trip it."""
import os
import tempfile

from vllm_amd import build as vbuild


def _scan(text):
    with tempfile.NamedTemporaryFile("w", suffix=".s", delete=False) as f:
        f.write(text)
    try:
        return vbuild.scan_mfma_hazards(f.name)
    finally:
        os.unlink(f.name)


def test_scan_flags_close_writes_and_accepts_distant_ones():
    mfma = "v_mfma_f32_16x16x32_f16 a[0:3], v[4:7], v[8:11], a[0:3]"
    assert _scan(f"v_and_or_b32 v5, v1, v2, v3\n{mfma}\n")[1]                      # A operand, 0 wait states
    assert _scan(f"v_pk_mul_f16 v10, v1, v2\nv_mov_b32 v20, v21\n{mfma}\n")[1]      # B operand, 1 wait state
    assert _scan(f"v_accvgpr_write_b32 a2, v1\n{mfma}\n")[1]                        # accumulator
    assert not _scan(f"v_pk_mul_f16 v10, v1, v2\nv_mov_b32 v20, v21\nv_mov_b32 v22, v21\n{mfma}\n")[1]
    assert not _scan(f"v_pk_mul_f16 v10, v1, v2\ns_nop 1\n{mfma}\n")[1]
    assert not _scan(f"v_and_or_b32 v12, v1, v2, v3\n{mfma}\n")[1]                  # unrelated register
    assert _scan(f"{mfma}\n{mfma}\n")[0] == 2


def test_no_valu_write_right_before_an_asm_mfma():
    assert vbuild.check_mfma_hazards() >= 3 * 1024
