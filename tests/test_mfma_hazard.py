"""Compiler-output check for the kernels that issue MFMAs through inline assembly (gemm_fat.hip, gemm_mid.hip,
gemm_kq.hip): no MFMA operand (A, B or the accumulator) may be written by a VALU instruction fewer than two wait states
before the MFMA reads it, along any control-flow path.  The scan lives in vllm_amd/build.py and runs in the build step on
the assembly the shipped objects are assembled from; here it runs on the compiler output for the same sources and flags
and on hand-written snippets that must (not) trip it."""
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


def test_scan_follows_branches_and_labels():
    mfma = "v_mfma_f32_16x16x32_f16 a[0:3], v[4:7], v[8:11], a[0:3]"
    # loop back-edge: the write at the bottom of the body is one wait state (the branch) away from the MFMA at the top
    loop = f".LBB0_1:\n{mfma}\nv_mov_b32 v20, v21\nv_mov_b32 v22, v21\nv_and_or_b32 v5, v1, v2, v3\ns_cbranch_scc1 .LBB0_1\n"
    assert _scan(loop)[1]
    safe = f".LBB0_1:\n{mfma}\nv_and_or_b32 v5, v1, v2, v3\nv_mov_b32 v20, v21\ns_cbranch_scc1 .LBB0_1\n"
    assert not _scan(safe)[1]
    # a forward branch over the padding reaches the MFMA right after the write
    fwd = f"v_and_or_b32 v5, v1, v2, v3\ns_cbranch_vccz .LBB0_2\ns_nop 4\n.LBB0_2:\n{mfma}\n"
    assert _scan(fwd)[1]
    # code behind an unconditional branch does not fall through into the label
    away = f"v_and_or_b32 v5, v1, v2, v3\ns_branch .LBB0_4\n.LBB0_3:\n{mfma}\n.LBB0_4:\ns_nop 0\n"
    assert not _scan(away)[1]


def test_no_valu_write_right_before_an_asm_mfma():
    assert vbuild.scan_sources() >= 3 * 1024
