"""Compiler-output check for the kernels that issue MFMAs through inline assembly (gemm_fat.hip, gemm_mid.hip,
gemm_kq.hip).

On gfx950 an MFMA that reads a VGPR fewer than two wait states after a VALU instruction wrote it sees the old value.
The compiler keeps that distance for MFMAs it knows; an inline-assembly MFMA is opaque to it.  This test compiles the
files to assembly (device pass only, no GPU needed) and fails if any MFMA source register is written by a VALU
instruction with fewer than two wait states in between (every instruction counts one, `s_nop N` counts N + 1)."""
import os
import re
import subprocess
import tempfile

import pytest

from vllm_amd import build as vbuild


def _regs(tok):
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def _violations(path):
    total, bad = 0, []
    hist = []  # (text, wait states it provides)
    for line in open(path):
        t = line.strip()
        if not t or t[0] in ";." or t.endswith(":"):
            continue
        op = t.split()[0]
        if op.startswith("v_mfma"):
            total += 1
            ops = [x.strip() for x in t[len(op):].split(",")]
            src = _regs(ops[1]) | _regs(ops[2])
            waited = 0
            for h, ws in reversed(hist[-3:]):
                hop = h.split()[0]
                if waited < 2 and hop.startswith("v_") and not hop.startswith(("v_mfma", "v_cmp")):
                    if _regs(h[len(hop):].split(",")[0].strip()) & src:
                        bad.append((h, t))
                waited += ws
        ws = 1
        if op == "s_nop":
            ws = int(t.split()[1]) + 1
        hist.append((t, ws))
    return total, bad


@pytest.mark.parametrize("src", ["gemm_fat.hip", "gemm_mid.hip", "gemm_kq.hip"])
def test_no_valu_write_right_before_an_asm_mfma(src):
    flags = [f for f in vbuild.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, src + ".s")
        cmd = [vbuild.hipcc_path()] + flags + ["-S", "--cuda-device-only", os.path.join(vbuild.CSRC, src), "-o", out]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        assert r.returncode == 0, r.stdout
        total, bad = _violations(out)
    assert total >= 1024, total  # the kernels are there (128 MFMAs per loop body and instantiation)
    assert not bad, bad[:5]
