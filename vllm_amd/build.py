"""Compile the gfx950 HIP sources into vllm_amd/libw4a16_gfx950.so (in-tree).

Usage: python -m vllm_amd.build
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libw4a16_gfx950.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

SOURCES = ["c_api.hip", "repack.hip", "gemm.hip", "gemm_skinny.hip", "gemm_decode.hip", "gemm_fat.hip", "gemm_mid.hip", "gemm_kq.hip", "moe_glue.hip"]

# packed-fp32 VALU forms are switched off for every device compile of this library
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build(verbose: bool = False, extra_flags: tuple = ()) -> str:
    """`extra_flags`, e.g. ("-DW4A16_TUNING",), are added to every compile (the planner's tuning overrides)."""
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    objs = []
    procs = []
    # compile translation units in parallel, then link
    for s in srcs:
        o = s[:-4] + ".o"
        objs.append(o)
        cmd = [hipcc_path()] + [f for f in HIPCC_FLAGS if f != "-shared"] + list(extra_flags) + ["-c", s, "-o", o]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for cmd, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
        if verbose and out.strip():
            print(out)
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed: %s\n%s" % (" ".join(cmd), r.stdout))
    os.replace(tmp, LIB_PATH)
    build_probe()
    return LIB_PATH


def build_probe() -> str:
    """The MFMA / VALU issue micro-benchmark of `bench.py --issue-probe`: a library of its own, not linked into the product."""
    out = os.path.join(HERE, "libw4a16_probe.so")
    cmd = [hipcc_path()] + HIPCC_FLAGS + [os.path.join(CSRC, "issue_probe.hip"), "-o", out + ".tmp"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), r.stdout))
    os.replace(out + ".tmp", out)
    return out


# ---------------------------------------------------------------------------------------------------------------
# MFMAs issued through inline assembly (gemm_fat.hip, gemm_mid.hip, gemm_kq.hip) are opaque to the compiler's hazard
# logic.  On gfx950 an MFMA that reads a register fewer than two wait states after a VALU instruction wrote it sees
# the old value.  The kernels keep their operand writes far from the MFMAs that read them; this check compiles the
# files to assembly (device pass only, no GPU needed) and reports every MFMA whose A, B or C operand is written by a
# VALU instruction (v_accvgpr_write included) with fewer than two wait states in between (every instruction counts
# one, `s_nop N` counts N + 1).
ASM_MFMA_SOURCES = ["gemm_fat.hip", "gemm_mid.hip", "gemm_kq.hip"]


def _regs(tok: str) -> set:
    import re
    m = re.match(r"([va])\[(\d+):(\d+)\]", tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.match(r"([va])(\d+)$", tok)
    return {(m.group(1), int(m.group(2)))} if m else set()


def scan_mfma_hazards(asm_path: str):
    """Returns (number of MFMAs seen, list of (writer, mfma) instruction pairs that are too close)."""
    total, bad = 0, []
    hist = []  # (instruction text, wait states it provides)
    for line in open(asm_path):
        t = line.strip()
        if not t or t[0] in ";." or t.endswith(":"):
            continue
        op = t.split()[0]
        if op.startswith("v_mfma"):
            total += 1
            ops = [x.strip() for x in t[len(op):].split(",")]
            src = set().union(*(_regs(o.split()[0]) for o in ops[1:4] if o))
            waited = 0
            for h, ws in reversed(hist):
                if waited >= 2:
                    break
                hop = h.split()[0]
                if hop.startswith("v_") and not hop.startswith(("v_mfma", "v_cmp")):
                    if _regs(h[len(hop):].split(",")[0].strip()) & src:
                        bad.append((h, t))
                waited += ws
        hist.append((t, int(t.split()[1]) + 1 if op == "s_nop" else 1))
        if len(hist) > 8:
            hist.pop(0)
    return total, bad


def check_mfma_hazards(verbose: bool = False) -> int:
    """Compiles the inline-assembly MFMA kernels to assembly and raises if a hazard is found; returns the MFMA count."""
    import tempfile
    flags = [f for f in HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    seen = 0
    with tempfile.TemporaryDirectory() as tmp:
        procs = []
        for src in ASM_MFMA_SOURCES:
            out = os.path.join(tmp, src + ".s")
            cmd = [hipcc_path()] + flags + ["-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", out]
            procs.append((src, out, cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        for src, out, cmd, p in procs:
            log, _ = p.communicate()
            if p.returncode != 0:
                raise RuntimeError("hipcc -S failed: %s\n%s" % (" ".join(cmd), log))
            total, bad = scan_mfma_hazards(out)
            if verbose:
                print(f"{src}: {total} MFMAs scanned, {len(bad)} too close to an operand write")
            if total < 1024:
                raise RuntimeError(f"{src}: only {total} MFMAs found in the compiler output; the scan is not seeing the kernels")
            if bad:
                raise RuntimeError(f"{src}: MFMA operand written fewer than two wait states before the MFMA: {bad[:3]}")
            seen += total
    return seen


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, extra_flags=tuple(a for a in sys.argv[1:] if a.startswith("-D"))))
    if "--check-hazards" in sys.argv:
        print(check_mfma_hazards(verbose=True), "MFMAs scanned, no operand hazard")
