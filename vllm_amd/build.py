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

# The 16-row kernel takes the values in front of its first loads as leading scalar arguments; with this option the first
# 14 dwords of a kernel's argument block arrive in SGPRs when a wavefront starts (gfx950 firmware loads them while it
# dispatches; the compiler keeps a fallback prologue that loads them itself).
FILE_FLAGS = {"gemm_decode.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=14"]}

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


def build(verbose: bool = False, extra_flags: tuple = (), check_hazards: bool = True) -> str:
    """`extra_flags`, e.g. ("-DW4A16_TUNING",), are added to every compile (the planner's tuning overrides).
    The files that issue MFMAs through inline assembly are compiled with -save-temps, and the device assembly their
    objects were assembled from is scanned for operand hazards (`check_mfma_hazards`) before the library is linked."""
    import shutil
    import tempfile
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    objs = []
    procs = []
    tmpdir = tempfile.mkdtemp(prefix="w4a16_build_")
    try:
        # compile translation units in parallel, then link
        for s in srcs:
            o = s[:-4] + ".o"
            objs.append(o)
            cmd = [hipcc_path()] + [f for f in HIPCC_FLAGS if f != "-shared"] + list(extra_flags) + FILE_FLAGS.get(os.path.basename(s), [])
            if os.path.basename(s) in ASM_MFMA_SOURCES:
                # intermediate files land beside the object: build it in the scratch folder and move it afterwards
                o_build = os.path.join(tmpdir, os.path.basename(o))
                cmd += ["-save-temps=obj", "-c", s, "-o", o_build]
            else:
                o_build = o
                cmd += ["-c", s, "-o", o]
            if verbose:
                print(" ".join(cmd), flush=True)
            procs.append((cmd, o_build, o, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        for cmd, o_build, o, p in procs:
            out, _ = p.communicate()
            if p.returncode != 0:
                raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
            if verbose and out.strip():
                print(out)
        scanned = 0
        for cmd, o_build, o, p in procs:
            if o_build == o:
                continue
            asm = o_build[:-2] + "-hip-amdgcn-amd-amdhsa-gfx950.s"
            if check_hazards:
                scanned += check_mfma_hazards(asm, verbose=verbose)
            shutil.move(o_build, o)
        if verbose and check_hazards:
            print(f"{scanned} inline-assembly MFMAs scanned in the assembly the objects were made from, no operand hazard")
        build.mfmas_scanned = scanned
    finally:
        shutil.rmtree(tmpdir, ignore_errors=True)
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed: %s\n%s" % (" ".join(cmd), r.stdout))
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


build.mfmas_scanned = 0

# ---------------------------------------------------------------------------------------------------------------
# MFMAs issued through inline assembly are opaque to the compiler's hazard logic.  On gfx950 an MFMA that reads a
# register fewer than two wait states after a VALU instruction wrote it sees the old value.  The kernels keep their
# operand writes far from the MFMAs that read them; the build reads the device assembly that each object file was
# assembled from (hipcc -save-temps) and fails on every MFMA whose A, B or C operand is written by a VALU instruction
# (v_accvgpr_write included) with fewer than two wait states in between, along any control-flow path: every
# instruction counts one wait state, `s_nop N` counts N + 1; a label's predecessors are the instruction above it
# (unless that is an unconditional branch or the end of the program) and every branch that names it.
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
    insts = []       # instruction texts in file order
    label_at = {}    # label -> index of the first instruction after it
    labels_before = {}  # instruction index -> labels directly in front of it
    pending = []
    for line in open(asm_path):
        t = line.split(";")[0].strip()
        if not t:
            continue
        if t.endswith(":"):
            pending.append(t[:-1])
            continue
        if t[0] == ".":
            # a new function starts a new instruction stream
            if t.startswith((".globl", ".section", ".text", ".type")):
                insts.append("s_endpgm")
            continue
        for lb in pending:
            label_at[lb] = len(insts)
        if pending:
            labels_before[len(insts)] = list(pending)
            pending = []
        insts.append(t)
    branches_to = {}  # instruction index of the target -> indices of the branches that name it
    for i, t in enumerate(insts):
        op = t.split()[0]
        if op.startswith(("s_cbranch", "s_branch")):
            tgt = t.split()[-1]
            if tgt in label_at:
                branches_to.setdefault(label_at[tgt], []).append(i)

    def preds(i):
        out = []
        if i > 0 and insts[i - 1].split()[0] not in ("s_branch", "s_endpgm", "s_setpc_b64"):
            out.append(i - 1)
        out.extend(branches_to.get(i, ()))
        return out

    def wait_states(t):
        parts = t.split()
        return int(parts[1], 0) + 1 if parts[0] == "s_nop" else 1

    total, bad = 0, []
    for i, t in enumerate(insts):
        op = t.split()[0]
        if not op.startswith("v_mfma"):
            continue
        total += 1
        ops = [x.strip() for x in t[len(op):].split(",")]
        src = set().union(*(_regs(o.split()[0]) for o in ops[1:4] if o))
        stack = [(p, 0) for p in preds(i)]
        seen = set()
        while stack:
            j, waited = stack.pop()
            if waited >= 2 or (j, waited) in seen:
                continue
            seen.add((j, waited))
            h = insts[j]
            hop = h.split()[0]
            if hop.startswith("v_") and not hop.startswith(("v_mfma", "v_cmp")):
                if _regs(h[len(hop):].split(",")[0].strip()) & src:
                    bad.append((h, t))
            w = waited + wait_states(h)
            stack.extend((p, w) for p in preds(j))
    return total, bad


def scan_sources(verbose: bool = False) -> int:
    """Compiles the inline-assembly MFMA sources exactly as build() does (same flags, -save-temps) into a scratch folder
    and scans the device assembly; for tests that must not replace the built library.  Returns the MFMA count."""
    import shutil
    import tempfile
    tmpdir = tempfile.mkdtemp(prefix="w4a16_scan_")
    try:
        procs = []
        for src in ASM_MFMA_SOURCES:
            o = os.path.join(tmpdir, src[:-4] + ".o")
            cmd = [hipcc_path()] + [f for f in HIPCC_FLAGS if f != "-shared"] + ["-save-temps=obj", "-c", os.path.join(CSRC, src), "-o", o]
            procs.append((cmd, o, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        total = 0
        for cmd, o, p in procs:
            out, _ = p.communicate()
            if p.returncode != 0:
                raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
            total += check_mfma_hazards(o[:-2] + "-hip-amdgcn-amd-amdhsa-gfx950.s", verbose=verbose)
        return total
    finally:
        shutil.rmtree(tmpdir, ignore_errors=True)


def check_mfma_hazards(asm_path: str, verbose: bool = False) -> int:
    """Scans one device assembly file written by the build and raises if an MFMA operand hazard is found; returns the
    number of MFMAs scanned."""
    total, bad = scan_mfma_hazards(asm_path)
    name = os.path.basename(asm_path)
    if verbose:
        print(f"{name}: {total} MFMAs scanned, {len(bad)} too close to an operand write")
    if total < 256:
        raise RuntimeError(f"{name}: only {total} MFMAs found in the compiler output; the scan is not seeing the kernels")
    if bad:
        raise RuntimeError(f"{name}: MFMA operand written fewer than two wait states before the MFMA: {bad[:3]}")
    return total


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, extra_flags=tuple(a for a in sys.argv[1:] if a.startswith("-D"))))
    print(build.mfmas_scanned, "inline-assembly MFMAs scanned, no operand hazard")
