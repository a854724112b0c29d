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
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, extra_flags=tuple(a for a in sys.argv[1:] if a.startswith("-D"))))
