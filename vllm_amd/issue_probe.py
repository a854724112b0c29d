"""MFMA / VALU issue micro-benchmark (`bench.py --issue-probe`): the measurement behind the prefill kernels' bound.

Every wavefront loops over independent in-place v_mfma_f32_16x16x32_f16 (32 accumulators) with NV v_and_or_b32 after
each MFMA, independent of each other or chained; one workgroup per compute unit with 4 or 8 wavefronts (one or two per
SIMD); operands random fp16 in [-2, 2) or all zero.  Printed per case: time per MFMA and SIMD, and the MFMA rate of the
whole chip as TFLOP/s (16384 flop per MFMA)."""
import ctypes
import os

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libw4a16_probe.so")


def run(dev, iters: int = 2000) -> list[dict]:
    lib = ctypes.CDLL(LIB_PATH)
    lib.w4a16_issue_probe.restype = ctypes.c_float
    lib.w4a16_issue_probe.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_int]
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    g = torch.Generator().manual_seed(1)
    rnd = (torch.rand(8192, generator=g) * 4 - 2).half().view(torch.int32).to(dev)       # 4096 dwords of fp16 pairs
    zero = torch.zeros(4096, dtype=torch.int32, device=dev)
    out = torch.empty(cus * 512, dtype=torch.float32, device=dev)
    rows = []
    torch.cuda.synchronize()
    for data, src in (("zeros", zero), ("random", rnd)):
        for waves in (4, 8):
            for dep in (0, 1):
                for nv in range(7):
                    if dep and nv == 0:
                        continue
                    if data == "zeros" and (nv > 0):
                        continue
                    ms = lib.w4a16_issue_probe(src.data_ptr(), out.data_ptr(), cus, waves, nv, dep, iters)
                    assert ms > 0, ms
                    per_simd_ns = ms * 1e6 / (iters * 32 * waves / 4)
                    tflops = cus * waves * iters * 32 * 16384.0 / (ms * 1e-3) / 1e12
                    rows.append(dict(data=data, waves_per_simd=waves // 4, valu_per_mfma=nv, dependent=bool(dep),
                                     ns_per_mfma_per_simd=per_simd_ns, tflops=tflops))
                    print(f"{data:6s} waves/SIMD={waves // 4} VALU/MFMA={nv} {'chained' if dep else 'independent'}: "
                          f"{per_simd_ns:6.2f} ns per MFMA and SIMD, {tflops:7.0f} TFLOP/s", flush=True)
    return rows
