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
                                      ctypes.c_int, ctypes.c_int, ctypes.c_int]
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
                    ms = lib.w4a16_issue_probe(src.data_ptr(), out.data_ptr(), cus, waves, nv, dep, iters, 0)
                    assert ms > 0, ms
                    per_simd_ns = ms * 1e6 / (iters * 32 * waves / 4)
                    tflops = cus * waves * iters * 32 * 16384.0 / (ms * 1e-3) / 1e12
                    rows.append(dict(data=data, waves_per_simd=waves // 4, valu_per_mfma=nv, dependent=bool(dep),
                                     ns_per_mfma_per_simd=per_simd_ns, tflops=tflops))
                    print(f"{data:6s} waves/SIMD={waves // 4} VALU/MFMA={nv} {'chained' if dep else 'independent'}: "
                          f"{per_simd_ns:6.2f} ns per MFMA and SIMD, {tflops:7.0f} TFLOP/s", flush=True)
    # the same VALU work per flop on v_mfma_f32_32x32x16_f16 (half as many, twice as long MFMAs)
    for waves in (4, 8):
        for nv in (0, 2, 4, 6, 8, 12):
            ms = lib.w4a16_issue_probe(rnd.data_ptr(), out.data_ptr(), cus, waves, nv, 0, iters, 1)
            assert ms > 0, ms
            tflops = cus * waves * iters * 16 * 32768.0 / (ms * 1e-3) / 1e12
            rows.append(dict(data="random", mfma="32x32x16", waves_per_simd=waves // 4, valu_per_mfma=nv, dependent=False,
                             ns_per_mfma_per_simd=ms * 1e6 / (iters * 16 * waves / 4), tflops=tflops))
            print(f"random 32x32x16 waves/SIMD={waves // 4} VALU/MFMA={nv} (= {nv / 2:g} per 16384 flop) independent: "
                  f"{tflops:7.0f} TFLOP/s", flush=True)
    return rows


def stream_floor(dev, layers: dict, time_graph, copies_needed) -> dict:
    """Streaming floor of the 16-row GEMM kernels (`bench.py --stream-probe`): a kernel with decode_kernel's work
    decomposition and loads that computes nothing, on weight buffers not touched for >= 512 MB of other traffic, replayed
    from a HIP graph like the GEMM rows of the bench table.  Per layer the best of the launch shapes the planner can
    choose from (tile width 64 / 128, K splits that keep the grid within one workgroup per compute unit, 3 or 6 stages in
    flight)."""
    lib = ctypes.CDLL(LIB_PATH)
    lib.w4a16_stream_probe.restype = ctypes.c_int
    lib.w4a16_stream_probe.argtypes = [ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 5 + [ctypes.c_void_p]
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.zeros(512, dtype=torch.int32, device=dev)
    out = {}
    for name, (k, n) in layers.items():
        nbytes = k * n // 2
        ncopy = copies_needed(nbytes)
        bufs = [torch.randint(-2**31, 2**31 - 1, (k // 16, 2 * n), dtype=torch.int32, device=dev) for _ in range(ncopy)]
        best = None
        for tn in (128, 64):
            for splits in (1, 2, 3, 4, 6, 8):
                if splits > 1 and (n // tn) * splits > cus:
                    continue
                if k // 64 // splits < 8:
                    continue
                for depth in (3, 6):
                    def launch(b):
                        rc = lib.w4a16_stream_probe(b.data_ptr(), sink.data_ptr(), k, n, tn, splits, depth,
                                                    torch.cuda.current_stream(dev).cuda_stream)
                        assert rc == 0, rc
                    fns = [(lambda b=bufs[i % ncopy]: launch(b)) for i in range(max(40, ncopy))]
                    us = time_graph(fns, reps=3, warmup=1) / len(fns) * 1e6
                    if best is None or us < best["us"]:
                        best = dict(us=us, tile_columns=tn, k_splits=splits, stages_in_flight=depth,
                                    GBps=nbytes / us / 1e3)
        # the same launch shape with every workgroup also storing 2 KB: what it costs a kernel to write at all
        big_sink = torch.zeros((n // best["tile_columns"]) * best["k_splits"] * 512, dtype=torch.int32, device=dev)

        def launch_w(b):
            rc = lib.w4a16_stream_probe(b.data_ptr(), big_sink.data_ptr(), k, n, best["tile_columns"], -best["k_splits"],
                                        best["stages_in_flight"], torch.cuda.current_stream(dev).cuda_stream)
            assert rc == 0, rc
        fns = [(lambda b=bufs[i % ncopy]: launch_w(b)) for i in range(max(40, ncopy))]
        best["us_with_stores"] = time_graph(fns, reps=3, warmup=1) / len(fns) * 1e6
        out[name] = best
        print(f"stream floor {name} ({k} x {n}, {nbytes / 1e6:.1f} MB): {best['us']:.2f} us = {best['GBps']:.0f} GB/s "
              f"(tiles of {best['tile_columns']} columns, {best['k_splits']} K splits, {best['stages_in_flight']} stages in "
              f"flight); {best['us_with_stores']:.2f} us when every workgroup also stores 2 KB", flush=True)
        del bufs
        torch.cuda.empty_cache()
    return out
