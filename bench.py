#!/usr/bin/env python3
"""Benchmark of the W4A16 Marlin-surface GEMM on one MI355X.

Default workload (`config.workload`): the four Llama-3-8B decode linears
(K,N) = (4096,6144) qkv, (4096,4096) o, (4096,28672) gate_up, (14336,4096) down at M = 16,
GPTQ uint4b8, group 128, fp16, no act-order.  One "step" = those four GEMMs, each on a weight
copy that has not been touched for >= 512 MB of other traffic (cold for L2 and the 256 MB
Infinity Cache), inputs resident in HBM, replayed from a HIP graph so host launch cost is not in
the timed region.  `value` = algorithmic bytes of the step / time = GB/s.

Also printed in the same JSON line:
  roofline      algorithmic bytes per launch / average launch duration (HIP events on the launch
                stream) against the 8 TB/s HBM peak, for the decode kernel
  cpu_baseline  the oracle's dequantize + torch.matmul path on the host cores, bounded sample
  detail        per-shape µs / GB/s / TFLOP/s / roofline fractions (decode M in {1,4,16,64,256},
                prefill M = 4096 bf16 AWQ; the latter against the 2.5 PFLOP/s dense MFMA peak)
"""
import argparse
import json
import os
import sys
import time

import torch

HBM_PEAK_GBPS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0
LAYERS = {"qkv": (4096, 6144), "o": (4096, 4096), "gate_up": (4096, 28672), "down": (14336, 4096)}
GROUP = 128
TRAFFIC_PROFILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                               "decode_kernel_llama3_8b_M16_hbm_traffic_pmc.txt")


def measured_traffic_bytes_per_launch():
    """HBM bytes per launch of the headline step's GEMM kernel (average of the four launches at M = 16) as the counter
    summary under profiles/ states it (`traffic_bytes_per_launch = N`, from FETCH_SIZE and WRITE_SIZE scaled by a copy of
    known size); None when the summary is missing or carries no such line."""
    try:
        for line in open(TRAFFIC_PROFILE):
            if line.startswith("traffic_bytes_per_launch"):
                return float(line.split("=")[1].split()[0])
    except OSError:
        pass
    return None


def algorithmic_bytes(m, k, n, zp=False, act_order=False):
    b = k * n // 2 + (k // GROUP) * n * 2 + m * k * 2 + m * n * 2
    if zp:
        b += (k // GROUP) * n // 2
    if act_order:
        b += 2 * k * 4
    return b


# ------------------------------------------------------------------ synthetic layers (on the GPU)
def _weights(k, n, dtype, dev, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(k, n, generator=g) * 0.02).to(dtype).to(dev)


def make_gptq_layer(ops, k, n, dtype, dev, seed):
    """N(0, 0.02) weights, symmetric uint4b8 RTN, s = absmax/7 per (group, column)."""
    from vllm_amd.marlin_utils_test import marlin_quantize
    from vllm_amd.scalar_type import scalar_types
    w_ref, mq, ms, _, _, _ = marlin_quantize(_weights(k, n, dtype, dev, seed), scalar_types.uint4b8, GROUP, False,
                                             rule="absmax")
    return {"k": k, "n": n, "q": mq, "s": ms, "zp": torch.empty(0, dtype=torch.int32, device=dev), "w_deq": w_ref}


def make_awq_layer(ops, k, n, dtype, dev, seed):
    """N(0, 0.02) weights, asymmetric uint4 RTN from per-group min/max, uint4 zero points."""
    from vllm_amd.marlin_utils_test import awq_marlin_quantize
    from vllm_amd.scalar_type import scalar_types
    w_ref, mq, ms, mz = awq_marlin_quantize(_weights(k, n, dtype, dev, seed), scalar_types.uint4, GROUP, rule="absmax")
    return {"k": k, "n": n, "q": mq, "s": ms, "zp": mz, "w_deq": w_ref}


def clone_weights(layer, seed):
    """A distinct copy of the streamed operands (random nibbles, same scales): only used to rotate
    buffers so that no launch finds its weights in a cache."""
    g = torch.Generator(device=layer["q"].device).manual_seed(seed)
    q = torch.randint(-2**31, 2**31 - 1, layer["q"].shape, generator=g, device=layer["q"].device, dtype=torch.int32)
    return {**layer, "q": q, "s": layer["s"].clone(), "zp": layer["zp"].clone(), "w_deq": None}


def gemm(ops, wtype, a, layer, workspace):
    e = torch.empty(0, dtype=torch.int32, device=a.device)
    return ops.gptq_marlin_gemm(a, None, layer["q"], None, layer["s"], None, layer["zp"], layer.get("g_idx", e),
                                layer.get("perm", e), workspace, wtype, a.shape[0], layer["n"], layer["k"], True, False,
                                True, False)


def time_graph(fn_list, reps, warmup, stats=False, eager_all=True):
    """Capture `fn_list` (a list of zero-arg launch closures) into one HIP graph, replay it `warmup`
    times untimed and `reps` times, every replay between its own pair of events on the launch stream;
    returns the median seconds/replay (with stats=True: (median, min)).  Before the capture every closure
    (eager_all=False: only the first) runs once eagerly."""
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for f in (fn_list if eager_all else fn_list[:1]):  # eager warm-up (module load, allocator)
            f()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for f in fn_list:
                f()
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize()
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
        evs[0].record(stream)
        for i in range(reps):
            graph.replay()
            evs[i + 1].record(stream)
        torch.cuda.synchronize()
    ts = sorted(evs[i].elapsed_time(evs[i + 1]) * 1e-3 for i in range(reps))
    med = ts[len(ts) // 2] if len(ts) % 2 else 0.5 * (ts[len(ts) // 2 - 1] + ts[len(ts) // 2])
    return (med, ts[0]) if stats else med


def copies_needed(weight_bytes):
    return max(2, -(-512 * 2**20 // weight_bytes) + 1)


def bench_shape(ops, wtype, layer_fn, m, k, n, dtype, dev, workspace, launches=40, zp=False, probe=False):
    """Cold (rotating weight copies) time of one shape; returns dict.  probe=True is the same launch sequence for a
    profiler run (`--probe-shape`): one eager launch, then the same graph replays, no warm-weights leg."""
    base = layer_fn(k, n, dtype, dev, 1)
    wbytes = base["q"].numel() * 4
    ncopy = min(copies_needed(wbytes), 64)
    copies = [base] + [clone_weights(base, 100 + i) for i in range(ncopy - 1)]
    g = torch.Generator(device="cpu").manual_seed(2)
    a = torch.randn(m, k, generator=g).to(dtype).to(dev)
    out = gemm(ops, wtype, a, base, workspace)
    ref = a.float() @ base["w_deq"].float()
    err = float((out.float() - ref).abs().max() / ref.abs().max())
    mean_rel = float((out.float() - ref).abs().mean() / ref.abs().mean())
    fns = [(lambda c=copies[i % ncopy]: gemm(ops, wtype, a, c, workspace)) for i in range(max(launches, ncopy))]
    if probe:  # more replays, so that the two eager launches in front weigh nothing in a trace's average
        sec, sec_min = (t / len(fns) for t in time_graph(fns, reps=11, warmup=1, stats=True, eager_all=False))
        return {"m": m, "k": k, "n": n, "us": sec * 1e6, "us_min": sec_min * 1e6, "launches_timed": 11 * len(fns),
                "launches_total": 2 + 12 * len(fns), "max_rel_err": err}
    sec, sec_min = (t / len(fns) for t in time_graph(fns, reps=5, warmup=1, stats=True))
    warm = time_graph([lambda: gemm(ops, wtype, a, base, workspace)] * 20, reps=5, warmup=1) / 20
    by, fl = algorithmic_bytes(m, k, n, zp=zp), 2.0 * m * n * k
    del copies
    torch.cuda.empty_cache()
    return {"m": m, "k": k, "n": n, "us": sec * 1e6, "us_min": sec_min * 1e6, "us_warm": warm * 1e6,
            "launches_timed": 5 * len(fns), "GBps": by / sec / 1e9,
            "TFLOPs": fl / sec / 1e12, "hbm_frac": by / sec / 1e9 / HBM_PEAK_GBPS,
            "mfma_frac": fl / sec / 1e12 / MFMA_PEAK_TFLOPS, "max_rel_err": err,
            "mean_rel_err": mean_rel}


def make_gptq_actorder_layer(ops, k, n, dtype, dev, seed):
    """GPTQ desc_act layer: rows arrive in a seeded random order, g_idx[i] = group of arriving row i
    (as the reference's permute_rows, quant_utils.py:346-373); weights are repacked in group-sorted order."""
    from vllm_amd.marlin_utils_test import marlin_quantize
    from vllm_amd.scalar_type import scalar_types
    perm = torch.randperm(k, generator=torch.Generator(device="cpu").manual_seed(seed + 7))
    w_ref, mq, ms, g_idx, sort_idx, _ = marlin_quantize(_weights(k, n, dtype, dev, seed), scalar_types.uint4b8, GROUP,
                                                        True, perm, rule="absmax")
    return {"k": k, "n": n, "q": mq, "s": ms, "zp": torch.empty(0, dtype=torch.int32, device=dev), "w_deq": w_ref,
            "g_idx": g_idx, "perm": sort_idx}


def bench_repack(ops, dev):
    """Load-time repack of the four layers (GPTQ and AWQ checkpoint layouts -> Marlin layout): K*N/2 bytes read and
    K*N/2 written per call, against the HBM peak."""
    out = {}
    empty = torch.empty(0, dtype=torch.int32, device=dev)
    for name, (k, n) in LAYERS.items():
        g = torch.Generator(device=dev).manual_seed(9)
        gq = torch.randint(-2**31, 2**31 - 1, (k // 8, n), generator=g, device=dev, dtype=torch.int32)
        aq = torch.randint(-2**31, 2**31 - 1, (k, n // 8), generator=g, device=dev, dtype=torch.int32)
        for kind, fn in (("gptq", lambda: ops.gptq_marlin_repack(gq, empty, k, n, 4)),
                         ("awq", lambda: ops.awq_marlin_repack(aq, k, n, 4))):
            sec = time_graph([fn] * 8, reps=3, warmup=1) / 8
            by = k * n  # bytes moved: half read, half written
            out[f"{kind}_{name}"] = {"k": k, "n": n, "us": sec * 1e6, "GBps": by / sec / 1e9,
                                     "hbm_frac": by / sec / 1e9 / HBM_PEAK_GBPS}
            print(f"[detail] {kind} repack {name}: {sec * 1e6:.1f} us, {by / sec / 1e9:.0f} GB/s = "
                  f"{100 * by / sec / 1e9 / HBM_PEAK_GBPS:.1f}% HBM", file=sys.stderr, flush=True)
    return out


def bench_load_path(ops, dev):
    """Load-time preparation of one Llama-3-8B decoder layer's four linears from checkpoint tensors (AWQ layout: packed
    weights, packed zero points, scales): repack + scale permutation + zero-point conversion, all on the device; bytes =
    checkpoint bytes read + Marlin bytes written.  Also projected to the 32 layers of the model."""
    from vllm_amd.marlin_utils import awq_to_marlin_zero_points, marlin_permute_scales
    layers = []
    for name, (k, n) in LAYERS.items():
        g = torch.Generator(device=dev).manual_seed(11)
        qw = torch.randint(-2**31, 2**31 - 1, (k, n // 8), generator=g, device=dev, dtype=torch.int32)
        qz = torch.randint(-2**31, 2**31 - 1, (k // GROUP, n // 8), generator=g, device=dev, dtype=torch.int32)
        sc = torch.rand(k // GROUP, n, generator=g, device=dev).to(torch.bfloat16)
        layers.append((k, n, qw, qz, sc))

    def prepare():
        for k, n, qw, qz, sc in layers:
            ops.awq_marlin_repack(qw, k, n, 4)
            marlin_permute_scales(sc, k, n, GROUP)
            awq_to_marlin_zero_points(qz, k // GROUP, n, 4)
    sec = time_graph([prepare], reps=5, warmup=1)
    by = sum(2 * (qw.numel() * 4 + qz.numel() * 4 + sc.numel() * 2) for _, _, qw, qz, sc in layers)
    out = {"us_per_decoder_layer": sec * 1e6, "GBps": by / sec / 1e9, "hbm_frac": by / sec / 1e9 / HBM_PEAK_GBPS,
           "launches_per_decoder_layer": 12, "ms_for_32_layers": 32 * sec * 1e3}
    print(f"[detail] load path, one decoder layer (4 linears, AWQ checkpoint -> Marlin operands): {sec * 1e6:.1f} us, "
          f"{by / sec / 1e9:.0f} GB/s = {100 * out['hbm_frac']:.1f}% HBM; 32 layers: {32 * sec * 1e3:.2f} ms",
          file=sys.stderr, flush=True)
    return out


def bench_act_order(ops, wtype, dev, workspace):
    """GPTQ act-order case: down_proj (K=14336, N=4096), g128, desc_act, fp16, M in {1, 16, 512}."""
    k, n = LAYERS["down"]
    base = make_gptq_actorder_layer(ops, k, n, torch.float16, dev, 21)
    ncopy = copies_needed(base["q"].numel() * 4)
    copies = [base] + [clone_weights(base, 300 + i) for i in range(ncopy - 1)]
    out = {}
    for m in (1, 16, 512):
        a = torch.randn(m, k, generator=torch.Generator().manual_seed(4)).half().to(dev)
        call = lambda l: ops.gptq_marlin_gemm(a, None, l["q"], None, l["s"], None, l["zp"], base["g_idx"], base["perm"],
                                              workspace, wtype, m, n, k, True, False, True, False)
        res = call(base)
        ref = a.float() @ base["w_deq"].float()
        err = float((res.float() - ref).abs().max() / ref.abs().max())
        fns = [(lambda c=copies[i % ncopy]: call(c)) for i in range(max(16, ncopy))]
        sec = time_graph(fns, reps=3, warmup=1) / len(fns)
        by, fl = algorithmic_bytes(m, k, n, act_order=True), 2.0 * m * n * k
        out[f"down_M{m}"] = {"m": m, "k": k, "n": n, "us": sec * 1e6, "GBps": by / sec / 1e9, "TFLOPs": fl / sec / 1e12,
                             "hbm_frac": by / sec / 1e9 / HBM_PEAK_GBPS, "mfma_frac": fl / sec / 1e12 / MFMA_PEAK_TFLOPS,
                             "max_rel_err": err}
        print(f"[detail] act-order down M={m}: {sec * 1e6:.2f} us, {by / sec / 1e9:.0f} GB/s = "
              f"{100 * by / sec / 1e9 / HBM_PEAK_GBPS:.1f}% HBM, {fl / sec / 1e12:.1f} TFLOP/s, err {err:.1e}",
              file=sys.stderr, flush=True)
    return out


def bench_moe(ops, wtype, dev):
    """Mixtral-8x7B fused MoE (8 experts, hidden 4096, intermediate 14336, top-2), uint4b8 g128
    fp16, T in {16, 512, 4096}; one call = align + GEMM1 + SiLU-and-mul + GEMM2 + top-k sum."""
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    e, hid, inter, topk = 8, 4096, 14336, 2
    w13 = [make_gptq_layer(ops, hid, 2 * inter, torch.float16, dev, 40 + i) for i in range(e)]
    w2 = [make_gptq_layer(ops, inter, hid, torch.float16, dev, 60 + i) for i in range(e)]
    q1, s1 = torch.stack([l["q"] for l in w13]), torch.stack([l["s"] for l in w13])
    q2, s2 = torch.stack([l["q"] for l in w2]), torch.stack([l["s"] for l in w2])
    deq13 = [l["w_deq"] for l in w13]
    deq2 = [l["w_deq"] for l in w2]
    del w13, w2
    per_expert = (hid * 2 * inter + inter * hid) // 2 + ((hid // GROUP) * 2 * inter + (inter // GROUP) * hid) * 2
    out = {}
    for t in (16, 512, 4096):
        g = torch.Generator().manual_seed(5)
        x = (torch.randn(t, hid, generator=g)).half().to(dev)
        logits = torch.randn(t, e, generator=g).to(dev)
        tw, ti = torch.topk(torch.softmax(logits.float(), dim=-1), topk)
        tw = (tw / tw.sum(dim=-1, keepdim=True)).contiguous()
        ti = ti.to(torch.int32).contiguous()
        call = lambda: fused_marlin_moe(x, q1, q2, None, None, s1, s2, logits, tw, ti, quant_type_id=wtype.id,
                                        global_num_experts=e)
        res = call()
        # check the first 4 tokens against dequantised fp32 matmuls on the GPU
        ref = torch.zeros(4, hid, device=dev)
        for r in range(min(4, t)):
            for j in range(topk):
                ex = int(ti[r, j])
                h = (x[r].float() @ deq13[ex].float()).half()
                act = (torch.nn.functional.silu(h[:inter].float()).half() * h[inter:])
                ref[r] += float(tw[r, j]) * (act.float() @ deq2[ex].float()).half().float()
        err = float((res[:4].float() - ref[:min(4, t)]).abs().max() / ref.abs().max())
        sec = time_graph([call] * 4, reps=3, warmup=1) / 4
        hit = int(ti.unique().numel())
        by = hit * per_expert + t * hid * 2 * 2 + t * topk * (2 * inter + inter + hid) * 2 * 2
        fl = 2.0 * t * topk * (hid * 2 * inter + inter * hid)
        out[f"T{t}"] = {"tokens": t, "experts_hit": hit, "us": sec * 1e6, "GBps": by / sec / 1e9, "TFLOPs": fl / sec / 1e12,
                        "hbm_frac": by / sec / 1e9 / HBM_PEAK_GBPS, "mfma_frac": fl / sec / 1e12 / MFMA_PEAK_TFLOPS,
                        "max_rel_err_first4": err}
        print(f"[detail] mixtral moe T={t}: {sec * 1e6:.1f} us, {by / sec / 1e9:.0f} GB/s = "
              f"{100 * by / sec / 1e9 / HBM_PEAK_GBPS:.1f}% HBM, {fl / sec / 1e12:.1f} TFLOP/s = "
              f"{100 * fl / sec / 1e12 / MFMA_PEAK_TFLOPS:.1f}% MFMA, err {err:.1e}", file=sys.stderr, flush=True)
    return out


def bench_moe_fine_grained(dev):
    """A fine-grained MoE layer (128 experts, hidden 2048, intermediate 768, top-8: the shape of Qwen3-30B-A3B), uint4b8
    g128 fp16 with random codes and scales, T in {16, 512, 4096}; one call = fused_marlin_moe (parity is the tests'
    business; this row only times the launch sequence)."""
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    from vllm_amd.scalar_type import scalar_types
    e, hid, inter, topk = 128, 2048, 768, 8
    gen = torch.Generator(device=dev).manual_seed(3)
    codes = lambda *shape: torch.randint(-2**31, 2**31 - 1, shape, dtype=torch.int32, device=dev, generator=gen)
    scales = lambda *shape: (torch.rand(shape, device=dev, generator=gen) * 0.01 + 0.001).half()
    q1, s1 = codes(e, hid // 16, 2 * inter * 2), scales(e, hid // GROUP, 2 * inter)
    q2, s2 = codes(e, inter // 16, hid * 2), scales(e, inter // GROUP, hid)
    per_expert = (hid * 2 * inter + inter * hid) // 2 + ((hid // GROUP) * 2 * inter + (inter // GROUP) * hid) * 2
    out = {}
    for t in (16, 512, 4096):
        x = (torch.randn(t, hid, device=dev, generator=gen) / 10).half()
        logits = torch.randn(t, e, device=dev, generator=gen)
        tw, ti = torch.topk(torch.softmax(logits, dim=-1), topk)
        tw, ti = (tw / tw.sum(dim=-1, keepdim=True)).contiguous(), ti.to(torch.int32).contiguous()
        call = lambda: fused_marlin_moe(x, q1, q2, None, None, s1, s2, logits, tw, ti,
                                        quant_type_id=scalar_types.uint4b8.id, global_num_experts=e)
        call()
        sec = time_graph([call] * 4, reps=3, warmup=1) / 4
        hit = int(ti.unique().numel())
        by = hit * per_expert + t * hid * 2 * 2 + t * topk * (2 * inter + inter + hid) * 2 * 2
        fl = 2.0 * t * topk * (hid * 2 * inter + inter * hid)
        out[f"T{t}"] = {"tokens": t, "experts_hit": hit, "us": sec * 1e6, "GBps": by / sec / 1e9, "TFLOPs": fl / sec / 1e12,
                        "hbm_frac": by / sec / 1e9 / HBM_PEAK_GBPS, "mfma_frac": fl / sec / 1e12 / MFMA_PEAK_TFLOPS}
        print(f"[detail] 128-expert top-8 moe T={t}: {sec * 1e6:.1f} us, {by / sec / 1e9:.0f} GB/s = "
              f"{100 * by / sec / 1e9 / HBM_PEAK_GBPS:.1f}% HBM, {fl / sec / 1e12:.1f} TFLOP/s", file=sys.stderr, flush=True)
    return out


def bench_other_types(ops, dev, workspace):
    """The other weight types of the operator on gate_up (4096 x 28672): uint8b128, float8_e4m3fn, NVFP4, MXFP4 and
    uint4 with fp16 zero points, at M = 16 and M = 4096 (warm weights, random codes; parity is the tests' business)."""
    from vllm_amd import marlin_utils_fp4 as f4, marlin_utils_fp8 as f8
    from vllm_amd.marlin_utils import marlin_permute_scales
    from vllm_amd.scalar_type import scalar_types as st
    k, n = LAYERS["gate_up"]
    e = torch.empty(0, dtype=torch.int32, device=dev)
    torch.manual_seed(0)
    w16 = torch.randn(n, k, dtype=torch.float16, device=dev) * 0.02
    cases = {}
    q8 = torch.randint(-2**31, 2**31 - 1, (k // 16, 4 * n), dtype=torch.int32, device=dev)
    s8 = marlin_permute_scales((torch.rand(k // GROUP, n, device=dev) * 0.01).half(), k, n, GROUP)
    cases["uint8b128_f16_g128"] = (torch.float16, 1.0, lambda a: ops.gptq_marlin_gemm(
        a, None, q8, None, s8, None, None, e, e, workspace, st.uint8b128, a.shape[0], n, k))
    _, qf8, sf8 = f8.marlin_quant_fp8_torch(w16, GROUP)
    cases["fp8_e4m3fn_f16_g128"] = (torch.float16, 1.0, lambda a: ops.gptq_marlin_gemm(
        a, None, qf8, None, sf8, None, None, None, None, workspace, st.float8_e4m3fn, a.shape[0], n, k))
    _, qn, sn, gn = f4.rand_marlin_weight_nvfp4_like(w16, 16)
    gn = gn.view(1)
    cases["nvfp4_f16"] = (torch.float16, 0.5, lambda a: ops.gptq_marlin_gemm(
        a, None, qn, None, sn, gn, None, None, None, workspace, st.float4_e2m1f, a.shape[0], n, k))
    _, qm, sm = f4.rand_marlin_weight_mxfp4_like(w16.bfloat16(), 32)
    cases["mxfp4_bf16"] = (torch.bfloat16, 0.5, lambda a: ops.gptq_marlin_gemm(
        a, None, qm, None, sm, None, None, None, None, workspace, st.float4_e2m1f, a.shape[0], n, k))
    qh = torch.randint(-2**31, 2**31 - 1, (k // 16, 2 * n), dtype=torch.int32, device=dev)
    sh = marlin_permute_scales(torch.rand(k // 64, n, dtype=torch.float16, device=dev) * 0.01, k, n, 64)
    zh = marlin_permute_scales(torch.rand(k // 64, n, dtype=torch.float16, device=dev) * 8, k, n, 64)
    cases["uint4_fp16_zero_points_g64"] = (torch.float16, 0.5, lambda a: ops.gptq_marlin_gemm(
        a, None, qh, None, sh, None, zh, e, e, workspace, st.uint4, a.shape[0], n, k, is_zp_float=True))
    out = {}
    for label, (dt, bytes_per_weight, fn) in cases.items():
        for m in (16, 4096):
            a = torch.randn(m, k, device=dev).to(dt)
            reps = 20 if m == 16 else 4
            sec = time_graph([lambda: fn(a)] * reps, reps=5, warmup=1) / reps
            out[f"{label}_M{m}"] = {"us": sec * 1e6, "TFLOPs": 2.0 * m * n * k / sec / 1e12,
                                    "weight_GBps": k * n * bytes_per_weight / sec / 1e9}
            print(f"[detail] gate_up {label} M={m}: {sec * 1e6:.1f} us, {2.0 * m * n * k / sec / 1e12:.0f} TFLOP/s, "
                  f"{k * n * bytes_per_weight / sec / 1e9:.0f} GB/s of weights", file=sys.stderr, flush=True)
    return out


def bench_practical_peak(dev):
    """What a dense 16-bit GEMM reaches on this GPU through the vendor library (torch.matmul -> hipBLASLt), same harness
    (graph replays on rotating weight copies), on the four M = 4096 shapes: activations [4096, K] times a dense weight
    stored [K, N] ("nn") or [N, K] ("nt", multiplied as its transpose).  No dequantisation: the practical ceiling that the
    2.5 PFLOP/s peak translates to for a GEMM of these shapes."""
    out = {}
    m = 4096
    for dt_name, dt in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        for name, (k, n) in LAYERS.items():
            gen = torch.Generator(device=dev).manual_seed(17)
            a = torch.randn(m, k, device=dev, generator=gen).to(dt)
            ncopy = min(copies_needed(k * n * 2), 3)
            row = {}
            for layout in ("nn", "nt"):
                shape = (k, n) if layout == "nn" else (n, k)
                ws = [(torch.randn(shape, device=dev, generator=gen) * 0.02).to(dt) for _ in range(ncopy)]
                c = torch.empty(m, n, dtype=dt, device=dev)
                fns = [(lambda w=ws[i % ncopy]: torch.matmul(a, w if layout == "nn" else w.t(), out=c)) for i in range(8)]
                sec = time_graph(fns, reps=5, warmup=1) / len(fns)
                row[layout] = {"us": sec * 1e6, "TFLOPs": 2.0 * m * n * k / sec / 1e12}
                del ws, c
                torch.cuda.empty_cache()
            best = max(row.values(), key=lambda r: r["TFLOPs"])
            out[f"{name}_M4096_{dt_name}"] = {"m": m, "k": k, "n": n, "nn_us": row["nn"]["us"], "nn_TFLOPs": row["nn"]["TFLOPs"],
                                              "nt_us": row["nt"]["us"], "nt_TFLOPs": row["nt"]["TFLOPs"],
                                              "best_TFLOPs": best["TFLOPs"], "best_frac_of_peak": best["TFLOPs"] / MFMA_PEAK_TFLOPS}
            print(f"[detail] dense torch.matmul {name} M=4096 {dt_name}: nn {row['nn']['us']:.1f} us "
                  f"({row['nn']['TFLOPs']:.0f} TFLOP/s), nt {row['nt']['us']:.1f} us ({row['nt']['TFLOPs']:.0f} TFLOP/s)",
                  file=sys.stderr, flush=True)
    return out


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(m, budget_s=12.0, matmul_only_budget_s=4.0):
    """The oracle's CPU path (unpack GPTQ nibbles, (q-8)*s group-broadcast, torch.matmul in fp32) on the
    host cores: whole passes over the four layers at M=`m`, repeated until `budget_s` seconds of CPU work
    (`value`, median pass); then the matmul alone on cached dequantised weights (`matmul_only_*`)."""
    from oracle import gemm_ref as gr
    from oracle import quant_utils as qu
    torch.manual_seed(0)
    layers = {}
    for name, (k, n) in LAYERS.items():
        q = torch.randint(0, 16, (k, n), dtype=torch.int32)
        layers[name] = (qu.gptq_pack(q), (torch.rand(k // GROUP, n) * 0.01 + 0.005).half(), torch.randn(m, k).half())
        del q
    step_bytes = sum(algorithmic_bytes(m, k, n) for k, n in LAYERS.values())
    pass_s, t_total = [], 0.0
    while t_total < budget_s or len(pass_s) < 3:
        t_pass = 0.0
        for name, (packed, s, a) in layers.items():
            t0 = time.perf_counter()
            w = gr.dequant_checkpoint(packed, s, None, None, "gptq", torch.float16)
            out = gr.gemm_ref(a, w)
            t_pass += time.perf_counter() - t0
            del w, out
        pass_s.append(t_pass)
        t_total += t_pass
    med = sorted(pass_s)[len(pass_s) // 2]
    # matmul only: the largest layer's dequantised fp32 weights are 470 MB, so one layer at a time
    mm_s = {}
    for name, (packed, s, a) in layers.items():
        w = gr.dequant_checkpoint(packed, s, None, None, "gptq", torch.float16).float()
        af, reps, t_mm = a.float(), 0, 0.0
        torch.matmul(af, w)
        while t_mm < matmul_only_budget_s / 4 or reps < 3:
            t0 = time.perf_counter()
            torch.matmul(af, w)
            t_mm += time.perf_counter() - t0
            reps += 1
        mm_s[name] = t_mm / reps
        del w
    mm_step = sum(mm_s.values())
    return {"value": step_bytes / med / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{len(pass_s)} passes of dequantize (unpack, (q-8)*s) + fp32 matmul over the four layers at "
                      f"M={m}, {t_total:.1f} s of CPU time, median pass",
            "ms_per_step": med * 1e3, "ms_per_step_min": min(pass_s) * 1e3,
            "matmul_only_value": step_bytes / mm_step / 1e9, "matmul_only_ms_per_step": mm_step * 1e3,
            "host_cpus": os.cpu_count(), "cpu_model": _cpu_model()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--m", type=int, default=16, help="decode batch of the headline workload")
    ap.add_argument("--no-detail", action="store_true", help="skip the per-shape table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--table", type=str, default="", help="also write the detail table to this JSON file")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="counter-collection workload: plain device copies of known size (calibration) followed by "
                         "eager launches of the headline GEMMs on cold weights; prints no JSON line")
    ap.add_argument("--probe-shape", type=str, default="",
                    help="counter-collection workload for one shape, LAYER:M:KIND with KIND gptq_f16, gptq_act_f16 or awq_bf16 "
                         "(e.g. gate_up:4096:awq_bf16): a few eager launches on rotating weight copies; prints no JSON line")
    ap.add_argument("--probe-moe", type=int, default=0, metavar="T",
                    help="kernel-trace workload: ten calls of the Mixtral-8x7B-shaped fused MoE (8 experts, top-2, uint4b8 "
                         "g128 fp16, random codes) on T tokens; prints no JSON line")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)

    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.scalar_type import scalar_types
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    workspace = marlin_make_workspace_new(dev)
    m = args.m

    if args.probe_moe:
        from vllm_amd.fused_marlin_moe import fused_marlin_moe
        e, hid, inter, topk, t = 8, 4096, 14336, 2, args.probe_moe
        gen = torch.Generator(device=dev).manual_seed(3)
        codes = lambda *shape: torch.randint(-2**31, 2**31 - 1, shape, dtype=torch.int32, device=dev, generator=gen)
        scales = lambda *shape: (torch.rand(shape, device=dev, generator=gen) * 0.01 + 0.001).half()
        q1, s1 = codes(e, hid // 16, 2 * inter * 2), scales(e, hid // GROUP, 2 * inter)
        q2, s2 = codes(e, inter // 16, hid * 2), scales(e, inter // GROUP, hid)
        x = (torch.randn(t, hid, device=dev, generator=gen) / 10).half()
        logits = torch.randn(t, e, device=dev, generator=gen)
        tw, ti = torch.topk(torch.softmax(logits, dim=-1), topk)
        tw, ti = (tw / tw.sum(dim=-1, keepdim=True)).contiguous(), ti.to(torch.int32).contiguous()
        call = lambda: fused_marlin_moe(x, q1, q2, None, None, s1, s2, logits, tw, ti, quant_type_id=scalar_types.uint4b8.id,
                                        global_num_experts=e)
        sec = time_graph([call] * 4, reps=5, warmup=1, eager_all=False) / 4
        print(f"probe-moe done: 1 eager call + 6 replays of 4 calls at T={t}, {int(ti.unique().numel())} experts hit, "
              f"{sec * 1e6:.1f} us per call (median replay)", file=sys.stderr)
        return
    if args.probe_shape:
        # the launch sequence of the `detail` row of the same shape (graph replays on rotating weight copies), so that a
        # kernel trace of this run averages over the launches that row times
        name, pm, kind = args.probe_shape.split(":")
        k, n = LAYERS[name]
        pm = int(pm)
        if kind == "awq_bf16":
            r = bench_shape(ops, scalar_types.uint4, lambda *a: make_awq_layer(ops, *a), pm, k, n, torch.bfloat16, dev,
                            workspace, launches=8 if pm >= 2048 else 40, zp=True, probe=True)
        elif kind == "gptq_act_f16":
            r = bench_shape(ops, scalar_types.uint4b8, lambda *a: make_gptq_actorder_layer(ops, *a), pm, k, n, torch.float16,
                            dev, workspace, launches=16, probe=True)
        else:
            r = bench_shape(ops, scalar_types.uint4b8, lambda *a: make_gptq_layer(ops, *a), pm, k, n, torch.float16, dev,
                            workspace, launches=8 if pm >= 2048 else 40, probe=True)
        print(f"probe-shape done: {name} M={pm} {kind}: {r['launches_total']} launches, the last {r['launches_timed']} "
              f"event-timed at {r['us']:.2f} us per launch (median replay; min {r['us_min']:.2f})", file=sys.stderr)
        return

    # ---- headline: one step = the four decode GEMMs, weights rotated over `nsets` full sets
    step_wbytes = sum(k * n // 2 for k, n in LAYERS.values())
    nsets = copies_needed(step_wbytes)
    base = {name: make_gptq_layer(ops, k, n, torch.float16, dev, 10 + i) for i, (name, (k, n)) in enumerate(LAYERS.items())}
    sets = [base] + [{name: clone_weights(l, 1000 * s + i) for i, (name, l) in enumerate(base.items())}
                     for s in range(1, nsets)]
    acts = {name: torch.randn(m, k, generator=torch.Generator().manual_seed(3)).half().to(dev)
            for name, (k, n) in LAYERS.items()}
    # correctness guard of the timed path (dequantised fp32 matmul on the GPU)
    errs = {}
    for name, l in base.items():
        out = gemm(ops, scalar_types.uint4b8, acts[name], l, workspace)
        ref = acts[name].float() @ l["w_deq"].float()
        errs[name] = float((out.float() - ref).abs().max() / ref.abs().max())
    assert max(errs.values()) < 2e-2, errs

    if args.pmc_probe:
        # 3 copies of 256 MiB (reads 256 MiB, writes 256 MiB each), then 3 steps on cold weight sets
        src = torch.empty(64 * 2**20, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        for i in range(1, 4):
            for name in LAYERS:
                gemm(ops, scalar_types.uint4b8, acts[name], sets[i % nsets][name], workspace)
        torch.cuda.synchronize()
        print("pmc-probe done: 3 x 256 MiB copy, 3 x (qkv, o, gate_up, down) at M=%d" % m, file=sys.stderr)
        return

    def step(i):
        s = sets[i % nsets]
        for name in LAYERS:
            gemm(ops, scalar_types.uint4b8, acts[name], s[name], workspace)

    # Exactly `--steps` steps are timed: whole graphs of `nsets` steps (one per weight set) plus, when `--steps` is
    # not a multiple of nsets, one shorter graph for the remainder.  Warm-up replays the same way.
    def capture(nsteps, stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(nsteps):
                step(i)
        return graph

    def run(nsteps, full, parts):
        for _ in range(nsteps // nsets):
            full.replay()
        if nsteps % nsets:
            parts[nsteps % nsets].replay()

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for i in range(nsets):
            step(i)
        torch.cuda.synchronize()
        full = capture(nsets, stream)
        parts = {r: capture(r, stream) for r in {args.steps % nsets, args.warmup % nsets} if r}
        run(args.warmup, full, parts)
        torch.cuda.synchronize()
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record(stream)
        run(args.steps, full, parts)
        t1.record(stream)
        torch.cuda.synchronize()
    timed_steps = args.steps
    sec_per_step = t0.elapsed_time(t1) * 1e-3 / max(timed_steps, 1)
    step_bytes = sum(algorithmic_bytes(m, k, n) for k, n in LAYERS.values())
    value = step_bytes / sec_per_step / 1e9
    launches = 4 * timed_steps
    avg_launch_s = sec_per_step / 4

    result = {
        "metric": "W4A16 GEMM \u00b5s + %HBM roofline (M\u226416), %MFMA peak (M=4096), Llama-3-8B shapes",
        "metric_detail": "value = algorithmic HBM bytes per second over one decode step = the four Llama-3-8B linears "
                         "(qkv, o, gate_up, down) at M=16; per-shape microseconds and roofline fractions are in "
                         "`detail` and `summary`",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": timed_steps, "warmup": args.warmup,
        "ms_per_step": sec_per_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"llama3-8b decode linears M={m}, GPTQ uint4b8 g128 fp16, no act-order, cold weights",
                   "shapes_KN": list(LAYERS.values()), "M": m, "weight_sets_rotated": nsets,
                   "timing": "HIP graph replay between two events on the launch stream"},
        "roofline": {"bound": "hbm", "achieved": step_bytes / 4 / avg_launch_s / 1e9, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": step_bytes / 4 / avg_launch_s / 1e9 / HBM_PEAK_GBPS, "traffic": measured_traffic_bytes_per_launch() if m == 16 else None,
                     "kernel": "w4a16::decode_kernel<f16, no-zp, grouped> (64- and 128-column instantiations, "
                               "average over the step's four launches)", "launches": launches,
                     "avg_launch_us": avg_launch_s * 1e6, "algorithmic_bytes_per_launch": step_bytes / 4},
        "us_per_gemm_avg": avg_launch_s * 1e6,
        "max_rel_err_vs_fp32": errs,
    }
    del sets, base
    torch.cuda.empty_cache()

    if not args.no_detail:
        detail = {"decode_fp16_gptq": {}, "prefill_bf16_awq": {}}  # + act_order_fp16_gptq, mixtral_moe_fp16_gptq
        for name, (k, n) in LAYERS.items():
            for mm in (1, 4, 16, 64, 256, 1024):
                r = bench_shape(ops, scalar_types.uint4b8, lambda *a: make_gptq_layer(ops, *a), mm, k, n,
                                torch.float16, dev, workspace)
                detail["decode_fp16_gptq"][f"{name}_M{mm}"] = r
                print(f"[detail] {name} M={mm}: {r['us']:.2f} us cold ({r['us_warm']:.2f} warm), "
                      f"{r['GBps']:.0f} GB/s = {100 * r['hbm_frac']:.1f}% HBM, {r['TFLOPs']:.1f} TFLOP/s",
                      file=sys.stderr, flush=True)
        for name, (k, n) in LAYERS.items():
            r = bench_shape(ops, scalar_types.uint4, lambda *a: make_awq_layer(ops, *a), 4096, k, n, torch.bfloat16,
                            dev, workspace, launches=8, zp=True)
            detail["prefill_bf16_awq"][f"{name}_M4096"] = r
            print(f"[detail] {name} M=4096 bf16 awq: {r['us']:.1f} us, {r['TFLOPs']:.1f} TFLOP/s = "
                  f"{100 * r['mfma_frac']:.1f}% MFMA peak", file=sys.stderr, flush=True)
        detail["act_order_fp16_gptq"] = bench_act_order(ops, scalar_types.uint4b8, dev, workspace)
        torch.cuda.empty_cache()
        detail["mixtral_moe_fp16_gptq"] = bench_moe(ops, scalar_types.uint4b8, dev)
        torch.cuda.empty_cache()
        detail["fine_grained_moe_fp16_gptq"] = bench_moe_fine_grained(dev)
        torch.cuda.empty_cache()
        detail["repack"] = bench_repack(ops, dev)
        detail["load_path"] = bench_load_path(ops, dev)
        torch.cuda.empty_cache()
        detail["other_weight_types_gate_up_warm"] = bench_other_types(ops, dev, workspace)
        result["detail"] = detail
        result["summary"] = {
            "decode_fp16_gptq_us": {k: round(v["us"], 2) for k, v in detail["decode_fp16_gptq"].items()},
            "decode_fp16_gptq_hbm_frac": {k: round(v["hbm_frac"], 3) for k, v in detail["decode_fp16_gptq"].items()},
            "prefill_bf16_awq_us": {k: round(v["us"], 1) for k, v in detail["prefill_bf16_awq"].items()},
            "prefill_bf16_awq_mfma_frac": {k: round(v["mfma_frac"], 3) for k, v in detail["prefill_bf16_awq"].items()},
        }
        # the M = 4096 half of the metric: the prefill kernel on the four bf16 AWQ layers, against the dense MFMA peak
        pf = detail["prefill_bf16_awq"]
        pf_flops = sum(2.0 * v["m"] * v["n"] * v["k"] for v in pf.values())
        pf_sec = sum(v["us"] for v in pf.values()) * 1e-6
        result["roofline_mfma"] = {
            "bound": "mfma", "achieved": pf_flops / pf_sec / 1e12, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": pf_flops / pf_sec / 1e12 / MFMA_PEAK_TFLOPS, "traffic": None,
            "kernel": "w4a16::fat_kernel<bf16, zero points, grouped> (qkv also runs its last 512-column strips on "
                      "w4a16::mid_kernel)", "launches": sum(v["launches_timed"] for v in pf.values()),
            "flops_per_launch_avg": pf_flops / 4, "avg_launch_us": pf_sec / 4 * 1e6,
            "workload": "llama3-8b linears at M=4096, bf16, AWQ uint4 + uint4 zero points g128 (qkv, o, gate_up, down), "
                        "time-weighted over the four layers",
            "per_layer_frac": {k: round(v["mfma_frac"], 3) for k, v in pf.items()}}
        pk = bench_practical_peak(dev)
        result["practical_peak"] = {
            "what": "dense 16-bit GEMM through torch.matmul (hipBLASLt), no dequantisation, same shapes and harness; "
                    "nn = weight stored [K, N], nt = stored [N, K]",
            "unit": "TFLOP/s", "per_shape": pk,
            "bf16_time_weighted_TFLOPs": sum(2.0 * v["m"] * v["n"] * v["k"] for kk, v in pk.items() if kk.endswith("bf16")) /
                                         sum(min(v["nn_us"], v["nt_us"]) for kk, v in pk.items() if kk.endswith("bf16")) / 1e6,
            "w4a16_bf16_awq_vs_dense_bf16": {name: round(pf[f"{name}_M4096"]["TFLOPs"] / pk[f"{name}_M4096_bf16"]["best_TFLOPs"], 3)
                                             for name in LAYERS}}
        if args.table:
            with open(args.table, "w") as f:
                json.dump(detail, f, indent=1)

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(m)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
