"""Every benchmark configuration at its stated shape, under a checker.

  config 1/2  Llama-3-8B linears (qkv, o, gate_up, down), GPTQ uint4b8 g128 fp16 (s = absmax/7), M in {1,4,16,64,256}
  config 3    the same four layers at M = 4096, bf16, AWQ-style uint4 + uint4 zero points from per-group min/max
  config 4    act-order down_proj (K = 14336, desc_act), M in {1,16,512}, is_k_full True and False
  config 5    Mixtral-8x7B fused MoE, 8 experts, top-2, T in {16,512,4096}

Layers are quantised on the GPU by vllm_amd.marlin_utils_test (the CPU oracle would need minutes per layer) and go
through the checkpoint packing and the repack kernels.  Two checks per case:
  * one-hot rows: 64 activation rows e_k; output row must equal, bit for bit, row k of the CPU ORACLE's dequantised
    weights, obtained by running the oracle's quantizer on the sampled groups only (so the GPU quantizer, packing,
    repack, scale / zero-point conversion and the kernel are all inside the comparison);
  * random activations against an fp32 matmul of the dequantised weights on the GPU, per 512-column strip:
    max|d| / max|ref| <= 2e-2 (fp16) / 4e-2 (bf16) and the reference's mean-relative gate 0.04
    (tests/kernels/quantization/test_marlin_gemm.py:359-361); MoE: atol 5e-2 (tests/kernels/moe/test_moe.py:744).
"""
import pytest
import torch

from oracle import quant_utils as qu
from oracle import scalar_types as ost

pytestmark = pytest.mark.gpu

LAYERS = {"qkv": (4096, 6144), "o": (4096, 4096), "gate_up": (4096, 28672), "down": (14336, 4096)}
GROUP = 128
_cache: dict = {}


def _weights(k, n, dtype, dev, seed):
    return (torch.randn(k, n, generator=torch.Generator().manual_seed(seed)) * 0.02).to(dtype).to(dev)


def _layer(kind, name, dev):
    """kind: gptq_f16 | awq_bf16 | act_f16 -> dict with the op's operands, the source weights and w_ref (arrival order)."""
    key = (kind, name)
    if key in _cache:
        return _cache[key]
    _cache.clear()                      # one layer resident at a time
    torch.cuda.empty_cache()
    from vllm_amd.marlin_utils_test import awq_marlin_quantize, marlin_quantize
    from vllm_amd.scalar_type import scalar_types as st
    k, n = LAYERS[name]
    e = torch.empty(0, dtype=torch.int32, device=dev)
    seed = 1000 + sorted(LAYERS).index(name)
    if kind == "awq_bf16":
        w = _weights(k, n, torch.bfloat16, dev, seed)
        w_ref, mq, ms, mz = awq_marlin_quantize(w, st.uint4, GROUP, rule="absmax")
        L = dict(w=w, w_ref=w_ref, q=mq, s=ms, zp=mz, g_idx=e, perm=e, wtype=st.uint4, rand_perm=None)
    else:
        w = _weights(k, n, torch.float16, dev, seed)
        act = kind == "act_f16"
        perm = torch.randperm(k, generator=torch.Generator().manual_seed(77)) if act else None
        w_ref, mq, ms, g_idx, sort_idx, rand_perm = marlin_quantize(w, st.uint4b8, GROUP, act, perm, rule="absmax")
        L = dict(w=w, w_ref=w_ref, q=mq, s=ms, zp=e, g_idx=g_idx, perm=sort_idx, wtype=st.uint4b8,
                 rand_perm=rand_perm if act else None)
    L.update(k=k, n=n, dtype=w.dtype, kind=kind)
    _cache[key] = L
    return L


def _gemm(L, a, ws, is_k_full=True):
    import vllm_amd.ops as ops
    return ops.gptq_marlin_gemm(a, None, L["q"], None, L["s"], None, L["zp"], L["g_idx"], L["perm"], ws, L["wtype"],
                                a.shape[0], L["n"], L["k"], is_k_full, False, True, False)


def _oracle_rows(L, rows):
    """Row i (arrival order) of the CPU oracle's dequantised weights, for the sampled rows: the oracle's quantizer runs
    on the 128-row group of the source weights that holds the row."""
    out = {}
    by_group = {}
    for i in rows:
        src = int(L["rand_perm"][i]) if L["rand_perm"] is not None else i
        by_group.setdefault(src // GROUP, []).append((i, src % GROUP))
    for g, items in by_group.items():
        wg = L["w"][g * GROUP:(g + 1) * GROUP].cpu()
        if L["kind"] == "awq_bf16":
            w_ref = qu.quantize_minmax_zp(wg, GROUP)[0]
        else:
            w_ref = qu.quantize_absmax7(wg, GROUP)[0]
        for i, r in items:
            out[i] = w_ref[r]
    return out


def _sample_rows(k):
    g = torch.Generator().manual_seed(k)
    groups = torch.randperm(k // GROUP, generator=g)[:6].tolist() + [0, k // GROUP - 1]
    rows = []
    for gi in groups:
        rows += [gi * GROUP + int(r) for r in torch.randperm(GROUP, generator=g)[:8]]
    rows[0], rows[-1] = 0, k - 1
    return rows                                                           # 64 rows in 8 groups


def _check_one_hot(L, m, ws, dev, is_k_full=True):
    rows = _sample_rows(L["k"])
    want = _oracle_rows(L, rows)
    step = min(m, 64)
    fill = torch.randn(max(m - 64, 0), L["k"], generator=torch.Generator().manual_seed(5)).to(L["dtype"]).to(dev)
    for c0 in range(0, 64, step):
        chunk = rows[c0:c0 + step]
        a = torch.zeros(len(chunk), L["k"], dtype=L["dtype"], device=dev)
        a[torch.arange(len(chunk)), torch.tensor(chunk)] = 1.0
        if m > 64:
            a = torch.cat([a, fill])
        out = _gemm(L, a, ws, is_k_full).cpu()
        for j, i in enumerate(chunk):
            assert torch.equal(out[j], want[i]), f"one-hot row {i} differs from the oracle's dequantised row"


def _check_random(L, m, ws, dev, is_k_full=True):
    a = torch.randn(m, L["k"], generator=torch.Generator().manual_seed(m)).to(L["dtype"]).to(dev)
    out = _gemm(L, a, ws, is_k_full).float()
    ref = a.float() @ L["w_ref"].float()
    tol = 2e-2 if L["dtype"] == torch.float16 else 4e-2
    d = (out - ref).abs()
    n = L["n"]
    dmax = d.view(m, n // 512, 512).amax(dim=(0, 2))
    rmax = ref.abs().view(m, n // 512, 512).amax(dim=(0, 2))
    assert float((dmax / rmax).max()) <= tol
    assert float(d.mean() / ref.abs().mean()) < 0.04
    assert int(ws.abs().sum()) == 0


@pytest.fixture(scope="module")
def ws(dev):
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    return marlin_make_workspace_new(dev)


@pytest.mark.parametrize("m", [1, 4, 16, 64, 256])
@pytest.mark.parametrize("name", ["qkv", "o", "gate_up", "down"])
def test_decode_gptq_fp16(dev, ws, name, m):
    print(f"baseline shape gptq fp16 {name} m={m}", flush=True)
    L = _layer("gptq_f16", name, dev)
    _check_one_hot(L, m, ws, dev)
    _check_random(L, m, ws, dev)


@pytest.mark.parametrize("name", ["qkv", "o", "gate_up", "down"])
def test_prefill_awq_bf16(dev, ws, name):
    print(f"baseline shape awq bf16 {name} m=4096", flush=True)
    L = _layer("awq_bf16", name, dev)
    _check_one_hot(L, 4096, ws, dev)
    _check_random(L, 4096, ws, dev)


@pytest.mark.parametrize("is_k_full", [True, False])
@pytest.mark.parametrize("m", [1, 16, 512])
def test_act_order_down(dev, ws, m, is_k_full):
    print(f"baseline shape act-order down m={m} is_k_full={is_k_full}", flush=True)
    L = _layer("act_f16", "down", dev)
    _check_one_hot(L, m, ws, dev, is_k_full)
    _check_random(L, m, ws, dev, is_k_full)


# ------------------------------------------------------------------------------------------- Mixtral fused MoE
@pytest.fixture(scope="module")
def mixtral(dev):
    from vllm_amd.marlin_utils_test import marlin_quantize
    from vllm_amd.scalar_type import scalar_types as st
    _cache.clear()
    torch.cuda.empty_cache()
    e, hid, inter = 8, 4096, 14336
    w13, w2 = [], []
    for i in range(e):
        w13.append(marlin_quantize(_weights(hid, 2 * inter, torch.float16, dev, 2000 + i), st.uint4b8, GROUP, False,
                                   rule="absmax")[:3])
        w2.append(marlin_quantize(_weights(inter, hid, torch.float16, dev, 3000 + i), st.uint4b8, GROUP, False,
                                  rule="absmax")[:3])
    M = dict(e=e, hid=hid, inter=inter,
             q1=torch.stack([x[1] for x in w13]), s1=torch.stack([x[2] for x in w13]),
             q2=torch.stack([x[1] for x in w2]), s2=torch.stack([x[2] for x in w2]),
             ref1=[x[0] for x in w13], ref2=[x[0] for x in w2])
    yield M
    M.clear()
    torch.cuda.empty_cache()


@pytest.mark.parametrize("t", [16, 512, 4096])
def test_mixtral_fused_moe(dev, mixtral, t):
    """fused_marlin_moe against the torch_experts computation on the dequantised weights (fp32 matmuls on the GPU,
    intermediate roundings as in tests/kernels/utils.py:900-1017); the reference's gate: atol 5e-2, rtol 0."""
    print(f"baseline shape mixtral T={t}", flush=True)
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    from vllm_amd.scalar_type import scalar_types as st
    M = mixtral
    e, hid, inter, topk = M["e"], M["hid"], M["inter"], 2
    g = torch.Generator().manual_seed(50 + t)
    x = torch.randn(t, hid, generator=g).half().to(dev)
    logits = torch.randn(t, e, generator=g).to(dev)
    tw, ti = torch.topk(torch.softmax(logits.float(), dim=-1), topk)
    tw = (tw / tw.sum(dim=-1, keepdim=True)).contiguous()
    ti = ti.to(torch.int32).contiguous()
    out = fused_marlin_moe(x, M["q1"], M["q2"], None, None, M["s1"], M["s2"], logits, tw, ti,
                           quant_type_id=st.uint4b8.id, global_num_experts=e)
    ref = torch.zeros(t, hid, dtype=torch.float32, device=dev)
    for ex in range(e):
        tok, slot = torch.nonzero(ti == ex, as_tuple=True)
        if tok.numel() == 0:
            continue
        h = (x[tok].float() @ M["ref1"][ex].float()).half()
        act = torch.nn.functional.silu(h[:, :inter].float()).half() * h[:, inter:]
        y = (act.float() @ M["ref2"][ex].float()).half()
        ref.index_add_(0, tok, y.float() * tw[tok, slot].unsqueeze(1))
    torch.testing.assert_close(out.float(), ref.half().float(), atol=5e-2, rtol=0)
    # the gate above is absolute; outputs here are O(1), so also bound the error relative to the largest output
    assert float((out.float() - ref).abs().max() / ref.abs().max()) <= 2e-2


@pytest.mark.parametrize("which", ["w13", "w2"])
def test_mixtral_moe_gemm_one_hot(dev, mixtral, which):
    """One-hot tokens through moe_wna16_marlin_gemm on the full expert tensors: output row (token, slot) must equal
    the oracle's dequantised row of the expert the slot routes to, bit for bit."""
    print(f"baseline shape mixtral one-hot {which}", flush=True)
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types as st
    M = mixtral
    e, topk, t = M["e"], 2, 64
    k, n = (M["hid"], 2 * M["inter"]) if which == "w13" else (M["inter"], M["hid"])
    q, s, seed0 = (M["q1"], M["s1"], 2000) if which == "w13" else (M["q2"], M["s2"], 3000)
    rows = _sample_rows(k)
    a = torch.zeros(t, k, dtype=torch.float16, device=dev)
    a[torch.arange(t), torch.tensor(rows)] = 1.0
    g = torch.Generator().manual_seed(9)
    ti = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(t)]).to(torch.int32).to(dev)
    toks = list(range(0, t, 7))                         # 10 tokens x 2 slots; each needs one oracle group
    want = {}
    for ex in sorted({int(ti[tok, slot]) for tok in toks for slot in range(topk)}):
        w_cpu = _weights(k, n, torch.float16, "cpu", seed0 + ex)
        for tok in toks:
            for slot in range(topk):
                if int(ti[tok, slot]) == ex:
                    r = rows[tok]
                    wg = w_cpu[r // GROUP * GROUP:(r // GROUP + 1) * GROUP]
                    want[(tok, slot)] = qu.quantize_absmax7(wg, GROUP)[0][r % GROUP].clone()
        del w_cpu
    for bs in (16, 64):
        sorted_ids, expert_ids, ntpp = moe_align_block_size(ti, bs, e)
        out = ops.moe_wna16_marlin_gemm(
            a, None, q, None, s, None, None, None, None, marlin_make_workspace_new(dev, 4), sorted_ids, expert_ids, ntpp,
            torch.ones(t, topk, device=dev), moe_block_size=bs, top_k=topk, mul_topk_weights=False, is_ep=False,
            b_q_type=st.uint4b8, size_m=t, size_n=n, size_k=k, is_k_full=True, use_atomic_add=False,
            use_fp32_reduce=True, is_zp_float=False).cpu()
        for (tok, slot), row in want.items():
            assert torch.equal(out[tok * topk + slot], row), (bs, tok, slot)


@pytest.mark.parametrize("m", [192, 320, 512, 768, 1024])
@pytest.mark.parametrize("kind", ["gptq_f16", "awq_bf16"])
@pytest.mark.parametrize("name", ["qkv", "o", "down"])
def test_narrow_layers_between_decode_and_prefill(dev, ws, name, kind, m):
    """129..1024 rows on the layers too narrow for the prefill kernel: the planner moves between the general kernel,
    64 x 256 tiles with the K range cut inside the workgroup (and, for down_proj's long K, across workgroups with a
    second pass over the partial tiles) and the 64 x 512 kernel."""
    print(f"narrow layer {kind} {name} m={m}", flush=True)
    L = _layer(kind, name, dev)
    _check_one_hot(L, m, ws, dev)
    _check_random(L, m, ws, dev)
