"""MoE glue and the fused-MoE W4A16 path on the GPU against the CPU oracle (reference tests:
tests/kernels/moe/test_moe.py:667-744, test_moe_align_block_size.py, test_moe.py:889)."""
import pytest
import torch

from helpers import make_layer, tol_for
from oracle import gemm_ref as gr
from oracle import moe_ref as mr

pytestmark = pytest.mark.gpu


def rand_topk(m, topk, e, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)


# ------------------------------------------------------------------------------ align / sum / silu
def test_align_docstring_example(dev):
    from vllm_amd.moe_align_block_size import moe_align_block_size
    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=torch.int32, device=dev)
    s, x, t = moe_align_block_size(ids, 4, 5)
    assert s[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert int(t) == 16 and x[:4].tolist() == [1, 2, 3, 4]


@pytest.mark.parametrize("m,topk,e,bs", [(1, 2, 8, 8), (16, 2, 8, 16), (123, 3, 12, 32), (666, 2, 4, 64),
                                         (4096, 2, 8, 64), (1000, 6, 256, 16), (3, 8, 1024, 8),
                                         # both kernels behind the op, one and several staged chunks of ids, an id
                                         # count that is no multiple of anything, more experts than the ranked kernel takes
                                         (512, 2, 8, 64), (9000, 2, 8, 64), (4321, 8, 200, 48), (2500, 7, 256, 64),
                                         (700, 3, 300, 16), (20000, 1, 3, 64)])
@pytest.mark.parametrize("pad", [False, True])
def test_align_equals_oracle(dev, m, topk, e, bs, pad):
    from vllm_amd.moe_align_block_size import moe_align_block_size
    ids = rand_topk(m, topk, e, seed=m + e)
    s, x, t = moe_align_block_size(ids.to(dev), bs, e, pad_sorted_ids=pad)
    ws, wx, wt = mr.moe_align_block_size(ids, bs, e, pad_sorted_ids=pad)
    assert torch.equal(t.cpu(), wt)
    assert torch.equal(s.cpu(), ws)
    assert torch.equal(x.cpu(), wx)


def test_align_expert_map(dev):
    from vllm_amd.moe_align_block_size import moe_align_block_size
    ids = rand_topk(50, 2, 8, seed=7)
    emap = torch.tensor([-1, 0, -1, 1, -1, 2, -1, 3], dtype=torch.int32)
    s, x, t = moe_align_block_size(ids.to(dev), 16, 8, expert_map=emap.to(dev))
    ws, wx, wt = mr.moe_align_block_size(ids, 16, 8, expert_map=emap)
    nb = int(wt) // 16
    assert torch.equal(t.cpu(), wt) and torch.equal(s.cpu(), ws) and torch.equal(x.cpu()[:nb], wx[:nb])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,topk,d", [(1, 2, 64), (37, 3, 4096), (512, 2, 1024)])
def test_moe_sum(dev, dtype, m, topk, d):
    import vllm_amd.ops as ops
    x = torch.randn(m, topk, d, generator=torch.Generator().manual_seed(0)).to(dtype)
    out = torch.empty(m, d, dtype=dtype, device=dev)
    ops.moe_sum(x.to(dev), out)
    want = x.float().sum(dim=1).to(dtype)                      # fp32 accumulate, one rounding
    assert torch.equal(out.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,d", [(1, 64), (33, 14336), (256, 1024)])
def test_silu_and_mul(dev, dtype, m, d):
    import vllm_amd.ops as ops
    x = torch.randn(m, 2 * d, generator=torch.Generator().manual_seed(1)).to(dtype)
    out = torch.empty(m, d, dtype=dtype, device=dev)
    ops.silu_and_mul(out, x.to(dev))
    xf = x[:, :d].float()
    want = ((xf / (1 + torch.exp(-xf))).to(dtype) * x[:, d:]).float()   # SiLU in fp32 -> T, then a T multiply
    got = out.cpu().float()
    # exp differs in the last ulp between devices: allow one rounding step of the result type
    eps = 2.0 ** (-10 if dtype == torch.float16 else -7)
    assert ((got - want).abs() <= eps * want.abs() + 1e-6).all()
    assert torch.allclose(got, mr.silu_and_mul(x.float()), rtol=4 * eps, atol=1e-3)
    # the reference's own bar (tests/kernels/core/test_activation.py:93-97): exactly the native PyTorch result on the device
    xd = x.to(dev)
    assert torch.equal(out, torch.nn.functional.silu(xd[:, :d]) * xd[:, d:])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("t,e,topk", [(1, 8, 2), (33, 8, 2), (7, 60, 6), (128, 64, 8), (5, 256, 8), (3, 1000, 4)])
@pytest.mark.parametrize("renorm", [False, True])
def test_topk_softmax(dev, dtype, t, e, topk, renorm):
    from vllm_amd.fused_moe import fused_topk
    g = torch.Generator().manual_seed(t + e)
    logits = (torch.randn(t, e, generator=g) * 2).to(dtype)
    w, ids, src = fused_topk(torch.empty(t, 4, device=dev), logits.to(dev), topk, renorm)
    p = torch.softmax(logits.float(), dim=-1)
    tw, ti = torch.topk(p, topk)
    if renorm:
        tw = tw / tw.sum(-1, keepdim=True)
    assert w.dtype == torch.float32 and ids.dtype == torch.int32
    # 16-bit logits can tie exactly: compare the selected probabilities, and the ids wherever they are unambiguous
    torch.testing.assert_close(w.cpu(), tw, rtol=2e-5, atol=1e-7)
    sel = torch.gather(p, 1, ids.cpu().long())
    assert torch.equal(sel, torch.gather(p, 1, ti))
    for r in range(t):
        assert len(set(ids[r].tolist())) == topk
    assert src.cpu().tolist() == [[k * t + r for k in range(topk)] for r in range(t)]
    if t * e <= 2048:
        ow, oi, _ = mr.topk_softmax(logits, topk, renorm)     # scalar oracle incl. lowest-index tie-break
        assert torch.equal(ids.cpu(), oi)
        torch.testing.assert_close(w.cpu(), ow, rtol=2e-5, atol=1e-7)


def test_topk_softmax_ties_take_lowest_index(dev):
    from vllm_amd.fused_moe import fused_topk
    logits = torch.zeros(2, 130, device=dev)
    logits[1, 70] = 1.0
    w, ids, _ = fused_topk(torch.empty(2, 4, device=dev), logits, 3, True)
    assert ids.cpu().tolist() == [[0, 1, 2], [70, 0, 1]]
    assert torch.allclose(w[0].cpu(), torch.full((3,), 1 / 3))


@pytest.mark.parametrize("max_tokens", [13, 64, 512])
@pytest.mark.parametrize("e", [8, 32])
@pytest.mark.parametrize("bs", [8, 16, 64])
@pytest.mark.parametrize("empty", [False, True])
def test_batched_align_equals_oracle(dev, max_tokens, e, bs, empty):
    from vllm_amd.moe_align_block_size import batched_moe_align_block_size
    g = torch.Generator().manual_seed(max_tokens + e)
    n = torch.randint(1, max_tokens + 1, (e,), generator=g, dtype=torch.int32)
    if empty:
        n[torch.randperm(e, generator=g)[:e // 2]] = 0
    s, x, t = batched_moe_align_block_size(max_tokens, bs, n.to(dev))
    ws, wx, wt = mr.batched_moe_align_block_size(max_tokens, bs, n)
    assert torch.equal(t.cpu(), wt) and torch.equal(s.cpu(), ws) and torch.equal(x.cpu(), wx)


# ------------------------------------------------------------------------------------- MoE GEMM
def make_experts(e, k, n, group, dtype, has_zp, act_order, seed):
    layers = [make_layer(k, n, group, dtype, has_zp=has_zp, act_order=act_order, seed=seed + i, w_std=0.1) for i in range(e)]
    st = lambda name: torch.stack([getattr(l, name) for l in layers])
    return layers, st("marlin_q"), st("marlin_s"), st("marlin_zp"), st("g_idx_sorted"), st("sort_indices")


@pytest.mark.parametrize("m,topk,e,bs", [(1, 2, 4, 8), (33, 2, 8, 16), (123, 3, 4, 32), (200, 2, 4, 48), (333, 2, 4, 64)])
@pytest.mark.parametrize("variant", ["gptq_f16_g128", "gptq_bf16_chan", "awq_bf16_g128", "gptq_f16_g32_act"])
@pytest.mark.parametrize("mul", [False, True])
def test_moe_gemm_equals_oracle(dev, m, topk, e, bs, variant, mul):
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    dtype = torch.bfloat16 if "bf16" in variant else torch.float16
    group = -1 if "chan" in variant else 32 if "g32" in variant else 128
    has_zp, act = variant.startswith("awq"), variant.endswith("act")
    k, n = 256, 192
    layers, mq, ms, mz, gi, perm = make_experts(e, k, n, group, dtype, has_zp, act, seed=10)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(5)).to(dtype)
    ids = rand_topk(m, topk, e, seed=6)
    tw = torch.rand(m, topk, generator=torch.Generator().manual_seed(7))
    s, x, t = moe_align_block_size(ids.to(dev), bs, e)
    ws = marlin_make_workspace_new(dev, 4)
    out = ops.moe_wna16_marlin_gemm(
        a.to(dev), None, mq.to(dev), None, ms.to(dev), None, mz.to(dev), gi.to(dev), perm.to(dev), ws, s, x, t,
        tw.to(dev), moe_block_size=bs, top_k=topk, mul_topk_weights=mul, is_ep=False,
        b_q_type=scalar_types.uint4 if has_zp else scalar_types.uint4b8, size_m=m, size_n=n, size_k=k,
        is_k_full=True, use_atomic_add=False, use_fp32_reduce=True, is_zp_float=False)
    assert out.shape == (m * topk, n)
    w_dense = torch.stack([l.w_ref for l in layers])
    ref = mr.moe_gemm_ref(a, w_dense, s.cpu(), x.cpu(), t.cpu(), tw, bs, topk, mul, m)
    mtr = gr.error_metrics(out, ref)
    assert mtr["max_rel"] <= tol_for(dtype) and mtr["mean_rel"] < 0.04, mtr
    assert int(ws.abs().sum()) == 0


def test_moe_gemm_split_k_blocks_of_64(dev):
    """Enough rows for blocks of 64 but fewer than 256 tiles: the 64-row kernel splits K and runs its reduction pass."""
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    m, topk, e, bs, k, n = 2048, 2, 4, 64, 2048, 1024
    layers, mq, ms, mz, gi, perm = make_experts(e, k, n, 128, torch.float16, False, False, seed=50)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(5)).half()
    ids = rand_topk(m, topk, e, seed=6)
    tw = torch.rand(m, topk, generator=torch.Generator().manual_seed(7))
    s, x, t = moe_align_block_size(ids.to(dev), bs, e)
    ws = marlin_make_workspace_new(dev, 4)
    out = ops.moe_wna16_marlin_gemm(
        a.to(dev), None, mq.to(dev), None, ms.to(dev), None, mz.to(dev), gi.to(dev), perm.to(dev), ws, s, x, t,
        tw.to(dev), moe_block_size=bs, top_k=topk, mul_topk_weights=True, is_ep=False, b_q_type=scalar_types.uint4b8,
        size_m=m, size_n=n, size_k=k, is_k_full=True, use_atomic_add=False, use_fp32_reduce=True, is_zp_float=False)
    # dense reference per expert on the gathered rows
    flat = ids.flatten().long()
    ref = torch.zeros(m * topk, n)
    for ex in range(e):
        rows = torch.nonzero(flat == ex).flatten()
        ref[rows] = (a[rows // topk].float() @ layers[ex].w_ref.float()) * tw.flatten()[rows].unsqueeze(1)
    mtr = gr.error_metrics(out, ref)
    assert mtr["max_rel"] <= 2e-2 and mtr["mean_rel"] < 0.04, mtr


@pytest.mark.parametrize("m,foreign", [(300, False), (300, True), (1200, False), (8300, False)])
def test_moe_gemm_tail_tiles_split_on_the_device(dev, m, foreign):
    """Blocks of 64 with a long K: the 64-row kernel cuts the tiles of its last, partly filled round of resident
    workgroups along K, by a number of pieces it derives from the live block count on the device, and a second pass adds
    the pieces.  24 live tiles -> 4 pieces each; 80 -> 4; about 520 -> 512 whole tiles and a few split ones; with blocks
    of experts held by another rank (left untouched) among them."""
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    topk, e, bs, k, n = 2, 4, 64, 4096, 1024
    print(f"tail split m={m} foreign={foreign}", flush=True)
    layers, mq, ms, mz, gi, perm = make_experts(e, k, n, 128, torch.float16, False, False, seed=80)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(5)).half()
    ids = rand_topk(m, topk, e, seed=6)
    tw = torch.rand(m, topk, generator=torch.Generator().manual_seed(7))
    emap = torch.tensor([0, -1, 1, 2], dtype=torch.int32) if foreign else None
    local = [0, 2, 3] if foreign else [0, 1, 2, 3]
    s, x, t = moe_align_block_size(ids.to(dev), bs, e, expert_map=emap.to(dev) if foreign else None)
    c = torch.full((m * topk, n), 7.0, dtype=torch.float16, device=dev)
    ws = marlin_make_workspace_new(dev, 4)
    out = ops.moe_wna16_marlin_gemm(
        a.to(dev), c, mq[local].to(dev), None, ms[local].to(dev), None, mz[local].to(dev), gi[local].to(dev),
        perm[local].to(dev), ws, s, x, t, tw.to(dev), moe_block_size=bs, top_k=topk, mul_topk_weights=True, is_ep=foreign,
        b_q_type=scalar_types.uint4b8, size_m=m, size_n=n, size_k=k, is_k_full=True, use_atomic_add=False,
        use_fp32_reduce=True, is_zp_float=False).cpu()
    flat = ids.flatten().long()
    for ex in range(e):
        rows = torch.nonzero(flat == ex).flatten()
        if foreign and ex == 1:
            assert (out[rows] == 7.0).all()
            continue
        ref = (a[rows // topk].float() @ layers[ex].w_ref.float()) * tw.flatten()[rows].unsqueeze(1)
        mtr = gr.error_metrics(out[rows], ref)
        assert mtr["max_rel"] <= 2e-2 and mtr["mean_rel"] < 0.04, (ex, mtr)
    assert int(ws.abs().sum()) == 0


def test_moe_gemm_more_than_65535_tiles(dev):
    """5000 blocks of 8 slots x 16 column tiles: the 16-row kernel's tile index spills into the grid's third dimension
    (workgroups past the last tile leave at once, after their share of the zero-fill side job)."""
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    m, topk, e, bs, k, n = 40000, 1, 2, 8, 128, 2048
    layers, mq, ms, mz, gi, perm = make_experts(e, k, n, 128, torch.float16, False, False, seed=90)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(5)).half()
    ids = rand_topk(m, topk, e, seed=6)
    tw = torch.rand(m, topk, generator=torch.Generator().manual_seed(7))
    s, x, t = moe_align_block_size(ids.to(dev), bs, e)
    ws = marlin_make_workspace_new(dev, 4)
    out = ops.moe_wna16_marlin_gemm(
        a.to(dev), None, mq.to(dev), None, ms.to(dev), None, mz.to(dev), gi.to(dev), perm.to(dev), ws, s, x, t,
        tw.to(dev), moe_block_size=bs, top_k=topk, mul_topk_weights=True, is_ep=False, b_q_type=scalar_types.uint4b8,
        size_m=m, size_n=n, size_k=k, is_k_full=True, use_atomic_add=False, use_fp32_reduce=True, is_zp_float=False).cpu()
    flat = ids.flatten().long()
    for ex in range(e):
        rows = torch.nonzero(flat == ex).flatten()
        ref = (a[rows].float() @ layers[ex].w_ref.float()) * tw.flatten()[rows].unsqueeze(1)
        mtr = gr.error_metrics(out[rows], ref)
        assert mtr["max_rel"] <= 2e-2 and mtr["mean_rel"] < 0.04, (ex, mtr)
    # the same launch through the fused operator with a buffer to clear on the side: every 16-byte piece is cleared
    fill = torch.full((3 * 1024 * 1024 + 40,), 1.0, dtype=torch.float16, device=dev)
    c = torch.empty(m * topk, n, dtype=torch.float16, device=dev)
    ops.moe_marlin_gemm_fused(a.to(dev), c, mq.to(dev), None, ms.to(dev), None, mz.to(dev), gi.to(dev), perm.to(dev), ws, s,
                              x, t, tw.to(dev), bs, topk, True, scalar_types.uint4b8, m, n, k, True, False, 0, fill)
    assert int(torch.count_nonzero(fill)) == 0
    assert torch.equal(c.cpu(), out)


def test_moe_gemm_skips_foreign_experts_and_bias(dev):
    """expert_ids = -1 blocks are left untouched (expert parallelism); per-expert bias is added."""
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new, marlin_permute_bias
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    m, topk, e, bs, k, n = 40, 2, 4, 16, 256, 128
    layers, mq, ms, mz, gi, perm = make_experts(e, k, n, 128, torch.float16, False, False, seed=30)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(8)).half()
    ids = rand_topk(m, topk, e, seed=9)
    emap = torch.tensor([0, -1, 1, -1], dtype=torch.int32)
    bias = torch.randn(e, n, generator=torch.Generator().manual_seed(10)).half()
    s, x, t = moe_align_block_size(ids.to(dev), bs, e, expert_map=emap.to(dev))
    c = torch.full((m * topk, n), 7.0, dtype=torch.float16, device=dev)
    # local experts 0, 1 hold global experts 0, 2
    local = [0, 2]
    pb = torch.stack([marlin_permute_bias(bias[g]) for g in local])
    out = ops.moe_wna16_marlin_gemm(
        a.to(dev), c, mq[local].to(dev), pb.to(dev), ms[local].to(dev), None, mz[local].to(dev), gi[local].to(dev),
        perm[local].to(dev), marlin_make_workspace_new(dev, 4), s, x, t, torch.ones(m, topk, device=dev),
        moe_block_size=bs, top_k=topk, mul_topk_weights=False, is_ep=True, b_q_type=scalar_types.uint4b8,
        size_m=m, size_n=n, size_k=k, is_k_full=True, use_atomic_add=False, use_fp32_reduce=True, is_zp_float=False)
    out = out.cpu().float()
    flat = ids.flatten()
    for i in range(m * topk):
        g = int(flat[i])
        if int(emap[g]) < 0:
            assert (out[i] == 7.0).all()
        else:
            want = a[i // topk].float() @ layers[g].w_ref.float() + bias[g].float()
            assert float((out[i] - want).abs().max() / want.abs().max()) <= 2e-2


# ----------------------------------------------------------------------------------- fused MoE
@pytest.mark.parametrize("m", [1, 33, 123, 666])
@pytest.mark.parametrize("e,topk", [(4, 2), (12, 3)])
@pytest.mark.parametrize("variant", ["gptq_f16_g128", "awq_bf16_g128", "gptq_bf16_chan"])
def test_fused_marlin_moe_vs_torch_moe(dev, m, e, topk, variant):
    """The reference's gate: atol 5e-2, rtol 0 against torch_moe on the dequantised weights."""
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    dtype = torch.bfloat16 if "bf16" in variant else torch.float16
    group = -1 if "chan" in variant else 128
    has_zp = variant.startswith("awq")
    k, inter = 256, 128
    l1, q1, s1, z1, _, _ = make_experts(e, k, 2 * inter, group, dtype, has_zp, False, seed=100)
    l2, q2, s2, z2, _, _ = make_experts(e, inter, k, group, dtype, has_zp, False, seed=200)
    g = torch.Generator().manual_seed(11)
    a = (torch.randn(m, k, generator=g) / 10).to(dtype)
    score = torch.randn(m, e, generator=g).to(dtype)
    p = torch.softmax(score.float(), dim=-1)
    tw, ti = torch.topk(p, topk)
    from helpers import Layer  # noqa: F401
    out = fused_marlin_moe(
        a.to(dev), q1.to(dev), q2.to(dev), None, None, s1.to(dev), s2.to(dev), score.to(dev), tw.to(dev),
        ti.to(torch.int32).to(dev), quant_type_id=l1[0].type_id, global_num_experts=e,
        w1_zeros=z1.to(dev) if has_zp else None, w2_zeros=z2.to(dev) if has_zp else None)
    w1 = torch.stack([l.w_ref.t() for l in l1])            # [E, 2I, K] as nn.Linear weights
    w2 = torch.stack([l.w_ref.t() for l in l2])            # [E, K, I]
    ref = mr.torch_experts(a, w1, w2, tw, ti)
    assert out.shape == (m, k)
    torch.testing.assert_close(out.cpu().float(), ref.float(), atol=5e-2, rtol=0)


@pytest.mark.parametrize("m", [1, 16, 300])
@pytest.mark.parametrize("e,topk", [(64, 6), (128, 8)])
def test_fused_marlin_moe_many_experts(dev, m, e, topk):
    """Expert counts and top-k of the fine-grained MoE models (64 experts / top-6, 128 / top-8): most blocks hold one or
    two slots, top-k above 2 takes the five-launch sequence.  Same gate as above."""
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    dtype, k, inter = torch.float16, 256, 128
    l1, q1, s1, _, _, _ = make_experts(e, k, 2 * inter, 128, dtype, False, False, seed=500)
    l2, q2, s2, _, _, _ = make_experts(e, inter, k, 128, dtype, False, False, seed=700)
    g = torch.Generator().manual_seed(13)
    a = (torch.randn(m, k, generator=g) / 10).to(dtype)
    score = torch.randn(m, e, generator=g).to(dtype)
    tw, ti = torch.topk(torch.softmax(score.float(), dim=-1), topk)
    tw = tw / tw.sum(dim=-1, keepdim=True)
    out = fused_marlin_moe(a.to(dev), q1.to(dev), q2.to(dev), None, None, s1.to(dev), s2.to(dev), score.to(dev),
                           tw.to(dev), ti.to(torch.int32).to(dev), quant_type_id=l1[0].type_id, global_num_experts=e)
    w1 = torch.stack([l.w_ref.t() for l in l1])
    w2 = torch.stack([l.w_ref.t() for l in l2])
    ref = mr.torch_experts(a, w1, w2, tw, ti)
    torch.testing.assert_close(out.cpu().float(), ref.float(), atol=5e-2, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,topk", [(64, 2), (24, 8)])
def test_fused_marlin_moe_more_tiles_than_compute_units(dev, dtype, m, topk):
    """128 experts, blocks of a few slots and four column tiles per block: both GEMMs launch more 16-row tiles than the
    chip has compute units, which the decode kernel runs as 4-wavefront workgroups (fused SiLU-and-mul epilogue, and for
    top-2 the fused sum, on that variant).  Same gate as above."""
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    e, k, inter = 128, 512, 256
    l1, q1, s1, _, _, _ = make_experts(e, k, 2 * inter, 128, dtype, False, False, seed=900)
    l2, q2, s2, _, _, _ = make_experts(e, inter, k, 128, dtype, False, False, seed=1100)
    g = torch.Generator().manual_seed(14)
    a = (torch.randn(m, k, generator=g) / 10).to(dtype)
    score = torch.randn(m, e, generator=g).to(dtype)
    tw, ti = torch.topk(torch.softmax(score.float(), dim=-1), topk)
    tw = tw / tw.sum(dim=-1, keepdim=True)
    out = fused_marlin_moe(a.to(dev), q1.to(dev), q2.to(dev), None, None, s1.to(dev), s2.to(dev), score.to(dev),
                           tw.to(dev), ti.to(torch.int32).to(dev), quant_type_id=l1[0].type_id, global_num_experts=e)
    w1 = torch.stack([l.w_ref.t() for l in l1])
    w2 = torch.stack([l.w_ref.t() for l in l2])
    ref = mr.torch_experts(a, w1, w2, tw, ti)
    torch.testing.assert_close(out.cpu().float(), ref.float(), atol=5e-2, rtol=0)


def test_fused_marlin_moe_mixtral_shape(dev):
    """Mixtral-8x7B expert shapes (hidden 4096, intermediate 14336, top-2) at T = 16; two experts instead of
    eight, so that quantising them with the CPU oracle stays within seconds."""
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    e, topk, k, inter, m = 2, 2, 4096, 14336, 16
    dtype = torch.float16
    l1, q1, s1, _, _, _ = make_experts(e, k, 2 * inter, 128, dtype, False, False, seed=300)
    l2, q2, s2, _, _, _ = make_experts(e, inter, k, 128, dtype, False, False, seed=400)
    g = torch.Generator().manual_seed(12)
    a = (torch.randn(m, k, generator=g) / 10).to(dtype)
    score = torch.randn(m, e, generator=g)
    tw, ti = torch.topk(torch.softmax(score, dim=-1), topk)
    tw = tw / tw.sum(dim=-1, keepdim=True)
    out = fused_marlin_moe(a.to(dev), q1.to(dev), q2.to(dev), None, None, s1.to(dev), s2.to(dev), score.to(dev),
                           tw.to(dev), ti.to(torch.int32).to(dev), quant_type_id=l1[0].type_id, global_num_experts=e)
    # oracle on the GPU-free path would need 8 x (4096x28672 + 14336x4096) fp32 matmuls: do the experts hit only
    w1 = {int(x): l1[int(x)].w_ref.float() for x in ti.unique()}
    w2 = {int(x): l2[int(x)].w_ref.float() for x in ti.unique()}
    ref = torch.zeros(m, k)
    for t in range(m):
        for j in range(topk):
            ex = int(ti[t, j])
            h = (a[t].float() @ w1[ex]).to(dtype)
            act = (torch.nn.functional.silu(h[:inter].float()).to(dtype) * h[inter:])
            ref[t] += float(tw[t, j]) * (act.float() @ w2[ex]).to(dtype).float()
    torch.testing.assert_close(out.cpu().float(), ref, atol=5e-2, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_batched_fused_marlin_moe_equals_standard(dev, dtype):
    """The reference's own check (tests/kernels/moe/test_moe.py:977-1135): batching tokens per expert and running the
    batched entry point gives what fused_marlin_moe gives for the same tokens (atol 1e-3)."""
    from vllm_amd.fused_marlin_moe import batched_fused_marlin_moe, fused_marlin_moe
    e, k, inter, max_tokens = 4, 256, 128, 70
    l1, q1, s1, _, _, _ = make_experts(e, k, 2 * inter, 128, dtype, False, False, seed=500)
    l2, q2, s2, _, _, _ = make_experts(e, inter, k, 128, dtype, False, False, seed=600)
    g = torch.Generator().manual_seed(13)
    n = torch.tensor([70, 0, 33, 64], dtype=torch.int32)
    x = (torch.randn(e, max_tokens, k, generator=g) / 10).to(dtype)
    out = batched_fused_marlin_moe(x.to(dev), n.to(dev), q1.to(dev), q2.to(dev), None, None, s1.to(dev), s2.to(dev), None,
                                   quant_type_id=l1[0].type_id)
    assert out.shape == (e, max_tokens, k)
    # the same tokens through the standard entry point: token i of expert ex routed to ex with weight 1
    for ex in range(e):
        cnt = int(n[ex])
        if cnt == 0:
            continue
        tok = x[ex, :cnt].contiguous().to(dev)
        ids = torch.full((cnt, 1), ex, dtype=torch.int32, device=dev)
        ones = torch.ones(cnt, 1, dtype=torch.float32, device=dev)
        want = fused_marlin_moe(tok, q1.to(dev), q2.to(dev), None, None, s1.to(dev), s2.to(dev), None, ones, ids,
                                quant_type_id=l1[0].type_id, global_num_experts=e)
        torch.testing.assert_close(out[ex, :cnt], want, atol=1e-3, rtol=0)
        ref = mr.torch_experts(x[ex, :cnt], torch.stack([l.w_ref.t() for l in l1]), torch.stack([l.w_ref.t() for l in l2]),
                               torch.ones(cnt, 1), torch.full((cnt, 1), ex))
        torch.testing.assert_close(out[ex, :cnt].cpu().float(), ref.float(), atol=5e-2, rtol=0)


def test_fused_marlin_moe_with_bias(dev):
    """Per-expert biases on both GEMMs (reference tests/kernels/moe/test_moe.py:750-830), atol 5e-2."""
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    from vllm_amd.marlin_utils import marlin_permute_bias
    dtype, e, topk, m, k, inter = torch.float16, 4, 2, 37, 256, 128
    l1, q1, s1, _, _, _ = make_experts(e, k, 2 * inter, 128, dtype, False, False, seed=700)
    l2, q2, s2, _, _, _ = make_experts(e, inter, k, 128, dtype, False, False, seed=800)
    g = torch.Generator().manual_seed(14)
    a = (torch.randn(m, k, generator=g) / 10).to(dtype)
    b1 = (torch.randn(e, 2 * inter, generator=g) / 10).to(dtype)
    b2 = (torch.randn(e, k, generator=g) / 10).to(dtype)
    score = torch.randn(m, e, generator=g)
    tw, ti = torch.topk(torch.softmax(score, dim=-1), topk)
    pb1 = torch.stack([marlin_permute_bias(b1[i].to(dev)) for i in range(e)])
    pb2 = torch.stack([marlin_permute_bias(b2[i].to(dev)) for i in range(e)])
    out = fused_marlin_moe(a.to(dev), q1.to(dev), q2.to(dev), pb1, pb2, s1.to(dev), s2.to(dev), score.to(dev), tw.to(dev),
                           ti.to(torch.int32).to(dev), quant_type_id=l1[0].type_id, global_num_experts=e)
    ref = torch.zeros(m, k)
    for t in range(m):
        for j in range(topk):
            ex = int(ti[t, j])
            h = (a[t].float() @ l1[ex].w_ref.float() + b1[ex].float()).to(dtype)
            act = torch.nn.functional.silu(h[:inter].float()).to(dtype) * h[inter:]
            ref[t] += float(tw[t, j]) * (act.float() @ l2[ex].w_ref.float() + b2[ex].float()).to(dtype).float()
    torch.testing.assert_close(out.cpu().float(), ref, atol=5e-2, rtol=0)


@pytest.mark.parametrize("bs", [16, 48])
def test_moe_gemm_never_uses_memory_past_sorted_ids(dev, bs):
    """sorted_token_ids of the usual length numel + E * (block - 1), not a multiple of the block size, as an exact-size
    view in front of slot ids that look valid: the launch's last, never-live block must not pick them up, and the result
    must equal the one computed from a tensor of its own."""
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    m, topk, e, k, n = 16, 2, 8, 256, 192
    layers, mq, ms, mz, gi, perm = make_experts(e, k, n, 128, torch.float16, False, False, seed=10)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(5)).half().to(dev)
    ids = rand_topk(m, topk, e, seed=6).to(dev)
    tw = torch.rand(m, topk, generator=torch.Generator().manual_seed(7)).to(dev)
    s, x, t = moe_align_block_size(ids, bs, e)
    assert s.numel() % bs != 0
    big = torch.zeros(s.numel() + 4 * bs, dtype=torch.int32, device=dev)   # id 0 behind the end: a valid-looking slot
    big[:s.numel()] = s
    ws = marlin_make_workspace_new(dev, 4)
    call = lambda sorted_ids: ops.moe_wna16_marlin_gemm(
        a, None, mq.to(dev), None, ms.to(dev), None, None, None, None, ws, sorted_ids, x, t, tw, moe_block_size=bs,
        top_k=topk, mul_topk_weights=True, is_ep=False, b_q_type=scalar_types.uint4b8, size_m=m, size_n=n, size_k=k,
        is_k_full=True, use_atomic_add=False, use_fp32_reduce=True, is_zp_float=False)
    want = call(s)
    got = call(big[:s.numel()])
    assert torch.equal(got, want)
