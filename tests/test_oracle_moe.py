"""Pins the MoE glue oracle (CPU only): alignment known answer and invariants, brute-force experts."""
import pytest
import torch

from oracle import moe_ref as mr


def test_align_docstring_example():
    """The worked example of the reference's contract docstring (moe_align_block_size.py:53-63)."""
    topk_ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=torch.int32)
    sorted_ids, expert_ids, total = mr.moe_align_block_size(topk_ids, 4, 5)
    assert sorted_ids[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert int(total) == 16
    assert expert_ids[:4].tolist() == [1, 2, 3, 4]
    assert (sorted_ids[16:] == 12).all()


@pytest.mark.parametrize("m,topk,e,bs", [(1, 2, 4, 8), (33, 2, 8, 16), (123, 3, 12, 64), (7, 6, 64, 16)])
def test_align_invariants(m, topk, e, bs):
    """What the reference's test asserts (test_moe_align_block_size.py:210-231) plus stability."""
    g = torch.Generator().manual_seed(m + e)
    topk_ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    sorted_ids, expert_ids, total = mr.moe_align_block_size(topk_ids, bs, e)
    numel = m * topk
    total = int(total)
    assert sorted_ids.numel() == numel + e * (bs - 1)
    assert total % bs == 0 and total <= sorted_ids.numel()
    counts = torch.bincount(topk_ids.flatten().long(), minlength=e)
    assert total == int(((counts + bs - 1) // bs * bs).sum())
    valid = sorted_ids[:total]
    real = valid[valid < numel]
    assert sorted(real.tolist()) == list(range(numel))            # every (token, slot) exactly once
    assert (sorted_ids[total:] == numel).all()
    flat = topk_ids.flatten()
    for b in range(total // bs):
        blk = valid[b * bs:(b + 1) * bs]
        ids = blk[blk < numel]
        assert ids.numel() > 0
        assert (flat[ids.long()] == expert_ids[b]).all()           # a block belongs to one expert
        assert (ids[1:] > ids[:-1]).all()                          # stable: ascending flat index
        pad = blk[ids.numel():]
        assert (pad == numel).all()                                # padding only at the tail of a block
    assert (expert_ids[total // bs:] == 0).all()
    assert (expert_ids[1:total // bs] >= expert_ids[:total // bs - 1]).all()


def test_align_expert_map_and_padded_length():
    topk_ids = torch.tensor([[0, 3], [3, 2]], dtype=torch.int32)
    emap = torch.tensor([-1, -1, 0, 1], dtype=torch.int32)
    sorted_ids, expert_ids, total = mr.moe_align_block_size(topk_ids, 4, 4, expert_map=emap, pad_sorted_ids=True)
    assert sorted_ids.numel() == 16 and int(total) == 12
    assert expert_ids[:3].tolist() == [-1, 0, 1]


def test_silu_and_mul_closed_form():
    x = torch.tensor([[0.0, 1.0, -2.0, 3.0, 2.0, 5.0]])
    want = torch.tensor([[0.0, 2.0 / (1 + torch.exp(torch.tensor(-1.0))), -10.0 / (1 + torch.exp(torch.tensor(2.0)))]])
    assert torch.allclose(mr.silu_and_mul(x), want, atol=1e-6)


def test_experts_brute_force():
    g = torch.Generator().manual_seed(0)
    m, k, inter, e, topk = 5, 8, 6, 4, 2
    a = torch.randn(m, k, generator=g)
    w1 = torch.randn(e, 2 * inter, k, generator=g)
    w2 = torch.randn(e, k, inter, generator=g)
    score = torch.randn(m, e, generator=g)
    got = mr.torch_moe(a, w1, w2, score, topk, renormalize=True)
    p = torch.softmax(score, -1)
    want = torch.zeros(m, k)
    for t in range(m):
        tw, ti = torch.topk(p[t], topk)
        tw = tw / tw.sum()
        for wgt, ex in zip(tw.tolist(), ti.tolist()):
            h = w1[ex] @ a[t]
            act = torch.nn.functional.silu(h[:inter]) * h[inter:]
            want[t] += wgt * (w2[ex] @ act)
    assert torch.allclose(got, want, atol=1e-5)


def test_moe_gemm_ref_is_dense_gemm_per_expert():
    g = torch.Generator().manual_seed(1)
    m, k, n, e, topk, bs = 9, 16, 12, 4, 2, 8
    a = torch.randn(m, k, generator=g)
    w = torch.randn(e, k, n, generator=g)
    topk_ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    tw = torch.rand(m, topk, generator=g)
    sorted_ids, expert_ids, total = mr.moe_align_block_size(topk_ids, bs, e)
    for mul in (False, True):
        out = mr.moe_gemm_ref(a, w, sorted_ids, expert_ids, total, tw, bs, topk, mul, m)
        for t in range(m):
            for s in range(topk):
                want = a[t] @ w[int(topk_ids[t, s])]
                if mul:
                    want = want * tw[t, s]
                assert torch.allclose(out[t * topk + s], want, atol=1e-5)


def test_topk_softmax_hand_case_and_torch_agreement():
    import math
    # logits (0, ln 2, ln 2, -inf-ish): probabilities 0.2, 0.4, 0.4, ~0; the tie goes to the lower index
    g = torch.tensor([[0.0, math.log(2.0), math.log(2.0), -50.0]])
    w, ids, src = mr.topk_softmax(g, 2, False)
    assert ids.tolist() == [[1, 2]] and src.tolist() == [[0, 1]]
    assert torch.allclose(w, torch.tensor([[0.4, 0.4]]), atol=1e-6)
    w, ids, _ = mr.topk_softmax(g, 3, True)
    assert ids.tolist() == [[1, 2, 0]] and torch.allclose(w, torch.tensor([[0.4, 0.4, 0.2]]), atol=1e-6)
    x = torch.randn(9, 16, generator=torch.Generator().manual_seed(3))
    w, ids, src = mr.topk_softmax(x, 4, True)
    tw, ti = torch.topk(torch.softmax(x, -1), 4)
    assert torch.equal(ids.long(), ti) and torch.allclose(w, tw / tw.sum(-1, keepdim=True), atol=1e-6)
    assert src.tolist() == [[k * 9 + r for k in range(4)] for r in range(9)]


def test_batched_align_docstring_example():
    """Worked example of the reference's docstring (moe_align_block_size.py:117-149)."""
    s, x, t = mr.batched_moe_align_block_size(8, 4, torch.tensor([2, 3, 0, 6, 8]))
    assert s[:28].tolist() == [0, 1, 40, 40, 8, 9, 10, 40, 24, 25, 26, 27, 28, 29, 40, 40, 32, 33, 34, 35, 36, 37, 38, 39,
                               40, 40, 40, 40]
    assert x.tolist() == [0, 1, 3, 3, 4, 4, -1, -1, -1, -1]
    assert int(t) == 24 and s.numel() == 40
