"""Fused epilogues of the MoE GEMM (SiLU-and-mul inside GEMM1, top-k sum inside GEMM2, the zero-fill side job) against
the separate launches they replace (reference: fused_marlin_moe.py:47-183 runs moe_wna16_marlin_gemm, silu_and_mul,
moe_wna16_marlin_gemm, moe_sum one after the other).  The fused results must be bit-identical: the epilogues round
exactly where the separate kernels do."""
import pytest
import torch

from test_gpu_moe import make_experts, rand_topk

pytestmark = pytest.mark.gpu

CASES = [(1, 2, 4, 8), (16, 2, 8, 8), (33, 2, 8, 16), (123, 2, 4, 32), (200, 2, 4, 48), (333, 2, 4, 64), (2048, 2, 4, 64)]


def _setup(dev, m, topk, e, bs, variant, k, n, seed):
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    dtype = torch.bfloat16 if "bf16" in variant else torch.float16
    group = -1 if "chan" in variant else 128
    has_zp = variant.startswith("awq")
    layers, mq, ms, mz, gi, perm = make_experts(e, k, n, group, dtype, has_zp, False, seed=seed)
    a = (torch.randn(m, k, generator=torch.Generator().manual_seed(5)) / 4).to(dtype).to(dev)
    ids = rand_topk(m, topk, e, seed=6).to(dev)
    tw = torch.rand(m, topk, generator=torch.Generator().manual_seed(7)).to(dev)
    s, x, t = moe_align_block_size(ids, bs, e)
    w = dict(q=mq.to(dev), s=ms.to(dev), z=mz.to(dev) if has_zp else None,
             wtype=scalar_types.uint4 if has_zp else scalar_types.uint4b8)
    return dtype, a, tw, (s, x, t), w, marlin_make_workspace_new(dev, 4)


def _plain(ops, a, w, ws, align, tw, bs, top_k, mul, m, n, k, bias=None):
    s, x, t = align
    return ops.moe_wna16_marlin_gemm(a, None, w["q"], bias, w["s"], None, w["z"], None, None, ws, s, x, t, tw, bs, top_k, mul,
                                     False, w["wtype"], m, n, k, True, False, True, False)


def _fused(ops, a, c, w, ws, align, tw, bs, top_k, mul, m, n, k, bias=None, **kw):
    s, x, t = align
    ops.moe_marlin_gemm_fused(a, c, w["q"], bias, w["s"], None, w["z"], None, None, ws, s, x, t, tw, bs, top_k, mul,
                              w["wtype"], m, n, k, True, **kw)
    return c


@pytest.mark.parametrize("m,topk,e,bs", CASES)
@pytest.mark.parametrize("variant", ["gptq_f16_g128", "gptq_bf16_chan", "awq_bf16_g128"])
@pytest.mark.parametrize("mul", [False, True])
def test_silu_and_mul_epilogue_equals_separate_launches(dev, m, topk, e, bs, variant, mul):
    import vllm_amd.ops as ops
    k, d = (2048, 512) if m == 2048 else (256, 192)
    dtype, a, tw, align, w, ws = _setup(dev, m, topk, e, bs, variant, k, 2 * d, seed=10)
    bias = (torch.randn(e, 2 * d, generator=torch.Generator().manual_seed(3)) / 8).to(dtype).to(dev)
    from vllm_amd.marlin_utils import marlin_permute_bias
    pbias = torch.stack([marlin_permute_bias(bias[i]) for i in range(e)])
    for b in (None, pbias):
        h = _plain(ops, a, w, ws, align, tw, bs, topk, mul, m, 2 * d, k, b)
        want = torch.empty(m * topk, d, dtype=dtype, device=dev)
        ops.silu_and_mul(want, h)
        got = torch.full((m * topk, d), 7.0, dtype=dtype, device=dev)
        _fused(ops, a, got, w, ws, align, tw, bs, topk, mul, m, 2 * d, k, b, silu_and_mul=True)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert float(want.float().abs().max()) > 0 and int(ws.abs().sum()) == 0


@pytest.mark.parametrize("m,topk,e,bs", CASES)
@pytest.mark.parametrize("variant", ["gptq_f16_g128", "gptq_bf16_chan", "awq_bf16_g128"])
def test_top2_sum_epilogue_equals_separate_launches(dev, m, topk, e, bs, variant):
    """GEMM2 as fused_marlin_moe calls it: A is [m * topk, k] (one row per slot), top_k = 1, rows scaled by the routing
    weight; the fused epilogue adds slot rows 2t and 2t + 1 into row t of a zeroed output."""
    import vllm_amd.ops as ops
    k, n = (2048, 1024) if m == 2048 else (256, 192)
    dtype, _, tw, align, w, ws = _setup(dev, m, topk, e, bs, variant, k, n, seed=20)
    a = (torch.randn(m * topk, k, generator=torch.Generator().manual_seed(9)) / 4).to(dtype).to(dev)
    y = _plain(ops, a, w, ws, align, tw, bs, 1, True, m * topk, n, k)
    want = torch.empty(m, n, dtype=dtype, device=dev)
    ops.moe_sum(y.view(m, topk, n), want)
    got = torch.zeros(m, n, dtype=dtype, device=dev)
    _fused(ops, a, got, w, ws, align, tw, bs, 1, True, m * topk, n, k, sum_top_k=2)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert float(want.float().abs().max()) > 0 and int(ws.abs().sum()) == 0


@pytest.mark.parametrize("m,bs", [(3, 8), (100, 32), (700, 64)])
def test_zero_fill_side_job(dev, m, bs):
    """The launch clears the given buffer completely, whatever share of its workgroups exits early (blocks past the
    padded total, experts of other ranks), and leaves its neighbours alone."""
    import vllm_amd.ops as ops
    topk, e, k, d = 2, 8, 256, 128
    dtype, a, tw, align, w, ws = _setup(dev, m, topk, e, bs, "gptq_f16_g128", k, 2 * d, seed=30)
    s, x, t = align
    x = torch.where(x % 2 == 1, torch.full_like(x, -1), x)          # every second expert lives elsewhere
    buf = torch.full((m * k + 64,), 3.0, dtype=dtype, device=dev)
    target = buf[32:32 + m * k].view(m, k)
    got = torch.empty(m * topk, d, dtype=dtype, device=dev)
    _fused(ops, a, got, w, ws, (s, x, t), tw, bs, topk, False, m, 2 * d, k, silu_and_mul=True, zero_fill=target)
    torch.cuda.synchronize()
    assert float(target.abs().max()) == 0.0
    assert float(buf[:32].min()) == 3.0 and float(buf[32 + m * k:].min()) == 3.0


@pytest.mark.parametrize("m,e,topk", [(1, 8, 2), (40, 8, 2), (300, 4, 2), (1500, 4, 2), (77, 6, 3), (50, 4, 1)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_marlin_moe_fused_path_equals_general_path(dev, m, e, topk, dtype):
    """fused_marlin_moe takes the three-launch path by default; handing it the default activation and sum as
    caller-supplied callables forces the five-launch path.  Same bits either way (top-3 always runs the general path and
    checks that both spellings agree there too)."""
    import vllm_amd.ops as ops
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    k, inter = 512, 256
    l1, q1, s1, _, _, _ = make_experts(e, k, 2 * inter, 128, dtype, False, False, seed=100)
    l2, q2, s2, _, _, _ = make_experts(e, inter, k, 128, dtype, False, False, seed=200)
    g = torch.Generator().manual_seed(11)
    a = (torch.randn(m, k, generator=g) / 10).to(dtype).to(dev)
    tw, ti = torch.topk(torch.softmax(torch.randn(m, e, generator=g), dim=-1), topk)
    args = (a, q1.to(dev), q2.to(dev), None, None, s1.to(dev), s2.to(dev), None, tw.to(dev), ti.to(torch.int32).to(dev))
    fast = fused_marlin_moe(*args, quant_type_id=l1[0].type_id, global_num_experts=e)
    slow = fused_marlin_moe(*args, quant_type_id=l1[0].type_id, global_num_experts=e,
                            activation_func=lambda name, out, x: ops.silu_and_mul(out, x),
                            moe_sum=lambda x, out: (ops.moe_sum(x.contiguous(), out), out)[1])
    assert torch.equal(fast, slow)
    inplace_in = a.clone()
    assert fused_marlin_moe(inplace_in, *args[1:], quant_type_id=l1[0].type_id, global_num_experts=e, inplace=True) is inplace_in
    assert torch.equal(inplace_in, fast)


def test_fused_marlin_moe_expert_parallel_fused_path(dev):
    """expert_map sends every second expert elsewhere: their slots contribute nothing, output rows of tokens with no
    local expert are zero."""
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    from oracle import moe_ref as mr
    dtype, e, topk, m, k, inter = torch.float16, 8, 2, 90, 256, 128
    local = [0, 2, 4, 6]
    emap = torch.full((e,), -1, dtype=torch.int32)
    emap[local] = torch.arange(len(local), dtype=torch.int32)
    l1, q1, s1, _, _, _ = make_experts(e, k, 2 * inter, 128, dtype, False, False, seed=300)
    l2, q2, s2, _, _, _ = make_experts(e, inter, k, 128, dtype, False, False, seed=400)
    g = torch.Generator().manual_seed(12)
    a = (torch.randn(m, k, generator=g) / 10).to(dtype)
    tw, ti = torch.topk(torch.softmax(torch.randn(m, e, generator=g), dim=-1), topk)
    out = fused_marlin_moe(a.to(dev), q1[local].to(dev), q2[local].to(dev), None, None, s1[local].to(dev), s2[local].to(dev),
                           None, tw.to(dev), ti.to(torch.int32).to(dev), quant_type_id=l1[0].type_id,
                           global_num_experts=e, expert_map=emap.to(dev))
    w1 = torch.stack([l.w_ref.t() for l in l1])
    w2 = torch.stack([l.w_ref.t() for l in l2])
    mask = torch.isin(ti, torch.tensor(local))
    ref = mr.torch_experts(a, w1, w2, tw * mask, ti)
    torch.testing.assert_close(out.cpu().float(), ref.float(), atol=5e-2, rtol=0)


@pytest.mark.parametrize("scales", [(1e-6, 1e-6), (1.0, 3e-4), (1e-5, 5e-5), (6e-5, -6.1e-5), (300.0, 1e-6)])
@pytest.mark.parametrize("dtype_variant", ["gptq_f16_g128", "gptq_bf16_chan"])
def test_top2_sum_epilogue_rounding_on_tiny_and_mixed_rows(dev, scales, dtype_variant):
    """The fused top-2 sum adds rounded 16-bit rows with packed 16-bit atomic adds; moe_sum adds them in fp32 and rounds.
    Both are the correctly rounded sum of two 16-bit numbers as long as the atomic unit rounds to nearest even and keeps
    subnormals: rows scaled into the subnormal range of fp16, rows whose two terms are many binades apart, and terms that
    nearly cancel, must give the same bits."""
    import vllm_amd.ops as ops
    m, topk, e, bs, k, n = 64, 2, 4, 16, 256, 192
    dtype, _, tw, align, w, ws = _setup(dev, m, topk, e, bs, dtype_variant, k, n, seed=21)
    tw = torch.empty(m, topk)
    tw[:, 0], tw[:, 1] = scales
    tw = (tw * (1 + torch.rand(m, topk, generator=torch.Generator().manual_seed(8)) / 8)).to(dev)
    a = (torch.randn(m * topk, k, generator=torch.Generator().manual_seed(9)) / 4).to(dtype).to(dev)
    y = _plain(ops, a, w, ws, align, tw, bs, 1, True, m * topk, n, k)
    want = torch.empty(m, n, dtype=dtype, device=dev)
    ops.moe_sum(y.view(m, topk, n), want)
    got = torch.zeros(m, n, dtype=dtype, device=dev)
    _fused(ops, a, got, w, ws, align, tw, bs, 1, True, m * topk, n, k, sum_top_k=2)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert float(want.float().abs().max()) > 0
    if dtype == torch.float16 and max(abs(s) for s in scales) < 1e-4:
        sub = (want.float().abs() < 6.1e-5) & (want != 0)          # subnormal results are what this case is about
        assert float(sub.float().mean()) > 0.5


@pytest.mark.parametrize("inter,strided", [(96, False), (128, True), (96, True)])
def test_fused_marlin_moe_falls_back_when_the_fused_epilogues_do_not_apply(dev, inter, strided):
    """An intermediate size that is not a multiple of 64 (no gate / up n-tile pairing) and a strided `output` must take
    the separate-launch path instead of failing the operator's argument checks."""
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    from oracle import moe_ref as mr
    dtype, e, topk, m, k = torch.float16, 4, 2, 50, 256
    l1, q1, s1, _, _, _ = make_experts(e, k, 2 * inter, 128, dtype, False, False, seed=500)
    l2, q2, s2, _, _, _ = make_experts(e, inter, k, 32, dtype, False, False, seed=600)
    g = torch.Generator().manual_seed(13)
    a = (torch.randn(m, k, generator=g) / 10).to(dtype)
    tw, ti = torch.topk(torch.softmax(torch.randn(m, e, generator=g), dim=-1), topk)
    out = torch.zeros(m, 2 * k, dtype=dtype, device=dev)[:, ::2] if strided else None
    res = fused_marlin_moe(a.to(dev), q1.to(dev), q2.to(dev), None, None, s1.to(dev), s2.to(dev), None, tw.to(dev),
                           ti.to(torch.int32).to(dev), quant_type_id=l1[0].type_id, global_num_experts=e, output=out)
    if strided:
        assert res is out
    w1 = torch.stack([l.w_ref.t() for l in l1])
    w2 = torch.stack([l.w_ref.t() for l in l2])
    ref = mr.torch_experts(a, w1, w2, tw, ti)
    torch.testing.assert_close(res.cpu().float(), ref.float(), atol=5e-2, rtol=0)
