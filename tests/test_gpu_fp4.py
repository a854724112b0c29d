"""float4_e2m1f weights on gptq_marlin_gemm: NVFP4 (group 16, float8_e4m3fn scales + global scale) and MXFP4
(group 32, E8M0 scales, bf16), as the reference's test grid feeds them
(tests/kernels/quantization/test_marlin_gemm.py:262-277 via rand_marlin_weight_{nvfp4,mxfp4}_like)."""
import pytest
import torch

from oracle import gemm_ref as gr

pytestmark = pytest.mark.gpu

MNK_FACTORS = [(1, 1, 1), (1, 4, 8), (1, 7, 5), (13, 17, 67), (26, 37, 13), (67, 13, 11), (257, 13, 11), (658, 13, 11)]
TOL = {torch.float16: 2e-2, torch.bfloat16: 4e-2}


@pytest.fixture(scope="module")
def ops():
    import vllm_amd.ops as o
    return o


@pytest.fixture(scope="module")
def workspace(dev):
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    return marlin_make_workspace_new(dev)


def make(kind, size_k, size_n, dtype, dev, seed):
    """Operands from the host mirror of the reference's random-weight helpers; w from the oracle's decode of the very
    tensors the op receives."""
    from vllm_amd import marlin_utils_fp4 as f4
    torch.manual_seed(seed)
    weight = torch.randn(size_n, size_k, dtype=dtype, device=dev)
    if kind == "nvfp4":
        w_helper, mq, ms, gs = f4.rand_marlin_weight_nvfp4_like(weight, 16)
    else:
        w_helper, mq, ms = f4.rand_marlin_weight_mxfp4_like(weight, 32)
        gs = None
    w = gr.dequant_marlin_fp4(mq.cpu(), ms.cpu().view(torch.uint8), None if gs is None else gs.cpu().view(1), size_k, size_n,
                              dtype)
    return w, w_helper, mq, ms, None if gs is None else gs.view(1)


def run(ops, a, mq, ms, gs, workspace, size_n, size_k, bias=None):
    import vllm_amd.scalar_type as vst
    return ops.gptq_marlin_gemm(a, None, mq, bias, ms, gs, None, None, None, workspace, vst.scalar_types.float4_e2m1f,
                                a.shape[0], size_n, size_k, is_k_full=True, use_fp32_reduce=True)


@pytest.mark.parametrize("kind,dtype", [("nvfp4", torch.float16), ("nvfp4", torch.bfloat16), ("mxfp4", torch.bfloat16)])
@pytest.mark.parametrize("size_m", [1, 16, 40])
def test_one_hot_rows_reproduce_the_decoded_weights(ops, dev, workspace, kind, dtype, size_m):
    size_k, size_n = 256, 192
    w, w_helper, mq, ms, gs = make(kind, size_k, size_n, dtype, dev, 3)
    # the helper's left-to-right product rounds twice: within one unit in the last place of the oracle
    assert ((w.double() - w_helper.cpu().double()).abs() <= w.double().abs() * torch.finfo(dtype).eps).all()
    rows = torch.randperm(size_k, generator=torch.Generator().manual_seed(size_m))[:size_m]
    a = torch.zeros(size_m, size_k, dtype=dtype)
    a[torch.arange(size_m), rows] = 1.0
    out = run(ops, a.to(dev), mq, ms, gs, workspace, size_n, size_k)
    assert torch.equal(out.cpu(), w[rows])
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("kind,dtype", [("nvfp4", torch.float16), ("nvfp4", torch.bfloat16), ("mxfp4", torch.bfloat16)])
@pytest.mark.parametrize("n_chunk", [64, 256])
@pytest.mark.parametrize("mnk", MNK_FACTORS)
def test_reference_grid(ops, dev, workspace, kind, dtype, n_chunk, mnk):
    mf, nf, kf = mnk
    size_m, size_k, size_n = mf, 128 * kf, n_chunk * nf
    print(f"fp4 grid {kind} dtype={dtype} m={size_m} n={size_n} k={size_k}", flush=True)
    w, w_helper, mq, ms, gs = make(kind, size_k, size_n, dtype, dev, 11 + mf)
    a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(2)).to(dtype)
    out = run(ops, a.to(dev), mq, ms, gs, workspace, size_n, size_k).cpu()
    m = gr.error_metrics(out, gr.gemm_ref(a, w))
    assert m["max_rel"] <= TOL[dtype] and m["mean_rel"] < 0.04, m
    # the reference's own check: mean|d| / mean|ref| < 0.04 against matmul(a, w_ref) of the helper
    ref = torch.matmul(a.float(), w_helper.cpu().float())
    assert float((out.float() - ref).abs().mean() / ref.abs().mean()) < 0.04


@pytest.mark.parametrize("kind,dtype", [("nvfp4", torch.float16), ("nvfp4", torch.bfloat16), ("mxfp4", torch.bfloat16)])
def test_prefill_tiles(ops, dev, workspace, kind, dtype):
    """Enough 128-row tiles for the prefill kernel, with a partial row tile and a partial 512-column strip: random
    activations against the oracle, one-hot rows bit-exact."""
    size_m, size_k, size_n = 1100, 512, 8256
    print(f"fp4 prefill {kind} dtype={dtype}", flush=True)
    w, _, mq, ms, gs = make(kind, size_k, size_n, dtype, dev, 9)
    a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(2)).to(dtype)
    out = run(ops, a.to(dev), mq, ms, gs, workspace, size_n, size_k).cpu()
    m = gr.error_metrics(out, gr.gemm_ref(a, w))
    assert m["max_rel"] <= TOL[dtype] and m["mean_rel"] < 0.04, m
    rows = torch.randint(0, size_k, (size_m,), generator=torch.Generator().manual_seed(5))
    hot = torch.zeros(size_m, size_k, dtype=dtype)
    hot[torch.arange(size_m), rows] = 1.0
    out = run(ops, hot.to(dev), mq, ms, gs, workspace, size_n, size_k)
    assert torch.equal(out.cpu(), w[rows])
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("kind,dtype", [("nvfp4", torch.float16), ("mxfp4", torch.bfloat16)])
def test_64_row_tiles_with_split_k(ops, dev, workspace, kind, dtype):
    """136 tiles of 64 x 512: the 64-row kernel splits K in two and a second kernel adds the partial tiles (and applies
    NVFP4's global scale)."""
    size_m, size_k, size_n = 512, 2048, 8704
    w, _, mq, ms, gs = make(kind, size_k, size_n, dtype, dev, 23)
    a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(2)).to(dtype)
    out = run(ops, a.to(dev), mq, ms, gs, workspace, size_n, size_k).cpu()
    m = gr.error_metrics(out, gr.gemm_ref(a, w))
    assert m["max_rel"] <= TOL[dtype] and m["mean_rel"] < 0.04, m
    rows = torch.randint(0, size_k, (size_m,), generator=torch.Generator().manual_seed(5))
    hot = torch.zeros(size_m, size_k, dtype=dtype)
    hot[torch.arange(size_m), rows] = 1.0
    out = run(ops, hot.to(dev), mq, ms, gs, workspace, size_n, size_k)
    assert torch.equal(out.cpu(), w[rows])
    assert int(workspace.abs().sum()) == 0


def test_linear_helpers_and_bias(ops, dev, workspace):
    from vllm_amd import marlin_utils_fp4 as f4
    from vllm_amd.marlin_utils import marlin_permute_bias
    size_k, size_n = 512, 256
    for kind, dtype in (("nvfp4", torch.float16), ("mxfp4", torch.bfloat16)):
        w, _, mq, ms, gs = make(kind, size_k, size_n, dtype, dev, 6)
        x = torch.randn(2, 5, size_k, generator=torch.Generator().manual_seed(7)).to(dtype)
        bias = torch.randn(size_n, generator=torch.Generator().manual_seed(8)).to(dtype)
        out = f4.apply_fp4_marlin_linear(x.to(dev), mq, ms, gs, workspace, size_n, size_k, marlin_permute_bias(bias.to(dev)))
        assert out.shape == (2, 5, size_n)
        m = gr.error_metrics(out.cpu().view(10, size_n), gr.gemm_ref(x.view(10, size_k), w, bias))
        assert m["max_rel"] <= TOL[dtype], m


def test_argument_errors(ops, dev, workspace):
    import vllm_amd.scalar_type as vst
    size_k, size_n = 256, 128
    _, _, mq, ms, gs = make("nvfp4", size_k, size_n, torch.float16, dev, 9)
    a = torch.randn(4, size_k).half().to(dev)
    fp4 = vst.scalar_types.float4_e2m1f
    with pytest.raises(RuntimeError, match="global_scale parameter must be passed"):
        ops.gptq_marlin_gemm(a, None, mq, None, ms, None, None, None, None, workspace, fp4, 4, size_n, size_k)
    with pytest.raises(RuntimeError, match="b_scales must be"):
        ops.gptq_marlin_gemm(a, None, mq, None, ms.view(torch.uint8).half(), gs, None, None, None, workspace, fp4, 4,
                             size_n, size_k)
    _, _, mq2, ms2, _ = make("mxfp4", size_k, size_n, torch.bfloat16, dev, 9)
    with pytest.raises(RuntimeError, match="bfloat16"):       # MXFP4 with fp16 activations
        ops.gptq_marlin_gemm(a, None, mq2, None, ms2, None, None, None, None, workspace, fp4, 4, size_n, size_k)
    with pytest.raises(RuntimeError, match="only be used for nvfp4"):
        ops.gptq_marlin_gemm(a.bfloat16(), None, mq2, None, ms2, gs.bfloat16(), None, None, None, workspace, fp4, 4,
                             size_n, size_k)
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("kind,dtype", [("nvfp4", torch.float16), ("nvfp4", torch.bfloat16), ("mxfp4", torch.bfloat16)])
# (600 tokens in blocks of 8: more 16-row tiles than compute units, the 4-wavefront form of the general kernel)
@pytest.mark.parametrize("m,topk,e,bs", [(3, 2, 4, 8), (123, 2, 4, 32), (333, 2, 4, 64), (600, 2, 4, 8)])
def test_moe_gemm_fp4_experts(ops, dev, kind, dtype, m, topk, e, bs):
    """Per-expert weights, scale bytes and (NVFP4) global scales through moe_wna16_marlin_gemm."""
    from oracle import moe_ref as mr
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    k, n = 256, 192
    experts = [make(kind, k, n, dtype, dev, 40 + i) for i in range(e)]
    mq, ms = torch.stack([x[2] for x in experts]), torch.stack([x[3] for x in experts])
    gs = torch.cat([x[4] for x in experts]) if kind == "nvfp4" else None
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(5)).to(dtype)
    g = torch.Generator().manual_seed(6)
    ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    tw = torch.rand(m, topk, generator=g)
    s, x, t = moe_align_block_size(ids.to(dev), bs, e)
    ws = marlin_make_workspace_new(dev, 4)
    out = ops.moe_wna16_marlin_gemm(
        a.to(dev), None, mq, None, ms, gs, None, None, None, ws, s, x, t, tw.to(dev), moe_block_size=bs, top_k=topk,
        mul_topk_weights=True, is_ep=False, b_q_type=scalar_types.float4_e2m1f, size_m=m, size_n=n, size_k=k,
        is_k_full=True, use_atomic_add=False, use_fp32_reduce=True, is_zp_float=False)
    ref = mr.moe_gemm_ref(a, torch.stack([x[0] for x in experts]), s.cpu(), x.cpu(), t.cpu(), tw, bs, topk, True, m)
    mtr = gr.error_metrics(out, ref)
    assert mtr["max_rel"] <= TOL[dtype] and mtr["mean_rel"] < 0.04, mtr
    assert int(ws.abs().sum()) == 0


@pytest.mark.parametrize("kind,dtype", [("nvfp4", torch.float16), ("mxfp4", torch.bfloat16), ("fp8", torch.bfloat16)])
@pytest.mark.parametrize("m", [1, 33, 200])
def test_fused_marlin_moe_with_float_weight_types(dev, kind, dtype, m):
    """fused_marlin_moe end to end (align, GEMM1, SiLU-and-mul, GEMM2, sum) with fp4 / fp8 experts and per-expert
    global scales, against torch_experts on the oracle's dequantised weights (the reference's gate: atol 5e-2)."""
    from oracle import marlin_layout as ml
    from oracle import moe_ref as mr
    from oracle import quant_utils as qu
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    from vllm_amd.scalar_type import scalar_types
    e, topk, k, inter = 4, 2, 256, 128

    def experts(size_k, size_n, seed):
        if kind == "fp8":
            ws, qs, ss = [], [], []
            for i in range(e):
                w = (torch.randn(size_k, size_n, generator=torch.Generator().manual_seed(seed + i)) * 0.1).to(dtype)
                w_ref, codes, s = qu.quantize_fp8(w, 128)
                ms = ml.marlin_permute_scales(s, size_k, size_n, 128)
                ws.append(w_ref)
                qs.append(ml.marlin_weights_closed_form8(codes.to(torch.int32)))
                ss.append((ms.double() * gr.fp8_scale_offset(dtype)).to(dtype))
            return torch.stack(ws), torch.stack(qs).to(dev), torch.stack(ss).to(dev), None
        made = [make(kind, size_k, size_n, dtype, dev, seed + i) for i in range(e)]
        gs = torch.cat([x[4] for x in made]) if kind == "nvfp4" else None
        return torch.stack([x[0] for x in made]), torch.stack([x[2] for x in made]), torch.stack([x[3] for x in made]), gs

    w1, q1, s1, g1 = experts(k, 2 * inter, 300)
    w2, q2, s2, g2 = experts(inter, k, 400)
    g = torch.Generator().manual_seed(12)
    a_scale = 0.1 if kind == "fp8" else 0.01
    a = (torch.randn(m, k, generator=g) * a_scale).to(dtype)
    score = torch.randn(m, e, generator=g).to(dtype)
    tw, ti = torch.topk(torch.softmax(score.float(), dim=-1), topk)
    wtype = scalar_types.float8_e4m3fn if kind == "fp8" else scalar_types.float4_e2m1f
    out = fused_marlin_moe(a.to(dev), q1, q2, None, None, s1, s2, score.to(dev), tw.to(dev), ti.to(torch.int32).to(dev),
                           quant_type_id=wtype.id, global_num_experts=e, global_scale1=g1, global_scale2=g2)
    ref = mr.torch_experts(a, w1.transpose(1, 2), w2.transpose(1, 2), tw, ti)
    assert out.shape == (m, k)
    torch.testing.assert_close(out.cpu().float(), ref.float(), atol=max(5e-2, 2e-2 * float(ref.abs().max())), rtol=0)
    mtr = gr.error_metrics(out, ref)          # and relative to the result's own size (two GEMMs and a 16-bit intermediate)
    assert mtr["max_rel"] <= 2 * TOL[dtype] and mtr["mean_rel"] < 0.04, mtr
