"""float8_e4m3fn weights (W8A16-fp8) on gptq_marlin_gemm, as the reference's test grid feeds them
(tests/kernels/quantization/test_marlin_gemm.py:280-289: group sizes -1 and 128, no act-order)."""
import pytest
import torch

from oracle import gemm_ref as gr
from oracle import marlin_layout as ml
from oracle import quant_utils as qu

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


def make_fp8(size_k, size_n, group, dtype, seed, w_std=1.0):
    w = (torch.randn(size_k, size_n, generator=torch.Generator().manual_seed(seed)) * w_std).to(dtype)
    w_ref, codes, s = qu.quantize_fp8(w, group)
    mq = ml.marlin_weights_closed_form8(codes.to(torch.int32))
    ms = ml.marlin_permute_scales(s, size_k, size_n, size_k if group == -1 else group)
    ms = (ms.double() * gr.fp8_scale_offset(dtype)).to(dtype)
    return w_ref, codes, mq, ms


def run(ops, a, mq, ms, workspace, size_n, size_k, bias=None):
    import vllm_amd.scalar_type as vst
    dev = a.device
    return ops.gptq_marlin_gemm(a, None, mq.to(dev), bias, ms.to(dev), None, None, None, None, workspace,
                                vst.scalar_types.float8_e4m3fn, a.shape[0], size_n, size_k, is_k_full=True,
                                use_fp32_reduce=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [-1, 128])
@pytest.mark.parametrize("size_m", [1, 16, 40])
def test_one_hot_rows_reproduce_w_ref(ops, dev, workspace, dtype, group, size_m):
    size_k, size_n = 256, 192
    w_ref, _, mq, ms = make_fp8(size_k, size_n, group, dtype, 4)
    rows = torch.randperm(size_k, generator=torch.Generator().manual_seed(size_m))[:size_m]
    a = torch.zeros(size_m, size_k, dtype=dtype)
    a[torch.arange(size_m), rows] = 1.0
    out = run(ops, a.to(dev), mq, ms, workspace, size_n, size_k)
    assert torch.equal(out.cpu(), w_ref[rows])
    assert int(workspace.abs().sum()) == 0


def test_every_fp8_code_is_decoded_exactly(ops, dev, workspace):
    """All 254 finite codes, unit scales, one-hot rows: the output is the code's value."""
    size_k, size_n = 256, 64
    codes = torch.arange(256, dtype=torch.int32).view(256, 1).expand(256, size_n).contiguous()
    codes[codes & 0x7F == 0x7F] = 0                           # the two NaN codes
    mq = ml.marlin_weights_closed_form8(codes)
    s = torch.ones(1, size_n, dtype=torch.float16)
    ms = (ml.marlin_permute_scales(s, size_k, size_n, size_k).double() * gr.fp8_scale_offset(torch.float16)).half()
    a = torch.eye(size_k, dtype=torch.float16)
    out = run(ops, a.to(dev), mq, ms, workspace, size_n, size_k).cpu()
    want = gr.fp8_e4m3fn_table()[codes.long()].half()
    assert torch.equal(out, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [-1, 128])
@pytest.mark.parametrize("n_chunk", [64, 256])
@pytest.mark.parametrize("mnk", MNK_FACTORS)
def test_reference_grid(ops, dev, workspace, dtype, group, n_chunk, mnk):
    mf, nf, kf = mnk
    size_m, size_k, size_n = mf, 128 * kf, n_chunk * nf
    print(f"fp8 grid dtype={dtype} g={group} m={size_m} n={size_n} k={size_k}", flush=True)
    w_ref, _, mq, ms = make_fp8(size_k, size_n, group, dtype, 11 + mf)
    a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(2)).to(dtype)
    out = run(ops, a.to(dev), mq, ms, workspace, size_n, size_k).cpu()
    m = gr.error_metrics(out, gr.gemm_ref(a, w_ref))
    assert m["max_rel"] <= TOL[dtype] and m["mean_rel"] < 0.04, m


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [-1, 128])
def test_prefill_tiles(ops, dev, workspace, dtype, group):
    """Enough 128-row tiles for the prefill kernel, with a partial row tile and a partial 512-column strip: random
    activations against the oracle, one-hot rows bit-exact."""
    size_m, size_k, size_n = 1100, 512, 8256
    print(f"fp8 prefill dtype={dtype} g={group}", flush=True)
    w_ref, _, mq, ms = make_fp8(size_k, size_n, group, dtype, 17)
    a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(2)).to(dtype)
    out = run(ops, a.to(dev), mq, ms, workspace, size_n, size_k).cpu()
    m = gr.error_metrics(out, gr.gemm_ref(a, w_ref))
    assert m["max_rel"] <= TOL[dtype] and m["mean_rel"] < 0.04, m
    rows = torch.randint(0, size_k, (size_m,), generator=torch.Generator().manual_seed(5))
    hot = torch.zeros(size_m, size_k, dtype=dtype)
    hot[torch.arange(size_m), rows] = 1.0
    out = run(ops, hot.to(dev), mq, ms, workspace, size_n, size_k)
    assert torch.equal(out.cpu(), w_ref[rows])
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("dtype,group", [(torch.float16, -1), (torch.bfloat16, 128)])
def test_64_row_tiles_with_split_k(ops, dev, workspace, dtype, group):
    """136 tiles of 64 x 512: the 64-row kernel splits K in two and a second kernel adds the partial tiles (and, with
    channel-wise scales, takes the exponent offset out of them)."""
    size_m, size_k, size_n = 512, 2048, 8704
    w_ref, _, mq, ms = make_fp8(size_k, size_n, group, dtype, 19)
    a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(2)).to(dtype)
    out = run(ops, a.to(dev), mq, ms, workspace, size_n, size_k).cpu()
    m = gr.error_metrics(out, gr.gemm_ref(a, w_ref))
    assert m["max_rel"] <= TOL[dtype] and m["mean_rel"] < 0.04, m
    rows = torch.randint(0, size_k, (size_m,), generator=torch.Generator().manual_seed(5))
    hot = torch.zeros(size_m, size_k, dtype=dtype)
    hot[torch.arange(size_m), rows] = 1.0
    out = run(ops, hot.to(dev), mq, ms, workspace, size_n, size_k)
    assert torch.equal(out.cpu(), w_ref[rows])
    assert int(workspace.abs().sum()) == 0


def test_host_helpers_match_the_oracle(ops, dev, workspace):
    """marlin_quant_fp8_torch (repack op + scale permutation + exponent offset) against the oracle's tensors, and
    apply_fp8_marlin_linear with a bias."""
    from vllm_amd.marlin_utils import marlin_permute_bias
    from vllm_amd.marlin_utils_fp8 import apply_fp8_marlin_linear, marlin_quant_fp8_torch
    size_k, size_n = 512, 256
    for dtype, group in ((torch.float16, 128), (torch.bfloat16, -1)):
        w = torch.randn(size_k, size_n, generator=torch.Generator().manual_seed(6)).to(dtype)
        w_ref_o, codes, s = qu.quantize_fp8(w, group)
        w_ref, mq, ms = marlin_quant_fp8_torch(w.t().contiguous().to(dev), group)
        assert torch.equal(w_ref.cpu(), w_ref_o)
        assert torch.equal(mq.cpu(), ml.marlin_weights_closed_form8(codes.to(torch.int32)))
        ms_o = ml.marlin_permute_scales(s, size_k, size_n, size_k if group == -1 else group)
        assert torch.equal(ms.cpu(), (ms_o.double() * gr.fp8_scale_offset(dtype)).to(dtype))
        x = torch.randn(2, 5, size_k, generator=torch.Generator().manual_seed(7)).to(dtype)
        bias = torch.randn(size_n, generator=torch.Generator().manual_seed(8)).to(dtype)
        out = apply_fp8_marlin_linear(x.to(dev), mq, ms, workspace, size_n, size_k, marlin_permute_bias(bias.to(dev)))
        assert out.shape == (2, 5, size_n)
        m = gr.error_metrics(out.cpu().view(10, size_n), gr.gemm_ref(x.view(10, size_k), w_ref_o, bias))
        assert m["max_rel"] <= TOL[dtype], m


def test_act_order_is_rejected(ops, dev, workspace):
    import vllm_amd.scalar_type as vst
    size_k, size_n = 256, 128
    _, _, mq, ms = make_fp8(size_k, size_n, 128, torch.float16, 1)
    a = torch.randn(4, size_k).half().to(dev)
    idx = torch.arange(size_k, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="Unsupported shapes"):
        ops.gptq_marlin_gemm(a, None, mq.to(dev), None, ms.to(dev), None, None, idx // 128, idx, workspace,
                             vst.scalar_types.float8_e4m3fn, 4, size_n, size_k)


# (600 tokens in blocks of 8: more 16-row tiles than compute units, the 4-wavefront form of the general kernel)
@pytest.mark.parametrize("m,topk,e,bs", [(3, 2, 4, 8), (123, 2, 4, 32), (333, 2, 4, 64), (600, 2, 4, 8)])
@pytest.mark.parametrize("dtype,group", [(torch.float16, 128), (torch.bfloat16, -1)])
def test_moe_gemm_fp8_experts(ops, dev, m, topk, e, bs, dtype, group):
    from oracle import moe_ref as mr
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    k, n = 256, 192
    experts = [make_fp8(k, n, group, dtype, 30 + i, w_std=0.1) for i in range(e)]
    mq, ms = torch.stack([x[2] for x in experts]), torch.stack([x[3] for x in experts])
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(5)).to(dtype)
    g = torch.Generator().manual_seed(6)
    ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    tw = torch.rand(m, topk, generator=g)
    s, x, t = moe_align_block_size(ids.to(dev), bs, e)
    ws = marlin_make_workspace_new(dev, 4)
    out = ops.moe_wna16_marlin_gemm(
        a.to(dev), None, mq.to(dev), None, ms.to(dev), None, None, None, None, ws, s, x, t, tw.to(dev),
        moe_block_size=bs, top_k=topk, mul_topk_weights=True, is_ep=False, b_q_type=scalar_types.float8_e4m3fn,
        size_m=m, size_n=n, size_k=k, is_k_full=True, use_atomic_add=False, use_fp32_reduce=True, is_zp_float=False)
    ref = mr.moe_gemm_ref(a, torch.stack([x[0] for x in experts]), s.cpu(), x.cpu(), t.cpu(), tw, bs, topk, True, m)
    mtr = gr.error_metrics(out, ref)
    assert mtr["max_rel"] <= TOL[dtype] and mtr["mean_rel"] < 0.04, mtr
    assert int(ws.abs().sum()) == 0
