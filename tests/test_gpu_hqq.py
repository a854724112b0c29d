"""Float zero points (HQQ: uint4 weights, fp16 scales and fp16 zero points, group 64) on gptq_marlin_gemm,
laid out as the reference's test does (tests/kernels/quantization/test_marlin_gemm.py:463-535)."""
import pytest
import torch

from oracle import gemm_ref as gr
from oracle import marlin_layout as ml
from oracle import quant_utils as qu

pytestmark = pytest.mark.gpu

MNK_FACTORS = [(1, 1, 1), (1, 4, 8), (1, 7, 5), (13, 17, 67), (26, 37, 13), (67, 13, 11), (257, 13, 11), (658, 13, 11)]


@pytest.fixture(scope="module")
def ops():
    import vllm_amd.ops as o
    return o


@pytest.fixture(scope="module")
def workspace(dev):
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    return marlin_make_workspace_new(dev)


def make_hqq(size_k, size_n, seed):
    """Operands as the reference test draws them: weights in [0, 10), scale and zero ~ N(0, 1) per (column, group)."""
    g = torch.Generator().manual_seed(seed)
    b_weight = torch.randint(0, 10, (size_n, size_k), generator=g, dtype=torch.uint8)
    scale = torch.randn(size_n, size_k // 64, generator=g).half()
    zero = torch.randn(size_n, size_k // 64, generator=g).half()
    q = b_weight.t().contiguous().to(torch.int32)
    mq = ml.gptq_marlin_repack(qu.gptq_pack(q), None, size_k, size_n)
    ms = ml.marlin_permute_scales(scale.t().contiguous(), size_k, size_n, 64)
    mz = ml.marlin_permute_scales(zero.t().contiguous(), size_k, size_n, 64)
    return b_weight, scale, zero, mq, ms, mz


def run(ops, a, mq, ms, mz, workspace, size_n, size_k, **kw):
    import vllm_amd.scalar_type as vst
    dev = a.device
    e = torch.empty(0, dtype=torch.int32, device=dev)
    return ops.gptq_marlin_gemm(a, None, mq.to(dev), None, ms.to(dev), None, mz.to(dev), e, e, workspace,
                                vst.scalar_types.uint4, a.shape[0], size_n, size_k, is_k_full=True,
                                use_fp32_reduce=True, is_zp_float=True, **kw)


@pytest.mark.parametrize("size_m", [1, 16, 33, 64])
def test_one_hot_rows_reproduce_the_dequantised_weights(ops, dev, workspace, size_m):
    size_k, size_n = 256, 192
    _, _, _, mq, ms, mz = make_hqq(size_k, size_n, 3)
    w = gr.dequant_marlin_float_zp(mq, ms, mz, size_k, size_n)
    rows = torch.randperm(size_k, generator=torch.Generator().manual_seed(size_m))[:size_m]
    a = torch.zeros(size_m, size_k, dtype=torch.float16)
    a[torch.arange(size_m), rows] = 1.0
    out = run(ops, a.to(dev), mq, ms, mz, workspace, size_n, size_k)
    assert torch.equal(out.cpu(), w[rows])
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("n_chunk", [64, 256])
@pytest.mark.parametrize("mnk", MNK_FACTORS)
def test_reference_grid(ops, dev, workspace, n_chunk, mnk):
    mf, nf, kf = mnk
    size_m, size_k, size_n = mf, 128 * kf, n_chunk * nf
    print(f"hqq grid m={size_m} n={size_n} k={size_k}", flush=True)
    b_weight, scale, zero, mq, ms, mz = make_hqq(size_k, size_n, 7 + mf)
    a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(1)).half()
    out = run(ops, a.to(dev), mq, ms, mz, workspace, size_n, size_k).cpu()
    m = gr.error_metrics(out, gr.gemm_ref(a, gr.dequant_marlin_float_zp(mq, ms, mz, size_k, size_n)))
    assert m["max_rel"] <= 2e-2 and m["mean_rel"] < 0.04, m
    # the reference's own check: mean|d| / mean|ref| < 0.04 against (q - zero) * scale in fp16
    ref = torch.matmul(a.float(), gr.float_zp_test_ref(b_weight, scale, zero, 64).float())
    assert float((out.float() - ref).abs().mean() / ref.abs().mean()) < 0.04


def test_llama_shape_decode_and_prefill_rows(ops, dev, workspace):
    size_k, size_n = 4096, 4096
    _, _, _, mq, ms, mz = make_hqq(size_k, size_n, 5)
    w = gr.dequant_marlin_float_zp(mq, ms, mz, size_k, size_n)
    for size_m in (16, 300):
        a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(size_m)).half()
        out = run(ops, a.to(dev), mq, ms, mz, workspace, size_n, size_k).cpu()
        m = gr.error_metrics(out, gr.gemm_ref(a, w))
        assert m["max_rel"] <= 2e-2 and m["mean_rel"] < 0.04, (size_m, m)


def test_prefill_tiles(ops, dev, workspace):
    """Enough 128-row tiles for the prefill kernel, with a partial row tile and a partial 512-column strip: random
    activations against the oracle, one-hot rows bit-exact."""
    size_m, size_k, size_n = 1100, 512, 8256
    _, _, _, mq, ms, mz = make_hqq(size_k, size_n, 13)
    w = gr.dequant_marlin_float_zp(mq, ms, mz, size_k, size_n)
    a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(2)).half()
    out = run(ops, a.to(dev), mq, ms, mz, workspace, size_n, size_k).cpu()
    m = gr.error_metrics(out, gr.gemm_ref(a, w))
    assert m["max_rel"] <= 2e-2 and m["mean_rel"] < 0.04, m
    rows = torch.randint(0, size_k, (size_m,), generator=torch.Generator().manual_seed(5))
    hot = torch.zeros(size_m, size_k, dtype=torch.float16)
    hot[torch.arange(size_m), rows] = 1.0
    out = run(ops, hot.to(dev), mq, ms, mz, workspace, size_n, size_k)
    assert torch.equal(out.cpu(), w[rows])
    assert int(workspace.abs().sum()) == 0


def test_64_row_tiles_with_split_k(ops, dev, workspace):
    """136 tiles of 64 x 512: the 64-row kernel splits K in two and a second kernel adds the partial tiles."""
    size_m, size_k, size_n = 512, 2048, 8704
    _, _, _, mq, ms, mz = make_hqq(size_k, size_n, 14)
    w = gr.dequant_marlin_float_zp(mq, ms, mz, size_k, size_n)
    a = torch.randn(size_m, size_k, generator=torch.Generator().manual_seed(2)).half()
    out = run(ops, a.to(dev), mq, ms, mz, workspace, size_n, size_k).cpu()
    m = gr.error_metrics(out, gr.gemm_ref(a, w))
    assert m["max_rel"] <= 2e-2 and m["mean_rel"] < 0.04, m
    rows = torch.randint(0, size_k, (size_m,), generator=torch.Generator().manual_seed(5))
    hot = torch.zeros(size_m, size_k, dtype=torch.float16)
    hot[torch.arange(size_m), rows] = 1.0
    out = run(ops, hot.to(dev), mq, ms, mz, workspace, size_n, size_k)
    assert torch.equal(out.cpu(), w[rows])
    assert int(workspace.abs().sum()) == 0


def test_argument_errors(ops, dev, workspace):
    import vllm_amd.scalar_type as vst
    size_k, size_n = 256, 128
    _, _, _, mq, ms, mz = make_hqq(size_k, size_n, 9)
    e = torch.empty(0, dtype=torch.int32, device=dev)
    a = torch.randn(4, size_k).to(dev)
    with pytest.raises(RuntimeError, match="float16"):           # bf16 activations
        ops.gptq_marlin_gemm(a.bfloat16(), None, mq.to(dev), None, ms.bfloat16().to(dev), None, mz.bfloat16().to(dev), e, e,
                             workspace, vst.scalar_types.uint4, 4, size_n, size_k, is_zp_float=True)
    with pytest.raises(RuntimeError, match="b_zeros dim 1"):     # packed integer zero points passed as float ones
        ops.gptq_marlin_gemm(a.half(), None, mq.to(dev), None, ms.to(dev), None, mz[:, :size_n // 8].contiguous().to(dev),
                             e, e, workspace, vst.scalar_types.uint4, 4, size_n, size_k, is_zp_float=True)
    with pytest.raises(RuntimeError, match="Unsupported shapes"):  # group size 128
        ops.gptq_marlin_gemm(a.half(), None, mq.to(dev), None, ms[:2].contiguous().to(dev), None, mz[:2].contiguous().to(dev),
                             e, e, workspace, vst.scalar_types.uint4, 4, size_n, size_k, is_zp_float=True)
    assert int(workspace.abs().sum()) == 0
