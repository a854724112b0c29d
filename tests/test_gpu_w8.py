"""uint8b128 (W8A16) on the same operator surface: repack bit-exact, GEMM against the CPU oracle."""
import pytest
import torch

from helpers import check_close, make_layer, run_gemm
from oracle import marlin_layout as ml
from oracle import quant_utils as qu

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import vllm_amd.ops as o
    return o


@pytest.fixture(scope="module")
def workspace(dev):
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    return marlin_make_workspace_new(dev)


@pytest.mark.parametrize("k,n", [(16, 64), (128, 192), (1024, 512)])
@pytest.mark.parametrize("act_order", [False, True])
def test_repack8_bit_exact(ops, dev, k, n, act_order):
    g = torch.Generator().manual_seed(k + n)
    q = torch.randint(0, 256, (k, n), generator=g, dtype=torch.int32)
    perm = torch.randperm(k, generator=g).to(torch.int32) if act_order else torch.empty(0, dtype=torch.int32)
    got = ops.gptq_marlin_repack(qu.pack_rows(q, 8).to(dev), perm.to(dev), k, n, 8)
    assert got.shape == (k // 16, 4 * n)
    assert torch.equal(got.cpu(), ml.gptq_marlin_repack(qu.pack_rows(q, 8), perm, k, n, 8))
    if not act_order:
        got = ops.awq_marlin_repack(qu.awq_pack(q, 8).to(dev), k, n, 8)
        assert torch.equal(got.cpu(), ml.marlin_weights_closed_form8(q))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [-1, 32, 128])
def test_one_hot_rows_are_exact_w8(ops, dev, workspace, dtype, group):
    k, n = 512, 192
    layer = make_layer(k, n, group, dtype, seed=3, bits=8)
    ks = torch.randperm(k, generator=torch.Generator().manual_seed(1))[:40]
    a = torch.zeros(40, k, dtype=dtype)
    a[torch.arange(40), ks] = 1.0
    out = run_gemm(ops, layer, a.to(dev), dev, workspace)
    assert torch.equal(out.cpu(), layer.w_ref[ks])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [-1, 128])
def test_wide_layer_more_tiles_than_compute_units_w8(ops, dev, workspace, dtype, group):
    """N / 128 = 300 column tiles of 16 rows: the general kernel's 4-wavefront form (final phase in two row passes)."""
    k, n = 128, 128 * 300
    layer = make_layer(k, n, group, dtype, seed=4, bits=8)
    ks = torch.randperm(k, generator=torch.Generator().manual_seed(1))[:16]
    a = torch.zeros(16, k, dtype=dtype)
    a[torch.arange(16), ks] = 1.0
    out = run_gemm(ops, layer, a.to(dev), dev, workspace)
    assert torch.equal(out.cpu(), layer.w_ref[ks])
    a = torch.randn(5, k, generator=torch.Generator().manual_seed(2)).to(dtype).to(dev)
    check_close(run_gemm(ops, layer, a, dev, workspace), a, layer)
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 16, 33, 100, 512])
@pytest.mark.parametrize("group,act_order,k_full", [(-1, False, True), (128, False, True), (64, True, True), (128, True, False)])
def test_gemm_w8(ops, dev, workspace, dtype, m, group, act_order, k_full):
    k, n = 1024, 384
    layer = make_layer(k, n, group, dtype, act_order=act_order, seed=m + k, bits=8)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(2)).to(dtype).to(dev)
    out = run_gemm(ops, layer, a, dev, workspace, is_k_full=k_full)
    check_close(out, a, layer)
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group,act_order", [(-1, False), (128, False), (64, True)])
def test_prefill_tiles_w8(ops, dev, workspace, dtype, group, act_order):
    """Enough 128-row tiles for the prefill kernel (M = 1100 leaves a partial row tile, N = 8256 a partial 512-column
    strip): random activations against the oracle, and one-hot rows bit-exact on the same launch shape."""
    m, k, n = 1100, 512, 8256
    print(f"w8 prefill dtype={dtype} g={group} act_order={act_order}", flush=True)
    layer = make_layer(k, n, group, dtype, act_order=act_order, seed=21, bits=8)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(3)).to(dtype).to(dev)
    out = run_gemm(ops, layer, a, dev, workspace)
    check_close(out, a, layer)
    ks = torch.randint(0, k, (m,), generator=torch.Generator().manual_seed(4))
    hot = torch.zeros(m, k, dtype=dtype)
    hot[torch.arange(m), ks] = 1.0
    out = run_gemm(ops, layer, hot.to(dev), dev, workspace)
    assert torch.equal(out.cpu(), layer.w_ref[ks])
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("dtype,group", [(torch.float16, 128), (torch.bfloat16, -1)])
def test_64_row_tiles_with_split_k_w8(ops, dev, workspace, dtype, group):
    """136 tiles of 64 x 512: the 64-row kernel splits K in two and a second kernel adds the partial tiles."""
    m, k, n = 512, 2048, 8704
    layer = make_layer(k, n, group, dtype, seed=22, bits=8)
    a = torch.randn(m, k, generator=torch.Generator().manual_seed(3)).to(dtype).to(dev)
    out = run_gemm(ops, layer, a, dev, workspace)
    check_close(out, a, layer)
    ks = torch.randint(0, k, (m,), generator=torch.Generator().manual_seed(4))
    hot = torch.zeros(m, k, dtype=dtype)
    hot[torch.arange(m), ks] = 1.0
    out = run_gemm(ops, layer, hot.to(dev), dev, workspace)
    assert torch.equal(out.cpu(), layer.w_ref[ks])
    assert int(workspace.abs().sum()) == 0


def test_linear_kernel_w8(dev):
    from vllm_amd.mixed_precision import MarlinLinearKernel, MPLinearLayerConfig, choose_mp_linear_kernel
    from vllm_amd.scalar_type import scalar_types
    from oracle import gemm_ref as gr
    from oracle import scalar_types as ost
    k, n, m = 512, 256, 20
    w = (torch.randn(k, n, generator=torch.Generator().manual_seed(0)) * 0.05).half()
    w_ref, q, s, _, _ = qu.gptq_quantize_weights(w, ost.uint8b128, 128, False, None)
    layer = torch.nn.Module()
    layer.qweight = torch.nn.Parameter(qu.pack_rows(q, 8).to(dev), requires_grad=False)
    layer.scales = torch.nn.Parameter(s.to(dev), requires_grad=False)
    cfg = MPLinearLayerConfig(full_weight_shape=(k, n), partition_weight_shape=(k, n), weight_type=scalar_types.uint8b128,
                              act_type=torch.float16, group_size=128, zero_points=False, has_g_idx=False)
    assert choose_mp_linear_kernel(cfg) is MarlinLinearKernel
    kern = MarlinLinearKernel(cfg, "qweight", "scales")
    kern.process_weights_after_loading(layer)
    assert tuple(layer.qweight.shape) == (k // 16, 4 * n)
    x = torch.randn(m, k, generator=torch.Generator().manual_seed(1)).half()
    out = kern.apply_weights(layer, x.to(dev))
    mt = gr.error_metrics(out, gr.gemm_ref(x, w_ref))
    assert mt["max_rel"] <= 2e-2 and mt["mean_rel"] < 0.04, mt


# (300 tokens in blocks of 8: more 16-row tiles than compute units, the 4-wavefront form of the general kernel)
@pytest.mark.parametrize("m,topk,e,bs", [(1, 2, 4, 8), (33, 2, 8, 16), (123, 3, 4, 32), (333, 2, 4, 64), (300, 4, 4, 8)])
@pytest.mark.parametrize("dtype,k_full", [(torch.float16, True), (torch.bfloat16, True), (torch.float16, False)])
def test_moe_gemm_w8_act_order(ops, dev, dtype, k_full, m, topk, e, bs):
    """uint8b128 experts with act-order (per-expert g_idx and column gather inside the kernel), which the reference
    instantiates for its MoE op (csrc/moe/marlin_moe_wna16/ops.cu:441); against the per-slot oracle, and one-hot rows
    bit-exactly."""
    from oracle import gemm_ref as gr
    from oracle import moe_ref as mr
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    from vllm_amd.scalar_type import scalar_types
    k, n = 256, 192
    layers = [make_layer(k, n, 32, dtype, act_order=True, seed=70 + i, w_std=0.1, bits=8) for i in range(e)]
    st = lambda name: torch.stack([getattr(l, name) for l in layers]).to(dev)
    g = torch.Generator().manual_seed(5)
    ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    tw = torch.rand(m, topk, generator=g)
    s, x, t = moe_align_block_size(ids.to(dev), bs, e)
    ws = marlin_make_workspace_new(dev, 4)

    def run(a):
        return ops.moe_wna16_marlin_gemm(
            a.to(dev), None, st("marlin_q"), None, st("marlin_s"), None, None, st("g_idx_sorted"), st("sort_indices"), ws,
            s, x, t, tw.to(dev), moe_block_size=bs, top_k=topk, mul_topk_weights=False, is_ep=False,
            b_q_type=scalar_types.uint8b128, size_m=m, size_n=n, size_k=k, is_k_full=k_full, use_atomic_add=False,
            use_fp32_reduce=True, is_zp_float=False)
    a = torch.randn(m, k, generator=g).to(dtype)
    out = run(a)
    w_dense = torch.stack([l.w_ref for l in layers])
    ref = mr.moe_gemm_ref(a, w_dense, s.cpu(), x.cpu(), t.cpu(), tw, bs, topk, False, m)
    mt = gr.error_metrics(out, ref)
    assert mt["max_rel"] <= (2e-2 if dtype == torch.float16 else 4e-2) and mt["mean_rel"] < 0.04, mt
    ks = torch.randint(0, k, (m,), generator=g)
    hot = torch.zeros(m, k, dtype=dtype)
    hot[torch.arange(m), ks] = 1.0
    out = run(hot).cpu()
    for i in range(m):
        for j in range(topk):
            assert torch.equal(out[i * topk + j], layers[int(ids[i, j])].w_ref[ks[i]])
    assert int(ws.abs().sum()) == 0
