"""The operator surface under PyTorch's own checks: torch.library.opcheck on every operator this package registers
(schema honesty, fake implementation against the real one, functionalisation through AOT dispatch), as the reference
does for its operators (tests/kernels/quantization/test_marlin_gemm.py:141-160, 310-330,
tests/kernels/moe/test_moe.py:820-880), and torch.compile(fullgraph=True) of the two host entry points against eager."""
import pytest
import torch

from helpers import make_layer
from test_gpu_moe import make_experts, rand_topk

pytestmark = pytest.mark.gpu

CHECKS = ("test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic")


def opcheck(op, args, kwargs=None):
    torch.library.opcheck(op, args, kwargs or {}, test_utils=CHECKS)


@pytest.fixture(scope="module")
def layer(dev):
    import vllm_amd.ops  # noqa: F401  (registers the operators)
    return make_layer(256, 128, 128, torch.float16, seed=1)


def test_opcheck_repacks_and_permute_cols(dev, layer):
    from oracle import quant_utils as qu
    k, n = layer.size_k, layer.size_n
    packed = qu.gptq_pack(layer.q).to(dev)
    empty = torch.empty(0, dtype=torch.int32, device=dev)
    perm = torch.randperm(k, generator=torch.Generator().manual_seed(0)).to(torch.int32).to(dev)
    opcheck(torch.ops._C.gptq_marlin_repack, (packed, empty, k, n, 4))
    opcheck(torch.ops._C.gptq_marlin_repack, (packed, perm, k, n, 4))
    opcheck(torch.ops._C.awq_marlin_repack, (qu.awq_pack(layer.q).to(dev), k, n, 4))
    a = torch.randn(5, k, dtype=torch.float16, device=dev)
    opcheck(torch.ops._C.permute_cols, (a, perm))


@pytest.mark.parametrize("m", [1, 40])
def test_opcheck_gptq_marlin_gemm(dev, layer, m):
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    k, n = layer.size_k, layer.size_n
    a = torch.randn(m, k, dtype=torch.float16, device=dev)
    e = torch.empty(0, dtype=torch.int32, device=dev)
    bias = torch.randn(n, dtype=torch.float16, device=dev)
    opcheck(torch.ops._C.gptq_marlin_gemm,
            (a, None, layer.marlin_q.to(dev), bias, layer.marlin_s.to(dev), None, e, e, e, marlin_make_workspace_new(dev),
             layer.type_id, m, n, k, True, False, True, False))


def test_opcheck_moe_ops(dev):
    import vllm_amd.ops  # noqa: F401
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.moe_align_block_size import moe_align_block_size
    m, topk, e, bs, k, d = 20, 2, 4, 16, 256, 128
    layers, mq, ms, _, _, _ = make_experts(e, k, 2 * d, 128, torch.float16, False, False, seed=3)
    ids = rand_topk(m, topk, e, seed=4).to(dev)
    numel = ids.numel()
    sorted_ids = torch.empty(numel + e * (bs - 1), dtype=torch.int32, device=dev)
    expert_ids = torch.empty(-(-sorted_ids.numel() // bs), dtype=torch.int32, device=dev)
    post = torch.empty(1, dtype=torch.int32, device=dev)
    opcheck(torch.ops._moe_C.moe_align_block_size, (ids, e, bs, sorted_ids, expert_ids, post))

    n_tok = torch.tensor([5, 0, 16, 9], dtype=torch.int32, device=dev)
    b_sorted = torch.empty(e * 16, dtype=torch.int32, device=dev)
    b_ids = torch.empty(e, dtype=torch.int32, device=dev)
    opcheck(torch.ops._moe_C.batched_moe_align_block_size, (16, 16, n_tok, b_sorted, b_ids, post.clone()))

    s, x, t = moe_align_block_size(ids, bs, e)
    a = torch.randn(m, k, dtype=torch.float16, device=dev) / 4
    tw = torch.rand(m, topk, device=dev)
    ws = marlin_make_workspace_new(dev, 4)
    wq, wsc = mq.to(dev), ms.to(dev)
    opcheck(torch.ops._moe_C.moe_wna16_marlin_gemm,
            (a, None, wq, None, wsc, None, None, None, None, ws, s, x, t, tw, bs, topk, False, False, layers[0].type_id,
             m, 2 * d, k, True, False, True, False))
    c = torch.empty(m * topk, d, dtype=torch.float16, device=dev)
    zf = torch.ones(m, k, dtype=torch.float16, device=dev)
    opcheck(torch.ops.w4a16.moe_marlin_gemm_fused,
            (a, c, wq, None, wsc, None, None, None, None, ws, s, x, t, tw, bs, topk, False, layers[0].type_id,
             m, 2 * d, k, True, True, 0, zf))

    y = torch.randn(m, topk, k, dtype=torch.float16, device=dev)
    opcheck(torch.ops._moe_C.moe_sum, (y, torch.empty(m, k, dtype=torch.float16, device=dev)))
    h = torch.randn(m, 2 * d, dtype=torch.float16, device=dev)
    opcheck(torch.ops._C.silu_and_mul, (torch.empty(m, d, dtype=torch.float16, device=dev), h))
    logits = torch.randn(m, e, device=dev)
    opcheck(torch.ops._moe_C.topk_softmax,
            (torch.empty(m, topk, device=dev), torch.empty(m, topk, dtype=torch.int32, device=dev),
             torch.empty(m, topk, dtype=torch.int32, device=dev), logits, True))


@pytest.mark.parametrize("mode", ["gptq", "awq"])
def test_compiled_apply_weights_equals_eager(dev, mode):
    from test_gpu_linear_kernel import build_layer
    from vllm_amd.mixed_precision import MarlinLinearKernel, MPLinearLayerConfig
    from vllm_amd.scalar_type import scalar_types
    k, n, group, dtype = 1024, 768, 128, torch.float16
    layer, _ = build_layer(dev, k, n, group, dtype, mode, seed=2)
    cfg = MPLinearLayerConfig(full_weight_shape=(k, n), partition_weight_shape=(k, n),
                              weight_type=scalar_types.uint4 if mode == "awq" else scalar_types.uint4b8, act_type=dtype,
                              group_size=group, zero_points=mode == "awq", has_g_idx=False)
    kern = MarlinLinearKernel(cfg, "qweight", "scales", "qzeros" if mode == "awq" else None, None)
    kern.process_weights_after_loading(layer)
    compiled = torch.compile(lambda x, b: kern.apply_weights(layer, x, b), fullgraph=True, backend="aot_eager", dynamic=False)
    for m in (3, 40):
        x = torch.randn(2, m, k, dtype=dtype, device=dev)
        b = torch.randn(n, dtype=dtype, device=dev)
        assert torch.equal(compiled(x, b), kern.apply_weights(layer, x, b))


@pytest.mark.parametrize("topk", [2, 3])
def test_compiled_fused_marlin_moe_equals_eager(dev, topk):
    from vllm_amd.fused_marlin_moe import fused_marlin_moe
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    dtype, e, m, k, inter = torch.float16, 4, 37, 256, 128
    l1, q1, s1, _, _, _ = make_experts(e, k, 2 * inter, 128, dtype, False, False, seed=100)
    l2, q2, s2, _, _, _ = make_experts(e, inter, k, 128, dtype, False, False, seed=200)
    g = torch.Generator().manual_seed(11)
    a = (torch.randn(m, k, generator=g) / 10).to(dtype).to(dev)
    tw, ti = torch.topk(torch.softmax(torch.randn(m, e, generator=g), dim=-1), topk)
    tw, ti = tw.to(dev), ti.to(torch.int32).to(dev)
    ws = marlin_make_workspace_new(dev, 4)
    w = (q1.to(dev), q2.to(dev), None, None, s1.to(dev), s2.to(dev))
    type_id = l1[0].type_id

    def run(x, weights, ids):
        return fused_marlin_moe(x, *w, None, weights, ids, quant_type_id=type_id, global_num_experts=e, workspace=ws)
    compiled = torch.compile(run, fullgraph=True, backend="aot_eager", dynamic=False)
    assert torch.equal(compiled(a, tw, ti), run(a, tw, ti))
