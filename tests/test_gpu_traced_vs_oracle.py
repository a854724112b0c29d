"""The GEMM operator under torch.compile and under HIP-graph capture, checked against the CPU oracle (not against the
eager run of the same code): a slice of the reference's kernel grid (tests/kernels/quantization/test_marlin_gemm.py:211-361)
through the traced operator and through graph replay, plus one dynamic-shape compile that varies M across calls so that
the `SymInt size_m` of the operator schema (csrc/torch_bindings.cpp:316-323) is traced as a symbol."""
import pytest
import torch

from helpers import check_close, make_layer

pytestmark = pytest.mark.gpu

K, N = 1024, 512
MODES = [("gptq", -1), ("gptq", 32), ("gptq", 128), ("act_order", 32), ("act_order", 128), ("awq", -1), ("awq", 32),
         ("awq", 128)]


def _operands(dev, mode, group, dtype, seed):
    layer = make_layer(K, N, group, dtype, has_zp=mode == "awq", act_order=mode == "act_order", seed=seed, w_std=0.05)
    import vllm_amd.scalar_type as vst
    wtype = vst.scalar_types.uint4 if layer.has_zp else vst.scalar_types.uint4b8
    dev_ops = (layer.marlin_q.to(dev), layer.marlin_s.to(dev), layer.marlin_zp.to(dev), layer.g_idx_sorted.to(dev),
               layer.sort_indices.to(dev))
    return layer, wtype, dev_ops


def _gemm(a, c, dev_ops, ws, type_id, bias=None):
    mq, ms, mz, gi, si = dev_ops
    return torch.ops._C.gptq_marlin_gemm(a, c, mq, bias, ms, None, mz, gi, si, ws, type_id, a.shape[0], N, K, True, False,
                                         True, False)


@pytest.mark.parametrize("m", [1, 37, 257])
@pytest.mark.parametrize("mode,group", MODES)
def test_compiled_gemm_matches_oracle(dev, mode, group, m):
    import vllm_amd.ops  # noqa: F401
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    dtype = torch.float16 if (m + group) % 2 else torch.bfloat16
    layer, wtype, dev_ops = _operands(dev, mode, group, dtype, seed=m + (group & 255))
    ws = marlin_make_workspace_new(dev)
    torch._dynamo.reset()   # every case compiles the same code object anew: start from an empty cache
    fn = torch.compile(lambda x: _gemm(x, None, dev_ops, ws, wtype.id), fullgraph=True, backend="aot_eager", dynamic=False)
    a = torch.randn(m, K, generator=torch.Generator().manual_seed(m)).to(dtype)
    out = fn(a.to(dev))
    torch.cuda.synchronize()
    check_close(out.cpu(), a, layer)
    assert int(ws.abs().sum()) == 0


@pytest.mark.parametrize("mode,group", [("gptq", 128), ("act_order", 128), ("awq", 128)])
def test_compiled_gemm_dynamic_m_matches_oracle(dev, mode, group):
    """One compiled function, M changing from call to call: the operator is traced with a symbolic size_m."""
    import vllm_amd.ops  # noqa: F401
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    dtype = torch.float16
    layer, wtype, dev_ops = _operands(dev, mode, group, dtype, seed=77)
    ws = marlin_make_workspace_new(dev)
    torch._dynamo.reset()
    type_id = int(wtype.id)   # (computed outside the traced function: only M is meant to be symbolic)
    fn = torch.compile(lambda x: _gemm(x, None, dev_ops, ws, type_id), fullgraph=True, backend="aot_eager", dynamic=True)
    for m in (5, 48, 19, 130, 2):
        a = torch.randn(m, K, generator=torch.Generator().manual_seed(m)).to(dtype)
        out = fn(a.to(dev))
        torch.cuda.synchronize()
        assert out.shape == (m, N)
        check_close(out.cpu(), a, layer)


@pytest.mark.parametrize("m", [1, 37, 257])
@pytest.mark.parametrize("mode,group", MODES)
def test_graph_replayed_gemm_matches_oracle(dev, mode, group, m):
    """Capture once, replay three times with new activations and eager work of the same operator in between; every
    replay is compared with the oracle's dequantize-then-matmul on that replay's activations."""
    import vllm_amd.ops  # noqa: F401
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    dtype = torch.bfloat16 if (m + group) % 2 else torch.float16
    layer, wtype, dev_ops = _operands(dev, mode, group, dtype, seed=3 * m + (group & 255))
    ws = marlin_make_workspace_new(dev)
    a_dev = torch.zeros(m, K, dtype=dtype, device=dev)
    out = torch.empty(m, N, dtype=dtype, device=dev)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        _gemm(a_dev, out, dev_ops, ws, wtype.id)   # warm-up outside capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            _gemm(a_dev, out, dev_ops, ws, wtype.id)
    torch.cuda.synchronize()
    for rep in range(3):
        a = torch.randn(m, K, generator=torch.Generator().manual_seed(100 * rep + m)).to(dtype)
        a_dev.copy_(a)
        _gemm(a_dev, None, dev_ops, ws, wtype.id)  # eager work between the replays
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        check_close(out.cpu(), a, layer)
        assert int(ws.abs().sum()) == 0


@pytest.mark.parametrize("mode", ["gptq", "gptq_act_order", "awq"])
def test_compiled_apply_weights_matches_oracle(dev, mode):
    """MarlinLinearKernel.apply_weights traced by torch.compile, against the oracle on the checkpoint tensors."""
    from oracle import gemm_ref as gr
    from helpers import tol_for
    from test_gpu_linear_kernel import build_layer
    from vllm_amd.marlin_utils import marlin_permute_bias
    from vllm_amd.mixed_precision import MarlinLinearKernel, MPLinearLayerConfig
    from vllm_amd.scalar_type import scalar_types
    k, n, group, dtype = 1024, 768, 128, torch.float16
    layer, w_ref = build_layer(dev, k, n, group, dtype, mode, seed=9)
    cfg = MPLinearLayerConfig(full_weight_shape=(k, n), partition_weight_shape=(k, n),
                              weight_type=scalar_types.uint4 if mode == "awq" else scalar_types.uint4b8, act_type=dtype,
                              group_size=group, zero_points=mode == "awq", has_g_idx=mode == "gptq_act_order")
    kern = MarlinLinearKernel(cfg, "qweight", "scales", "qzeros" if mode == "awq" else None,
                              "g_idx" if mode == "gptq_act_order" else None)
    kern.process_weights_after_loading(layer)
    torch._dynamo.reset()
    compiled = torch.compile(lambda x, b: kern.apply_weights(layer, x, b), fullgraph=True, backend="aot_eager", dynamic=False)
    for m in (3, 40, 200):
        g = torch.Generator().manual_seed(m)
        x = torch.randn(2, m, k, generator=g).to(dtype)
        bias = torch.randn(n, generator=g).to(dtype)
        out = compiled(x.to(dev), marlin_permute_bias(bias.to(dev)))
        ref = gr.gemm_ref(x.reshape(-1, k), w_ref, bias).reshape(2, m, n)
        mt = gr.error_metrics(out, ref)
        assert mt["max_rel"] <= tol_for(dtype) and mt["mean_rel"] < 0.04, mt
