"""MarlinLinearKernel end to end on the GPU (load-time conversion + apply) and HIP-graph replay of the GEMM.

Follows the choreography of the reference's kernel class
(vllm/model_executor/layers/quantization/kernels/mixed_precision/marlin.py:66-166): checkpoint-layout
parameters on a layer -> process_weights_after_loading -> apply_weights, compared with the CPU oracle's
dequantize-then-matmul on the same checkpoint tensors."""
import pytest
import torch

from helpers import tol_for
from oracle import gemm_ref as gr
from oracle import quant_utils as qu
from oracle import scalar_types as ost

pytestmark = pytest.mark.gpu


def build_layer(dev, k, n, group, dtype, mode, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(k, n, generator=g) * 0.05).to(dtype)
    layer = torch.nn.Module()
    if mode == "awq":
        w_ref, q, s, zp = qu.quantize_weights(w, ost.uint4, group, zero_points=True)
        layer.qweight = torch.nn.Parameter(qu.gptq_pack(q).to(dev), requires_grad=False)       # packed along K
        # zero points arrive packed along N and transposed: [N/8, G]
        layer.qzeros = torch.nn.Parameter(qu.pack_cols(zp, 4).t().contiguous().to(dev), requires_grad=False)
        g_idx = None
    else:
        act = mode == "gptq_act_order"
        w_ref, q, s, g_idx, _ = qu.gptq_quantize_weights(w, ost.uint4b8, group, act,
                                                         torch.randperm(k, generator=g) if act else None)
        layer.qweight = torch.nn.Parameter(qu.gptq_pack(q).to(dev), requires_grad=False)
        if act:
            layer.g_idx = torch.nn.Parameter(g_idx.to(dev), requires_grad=False)
    layer.scales = torch.nn.Parameter(s.to(dev), requires_grad=False)
    return layer, w_ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode,group", [("gptq", 128), ("gptq", -1), ("gptq_act_order", 128), ("gptq_act_order", 32),
                                        ("awq", 128), ("awq", 64)])
@pytest.mark.parametrize("m", [1, 16, 77, 300])
def test_marlin_linear_kernel_end_to_end(dev, dtype, mode, group, m):
    from vllm_amd.mixed_precision import MarlinLinearKernel, MPLinearLayerConfig, choose_mp_linear_kernel
    from vllm_amd.scalar_type import scalar_types
    k, n = 1024, 768
    layer, w_ref = build_layer(dev, k, n, group, dtype, mode, seed=m + k)
    cfg = MPLinearLayerConfig(full_weight_shape=(k, n), partition_weight_shape=(k, n),
                              weight_type=scalar_types.uint4 if mode == "awq" else scalar_types.uint4b8,
                              act_type=dtype, group_size=group, zero_points=mode == "awq",
                              has_g_idx=mode == "gptq_act_order")
    assert choose_mp_linear_kernel(cfg) is MarlinLinearKernel
    kern = MarlinLinearKernel(cfg, w_q_param_name="qweight", w_s_param_name="scales",
                              w_zp_param_name="qzeros" if mode == "awq" else None,
                              w_gidx_param_name="g_idx" if mode == "gptq_act_order" else None)
    kern.process_weights_after_loading(layer)
    assert tuple(layer.qweight.shape) == (k // 16, 2 * n) and layer.qweight.dtype == torch.int32
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, m, k, generator=g).to(dtype)            # leading batch dims are flattened by apply
    bias = torch.randn(n, generator=g).to(dtype)
    from vllm_amd.marlin_utils import marlin_permute_bias
    out = kern.apply_weights(layer, x.to(dev), marlin_permute_bias(bias.to(dev)))
    assert out.shape == (2, m, n) and out.dtype == dtype
    ref = gr.gemm_ref(x.reshape(-1, k), w_ref, bias).reshape(2, m, n)
    mt = gr.error_metrics(out, ref)
    assert mt["max_rel"] <= tol_for(dtype) and mt["mean_rel"] < 0.04, mt


def test_kernel_selection_errors(dev):
    from vllm_amd.mixed_precision import MPLinearLayerConfig, choose_mp_linear_kernel
    from vllm_amd.scalar_type import scalar_types
    bad = MPLinearLayerConfig(full_weight_shape=(1024, 100), partition_weight_shape=(1024, 100),
                              weight_type=scalar_types.uint4b8, act_type=torch.float16, group_size=128,
                              zero_points=False, has_g_idx=False)
    with pytest.raises(ValueError, match="min_thread_n"):
        choose_mp_linear_kernel(bad)
    bad8 = MPLinearLayerConfig(full_weight_shape=(1024, 128), partition_weight_shape=(1024, 128),
                               weight_type=scalar_types.int8, act_type=torch.float16, group_size=128,
                               zero_points=False, has_g_idx=False)
    with pytest.raises(ValueError, match="not supported"):
        choose_mp_linear_kernel(bad8)


@pytest.mark.parametrize("m,k,n", [(16, 4096, 4096), (16, 2048, 512), (64, 1024, 4096), (200, 1024, 1024)])
def test_gemm_under_hip_graph_replay(dev, m, k, n):
    """Capture the GEMM (split-K paths included: counters in `workspace`, partials in the scratch tensor) in a HIP
    graph; replay it several times with new activations and eager work in between; every replay must equal eager."""
    import vllm_amd.ops as ops
    from helpers import make_layer, run_gemm
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    layer = make_layer(k, n, 128, torch.float16, seed=3, rule="absmax7", w_std=0.05)
    ws = marlin_make_workspace_new(dev)
    a = torch.zeros(m, k, dtype=torch.float16, device=dev)
    out = torch.empty(m, n, dtype=torch.float16, device=dev)
    mq, ms = layer.marlin_q.to(dev), layer.marlin_s.to(dev)
    e = torch.empty(0, dtype=torch.int32, device=dev)
    from vllm_amd.scalar_type import scalar_types

    def call(c):
        return ops.gptq_marlin_gemm(a, c, mq, None, ms, None, e, e, e, ws, scalar_types.uint4b8, m, n, k, True, False,
                                    True, False)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        call(out)                      # warm-up outside capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            call(out)
    torch.cuda.synchronize()
    for rep in range(4):
        a.copy_(torch.randn(m, k, generator=torch.Generator().manual_seed(rep)).half())
        eager = call(None).clone()     # eager work between replays
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        assert int(ws.abs().sum()) == 0
