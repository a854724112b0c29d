"""Vocabulary-sized N and long K (an lm_head of 128256 columns, K = 28672): index arithmetic beyond 2^31 bits of weight
data, tile counts in the thousands.  The weights are quantised on the GPU (vllm_amd.marlin_utils_test, checked
against the CPU oracle in test_host_quantize.py and test_gpu_baseline_shapes.py) and the result is compared with a
dequantised fp32 matmul there (the CPU oracle would need minutes for these sizes); tolerances as in test_gpu_gemm.py."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("k,n", [(4096, 128256), (28672, 8192)])
@pytest.mark.parametrize("mode", ["gptq_f16", "awq_bf16"])
def test_large_shape(dev, k, n, mode):
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.marlin_utils_test import awq_marlin_quantize, marlin_quantize
    from vllm_amd.scalar_type import scalar_types
    ws = marlin_make_workspace_new(dev)
    e = torch.empty(0, dtype=torch.int32, device=dev)
    gen = torch.Generator().manual_seed(1)
    if mode == "gptq_f16":
        wtype, dtype, tol = scalar_types.uint4b8, torch.float16, 2e-2
        w = (torch.randn(k, n, generator=gen) * 0.02).to(dtype).to(dev)
        w_deq, mq, ms, _, _, _ = marlin_quantize(w, wtype, 128, False, rule="absmax")
        mz = e
    else:
        wtype, dtype, tol = scalar_types.uint4, torch.bfloat16, 4e-2
        w = (torch.randn(k, n, generator=gen) * 0.02).to(dtype).to(dev)
        w_deq, mq, ms, mz = awq_marlin_quantize(w, wtype, 128, rule="absmax")
    del w
    for m in (1, 16, 50, 300, 2100):
        print(f"large shape {mode} k={k} n={n} m={m}", flush=True)
        a = torch.randn(m, k, generator=torch.Generator().manual_seed(m)).to(dtype).to(dev)
        out = ops.gptq_marlin_gemm(a, None, mq, None, ms, None, mz, e, e, ws, wtype, m, n, k, True, False, True, False)
        ref = a.float() @ w_deq.float()
        # per 512-column strip, so that one wrong tile cannot hide behind the largest value of the whole matrix
        d = (out.float() - ref).abs()
        pad = (-n) % 512
        dmax = torch.nn.functional.pad(d, (0, pad)).view(m, -1, 512).amax(dim=(0, 2))
        rmax = torch.nn.functional.pad(ref.abs(), (0, pad)).view(m, -1, 512).amax(dim=(0, 2))
        assert float((dmax / rmax).max()) <= tol
        assert float(d.mean() / ref.abs().mean()) < 0.04
        assert int(ws.abs().sum()) == 0
    del w_deq, mq, ms, mz
    torch.cuda.empty_cache()
