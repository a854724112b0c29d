"""Accuracy of the 16-row kernels' fold arithmetic (raw E + q operands, one subtraction of (E + z) * sum(a) per scale
group) on activations that are not zero-mean unit-variance: all-positive rows (what follows a SiLU), rows with a large
common offset, and rows of magnitude 1e-4, at K = 14336 (down_proj), for group-128 and channel-wise scales, fp16 and
bf16.  Gates as everywhere: max|d| / max|ref| <= 2e-2 (fp16) / 4e-2 (bf16), mean-relative < 0.04; the error is also
required to stay within 4x of what rounding the exact result to the output type costs."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [128, -1])
@pytest.mark.parametrize("zp", [False, True])
@pytest.mark.parametrize("kind", ["positive", "offset", "tiny"])
@pytest.mark.parametrize("m", [1, 16])
def test_fold_arithmetic_on_biased_activations(dev, dtype, group, zp, kind, m):
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.marlin_utils_test import awq_marlin_quantize, marlin_quantize
    from vllm_amd.scalar_type import scalar_types as st
    k, n = 14336, 4096
    g = torch.Generator().manual_seed(7)
    w = (torch.randn(k, n, generator=g) * 0.02).to(dtype).to(dev)
    e = torch.empty(0, dtype=torch.int32, device=dev)
    if zp:
        w_ref, mq, ms, mz = awq_marlin_quantize(w, st.uint4, group, rule="absmax")
        wtype = st.uint4
    else:
        w_ref, mq, ms, _, _, _ = marlin_quantize(w, st.uint4b8, group, False, rule="absmax")
        mz, wtype = e, st.uint4b8
    base = torch.randn(m, k, generator=g)
    a = {"positive": base.abs() + 0.5, "offset": base + 8.0, "tiny": base * 1e-4}[kind].to(dtype).to(dev)
    out = ops.gptq_marlin_gemm(a, None, mq, None, ms, None, mz, e, e, marlin_make_workspace_new(dev), wtype, m, n, k,
                               True, False, True, False).double()
    ref = a.double() @ w_ref.double()
    d = (out - ref).abs()
    tol = 2e-2 if dtype == torch.float16 else 4e-2
    assert float(d.max() / ref.abs().max()) <= tol
    assert float(d.mean() / ref.abs().mean()) < 0.04
    rounding = (ref.to(dtype).double() - ref).abs()          # cost of the final rounding alone
    print(f"{kind} {dtype} g={group} zp={zp} m={m}: mean err / mean rounding err = {float(d.mean() / rounding.mean()):.2f}",
          flush=True)
    assert float(d.mean()) <= 4.0 * float(rounding.mean()) + 1e-12
