"""Many back-to-back launches of the paths that add K splits across workgroups (the 16-row kernel's in-kernel
exchange on o_proj- and down_proj-sized layers at M = 16; the two-pass K split of the 64 x 256 and the 64 x 512 kernels):
every result must equal the first bit for bit, and the workspace counters must be zero at the end.  The launches of a
burst go out on one stream without host synchronisation in between."""
import pytest
import torch

pytestmark = pytest.mark.gpu

BURST, BURSTS = 50, 40   # 2000 launches per case

# (name, M, K, N)
CASES = [("o M=16, 16-row kernel", 16, 4096, 4096), ("down M=16, 16-row kernel", 16, 14336, 4096),
         ("qkv M=4, 16-row kernel", 4, 4096, 6144),
         ("down M=256, 64 x 256 tiles + second pass", 256, 14336, 4096),
         ("gate_up M=192, 64 x 512 tiles + second pass", 192, 4096, 28672)]


@pytest.mark.parametrize("name,m,k,n", CASES)
def test_split_k_paths_are_stable_over_many_launches(dev, name, m, k, n):
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.scalar_type import scalar_types
    print(f"split-K stress: {name}", flush=True)
    gen = torch.Generator(device=dev).manual_seed(k + n + m)
    q = torch.randint(-2**31, 2**31 - 1, (k // 16, 2 * n), dtype=torch.int32, device=dev, generator=gen)
    s = (torch.rand(k // 128, n, device=dev, generator=gen) * 0.01 + 0.001).half()
    a = torch.randn(m, k, device=dev, generator=gen).half()
    ws = marlin_make_workspace_new(dev)
    e = torch.empty(0, dtype=torch.int32, device=dev)
    outs = [torch.empty(m, n, dtype=torch.float16, device=dev) for _ in range(BURST)]

    def launch(c):
        ops.gptq_marlin_gemm(a, c, q, None, s, None, e, e, e, ws, scalar_types.uint4b8, m, n, k, True, False, True, False)
    first = torch.empty(m, n, dtype=torch.float16, device=dev)
    launch(first)
    torch.cuda.synchronize()
    assert float(first.float().abs().max()) > 0 and bool(torch.isfinite(first).all())
    for burst in range(BURSTS):
        for c in outs:
            launch(c)
        torch.cuda.synchronize()
        for i, c in enumerate(outs):
            assert torch.equal(c, first), f"{name}: launch {burst * BURST + i} differs from the first"
        if burst == 0:
            for c in outs:
                c.zero_()
    assert int(ws.abs().sum()) == 0
