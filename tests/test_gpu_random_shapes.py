"""Seeded random problem shapes for the dense W4A16 GEMM, checked against the CPU oracle through the torch op.

The fixed grids of the other GPU tests follow the reference's own test parameters; this file walks shapes between
them (row counts around every tile height, N and K that are odd multiples of the tile sizes, every group size and
quantization mode, bias, strided activations) so that a launch-plan boundary with a wrong tail shows up.
Tolerances as in test_gpu_gemm.py (tests/kernels/quantization/test_marlin_gemm.py:359-361 in the reference)."""
import random

import pytest
import torch

from helpers import check_close, make_layer, run_gemm

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(dev):
    import vllm_amd.ops as o
    return o


@pytest.fixture(scope="module")
def workspace(dev):
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    return marlin_make_workspace_new(dev)


def _configs(n, seed, large=False):
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        mode = rng.choice(["gptq", "gptq", "awq", "act_order", "act_order_partial_k"])
        group = rng.choice([-1, 32, 64, 128])
        if mode.startswith("act_order") and group == -1:
            continue
        k = 128 * (rng.randint(8, 32) if large else rng.randint(1, 20))
        if group > 0 and mode.startswith("act_order") and k // group < 2:
            continue
        nn = 64 * (rng.choice([8, 9, 16, 23, 24, 32, 40, 47, 64, 72, 96]) if large else
                   rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 15, 16, 17, 24, 31, 40]))
        m = rng.randint(300, 3000) if large else rng.choice([1, 2, 7, 15, 16, 17, 31, 32, 33, 47, 63, 64, 65, 100, 127, 128, 129, 191, 200, 255, 256, 257,
                        300, 511, 513, 700])
        dtype = rng.choice([torch.float16, torch.bfloat16])
        out.append((mode, group, m, nn, k, dtype, rng.random() < 0.3, rng.random() < 0.3))
    return out


@pytest.mark.parametrize("cfg", _configs(160, 20240611) + _configs(16, 77, large=True), ids=lambda c: f"{c[0]}-g{c[1]}-m{c[2]}-n{c[3]}-k{c[4]}-"
                         f"{'f16' if c[5] == torch.float16 else 'bf16'}{'-bias' if c[6] else ''}{'-strided' if c[7] else ''}")
def test_random_shape(ops, dev, workspace, cfg):
    from vllm_amd.marlin_utils import marlin_permute_bias
    mode, group, m, n, k, dtype, with_bias, strided = cfg
    print(f"random_shape {cfg}", flush=True)
    layer = make_layer(k, n, group, dtype, has_zp=(mode == "awq"), act_order=mode.startswith("act_order"),
                       seed=m * 7 + n + k)
    g = torch.Generator().manual_seed(m + 3 * n + 5 * k)
    if strided:  # a column slice of a wider tensor: rows are k + 64 elements apart
        wide = torch.randn(m, k + 64, generator=g).to(dtype).to(dev)
        a = wide[:, 32:32 + k]
        assert a.stride(0) == k + 64
    else:
        a = torch.randn(m, k, generator=g).to(dtype).to(dev)
    bias = torch.randn(n, generator=g).to(dtype).to(dev) if with_bias else None
    out = run_gemm(ops, layer, a, dev, workspace, is_k_full=(mode != "act_order_partial_k"),
                   bias=None if bias is None else marlin_permute_bias(bias))
    torch.cuda.synchronize()
    assert out.shape == (m, n) and out.dtype == dtype
    check_close(out, a.contiguous(), layer, bias=bias)
    assert int(workspace.abs().sum()) == 0
