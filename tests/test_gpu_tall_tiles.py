"""Problems that run on 128 x 256 tiles whose K halves are added inside the workgroup (gemm_kq.hip with 8 m-blocks): on
their own when those tiles fill between 3/4 and all of the 256 compute units in one round, and as the last, partly filled
round of a prefill launch (the trailing 512-column strips of 4096 x 6144).  Compared with the CPU oracle's
dequantise-then-matmul (gates as in test_gpu_gemm.py, which follow tests/kernels/quantization/test_marlin_gemm.py:359-361)
and, with one-hot rows, bit for bit with the dequantised weights."""
import pytest
import torch

from helpers import check_close, make_layer, run_gemm

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import vllm_amd.ops as o
    return o


@pytest.fixture()
def workspace(dev):
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    return marlin_make_workspace_new(dev)


MODES = [
    # (dtype, zero points, act-order, group, bias)
    (torch.float16, False, False, 128, False),
    (torch.bfloat16, True, False, 128, True),
    (torch.bfloat16, False, False, -1, False),
    (torch.float16, True, False, 32, False),
    (torch.float16, False, True, 128, True),
]

SHAPES = [
    # (M, K, N): tiles of 128 x 256
    (200, 512, 28672),    # 2 x 112, a ragged last row tile
    (256, 256, 32768),    # 2 x 128: every compute unit, one loop iteration per K half
    (1536, 768, 4096),    # 12 x 16 = 192: the smallest grid that takes this path
    (4000, 512, 1600),    # 32 x 7, the last strip 64 columns wide
    # prefill kernel on the first 4096 columns, these tiles on the rest
    (4096, 512, 6144),
    (4090, 256, 6080),
]


@pytest.mark.parametrize("m,k,n", SHAPES)
@pytest.mark.parametrize("dtype,zp,act_order,group,with_bias", MODES)
def test_tall_tiles_match_oracle(ops, dev, workspace, m, k, n, dtype, zp, act_order, group, with_bias):
    print(f"tall tiles m={m} k={k} n={n} dtype={dtype} zp={zp} act_order={act_order} group={group}", flush=True)
    layer = make_layer(k, n, group, dtype, has_zp=zp, act_order=act_order, seed=m + n, w_std=0.05)
    g = torch.Generator().manual_seed(k)
    a = torch.randn(m, k, generator=g).to(dtype)
    bias = torch.randn(n, generator=g).to(dtype) if with_bias else None
    bias_dev = None
    if with_bias:
        from vllm_amd.marlin_utils import marlin_permute_bias
        bias_dev = marlin_permute_bias(bias.to(dev))
    out = run_gemm(ops, layer, a.to(dev), dev, workspace, bias=bias_dev)
    torch.cuda.synchronize()
    check_close(out.cpu(), a, layer, bias)
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("m,k,n", [(256, 512, 28672), (4096, 512, 6144)])
@pytest.mark.parametrize("dtype,zp,group", [(torch.float16, False, 128), (torch.bfloat16, True, 128),
                                            (torch.bfloat16, False, 32), (torch.float16, True, -1)])
def test_tall_tiles_one_hot_rows_are_exact(ops, dev, workspace, m, k, n, dtype, zp, group):
    """Row r of A is the unit vector of K position (7 r) mod K: the output row is one product 1 * w, so it must equal
    the dequantised weight row exactly, whichever K half and whichever tile it falls into."""
    print(f"tall tiles one-hot m={m} k={k} n={n} dtype={dtype} zp={zp} group={group}", flush=True)
    layer = make_layer(k, n, group, dtype, has_zp=zp, seed=3)
    ks = (7 * torch.arange(m)) % k
    a = torch.zeros(m, k, dtype=dtype)
    a[torch.arange(m), ks] = 1.0
    out = run_gemm(ops, layer, a.to(dev), dev, workspace)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), layer.w_ref[ks])


def _random_tall_shapes(count, seed):
    """Shapes whose 128 x 256 tiles number between 192 and 256: ragged last row tile, last strip 64..256 columns wide."""
    import random
    rng = random.Random(seed)
    out = []
    while len(out) < count:
        rows, strips = rng.randint(2, 32), rng.randint(6, 128)
        if not 192 <= rows * strips <= 256:
            continue
        m = 128 * (rows - 1) + rng.randint(1, 128)
        n = 256 * (strips - 1) + 64 * rng.randint(1, 4)
        k = 256 * rng.randint(1, 5)
        mode = rng.choice(["gptq", "awq", "act_order"])
        group = rng.choice([32, 64, 128] if mode == "act_order" else [-1, 32, 64, 128])
        out.append((m, k, n, mode, group, rng.choice([torch.float16, torch.bfloat16]), rng.random() < 0.5))
    return out


@pytest.mark.parametrize("cfg", _random_tall_shapes(12, 4242), ids=lambda c: f"m{c[0]}-k{c[1]}-n{c[2]}-{c[3]}-g{c[4]}-"
                         f"{'f16' if c[5] == torch.float16 else 'bf16'}{'-strided' if c[6] else ''}")
def test_tall_tiles_random_shapes(ops, dev, workspace, cfg):
    m, k, n, mode, group, dtype, strided = cfg
    print(f"tall tiles random {cfg}", flush=True)
    layer = make_layer(k, n, group, dtype, has_zp=mode == "awq", act_order=mode == "act_order", seed=m + n + k, w_std=0.05)
    g = torch.Generator().manual_seed(m * 3 + n)
    if strided:  # a column slice of a wider tensor: rows are k + 64 elements apart
        a = torch.randn(m, k + 64, generator=g).to(dtype).to(dev)[:, 32:32 + k]
    else:
        a = torch.randn(m, k, generator=g).to(dtype).to(dev)
    out = run_gemm(ops, layer, a, dev, workspace)
    torch.cuda.synchronize()
    check_close(out.cpu(), a.contiguous().cpu(), layer)
    assert int(workspace.abs().sum()) == 0
