"""GPU parity: repack kernels are bit-exact against the CPU oracle, called through the torch ops
(which go through the C ABI).  Grid follows the reference's test_gptq_marlin_repack /
test_awq_marlin_repack (tests/kernels/quantization/test_marlin_gemm.py:55-73, 98-209)."""
import pytest
import torch

from oracle import marlin_layout as ml
from oracle import quant_utils as qu

pytestmark = pytest.mark.gpu

MNK_FACTORS = [(1, 1, 1), (1, 4, 8), (26, 37, 13), (257, 13, 11)]


@pytest.fixture(scope="module")
def ops(dev):
    import vllm_amd.ops as o
    return o


@pytest.mark.parametrize("n_chunk", [64, 256])
@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("mnk", MNK_FACTORS)
def test_gptq_marlin_repack(ops, dev, n_chunk, act_order, mnk):
    _, nf, kf = mnk
    size_k, size_n = 128 * kf, n_chunk * nf
    print(f"gptq_repack k={size_k} n={size_n} act_order={act_order}", flush=True)
    g = torch.Generator().manual_seed(size_k * 7 + size_n)
    q = torch.randint(0, 16, (size_k, size_n), generator=g, dtype=torch.int32)
    packed = qu.gptq_pack(q)
    perm = torch.randperm(size_k, generator=g).to(torch.int32) if act_order else torch.empty(0, dtype=torch.int32)
    want = ml.marlin_weights_closed_form(q, perm if act_order else None)
    got = ops.gptq_marlin_repack(packed.to(dev), perm.to(dev), size_k, size_n, 4)
    torch.cuda.synchronize()
    assert got.dtype == torch.int32 and tuple(got.shape) == (size_k // 16, 2 * size_n)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("n_chunk", [64, 256])
@pytest.mark.parametrize("mnk", MNK_FACTORS)
def test_awq_marlin_repack(ops, dev, n_chunk, mnk):
    _, nf, kf = mnk
    size_k, size_n = 128 * kf, n_chunk * nf
    print(f"awq_repack k={size_k} n={size_n}", flush=True)
    g = torch.Generator().manual_seed(size_k * 5 + size_n)
    q = torch.randint(0, 16, (size_k, size_n), generator=g, dtype=torch.int32)
    want = ml.marlin_weights_closed_form(q)
    got = ops.awq_marlin_repack(qu.awq_pack(q).to(dev), size_k, size_n, 4)
    torch.cuda.synchronize()
    assert torch.equal(got.cpu(), want)


def test_repack_full_size_roundtrip(ops, dev):
    """Llama-3-8B down_proj size: GPU repack of a GPTQ pack, unpacked again on the host, is the input."""
    size_k, size_n = 14336, 4096
    print("gptq_repack full size", flush=True)
    g = torch.Generator().manual_seed(3)
    q = torch.randint(0, 16, (size_k, size_n), generator=g, dtype=torch.int32)
    got = ops.gptq_marlin_repack(qu.gptq_pack(q).to(dev), torch.empty(0, dtype=torch.int32, device=dev), size_k, size_n, 4)
    got_awq = ops.awq_marlin_repack(qu.awq_pack(q).to(dev), size_k, size_n, 4)
    torch.cuda.synchronize()
    assert torch.equal(got, got_awq)
    assert torch.equal(ml.marlin_unpack_weights(got.cpu()), q)


def test_permute_cols(ops, dev):
    """y == x[:, perm] (reference tests/kernels/core/test_permute_cols.py), including a strided view."""
    g = torch.Generator().manual_seed(1)
    # (rows, columns, extra row stride): both kernels behind the op (element-wise for few rows or short / odd rows, rows
    # staged in LDS otherwise), rows shared between workgroups (32..127 rows), several rows per workgroup (> 1024 rows),
    # the longest row the staged kernel takes and the first one it does not
    for m, k, pad in [(1, 128, 64), (33, 4096, 64), (31, 4096, 0), (100, 1024, 8), (512, 14336, 64), (1500, 2048, 0),
                      (40, 32768, 0), (40, 32776, 0), (64, 1028, 4), (300, 4096, 4)]:
        x = torch.randn(m, k + pad, generator=g).half().to(dev)[:, :k]
        perm = torch.randperm(k, generator=g).to(torch.int32).to(dev)
        y = ops.permute_cols(x, perm)
        assert torch.equal(y, x[:, perm.long()]), (m, k, pad)
    x = torch.randn(200, 2048, generator=g).to(torch.bfloat16).to(dev)
    perm = torch.randperm(2048, generator=g).to(torch.int32).to(dev)
    assert torch.equal(ops.permute_cols(x, perm), x[:, perm.long()])


def test_repack_errors(ops, dev):
    q = torch.zeros(16, 64, dtype=torch.int32, device=dev)
    e = torch.empty(0, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):
        ops.gptq_marlin_repack(q, e, 100, 64, 4)        # size_k not divisible by 16
    with pytest.raises(RuntimeError):
        ops.gptq_marlin_repack(q, e, 128, 96, 4)        # size_n not divisible by 64
    with pytest.raises(RuntimeError):
        ops.gptq_marlin_repack(q, e, 256, 64, 4)        # shape mismatch
    with pytest.raises(RuntimeError):
        ops.awq_marlin_repack(q, 128, 64, 3)            # bad bits


@pytest.mark.parametrize("num_bits", [4, 8])
def test_moe_repack_wrappers(ops, dev, num_bits):
    """Per-expert repack loops (reference vllm/_custom_ops.py:1221-1260): [E, K/pf, N] -> [E, K/16, N * bits / 2]."""
    e, size_k, size_n = 3, 128, 192
    g = torch.Generator().manual_seed(17)
    q = torch.randint(0, 1 << num_bits, (e, size_k, size_n), generator=g, dtype=torch.int32)
    perm = torch.stack([torch.randperm(size_k, generator=g) for _ in range(e)]).to(torch.int32)
    layout = ml.marlin_weights_closed_form if num_bits == 4 else ml.marlin_weights_closed_form8
    packed = torch.stack([qu.pack_rows(q[i], num_bits) for i in range(e)])
    got = ops.gptq_marlin_moe_repack(packed.to(dev), perm.to(dev), size_k, size_n, num_bits)
    assert tuple(got.shape) == (e, size_k // 16, size_n * num_bits // 2)
    for i in range(e):
        assert torch.equal(got[i].cpu(), layout(q[i], perm[i]))
    packed = torch.stack([qu.awq_pack(q[i], num_bits) for i in range(e)])
    got = ops.awq_marlin_moe_repack(packed.to(dev), perm.to(dev), size_k, size_n, num_bits)
    for i in range(e):
        assert torch.equal(got[i].cpu(), layout(q[i]))
