"""Load-time preparation kernels (scale / bias permutation, zero-point conversion) against the CPU oracle, bit for bit
(reference marlin_utils.py:278-370; the reference's own check is indirect, through test_marlin_gemm.py)."""
import pytest
import torch

from oracle import marlin_layout as ml
from oracle import quant_utils as qu

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k,n,group", [(256, 64, 128), (4096, 4096, 128), (1024, 28672, 32), (512, 192, -1),
                                       (14336, 4096, -1)])
def test_permute_scales_kernel(dev, dtype, k, n, group):
    from vllm_amd.marlin_utils import marlin_permute_bias, marlin_permute_scales
    gs = k if group == -1 else group
    s = torch.randn(k // gs, n, generator=torch.Generator().manual_seed(n)).to(dtype)
    got = marlin_permute_scales(s.to(dev), k, n, group)
    assert torch.equal(got.cpu(), ml.marlin_permute_scales(s, k, n, gs))
    b = torch.randn(n, generator=torch.Generator().manual_seed(k)).to(dtype)
    assert torch.equal(marlin_permute_bias(b.to(dev)).cpu(), ml.marlin_permute_bias(b))


def test_permute_scales_moe_and_strided(dev):
    from vllm_amd.marlin_utils import marlin_moe_permute_scales, marlin_permute_scales
    e, k, n, g = 5, 512, 320, 128
    s = torch.randn(e, k // g, n, generator=torch.Generator().manual_seed(3)).half()
    got = marlin_moe_permute_scales(s.to(dev), k, n, g)
    want = torch.stack([ml.marlin_permute_scales(s[i], k, n, g) for i in range(e)])
    assert torch.equal(got.cpu(), want)
    # a transposed (non-contiguous) view, as a checkpoint parameter with output_dim = 0 arrives
    t = torch.randn(n, k // g, generator=torch.Generator().manual_seed(4)).half()
    assert torch.equal(marlin_permute_scales(t.to(dev).t(), k, n, g).cpu(), ml.marlin_permute_scales(t.t(), k, n, g))


@pytest.mark.parametrize("groups,n", [(1, 64), (32, 4096), (112, 4096), (32, 28672), (7, 192)])
def test_zero_point_kernel_all_source_formats(dev, groups, n):
    from vllm_amd.marlin_utils import awq_to_marlin_zero_points, marlin_zero_points, marlin_zero_points_from_packed
    zp = torch.randint(0, 16, (groups, n), generator=torch.Generator().manual_seed(groups + n), dtype=torch.int32)
    want = ml.marlin_zero_points(zp, groups, n)
    assert torch.equal(want, ml.marlin_zero_points_closed_form(zp))
    assert torch.equal(marlin_zero_points(zp.to(dev), groups, n, 4).cpu(), want)
    assert torch.equal(marlin_zero_points_from_packed(qu.pack_cols(zp, 4).to(dev), groups, n, 4).cpu(), want)
    assert torch.equal(awq_to_marlin_zero_points(qu.awq_pack(zp, 4).to(dev), groups, n, 4).cpu(), want)


def test_zero_points_moe(dev):
    from vllm_amd.marlin_utils import moe_awq_to_marlin_zero_points
    e, groups, n = 3, 8, 256
    zp = torch.randint(0, 16, (e, groups, n), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    packed = torch.stack([qu.awq_pack(zp[i], 4) for i in range(e)])
    got = moe_awq_to_marlin_zero_points(packed.to(dev), groups, n, 4)
    want = torch.stack([ml.marlin_zero_points(zp[i], groups, n) for i in range(e)])
    assert torch.equal(got.cpu(), want)
