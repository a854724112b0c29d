"""GPU results against the committed golden fixtures (tests/golden/*.npz), through the operator surface."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def cases(z):
    return sorted({k.split(".")[0] for k in z.files})


def test_repack_fixtures_bit_exact(dev):
    import vllm_amd.ops as ops
    z = load("repack.npz")
    for c in cases(z):
        k, n = z[f"{c}.awq_in"].shape[0], z[f"{c}.gptq_in"].shape[1]
        perm = torch.from_numpy(z[f"{c}.perm"]).to(dev)
        got = ops.gptq_marlin_repack(torch.from_numpy(z[f"{c}.gptq_in"]).to(dev), perm, k, n, 4)
        assert np.array_equal(got.cpu().numpy(), z[f"{c}.gptq_out"]), c
        got = ops.awq_marlin_repack(torch.from_numpy(z[f"{c}.awq_in"]).to(dev), k, n, 4)
        assert np.array_equal(got.cpu().numpy(), z[f"{c}.awq_out"]), c


def test_gemm_fixtures(dev):
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.scalar_type import scalar_types
    z = load("gemm.npz")
    ws = marlin_make_workspace_new(dev)
    for c in cases(z):
        dtype = torch.bfloat16 if "bf16" in c else torch.float16
        t = lambda key, dt=None: (torch.from_numpy(z[f"{c}.{key}"].copy()).view(dt) if dt else
                                  torch.from_numpy(z[f"{c}.{key}"].copy())).to(dev)
        a, s = t("a", dtype), t("b_scales", dtype)
        zeros = t("b_zeros")
        wtype = scalar_types.uint4 if zeros.numel() else scalar_types.uint4b8
        out = ops.gptq_marlin_gemm(a, None, t("b_q_weight"), None, s, None, zeros, t("g_idx"), t("perm"), ws, wtype,
                                   a.shape[0], s.shape[1], a.shape[1], True, False, True, False)
        ref = torch.from_numpy(z[f"{c}.c_ref"])
        d = (out.float().cpu() - ref).abs()
        tol = 4e-2 if dtype == torch.bfloat16 else 2e-2      # stated gate: max|d| / max|ref|
        assert float(d.max() / ref.abs().max()) <= tol, c
        assert float(d.mean() / ref.abs().mean()) < 0.04, c
        assert int(ws.abs().sum()) == 0

        # one-hot rows select dequantised weight rows: bit-exact against the fixture's w_ref
        k = a.shape[1]
        rows = torch.tensor([0, 1, 17, k // 2 + 3, k - 1])
        onehot = torch.zeros(len(rows), k, dtype=dtype)
        onehot[torch.arange(len(rows)), rows] = 1
        out = ops.gptq_marlin_gemm(onehot.to(dev), None, t("b_q_weight"), None, s, None, zeros, t("g_idx"), t("perm"),
                                   ws, wtype, len(rows), s.shape[1], k, True, False, True, False)
        w_ref = torch.from_numpy(z[f"{c}.w_ref"].copy())
        assert torch.equal(out.cpu().view(torch.int16) , w_ref[rows]), c


def test_moe_align_fixtures_exact(dev):
    from vllm_amd.moe_align_block_size import moe_align_block_size
    z = load("moe_align.npz")
    for c in cases(z):
        parts = {p[0]: int(p[1:]) for p in c.split("_")}
        ids = torch.from_numpy(z[f"{c}.topk_ids"]).to(dev)
        s, x, t = moe_align_block_size(ids, parts["b"], parts["e"])
        assert np.array_equal(t.cpu().numpy(), z[f"{c}.total"]), c
        assert np.array_equal(s.cpu().numpy(), z[f"{c}.sorted_ids"]), c
        assert np.array_equal(x.cpu().numpy(), z[f"{c}.expert_ids"]), c
