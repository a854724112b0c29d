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


def test_other_type_fixtures(dev):
    """uint8b128, float zero points, float8_e4m3fn and float4_e2m1f operands of tests/golden/other_types.npz."""
    import vllm_amd.ops as ops
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    from vllm_amd.scalar_type import scalar_types
    z = load("other_types.npz")
    ws = marlin_make_workspace_new(dev)
    wtypes = {"u8b128": scalar_types.uint8b128, "hqq": scalar_types.uint4, "fp8": scalar_types.float8_e4m3fn,
              "nvfp4": scalar_types.float4_e2m1f, "mxfp4": scalar_types.float4_e2m1f}
    for c in cases(z):
        kind = c.split("_")[0]
        dtype = torch.bfloat16 if "bf16" in c else torch.float16
        bits = lambda key: torch.from_numpy(z[f"{c}.{key}"].copy()).view(dtype).to(dev)
        a = bits("a")
        mq = torch.from_numpy(z[f"{c}.b_q_weight"].copy()).to(dev)
        k = a.shape[1]
        n = mq.shape[1] // (4 if kind in ("u8b128", "fp8") else 2)
        zeros, gs, zp_float = None, None, False
        if kind in ("nvfp4", "mxfp4"):
            raw = torch.from_numpy(z[f"{c}.b_scales"].copy()).to(dev)
            scales = raw.view(torch.float8_e4m3fn if kind == "nvfp4" else torch.float8_e8m0fnu)
            gs = bits("global_scale") if kind == "nvfp4" else None
        else:
            scales = bits("b_scales")
        if kind == "hqq":
            zeros, zp_float = bits("b_zeros_f16"), True

        def run(x):
            return ops.gptq_marlin_gemm(x, None, mq, None, scales, gs, zeros, None, None, ws, wtypes[kind], x.shape[0], n, k,
                                        True, False, True, zp_float)
        ref = torch.from_numpy(z[f"{c}.c_ref"])
        d = (run(a).float().cpu() - ref).abs()
        assert float(d.max() / ref.abs().max()) <= (4e-2 if dtype == torch.bfloat16 else 2e-2), c
        assert float(d.mean() / ref.abs().mean()) < 0.04, c
        rows = torch.tensor([0, 1, 17, k // 2 + 3, k - 1])
        onehot = torch.zeros(len(rows), k, dtype=dtype)
        onehot[torch.arange(len(rows)), rows] = 1
        w_ref = torch.from_numpy(z[f"{c}.w_ref"].copy()).view(dtype)
        assert torch.equal(run(onehot.to(dev)).cpu(), w_ref[rows]), c
        assert int(ws.abs().sum()) == 0
