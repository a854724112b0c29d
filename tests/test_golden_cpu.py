"""The oracle reproduces the committed golden fixtures (tests/golden/*.npz, written by make_golden.py)."""
import os

import numpy as np
import torch

from oracle import gemm_ref as gr
from oracle import marlin_layout as ml
from oracle import moe_ref as mr

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def cases(z):
    return sorted({k.split(".")[0] for k in z.files})


def from_bits(a, dtype):
    return torch.from_numpy(a.copy()).view(dtype)


def test_repack_fixtures():
    z = load("repack.npz")
    assert len(cases(z)) == 3
    for c in cases(z):
        k, n = z[f"{c}.awq_in"].shape[0], z[f"{c}.gptq_in"].shape[1]
        perm = torch.from_numpy(z[f"{c}.perm"])
        got = ml.gptq_marlin_repack(torch.from_numpy(z[f"{c}.gptq_in"]), perm, k, n)
        assert np.array_equal(got.numpy(), z[f"{c}.gptq_out"])
        got = ml.awq_marlin_repack(torch.from_numpy(z[f"{c}.awq_in"]), k, n)
        assert np.array_equal(got.numpy(), z[f"{c}.awq_out"])
        if perm.numel() == 0:
            assert np.array_equal(z[f"{c}.gptq_out"], z[f"{c}.awq_out"])


def test_gemm_fixtures():
    z = load("gemm.npz")
    assert len(cases(z)) == 5
    for c in cases(z):
        dtype = torch.bfloat16 if "bf16" in c else torch.float16
        a = from_bits(z[f"{c}.a"], dtype)
        s = from_bits(z[f"{c}.b_scales"], dtype)
        k, n = a.shape[1], s.shape[1]
        zeros = torch.from_numpy(z[f"{c}.b_zeros"])
        g_idx = torch.from_numpy(z[f"{c}.g_idx"])
        w = gr.dequant_marlin(torch.from_numpy(z[f"{c}.b_q_weight"]), s, zeros, g_idx, k, n, zeros.numel() == 0, dtype)
        perm = torch.from_numpy(z[f"{c}.perm"]).long()
        w_ref = from_bits(z[f"{c}.w_ref"], dtype)
        assert torch.equal(w, w_ref[perm] if perm.numel() else w_ref)
        a_in = a[:, perm] if perm.numel() else a                    # the kernel gathers A columns the same way
        assert np.array_equal(gr.gemm_ref(a_in, w).numpy(), gr.gemm_ref(a[:, perm], w_ref[perm]).numpy()
                              if perm.numel() else z[f"{c}.c_ref"])
        assert np.allclose(gr.gemm_ref(a_in, w).numpy(), z[f"{c}.c_ref"], rtol=1e-5, atol=1e-5)


def test_moe_align_fixtures():
    z = load("moe_align.npz")
    for c in cases(z):
        parts = {p[0]: int(p[1:]) for p in c.split("_")}
        ids = torch.from_numpy(z[f"{c}.topk_ids"])
        s, x, t = mr.moe_align_block_size(ids, parts["b"], parts["e"])
        assert np.array_equal(s.numpy(), z[f"{c}.sorted_ids"])
        assert np.array_equal(x.numpy(), z[f"{c}.expert_ids"])
        assert np.array_equal(t.numpy(), z[f"{c}.total"])


def _other_type_w(z, c):
    """The oracle's dequantised weights for one case of other_types.npz, from the stored operands."""
    dtype = torch.bfloat16 if "bf16" in c else torch.float16
    mq = torch.from_numpy(z[f"{c}.b_q_weight"].copy())
    k = mq.shape[0] * 16
    if c.startswith("u8b128"):
        n = mq.shape[1] // 4
        return gr.dequant_marlin(mq, from_bits(z[f"{c}.b_scales"], dtype), None, None, k, n, True, dtype, num_bits=8)
    if c.startswith("fp8"):
        return gr.dequant_marlin_fp8(mq, from_bits(z[f"{c}.b_scales"], dtype), k, mq.shape[1] // 4, dtype)
    n = mq.shape[1] // 2
    if c.startswith("hqq"):
        return gr.dequant_marlin_float_zp(mq, from_bits(z[f"{c}.b_scales"], dtype),
                                          from_bits(z[f"{c}.b_zeros_f16"], dtype), k, n)
    byts = torch.from_numpy(z[f"{c}.b_scales"].copy())
    gs = from_bits(z[f"{c}.global_scale"], dtype) if f"{c}.global_scale" in z.files else None
    return gr.dequant_marlin_fp4(mq, byts, gs, k, n, dtype)


def test_other_type_fixtures():
    z = load("other_types.npz")
    assert cases(z) == ["fp8_f16_chan", "hqq_f16_g64", "mxfp4_bf16", "nvfp4_f16", "u8b128_bf16_g128"]
    for c in cases(z):
        dtype = torch.bfloat16 if "bf16" in c else torch.float16
        w = _other_type_w(z, c)
        assert torch.equal(w, from_bits(z[f"{c}.w_ref"], dtype)), c
        a = from_bits(z[f"{c}.a"], dtype)
        assert np.array_equal(gr.gemm_ref(a, w).numpy(), z[f"{c}.c_ref"]), c
