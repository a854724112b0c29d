"""Writes the golden fixtures of this folder from the CPU oracle (run from the repository root:
`python tests/golden/make_golden.py`).  The fixtures are plain data (.npz, no pickles): seeded inputs in
the layouts the operators receive and the outputs the oracle derives for them.  They freeze the oracle's
answers so that a later change to the oracle, or a GPU result, is compared with fixed numbers."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import gemm_ref as gr  # noqa: E402
from oracle import marlin_layout as ml  # noqa: E402
from oracle import moe_ref as mr  # noqa: E402
from oracle import quant_utils as qu  # noqa: E402
from oracle import scalar_types as st  # noqa: E402


def bits16(t):
    """fp16 / bf16 tensors are stored as their 16-bit patterns (numpy has no bfloat16)."""
    return t.contiguous().view(torch.int16).numpy()


def repack_cases():
    g = torch.Generator().manual_seed(11)
    out = {}
    for name, (k, n, act) in {"k16n64": (16, 64, False), "k32n128_perm": (32, 128, True),
                              "k128n192": (128, 192, False)}.items():
        q = torch.randint(0, 16, (k, n), generator=g, dtype=torch.int32)
        perm = torch.randperm(k, generator=g).to(torch.int32) if act else torch.empty(0, dtype=torch.int32)
        out[f"{name}.gptq_in"] = qu.gptq_pack(q).numpy()
        out[f"{name}.awq_in"] = qu.awq_pack(q).numpy()
        out[f"{name}.perm"] = perm.numpy()
        out[f"{name}.gptq_out"] = ml.gptq_marlin_repack(qu.gptq_pack(q), perm, k, n).numpy()
        out[f"{name}.awq_out"] = ml.awq_marlin_repack(qu.awq_pack(q), k, n).numpy()
    np.savez_compressed(os.path.join(HERE, "repack.npz"), **out)


def gemm_cases():
    out = {}
    g = torch.Generator().manual_seed(12)
    cases = {
        "gptq_f16_g128": (torch.float16, 128, "gptq"), "gptq_bf16_chan": (torch.bfloat16, -1, "gptq"),
        "gptq_f16_g32_act": (torch.float16, 32, "act"), "awq_bf16_g128": (torch.bfloat16, 128, "awq"),
        "awq_f16_g64": (torch.float16, 64, "awq"),
    }
    for name, (dtype, group, mode) in cases.items():
        m, k, n = 5, 256, 64
        gs = k if group == -1 else group
        w = (torch.randn(k, n, generator=g) * 0.05).to(dtype)
        a = torch.randn(m, k, generator=g).to(dtype)
        e = torch.empty(0, dtype=torch.int32)
        zp_m, g_idx, order = e, e, e
        if mode == "awq":
            w_ref, q, s, zp = qu.quantize_weights(w, st.uint4, group, zero_points=True)
            mq = ml.awq_marlin_repack(qu.awq_pack(q), k, n)
            zp_m = ml.marlin_zero_points(zp, zp.shape[0], n)
        else:
            act = mode == "act"
            w_ref, q, s, gi, _ = qu.gptq_quantize_weights(w, st.uint4b8, group, act,
                                                          torch.randperm(k, generator=g) if act else None)
            if act:
                _, g_idx, order = qu.sort_weights(q, gi)
                g_idx = g_idx.to(torch.int32)
            mq = ml.gptq_marlin_repack(qu.gptq_pack(q), order, k, n)
        out[f"{name}.a"] = bits16(a)
        out[f"{name}.b_q_weight"] = mq.numpy()
        out[f"{name}.b_scales"] = bits16(ml.marlin_permute_scales(s, k, n, gs))
        out[f"{name}.b_zeros"] = zp_m.numpy()
        out[f"{name}.g_idx"] = g_idx.numpy()
        out[f"{name}.perm"] = order.numpy()
        out[f"{name}.w_ref"] = bits16(w_ref)                       # rows in the order activations arrive
        out[f"{name}.c_ref"] = gr.gemm_ref(a, w_ref).numpy()       # fp32
    np.savez_compressed(os.path.join(HERE, "gemm.npz"), **out)


def moe_align_cases():
    out = {}
    g = torch.Generator().manual_seed(13)
    for name, (m, topk, e, bs) in {"m33_k2_e8_b16": (33, 2, 8, 16), "m7_k3_e12_b8": (7, 3, 12, 8),
                                   "m200_k2_e64_b64": (200, 2, 64, 64)}.items():
        ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
        s, x, t = mr.moe_align_block_size(ids, bs, e)
        out[f"{name}.topk_ids"] = ids.numpy()
        out[f"{name}.sorted_ids"] = s.numpy()
        out[f"{name}.expert_ids"] = x.numpy()
        out[f"{name}.total"] = t.numpy()
    np.savez_compressed(os.path.join(HERE, "moe_align.npz"), **out)


def _regroup_fp4_scales(t):
    """Regrouping of a Marlin-permuted [G, N] scale matrix for fp4 weights (row pairs interleaved per 8-column chunk,
    the middle two of every four swapped), the layout the op receives."""
    g, n = t.shape
    t = t.view(g // 2, 2, -1, 8).permute(0, 2, 1, 3).reshape(g, n)
    return t.reshape(-1, 4)[:, [0, 2, 1, 3]].reshape(g, n)


def other_type_cases():
    """uint8b128, float zero points (HQQ), float8_e4m3fn and float4_e2m1f (NVFP4, MXFP4): operands as the dense op
    receives them, the oracle's dequantised weights and its fp32 result."""
    out = {}
    g = torch.Generator().manual_seed(14)
    m, k, n = 5, 256, 64
    e = torch.empty(0, dtype=torch.int32)

    def put(name, a, mq, scales, w_ref, **extra):
        out[f"{name}.a"] = bits16(a)
        out[f"{name}.b_q_weight"] = mq.numpy()
        out[f"{name}.b_scales"] = scales
        out[f"{name}.w_ref"] = bits16(w_ref)
        out[f"{name}.c_ref"] = gr.gemm_ref(a, w_ref).numpy()
        for key, v in extra.items():
            out[f"{name}.{key}"] = v

    # uint8b128, group 128, bf16
    w = (torch.randn(k, n, generator=g) * 0.05).bfloat16()
    a = torch.randn(m, k, generator=g).bfloat16()
    w_ref, q, s, _ = qu.quantize_weights(w, st.uint8b128, 128)
    put("u8b128_bf16_g128", a, ml.gptq_marlin_repack(qu.pack_rows(q, 8), None, k, n, 8),
        bits16(ml.marlin_permute_scales(s, k, n, 128)), w_ref)

    # HQQ: uint4, fp16 scales and fp16 zero points, group 64
    q = torch.randint(0, 10, (k, n), generator=g, dtype=torch.int32)
    s = torch.randn(k // 64, n, generator=g).half()
    z = torch.randn(k // 64, n, generator=g).half()
    a = torch.randn(m, k, generator=g).half()
    mq = ml.gptq_marlin_repack(qu.gptq_pack(q), None, k, n)
    ms, mz = ml.marlin_permute_scales(s, k, n, 64), ml.marlin_permute_scales(z, k, n, 64)
    put("hqq_f16_g64", a, mq, bits16(ms), gr.dequant_marlin_float_zp(mq, ms, mz, k, n), b_zeros_f16=bits16(mz))

    # float8_e4m3fn, channel-wise scales, fp16 (scales carry the exponent offset 2^8)
    w = torch.randn(k, n, generator=g).half()
    a = torch.randn(m, k, generator=g).half()
    w_ref, codes, s = qu.quantize_fp8(w, -1)
    ms = (ml.marlin_permute_scales(s, k, n, k).double() * gr.fp8_scale_offset(torch.float16)).half()
    put("fp8_f16_chan", a, ml.marlin_weights_closed_form8(codes.to(torch.int32)), bits16(ms), w_ref)

    # float4_e2m1f, NVFP4 (fp16) and MXFP4 (bf16)
    codes = torch.randint(0, 16, (k, n), generator=g, dtype=torch.int32)
    mq = ml.gptq_marlin_repack(qu.gptq_pack(codes), None, k, n)
    a = torch.randn(m, k, generator=g).half()
    s = (torch.rand(k // 16, n, generator=g) * 3 + 0.02).to(torch.float8_e4m3fn).half()
    ms = _regroup_fp4_scales(ml.marlin_permute_scales(s, k, n, 16))
    byts = ((ms * 128).view(torch.int16) << 1).view(torch.uint8)[:, 1::2].contiguous()
    gs = torch.tensor([0.0371], dtype=torch.float16)
    gs_proc = (gs.double() * 2.0 ** 7).half()
    put("nvfp4_f16", a, mq, byts.numpy(), gr.dequant_marlin_fp4(mq, byts, gs_proc, k, n, torch.float16),
        global_scale=bits16(gs_proc))
    a = torch.randn(m, k, generator=g).bfloat16()
    sb = torch.randint(110, 125, (k // 32, n), generator=g, dtype=torch.uint8)
    ms = _regroup_fp4_scales(ml.marlin_permute_scales(sb.view(torch.float8_e8m0fnu).to(torch.bfloat16), k, n, 32))
    byts = ms.to(torch.float8_e8m0fnu).view(torch.uint8).contiguous()
    put("mxfp4_bf16", a, mq, byts.numpy(), gr.dequant_marlin_fp4(mq, byts, None, k, n, torch.bfloat16))
    np.savez_compressed(os.path.join(HERE, "other_types.npz"), **out)


if __name__ == "__main__":
    repack_cases()
    gemm_cases()
    moe_align_cases()
    other_type_cases()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
