"""Pins the oracle's quantizers, checkpoint packers, type ids and dequantisation (CPU only)."""
import numpy as np
import pytest
import torch

from oracle import gemm_ref as gr
from oracle import marlin_layout as ml
from oracle import quant_utils as qu
from oracle import scalar_types as st


def u32(t):
    return t.numpy().view(np.uint32)


# ---------------------------------------------------------------------------------- type ids
def test_type_ids_literal():
    # mantissa << 8 | bias << 17 | nan_repr(IEEE = 1) << 50
    assert st.uint4.id == (4 << 8) | (1 << 50) == 1125899906843648
    assert st.uint4b8.id == (4 << 8) | (8 << 17) | (1 << 50) == 1125899907892224
    assert st.uint8b128.id == (8 << 8) | (128 << 17) | (1 << 50) == 1125899923621888
    assert (st.uint4b8.min(), st.uint4b8.max()) == (-8, 7)
    assert (st.uint4.min(), st.uint4.max()) == (0, 15)


# ----------------------------------------------------------------------------------- packers
def test_pack_rows_literal_and_roundtrip():
    q = torch.arange(8, dtype=torch.int32).view(8, 1)            # rows 0..7 -> nibble i = i
    assert int(u32(qu.pack_rows(q, 4))[0, 0]) == 0x76543210
    q = torch.tensor([[15]] * 8, dtype=torch.int32)
    assert int(qu.pack_rows(q, 4)[0, 0]) == -1                   # 0xffffffff as int32
    r = torch.randint(0, 16, (64, 24), generator=torch.Generator().manual_seed(0), dtype=torch.int32)
    assert torch.equal(qu.unpack_rows(qu.pack_rows(r, 4), 4), r)
    assert qu.gptq_pack(r).shape == (8, 24)


def test_pack_cols_literal_and_roundtrip():
    q = torch.arange(8, dtype=torch.int32).view(1, 8)
    assert int(u32(qu.pack_cols(q, 4))[0, 0]) == 0x76543210
    r = torch.randint(0, 16, (5, 64), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    assert torch.equal(qu.unpack_cols(qu.pack_cols(r, 4), 4), r)


def test_awq_pack_literal_and_roundtrip():
    # nibble t of the word holds column (0,2,4,6,1,3,5,7)[t]
    q = torch.arange(8, dtype=torch.int32).view(1, 8)
    assert int(u32(qu.awq_pack(q))[0, 0]) == 0x75316420
    r = torch.randint(0, 16, (7, 128), generator=torch.Generator().manual_seed(2), dtype=torch.int32)
    assert torch.equal(qu.awq_unpack(qu.awq_pack(r)), r)
    # brute force
    p = u32(qu.awq_pack(r))
    for c in range(16):
        word = 0
        for t, o in enumerate((0, 2, 4, 6, 1, 3, 5, 7)):
            word |= int(r[3, 8 * c + o]) << (4 * t)
        assert int(p[3, c]) == word


# -------------------------------------------------------------------------------- quantizers
def test_symmetric_rule_hand_built_groups():
    """uint4b8: s = max(|max/7|, |min/-8|); stored value = round(w/s) + 8."""
    w = torch.zeros(8, 2, dtype=torch.float32)
    w[:, 0] = torch.tensor([7.0, -3.5, 0, 1, 2, 3, -1, -2])      # max 7 -> s = 1 ; -3.5 -> round-half-even -4
    w[:, 1] = torch.tensor([-16.0, 14, 0, 2, 4, 6, -2, -4])      # |min|/8 = 2 = max/7
    w_ref, q, s, zp = qu.quantize_weights(w, st.uint4b8, 8)
    assert zp is None
    assert s.tolist() == [[1.0, 2.0]]
    assert q[:, 0].tolist() == [15, 4, 8, 9, 10, 11, 7, 6]
    assert q[:, 1].tolist() == [0, 15, 8, 9, 10, 11, 7, 6]
    assert torch.equal(w_ref, (q - 8).float() * s.repeat_interleave(8, 0))


def test_zero_point_rule_hand_built_group():
    """uint4 + zp: s = (max-min)/15, zp = round(|min/s|), q = clamp(round(w/s) + zp, 0, 15)."""
    w = torch.tensor([[-5.0], [10.0], [0.0], [1.0], [2.4], [-1.0], [7.0], [9.6]])
    w_ref, q, s, zp = qu.quantize_weights(w, st.uint4, 8, zero_points=True)
    assert s.tolist() == [[1.0]] and zp.tolist() == [[5]]
    assert q[:, 0].tolist() == [0, 15, 5, 6, 7, 4, 12, 15]
    assert torch.equal(w_ref[:, 0], (q[:, 0] - 5).float())


def test_benchmark_rules():
    g = torch.Generator().manual_seed(0)
    w = (torch.randn(256, 16, generator=g) * 0.02).half()
    w_ref, q, s = qu.quantize_absmax7(w, 128)
    wg = w.float().view(2, 128, 16)
    assert torch.equal(s, (wg.abs().amax(1) / 7).half())
    assert q.min() >= 1 and q.max() <= 15                       # absmax/7 never reaches -8
    assert torch.equal(w_ref, ((q - 8).half().view(2, 128, 16) * s.view(2, 1, 16)).view(256, 16))
    w_ref, q, s, zp = qu.quantize_minmax_zp(w.bfloat16(), 128)
    assert q.min() >= 0 and q.max() <= 15 and zp.min() >= 0 and zp.max() <= 15
    assert torch.equal(w_ref, ((q.view(2, 128, 16) - zp.view(2, 1, 16)).bfloat16() * s.view(2, 1, 16)).view(256, 16))


@pytest.mark.parametrize("group", [-1, 32, 128])
def test_channelwise_and_group_shapes(group):
    w = torch.randn(256, 64, generator=torch.Generator().manual_seed(3)).half()
    w_ref, q, s, _ = qu.quantize_weights(w, st.uint4b8, group)
    assert s.shape == (1 if group == -1 else 256 // group, 64)
    assert q.min() >= 0 and q.max() <= 15
    # reconstruction error bounded by half a step per element
    gs = 256 if group == -1 else group
    step = s.float().repeat_interleave(gs, 0)
    assert ((w.float() - w_ref.float()).abs() <= 0.5 * step * 1.01 + 1e-3).all()


def test_act_order_identities():
    g = torch.Generator().manual_seed(4)
    w = torch.randn(256, 64, generator=g).half()
    perm = torch.randperm(256, generator=g)
    w_ref, q, s, g_idx, rp = qu.gptq_quantize_weights(w, st.uint4b8, 64, True, perm)
    w0, q0, s0, _ = qu.quantize_weights(w, st.uint4b8, 64)
    assert torch.equal(rp, perm) and torch.equal(s, s0)
    assert torch.equal(q, q0[perm]) and torch.equal(w_ref, w0[perm])
    assert torch.equal(g_idx.long(), perm // 64)
    qs, gs, order = qu.sort_weights(q, g_idx)
    assert (gs[1:] >= gs[:-1]).all()
    assert torch.equal(qs, q[order.long()])
    assert torch.equal(torch.bincount(gs.long()), torch.full((4,), 64))


# -------------------------------------------------------------------- dequantisation identity
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [-1, 32, 128])
@pytest.mark.parametrize("mode", ["gptq", "gptq_act_order", "awq"])
def test_dequant_reproduces_quantizer_w_ref(dtype, group, mode):
    k, n = 256, 128
    if mode == "gptq_act_order" and group == -1:
        pytest.skip("act-order needs groups")
    g = torch.Generator().manual_seed(5)
    w = torch.randn(k, n, generator=g).to(dtype)
    gs = k if group == -1 else group
    if mode == "awq":
        w_ref, q, s, zp = qu.quantize_weights(w, st.uint4, group, zero_points=True)
        mq = ml.awq_marlin_repack(qu.awq_pack(q), k, n)
        mz = ml.awq_to_marlin_zero_points(qu.awq_pack(zp), zp.shape[0], n)
        ms = ml.marlin_permute_scales(s, k, n, gs)
        assert torch.equal(gr.dequant_marlin(mq, ms, mz, None, k, n, False, dtype), w_ref)
        assert torch.equal(gr.dequant_checkpoint(qu.awq_pack(q), s, qu.awq_pack(zp), None, "awq", dtype), w_ref)
        return
    act = mode == "gptq_act_order"
    w_ref, q, s, g_idx, _ = qu.gptq_quantize_weights(w, st.uint4b8, group, act, torch.randperm(k, generator=g) if act else None)
    ms = ml.marlin_permute_scales(s, k, n, gs)
    if act:
        _, g_sorted, order = qu.sort_weights(q, g_idx)
        mq = ml.gptq_marlin_repack(qu.gptq_pack(q), order, k, n)
        w_sorted = gr.dequant_marlin(mq, ms, None, g_sorted, k, n, True, dtype)
        assert torch.equal(w_sorted, w_ref[order.long()])
        assert torch.equal(gr.dequant_checkpoint(qu.gptq_pack(q), s, None, g_idx, "gptq", dtype), w_ref)
    else:
        mq = ml.gptq_marlin_repack(qu.gptq_pack(q), None, k, n)
        assert torch.equal(gr.dequant_marlin(mq, ms, None, None, k, n, True, dtype), w_ref)
        assert torch.equal(gr.dequant_checkpoint(qu.gptq_pack(q), s, None, None, "gptq", dtype), w_ref)


def test_gemm_ref_is_fp32_matmul_plus_bias():
    a = torch.tensor([[1.0, 2.0], [0.5, -1.0]]).half()
    w = torch.tensor([[2.0, 0.0], [1.0, 4.0]]).half()
    out = gr.gemm_ref(a, w, torch.tensor([1.0, -1.0]).half())
    assert out.dtype == torch.float32
    assert out.tolist() == [[5.0, 7.0], [1.0, -5.0]]
    m = gr.error_metrics(out + torch.tensor([[0.0, 0.7], [0.0, 0.0]]), out)
    assert abs(m["max_rel"] - 0.1) < 1e-6 and abs(m["mean_rel"] - 0.7 / 18.0) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [-1, 128])
def test_uint8b128_quantizer_and_dequant(dtype, group):
    k, n = 256, 64
    w = torch.randn(k, n, generator=torch.Generator().manual_seed(6)).to(dtype)
    w_ref, q, s, zp = qu.quantize_weights(w, st.uint8b128, group)
    assert zp is None and q.min() >= 0 and q.max() <= 255
    gs = k if group == -1 else group
    assert torch.equal(w_ref, (q - 128).to(dtype) * s.repeat_interleave(gs, 0))
    mq = ml.gptq_marlin_repack(qu.pack_rows(q, 8), None, k, n, 8)
    ms = ml.marlin_permute_scales(s, k, n, gs)
    assert torch.equal(gr.dequant_marlin(mq, ms, None, None, k, n, True, dtype, num_bits=8), w_ref)
    # symmetric rule: s = max(|max| / 127, |min| / 128)
    wg = w.float().view(k // gs, gs, n)
    want = torch.maximum(wg.amax(1).abs() / 127, wg.amin(1).abs() / 128)
    assert torch.allclose(s.float(), want, rtol=2e-2)


# ------------------------------------------------------------------ float zero points (HQQ)
def _hqq_operands(q, s, z):
    """q int [K, N], s / z fp16 [G, N] -> Marlin operands (group 64)."""
    k, n = q.shape
    mq = ml.gptq_marlin_repack(qu.gptq_pack(q.to(torch.int32)), None, k, n)
    return mq, ml.marlin_permute_scales(s, k, n, 64), ml.marlin_permute_scales(z, k, n, 64)


def test_float_zp_reduces_to_integer_zero_points():
    """s = 1 and integer zero points: every step is exact, so the result is q - z, which is also what the packed
    integer zero-point path (pinned above against the quantizer's w_ref) gives."""
    g = torch.Generator().manual_seed(11)
    k, n = 128, 64
    q = torch.randint(0, 16, (k, n), generator=g, dtype=torch.int32)
    z = torch.randint(0, 16, (k // 64, n), generator=g, dtype=torch.int32)
    s = torch.ones(k // 64, n, dtype=torch.float16)
    mq, ms, mz = _hqq_operands(q, s, z.half())
    w = gr.dequant_marlin_float_zp(mq, ms, mz, k, n)
    assert torch.equal(w, (q - z.repeat_interleave(64, 0)).half())
    mz_int = ml.marlin_zero_points(z, k // 64, n)
    assert torch.equal(w, gr.dequant_marlin(mq, ms, mz_int, None, k, n, False, torch.float16))


def test_float_zp_zero_is_plain_scaling_and_pow2_scales_match_the_test_formula():
    g = torch.Generator().manual_seed(12)
    k, n = 128, 128
    q = torch.randint(0, 16, (k, n), generator=g, dtype=torch.int32)
    s = torch.randn(k // 64, n, generator=g).half()
    z0 = torch.zeros(k // 64, n, dtype=torch.float16)
    mq, ms, mz = _hqq_operands(q, s, z0)
    assert torch.equal(gr.dequant_marlin_float_zp(mq, ms, mz, k, n), q.half() * s.repeat_interleave(64, 0))
    # power-of-two scales: zp * s is exact, and so is (q - zp) * s whenever q - zp is representable
    s2 = torch.tensor([0.25, 2.0]).half().view(2, 1).expand(2, n).contiguous()
    z = (torch.randint(0, 64, (k // 64, n), generator=g).half() / 4)            # multiples of 1/4 below 16
    mq, ms, mz = _hqq_operands(q, s2, z)
    ref = gr.float_zp_test_ref(q.t().contiguous().to(torch.uint8), s2.t().contiguous(), z.t().contiguous(), 64)
    assert torch.equal(gr.dequant_marlin_float_zp(mq, ms, mz, k, n), ref)


def test_float_zp_hand_derived_rounding_case():
    """s = zp = 1 + 2^-10, q = 1:  zp*s = 1 + 2^-9 + 2^-20 rounds to 1 + 2^-9;  q*s - zs = -2^-10 exactly.
    (The reference test's formula (q - zp) * s gives -2^-10 (1 + 2^-10) instead: the kernel's two roundings differ.)"""
    k, n = 64, 64
    q = torch.ones(k, n, dtype=torch.int32)
    v = torch.full((1, n), 1.0 + 2.0 ** -10, dtype=torch.float16)
    mq, ms, mz = _hqq_operands(q, v, v)
    w = gr.dequant_marlin_float_zp(mq, ms, mz, k, n)
    assert torch.equal(w, torch.full((k, n), -(2.0 ** -10), dtype=torch.float16))
    ref = gr.float_zp_test_ref(q.t().contiguous().to(torch.uint8), v.t().contiguous(), v.t().contiguous(), 64)
    assert float(ref[0, 0]) == -(2.0 ** -10) * (1 + 2.0 ** -10)


def test_float_zp_close_to_the_reference_test_formula():
    g = torch.Generator().manual_seed(13)
    k, n = 256, 128
    q = torch.randint(0, 10, (k, n), generator=g, dtype=torch.int32)             # as the reference test draws them
    s = torch.randn(k // 64, n, generator=g).half()
    z = torch.randn(k // 64, n, generator=g).half()
    mq, ms, mz = _hqq_operands(q, s, z)
    w = gr.dequant_marlin_float_zp(mq, ms, mz, k, n).float()
    ref = gr.float_zp_test_ref(q.t().contiguous().to(torch.uint8), s.t().contiguous(), z.t().contiguous(), 64).float()
    s_full, z_full = s.float().repeat_interleave(64, 0), z.float().repeat_interleave(64, 0)
    bound = 2.0 ** -9 * torch.maximum((q.float() * s_full).abs(), (z_full * s_full).abs()) + 1e-7
    assert ((w - ref).abs() <= bound).all()


# ------------------------------------------------------------------------------ fp8 weights
def test_fp8_table_literals_and_torch_conversion():
    t = gr.fp8_e4m3fn_table()
    assert t[0x38] == 1.0 and t[0x7E] == 448.0 and t[0x01] == 2.0 ** -9 and t[0x08] == 2.0 ** -6 and t[0xC0] == -2.0
    assert t[0x00] == 0.0 and t[0x7F].isnan() and t[0xFF].isnan()
    finite = [c for c in range(256) if c & 0x7F != 0x7F]
    codes = torch.tensor(finite, dtype=torch.uint8)
    assert torch.equal(codes.view(torch.float8_e4m3fn).double(), t[codes.long()])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [-1, 128])
def test_fp8_dequant_reproduces_quantizer_w_ref(dtype, group):
    k, n = 256, 128
    w = torch.randn(k, n, generator=torch.Generator().manual_seed(21)).to(dtype)
    w_ref, codes, s = qu.quantize_fp8(w, group)
    assert codes.dtype == torch.uint8 and s.shape == (1 if group == -1 else k // group, n)
    assert (codes & 0x7F != 0x7F).all()
    # |w - w_ref| within half an fp8 step (2^-4 relative) plus the 16-bit roundings
    assert ((w.float() - w_ref.float()).abs() <= w.float().abs() * 2.0 ** -4 + s.float().repeat_interleave(k // s.shape[0], 0) * 2.0 ** -9).all()
    mq = ml.marlin_weights_closed_form8(codes.to(torch.int32))
    ms = ml.marlin_permute_scales(s, k, n, k if group == -1 else group)
    ms_fused = (ms.double() * gr.fp8_scale_offset(dtype)).to(dtype)
    assert torch.equal(gr.dequant_marlin_fp8(mq, ms_fused, k, n, dtype), w_ref)


# ------------------------------------------------------------------------------ fp4 weights
def _regroup_restated(t):
    """The reference's regrouping of a Marlin-permuted [G, N] tensor, restated with its own tensor ops
    (marlin_utils_fp4.py:38-47), as the thing the closed-form byte position is checked against."""
    g, n = t.shape
    t = t.view(g // 2, 2, -1, 8).permute(0, 2, 1, 3).reshape(g, n)
    return t.reshape(-1, 4)[:, [0, 2, 1, 3]].reshape(g, n)


def test_fp4_code_table_and_scale_byte_literals():
    assert gr.FP4_E2M1_VALUES == (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
    # NVFP4 scale byte: high byte of half(s * 2^7) << 1.  1.0 -> half(128) = 0x5800 -> 0xB0; 448 -> 0x7B00 -> 0xF6;
    # 2^-9 -> half(2^-2) = 0x3400 -> 0x68
    for s, byte in ((1.0, 0xB0), (448.0, 0xF6), (2.0 ** -9, 0x68), (0.5, 0xA8)):
        raw = torch.tensor([[byte] * 8] * 2, dtype=torch.uint8)
        assert torch.all(gr.fp4_unprocess_scales(raw, "nvfp4") == s)
    raw = torch.tensor([[127, 100, 120, 130] * 2] * 2, dtype=torch.uint8)
    got = gr.fp4_unprocess_scales(raw, "mxfp4")
    assert set(got.flatten().tolist()) == {1.0, 2.0 ** -27, 2.0 ** -7, 8.0}


def test_fp4_scale_byte_position_matches_the_regrouping():
    g, n = 6, 128
    ident = torch.arange(g * n, dtype=torch.int32).view(g, n)         # value = flat index in the permuted matrix
    out = _regroup_restated(ident).reshape(-1)
    for r in range(g):
        for c in range(n):
            assert int(out[gr.fp4_scale_byte_position(r, c, n)]) == r * n + c
    # hand-derived: rows 2, 3 (second pair), permuted column 8*5 + 3 of row 3: pair offset 2n*1, chunk 5 -> 80,
    # second row of the pair -> +8, element 3 of (0,2,1,3)-swapped run -> position 3
    assert gr.fp4_scale_byte_position(3, 43, n) == 2 * n + 80 + 8 + 3
    assert gr.fp4_scale_byte_position(0, 1, n) == 2 and gr.fp4_scale_byte_position(0, 2, n) == 1


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_nvfp4_dequant_against_the_test_helper_formula(dtype):
    """w = value * global_scale * scale evaluated left to right in `dtype` (the reference helper's w_ref) agrees with
    the single-rounding oracle to one unit in the last place, and exactly when the global scale is a power of two."""
    k, n, group = 128, 64, 16
    g = torch.Generator().manual_seed(31)
    codes = torch.randint(0, 16, (k, n), generator=g, dtype=torch.int32)
    scales = (torch.rand(k // group, n, generator=g) * 4 + 0.01).to(torch.float8_e4m3fn)
    table = torch.tensor(gr.FP4_E2M1_VALUES + tuple(-v for v in gr.FP4_E2M1_VALUES), dtype=dtype)
    mq = ml.gptq_marlin_repack(qu.gptq_pack(codes), None, k, n)
    ms = ml.marlin_permute_scales(scales.to(dtype), k, n, group)
    byts = ((_regroup_restated(ms.to(torch.half)) * 128).view(torch.int16) << 1).view(torch.uint8)[:, 1::2].contiguous()
    for gs_val in (0.25, 0.0123):
        gs = torch.tensor(gs_val, dtype=dtype)
        gs_proc = (gs.double() * (2.0 ** 7 if dtype == torch.float16 else 2.0 ** 119)).to(dtype).view(1)
        w = gr.dequant_marlin_fp4(mq, byts, gs_proc, k, n, dtype)
        helper = table[codes.long()] * gs * scales.to(dtype).repeat_interleave(group, 0)
        if gs_val == 0.25:
            assert torch.equal(w, helper)
        else:
            ulp = torch.finfo(dtype).eps
            assert ((w.double() - helper.double()).abs() <= helper.double().abs() * ulp).all()


def test_mxfp4_dequant_is_exact():
    k, n, group = 128, 128, 32
    g = torch.Generator().manual_seed(32)
    codes = torch.randint(0, 16, (k, n), generator=g, dtype=torch.int32)
    sbytes = torch.randint(100, 125, (k // group, n), generator=g, dtype=torch.uint8)
    scales = sbytes.view(torch.float8_e8m0fnu).to(torch.bfloat16)
    table = torch.tensor(gr.FP4_E2M1_VALUES + tuple(-v for v in gr.FP4_E2M1_VALUES), dtype=torch.bfloat16)
    mq = ml.gptq_marlin_repack(qu.gptq_pack(codes), None, k, n)
    ms = ml.marlin_permute_scales(scales, k, n, group)
    byts = _regroup_restated(ms).to(torch.float8_e8m0fnu).view(torch.uint8)
    w = gr.dequant_marlin_fp4(mq, byts, None, k, n, torch.bfloat16)
    assert torch.equal(w, table[codes.long()] * scales.repeat_interleave(group, 0))
