"""Dequantize-then-matmul reference for the W4A16 GEMM (CPU oracle, test infrastructure only).

The reference's kernel test (tests/kernels/quantization/test_marlin_gemm.py:228-361)
checks `gptq_marlin_gemm` against `torch.matmul(a, w_ref)` where `w_ref` is the
dequantised weight produced by the quantizer (quant_utils.py:427-432:
w_ref = (q - zp) * s in the weight dtype).  Here the same thing is computed from the
tensors the op actually receives, so layout decode, scale/zero indexing and act-order
are all part of what is checked:

  dequant_marlin(...)   Marlin-layout operands  -> w [K, N] in the activation dtype
  dequant_marlin_float_zp(...)  the same for fp16 zero points (HQQ)
  dequant_marlin_fp8(...)       the same for float8_e4m3fn weights
  dequant_marlin_fp4(...)       the same for float4_e2m1f weights (NVFP4 / MXFP4 scale bytes)
  dequant_checkpoint()  GPTQ / AWQ checkpoint   -> w [K, N]   (the CPU baseline path:
                        unpack nibbles, (q-8)*s or (q-z)*s group-broadcast)
  gemm_ref(a, w)        fp32 matmul (+ bias), result in fp32

Pinned by (tests/test_oracle_quant.py, the dequantisation section): dequant_marlin(repack(x)) == w_ref of the
quantizer bit-for-bit for every (type, group, act-order) combination;
dequant_checkpoint == w_ref likewise; fp32 matmul is torch's.
"""
import numpy as np
import torch

from .marlin_layout import (marlin_unpack_weights, marlin_unpack_weights8, marlin_unpack_zero_points,
                            marlin_unpermute_scales)
from .quant_utils import awq_unpack, unpack_rows


def _expand_groups(t: torch.Tensor, size_k: int, g_idx=None) -> torch.Tensor:
    """[G, N] -> [K, N] by group broadcast (contiguous groups) or g_idx lookup."""
    g = t.shape[0]
    if g_idx is not None and len(g_idx) > 0:
        return t[g_idx.long()]
    if g == 1:
        return t.expand(size_k, -1)
    assert size_k % g == 0
    return t.repeat_interleave(size_k // g, dim=0)


def dequant_marlin(b_q_weight, b_scales, b_zeros, g_idx, size_k, size_n, bias8: bool, dtype, num_bits: int = 4):
    """Marlin operands -> dense w[K, N] (row i = Marlin row i, i.e. after act-order sort).

    b_scales [G, N] Marlin-permuted; b_zeros int32 [G, N/8] Marlin-packed or None; bias8: the stored value
    carries the type's bias (8 for uint4b8, 128 for uint8b128);
    g_idx: sorted group id per Marlin row (only when the scale row is looked up per row).
    """
    q = marlin_unpack_weights(b_q_weight) if num_bits == 4 else marlin_unpack_weights8(b_q_weight)
    assert tuple(q.shape) == (size_k, size_n)
    num_groups = b_scales.shape[0]
    grouped = num_groups > 1
    s = marlin_unpermute_scales(b_scales, grouped).to(dtype)
    s_full = _expand_groups(s, size_k, g_idx)
    if b_zeros is not None and b_zeros.numel() > 0:
        z = marlin_unpack_zero_points(b_zeros)
        z_full = _expand_groups(z, size_k, g_idx)
        qz = q - z_full
    else:
        qz = q - ((8 if num_bits == 4 else 128) if bias8 else 0)
    return qz.to(dtype) * s_full


def dequant_marlin_float_zp(b_q_weight, b_scales, b_zeros, size_k, size_n):
    """HQQ operands (uint4 weights, fp16 scales and fp16 zero points, both [G, N] and Marlin-permuted like scales)
    -> dense fp16 w[K, N] as the reference kernel forms its B operand: zs = half(zp * s) rounded once, then
    w = fma(q, s, -zs) rounded once (marlin_template.h:174-181 scale_and_sub, :1235-1240).  Computed in float64,
    where q * s - zs is exact, and rounded to fp16 once.

    The reference's test compares against (q - zp) * s in fp16 tensor arithmetic with a mean-relative gate of 0.04
    (tests/kernels/quantization/test_marlin_gemm.py:524-535); `float_zp_test_ref` below is that formula.
    Pinned by (tests/test_oracle_quant.py): hand-computed words where the two roundings differ from the test
    formula, zp = 0 reducing to the plain q * s product, and agreement with `float_zp_test_ref` to 2 fp16 ulps of
    max(|q s|, |zp s|) on random data."""
    q = marlin_unpack_weights(b_q_weight)
    assert tuple(q.shape) == (size_k, size_n)
    assert b_scales.dtype == torch.float16 and b_zeros.dtype == torch.float16
    s = marlin_unpermute_scales(b_scales, True)
    z = marlin_unpermute_scales(b_zeros, True)
    zs = (z * s)                                  # fp16 product, one rounding
    s_full = _expand_groups(s, size_k).double()
    zs_full = _expand_groups(zs, size_k).double()
    return (q.double() * s_full - zs_full).to(torch.float16)


def float_zp_test_ref(q, scale, zero, group_size: int):
    """The reference test's dequantisation for HQQ (test_marlin_gemm.py:524-529): q uint8 [N, K], scale and zero
    fp16 [N, K/group]; returns w [K, N] = ((q - zero) * scale) evaluated in fp16 tensor arithmetic."""
    n, k = q.shape
    b_flat = q.reshape(-1, group_size)
    dequant = (b_flat.to(torch.float16) - zero.reshape(-1, 1)) * scale.reshape(-1, 1)
    return dequant.reshape(n, k).transpose(1, 0).contiguous()


def fp8_e4m3fn_table() -> torch.Tensor:
    """float64 value of each of the 256 float8_e4m3fn codes by the format's closed form (OCP 8-bit float spec,
    E4M3: bias 7, no infinities, S.1111.111 = NaN): (-1)^s 2^(e-7) (1 + m/8) for e > 0, (-1)^s 2^-6 (m/8) for e = 0.
    Pinned by (tests/test_oracle_quant.py): literal codes (0x38 = 1, 0x7E = 448, 0x01 = 2^-9, 0x08 = 2^-6,
    0xC0 = -2) and agreement with torch's own float8_e4m3fn -> float conversion on all 254 finite codes."""
    vals = []
    for code in range(256):
        sgn = -1.0 if code & 0x80 else 1.0
        e, m = (code >> 3) & 0xF, code & 7
        if e == 15 and m == 7:
            vals.append(float("nan"))
        elif e == 0:
            vals.append(sgn * 2.0 ** -6 * (m / 8.0))
        else:
            vals.append(sgn * 2.0 ** (e - 7) * (1.0 + m / 8.0))
    return torch.tensor(vals, dtype=torch.float64)


def fp8_scale_offset(dtype) -> float:
    """Factor the reference folds into fp8 Marlin scales at load time (marlin_utils_fp8.py:25-37)."""
    return 2.0 ** 8 if dtype == torch.float16 else 2.0 ** 120


def dequant_marlin_fp8(b_q_weight, b_scales_fused, size_k, size_n, dtype):
    """fp8 bytes in the 8-bit Marlin layout + Marlin-permuted scales carrying the exponent offset -> dense w[K, N]
    = fp8.to(dtype) * s evaluated in `dtype` (one rounding), the w_ref of the reference's marlin_quant_fp8_torch
    (marlin_utils_fp8.py:313-351)."""
    codes = marlin_unpack_weights8(b_q_weight)
    assert tuple(codes.shape) == (size_k, size_n)
    x = fp8_e4m3fn_table()[codes.long()].to(dtype)
    grouped = b_scales_fused.shape[0] > 1
    s = marlin_unpermute_scales(b_scales_fused, grouped)
    s = (s.double() / fp8_scale_offset(dtype)).to(dtype)
    return x * _expand_groups(s, size_k)


FP4_E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)   # magnitude of codes 0..7; bit 3 is the sign (OCP MX v1.0)


def fp4_scale_byte_position(group: int, perm_col: int, size_n: int) -> int:
    """Flat byte offset, in the processed fp4 scale tensor [G, N], of the scale that sits at (group, perm_col) of
    the Marlin-permuted scale matrix — closed form of the regrouping in marlin_utils_fp4.py:38-47:
    rows are taken in pairs; inside a pair the 16 values (row 2i | row 2i+1) of each 8-column chunk are adjacent;
    inside every run of 4 the middle two are swapped."""
    chunk, e = perm_col // 8, perm_col % 8
    pos = (e & 4) | ((e & 1) << 1) | ((e >> 1) & 1)          # (0, 2, 1, 3) applied to the low two bits
    return (group // 2) * 2 * size_n + chunk * 16 + (group % 2) * 8 + pos


def fp4_unprocess_scales(b_scales, fmt: str) -> torch.Tensor:
    """Processed scale bytes [G, N] (uint8 view) -> true scales float64 [G, N] in Marlin-permuted column order.
    fmt "nvfp4": byte = high byte of half(s * 2^7) << 1, i.e. s = half(byte << 7) / 2^7;  "mxfp4": s = 2^(byte - 127)."""
    raw = b_scales.view(torch.uint8)
    g, n = raw.shape
    flat = raw.reshape(-1)
    idx = torch.tensor([[fp4_scale_byte_position(r, c, n) for c in range(n)] for r in range(g)])
    by = flat[idx].to(torch.int32)
    if fmt == "nvfp4":
        return (by << 7).to(torch.int16).view(torch.float16).double() / 128.0
    return torch.pow(torch.tensor(2.0, dtype=torch.float64), (by - 127).double())


def dequant_marlin_fp4(b_q_weight, b_scales, global_scale, size_k, size_n, dtype):
    """float4_e2m1f codes in the 4-bit Marlin layout + processed scale bytes (+ processed NVFP4 global scale, or None
    for MXFP4) -> dense w[K, N] = code value * scale * global scale, exact in float64 and rounded once to `dtype`.
    (The reference's test helper multiplies in `dtype` from left to right, marlin_utils_fp4.py:325-333, which rounds
    twice: the two agree to one unit in the last place.)
    Pinned by (tests/test_oracle_quant.py): the code table and byte literals, the closed-form byte position against the
    restated regrouping, round trips of random scales, and agreement with the test helper's formula to 1 ulp."""
    codes = marlin_unpack_weights(b_q_weight)
    assert tuple(codes.shape) == (size_k, size_n)
    mag = torch.tensor(FP4_E2M1_VALUES, dtype=torch.float64)[(codes & 7).long()]
    x = torch.where((codes & 8) != 0, -mag, mag)
    fmt = "nvfp4" if global_scale is not None else "mxfp4"
    s_perm = fp4_unprocess_scales(b_scales, fmt)
    s = marlin_unpermute_scales(s_perm, True)
    gs = 1.0
    if global_scale is not None:
        gs = float(global_scale.double().reshape(-1)[0]) / (2.0 ** 7 if dtype == torch.float16 else 2.0 ** 119)
    return (x * _expand_groups(s, size_k) * gs).to(dtype)


def dequant_checkpoint(qweight, scales, qzeros, g_idx, fmt: str, dtype):
    """Checkpoint tensors -> dense w[K, N] in original row order.

    fmt "gptq": qweight int32 [K/8, N], symmetric uint4b8 (qzeros ignored), g_idx optional.
    fmt "awq":  qweight int32 [K, N/8], qzeros int32 [G, N/8] (AWQ interleave), scales [G, N].
    """
    if fmt == "gptq":
        q = unpack_rows(qweight, 4) - 8
    elif fmt == "awq":
        q = awq_unpack(qweight, 4)
    else:
        raise ValueError(fmt)
    k = q.shape[0]
    s_full = _expand_groups(scales.to(dtype), k, g_idx)
    if fmt == "awq":
        q = q - _expand_groups(awq_unpack(qzeros, 4), k, g_idx)
    return q.to(dtype) * s_full


def gemm_ref(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    out = a.float() @ w.float()
    if bias is not None:
        out = out + bias.float()
    return out


def error_metrics(out: torch.Tensor, ref: torch.Tensor) -> dict:
    """max|d|/max|ref| (the stated 2e-2 / 4e-2 gate) and the reference test's
    mean|d|/mean|ref| (< 0.04, test_marlin_gemm.py:78-81)."""
    d = (out.float().cpu() - ref.float().cpu()).abs()
    r = ref.float().cpu().abs()
    return {"max_rel": float(d.max() / r.max().clamp(min=1e-30)),
            "mean_rel": float(d.mean() / r.mean().clamp(min=1e-30))}
