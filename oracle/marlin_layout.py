"""Marlin weight / scale / zero-point / bias layouts (CPU oracle, test infrastructure only).

Reference statements followed:
  weights   vllm/model_executor/layers/quantization/utils/marlin_utils_test.py:32-93
            (marlin_permute_weights, marlin_weights, get_weight_perm) and the per-thread
            index arithmetic of csrc/quantization/gptq_marlin/gptq_marlin_repack.cu:107-204,
            csrc/quantization/gptq_marlin/awq_marlin_repack.cu:68-148
  scales    marlin_utils.py:278-298 (get_scale_perms, marlin_permute_scales)
  bias      marlin_utils.py:301-305
  zeros     marlin_utils.py:326-370 (marlin_zero_points, awq_to_marlin_zero_points)

The 8-bit weight layout (uint8b128) has the same two formulations (`marlin_weights_closed_form8`,
`marlin_weights_perm_table(num_bits=8)`) and is pinned the same way (tests/test_oracle_layout.py).

Two independent formulations of the weight layout are kept on purpose:
`marlin_weights_closed_form` (index arithmetic per output nibble) and
`marlin_weights_perm_table` (tile transpose + 1024-entry permutation + pack).
Pinned by (tests/test_oracle_layout.py): the two formulations agree; hand-derived
words for q[k,n]=k and q[k,n]=n%16; nibble-multiset conservation; brute-force
inverse on the minimal 16x64 tile; GPTQ-packed and AWQ-packed inputs of one logical
matrix repack to the same words; act-order repack == repack of the row-gathered
matrix; scale permutation closed forms and the 8x8-transpose involution; zero-point
closed form (word 8*ch+i, nibble t <- column 64*ch + i + 8*order[t]).
"""
import numpy as np
import torch

from .quant_utils import (AWQ_NIBBLE_ORDER, _to_i32_tensor, _u32, awq_unpack, pack_cols,
                          unpack_cols, unpack_rows)

TILE_K = 16
TILE_N = 64


# ----------------------------------------------------------------------------- weights
def marlin_weights_closed_form(q, perm=None) -> torch.Tensor:
    """4-bit layout by direct index arithmetic.

    Output int32 [K/16, 2N].  Word (kt, nt*128 + th*4 + w), th in [0,32), w in [0,4):
      r = 2*(th % 4), c = th // 4, n0 = 64*nt + 16*w + c, k0 = 16*kt + r
      nibble j holds q[k0 + dk[j], n0 + dn[j]] with
      dk = (0, 8, 0, 8, 1, 9, 1, 9), dn = (0, 0, 8, 8, 0, 0, 8, 8).
    With act-order, source row k is replaced by perm[k].
    """
    qa = _u32(q)
    k, n = qa.shape
    assert k % TILE_K == 0 and n % TILE_N == 0
    if perm is not None and len(perm) > 0:
        qa = qa[np.asarray(perm, dtype=np.int64)]
    kt = np.arange(k // 16)[:, None, None, None]
    nt = np.arange(n // 64)[None, :, None, None]
    th = np.arange(32)[None, None, :, None]
    w = np.arange(4)[None, None, None, :]
    k0 = 16 * kt + 2 * (th % 4)
    n0 = 64 * nt + 16 * w + th // 4
    dk = (0, 8, 0, 8, 1, 9, 1, 9)
    dn = (0, 0, 8, 8, 0, 0, 8, 8)
    out = np.zeros((k // 16, n // 64, 32, 4), dtype=np.uint32)
    for j in range(8):
        kk, nn = np.broadcast_arrays(k0 + dk[j], n0 + dn[j])
        out |= (qa[kk, nn] & 0xF) << np.uint32(4 * j)
    return _to_i32_tensor(out.reshape(k // 16, 2 * n))


def marlin_weights_closed_form8(q, perm=None) -> torch.Tensor:
    """8-bit layout by direct index arithmetic (gptq_marlin_repack.cu:119-203 with num_bits = 8).

    Output int32 [K/16, 4N].  Per k-tile and 64-column n-tile 256 words; word nt*256 + th*8 + 2*w + half
    (th in [0,32), w in [0,4), half in {0,1}) holds, with r = 2*(th % 4), c = th // 4, n = 64*nt + 16*w + c + 8*half,
    k0 = 16*kt + r, the bytes q[k0 + (0, 8, 1, 9)[j], n] for j = 0..3."""
    qa = _u32(q)
    k, n = qa.shape
    assert k % TILE_K == 0 and n % TILE_N == 0
    if perm is not None and len(perm) > 0:
        qa = qa[np.asarray(perm, dtype=np.int64)]
    kt = np.arange(k // 16)[:, None, None, None, None]
    nt = np.arange(n // 64)[None, :, None, None, None]
    th = np.arange(32)[None, None, :, None, None]
    w = np.arange(4)[None, None, None, :, None]
    half = np.arange(2)[None, None, None, None, :]
    k0 = 16 * kt + 2 * (th % 4)
    nn = 64 * nt + 16 * w + th // 4 + 8 * half
    out = np.zeros((k // 16, n // 64, 32, 4, 2), dtype=np.uint32)
    for j, dk in enumerate((0, 8, 1, 9)):
        kk, n2 = np.broadcast_arrays(k0 + dk, nn)
        out |= (qa[kk, n2] & 0xFF) << np.uint32(8 * j)
    return _to_i32_tensor(out.reshape(k // 16, 4 * n))


def marlin_unpack_weights8(marlin_w) -> torch.Tensor:
    """Inverse of the 8-bit layout: int32 [K/16, 4N] -> int32 [K, N] bytes."""
    wa = _u32(marlin_w)
    kt_n, words = wa.shape
    n = words // 4
    out = np.zeros((kt_n * 16, n), dtype=np.int32)
    wa = wa.reshape(kt_n, n // 64, 32, 4, 2)
    kt = np.arange(kt_n)[:, None, None, None, None]
    nt = np.arange(n // 64)[None, :, None, None, None]
    th = np.arange(32)[None, None, :, None, None]
    w = np.arange(4)[None, None, None, :, None]
    half = np.arange(2)[None, None, None, None, :]
    k0 = 16 * kt + 2 * (th % 4)
    nn = 64 * nt + 16 * w + th // 4 + 8 * half
    for j, dk in enumerate((0, 8, 1, 9)):
        kk, n2 = np.broadcast_arrays(k0 + dk, nn)
        out[kk, n2] = (wa >> np.uint32(8 * j)) & 0xFF
    return torch.from_numpy(out)


def weight_perm_table(num_bits: int = 4) -> np.ndarray:
    """1024-entry permutation over a flattened [64 n-cols ... ] 16x64 tile, built from the
    thread/fragment description: 32 threads x 4 sub-tiles x 8 values, then the
    within-word interleave (0,2,4,6,1,3,5,7)."""
    entries = []
    for th in range(32):
        col = th // 4
        base = []
        for blk in (0, 1):
            for row in (2 * (th % 4), 2 * (th % 4) + 1, 2 * (th % 4 + 4), 2 * (th % 4 + 4) + 1):
                base.append(16 * row + col + 8 * blk)
        for j in range(4):
            entries.extend(b + 256 * j for b in base)
    table = np.array(entries)
    order = np.array(AWQ_NIBBLE_ORDER if num_bits == 4 else (0, 2, 1, 3))
    return table.reshape(-1, len(order))[:, order].ravel()


def marlin_weights_perm_table(q, perm=None, num_bits: int = 4) -> torch.Tensor:
    """Same layout through the reference's test formulation
    (marlin_utils_test.py:32-63): 16x16 tile transpose, table gather, pack."""
    qa = _u32(q)
    k, n = qa.shape
    if perm is not None and len(perm) > 0:
        qa = qa[np.asarray(perm, dtype=np.int64)]
    t = qa.reshape(k // 16, 16, n // 16, 16).transpose(0, 2, 1, 3).reshape(k // 16, n * 16)
    table = weight_perm_table(num_bits)
    t = t.reshape(-1, table.size)[:, table].reshape(k // 16, n * 16)
    pf = 32 // num_bits
    out = np.zeros((k // 16, n * 16 // pf), dtype=np.uint32)
    for i in range(pf):
        out |= (t[:, i::pf] & ((1 << num_bits) - 1)) << np.uint32(num_bits * i)
    return _to_i32_tensor(out)


def gptq_marlin_repack(b_q_weight, perm, size_k: int, size_n: int, num_bits: int = 4) -> torch.Tensor:
    """GPTQ checkpoint int32 [K/pf, N] (+ optional row order) -> Marlin int32 [K/16, N*16/pf], pf = 32/num_bits."""
    assert num_bits in (4, 8)
    assert tuple(b_q_weight.shape) == (size_k // (32 // num_bits), size_n)
    q = unpack_rows(b_q_weight, num_bits)
    p = perm if perm is not None and len(perm) else None
    return marlin_weights_closed_form(q, p) if num_bits == 4 else marlin_weights_closed_form8(q, p)


def awq_marlin_repack(b_q_weight, size_k: int, size_n: int, num_bits: int = 4) -> torch.Tensor:
    """AWQ checkpoint int32 [K, N/pf] -> Marlin int32 [K/16, N*16/pf], pf = 32/num_bits."""
    assert num_bits in (4, 8)
    assert tuple(b_q_weight.shape) == (size_k, size_n // (32 // num_bits))
    q = awq_unpack(b_q_weight, num_bits)
    return marlin_weights_closed_form(q) if num_bits == 4 else marlin_weights_closed_form8(q)


def marlin_unpack_weights(marlin_w) -> torch.Tensor:
    """Inverse of the 4-bit layout: int32 [K/16, 2N] -> int32 [K, N] nibbles."""
    wa = _u32(marlin_w)
    kt_n, words = wa.shape
    n = words // 2
    k = kt_n * 16
    out = np.zeros((k, n), dtype=np.int32)
    wa = wa.reshape(kt_n, n // 64, 32, 4)
    kt = np.arange(kt_n)[:, None, None, None]
    nt = np.arange(n // 64)[None, :, None, None]
    th = np.arange(32)[None, None, :, None]
    w = np.arange(4)[None, None, None, :]
    k0 = 16 * kt + 2 * (th % 4)
    n0 = 64 * nt + 16 * w + th // 4
    dk = (0, 8, 0, 8, 1, 9, 1, 9)
    dn = (0, 0, 8, 8, 0, 0, 8, 8)
    for j in range(8):
        kk, nn = np.broadcast_arrays(k0 + dk[j], n0 + dn[j])
        out[kk, nn] = (wa >> np.uint32(4 * j)) & 0xF
    return torch.from_numpy(out)


# ------------------------------------------------------------------- scales / bias / zeros
def scale_perm_grouped() -> list[int]:
    return [i + 8 * j for i in range(8) for j in range(8)]


def scale_perm_single() -> list[int]:
    return [2 * i + j for i in range(4) for j in (0, 1, 8, 9, 16, 17, 24, 25)]


def marlin_permute_scales(s: torch.Tensor, size_k: int, size_n: int, group_size: int) -> torch.Tensor:
    if group_size < size_k and group_size != -1:
        p = scale_perm_grouped()
    else:
        p = scale_perm_single()
    return s.reshape(-1, len(p))[:, p].reshape(-1, size_n).contiguous()


def marlin_permute_bias(b: torch.Tensor) -> torch.Tensor:
    p = scale_perm_single()
    return b.reshape(-1, len(p))[:, p].reshape(b.shape).contiguous()


def marlin_zero_points(zp: torch.Tensor, num_groups: int, size_n: int, num_bits: int = 4) -> torch.Tensor:
    """Unpacked zp int [G, N] -> Marlin-packed int32 [G, N/8]."""
    assert num_bits == 4
    p = scale_perm_grouped()
    z = zp.reshape(-1, len(p))[:, p]
    z = z.reshape(-1, 8)[:, list(AWQ_NIBBLE_ORDER)].reshape(-1, size_n).contiguous()
    return pack_cols(z, num_bits)


def awq_to_marlin_zero_points(q_zp_packed: torch.Tensor, num_groups: int, size_n: int, num_bits: int = 4):
    """AWQ-packed zp int32 [G, N/8] -> Marlin-packed int32 [G, N/8]."""
    return marlin_zero_points(awq_unpack(q_zp_packed, num_bits), num_groups, size_n, num_bits)


def marlin_zero_points_closed_form(zp: torch.Tensor) -> torch.Tensor:
    """Independent statement: word 8*ch + i, nibble t <- zp[g, 64*ch + i + 8*order[t]]."""
    za = _u32(zp)
    g, n = za.shape
    out = np.zeros((g, n // 8), dtype=np.uint32)
    for ch in range(n // 64):
        for i in range(8):
            for t in range(8):
                out[:, 8 * ch + i] |= (za[:, 64 * ch + i + 8 * AWQ_NIBBLE_ORDER[t]] & 0xF) << np.uint32(4 * t)
    return _to_i32_tensor(out)


def marlin_unpermute_scales(s_perm: torch.Tensor, grouped: bool) -> torch.Tensor:
    """Inverse of marlin_permute_scales (used by the dequantising GEMM oracle)."""
    p = scale_perm_grouped() if grouped else scale_perm_single()
    inv = np.argsort(np.array(p))
    n = s_perm.shape[-1]
    return s_perm.reshape(-1, len(p))[:, torch.from_numpy(inv)].reshape(-1, n).contiguous()


def marlin_unpack_zero_points(zp_marlin: torch.Tensor) -> torch.Tensor:
    """Inverse of marlin_zero_points: int32 [G, N/8] -> int32 [G, N]."""
    raw = unpack_cols(zp_marlin, 4).numpy()                      # interleaved, scale-permuted
    g, n = raw.shape
    de = np.empty_like(raw).reshape(-1, 8)
    de[:, list(AWQ_NIBBLE_ORDER)] = raw.reshape(-1, 8)           # undo nibble interleave
    de = de.reshape(-1, 64)
    inv = np.argsort(np.array(scale_perm_grouped()))
    return torch.from_numpy(de[:, inv].reshape(g, n).astype(np.int32))
