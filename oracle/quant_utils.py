"""RTN quantizers and checkpoint packers (CPU oracle, test infrastructure only).

Restates the semantics of the reference's test/benchmark helpers in
vllm/model_executor/layers/quantization/utils/quant_utils.py:
  quantize_weights :376-468, gptq_quantize_weights :475-506, permute_rows :346-373,
  sort_weights :509-521, pack_rows :524-545, pack_cols :548-571, unpack_cols :574-602,
  gptq_pack :605-611, awq_pack :614-633.

Pinned by (tests/test_oracle_*.py): pack/unpack round trips and literal packed
words for hand-written matrices; quantizer closed forms on hand-built groups
(max/7 vs |min|/8 rule, zero-point = round(|min|/s)); dequantisation identity
w_ref == (q - bias - zp) * s recomputed with independent indexing; act-order
identities (g_idx sorted is non-decreasing, rows follow the same permutation).
The quantizers only have to be self-consistent: GPU results are compared with
this module's own dequantisation of the same integers.
"""
import numpy as np
import torch

from .scalar_types import WType

AWQ_NIBBLE_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)
AWQ_BYTE_ORDER = (0, 2, 1, 3)


def pack_factor(num_bits: int) -> int:
    assert 32 % num_bits == 0
    return 32 // num_bits


def _group_view(w: torch.Tensor, group_size: int):
    """[K, N] -> [K/g, g, N] view (no copy)."""
    k, n = w.shape
    return w.reshape(k // group_size, group_size, n)


def quantize_weights(w: torch.Tensor, wtype: WType, group_size: int, zero_points: bool = False):
    """Reference rule (quant_utils.py:376-468); arithmetic stays in w's own dtype.

    Returns (w_ref [K,N] dtype, q [K,N] int32 *stored* value (bias added),
             s [G,N] dtype, zp [G,N] int32 or None).
    """
    assert w.is_floating_point() and w.dim() == 2
    k, n = w.shape
    if group_size == -1:
        group_size = k
    assert k % group_size == 0
    wg = _group_view(w, group_size)                      # [G, g, N]
    hi = wg.max(dim=1, keepdim=True).values              # [G, 1, N]
    lo = wg.min(dim=1, keepdim=True).values
    qmax, qmin = wtype.max(), wtype.min()
    if zero_points:
        assert wtype.bias == 0 and not wtype.signed
        s = (hi - lo).clamp(min=1e-5) / qmax
        zp = torch.round(torch.abs(lo / s)).clamp(qmin, qmax).int()
        q = torch.round(wg / s).int() + zp
        q = torch.clamp(q, qmin, qmax)
        w_ref = (q - zp).to(w.dtype) * s
    else:
        zp = None
        a = torch.abs(hi / qmax) if qmax != 0 else torch.zeros_like(hi)
        b = torch.abs(lo / qmin) if qmin != 0 else torch.zeros_like(lo)
        s = torch.maximum(a, b)
        q = torch.clamp(torch.round(wg / s).int(), qmin, qmax)
        w_ref = q.to(w.dtype) * s
    q = q + wtype.bias
    g = k // group_size
    return (w_ref.reshape(k, n).contiguous(), q.reshape(k, n).contiguous().int(),
            s.reshape(g, n).contiguous(),
            None if zp is None else zp.reshape(g, n).contiguous())


def quantize_absmax7(w: torch.Tensor, group_size: int):
    """Symmetric uint4b8 RTN with s = absmax/7 per (group, column): the rule the
    benchmark configurations are stated with.  Returns (w_ref, q_stored, s)."""
    k, n = w.shape
    if group_size == -1:
        group_size = k
    wg = _group_view(w, group_size)
    s = (wg.abs().max(dim=1, keepdim=True).values / 7).clamp(min=1e-5)
    q = torch.clamp(torch.round(wg / s).int(), -8, 7)
    w_ref = q.to(w.dtype) * s
    return (w_ref.reshape(k, n).contiguous(), (q + 8).reshape(k, n).contiguous().int(),
            s.reshape(k // group_size, n).contiguous())


def quantize_minmax_zp(w: torch.Tensor, group_size: int):
    """Asymmetric uint4 RTN from per-group min/max (AWQ-style benchmark rule):
    s = (max-min)/15 clamped to >= 1e-5, z = clamp(round(-min/s), 0, 15),
    q = clamp(round(w/s) + z, 0, 15).  Returns (w_ref, q, s, zp)."""
    k, n = w.shape
    if group_size == -1:
        group_size = k
    wg = _group_view(w, group_size)
    hi = wg.max(dim=1, keepdim=True).values
    lo = wg.min(dim=1, keepdim=True).values
    s = ((hi - lo) / 15).clamp(min=1e-5)
    zp = torch.clamp(torch.round(-lo / s), 0, 15).int()
    q = torch.clamp(torch.round(wg / s).int() + zp, 0, 15)
    w_ref = (q - zp).to(w.dtype) * s
    g = k // group_size
    return (w_ref.reshape(k, n).contiguous(), q.reshape(k, n).contiguous().int(),
            s.reshape(g, n).contiguous(), zp.reshape(g, n).contiguous())


def permute_rows(q: torch.Tensor, w_ref: torch.Tensor, group_size: int, perm: torch.Tensor | None = None):
    """Act-order simulation (quant_utils.py:346-373): rows are shuffled by `perm`,
    g_idx[i] = perm[i] // group_size is the group of shuffled row i."""
    k = q.shape[0]
    if perm is None:
        perm = torch.randperm(k)
    perm = perm.long()
    g_idx = (perm // group_size).to(torch.int32)
    return w_ref[perm].contiguous(), q[perm].contiguous(), g_idx.contiguous(), perm


def gptq_quantize_weights(w, wtype: WType, group_size: int, act_order: bool, perm=None):
    """quant_utils.py:475-506.  Returns (w_ref, q, s, g_idx, rand_perm)."""
    k = w.shape[0]
    w_ref, q, s, _ = quantize_weights(w, wtype, group_size)
    g_idx = torch.empty(0, dtype=torch.int32)
    rand_perm = torch.empty(0, dtype=torch.int64)
    if act_order:
        assert group_size != -1 and group_size < k
        w_ref, q, g_idx, rand_perm = permute_rows(q, w_ref, group_size, perm)
    return w_ref, q, s, g_idx, rand_perm


def sort_weights(q: torch.Tensor, g_idx: torch.Tensor):
    """quant_utils.py:509-521: order rows by group id (stable)."""
    order = torch.argsort(g_idx.long(), stable=True).to(torch.int32)
    return q[order.long()].contiguous(), g_idx[order.long()].contiguous(), order


def _u32(t) -> np.ndarray:
    if isinstance(t, torch.Tensor):
        t = t.cpu().numpy()
    return np.ascontiguousarray(t).astype(np.int64).astype(np.uint32)


def _to_i32_tensor(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).astype(np.uint32).view(np.int32).copy())


def pack_rows(q, num_bits: int) -> torch.Tensor:
    """[K, N] -> int32 [K/pf, N]; field i of word (r, n) = q[pf*r + i, n]."""
    qa = _u32(q)
    pf = pack_factor(num_bits)
    k, n = qa.shape
    assert k % pf == 0
    fields = qa.reshape(k // pf, pf, n)
    out = np.zeros((k // pf, n), dtype=np.uint32)
    for i in range(pf):
        out |= (fields[:, i, :] & ((1 << num_bits) - 1)) << np.uint32(num_bits * i)
    return _to_i32_tensor(out)


def pack_cols(q, num_bits: int) -> torch.Tensor:
    """[K, N] -> int32 [K, N/pf]; field i of word (k, c) = q[k, pf*c + i]."""
    qa = _u32(q)
    pf = pack_factor(num_bits)
    k, n = qa.shape
    assert n % pf == 0
    fields = qa.reshape(k, n // pf, pf)
    out = np.zeros((k, n // pf), dtype=np.uint32)
    for i in range(pf):
        out |= (fields[:, :, i] & ((1 << num_bits) - 1)) << np.uint32(num_bits * i)
    return _to_i32_tensor(out)


def unpack_rows(packed, num_bits: int) -> torch.Tensor:
    pa = _u32(packed)
    pf = pack_factor(num_bits)
    r, n = pa.shape
    out = np.zeros((r, pf, n), dtype=np.uint32)
    for i in range(pf):
        out[:, i, :] = (pa >> np.uint32(num_bits * i)) & ((1 << num_bits) - 1)
    return torch.from_numpy(out.reshape(r * pf, n).astype(np.int32))


def unpack_cols(packed, num_bits: int) -> torch.Tensor:
    pa = _u32(packed)
    pf = pack_factor(num_bits)
    k, c = pa.shape
    out = np.zeros((k, c, pf), dtype=np.uint32)
    for i in range(pf):
        out[:, :, i] = (pa >> np.uint32(num_bits * i)) & ((1 << num_bits) - 1)
    return torch.from_numpy(out.reshape(k, c * pf).astype(np.int32))


def gptq_pack(q, num_bits: int = 4) -> torch.Tensor:
    return pack_rows(q, num_bits)


def _interleave(num_bits: int):
    return AWQ_NIBBLE_ORDER if num_bits == 4 else AWQ_BYTE_ORDER


def awq_pack(q, num_bits: int = 4) -> torch.Tensor:
    """[K, N] -> int32 [K, N/pf]; field t of word (k, c) = q[k, pf*c + order[t]]."""
    qa = _u32(q)
    order = np.array(_interleave(num_bits))
    k, n = qa.shape
    pf = pack_factor(num_bits)
    shuffled = qa.reshape(k, n // pf, pf)[:, :, order].reshape(k, n)
    return pack_cols(shuffled, num_bits)


def awq_unpack(packed, num_bits: int = 4) -> torch.Tensor:
    """Inverse of awq_pack: int32 [K, N/pf] -> [K, N] logical values."""
    raw = unpack_cols(packed, num_bits).numpy()
    order = np.array(_interleave(num_bits))
    pf = pack_factor(num_bits)
    k, n = raw.shape
    out = np.empty_like(raw).reshape(k, n // pf, pf)
    out[:, :, order] = raw.reshape(k, n // pf, pf)
    return torch.from_numpy(out.reshape(k, n))


def quantize_fp8(w: torch.Tensor, group_size: int):
    """Weight-only fp8 quantizer of the reference's test helper (marlin_utils_fp8.py:313-335), on w [K, N]:
    scale = absmax / 448 per (group, column) in the weight dtype, codes = (w / scale) cast to float8_e4m3fn
    (torch's round-to-nearest-even cast), w_ref = codes.to(dtype) * scale.
    Returns (w_ref [K, N], codes uint8 [K, N], scales [G, N])."""
    size_k, size_n = w.shape
    gs = size_k if group_size == -1 else group_size
    wg = w.t().contiguous().view(size_n, -1, gs)
    scales = wg.abs().amax(-1) / 448                       # [N, G]
    rep = scales.repeat_interleave(gs, 1)                  # [N, K]
    fp8 = (w.t() / rep).to(torch.float8_e4m3fn)
    w_ref = fp8.to(w.dtype) * rep
    return w_ref.t().contiguous(), fp8.view(torch.uint8).t().contiguous(), scales.t().contiguous()
