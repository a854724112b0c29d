"""Column pack / unpack of sub-byte integers on whatever device the tensor lives on.

Same results as the reference's numpy helpers `pack_cols` / `unpack_cols`
(vllm/model_executor/layers/quantization/utils/quant_utils.py:548-602), but computed with torch
integer ops so load-time zero-point conversion stays on the GPU instead of a host round trip.
"""
import torch


def get_pack_factor(num_bits: int) -> int:
    assert 32 % num_bits == 0, f"Unsupported num_bits = {num_bits}"
    return 32 // num_bits


def pack_cols(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    assert q_w.shape == (size_k, size_n)
    pf = get_pack_factor(num_bits)
    assert size_n % pf == 0
    fields = q_w.to(torch.int64).reshape(size_k, size_n // pf, pf) & ((1 << num_bits) - 1)
    shifts = torch.arange(pf, device=q_w.device, dtype=torch.int64) * num_bits
    word = (fields << shifts).sum(dim=-1)                       # disjoint bit fields: sum == or
    word = torch.where(word >= 2**31, word - 2**32, word)       # to two's-complement int32 range
    return word.to(torch.int32).contiguous()


def unpack_cols(packed_q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    pf = get_pack_factor(num_bits)
    assert size_n % pf == 0
    assert packed_q_w.shape == (size_k, size_n // pf), (
        f"packed_q_w.shape = {tuple(packed_q_w.shape)} size_k = {size_k}, size_n = {size_n} pack_factor = {pf}")
    shifts = torch.arange(pf, device=packed_q_w.device, dtype=torch.int64) * num_bits
    wide = packed_q_w.to(torch.int64) & 0xFFFFFFFF
    vals = (wide.unsqueeze(-1) >> shifts) & ((1 << num_bits) - 1)
    return vals.reshape(size_k, size_n).to(torch.int32).contiguous()


def pack_rows(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    """[size_k, size_n] -> int32 [size_k / pack_factor, size_n]; field i of word (r, n) = q_w[pack_factor * r + i, n]
    (the GPTQ checkpoint packing; reference quant_utils.py:524-545)."""
    assert q_w.shape == (size_k, size_n)
    pf = get_pack_factor(num_bits)
    assert size_k % pf == 0
    word = torch.zeros((size_k // pf, size_n), dtype=torch.int64, device=q_w.device)
    fields = q_w.reshape(size_k // pf, pf, size_n)
    for i in range(pf):                                          # one field at a time: no [K, N] int64 temporary
        word |= (fields[:, i, :].to(torch.int64) & ((1 << num_bits) - 1)) << (num_bits * i)
    word = torch.where(word >= 2**31, word - 2**32, word)
    return word.to(torch.int32).contiguous()


def unpack_rows(packed_q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    pf = get_pack_factor(num_bits)
    assert packed_q_w.shape == (size_k // pf, size_n)
    shifts = (torch.arange(pf, device=packed_q_w.device, dtype=torch.int64) * num_bits).view(1, pf, 1)
    wide = (packed_q_w.to(torch.int64) & 0xFFFFFFFF).unsqueeze(1)
    return ((wide >> shifts) & ((1 << num_bits) - 1)).reshape(size_k, size_n).to(torch.int32).contiguous()


def gptq_pack(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    """Reference quant_utils.py:605-611."""
    return pack_rows(q_w, num_bits, size_k, size_n)


def awq_pack(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    """AWQ checkpoint packing (reference quant_utils.py:614-633): inside every run of pack_factor columns the fields
    are stored in the order (0, 2, 4, 6, 1, 3, 5, 7) [4-bit] or (0, 2, 1, 3) [8-bit], then packed along columns."""
    assert q_w.shape == (size_k, size_n)
    order = (0, 2, 4, 6, 1, 3, 5, 7) if num_bits == 4 else (0, 2, 1, 3)
    pf = get_pack_factor(num_bits)
    idx = torch.tensor(order, device=q_w.device)
    shuffled = q_w.reshape(size_k, size_n // pf, pf)[:, :, idx].reshape(size_k, size_n)
    return pack_cols(shuffled, num_bits, size_k, size_n)
