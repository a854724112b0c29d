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
