"""Token -> expert block alignment; host wrapper with the reference's signature and result contract
(vllm/model_executor/layers/fused_moe/moe_align_block_size.py:11-85)."""
import torch

from . import _custom_ops as ops


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int,
                         expert_map: torch.Tensor | None = None,
                         pad_sorted_ids: bool = False) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns (sorted_token_ids, expert_ids, num_tokens_post_padded).

    sorted_token_ids: flat (token, slot) indices grouped by expert, each expert's run padded to a
    multiple of block_size with the value topk_ids.numel(); expert_ids: expert of every block (-1 after
    `expert_map` for experts not on this rank); num_tokens_post_padded: padded total, int32 [1].
    """
    max_num_tokens_padded = topk_ids.numel() + num_experts * (block_size - 1)
    if pad_sorted_ids:
        max_num_tokens_padded = -(-max_num_tokens_padded // block_size) * block_size
    sorted_ids = torch.empty((max_num_tokens_padded,), dtype=torch.int32, device=topk_ids.device)
    max_num_m_blocks = -(-max_num_tokens_padded // block_size)
    expert_ids = torch.empty((max_num_m_blocks,), dtype=torch.int32, device=topk_ids.device)
    num_tokens_post_pad = torch.empty((1,), dtype=torch.int32, device=topk_ids.device)
    ops.moe_align_block_size(topk_ids, num_experts, block_size, sorted_ids, expert_ids, num_tokens_post_pad)
    if expert_map is not None:
        expert_ids = expert_map[expert_ids.long()].to(torch.int32)
    return sorted_ids, expert_ids, num_tokens_post_pad


def batched_moe_align_block_size(max_tokens_per_batch: int, block_size: int,
                                 expert_num_tokens: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Alignment for activations that are already batched per expert, [E, max_tokens_per_batch, K] with
    expert_num_tokens[e] valid rows in batch e; same result contract as the reference's function of this name
    (vllm/model_executor/layers/fused_moe/moe_align_block_size.py:88-172): row index e * max_tokens_per_batch + j
    for the valid rows of expert e, each expert padded to a multiple of block_size with the value
    E * max_tokens_per_batch, experts with no tokens skipped, expert_ids = -1 past the last block."""
    e = expert_num_tokens.size(0)
    dev = expert_num_tokens.device
    padded = e * (-(-max_tokens_per_batch // block_size) * block_size)
    sorted_ids = torch.empty((padded,), dtype=torch.int32, device=dev)
    expert_ids = torch.empty((padded // block_size,), dtype=torch.int32, device=dev)
    num_tokens_post_pad = torch.empty((1,), dtype=torch.int32, device=dev)
    ops.batched_moe_align_block_size(max_tokens_per_batch, block_size, expert_num_tokens, sorted_ids, expert_ids,
                                     num_tokens_post_pad)
    return sorted_ids, expert_ids, num_tokens_post_pad
