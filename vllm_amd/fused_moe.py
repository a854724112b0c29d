"""Expert routing for the fused MoE path; mirrors `fused_topk` of the reference
(vllm/model_executor/layers/fused_moe/fused_moe.py:1099-1128) on the gfx950 topk_softmax kernel."""
import torch

from . import _custom_ops as ops


def fused_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int, renormalize: bool,
               indices_type: torch.dtype | None = None) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns (topk_weights fp32 [M, topk], topk_ids [M, topk], token_expert_indices int32 [M, topk])."""
    assert hidden_states.size(0) == gating_output.size(0), "Number of tokens mismatch"
    m = hidden_states.size(0)
    topk_weights = torch.empty(m, topk, dtype=torch.float32, device=hidden_states.device)
    topk_ids = torch.empty(m, topk, dtype=torch.int32 if indices_type is None else indices_type,
                           device=hidden_states.device)
    token_expert_indices = torch.empty(m, topk, dtype=torch.int32, device=hidden_states.device)
    ops.topk_softmax(topk_weights, topk_ids, token_expert_indices, gating_output.contiguous(), renormalize)
    return topk_weights, topk_ids, token_expert_indices
