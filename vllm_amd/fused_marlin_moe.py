"""Fused MoE on the Marlin-layout W4A16 kernels; host choreography with the reference's signature
(vllm/model_executor/layers/fused_moe/fused_marlin_moe.py:47-340): block-size pick, token alignment,
GEMM1 (gate|up) -> SiLU-and-mul -> GEMM2 (down, scaled by routing weights) -> sum over top-k."""
from collections.abc import Callable

import torch

from . import _custom_ops as ops
from .marlin_utils import marlin_make_workspace_new, marlin_moe_intermediate_size
from .moe_align_block_size import batched_moe_align_block_size, moe_align_block_size
from .scalar_type import ScalarType, scalar_types


def default_activation_func(activation: str, output: torch.Tensor, input: torch.Tensor) -> None:
    if activation == "silu":
        ops.silu_and_mul(output, input)
    else:
        raise ValueError(f"Unsupported activation: {activation}. Only silu is implemented.")


def _fused_marlin_moe(hidden_states, w1, w2, bias1, bias2, w1_scale, w2_scale, topk_weights, num_topk: int,
                      quant_type: ScalarType, apply_router_weight_on_input: bool, expert_map, block_size_m: int,
                      sorted_token_ids, expert_ids, num_tokens_post_padded, activation: str = "silu",
                      activation_func: Callable = default_activation_func, global_scale1=None, global_scale2=None,
                      g_idx1=None, g_idx2=None, sort_indices1=None, sort_indices2=None, w1_zeros=None, w2_zeros=None,
                      workspace=None, intermediate_cache13=None, intermediate_cache2=None, output=None,
                      is_k_full: bool = True) -> torch.Tensor:
    assert hidden_states.ndim == 2
    M, K = hidden_states.size()
    N = marlin_moe_intermediate_size(w1, w2)
    if workspace is None:
        workspace = marlin_make_workspace_new(hidden_states.device, 4)
    if intermediate_cache13 is None:
        intermediate_cache13 = torch.empty((M * num_topk * max(2 * N, K),), device=hidden_states.device,
                                           dtype=hidden_states.dtype)
    if intermediate_cache2 is None:
        intermediate_cache2 = torch.empty((M * num_topk, N), device=hidden_states.device, dtype=hidden_states.dtype)
    cache1 = intermediate_cache13[:M * num_topk * 2 * N].view(M * num_topk, 2 * N)
    cache3 = intermediate_cache13[:M * num_topk * K].view(M * num_topk, K)
    cache2 = intermediate_cache2.view(-1)[:M * num_topk * N].view(M * num_topk, N)
    use_atomic_add = hidden_states.dtype == torch.half

    cache1 = ops.moe_wna16_marlin_gemm(
        hidden_states, cache1, w1, bias1, w1_scale, global_scale1, w1_zeros, g_idx1, sort_indices1, workspace,
        sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, moe_block_size=block_size_m,
        top_k=num_topk, mul_topk_weights=apply_router_weight_on_input, is_ep=expert_map is not None,
        b_q_type=quant_type, size_m=M, size_n=2 * N, size_k=K, is_k_full=is_k_full,
        use_atomic_add=use_atomic_add, use_fp32_reduce=True, is_zp_float=False)

    activation_func(activation, cache2, cache1.view(-1, 2 * N))

    if output is None:
        output = cache3
    if expert_map is not None:
        output.zero_()

    output = ops.moe_wna16_marlin_gemm(
        cache2, output, w2, bias2, w2_scale, global_scale2, w2_zeros, g_idx2, sort_indices2, workspace,
        sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, moe_block_size=block_size_m,
        top_k=1, mul_topk_weights=not apply_router_weight_on_input, is_ep=expert_map is not None,
        b_q_type=quant_type, size_m=M * num_topk, size_n=K, size_k=N, is_k_full=is_k_full,
        use_atomic_add=use_atomic_add, use_fp32_reduce=True, is_zp_float=False)
    return output


def fused_marlin_moe(hidden_states, w1, w2, bias1, bias2, w1_scale, w2_scale, gating_output, topk_weights,
                     topk_ids, quant_type_id: int, apply_router_weight_on_input: bool = False,
                     global_num_experts: int = -1, activation: str = "silu",
                     activation_func: Callable = default_activation_func, moe_sum: Callable | None = None,
                     expert_map=None, global_scale1=None, global_scale2=None, g_idx1=None, g_idx2=None,
                     sort_indices1=None, sort_indices2=None, w1_zeros=None, w2_zeros=None, workspace=None,
                     intermediate_cache13=None, intermediate_cache2=None, is_k_full: bool = True, output=None,
                     inplace: bool = False) -> torch.Tensor:
    """Mixture-of-experts layer over Marlin-layout 4-bit expert weights w1 [E, K/16, 2*(2N)] and
    w2 [E, N/16, 2*K]; returns [M, K]."""
    if inplace:
        assert output is None, "Conflicting request"
    quant_type = ScalarType.from_id(quant_type_id)
    assert quant_type in (scalar_types.uint4, scalar_types.uint4b8, scalar_types.uint8b128,
                          scalar_types.float8_e4m3fn, scalar_types.float4_e2m1f), \
        f"unsupported MoE weight type {quant_type}"
    num_bits = quant_type.size_bits
    M, K = hidden_states.size()
    E = w1.size(0)
    topk = topk_ids.size(1)
    if gating_output is not None:
        assert gating_output.size(0) == M, "Number of tokens mismatch"
    assert w1.size(1) * 16 == K, "Hidden size mismatch w1"
    assert w2.size(2) // (num_bits // 2) == K, "Hidden size mismatch w2"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.is_contiguous(), "Expert weights1 must be contiguous"
    assert w2.is_contiguous(), "Expert weights2 must be contiguous"
    assert hidden_states.dtype in (torch.float16, torch.bfloat16)
    assert topk_weights.dtype == torch.float32

    for block_size_m in (8, 16, 32, 48, 64):
        if M * topk / E / block_size_m < 0.9:
            break
    if global_num_experts == -1:
        global_num_experts = E
    sorted_token_ids, expert_ids, num_tokens_post_padded = moe_align_block_size(
        topk_ids, block_size_m, global_num_experts, expert_map)

    moe_output = _fused_marlin_moe(
        hidden_states=hidden_states, w1=w1, w2=w2, bias1=bias1, bias2=bias2, w1_scale=w1_scale, w2_scale=w2_scale,
        topk_weights=topk_weights, num_topk=topk, quant_type=quant_type,
        apply_router_weight_on_input=apply_router_weight_on_input, expert_map=expert_map,
        block_size_m=block_size_m, sorted_token_ids=sorted_token_ids, expert_ids=expert_ids,
        num_tokens_post_padded=num_tokens_post_padded, activation=activation, activation_func=activation_func,
        global_scale1=global_scale1, global_scale2=global_scale2, g_idx1=g_idx1, g_idx2=g_idx2,
        sort_indices1=sort_indices1, sort_indices2=sort_indices2, w1_zeros=w1_zeros, w2_zeros=w2_zeros,
        workspace=workspace, intermediate_cache13=intermediate_cache13, intermediate_cache2=intermediate_cache2,
        output=None, is_k_full=is_k_full).view(-1, topk, K)

    if output is None:
        output = hidden_states if inplace else torch.empty_like(hidden_states)
    if moe_sum is None:
        ops.moe_sum(moe_output.contiguous(), output)
        return output
    return moe_sum(moe_output, output)


def batched_fused_marlin_moe(hidden_states, expert_num_tokens, w1, w2, bias1, bias2, w1_scale, w2_scale, gating_output,
                             quant_type_id: int, apply_router_weight_on_input: bool = False,
                             global_num_experts: int = -1, activation: str | None = "silu", expert_map=None,
                             global_scale1=None, global_scale2=None, g_idx1=None, g_idx2=None, sort_indices1=None,
                             sort_indices2=None, w1_zeros=None, w2_zeros=None, workspace=None,
                             intermediate_cache13=None, intermediate_cache2=None, is_k_full: bool = True, output=None,
                             inplace: bool = False) -> torch.Tensor:
    """MoE over activations already batched per expert, hidden_states [E, max_tokens, K] with expert_num_tokens[e]
    valid rows in batch e (reference fused_marlin_moe.py:343-498): the batch is viewed as [E * max_tokens, K] with
    top_k = 1 and unit routing weights, and the alignment comes from the row counts.  Returns [E, max_tokens, K];
    rows past expert_num_tokens[e] are not written."""
    assert hidden_states.ndim == 3, f"hidden states must be batched. e.g. [B, MAX_TOKENS, K]. But got {hidden_states.size()}"
    if inplace:
        assert output is None, "Conflicting request."
    quant_type = ScalarType.from_id(quant_type_id)
    assert quant_type in (scalar_types.uint4, scalar_types.uint4b8, scalar_types.uint8b128,
                          scalar_types.float8_e4m3fn, scalar_types.float4_e2m1f), \
        f"unsupported MoE weight type {quant_type}"
    num_bits = quant_type.size_bits
    B, batch_tokens_max, K = hidden_states.size()
    M = B * batch_tokens_max
    E = w1.size(0)
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert hidden_states.dtype in (torch.float16, torch.bfloat16)
    assert expert_num_tokens.size(0) == E
    assert B == E, "Batch must be as big as number of experts as the tokens are sorted into the batch/expert they belong to"
    assert w1.size(1) * 16 == K, "Hidden size mismatch w1"
    assert w2.size(2) // (num_bits // 2) == K, "Hidden size mismatch w2"
    assert w1.is_contiguous(), "Expert weights1 must be contiguous"
    assert w2.is_contiguous(), "Expert weights2 must be contiguous"
    assert activation is not None
    topk = 1
    block_size_m = 64
    sorted_token_ids, expert_ids, num_tokens_post_padded = batched_moe_align_block_size(
        max_tokens_per_batch=batch_tokens_max, block_size=block_size_m, expert_num_tokens=expert_num_tokens)
    if output is None and inplace:
        output = hidden_states
    topk_weights = torch.ones((M, topk), device=hidden_states.device, dtype=torch.float32)
    output = _fused_marlin_moe(
        hidden_states=hidden_states.view(-1, K), w1=w1, w2=w2, bias1=bias1, bias2=bias2, w1_scale=w1_scale,
        w2_scale=w2_scale, topk_weights=topk_weights, num_topk=topk, quant_type=quant_type,
        apply_router_weight_on_input=apply_router_weight_on_input, activation=activation, expert_map=expert_map,
        block_size_m=block_size_m, sorted_token_ids=sorted_token_ids, expert_ids=expert_ids,
        num_tokens_post_padded=num_tokens_post_padded, global_scale1=global_scale1, global_scale2=global_scale2,
        g_idx1=g_idx1, g_idx2=g_idx2, sort_indices1=sort_indices1, sort_indices2=sort_indices2, w1_zeros=w1_zeros,
        w2_zeros=w2_zeros, workspace=workspace, intermediate_cache13=intermediate_cache13,
        intermediate_cache2=intermediate_cache2, output=output.view(-1, K) if output is not None else output,
        is_k_full=is_k_full)
    return output.view(B, batch_tokens_max, K)
