"""Mixture-of-experts layer over Marlin-layout expert weights on the gfx950 MoE GEMM.

Public functions keep the reference's names and argument lists
(vllm/model_executor/layers/fused_moe/fused_marlin_moe.py: `fused_marlin_moe` :186-340,
`batched_fused_marlin_moe` :343-498), so a caller written against the reference works unchanged.
The launch sequence is this library's own.  Where the reference runs five launches

    align -> GEMM1 -> silu_and_mul -> GEMM2 (x routing weight) -> moe_sum,

the default path here runs three:

    align -> GEMM1 with SiLU-and-mul in its epilogue (and the final output cleared on the side)
          -> GEMM2 x routing weight, each token's top-k rows added into the output by the epilogue.

The [tokens * topk, 2 * inter] GEMM1 result and the [tokens, topk, hidden] GEMM2 result never reach memory.  Results
are those of the five-launch sequence (the epilogues round where the separate kernels would have).  The five-launch
sequence remains for what the fused epilogues do not cover: a caller-supplied activation or sum function, more than
two experts per token.
"""
from collections.abc import Callable
from dataclasses import dataclass

import torch

from . import _custom_ops as ops
from .marlin_utils import marlin_make_workspace_new, marlin_moe_intermediate_size
from .moe_align_block_size import batched_moe_align_block_size, moe_align_block_size
from .scalar_type import ScalarType, scalar_types

_MOE_WEIGHT_TYPES = (scalar_types.uint4, scalar_types.uint4b8, scalar_types.uint8b128, scalar_types.float8_e4m3fn,
                     scalar_types.float4_e2m1f)
_BLOCK_SIZES = (8, 16, 32, 48, 64)  # token slots per expert block the MoE GEMM accepts


def default_activation_func(activation: str, output: torch.Tensor, input: torch.Tensor) -> None:
    if activation != "silu":
        raise ValueError(f"Unsupported activation: {activation}. Only silu is implemented.")
    ops.silu_and_mul(output, input)


def pick_block_size(tokens: int, topk: int, num_experts: int, expert_bytes: int = 1 << 30) -> int:
    """Token slots per expert block, from the average expert's share of the slots (the quantity the reference's rule
    uses, fused_marlin_moe.py:279-282), fitted to the kernels behind each size on MI355X: blocks of 16 slots run on the
    weight-streaming kernel, whose cost is one pass over the expert's weights per block; blocks of 64 on the 64-row
    kernel, which costs about two such passes per block, so it wins once an expert fills more than one and a quarter
    blocks of 16 (sooner for experts of a few MB, where the per-block fixed costs count).  Blocks of 8 never beat 16,
    and 32 / 48 lost their niche (few, large experts) when the 64-row kernel began to split K for a thin last round."""
    per_expert = tokens * topk / num_experts
    return 16 if per_expert < (20 if expert_bytes >= (12 << 20) else 14) else 64


@dataclass
class _Experts:
    """The operands that stay the same across the two GEMMs of one layer call."""
    quant_type: ScalarType
    w: tuple            # (w1, w2)
    scale: tuple
    bias: tuple
    global_scale: tuple
    zeros: tuple
    g_idx: tuple
    sort_indices: tuple
    is_k_full: bool
    workspace: torch.Tensor

    def operands(self, i: int):
        return (self.w[i], self.bias[i], self.scale[i], self.global_scale[i], self.zeros[i], self.g_idx[i],
                self.sort_indices[i])


@dataclass
class _Routing:
    sorted_token_ids: torch.Tensor
    expert_ids: torch.Tensor
    num_tokens_post_padded: torch.Tensor
    topk_weights: torch.Tensor
    block_size: int
    topk: int
    expert_parallel: bool


def _gemm(ex: _Experts, which: int, rt: _Routing, a, c, size_m, size_n, size_k, top_k, mul_weights, **fused):
    w, bias, scale, gscale, zeros, g_idx, sort_idx = ex.operands(which)
    common = (a, c, w, bias, scale, gscale, zeros, g_idx, sort_idx, ex.workspace, rt.sorted_token_ids, rt.expert_ids,
              rt.num_tokens_post_padded, rt.topk_weights, rt.block_size, top_k, mul_weights)
    if fused:
        ops.moe_marlin_gemm_fused(*common, ex.quant_type, size_m, size_n, size_k, ex.is_k_full, **fused)
        return c
    return ops.moe_wna16_marlin_gemm(*common, rt.expert_parallel, ex.quant_type, size_m, size_n, size_k, ex.is_k_full,
                                     a.dtype == torch.half, True, False)


def _run_experts(x: torch.Tensor, ex: _Experts, rt: _Routing, weight_on_input: bool, activation: str,
                 activation_func: Callable, moe_sum: Callable | None, out: torch.Tensor | None, inter_buf, gemm_buf,
                 reduce_topk: bool) -> torch.Tensor:
    """x [M, K] -> [M, K] (reduce_topk) or [M * topk, K].  `out` receives the result when given."""
    m, k = x.shape
    n = marlin_moe_intermediate_size(*ex.w)
    slots = m * rt.topk
    dev, dt = x.device, x.dtype
    act = inter_buf.view(-1)[:slots * n].view(slots, n) if inter_buf is not None else torch.empty((slots, n), device=dev, dtype=dt)
    # what the GEMM launches can take over: SiLU-and-mul in GEMM1's epilogue whenever the default activation is asked
    # for; the top-k sum in GEMM2's epilogue for two terms (a sum of two does not depend on their order)
    # (the fused activation pairs gate and up n-tiles of 64 columns: the intermediate size must be a multiple of 64; the
    #  GEMM writes rows of a contiguous output: a strided `out` takes the separate-launch path and a final copy)
    act_fused = activation == "silu" and activation_func is default_activation_func and n % 64 == 0
    out_ok = out is None or out.is_contiguous()
    sum_fused = reduce_topk and moe_sum is None and rt.topk == 2 and out_ok
    direct = (not reduce_topk or (moe_sum is None and rt.topk == 1)) and out_ok   # GEMM2 writes the result rows themselves
    if (sum_fused or direct) and out is None:
        out = torch.empty((m if reduce_topk else slots, k), device=dev, dtype=dt)
    needs_zero = sum_fused or (direct and rt.expert_parallel)    # rows of experts on other ranks are never written
    big = max(0 if act_fused else 2 * n, 0 if (sum_fused or direct) else k)
    shared = None
    if big:
        shared = gemm_buf if gemm_buf is not None else torch.empty((slots * big,), device=dev, dtype=dt)
    # ---- GEMM1 (+ activation)
    cleared = False
    if act_fused:
        # the launch can clear GEMM2's output on the side, unless GEMM1 still reads it (inplace) or it is a strided view
        side_job = out if needs_zero and out is not x and out.is_contiguous() else None
        _gemm(ex, 0, rt, x, act, m, 2 * n, k, rt.topk, weight_on_input, silu_and_mul=True, sum_top_k=0, zero_fill=side_job)
        cleared = side_job is not None
    else:
        h = _gemm(ex, 0, rt, x, shared.view(-1)[:slots * 2 * n].view(slots, 2 * n), m, 2 * n, k, rt.topk, weight_on_input)
        activation_func(activation, act, h)
    # ---- GEMM2 (+ top-k sum)
    if sum_fused or direct:
        if needs_zero and not cleared:
            out.zero_()
        _gemm(ex, 1, rt, act, out, slots, k, n, 1, not weight_on_input, silu_and_mul=False,
              sum_top_k=2 if sum_fused else 0, zero_fill=None)
        return out
    y = shared.view(-1)[:slots * k].view(slots, k)
    if rt.expert_parallel:
        y.zero_()
    y = _gemm(ex, 1, rt, act, y, slots, k, n, 1, not weight_on_input)
    if out is None:
        out = torch.empty((m, k), device=dev, dtype=dt)
    if not reduce_topk:          # (a strided `out` for the unreduced rows)
        out.copy_(y)
        return out
    y3 = y.view(m, rt.topk, k)
    if moe_sum is None:
        if out.is_contiguous():
            ops.moe_sum(y3, out)
        else:
            dense = torch.empty((m, k), device=dev, dtype=dt)
            ops.moe_sum(y3, dense)
            out.copy_(dense)
        return out
    return moe_sum(y3, out)


def _check_layer(hidden_2d_k: int, w1, w2, quant_type: ScalarType, dtype) -> None:
    assert quant_type in _MOE_WEIGHT_TYPES, f"unsupported MoE weight type {quant_type}"
    assert w1.size(1) * 16 == hidden_2d_k, "Hidden size mismatch w1"
    assert w2.size(2) // (quant_type.size_bits // 2) == hidden_2d_k, "Hidden size mismatch w2"
    assert w1.is_contiguous(), "Expert weights1 must be contiguous"
    assert w2.is_contiguous(), "Expert weights2 must be contiguous"
    assert dtype in (torch.float16, torch.bfloat16)


def fused_marlin_moe(hidden_states, w1, w2, bias1, bias2, w1_scale, w2_scale, gating_output, topk_weights,
                     topk_ids, quant_type_id: int, apply_router_weight_on_input: bool = False,
                     global_num_experts: int = -1, activation: str = "silu",
                     activation_func: Callable = default_activation_func, moe_sum: Callable | None = None,
                     expert_map=None, global_scale1=None, global_scale2=None, g_idx1=None, g_idx2=None,
                     sort_indices1=None, sort_indices2=None, w1_zeros=None, w2_zeros=None, workspace=None,
                     intermediate_cache13=None, intermediate_cache2=None, is_k_full: bool = True, output=None,
                     inplace: bool = False) -> torch.Tensor:
    """hidden_states [M, K]; w1 [E, K/16, 2N * bits/2] (gate | up), w2 [E, N/16, K * bits/2] in Marlin layout;
    topk_weights fp32 [M, topk], topk_ids [M, topk]; returns [M, K]."""
    assert not (inplace and output is not None), "Conflicting request"
    assert hidden_states.ndim == 2 and hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert topk_weights.dtype == torch.float32
    m, k = hidden_states.shape
    assert gating_output is None or gating_output.size(0) == m, "Number of tokens mismatch"
    quant_type = ScalarType.from_id(quant_type_id)
    _check_layer(k, w1, w2, quant_type, hidden_states.dtype)
    num_local = w1.size(0)
    topk = topk_ids.size(1)
    bs = pick_block_size(m, topk, num_local, (w1[0].numel() + w2[0].numel()) * 4)
    sorted_ids, expert_ids, post_pad = moe_align_block_size(
        topk_ids, bs, num_local if global_num_experts == -1 else global_num_experts, expert_map)
    ex = _Experts(quant_type, (w1, w2), (w1_scale, w2_scale), (bias1, bias2), (global_scale1, global_scale2),
                  (w1_zeros, w2_zeros), (g_idx1, g_idx2), (sort_indices1, sort_indices2), is_k_full,
                  workspace if workspace is not None else marlin_make_workspace_new(hidden_states.device, 4))
    rt = _Routing(sorted_ids, expert_ids, post_pad, topk_weights, bs, topk, expert_map is not None)
    return _run_experts(hidden_states, ex, rt, apply_router_weight_on_input, activation, activation_func, moe_sum,
                        hidden_states if inplace else output, intermediate_cache2, intermediate_cache13, True)


def batched_fused_marlin_moe(hidden_states, expert_num_tokens, w1, w2, bias1, bias2, w1_scale, w2_scale, gating_output,
                             quant_type_id: int, apply_router_weight_on_input: bool = False,
                             global_num_experts: int = -1, activation: str | None = "silu", expert_map=None,
                             global_scale1=None, global_scale2=None, g_idx1=None, g_idx2=None, sort_indices1=None,
                             sort_indices2=None, w1_zeros=None, w2_zeros=None, workspace=None,
                             intermediate_cache13=None, intermediate_cache2=None, is_k_full: bool = True, output=None,
                             inplace: bool = False) -> torch.Tensor:
    """Activations already batched per expert: hidden_states [E, max_tokens, K] with expert_num_tokens[e] valid rows in
    batch e.  The batch is the flat [E * max_tokens, K] problem with one expert per token and unit routing weights;
    the alignment comes from the row counts.  Returns [E, max_tokens, K]; rows past expert_num_tokens[e] are not written."""
    assert hidden_states.ndim == 3, f"hidden states must be batched. e.g. [B, MAX_TOKENS, K]. But got {hidden_states.size()}"
    assert not (inplace and output is not None), "Conflicting request."
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert activation is not None
    batches, max_tokens, k = hidden_states.shape
    quant_type = ScalarType.from_id(quant_type_id)
    _check_layer(k, w1, w2, quant_type, hidden_states.dtype)
    assert expert_num_tokens.size(0) == w1.size(0) == batches, \
        "Batch must be as big as number of experts as the tokens are sorted into the batch/expert they belong to"
    bs = _BLOCK_SIZES[-1]
    sorted_ids, expert_ids, post_pad = batched_moe_align_block_size(max_tokens, bs, expert_num_tokens)
    flat = hidden_states.view(-1, k)
    ones = torch.ones((flat.size(0), 1), device=flat.device, dtype=torch.float32)
    ex = _Experts(quant_type, (w1, w2), (w1_scale, w2_scale), (bias1, bias2), (global_scale1, global_scale2),
                  (w1_zeros, w2_zeros), (g_idx1, g_idx2), (sort_indices1, sort_indices2), is_k_full,
                  workspace if workspace is not None else marlin_make_workspace_new(flat.device, 4))
    rt = _Routing(sorted_ids, expert_ids, post_pad, ones, bs, 1, expert_map is not None)
    dest = flat if inplace else (output.view(-1, k) if output is not None else None)
    y = _run_experts(flat, ex, rt, apply_router_weight_on_input, activation, default_activation_func, None, dest,
                     intermediate_cache2, intermediate_cache13, False)
    return y.view(batches, max_tokens, k)
