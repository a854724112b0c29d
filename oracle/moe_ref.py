"""MoE glue oracle (CPU, test infrastructure only).

Follows: torch_moe_align_block_size (reference tests/kernels/moe/test_moe_align_block_size.py:92-168),
the contract docstring of moe_align_block_size (vllm/model_executor/layers/fused_moe/
moe_align_block_size.py:11-85), torch_experts / torch_moe (tests/kernels/utils.py:900-1043) and the
choreography of fused_marlin_moe (fused_moe/fused_marlin_moe.py:47-340).

Pinned by (tests/test_oracle_moe.py): the docstring example (topk_ids
[[2,3,4],[1,2,4],[1,3,4],[1,2,3]], block 4 -> sorted ids
[3,6,9,12,0,4,10,12,1,7,11,12,2,5,8,12] once the unused expert 0 is skipped), the
invariants of test_moe_align_block_size.py:210-231, a brute-force per-token loop for the
experts computation, moe_gemm_ref == dense gemm_ref per expert on gathered rows, and for topk_softmax a
hand-computed three-expert case with a tie plus agreement with torch.topk on tie-free inputs.
"""
import torch


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int,
                         expert_map: torch.Tensor | None = None, pad_sorted_ids: bool = False):
    numel = topk_ids.numel()
    max_padded = numel + num_experts * (block_size - 1)
    if pad_sorted_ids:
        max_padded = -(-max_padded // block_size) * block_size
    flat = topk_ids.flatten().long()
    sorted_ids = torch.full((max_padded,), numel, dtype=torch.int32)
    n_blocks = -(-max_padded // block_size)
    expert_ids = torch.zeros(n_blocks, dtype=torch.int32)
    pos = 0
    blk = 0
    for e in range(num_experts):
        tok = torch.nonzero(flat == e).flatten().to(torch.int32)   # ascending = stable order
        cnt = tok.numel()
        if cnt == 0:
            continue
        nb = -(-cnt // block_size)
        sorted_ids[pos:pos + cnt] = tok
        expert_ids[blk:blk + nb] = e
        pos += nb * block_size
        blk += nb
    total = torch.tensor([pos], dtype=torch.int32)
    if expert_map is not None:
        expert_ids = expert_map[expert_ids.long()].to(torch.int32)
    return sorted_ids, expert_ids, total


def topk_softmax(gating_output: torch.Tensor, topk: int, renormalize: bool):
    """Routing as the reference's topk_softmax op (csrc/moe/topk_softmax_kernels.cu:127-211): fp32 softmax,
    k rounds of arg-max with ties going to the lowest expert index, optional renormalisation (zero sum -> divide
    by 1), token_expert_indices[t, k] = k * num_tokens + t.  Scalar loops: small cases only."""
    t, e = gating_output.shape
    p = torch.softmax(gating_output.float(), dim=-1)
    w = torch.zeros(t, topk, dtype=torch.float32)
    ids = torch.zeros(t, topk, dtype=torch.int32)
    src = torch.zeros(t, topk, dtype=torch.int32)
    for r in range(t):
        taken = set()
        for k in range(topk):
            best, be = -1.0, -1
            for x in range(e):
                if x not in taken and float(p[r, x]) > best:
                    best, be = float(p[r, x]), x
            taken.add(be)
            w[r, k], ids[r, k], src[r, k] = p[r, be], be, k * t + r
        if renormalize:
            d = w[r].sum()
            w[r] = w[r] / (d if d > 0 else 1.0)
    return w, ids, src


def batched_moe_align_block_size(max_tokens_per_batch: int, block_size: int, expert_num_tokens: torch.Tensor):
    """Alignment for per-expert batches, as the reference's test states it
    (tests/kernels/moe/test_moe_align_block_size.py:316-352) and its docstring example
    (moe_align_block_size.py:117-149): rows e*MAX + j for j < n_e, experts padded to block_size with the value
    E*MAX, empty experts skipped, expert_ids -1 past the end."""
    e = expert_num_tokens.numel()
    padded = -(-max_tokens_per_batch // block_size) * block_size * e
    sentinel = e * max_tokens_per_batch
    sorted_ids = torch.full((padded,), sentinel, dtype=torch.int32)
    expert_ids = torch.full((padded // block_size,), -1, dtype=torch.int32)
    i = 0
    for ex, nt in enumerate(expert_num_tokens.tolist()):
        first = i
        for j in range(nt):
            sorted_ids[i] = ex * max_tokens_per_batch + j
            i += 1
        i = -(-i // block_size) * block_size
        expert_ids[first // block_size:i // block_size] = ex
    return sorted_ids, expert_ids, torch.tensor([i], dtype=torch.int32)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    return torch.nn.functional.silu(x[..., :d]) * x[..., d:]


def torch_experts(a, w1, w2, topk_weight, topk_ids, expert_map=None):
    """a [M,K]; w1 [E, 2I, K]; w2 [E, K, I] dense (dequantised, transposed as nn.Linear
    weights); arithmetic in a's dtype like the reference; fp32 weighted sum over top-k."""
    m, k = a.shape
    topk = topk_ids.shape[1]
    rep = a.view(m, 1, k).repeat(1, topk, 1).reshape(-1, k)
    out = torch.zeros(m * topk, w2.shape[1], dtype=a.dtype)
    ids = topk_ids.reshape(-1).long()
    if expert_map is not None:
        ids = expert_map[ids].long()
    for e in range(w1.shape[0]):
        mask = ids == e
        if mask.any():
            h = rep[mask] @ w1[e].t()
            out[mask] = silu_and_mul(h) @ w2[e].t()
    return (out.view(m, topk, -1).float() * topk_weight.view(m, topk, 1).float()).sum(dim=1).to(a.dtype)


def torch_moe(a, w1, w2, score, topk, renormalize=False, expert_map=None):
    p = torch.softmax(score.float(), dim=-1)
    tw, ti = torch.topk(p, topk)
    if renormalize:
        tw = tw / tw.sum(dim=-1, keepdim=True)
    return torch_experts(a, w1, w2, tw, ti, expert_map)


def moe_gemm_ref(a, w_dense, sorted_ids, expert_ids, num_post_pad, topk_weights, block_size, top_k,
                 mul_topk_weights, size_m):
    """What one moe_wna16_marlin_gemm call computes, in fp32:
    for each valid sorted slot i with id = sorted_ids[i] < size_m*top_k:
      out[id] = a[id // top_k] @ w_dense[expert_ids[i // block]] (* topk_weights[id])."""
    n = w_dense.shape[2]
    out = torch.zeros(size_m * top_k, n, dtype=torch.float32)
    total = int(num_post_pad.item())
    for i in range(total):
        sid = int(sorted_ids[i])
        e = int(expert_ids[i // block_size])
        if sid >= size_m * top_k or e < 0:
            continue
        row = a[sid // top_k].float() @ w_dense[e].float()
        if mul_topk_weights:
            row = row * float(topk_weights.flatten()[sid])
        out[sid] = row
    return out
