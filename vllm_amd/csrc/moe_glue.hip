// MoE glue kernels for gfx950: token->expert block alignment, top-k sum, SiLU-and-mul.
//
// moe_align_block_size follows the contract of the reference op
// (vllm/model_executor/layers/fused_moe/moe_align_block_size.py:11-85, kernels
// csrc/moe/moe_align_sum_kernels.cu:83-268): sort the flattened (token, slot) indices by expert,
// pad every expert's run to a multiple of block_size with the value `numel`, emit one expert id
// per block (tail zero-filled) and the padded total.  Unlike the reference (atomic ranks, order
// inside an expert unspecified) the order here is stable — ascending flat index inside each
// expert — so the result is deterministic and equals the reference's torch golden
// (tests/kernels/moe/test_moe_align_block_size.py:92-168) element for element.
#include "gemm_common.h"

namespace w4a16 {

constexpr int ALIGN_THREADS = 1024;
constexpr int ALIGN_WAVES = ALIGN_THREADS / 64;
constexpr int ALIGN_MAX_EXPERTS = 1024;

// Every workgroup recomputes the histogram and the scan (numel and E are small), then its 16
// wavefronts each place the tokens of experts wg*16 + wave, +gridDim*16, ... by ballot ranking.
__global__ __launch_bounds__(ALIGN_THREADS) void moe_align_kernel(
    const int32_t* __restrict__ topk_ids, int numel, int num_experts, int block_size,
    int32_t* __restrict__ sorted_ids, int sorted_len, int32_t* __restrict__ expert_ids, int expert_ids_len,
    int32_t* __restrict__ num_post_pad) {
  __shared__ int cnt[ALIGN_MAX_EXPERTS];
  __shared__ int off[ALIGN_MAX_EXPERTS + 1];
  const int t = threadIdx.x;
  for (int e = t; e < num_experts; e += ALIGN_THREADS) cnt[e] = 0;
  __syncthreads();
  for (int i = t; i < numel; i += ALIGN_THREADS) {
    const int e = topk_ids[i];
    if (e >= 0 && e < num_experts) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (t < 64) {  // wave 0: exclusive scan of padded counts, 64 experts per round
    int run = 0;
    for (int base = 0; base < num_experts; base += 64) {
      const int e = base + t;
      const int padded = e < num_experts ? (cnt[e] + block_size - 1) / block_size * block_size : 0;
      int incl = padded;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int v = __shfl_up(incl, d, 64);
        if (t >= d) incl += v;
      }
      if (e < num_experts) off[e] = run + incl - padded;
      run += __shfl(incl, 63, 64);
    }
    if (t == 0) off[num_experts] = run;
  }
  __syncthreads();
  const int total = off[num_experts];

  if (blockIdx.x == 0) {
    if (t == 0) *num_post_pad = total;
    // expert id of every block; blocks past the padded total are zero-filled
    for (int e = t; e < num_experts; e += ALIGN_THREADS) {
      const int b0 = off[e] / block_size, b1 = off[e + 1] / block_size;
      for (int b = b0; b < b1 && b < expert_ids_len; ++b) expert_ids[b] = e;
    }
    for (int b = total / block_size + t; b < expert_ids_len; b += ALIGN_THREADS) expert_ids[b] = 0;
    for (int i = total + t; i < sorted_len; i += ALIGN_THREADS) sorted_ids[i] = numel;
  }

  const int lane = t & 63, wv = t >> 6;
  for (int e = blockIdx.x * ALIGN_WAVES + wv; e < num_experts; e += gridDim.x * ALIGN_WAVES) {
    int pos = off[e];
    const int end = off[e + 1];
    if (pos == end) continue;
    // four independent loads per round trip (the loop is latency-bound: 64 ids per wavefront and load otherwise)
    for (int base = 0; base < numel; base += 256) {
      int id[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + 64 * u + lane;
        id[u] = i < numel ? topk_ids[i] : -1;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + 64 * u + lane;
        const bool hit = id[u] == e;  // (e >= 0: padding ids never match)
        const unsigned long long m = __ballot(hit);
        if (hit) {
          const int rank = __popcll(m & ((1ull << lane) - 1ull));
          if (pos + rank < sorted_len) sorted_ids[pos + rank] = i;
        }
        pos += __popcll(m);
      }
    }
    for (int i = pos + lane; i < end && i < sorted_len; i += 64) sorted_ids[i] = numel;
  }
}

// The same contract for long id lists (prefill): the kernel above walks all ids once per expert with one wavefront, four
// dependent 4-byte loads per round trip, and re-reads them with as many round trips for the histogram; here
//   * every thread fetches its ids with 16-byte loads, several in flight, for the histogram (LDS atomics: per-expert
//     ballot counts for the few-expert case, where lanes queue on a few addresses, measured slower);
//   * the ids of an expert are placed by `spe` wavefronts of a workgroup, each on a contiguous slice of the ids:
//     count the matches of the slice, exchange the counts through LDS, place from the slice's start position.  A lane
//     holds four consecutive ids; a match's rank is the matches of the lanes in front plus its own earlier components,
//     so the order inside an expert stays the order of the ids (stable, deterministic).
using i32x4 = int32_t __attribute__((ext_vector_type(4)));
constexpr int ALIGN_ROUND = 8;  // 16-byte loads in flight per lane in the placement passes (2048 ids per wavefront round)
__global__ __launch_bounds__(ALIGN_THREADS) void moe_align_sliced_kernel(
    const int32_t* __restrict__ topk_ids, int numel, int num_experts, int block_size, int spe,
    int32_t* __restrict__ sorted_ids, int sorted_len, int32_t* __restrict__ expert_ids, int expert_ids_len,
    int32_t* __restrict__ num_post_pad) {
  __shared__ int cnt[ALIGN_MAX_EXPERTS];
  __shared__ int off[ALIGN_MAX_EXPERTS + 1];
  __shared__ int slice_cnt[ALIGN_WAVES];
  const int t = threadIdx.x, lane = t & 63, wv = t >> 6;
  const unsigned long long lt = (1ull << lane) - 1ull;
  for (int e = t; e < num_experts; e += ALIGN_THREADS) cnt[e] = 0;
  __syncthreads();
  const int nvec = numel >> 2;  // whole 16-byte groups; the last numel & 3 ids are handled one by one
  const i32x4* vids = (const i32x4*)topk_ids;

  // ---- histogram
  for (int v0 = 0; v0 < nvec; v0 += 4 * ALIGN_THREADS) {
    i32x4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int vi = v0 + j * ALIGN_THREADS + t;
      v[j] = vi < nvec ? vids[vi] : i32x4{-1, -1, -1, -1};
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int e = v[j][q];
        if (e >= 0 && e < num_experts) atomicAdd(&cnt[e], 1);
      }
    }
  }
  if (t < (numel & 3)) {
    const int e = topk_ids[4 * nvec + t];
    if (e >= 0 && e < num_experts) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (t < 64) {  // wave 0: exclusive scan of padded counts, 64 experts per round
    int acc = 0;
    for (int base = 0; base < num_experts; base += 64) {
      const int e = base + t;
      const int padded = e < num_experts ? (cnt[e] + block_size - 1) / block_size * block_size : 0;
      int incl = padded;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int v = __shfl_up(incl, d, 64);
        if (t >= d) incl += v;
      }
      if (e < num_experts) off[e] = acc + incl - padded;
      acc += __shfl(incl, 63, 64);
    }
    if (t == 0) off[num_experts] = acc;
  }
  __syncthreads();
  const int total = off[num_experts];
  if (blockIdx.x == 0) {
    if (t == 0) *num_post_pad = total;
    // expert id of every block; blocks past the padded total are zero-filled; slots past the total hold numel
    for (int e = t; e < num_experts; e += ALIGN_THREADS) {
      const int b0 = off[e] / block_size, b1 = off[e + 1] / block_size;
      for (int b = b0; b < b1 && b < expert_ids_len; ++b) expert_ids[b] = e;
    }
    for (int b = total / block_size + t; b < expert_ids_len; b += ALIGN_THREADS) expert_ids[b] = 0;
    for (int i = total + t; i < sorted_len; i += ALIGN_THREADS) sorted_ids[i] = numel;
  }

  // ---- placement: workgroup turn `eg` handles experts eg * epw .. + epw - 1, `spe` wavefronts each
  const int epw = ALIGN_WAVES / spe;
  const int j = wv / spe, sl = wv % spe;
  // slice of the 16-byte groups: whole wavefront loads (64 groups)
  const int per = ((nvec + spe - 1) / spe + 63) / 64 * 64;
  const int vb = min(sl * per, nvec), ve = min(vb + per, nvec);
  for (int eg = blockIdx.x; eg * epw < num_experts; eg += gridDim.x) {
    const int e = eg * epw + j;
    const bool live = e < num_experts && cnt[e] > 0;
    // matches of expert e in groups [vb, ve): pass 0 counts, pass 1 places from `pos`
    int pos = 0;
    for (int pass = 0; pass < 2; ++pass) {
      int seen = 0;
      if (live) {
        for (int v0 = vb; v0 < ve; v0 += 64 * ALIGN_ROUND) {
          i32x4 v[ALIGN_ROUND];
#pragma unroll
          for (int r = 0; r < ALIGN_ROUND; ++r) {
            const int vi = v0 + 64 * r + lane;
            v[r] = vi < ve ? vids[vi] : i32x4{-1, -1, -1, -1};
          }
#pragma unroll
          for (int r = 0; r < ALIGN_ROUND; ++r) {
            unsigned long long m[4];
            int before = 0, all = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              m[q] = __ballot(v[r][q] == e);
              before += __popcll(m[q] & lt);
              all += __popcll(m[q]);
            }
            if (pass == 1 && all) {
              int p = pos + seen + before;
              const int idx = 4 * (v0 + 64 * r + lane);
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                if (v[r][q] == e) {
                  if (p < sorted_len) sorted_ids[p] = idx + q;
                  ++p;
                }
              }
            }
            seen += all;
          }
        }
        // the last slice also owns the numel & 3 ids past the 16-byte groups
        if (sl == spe - 1) {
          const int i = 4 * nvec + lane;
          const bool hit = lane < (numel & 3) && topk_ids[i] == e;
          const unsigned long long m = __ballot(hit);
          if (pass == 1 && hit) {
            const int p = pos + seen + __popcll(m & lt);
            if (p < sorted_len) sorted_ids[p] = i;
          }
          seen += __popcll(m);
        }
      }
      if (pass == 0) {
        if (lane == 0) slice_cnt[wv] = seen;
        __syncthreads();
        if (live) {
          pos = off[e];
          for (int s2 = 0; s2 < sl; ++s2) pos += slice_cnt[j * spe + s2];
        }
        __syncthreads();  // slice_cnt is rewritten in the next turn
      }
    }
    // padding slots of the expert: by its first slice's wavefront
    if (e < num_experts && sl == 0) {
      const int padded = (cnt[e] + block_size - 1) / block_size * block_size;
      for (int i = off[e] + cnt[e] + lane; i < off[e] + padded && i < sorted_len; i += 64) sorted_ids[i] = numel;
    }
  }
}

// B terms' loads in flight together (a few tokens give too few wavefronts to hide one round trip per term); added in
// term order
template <int DT, int B>
__device__ __forceinline__ void moe_sum_terms(const uint16_t* __restrict__ in, int64_t tok, int top_k, int64_t hidden8,
                                              int64_t col, float* acc) {
  for (int k0 = 0; k0 < top_k; k0 += B) {
    u32x4 v[B];
#pragma unroll
    for (int i = 0; i < B; ++i)
      v[i] = *(const u32x4*)(in + ((tok * top_k + min(k0 + i, top_k - 1)) * hidden8 + col) * 8);
#pragma unroll
    for (int i = 0; i < B; ++i) {
      if (k0 + i < top_k) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[2 * j] += DT == DT_F16 ? f16_lo_f32(v[i][j]) : bf16_lo_f32(v[i][j]);
          acc[2 * j + 1] += DT == DT_F16 ? f16_hi_f32(v[i][j]) : bf16_hi_f32(v[i][j]);
        }
      }
    }
  }
}

template <int DT>
__global__ __launch_bounds__(256) void moe_sum_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                      int64_t total8, int top_k, int64_t hidden8) {
  // one thread per 8 consecutive output elements
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total8; idx += (int64_t)gridDim.x * 256) {
    const int64_t tok = idx / hidden8, col = idx % hidden8;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (top_k <= 2)
      moe_sum_terms<DT, 2>(in, tok, top_k, hidden8, col, acc);
    else if (top_k <= 4)
      moe_sum_terms<DT, 4>(in, tok, top_k, hidden8, col, acc);
    else
      moe_sum_terms<DT, 8>(in, tok, top_k, hidden8, col, acc);
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      o[j] = DT == DT_F16 ? pack_f16(acc[2 * j], acc[2 * j + 1]) : pack_bf16(acc[2 * j], acc[2 * j + 1]);
    *(u32x4*)(out + idx * 8) = o;
  }
}

// out = T(silu_f32(x)) * y evaluated like the reference's act_and_mul_kernel<silu>
// (csrc/activation_kernels.cu:22-40): SiLU in fp32 rounded to T, then one multiply rounded to T.
template <int DT>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const uint16_t* __restrict__ in,
                                                           uint16_t* __restrict__ out, int64_t total8,
                                                           int64_t d8) {
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total8; idx += (int64_t)gridDim.x * 256) {
    const int64_t tok = idx / d8, col = idx % d8;
    const u32x4 x = *(const u32x4*)(in + (tok * 2 * d8 + col) * 8);
    const u32x4 y = *(const u32x4*)(in + (tok * 2 * d8 + d8 + col) * 8);
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float xv[2], yv[2], r[2];
      xv[0] = DT == DT_F16 ? f16_lo_f32(x[j]) : bf16_lo_f32(x[j]);
      xv[1] = DT == DT_F16 ? f16_hi_f32(x[j]) : bf16_hi_f32(x[j]);
      yv[0] = DT == DT_F16 ? f16_lo_f32(y[j]) : bf16_lo_f32(y[j]);
      yv[1] = DT == DT_F16 ? f16_hi_f32(y[j]) : bf16_hi_f32(y[j]);
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const float s = silu_f32(xv[q]);
        const uint32_t sr = DT == DT_F16 ? pack_f16(s, 0.f) : pack_bf16(s, 0.f);
        const float st = DT == DT_F16 ? f16_lo_f32(sr) : bf16_lo_f32(sr);
        r[q] = st * yv[q];
      }
      o[j] = DT == DT_F16 ? pack_f16(r[0], r[1]) : pack_bf16(r[0], r[1]);
    }
    *(u32x4*)(out + idx * 8) = o;
  }
}


// Routing: fp32 softmax over the experts of one token, then top-k by repeated arg-max (ties -> lowest expert
// index), as the reference's topk_softmax (csrc/moe/topk_softmax_kernels.cu:127-211, 676-705):
// weights are the softmax probabilities of the chosen experts, optionally renormalised to sum to 1
// (a zero sum divides by 1); token_expert_indices[t, k] = k * num_tokens + t.
// One wavefront per token; lane l holds experts l, l + 64, ... (at most TOPK_PER_LANE of them) in registers.
constexpr int TOPK_PER_LANE = 16;  // up to 1024 experts

template <typename T>
__device__ __forceinline__ float gate_to_f32(T v);
template <>
__device__ __forceinline__ float gate_to_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ float gate_to_f32<_Float16>(_Float16 v) { return (float)v; }
template <>
__device__ __forceinline__ float gate_to_f32<__bf16>(__bf16 v) { return (float)v; }

template <typename T>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const T* __restrict__ gating, float* __restrict__ weights,
                                                           int32_t* __restrict__ ids, int32_t* __restrict__ src_rows,
                                                           int num_tokens, int num_experts, int topk, int renormalize) {
  const int lane = threadIdx.x & 63;
  const int tok = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tok >= num_tokens) return;
  const T* row = gating + (int64_t)tok * num_experts;
  float v[TOPK_PER_LANE];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < TOPK_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < num_experts ? gate_to_f32<T>(row[e]) : -INFINITY;
    mx = fmaxf(mx, v[i]);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < TOPK_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < num_experts ? expf(v[i] - mx) : 0.f;
    sum += v[i];
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d, 64);
#pragma unroll
  for (int i = 0; i < TOPK_PER_LANE; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < num_experts ? v[i] / sum : -1.f;  // probabilities are >= 0: -1 marks "not a candidate"
  }
  float selected = 0.f;
  for (int k = 0; k < topk; ++k) {
    float bv = -1.f;
    int be = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < TOPK_PER_LANE; ++i) {  // ascending expert index inside the lane: strict > keeps the lowest
      if (v[i] > bv) {
        bv = v[i];
        be = lane + 64 * i;
      }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      const float ov = __shfl_xor(bv, d, 64);
      const int oe = __shfl_xor(be, d, 64);
      if (ov > bv || (ov == bv && oe < be)) {
        bv = ov;
        be = oe;
      }
    }
    if (lane == 0) {
      weights[(int64_t)tok * topk + k] = bv;
      ids[(int64_t)tok * topk + k] = be;
      src_rows[(int64_t)tok * topk + k] = k * num_tokens + tok;
    }
    selected += bv;
    if ((be & 63) == lane) {
#pragma unroll
      for (int i = 0; i < TOPK_PER_LANE; ++i)
        if (i == (be >> 6)) v[i] = -1.f;
    }
  }
  // (lane 0 wrote the weights, so lane 0 rescales them: same-thread program order)
  if (renormalize && lane == 0) {
    const float denom = selected > 0.f ? selected : 1.f;
    for (int k = 0; k < topk; ++k) weights[(int64_t)tok * topk + k] /= denom;
  }
}

}  // namespace w4a16

using namespace w4a16;

// Alignment for activations already batched per expert ([B, max_tokens, K], batch_num_tokens[b] valid rows in batch
// b), the contract of the reference's batched_moe_align_block_size (csrc/moe/moe_align_sum_kernels.cu:18-80, 348-373):
// batch b's rows b * max_tokens + j, j < n_b, padded to a multiple of block_size with the value B * max_tokens, runs
// packed in batch order; one batch id per block, -1 past the last; the padded total.  One workgroup: an inclusive scan
// of the padded counts in LDS, then every output slot is written exactly once (its batch found by bisection).
__global__ __launch_bounds__(ALIGN_THREADS) void batched_moe_align_kernel(
    int num_batches, int max_tokens, int block_size, const int32_t* __restrict__ batch_num_tokens,
    int32_t* __restrict__ sorted_ids, int sorted_len, int32_t* __restrict__ block_ids, int32_t* __restrict__ num_post_pad) {
  __shared__ int incl[ALIGN_MAX_EXPERTS];  // inclusive scan of padded counts
  __shared__ int cnt[ALIGN_MAX_EXPERTS];
  const int t = threadIdx.x;
  const int n = t < num_batches ? min(max(batch_num_tokens[t], 0), max_tokens) : 0;
  cnt[t] = n;
  incl[t] = (n + block_size - 1) / block_size * block_size;
  __syncthreads();
  for (int d = 1; d < ALIGN_THREADS; d <<= 1) {
    const int add = t >= d ? incl[t - d] : 0;
    __syncthreads();
    incl[t] += add;
    __syncthreads();
  }
  const int total = incl[ALIGN_THREADS - 1];
  if (t == 0) *num_post_pad = total;
  const int sentinel = num_batches * max_tokens;
  auto batch_of = [&](int pos) {  // first b with incl[b] > pos (pos < total)
    int lo = 0, hi = num_batches - 1;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (incl[mid] > pos) hi = mid; else lo = mid + 1;
    }
    return lo;
  };
  for (int i = t; i < sorted_len; i += ALIGN_THREADS) {
    int v = sentinel;
    if (i < total) {
      const int b = batch_of(i);
      const int start = b == 0 ? 0 : incl[b - 1];
      if (i - start < cnt[b]) v = b * max_tokens + (i - start);
    }
    sorted_ids[i] = v;
  }
  for (int i = t; i < sorted_len / block_size; i += ALIGN_THREADS)
    block_ids[i] = i * block_size < total ? batch_of(i * block_size) : -1;
}

extern "C" int w4a16_moe_align_block_size(const int32_t* topk_ids, int64_t numel, int32_t num_experts,
                                          int32_t block_size, int32_t* sorted_token_ids, int64_t sorted_len,
                                          int32_t* expert_ids, int64_t expert_ids_len,
                                          int32_t* num_tokens_post_pad, void* stream) {
  W4A16_CHECK(topk_ids && sorted_token_ids && expert_ids && num_tokens_post_pad, "null pointer");
  W4A16_CHECK(num_experts >= 1 && num_experts <= ALIGN_MAX_EXPERTS, "num_experts = %d must be in [1, %d]",
              num_experts, ALIGN_MAX_EXPERTS);
  W4A16_CHECK(block_size >= 1, "block_size must be positive");
  W4A16_CHECK(numel >= 0 && numel < (1LL << 30), "bad topk_ids.numel()");
  W4A16_CHECK(sorted_len >= numel, "sorted_token_ids is shorter than topk_ids");
  if (numel >= 2048 && ((uintptr_t)topk_ids & 15) == 0) {
    // slices per expert: enough wavefronts for 64 and more workgroups, slices of at least 256 ids
    int spe = 1;
    while (spe < ALIGN_WAVES && num_experts * spe < 1024 && numel / (2 * spe) >= 256) spe *= 2;
    const int64_t turns = ceil_div(num_experts, ALIGN_WAVES / spe);
    const int grid = (int)(turns < 256 ? turns : 256);
    moe_align_sliced_kernel<<<grid, ALIGN_THREADS, 0, (hipStream_t)stream>>>(
        topk_ids, (int)numel, num_experts, block_size, spe, sorted_token_ids, (int)sorted_len, expert_ids,
        (int)expert_ids_len, num_tokens_post_pad);
    W4A16_HIP(hipGetLastError());
    return 0;
  }
  const int grid = (int)ceil_div(num_experts, ALIGN_WAVES);
  moe_align_kernel<<<grid, ALIGN_THREADS, 0, (hipStream_t)stream>>>(
      topk_ids, (int)numel, num_experts, block_size, sorted_token_ids, (int)sorted_len, expert_ids,
      (int)expert_ids_len, num_tokens_post_pad);
  W4A16_HIP(hipGetLastError());
  return 0;
}

// MoE act-order gather in front of the GEMM (the role of the reference's permute_cols_kernel<moe_block_size>,
// csrc/moe/marlin_moe_wna16/ops.cu:75-149): out[slot, k] = a[sorted_ids[slot] / top_k, perm_e[k]] for every valid slot,
// perm_e = the column order of the expert that owns the slot's block.  One workgroup per slot and turn: the source row is
// staged in LDS with 16-byte loads, every thread assembles 16-byte pieces of the output row from eight 2-byte LDS reads.
// Slots past the padded total, padding slots and blocks of experts of other ranks are skipped (their rows of `out` stay
// as they are: the GEMM kernels never store results of such rows).
namespace w4a16 {
constexpr int MG_MAX_K = 32768;  // 64 KB of LDS
template <bool STAGED>
__global__ __launch_bounds__(256) void moe_gather_rows_kernel(const uint16_t* __restrict__ a, int64_t lda,
                                                             const int32_t* __restrict__ perm,
                                                             const int32_t* __restrict__ sorted_ids,
                                                             const int32_t* __restrict__ expert_ids,
                                                             const int32_t* __restrict__ ntpp, int n_sorted, int block,
                                                             int top_k, int c_rows, int size_k,
                                                             uint16_t* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char mg_smem[];
  uint16_t* row = (uint16_t*)mg_smem;
  const int t = threadIdx.x;
  const int total = min(*ntpp, n_sorted);
  const int pieces = size_k >> 3;
  for (int slot = blockIdx.x; slot < total; slot += gridDim.x) {
    const int id = sorted_ids[slot];
    const int e = expert_ids[slot / block];
    if ((unsigned)id >= (unsigned)c_rows || e < 0) continue;  // (uniform over the workgroup)
    const uint16_t* src = a + (int64_t)(id / top_k) * lda;
    const int32_t* pe = perm + (int64_t)e * size_k;
    uint16_t* dst = out + (int64_t)slot * size_k;
    if constexpr (STAGED) {
      __syncthreads();  // the previous turn's gathers are done
      for (int p = t; p < pieces; p += 256) ((u32x4*)row)[p] = ((const u32x4*)src)[p];
      __syncthreads();
      for (int p = t; p < pieces; p += 256) {
        const u32x4 i0 = *(const u32x4*)(pe + 8 * p), i1 = *(const u32x4*)(pe + 8 * p + 4);
        u32x4 v;
        v[0] = (uint32_t)row[i0[0]] | ((uint32_t)row[i0[1]] << 16);
        v[1] = (uint32_t)row[i0[2]] | ((uint32_t)row[i0[3]] << 16);
        v[2] = (uint32_t)row[i1[0]] | ((uint32_t)row[i1[1]] << 16);
        v[3] = (uint32_t)row[i1[2]] | ((uint32_t)row[i1[3]] << 16);
        ((u32x4*)dst)[p] = v;
      }
    } else {
      for (int k = t; k < size_k; k += 256) dst[k] = src[pe[k]];
    }
  }
}

int moe_gather_rows(const w4a16_gemm_args* a, void* out, hipStream_t stream) {
  const int64_t k = a->size_k;
  if (a->n_sorted <= 0 || k == 0) return 0;
  const int64_t slots = a->n_sorted;
  const unsigned grid = (unsigned)(slots < 8 * (int64_t)num_cus() ? slots : 8 * (int64_t)num_cus());
  const int c_rows = (int)(a->size_m * a->top_k);
  const bool staged = k % 8 == 0 && k <= MG_MAX_K && a->lda % 8 == 0 && ((uintptr_t)a->a & 15) == 0 &&
                      ((uintptr_t)out & 15) == 0 && ((uintptr_t)a->perm & 15) == 0;
  if (staged)
    moe_gather_rows_kernel<true><<<grid, 256, (size_t)k * 2, stream>>>(
        (const uint16_t*)a->a, a->lda, a->perm, a->sorted_token_ids, a->expert_ids, a->num_tokens_past_padded,
        (int)a->n_sorted, a->moe_block_size, a->top_k, c_rows, (int)k, (uint16_t*)out);
  else
    moe_gather_rows_kernel<false><<<grid, 256, 0, stream>>>(
        (const uint16_t*)a->a, a->lda, a->perm, a->sorted_token_ids, a->expert_ids, a->num_tokens_past_padded,
        (int)a->n_sorted, a->moe_block_size, a->top_k, c_rows, (int)k, (uint16_t*)out);
  W4A16_HIP(hipGetLastError());
  return 0;
}
}  // namespace w4a16

extern "C" int w4a16_moe_sum(const void* in, void* out, int64_t tokens, int32_t top_k, int64_t hidden,
                             int32_t dtype, void* stream) {
  W4A16_CHECK(in && out, "null pointer");
  W4A16_CHECK(hidden % 8 == 0, "hidden = %lld must be divisible by 8", (long long)hidden);
  W4A16_CHECK(dtype == W4A16_DTYPE_F16 || dtype == W4A16_DTYPE_BF16, "unsupported dtype");
  const int64_t total8 = tokens * (hidden / 8);
  if (total8 == 0) return 0;
  const int64_t blocks = ceil_div(total8, 256);
  const unsigned grid = (unsigned)(blocks < 65536 ? blocks : 65536);
  if (dtype == W4A16_DTYPE_F16)
    moe_sum_kernel<DT_F16><<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)in, (uint16_t*)out, total8, top_k, hidden / 8);
  else
    moe_sum_kernel<DT_BF16><<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)in, (uint16_t*)out, total8, top_k, hidden / 8);
  W4A16_HIP(hipGetLastError());
  return 0;
}

extern "C" int w4a16_silu_and_mul(const void* in, void* out, int64_t tokens, int64_t d, int32_t dtype,
                                  void* stream) {
  W4A16_CHECK(in && out, "null pointer");
  W4A16_CHECK(d % 8 == 0, "d = %lld must be divisible by 8", (long long)d);
  W4A16_CHECK(dtype == W4A16_DTYPE_F16 || dtype == W4A16_DTYPE_BF16, "unsupported dtype");
  const int64_t total8 = tokens * (d / 8);
  if (total8 == 0) return 0;
  const int64_t blocks = ceil_div(total8, 256);
  const unsigned grid = (unsigned)(blocks < 65536 ? blocks : 65536);
  if (dtype == W4A16_DTYPE_F16)
    silu_and_mul_kernel<DT_F16><<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)in, (uint16_t*)out, total8, d / 8);
  else
    silu_and_mul_kernel<DT_BF16><<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)in, (uint16_t*)out, total8, d / 8);
  W4A16_HIP(hipGetLastError());
  return 0;
}

extern "C" int w4a16_topk_softmax(const void* gating_output, int32_t gating_dtype, float* topk_weights,
                                  int32_t* topk_ids, int32_t* token_expert_indices, int64_t num_tokens,
                                  int32_t num_experts, int32_t topk, int32_t renormalize, void* stream) {
  W4A16_CHECK(gating_output && topk_weights && topk_ids && token_expert_indices, "null pointer");
  W4A16_CHECK(num_experts >= 1 && num_experts <= 64 * TOPK_PER_LANE, "num_experts = %d must be in [1, %d]", num_experts,
              64 * TOPK_PER_LANE);
  W4A16_CHECK(topk >= 1 && topk <= num_experts, "topk = %d must be in [1, num_experts]", topk);
  W4A16_CHECK(num_tokens >= 0 && num_tokens < (1LL << 30), "bad num_tokens");
  if (num_tokens == 0) return 0;
  const unsigned grid = (unsigned)ceil_div(num_tokens, 4);
  hipStream_t st = (hipStream_t)stream;
  if (gating_dtype == W4A16_DTYPE_F16)
    topk_softmax_kernel<_Float16><<<grid, 256, 0, st>>>((const _Float16*)gating_output, topk_weights, topk_ids,
                                                       token_expert_indices, (int)num_tokens, num_experts, topk, renormalize);
  else if (gating_dtype == W4A16_DTYPE_BF16)
    topk_softmax_kernel<__bf16><<<grid, 256, 0, st>>>((const __bf16*)gating_output, topk_weights, topk_ids,
                                                     token_expert_indices, (int)num_tokens, num_experts, topk, renormalize);
  else if (gating_dtype == W4A16_DTYPE_F32)
    topk_softmax_kernel<float><<<grid, 256, 0, st>>>((const float*)gating_output, topk_weights, topk_ids,
                                                    token_expert_indices, (int)num_tokens, num_experts, topk, renormalize);
  else
    return fail(W4A16_EINVAL, "gating_output must be fp16, bf16 or fp32");
  W4A16_HIP(hipGetLastError());
  return 0;
}

extern "C" int w4a16_batched_moe_align_block_size(int64_t max_tokens_per_batch, int32_t block_size,
                                                  const int32_t* batch_num_tokens, int32_t num_batches,
                                                  int32_t* sorted_ids, int64_t sorted_len, int32_t* block_ids,
                                                  int64_t block_ids_len, int32_t* num_tokens_post_pad, void* stream) {
  W4A16_CHECK(batch_num_tokens && sorted_ids && block_ids && num_tokens_post_pad, "null pointer");
  W4A16_CHECK(block_size > 0 && max_tokens_per_batch >= 0, "bad block_size / max_tokens_per_batch");
  W4A16_CHECK(num_batches >= 1 && num_batches <= ALIGN_MAX_EXPERTS, "num_batches = %d must be in [1, %d]", num_batches,
              ALIGN_MAX_EXPERTS);
  const int64_t want = ceil_div(max_tokens_per_batch, block_size) * block_size * num_batches;
  W4A16_CHECK(sorted_len == want, "sorted_ids has %lld elements, expected %lld", (long long)sorted_len, (long long)want);
  W4A16_CHECK(block_ids_len == want / block_size, "batch_ids has %lld elements, expected %lld", (long long)block_ids_len,
              (long long)(want / block_size));
  W4A16_CHECK(want < (1LL << 31) && num_batches * max_tokens_per_batch < (1LL << 31), "problem too large");
  batched_moe_align_kernel<<<1, ALIGN_THREADS, 0, (hipStream_t)stream>>>(num_batches, (int)max_tokens_per_batch, block_size,
                                                                         batch_num_tokens, sorted_ids, (int)sorted_len,
                                                                         block_ids, num_tokens_post_pad);
  W4A16_HIP(hipGetLastError());
  return 0;
}
