// Kernel parameter block and cross-workgroup helpers shared by the W4A16 GEMM kernels.
#pragma once
#include <mutex>

#include "gemm_plan.h"

namespace w4a16 {

struct KParams {
  const void* A;
  int64_t lda;
  void* C;
  const uint32_t* B;
  const void* S;
  const uint32_t* Z;
  const int32_t* gidx;
  const void* bias;
  const void* gscale;  // NVFP4 global scale (one element of the activation type per expert), else null
  int fp8;             // weights are float8_e4m3fn (their stored scales carry an exponent offset)
  float* ctmp;
  int32_t* locks;
  int lock_stride;
  int M;       // rows of A
  int c_rows;  // rows of C (M, or M*top_k for MoE)
  int N, K;
  int group_ksteps;  // GM_GROUPED: group_size / 32
  int group_shift;   // log2(group_ksteps) when that is a power of two, else -1
  int ncp;           // column tiles = ceil(N / tile width)
  int tiles;         // output tiles of the launch (ncp x m-tiles)
  int splits, ksteps_per_split, total_ksteps;
  int xcd_map;
  int tn;        // tile width in columns (128, or 64 for the narrow decode tiles)
  int strip0;    // 64-row kernel / K-split kernel: first 512- / 256-column strip of this launch (it may finish what the prefill kernel left)
  int dyn_slots; // 64-row kernel, MoE: > 0 = the K split is chosen on the device from the number of live blocks (tail_split)
  // MoE
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* ntpp;
  const float* topk_w;
  int moe, moe_bs, top_k, mul_topk;
  int n_sorted;  // usable length of sorted_ids
  int64_t b_estride, s_estride, z_estride, k_estride, n_estride;  // per-expert strides (elements)
  // fused epilogues
  int a_by_slot;  // MoE: row r of block mt reads A row mt * block + r (gathered in front of the launch), not id / top_k
  int act;        // 1: column halves are gate | up; C is [rows, N / 2] = silu(gate) * up
  int sum_div;    // > 0: result row i is added atomically into C row i / sum_div
  uint32_t* zero_ptr;  // side job: zero_n16 16-byte pieces to clear, spread over the grid
  int64_t zero_n16;
};

// 64-row kernel on MoE problems.  The number of live tiles L (blocks that hold tokens x column strips) is only known on
// the device, and whole tiles run in rounds of `slots` resident workgroups.  The tiles of the last, partly filled round
// (all tiles, when there are fewer than `slots`) are therefore cut along K into S pieces each, as many as still fit that
// round, and a second pass adds the pieces: F tiles run whole, the R = L - F tail tiles as R * S pieces of kps k-steps
// (a multiple of 4, at least 32).  Only from S = 3 on: a tail of more than slots / 3 tiles already runs with fewer
// workgroups per compute unit, hence faster, and halving it gains less than the partial tiles cost.  Both passes derive
// the same numbers from L.
constexpr int TAIL_MIN_KSTEPS = 32;
struct TailSplit {
  int F, R, S, kps;
};
__host__ __device__ inline TailSplit tail_split(int live_tiles, int slots, int total_ksteps) {
  TailSplit d;
  d.F = (live_tiles / slots) * slots;
  d.R = live_tiles - d.F;
  d.S = 1;
  d.kps = total_ksteps;
  if (d.R > 0) {
    int s = slots / d.R;
    if (s > 8) s = 8;
    if (s > total_ksteps / TAIL_MIN_KSTEPS) s = total_ksteps / TAIL_MIN_KSTEPS;
    if (s >= 3) {
      d.kps = ((total_ksteps + s - 1) / s + 3) / 4 * 4;
      d.S = (total_ksteps + d.kps - 1) / d.kps;
    }
  }
  return d;
}

// Side job of a launch: the grid clears `zero_n16` 16-byte pieces at `zero_ptr` (the output of a later launch that
// accumulates with atomic adds).  Every workgroup of the grid calls this first, before any early exit.
__device__ __forceinline__ void zero_fill_side_job(const KParams& p, unsigned block, unsigned nblocks) {
  if (p.zero_n16 <= 0) return;
  const int64_t per = (p.zero_n16 + nblocks - 1) / nblocks;
  const int64_t b = (int64_t)block * per, e = b + per < p.zero_n16 ? b + per : p.zero_n16;
  for (int64_t i = b + threadIdx.x; i < e; i += blockDim.x) ((u32x4*)p.zero_ptr)[i] = u32x4{0, 0, 0, 0};
}
__device__ __forceinline__ void zero_fill_side_job(const KParams& p) { zero_fill_side_job(p, blockIdx.x, gridDim.x); }

template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  return DT == DT_F16 ? pack_f16(lo, hi) : pack_bf16(lo, hi);
}
template <int DT>
__device__ __forceinline__ float lo_f32(uint32_t x) { return DT == DT_F16 ? f16_lo_f32(x) : bf16_lo_f32(x); }
template <int DT>
__device__ __forceinline__ float hi_f32(uint32_t x) { return DT == DT_F16 ? f16_hi_f32(x) : bf16_hi_f32(x); }

// Four finished fp32 results of C row `crow`, columns ncol .. ncol + 3: rounded to the 16-bit type, then stored, or
// (sum_div > 0) added into row crow / sum_div with packed 16-bit atomic adds.
template <int DT, bool MOE = true>
__device__ __forceinline__ void store_row4(const KParams& p, int crow, int ncol, f32x4 v) {
  const uint32_t o0 = pack2<DT>(v[0], v[1]), o1 = pack2<DT>(v[2], v[3]);
  if (MOE && p.sum_div > 0) {
    uint16_t* dst = (uint16_t*)p.C + (int64_t)(crow / p.sum_div) * p.N + ncol;
    if constexpr (DT == DT_F16) {
      typedef _Float16 h2 __attribute__((ext_vector_type(2)));
      __builtin_amdgcn_global_atomic_fadd_v2f16((h2*)dst, __builtin_bit_cast(h2, o0));
      __builtin_amdgcn_global_atomic_fadd_v2f16((h2*)(dst + 2), __builtin_bit_cast(h2, o1));
    } else {
      typedef short s2 __attribute__((ext_vector_type(2)));
      __builtin_amdgcn_global_atomic_fadd_v2bf16((s2*)dst, __builtin_bit_cast(s2, o0));
      __builtin_amdgcn_global_atomic_fadd_v2bf16((s2*)(dst + 2), __builtin_bit_cast(s2, o1));
    }
  } else {
    *(u32x2*)((uint16_t*)p.C + (int64_t)crow * p.N + ncol) = u32x2{o0, o1};
  }
}

// silu(gate) * up on finished fp32 results, with the roundings of a GEMM store followed by the reference's
// act_and_mul_kernel<silu> (csrc/activation_kernels.cu:22-40): gate and up rounded to the 16-bit type, SiLU evaluated
// in fp32 and rounded, the product rounded.  Stored at C[crow][ocol .. ocol + 3], row stride N / 2.
template <int DT>
__device__ __forceinline__ void store_row4_silu_mul(const KParams& p, int crow, int ocol, f32x4 gate, f32x4 up) {
  float r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t gu = pack2<DT>(gate[j], up[j]);
    const float gv = lo_f32<DT>(gu), uv = hi_f32<DT>(gu);
    r[j] = lo_f32<DT>(pack2<DT>(silu_f32(gv), 0.f)) * uv;
  }
  *(u32x2*)((uint16_t*)p.C + (int64_t)crow * (p.N >> 1) + ocol) = u32x2{pack2<DT>(r[0], r[1]), pack2<DT>(r[2], r[3])};
}

// Split-K partials cross XCDs (each XCD has its own L2).  A plain store stays dirty in the writer's L2,
// and an agent-scope release fence (an L2 write-back) costs ~0.5 us per workgroup, serialised per L2.
// Instead every partial is written with relaxed agent-scope atomic stores (global_store ... sc1: written
// through to the device-coherent level) and read back with agent-scope loads (sc1: never served from a
// non-coherent line), 8 bytes at a time.  The writer waits for its stores (s_waitcnt) before it counts
// itself as arrived; the reader is whoever sees the last arrival.
//
// Why the last arriver reads complete partial tiles, instruction by instruction (16-row kernels, gemm_decode.hip /
// gemm_skinny.hip epilogue):
//   1. every thread of a writing workgroup issues its partial sums as `global_store_dwordx2 ... sc1`: the store is
//      performed at the device-coherent level, not left dirty in the XCD's L2;
//   2. `s_waitcnt vmcnt(0)` (__builtin_amdgcn_s_waitcnt(0)) in every thread: vmcnt only drops when the memory system has
//      acknowledged the store, i.e. when it is performed at that level, so after the wait the thread's words are visible
//      to any later sc1 load of any compute unit;
//   3. `s_barrier`: all threads of the workgroup have passed step 2 before thread 0 goes on;
//   4. thread 0 executes `global_atomic_inc ... sc0` at agent scope on the tile's counter: a read-modify-write performed
//      at the same coherent level, issued after (program order + the barrier) every store of its workgroup was
//      acknowledged.  Read-modify-writes on one address are totally ordered, so exactly one workgroup reads the value
//      splits - 1, and at that point every other workgroup's increment, hence (steps 2-3) every other workgroup's stores,
//      have been performed;
//   5. the returned value reaches the other threads through LDS and a second `s_barrier`; their `global_load_dwordx2
//      ... sc1` are issued after that barrier, cannot be served from a stale line of the compute unit's or the XCD's
//      cache, and therefore return the performed stores.
// What this does not use: a release/acquire fence pair (buffer_wbl2 / buffer_inv).  The argument rests on sc1 accesses
// being performed at one common level in issue order per thread after an acknowledged wait, which is how the ISA defines
// them, not on the HIP memory model's fences; tests/test_gpu_splitk_stress.py runs thousands of back-to-back launches of
// these paths and compares every result bit for bit.
__device__ __forceinline__ void store_coherent2(float* ptr, float f0, float f1) {
  using u64 = unsigned long long;
  const u64 a = (u64)__builtin_bit_cast(uint32_t, f0) | ((u64)__builtin_bit_cast(uint32_t, f1) << 32);
  __hip_atomic_store((u64*)ptr, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_coherent(float* ptr, f32x4 v) {
  // (elements are copied to scalars first: bit-casting a vector element directly reads element 0)
  const float f0 = v[0], f1 = v[1], f2 = v[2], f3 = v[3];
  store_coherent2(ptr, f0, f1);
  store_coherent2(ptr + 2, f2, f3);
}
__device__ __forceinline__ void load_coherent2(const float* ptr, float& f0, float& f1) {
  using u64 = unsigned long long;
  const u64 a = __hip_atomic_load((const u64*)ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  f0 = __builtin_bit_cast(float, (uint32_t)a);
  f1 = __builtin_bit_cast(float, (uint32_t)(a >> 32));
}
__device__ __forceinline__ f32x4 load_coherent(const float* ptr) {
  float f0, f1, f2, f3;
  load_coherent2(ptr, f0, f1);
  load_coherent2(ptr + 2, f2, f3);
  return f32x4{f0, f1, f2, f3};
}

// Arrival at a tile's counter: a wrapping increment (old >= splits - 1 ? 0 : old + 1), so the last of `splits`
// arrivals leaves the counter at zero again without a second access; returns true for that last arrival.
// Measured on the part this is ~1 us shorter than fetch-add + reset store.
__device__ __forceinline__ bool arrive_last(int32_t* counter, int splits) {
  const unsigned old = __builtin_amdgcn_atomic_inc32((unsigned*)counter, (unsigned)(splits - 1), __ATOMIC_RELAXED, "agent");
  return old == (unsigned)(splits - 1);
}

// Host: more than 64 KiB of dynamic LDS has to be allowed per kernel function; done once per function, device and
// process (thread-safe).  Returns a HIP error code.
inline hipError_t allow_dynamic_lds(const void* fn, int bytes) {
  if (bytes <= 64 * 1024) return hipSuccess;
  struct Key { const void* fn; int dev; };
  static std::mutex mu;
  static Key seen[256];
  static int n_seen = 0;
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  std::lock_guard<std::mutex> lock(mu);
  for (int i = 0; i < n_seen; ++i)
    if (seen[i].fn == fn && seen[i].dev == dev) return hipSuccess;
  if (hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes)) return e;
  if (n_seen < 256) seen[n_seen++] = Key{fn, dev};
  return hipSuccess;
}

// Host: translate the C-ABI arguments and the launch plan into the kernel parameter block.
inline KParams make_kparams(const w4a16_gemm_args* a, const Plan& pl) {
  const bool moe = (a->flags & W4A16_F_MOE) != 0;
  KParams p{};
  p.A = a->a;
  p.lda = a->lda;
  p.C = a->c;
  p.B = a->b_q_weight;
  p.S = a->b_scales;
  p.Z = a->b_zeros;
  p.gidx = pl.gm == GM_GIDX ? a->g_idx : nullptr;
  p.bias = a->b_bias;
  p.gscale = a->global_scale;
  p.fp8 = a->wtype == W4A16_WTYPE_FE4M3;
  p.ctmp = a->c_tmp;
  p.locks = a->workspace;
  // counters of neighbouring tiles 16 bytes apart when the workspace is long enough (arrivals complete sooner)
  p.lock_stride = a->workspace_len >= 4 * (int64_t)pl.tiles ? 4 : (a->workspace_len >= 2 * (int64_t)pl.tiles ? 2 : 1);
  p.M = (int)a->size_m;
  p.c_rows = (int)(moe ? a->size_m * a->top_k : a->size_m);
  p.N = (int)a->size_n;
  p.K = (int)a->size_k;
  p.group_ksteps = pl.group_ksteps;
  p.group_shift = -1;
  for (int sh = 0; sh < 20; ++sh)
    if ((1 << sh) == pl.group_ksteps) p.group_shift = sh;
  p.ncp = pl.ncp;
  p.tiles = pl.tiles;
  p.splits = pl.splits;
  p.ksteps_per_split = pl.kps;
  p.total_ksteps = pl.total_ksteps;
  p.xcd_map = pl.xcd_map;
  p.tn = pl.tn;
  p.strip0 = pl.strip0;
  p.dyn_slots = pl.dyn_slots;
  p.sorted_ids = a->sorted_token_ids;
  p.expert_ids = a->expert_ids;
  p.ntpp = a->num_tokens_past_padded;
  p.topk_w = a->topk_weights;
  p.moe = moe;
  p.moe_bs = a->moe_block_size;
  p.top_k = moe ? a->top_k : 1;
  p.mul_topk = moe && (a->flags & W4A16_F_MUL_TOPK_WEIGHTS);
  p.n_sorted = moe ? (int)a->n_sorted : 0;
  p.b_estride = (a->size_k / 16) * ((a->wtype == W4A16_WTYPE_U8B128 || a->wtype == W4A16_WTYPE_FE4M3) ? 4 : 2) * a->size_n;
  // scale elements are addressed as 16-bit words; fp4 scales are one byte each
  p.s_estride = a->num_groups * a->size_n / (a->wtype == W4A16_WTYPE_FE2M1 ? 2 : 1);
  p.z_estride = a->num_groups * (a->size_n / 8);
  p.k_estride = a->size_k;
  p.n_estride = a->size_n;
  p.a_by_slot = moe && pl.a_by_slot;
  p.act = moe && (a->flags & W4A16_F_SILU_AND_MUL);
  p.sum_div = (moe && (a->flags & W4A16_F_SUM_TOPK)) ? a->sum_top_k : 0;
  p.zero_ptr = (uint32_t*)a->zero_fill;
  p.zero_n16 = a->zero_fill ? a->zero_fill_bytes / 16 : 0;
  return p;
}

// In-place MFMA on an accumulator pinned to AGPRs.  With 128 or 256 accumulators per lane the register allocator
// otherwise assigns different registers to an MFMA's source and destination accumulator and fills the loop
// with v_accvgpr moves (more of them than dequantisation instructions).  Source C == destination is the form
// the matrix pipe forwards without extra wait states; results are only read again after the main loop.
// The statement is opaque to the compiler's hazard logic: an operand register must not be written by a VALU
// instruction in the two wait states before it.  Callers dequantise every operand register at least one MFMA (16 cycles)
// ahead of its use and pin that order with scheduling barriers; the build step verifies the compiler's output.
// (Two wait states in front of every such MFMA, `s_nop 1` inside the statement, would make this unconditional; it costs
// 5-8 % of the prefill kernels' throughput and is only compiled in with -DW4A16_MFMA_NOP.  The shipped build instead
// scans its own compiler output for the hazard, see vllm_amd/build.py: check_mfma_hazards.)
#ifdef W4A16_MFMA_NOP
#define W4A16_MFMA_PRE "s_nop 1\n\t"
#else
#define W4A16_MFMA_PRE ""
#endif
template <int DT>
__device__ __forceinline__ void mfma_inplace(f32x4& acc, const u32x4& a, const u32x4& b) {
  if constexpr (DT == DT_F16)
    asm(W4A16_MFMA_PRE "v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  else
    asm(W4A16_MFMA_PRE "v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

constexpr int RED_RS = 148;  // row stride (floats) of the 128-column reduction slab (4 mod 16: conflict-free)

}  // namespace w4a16
