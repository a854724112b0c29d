// W4A16 "skinny" GEMM for gfx950: C[M,N] = A[M,K] * dequant(Bq)[K,N] (+bias), dense or fused-MoE.
//
// Stands in for the reference's Marlin<> kernel (csrc/quantization/gptq_marlin/marlin_template.h:273-1804)
// and its MoE twin (csrc/moe/marlin_moe_wna16/marlin_template.h:298-2009); written from scratch for
// wave64 + MFMA, see gemm_common.h for how a wavefront reads the Marlin layout.
//
// Work decomposition
//   tile  = (m-tile of BM = 16*MB rows) x (column pair = 128 columns)
//   split = contiguous range of k-steps (32 K-rows each) of that tile
//   one workgroup of 8 wavefronts per (tile, split), meant to own a compute unit.  The wavefronts
//   share the tile's rows and columns and cut the split's k-steps into 8 contiguous parts, so no
//   wavefront waits on another inside the main loop:
//     weights      global -> registers, 128-bit per lane, 1 KiB contiguous per wavefront instruction,
//                  D k-steps (2D KiB) in flight per wavefront
//     activations  global -> registers, 16 bytes per lane (row l&15, 8 consecutive K), turned into the
//                  MFMA A operand by a 4x4 lane-group/register transpose (4 v_permlane*_swap); no LDS
//     scales/zeros one 16-byte / 4-byte load per k-step (cache hits after the first of a group)
//   The 8 partial tiles are summed through LDS.  Splits are summed by the last workgroup to arrive
//   at the tile's counter in `workspace`, in split order (deterministic); the counter is reset so
//   the workspace is all-zero on exit, as the reference requires (csrc/torch_bindings.cpp:255-267).
// HBM traffic per launch: every weight byte once (K*N/2), scales (K/g)*N*2, C once; A is re-read
// once per column pair (from L2), split partials move 2 * splits * M * N * 4 bytes.
#include <stdlib.h>

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
  const int32_t* perm;
  const void* bias;
  float* ctmp;
  int32_t* locks;
  int M;       // rows of A
  int c_rows;  // rows of C (M, or M*top_k for MoE)
  int N, K;
  int group_ksteps;  // GM_GROUPED: group_size / 32
  int ncp;           // column pairs = ceil(N / 128)
  int splits, ksteps_per_split, total_ksteps;
  int xcd_map;
  int fix_mode;
  // MoE
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* ntpp;
  const float* topk_w;
  int moe, moe_bs, top_k, mul_topk;
  int64_t b_estride, s_estride, z_estride, k_estride, n_estride;  // per-expert strides (elements)
};

// Split partials cross XCDs (each XCD has its own L2).  A plain store stays dirty in the writer's L2
// and an agent-scope release fence (L2 write-back) costs ~0.5 us per workgroup, serialised per L2.
// Instead every partial word is written with an agent-scope atomic exchange, which is performed at
// the device-coherent level, and read back with agent-scope loads (sc1: bypass non-coherent lines).
__device__ __forceinline__ void store_coherent(float* ptr, f32x4 v, int mode) {
  using u64 = unsigned long long;
  // (elements are copied to scalars first: bit-casting a vector element directly reads element 0)
  const float f0 = v[0], f1 = v[1], f2 = v[2], f3 = v[3];
  const u64 a = (u64)__builtin_bit_cast(uint32_t, f0) | ((u64)__builtin_bit_cast(uint32_t, f1) << 32);
  const u64 b = (u64)__builtin_bit_cast(uint32_t, f2) | ((u64)__builtin_bit_cast(uint32_t, f3) << 32);
  if (mode == 3) {
    __hip_atomic_store((u64*)ptr, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __hip_atomic_store((u64*)ptr + 1, b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  } else if (mode == 0) {
    __hip_atomic_store((u64*)ptr, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store((u64*)ptr + 1, b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
    __hip_atomic_exchange((u64*)ptr, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_exchange((u64*)ptr + 1, b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}
__device__ __forceinline__ f32x4 load_coherent(const float* ptr, int mode) {
  using u64 = unsigned long long;
  u64 a, b;
  if (mode == 3) {
    a = __hip_atomic_load((const u64*)ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    b = __hip_atomic_load((const u64*)ptr + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  } else {
    a = __hip_atomic_load((const u64*)ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    b = __hip_atomic_load((const u64*)ptr + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  return f32x4{__builtin_bit_cast(float, (uint32_t)a), __builtin_bit_cast(float, (uint32_t)(a >> 32)),
               __builtin_bit_cast(float, (uint32_t)b), __builtin_bit_cast(float, (uint32_t)(b >> 32))};
}

constexpr int NW = 8;        // wavefronts per workgroup
constexpr int RED_RS = 148;  // row stride (floats) of the reduction slab; see epilogue

template <int MB>
struct SkinnyCfg {
  static constexpr int D = (MB >= 4) ? 3 : (MB == 2 ? 6 : 8);  // k-steps in flight per wavefront
  static constexpr int SMEM = NW * 16 * RED_RS * 4;             // reduction slab only
};


template <int DT, int MB, bool ZP, int GM, bool PERM>
__global__ __launch_bounds__(NW * 64) void skinny_kernel(const KParams p) {
  constexpr int BM = 16 * MB;
  constexpr int D = SkinnyCfg<MB>::D;
  constexpr bool UNIT = (GM == GM_CHANNEL);
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int s_crow[BM];  // C row of each tile row, -1 = not written
  __shared__ int s_last;

  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 7, h = (lane >> 3) & 1, g = lane >> 4;
  const int am = lane & 15;  // activation row inside an m-block (MFMA A operand row)

  int tile, split;
  {
    const int b = blockIdx.x;
    if (p.xcd_map) {  // all splits of a tile on one XCD (consecutive workgroup ids rotate over 8 XCDs)
      const int idx = b >> 3;
      tile = (idx / p.splits) * 8 + (b & 7);
      split = idx % p.splits;
    } else {
      tile = b / p.splits;
      split = b % p.splits;
    }
  }
  const int cp = tile % p.ncp, mt = tile / p.ncp;

  const uint32_t* Bq = p.B;
  const uint16_t* Sc = (const uint16_t*)p.S;
  const uint32_t* Zp = p.Z;
  const int32_t* gidx = p.gidx;
  const int32_t* perm = p.perm;
  const uint16_t* bias = (const uint16_t*)p.bias;
  if (p.moe) {
    if (mt * p.moe_bs >= *p.ntpp) return;
    const int e = p.expert_ids[mt];
    if (e < 0) return;
    Bq += e * p.b_estride;
    Sc += e * p.s_estride;
    if (ZP) Zp += e * p.z_estride;
    if (gidx) gidx += e * p.k_estride;
    if (PERM) perm += e * p.k_estride;
    if (bias) bias += e * p.n_estride;
  }

  // ---- which A row feeds each tile row, which C row it is written to.  Rows past the end of the
  // problem read the tile's first row (always valid) so that LDS never holds uninitialised data;
  // their results are never stored.
  auto tile_row_ids = [&](int r, int& src, int& dst) {
    src = -1;
    dst = -1;
    if (p.moe) {
      if (r < p.moe_bs) {
        const int id = p.sorted_ids[mt * p.moe_bs + r];
        if (id < p.c_rows) {
          src = id / p.top_k;
          dst = id;
        }
      }
    } else {
      const int gr = mt * BM + r;
      if (gr < p.M) src = dst = gr;
    }
  };
  const uint16_t* arow[MB];
  {
    int src0, dst0;
    tile_row_ids(0, src0, dst0);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      int src, dst;
      tile_row_ids(mb * 16 + am, src, dst);
      arow[mb] = (const uint16_t*)p.A + (int64_t)(src >= 0 ? src : src0) * p.lda + g * 8;
    }
  }
  if (threadIdx.x < BM) {
    int src, dst;
    tile_row_ids(threadIdx.x, src, dst);
    s_crow[threadIdx.x] = dst;
  }

  // ---- this wavefront's k-steps
  const int ks_b = split * p.ksteps_per_split;
  const int ks_e = min(ks_b + p.ksteps_per_split, p.total_ksteps);
  const int per = (ks_e - ks_b + NW - 1) / NW;
  const int w_b = min(ks_b + wv * per, ks_e), w_e = min(w_b + per, ks_e);
  const int nks = (p.fix_mode == 12 || p.fix_mode == 13) ? 0 : w_e - w_b;

  // lanes of an n-tile past the end of N (odd number of n-tiles) read n-tile 0; their columns are never stored
  const int nt = (2 * cp + h) * 64 < p.N ? 2 * cp + h : 0;
  const int64_t b_row = p.N >> 1;  // u32x4 per k-tile row
  const u32x4* bp = (const u32x4*)Bq + nt * 32 + (4 * c + g);
  const int64_t s_row = p.N >> 3;  // u32x4 (8 scales) per scale row; also words per zero-point row
  const u32x4* sp = (const u32x4*)Sc + nt * 8 + c;
  const uint32_t* zp = ZP ? Zp + nt * 8 + c : nullptr;

  // Activations: lane (row am, piece g) loads the 16 bytes A[row][32ks + 8g .. +8) = K pairs 8g+2q, q=0..3.
  // The MFMA lane (row, g) needs pair 8s+2g for s=0..3, i.e. register g of the lane 16s+row: a 4x4
  // transpose between the four 16-lane groups and the four registers, done with permlane swaps.
  struct Stage {
    u32x4 b0, b1, sc;
    u32x4 a[MB];
    uint32_t zq;
    int gi;
    bool uni;
  };
  Stage st[D];

  auto issue = [&](Stage& s, int ks) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      if constexpr (PERM) {
        uint16_t e[8];
        const uint16_t* row = arow[mb] - g * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = row[perm[ks * 32 + g * 8 + j]];
        s.a[mb] = u32x4{(uint32_t)e[0] | ((uint32_t)e[1] << 16), (uint32_t)e[2] | ((uint32_t)e[3] << 16),
                        (uint32_t)e[4] | ((uint32_t)e[5] << 16), (uint32_t)e[6] | ((uint32_t)e[7] << 16)};
      } else {
        s.a[mb] = *(const u32x4*)(arow[mb] + ks * 32);
      }
    }
    int gi = 0;
    s.uni = true;
    if (GM == GM_GROUPED) gi = ks / p.group_ksteps;
    if (GM == GM_GIDX) {
      gi = gidx[ks * 32];
      s.uni = (gidx[ks * 32 + 31] == gi);
    }
    s.gi = gi;
    if (GM != GM_CHANNEL) s.sc = sp[(int64_t)gi * s_row];
    if (ZP) s.zq = zp[(int64_t)gi * s_row];
    s.b0 = __builtin_nontemporal_load(bp + (int64_t)(2 * ks) * b_row);
    s.b1 = __builtin_nontemporal_load(bp + (int64_t)(2 * ks + 1) * b_row);
  };

  f32x4 acc[MB][4][2];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      acc[mb][w][0] = f32x4{0, 0, 0, 0};
      acc[mb][w][1] = f32x4{0, 0, 0, 0};
    }

  auto consume = [&](const Stage& s, int ks) {
    u32x4 af[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      uint32_t r0 = s.a[mb][0], r1 = s.a[mb][1], r2 = s.a[mb][2], r3 = s.a[mb][3];
      typedef uint32_t u2 __attribute__((ext_vector_type(2)));
      u2 t;
      t = __builtin_amdgcn_permlane32_swap(r0, r2, false, false); r0 = t[0]; r2 = t[1];
      t = __builtin_amdgcn_permlane32_swap(r1, r3, false, false); r1 = t[0]; r3 = t[1];
      t = __builtin_amdgcn_permlane16_swap(r0, r1, false, false); r0 = t[0]; r1 = t[1];
      t = __builtin_amdgcn_permlane16_swap(r2, r3, false, false); r2 = t[0]; r3 = t[1];
      af[mb] = u32x4{r0, r1, r2, r3};
    }
    if (GM == GM_GIDX && !s.uni) {
      // group boundary inside the k-step: fetch the scale row of every K-row separately
      const int kb = ks * 32 + 2 * g;
      u32x4 se[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int kk = kb + (e & 1) + ((e >> 1) & 1) * 8 + (e >> 2) * 16;
        se[e] = sp[(int64_t)gidx[kk] * s_row];
      }
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const ColConst<DT> cc = make_col_const<DT, true>(0, 8, 8);
        u32x4 o[2];
        dequant_pair<DT, true>(s.b0[w], s.b1[w], cc, o[0], o[1]);
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          u32x4 r;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t sa = (se[2 * q][w] >> (16 * hf)) & 0xffffu;
            const uint32_t sb = (se[2 * q + 1][w] >> (16 * hf)) & 0xffffu;
            const uint32_t spair = sa | (sb << 16);
            if constexpr (DT == DT_F16)
              r[q] = as_u32(as_h2(o[hf][q]) * as_h2(spair));
            else
              r[q] = pack_bf16(bf16_lo_f32(o[hf][q]) * bf16_lo_f32(spair),
                               bf16_hi_f32(o[hf][q]) * bf16_hi_f32(spair));
          }
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) acc[mb][w][hf] = mfma16x16x32<DT>(af[mb], r, acc[mb][w][hf]);
        }
      }
      return;
    }
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t z0 = 8, z1 = 8;
      if (ZP) {
        z0 = (s.zq >> (4 * w)) & 0xf;
        z1 = (s.zq >> (4 * w + 16)) & 0xf;
      }
      const ColConst<DT> cc = make_col_const<DT, UNIT>(GM == GM_CHANNEL ? 0u : s.sc[w], z0, z1);
      u32x4 o0, o1;
      dequant_pair<DT, UNIT>(s.b0[w], s.b1[w], cc, o0, o1);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        acc[mb][w][0] = mfma16x16x32<DT>(af[mb], o0, acc[mb][w][0]);
        acc[mb][w][1] = mfma16x16x32<DT>(af[mb], o1, acc[mb][w][1]);
      }
    }
  };

  // ---- software pipeline: D k-steps in flight.  The steady-state loop is free of conditionals so
  // that every stage waits only for its own loads; the last (at most 2D-1) k-steps drain the ring.
  int done = 0;
  if (nks >= D) {
#pragma unroll
    for (int j = 0; j < D; ++j) issue(st[j], w_b + j);
    for (; done + 2 * D <= nks; done += D) {
#pragma unroll
      for (int j = 0; j < D; ++j) {
        consume(st[j], w_b + done + j);
        __builtin_amdgcn_sched_barrier(0);  // keep each stage's loads where they are issued:
        issue(st[j], w_b + done + j + D);   // the scheduler would otherwise sink them to the loop end
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < D; ++j)
      if (j < nks) issue(st[j], w_b + j);
  }
#pragma unroll 1
  for (; done < nks; done += D) {
#pragma unroll
    for (int j = 0; j < D; ++j) {
      const int i = done + j;
      if (i < nks) {
        consume(st[j], w_b + i);
        if (i + D < nks) {
            issue(st[j], w_b + i + D);
        }
      }
    }
  }

  // ------------------------------------------------------------------------------ epilogue
  // Reduction slab: red[wave][row 0..15][RED_RS floats]; column position of real column
  // (h, w, half, c) is 72h + 16w + 8half + c.  With RED_RS = 148 (= 4 mod 16) the 64 lanes of one
  // store hit 64 distinct banks: c + 8h + 16*(row/4).
  float* red = (float*)smem;
  const int t = threadIdx.x;
  const int fr = t >> 5;            // 0..15: tile row handled in the final phase
  const int fc4 = (t & 31) * 4;     // first of 4 consecutive columns inside the column pair
  const int fpos = fc4 + (fc4 >= 64 ? 8 : 0);
  const int ncol = cp * 128 + fc4;  // real column
  const bool fcol_ok = ncol < p.N;
  const bool single = p.splits == 1;
  float* my_part = p.ctmp + ((int64_t)tile * p.splits + split) * (BM * 128);

  auto finalize = [&](int r, f32x4 v) {
    const int crow = s_crow[r];
    if (crow < 0 || !fcol_ok) return;
    if (GM == GM_CHANNEL) {
      const int base = ncol & ~31, cl = ncol & 31;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint16_t sv = Sc[base + single_perm_pos(cl + j)];
        v[j] *= (DT == DT_F16) ? f16_lo_f32(sv) : bf16_lo_f32(sv);
      }
    }
    if (bias) {
      const int base = ncol & ~31, cl = ncol & 31;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint16_t bv = bias[base + single_perm_pos(cl + j)];
        v[j] += (DT == DT_F16) ? f16_lo_f32(bv) : bf16_lo_f32(bv);
      }
    }
    if (p.mul_topk) {
      const float tw = p.topk_w[crow];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] *= tw;
    }
    u32x2 o;
    if constexpr (DT == DT_F16)
      o = u32x2{pack_f16(v[0], v[1]), pack_f16(v[2], v[3])};
    else
      o = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
    *(u32x2*)((uint16_t*)p.C + (int64_t)crow * p.N + ncol) = o;
  };

#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    if (mb) __syncthreads();  // previous m-block's slab no longer read
    {
      float* mine = red + wv * (16 * RED_RS);
#pragma unroll
      for (int w = 0; w < 4; ++w)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            mine[(4 * g + r) * RED_RS + 72 * h + 16 * w + 8 * hf + c] = acc[mb][w][hf][r];
    }
    __syncthreads();
    f32x4 v = *(const f32x4*)(red + fr * RED_RS + fpos);
#pragma unroll
    for (int ww = 1; ww < NW; ++ww) v += *(const f32x4*)(red + ww * (16 * RED_RS) + fr * RED_RS + fpos);
    const int r = mb * 16 + fr;
    if (single)
      finalize(r, v);
    else if (s_crow[r] >= 0)
      store_coherent(my_part + r * 128 + fc4, v, p.fix_mode);
  }
  if (single) return;
  if (p.fix_mode == 10 || p.fix_mode == 13) return;

  // ---- cross-workgroup reduction: the last split to arrive sums all partials in split order.
  // The wait makes every partial of this workgroup complete before its arrival is counted.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (t == 0) {
    const int old = __hip_atomic_fetch_add(&p.locks[tile], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (old == p.splits - 1);
  }
  __syncthreads();
  if (!s_last) return;
  const float* parts = p.ctmp + (int64_t)tile * p.splits * (BM * 128);
#pragma unroll 1
  for (int r = fr; r < BM; r += 16) {
    if (s_crow[r] < 0) continue;
    f32x4 v = {0, 0, 0, 0};
    for (int s = 0; s < p.splits; ++s)
      v += load_coherent(parts + (int64_t)s * (BM * 128) + r * 128 + fc4, p.fix_mode);
    finalize(r, v);
  }
  if (t == 0) __hip_atomic_store(&p.locks[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------------------------ host side
typedef void (*skinny_fn)(const KParams);

template <int DT, int MB, bool PERM>
static skinny_fn pick_zp_gm(bool zp, int gm) {
  if (zp) {
    if (gm == GM_GROUPED) return skinny_kernel<DT, MB, true, GM_GROUPED, PERM>;
    if (gm == GM_CHANNEL) return skinny_kernel<DT, MB, true, GM_CHANNEL, PERM>;
    return nullptr;
  }
  if (gm == GM_GROUPED) return skinny_kernel<DT, MB, false, GM_GROUPED, PERM>;
  if (gm == GM_CHANNEL) {
    if constexpr (PERM) return nullptr; else return skinny_kernel<DT, MB, false, GM_CHANNEL, false>;
  }
  if constexpr (PERM) return skinny_kernel<DT, MB, false, GM_GIDX, true>; else return nullptr;
}

template <int DT, bool PERM>
static skinny_fn pick_mb(int mb, bool zp, int gm) {
  switch (mb) {
    case 1: return pick_zp_gm<DT, 1, PERM>(zp, gm);
    case 2: return pick_zp_gm<DT, 2, PERM>(zp, gm);
    default: return pick_zp_gm<DT, 4, PERM>(zp, gm);
  }
}

static skinny_fn pick_skinny(int dt, int mb, bool zp, int gm, bool perm) {
  if (perm) return dt == DT_F16 ? pick_mb<DT_F16, true>(mb, zp, gm) : pick_mb<DT_BF16, true>(mb, zp, gm);
  return dt == DT_F16 ? pick_mb<DT_F16, false>(mb, zp, gm) : pick_mb<DT_BF16, false>(mb, zp, gm);
}

static int skinny_smem_bytes(int mb) {
  return mb == 1 ? SkinnyCfg<1>::SMEM : mb == 2 ? SkinnyCfg<2>::SMEM : SkinnyCfg<4>::SMEM;
}

int launch_skinny(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream) {
  const bool zp = a->b_zeros != nullptr;
  skinny_fn fn = pick_skinny(a->dtype, pl.mb, zp, pl.gm, pl.use_perm);
  if (!fn) return fail(W4A16_EINVAL, "unsupported kernel variant");
  const bool moe = (a->flags & W4A16_F_MOE) != 0;
  KParams p{};
  p.A = a->a;
  p.lda = a->lda;
  p.C = a->c;
  p.B = a->b_q_weight;
  p.S = a->b_scales;
  p.Z = a->b_zeros;
  p.gidx = pl.gm == GM_GIDX ? a->g_idx : nullptr;
  p.perm = pl.use_perm ? a->perm : nullptr;
  p.bias = a->b_bias;
  p.ctmp = a->c_tmp;
  p.locks = a->workspace;
  p.M = (int)a->size_m;
  p.c_rows = (int)(moe ? a->size_m * a->top_k : a->size_m);
  p.N = (int)a->size_n;
  p.K = (int)a->size_k;
  p.group_ksteps = pl.group_ksteps;
  p.ncp = pl.ncp;
  p.splits = pl.splits;
  p.ksteps_per_split = pl.kps;
  p.total_ksteps = pl.total_ksteps;
  p.xcd_map = pl.xcd_map;
  {
    static const char* fm = getenv("W4A16_FIXMODE");
    p.fix_mode = fm ? atoi(fm) : 2;
  }
  p.sorted_ids = a->sorted_token_ids;
  p.expert_ids = a->expert_ids;
  p.ntpp = a->num_tokens_past_padded;
  p.topk_w = a->topk_weights;
  p.moe = moe;
  p.moe_bs = a->moe_block_size;
  p.top_k = moe ? a->top_k : 1;
  p.mul_topk = moe && (a->flags & W4A16_F_MUL_TOPK_WEIGHTS);
  p.b_estride = (a->size_k / 16) * (2 * a->size_n);
  p.s_estride = a->num_groups * a->size_n;
  p.z_estride = a->num_groups * (a->size_n / 8);
  p.k_estride = a->size_k;
  p.n_estride = a->size_n;
  const int smem = skinny_smem_bytes(pl.mb);
  if (smem > 64 * 1024) {
    // more than 64 KiB of dynamic LDS has to be allowed per kernel function; do it once per function
    static const void* allowed[64];
    static int n_allowed = 0;
    bool seen = false;
    for (int i = 0; i < n_allowed; ++i) seen |= allowed[i] == (const void*)fn;
    if (!seen) {
      W4A16_HIP(hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, smem));
      if (n_allowed < 64) allowed[n_allowed++] = (const void*)fn;
    }
  }
  const int64_t grid = (int64_t)pl.tiles * pl.splits;
  if (grid <= 0) return 0;
  hipLaunchKernelGGL(fn, dim3((unsigned)grid), dim3(NW * 64), smem, stream, p);
  W4A16_HIP(hipGetLastError());
  return 0;
}

}  // namespace w4a16
