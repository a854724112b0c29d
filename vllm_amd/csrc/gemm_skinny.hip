// W4A16 "skinny" GEMM for gfx950: C[M,N] = A[M,K] * dequant(Bq)[K,N] (+bias), dense or fused-MoE.
//
// Stands in for the reference's Marlin<> kernel (csrc/quantization/gptq_marlin/marlin_template.h:273-1804)
// and its MoE twin (csrc/moe/marlin_moe_wna16/marlin_template.h:298-2009); written from scratch for
// wave64 + MFMA, see gemm_common.h for how a wavefront reads the Marlin layout.
//
// Work decomposition
//   tile  = (m-tile of BM = 16*MB rows) x (column pair = 128 columns)
//   split = contiguous range of k-steps (32 K-rows each) of that tile
//   one workgroup (4 wavefronts) per (tile, split); the 4 wavefronts share the tile's columns
//   and rows and cut the split's k-steps into 4 contiguous quarters, so no wavefront ever waits
//   on another inside the main loop: weights stream global -> registers (128-bit, 1 KiB contiguous
//   per wavefront instruction), activations are staged per wavefront in a private LDS slab.
//   The quarters are summed through LDS; splits are summed through an fp32 scratch (c_tmp) by the
//   last workgroup to arrive at the tile's counter in `workspace` (ordered sum => deterministic;
//   the counter is reset so the workspace is all-zero on exit, as the reference requires,
//   csrc/torch_bindings.cpp:255-267).
// HBM traffic per launch: every weight byte once (K*N/2), scales (K/g)*N*2, A re-read once per
// column pair from L2, C once, plus 2 * splits * M * N * 4 bytes of L2-resident partials.
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
  // MoE
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* ntpp;
  const float* topk_w;
  int moe, moe_bs, top_k, mul_topk;
  int64_t b_estride, s_estride, z_estride, k_estride, n_estride;  // per-expert strides (elements)
};

constexpr int RED_RS = 148;  // row stride (floats) of the reduction slab; see epilogue

template <int MB>
struct SkinnyCfg {
  static constexpr int CH = (MB >= 4) ? 2 : 4;  // k-steps staged per wavefront per chunk
  static constexpr int STAGE_BYTES = 4 * CH * MB * 1024;
  static constexpr int RED_BYTES = 4 * 16 * RED_RS * 4;
  static constexpr int SMEM = STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES;
};

template <int DT, int MB, bool ZP, int GM>
__global__ __launch_bounds__(256) void skinny_kernel(const KParams p) {
  constexpr int BM = 16 * MB;
  constexpr int CH = SkinnyCfg<MB>::CH;
  constexpr bool UNIT = (GM == GM_CHANNEL);
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int s_crow[BM];  // C row of each tile row, -1 = not written
  __shared__ int s_last;

  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int c = lane & 7, h = (lane >> 3) & 1, g = lane >> 4;

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
    if (perm) perm += e * p.k_estride;
    if (bias) bias += e * p.n_estride;
  }

  // ---- which A row feeds each staged row; which C row each tile row is written to
  // staging lane layout: row ms = lane >> 2 of the m-block, 16-byte piece pc = lane & 3 of the k-step
  const int ms = lane >> 2, pc = lane & 3;
  const uint16_t* arow[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int r = mb * 16 + ms;
    int64_t src = -1;
    if (p.moe) {
      if (r < p.moe_bs) {
        const int id = p.sorted_ids[mt * p.moe_bs + r];
        if (id < p.c_rows) src = id / p.top_k;
      }
    } else {
      const int gr = mt * BM + r;
      if (gr < p.M) src = gr;
    }
    arow[mb] = src >= 0 ? (const uint16_t*)p.A + src * p.lda : nullptr;
  }
  if (threadIdx.x < BM) {
    const int r = threadIdx.x;
    int crow = -1;
    if (p.moe) {
      if (r < p.moe_bs) {
        const int id = p.sorted_ids[mt * p.moe_bs + r];
        if (id < p.c_rows) crow = id;
      }
    } else {
      const int gr = mt * BM + r;
      if (gr < p.M) crow = gr;
    }
    s_crow[r] = crow;
  }

  // ---- this wavefront's k-steps
  const int ks_b = split * p.ksteps_per_split;
  const int ks_e = min(ks_b + p.ksteps_per_split, p.total_ksteps);
  const int per = (ks_e - ks_b + 3) >> 2;
  const int w_b = min(ks_b + wv * per, ks_e), w_e = min(w_b + per, ks_e);

  const bool col_ok = (2 * cp + h) * 64 < p.N;
  const int64_t b_row = p.N >> 1;  // u32x4 per k-tile row
  const u32x4* bp = (const u32x4*)Bq + (2 * cp + h) * 32 + (4 * c + g);
  const int64_t s_row = p.N >> 3;  // u32x4 (8 scales) per scale row; also words per zero-point row
  const u32x4* sp = (const u32x4*)Sc + (2 * cp + h) * 8 + c;
  const uint32_t* zp = ZP ? Zp + (2 * cp + h) * 8 + c : nullptr;

  u32x4* stage = (u32x4*)smem + wv * (CH * MB * 64);

  struct Chunk {
    u32x4 bq[CH][2];
    u32x4 sc[CH];
    uint32_t zq[CH];
    u32x4 av[CH][MB];
    int gi[CH];
    bool uni[CH];
  };

  auto load_chunk = [&](Chunk& ck, int ks0) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int ks = ks0 + i;
      const bool on = ks < w_e;
      // weights
      if (on && col_ok) {
        ck.bq[i][0] = __builtin_nontemporal_load(bp + (int64_t)(2 * ks) * b_row);
        ck.bq[i][1] = __builtin_nontemporal_load(bp + (int64_t)(2 * ks + 1) * b_row);
      } else {
        ck.bq[i][0] = u32x4{0, 0, 0, 0};
        ck.bq[i][1] = u32x4{0, 0, 0, 0};
      }
      // scales / zero points of the k-step's group
      int gi = 0;
      ck.uni[i] = true;
      if (GM == GM_GROUPED) gi = on ? ks / p.group_ksteps : 0;
      if (GM == GM_GIDX && on) {
        gi = gidx[ks * 32];
        ck.uni[i] = (gidx[ks * 32 + 31] == gi);
      }
      ck.gi[i] = gi;
      if (GM != GM_CHANNEL) ck.sc[i] = col_ok ? sp[(int64_t)gi * s_row] : u32x4{0, 0, 0, 0};
      if (ZP) ck.zq[i] = col_ok ? zp[(int64_t)gi * s_row] : 0u;
      // activations: 16 bytes = 8 consecutive K of one row
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        u32x4 v = {0, 0, 0, 0};
        if (on && arow[mb]) {
          const int k8 = ks * 32 + pc * 8;
          if (perm) {
            uint16_t e[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) e[j] = arow[mb][perm[k8 + j]];
            v = u32x4{(uint32_t)e[0] | ((uint32_t)e[1] << 16), (uint32_t)e[2] | ((uint32_t)e[3] << 16),
                      (uint32_t)e[4] | ((uint32_t)e[5] << 16), (uint32_t)e[6] | ((uint32_t)e[7] << 16)};
          } else {
            v = *(const u32x4*)(arow[mb] + k8);
          }
        }
        ck.av[i][mb] = v;
      }
    }
  };

  // LDS slab of one wavefront: [k-step i][m-block][g][m][4 dwords]; lane (ms, pc) owns K pairs
  // (8pc+2q, 8pc+2q+1), q = 0..3, which belong to K-group g = q, dword slot pc.
  auto stage_chunk = [&](const Chunk& ck) {
    uint32_t* sl = (uint32_t*)stage;
#pragma unroll
    for (int i = 0; i < CH; ++i)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int base = ((i * MB + mb) * 64) * 4;
        sl[base + (0 * 16 + ms) * 4 + pc] = ck.av[i][mb].x;
        sl[base + (1 * 16 + ms) * 4 + pc] = ck.av[i][mb].y;
        sl[base + (2 * 16 + ms) * 4 + pc] = ck.av[i][mb].z;
        sl[base + (3 * 16 + ms) * 4 + pc] = ck.av[i][mb].w;
      }
  };

  f32x4 acc[MB][4][2];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      acc[mb][w][0] = f32x4{0, 0, 0, 0};
      acc[mb][w][1] = f32x4{0, 0, 0, 0};
    }

  auto compute_chunk = [&](const Chunk& ck, int ks0) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      if (ks0 + i >= w_e) break;
      u32x4 af[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) af[mb] = stage[(i * MB + mb) * 64 + lane];

      if (GM == GM_GIDX && !ck.uni[i]) {
        // group boundary inside the k-step: fetch the scale row of every K-row separately
        const int kb = (ks0 + i) * 32 + 2 * g;
        u32x4 se[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int kk = kb + (e & 1) + ((e >> 1) & 1) * 8 + (e >> 2) * 16;
          se[e] = col_ok ? sp[(int64_t)gidx[kk] * s_row] : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const ColConst<DT> cc = make_col_const<DT, true>(0, 8, 8);
          u32x4 o[2];
          dequant_pair<DT, true>(ck.bq[i][0][w], ck.bq[i][1][w], cc, o[0], o[1]);
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
        continue;
      }

#pragma unroll
      for (int w = 0; w < 4; ++w) {
        uint32_t z0 = 8, z1 = 8;
        if (ZP) {
          z0 = (ck.zq[i] >> (4 * w)) & 0xf;
          z1 = (ck.zq[i] >> (4 * w + 16)) & 0xf;
        }
        const ColConst<DT> cc = make_col_const<DT, UNIT>(GM == GM_CHANNEL ? 0u : ck.sc[i][w], z0, z1);
        u32x4 o0, o1;
        dequant_pair<DT, UNIT>(ck.bq[i][0][w], ck.bq[i][1][w], cc, o0, o1);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          acc[mb][w][0] = mfma16x16x32<DT>(af[mb], o0, acc[mb][w][0]);
          acc[mb][w][1] = mfma16x16x32<DT>(af[mb], o1, acc[mb][w][1]);
        }
      }
    }
  };

  if (w_b < w_e) {
    Chunk cur;
    load_chunk(cur, w_b);
    for (int ks0 = w_b; ks0 < w_e; ks0 += CH) {
      stage_chunk(cur);
      __builtin_amdgcn_wave_barrier();
      Chunk nxt;
      const bool more = ks0 + CH < w_e;
      if (more) load_chunk(nxt, ks0 + CH);
      compute_chunk(cur, ks0);
      __builtin_amdgcn_wave_barrier();
      if (more) cur = nxt;
    }
  }

  // ------------------------------------------------------------------------------ epilogue
  // Reduction slab: red[wave][row 0..15][RED_RS floats]; column position of real column
  // (h, w, half, c) is 72h + 16w + 8half + c.  With RED_RS = 148 (= 4 mod 16) the 64 lanes of one
  // store hit 64 distinct banks: c + 8h + 16*(row/4).
  float* red = (float*)smem;
  const int t = threadIdx.x;
  const int fr = t >> 5;               // 0..7: row (and row + 8) handled in the final phase
  const int fc4 = (t & 31) * 4;        // first of 4 consecutive columns inside the column pair
  const int fpos = fc4 + (fc4 >= 64 ? 8 : 0);
  const int ncol = cp * 128 + fc4;     // real column
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
    __syncthreads();  // staging slabs / previous m-block's slab no longer read
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
#pragma unroll
    for (int half_rows = 0; half_rows < 2; ++half_rows) {
      const int r16 = fr + 8 * half_rows;
      f32x4 v = *(const f32x4*)(red + r16 * RED_RS + fpos);
#pragma unroll
      for (int ww = 1; ww < 4; ++ww) v += *(const f32x4*)(red + ww * (16 * RED_RS) + r16 * RED_RS + fpos);
      const int r = mb * 16 + r16;
      if (single)
        finalize(r, v);
      else
        *(f32x4*)(my_part + r * 128 + fc4) = v;
    }
  }
  if (single) return;

  // ---- cross-workgroup reduction: the last split to arrive sums all partials in split order
  __threadfence();
  __syncthreads();
  if (t == 0) {
    const int old = __hip_atomic_fetch_add(&p.locks[tile], 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (old == p.splits - 1);
  }
  __syncthreads();
  if (!s_last) return;
  __threadfence();
  const float* parts = p.ctmp + (int64_t)tile * p.splits * (BM * 128);
#pragma unroll 1
  for (int r = fr; r < BM; r += 8) {
    if (s_crow[r] < 0) continue;
    f32x4 v = {0, 0, 0, 0};
    for (int s = 0; s < p.splits; ++s)
      v += __builtin_nontemporal_load((const f32x4*)(parts + (int64_t)s * (BM * 128) + r * 128 + fc4));
    finalize(r, v);
  }
  if (t == 0) __hip_atomic_store(&p.locks[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------------------------ host side
typedef void (*skinny_fn)(const KParams);

template <int DT, int MB>
static skinny_fn pick_zp_gm(bool zp, int gm) {
  if (zp) {
    if (gm == GM_GROUPED) return skinny_kernel<DT, MB, true, GM_GROUPED>;
    if (gm == GM_CHANNEL) return skinny_kernel<DT, MB, true, GM_CHANNEL>;
    return nullptr;
  }
  if (gm == GM_GROUPED) return skinny_kernel<DT, MB, false, GM_GROUPED>;
  if (gm == GM_CHANNEL) return skinny_kernel<DT, MB, false, GM_CHANNEL>;
  return skinny_kernel<DT, MB, false, GM_GIDX>;
}

template <int DT>
static skinny_fn pick_mb(int mb, bool zp, int gm) {
  switch (mb) {
    case 1: return pick_zp_gm<DT, 1>(zp, gm);
    case 2: return pick_zp_gm<DT, 2>(zp, gm);
    default: return pick_zp_gm<DT, 4>(zp, gm);
  }
}

static skinny_fn pick_skinny(int dt, int mb, bool zp, int gm) {
  return dt == DT_F16 ? pick_mb<DT_F16>(mb, zp, gm) : pick_mb<DT_BF16>(mb, zp, gm);
}

static int skinny_smem_bytes(int mb) {
  return mb == 1 ? SkinnyCfg<1>::SMEM : mb == 2 ? SkinnyCfg<2>::SMEM : SkinnyCfg<4>::SMEM;
}

int launch_skinny(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream) {
  const bool zp = a->b_zeros != nullptr;
  skinny_fn fn = pick_skinny(a->dtype, pl.mb, zp, pl.gm);
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
  const int64_t grid = (int64_t)pl.tiles * pl.splits;
  if (grid <= 0) return 0;
  hipLaunchKernelGGL(fn, dim3((unsigned)grid), dim3(256), smem, stream, p);
  W4A16_HIP(hipGetLastError());
  return 0;
}

}  // namespace w4a16
