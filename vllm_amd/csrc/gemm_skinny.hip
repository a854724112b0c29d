// W4A16 (and W8A16, uint8b128) "skinny" GEMM for gfx950: C[M,N] = A[M,K] * dequant(Bq)[K,N] (+bias), dense or fused-MoE.
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
//     activations  global -> registers, 16 bytes per lane (coalesced rows), bounced through a
//                  wavefront-private LDS slab into the MFMA A operand order (no barrier needed)
//     scales/zeros one 16-byte / 4-byte load per k-step (cache hits after the first of a group)
//   The 8 partial tiles are summed through LDS.  Splits are summed by the last workgroup to arrive
//   at the tile's counter in `workspace`, in split order (deterministic); arrivals are wrapping increments, so
//   the workspace is all-zero on exit, as the reference requires (csrc/torch_bindings.cpp:255-267).
// HBM traffic per launch: every weight byte once (K*N/2), scales (K/g)*N*2, C once; A is re-read
// once per column pair (from L2), split partials move 2 * splits * M * N * 4 bytes.
#include <stdlib.h>

#include <mutex>
#include <type_traits>

#include "gemm_kernels.h"

namespace w4a16 {

// Wavefronts per workgroup (template parameter NW): 8; one-m-block tiles also come with 4, for launches with more
// workgroups than compute units, where two 4-wavefront workgroups share a compute unit and each one's prologue and
// epilogue run under the other's weight stream.

template <int MB>
struct SkinnyCfg {
  // k-steps in flight per wavefront (measured: deeper rings on the taller tiles cost registers, hence spills, and time)
  static constexpr int D = (MB >= 4) ? 2 : (MB == 2) ? 4 : 6;
  static constexpr int smem(int nw) { return nw * 16 * RED_RS * 4; }  // reduction slab; its head doubles as the A bounce slabs
};


// FP4: 0 = integer weights, 1 = float4_e2m1f with NVFP4 scales (per k-tile), 2 = with MXFP4 scales (per k-step)
template <int DT, int MB, bool ZP, int GM, int BITS = 4, bool ZPF = false, bool FP8 = false, int FP4 = 0, int NW = 8>
__global__ __launch_bounds__(NW * 64, 2) void skinny_kernel(const KParams p) {
  static_assert(NW == 8 || (NW == 4 && MB == 1), "4-wavefront workgroups: one-m-block tiles only");
  static_assert(BITS == 4 || (BITS == 8 && !ZP), "8-bit weights are uint8b128 (no zero points)");
  // ZPF: fp16 zero points laid out like the scales (HQQ); element-wise dequantisation on every tile size
  static_assert(FP4 == 0 || (BITS == 4 && !ZP && !ZPF && GM == GM_GROUPED), "fp4 weights: grouped scale records");
  static_assert(!FP8 || (BITS == 8 && GM != GM_GIDX), "fp8 weights use the 8-bit layout, no act-order");
  static_assert(!ZPF || (DT == DT_F16 && !ZP && GM == GM_GROUPED && BITS == 4), "float zero points: fp16 uint4 grouped");
  constexpr int BM = 16 * MB;
  // 8-bit stages hold twice the weight registers: shorter ring
  // ... and so do the variants that keep extra per-stage state (per-row scale lookup, fp4 scale records)
  constexpr int D = (BITS == 8) ? (MB >= 4 ? 2 : 3) : ((FP4 != 0 || GM == GM_GIDX) && MB >= 2) ? 2 : SkinnyCfg<MB>::D;
  constexpr bool UNIT = (GM == GM_CHANNEL);
  // Decode tiles (one m-block) keep the weights as raw magic numbers E+q in the MFMA and apply
  // "-(E+z)" and the group scale to the fp32 accumulator once per group (see fold() below).
  constexpr bool FOLD = (MB == 1) && (GM != GM_GIDX) && (BITS == 4) && !ZPF && FP4 == 0;
  constexpr bool HI_TRICK = FOLD && (DT == DT_F16) && !ZP;
  // fp4 codes converted straight to the 16-bit type (A reordered to the resulting K order); NVFP4 with bf16 has no
  // packed multiply for the scale mantissa and stays on the fp32 route
  constexpr bool FP4_DIRECT = (FP4 == 2) || (FP4 == 1 && DT == DT_F16);
  // fp8 likewise, where the scale can follow as a packed fp16 multiply or is applied to the accumulator (channel-wise)
  constexpr bool FP8_DIRECT = FP8 && (DT == DT_F16 || GM == GM_CHANNEL);
  constexpr bool A_PAIR_ORDER = FP4_DIRECT || FP8_DIRECT;  // A fragments in the K order (k0, k0+8, k0+1, k0+9, ...)
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int s_crow[BM];  // C row of each tile row, -1 = not written
  __shared__ float s_tw[BM];  // MoE: routing weight of each tile row
  __shared__ int s_last;

  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 7, h = (lane >> 3) & 1, g = lane >> 4;
  const int am = lane >> 2;  // activation row (inside an m-block) this lane loads
  const int ap = lane & 3;   // ... and which 16-byte piece of the k-step's 64 bytes

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
  zero_fill_side_job(p);

  const uint32_t* Bq = p.B;
  const uint16_t* Sc = (const uint16_t*)p.S;
  const uint32_t* Zp = p.Z;
  const int32_t* gidx = p.gidx;
  const uint16_t* bias = (const uint16_t*)p.bias;
  const uint16_t* gscale = (const uint16_t*)p.gscale;
  // MoE: slot ids of tile rows 0, 16 mb + am and (threadIdx.x % BM) (clamped into the block; checked against the block
  // size below), the block's expert and the number of live slots, all loaded together: one round trip, not several in a
  // row, before the workgroup can address its weights and activations
  const int tr = threadIdx.x < BM ? threadIdx.x : 0;
  int id_0 = 0, id_t = 0, id_a[MB], moe_e = 0, moe_ntp = 0;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) id_a[mb] = 0;
  if (p.moe) {
    // (the last block of the grid may reach past the end of sorted_ids, whose length need not be a multiple of the block
    //  size; such a block is never live, and its loads are clamped onto the array's last element)
    const int first = mt * p.moe_bs, last = p.moe_bs - 1, end = p.n_sorted - 1;
    id_0 = p.sorted_ids[min(first, end)];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) id_a[mb] = p.sorted_ids[min(first + min(mb * 16 + am, last), end)];
    id_t = p.sorted_ids[min(first + min(tr, last), end)];
    moe_ntp = *p.ntpp;
    moe_e = p.expert_ids[mt];
  }

  // ---- which A row feeds each tile row, which C row it is written to.  Rows past the end of the
  // problem read the tile's first row (always valid) so that LDS never holds uninitialised data;
  // their results are never stored.  id: the row's slot id (MoE).
  auto tile_row_ids = [&](int r, int id, int& src, int& dst) {
    src = -1;
    dst = -1;
    if (p.moe) {
      if (r < p.moe_bs && (unsigned)id < (unsigned)p.c_rows) {
        src = p.a_by_slot ? mt * p.moe_bs + r : id / p.top_k;
        dst = id;
      }
    } else {
      const int gr = mt * BM + r;
      if (gr < p.M) src = dst = gr;
    }
  };
  const uint16_t* arow[MB];
  {
    int src0, dst0;
    tile_row_ids(0, id_0, src0, dst0);
    if (src0 < 0) src0 = 0;  // a block whose first slot is padding still reads inside A
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      int src, dst;
      tile_row_ids(mb * 16 + am, id_a[mb], src, dst);
      arow[mb] = (const uint16_t*)p.A + (int64_t)(src >= 0 ? src : src0) * p.lda + ap * 8;
    }
  }
  if (threadIdx.x < BM) {
    int src, dst;
    tile_row_ids(tr, id_t, src, dst);
    s_crow[tr] = dst;
    if (p.mul_topk) s_tw[tr] = dst >= 0 ? p.topk_w[dst] : 0.f;
  }
  if (p.moe) {
    if (mt * p.moe_bs >= moe_ntp || moe_e < 0) return;
    Bq += moe_e * p.b_estride;
    Sc += moe_e * p.s_estride;
    if (FP4 == 1) gscale += moe_e;
    if (ZP) Zp += moe_e * p.z_estride;
    if (gidx) gidx += moe_e * p.k_estride;
    if (bias) bias += moe_e * p.n_estride;
  }

  // ---- this wavefront's k-steps
  const int ks_b = split * p.ksteps_per_split;
  const int ks_e = min(ks_b + p.ksteps_per_split, p.total_ksteps);
  const int per = (ks_e - ks_b + NW - 1) / NW;
  const int w_b = min(ks_b + wv * per, ks_e), w_e = min(w_b + per, ks_e);
  const int nks = w_e - w_b;

  // lanes of an n-tile past the end of N (odd number of n-tiles) read n-tile 0; their columns are never stored
  // (fused SiLU-and-mul: the tile pairs gate n-tile cp with the up n-tile of the same output columns, N/128 + cp)
  const int nt = p.act ? (h ? (p.N >> 7) + cp : cp) : ((2 * cp + h) * 64 < p.N ? 2 * cp + h : 0);
  // 4-bit: 32 u32x4 per n-tile and k-tile, one per Marlin thread; 8-bit: 64, two per thread (words 2w + half)
  const int64_t b_row = (BITS == 4) ? (p.N >> 1) : p.N;  // u32x4 per k-tile row
  const u32x4* bp = (const u32x4*)Bq + nt * (8 * BITS) + (4 * c + g) * (BITS / 4);
  const int64_t s_row = p.N >> 3;  // u32x4 (8 scales) per scale row; also words per zero-point row
  const u32x4* sp = (const u32x4*)Sc + nt * 8 + c;
  const uint32_t* zp = ZP ? Zp + nt * 8 + c : nullptr;
  const u32x4* zfp = ZPF ? (const u32x4*)Zp + nt * 8 + c : nullptr;  // fp16 zero points: indexed like the scales

  // Activations: lane (row am = l>>2, piece ap = l&3) loads the 16 bytes A[row][32ks + 8ap .. +8), so one
  // 16-lane pass of the load covers 4 rows x 64 contiguous bytes.  The MFMA lane (row m = l&15, g = l>>4)
  // needs K pairs 8s+2g, s = 0..3, i.e. dword g of pieces 0..3 of row m: the 1 KiB is bounced through a
  // wavefront-private LDS slab laid out [row][piece][dword] with an 80-byte row stride (conflict-free:
  // bank = 20*row + 4*piece + dword).  LDS ops of one wavefront execute in order, so no barrier is needed.
  constexpr int A_ROW = 20;  // dwords per row (16 + 4 pad)
  uint32_t* slab = (uint32_t*)smem + wv * (MB * 16 * A_ROW);
  uint32_t* slab_wr = slab + am * A_ROW + ap * 4;
  const uint32_t* slab_rd = slab + (lane & 15) * A_ROW + g;
  struct Stage {
    u32x4 b0, b1, sc;
    u32x4 b0h, b1h;  // 8-bit weights only: second half of the thread's words (w = 2, 3)
    u32x4 zf;        // float zero points only
    u32x4 a[MB];
    uint32_t zq;
    int gi;
    bool uni;
  };
  Stage st[D];

  auto issue = [&](Stage& s, int ks) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      s.a[mb] = *(const u32x4*)(arow[mb] + ks * 32);
    }
    int gi = 0;
    s.uni = true;
    if (GM == GM_GROUPED) gi = ks / p.group_ksteps;
    // channel-wise scales on the fold path: fold every 128 K rows all the same, so that the raw partial sums (biased
    // by E * sum(a)) stay small next to fp32's 24 bits whatever the activations' mean
    if (FOLD && GM == GM_CHANNEL) gi = ks >> 2;
    if (GM == GM_GIDX) {
      gi = gidx[ks * 32];
      s.uni = (gidx[ks * 32 + 31] == gi);
    }
    s.gi = gi;
    if (GM != GM_CHANNEL) s.sc = sp[(int64_t)gi * s_row];
    if (ZP) s.zq = zp[(int64_t)(GM == GM_CHANNEL ? 0 : gi) * s_row];
    if (ZPF) s.zf = zfp[(int64_t)gi * s_row];
    if (FP4 == 2) s.zq = ks & 1;  // which half of the two-k-step scale record
    s.b0 = __builtin_nontemporal_load(bp + (int64_t)(2 * ks) * b_row);
    s.b1 = __builtin_nontemporal_load(bp + (int64_t)(2 * ks + 1) * b_row);
    if constexpr (BITS == 8) {
      s.b0h = __builtin_nontemporal_load(bp + (int64_t)(2 * ks) * b_row + 1);
      s.b1h = __builtin_nontemporal_load(bp + (int64_t)(2 * ks + 1) * b_row + 1);
    }
  };
  // B operands (column half 0 / 1) of Marlin word position w of a stage; unit: leave the scale out
  auto dequant_word = [&](const Stage& s, auto w_tag, auto unit_tag, u32x4& o0, u32x4& o1) {
    constexpr int w = decltype(w_tag)::value;
    constexpr bool unit = decltype(unit_tag)::value;
    if constexpr (FP4 == 1 && FP4_DIRECT) {
      const uint32_t ba = fp4_scale_bytes(s.sc[0], s.sc[1], w), bb = fp4_scale_bytes(s.sc[2], s.sc[3], w);
      dequant_pair_nvfp4_f16_direct(s.b0[w], s.b1[w], ba, bb, o0, o1);
    } else if constexpr (FP4 == 2 && FP4_DIRECT) {
      const uint32_t bs = s.zq ? fp4_scale_bytes(s.sc[2], s.sc[3], w) : fp4_scale_bytes(s.sc[0], s.sc[1], w);
      dequant_pair_mxfp4_direct<DT>(s.b0[w], s.b1[w], mxfp4_scale_f32(bs & 0xff), mxfp4_scale_f32(bs >> 16), o0, o1);
    } else if constexpr (FP4 == 1) {
      const uint32_t ba = fp4_scale_bytes(s.sc[0], s.sc[1], w), bb = fp4_scale_bytes(s.sc[2], s.sc[3], w);
      dequant_pair_fp4<DT>(s.b0[w], s.b1[w], nvfp4_scale_f32(ba & 0xff), nvfp4_scale_f32(ba >> 16),
                           nvfp4_scale_f32(bb & 0xff), nvfp4_scale_f32(bb >> 16), o0, o1);
    } else if constexpr (FP4 == 2) {
      const uint32_t bs = s.zq ? fp4_scale_bytes(s.sc[2], s.sc[3], w) : fp4_scale_bytes(s.sc[0], s.sc[1], w);
      const float s0 = mxfp4_scale_f32(bs & 0xff), s1 = mxfp4_scale_f32(bs >> 16);
      dequant_pair_fp4<DT>(s.b0[w], s.b1[w], s0, s1, s0, s1, o0, o1);
    } else if constexpr (ZPF) {
      const uint32_t zs = as_u32(as_h2(s.zf[w]) * as_h2(s.sc[w]));
      dequant_pair_zpf(s.b0[w], s.b1[w], s.sc[w], zs, o0, o1);
    } else if constexpr (BITS == 4) {
      uint32_t z0 = 8, z1 = 8;
      if (ZP) {
        z0 = (s.zq >> (4 * w)) & 0xf;
        z1 = (s.zq >> (4 * w + 16)) & 0xf;
      }
      const ColConst<DT> cc = make_col_const<DT, unit>(unit ? 0u : s.sc[w], z0, z1);
      dequant_pair<DT, unit>(s.b0[w], s.b1[w], cc, o0, o1);
    } else {
      const u32x4& la = (w < 2) ? s.b0 : s.b0h;
      const u32x4& lb = (w < 2) ? s.b1 : s.b1h;
      if constexpr (FP8_DIRECT)
        dequant_pair8_fp8_direct<DT, unit>(la[2 * (w & 1)], la[2 * (w & 1) + 1], lb[2 * (w & 1)], lb[2 * (w & 1) + 1],
                                           unit ? 0u : s.sc[w], o0, o1);
      else if constexpr (FP8)
        dequant_pair8_fp8<DT, unit>(la[2 * (w & 1)], la[2 * (w & 1) + 1], lb[2 * (w & 1)], lb[2 * (w & 1) + 1],
                                    unit ? 0u : s.sc[w], o0, o1);
      else
        dequant_pair8<DT, unit>(la[2 * (w & 1)], la[2 * (w & 1) + 1], lb[2 * (w & 1)], lb[2 * (w & 1) + 1],
                                unit ? 0u : s.sc[w], o0, o1);
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

  // ---- fold scheme state (FOLD only): tmp = sum_k a_k (E + q_k) over the k-steps of the current group,
  // rs = sum_k a_k * v_k, the matching bias term (v = E + 8 for uint4b8 in the HI_TRICK form, else 1).
  f32x4 tmp[4][2];
  f32x4 rs = {0, 0, 0, 0};
  int cur_gi = -1;
  bool fresh = true;
  u32x4 cur_sc = {0, 0, 0, 0};
  uint32_t cur_zq = 0;
  // acc += s * (tmp - (E + z) * rs)   [HI_TRICK: acc += s * (tmp - rs)]
  auto fold = [&]() {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float s0 = 1.0f, s1 = 1.0f;
      if (GM != GM_CHANNEL) {
        s0 = (DT == DT_F16) ? f16_lo_f32(cur_sc[w]) : bf16_lo_f32(cur_sc[w]);
        s1 = (DT == DT_F16) ? f16_hi_f32(cur_sc[w]) : bf16_hi_f32(cur_sc[w]);
      }
      float e0 = 1.0f, e1 = 1.0f;
      if constexpr (!HI_TRICK) {
        const float E = (DT == DT_F16) ? 1024.0f : 128.0f;
        e0 = E + (ZP ? (float)((cur_zq >> (4 * w)) & 0xf) : 8.0f);
        e1 = E + (ZP ? (float)((cur_zq >> (4 * w + 16)) & 0xf) : 8.0f);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float d0 = __builtin_fmaf(-e0, rs[r], tmp[w][0][r]);
        const float d1 = __builtin_fmaf(-e1, rs[r], tmp[w][1][r]);
        acc[0][w][0][r] = __builtin_fmaf(s0, d0, acc[0][w][0][r]);
        acc[0][w][1][r] = __builtin_fmaf(s1, d1, acc[0][w][1][r]);
      }
    }
  };

  auto consume = [&](const Stage& s, int ks) {
    u32x4 af[MB];
    {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) *(u32x4*)(slab_wr + mb * 16 * A_ROW) = s.a[mb];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const uint32_t* q = slab_rd + mb * 16 * A_ROW;
      af[mb] = u32x4{q[0], q[4], q[8], q[12]};
      if constexpr (A_PAIR_ORDER) af[mb] = a_frag_fp4_order(af[mb]);
    }
    }
    if constexpr (FOLD) {
      if (s.gi != cur_gi) {
        if (cur_gi >= 0) fold();
        cur_gi = s.gi;
        cur_sc = s.sc;
        cur_zq = s.zq;
        fresh = true;
      }
      u32x4 vb;  // B operand of the bias-term MFMA
      if constexpr (HI_TRICK) {
        vb = u32x4{RAW_BIAS_LO, RAW_BIAS_HI, RAW_BIAS_LO, RAW_BIAS_HI};
      } else {
        const uint32_t one = (DT == DT_F16) ? 0x3c003c00u : 0x3f803f80u;
        vb = u32x4{one, one, one, one};
      }
      u32x4 o[4][2];
#pragma unroll
      for (int w = 0; w < 4; ++w) raw_pair<DT, HI_TRICK>(s.b0[w], s.b1[w], o[w][0], o[w][1]);
      const f32x4 zero = {0, 0, 0, 0};
      if (fresh) {
        fresh = false;
        rs = mfma16x16x32<DT>(af[0], vb, zero);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          tmp[w][0] = mfma16x16x32<DT>(af[0], o[w][0], zero);
          tmp[w][1] = mfma16x16x32<DT>(af[0], o[w][1], zero);
        }
      } else {
        rs = mfma16x16x32<DT>(af[0], vb, rs);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          tmp[w][0] = mfma16x16x32<DT>(af[0], o[w][0], tmp[w][0]);
          tmp[w][1] = mfma16x16x32<DT>(af[0], o[w][1], tmp[w][1]);
        }
      }
      return;
    }
    if constexpr (GM == GM_GIDX) {
      // Per-row scale lookup.  A k-step inside one group dequantises with the stage's scale row like the grouped form;
      // one that crosses a group boundary dequantises without a scale and multiplies every operand register (two K rows
      // of one column) by its own scale pair, fetched as word w of the scale rows of the lane's eight K rows (eight 4-byte
      // loads per Marlin word, cache hits).  The two forms only differ in how the eight operand registers of a word are
      // made; the MFMAs follow the merge, so the 32 * MB accumulators are not merged from two branches.
      const int kb = ks * 32 + 2 * g;
      int64_t srow[8];
      if (!s.uni) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int kk = kb + (e & 1) + ((e >> 1) & 1) * 8 + (e >> 2) * 16;
          srow[e] = (int64_t)gidx[kk] * s_row;
        }
      }
      auto gidx_word = [&](auto w_tag) {
        constexpr int w = decltype(w_tag)::value;
        u32x4 r[2];
        if (s.uni) {
          dequant_word(s, w_tag, std::false_type{}, r[0], r[1]);
        } else {
          uint32_t se[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) se[e] = ((const uint32_t*)(sp + srow[e]))[w];
          u32x4 o[2];
          dequant_word(s, w_tag, std::true_type{}, o[0], o[1]);
#pragma unroll
          for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const uint32_t sa = (se[2 * q] >> (16 * hf)) & 0xffffu;
              const uint32_t sb = (se[2 * q + 1] >> (16 * hf)) & 0xffffu;
              const uint32_t spair = sa | (sb << 16);
              if constexpr (DT == DT_F16)
                r[hf][q] = as_u32(as_h2(o[hf][q]) * as_h2(spair));
              else
                r[hf][q] = pack_bf16(bf16_lo_f32(o[hf][q]) * bf16_lo_f32(spair),
                                     bf16_hi_f32(o[hf][q]) * bf16_hi_f32(spair));
            }
          }
        }
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) acc[mb][w][hf] = mfma16x16x32<DT>(af[mb], r[hf], acc[mb][w][hf]);
      };
      gidx_word(std::integral_constant<int, 0>{});
      gidx_word(std::integral_constant<int, 1>{});
      gidx_word(std::integral_constant<int, 2>{});
      gidx_word(std::integral_constant<int, 3>{});
      return;
    }
    auto plain_word = [&](auto w_tag) {
      constexpr int w = decltype(w_tag)::value;
      u32x4 o0, o1;
      dequant_word(s, w_tag, std::integral_constant<bool, UNIT>{}, o0, o1);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        acc[mb][w][0] = mfma16x16x32<DT>(af[mb], o0, acc[mb][w][0]);
        acc[mb][w][1] = mfma16x16x32<DT>(af[mb], o1, acc[mb][w][1]);
      }
    };
    plain_word(std::integral_constant<int, 0>{});
    plain_word(std::integral_constant<int, 1>{});
    plain_word(std::integral_constant<int, 2>{});
    plain_word(std::integral_constant<int, 3>{});
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

  if constexpr (FOLD) {
    if (cur_gi >= 0) fold();
  }

  // ------------------------------------------------------------------------------ epilogue
  // Reduction slab: red[wave][row 0..15][RED_RS floats]; column position of real column
  // (h, w, half, c) is 72h + 16w + 8half + c.  With RED_RS = 148 (= 4 mod 16) the 64 lanes of one
  // store hit 64 distinct banks: c + 8h + 16*(row/4).
  float* red = (float*)smem;
  const int t = threadIdx.x;
  constexpr int RPP = NW * 2;       // tile rows per pass of the final phase (32 threads per row)
  const int fr0 = t >> 5;           // 0..RPP-1: tile row handled in the first pass
  const int fc4 = (t & 31) * 4;     // first of 4 consecutive columns inside the column pair
  const int fpos = fc4 + (fc4 >= 64 ? 8 : 0);
  const int ncol = cp * 128 + fc4;  // real column
  const bool fcol_ok = ncol < p.N;
  const bool single = p.splits == 1;
  float* my_part = p.ctmp + ((int64_t)tile * p.splits + split) * (BM * 128);

  // channel scale (times the global scale) and bias of four finished columns starting at real column `col`; read once,
  // in front of the m-block loop (inside it every load would wait behind the stores of the rows before)
  struct ColConsts { f32x4 sc, bo; };
  auto col_consts = [&](int col) {
    ColConsts cc{f32x4{1.f, 1.f, 1.f, 1.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
    const int base = col & ~31, cl = col & 31;
    if (GM == GM_CHANNEL) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint16_t sv = Sc[base + single_perm_pos(cl + j)];
        cc.sc[j] = ((DT == DT_F16) ? f16_lo_f32(sv) : bf16_lo_f32(sv)) * (FP8 ? fp8_scale_unbias<DT>() : 1.0f);
      }
    }
    if (bias) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint16_t bv = bias[base + single_perm_pos(cl + j)];
        cc.bo[j] = (DT == DT_F16) ? f16_lo_f32(bv) : bf16_lo_f32(bv);
      }
    }
    return cc;
  };
  float gs = 1.0f;
  if constexpr (FP4 == 1) {
    // NVFP4 global scale: stored times 2^7 (fp16) / 2^119 (bf16) by the reference's load-time processing
    const uint16_t gv = *gscale;
    gs = (DT == DT_F16) ? f16_lo_f32(gv) * 0x1.0p-7f : bf16_lo_f32(gv) * 0x1.0p-119f;
  }
  // ... applied, with the row's routing weight, to finished values
  auto finish = [&](f32x4 v, const ColConsts& cc, int r) {
    if (GM == GM_CHANNEL) {
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] *= cc.sc[j];
    }
    if constexpr (FP4 == 1) {
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] *= gs;
    }
    if (bias) {
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] += cc.bo[j];
    }
    if (p.mul_topk) {
      const float tw = s_tw[r];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] *= tw;
    }
    return v;
  };
  // v: the thread's four columns; u (fused SiLU-and-mul, threads of the gate half only): the up half's same columns
  const bool act_lane = p.act && fc4 < 64;
  ColConsts ccv{f32x4{1.f, 1.f, 1.f, 1.f}, f32x4{0.f, 0.f, 0.f, 0.f}}, ccu = ccv;
  if (p.act) {
    if (act_lane) {
      ccv = col_consts(cp * 64 + fc4);
      ccu = col_consts((p.N >> 1) + cp * 64 + fc4);
    }
  } else if (fcol_ok) {
    ccv = col_consts(ncol);
  }
  auto finalize = [&](int r, f32x4 v, f32x4 u) {
    const int crow = s_crow[r];
    if (crow < 0) return;
    if (p.act) {
      if (!act_lane) return;
      store_row4_silu_mul<DT>(p, crow, cp * 64 + fc4, finish(v, ccv, r), finish(u, ccu, r));
    } else if (fcol_ok) {
      store_row4<DT>(p, crow, ncol, finish(v, ccv, r));
    }
  };

#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    __syncthreads();  // A bounce slabs / previous m-block's slab no longer read
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
    for (int ps = 0; ps < 16 / RPP; ++ps) {
      const int fr = fr0 + ps * RPP;
      f32x4 v = *(const f32x4*)(red + fr * RED_RS + fpos);
#pragma unroll
      for (int ww = 1; ww < NW; ++ww) v += *(const f32x4*)(red + ww * (16 * RED_RS) + fr * RED_RS + fpos);
      const int r = mb * 16 + fr;
      if (single) {
        f32x4 u = {0, 0, 0, 0};
        if (act_lane) {
#pragma unroll
          for (int ww = 0; ww < NW; ++ww) u += *(const f32x4*)(red + ww * (16 * RED_RS) + fr * RED_RS + fpos + 72);
        }
        finalize(r, v, u);
      } else if (s_crow[r] >= 0) {
        store_coherent(my_part + r * 128 + fc4, v);
      }
    }
  }
  if (single) return;

  // ---- cross-workgroup reduction: the last split to arrive sums all partials in split order.
  // The wait makes every partial of this workgroup complete before its arrival is counted.
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (t == 0) s_last = arrive_last(p.locks + tile * p.lock_stride, p.splits);
  __syncthreads();
  if (!s_last) return;
  const float* parts = p.ctmp + (int64_t)tile * p.splits * (BM * 128);
  auto sum_parts = [&](int r, int col4) {
    f32x4 v = {0, 0, 0, 0};
    // four splits' loads are in flight together; summed in split order
    for (int s0 = 0; s0 < p.splits; s0 += 4) {
      f32x4 a[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a[i] = load_coherent(parts + (int64_t)min(s0 + i, p.splits - 1) * (BM * 128) + r * 128 + col4);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (s0 + i < p.splits) v += a[i];
    }
    return v;
  };
#pragma unroll 1
  for (int r = fr0; r < BM; r += RPP) {
    if (s_crow[r] < 0) continue;
    const f32x4 v = sum_parts(r, fc4);
    f32x4 u = {0, 0, 0, 0};
    if (act_lane) u = sum_parts(r, fc4 + 64);
    finalize(r, v, u);
  }
}

// ------------------------------------------------------------------------------------ host side
typedef void (*skinny_fn)(const KParams);

template <int DT, int MB, int NW = 8>
static skinny_fn pick_zp_gm(bool zp, int gm) {
  if (zp) {
    if (gm == GM_GROUPED) return skinny_kernel<DT, MB, true, GM_GROUPED, 4, false, false, 0, NW>;
    if (gm == GM_CHANNEL) return skinny_kernel<DT, MB, true, GM_CHANNEL, 4, false, false, 0, NW>;
    return nullptr;
  }
  if (gm == GM_GROUPED) return skinny_kernel<DT, MB, false, GM_GROUPED, 4, false, false, 0, NW>;
  if (gm == GM_CHANNEL) return skinny_kernel<DT, MB, false, GM_CHANNEL, 4, false, false, 0, NW>;
  return skinny_kernel<DT, MB, false, GM_GIDX, 4, false, false, 0, NW>;
}

// (nw = 4 exists for one-m-block tiles only; the planner asks for it nowhere else)
template <int DT>
static skinny_fn pick_mb(int mb, int nw, bool zp, int gm) {
  switch (mb) {
    case 1: return nw == 4 ? pick_zp_gm<DT, 1, 4>(zp, gm) : pick_zp_gm<DT, 1>(zp, gm);
    case 2: return pick_zp_gm<DT, 2>(zp, gm);
    default: return pick_zp_gm<DT, 4>(zp, gm);
  }
}

template <int DT, int MB, int NW = 8>
static skinny_fn pick_w8_gm(int gm) {  // uint8b128: no zero points
  return gm == GM_GROUPED ? skinny_kernel<DT, MB, false, GM_GROUPED, 8, false, false, 0, NW>
         : gm == GM_CHANNEL ? skinny_kernel<DT, MB, false, GM_CHANNEL, 8, false, false, 0, NW>
                            : skinny_kernel<DT, MB, false, GM_GIDX, 8, false, false, 0, NW>;
}

template <int DT>
static skinny_fn pick_w8(int mb, int nw, int gm) {
  return mb == 1 ? (nw == 4 ? pick_w8_gm<DT, 1, 4>(gm) : pick_w8_gm<DT, 1>(gm))
         : mb == 2 ? pick_w8_gm<DT, 2>(gm) : pick_w8_gm<DT, 4>(gm);
}

// (act-order never reaches a kernel as such: the host gathers A's columns in front of the launch, see gemm.hip)
static skinny_fn pick_skinny(int dt, int mb, int nw, bool zp, int gm, bool w8) {
  if (w8) {
    if (zp) return nullptr;
    return dt == DT_F16 ? pick_w8<DT_F16>(mb, nw, gm) : pick_w8<DT_BF16>(mb, nw, gm);
  }
  return dt == DT_F16 ? pick_mb<DT_F16>(mb, nw, zp, gm) : pick_mb<DT_BF16>(mb, nw, zp, gm);
}

static int skinny_smem_bytes(int mb, int nw) {
  return mb == 1 ? SkinnyCfg<1>::smem(nw) : mb == 2 ? SkinnyCfg<2>::smem(nw) : SkinnyCfg<4>::smem(nw);
}

template <int DT>
static skinny_fn pick_fp8(int mb, int nw, int gm) {  // float8_e4m3fn: grouped or channel-wise scales, no act-order
  switch (mb) {
    case 1:
      if (nw == 4)
        return gm == GM_GROUPED ? skinny_kernel<DT, 1, false, GM_GROUPED, 8, false, true, 0, 4>
                                : skinny_kernel<DT, 1, false, GM_CHANNEL, 8, false, true, 0, 4>;
      return gm == GM_GROUPED ? skinny_kernel<DT, 1, false, GM_GROUPED, 8, false, true>
                              : skinny_kernel<DT, 1, false, GM_CHANNEL, 8, false, true>;
    case 2:
      return gm == GM_GROUPED ? skinny_kernel<DT, 2, false, GM_GROUPED, 8, false, true>
                              : skinny_kernel<DT, 2, false, GM_CHANNEL, 8, false, true>;
    default:
      return gm == GM_GROUPED ? skinny_kernel<DT, 4, false, GM_GROUPED, 8, false, true>
                              : skinny_kernel<DT, 4, false, GM_CHANNEL, 8, false, true>;
  }
}

template <int DT, int FP4>
static skinny_fn pick_fp4(int mb, int nw) {  // float4_e2m1f (validated on the host: grouped records, no act-order)
  switch (mb) {
    case 1:
      return nw == 4 ? skinny_kernel<DT, 1, false, GM_GROUPED, 4, false, false, FP4, 4>
                     : skinny_kernel<DT, 1, false, GM_GROUPED, 4, false, false, FP4>;
    case 2: return skinny_kernel<DT, 2, false, GM_GROUPED, 4, false, false, FP4>;
    default: return skinny_kernel<DT, 4, false, GM_GROUPED, 4, false, false, FP4>;
  }
}

static skinny_fn pick_zpf(int mb, int nw) {  // fp16 zero points (validated on the host: fp16, uint4, grouped, no act-order)
  switch (mb) {
    case 1:
      return nw == 4 ? skinny_kernel<DT_F16, 1, false, GM_GROUPED, 4, true, false, 0, 4>
                     : skinny_kernel<DT_F16, 1, false, GM_GROUPED, 4, true>;
    case 2: return skinny_kernel<DT_F16, 2, false, GM_GROUPED, 4, true>;
    default: return skinny_kernel<DT_F16, 4, false, GM_GROUPED, 4, true>;
  }
}

int launch_skinny(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream) {
  const bool zp = a->b_zeros != nullptr;
  const int nw = (pl.nw == 4 && pl.mb == 1) ? 4 : 8;
  skinny_fn fn;
  if (a->flags & W4A16_F_ZP_FLOAT)
    fn = pick_zpf(pl.mb, nw);
  else if (a->wtype == W4A16_WTYPE_FE2M1)
    fn = a->global_scale ? (a->dtype == DT_F16 ? pick_fp4<DT_F16, 1>(pl.mb, nw) : pick_fp4<DT_BF16, 1>(pl.mb, nw))
                         : pick_fp4<DT_BF16, 2>(pl.mb, nw);
  else if (a->wtype == W4A16_WTYPE_FE4M3)
    fn = pl.gm == GM_GIDX     ? nullptr
         : a->dtype == DT_F16 ? pick_fp8<DT_F16>(pl.mb, nw, pl.gm)
                              : pick_fp8<DT_BF16>(pl.mb, nw, pl.gm);
  else
    fn = pick_skinny(a->dtype, pl.mb, nw, zp, pl.gm, a->wtype == W4A16_WTYPE_U8B128);
  if (!fn || pl.use_perm) return fail(W4A16_EINVAL, "unsupported kernel variant");
  KParams p = make_kparams(a, pl);
  const int smem = skinny_smem_bytes(pl.mb, nw);
  W4A16_HIP(allow_dynamic_lds((const void*)fn, smem));
  const int64_t grid = (int64_t)pl.tiles * pl.splits;
  if (grid <= 0) return 0;
  hipLaunchKernelGGL(fn, dim3((unsigned)grid), dim3(nw * 64), smem, stream, p);
  W4A16_HIP(hipGetLastError());
  return 0;
}

}  // namespace w4a16
