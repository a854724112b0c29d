// W4A16 decode GEMM for gfx950 (M-tiles of 16 rows): C[M,N] = A[M,K] * dequant(Bq)[K,N] (+bias).
//
// Specialisation of the skinny kernel for the weight-streaming regime, where the kernel is bound by HBM
// and by fixed latencies rather than by the matrix cores.  Same operand layouts and the same workgroup
// decomposition (tile x split, 8 wavefronts cutting the split's K range into contiguous parts, LDS sum,
// ordered cross-workgroup sum), with these differences:
//   * tile width TN = 128 columns (a column pair, 128-bit loads) or 64 columns (one n-tile, 64-bit loads);
//     narrow tiles give twice as many workgroups, so small-N layers can cover enough compute units without
//     splitting K across workgroups (a cross-workgroup sum costs ~4 us of dependent device-scope round trips).
//   * a pipeline stage is two k-steps (64 K rows): 4 weight loads, 2 activation loads that read 128
//     contiguous bytes per row (full cache lines), one scale load, one zero-point load.
//   * "fold" arithmetic: nibbles are only OR-ed into the mantissa of a magic exponent (fp16: 1024+q or, for
//     the high nibbles, which stay at bits 4..7, 64+q; bf16: 128+q) and fed to the MFMA as
//     they are; one extra MFMA per k-step against a constant operand accumulates the bias term
//     sum_k a_k * (E+8)  [or sum_k a_k when zero points vary per column].  Once per quantization group the fp32
//     partial is folded:  acc += s * (tmp - (E+z) * rs).  Exact integer dequantisation happens in fp32, the
//     scale is applied once per group in fp32; a one-hot activation row still reproduces half(q-z)*half(s)
//     rounded once, bit for bit.  ~45 VALU instructions per k-step instead of ~135.
// Requirements (checked on the host, which otherwise falls back to the skinny kernel): K % 64 == 0,
// group size a multiple of 64 (or channel-wise), no per-row g_idx lookup.
#include "gemm_kernels.h"

namespace w4a16 {

// Wavefronts per workgroup: 8, or 4 when a launch has several workgroups per compute unit in turn: two 4-wavefront
// workgroups share a compute unit (same registers and loads in flight as one of 8), so one's prologue and
// epilogue latencies run under the other's weight stream.
// Stages (of two k-steps) in flight per wavefront.  Two: with three to five the kernel is slower on every layer of the
// decode step (a wavefront's loads are consumed in order, the eight wavefronts of a workgroup already keep ~64 KB per
// compute unit in flight, and every further stage costs 20-29 registers and lengthens the prologue); with one, 64-column
// tiles lose a few per cent.
constexpr int DD = 2;

template <int TN>
struct DecodeCfg {
  static constexpr int RS = (TN == 128) ? RED_RS : 84;  // reduction slab row stride (floats), 4 mod 16
  static constexpr int smem(int nw) { return nw * 16 * RS * 4; }
};

// MOE: the launch walks MoE blocks (slot ids, expert ids, fused epilogues); the dense instantiations carry none of that
// code, which shortens the chain of argument loads in front of a small layer's first weight load
// The leading scalar arguments repeat fields of `p`: the file is compiled with kernel-argument preloading, which hands
// the first 14 dwords of the argument block to a wavefront in SGPRs when it starts.  Everything in front of the first
// weight and activation loads (tile and K range of the workgroup, the operands' addresses) is computed from those
// registers alone, so a small layer's first loads do not wait for a fetch of the argument block from memory (a round
// trip as long as the weight load itself when the launch comes from a graph and the block is cold).
//   eNcpX: column tiles, bit 30 set for the XCD-aware grid; eKpsG: k-steps per split, (group_shift + 1) << 24
template <int DT, bool ZP, bool CHANNEL, int TN, int DNW, bool MOE>
__global__ __launch_bounds__(DNW * 64, 2) void decode_kernel(const uint32_t* eB, const void* eA, const void* eS,
                                                             int64_t eLda, int eN, int eKpsG, int eTotal, int eTiles,
                                                             int eNcpX, int eM, const KParams p) {
  const int eNcp = eNcpX & 0x3fffffff;
  const bool eXcd = (eNcpX >> 30) & 1;
  const int eKps = eKpsG & 0xffffff, eGroupShift = (eKpsG >> 24) - 1;
  constexpr int W = TN / 32;  // Marlin words per lane and k-tile: 4 (128-bit load) or 2 (64-bit load)
  constexpr bool HI_TRICK = (DT == DT_F16) && !ZP;
  constexpr int RS = DecodeCfg<TN>::RS;
  using bvec = uint32_t __attribute__((ext_vector_type(W)));
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int s_crow[16];
  __shared__ float s_tw[16];  // MoE: routing weight of each tile row
  __shared__ int s_last;

  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // weight-side roles: c = column inside an 8-column block, h = which half of the tile's columns, g = K group
  const int c = lane & 7, h = (lane >> 3) & 1, g = lane >> 4;

  // The grid is three-dimensional so that (tile, split) come from the block indices without an integer division (a
  // small layer's first weight load waits for every instruction in front of it); workgroups are dispatched x fastest:
  //   plain:   x = split, y + 65535 z = tile                       (the splits of a tile are neighbours)
  //   xcd_map: x = tile % 8, y = split, z = tile / 8               (consecutive workgroups go round the eight XCDs, so
  //            all splits of a tile share one XCD's L2)
  // (every workgroup of the grid takes its share of the side job, also one that has no tile)
  if constexpr (MOE)
    zero_fill_side_job(p, (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x, gridDim.x * gridDim.y * gridDim.z);
  int tile, split;
  if (eXcd) {
    tile = blockIdx.z * 8 + blockIdx.x;
    split = blockIdx.y;
  } else {
    tile = blockIdx.z * 65535 + blockIdx.y;
    split = blockIdx.x;
    if (tile >= eTiles) return;
  }
  int ct = tile, mt = 0;  // column tile, m-tile
  if (eNcp != eTiles) {
    ct = tile % eNcp;
    mt = tile / eNcp;
  }

  const uint32_t* Bq = eB;
  const uint16_t* Sc = (const uint16_t*)eS;
  const uint32_t* Zp = p.Z;
  const uint16_t* bias = (const uint16_t*)p.bias;
  // activation loads: lane -> row (lane >> 3) [+ 8 for the second load], 16-byte piece (lane & 7) of the
  // stage's 128 bytes.  Rows past the end of the problem read the tile's first row; never stored.
  const int ar = lane >> 3, ap = lane & 7;
  const int tr = threadIdx.x & 15;
  // MoE: slot ids of tile rows 0, ar, ar + 8 and tr (clamped into the block; checked against the block size below), the
  // block's expert and the number of live slots, all loaded together: a workgroup then waits for one round trip, not
  // five in a row, before it can address its weights and activations (short-K expert GEMMs live only a few of them)
  int id_0 = 0, id_a0 = 0, id_a1 = 0, id_t = 0, moe_e = 0, moe_ntp = 0;
  if constexpr (MOE) {
    // (the last block of the grid may reach past the end of sorted_ids, whose length need not be a multiple of the block
    //  size; such a block is never live, and its loads are clamped onto the array's last element)
    const int first = mt * p.moe_bs, last = p.moe_bs - 1, end = p.n_sorted - 1;
    id_0 = p.sorted_ids[min(first, end)];
    id_a0 = p.sorted_ids[min(first + min(ar, last), end)];
    id_a1 = p.sorted_ids[min(first + min(ar + 8, last), end)];
    id_t = p.sorted_ids[min(first + min(tr, last), end)];
    moe_ntp = *p.ntpp;
    moe_e = p.expert_ids[mt];
  }
  // which A row feeds tile row r and which C row receives it (-1: none); id: the row's slot id (MoE)
  auto tile_row_ids = [&](int r, int id, int& src, int& dst) {
    src = -1;
    dst = -1;
    if constexpr (MOE) {
      if (r < p.moe_bs && (unsigned)id < (unsigned)p.c_rows) {
        src = p.a_by_slot ? mt * p.moe_bs + r : id / p.top_k;
        dst = id;
      }
    } else {
      const int gr = mt * 16 + r;
      if (gr < eM) src = dst = gr;
    }
  };
  const uint16_t* arow[2];
  {
    int src0, dst0;
    tile_row_ids(0, id_0, src0, dst0);
    if (src0 < 0) src0 = 0;  // a block whose first slot is padding still reads inside A
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      int src, dst;
      tile_row_ids(ar + 8 * i, i ? id_a1 : id_a0, src, dst);
      arow[i] = (const uint16_t*)eA + (int64_t)(src >= 0 ? src : src0) * eLda + ap * 8;
    }
  }
  if (threadIdx.x < 16) {
    int src, dst;
    tile_row_ids(tr, id_t, src, dst);
    s_crow[tr] = dst;
    if (MOE && p.mul_topk) s_tw[tr] = dst >= 0 ? p.topk_w[dst] : 0.f;
  }
  if constexpr (MOE) {
    if (mt * p.moe_bs >= moe_ntp || moe_e < 0) return;
    Bq += moe_e * p.b_estride;
    Sc += moe_e * p.s_estride;
    if (ZP) Zp += moe_e * p.z_estride;
    if (bias) bias += moe_e * p.n_estride;
  }

  // ---- this wavefront's stages (pairs of k-steps)
  const int st_b = split * eKps / 2;
  const int st_e = min(st_b + eKps / 2, eTotal / 2);
  const int per = (st_e - st_b + DNW - 1) / DNW;
  const int w_b = min(st_b + wv * per, st_e), w_e = min(w_b + per, st_e);
  const int nst = w_e - w_b;

  // n-tile this lane reads (TN=128: 2ct+h, TN=64: ct); a missing second n-tile (N/64 odd) aliases n-tile 0
  int nt;
  if (TN == 128)  // (fused SiLU-and-mul: gate n-tile ct paired with the up n-tile of the same output columns)
    nt = (MOE && p.act) ? (h ? (eN >> 7) + ct : ct) : ((2 * ct + h) * 64 < eN ? 2 * ct + h : 0);
  else
    nt = ct;
  const int64_t b_row = (int64_t)eN * 2;  // words per k-tile row
  // TN=128: words th*4 .. +4 of the n-tile, th = 4c+g.  TN=64: words th*4 + 2h .. +2.
  const uint32_t* bnext = Bq + (int64_t)nt * 128 + (4 * c + g) * 4 + (TN == 64 ? 2 * h : 0) + (int64_t)(4 * w_b) * b_row;
  // scales of the lane's columns: permuted position 8c + j, j = 2w + half; TN=64 covers w = 2h, 2h+1 only
  const uint16_t* sp = Sc + (int64_t)nt * 64 + 8 * c + (TN == 64 ? 4 * h : 0);
  const uint32_t* zp = ZP ? Zp + nt * 8 + c : nullptr;

  // wavefront-private LDS slab for the A bounce: [row 16][36 dwords]: 32 dwords = 8 pieces x 4, +4 pad
  // (bank = 36*row + 4*piece + dword is conflict-free for the reads below).
  constexpr int A_ROW = 36;
  uint32_t* slab = (uint32_t*)smem + wv * (16 * A_ROW);
  uint32_t* slab_wr = slab + ar * A_ROW + ap * 4;
  const uint32_t* slab_rd = slab + (lane & 15) * A_ROW + g;

  // rows 8..15 of the tile exist?  (otherwise their activation loads are skipped)
  const bool rows_hi = MOE ? (p.moe_bs > 8) : (mt * 16 + 8 < eM);
  // scale group of an absolute stage index (channel-wise scales: pseudo-groups of 128 K rows, so that the raw partial
  // sums, biased by E * sum(a), stay small next to fp32's 24 bits whatever the activations' mean)
  // (grouped scales: the host only picks this kernel for power-of-two groups of at least one stage)
  auto group_of = [&](int sidx) { return CHANNEL ? (sidx >> 1) : ((2 * sidx) >> eGroupShift); };
  const int gmask = CHANNEL ? 1 : (((1 << eGroupShift) - 1) >> 1);  // stage index bits inside a group
  struct Stage {
    bvec b[4];   // k-tiles 4s .. 4s+3
    u32x4 a[2];  // rows ar, ar+8
    bvec sc;     // scales (pairs half0|half1 per word)
    uint32_t zq;
    int gi;
  };
  Stage st[DD];

  auto issue = [&](Stage& s, int sidx) {  // sidx: absolute stage index (2 k-steps = 4 k-tiles = 64 K rows)
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (i == 1 && !rows_hi) {
        s.a[i] = u32x4{0, 0, 0, 0};  // the tile has no rows 8..15
      } else {
        s.a[i] = *(const u32x4*)(arow[i] + sidx * 64);
      }
    }
    const int gi = group_of(sidx);
    s.gi = gi;
    if (sidx == w_b || (sidx & gmask) == 0) {  // uniform: only the first stage of a group carries its scales
      if (!CHANNEL) s.sc = *(const bvec*)(sp + (int64_t)gi * eN);
      if (ZP) s.zq = zp[(int64_t)(CHANNEL ? 0 : gi) * (eN >> 3)];
    }
    const uint32_t* q = bnext;  // (stages are issued in order: a running pointer instead of a 64-bit product per stage)
    bnext += 4 * b_row;
#pragma unroll
    for (int t = 0; t < 4; ++t) s.b[t] = __builtin_nontemporal_load((const bvec*)(q + t * b_row));
  };

  f32x4 acc[W][2], tmp[W][2];
  f32x4 rs = {0, 0, 0, 0};
#pragma unroll
  for (int w = 0; w < W; ++w) {
    acc[w][0] = f32x4{0, 0, 0, 0};
    acc[w][1] = f32x4{0, 0, 0, 0};
    tmp[w][0] = f32x4{0, 0, 0, 0};
    tmp[w][1] = f32x4{0, 0, 0, 0};
  }
  int cur_gi = -1;
  bool fresh = true;
  bvec cur_sc;
  uint32_t cur_zq = 0;
#pragma unroll
  for (int w = 0; w < W; ++w) cur_sc[w] = 0;

  // acc += s * (tmp - e * rs),  e = E + z  (HI_TRICK: the bias operand already carries E + 8, e = 1)
  auto fold = [&]() {
#pragma unroll
    for (int w = 0; w < W; ++w) {
      float s0 = 1.0f, s1 = 1.0f;
      if (!CHANNEL) {
        const uint32_t sw = cur_sc[w];
        s0 = (DT == DT_F16) ? f16_lo_f32(sw) : bf16_lo_f32(sw);
        s1 = (DT == DT_F16) ? f16_hi_f32(sw) : bf16_hi_f32(sw);
      }
      float e0 = 1.0f, e1 = 1.0f;
      if constexpr (!HI_TRICK) {
        const float E = (DT == DT_F16) ? 1024.0f : 128.0f;
        const int wa = (TN == 64) ? 2 * h + w : w;  // absolute word index of the n-tile
        e0 = E + (ZP ? (float)((cur_zq >> (4 * wa)) & 0xf) : 8.0f);
        e1 = E + (ZP ? (float)((cur_zq >> (4 * wa + 16)) & 0xf) : 8.0f);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float d0 = __builtin_fmaf(-e0, rs[r], tmp[w][0][r]);
        const float d1 = __builtin_fmaf(-e1, rs[r], tmp[w][1][r]);
        acc[w][0][r] = __builtin_fmaf(s0, d0, acc[w][0][r]);
        acc[w][1][r] = __builtin_fmaf(s1, d1, acc[w][1][r]);
      }
    }
  };

  auto consume = [&](const Stage& s) {
    if (s.gi != cur_gi) {
      if (cur_gi >= 0) fold();
      cur_gi = s.gi;
      cur_sc = s.sc;
      cur_zq = s.zq;
      fresh = true;
    }
    // A bounce: natural [row][128 B] layout in, MFMA operand (row m, K pairs 8s+2g) out
    *(u32x4*)slab_wr = s.a[0];
    *(u32x4*)(slab_wr + 8 * A_ROW) = s.a[1];
    u32x4 af[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const uint32_t* q = slab_rd + kk * 16;
      af[kk] = u32x4{q[0], q[4], q[8], q[12]};
    }
    u32x4 vb;  // B operand of the bias-term MFMA
    if constexpr (HI_TRICK) {
      vb = u32x4{RAW_BIAS_LO, RAW_BIAS_HI, RAW_BIAS_LO, RAW_BIAS_HI};
    } else {
      const uint32_t one = (DT == DT_F16) ? 0x3c003c00u : 0x3f803f80u;
      vb = u32x4{one, one, one, one};
    }
    const f32x4 zero = {0, 0, 0, 0};
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      u32x4 o[W][2];
#pragma unroll
      for (int w = 0; w < W; ++w) raw_pair<DT, HI_TRICK>(s.b[2 * kk][w], s.b[2 * kk + 1][w], o[w][0], o[w][1]);
      if (kk == 0 && fresh) {
        rs = mfma16x16x32<DT>(af[kk], vb, zero);
#pragma unroll
        for (int w = 0; w < W; ++w) {
          tmp[w][0] = mfma16x16x32<DT>(af[kk], o[w][0], zero);
          tmp[w][1] = mfma16x16x32<DT>(af[kk], o[w][1], zero);
        }
      } else {
        rs = mfma16x16x32<DT>(af[kk], vb, rs);
#pragma unroll
        for (int w = 0; w < W; ++w) {
          tmp[w][0] = mfma16x16x32<DT>(af[kk], o[w][0], tmp[w][0]);
          tmp[w][1] = mfma16x16x32<DT>(af[kk], o[w][1], tmp[w][1]);
        }
      }
    }
    fresh = false;
  };

  // ---- software pipeline over stages (see the skinny kernel for why the scheduling barriers are there)
  int done = 0;
  if (nst >= DD) {
#pragma unroll
    for (int j = 0; j < DD; ++j) issue(st[j], w_b + j);
    for (; done + 2 * DD <= nst; done += DD) {
#pragma unroll
      for (int j = 0; j < DD; ++j) {
        consume(st[j]);
        __builtin_amdgcn_sched_barrier(0);
        issue(st[j], w_b + done + j + DD);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < DD; ++j)
      if (j < nst) issue(st[j], w_b + j);
  }
#pragma unroll 1
  for (; done < nst; done += DD) {
#pragma unroll
    for (int j = 0; j < DD; ++j) {
      const int i = done + j;
      if (i < nst) {
        consume(st[j]);
        __builtin_amdgcn_sched_barrier(0);
        if (i + DD < nst) issue(st[j], w_b + i + DD);
      }
    }
  }
  if (cur_gi >= 0) fold();

  // ------------------------------------------------------------------------------ epilogue
  // red[wave][row 16][RS floats]; column position inside the tile: TN=128: 72h + 16w + 8half + c
  // (real column 64h + 16w + 8half + c), TN=64: 40h + 16w + 8half + c (real column 32h + 16w + 8half + c).
  float* red = (float*)smem;
  const int t = threadIdx.x;
  constexpr int CPT = TN / 32;          // consecutive columns per thread in the final phase (4 or 2)
  constexpr int RPP = DNW * 2;          // tile rows per pass of the final phase (32 threads per row)
  constexpr int NP = 16 / RPP;          // passes: thread t has rows (t >> 5) + RPP * pass
  const int fr0 = t >> 5;
  const int fc = (t & 31) * CPT;        // first column inside the tile
  const int fpos = (TN == 128) ? fc + (fc >= 64 ? 8 : 0) : fc + (fc >= 32 ? 8 : 0);
  const int ncol = ct * TN + fc;
  const bool fcol_ok = ncol < eN;
  const bool single = p.splits == 1;
  float* my_part = p.ctmp + ((int64_t)tile * p.splits + split) * (16 * TN);

  // channel scale and bias of CPT finished columns starting at real column `col`; read once, in front of the barriers
  // below (inside the row passes every load would wait behind the stores of the pass before)
  auto col_consts = [&](int col, float* sc, float* bo) {
    const int base = col & ~31, cl = col & 31;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      sc[j] = 1.0f;
      bo[j] = 0.0f;
      if (CHANNEL) {
        const uint16_t sv = Sc[base + single_perm_pos(cl + j)];
        sc[j] = (DT == DT_F16) ? f16_lo_f32(sv) : bf16_lo_f32(sv);
      }
      if (bias) {
        const uint16_t bv = bias[base + single_perm_pos(cl + j)];
        bo[j] = (DT == DT_F16) ? f16_lo_f32(bv) : bf16_lo_f32(bv);
      }
    }
  };
  // ... applied, with the row's routing weight, to finished values
  auto finish = [&](float* v, const float* sc, const float* bo, int fr) {
    if (CHANNEL) {
#pragma unroll
      for (int j = 0; j < CPT; ++j) v[j] *= sc[j];
    }
    if (bias) {
#pragma unroll
      for (int j = 0; j < CPT; ++j) v[j] += bo[j];
    }
    if (MOE && p.mul_topk) {
      const float tw = s_tw[fr];
#pragma unroll
      for (int j = 0; j < CPT; ++j) v[j] *= tw;
    }
  };
  // fused SiLU-and-mul (TN = 128 only, host-checked): the threads of the gate half also take the up half's columns
  const bool act_lane = MOE && TN == 128 && p.act && fc < 64;
  float cs[CPT], bs[CPT], cu[CPT], bu[CPT];
#pragma unroll
  for (int j = 0; j < CPT; ++j) cs[j] = cu[j] = 1.0f, bs[j] = bu[j] = 0.0f;
  if (MOE && TN == 128 && p.act) {
    if (act_lane) {
      col_consts(ct * 64 + fc, cs, bs);
      col_consts((eN >> 1) + ct * 64 + fc, cu, bu);
    }
  } else if (fcol_ok) {
    col_consts(ncol, cs, bs);
  }
  auto finalize = [&](float* v, float* u, int fr) {
    const int crow = s_crow[fr];
    if (crow < 0) return;
    if constexpr (TN == 128) {
      if (MOE && p.act) {
        if (!act_lane) return;
        const int oc = ct * 64 + fc;
        finish(v, cs, bs, fr);
        finish(u, cu, bu, fr);
        store_row4_silu_mul<DT>(p, crow, oc, f32x4{v[0], v[1], v[2], v[3]}, f32x4{u[0], u[1], u[2], u[3]});
        return;
      }
    }
    if (!fcol_ok) return;
    finish(v, cs, bs, fr);
    if constexpr (CPT == 4) {
      store_row4<DT, MOE>(p, crow, ncol, f32x4{v[0], v[1], v[2], v[3]});
    } else {
      const uint32_t o = pack2<DT>(v[0], v[1]);
      if (MOE && p.sum_div > 0) {
        uint16_t* dst = (uint16_t*)p.C + (int64_t)(crow / p.sum_div) * eN + ncol;
        if constexpr (DT == DT_F16) {
          typedef _Float16 h2 __attribute__((ext_vector_type(2)));
          __builtin_amdgcn_global_atomic_fadd_v2f16((h2*)dst, __builtin_bit_cast(h2, o));
        } else {
          typedef short s2 __attribute__((ext_vector_type(2)));
          __builtin_amdgcn_global_atomic_fadd_v2bf16((s2*)dst, __builtin_bit_cast(s2, o));
        }
      } else {
        *(uint32_t*)((uint16_t*)p.C + (int64_t)crow * eN + ncol) = o;
      }
    }
  };

  __syncthreads();  // A bounce slabs no longer read
  {
    float* mine = red + wv * (16 * RS);
    constexpr int HS = (TN == 128) ? 72 : 40;
#pragma unroll
    for (int w = 0; w < W; ++w)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int r = 0; r < 4; ++r) mine[(4 * g + r) * RS + HS * h + 16 * w + 8 * hf + c] = acc[w][hf][r];
  }
  __syncthreads();
  float v[NP][CPT], u[NP][CPT];
#pragma unroll
  for (int ps = 0; ps < NP; ++ps) {
    const int fr = fr0 + RPP * ps;
#pragma unroll
    for (int j = 0; j < CPT; ++j) v[ps][j] = u[ps][j] = 0.0f;
#pragma unroll
    for (int ww = 0; ww < DNW; ++ww) {
      const float* src = red + ww * (16 * RS) + fr * RS + fpos;
#pragma unroll
      for (int j = 0; j < CPT; ++j) v[ps][j] += src[j];
    }
  }
  if (single) {
#pragma unroll
    for (int ps = 0; ps < NP; ++ps) {
      const int fr = fr0 + RPP * ps;
      if (act_lane) {
#pragma unroll
        for (int ww = 0; ww < DNW; ++ww) {
          const float* src = red + ww * (16 * RS) + fr * RS + fpos + 72;
#pragma unroll
          for (int j = 0; j < CPT; ++j) u[ps][j] += src[j];
        }
      }
      finalize(v[ps], u[ps], fr);
    }
    return;
  }
#pragma unroll
  for (int ps = 0; ps < NP; ++ps) {
    const int fr = fr0 + RPP * ps;
    if (s_crow[fr] >= 0) {
#pragma unroll
      for (int j = 0; j < CPT; j += 2) store_coherent2(my_part + fr * TN + fc + j, v[ps][j], v[ps][j + 1]);
    }
  }
  // ---- cross-workgroup reduction: the last split to arrive sums all partials in split order
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (t == 0) s_last = arrive_last(p.locks + tile * p.lock_stride, p.splits);
  __syncthreads();
  if (!s_last) return;
#pragma unroll
  for (int ps = 0; ps < NP; ++ps) {
    const int fr = fr0 + RPP * ps;
    if (s_crow[fr] < 0) continue;
    auto sum_parts = [&](float* out, int col) {
      const float* parts = p.ctmp + (int64_t)tile * p.splits * (16 * TN) + fr * TN + col;
#pragma unroll
      for (int j = 0; j < CPT; ++j) out[j] = 0.0f;
      // four splits' loads are in flight together (a loop of dependent round trips would cost ~0.3 us per split)
      for (int s0 = 0; s0 < p.splits; s0 += 4) {
        float a[4][CPT];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int s = min(s0 + i, p.splits - 1);
#pragma unroll
          for (int j = 0; j < CPT; j += 2) load_coherent2(parts + (int64_t)s * (16 * TN) + j, a[i][j], a[i][j + 1]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (s0 + i < p.splits) {
#pragma unroll
            for (int j = 0; j < CPT; ++j) out[j] += a[i][j];
          }
      }
    };
    sum_parts(v[ps], fc);
    if (act_lane) sum_parts(u[ps], fc + 64);
    finalize(v[ps], u[ps], fr);
  }
}

// ------------------------------------------------------------------------------------ host side
typedef void (*decode_fn)(const uint32_t*, const void*, const void*, int64_t, int, int, int, int, int, int, const KParams);

template <int DT, int TN, int NW, bool MOE>
static decode_fn pick5(bool zp, bool channel) {
  if (zp) return channel ? decode_kernel<DT, true, true, TN, NW, MOE> : decode_kernel<DT, true, false, TN, NW, MOE>;
  return channel ? decode_kernel<DT, false, true, TN, NW, MOE> : decode_kernel<DT, false, false, TN, NW, MOE>;
}
template <int DT, int TN, int NW>
static decode_fn pick4(bool moe, bool zp, bool channel) {
  return moe ? pick5<DT, TN, NW, true>(zp, channel) : pick5<DT, TN, NW, false>(zp, channel);
}
template <int DT, int TN>
static decode_fn pick3(int nw, bool moe, bool zp, bool channel) {
  return nw == 4 ? pick4<DT, TN, 4>(moe, zp, channel) : pick4<DT, TN, 8>(moe, zp, channel);
}
template <int DT>
static decode_fn pick2(int tn, int nw, bool moe, bool zp, bool channel) {
  return tn == 64 ? pick3<DT, 64>(nw, moe, zp, channel) : pick3<DT, 128>(nw, moe, zp, channel);
}

// (act-order never reaches the kernel as such: the host gathers A's columns in front of the launch, see gemm.hip)
static decode_fn pick_decode(int dt, int tn, int nw, bool moe, bool zp, bool channel) {
  return dt == DT_F16 ? pick2<DT_F16>(tn, nw, moe, zp, channel) : pick2<DT_BF16>(tn, nw, moe, zp, channel);
}

int launch_decode(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream) {
  const bool zp = a->b_zeros != nullptr;
  if (pl.use_perm) return fail(W4A16_EINVAL, "unsupported kernel variant");
  const int nw = pl.nw == 4 ? 4 : 8;
  decode_fn fn = pick_decode(a->dtype, pl.tn, nw, (a->flags & W4A16_F_MOE) != 0, zp, pl.gm == GM_CHANNEL);
  KParams p = make_kparams(a, pl);
  const int smem = pl.tn == 64 ? DecodeCfg<64>::smem(nw) : DecodeCfg<128>::smem(nw);
  W4A16_HIP(allow_dynamic_lds((const void*)fn, smem));
  if ((int64_t)pl.tiles * pl.splits <= 0) return 0;
  dim3 grid;
  if (pl.xcd_map) {
    if (pl.tiles % 8 != 0 || pl.tiles / 8 > 65535 || pl.splits > 65535) return fail(W4A16_EINVAL, "unsupported launch shape");
    grid = dim3(8, (unsigned)pl.splits, (unsigned)(pl.tiles / 8));
  } else {
    if (pl.splits > 65535) return fail(W4A16_EINVAL, "unsupported launch shape");
    const unsigned gy = pl.tiles < 65535 ? (unsigned)pl.tiles : 65535u;
    grid = dim3((unsigned)pl.splits, gy, (unsigned)((pl.tiles + 65534) / 65535));
  }
  hipLaunchKernelGGL(fn, grid, dim3(nw * 64), smem, stream, p.B, p.A, p.S, p.lda, p.N, p.ksteps_per_split | ((p.group_shift + 1) << 24), p.total_ksteps,
                     p.tiles, p.ncp | (p.xcd_map ? (1 << 30) : 0), p.M, p);
  W4A16_HIP(hipGetLastError());
  return 0;
}

}  // namespace w4a16
