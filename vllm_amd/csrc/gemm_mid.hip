// W4A16 GEMM for gfx950 with 64-row tiles: C[M,N] = A[M,K] * dequant(Bq)[K,N] (+bias), dense (64 < M, too few
// rows or tiles for the 128-row prefill kernel) and MoE blocks of 64 sorted token slots
// (the counterpart of the reference's thread_m_blocks = 4 configurations, csrc/moe/marlin_moe_wna16/ops.cu:451-512).
//
//   workgroup tile 64 rows x 512 columns, 4 wavefronts, each owning 64 rows x 128 columns (one column pair):
//   4 m-blocks x 8 MFMA column groups = 32 v_mfma_f32_16x16x32 per k-step, 128 fp32 accumulators per lane in
//   AGPRs and fewer than 128 VGPRs, so two workgroups share a compute unit (two wavefronts per SIMD): one
//   wavefront's dequantisation and waits run under the other's MFMAs.
//   weights      each wavefront streams its column pair global -> registers (128-bit loads, four k-steps in
//                flight) and dequantises each Marlin word right before its 8 MFMAs, one operand register per MFMA
//                (scale applied per element: the B operand equals the reference's half(q - z) * half(s)).
//   activations  the workgroup stages 64 rows x 64 K (two k-steps) into LDS, double buffered, in MFMA fragment
//                order (one conflict-free ds_read_b128 per operand); MoE rows are gathered through sorted_token_ids
//                while staging.  One barrier per two k-steps.
//   split-K      with too few tiles to fill the chip, K is cut into splits of whole loop iterations (multiples of
//                128 K rows); each workgroup writes its fp32 partial tile to scratch with plain 128-bit stores and
//                mid_reduce_kernel, launched right behind, adds the splits in order and finishes the rows.  (Passing
//                128 KB partial tiles between running workgroups through device-coherent 8-byte accesses, as the
//                16-row kernels do with their 4 KB tiles, was measured slower than not splitting at all.)
// Requirements (host-checked): K % 128 == 0, scales grouped or channelwise (no per-row g_idx), A's columns already
// in weight order (dense act-order is gathered beforehand), MoE block size 64.
#include <type_traits>

#include "gemm_kernels.h"

namespace w4a16 {

constexpr int MD_MB = 4;     // m-blocks per tile
constexpr int MD_BM = 64;    // rows per tile
constexpr int MD_D = 4;      // weight k-steps in flight per wavefront
constexpr int MD_ABUF = 2 * MD_MB * 64 * 16;            // one A buffer: 2 k-steps x 4 m-blocks x 64 lanes x 16 B
constexpr int MD_SLABS = 4 * 16 * RED_RS * 4;           // four wavefront slabs of the epilogue
constexpr int MD_SMEM = (2 * MD_ABUF > MD_SLABS ? 2 * MD_ABUF : MD_SLABS) + MD_BM * 8;  // + C row and routing weight of each tile row

// FP4 = 1 / 2: float4_e2m1f weights with NVFP4 / MXFP4 scale records (one 16-byte record per lane and k-step / two
// k-steps); NVFP4's per-expert global scale is applied to the accumulator.
// BITS = 8: uint8b128 or (FP8) float8_e4m3fn weights in the 8-bit Marlin layout; their stages hold twice the weight
// registers, which still fits the two-workgroups-per-compute-unit budget (the grouped variants spill 2-9 registers).
// ZPF: uint4 weights with fp16 zero points laid out like the scales (HQQ; dense only).
template <int DT, bool ZP, bool CHANNEL, bool MOE, int FP4 = 0, int BITS = 4, bool FP8 = false, bool ZPF = false>
__global__ __launch_bounds__(256, 2) void mid_kernel(const KParams p) {
  static_assert(!ZPF || (DT == DT_F16 && !ZP && !CHANNEL && !MOE && BITS == 4 && FP4 == 0), "float zero points: fp16 uint4 grouped, dense");
  static_assert(FP4 == 0 || (!ZP && !CHANNEL && BITS == 4), "fp4 weights: grouped scale records, no zero points");
  static_assert(BITS == 4 || (BITS == 8 && !ZP), "8-bit weights have no zero points");
  static_assert(!FP8 || BITS == 8, "fp8 weights use the 8-bit layout");
  constexpr bool UNIT = CHANNEL;
  extern __shared__ __align__(16) unsigned char smem[];
  int* s_crow = (int*)(smem + MD_SMEM - MD_BM * 8);
  float* s_tw = (float*)(smem + MD_SMEM - MD_BM * 4);
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wv = __builtin_amdgcn_readfirstlane(t >> 6);
  const int c = lane & 7, h = (lane >> 3) & 1, g = lane >> 4;

  // tile order: consecutive workgroups walk M first, so workgroups resident together share weight strips
  // (MoE: neighbouring blocks mostly belong to the same expert)
  const int mtiles = MOE ? (p.n_sorted + MD_BM - 1) / MD_BM : (p.M + MD_BM - 1) / MD_BM;
  zero_fill_side_job(p);
  int mt = blockIdx.x % mtiles;
  int split = (blockIdx.x / mtiles) % p.splits, st_l = blockIdx.x / (mtiles * p.splits);
  int tile = st_l * mtiles + mt;               // index of the output tile inside this launch (partials)
  int nsplit = p.splits, kps = p.ksteps_per_split;
  int moe_ntp = 0;
  if (MOE) moe_ntp = *p.ntpp;
  if (MOE && p.dyn_slots > 0) {
    // live tiles in M-first order; the tail tiles' pieces walk the tiles first, then K (see tail_split)
    const int live = min((moe_ntp + MD_BM - 1) / MD_BM, mtiles);
    if (live == 0) return;
    const TailSplit d = tail_split(live * p.ncp, p.dyn_slots, p.total_ksteps);
    int j = blockIdx.x;
    if (j < d.F) {
      split = 0, nsplit = 1, kps = p.total_ksteps, tile = 0;
    } else {
      const int u = j - d.F;
      if (u >= d.R * d.S) return;
      tile = u % d.R, split = u / d.R, nsplit = d.S, kps = d.kps;
      j = d.F + tile;
    }
    st_l = j / live, mt = j % live;
  }
  const int nt4 = p.strip0 + st_l;             // 512-column strip
  const int cp = nt4 * 4 + wv;                 // column pair of this wavefront
  const bool wave_on = cp * 128 < p.N;         // N not a multiple of 512: trailing wavefronts only help staging
  const int row0 = mt * MD_BM;

  const uint32_t* Bq = p.B;
  const uint16_t* Sc = (const uint16_t*)p.S;
  const uint32_t* Zp = p.Z;
  const uint16_t* bias = (const uint16_t*)p.bias;
  const uint16_t* gscale = (const uint16_t*)p.gscale;
  if (MOE) {
    if (row0 >= moe_ntp) return;
    const int e = p.expert_ids[mt];
    if (e < 0) return;  // expert of another rank
    Bq += e * p.b_estride;
    Sc += e * p.s_estride;
    if (FP4 == 1) gscale += e;
    if (ZP) Zp += e * p.z_estride;
    if (bias) bias += e * p.n_estride;
  }
  // which A row feeds tile row r and which C row receives it (-1: none)
  auto tile_row_ids = [&](int r, int& src, int& dst) {
    src = dst = -1;
    if (MOE) {
      const int id = p.sorted_ids[row0 + r];
      if ((unsigned)id < (unsigned)p.c_rows) {
        src = p.a_by_slot ? row0 + r : id / p.top_k;
        dst = id;
      }
    } else if (row0 + r < p.M) {
      src = dst = row0 + r;
    }
  };
  if (t < MD_BM) {
    int src, dst;
    tile_row_ids(t, src, dst);
    s_crow[t] = dst;
    // (read here once: in the epilogue a load per row would wait behind every store in front of it)
    if (MOE && p.mul_topk) s_tw[t] = dst >= 0 ? p.topk_w[dst] : 0.f;
  }

  // ---- weights of this wavefront
  // (fused SiLU-and-mul: gate n-tile cp paired with the up n-tile of the same output columns, N/128 + cp)
  const int nt = !wave_on ? 0 : (MOE && p.act) ? (h ? (p.N >> 7) + cp : cp) : ((2 * cp + h) * 64 < p.N ? 2 * cp + h : 0);
  // 4-bit: 32 u32x4 per n-tile and k-tile, one per Marlin thread; 8-bit: 64, two per thread (words 2w + half)
  const int64_t b_row = (BITS == 4) ? (p.N >> 1) : p.N;
  const u32x4* bp = (const u32x4*)Bq + nt * (8 * BITS) + (4 * c + g) * (BITS / 4);
  const int64_t s_row = p.N >> 3;
  const u32x4* sp = (const u32x4*)Sc + nt * 8 + c;
  const uint32_t* zp = ZP ? Zp + nt * 8 + c : nullptr;
  const u32x4* zfp = ZPF ? (const u32x4*)Zp + nt * 8 + c : nullptr;  // fp16 zero points: indexed like the scales

  // ---- activation staging: thread t loads piece (t & 7) of tile rows (t >> 3) + 32 i, i = 0..1
  // (rows without a source read row 0 of A; their results are never stored)
  const int piece = t & 7;
  const uint16_t* arow[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    int src, dst;
    tile_row_ids((t >> 3) + 32 * i, src, dst);
    arow[i] = (const uint16_t*)p.A + (int64_t)(src < 0 ? 0 : src) * p.lda + piece * 8;
  }
  // LDS A layout: [buffer][k-step 2][m-block 4][lane 64][4 dwords]; the 16 bytes of (row, piece) are the K
  // pairs 8*pp + 2q (pp = piece & 3), which belong to lane (q*16 + row%16), dword pp, of k-step piece >> 2.
  uint32_t* lds = (uint32_t*)smem;
  int a_wr[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = (t >> 3) + 32 * i;
    a_wr[i] = (((piece >> 2) * MD_MB + (r >> 4)) * 64 + (r & 15)) * 4 + (piece & 3);
  }
  u32x4 areg[2];
  // this workgroup's k-steps: [ks_b, ks_e), a multiple of 4 long (the host splits K in multiples of 4 k-steps)
  const int ks_b = split * kps;
  const int ks_e = min(ks_b + kps, p.total_ksteps);
  // (chunk and k-step indices are clamped instead of guarded: the last iteration re-reads its own data, which
  //  keeps the main loop free of branches)
  auto load_a = [&](int chunk) {  // chunk: relative to ks_b
    chunk = min(ks_b / 2 + chunk, ks_e / 2 - 1);
#pragma unroll
    for (int i = 0; i < 2; ++i) areg[i] = *(const u32x4*)(arow[i] + chunk * 64);
  };
  auto store_a = [&](int buf) {
    uint32_t* dst = lds + buf * (MD_ABUF / 4);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) dst[a_wr[i] + q * 64] = areg[i][q];
    }
  };

  struct Stage {
    u32x4 b0, b1, sc;
    u32x4 b0h, b1h;  // 8-bit weights only: the thread's words 2, 3
    u32x4 zf;        // float zero points only
    uint32_t zq;
  };
  Stage st[MD_D];
  auto issue = [&](Stage& s, int ks) {  // ks: relative to ks_b
    ks = min(ks_b + ks, ks_e - 1);
    int gi = 0;
    if (!CHANNEL) gi = ks >> p.group_shift;  // the host only picks this kernel for power-of-two group sizes
    if (!CHANNEL) s.sc = sp[(int64_t)gi * s_row];
    if (ZP) s.zq = zp[(int64_t)gi * s_row];
    if (FP4 == 2) s.zq = ks & 1;  // which half of the two-k-step scale record
    if (ZPF) s.zf = zfp[(int64_t)gi * s_row];
    s.b0 = bp[(int64_t)(2 * ks) * b_row];
    s.b1 = bp[(int64_t)(2 * ks + 1) * b_row];
    if constexpr (BITS == 8) {
      s.b0h = bp[(int64_t)(2 * ks) * b_row + 1];
      s.b1h = bp[(int64_t)(2 * ks + 1) * b_row + 1];
    }
  };
  // 8-bit: the words of Marlin word position w are elements 2(w & 1) [column half 0] and 2(w & 1) + 1 [half 1] of
  // the thread's first (w < 2) or second 16 bytes, per k-tile
  auto word8 = [&](const Stage& s, int w, int ktile, int half) -> uint32_t {
    const u32x4& v = ktile == 0 ? (w < 2 ? s.b0 : s.b0h) : (w < 2 ? s.b1 : s.b1h);
    return v[2 * (w & 1) + half];
  };
  struct Fp4Scales { float a0, a1, b0, b1; };  // k-tile a / b, column half 0 / 1
  auto fp4_scales = [&](const Stage& s, int w) {
    Fp4Scales r{1.f, 1.f, 1.f, 1.f};
    if constexpr (FP4 == 1) {
      const uint32_t ba = fp4_scale_bytes(s.sc[0], s.sc[1], w), bb = fp4_scale_bytes(s.sc[2], s.sc[3], w);
      r = Fp4Scales{nvfp4_scale_f32(ba & 0xff), nvfp4_scale_f32(ba >> 16), nvfp4_scale_f32(bb & 0xff), nvfp4_scale_f32(bb >> 16)};
    } else if constexpr (FP4 == 2) {
      const uint32_t bs = s.zq ? fp4_scale_bytes(s.sc[2], s.sc[3], w) : fp4_scale_bytes(s.sc[0], s.sc[1], w);
      const float s0 = mxfp4_scale_f32(bs & 0xff), s1 = mxfp4_scale_f32(bs >> 16);
      r = Fp4Scales{s0, s1, s0, s1};
    }
    return r;
  };
  auto col_const = [&](const Stage& s, int w) {
    uint32_t z0 = 8, z1 = 8;
    if (ZP) {
      z0 = (s.zq >> (4 * w)) & 0xf;
      z1 = (s.zq >> (4 * w + 16)) & 0xf;
    }
    return make_col_const<DT, UNIT>(CHANNEL ? 0u : s.sc[w], z0, z1);
  };

  f32x4 acc[MD_MB][4][2];
#pragma unroll
  for (int mb = 0; mb < MD_MB; ++mb)
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      acc[mb][w][0] = f32x4{0, 0, 0, 0};
      acc[mb][w][1] = f32x4{0, 0, 0, 0};
    }

  const int nchunks = (ks_e - ks_b) / 2;  // even: K % 128 == 0 and splits are multiples of 4 k-steps

  // ---- prologue
  load_a(0);
#pragma unroll
  for (int j = 0; j < MD_D; ++j) issue(st[j], j);
  store_a(0);
  // B operands of two Marlin words: the one whose MFMAs are being issued and the one being dequantised
  u32x4 ob[2][2];
  if constexpr (ZPF) {
    dequant_pair_zpf(st[0].b0[0], st[0].b1[0], st[0].sc[0], as_u32(as_h2(st[0].zf[0]) * as_h2(st[0].sc[0])), ob[0][0],
                     ob[0][1]);
  } else if constexpr (FP4 != 0) {
    const Fp4Scales fs = fp4_scales(st[0], 0);
    dequant_pair_fp4<DT>(st[0].b0[0], st[0].b1[0], fs.a0, fs.a1, fs.b0, fs.b1, ob[0][0], ob[0][1]);
  } else if constexpr (FP8) {
    dequant_pair8_fp8<DT, UNIT>(word8(st[0], 0, 0, 0), word8(st[0], 0, 0, 1), word8(st[0], 0, 1, 0), word8(st[0], 0, 1, 1),
                                CHANNEL ? 0u : st[0].sc[0], ob[0][0], ob[0][1]);
  } else if constexpr (BITS == 8) {
    dequant_pair8<DT, UNIT>(word8(st[0], 0, 0, 0), word8(st[0], 0, 0, 1), word8(st[0], 0, 1, 0), word8(st[0], 0, 1, 1),
                            CHANNEL ? 0u : st[0].sc[0], ob[0][0], ob[0][1]);
  } else {
    const ColConst<DT> cc = col_const(st[0], 0);
    dequant_pair<DT, UNIT>(st[0].b0[0], st[0].b1[0], cc, ob[0][0], ob[0][1]);
  }
  __syncthreads();

  // One k-step: per Marlin word w, 8 MFMAs on ob[w & 1]; after each MFMA one register of the following word's
  // operands (word w + 1 of this k-step, or word 0 of the next k-step `nxt`) is dequantised into ob[(w + 1) & 1].
  // The scheduling barriers keep the compiler from regrouping this into MFMA-only and VALU-only blocks.
  auto kstep = [&](int buf, int kk, const Stage& cur, const Stage& nxt) {
    const u32x4* abase = (const u32x4*)(lds + buf * (MD_ABUF / 4)) + (kk * MD_MB) * 64 + lane;
    u32x4 af[MD_MB];
#pragma unroll
    for (int mb = 0; mb < MD_MB; ++mb) af[mb] = abase[mb * 64];
    auto word = [&](auto w_tag) {
      constexpr int w = decltype(w_tag)::value;
      constexpr int wn = (w + 1) & 3;
      const Stage& src = w == 3 ? nxt : cur;
      const ColConst<DT> cc = col_const(src, wn);
      const Fp4Scales fs = fp4_scales(src, wn);
      uint32_t zs = 0;
      if constexpr (ZPF) zs = as_u32(as_h2(src.zf[wn]) * as_h2(src.sc[wn]));
      const uint32_t xa = src.b0[wn], xb = src.b1[wn];
      auto step = [&](auto j_tag) {
        constexpr int J = decltype(j_tag)::value;
        mfma_inplace<DT>(acc[J >> 1][w][J & 1], af[J >> 1], ob[w & 1][J & 1]);
        uint32_t r;
        if constexpr (ZPF)
          r = dequant_piece_zpf<J>(xa, xb, src.sc[wn], zs);
        else if constexpr (FP4 != 0)
          r = ((J & 3) < 2) ? dequant_piece_fp4<DT, J>(xa, fs.a0, fs.a1) : dequant_piece_fp4<DT, J>(xb, fs.b0, fs.b1);
        else if constexpr (BITS == 8)
          r = dequant_piece8<DT, UNIT, FP8, J>(word8(src, wn, (J & 3) >> 1, 0), word8(src, wn, (J & 3) >> 1, 1),
                                               CHANNEL ? 0u : src.sc[wn]);
        else
          r = dequant_piece<DT, UNIT, J>(xa, xb, cc);
        if constexpr (J < 4)
          ob[wn & 1][0][J] = r;
        else
          ob[wn & 1][1][J - 4] = r;
        __builtin_amdgcn_sched_barrier(0);
      };
      step(std::integral_constant<int, 0>{});
      step(std::integral_constant<int, 1>{});
      step(std::integral_constant<int, 2>{});
      step(std::integral_constant<int, 3>{});
      step(std::integral_constant<int, 4>{});
      step(std::integral_constant<int, 5>{});
      step(std::integral_constant<int, 6>{});
      step(std::integral_constant<int, 7>{});
    };
    word(std::integral_constant<int, 0>{});
    word(std::integral_constant<int, 1>{});
    word(std::integral_constant<int, 2>{});
    word(std::integral_constant<int, 3>{});
  };

  // ---- main loop: two chunks (four k-steps = the weight ring) per iteration
#pragma unroll 1
  for (int c0 = 0; c0 < nchunks; c0 += 2) {
    const int ks0 = 2 * c0;
    // chunk c0 in buffer 0
    load_a(c0 + 1);
    kstep(0, 0, st[0], st[1]);
    issue(st[0], ks0 + 4);
    kstep(0, 1, st[1], st[2]);
    issue(st[1], ks0 + 5);
    store_a(1);
    __syncthreads();
    // chunk c0+1 in buffer 1
    load_a(c0 + 2);
    kstep(1, 0, st[2], st[3]);
    issue(st[2], ks0 + 6);
    kstep(1, 1, st[3], st[0]);
    issue(st[3], ks0 + 7);
    store_a(0);
    __syncthreads();
  }

  // ------------------------------------------------------------------------------ epilogue
  // (the inline-asm MFMAs are opaque to the compiler's hazard logic: let the matrix pipe drain before the
  //  accumulators are read)
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  // per wavefront and m-block: accumulators -> private LDS slab [16 rows][RED_RS] -> 8-byte row stores.
  // (the last barrier of the loop separates the slabs from the A buffers they overlay)
  float* slab = (float*)smem + wv * (16 * RED_RS);
  const int fc4 = (lane & 31) * 4;
  const int fpos = fc4 + (fc4 >= 64 ? 8 : 0);
  const int ncol = cp * 128 + fc4;
  const bool fcol_ok = wave_on && ncol < p.N;
  const bool act = MOE && p.act;
  // cs / bs: channel (and global) scale and bias of the thread's four columns; cu / bu: of the up half's columns
  float cs[4] = {1.f, 1.f, 1.f, 1.f}, bs[4] = {0.f, 0.f, 0.f, 0.f}, cu[4] = {1.f, 1.f, 1.f, 1.f}, bu[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (FP4 == 1) {
    // NVFP4 global scale: stored times 2^7 (fp16) / 2^119 (bf16) by the reference's load-time processing
    const uint16_t gv = *gscale;
    const float gs = (DT == DT_F16) ? f16_lo_f32(gv) * 0x1.0p-7f : bf16_lo_f32(gv) * 0x1.0p-119f;
#pragma unroll
    for (int j = 0; j < 4; ++j) cs[j] = cu[j] = gs;
  }
  auto col_consts = [&](int col, float* sc_out, float* b_out) {
    const int base = col & ~31, cl = col & 31;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (CHANNEL) {
        const uint16_t sv = Sc[base + single_perm_pos(cl + j)];
        sc_out[j] = ((DT == DT_F16) ? f16_lo_f32(sv) : bf16_lo_f32(sv)) * (p.fp8 ? fp8_scale_unbias<DT>() : 1.0f);
      }
      if (bias) {
        const uint16_t bv = bias[base + single_perm_pos(cl + j)];
        b_out[j] = (DT == DT_F16) ? f16_lo_f32(bv) : bf16_lo_f32(bv);
      }
    }
  };
  // fused SiLU-and-mul, unsplit: lane -> row (lane >> 4) + 4 i, gate columns 4 (lane & 15) .. + 3 and the up columns of
  // the same outputs, so that all 64 lanes take part
  const int ac4 = (lane & 15) * 4;
  const int ocol = cp * 64 + ac4;
  if (act) {
    if (wave_on) {
      col_consts(ocol, cs, bs);
      col_consts((p.N >> 1) + ocol, cu, bu);
    }
  } else if (fcol_ok) {
    col_consts(ncol, cs, bs);
  }
#pragma unroll
  for (int mb = 0; mb < MD_MB; ++mb) {
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int r = 0; r < 4; ++r) slab[(4 * g + r) * RED_RS + 72 * h + 16 * w + 8 * hf + c] = acc[mb][w][hf][r];
    __builtin_amdgcn_wave_barrier();
    if (act && nsplit == 1) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r16 = (lane >> 4) + 4 * i;
        const int crow = s_crow[mb * 16 + r16];
        if (crow < 0 || !wave_on) continue;
        f32x4 v = *(const f32x4*)(slab + r16 * RED_RS + ac4);
        f32x4 u = *(const f32x4*)(slab + r16 * RED_RS + ac4 + 72);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v[j] = v[j] * cs[j] + bs[j];
          u[j] = u[j] * cu[j] + bu[j];
        }
        if (p.mul_topk) {
          const float tw = s_tw[mb * 16 + r16];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[j] *= tw;
            u[j] *= tw;
          }
        }
        store_row4_silu_mul<DT>(p, crow, ocol, v, u);
      }
      __builtin_amdgcn_wave_barrier();
      continue;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r16 = (lane >> 5) + 2 * i;
      const int crow = s_crow[mb * 16 + r16];
      f32x4 v = *(const f32x4*)(slab + r16 * RED_RS + fpos);
      if (nsplit > 1) {
        // K is split: the fp32 partial tile [row 64][column 512] goes to scratch with plain stores; the reduction
        // kernel launched behind this one adds the splits and finishes the rows
        if (fcol_ok && crow >= 0)
          *(f32x4*)(p.ctmp + (((int64_t)tile * nsplit + split) * MD_BM + mb * 16 + r16) * 512 + wv * 128 + fc4) = v;
        continue;
      }
      if (crow < 0) continue;
      if (fcol_ok) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = v[j] * cs[j] + bs[j];
        if (MOE && p.mul_topk) {
          const float tw = s_tw[mb * 16 + r16];
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] *= tw;
        }
        store_row4<DT>(p, crow, ncol, v);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// Second pass of a split-K launch of mid_kernel: out tile = sum over splits of the fp32 partial tiles (in split order,
// so the result does not depend on timing), then channel scale, bias, routing weight, conversion and the row scatter
// exactly as mid_kernel's own epilogue does.  One workgroup per (tile, 16-row block); thread -> 4 columns of 2 rows per pass.
template <int DT, bool CHANNEL, bool MOE>
__global__ __launch_bounds__(256) void mid_reduce_kernel(const KParams p) {
  const int t = threadIdx.x;
  const int mtiles = MOE ? (p.n_sorted + MD_BM - 1) / MD_BM : (p.M + MD_BM - 1) / MD_BM;
  const int tile = blockIdx.x >> 2, rb = blockIdx.x & 3;
  int mt = tile % mtiles, nt4 = p.strip0 + tile / mtiles, nsplit = p.splits;
  if (MOE && p.dyn_slots > 0) {  // tile: index among the tail tiles (see tail_split)
    const int live = min((*p.ntpp + MD_BM - 1) / MD_BM, mtiles);
    if (live == 0) return;
    const TailSplit d = tail_split(live * p.ncp, p.dyn_slots, p.total_ksteps);
    if (d.S == 1 || tile >= d.R) return;
    const int j = d.F + tile;
    mt = j % live, nt4 = p.strip0 + j / live, nsplit = d.S;
  }
  const int row0 = mt * MD_BM;
  const uint16_t* Sc = (const uint16_t*)p.S;
  const uint16_t* bias = (const uint16_t*)p.bias;
  const uint16_t* gscale = (const uint16_t*)p.gscale;  // NVFP4 only, else null
  if (MOE) {
    if (row0 >= *p.ntpp) return;
    const int e = p.expert_ids[mt];
    if (e < 0) return;
    Sc += e * p.s_estride;
    if (gscale) gscale += e;
    if (bias) bias += e * p.n_estride;
  }
  const int fc4 = (t & 127) * 4;
  const bool act = MOE && p.act;
  // fused SiLU-and-mul: the 128 columns of wavefront block fc4 / 128 are 64 gate columns followed by the 64 up columns
  // of the same outputs; only the gate half's threads finish rows
  const int cp = nt4 * 4 + (fc4 >> 7);
  const int ncol = act ? cp * 64 + (fc4 & 127) : nt4 * 512 + fc4;
  if (act ? ((fc4 & 127) >= 64 || cp * 128 >= p.N) : ncol >= p.N) return;
  float cs[4] = {1.f, 1.f, 1.f, 1.f}, bs[4] = {0.f, 0.f, 0.f, 0.f}, cu[4] = {1.f, 1.f, 1.f, 1.f}, bu[4] = {0.f, 0.f, 0.f, 0.f};
  if (gscale) {
    const uint16_t gv = *gscale;
    const float gs = (DT == DT_F16) ? f16_lo_f32(gv) * 0x1.0p-7f : bf16_lo_f32(gv) * 0x1.0p-119f;
#pragma unroll
    for (int j = 0; j < 4; ++j) cs[j] = cu[j] = gs;
  }
  auto col_consts = [&](int col, float* sc_out, float* b_out) {
    const int base = col & ~31, cl = col & 31;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (CHANNEL) {
        const uint16_t sv = Sc[base + single_perm_pos(cl + j)];
        sc_out[j] = ((DT == DT_F16) ? f16_lo_f32(sv) : bf16_lo_f32(sv)) * (p.fp8 ? fp8_scale_unbias<DT>() : 1.0f);
      }
      if (bias) {
        const uint16_t bv = bias[base + single_perm_pos(cl + j)];
        b_out[j] = (DT == DT_F16) ? f16_lo_f32(bv) : bf16_lo_f32(bv);
      }
    }
  };
  col_consts(ncol, cs, bs);
  if (act) col_consts((p.N >> 1) + ncol, cu, bu);
  const float* parts = p.ctmp + (int64_t)tile * nsplit * (MD_BM * 512) + fc4;
  // (the rows' slot ids, then per row the partial tiles of four splits at a time, are loaded together: the pass is bound
  //  by round trips, not by bytes)
  int crows[8];
  float tws[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = rb * 16 + (t >> 7) + 2 * i;
    crows[i] = -1;
    if (MOE) {
      const int id = p.sorted_ids[row0 + r];
      if ((unsigned)id < (unsigned)p.c_rows) crows[i] = id;
    } else if (row0 + r < p.M) {
      crows[i] = row0 + r;
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) tws[i] = (MOE && p.mul_topk && crows[i] >= 0) ? p.topk_w[crows[i]] : 1.0f;
  auto sum_splits = [&](const float* src) {  // src: the row's columns in split 0; added in split order
    f32x4 acc = {0, 0, 0, 0};
    for (int s0 = 0; s0 < nsplit; s0 += 4) {
      f32x4 a[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) a[q] = *(const f32x4*)(src + (int64_t)min(s0 + q, nsplit - 1) * (MD_BM * 512));
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (s0 + q < nsplit) acc += a[q];
    }
    return acc;
  };
#pragma unroll 2
  for (int i = 0; i < 8; ++i) {
    const int r = rb * 16 + (t >> 7) + 2 * i;
    const int crow = crows[i];
    if (crow < 0) continue;
    f32x4 v = sum_splits(parts + (int64_t)r * 512), u = {0, 0, 0, 0};
    if (act) u = sum_splits(parts + (int64_t)r * 512 + 64);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[j] = v[j] * cs[j] + bs[j];
      u[j] = u[j] * cu[j] + bu[j];
    }
    if (MOE && p.mul_topk) {
      const float tw = tws[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[j] *= tw;
        u[j] *= tw;
      }
    }
    if (act)
      store_row4_silu_mul<DT>(p, crow, ncol, v, u);
    else
      store_row4<DT>(p, crow, ncol, v);
  }
}

typedef void (*mid_fn)(const KParams);

template <int DT, bool MOE>
static mid_fn pick_mid2(bool zp, bool channel) {
  if (zp) return channel ? mid_kernel<DT, true, true, MOE> : mid_kernel<DT, true, false, MOE>;
  return channel ? mid_kernel<DT, false, true, MOE> : mid_kernel<DT, false, false, MOE>;
}
template <int DT, bool MOE>
static mid_fn pick_mid8(bool fp8, bool channel) {
  if (fp8) return channel ? mid_kernel<DT, false, true, MOE, 0, 8, true> : mid_kernel<DT, false, false, MOE, 0, 8, true>;
  return channel ? mid_kernel<DT, false, true, MOE, 0, 8, false> : mid_kernel<DT, false, false, MOE, 0, 8, false>;
}
template <int DT, bool MOE>
static mid_fn pick_reduce(bool channel) {
  return channel ? mid_reduce_kernel<DT, true, MOE> : mid_reduce_kernel<DT, false, MOE>;
}

int launch_mid(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream) {
  const bool zp = a->b_zeros != nullptr, channel = pl.gm == GM_CHANNEL;
  const bool moe = (a->flags & W4A16_F_MOE) != 0;
  mid_fn fn, red;
  if (a->flags & W4A16_F_ZP_FLOAT) {
    if (a->dtype != DT_F16 || channel || moe) return fail(W4A16_EINVAL, "unsupported kernel variant");
    fn = mid_kernel<DT_F16, false, false, false, 0, 4, false, true>;
    red = pick_reduce<DT_F16, false>(false);
  } else if (a->wtype == W4A16_WTYPE_U8B128 || a->wtype == W4A16_WTYPE_FE4M3) {
    if (zp) return fail(W4A16_EINVAL, "unsupported kernel variant");
    const bool fp8 = a->wtype == W4A16_WTYPE_FE4M3;
    if (a->dtype == DT_F16) {
      fn = moe ? pick_mid8<DT_F16, true>(fp8, channel) : pick_mid8<DT_F16, false>(fp8, channel);
      red = moe ? pick_reduce<DT_F16, true>(channel) : pick_reduce<DT_F16, false>(channel);
    } else {
      fn = moe ? pick_mid8<DT_BF16, true>(fp8, channel) : pick_mid8<DT_BF16, false>(fp8, channel);
      red = moe ? pick_reduce<DT_BF16, true>(channel) : pick_reduce<DT_BF16, false>(channel);
    }
  } else if (a->wtype == W4A16_WTYPE_FE2M1) {
    if (zp || channel) return fail(W4A16_EINVAL, "unsupported kernel variant");
    if (a->global_scale)
      fn = a->dtype == DT_F16 ? (moe ? mid_kernel<DT_F16, false, false, true, 1> : mid_kernel<DT_F16, false, false, false, 1>)
                              : (moe ? mid_kernel<DT_BF16, false, false, true, 1> : mid_kernel<DT_BF16, false, false, false, 1>);
    else
      fn = moe ? mid_kernel<DT_BF16, false, false, true, 2> : mid_kernel<DT_BF16, false, false, false, 2>;
    red = a->dtype == DT_F16 ? (moe ? pick_reduce<DT_F16, true>(false) : pick_reduce<DT_F16, false>(false))
                             : (moe ? pick_reduce<DT_BF16, true>(false) : pick_reduce<DT_BF16, false>(false));
  } else if (a->dtype == DT_F16) {
    fn = moe ? pick_mid2<DT_F16, true>(zp, channel) : pick_mid2<DT_F16, false>(zp, channel);
    red = moe ? pick_reduce<DT_F16, true>(channel) : pick_reduce<DT_F16, false>(channel);
  } else {
    fn = moe ? pick_mid2<DT_BF16, true>(zp, channel) : pick_mid2<DT_BF16, false>(zp, channel);
    red = moe ? pick_reduce<DT_BF16, true>(channel) : pick_reduce<DT_BF16, false>(channel);
  }
  KParams p = make_kparams(a, pl);
  if (pl.tiles <= 0) return 0;
  if (pl.dyn_slots > 0) {
    // device-side K split of the tail tiles: at most dyn_slots pieces behind the whole tiles, at most that many tail tiles
    if (!moe || pl.splits != 1) return fail(W4A16_EINVAL, "unsupported kernel variant");
    const int64_t pieces = mid_tail_pieces(pl.tiles, pl.dyn_slots);
    hipLaunchKernelGGL(fn, dim3((unsigned)(pl.tiles + pieces)), dim3(256), MD_SMEM, stream, p);
    W4A16_HIP(hipGetLastError());
    const int64_t tail = pl.tiles < pl.dyn_slots ? pl.tiles : pl.dyn_slots;
    hipLaunchKernelGGL(red, dim3((unsigned)(tail * 4)), dim3(256), 0, stream, p);
    W4A16_HIP(hipGetLastError());
    return 0;
  }
  const int64_t grid = (int64_t)pl.tiles * pl.splits;
  hipLaunchKernelGGL(fn, dim3((unsigned)grid), dim3(256), MD_SMEM, stream, p);
  W4A16_HIP(hipGetLastError());
  if (pl.splits > 1) {
    hipLaunchKernelGGL(red, dim3((unsigned)(pl.tiles * 4)), dim3(256), 0, stream, p);
    W4A16_HIP(hipGetLastError());
  }
  return 0;
}

}  // namespace w4a16
