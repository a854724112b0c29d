// W4A16 GEMM for gfx950 with an in-workgroup K split: C[M,N] = A[M,K] * dequant(Bq)[K,N] (+bias), dense, in two shapes.
// First shape, 64-row tiles: 33..128 rows and wide N, where the 64 x 512 tiles of the 64-row kernel are too few to fill
// the chip (the reference's small-batch thread configurations, csrc/quantization/gptq_marlin/gptq_marlin.cu:120-170).
//
//   workgroup tile 64 rows x 256 columns, 8 wavefronts = 2 column pairs x 4 K-quarters: every wavefront owns
//   64 rows x 128 columns (32 v_mfma_f32_16x16x32 per k-step, 128 fp32 accumulators in AGPRs) over a quarter of the
//   K range, two wavefronts per SIMD.
//   weights      streamed global -> registers per wavefront and dequantised one operand register per MFMA, exactly as
//                in the 64-row kernel (B operand = the reference's half(q - z) * half(s)).
//   activations  each K-quarter stages its own 64 rows x 64 K chunk into LDS in MFMA fragment order (its two
//                wavefronts share it), double buffered; one workgroup barrier per two k-steps.
//   epilogue     the four quarters' partial tiles are added through LDS, one 16-row block at a time.
//   split-K      with fewer tiles than compute units (129..~1000 rows of a narrow layer) K is also cut across
//                workgroups, in splits of whole multiples of 512 K rows: the workgroup writes its 64 x 256 fp32 partial
//                tile (already summed over its quarters) to scratch with plain 128-bit stores and kq_reduce_kernel,
//                launched right behind, adds the splits in order and finishes the rows.  A quarter of the 64 x 512
//                kernel's partial bytes for the same number of wavefronts on the problem.
// Compared with 16-row tiles (which re-read and re-convert the weight strip once per 16 rows) every weight is fetched
// and dequantised once per 64 rows; compared with the 64 x 512 tile there are 2 x 4 times as many independent streams.
// A second shape of the same kernel (MB = 8, Q = 2: 4 wavefronts, one per SIMD, 128 rows x 256 columns, K in halves, 256
// accumulators per lane) serves problems with 128-row tiles that are too few for the prefill kernel's 128 x 512 tiles:
// every dequantised operand register feeds eight row blocks as in the prefill kernel, and the two K halves are added
// through LDS instead of through memory.  The host uses it for more than 128 rows when these tiles fill 3/4 to all of the
// compute units in one round, and for the trailing strips of a prefill launch whose last round is at most half full
// (KParams.strip0: first 256-column strip of the launch).
// Requirements (host-checked): K % 512 == 0 (second shape: K % 256 == 0), so that every K part runs whole ring periods of
// 4 k-steps; scales grouped (a power-of-two number of k-steps) or channelwise, no per-row g_idx, A's columns already in
// weight order.
#include <type_traits>

#include "gemm_kernels.h"

namespace w4a16 {

constexpr int KQ_TN = 256;   // columns per tile
constexpr int KQ_D = 4;      // weight k-steps in flight per wavefront
// MB m-blocks of 16 rows per tile, K cut into Q parts inside the workgroup (2 Q wavefronts)
constexpr int kq_abuf(int MB) { return 2 * MB * 64 * 16; }  // one A buffer of one K part: 2 k-steps x MB m-blocks x 64 lanes x 16 B
constexpr int kq_smem(int MB, int Q) {
  const int stage = Q * 2 * kq_abuf(MB), slabs = 2 * Q * 16 * RED_RS * 4;  // staging rings | the wavefronts' epilogue slabs
  return (stage > slabs ? stage : slabs) + 16 * MB * 4;                     // + C row of each tile row
}

template <int DT, bool ZP, bool CHANNEL, int MB = 4, int Q = 4>
__global__ __launch_bounds__(128 * Q) void kq_kernel(const KParams p) {
  static_assert((MB == 4 && Q == 4) || (MB == 8 && Q == 2), "64 x 256 in K quarters or 128 x 256 in K halves");
  constexpr int KQ_MB = MB, KQ_BM = 16 * MB, KQ_Q = Q, KQ_ABUF = kq_abuf(MB), KQ_SMEM = kq_smem(MB, Q);
  constexpr bool UNIT = CHANNEL;
  extern __shared__ __align__(16) unsigned char smem[];
  int* s_crow = (int*)(smem + KQ_SMEM - KQ_BM * 4);
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wv = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wn = wv & 1, q = wv >> 1;  // column pair inside the tile, K-quarter
  const int c = lane & 7, h = (lane >> 3) & 1, g = lane >> 4;

  // tile order: consecutive workgroups walk M first, so workgroups resident together share weight strips
  const int mtiles = (p.M + KQ_BM - 1) / KQ_BM;
  const int mt = blockIdx.x % mtiles;
  const int split = (blockIdx.x / mtiles) % p.splits, strip = blockIdx.x / (mtiles * p.splits);
  const int cp = (p.strip0 + strip) * 2 + wn;  // column pair of this wavefront (strip0: first 256-column strip of the launch)
  const bool wave_on = cp * 128 < p.N;         // N not a multiple of 256: the trailing wavefronts only help staging
  const int row0 = mt * KQ_BM;

  const uint32_t* Bq = p.B;
  const uint16_t* Sc = (const uint16_t*)p.S;
  const uint32_t* Zp = p.Z;
  const uint16_t* bias = (const uint16_t*)p.bias;
  // which A row feeds tile row r and which C row receives it (-1: none)
  auto tile_row_ids = [&](int r, int& src, int& dst) {
    src = dst = -1;
    if (row0 + r < p.M) src = dst = row0 + r;
  };
  if (t < KQ_BM) {
    int src, dst;
    tile_row_ids(t, src, dst);
    s_crow[t] = dst;
  }

  // ---- weights of this wavefront
  const int nt = (wave_on && (2 * cp + h) * 64 < p.N) ? 2 * cp + h : 0;
  const int64_t b_row = p.N >> 1;
  const u32x4* bp = (const u32x4*)Bq + nt * 32 + (4 * c + g);
  const int64_t s_row = p.N >> 3;
  const u32x4* sp = (const u32x4*)Sc + nt * 8 + c;
  const uint32_t* zp = ZP ? Zp + nt * 8 + c : nullptr;

  // ---- this quarter's k-steps: [ks_b, ks_e), a multiple of 4 long
  const int per_q = p.ksteps_per_split / KQ_Q;  // host: a multiple of 4, and the splits are equally long
  const int ks_b = split * p.ksteps_per_split + q * per_q, ks_e = ks_b + per_q;

  // ---- activation staging: the K part's 128 threads; thread tq loads piece (tq & 7) of tile rows (tq >> 3) + 16 i
  // (rows without a source read row 0 of A; their results are never stored)
  const int tq = wn * 64 + lane;
  const int piece = tq & 7;
  const uint16_t* arow[KQ_MB];
#pragma unroll
  for (int i = 0; i < KQ_MB; ++i) {
    int src, dst;
    tile_row_ids((tq >> 3) + 16 * i, src, dst);
    arow[i] = (const uint16_t*)p.A + (int64_t)(src < 0 ? 0 : src) * p.lda + piece * 8;
  }
  // LDS A layout per quarter: [buffer][k-step 2][m-block 4][lane 64][4 dwords]; the 16 bytes of (row, piece) are the
  // K pairs 8*pp + 2j (pp = piece & 3), which belong to lane (j*16 + row%16), dword pp, of k-step piece >> 2.
  uint32_t* lds = (uint32_t*)smem + q * (2 * KQ_ABUF / 4);
  int a_wr[KQ_MB];
#pragma unroll
  for (int i = 0; i < KQ_MB; ++i) {
    const int r = (tq >> 3) + 16 * i;
    a_wr[i] = (((piece >> 2) * KQ_MB + (r >> 4)) * 64 + (r & 15)) * 4 + (piece & 3);
  }
  u32x4 areg[KQ_MB];
  // (chunk and k-step indices are clamped instead of guarded: the last iteration re-reads its own data, which
  //  keeps the main loop free of branches)
  auto load_a = [&](int chunk) {  // chunk: relative to ks_b
    chunk = min(ks_b / 2 + chunk, ks_e / 2 - 1);
#pragma unroll
    for (int i = 0; i < KQ_MB; ++i) areg[i] = *(const u32x4*)(arow[i] + chunk * 64);
  };
  auto store_a = [&](int buf) {
    uint32_t* dst = lds + buf * (KQ_ABUF / 4);
#pragma unroll
    for (int i = 0; i < KQ_MB; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) dst[a_wr[i] + j * 64] = areg[i][j];
    }
  };

  struct Stage {
    u32x4 b0, b1, sc;
    uint32_t zq;
  };
  Stage st[KQ_D];
  auto issue = [&](Stage& s, int ks) {  // ks: relative to ks_b
    ks = min(ks_b + ks, ks_e - 1);
    int gi = 0;
    if (!CHANNEL) gi = ks >> p.group_shift;
    if (!CHANNEL) s.sc = sp[(int64_t)gi * s_row];
    if (ZP) s.zq = zp[(int64_t)gi * s_row];
    s.b0 = bp[(int64_t)(2 * ks) * b_row];
    s.b1 = bp[(int64_t)(2 * ks + 1) * b_row];
  };
  auto col_const = [&](const Stage& s, int w) {
    uint32_t z0 = 8, z1 = 8;
    if (ZP) {
      z0 = (s.zq >> (4 * w)) & 0xf;
      z1 = (s.zq >> (4 * w + 16)) & 0xf;
    }
    return make_col_const<DT, UNIT>(CHANNEL ? 0u : s.sc[w], z0, z1);
  };

  f32x4 acc[KQ_MB][4][2];
#pragma unroll
  for (int mb = 0; mb < KQ_MB; ++mb)
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      acc[mb][w][0] = f32x4{0, 0, 0, 0};
      acc[mb][w][1] = f32x4{0, 0, 0, 0};
    }

  const int nchunks = per_q / 2;  // even

  // ---- prologue
  load_a(0);
#pragma unroll
  for (int j = 0; j < KQ_D; ++j) issue(st[j], j);
  store_a(0);
  // B operands of two Marlin words: the one whose MFMAs are being issued and the one being dequantised
  u32x4 ob[2][2];
  // dequantisation constants of the four word positions for the k-step whose operands are being built.  A loop iteration
  // covers four k-steps (128 rows of K, aligned: every K part starts at a multiple of four k-steps), so with groups of
  // 128 rows or more, or one scale per column, they are rebuilt once per iteration instead of once per k-step.
  // (128-row tiles only: with two wavefronts per SIMD the 64-row tiles have no registers to spare for them.)
  constexpr bool HOIST = (KQ_MB == 8);
  ColConst<DT> ccs[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) ccs[w] = col_const(st[0], w);
  dequant_pair<DT, UNIT>(st[0].b0[0], st[0].b1[0], ccs[0], ob[0][0], ob[0][1]);
  __syncthreads();

  // One k-step: per Marlin word w, 2 MB MFMAs on ob[w & 1]; after each MFMA (MB = 8: pair of MFMAs) one register of the following word's
  // operands (word w + 1 of this k-step, or word 0 of the next k-step `nxt`) is dequantised into ob[(w + 1) & 1].
  // The scheduling barriers keep the compiler from regrouping this into MFMA-only and VALU-only blocks.
  auto kstep = [&](int buf, int kk, const Stage& cur, const Stage& nxt, auto refresh_tag) {
    const u32x4* abase = (const u32x4*)(lds + buf * (KQ_ABUF / 4)) + (kk * KQ_MB) * 64 + lane;
    u32x4 af[KQ_MB];
#pragma unroll
    for (int mb = 0; mb < KQ_MB; ++mb) af[mb] = abase[mb * 64];
    auto word = [&](auto w_tag) {
      constexpr int w = decltype(w_tag)::value;
      constexpr int wn2 = (w + 1) & 3;
      const Stage& src = w == 3 ? nxt : cur;
      ColConst<DT> cc_word;
      if constexpr (!HOIST) {
        cc_word = col_const(src, wn2);
      } else if constexpr (w == 3 && decltype(refresh_tag)::value) {  // the words of `cur` are done: constants of `nxt`
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) ccs[ww] = col_const(nxt, ww);
      }
      const ColConst<DT>& cc = HOIST ? ccs[wn2] : cc_word;
      const uint32_t xa = src.b0[wn2], xb = src.b1[wn2];
      auto step = [&](auto j_tag) {
        constexpr int J = decltype(j_tag)::value;
        if constexpr (KQ_MB == 4) {
          mfma_inplace<DT>(acc[J >> 1][w][J & 1], af[J >> 1], ob[w & 1][J & 1]);
        } else {
          mfma_inplace<DT>(acc[J][w][0], af[J], ob[w & 1][0]);
          mfma_inplace<DT>(acc[J][w][1], af[J], ob[w & 1][1]);
        }
        const uint32_t r = dequant_piece<DT, UNIT, J>(xa, xb, cc);
        if constexpr (J < 4)
          ob[wn2 & 1][0][J] = r;
        else
          ob[wn2 & 1][1][J - 4] = r;
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

  // ---- main loop: two chunks (four k-steps = the weight ring) per iteration; all K parts run the same count.  The
  // last k-step of an iteration builds the first operands of the next 128 rows of K: the constants are rebuilt there,
  // and in the other three k-steps too when a group is shorter than 128 rows.
  auto main_loop = [&](auto every_tag) {
    const std::true_type refresh{};
#pragma unroll 1
    for (int c0 = 0; c0 < nchunks; c0 += 2) {
      const int ks0 = 2 * c0;
      load_a(c0 + 1);
      kstep(0, 0, st[0], st[1], every_tag);
      issue(st[0], ks0 + 4);
      kstep(0, 1, st[1], st[2], every_tag);
      issue(st[1], ks0 + 5);
      store_a(1);
      __syncthreads();
      load_a(c0 + 2);
      kstep(1, 0, st[2], st[3], every_tag);
      issue(st[2], ks0 + 6);
      kstep(1, 1, st[3], st[0], refresh);
      issue(st[3], ks0 + 7);
      store_a(0);
      __syncthreads();
    }
  };
  if constexpr (CHANNEL || !HOIST) {
    main_loop(std::false_type{});
  } else {
    if (p.group_shift < 2)
      main_loop(std::true_type{});
    else
      main_loop(std::false_type{});
  }

  // ------------------------------------------------------------------------------ epilogue
  // (the inline-asm MFMAs are opaque to the compiler's hazard logic: let the matrix pipe drain before the
  //  accumulators are read)
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  // per m-block: every wavefront writes its 16 x 128 partial to its slab [16 rows][RED_RS]; after a barrier the
  // wavefront of K part q adds the Q parts' slabs of its column pair for rows (16 / Q) q .. and finishes them.
  // (the last barrier of the loop separates the slabs from the A buffers they overlay)
  float* slabs = (float*)smem;
  float* mine = slabs + wv * (16 * RED_RS);
  const int fc4 = (lane & 31) * 4;
  const int fpos = fc4 + (fc4 >= 64 ? 8 : 0);
  const int ncol = cp * 128 + fc4;
  const bool fcol_ok = wave_on && ncol < p.N;
  float cs[4] = {1.f, 1.f, 1.f, 1.f}, bs[4] = {0.f, 0.f, 0.f, 0.f};
  if (fcol_ok) {
    const int base = ncol & ~31, cl = ncol & 31;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (CHANNEL) {
        const uint16_t sv = Sc[base + single_perm_pos(cl + j)];
        cs[j] = (DT == DT_F16) ? f16_lo_f32(sv) : bf16_lo_f32(sv);
      }
      if (bias) {
        const uint16_t bv = bias[base + single_perm_pos(cl + j)];
        bs[j] = (DT == DT_F16) ? f16_lo_f32(bv) : bf16_lo_f32(bv);
      }
    }
  }
#pragma unroll
  for (int mb = 0; mb < KQ_MB; ++mb) {
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int r = 0; r < 4; ++r) mine[(4 * g + r) * RED_RS + 72 * h + 16 * w + 8 * hf + c] = acc[mb][w][hf][r];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8 / KQ_Q; ++i) {
      const int r16 = (16 / KQ_Q) * q + (lane >> 5) + 2 * i;
      const int crow = s_crow[mb * 16 + r16];
      f32x4 v = {0, 0, 0, 0};
#pragma unroll
      for (int qq = 0; qq < KQ_Q; ++qq) v += *(const f32x4*)(slabs + (qq * 2 + wn) * (16 * RED_RS) + r16 * RED_RS + fpos);
      if (p.splits > 1) {
        if (crow >= 0)
          *(f32x4*)(p.ctmp + (((int64_t)(strip * mtiles + mt) * p.splits + split) * KQ_BM + mb * 16 + r16) * KQ_TN +
                    wn * 128 + fc4) = v;
      } else if (fcol_ok && crow >= 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = v[j] * cs[j] + bs[j];
        u32x2 o;
        if constexpr (DT == DT_F16)
          o = u32x2{pack_f16(v[0], v[1]), pack_f16(v[2], v[3])};
        else
          o = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
        *(u32x2*)((uint16_t*)p.C + (int64_t)crow * p.N + ncol) = o;
      }
    }
    __syncthreads();
  }
}

// Second pass of a split-K launch: adds the splits' partial tiles in split order, then channel scale, bias and
// conversion as kq_kernel's own epilogue.  One workgroup per (tile, 16-row block); thread -> 4 columns of 4 rows.
template <int DT, bool CHANNEL, int MB = 4>
__global__ __launch_bounds__(256) void kq_reduce_kernel(const KParams p) {
  constexpr int KQ_BM = 16 * MB;
  const int t = threadIdx.x;
  const int mtiles = (p.M + KQ_BM - 1) / KQ_BM;
  const int tile = blockIdx.x / MB, rb = blockIdx.x % MB;
  const int mt = tile % mtiles, strip = tile / mtiles;
  const int fc4 = (t & 63) * 4;
  const int ncol = (p.strip0 + strip) * KQ_TN + fc4;
  if (ncol >= p.N) return;
  const uint16_t* Sc = (const uint16_t*)p.S;
  const uint16_t* bias = (const uint16_t*)p.bias;
  float cs[4] = {1.f, 1.f, 1.f, 1.f}, bs[4] = {0.f, 0.f, 0.f, 0.f};
  {
    const int base = ncol & ~31, cl = ncol & 31;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (CHANNEL) {
        const uint16_t sv = Sc[base + single_perm_pos(cl + j)];
        cs[j] = (DT == DT_F16) ? f16_lo_f32(sv) : bf16_lo_f32(sv);
      }
      if (bias) {
        const uint16_t bv = bias[base + single_perm_pos(cl + j)];
        bs[j] = (DT == DT_F16) ? f16_lo_f32(bv) : bf16_lo_f32(bv);
      }
    }
  }
  const float* parts = p.ctmp + (int64_t)tile * p.splits * (KQ_BM * KQ_TN) + fc4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = rb * 16 + (t >> 6) + 4 * i;
    const int crow = mt * KQ_BM + r;
    if (crow >= p.M) continue;
    f32x4 v = {0, 0, 0, 0};
    for (int sidx = 0; sidx < p.splits; ++sidx) v += *(const f32x4*)(parts + ((int64_t)sidx * KQ_BM + r) * KQ_TN);
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = v[j] * cs[j] + bs[j];
    u32x2 o;
    if constexpr (DT == DT_F16)
      o = u32x2{pack_f16(v[0], v[1]), pack_f16(v[2], v[3])};
    else
      o = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
    *(u32x2*)((uint16_t*)p.C + (int64_t)crow * p.N + ncol) = o;
  }
}

typedef void (*kq_fn)(const KParams);

template <int DT, int MB, int Q>
static kq_fn pick_kq(bool zp, bool channel) {
  if (zp) return channel ? kq_kernel<DT, true, true, MB, Q> : kq_kernel<DT, true, false, MB, Q>;
  return channel ? kq_kernel<DT, false, true, MB, Q> : kq_kernel<DT, false, false, MB, Q>;
}
template <int DT, int MB>
static kq_fn pick_kq_reduce(bool channel) {
  return channel ? kq_reduce_kernel<DT, true, MB> : kq_reduce_kernel<DT, false, MB>;
}

int launch_kq(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream) {
  const bool zp = a->b_zeros != nullptr, channel = pl.gm == GM_CHANNEL;
  const bool tall = pl.mb == 8;  // 128 x 256 tiles with K in halves; otherwise 64 x 256 with K in quarters
  const int parts = tall ? 2 : 4;
  if ((a->wtype != W4A16_WTYPE_U4B8 && a->wtype != W4A16_WTYPE_U4) || (a->flags & (W4A16_F_ZP_FLOAT | W4A16_F_MOE)) ||
      pl.gm == GM_GIDX || pl.use_perm || pl.splits < 1 || pl.kps * pl.splits != pl.total_ksteps ||
      pl.kps % (4 * parts) != 0 || pl.tn != KQ_TN || (pl.mb != 4 && pl.mb != 8))
    return fail(W4A16_EINVAL, "unsupported kernel variant");
  const bool f16 = a->dtype == DT_F16;
  const kq_fn fn = tall ? (f16 ? pick_kq<DT_F16, 8, 2>(zp, channel) : pick_kq<DT_BF16, 8, 2>(zp, channel))
                        : (f16 ? pick_kq<DT_F16, 4, 4>(zp, channel) : pick_kq<DT_BF16, 4, 4>(zp, channel));
  const int smem = tall ? kq_smem(8, 2) : kq_smem(4, 4);
  KParams p = make_kparams(a, pl);
  if (pl.tiles <= 0) return 0;
  W4A16_HIP(allow_dynamic_lds((const void*)fn, smem));
  hipLaunchKernelGGL(fn, dim3((unsigned)((int64_t)pl.tiles * pl.splits)), dim3(128 * parts), smem, stream, p);
  W4A16_HIP(hipGetLastError());
  if (pl.splits > 1) {
    const kq_fn red = tall ? (f16 ? pick_kq_reduce<DT_F16, 8>(channel) : pick_kq_reduce<DT_BF16, 8>(channel))
                           : (f16 ? pick_kq_reduce<DT_F16, 4>(channel) : pick_kq_reduce<DT_BF16, 4>(channel));
    hipLaunchKernelGGL(red, dim3((unsigned)pl.tiles * pl.mb), dim3(256), 0, stream, p);
    W4A16_HIP(hipGetLastError());
  }
  return 0;
}

}  // namespace w4a16
