// Host side of the W4A16 GEMM entry points: argument checks in the spirit of the reference's
// gptq_marlin_gemm / moe_wna16_marlin_gemm hosts (csrc/quantization/gptq_marlin/gptq_marlin.cu:674-959,
// csrc/moe/marlin_moe_wna16/ops.cu:691-993), launch planning, kernel dispatch.
#include <stdlib.h>

#include "gemm_kernels.h"

namespace w4a16 {

// Planner overrides for tuning runs exist only in builds made with -DW4A16_TUNING: W4A16_SPLITS, W4A16_TN and
// W4A16_KIND (0 general, 1 decode, 2 prefill, 3 64-row, 5 64-row with in-workgroup K split) force the K split count, the
// decode tile width and the kernel kind, W4A16_NW (4 or 8) the wavefronts per workgroup of the 16-row kernels;
// W4A16_DEBUG=1 prints the chosen plan to stderr, =2 every candidate.
// The shipped library reads no environment variable and prints nothing.
#ifdef W4A16_TUNING
static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : dflt;
}
#endif

static int validate(const w4a16_gemm_args* a) {
  W4A16_CHECK(a != nullptr, "null args");
  W4A16_CHECK(a->struct_size == sizeof(w4a16_gemm_args), "w4a16_gemm_args size mismatch: got %u, expected %zu",
              a->struct_size, sizeof(w4a16_gemm_args));
  W4A16_CHECK(a->dtype == W4A16_DTYPE_F16 || a->dtype == W4A16_DTYPE_BF16,
              "gpt_marlin_gemm only supports bfloat16 and float16");
  W4A16_CHECK(a->wtype == W4A16_WTYPE_U4B8 || a->wtype == W4A16_WTYPE_U4 || a->wtype == W4A16_WTYPE_U8B128 ||
                  a->wtype == W4A16_WTYPE_FE4M3 || a->wtype == W4A16_WTYPE_FE2M1,
              "unsupported b_q_type");
  W4A16_CHECK(a->size_m >= 0 && a->size_n > 0 && a->size_k > 0, "bad problem size");
  W4A16_CHECK(a->size_k % 32 == 0, "size_k = %lld is not divisible by 32", (long long)a->size_k);
  W4A16_CHECK(a->size_n % 64 == 0, "size_n = %lld is not divisible by tile_n_size = 64", (long long)a->size_n);
  W4A16_CHECK(a->size_n < (1LL << 30) && a->size_k < (1LL << 30) && a->size_m < (1LL << 30), "problem too large");
  if (a->size_m == 0) return 0;
  W4A16_CHECK(a->a && a->c && a->b_q_weight && a->b_scales, "null operand pointer");
  W4A16_CHECK(a->lda % 8 == 0, "A.stride(0) must be divisible by 8");
  W4A16_CHECK(((uintptr_t)a->a & 15) == 0, "A must be 16-byte aligned");
  W4A16_CHECK(a->lda >= a->size_k, "A.stride(0) smaller than size_k");
  W4A16_CHECK(a->num_groups >= 1, "b_scales must have at least one row");
  const bool has_zp = a->b_zeros != nullptr;
  if (has_zp)
    W4A16_CHECK(a->wtype == W4A16_WTYPE_U4, "b_q_type must be uint4 when has_zp = True");
  else
    W4A16_CHECK(a->wtype == W4A16_WTYPE_U4B8 || a->wtype == W4A16_WTYPE_U8B128 || a->wtype == W4A16_WTYPE_FE4M3 ||
                    a->wtype == W4A16_WTYPE_FE2M1,
                "b_q_type must be uint4b8, uint8b128, float8_e4m3fn or float4_e2m1f when has_zp = False");
  if (a->wtype == W4A16_WTYPE_FE2M1) {
    const int64_t gs = a->num_groups > 0 && a->size_k % a->num_groups == 0 ? a->size_k / a->num_groups : 0;
    W4A16_CHECK(gs == 16 || gs == 32, "float4_e2m1f only supports group_size == 16 (NVFP4) and group_size == 32 (MXFP4)");
    W4A16_CHECK(a->g_idx == nullptr, "Unsupported shapes: act-order with float4_e2m1f weights");
    // scale bytes of two k-tiles (NVFP4) or two k-steps (MXFP4) are interleaved: whole pairs only
    W4A16_CHECK(a->num_groups % 2 == 0, "float4_e2m1f: the number of scale groups must be even");
    if (gs == 16)
      W4A16_CHECK(a->global_scale != nullptr, "the global_scale parameter must be passed for nvfp4 format.");
    else
      W4A16_CHECK(a->global_scale == nullptr, "global_scale can only be used for nvfp4 format.");
    if (gs == 32)
      W4A16_CHECK(a->dtype == W4A16_DTYPE_BF16, "MXFP4 (group_size == 32) needs bfloat16 activations");
  } else {
    W4A16_CHECK(a->global_scale == nullptr, "global_scale can only be used for nvfp4 format.");
  }
  if (a->wtype == W4A16_WTYPE_FE4M3) {
    // the reference instantiates fp8 weights for channel-wise and group-128 scales without act-order
    // (csrc/quantization/gptq_marlin/gptq_marlin.cu:266-300 COMMON / BIGGROUP cases); any whole group size is accepted here
    W4A16_CHECK(a->g_idx == nullptr,
                "Unsupported shapes: MNK = [%lld, %lld, %lld], has_act_order = 1 with float8_e4m3fn weights",
                (long long)a->size_m, (long long)a->size_n, (long long)a->size_k);
  }
  W4A16_CHECK((a->g_idx == nullptr) == (a->perm == nullptr),
              "g_idx and perm must both be given (act-order) or both be empty");
  if (a->flags & W4A16_F_ZP_FLOAT) {
    W4A16_CHECK(has_zp, "float zero points requested but b_zeros is null");
    W4A16_CHECK(a->dtype == W4A16_DTYPE_F16, "Computation type must be float16 (half) when using float zero points.");
    if (a->flags & W4A16_F_MOE)
      return fail(W4A16_ENOTIMPL, "float zero points are not implemented for the MoE op in this build");
    // the reference instantiates float zero points for group size 64 without act-order only
    // (csrc/quantization/gptq_marlin/gptq_marlin.cu:364-379)
    W4A16_CHECK(a->g_idx == nullptr && a->num_groups > 0 && a->size_k == a->num_groups * 64,
                "Unsupported shapes: MNK = [%lld, %lld, %lld], has_act_order = %d, num_groups = %lld, is_zp_float = 1 "
                "(float zero points need group_size = 64 and no act-order)",
                (long long)a->size_m, (long long)a->size_n, (long long)a->size_k, a->g_idx != nullptr,
                (long long)a->num_groups);
  }
  if (a->flags & (W4A16_F_SILU_AND_MUL | W4A16_F_SUM_TOPK))
    W4A16_CHECK((a->flags & W4A16_F_MOE) != 0, "the fused SiLU-and-mul / top-k sum epilogues exist for the MoE GEMM only");
  if (a->flags & W4A16_F_SILU_AND_MUL) {
    W4A16_CHECK(a->size_n % 128 == 0, "fused SiLU-and-mul: size_n = %lld must be 2 * d with d a multiple of 64",
                (long long)a->size_n);
    W4A16_CHECK(!(a->flags & W4A16_F_SUM_TOPK), "fused SiLU-and-mul and the top-k sum cannot be combined");
  }
  if (a->flags & W4A16_F_SUM_TOPK)
    W4A16_CHECK(a->sum_top_k == 1 || a->sum_top_k == 2, "fused top-k sum: sum_top_k = %d must be 1 or 2", a->sum_top_k);
  if (a->zero_fill)
    W4A16_CHECK((a->flags & W4A16_F_MOE) != 0, "zero_fill is a side job of the MoE GEMM only");
  if (a->zero_fill)
    W4A16_CHECK(a->zero_fill_bytes >= 0 && a->zero_fill_bytes % 16 == 0 && ((uintptr_t)a->zero_fill & 15) == 0,
                "zero_fill must be 16-byte aligned and a multiple of 16 bytes long");
  if (a->flags & W4A16_F_MOE) {
    W4A16_CHECK(a->sorted_token_ids && a->expert_ids && a->num_tokens_past_padded, "null MoE index pointer");
    W4A16_CHECK(a->moe_block_size == 8 || (a->moe_block_size % 16 == 0 && a->moe_block_size >= 16 &&
                                           a->moe_block_size <= 64),
                "unsupported moe_block_size=%d", a->moe_block_size);
    W4A16_CHECK(a->top_k >= 1, "top_k must be >= 1");
    W4A16_CHECK(a->lda == a->size_k, "A is not contiguous");
    if (a->flags & W4A16_F_MUL_TOPK_WEIGHTS) W4A16_CHECK(a->topk_weights, "topk_weights is null");
    W4A16_CHECK(a->n_sorted >= 0, "bad sorted_token_ids length");
  }
  return 0;
}

static int make_plan(const w4a16_gemm_args* a, Plan& pl) {
  const bool act_order = a->g_idx != nullptr;
  const bool k_full = (a->flags & W4A16_F_IS_K_FULL) != 0;
  pl.use_perm = act_order;
  pl.group_ksteps = 1;
  if (act_order && !k_full) {
    W4A16_CHECK(a->b_zeros == nullptr, "act-order with partial groups does not support zero points");
    pl.gm = GM_GIDX;
  } else if (a->wtype == W4A16_WTYPE_FE2M1) {
    // one 16-byte scale record per lane and k-step (NVFP4: its two k-tiles) or per two k-steps (MXFP4)
    pl.gm = GM_GROUPED;
    pl.group_ksteps = a->size_k / a->num_groups == 16 ? 1 : 2;
  } else if (a->num_groups > 1) {
    W4A16_CHECK(a->size_k % a->num_groups == 0, "size_k = %lld, is not divisible by b_scales.size(0) = %lld",
                (long long)a->size_k, (long long)a->num_groups);
    const int64_t gs = a->size_k / a->num_groups;
    W4A16_CHECK(gs % 32 == 0, "Unsupported group_size = %lld", (long long)gs);
    pl.gm = GM_GROUPED;
    pl.group_ksteps = (int)(gs / 32);
  } else {
    W4A16_CHECK(!(act_order && k_full), "For act_order, num_groups must be > 1");
    pl.gm = GM_CHANNEL;
  }

  const bool moe = (a->flags & W4A16_F_MOE) != 0;
  // 8-bit weights and float zero points run on the general (skinny) kernel only
  const bool general_only = a->wtype == W4A16_WTYPE_U8B128 || a->wtype == W4A16_WTYPE_FE4M3 ||
                            a->wtype == W4A16_WTYPE_FE2M1 ||
                            (a->flags & W4A16_F_ZP_FLOAT) != 0;
  // ... except that the prefill kernel also has 8-bit (uint8b128, fp8), fp4 and float-zero-point instantiations
  const bool w8 = a->wtype == W4A16_WTYPE_U8B128 || a->wtype == W4A16_WTYPE_FE4M3;
  const bool fat_ok = !general_only || w8 || a->wtype == W4A16_WTYPE_FE2M1 || (a->flags & W4A16_F_ZP_FLOAT);
  // the 64-row kernel has instantiations for all of them
  const bool mid_ok = !general_only || a->wtype == W4A16_WTYPE_FE2M1 || w8 || ((a->flags & W4A16_F_ZP_FLOAT) && !moe);
  const bool pow2_group = (pl.group_ksteps & (pl.group_ksteps - 1)) == 0;  // prefill / 64-row kernels shift
  if (moe) {
    const int bs = a->moe_block_size;
    pl.mb = bs <= 16 ? 1 : bs <= 32 ? 2 : 4;
    pl.bm = 16 * pl.mb;
    pl.mtiles = (int)ceil_div(a->n_sorted, bs);
  } else {
    pl.mb = a->size_m <= 16 ? 1 : a->size_m <= 32 ? 2 : 4;
    pl.bm = 16 * pl.mb;
    pl.mtiles = (int)ceil_div(a->size_m, pl.bm);
  }
  pl.total_ksteps = (int)(a->size_k / 32);
  const int cus = num_cus();
#ifdef W4A16_TUNING
  static const int forced_splits = env_int("W4A16_SPLITS", 0);
  static const int forced_tn = env_int("W4A16_TN", 0);
  static const int forced_kind = env_int("W4A16_KIND", -1);
  static const int debug_plan = env_int("W4A16_DEBUG", 0);
  static const int forced_nw = env_int("W4A16_NW", 0);
#else
  constexpr int forced_splits = 0, forced_tn = 0, forced_kind = -1, debug_plan = 0, forced_nw = 0;
#endif

  // Dense act-order: A's columns are gathered once into a_tmp by permute_cols (as the reference's
  // permute_cols_kernel, csrc/quantization/gptq_marlin/gptq_marlin.cu:68-120), so the GEMM kernels read A with
  // plain 128-bit loads.  MoE: rows and per-expert column order are gathered together, one row of a_tmp per sorted
  // slot (moe_gather_rows), and the kernels read row `slot` instead of row id / top_k.
  pl.atmp_bytes = act_order ? (moe ? a->n_sorted : a->size_m) * a->size_k * 2 : 0;
  // Prefill kernel: dense, at least one full 128-row tile's worth of rows, K a multiple of 128.
  const int64_t fat_tiles = ceil_div(a->size_m, 128) * ceil_div(a->size_n, 512);
  // ... unless the same problem cut into 64-row tiles finishes sooner.  In units of one 128 x 512 tile's time (measured):
  // a round of 128-row tiles costs 1 (0.6 when its trailing strips are handed to the 64-row kernel); 64-row tiles cost
  // 0.75 with one workgroup per compute unit and 1.15 per pair with two.  (2048 x 4096: 128 tiles of 128 rows leave
  // half the compute units idle, 256 tiles of 64 rows do not: 99 -> 75 us at K = 4096.)
  const bool kq_types = !general_only && !w8 && a->wtype != W4A16_WTYPE_FE2M1 && !(a->flags & W4A16_F_ZP_FLOAT);
  bool prefer_mid = false;
  if (fat_tiles >= cus / 2 && forced_kind < 0 && mid_ok && !w8) {  // (the unit costs below are the 4-bit kernels')
    const int64_t mt128 = ceil_div(a->size_m, 128), tail = fat_tiles % cus;
    const bool handoff = fat_tiles >= cus && tail > 0 && ceil_div(tail, mt128) * ceil_div(a->size_m, 64) <= cus;
    const double fat_units = (double)(fat_tiles / cus) + (tail == 0 ? 0.0 : handoff ? 0.7 : 1.0);
    const int64_t mid_tiles = ceil_div(a->size_m, 64) * ceil_div(a->size_n, 512), rem = mid_tiles % (2 * cus);
    const double mid_units = 1.15 * (double)(mid_tiles / (2 * cus)) + (rem == 0 ? 0.0 : rem <= cus ? 0.75 : 1.15);
    prefer_mid = mid_units < 0.95 * fat_units;
  }
  // 128 x 256 tiles with the K halves inside the workgroup (gemm_kq.hip, MB = 8): the prefill kernel's operand reuse for
  // problems whose 128 x 512 tiles would leave half the compute units idle.  One round only.
  {
    const int64_t tall_tiles = ceil_div(a->size_m, 128) * ceil_div(a->size_n, 256);
    const bool tall_shape = !moe && kq_types && pow2_group && pl.gm != GM_GIDX && a->size_k % 256 == 0 && a->size_m > 128;
    const bool tall_pays = tall_tiles <= cus && tall_tiles * 4 >= cus * 3;
    if (tall_shape && (forced_kind == 6 || (forced_kind < 0 && tall_pays))) {
      pl.kind = 5;
      pl.tn = 256;
      pl.mb = 8;
      pl.bm = 128;
      pl.mtiles = (int)ceil_div(a->size_m, 128);
      pl.ncp = (int)ceil_div(a->size_n, 256);
      W4A16_CHECK(tall_tiles < (1LL << 31) / 64, "too many tiles");
      pl.tiles = (int)tall_tiles;
      pl.splits = 1;
      pl.kps = pl.total_ksteps;
      pl.xcd_map = 0;
      pl.ctmp_bytes = 0;
      if (debug_plan)
        fprintf(stderr, "[w4a16] M=%lld N=%lld K=%lld kind=5 (128 x 256) tiles=%d\n", (long long)a->size_m,
                (long long)a->size_n, (long long)a->size_k, pl.tiles);
      return 0;
    }
  }
  if (!moe && fat_ok && pow2_group && a->size_m >= 128 && !prefer_mid && (fat_tiles >= cus / 2 || forced_kind == 2) && a->size_k % 128 == 0 &&
      pl.gm != GM_GIDX && forced_kind != 0 && forced_kind != 1 && forced_kind != 3 && forced_kind != 5) {
    pl.kind = 2;
    pl.tn = 512;
    pl.mb = 8;
    pl.bm = 128;
    pl.mtiles = (int)ceil_div(a->size_m, 128);
    pl.ncp = (int)ceil_div(a->size_n, 512);
    const int64_t tiles = (int64_t)pl.mtiles * pl.ncp;
    W4A16_CHECK(tiles < (1LL << 31) / 64, "too many tiles");
    pl.tiles = (int)tiles;
    pl.splits = 1;
    pl.kps = pl.total_ksteps;
    pl.xcd_map = 0;
    pl.ctmp_bytes = 0;
    // One workgroup fills a compute unit, so tiles run in rounds of `cus`.  The strips that reach into a partly filled
    // last round (tiles are ordered M first) go to the 64-row kernel instead when it can hold them with one workgroup
    // per compute unit: that takes about 0.75 of a round instead of a whole one.
    {
      const int64_t rounds = tiles / cus, tail = tiles - rounds * cus;
      const int64_t strips = ceil_div(tail, (int64_t)pl.mtiles);
      if (rounds >= 1 && tail > 0 && strips < pl.ncp && forced_kind != 2) {
        // ... or, better, to 128 x 256 tiles whose K halves run on the four wavefronts of one workgroup (the operand reuse
        // of the prefill kernel, half a round) when those fit one round
        if (kq_types && a->size_k % 256 == 0 && 2 * strips * pl.mtiles <= cus) {
          pl.tail_strips = (int)strips;
          pl.tail_kind = 5;
        } else if (strips * ceil_div(a->size_m, 64) <= cus && mid_ok) {
          pl.tail_strips = (int)strips;
          pl.tail_kind = 3;
        }
      }
    }
    return 0;
  }

  // 64-row tiles of 256 columns with the K range cut in four inside the workgroup (one workgroup per compute unit).
  {
    const bool kq_shape = !moe && !general_only && pow2_group && pl.gm != GM_GIDX && a->size_k % 512 == 0 && a->size_m > 32;
    // measured against the alternatives (16-row tiles, general kernel): ahead by 13-25 % at 33..128 rows when its tiles
    // give between 3/4 and all of the compute units a workgroup (4096 x 28672: 45 / 44 us at 96 / 128 rows against
    // 54 / 58; 8192 x 57344: 75-82 us at 33-64 rows against 87-101), level at 1.75 rounds, behind with fewer tiles
    const int64_t kq_tiles = ceil_div(a->size_m, 64) * ceil_div(a->size_n, 256);
    // Above 128 rows (layers too narrow for the prefill kernel's 128 x 512 tiles): against the 64 x 512 kernel these
    // tiles win whenever they fit one round (4096 x 4096 at 1024 rows: 44 against 59 us); against the general kernel's
    // 64 x 128 tiles once those need a second round (4096 x 6144 at 384 rows: 38 against 50 us).  With a long K and
    // few tiles, K is also split across workgroups while every wavefront keeps at least 24 k-steps (14336 x 4096 at
    // 192..512 rows: 5-9 % ahead of the general kernel; with shorter splits the fixed costs of the two launches win).
    int kq_sp = 1;
    const int64_t gen_tiles = ceil_div(a->size_m, 64) * ceil_div(a->size_n, 128);
    const bool kq_tall = a->size_m > 128 && kq_tiles <= cus;
    if (kq_tall)
      while (kq_sp < 8 && kq_tiles * kq_sp * 2 <= cus && pl.total_ksteps % (32 * kq_sp) == 0 &&
             pl.total_ksteps / (8 * kq_sp) >= 24)
        kq_sp *= 2;
    if (forced_splits > 0 && forced_kind == 5 && pl.total_ksteps % (16 * forced_splits) == 0) kq_sp = forced_splits;
    const bool kq_pays = (a->size_m <= 128 && kq_tiles >= cus * 3 / 4 && kq_tiles <= cus) ||
                         (kq_tall && kq_tiles * kq_sp >= cus / 2 && (kq_sp > 1 || gen_tiles > cus));
    if (kq_shape && (forced_kind == 5 || (forced_kind < 0 && kq_pays))) {
      pl.kind = 5;
      pl.tn = 256;
      pl.mb = 4;
      pl.bm = 64;
      pl.mtiles = (int)ceil_div(a->size_m, 64);
      pl.ncp = (int)ceil_div(a->size_n, 256);
      const int64_t tiles = (int64_t)pl.mtiles * pl.ncp;
      W4A16_CHECK(tiles * kq_sp < (1LL << 31) / 64, "too many tiles");
      pl.tiles = (int)tiles;
      pl.splits = kq_sp;
      pl.kps = pl.total_ksteps / kq_sp;
      pl.xcd_map = 0;
      pl.ctmp_bytes = kq_sp > 1 ? tiles * kq_sp * 64 * 256 * 4 : 0;
      if (debug_plan)
        fprintf(stderr, "[w4a16] M=%lld N=%lld K=%lld kind=5 tiles=%d splits=%d kps=%d\n", (long long)a->size_m,
                (long long)a->size_n, (long long)a->size_k, pl.tiles, pl.splits, pl.kps);
      return 0;
    }
  }

  // 64-row kernel: MoE blocks of 64 slots, and dense problems with too few rows or tiles for the prefill kernel.
  // It holds two workgroups per compute unit; with fewer tiles than that, K is split (>= 32 k-steps per split, in
  // multiples of 4) and a second small kernel adds the partial tiles (~2 us launch + the partials' traffic).
  {
    const int64_t mid_mtiles = moe ? ceil_div(a->n_sorted, 64) : ceil_div(a->size_m, 64);
    const int64_t mid_tiles = mid_mtiles * ceil_div(a->size_n, 512);
    int sp = 1;
    // 8-bit weights at 65..128 rows: the general kernel would stream the (twice as large) weights once per 64-row tile;
    // two K splits of the 64-row kernel win from cus/4 tiles on (gate_up, 96 / 128 rows: 81 / 85 -> 66 / 67 us)
    const bool w8_two_tiles = w8 && !moe && a->size_m > 64 && a->size_m <= 128 && mid_tiles >= cus / 4 && mid_tiles < cus / 2;
    // (measured: worth it from about cus/2 tiles up to 3/4 cus dense, up to cus for MoE, whose tile count is an upper bound)
    if (w8_two_tiles) {
      sp = 2;
    } else if ((mid_tiles >= cus / 2 || forced_kind == 3) && mid_tiles < (moe ? cus : cus * 3 / 4)) {
      const int by_k = pl.total_ksteps / 32;
      const int by_cus = (int)(2 * cus / mid_tiles);
      sp = by_k < by_cus ? by_k : by_cus;
      if (sp < 1) sp = 1;
      if (sp > 16) sp = 16;
    }
    // MoE: the number of live tiles is only known on the device, which then splits K for the tiles of the last, partly
    // filled round of resident workgroups (two per compute unit); see tail_split
    const bool tail_dyn = moe && forced_splits <= 0 && pl.total_ksteps >= 3 * TAIL_MIN_KSTEPS;  // (else it never splits)
    if (tail_dyn) sp = 1;
    if (forced_splits > 0) sp = forced_splits;
    int kps = (int)ceil_div(pl.total_ksteps, sp);
    kps = (kps + 3) / 4 * 4;
    sp = (int)ceil_div(pl.total_ksteps, kps);
    const bool mid_shape = mid_ok && pow2_group && a->size_k % 128 == 0 && pl.gm != GM_GIDX &&
                           (moe ? a->moe_block_size == 64
                                : (a->size_m > 32 && (mid_tiles >= cus / 2 || w8_two_tiles ||
                                                      (forced_kind == 3 && mid_tiles >= cus / 16))));
    if ((mid_shape && forced_kind < 0) || (forced_kind == 3 && mid_shape)) {
      W4A16_CHECK(mid_tiles * sp < (1LL << 31) / 64, "too many tiles");
      pl.kind = 3;
      pl.tn = 512;
      pl.mb = 4;
      pl.bm = 64;
      pl.mtiles = (int)mid_mtiles;
      pl.ncp = (int)ceil_div(a->size_n, 512);
      pl.tiles = (int)mid_tiles;
      pl.splits = sp;
      pl.kps = kps;
      pl.xcd_map = 0;
      pl.ctmp_bytes = sp > 1 ? mid_tiles * sp * 64 * 512 * 4 : 0;
      if (tail_dyn) {
        pl.dyn_slots = (int)(2 * cus);
        pl.ctmp_bytes = mid_tail_pieces(mid_tiles, pl.dyn_slots) * 64 * 512 * 4;
      }
      if (debug_plan)
        fprintf(stderr, "[w4a16] M=%lld N=%lld K=%lld kind=3 tiles=%d splits=%d kps=%d dyn=%d\n", (long long)a->size_m,
                (long long)a->size_n, (long long)a->size_k, pl.tiles, pl.splits, pl.kps, pl.dyn_slots);
      return 0;
    }
  }

  // The decode kernel handles 16-row tiles whose scale groups span whole stages of 64 K rows.
  const bool decode_shape = !general_only && pl.gm != GM_GIDX && pl.total_ksteps % 2 == 0 &&
                            (pl.gm == GM_CHANNEL || (pl.group_ksteps % 2 == 0 && pow2_group)) && forced_kind != 0;

  // Launch-shape choice by a small cost model (microseconds) fitted to MI355X measurements of these
  // kernels.  One 8-wavefront workgroup sustains ~33 GB/s on a 128-column strip and ~20 GB/s on a 64-column
  // strip with 16-row tiles (instruction-issue bound), ~12 / ~9 GB/s with 32- / 64-row tiles (dequantisation
  // per element); the whole chip ~4.7 TB/s; summing K-splits across workgroups adds ~1.5 us of dependent
  // device-scope round trips plus the last workgroup's pass over the partial tiles.  Only one such workgroup
  // fits a compute unit, so a grid larger than the number of compute units runs in rounds.  Each split needs
  // >= 1 stage per wavefront and one workspace counter per tile.
  // Dense problems of up to 128 rows may also run as several 16-row tiles of the decode kernel: the weight strip
  // is then re-read from L2 by every row tile, but there is no per-element dequantisation and no K split.
  struct Cand { int kind, tn, splits, mb; double t; };
  Cand best{0, 128, 1, pl.mb, 1e30};
  const int natural_mb = pl.mb;
  for (int mi = 0; mi < 2; ++mi) {
    const int mb = mi == 0 ? natural_mb : 1;
    if (mi == 1 && (natural_mb == 1 || moe || a->size_m > 128 || !decode_shape)) continue;
    const bool decode_ok = mb == 1 && decode_shape;
    const int64_t mtiles = moe ? pl.mtiles : ceil_div(a->size_m, 16 * mb);
    const int n_tn = decode_ok ? 2 : 1;
    for (int ti = 0; ti < n_tn; ++ti) {
      const int tn = ti == 0 ? 128 : 64;
      if (forced_tn && tn != forced_tn && decode_ok) continue;
      if (tn == 64 && (a->flags & W4A16_F_SILU_AND_MUL)) continue;  // gate and up n-tiles are paired in 128-column tiles
      const int64_t ncol_tiles = ceil_div(a->size_n, tn);
      const int64_t tiles = mtiles * ncol_tiles;
      if (tiles <= 0 || tiles >= (1LL << 31) / 64) continue;
      const double bytes = (double)tiles * a->size_k * tn / 2.0;
      const double wg_rate = mb == 1 ? (tn == 64 ? 20e3 : 33e3) : mb == 2 ? 12e3 : 9e3;  // bytes per us
      const double chip_rate = 4.7e6;
      const double t_xchg = 2.2;
      const int unit = decode_ok ? 16 : 8;  // k-steps per split needed to give every wavefront work
      const int max_splits = pl.total_ksteps / unit > 0 ? pl.total_ksteps / unit : 1;
      for (int sp = 1; sp <= 16; ++sp) {
        if (sp > max_splits) break;
        if (sp > 1 && (!a->workspace || tiles > a->workspace_len)) break;
        if (forced_splits > 0 && sp != (forced_splits < max_splits ? forced_splits : max_splits)) continue;
        const int64_t wgs = tiles * sp;
        if (sp > 1 && wgs > cus) break;
        const int64_t rounds = ceil_div(wgs, cus);
        const double rate = (double)wgs / (double)rounds * wg_rate;  // workgroups resident at a time
        // the last workgroup of a tile re-reads every split's partial tile at about one workgroup's stream rate
        const double t_fix = sp > 1 ? t_xchg + sp * (double)(16 * mb * tn * 4) / 20e3 : 0.0;
        // HBM sees every weight byte once; further row tiles re-read the strips, from L2 at about twice that rate when
        // the whole weight fits the eight 4 MB L2s (down_proj at 64 rows: 128-column tiles with two splits take 22 us,
        // 64-column tiles without 27), else at the same rate again (gate_up: 2 row tiles cost 28 us, not 19)
        const double unique = (double)ncol_tiles * a->size_k * tn / 2.0;
        const double t_mem = unique / chip_rate + (bytes - unique) / (unique <= 32e6 ? 9.2e6 : chip_rate);
        const double t_wg = bytes / rate;
        const double t = (t_wg > t_mem ? t_wg : t_mem) + t_fix;
        if (debug_plan >= 2)
          fprintf(stderr, "[w4a16]   cand kind=%d tn=%d mb=%d tiles=%lld sp=%d: wg %.2f mem %.2f fix %.2f -> %.2f\n", decode_ok ? 1 : 0,
                  tn, mb, (long long)tiles, sp, t_wg, t_mem, t_fix, t);
        if (t < best.t) best = Cand{decode_ok ? 1 : 0, tn, sp, mb, t};
      }
    }
  }
  W4A16_CHECK(best.t < 1e30, "no launch shape for this problem (too many tiles)");
  pl.kind = best.kind;
  pl.tn = best.tn;
  if (!moe) {
    pl.mb = best.mb;
    pl.bm = 16 * pl.mb;
    pl.mtiles = (int)ceil_div(a->size_m, pl.bm);
  }
  pl.ncp = (int)ceil_div(a->size_n, pl.tn);
  pl.tiles = pl.mtiles * pl.ncp;
  {
    const int align = pl.kind == 1 ? 2 : 1;  // decode stages are two k-steps
    int kps = (int)ceil_div(pl.total_ksteps, best.splits);
    kps = (kps + align - 1) / align * align;
    pl.kps = kps;
    pl.splits = (int)ceil_div(pl.total_ksteps, kps);
  }
  // 16-row tiles, more workgroups than compute units -> 4-wavefront workgroups, two to a compute unit
  pl.nw = forced_nw ? forced_nw
          : ((pl.kind == 1 || (pl.kind == 0 && pl.mb == 1)) && (int64_t)pl.tiles * pl.splits > cus) ? 4 : 8;
  if (debug_plan)
    fprintf(stderr, "[w4a16] M=%lld N=%lld K=%lld kind=%d tn=%d mb=%d tiles=%d splits=%d kps=%d nw=%d model_us=%.2f\n",
            (long long)a->size_m, (long long)a->size_n, (long long)a->size_k, pl.kind, pl.tn, pl.mb, pl.tiles,
            pl.splits, pl.kps, pl.nw, best.t);
  pl.xcd_map = (pl.splits > 1 && pl.tiles % 8 == 0) ? 1 : 0;
  pl.ctmp_bytes = pl.splits > 1 ? (int64_t)pl.tiles * pl.splits * pl.bm * pl.tn * 4 : 0;
  return 0;
}

}  // namespace w4a16

using namespace w4a16;

extern "C" int64_t w4a16_gemm_scratch_bytes(const w4a16_gemm_args* args) {
  if (int rc = validate(args)) return rc;
  if (args->size_m == 0) return 0;
  Plan pl;
  if (int rc = make_plan(args, pl)) return rc;
  return ((pl.ctmp_bytes + 255) & ~255LL) + pl.atmp_bytes;
}

// Launches the planned kernels; `args` already carries the scratch (c_tmp) and counter (workspace) pointers to use.
static int run_planned(const w4a16_gemm_args* args, Plan& pl, void* stream) {
  w4a16_gemm_args b = *args;
  if (pl.atmp_bytes > 0) {
    void* a_tmp = (char*)args->c_tmp + ((pl.ctmp_bytes + 255) & ~255LL);
    if (args->flags & W4A16_F_MOE) {
      if (int rc = moe_gather_rows(args, a_tmp, (hipStream_t)stream)) return rc;
      pl.a_by_slot = true;
    } else {
      if (int rc = w4a16_permute_cols(args->a, args->perm, a_tmp, args->size_m, args->size_k, args->lda, stream)) return rc;
    }
    b.a = a_tmp;
    b.lda = args->size_k;
    pl.use_perm = false;
  }
  if (pl.kind == 2) {
    if (pl.tail_strips == 0) return launch_fat(&b, pl, (hipStream_t)stream);
    Plan head = pl, tail = pl;
    head.ncp = pl.ncp - pl.tail_strips;
    head.tiles = head.ncp * pl.mtiles;
    if (int rc = launch_fat(&b, head, (hipStream_t)stream)) return rc;
    if (pl.tail_kind == 5) {  // 128 x 256 tiles, K halves inside the workgroup
      tail.kind = 5;
      tail.tn = 256;
      tail.ncp = 2 * pl.tail_strips;
      tail.tiles = tail.mtiles * tail.ncp;
      tail.strip0 = 2 * head.ncp;
      return launch_kq(&b, tail, (hipStream_t)stream);
    }
    tail.kind = 3;
    tail.mb = 4;
    tail.bm = 64;
    tail.mtiles = (int)ceil_div(args->size_m, 64);
    tail.ncp = pl.tail_strips;
    tail.tiles = tail.mtiles * tail.ncp;
    tail.strip0 = head.ncp;
    return launch_mid(&b, tail, (hipStream_t)stream);
  }
  if (pl.kind == 3) return launch_mid(&b, pl, (hipStream_t)stream);
  if (pl.kind == 5) return launch_kq(&b, pl, (hipStream_t)stream);
  return pl.kind == 1 ? launch_decode(&b, pl, (hipStream_t)stream) : launch_skinny(&b, pl, (hipStream_t)stream);
}

extern "C" int w4a16_marlin_gemm(const w4a16_gemm_args* args, void* stream) {
  if (int rc = validate(args)) return rc;
  if (args->size_m == 0) return 0;
  Plan pl;
  if (int rc = make_plan(args, pl)) return rc;
  if (pl.mtiles == 0) return 0;
  if (pl.ctmp_bytes + pl.atmp_bytes > 0)
    W4A16_CHECK(args->c_tmp != nullptr, "c_tmp is null but %lld bytes are needed",
                (long long)(pl.ctmp_bytes + pl.atmp_bytes));
  return run_planned(args, pl, stream);
}

// ---------------------------------------------------------------- the entry point that allocates nothing
// Split-K partial tiles, the column-gathered copy of A (act-order) and the tiles' arrival counters live in one array
// in the library's own device memory: W4A16_STATIC_SCRATCH_BYTES of data followed by STATIC_COUNTERS counters.
// Every GPU the library runs on holds its own copy at its own address; host code only ever uses the address that
// hipGetSymbolAddress returned for the current device.
namespace w4a16 {
constexpr int64_t STATIC_COUNTERS = 4096;
static __device__ __align__(256) unsigned char scratch[W4A16_STATIC_SCRATCH_BYTES + STATIC_COUNTERS * 4];

static int static_scratch(unsigned char** out) {
  static std::mutex mu;
  static unsigned char* ptrs[64] = {nullptr};
  int dev = 0;
  W4A16_HIP(hipGetDevice(&dev));
  W4A16_CHECK(dev >= 0 && dev < 64, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    W4A16_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    W4A16_CHECK(p != nullptr, "hipGetSymbolAddress returned a null address for the static scratch");
    ptrs[dev] = (unsigned char*)p;
  }
  *out = ptrs[dev];
  return 0;
}

__global__ void clear_counters_kernel(int32_t* counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0;
}
}  // namespace w4a16

extern "C" int w4a16_marlin_gemm_static(const w4a16_gemm_args* args, void* stream) {
  if (int rc = validate(args)) return rc;
  if (args->size_m == 0) return 0;
  unsigned char* base = nullptr;
  if (int rc = static_scratch(&base)) return rc;
  w4a16_gemm_args b = *args;
  b.c_tmp = (float*)base;
  b.workspace = (int32_t*)(base + W4A16_STATIC_SCRATCH_BYTES);
  b.workspace_len = STATIC_COUNTERS;
  Plan pl;
  if (int rc = make_plan(&b, pl)) return rc;
  if (pl.mtiles == 0) return 0;
  const int64_t need = ((pl.ctmp_bytes + 255) & ~255LL) + pl.atmp_bytes;
  W4A16_CHECK(need <= (int64_t)W4A16_STATIC_SCRATCH_BYTES,
              "w4a16_marlin_gemm_static: this problem needs %lld bytes of scratch, the library's static buffer holds "
              "%lld; use w4a16_marlin_gemm with a caller-owned c_tmp",
              (long long)need, (long long)W4A16_STATIC_SCRATCH_BYTES);
  if (pl.splits > 1 && (pl.kind == 0 || pl.kind == 1)) {
    // arrival counters must start at zero; a fill kernel rather than a memset node, so that the call can be captured
    const KParams kp = make_kparams(&b, pl);
    const int n = pl.tiles * kp.lock_stride;
    W4A16_CHECK(n <= STATIC_COUNTERS, "w4a16_marlin_gemm_static: %d arrival counters needed, %lld available", n,
                (long long)STATIC_COUNTERS);
    hipLaunchKernelGGL(clear_counters_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, b.workspace, n);
    W4A16_HIP(hipGetLastError());
  }
  return run_planned(&b, pl, stream);
}
