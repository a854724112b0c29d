// Host side of the W4A16 GEMM entry points: argument checks in the spirit of the reference's
// gptq_marlin_gemm / moe_wna16_marlin_gemm hosts (csrc/quantization/gptq_marlin/gptq_marlin.cu:674-959,
// csrc/moe/marlin_moe_wna16/ops.cu:691-993), launch planning, kernel dispatch.
#include <stdlib.h>

#include "gemm_plan.h"

namespace w4a16 {

static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : dflt;
}

static int validate(const w4a16_gemm_args* a) {
  W4A16_CHECK(a != nullptr, "null args");
  W4A16_CHECK(a->struct_size == sizeof(w4a16_gemm_args), "w4a16_gemm_args size mismatch: got %u, expected %zu",
              a->struct_size, sizeof(w4a16_gemm_args));
  W4A16_CHECK(a->dtype == W4A16_DTYPE_F16 || a->dtype == W4A16_DTYPE_BF16,
              "gpt_marlin_gemm only supports bfloat16 and float16");
  W4A16_CHECK(a->wtype == W4A16_WTYPE_U4B8 || a->wtype == W4A16_WTYPE_U4, "unsupported b_q_type");
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
    W4A16_CHECK(a->wtype == W4A16_WTYPE_U4B8, "b_q_type must be uint4b8 when has_zp = False");
  W4A16_CHECK((a->g_idx == nullptr) == (a->perm == nullptr),
              "g_idx and perm must both be given (act-order) or both be empty");
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
  pl.ncp = (int)ceil_div(a->size_n, 128);
  const int64_t tiles = (int64_t)pl.mtiles * pl.ncp;
  W4A16_CHECK(tiles < (1LL << 31) / 64, "too many tiles");
  pl.tiles = (int)tiles;
  pl.total_ksteps = (int)(a->size_k / 32);

  // One workgroup (8 wavefronts) per compute unit: split K until the grid covers the chip, keeping at
  // least one k-step per wavefront.  Splitting needs one counter per tile in the caller's workspace.
  static const int forced_splits = env_int("W4A16_SPLITS", 0);
  static const int target_mult = env_int("W4A16_TARGET_WG_PER_CU", 1);
  const int target = num_cus() * target_mult;
  int splits = 1;
  if (pl.tiles > 0 && pl.tiles < target && a->workspace && pl.tiles <= a->workspace_len) {
    splits = (target + pl.tiles / 2) / pl.tiles;
    const int max_splits = pl.total_ksteps / 8 > 0 ? pl.total_ksteps / 8 : 1;
    if (forced_splits > 0) splits = forced_splits;
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
  }
  pl.kps = (int)ceil_div(pl.total_ksteps, splits);
  pl.splits = (int)ceil_div(pl.total_ksteps, pl.kps);
  pl.xcd_map = (pl.splits > 1 && pl.tiles % 8 == 0) ? 1 : 0;
  pl.ctmp_bytes = pl.splits > 1 ? (int64_t)pl.tiles * pl.splits * pl.bm * 128 * 4 : 0;
  return 0;
}

}  // namespace w4a16

using namespace w4a16;

extern "C" int64_t w4a16_gemm_scratch_bytes(const w4a16_gemm_args* args) {
  if (int rc = validate(args)) return rc;
  if (args->size_m == 0) return 0;
  Plan pl;
  if (int rc = make_plan(args, pl)) return rc;
  return pl.ctmp_bytes;
}

extern "C" int w4a16_marlin_gemm(const w4a16_gemm_args* args, void* stream) {
  if (int rc = validate(args)) return rc;
  if (args->size_m == 0) return 0;
  Plan pl;
  if (int rc = make_plan(args, pl)) return rc;
  if (pl.mtiles == 0) return 0;
  if (pl.ctmp_bytes > 0) W4A16_CHECK(args->c_tmp != nullptr, "c_tmp is null but %lld bytes are needed", (long long)pl.ctmp_bytes);
  return launch_skinny(args, pl, (hipStream_t)stream);
}
