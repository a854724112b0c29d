// Launch plan shared between the host entry point and the kernel launchers.
#pragma once
#include "gemm_common.h"

namespace w4a16 {

struct Plan {
  int gm;            // GM_*: how scale rows are found
  int group_ksteps;  // GM_GROUPED: group_size / 32
  bool use_perm;     // gather A columns through perm (act-order)
  bool a_by_slot = false;  // MoE: A already holds one row per sorted slot (act-order gather done in front of the GEMM)
  int mb, bm;        // m-blocks of 16 rows per tile, rows per tile
  int mtiles, ncp, tiles;
  int total_ksteps, splits, kps;  // k-steps of 32 rows; K splits; k-steps per split
  int xcd_map;
  int kind;  // 0: skinny kernel, 1: decode kernel, 2: prefill ("fat") kernel, 3: 64-row ("mid") kernel,
             // 5: in-workgroup K split (gemm_kq.hip): 64 x 256 tiles in K quarters (mb = 4), 128 x 256 in halves (mb = 8)
  int tn;    // tile width in columns (128; the decode kernel also has 64)
  int nw = 8;  // 16-row tiles (decode kernel, general kernel with one m-block): wavefronts per workgroup (8 or 4)
  int strip0 = 0;      // 64-row kernel / K-split kernel: first 512- / 256-column strip handled by the launch
  int dyn_slots = 0;   // 64-row kernel, MoE: resident workgroups that the device-side K split of the tail tiles fills
  int tail_strips = 0; // prefill plan: trailing 512-column strips handed to another kernel (0 = none)
  int tail_kind = 3;   // ... which one: 3 = 64-row kernel, 5 = 128 x 256 tiles with the K halves inside the workgroup
  int64_t ctmp_bytes;  // fp32 split-K partials
  int64_t atmp_bytes;  // column-permuted copy of A (act-order), after the partials; MoE: one row per sorted slot
};

// MoE act-order: out[slot, :] = a[sorted_ids[slot] / top_k, perm[expert of the slot's block][:]] for the valid slots
// (gemm.hip runs it in front of the GEMM kernels, which then read row `slot`).
int moe_gather_rows(const w4a16_gemm_args* a, void* out, hipStream_t stream);

// 64-row kernel, MoE: upper bound of the tail pieces (tail_split) for a launch of `tiles` tiles at most
inline int64_t mid_tail_pieces(int64_t tiles, int slots) { return tiles * 8 < slots ? tiles * 8 : slots; }

int launch_skinny(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream);
int launch_decode(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream);
int launch_fat(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream);
int launch_mid(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream);
int launch_kq(const w4a16_gemm_args* a, const Plan& pl, hipStream_t stream);

}  // namespace w4a16
