/*
 * w4a16_gfx950.h — C ABI of the MI355X (gfx950) weight-only int4 GEMM library.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void*; NULL = the default stream), launches asynchronously on
 * that stream, never synchronises the host, and returns 0 on success or a
 * negative W4A16_E* code.  After a failure w4a16_last_error() returns a
 * message worded like the reference's TORCH_CHECK texts (thread-local).
 * The caller owns every buffer.  Nothing here allocates device memory.
 *
 * Each function names the reference operator it stands in for.
 */
#ifndef W4A16_GFX950_H
#define W4A16_GFX950_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define W4A16_ABI_VERSION 3

enum {
  W4A16_OK = 0,
  W4A16_EINVAL = -1,   /* shape / argument check failed (reference: TORCH_CHECK)     */
  W4A16_ENOTIMPL = -2, /* valid in the reference, not built here (e.g. fp4 weights)  */
  W4A16_EHIP = -3      /* a HIP runtime call failed                                  */
};

/* weight types (decoded from the reference's ScalarType ids by the host layer,
 * vllm/scalar_type.py:136-164, csrc/core/scalar_type.hpp:143-160) */
enum {
  W4A16_WTYPE_U4B8 = 0,
  W4A16_WTYPE_U4 = 1,
  W4A16_WTYPE_U8B128 = 2,
  /* float8_e4m3fn bytes in the 8-bit Marlin layout; b_scales carry the exponent offset the reference folds in at
     load time (marlin_utils_fp8.py:25-37: x 2^8 for fp16, x 2^120 for bf16); no zero points, no act-order */
  W4A16_WTYPE_FE4M3 = 3,
  /* float4_e2m1f codes in the 4-bit Marlin layout.  b_scales holds one byte per (group, column) in the order the
     reference's nvfp4_marlin_process_scales / mxfp4_marlin_process_scales produce
     (marlin_utils_fp4.py:28-79): group size 16 (NVFP4): scale * 2^7 as unsigned E5M3, with global_scale;
     group size 32 (MXFP4, bf16 only): E8M0.  No zero points, no act-order */
  W4A16_WTYPE_FE2M1 = 4
};
/* activation / output / scale element type */
enum { W4A16_DTYPE_F16 = 0, W4A16_DTYPE_BF16 = 1, W4A16_DTYPE_F32 = 2 /* router logits only */ };

int w4a16_abi_version(void);
const char* w4a16_last_error(void);

/* Replaces torch.ops._C.gptq_marlin_repack
 * (csrc/quantization/gptq_marlin/gptq_marlin_repack.cu:251-322, schema csrc/torch_bindings.cpp:327-329).
 * b_q_weight: int32 [size_k/8, size_n] GPTQ packing (nibble i of word (r,n) = q[8r+i, n]);
 *             num_bits = 8: int32 [size_k/4, size_n], byte i of word (r,n) = q[4r+i, n].
 * perm: int32 [size_k] source-row order (act-order) or NULL.
 * out: int32 [size_k/16, 2*size_n] Marlin layout (num_bits = 8: [size_k/16, 4*size_n]). */
int w4a16_gptq_marlin_repack(const uint32_t* b_q_weight, const int32_t* perm, uint32_t* out,
                             int64_t size_k, int64_t size_n, int num_bits, void* stream);

/* Replaces torch.ops._C.awq_marlin_repack
 * (csrc/quantization/gptq_marlin/awq_marlin_repack.cu:189-248, schema csrc/torch_bindings.cpp:333-335).
 * b_q_weight: int32 [size_k, size_n/8] AWQ packing (nibble t of word (k,c) = q[k, 8c+{0,2,4,6,1,3,5,7}[t]]);
 *             num_bits = 8: int32 [size_k, size_n/4], byte t of word (k,c) = q[k, 4c+{0,2,1,3}[t]]. */
int w4a16_awq_marlin_repack(const uint32_t* b_q_weight, uint32_t* out, int64_t size_k,
                            int64_t size_n, int num_bits, void* stream);

/* Replaces torch.ops._C.permute_cols (csrc/permute_cols.cu:14-88, schema csrc/torch_bindings.cpp:312):
 * out[m, k] = a[m, perm[k]] for 16-bit elements; a has row stride lda (elements), out is dense. */
int w4a16_permute_cols(const void* a, const int32_t* perm, void* out, int64_t size_m,
                       int64_t size_k, int64_t lda, void* stream);

/* Replaces the load-time helper marlin_permute_scales / marlin_permute_bias
 * (vllm/model_executor/layers/quantization/utils/marlin_utils.py:278-305), which the reference runs as torch index
 * ops.  s, out: 16-bit elements [num_rows, size_n], size_n a multiple of 64.  grouped != 0: the 8 x 8 transpose inside
 * every 64-column chunk (group scales); grouped == 0: the "single" permutation inside every 32-column chunk
 * (channel-wise scales, bias). */
int w4a16_marlin_permute_scales(const void* s, void* out, int64_t num_rows, int64_t size_n, int grouped,
                                void* stream);

/* Replaces the load-time helpers marlin_zero_points / awq_to_marlin_zero_points (marlin_utils.py:326-370), which the
 * reference runs in numpy on the host (quant_utils.py:548-602).  out: int32 [num_groups, size_n/8], Marlin packing.
 * format 0: zp int32 [num_groups, size_n/8], nibble j of word c = column 8c + j (what
 *           unpack_cols(x.t()) of MarlinLinearKernel.process_weights_after_loading starts from, marlin.py:115-133);
 * format 1: the same shape in AWQ packing (column 8c + j in nibble {0,4,1,5,2,6,3,7}[j]);
 * format 2: unpacked int32 [num_groups, size_n] (the argument of marlin_zero_points). */
int w4a16_marlin_zero_points(const uint32_t* zp, uint32_t* out, int64_t num_groups, int64_t size_n, int format,
                             void* stream);

/* Operands of one W4A16 GEMM  C[M,N] = A[M,K] * dequant(Bq)[K,N] (+ bias).
 * Mirrors the tensor arguments of torch.ops._C.gptq_marlin_gemm
 * (csrc/quantization/gptq_marlin/gptq_marlin.cu:674-959, schema csrc/torch_bindings.cpp:316-323)
 * and, when the moe_* fields are set, of torch.ops._moe_C.moe_wna16_marlin_gemm
 * (csrc/moe/marlin_moe_wna16/ops.cu:691-993, schema csrc/moe/torch_bindings.cpp:63-75). */
typedef struct w4a16_gemm_args {
  uint32_t struct_size;       /* sizeof(w4a16_gemm_args), checked                         */
  int32_t dtype;              /* W4A16_DTYPE_*: element type of a, c, b_scales, b_bias    */
  int32_t wtype;              /* W4A16_WTYPE_*                                            */
  int32_t flags;              /* W4A16_F_* bits                                           */
  const void* a;              /* [size_m, size_k], row stride lda elements, 16-B aligned  */
  int64_t lda;
  void* c;                    /* [size_m(*top_k), size_n] dense                           */
  const uint32_t* b_q_weight; /* [E,] [size_k/16, 2*size_n] Marlin layout                 */
  const void* b_scales;       /* [E,] [num_groups, size_n] Marlin-permuted                */
  const uint32_t* b_zeros;    /* [E,] [num_groups, size_n/8] Marlin-packed, or NULL;
                                 with W4A16_F_ZP_FLOAT: fp16 [num_groups, size_n]        */
  const int32_t* g_idx;       /* [E,] [size_k] sorted group of each Marlin row, or NULL   */
  const int32_t* perm;        /* [E,] [size_k] act-order column gather for a, or NULL     */
  const void* b_bias;         /* [E,] [size_n] Marlin-permuted bias, or NULL              */
  float* c_tmp;               /* fp32 scratch, >= w4a16_gemm_scratch_bytes(); may be NULL
                                 when that returns 0                                      */
  int32_t* workspace;         /* int32 counters, all zero on entry, all zero on exit      */
  int64_t workspace_len;      /* elements                                                 */
  int64_t size_m, size_n, size_k;
  int64_t num_groups;         /* rows of b_scales (per expert)                            */
  /* ---- fused-MoE variant (all NULL/0 for the dense op) ---- */
  const int32_t* sorted_token_ids;       /* [n_sorted]  (pad value >= size_m*top_k)       */
  const int32_t* expert_ids;             /* [ceil(n_sorted/moe_block_size)], -1 = skip    */
  const int32_t* num_tokens_past_padded; /* [1] device scalar                             */
  const float* topk_weights;             /* flat, indexed by sorted token id              */
  int64_t n_sorted;
  int32_t moe_block_size;     /* 8 or a multiple of 16 in [16, 64]                        */
  int32_t top_k;
  int32_t num_experts;
  int32_t reserved;
  const void* global_scale;   /* NVFP4 only: [E,] one element of the activation type, as the reference's
                                 nvfp4_marlin_process_global_scale leaves it (marlin_utils_fp4.py:82-93:
                                 x 2^7 for fp16, x 2^119 for bf16); NULL otherwise            */
  /* ---- fused MoE epilogues (no counterpart in the reference's operator, which runs them as separate launches:
     fused_marlin_moe.py:47-183, csrc/activation_kernels.cu:85, csrc/moe/moe_align_sum_kernels.cu:375) ---- */
  void* zero_fill;            /* optional side job of the launch: zero_fill_bytes bytes (a multiple of 16, 16-byte
                                 aligned) at this address are set to zero; must not overlap any operand of the call */
  int64_t zero_fill_bytes;
  int32_t sum_top_k;          /* W4A16_F_SUM_TOPK: result row i is added into c[i / sum_top_k]                     */
  int32_t reserved2;
} w4a16_gemm_args;

enum {
  W4A16_F_IS_K_FULL = 1,        /* act-order: groups are whole on this shard              */
  W4A16_F_USE_ATOMIC_ADD = 2,   /* accepted; the split-K reduction here is always ordered */
  W4A16_F_USE_FP32_REDUCE = 4,  /* accepted; partial sums are always fp32                 */
  W4A16_F_MUL_TOPK_WEIGHTS = 8, /* MoE: scale each output row by its routing weight       */
  W4A16_F_MOE = 16,
  W4A16_F_ZP_FLOAT = 32,        /* b_zeros holds fp16 zero points [num_groups, size_n], Marlin-permuted like the
                                   scales (HQQ; reference is_zp_float, gptq_marlin.cu:866-880): w = q*s - zp*s.
                                   fp16, uint4, group size 64, dense op only */
  W4A16_F_SILU_AND_MUL = 64,    /* MoE only: the weights hold gate | up column halves (size_n = 2 * d, d % 64 == 0);
                                   c is [size_m * top_k, d] and receives silu(gate) * up, rounded exactly as
                                   silu_and_mul does on the rounded GEMM result (each of gate, up, silu, product
                                   rounded once to the activation type) */
  W4A16_F_SUM_TOPK = 128        /* MoE only: c is [size_m / sum_top_k, size_n], zero on entry (zero_fill of an earlier
                                   launch on the same stream can do that); every result row i, rounded to the
                                   activation type, is added to c[i / sum_top_k] with packed 16-bit atomic adds.
                                   sum_top_k <= 2 (a sum of two rounded terms does not depend on their order) */
};

/* Bytes of fp32 scratch (c_tmp) a call with these operands may use (0 = none).
 * The reference allocates the equivalent inside the op (gptq_marlin.cu:751-763). */
int64_t w4a16_gemm_scratch_bytes(const w4a16_gemm_args* args);

/* Replaces torch.ops._C.gptq_marlin_gemm / torch.ops._moe_C.moe_wna16_marlin_gemm (see above). */
int w4a16_marlin_gemm(const w4a16_gemm_args* args, void* stream);

/* The same GEMM for callers that cannot allocate device memory (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc).  No counterpart in the reference, whose op allocates c_tmp and a_tmp itself
 * (gptq_marlin.cu:751-763).  args->c_tmp, args->workspace and args->workspace_len are ignored: split-K partial
 * tiles, the column-gathered copy of A (act-order) and the arrival counters live in a buffer of
 * W4A16_STATIC_SCRATCH_BYTES (+ 16 KiB of counters) inside the library's own device memory: resident on every GPU of
 * every process that loads the library, whether or not this entry point is ever called, until the process ends.
 * A problem that needs more scratch than that (w4a16_gemm_scratch_bytes says how much) fails with W4A16_EINVAL and a
 * message; nothing is launched then.  The call allocates and frees nothing.  All calls on one GPU share that GPU's
 * buffer: calls that overlap in time on one GPU (two streams, two host threads) race and must be serialised by the
 * caller.  Inputs and the output are the caller's, as in w4a16_marlin_gemm, and results are identical to those of
 * w4a16_marlin_gemm called with a workspace of 4096 counters (the launch plan looks at the workspace length: a shorter
 * workspace can rule out a K split).  MoE calls whose 64-row tiles may split K on the device ask for the buffer's
 * whole size in partial tiles when the tile count is large; add the act-order copy of A and they are refused. */
#define W4A16_STATIC_SCRATCH_BYTES (64u << 20)
int w4a16_marlin_gemm_static(const w4a16_gemm_args* args, void* stream);

/* Replaces torch.ops._moe_C.moe_align_block_size
 * (csrc/moe/moe_align_sum_kernels.cu:275-346, schema csrc/moe/torch_bindings.cpp:17-23).
 * topk_ids int32 [numel]; sorted_token_ids int32 [sorted_len] (pre-filled with numel by this call);
 * expert_ids int32 [expert_ids_len] (tail zero-filled); num_tokens_post_pad int32 [1]. */
int w4a16_moe_align_block_size(const int32_t* topk_ids, int64_t numel, int32_t num_experts,
                               int32_t block_size, int32_t* sorted_token_ids, int64_t sorted_len,
                               int32_t* expert_ids, int64_t expert_ids_len,
                               int32_t* num_tokens_post_pad, void* stream);

/* Replaces torch.ops._moe_C.batched_moe_align_block_size
 * (csrc/moe/moe_align_sum_kernels.cu:18-80, 348-373, schema csrc/moe/torch_bindings.cpp:27-34): alignment for
 * activations already batched per expert.  batch_num_tokens int32 [num_batches <= 1024];
 * sorted_ids int32 [num_batches * round_up(max_tokens_per_batch, block_size)] (pad value num_batches *
 * max_tokens_per_batch); block_ids int32 [that / block_size] (-1 past the last block); num_tokens_post_pad int32 [1]. */
int w4a16_batched_moe_align_block_size(int64_t max_tokens_per_batch, int32_t block_size,
                                       const int32_t* batch_num_tokens, int32_t num_batches, int32_t* sorted_ids,
                                       int64_t sorted_len, int32_t* block_ids, int64_t block_ids_len,
                                       int32_t* num_tokens_post_pad, void* stream);

/* Replaces torch.ops._moe_C.moe_sum (csrc/moe/moe_align_sum_kernels.cu:375-416, schema
 * csrc/moe/torch_bindings.cpp:13): out[t, :] = sum_k in[t, k, :], 16-bit elements, fp32 sum. */
int w4a16_moe_sum(const void* in, void* out, int64_t tokens, int32_t top_k, int64_t hidden,
                  int32_t dtype, void* stream);

/* Replaces torch.ops._C.silu_and_mul (csrc/activation_kernels.cu:22-32,85; schema
 * csrc/torch_bindings.cpp:118): out[t, j] = silu(in[t, j]) * in[t, d + j]. */
int w4a16_silu_and_mul(const void* in, void* out, int64_t tokens, int64_t d, int32_t dtype,
                       void* stream);

/* Replaces torch.ops._moe_C.topk_softmax (csrc/moe/topk_softmax_kernels.cu:676-705, schema
 * csrc/moe/torch_bindings.cpp:6-8): fp32 softmax over num_experts router logits per token (fp16 / bf16 / fp32),
 * top-k by repeated arg-max (ties: lowest index), weights optionally renormalised to sum to 1;
 * token_expert_indices[t, k] = k * num_tokens + t.  All outputs [num_tokens, topk]. */
int w4a16_topk_softmax(const void* gating_output, int32_t gating_dtype, float* topk_weights,
                       int32_t* topk_ids, int32_t* token_expert_indices, int64_t num_tokens,
                       int32_t num_experts, int32_t topk, int32_t renormalize, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* W4A16_GFX950_H */
