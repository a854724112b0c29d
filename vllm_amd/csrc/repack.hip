// Checkpoint -> Marlin-layout repack kernels (4-bit, and a simple 8-bit variant), written for gfx950.
//
// Output layout (int32 [K/16, 2N]): for k-tile kt (16 rows) and n-tile nt (64 cols) the 128
// words nt*128 + th*4 + w (th in [0,32), w in [0,4)) hold, with r = 2*(th%4), c = th/4,
// n0 = 64*nt + 16*w + c, k0 = 16*kt + r, the nibbles
//   j:   0        1        2          3          4        5        6          7
//   q[k0,n0] q[k0+8,n0] q[k0,n0+8] q[k0+8,n0+8] q[k0+1,n0] q[k0+9,n0] q[k0+1,n0+8] q[k0+9,n0+8]
// which is the layout produced by the reference's gptq_marlin_repack / awq_marlin_repack
// (csrc/quantization/gptq_marlin/gptq_marlin_repack.cu:107-204, awq_marlin_repack.cu:68-148)
// and by its numpy statement (marlin_utils_test.py:32-93).
//
// One workgroup of 256 threads produces the 256 output words of (one k-tile) x (two n-tiles,
// 128 columns).  The source words of that 16 x 128 patch are staged in LDS with coalesced
// loads, then each thread assembles one output word, so global reads and writes are both
// contiguous per wavefront.  The work is pure HBM streaming: K*N/2 bytes in, K*N/2 bytes out.
#include "common.h"

namespace w4a16 {

// nibble j of the output word takes source row k0 + DK[j], column n0 + DN[j]
__device__ __constant__ const int kDK[8] = {0, 8, 0, 8, 1, 9, 1, 9};
// k-tiles one workgroup of the 4-bit repack kernels walks through (16 KB of output per workgroup)
constexpr int KT_PER_WG = 16;
// ... of the 512-column kernels: as many as leave about 2048 workgroups (between 2 and 16)
static int wide_kt_per_wg(int64_t size_k, int64_t size_n) {
  const int64_t kt = (size_k / 16) * ((size_n + 511) / 512) / 2048;
  return kt < 2 ? 2 : kt > KT_PER_WG ? KT_PER_WG : (int)kt;
}

// GPTQ source: word (r, n), nibble i = q[8r + i, n].  Without perm a k-tile is two source rows.
template <bool HAS_PERM>
__global__ __launch_bounds__(256) void gptq_repack_kernel(const uint32_t* __restrict__ in,
                                                          const int32_t* __restrict__ perm,
                                                          uint32_t* __restrict__ out, int size_k,
                                                          int size_n) {
  // LDS: 16 logical rows x 128 columns of source words (HAS_PERM) or 2 x 128 (plain).
  __shared__ uint32_t tile[HAS_PERM ? 16 : 2][128];
  __shared__ int src_row[16];
  const int t = threadIdx.x;
  const int ncol0 = blockIdx.x * 128;
  const int ncols = min(128, size_n - ncol0);  // 64 or 128
  const int kt_end = min((int)(blockIdx.y + 1) * KT_PER_WG, size_k / 16);
  for (int kt = blockIdx.y * KT_PER_WG; kt < kt_end; ++kt) {
  __syncthreads();  // the previous k-tile's LDS reads are done

  if (HAS_PERM) {
    if (t < 16) src_row[t] = perm[kt * 16 + t];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = i * 2 + (t >> 7);
      const int col = t & 127;
      if (col < ncols) tile[row][col] = in[(size_t)(src_row[row] >> 3) * size_n + ncol0 + col];
    }
  } else {
    const int row = t >> 7, col = t & 127;
    if (col < ncols) tile[row][col] = in[(size_t)(kt * 2 + row) * size_n + ncol0 + col];
  }
  __syncthreads();

  const int nt = t >> 7;        // n-tile inside the 128-column span
  const int th = (t >> 2) & 31; // "thread" of the Marlin fragment
  const int w = t & 3;
  if (nt * 64 < ncols) {
  const int r = 2 * (th & 3);
  const int c = th >> 2;
  const int n0 = nt * 64 + 16 * w + c;
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int kk = r + kDK[j];                 // row inside the k-tile
    const int nn = n0 + ((j >> 1) & 1) * 8;
    uint32_t src;
    int nib;
    if (HAS_PERM) {
      src = tile[kk][nn];
      nib = src_row[kk] & 7;
    } else {
      src = tile[kk >> 3][nn];
      nib = kk & 7;
    }
    word |= ((src >> (4 * nib)) & 0xFu) << (4 * j);
  }
  out[(size_t)kt * (2 * size_n) + (size_t)(blockIdx.x * 2 + nt) * 128 + th * 4 + w] = word;
  }
  }
}

// GPTQ source without a row permutation, layers of at least 512 columns: a workgroup walks kt_per_wg k-tiles of a
// 512-column span, reads the two source rows of a k-tile (2 KB contiguous each) with 16-byte loads, the next k-tile's in
// flight while this one is assembled, and stores 16 bytes per thread: thread t makes the four words (w = 0..3) of Marlin
// thread t % 32 in n-tile t / 32.
__global__ __launch_bounds__(256) void gptq_repack_wide_kernel(const uint32_t* __restrict__ in,
                                                               uint32_t* __restrict__ out, int size_k,
                                                               int size_n, int kt_per_wg) {
  using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
  __shared__ __align__(16) uint32_t tile[2][512];
  const int t = threadIdx.x;
  const int ncol0 = blockIdx.x * 512;
  const int ncols = min(512, size_n - ncol0);  // a multiple of 64
  const int kt_begin = blockIdx.y * kt_per_wg, kt_end = min(kt_begin + kt_per_wg, size_k / 16);
  const int row = t >> 7, c4 = (t & 127) * 4;
  const bool ld_on = c4 < ncols;
  const uint32_t* src = in + (size_t)row * size_n + ncol0 + c4;
  const size_t kt_stride = (size_t)2 * size_n;
  const int nt = t >> 5, th = t & 31;
  const bool st_on = nt * 64 < ncols;
  const int r = 2 * (th & 3), c = th >> 2;
  u32x4 cur = {0, 0, 0, 0};
  if (ld_on && kt_begin < kt_end) cur = *(const u32x4*)(src + kt_begin * kt_stride);
  for (int kt = kt_begin; kt < kt_end; ++kt) {
    u32x4 nxt = {0, 0, 0, 0};
    if (ld_on && kt + 1 < kt_end) nxt = *(const u32x4*)(src + (kt + 1) * kt_stride);
    __syncthreads();  // the previous k-tile's LDS reads are done
    if (ld_on) *(u32x4*)&tile[row][c4] = cur;
    __syncthreads();
    if (st_on) {
      u32x4 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int kk = r + kDK[j];
          const uint32_t sw = tile[kk >> 3][nt * 64 + 16 * w + c + ((j >> 1) & 1) * 8];
          word |= ((sw >> (4 * (kk & 7))) & 0xFu) << (4 * j);
        }
        o[w] = word;
      }
      *(u32x4*)(out + (size_t)kt * (2 * size_n) + (size_t)(blockIdx.x * 8 + nt) * 128 + th * 4) = o;
    }
    cur = nxt;
  }
}

// GPTQ source with a row permutation (act-order), layers of at least 512 columns: as above, but a k-tile gathers its 16
// rows through perm (row perm[k] lives in source word row perm[k] / 8, nibble perm[k] % 8).  The workgroup's slice of
// perm is read into LDS once; the 16 source rows' 2 KB pieces of the next k-tile are in flight (eight 16-byte loads
// per thread) while this one is assembled.
__global__ __launch_bounds__(256) void gptq_repack_perm_wide_kernel(const uint32_t* __restrict__ in,
                                                                    const int32_t* __restrict__ perm,
                                                                    uint32_t* __restrict__ out, int size_k,
                                                                    int size_n, int kt_per_wg) {
  using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
  __shared__ __align__(16) uint32_t tile[16][512];
  __shared__ int src_rows[KT_PER_WG * 16];
  const int t = threadIdx.x;
  const int ncol0 = blockIdx.x * 512;
  const int ncols = min(512, size_n - ncol0);  // a multiple of 64
  const int kt_begin = blockIdx.y * kt_per_wg, kt_end = min(kt_begin + kt_per_wg, size_k / 16);
  if (t < (kt_end - kt_begin) * 16) src_rows[t] = perm[kt_begin * 16 + t];
  __syncthreads();
  const int rh = t >> 7, c4 = (t & 127) * 4;
  const bool ld_on = c4 < ncols;
  const uint32_t* src = in + ncol0 + c4;
  const int nt = t >> 5, th = t & 31;
  const bool st_on = nt * 64 < ncols;
  const int r = 2 * (th & 3), c = th >> 2;
  u32x4 cur[8], nxt[8];
  auto load = [&](u32x4* dst, int kt) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      dst[i] = u32x4{0, 0, 0, 0};
      if (ld_on && kt < kt_end) dst[i] = *(const u32x4*)(src + (size_t)(src_rows[(kt - kt_begin) * 16 + 2 * i + rh] >> 3) * size_n);
    }
  };
  load(cur, kt_begin);
  for (int kt = kt_begin; kt < kt_end; ++kt) {
    load(nxt, kt + 1);
    __syncthreads();  // the previous k-tile's LDS reads are done
    if (ld_on) {
#pragma unroll
      for (int i = 0; i < 8; ++i) *(u32x4*)&tile[2 * i + rh][c4] = cur[i];
    }
    __syncthreads();
    if (st_on) {
      const int* rows = src_rows + (kt - kt_begin) * 16;
      u32x4 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int kk = r + kDK[j];
          const uint32_t sw = tile[kk][nt * 64 + 16 * w + c + ((j >> 1) & 1) * 8];
          word |= ((sw >> (4 * (rows[kk] & 7))) & 0xFu) << (4 * j);
        }
        o[w] = word;
      }
      *(u32x4*)(out + (size_t)kt * (2 * size_n) + (size_t)(blockIdx.x * 8 + nt) * 128 + th * 4) = o;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) cur[i] = nxt[i];
  }
}

// AWQ source: word (k, cw), nibble t = q[k, 8*cw + {0,2,4,6,1,3,5,7}[t]]  =>  column 8*cw + j sits
// in nibble {0,4,1,5,2,6,3,7}[j].
__global__ __launch_bounds__(256) void awq_repack_kernel(const uint32_t* __restrict__ in,
                                                         uint32_t* __restrict__ out, int size_k,
                                                         int size_n) {
  __shared__ uint32_t tile[16][16];  // 16 rows x 16 words (128 columns)
  const int t = threadIdx.x;
  const int ncol0 = blockIdx.x * 128;
  const int ncols = min(128, size_n - ncol0);
  const int kt_end = min((int)(blockIdx.y + 1) * KT_PER_WG, size_k / 16);
  for (int kt = blockIdx.y * KT_PER_WG; kt < kt_end; ++kt) {
  __syncthreads();  // the previous k-tile's LDS reads are done
  {
    const int row = t >> 4, cw = t & 15;
    if (cw * 8 < ncols) tile[row][cw] = in[(size_t)(kt * 16 + row) * (size_n >> 3) + (ncol0 >> 3) + cw];
  }
  __syncthreads();
  const int nt = t >> 7;
  const int th = (t >> 2) & 31;
  const int w = t & 3;
  if (nt * 64 < ncols) {
  const int r = 2 * (th & 3);
  const int c = th >> 2;
  const int n0 = nt * 64 + 16 * w + c;
  const int nib = ((c & 1) << 2) | (c >> 1);  // {0,4,1,5,2,6,3,7}[c]; n0 % 8 == c
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int kk = r + kDK[j];
    const int nn = n0 + ((j >> 1) & 1) * 8;
    const uint32_t src = tile[kk][nn >> 3];
    word |= ((src >> (4 * nib)) & 0xFu) << (4 * j);
  }
  out[(size_t)kt * (2 * size_n) + (size_t)(blockIdx.x * 2 + nt) * 128 + th * 4 + w] = word;
  }
  }
}

// The same for layers of at least 512 columns: a workgroup walks 16 k-tiles of a 512-column span, reads every source
// row's 256 contiguous bytes with 16-byte loads (the next k-tile's are in flight while this one is assembled) and
// stores 16 bytes per thread; thread t makes the four words (w = 0..3) of Marlin thread t % 32 in n-tile t / 32.
__global__ __launch_bounds__(256) void awq_repack_wide_kernel(const uint32_t* __restrict__ in,
                                                              uint32_t* __restrict__ out, int size_k,
                                                              int size_n, int kt_per_wg) {
  using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
  __shared__ __align__(16) uint32_t tile[16][64];  // 16 rows x 64 words (512 columns)
  const int t = threadIdx.x;
  const int ncol0 = blockIdx.x * 512;
  const int ncols = min(512, size_n - ncol0);  // a multiple of 64
  const int kt_begin = blockIdx.y * kt_per_wg, kt_end = min(kt_begin + kt_per_wg, size_k / 16);
  const int row = t >> 4, cw4 = (t & 15) * 4;
  const bool ld_on = cw4 * 8 < ncols;
  const uint32_t* src = in + (size_t)row * (size_n >> 3) + (ncol0 >> 3) + cw4;
  const size_t kt_stride = (size_t)16 * (size_n >> 3);
  const int nt = t >> 5, th = t & 31;
  const bool st_on = nt * 64 < ncols;
  const int r = 2 * (th & 3), c = th >> 2;
  const int nib = ((c & 1) << 2) | (c >> 1);  // {0,4,1,5,2,6,3,7}[c]
  u32x4 cur = {0, 0, 0, 0};
  if (ld_on && kt_begin < kt_end) cur = *(const u32x4*)(src + kt_begin * kt_stride);
  for (int kt = kt_begin; kt < kt_end; ++kt) {
    u32x4 nxt = {0, 0, 0, 0};
    if (ld_on && kt + 1 < kt_end) nxt = *(const u32x4*)(src + (kt + 1) * kt_stride);
    __syncthreads();  // the previous k-tile's LDS reads are done
    if (ld_on) *(u32x4*)&tile[row][cw4] = cur;
    __syncthreads();
    if (st_on) {
      u32x4 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int kk = r + kDK[j];
          const uint32_t sw = tile[kk][nt * 8 + 2 * w + ((j >> 1) & 1)];
          word |= ((sw >> (4 * nib)) & 0xFu) << (4 * j);
        }
        o[w] = word;
      }
      *(u32x4*)(out + (size_t)kt * (2 * size_n) + (size_t)(blockIdx.x * 8 + nt) * 128 + th * 4) = o;
    }
    cur = nxt;
  }
}

// 8-bit variant (uint8b128): output int32 [K/16, 4N]; per k-tile and n-tile 256 words; word
// nt*256 + th*8 + 2w + half holds the bytes q[k0 + {0, 8, 1, 9}[j], 64nt + 16w + c + 8 half], j = 0..3
// (gptq_marlin_repack.cu:119-203 with num_bits = 8).  One thread per output word; load-time only, so the
// gathers are not staged.  GPTQ source: word (r, n), byte i = q[4r + i, n]; AWQ source: word (k, cw),
// byte t = q[k, 4cw + {0, 2, 1, 3}[t]].
template <bool AWQ, bool HAS_PERM>
__global__ __launch_bounds__(256) void repack8_kernel(const uint32_t* __restrict__ in, const int32_t* __restrict__ perm,
                                                      uint32_t* __restrict__ out, int size_k, int size_n) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // output word
  const int64_t row_words = 4LL * size_n;
  if (idx >= (int64_t)(size_k / 16) * row_words) return;
  const int kt = (int)(idx / row_words);
  const int rem = (int)(idx % row_words);
  const int nt = rem >> 8, th = (rem >> 3) & 31, w = (rem >> 1) & 3, half = rem & 1;
  const int k0 = 16 * kt + 2 * (th & 3);
  const int n = 64 * nt + 16 * w + (th >> 2) + 8 * half;
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int k = k0 + ((j & 1) ? 8 : 0) + (j >> 1);  // {0, 8, 1, 9}[j]
    if (HAS_PERM) k = perm[k];
    uint32_t b;
    if (AWQ) {
      const uint32_t src = in[(size_t)k * (size_n >> 2) + (n >> 2)];
      const int pos = ((n & 1) << 1) | ((n >> 1) & 1);  // {0, 2, 1, 3}[n % 4]
      b = (src >> (8 * pos)) & 0xFFu;
    } else {
      const uint32_t src = in[(size_t)(k >> 2) * size_n + n];
      b = (src >> (8 * (k & 3))) & 0xFFu;
    }
    word |= b << (8 * j);
  }
  out[idx] = word;
}

// out[m, k] = a[m, perm[k]], 16-bit elements.
__global__ __launch_bounds__(256) void permute_cols_kernel(const uint16_t* __restrict__ a,
                                                           const int32_t* __restrict__ perm,
                                                           uint16_t* __restrict__ out, int size_m,
                                                           int size_k, int64_t lda) {
  const int m = blockIdx.y;
  for (int k = blockIdx.x * 256 + threadIdx.x; k < size_k; k += gridDim.x * 256)
    out[(size_t)m * size_k + k] = a[(size_t)m * lda + perm[k]];
}

// The same gather with rows staged in LDS: a workgroup copies one row of `a` into LDS with 16-byte loads (the next
// row's loads are in flight meanwhile), every thread then assembles 16-byte pieces of the output row from eight 2-byte
// LDS reads and stores them whole.  Global memory only sees 16-byte accesses; the random 2-byte reads hit LDS.
// grid = (row walkers, piece slices): with few rows the pieces of a row are shared out over several workgroups, each
// of which stages the whole row.  Needs size_k % 8 == 0, 16-byte aligned rows and a row that fits the LDS budget.
constexpr int PC_MAX_K = 32768;  // 64 KB of LDS
using pc_u32x4 = uint32_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void permute_cols_lds_kernel(const uint16_t* __restrict__ a,
                                                               const int32_t* __restrict__ perm,
                                                               uint16_t* __restrict__ out, int size_m, int size_k,
                                                               int64_t lda) {
  extern __shared__ __align__(16) unsigned char pc_smem[];
  uint16_t* row = (uint16_t*)pc_smem;
  const int t = threadIdx.x;
  const int pieces = size_k >> 3;                       // 16-byte pieces per row
  constexpr int MAXP = PC_MAX_K / 8 / 256;              // pieces a thread stages per row
  const int per_slice = (pieces + gridDim.y - 1) / gridDim.y;
  const int p_b = blockIdx.y * per_slice, p_e = min(p_b + per_slice, pieces);
  pc_u32x4 stage[MAXP];
  auto load_row = [&](int m) {
    const pc_u32x4* src = (const pc_u32x4*)(a + (int64_t)m * lda);
#pragma unroll
    for (int i = 0; i < MAXP; ++i)
      if (t + 256 * i < pieces) stage[i] = src[t + 256 * i];
  };
  int m = blockIdx.x;
  if (m < size_m) load_row(m);
  for (; m < size_m; m += gridDim.x) {
    __syncthreads();  // the previous row's gathers are done
#pragma unroll
    for (int i = 0; i < MAXP; ++i)
      if (t + 256 * i < pieces) ((pc_u32x4*)row)[t + 256 * i] = stage[i];
    __syncthreads();
    if (m + (int)gridDim.x < size_m) load_row(m + gridDim.x);
    pc_u32x4* dst = (pc_u32x4*)(out + (int64_t)m * size_k);
    for (int p = p_b + t; p < p_e; p += 256) {
      const pc_u32x4 i0 = *(const pc_u32x4*)(perm + 8 * p), i1 = *(const pc_u32x4*)(perm + 8 * p + 4);
      pc_u32x4 v;
      v[0] = (uint32_t)row[i0[0]] | ((uint32_t)row[i0[1]] << 16);
      v[1] = (uint32_t)row[i0[2]] | ((uint32_t)row[i0[3]] << 16);
      v[2] = (uint32_t)row[i1[0]] | ((uint32_t)row[i1[1]] << 16);
      v[3] = (uint32_t)row[i1[2]] | ((uint32_t)row[i1[3]] << 16);
      dst[p] = v;
    }
  }
}

// Scale (and bias) permutation of the Marlin layout, 16-bit elements, rows of size_n (a multiple of 64):
//   grouped:  inside every 64-column chunk, position 8i + j takes the chunk's column i + 8j (an 8 x 8 transpose);
//   single:   inside every 32-column chunk, position 8i + jj takes column 2i + (jj & 1) + 8 (jj >> 1)
// (reference marlin_utils.py:278-305).  One thread per output element pair.
__global__ __launch_bounds__(256) void permute_scales_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                             int64_t total, int grouped) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  int64_t src;
  if (grouped) {
    const int p = (int)(idx & 63);
    src = (idx & ~63LL) + (p >> 3) + 8 * (p & 7);
  } else {
    const int p = (int)(idx & 31), i = p >> 3, jj = p & 7;
    src = (idx & ~31LL) + 2 * i + (jj & 1) + 8 * (jj >> 1);
  }
  out[idx] = in[src];
}

// Zero points -> Marlin packing: output word 8ch + i of a group row (chunk ch of 64 columns), nibble t, holds the
// zero point of column 64ch + i + 8 * {0,2,4,6,1,3,5,7}[t] (reference marlin_utils.py:326-370).
// FORMAT 0: packed int32 [G, N/8], nibble j of word c = column 8c + j (compressed-tensors, transposed by the caller);
// FORMAT 1: AWQ packing, column 8c + j sits in nibble {0,4,1,5,2,6,3,7}[j]; FORMAT 2: unpacked int32 [G, N].
template <int FORMAT>
__global__ __launch_bounds__(256) void marlin_zero_points_kernel(const uint32_t* __restrict__ in, uint32_t* __restrict__ out,
                                                                 int64_t total_words, int size_n) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // output word
  if (idx >= total_words) return;
  const int words_per_row = size_n >> 3;
  const int64_t g = idx / words_per_row;
  const int wi = (int)(idx % words_per_row), ch = wi >> 3, i = wi & 7;
  uint32_t word = 0;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int m = ((t & 3) << 1) | (t >> 2);  // {0,2,4,6,1,3,5,7}[t]
    const int col = 64 * ch + i + 8 * m;
    uint32_t z;
    if (FORMAT == 2) {
      z = in[g * size_n + col] & 0xFu;
    } else {
      const uint32_t src = in[g * words_per_row + (col >> 3)];
      const int j = col & 7;
      const int nib = FORMAT == 1 ? (((j & 1) << 2) | (j >> 1)) : j;
      z = (src >> (4 * nib)) & 0xFu;
    }
    word |= z << (4 * t);
  }
  out[idx] = word;
}

static int check_repack(int64_t size_k, int64_t size_n, int num_bits) {
  W4A16_CHECK(size_k % 16 == 0, "size_k = %lld is not divisible by tile_k_size = 16", (long long)size_k);
  W4A16_CHECK(size_n % 64 == 0, "size_n = %lld is not divisible by tile_n_size = 64", (long long)size_n);
  W4A16_CHECK(num_bits == 4 || num_bits == 8, "num_bits must be 4 or 8. Got = %d", num_bits);
  W4A16_CHECK(size_k / 16 / KT_PER_WG <= 65535, "size_k = %lld too large", (long long)size_k);
  W4A16_CHECK(size_k / 16 * 4 * size_n < (1LL << 31) * 256, "problem too large");
  return 0;
}

}  // namespace w4a16

using namespace w4a16;

extern "C" int w4a16_gptq_marlin_repack(const uint32_t* b_q_weight, const int32_t* perm, uint32_t* out,
                                        int64_t size_k, int64_t size_n, int num_bits, void* stream) {
  if (int rc = check_repack(size_k, size_n, num_bits)) return rc;
  W4A16_CHECK(b_q_weight && out, "null weight pointer");
  if (size_k == 0 || size_n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (num_bits == 8) {
    const unsigned blocks = (unsigned)ceil_div(size_k / 16 * 4 * size_n, 256);
    if (perm)
      repack8_kernel<false, true><<<blocks, 256, 0, s>>>(b_q_weight, perm, out, (int)size_k, (int)size_n);
    else
      repack8_kernel<false, false><<<blocks, 256, 0, s>>>(b_q_weight, nullptr, out, (int)size_k, (int)size_n);
    W4A16_HIP(hipGetLastError());
    return 0;
  }
  if (size_n >= 512 && size_n % 4 == 0 && ((uintptr_t)b_q_weight & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    const int kt_per_wg = wide_kt_per_wg(size_k, size_n);
    dim3 wgrid((unsigned)ceil_div(size_n, 512), (unsigned)ceil_div(size_k / 16, kt_per_wg));
    if (perm)
      gptq_repack_perm_wide_kernel<<<wgrid, 256, 0, s>>>(b_q_weight, perm, out, (int)size_k, (int)size_n, kt_per_wg);
    else
      gptq_repack_wide_kernel<<<wgrid, 256, 0, s>>>(b_q_weight, out, (int)size_k, (int)size_n, kt_per_wg);
    W4A16_HIP(hipGetLastError());
    return 0;
  }
  dim3 grid((unsigned)ceil_div(size_n, 128), (unsigned)ceil_div(size_k / 16, KT_PER_WG));
  if (perm)
    gptq_repack_kernel<true><<<grid, 256, 0, s>>>(b_q_weight, perm, out, (int)size_k, (int)size_n);
  else
    gptq_repack_kernel<false><<<grid, 256, 0, s>>>(b_q_weight, nullptr, out, (int)size_k, (int)size_n);
  W4A16_HIP(hipGetLastError());
  return 0;
}

extern "C" int w4a16_awq_marlin_repack(const uint32_t* b_q_weight, uint32_t* out, int64_t size_k,
                                       int64_t size_n, int num_bits, void* stream) {
  if (int rc = check_repack(size_k, size_n, num_bits)) return rc;
  W4A16_CHECK(b_q_weight && out, "null weight pointer");
  if (size_k == 0 || size_n == 0) return 0;
  if (num_bits == 8) {
    const unsigned blocks = (unsigned)ceil_div(size_k / 16 * 4 * size_n, 256);
    repack8_kernel<true, false><<<blocks, 256, 0, (hipStream_t)stream>>>(b_q_weight, nullptr, out, (int)size_k, (int)size_n);
    W4A16_HIP(hipGetLastError());
    return 0;
  }
  if (size_n >= 512 && ((uintptr_t)b_q_weight & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    const int kt_per_wg = wide_kt_per_wg(size_k, size_n);
    dim3 grid((unsigned)ceil_div(size_n, 512), (unsigned)ceil_div(size_k / 16, kt_per_wg));
    awq_repack_wide_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(b_q_weight, out, (int)size_k, (int)size_n, kt_per_wg);
    W4A16_HIP(hipGetLastError());
    return 0;
  }
  dim3 grid((unsigned)ceil_div(size_n, 128), (unsigned)ceil_div(size_k / 16, KT_PER_WG));
  awq_repack_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(b_q_weight, out, (int)size_k, (int)size_n);
  W4A16_HIP(hipGetLastError());
  return 0;
}

extern "C" int w4a16_permute_cols(const void* a, const int32_t* perm, void* out, int64_t size_m,
                                  int64_t size_k, int64_t lda, void* stream) {
  W4A16_CHECK(a && perm && out, "null pointer");
  W4A16_CHECK(size_m <= 65535 * 1024LL, "size_m too large");
  if (size_m == 0 || size_k == 0) return 0;
  // (measured: ahead of the element-wise kernel from about 32 rows of 1024 columns on, 4 - 6 x at 512 rows and more)
  if (size_m >= 32 && size_k >= 1024 && size_k % 8 == 0 && size_k <= PC_MAX_K && lda % 8 == 0 && ((uintptr_t)a & 15) == 0 && ((uintptr_t)out & 15) == 0 &&
      ((uintptr_t)perm & 15) == 0 && size_m < (1LL << 31)) {
    const int cus = num_cus();
    // one row walker per compute unit and more; with few rows, up to 8 workgroups share a row's pieces
    const int walkers = (int)(size_m < 4 * cus ? size_m : 4 * cus);
    int slices = (int)(2 * cus / walkers);
    slices = slices < 1 ? 1 : slices > 8 ? 8 : slices;
    permute_cols_lds_kernel<<<dim3((unsigned)walkers, (unsigned)slices), 256, (size_t)size_k * 2, (hipStream_t)stream>>>(
        (const uint16_t*)a, perm, (uint16_t*)out, (int)size_m, (int)size_k, lda);
    W4A16_HIP(hipGetLastError());
    return 0;
  }
  // grid.y is limited to 65535: walk M in slabs
  for (int64_t m0 = 0; m0 < size_m; m0 += 65535) {
    const int rows = (int)((size_m - m0) < 65535 ? (size_m - m0) : 65535);
    dim3 grid((unsigned)((size_k + 255) / 256 < 64 ? (size_k + 255) / 256 : 64), (unsigned)rows);
    permute_cols_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(
        (const uint16_t*)a + m0 * lda, perm, (uint16_t*)out + m0 * size_k, rows, (int)size_k, lda);
  }
  W4A16_HIP(hipGetLastError());
  return 0;
}

extern "C" int w4a16_marlin_permute_scales(const void* s, void* out, int64_t num_rows, int64_t size_n, int grouped,
                                           void* stream) {
  W4A16_CHECK(s && out, "null pointer");
  W4A16_CHECK(size_n % 64 == 0, "size_n = %lld is not divisible by 64", (long long)size_n);
  const int64_t total = num_rows * size_n;
  if (total == 0) return 0;
  W4A16_CHECK(total < (1LL << 31) * 256, "problem too large");
  permute_scales_kernel<<<(unsigned)ceil_div(total, 256), 256, 0, (hipStream_t)stream>>>(
      (const uint16_t*)s, (uint16_t*)out, total, grouped);
  W4A16_HIP(hipGetLastError());
  return 0;
}

extern "C" int w4a16_marlin_zero_points(const uint32_t* zp, uint32_t* out, int64_t num_groups, int64_t size_n,
                                        int format, void* stream) {
  W4A16_CHECK(zp && out, "null pointer");
  W4A16_CHECK(size_n % 64 == 0, "size_n = %lld is not divisible by 64", (long long)size_n);
  W4A16_CHECK(format >= 0 && format <= 2, "unknown zero-point source format %d", format);
  const int64_t total = num_groups * (size_n / 8);
  if (total == 0) return 0;
  W4A16_CHECK(total < (1LL << 31) * 256 && size_n < (1LL << 31), "problem too large");
  const unsigned blocks = (unsigned)ceil_div(total, 256);
  hipStream_t st = (hipStream_t)stream;
  if (format == 0) marlin_zero_points_kernel<0><<<blocks, 256, 0, st>>>(zp, out, total, (int)size_n);
  if (format == 1) marlin_zero_points_kernel<1><<<blocks, 256, 0, st>>>(zp, out, total, (int)size_n);
  if (format == 2) marlin_zero_points_kernel<2><<<blocks, 256, 0, st>>>(zp, out, total, (int)size_n);
  W4A16_HIP(hipGetLastError());
  return 0;
}
