// Device-side building blocks shared by the W4A16 GEMM kernels (gfx950, wave64).
//
// How a wavefront consumes the Marlin weight layout with v_mfma_f32_16x16x32_{f16,bf16}
// -----------------------------------------------------------------------------------
// Lane l is split as c = l & 7, h = (l >> 3) & 1, g = l >> 4.  For a "column pair" cp (two
// adjacent 64-column n-tiles, 128 columns) and a k-step ks (two adjacent 16-row k-tiles, 32 rows)
// the lane issues two 128-bit loads, one per k-tile, at Marlin word
//     kt*2N + (2cp+h)*128 + (4c+g)*4 ,  kt = 2ks, 2ks+1
// i.e. it plays Marlin "thread" th = 4c+g of n-tile 2cp+h.  The 64 lanes of one load cover one
// contiguous KiB.  Word w (0..3) of a load holds rows {2g, 2g+1, 2g+8, 2g+9} of the k-tile for
// columns n0 = 64(2cp+h) + 16w + c and n0 + 8.  Across the two k-tiles the lane therefore owns,
// for each of its 8 columns, the 8 K-rows  {2g, 2g+1, 2g+8, 2g+9, 16+2g, 16+2g+1, 16+2g+8, 16+2g+9}
// — exactly what one lane of the MFMA's 32x16 B operand holds (column label l & 15, K-block
// l >> 4).  So 8 MFMAs per k-step, one per (w, half), each covering the 16 columns
//     { 64(2cp+h) + 16w + 8half + c : h in {0,1}, c in [0,8) }      (label = 8h + c)
// K order inside the MFMA is arbitrary as long as the activation operand agrees: activations are
// staged in LDS as [k-step][g][row m][8 halves in the K order above], so lane (m = l & 15,
// g = l >> 4) fetches its A operand with one conflict-free ds_read_b128.
// The accumulator of lane l holds rows 4(l>>4) .. +3 of column label l & 15 — the lane's own
// columns, so per-column scales / zero-points / bias never cross lanes.
#pragma once
#include <type_traits>

#include "common.h"

namespace w4a16 {

using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
using u32x2 = uint32_t __attribute__((ext_vector_type(2)));
using f32x4 = float __attribute__((ext_vector_type(4)));
using f16x8 = _Float16 __attribute__((ext_vector_type(8)));
using f16x2 = _Float16 __attribute__((ext_vector_type(2)));
using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));

enum { DT_F16 = 0, DT_BF16 = 1 };
// how the scale row of a K-row is found
enum {
  GM_GROUPED = 0,  // contiguous groups of group_size rows (multiple of 32), scale per element
  GM_CHANNEL = 1,  // one scale row for all K: applied once to the fp32 accumulator
  GM_GIDX = 2      // scale row = g_idx[row] (act-order shard with partial groups)
};

template <int DT>
__device__ __forceinline__ f32x4 mfma16x16x32(u32x4 a, u32x4 b, f32x4 c) {
  if constexpr (DT == DT_F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ f16x2 as_h2(uint32_t x) { return __builtin_bit_cast(f16x2, x); }
__device__ __forceinline__ uint32_t as_u32(f16x2 x) { return __builtin_bit_cast(uint32_t, x); }
__device__ __forceinline__ float bf16_lo_f32(uint32_t x) { return __builtin_bit_cast(float, x << 16); }
__device__ __forceinline__ float bf16_hi_f32(uint32_t x) { return __builtin_bit_cast(float, x & 0xffff0000u); }
__device__ __forceinline__ float f16_lo_f32(uint32_t x) { return (float)as_h2(x).x; }
__device__ __forceinline__ float f16_hi_f32(uint32_t x) { return (float)as_h2(x).y; }

// round-to-nearest-even pack of two fp32 into bf16x2 (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  bf2 r = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  f16x2 r = {(_Float16)lo, (_Float16)hi};
  return as_u32(r);
}

// Per-lane dequantisation constants of one Marlin word position w (two columns: half 0 / half 1).
//  fp16:  value = (1024+q) - zl  |  (1024+16q)/16 - zh , then * s         (all packed-half ops;
//         every step is exact except the final multiply, so the operand equals
//         half(q - z) * half(s) rounded once — the reference's w_ref)
//  bf16:  the nibbles are turned into the same exact fp16 pairs, (1024+q) and (1024+16q), and one mixed-precision
//         FMA per value (v_fma_mix_f32: fp16 x fp32 + fp32 -> fp32) gives (q - z) * s in fp32:
//         fma(1024+q, s, -(1024+z) s)  |  fma(1024+16q, s/16, -(64+z) s).  The constants are exact in fp32 (at most
//         11 + 8 bits) and so is the result (at most 5 + 8 bits), which v_cvt_pk_bf16_f32 then rounds once:
//         bf16_rne((q - z) * s), the reference's w_ref.
template <int DT>
struct ColConst;

template <>
struct ColConst<DT_F16> {
  uint32_t s;   // (s_half0, s_half1)
  uint32_t zl;  // (1024+z_half0, 1024+z_half1)
  uint32_t zh;  // (64+z_half0, 64+z_half1)
};
template <>
struct ColConst<DT_BF16> {
  float s0, s1;  // scale of half 0 / half 1
  float c0, c1;  // -(1024+z)*s
  float h0, h1;  // s/16
  float d0, d1;  // -(64+z)*s
};

// raw: (s_half0, s_half1) packed 16-bit pair as loaded; z0/z1: integer zero points (8 for uint4b8)
template <int DT, bool UNIT_SCALE>
__device__ __forceinline__ ColConst<DT> make_col_const(uint32_t s_pair, uint32_t z0, uint32_t z1) {
  ColConst<DT> cc;
  if constexpr (DT == DT_F16) {
    cc.s = UNIT_SCALE ? 0x3c003c00u : s_pair;
    // 1024+z and 64+z are exact fp16 integers: 0x6400 | z  and  0x5400 + (z << 4) (ulp of 64.. is 1/16)
    cc.zl = 0x64006400u | z0 | (z1 << 16);
    cc.zh = 0x54005400u + ((z0 << 4) | (z1 << 20));
  } else {
    cc.s0 = UNIT_SCALE ? 1.0f : bf16_lo_f32(s_pair);
    cc.s1 = UNIT_SCALE ? 1.0f : bf16_hi_f32(s_pair);
    // 1024+z as fp32 bits: 2^10 has its ulp at 2^-13, so z sits at bit 13 of the mantissa
    const float t0 = __builtin_bit_cast(float, 0x44800000u | (z0 << 13));
    const float t1 = __builtin_bit_cast(float, 0x44800000u | (z1 << 13));
    cc.c0 = -t0 * cc.s0;
    cc.c1 = -t1 * cc.s1;
    cc.h0 = cc.s0 * 0.0625f;
    cc.h1 = cc.s1 * 0.0625f;
    cc.d0 = __builtin_fmaf(960.0f, cc.s0, cc.c0);
    cc.d1 = __builtin_fmaf(960.0f, cc.s1, cc.c1);
  }
  return cc;
}

// xa, xb: word w of the lane's 128-bit loads from k-tile 2ks and 2ks+1.
// o0 / o1: MFMA B operand (8 values in the lane's K order) for column half 0 / half 1.
template <int DT, bool UNIT_SCALE>
__device__ __forceinline__ void dequant_pair(uint32_t xa, uint32_t xb, const ColConst<DT>& cc, u32x4& o0,
                                             u32x4& o1) {
  if constexpr (DT == DT_F16) {
    const uint32_t MLO = 0x000f000fu, MHI = 0x00f000f0u;
    // keep the exponent pattern in a VGPR so that (x & mask) | EX is one v_and_or_b32
    uint32_t EX = 0x64006400u;
    asm("" : "+v"(EX));
    const f16x2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
    const f16x2 s = as_h2(cc.s), zl = as_h2(cc.zl), zh = as_h2(cc.zh);
    const f16x2 s0 = {s.x, s.x}, s1 = {s.y, s.y};
    const f16x2 zl0 = {zl.x, zl.x}, zl1 = {zl.y, zl.y};
    const f16x2 zh0 = {zh.x, zh.x}, zh1 = {zh.y, zh.y};
    auto lo = [&](uint32_t x, f16x2 z, f16x2 sc) {
      const f16x2 v = as_h2((x & MLO) | EX) - z;
      return as_u32(UNIT_SCALE ? v : v * sc);
    };
    auto hi = [&](uint32_t x, f16x2 z, f16x2 sc) {
      const f16x2 v = as_h2((x & MHI) | EX) * sixteenth - z;
      return as_u32(UNIT_SCALE ? v : v * sc);
    };
    const uint32_t ya = xa >> 8, yb = xb >> 8;
    o0 = u32x4{lo(xa, zl0, s0), hi(xa, zh0, s0), lo(xb, zl0, s0), hi(xb, zh0, s0)};
    o1 = u32x4{lo(ya, zl1, s1), hi(ya, zh1, s1), lo(yb, zl1, s1), hi(yb, zh1, s1)};
  } else {
    // nibble j of a word: j=0 (k0,n0) 1 (k0+8,n0) 2 (k0,n0+8) 3 (k0+8,n0+8) 4..7 same with k0+1
    uint32_t EX = 0x64006400u;
    asm("" : "+v"(EX));
    auto lo = [&](uint32_t x, float sf, float cf) {   // nibbles 0 and 4 of x: 1024+q
      const f16x2 v = as_h2((x & 0x000f000fu) | EX);
      return pack_bf16(__builtin_fmaf((float)v.x, sf, cf), __builtin_fmaf((float)v.y, sf, cf));
    };
    auto hi = [&](uint32_t x, float hf, float df) {   // nibbles 1 and 5 of x: 1024+16q
      const f16x2 v = as_h2((x & 0x00f000f0u) | EX);
      return pack_bf16(__builtin_fmaf((float)v.x, hf, df), __builtin_fmaf((float)v.y, hf, df));
    };
    const uint32_t ya = xa >> 8, yb = xb >> 8;
    o0 = u32x4{lo(xa, cc.s0, cc.c0), hi(xa, cc.h0, cc.d0), lo(xb, cc.s0, cc.c0), hi(xb, cc.h0, cc.d0)};
    o1 = u32x4{lo(ya, cc.s1, cc.c1), hi(ya, cc.h1, cc.d1), lo(yb, cc.s1, cc.c1), hi(yb, cc.h1, cc.d1)};
  }
}

// Float zero points (HQQ; fp16 only): the B operand is fma(q, s, -zs) with zs = half(zp * s) rounded once, as the
// reference computes it (marlin_template.h:174-181 scale_and_sub, :1235-1240).  q is made exact first:
// (1024+q) - 1024 for the low nibbles, (1024+16q)/16 - 64 for the high ones.
__device__ __forceinline__ void dequant_pair_zpf(uint32_t xa, uint32_t xb, uint32_t s_pair, uint32_t zs_pair,
                                                 u32x4& o0, u32x4& o1) {
  const uint32_t MLO = 0x000f000fu, MHI = 0x00f000f0u;
  uint32_t EX = 0x64006400u;
  asm("" : "+v"(EX));
  const f16x2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  const f16x2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f}, k64 = {(_Float16)64.0f, (_Float16)64.0f};
  const f16x2 s = as_h2(s_pair), zs = as_h2(zs_pair);
  const f16x2 s0 = {s.x, s.x}, s1 = {s.y, s.y};
  const f16x2 nz0 = {-zs.x, -zs.x}, nz1 = {-zs.y, -zs.y};
  auto lo = [&](uint32_t x, f16x2 sc, f16x2 nz) {
    const f16x2 q = as_h2((x & MLO) | EX) - k1024;
    return as_u32(__builtin_elementwise_fma(q, sc, nz));
  };
  auto hi = [&](uint32_t x, f16x2 sc, f16x2 nz) {
    const f16x2 q = as_h2((x & MHI) | EX) * sixteenth - k64;
    return as_u32(__builtin_elementwise_fma(q, sc, nz));
  };
  const uint32_t ya = xa >> 8, yb = xb >> 8;
  o0 = u32x4{lo(xa, s0, nz0), hi(xa, s0, nz0), lo(xb, s0, nz0), hi(xb, s0, nz0)};
  o1 = u32x4{lo(ya, s1, nz1), hi(ya, s1, nz1), lo(yb, s1, nz1), hi(yb, s1, nz1)};
}

// One register (J = 0..7, as dequant_piece) of what dequant_pair_zpf produces, for the prefill kernel.
template <int J>
__device__ __forceinline__ uint32_t dequant_piece_zpf(uint32_t xa, uint32_t xb, uint32_t s_pair, uint32_t zs_pair) {
  constexpr int HF = J >> 2, Q = J & 3;
  uint32_t EX = 0x64006400u;
  asm("" : "+v"(EX));
  const uint32_t x = (Q < 2) ? xa : xb;
  const uint32_t y = HF ? (x >> 8) : x;
  const f16x2 s = as_h2(s_pair), zs = as_h2(zs_pair);
  const f16x2 sc = HF ? f16x2{s.y, s.y} : f16x2{s.x, s.x};
  const f16x2 nz = HF ? f16x2{-zs.y, -zs.y} : f16x2{-zs.x, -zs.x};
  f16x2 q;
  if constexpr ((Q & 1) == 0) {
    const f16x2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    q = as_h2((y & 0x000f000fu) | EX) - k1024;
  } else {
    const f16x2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f}, k64 = {(_Float16)64.0f, (_Float16)64.0f};
    q = as_h2((y & 0x00f000f0u) | EX) * sixteenth - k64;
  }
  return as_u32(__builtin_elementwise_fma(q, sc, nz));
}

// byte N of x as float (v_cvt_f32_ubyteN; the compiler only finds the byte-0 form on its own)
template <int N>
__device__ __forceinline__ float ubyte_f32(uint32_t x) {
  float f;
  if constexpr (N == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(x));
  if constexpr (N == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(x));
  if constexpr (N == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(x));
  if constexpr (N == 3) asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(x));
  return f;
}

// bf16, the two steps of one operand register apart (the prefill kernel issues them between different MFMAs):
// the exact fp16 pair of nibbles 2*HF + ODD and that + 4 of x, then the two mixed FMAs and the pack.
template <int HF, int ODD>
__device__ __forceinline__ uint32_t bf16_piece_halves(uint32_t x) {
  uint32_t EX = 0x64006400u;
  asm("" : "+v"(EX));
  const uint32_t y = HF ? (x >> 8) : x;
  return (y & (ODD ? 0x00f000f0u : 0x000f000fu)) | EX;
}
template <int HF, int ODD>
__device__ __forceinline__ void bf16_piece_fma(uint32_t halves, const ColConst<DT_BF16>& cc, float& f0, float& f1) {
  const f16x2 v = as_h2(halves);
  const float m = ODD ? (HF ? cc.h1 : cc.h0) : (HF ? cc.s1 : cc.s0);
  const float a = ODD ? (HF ? cc.d1 : cc.d0) : (HF ? cc.c1 : cc.c0);
  f0 = __builtin_fmaf((float)v.x, m, a);
  f1 = __builtin_fmaf((float)v.y, m, a);
}
template <int HF, int ODD>
__device__ __forceinline__ uint32_t bf16_piece_pack(uint32_t halves, const ColConst<DT_BF16>& cc) {
  float f0, f1;
  bf16_piece_fma<HF, ODD>(halves, cc, f0, f1);
  return pack_bf16(f0, f1);
}

// One register (J = 0..7) of what dequant_pair produces: J < 4 -> o0[J], else o1[J - 4].  Lets a caller spread
// the dequantisation of a Marlin word pair between MFMAs a few instructions at a time.
template <int DT, bool UNIT_SCALE, int J>
__device__ __forceinline__ uint32_t dequant_piece(uint32_t xa, uint32_t xb, const ColConst<DT>& cc) {
  constexpr int HF = J >> 2, Q = J & 3;
  const uint32_t x = (Q < 2) ? xa : xb;
  if constexpr (DT == DT_F16) {
    uint32_t EX = 0x64006400u;
    asm("" : "+v"(EX));
    const uint32_t y = HF ? (x >> 8) : x;
    const f16x2 s = as_h2(cc.s);
    const f16x2 sc = HF ? f16x2{s.y, s.y} : f16x2{s.x, s.x};
    f16x2 v;
    if constexpr ((Q & 1) == 0) {
      const f16x2 z = as_h2(cc.zl);
      v = as_h2((y & 0x000f000fu) | EX) - (HF ? f16x2{z.y, z.y} : f16x2{z.x, z.x});
    } else {
      const f16x2 z = as_h2(cc.zh);
      const f16x2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
      v = as_h2((y & 0x00f000f0u) | EX) * sixteenth - (HF ? f16x2{z.y, z.y} : f16x2{z.x, z.x});
    }
    return as_u32(UNIT_SCALE ? v : v * sc);
  } else {
    return bf16_piece_pack<HF, Q & 1>(bf16_piece_halves<HF, Q & 1>(x), cc);
  }
}

// 8-bit weights (uint8b128: stored byte = value + 128).  A lane's Marlin word holds the bytes of one column for
// K rows (k0, k0+8, k0+1, k0+9); ha / hb: the words of column half 0 / half 1, a / b: k-tiles 2ks / 2ks+1.
//  fp16:  (1024 + b) - 1152 is exact, then one multiply by s (= half(q - 128) * half(s), the reference's w_ref)
//  bf16:  bf16_rne(fma(float(b), s, -128 s))
template <int DT, bool UNIT_SCALE>
__device__ __forceinline__ void dequant_pair8(uint32_t xa0, uint32_t xa1, uint32_t xb0, uint32_t xb1,
                                              uint32_t s_pair, u32x4& o0, u32x4& o1) {
  if constexpr (DT == DT_F16) {
    uint32_t EX = 0x64006400u;
    asm("" : "+v"(EX));
    const f16x2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    const f16x2 s = as_h2(s_pair);
    auto lo = [&](uint32_t x, f16x2 sc) {
      const f16x2 v = as_h2((x & 0x00ff00ffu) | EX) - bias;
      return as_u32(UNIT_SCALE ? v : v * sc);
    };
    auto hi = [&](uint32_t x, f16x2 sc) { return lo(x >> 8, sc); };
    const f16x2 s0 = {s.x, s.x}, s1 = {s.y, s.y};
    o0 = u32x4{lo(xa0, s0), hi(xa0, s0), lo(xb0, s0), hi(xb0, s0)};
    o1 = u32x4{lo(xa1, s1), hi(xa1, s1), lo(xb1, s1), hi(xb1, s1)};
  } else {
    const float s0 = UNIT_SCALE ? 1.0f : bf16_lo_f32(s_pair), s1 = UNIT_SCALE ? 1.0f : bf16_hi_f32(s_pair);
    const float c0 = -128.0f * s0, c1 = -128.0f * s1;
    auto lo = [&](uint32_t x, float sf, float cf) {
      return pack_bf16(__builtin_fmaf(ubyte_f32<0>(x), sf, cf), __builtin_fmaf(ubyte_f32<2>(x), sf, cf));
    };
    auto hi = [&](uint32_t x, float sf, float cf) {
      return pack_bf16(__builtin_fmaf(ubyte_f32<1>(x), sf, cf), __builtin_fmaf(ubyte_f32<3>(x), sf, cf));
    };
    o0 = u32x4{lo(xa0, s0, c0), hi(xa0, s0, c0), lo(xb0, s0, c0), hi(xb0, s0, c0)};
    o1 = u32x4{lo(xa1, s1, c1), hi(xa1, s1, c1), lo(xb1, s1, c1), hi(xb1, s1, c1)};
  }
}

// One register (J = 0..7, as dequant_piece) of what dequant_pair8 / dequant_pair8_fp8 produce, for the prefill kernel.
// x0 / x1: the word of column half 0 / 1 of the k-tile that register J draws on (Q < 2: k-tile a, else b).
template <int DT, bool UNIT_SCALE, bool FP8, int J>
__device__ __forceinline__ uint32_t dequant_piece8(uint32_t x0, uint32_t x1, uint32_t s_pair) {
  constexpr int HF = J >> 2, Q = J & 3;
  const uint32_t x = HF ? x1 : x0;
  if constexpr (FP8) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    float sf = 1.0f;
    if (!UNIT_SCALE)
      sf = ((DT == DT_F16) ? (HF ? f16_hi_f32(s_pair) : f16_lo_f32(s_pair))
                           : (HF ? bf16_hi_f32(s_pair) : bf16_lo_f32(s_pair))) *
           ((DT == DT_F16) ? 0x1.0p-8f : 0x1.0p-120f);
    // bytes (k0, k0+8, k0+1, k0+9): register Q & 1 = 0 pairs (k0, k0+1), 1 pairs (k0+8, k0+9)
    const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)x, false);
    const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)x, true);
    const float lo = (Q & 1) ? a.y : a.x, hi = (Q & 1) ? b.y : b.x;
    return DT == DT_F16 ? pack_f16(lo * sf, hi * sf) : pack_bf16(lo * sf, hi * sf);
  } else if constexpr (DT == DT_F16) {
    uint32_t EX = 0x64006400u;
    asm("" : "+v"(EX));
    const f16x2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    const uint32_t y = (Q & 1) ? (x >> 8) : x;
    const f16x2 v = as_h2((y & 0x00ff00ffu) | EX) - bias;
    const f16x2 s = as_h2(s_pair);
    return as_u32(UNIT_SCALE ? v : v * (HF ? f16x2{s.y, s.y} : f16x2{s.x, s.x}));
  } else {
    const float sf = UNIT_SCALE ? 1.0f : (HF ? bf16_hi_f32(s_pair) : bf16_lo_f32(s_pair));
    const float cf = -128.0f * sf;
    return pack_bf16(__builtin_fmaf(ubyte_f32<(Q & 1)>(x), sf, cf), __builtin_fmaf(ubyte_f32<(Q & 1) + 2>(x), sf, cf));
  }
}

// fp8 (OCP e4m3fn) weights in the 8-bit Marlin layout.  The scales the op receives carry the exponent offset the
// reference folds into them at load time (marlin_utils_fp8.py:25-37: s * 2^8 for fp16, s * 2^120 for bf16, because
// its kernel moves the fp8 bits into the 16-bit format without re-biasing the exponent, dequant.h:320-373).  Here the
// bytes are converted by v_cvt_pk_f32_fp8 (exact), so the offset is taken out of the scale again (exact, a power of
// two) and the operand is x * s rounded once to the 16-bit type: the reference's w_ref = fp8.to(dtype) * s.
template <int DT>
__device__ __forceinline__ float fp8_scale_unbias() {
  return (DT == DT_F16) ? 0x1.0p-8f : 0x1.0p-120f;
}
template <int DT, bool UNIT_SCALE>
__device__ __forceinline__ void dequant_pair8_fp8(uint32_t xa0, uint32_t xa1, uint32_t xb0, uint32_t xb1,
                                                  uint32_t s_pair, u32x4& o0, u32x4& o1) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  float s0 = 1.0f, s1 = 1.0f;
  if (!UNIT_SCALE) {
    s0 = ((DT == DT_F16) ? f16_lo_f32(s_pair) : bf16_lo_f32(s_pair)) * fp8_scale_unbias<DT>();
    s1 = ((DT == DT_F16) ? f16_hi_f32(s_pair) : bf16_hi_f32(s_pair)) * fp8_scale_unbias<DT>();
  }
  // a word holds K rows (k0, k0+8, k0+1, k0+9): low half -> (k0, k0+8), high half -> (k0+1, k0+9)
  auto cvt = [&](uint32_t x, float sf, uint32_t& p_lo, uint32_t& p_hi) {
    const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)x, false);
    const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)x, true);
    if constexpr (DT == DT_F16) {
      p_lo = pack_f16(a.x * sf, b.x * sf);  // (k0, k0+1)
      p_hi = pack_f16(a.y * sf, b.y * sf);  // (k0+8, k0+9)
    } else {
      p_lo = pack_bf16(a.x * sf, b.x * sf);
      p_hi = pack_bf16(a.y * sf, b.y * sf);
    }
  };
  uint32_t p0, p1, p2, p3, q0, q1, q2, q3;
  cvt(xa0, s0, p0, p1);
  cvt(xb0, s0, p2, p3);
  cvt(xa1, s1, q0, q1);
  cvt(xb1, s1, q2, q3);
  o0 = u32x4{p0, p1, p2, p3};
  o1 = u32x4{q0, q1, q2, q3};
}

// The same weights converted straight to the 16-bit type: v_cvt_scalef32_pk_{f16,bf16}_fp8 turns the two low (or high)
// bytes of a word, K rows (k0, k0+8) or (k0+1, k0+9), into a packed pair times 2^(exponent of scale - 127); the B
// operand is then in the K order (k0, k0+8, k0+1, k0+9, ...) and A is reordered to match (a_frag_fp4_order).
// fp16: codes * 2^-8 (exact, takes the exponent offset out of the stored scale), then one packed multiply by the
// stored scale: x * s rounded once, as above.  Without a per-element scale (channel-wise) the conversion alone is exact
// in either type.
template <int DT, bool UNIT_SCALE>
__device__ __forceinline__ void dequant_pair8_fp8_direct(uint32_t xa0, uint32_t xa1, uint32_t xb0, uint32_t xb1,
                                                         uint32_t s_pair, u32x4& o0, u32x4& o1) {
  static_assert(DT == DT_F16 || UNIT_SCALE, "bf16 has no packed multiply");
  const float pre = UNIT_SCALE ? 1.0f : 0x1.0p-8f;
  auto cvt = [&](uint32_t x, auto hi_tag) {
    constexpr bool hi = decltype(hi_tag)::value;
    if constexpr (DT == DT_F16) {
      return as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(x, pre, hi));
    } else {
      typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
      const bf2 r = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(x, pre, hi);
      return __builtin_bit_cast(uint32_t, r);
    }
  };
  using T = std::integral_constant<bool, true>;
  using F = std::integral_constant<bool, false>;
  u32x4 r0 = {cvt(xa0, F{}), cvt(xa0, T{}), cvt(xb0, F{}), cvt(xb0, T{})};
  u32x4 r1 = {cvt(xa1, F{}), cvt(xa1, T{}), cvt(xb1, F{}), cvt(xb1, T{})};
  if constexpr (!UNIT_SCALE) {
    const f16x2 s = as_h2(s_pair);
    const f16x2 s0 = {s.x, s.x}, s1 = {s.y, s.y};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      r0[i] = as_u32(as_h2(r0[i]) * s0);
      r1[i] = as_u32(as_h2(r1[i]) * s1);
    }
  }
  o0 = r0;
  o1 = r1;
}

// fp4 (float4_e2m1f) weights in the 4-bit Marlin layout.  A byte of a Marlin word holds the codes of K rows (k0, k0+8)
// [bytes 0, 1: columns n0, n0+8] or (k0+1, k0+9) [bytes 2, 3]; v_cvt_scalef32_pk_f32_fp4 turns one byte into two exact
// fp32 values.  sa* / sb*: true scales (fp32) of k-tile a / b for column half 0 / 1; x * s has at most 6 significant
// bits, so the operand is exact in either 16-bit type.
template <int DT>
__device__ __forceinline__ void dequant_pair_fp4(uint32_t xa, uint32_t xb, float sa0, float sa1, float sb0, float sb1,
                                                 u32x4& o0, u32x4& o1) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  auto pack = [](float lo, float hi) { return DT == DT_F16 ? pack_f16(lo, hi) : pack_bf16(lo, hi); };
  auto tile = [&](uint32_t x, float s0, float s1, uint32_t& p0_lo, uint32_t& p0_hi, uint32_t& p1_lo, uint32_t& p1_hi) {
    const f32x2 c0a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, 0);  // column n0:   (k0, k0+8)
    const f32x2 c1a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, 1);  // column n0+8: (k0, k0+8)
    const f32x2 c0b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, 2);  // column n0:   (k0+1, k0+9)
    const f32x2 c1b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, 3);  // column n0+8: (k0+1, k0+9)
    p0_lo = pack(c0a.x * s0, c0b.x * s0);  // (k0, k0+1)
    p0_hi = pack(c0a.y * s0, c0b.y * s0);  // (k0+8, k0+9)
    p1_lo = pack(c1a.x * s1, c1b.x * s1);
    p1_hi = pack(c1a.y * s1, c1b.y * s1);
  };
  uint32_t p0, p1, p2, p3, q0, q1, q2, q3;
  tile(xa, sa0, sa1, p0, p1, q0, q1);
  tile(xb, sb0, sb1, p2, p3, q2, q3);
  o0 = u32x4{p0, p1, p2, p3};
  o1 = u32x4{q0, q1, q2, q3};
}
// Direct fp4 -> 16-bit conversion: v_cvt_scalef32_pk_{f16,bf16}_fp4 turns one byte (the codes of K rows k0 and
// k0+8 of one column) into a packed 16-bit pair, times 2^(exponent of `scale` - 127).  The B operand of a column half
// is then in the K order (k0, k0+8, k0+1, k0+9, 16+k0, 24+k0, 17+k0, 25+k0) instead of (k0, k0+1, k0+8, k0+9, ...):
// the A operand is reordered to match (a_frag_fp4_order), which costs 4 v_perm_b32 per m-block and k-step instead of
// two multiplies and a pack per weight pair.
template <int DT, int BYTE>
__device__ __forceinline__ uint32_t cvt_fp4x2(uint32_t x, float scale) {
  if constexpr (DT == DT_F16) {
    return as_u32(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(x, scale, BYTE));
  } else {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    const bf2 r = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(x, scale, BYTE);
    return __builtin_bit_cast(uint32_t, r);
  }
}
__device__ __forceinline__ u32x4 a_frag_fp4_order(u32x4 a) {
  return u32x4{__builtin_amdgcn_perm(a[1], a[0], 0x05040100u), __builtin_amdgcn_perm(a[1], a[0], 0x07060302u),
               __builtin_amdgcn_perm(a[3], a[2], 0x05040100u), __builtin_amdgcn_perm(a[3], a[2], 0x07060302u)};
}
// MXFP4: the E8M0 group scale is the conversion's scale operand (exact: a power of two).  s0 / s1: scale of column
// half 0 / 1 as fp32 (only its exponent is used).
template <int DT>
__device__ __forceinline__ void dequant_pair_mxfp4_direct(uint32_t xa, uint32_t xb, float s0, float s1, u32x4& o0,
                                                          u32x4& o1) {
  o0 = u32x4{cvt_fp4x2<DT, 0>(xa, s0), cvt_fp4x2<DT, 2>(xa, s0), cvt_fp4x2<DT, 0>(xb, s0), cvt_fp4x2<DT, 2>(xb, s0)};
  o1 = u32x4{cvt_fp4x2<DT, 1>(xa, s1), cvt_fp4x2<DT, 3>(xa, s1), cvt_fp4x2<DT, 1>(xb, s1), cvt_fp4x2<DT, 3>(xb, s1)};
}
// NVFP4, fp16: the scale byte b stands for the half (b << 7) = s * 2^7.  The codes are converted times 2^-7 (exact,
// >= 2^-8) and multiplied by that half with one packed multiply: value * s rounded once, as the fp32 route gives.
// ba / bb: scale bytes of k-tile a / b, column half 0 in bits 0..7, half 1 in bits 16..23.
__device__ __forceinline__ void dequant_pair_nvfp4_f16_direct(uint32_t xa, uint32_t xb, uint32_t ba, uint32_t bb,
                                                              u32x4& o0, u32x4& o1) {
  const float pre = 0x1.0p-7f;
  auto h2 = [](uint32_t byte) { return as_h2(byte * 0x00800080u); };  // (b << 7) in both halves
  const f16x2 sa0 = h2(ba & 0xffu), sa1 = h2(ba >> 16), sb0 = h2(bb & 0xffu), sb1 = h2(bb >> 16);
  auto m = [](uint32_t v, f16x2 sc) { return as_u32(as_h2(v) * sc); };
  o0 = u32x4{m(cvt_fp4x2<DT_F16, 0>(xa, pre), sa0), m(cvt_fp4x2<DT_F16, 2>(xa, pre), sa0),
             m(cvt_fp4x2<DT_F16, 0>(xb, pre), sb0), m(cvt_fp4x2<DT_F16, 2>(xb, pre), sb0)};
  o1 = u32x4{m(cvt_fp4x2<DT_F16, 1>(xa, pre), sa1), m(cvt_fp4x2<DT_F16, 3>(xa, pre), sa1),
             m(cvt_fp4x2<DT_F16, 1>(xb, pre), sb1), m(cvt_fp4x2<DT_F16, 3>(xb, pre), sb1)};
}
// One register (J = 0..7, as dequant_piece) of what dequant_pair_fp4 produces, for the prefill kernel.  x: the word of
// the k-tile register J draws on; s0 / s1: that k-tile's true scale for column half 0 / 1.
template <int DT, int J>
__device__ __forceinline__ uint32_t dequant_piece_fp4(uint32_t x, float s0, float s1) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  constexpr int HF = J >> 2, Q = J & 3;
  const float sf = HF ? s1 : s0;
  // bytes 0, 1: K rows (k0, k0+8) of columns n0, n0+8; bytes 2, 3: rows (k0+1, k0+9)
  const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, HF);
  const f32x2 b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, HF + 2);
  const float lo = (Q & 1) ? a.y : a.x, hi = (Q & 1) ? b.y : b.x;
  return DT == DT_F16 ? pack_f16(lo * sf, hi * sf) : pack_bf16(lo * sf, hi * sf);
}
// Scale bytes of Marlin word w in a lane's 16-byte fp4 scale record: 8 bytes per k-tile (NVFP4) or k-step (MXFP4),
// stored in the order (e0, e2, e1, e3, e4, e6, e5, e7) with e = 2w + half (marlin_utils_fp4.py:44-47, 68-71).
// half_rec: the 8 bytes as two dwords; returns byte of column half 0 in bits 0..7 and of half 1 in bits 16..23.
__device__ __forceinline__ uint32_t fp4_scale_bytes(uint32_t d_lo, uint32_t d_hi, int w) {
  const uint32_t d = (w >> 1) ? d_hi : d_lo;
  return (d >> (8 * (w & 1))) & 0x00ff00ffu;
}
// NVFP4 scale byte -> fp32: the byte is the top byte of half(s * 2^7) << 1 (unsigned E5M3)
__device__ __forceinline__ float nvfp4_scale_f32(uint32_t byte) {
  return f16_lo_f32(byte << 7) * 0x1.0p-7f;
}
// MXFP4 scale byte (E8M0) -> fp32: 2^(b - 127)
__device__ __forceinline__ float mxfp4_scale_f32(uint32_t byte) { return __builtin_bit_cast(float, byte << 23); }

// "Raw" B operands for the fold scheme of the 16-row kernels: nibbles are only moved into the mantissa of a magic
// exponent, value = E + q (E = 1024 for fp16, 128 for bf16).  With HI_TRICK (fp16) the high nibbles stay where they
// are, bits 4..7, under the exponent of 64, whose mantissa bits 4..7 weigh 1, 2, 4, 8: value = 64 + q exactly, for the
// K rows k0+8, k0+9 (slots 1 and 3), so no shift is needed.  No subtract, no scale: both are applied to the fp32
// accumulator once per quantization group, through a bias-term MFMA whose operand carries 1024 + 8 in the low-nibble
// slots and 64 + 8 in the high-nibble slots (RAW_BIAS_LO / RAW_BIAS_HI).
constexpr uint32_t RAW_BIAS_LO = 0x64086408u;  // (1032, 1032)
constexpr uint32_t RAW_BIAS_HI = 0x54805480u;  // (72, 72)
template <int DT, bool HI_TRICK>
__device__ __forceinline__ void raw_pair(uint32_t xa, uint32_t xb, u32x4& o0, u32x4& o1) {
  const uint32_t M = 0x000f000fu;
  uint32_t E = (DT == DT_F16) ? 0x64006400u : 0x43004300u;
  asm("" : "+v"(E));  // keep in a VGPR: (x & mask) | E becomes one v_and_or_b32
  if constexpr (HI_TRICK) {
    const uint32_t MH = 0x00f000f0u;
    uint32_t EH = 0x54005400u;
    asm("" : "+v"(EH));
    const uint32_t ya = xa >> 8, yb = xb >> 8;
    o0 = u32x4{(xa & M) | E, (xa & MH) | EH, (xb & M) | E, (xb & MH) | EH};
    o1 = u32x4{(ya & M) | E, (ya & MH) | EH, (yb & M) | E, (yb & MH) | EH};
  } else {
    o0 = u32x4{(xa & M) | E, ((xa >> 4) & M) | E, (xb & M) | E, ((xb >> 4) & M) | E};
    o1 = u32x4{((xa >> 8) & M) | E, ((xa >> 12) & M) | E, ((xb >> 8) & M) | E, ((xb >> 12) & M) | E};
  }
}

// SiLU in fp32 exactly as PyTorch's device kernel and the reference's act_and_mul_kernel evaluate it
// (csrc/activation_kernels.cu:28-32): x / (1 + expf(-x)) with the correctly rounded quotient, so that results equal
// torch.nn.functional.silu on the same device bit for bit (the reference tests this op for exact equality,
// tests/kernels/core/test_activation.py:93-97).
__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

// Position of real column `cl` (0..31 inside its 32-column chunk) in a tensor permuted with the
// reference's "single" permutation (marlin_utils.py:278-286, used for channel-wise scales and bias).
__device__ __forceinline__ int single_perm_pos(int cl) {
  return 8 * ((cl & 7) >> 1) + 2 * (cl >> 3) + (cl & 1);
}

}  // namespace w4a16
