// In-register dequantisation of one gfx950 weight word (eight 4-bit codes of
// one column, rows t = 0..7 at nibble slots t/2 + 4*(t%2)) into the eight
// 16-bit values of one v_mfma_f32_16x16x32 operand, plus the per-column
// constants it needs.  The result is round_to_dtype((code - z) * s) with a
// single round-to-nearest-even, the value the reference forms with
// dequant<...> followed by scale()/sub_zp()
// (csrc/libtorch_stable/quantization/marlin/dequant.h:107-216,
// marlin_template.h:107-142,1182-1299).
#pragma once

#include "common.hpp"

namespace sonar {

// Where column `nl` (0..63) of a 64-column block sits after
// marlin_permute_scales (aphrodite/.../utils/marlin_utils.py:406-426).
// grouped: 8x8 transpose of the block; single: scale_perm_single inside each
// 32 columns.
__device__ __forceinline__ int scale_slot(int nl, bool grouped) {
  if (grouped) return 8 * (nl & 7) + (nl >> 3);
  const int n32 = nl & 31;
  return (nl & 32) + 8 * ((n32 & 7) >> 1) + 2 * (n32 >> 3) + (n32 & 1);
}

// Zero point of column `nl` of a 64-column block from the eight words that
// marlin_zero_points (marlin_utils.py:456-477) makes of the block: word nl%8,
// nibble slot {0,4,1,5,2,6,3,7}[nl/8] = (nl/8)/2 + 4*((nl/8)%2).
__device__ __forceinline__ int zero_point_word(int nl) { return nl & 7; }
__device__ __forceinline__ int zero_point_shift(int nl) {
  const int t = nl >> 3;
  return 4 * ((t >> 1) + 4 * (t & 1));
}

// (q & mask) | magic, which the compiler emits as one v_and_or_b32 when the
// constant that is OR-ed in sits in a vector register it cannot see through
// (`magic_register`); with a visible constant it splits the expression into
// an AND and an OR with literals.  The expression itself must stay visible to
// the compiler: it pads the matrix-core hazards (a VALU write to a register an
// MFMA in flight still reads) only around instructions it generated itself.
__device__ __forceinline__ uint32_t magic_register(uint32_t m = 0x64006400u) {
  asm("" : "+v"(m));
  return m;
}
__device__ __forceinline__ uint32_t and_or(uint32_t q, uint32_t mask, uint32_t magic) {
  return (q & mask) | magic;
}

template <typename T>
struct Dq;

// ---------------------------------------------------------------- fp16
// (q & 0x000f000f) | 0x64006400 is the half2 (1024 + v_lo, 1024 + v_hi);
// with mask 0x00f000f0 it is 1024 + 16 v.  Subtracting 1024 + z, or
// fma(x, 1/16, -(64 + z)), gives v - z exactly; one packed multiply by the
// scale then rounds once.
template <>
struct Dq<_Float16> {
  typedef half8_t vec8;
  struct Col {
    half2_t s;    // (s, s)
    half2_t c0;   // 1024 + z
    half2_t c1;   // -(64 + z)
  };
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits, int z) {
    Col c;
    const _Float16 s = __builtin_bit_cast(_Float16, scale_bits);
    c.s = half2_t{s, s};
    const _Float16 a = (_Float16)(float)(1024 + z);
    const _Float16 b = (_Float16)(float)(-(64 + z));
    c.c0 = half2_t{a, a};
    c.c1 = half2_t{b, b};
    return c;
  }
  static __device__ __forceinline__ vec8 word(uint32_t q, const Col& c, uint32_t magic) {
    const half2_t r16 = half2_t{(_Float16)0.0625f, (_Float16)0.0625f};
    const uint32_t lo0 = and_or(q, 0x000f000fu, magic);
    const uint32_t hi0 = and_or(q, 0x00f000f0u, magic);
    q >>= 8;
    const uint32_t lo1 = and_or(q, 0x000f000fu, magic);
    const uint32_t hi1 = and_or(q, 0x00f000f0u, magic);
    const half2_t d0 = __builtin_bit_cast(half2_t, lo0) - c.c0;
    const half2_t d1 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, hi0), r16, c.c1);
    const half2_t d2 = __builtin_bit_cast(half2_t, lo1) - c.c0;
    const half2_t d3 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, hi1), r16, c.c1);
    const half2_t w0 = d0 * c.s, w1 = d1 * c.s, w2 = d2 * c.s, w3 = d3 * c.s;
    return vec8{w0.x, w0.y, w1.x, w1.y, w2.x, w2.y, w3.x, w3.y};
  }
  // word() one instruction at a time, for kernels that place the instructions themselves: pair
  // `part` (0..3) of the word is stage3(stage2(stage1(part < 2 ? q : q >> 8, part, magic), c, part), c)
  typedef half2_t Mid;
  static __device__ __forceinline__ uint32_t stage1(uint32_t q, int part, uint32_t magic) {
    return and_or(q, (part & 1) ? 0x00f000f0u : 0x000f000fu, magic);
  }
  static __device__ __forceinline__ Mid stage2(uint32_t x, const Col& c, int part) {
    const half2_t r16 = half2_t{(_Float16)0.0625f, (_Float16)0.0625f};
    if (part & 1) return __builtin_elementwise_fma(__builtin_bit_cast(half2_t, x), r16, c.c1);
    return __builtin_bit_cast(half2_t, x) - c.c0;
  }
  static __device__ __forceinline__ uint32_t stage3(Mid y, const Col& c) {
    return __builtin_bit_cast(uint32_t, y * c.s);
  }
  static __device__ __forceinline__ floatx4_t mfma(vec8 w, vec8 a, floatx4_t acc) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(w, a, acc, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    return __builtin_bit_cast(uint16_t, (_Float16)f);
  }
  static __device__ __forceinline__ float to_float(uint16_t b) {
    return (float)__builtin_bit_cast(_Float16, b);
  }
};

// ---------------------------------------------------------------- bf16
// gfx950 has no packed bf16 arithmetic.  The same fp16 magic numbers are used
// and each half is widened inside a mixed-precision fma: with S = float(s),
// fma(1024 + v, S, -(1024 + z) S) and fma(1024 + 16 v, S/16, -(64 + z) S) are
// exact in fp32 (at most 19 significant bits per term, result (v - z) S has at
// most 12), so the only rounding is the fp32 -> bf16 conversion
// (v_cvt_pk_bf16_f32, round to nearest even).
template <>
struct Dq<__bf16> {
  typedef bf16x8_t vec8;
  struct Col {
    float s, s16, c0, c1;
  };
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits, int z) {
    Col c;
    c.s = __builtin_bit_cast(float, (uint32_t)scale_bits << 16);
    c.s16 = c.s * 0.0625f;
    c.c0 = -(float)(1024 + z) * c.s;
    c.c1 = -(float)(64 + z) * c.s;
    return c;
  }
  static __device__ __forceinline__ bf16x2_t pair(uint32_t bits, float mul, float add) {
    const half2_t h = __builtin_bit_cast(half2_t, bits);
    const floatx2_t f = floatx2_t{__builtin_fmaf((float)h.x, mul, add),
                                  __builtin_fmaf((float)h.y, mul, add)};
    return __builtin_convertvector(f, bf16x2_t);
  }
  static __device__ __forceinline__ vec8 word(uint32_t q, const Col& c, uint32_t magic) {
    const uint32_t lo0 = and_or(q, 0x000f000fu, magic);
    const uint32_t hi0 = and_or(q, 0x00f000f0u, magic);
    q >>= 8;
    const uint32_t lo1 = and_or(q, 0x000f000fu, magic);
    const uint32_t hi1 = and_or(q, 0x00f000f0u, magic);
    const bf16x2_t w0 = pair(lo0, c.s, c.c0);
    const bf16x2_t w1 = pair(hi0, c.s16, c.c1);
    const bf16x2_t w2 = pair(lo1, c.s, c.c0);
    const bf16x2_t w3 = pair(hi1, c.s16, c.c1);
    return vec8{w0.x, w0.y, w1.x, w1.y, w2.x, w2.y, w3.x, w3.y};
  }
  // word() in three stages (see Dq<_Float16>)
  typedef floatx2_t Mid;
  static __device__ __forceinline__ uint32_t stage1(uint32_t q, int part, uint32_t magic) {
    return and_or(q, (part & 1) ? 0x00f000f0u : 0x000f000fu, magic);
  }
  static __device__ __forceinline__ Mid stage2(uint32_t x, const Col& c, int part) {
    const half2_t h = __builtin_bit_cast(half2_t, x);
    const float mul = (part & 1) ? c.s16 : c.s, add = (part & 1) ? c.c1 : c.c0;
    return floatx2_t{__builtin_fmaf((float)h.x, mul, add), __builtin_fmaf((float)h.y, mul, add)};
  }
  static __device__ __forceinline__ uint32_t stage3(Mid y, const Col&) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(y, bf16x2_t));
  }
  static __device__ __forceinline__ floatx4_t mfma(vec8 w, vec8 a, floatx4_t acc) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, a, acc, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);
  }
  static __device__ __forceinline__ float to_float(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
  }
};

// Per-lane constants of the four columns (j = 0..3) a lane dequantises, for
// the group `g` of strip `strip`.
template <typename T, bool HAS_ZP, typename D = Dq<T>>
__device__ __forceinline__ void load_cols(typename D::Col (&cols)[4], const uint16_t* scales,
                                          const uint32_t* zeros, int size_n, int strip, int g,
                                          int col16, bool grouped) {
  const uint16_t* srow = scales + (long)g * size_n + strip * kStripN;
  uint32_t zword = 0;
  if (HAS_ZP) zword = zeros[(long)g * (size_n / 8) + strip * 8 + zero_point_word(col16)];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int nl = 16 * j + col16;
    int z = 8;
    if (HAS_ZP) z = (int)((zword >> zero_point_shift(nl)) & 0xFu);
    cols[j] = D::make_col(srow[scale_slot(nl, grouped)], z);
  }
}

// 4-bit floating-point codes (float4_e2m1f: sign, 2 exponent bits with bias 1,
// 1 mantissa bit: 0, 0.5, 1, 1.5, 2, 3, 4, 6 and their negatives;
// dequant.h:397-470 of the reference).  With its sign at bit 15 and the other
// three bits at bits 11-9, a code is the fp16 number value * 2^-14 (the two
// subnormal codes become fp16 subnormals).  The scales are powers of two held
// in the activation type (the MX block scales, 2^(e - 127)); value * scale is
// exact, so the one conversion rounds nothing.  Same interface and row order
// as Dq: word() returns rows 0..7 of the column.  (This generic form is the
// arithmetic the bf16 specialisation below must reproduce; only bf16 is launched.)
template <typename T>
struct DqF4Generic {
  typedef typename Dq<T>::vec8 vec8;
  struct Col {
    float s;   // scale * 2^14
  };
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits, int) {
    return Col{Dq<T>::to_float(scale_bits) * 0x1p14f};
  }
  // codes in bits 12-15 and 28-31 of y -> two scaled values of T
  static __device__ __forceinline__ uint32_t pair(uint32_t y, float s) {
    const half2_t h = __builtin_bit_cast(half2_t, (y & 0x80008000u) | ((y & 0x70007000u) >> 3));
    return (uint32_t)Dq<T>::from_float((float)h.x * s) | ((uint32_t)Dq<T>::from_float((float)h.y * s) << 16);
  }
  static __device__ __forceinline__ vec8 word(uint32_t q, const Col& c, uint32_t) {
    // rows 0,1 are nibbles 0,4; rows 2,3 nibbles 1,5; rows 4,5 nibbles 2,6; rows 6,7 nibbles 3,7
    return __builtin_bit_cast(vec8, u32x4_t{pair(q << 12, c.s), pair(q << 8, c.s), pair(q << 4, c.s), pair(q, c.s)});
  }
};
template <typename T>
struct DqF4 : DqF4Generic<T> {};
// NVFP4 (dequant.h:397-470,518-549 of the reference): the same codes with one scale per column
// and 16 rows that is any number of the activation type with few significant bits (the
// reference's fp8 block scales, decoded by the caller): value * scale has at most five, so the
// generic form, which multiplies in fp32 and converts once, rounds nothing either.
template <typename T>
struct DqNvF4 : DqF4Generic<T> {};
// fp16: the code read as an fp16 number (value * 2^-14) times the scale * 2^14 in one packed
// multiply, the reference's own arithmetic (dequant.h:397-420, 520-531): scale * 2^14 is what
// the reference reads a scale byte as, at most 448 * 2^7.
template <>
struct DqNvF4<_Float16> {
  typedef Dq<_Float16>::vec8 vec8;
  struct Col {
    uint32_t s2;   // scale * 2^14, twice
  };
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits, int) {
    const _Float16 s = __builtin_bit_cast(_Float16, scale_bits) * (_Float16)16384.0f;
    const uint32_t b = __builtin_bit_cast(uint16_t, s);
    return Col{b | (b << 16)};
  }
  static __device__ __forceinline__ uint32_t pair(uint32_t y, uint32_t s2) {
    const half2_t h = __builtin_bit_cast(half2_t, (y & 0x80008000u) | ((y & 0x70007000u) >> 3));
    return __builtin_bit_cast(uint32_t, h * __builtin_bit_cast(half2_t, s2));
  }
  static __device__ __forceinline__ vec8 word(uint32_t q, const Col& c, uint32_t) {
    return __builtin_bit_cast(vec8, u32x4_t{pair(q << 12, c.s2), pair(q << 8, c.s2), pair(q << 4, c.s2), pair(q, c.s2)});
  }
};

// bf16: the matrix-core generation this is written for converts two 4-bit
// floats of a byte to bf16 and applies a power-of-two scale in one instruction
// (v_cvt_scalef32_pk_bf16_fp4: low nibble to the low half; only the exponent of
// the scale operand counts, and the MX block scales are powers of two).  Byte b
// of a word holds nibble slots 2b, 2b + 1, i.e. rows (0,2), (4,6), (1,3), (5,7);
// four byte permutes put the rows in order.
template <>
struct DqF4<__bf16> {
  typedef Dq<__bf16>::vec8 vec8;
  struct Col {
    float s;   // the block scale, a power of two
  };
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits, int) {
    return Col{Dq<__bf16>::to_float(scale_bits)};
  }
  static __device__ __forceinline__ vec8 word(uint32_t q, const Col& c, uint32_t) {
    const uint32_t r02 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, c.s, 0));
    const uint32_t r46 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, c.s, 1));
    const uint32_t r13 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, c.s, 2));
    const uint32_t r57 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, c.s, 3));
    // __builtin_amdgcn_perm(a, b, sel): bytes 0-3 of the selector space are b, 4-7 are a
    return __builtin_bit_cast(vec8, u32x4_t{__builtin_amdgcn_perm(r13, r02, 0x05040100u),
                                            __builtin_amdgcn_perm(r13, r02, 0x07060302u),
                                            __builtin_amdgcn_perm(r57, r46, 0x05040100u),
                                            __builtin_amdgcn_perm(r57, r46, 0x07060302u)});
  }
};

// bf16: the hardware conversion with a unit scale gives the code's value; the two values of a
// register (two rows of one column) are widened, multiplied by the scale in fp32 and cut back
// (the product has at most five significant bits: nothing is lost).
template <>
struct DqNvF4<__bf16> {
  typedef Dq<__bf16>::vec8 vec8;
  struct Col {
    float s;   // the block scale
  };
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits, int) {
    return Col{Dq<__bf16>::to_float(scale_bits)};
  }
  static __device__ __forceinline__ uint32_t scaled(uint32_t r, float s) {
    const float lo = __uint_as_float(r << 16) * s, hi = __uint_as_float(r & 0xFFFF0000u) * s;
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
  }
  static __device__ __forceinline__ vec8 word(uint32_t q, const Col& c, uint32_t) {
    const uint32_t r02 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, 1.0f, 0));
    const uint32_t r46 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, 1.0f, 1));
    const uint32_t r13 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, 1.0f, 2));
    const uint32_t r57 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, 1.0f, 3));
    return __builtin_bit_cast(vec8, u32x4_t{scaled(__builtin_amdgcn_perm(r13, r02, 0x05040100u), c.s),
                                            scaled(__builtin_amdgcn_perm(r13, r02, 0x07060302u), c.s),
                                            scaled(__builtin_amdgcn_perm(r57, r46, 0x05040100u), c.s),
                                            scaled(__builtin_amdgcn_perm(r57, r46, 0x07060302u), c.s)});
  }
};

// Eight neighbours of a permuted scale row of grouped scales, slots
// 8 (col16 % 8) .. + 7, hold the scales of columns 16 j + col16 (j = 0..3) and
// of their partners col16 +- 8: column 16 j + col16 is slot 2 j + col16 / 8
// (scale_slot with grouped = true).
__device__ __forceinline__ uint16_t chunk_scale(const uint4& sv, int j, int col16) {
  const uint32_t word = j == 0 ? sv.x : (j == 1 ? sv.y : (j == 2 ? sv.z : sv.w));
  return (uint16_t)(word >> (16 * (col16 >> 3)));
}

// The dequantiser of a 4-bit weight type (NV: float4 codes with arbitrary scales per 16 rows).
template <typename T, bool FP4, bool NV = false>
struct Dq4Of {
  typedef Dq<T> type;
};
template <typename T>
struct Dq4Of<T, true, false> {
  typedef DqF4<T> type;
};
template <typename T>
struct Dq4Of<T, true, true> {
  typedef DqNvF4<T> type;
};

// 8-bit codes (uint8b128, symmetric): (v - 128) * s with one rounding.  A
// packed word holds four rows of one column; word4 returns them as two
// registers (rows 0,1 and rows 2,3).  The code is OR-ed into the mantissa of
// fp16 1024.0 for both activation types (bf16 has too few mantissa bits for
// 128 + v); 1024 + 128 = 1152 comes off exactly, in fp16 or in fp32.
template <typename T>
struct Dq8;

template <>
struct Dq8<_Float16> {
  struct Col {
    half2_t s;
  };
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits) {
    const _Float16 s = __builtin_bit_cast(_Float16, scale_bits);
    return Col{half2_t{s, s}};
  }
  static __device__ __forceinline__ uint2 word4(uint32_t q, const Col& c, uint32_t magic) {
    const half2_t off = half2_t{(_Float16)1152.f, (_Float16)1152.f};
    const uint32_t lo = and_or(q, 0x00ff00ffu, magic);
    const uint32_t hi = and_or(q >> 8, 0x00ff00ffu, magic);
    const half2_t w0 = (__builtin_bit_cast(half2_t, lo) - off) * c.s;
    const half2_t w1 = (__builtin_bit_cast(half2_t, hi) - off) * c.s;
    return make_uint2(__builtin_bit_cast(uint32_t, w0), __builtin_bit_cast(uint32_t, w1));
  }
};

template <>
struct Dq8<__bf16> {
  struct Col {
    float s, c0;
  };
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits) {
    Col c;
    c.s = __builtin_bit_cast(float, (uint32_t)scale_bits << 16);
    c.c0 = -1152.f * c.s;  // 9 * 2^7 times an 8-bit mantissa: exact
    return c;
  }
  static __device__ __forceinline__ uint2 word4(uint32_t q, const Col& c, uint32_t magic) {
    const uint32_t lo = and_or(q, 0x00ff00ffu, magic);
    const uint32_t hi = and_or(q >> 8, 0x00ff00ffu, magic);
    // (1024 + v) * s - 1152 s: both products and their sum are exact in fp32
    const bf16x2_t w0 = Dq<__bf16>::pair(lo, c.s, c.c0);
    const bf16x2_t w1 = Dq<__bf16>::pair(hi, c.s, c.c0);
    return make_uint2(__builtin_bit_cast(uint32_t, w0), __builtin_bit_cast(uint32_t, w1));
  }
};

// 8-bit floating-point codes (float8_e4m3fn: sign, 4 exponent bits with bias
// 7, 3 mantissa bits; dequant.h:320-380 of the reference).  Moved one bit to
// the right below the sign, a code is the fp16 number v * 2^-8 (subnormal
// codes become fp16 subnormals, so this holds for all of them; the two NaN
// codes read as +-480).  The scales arrive with the exponent bias already
// folded in (marlin_utils_fp8.py:35-46): s * 2^8 for fp16, s * 2^120 for bf16.
// fp16: one packed multiply by that scale, as the reference's.  bf16: the
// reference reads the code as the bf16 number v * 2^-120 and multiplies by
// s * 2^120; here the fp16 reading is widened and multiplied by
// (s * 2^120) * 2^-112 in fp32 -- the same exact product v * s, rounded once.
// Same interface and row order as Dq8.
template <typename T>
struct Dq8F;

__device__ __forceinline__ uint32_t fp8_pair_as_fp16(uint32_t y) {  // codes in bits 8-15 and 24-31
  return (y & 0x80008000u) | ((y & 0x7f007f00u) >> 1);
}

template <>
struct Dq8F<_Float16> {
  typedef Dq8<_Float16>::Col Col;
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits) { return Dq8<_Float16>::make_col(scale_bits); }
  static __device__ __forceinline__ uint2 word4(uint32_t q, const Col& c, uint32_t) {
    const half2_t w0 = __builtin_bit_cast(half2_t, fp8_pair_as_fp16(q << 8)) * c.s;
    const half2_t w1 = __builtin_bit_cast(half2_t, fp8_pair_as_fp16(q)) * c.s;
    return make_uint2(__builtin_bit_cast(uint32_t, w0), __builtin_bit_cast(uint32_t, w1));
  }
};

template <>
struct Dq8F<__bf16> {
  struct Col {
    float s;
  };
  static __device__ __forceinline__ Col make_col(uint16_t scale_bits) {
    return Col{__builtin_bit_cast(float, (uint32_t)scale_bits << 16) * 0x1p-112f};
  }
  static __device__ __forceinline__ bf16x2_t scaled(uint32_t fp16_pair, float s) {
    const half2_t h = __builtin_bit_cast(half2_t, fp16_pair);
    return __builtin_convertvector(floatx2_t{(float)h.x * s, (float)h.y * s}, bf16x2_t);
  }
  static __device__ __forceinline__ uint2 word4(uint32_t q, const Col& c, uint32_t) {
    const bf16x2_t w0 = scaled(fp8_pair_as_fp16(q << 8), c.s);
    const bf16x2_t w1 = scaled(fp8_pair_as_fp16(q), c.s);
    return make_uint2(__builtin_bit_cast(uint32_t, w0), __builtin_bit_cast(uint32_t, w1));
  }
};

// The dequantiser of an 8-bit weight type.
template <typename T, bool FP8>
struct Dq8Of {
  typedef Dq8<T> type;
};
template <typename T>
struct Dq8Of<T, true> {
  typedef Dq8F<T> type;
};

// One packed word whose eight rows (8 consecutive k) may lie in different groups:
// a shard of an act-order matrix that does not hold whole groups.  `groups`
// holds the group of each row, `scale_col` points at this column's scale of
// group 0, `group_stride` is the distance between groups in elements.  The
// exact integers v - 8 times the scale of the row's group, rounded once, as
// the reference's dequantise-then-scale (products of two 16-bit floats are
// exact in fp32, so rounding the fp32 product is the 16-bit multiply).
template <typename T>
__device__ __forceinline__ typename Dq<T>::vec8 word_by_row_groups(uint32_t q, const int (&groups)[8],
                                                                  const uint16_t* scale_col, long group_stride,
                                                                  uint32_t magic) {
  typedef typename Dq<T>::vec8 vec8;
  const typename Dq<T>::Col unit = Dq<T>::make_col(Dq<T>::from_float(1.0f), 8);
  const vec8 w0 = Dq<T>::word(q, unit, magic);
  const u32x4_t in = __builtin_bit_cast(u32x4_t, w0);
  const uint32_t regs[4] = {in.x, in.y, in.z, in.w};
  uint32_t out[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float lo = Dq<T>::to_float((uint16_t)(regs[r] & 0xffffu)) *
                     Dq<T>::to_float(scale_col[(long)groups[2 * r] * group_stride]);
    const float hi = Dq<T>::to_float((uint16_t)(regs[r] >> 16)) *
                     Dq<T>::to_float(scale_col[(long)groups[2 * r + 1] * group_stride]);
    out[r] = (uint32_t)Dq<T>::from_float(lo) | ((uint32_t)Dq<T>::from_float(hi) << 16);
  }
  return __builtin_bit_cast(vec8, u32x4_t{out[0], out[1], out[2], out[3]});
}

// The same for one packed word of 8-bit codes (four rows of one column, uint8b128):
// the exact integers v - 128 times the scale of each row's group, rounded once.
template <typename T>
__device__ __forceinline__ uint2 word4_by_row_groups8(uint32_t q, const int* groups4, const uint16_t* scale_col,
                                                      long group_stride, uint32_t magic) {
  const uint2 w0 = Dq8<T>::word4(q, Dq8<T>::make_col(Dq<T>::from_float(1.0f)), magic);
  const uint32_t regs[2] = {w0.x, w0.y};
  uint32_t out[2];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const float lo = Dq<T>::to_float((uint16_t)(regs[r] & 0xffffu)) *
                     Dq<T>::to_float(scale_col[(long)groups4[2 * r] * group_stride]);
    const float hi = Dq<T>::to_float((uint16_t)(regs[r] >> 16)) *
                     Dq<T>::to_float(scale_col[(long)groups4[2 * r + 1] * group_stride]);
    out[r] = (uint32_t)Dq<T>::from_float(lo) | ((uint32_t)Dq<T>::from_float(hi) << 16);
  }
  return make_uint2(out[0], out[1]);
}

}  // namespace sonar
