// Device helpers shared by the GEMM kernels: vector types for the MFMA builtins and the
// nibble -> fp16 conversion applied in registers right before an MFMA.
//
// Dequantized value: fp16( scale * (q - zp) ) with ONE rounding -- bit-identical to the reference's
// host-side dequantization (reference: test/blkq4_fp16_gemm_sm80_test.cu:314-328).  The packed word
// layout (see blkq4_device.h) puts the pair (k0+2i, k0+2i+1) at nibble positions i and i+4, so
//   (w & 0x000f000f) | 0x64006400  is the fp16 pair (1024 + q, 1024 + q)   (ulp of 1024 is 1)
//   (w & 0x00f000f0) | 0x54005400  is the fp16 pair (  64 + q,   64 + q)   (ulp of 64 is 1/16)
// and one shift by 8 exposes the other two pairs the same way.  Adding -(1024 + zp) resp. -(64 + zp)
// is exact (small integers), the multiplication by the scale rounds once.  Per 8 weights: 1 shift,
// 4 and-or, 4 packed adds, 4 packed multiplies.

#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace blkq4 {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half2_t as_half2(uint32_t x) { return __builtin_bit_cast(half2_t, x); }
__device__ __forceinline__ uint32_t as_u32(half2_t x) { return __builtin_bit_cast(uint32_t, x); }

// Per-(block, column) constants of the conversion.
struct DequantConsts {
  half2_t scale2;  // (s, s)
  half2_t neg_c0;  // (-(1024 + zp), -(1024 + zp))
  half2_t neg_c1;  // (-(64 + zp),   -(64 + zp))
};

// scale_bits: fp16 bit pattern; zp: 0..15
__device__ __forceinline__ DequantConsts make_dequant_consts(uint32_t scale_bits, uint32_t zp) {
  DequantConsts c;
  c.scale2 = as_half2(scale_bits | (scale_bits << 16));
  const uint32_t c0 = 0xE400u | zp;         // -(1024 + zp): 0x6400 is 1024.0, ulp 1, sign bit set
  const uint32_t c1 = 0xD400u | (zp << 4);  // -(64 + zp):   0x5400 is 64.0, ulp 1/16, sign bit set
  c.neg_c0 = as_half2(c0 | (c0 << 16));
  c.neg_c1 = as_half2(c1 | (c1 << 16));
  return c;
}

// One packed word (8 weights k0..k0+7 of one column) -> 8 fp16 in k order.
__device__ __forceinline__ half8_t dequant_word(uint32_t w, const DequantConsts& c) {
  const uint32_t y = w >> 8;
  const half2_t p0 = (as_half2((w & 0x000f000fu) | 0x64006400u) + c.neg_c0) * c.scale2;  // k0, k0+1
  const half2_t p1 = (as_half2((w & 0x00f000f0u) | 0x54005400u) + c.neg_c1) * c.scale2;  // k0+2, k0+3
  const half2_t p2 = (as_half2((y & 0x000f000fu) | 0x64006400u) + c.neg_c0) * c.scale2;  // k0+4, k0+5
  const half2_t p3 = (as_half2((y & 0x00f000f0u) | 0x54005400u) + c.neg_c1) * c.scale2;  // k0+6, k0+7
  half8_t r;
  r[0] = p0[0]; r[1] = p0[1];
  r[2] = p1[0]; r[3] = p1[1];
  r[4] = p2[0]; r[5] = p2[1];
  r[6] = p3[0]; r[7] = p3[1];
  return r;
}

// The four literals of the conversion, held in VGPRs: with register operands `(w & mask) | magic`
// is one v_and_or_b32 (a VOP3 instruction can carry at most one literal, so with literal operands
// it becomes two instructions).  `opaque()` hides the value from constant propagation.
struct DequantMasks {
  uint32_t lo_mask, hi_mask, magic_1024, magic_64;
  __device__ __forceinline__ static uint32_t opaque(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
  }
  __device__ __forceinline__ static DequantMasks make() {
    DequantMasks m;
    m.lo_mask = opaque(0x000f000fu);
    m.hi_mask = opaque(0x00f000f0u);
    m.magic_1024 = opaque(0x64006400u);
    m.magic_64 = opaque(0x54005400u);
    return m;
  }
};

// Pair `pair` (0..3) of a packed word: the fp16 values of weights k0 + 2*pair and k0 + 2*pair + 1.
// `w_shifted` is the word itself for pairs 0/1 and the word shifted right by 8 for pairs 2/3.
// Three instructions: v_and_or_b32, v_pk_add_f16, v_pk_mul_f16.
__device__ __forceinline__ half2_t dequant_pair(uint32_t w_shifted, int pair, const DequantConsts& c,
                                                const DequantMasks& m) {
  if ((pair & 1) == 0) return (as_half2((w_shifted & m.lo_mask) | m.magic_1024) + c.neg_c0) * c.scale2;
  return (as_half2((w_shifted & m.hi_mask) | m.magic_64) + c.neg_c1) * c.scale2;
}

// Blocks along N: the constants that one pair of weights is added to, built from the packed zero-point
// word of the pair (reference order: bytes 0 and 2 of the word are rows 2p and 2p + 1 of the 16-row group,
// bytes 1 and 3 rows 2p + 8 and 2p + 9).  hh selects the rows (0: the first eight of the group), pair
// parity the magic number (even pairs 1024 + q, odd pairs 64 + q with the zero-point shifted likewise).
struct RowMetaMasks {
  uint32_t byte_pair, byte_pair_x16, neg_1024, neg_64;
  __device__ __forceinline__ static RowMetaMasks make() {
    RowMetaMasks m;
    m.byte_pair = DequantMasks::opaque(0x00ff00ffu);
    m.byte_pair_x16 = DequantMasks::opaque(0x0ff00ff0u);
    m.neg_1024 = DequantMasks::opaque(0xE400E400u);
    m.neg_64 = DequantMasks::opaque(0xD400D400u);
    return m;
  }
};
template <bool HAS_ZP>
__device__ __forceinline__ half2_t row_neg_c(uint32_t zp_word, int pair, int hh, const RowMetaMasks& m) {
  if (!HAS_ZP) return as_half2((pair & 1) == 0 ? 0xE408E408u : 0xD480D480u);  // zero-point 8
  if ((pair & 1) == 0) return as_half2((((hh == 0) ? zp_word : (zp_word >> 8)) & m.byte_pair) | m.neg_1024);
  return as_half2((((hh == 0) ? (zp_word << 4) : (zp_word >> 4)) & m.byte_pair_x16) | m.neg_64);
}
// component c of a 4-word vector, c known at compile time after unrolling
__device__ __forceinline__ uint32_t vec_word(const uint4& v, int c) { return c == 0 ? v.x : c == 1 ? v.y : c == 2 ? v.z : v.w; }

__device__ __forceinline__ half8_t as_half8(uint4 v) {
  uint4_t t = {v.x, v.y, v.z, v.w};
  return __builtin_bit_cast(half8_t, t);
}

__device__ __forceinline__ uint16_t float_to_half_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h)));
}

// ---- bf16 ------------------------------------------------------------------------------------------------
// Dequantized value: bf16( scale * (q - zp) ) with ONE rounding, the same definition as for fp16 with the
// other 16-bit type.  The nibbles become fp16 pairs (1024 + q) resp. (64 + q) exactly as above; each half is
// then the fp16 operand of a mixed-precision fma with the scale and -(1024 + zp) * scale resp. -(64 + zp) * scale
// in fp32 (v_fma_mix_f32 converts the fp16 operand exactly).  A bf16 scale is m * 2^e with an 8-bit m, 1024 + zp
// has 11 bits, so the constant is exact in fp32 (19 bits) and the fma returns scale * (q - zp) exactly (12
// bits); the packed conversion to bf16 does the one rounding.  Per 8 weights: 1 shift, 4 and-or, 8 fmas,
// 4 packed conversions.  Scales beyond 2^118 overflow the constant (1039 * scale) although 15 * scale would
// still be finite: such scales are outside the GEMM's range.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __builtin_bit_cast(float, b << 16); }
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));  // round to nearest even
}

struct Bf16Consts {
  float scale;   // s
  float neg_c0;  // -(1024 + zp) * s, exact
  float neg_c1;  // -(64 + zp) * s, exact
};
__device__ __forceinline__ Bf16Consts make_bf16_consts(uint32_t scale_bits, uint32_t zp) {
  Bf16Consts c;
  c.scale = bf16_bits_to_float(scale_bits);
  c.neg_c0 = -(static_cast<float>(1024u + zp) * c.scale);
  c.neg_c1 = -(static_cast<float>(64u + zp) * c.scale);
  return c;
}
// One packed word (8 weights k0..k0+7 of one column) -> 8 bf16 in k order.
__device__ __forceinline__ bf16x8_t dequant_word_bf16(uint32_t w, const Bf16Consts& c, const DequantMasks& m) {
  const uint32_t y = w >> 8;
  const half2_t p0 = as_half2((w & m.lo_mask) | m.magic_1024);  // 1024 + q of k0, k0+1
  const half2_t p1 = as_half2((w & m.hi_mask) | m.magic_64);    //   64 + q of k0+2, k0+3
  const half2_t p2 = as_half2((y & m.lo_mask) | m.magic_1024);  // k0+4, k0+5
  const half2_t p3 = as_half2((y & m.hi_mask) | m.magic_64);    // k0+6, k0+7
  bf16x8_t r;
  r[0] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(p0[0]), c.scale, c.neg_c0));
  r[1] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(p0[1]), c.scale, c.neg_c0));
  r[2] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(p1[0]), c.scale, c.neg_c1));
  r[3] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(p1[1]), c.scale, c.neg_c1));
  r[4] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(p2[0]), c.scale, c.neg_c0));
  r[5] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(p2[1]), c.scale, c.neg_c0));
  r[6] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(p3[0]), c.scale, c.neg_c1));
  r[7] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(p3[1]), c.scale, c.neg_c1));
  return r;
}
// Blocks along N: the weights k and k + 1 of a pair have scales of their own (a packed pair of bf16).  d holds
// q - zp of both, exact in fp16; each product with its scale is exact in fp32 (4 + 8 bits), the packed
// conversion does the one rounding.  Two instructions for the scales, two mixed-precision fmas, one conversion.
__device__ __forceinline__ uint32_t row_pair_bf16(half2_t d, uint32_t scale_pair) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const float s0 = __builtin_bit_cast(float, scale_pair << 16);
  const float s1 = __builtin_bit_cast(float, scale_pair & 0xffff0000u);
  bf16x2_t v;
  // (written as fmas with a zero addend: one v_fma_mix_f32 per weight, where a conversion and a multiply would be two;
  // a zero weight comes out as +0 whatever the scale's sign, which no sum can tell from -0)
  v[0] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(d[0]), s0, 0.0f));
  v[1] = static_cast<__bf16>(__builtin_fmaf(static_cast<float>(d[1]), s1, 0.0f));
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ bf16x8_t as_bf16x8(uint4 v) {
  uint4_t t = {v.x, v.y, v.z, v.w};
  return __builtin_bit_cast(bf16x8_t, t);
}

// c + bias the way an fp16 tensor library adds two fp16 tensors: in fp32, rounded to fp16 (the reference
// module adds its bias to the fp16 output of the GEMM, python/ms_blkq4linear.py:26-27).
__device__ __forceinline__ uint32_t add_bias_bits(uint32_t c, uint32_t bias) {
  return float_to_half_bits(half_bits_to_float(c) + half_bits_to_float(bias));
}
__device__ __forceinline__ uint32_t add_bias_pair(uint32_t c, uint32_t bias) {
  return add_bias_bits(c & 0xffffu, bias & 0xffffu) | (add_bias_bits(c >> 16, bias >> 16) << 16);
}

// the same for either 16-bit type
template <bool BF>
__device__ __forceinline__ uint32_t float_to_bits(float f) {
  return BF ? float_to_bf16_bits(f) : float_to_half_bits(f);
}
template <bool BF>
__device__ __forceinline__ uint32_t add_bias_bits_t(uint32_t c, uint32_t bias) {
  if (BF) return float_to_bf16_bits(bf16_bits_to_float(c) + bf16_bits_to_float(bias));
  return add_bias_bits(c, bias);
}
template <bool BF>
__device__ __forceinline__ uint32_t add_bias_pair_t(uint32_t c, uint32_t bias) {
  return add_bias_bits_t<BF>(c & 0xffffu, bias & 0xffffu) | (add_bias_bits_t<BF>(c >> 16, bias >> 16) << 16);
}

}  // namespace blkq4
