// Fused quantize + pack kernel and the layout conversion kernels (gfx950).
//
// One pass: every fp16 weight is read once (coalesced 16-byte loads along K), the block range is
// reduced across the 2/4/8 neighbouring lanes that share a quantization block, scale and zero-point
// are derived, the eight weights a lane holds become one packed 32-bit word, and words, scales and
// zero-points leave through LDS so that global stores are coalesced in the packed layouts described
// in blkq4_device.h.  No temporary device buffers.
//
// Arithmetic (every rounding point) follows the reference quantizer
// (reference: src/mickey/blk_q4/f16_quant_sm80.cuh:96-141 and :261-313):
//   fp16 -> fp32 exactly; min/max with strict compares in ascending k; asymmetric: range widened to
//   include 0, scale_f = (max - min) / 15 (IEEE divide), zp = roundf(0 - min / scale_f) clamped to
//   0..15, scale = fp16(scale_f); symmetric: scale = fp16(extreme / -8) with ties going to min;
//   q = clamp(roundf(fmaf(v, 1 / float(scale), zp)), 0, 15) with the fp16-rounded scale re-read.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_device.h"
#include "blkq4_launch.h"

namespace {

constexpr int kTileN = 64;    // columns (n) per workgroup, blocks along N
constexpr int kTileK = 256;   // rows (k) per workgroup
// Blocks along K: 32 columns per workgroup, four 16-byte loads per lane.  A kernel that moves the same bytes the same
// way and computes nothing was measured on K = 8192, N = 28672 with blocks of 16 for several tile shapes: 64 x 256
// (eight loads per lane) 105.4 - 106.5 us, 32 x 256 103.6, 32 x 512 with 1 KiB per wave-load 105.7, 64 x 512 and 128 x 256
// (sixteen loads per lane) 108 - 109; a pure read of the source takes 67 us, a fill of the outputs 26 us.
constexpr int kColTileN = 32;
constexpr int kThreads = 256;

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h)));
}

__device__ __forceinline__ uint16_t float_to_half_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));  // v_cvt_f16_f32, round to nearest even
}

// roundf (halves away from zero) for 0 <= x <= 15 as one add and one truncating conversion.  The
// constant is the largest float below 0.5: x + c lands on the next integer exactly when
// x - floor(x) >= 0.5 (checked against roundf for every float in [0, 16]); adding 0.5 itself would
// round 0.49999997 up to 1.
__device__ __forceinline__ uint32_t round_0_to_15(float x) {
  return static_cast<uint32_t>(__fadd_rn(x, 0.49999997f));
}

// x / 15 with IEEE rounding for 0 <= x < 2^19 (the range of a block of fp16 values is 0 or lies in
// [2^-24, 131008]): estimate with the rounded reciprocal, exact residual, one correction.  Checked
// against the division for every float in [2^-30, 2^19].
__device__ __forceinline__ float div_by_15(float x) {
  const float y = 1.0f / 15.0f;
  const float q = __fmul_rn(x, y);
  const float r = __fmaf_rn(-q, 15.0f, x);
  return __fmaf_rn(r, y, q);
}

// ---- shortened forms of the quantizer's divisions and of its rounding (fp16 only) ----------------------------
// The full IEEE division is a sequence of about eleven instructions, and the quantizer is bound by its vector
// instructions, not by memory.  Over the quantizer's domain the short sequences below give the very same bits;
// that is not argued but checked: quant_selfcheck_kernel (at the end of this file) compares each of them with
// the IEEE form over its WHOLE domain on the GPU it runs on, and a test runs that check.

// 1 / s for s = an fp16 value (normal or subnormal, not 0, inf or nan) widened to fp32: one Newton step on the
// hardware's reciprocal estimate.
__device__ __forceinline__ float reciprocal_of_fp16_value(float s) {
  const float y = __builtin_amdgcn_rcpf(s);
  const float e = __fmaf_rn(-s, y, 1.0f);
  return __fmaf_rn(e, y, y);
}

// a / b where b = RN((mx - a) / 15) for fp16 values a <= 0 <= mx, b != 0 (the zero-point's division): estimate
// with the reciprocal, exact residual, one correction.
__device__ __forceinline__ float zero_point_quotient(float a, float b) {
  const float y = __builtin_amdgcn_rcpf(b);
  const float q = __fmul_rn(a, y);
  const float r = __fmaf_rn(-b, q, a);
  return __fmaf_rn(r, y, q);
}

// roundf for 0 <= x <= 15 in one instruction: v_cvt_rpi_i32_f32 is floor(x + 0.5) of the exact sum
__device__ __forceinline__ uint32_t round_0_to_15_rpi(float x) {
  uint32_t r;
  asm("v_cvt_rpi_i32_f32 %0, %1" : "=v"(r) : "v"(x));
  return r;
}

// A lane's value exchanged with lane ^ 1, lane ^ 2 and with the mirrored lane of its group of eight (which lies
// in the other group of four): the three steps of a reduction over 2, 4 or 8 neighbouring lanes, without LDS.
template <int kStep>
__device__ __forceinline__ uint32_t exchange_in_group(uint32_t x) {
  constexpr int kCtrl = kStep == 1 ? 0xB1    // quad_perm [1, 0, 3, 2]
                        : kStep == 2 ? 0x4E  // quad_perm [2, 3, 0, 1]
                                     : 0x141;  // row_half_mirror
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), kCtrl, 0xf, 0xf, true));
}

// The scale is rounded twice: to fp32 by the division, then to the 16-bit type.  Handed the two steps as one
// expression the compiler folds the division's last fused multiply-add and the conversion into ONE instruction
// (v_fma_mixlo_f16) that rounds once, which differs from the reference in about one scale of 10^4.  The value passes
// through this (empty) statement so that it exists as an fp32 number before it is converted.
__device__ __forceinline__ float rounded_to_fp32(float x) {
  asm volatile("" : "+v"(x));
  return x;
}

// source and packed weights are touched once per launch: non-temporal requests
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_once_16(const void* p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store_once_16(void* p, const uint4& v) {
  __builtin_nontemporal_store(u32x4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4_t*>(p));
}

// nibble position of weight t (0..7) inside its 32-bit word
__device__ __forceinline__ constexpr int nibble_shift(int t) { return 4 * ((t >> 1) + 4 * (t & 1)); }

// bf16: the other 16-bit type, the same arithmetic (a block's range is not bounded by 2^19 there, so the
// division by 15 is the plain IEEE one)
__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __builtin_bit_cast(float, b << 16); }
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));  // round to nearest even
}
template <bool BF>
__device__ __forceinline__ float bits_to_float(uint32_t b) { return BF ? bf16_bits_to_float(b) : half_bits_to_float(b); }
template <bool BF>
__device__ __forceinline__ uint16_t float_to_bits(float f) { return BF ? float_to_bf16_bits(f) : float_to_half_bits(f); }

// What the quantizer derives from a block's range: the scale as it is stored, the zero-point, and the reciprocal of
// the stored scale (0 when that scale is zero) that the weights are multiplied with.
struct BlockQuant {
  uint32_t scale_bits;
  uint32_t zp;
  float reciprocal_scale;
};

// The definition (IEEE divisions throughout), both element types.
//   asymmetric: range2scalezp, reference f16_quant_sm80.cuh:96-122; symmetric: range2scale, :124-135 (the all-zero
//   block's sign is the caller's business); the scale re-read after its rounding, :291-297 (-0.0 counts as zero).
template <bool HAS_ZP, bool BF>
__device__ __forceinline__ BlockQuant block_quant_ieee(float mn, float mx) {
  BlockQuant b;
  if constexpr (HAS_ZP) {
    const float rmn = fminf(mn, 0.0f);
    const float rmx = fmaxf(mx, 0.0f);
    const float scale_f = rounded_to_fp32(BF ? __fdiv_rn(__fsub_rn(rmx, rmn), 15.0f) : div_by_15(__fsub_rn(rmx, rmn)));
    float zero_point_fp = rmn;
    if (scale_f != 0.0f) zero_point_fp = __fsub_rn(0.0f, __fdiv_rn(rmn, scale_f));
    if (zero_point_fp < 0.0f) {
      b.zp = 0;
    } else if (zero_point_fp > 15.0f) {
      b.zp = 15;
    } else {
      b.zp = round_0_to_15(zero_point_fp);
    }
    b.scale_bits = float_to_bits<BF>(scale_f);
  } else {
    const float m = fabsf(mx) > fabsf(mn) ? mx : mn;
    b.scale_bits = float_to_bits<BF>(rounded_to_fp32(__fdiv_rn(m, -8.0f)));
    b.zp = 8;
  }
  const float scale = bits_to_float<BF>(b.scale_bits);
  b.reciprocal_scale = (scale != 0.0f) ? __fdiv_rn(1.0f, scale) : 0.0f;
  return b;
}

// The same for fp16 with the shortened sequences (about 20 instructions instead of 45, no branches).
template <bool HAS_ZP>
__device__ __forceinline__ BlockQuant block_quant_fp16(float mn, float mx) {
  BlockQuant b;
  if constexpr (HAS_ZP) {
    const float rmn = fminf(mn, 0.0f);
    const float rmx = fmaxf(mx, 0.0f);
    const float scale_f = rounded_to_fp32(div_by_15(__fsub_rn(rmx, rmn)));
    // scale_f is zero only for rmn = rmx = 0: the quotient is then 0 * (1 / 1e-30) = 0 and the zero-point 0, which is
    // what the definition gives; every other scale_f is at least 2^-24 / 15.  Clamping before rounding equals the
    // definition's compare-then-round: round(0) = 0, round(15) = 15.
    const float q = zero_point_quotient(rmn, fmaxf(scale_f, 1e-30f));
    b.zp = round_0_to_15_rpi(__builtin_amdgcn_fmed3f(-q, 0.0f, 15.0f));
    b.scale_bits = float_to_half_bits(scale_f);
  } else {
    const float m = fabsf(mx) > fabsf(mn) ? mx : mn;
    b.scale_bits = float_to_half_bits(__fmul_rn(m, -0.125f));  // exact: a power of two
    b.zp = 8;
  }
  const float scale = half_bits_to_float(b.scale_bits);
  // normal or subnormal of either sign: everything but zero, infinity and nan
  const bool invertible = __builtin_amdgcn_classf(scale, 0x008 | 0x010 | 0x080 | 0x100);
  b.reciprocal_scale = invertible ? reciprocal_of_fp16_value(scale) : 0.0f;
  return b;
}

template <bool HAS_ZP, bool BF>
__device__ __forceinline__ BlockQuant block_quant(float mn, float mx) {
  if constexpr (BF) {
    return block_quant_ieee<HAS_ZP, true>(mn, mx);
  } else {
    return block_quant_fp16<HAS_ZP>(mn, mx);
  }
}

// One weight: clamp(roundf(fmaf(v, reciprocal_scale, zp)), 0, 15) (reference: f16_quant_sm80.cuh:296-313); clamping
// before rounding gives the same nibble as the reference's round-then-clamp (both are monotonic).
template <bool BF>
__device__ __forceinline__ uint32_t quantize_one(float v, float reciprocal_scale, float zp_f) {
  const float r = __builtin_amdgcn_fmed3f(__fmaf_rn(v, reciprocal_scale, zp_f), 0.0f, 15.0f);
  return BF ? round_0_to_15(r) : round_0_to_15_rpi(r);
}

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
// (inline assembly: written as minnum / maxnum the compiler first canonicalises every loaded word with an instruction
// of its own, which is what these instructions do to their operands anyway)
__device__ __forceinline__ uint32_t pk_min_f16(uint32_t a, uint32_t b) {
  uint32_t d;
  asm("v_pk_min_f16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
__device__ __forceinline__ uint32_t pk_max_f16(uint32_t a, uint32_t b) {
  uint32_t d;
  asm("v_pk_max_f16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
// minimum / maximum of the two halves of a, in the low half of the result
__device__ __forceinline__ uint32_t pk_min_f16_halves(uint32_t a) {
  uint32_t d;
  asm("v_pk_min_f16 %0, %1, %1 op_sel:[0,1] op_sel_hi:[1,0]" : "=v"(d) : "v"(a));
  return d;
}
__device__ __forceinline__ uint32_t pk_max_f16_halves(uint32_t a) {
  uint32_t d;
  asm("v_pk_max_f16 %0, %1, %1 op_sel:[0,1] op_sel_hi:[1,0]" : "=v"(d) : "v"(a));
  return d;
}

template <int BS, bool HAS_ZP, bool ALIGNED, bool BF = false>
__global__ __launch_bounds__(kThreads) void prepack_kernel(const uint16_t* __restrict__ src, int K,
                                                           int N, int ld,
                                                           uint4* __restrict__ packed_w,
                                                           uint16_t* __restrict__ scales,
                                                           uint8_t* __restrict__ zps, unsigned k_tiles,
                                                           bool wide_meta) {
  constexpr int kLanesPerBlock = BS / 8;     // lanes sharing one quantization block
  constexpr int kBlocksPerTile = kTileK / BS;  // quantization blocks along K in one tile
  __shared__ uint32_t w_lds[kTileK / 32][kColTileN][4];
  __shared__ __attribute__((aligned(8))) uint16_t s_lds[kBlocksPerTile][kColTileN];
  __shared__ __attribute__((aligned(4))) uint8_t z_lds[kBlocksPerTile][kColTileN];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  // consecutive workgroups walk along k: they read consecutive 512-byte pieces of the same 32 rows
  const int k0 = static_cast<int>(blockIdx.x % k_tiles) * kTileK;
  const int n0 = static_cast<int>(blockIdx.x / k_tiles) * kColTileN;

  const int kl = (lane & 31) * 8;  // this lane's first k inside the tile

  // Issue every load of the wave first: 4 x 16 bytes per lane in flight.  Lanes past the end of the matrix (K is a
  // multiple of 64, so a lane's 8 weights and the lanes that share a block are all in or all out) read the last valid
  // place instead: what they compute is never stored, and the loads need no branches.
  constexpr int kLoads = kColTileN / 8;  // per lane: a wave covers two columns per load
  uint4 raw[kLoads];
  {
    const int kc = min(k0 + kl, K - 8);
    const int nl0 = wave * (2 * kLoads) + (lane >> 5);
    const uint16_t* p = src + static_cast<size_t>(min(n0 + nl0, N - 1)) * ld + kc;
    const size_t step = static_cast<size_t>(ld) * 2;  // two columns further per load
#pragma unroll
    for (int it = 0; it < kLoads; ++it) {
      // the column tile's last columns may lie past N: stay on the last one
      const uint16_t* q = (n0 + nl0 + 2 * it < N) ? p + it * step : src + static_cast<size_t>(N - 1) * ld + kc;
      if constexpr (ALIGNED) {
        raw[it] = load_once_16(q);
      } else {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = static_cast<uint32_t>(q[2 * i]) | (static_cast<uint32_t>(q[2 * i + 1]) << 16);
        raw[it] = make_uint4(w[0], w[1], w[2], w[3]);
      }
    }
  }

#pragma unroll
  for (int it = 0; it < kLoads; ++it) {
    const int nl = wave * (2 * kLoads) + it * 2 + (lane >> 5);
    const uint32_t words[4] = {raw[it].x, raw[it].y, raw[it].z, raw[it].w};
    // Range of the block: this lane's 8 weights, then the lanes that share the block.  The reference
    // scans in ascending k with strict compares, i.e. among equal values the first wins; that only
    // shows when +0 and -0 tie, and only matters for an all-zero block without zero-points, whose
    // scale takes the sign of the block's first weight: handled below from that weight itself.
    float mn, mx;
    if constexpr (BF) {
      float v[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] = bf16_bits_to_float(words[i] & 0xffffu);
        v[2 * i + 1] = bf16_bits_to_float(words[i] >> 16);
      }
      mn = v[0];
      mx = v[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) {
        mn = fminf(mn, v[i]);
        mx = fmaxf(mx, v[i]);
      }
#pragma unroll
      for (int mask = 1; mask < kLanesPerBlock; mask <<= 1) {
        mn = fminf(mn, __shfl_xor(mn, mask));
        mx = fmaxf(mx, __shfl_xor(mx, mask));
      }
    } else {
      // fp16: minimum and maximum of the pairs as they lie in the words (comparisons are exact in any precision),
      // the neighbouring lanes' through DPP, the two halves last
      uint32_t mn2 = pk_min_f16(pk_min_f16(words[0], words[1]), pk_min_f16(words[2], words[3]));
      uint32_t mx2 = pk_max_f16(pk_max_f16(words[0], words[1]), pk_max_f16(words[2], words[3]));
      if constexpr (kLanesPerBlock >= 2) {
        mn2 = pk_min_f16(mn2, exchange_in_group<1>(mn2));
        mx2 = pk_max_f16(mx2, exchange_in_group<1>(mx2));
      }
      if constexpr (kLanesPerBlock >= 4) {
        mn2 = pk_min_f16(mn2, exchange_in_group<2>(mn2));
        mx2 = pk_max_f16(mx2, exchange_in_group<2>(mx2));
      }
      if constexpr (kLanesPerBlock >= 8) {
        mn2 = pk_min_f16(mn2, exchange_in_group<4>(mn2));
        mx2 = pk_max_f16(mx2, exchange_in_group<4>(mx2));
      }
      mn = half_bits_to_float(pk_min_f16_halves(mn2));
      mx = half_bits_to_float(pk_max_f16_halves(mx2));
    }

    BlockQuant b = block_quant<HAS_ZP, BF>(mn, mx);
    if constexpr (!HAS_ZP) {
      // (+-0) / -8 is a zero of the opposite sign (an all-zero block of +0 gives the scale -0.0): the
      // zero case takes its sign from the bits of the block's first weight, which is the value the
      // reference's scan ends with.
      if (mn == 0.0f && mx == 0.0f) {
        const uint32_t first = __shfl(words[0], lane & ~(kLanesPerBlock - 1));  // block's first weight, its bits
        b.scale_bits = ~first & 0x8000u;
      }
    }
    const uint32_t zp = b.zp;
    const uint16_t scale_bits = static_cast<uint16_t>(b.scale_bits);
    const float zp_f = static_cast<float>(zp);
    uint32_t word = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      float v;
      if constexpr (BF) {
        v = bf16_bits_to_float((words[t >> 1] >> (16 * (t & 1))) & 0xffffu);
      } else {
        v = static_cast<float>(__builtin_bit_cast(half2_t, words[t >> 1])[t & 1]);  // folded into the fma
      }
      word |= quantize_one<BF>(v, b.reciprocal_scale, zp_f) << nibble_shift(t);
    }

    w_lds[kl >> 5][nl][(kl >> 3) & 3] = word;
    if ((lane & (kLanesPerBlock - 1)) == 0) {
      s_lds[kl / BS][nl] = scale_bits;
      if constexpr (HAS_ZP) z_lds[kl / BS][nl] = static_cast<uint8_t>(zp);
    }
  }
  __syncthreads();

  // packed weights: one 16-byte unit per thread and pass, 1 KiB contiguous per wave
#pragma unroll
  for (int r = 0; r < (kTileK / 32) * kColTileN / kThreads; ++r) {
    const int u = tid + r * kThreads;
    const int ksl = u / kColTileN;
    const int nl = u % kColTileN;
    const int k = k0 + ksl * 32;
    const int n = n0 + nl;
    if (k < K && n < N) {
      const uint4 val = *reinterpret_cast<const uint4*>(&w_lds[ksl][nl][0]);
      store_once_16(&packed_w[static_cast<size_t>(k >> 5) * N + n], val);
    }
  }
  // scales / zero-points: row-major [K/BS][N]; four columns per thread (8-byte and 4-byte stores) when the
  // buffers are aligned for that (N and the tile's first column are multiples of 32)
  if (wide_meta) {
#pragma unroll
    for (int r = 0; r < (kBlocksPerTile * kColTileN / 4 + kThreads - 1) / kThreads; ++r) {
      const int u = tid + r * kThreads;
      const int bl = u / (kColTileN / 4);
      const int nl = (u % (kColTileN / 4)) * 4;
      const int k = k0 + bl * BS;
      const int n = n0 + nl;
      if (bl < kBlocksPerTile && k < K && n < N) {
        const size_t idx = static_cast<size_t>(k / BS) * N + n;
        *reinterpret_cast<uint2*>(scales + idx) = *reinterpret_cast<const uint2*>(&s_lds[bl][nl]);
        if constexpr (HAS_ZP) *reinterpret_cast<uint32_t*>(zps + idx) = *reinterpret_cast<const uint32_t*>(&z_lds[bl][nl]);
      }
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < (kBlocksPerTile * kColTileN + kThreads - 1) / kThreads; ++r) {
    const int u = tid + r * kThreads;
    const int bl = u / kColTileN;
    const int nl = u % kColTileN;
    const int k = k0 + bl * BS;
    const int n = n0 + nl;
    if (bl < kBlocksPerTile && k < K && n < N) {
      const size_t idx = static_cast<size_t>(k / BS) * N + n;
      scales[idx] = s_lds[bl][nl];
      if constexpr (HAS_ZP) zps[idx] = z_lds[bl][nl];
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Row-wise blocking: a quantization block is one k and BS consecutive columns, so every k of a lane's
// eight has its own scale and zero-point (reference: the [1, bs] block shape of
// src/mickey/blk_q4/f16_quant_sm80.cuh:206-212, 225-315).  Same tile, same packed weight layout and
// the same arithmetic as above; only the reduction runs across columns.  A wave covers 64 k of all
// 64 columns of the tile: lane = (column & 7) * 8 + (k / 8), eight passes of 8 columns, so a block
// is BS/8 passes times 8 lanes.
//
// Scales and zero-points leave in the reference's packed order for this blocking
// (f16_quant_sm80.cuh:506-512, 528-539): column-major [K][N/BS], and inside every group of 16
// rows scale rows (2t, 2t+1, 2t+8, 2t+9) and zero-point rows (2t, 2t+8, 2t+1, 2t+9) sit at
// positions 4t .. 4t+3.
// ------------------------------------------------------------------------------------------------
template <int BS, bool HAS_ZP, bool ALIGNED, bool BF = false>
__global__ __launch_bounds__(kThreads) void prepack_rowwise_kernel(const uint16_t* __restrict__ src, int K,
                                                                   int N, int ld,
                                                                   uint4* __restrict__ packed_w,
                                                                   uint16_t* __restrict__ scales,
                                                                   uint8_t* __restrict__ zps, unsigned k_tiles,
                                                                   bool /*wide_meta*/) {
  constexpr int kPasses = BS / 8;            // passes of 8 columns that make up one block
  constexpr int kGroups = kTileN / BS;       // blocks along N in one tile
  __shared__ uint32_t w_lds[kTileK / 32][kTileN][4];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int c8 = lane >> 3;  // column inside a pass
  const int kq = lane & 7;   // which 8 k of the wave's 64
  const int k0 = static_cast<int>(blockIdx.x % k_tiles) * kTileK;
  const int n0 = static_cast<int>(blockIdx.x / k_tiles) * kTileN;
  const int kl = wave * 64 + kq * 8;  // this lane's first k inside the tile
  const bool k_ok = (k0 + kl) < K;    // K is a multiple of 64: a wave's 64 k are all in or all out

  uint4 raw[8];
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int n = n0 + it * 8 + c8;
    raw[it] = make_uint4(0, 0, 0, 0);
    if (k_ok && n < N) {  // N is a multiple of BS: a block is all in or all out
      const uint16_t* p = src + static_cast<size_t>(n) * ld + (k0 + kl);
      if constexpr (ALIGNED) {
        raw[it] = load_once_16(p);
      } else {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = static_cast<uint32_t>(p[2 * i]) | (static_cast<uint32_t>(p[2 * i + 1]) << 16);
        raw[it] = make_uint4(w[0], w[1], w[2], w[3]);
      }
    }
  }
#define BLKQ4_VALUE(it_, t_) \
  bits_to_float<BF>((((t_) >> 1) == 0 ? raw[it_].x : ((t_) >> 1) == 1 ? raw[it_].y : ((t_) >> 1) == 2 ? raw[it_].z : raw[it_].w) >> (16 * ((t_) & 1)) & 0xffffu)

#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    float rs[8], zf[8];
    uint32_t sbits[8], zq[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      // range of the block of k = k0 + kl + t: the passes of this group, then the 8 column lanes
      float mn = BLKQ4_VALUE(g * kPasses, t), mx = mn;
#pragma unroll
      for (int q = 1; q < kPasses; ++q) {
        const float v = BLKQ4_VALUE(g * kPasses + q, t);
        mn = fminf(mn, v);
        mx = fmaxf(mx, v);
      }
#pragma unroll
      for (int mask = 8; mask < 64; mask <<= 1) {
        mn = fminf(mn, __shfl_xor(mn, mask));
        mx = fmaxf(mx, __shfl_xor(mx, mask));
      }
      BlockQuant b = block_quant<HAS_ZP, BF>(mn, mx);
      if constexpr (!HAS_ZP) {
        if (mn == 0.0f && mx == 0.0f) {
          // all-zero block: the sign comes from the block's first weight (its first column, this k)
          const uint32_t w0 = ((t >> 1) == 0 ? raw[g * kPasses].x : (t >> 1) == 1 ? raw[g * kPasses].y
                               : (t >> 1) == 2 ? raw[g * kPasses].z : raw[g * kPasses].w) >> (16 * (t & 1));
          const uint32_t first = __shfl(w0, kq);
          b.scale_bits = ~first & 0x8000u;
        }
      }
      rs[t] = b.reciprocal_scale;
      zf[t] = static_cast<float>(b.zp);
      sbits[t] = b.scale_bits & 0xffffu;
      zq[t] = b.zp;
    }
#pragma unroll
    for (int q = 0; q < kPasses; ++q) {
      const int it = g * kPasses + q;
      uint32_t word = 0;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        word |= quantize_one<BF>(BLKQ4_VALUE(it, t), rs[t], zf[t]) << nibble_shift(t);
      }
      w_lds[kl >> 5][it * 8 + c8][(kl >> 3) & 3] = word;
    }
    // meta data of the group: one lane per 8 rows writes them
    const int n_first = n0 + g * BS;
    if (c8 == 0 && k_ok && n_first < N) {
      const int row16 = (k0 + kl) & ~15;   // first row of the 16-row group
      const int upper = ((k0 + kl) >> 3) & 1;  // this lane holds rows 8..15 of the group
      const size_t base = static_cast<size_t>(n_first / BS) * K + row16;
#pragma unroll
      for (int tp = 0; tp < 4; ++tp) {
        // rows (2tp, 2tp+1) of this lane's eight
        const uint32_t pair = sbits[2 * tp] | (sbits[2 * tp + 1] << 16);
        *reinterpret_cast<uint32_t*>(scales + base + 4 * tp + 2 * upper) = pair;
        if constexpr (HAS_ZP) {
          zps[base + 4 * tp + upper] = static_cast<uint8_t>(zq[2 * tp]);
          zps[base + 4 * tp + upper + 2] = static_cast<uint8_t>(zq[2 * tp + 1]);
        }
      }
    }
  }
#undef BLKQ4_VALUE
  __syncthreads();

  // packed weights: one 16-byte unit per thread and pass, 1 KiB contiguous per wave
#pragma unroll
  for (int r = 0; r < (kTileK / 32) * kTileN / kThreads; ++r) {
    const int u = tid + r * kThreads;
    const int ksl = u / kTileN;
    const int nl = u % kTileN;
    const int k = k0 + ksl * 32;
    const int n = n0 + nl;
    if (k < K && n < N) {
      const uint4 val = *reinterpret_cast<const uint4*>(&w_lds[ksl][nl][0]);
      store_once_16(&packed_w[static_cast<size_t>(k >> 5) * N + n], val);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Layout conversion between the packed layout above and the reference's sm80 layout
// (reference: src/mickey/blk_q4/f16_quant_sm80.cuh:362-417): uint8[K, N/2] column-major, where for
// each 16x16 weight tile at (k0, n0), row in 0..3, col in 0..7, s in 0..3 the byte at
// (k0 + 4*row + s, n0/2 + col) holds  low = q(k0 + 2*row + (s>>1), n0 + col + 8*(s&1))  and
// high = the same with k + 8.  One thread converts one 16-byte unit (32 k of one n).
// ------------------------------------------------------------------------------------------------

template <bool TO_SM80>
__global__ __launch_bounds__(256) void repack_kernel(const uint8_t* __restrict__ src,
                                                     uint8_t* __restrict__ dst, int K, int N) {
  const size_t unit = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t units = static_cast<size_t>(K / 32) * N;
  if (unit >= units) return;
  const int ks = static_cast<int>(unit / N);
  const int n = static_cast<int>(unit % N);
  const int hi_n = (n & 15) >> 3;
  const size_t pc = static_cast<size_t>((n & ~15) >> 1) + (n & 7);
  const size_t col_base = pc * K + static_cast<size_t>(ks) * 32;

  if constexpr (TO_SM80) {
    const uint4 u = reinterpret_cast<const uint4*>(src)[unit];
    const uint32_t words[4] = {u.x, u.y, u.z, u.w};
    uint32_t q[32];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int t = 0; t < 8; ++t) q[8 * j + t] = (words[j] >> nibble_shift(t)) & 0xfu;
#pragma unroll
    for (int tile = 0; tile < 2; ++tile)
#pragma unroll
      for (int row = 0; row < 4; ++row)
#pragma unroll
        for (int odd = 0; odd < 2; ++odd) {
          const int kk = 16 * tile + 2 * row + odd;
          dst[col_base + 16 * tile + 4 * row + 2 * odd + hi_n] = static_cast<uint8_t>(q[kk] | (q[kk + 8] << 4));
        }
  } else {
    uint32_t q[32];
#pragma unroll
    for (int tile = 0; tile < 2; ++tile)
#pragma unroll
      for (int row = 0; row < 4; ++row)
#pragma unroll
        for (int odd = 0; odd < 2; ++odd) {
          const int kk = 16 * tile + 2 * row + odd;
          const uint32_t b = src[col_base + 16 * tile + 4 * row + 2 * odd + hi_n];
          q[kk] = b & 0xfu;
          q[kk + 8] = b >> 4;
        }
    uint32_t words[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int t = 0; t < 8; ++t) words[j] |= q[8 * j + t] << nibble_shift(t);
    reinterpret_cast<uint4*>(dst)[unit] = make_uint4(words[0], words[1], words[2], words[3]);
  }
}

// ------------------------------------------------------------------------------------------------
// The shortened arithmetic of the fp16 quantizer against its definition, over the whole domain, on the GPU this
// runs on (the hardware's reciprocal estimate is part of what is checked):
//   counts[0]  asymmetric blocks: every pair of finite fp16 values mn <= 0 <= mx (31 745 x 31 744 pairs, which is every range a
//              block can have once it has been widened to include 0): scale bits, zero-point and the bits of the
//              reciprocal of the stored scale from block_quant_fp16 against block_quant_ieee;
//   counts[1]  symmetric blocks: every finite fp16 extreme but zero (an all-zero block's scale is a sign rule of
//              its own in the kernels);
//   counts[2]  the rounding: every float in [0, 15] through v_cvt_rpi_i32_f32 against roundf and against the
//              add-and-truncate form the bf16 quantizer uses;
//   counts[3]  cases looked at (1 007 713 280 + 63 486 + 1 097 859 073).
// counts[0..2] count disagreements: all three must be zero.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ bool same_block_quant(const BlockQuant& a, const BlockQuant& b) {
  return a.scale_bits == b.scale_bits && a.zp == b.zp &&
         __float_as_uint(a.reciprocal_scale) == __float_as_uint(b.reciprocal_scale);
}

__global__ __launch_bounds__(256) void quant_selfcheck_kernel(unsigned long long* __restrict__ counts) {
  constexpr uint32_t kFinite = 0x7c00u;  // fp16 bit patterns 0 .. 0x7bff are the finite non-negative values
  unsigned long long bad_asym = 0, bad_sym = 0, bad_round = 0, looked_at = 0;
  const uint64_t threads = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  const uint64_t me = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  // mn = -(pattern a), with a = kFinite standing for +0 (pattern 0 is -0); mx = pattern x
  for (uint64_t idx = me; idx < static_cast<uint64_t>(kFinite + 1) * kFinite; idx += threads) {
    const uint32_t a = static_cast<uint32_t>(idx / kFinite), x = static_cast<uint32_t>(idx % kFinite);
    const float mn = half_bits_to_float(a == kFinite ? 0u : (0x8000u | a));
    const float mx = half_bits_to_float(x);
    bad_asym += same_block_quant(block_quant_fp16<true>(mn, mx), block_quant_ieee<true, false>(mn, mx)) ? 0 : 1;
    ++looked_at;
  }
  for (uint64_t idx = me; idx < 2 * kFinite; idx += threads) {
    const uint32_t bits = static_cast<uint32_t>(idx % kFinite) | (idx >= kFinite ? 0x8000u : 0u);
    if ((bits & 0x7fffu) == 0) continue;  // the all-zero block's scale is set by the kernels from the block's first weight
    const float m = half_bits_to_float(bits);
    bad_sym += same_block_quant(block_quant_fp16<false>(m, m), block_quant_ieee<false, false>(m, m)) ? 0 : 1;
    ++looked_at;
  }
  for (uint64_t idx = me; idx <= 0x41700000u; idx += threads) {  // 0x41700000 is 15.0f
    const float v = __uint_as_float(static_cast<uint32_t>(idx));
    const uint32_t r = round_0_to_15_rpi(v);
    bad_round += (r == static_cast<uint32_t>(roundf(v)) && r == round_0_to_15(v)) ? 0 : 1;
    ++looked_at;
  }
  if (bad_asym) atomicAdd(&counts[0], bad_asym);
  if (bad_sym) atomicAdd(&counts[1], bad_sym);
  if (bad_round) atomicAdd(&counts[2], bad_round);
  atomicAdd(&counts[3], looked_at);
}

__global__ void quant_selfcheck_clear(unsigned long long* counts) {
  if (threadIdx.x < 4) counts[threadIdx.x] = 0;
}

// All instantiations of a prepack kernel share one signature; `launch` starts the chosen one and returns the
// launch's own status.
template <int BS>
int launch_prepack(const blkq4_prepack_args* a) {
  const int tile_n = a->column_wise ? kColTileN : kTileN;
  const unsigned k_tiles = (a->rows + kTileK - 1) / kTileK;
  const dim3 grid(k_tiles * static_cast<unsigned>((a->columns + tile_n - 1) / tile_n));
  const bool aligned = (reinterpret_cast<uintptr_t>(a->src) & 15u) == 0 && (a->ld % 8) == 0;
  const bool has_zp = a->zero_points != nullptr;
  // scales stored eight bytes, zero-points four bytes at a time (columns is a multiple of 32)
  const bool wide_meta = (reinterpret_cast<uintptr_t>(a->scales) & 7u) == 0 &&
                         (reinterpret_cast<uintptr_t>(a->zero_points) & 3u) == 0 && (a->columns % 4) == 0;
  auto launch = [&](auto* kernel) {
    return static_cast<int>(blkq4::launch_status(kernel, grid, dim3(kThreads), 0, a->stream,
                                          static_cast<const uint16_t*>(a->src), a->rows, a->columns, a->ld,
                                          static_cast<uint4*>(a->packed_w), static_cast<uint16_t*>(a->scales),
                                          static_cast<uint8_t*>(a->zero_points), k_tiles, wide_meta));
  };
  // (has zero-points, aligned source, bf16) -> instantiation
#define BLKQ4_PICK(KERNEL_)                                                                   \
  if (a->bf16) {                                                                              \
    if (has_zp) return aligned ? launch(KERNEL_<BS, true, true, true>) : launch(KERNEL_<BS, true, false, true>);   \
    return aligned ? launch(KERNEL_<BS, false, true, true>) : launch(KERNEL_<BS, false, false, true>);             \
  }                                                                                           \
  if (has_zp) return aligned ? launch(KERNEL_<BS, true, true, false>) : launch(KERNEL_<BS, true, false, false>);   \
  return aligned ? launch(KERNEL_<BS, false, true, false>) : launch(KERNEL_<BS, false, false, false>);
  if (!a->column_wise) {
    BLKQ4_PICK(prepack_rowwise_kernel)
  }
  BLKQ4_PICK(prepack_kernel)
#undef BLKQ4_PICK
}

}  // namespace

extern "C" int blkq4_dev_prepack(const blkq4_prepack_args* a) {
  if ((reinterpret_cast<uintptr_t>(a->packed_w) & 15u) != 0) return static_cast<int>(hipErrorInvalidValue);
  // row-wise blocking: scale pairs are stored as 32-bit words; a block may not straddle the tile edge
  if (!a->column_wise && ((reinterpret_cast<uintptr_t>(a->scales) & 3u) != 0 || (a->columns % a->block_size) != 0)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  switch (a->block_size) {
    case 16: return launch_prepack<16>(a);
    case 32: return launch_prepack<32>(a);
    case 64: return launch_prepack<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}

extern "C" int blkq4_dev_quant_selfcheck(void* counts, void* stream) {
  auto* c = static_cast<unsigned long long*>(counts);
  if (hipError_t e = blkq4::launch_status(quant_selfcheck_clear, dim3(1), dim3(64), 0, stream, c); e != hipSuccess) {
    return static_cast<int>(e);
  }
  return static_cast<int>(blkq4::launch_status(quant_selfcheck_kernel, dim3(256 * 16), dim3(256), 0, stream, c));
}

extern "C" int blkq4_dev_repack(const blkq4_repack_args* a) {
  const size_t units = static_cast<size_t>(a->rows / 32) * a->columns;
  const dim3 grid(static_cast<unsigned>((units + 255) / 256));
  const auto* src = static_cast<const uint8_t*>(a->src);
  auto* dst = static_cast<uint8_t*>(a->dst);
  auto* kernel = a->to_sm80 ? repack_kernel<true> : repack_kernel<false>;
  return static_cast<int>(blkq4::launch_status(kernel, grid, dim3(256), 0, a->stream, src, dst, a->rows, a->columns));
}

extern "C" const char* blkq4_dev_error_string(int code) {
  return hipGetErrorString(static_cast<hipError_t>(code));
}
