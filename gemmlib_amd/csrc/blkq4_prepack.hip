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

constexpr int kTileN = 64;    // columns (n) per workgroup
constexpr int kTileK = 256;   // rows (k) per workgroup
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

template <int BS, bool HAS_ZP, bool ALIGNED, bool BF = false>
__global__ __launch_bounds__(kThreads) void prepack_kernel(const uint16_t* __restrict__ src, int K,
                                                           int N, int ld,
                                                           uint4* __restrict__ packed_w,
                                                           uint16_t* __restrict__ scales,
                                                           uint8_t* __restrict__ zps, unsigned k_tiles) {
  constexpr int kLanesPerBlock = BS / 8;     // lanes sharing one quantization block
  constexpr int kBlocksPerTile = kTileK / BS;  // quantization blocks along K in one tile
  __shared__ uint32_t w_lds[kTileK / 32][kTileN][4];
  __shared__ uint16_t s_lds[kBlocksPerTile][kTileN];
  __shared__ uint8_t z_lds[kBlocksPerTile][kTileN];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  // consecutive workgroups walk along k: they read consecutive 512-byte pieces of the same 64 rows
  const int k0 = static_cast<int>(blockIdx.x % k_tiles) * kTileK;
  const int n0 = static_cast<int>(blockIdx.x / k_tiles) * kTileN;

  const int kl = (lane & 31) * 8;  // this lane's first k inside the tile
  const bool k_ok = (k0 + kl) < K;  // K is a multiple of 64, so a lane's 8 weights are all in or all out

  // Issue every load of the wave first: 8 x 16 bytes per lane in flight.
  uint4 raw[8];
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int nl = wave * 16 + it * 2 + (lane >> 5);
    const int n = n0 + nl;
    raw[it] = make_uint4(0, 0, 0, 0);
    if (k_ok && n < N) {
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

#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int nl = wave * 16 + it * 2 + (lane >> 5);
    const uint32_t words[4] = {raw[it].x, raw[it].y, raw[it].z, raw[it].w};
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = bits_to_float<BF>(words[i] & 0xffffu);
      v[2 * i + 1] = bits_to_float<BF>(words[i] >> 16);
    }
    // Range of the block: this lane's 8 weights, then the lanes that share the block.  The reference
    // scans in ascending k with strict compares, i.e. among equal values the first wins; that only
    // shows when +0 and -0 tie, and only matters for an all-zero block without zero-points, whose
    // scale takes the sign of the block's first weight: handled below from that weight itself.
    float mn = v[0], mx = v[0];
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

    uint16_t scale_bits;
    uint32_t zp;
    if constexpr (HAS_ZP) {
      // reference: range2scalezp, f16_quant_sm80.cuh:96-122
      const float rmn = fminf(mn, 0.0f);
      const float rmx = fmaxf(mx, 0.0f);
      const float scale_f = BF ? __fdiv_rn(__fsub_rn(rmx, rmn), 15.0f) : div_by_15(__fsub_rn(rmx, rmn));
      float zero_point_fp = rmn;
      if (scale_f != 0.0f) zero_point_fp = __fsub_rn(0.0f, __fdiv_rn(rmn, scale_f));
      if (zero_point_fp < 0.0f) {
        zp = 0;
      } else if (zero_point_fp > 15.0f) {
        zp = 15;
      } else {
        zp = round_0_to_15(zero_point_fp);
      }
      scale_bits = float_to_bits<BF>(scale_f);
    } else {
      // reference: range2scale, f16_quant_sm80.cuh:124-135
      const float m = fabsf(mx) > fabsf(mn) ? mx : mn;
      scale_bits = float_to_bits<BF>(__fdiv_rn(m, -8.0f));
      // (+-0) / -8 is a zero of the opposite sign (an all-zero block of +0 gives the scale -0.0): the
      // zero case takes its sign from the bits of the block's first weight, which is the value the
      // reference's scan ends with.
      if (m == 0.0f) {
        const uint32_t first = __shfl(words[0], lane & ~(kLanesPerBlock - 1));  // block's first weight, fp16 bits
        scale_bits = static_cast<uint16_t>(~first & 0x8000u);
      }
      zp = 8;
    }

    // reference: f16_quant_sm80.cuh:291-297 (scale re-read after fp16 rounding; -0.0 counts as zero)
    const float scale = bits_to_float<BF>(scale_bits);
    const float reciprocal_scale = (scale != 0.0f) ? __fdiv_rn(1.0f, scale) : 0.0f;
    const float zp_f = static_cast<float>(zp);
    uint32_t word = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      // clamping before rounding gives the same nibble as the reference's round-then-clamp (both
      // are monotonic)
      const float r = __builtin_amdgcn_fmed3f(__fmaf_rn(v[t], reciprocal_scale, zp_f), 0.0f, 15.0f);
      word |= round_0_to_15(r) << nibble_shift(t);
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
  // scales / zero-points: row-major [K/BS][N]
#pragma unroll
  for (int r = 0; r < (kBlocksPerTile * kTileN + kThreads - 1) / kThreads; ++r) {
    const int u = tid + r * kThreads;
    const int bl = u / kTileN;
    const int nl = u % kTileN;
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
                                                                   uint8_t* __restrict__ zps, unsigned k_tiles) {
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
      uint16_t scale_bits;
      uint32_t zp;
      if constexpr (HAS_ZP) {
        const float rmn = fminf(mn, 0.0f);
        const float rmx = fmaxf(mx, 0.0f);
        const float scale_f = BF ? __fdiv_rn(__fsub_rn(rmx, rmn), 15.0f) : div_by_15(__fsub_rn(rmx, rmn));
        float zero_point_fp = rmn;
        if (scale_f != 0.0f) zero_point_fp = __fsub_rn(0.0f, __fdiv_rn(rmn, scale_f));
        if (zero_point_fp < 0.0f) {
          zp = 0;
        } else if (zero_point_fp > 15.0f) {
          zp = 15;
        } else {
          zp = round_0_to_15(zero_point_fp);
        }
        scale_bits = float_to_bits<BF>(scale_f);
      } else {
        const float m = fabsf(mx) > fabsf(mn) ? mx : mn;
        scale_bits = float_to_bits<BF>(__fdiv_rn(m, -8.0f));
        if (m == 0.0f) {
          // all-zero block: the sign comes from the block's first weight (its first column, this k)
          const uint32_t w0 = ((t >> 1) == 0 ? raw[g * kPasses].x : (t >> 1) == 1 ? raw[g * kPasses].y
                               : (t >> 1) == 2 ? raw[g * kPasses].z : raw[g * kPasses].w) >> (16 * (t & 1));
          const uint32_t first = __shfl(w0, kq);
          scale_bits = static_cast<uint16_t>(~first & 0x8000u);
        }
        zp = 8;
      }
      const float scale = bits_to_float<BF>(scale_bits);
      rs[t] = (scale != 0.0f) ? __fdiv_rn(1.0f, scale) : 0.0f;
      zf[t] = static_cast<float>(zp);
      sbits[t] = scale_bits;
      zq[t] = zp;
    }
#pragma unroll
    for (int q = 0; q < kPasses; ++q) {
      const int it = g * kPasses + q;
      uint32_t word = 0;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const float r = __builtin_amdgcn_fmed3f(__fmaf_rn(BLKQ4_VALUE(it, t), rs[t], zf[t]), 0.0f, 15.0f);
        word |= round_0_to_15(r) << nibble_shift(t);
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

// All instantiations of a prepack kernel share one signature; `launch` starts the chosen one and returns the
// launch's own status.
template <int BS>
int launch_prepack(const blkq4_prepack_args* a) {
  const unsigned k_tiles = (a->rows + kTileK - 1) / kTileK;
  const dim3 grid(k_tiles * static_cast<unsigned>((a->columns + kTileN - 1) / kTileN));
  const bool aligned = (reinterpret_cast<uintptr_t>(a->src) & 15u) == 0 && (a->ld % 8) == 0;
  const bool has_zp = a->zero_points != nullptr;
  auto launch = [&](auto* kernel) {
    return static_cast<int>(blkq4::launch_status(kernel, grid, dim3(kThreads), 0, a->stream,
                                          static_cast<const uint16_t*>(a->src), a->rows, a->columns, a->ld,
                                          static_cast<uint4*>(a->packed_w), static_cast<uint16_t*>(a->scales),
                                          static_cast<uint8_t*>(a->zero_points), k_tiles));
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
