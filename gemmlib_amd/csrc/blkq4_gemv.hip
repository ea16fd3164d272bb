// GEMV without matrix instructions, for 1 to 4 activation rows and blocks along K: the form the reference's
// small-M path has in spirit (src/mickey/blk_q4/f16_gemm_sm80.h:63-72 gives M <= 16 a kernel of its own) and the
// alternative to the MFMA form in blkq4_skinny.hip, against which it is measured.
//
//   - a workgroup of kWaves waves owns 16 output columns and all of K; the waves split K in 128-deep slices and
//     a lane (column nl, k-unit g of the slice) loads one 16-byte unit per slice: four contiguous 256-byte runs
//     per wave, the same requests as the MFMA form;
//   - every lane keeps a fp32 partial sum per activation row: it dequantizes its 32 weights in registers
//     (blkq4_dequant.h, one rounding per weight) and multiplies them pairwise with the matching activations by
//     v_dot2_f32_f16;
//   - the activation rows are staged in LDS once per workgroup, after the first weight requests have been
//     issued; the 16 lanes of a k-unit read the same addresses (a broadcast);
//   - sums across K: inside the wave over the four k-units by two lane exchanges (lanes nl, nl + 16, nl + 32,
//     nl + 48), across the waves through 64 bytes of LDS per wave and row and one barrier; a fixed order, so
//     every call gives the same bits.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_choose.h"
#include "blkq4_dequant.h"
#include "blkq4_device.h"
#include "blkq4_launch.h"

namespace {

using namespace blkq4;

constexpr int kDepth = 2;  // slices a wave keeps in flight

template <int BS>
struct DotSlot {
  static constexpr int kMeta = (BS == 16) ? 2 : 1;  // quantization blocks inside one 32-deep unit
  uint4 w;
  uint32_t sc[kMeta];
  uint32_t zp[kMeta];
};

// R: activation rows kept (1, 2 or 4; M <= R)
template <int BS, bool HAS_ZP, int R, int kWaves>
__global__ __launch_bounds__(64 * kWaves) void gemv_dot_kernel(const uint16_t* __restrict__ A,
                                                              const uint4* __restrict__ W,
                                                              const uint16_t* __restrict__ S,
                                                              const uint8_t* __restrict__ Z,
                                                              uint16_t* __restrict__ C,
                                                              const uint16_t* __restrict__ bias, int M, int N, int K) {
  constexpr int kMeta = DotSlot<BS>::kMeta;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // [R][K] fp16, then [kWaves][R][16] floats
  float* red = reinterpret_cast<float*>(smem + static_cast<size_t>(R) * K * 2);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int nl = lane & 15;
  const int g = lane >> 4;
  const int col = blockIdx.x * 16 + nl;
  const int units = K >> 5;
  const int slices = (units + 3) >> 2;
  const int my_slices = (slices - wave + kWaves - 1) / kWaves;  // slices wave, wave + kWaves, ...
  const DequantMasks masks = DequantMasks::make();

  // a unit past the end of K asks for unit 0 instead; its scale is zeroed when it is consumed, so it adds 0
  auto load = [&](DotSlot<BS>& s, int slice) {
    const int unit = 4 * slice + g;
    const int u = unit < units ? unit : 0;
    // (read once per launch: non-temporal)
    const uint4_t v = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(
        reinterpret_cast<const char*>(W) + (static_cast<size_t>(u) * N + col) * 16));
    s.w = make_uint4(v[0], v[1], v[2], v[3]);
#pragma unroll
    for (int q = 0; q < kMeta; ++q) {
      const size_t blk = (BS == 64) ? (u >> 1) : (BS == 32) ? u : 2 * u + q;
      s.sc[q] = S[blk * N + col];
      s.zp[q] = HAS_ZP ? Z[blk * N + col] : 8u;
    }
  };

  DotSlot<BS> slot[kDepth];
#pragma unroll
  for (int d = 0; d < kDepth; ++d) load(slot[d], wave + kWaves * d);  // (past the wave's last slice: unit 0, unused)

  // the rows, as they lie in memory (rows past M: zeros)
  for (int c = tid; c < R * (K >> 3); c += 64 * kWaves) {
    const int row = c / (K >> 3);
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row < M) v = *reinterpret_cast<const uint4*>(A + static_cast<size_t>(c) * 8);
    *reinterpret_cast<uint4*>(smem + static_cast<size_t>(c) * 16) = v;
  }
  __syncthreads();

  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;

  auto consume = [&](const DotSlot<BS>& s, int slice) {
    const int unit = 4 * slice + g;
    const bool valid = slice < slices && unit < units;
    const uint32_t keep = valid ? 0xffffffffu : 0u;
    const int u = valid ? unit : 0;
    DequantConsts dc[kMeta];
#pragma unroll
    for (int q = 0; q < kMeta; ++q) dc[q] = make_dequant_consts(s.sc[q] & keep, s.zp[q]);
    const uint32_t words[4] = {s.w.x, s.w.y, s.w.z, s.w.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const DequantConsts& c = dc[(kMeta == 2) ? (j >> 1) : 0];
      const uint32_t y = words[j] >> 8;
      half2_t p[4];
      p[0] = dequant_pair(words[j], 0, c, masks);
      p[1] = dequant_pair(words[j], 1, c, masks);
      p[2] = dequant_pair(y, 2, c, masks);
      p[3] = dequant_pair(y, 3, c, masks);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint4 a8 = *reinterpret_cast<const uint4*>(smem + (static_cast<size_t>(r) * K + u * 32 + j * 8) * 2);
        acc[r] = __builtin_amdgcn_fdot2(p[0], as_half2(a8.x), acc[r], false);
        acc[r] = __builtin_amdgcn_fdot2(p[1], as_half2(a8.y), acc[r], false);
        acc[r] = __builtin_amdgcn_fdot2(p[2], as_half2(a8.z), acc[r], false);
        acc[r] = __builtin_amdgcn_fdot2(p[3], as_half2(a8.w), acc[r], false);
      }
    }
  };

  for (int i0 = 0; i0 < my_slices; i0 += kDepth) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      consume(slot[d], wave + kWaves * (i0 + d));
      if (i0 + kDepth < my_slices) load(slot[d], wave + kWaves * (i0 + d + kDepth));
    }
  }

  // over the four k-units of the wave: lanes nl, nl + 16, nl + 32, nl + 48
#pragma unroll
  for (int r = 0; r < R; ++r) {
    acc[r] += __shfl_xor(acc[r], 16);
    acc[r] += __shfl_xor(acc[r], 32);
  }
  if (g == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) red[(wave * R + r) * 16 + nl] = acc[r];
  }
  __syncthreads();
  if (tid < 16 * R) {
    const int r = tid >> 4, c = tid & 15;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) sum += red[(w * R + r) * 16 + c];
    if (r < M) {
      uint32_t h = float_to_half_bits(sum);
      if (bias != nullptr) h = add_bias_bits(h, bias[blockIdx.x * 16 + c]);
      C[static_cast<size_t>(r) * N + blockIdx.x * 16 + c] = static_cast<uint16_t>(h);
    }
  }
}

template <auto kKernel>
hipError_t raise_lds_limit() {
  return raise_lds_limit_once(reinterpret_cast<const void*>(kKernel), kMaxLdsBytes, &lds_limit_flags<kKernel>());
}

template <int BS, bool HAS_ZP, int R, int kWaves>
int launch_dot(const blkq4_gemm_args* a) {
  const size_t lds = static_cast<size_t>(R) * a->k * 2 + static_cast<size_t>(kWaves) * R * 16 * 4;
  if (a->launched_id != nullptr) *a->launched_id = valu_gemv_id(R, kWaves);
  if (a->dry_run) return 0;
  if (lds > kMaxLdsBytes) return static_cast<int>(hipErrorInvalidValue);
  constexpr auto kernel = gemv_dot_kernel<BS, HAS_ZP, R, kWaves>;
  if (hipError_t e = raise_lds_limit<kernel>(); e != hipSuccess) return static_cast<int>(e);
  return static_cast<int>(launch_status(kernel, dim3(a->n / 16), dim3(64 * kWaves), lds, a->stream,
                                        static_cast<const uint16_t*>(a->a), static_cast<const uint4*>(a->packed_w),
                                        static_cast<const uint16_t*>(a->scales),
                                        static_cast<const uint8_t*>(a->zero_points), static_cast<uint16_t*>(a->c),
                                        static_cast<const uint16_t*>(a->bias), a->m, a->n, a->k));
}

template <int BS, bool HAS_ZP, int R>
int launch_waves(const blkq4_gemm_args* a) {
  switch (valu_gemv_waves(a->k)) {
    case 16: return launch_dot<BS, HAS_ZP, R, 16>(a);
    case 8: return launch_dot<BS, HAS_ZP, R, 8>(a);
    default: return launch_dot<BS, HAS_ZP, R, 4>(a);
  }
}

template <int BS, bool HAS_ZP>
int launch_rows(const blkq4_gemm_args* a) {
  switch (valu_gemv_rows(a->m)) {
    case 1: return launch_waves<BS, HAS_ZP, 1>(a);
    case 2: return launch_waves<BS, HAS_ZP, 2>(a);
    default: return launch_waves<BS, HAS_ZP, 4>(a);
  }
}

template <int BS>
int launch_bs(const blkq4_gemm_args* a) {
  return a->zero_points ? launch_rows<BS, true>(a) : launch_rows<BS, false>(a);
}

}  // namespace

// fp16, blocks along K, 1 <= m <= 4, the rows' m * k * 2 bytes (m rounded up to 1, 2 or 4) within 150 KiB of LDS
extern "C" int blkq4_dev_gemv_dot(const blkq4_gemm_args* a) {
  if (a->m < 1 || a->m > 4 || !a->column_wise || (a->n % 16) != 0 || (a->k % 64) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  switch (a->block_size) {
    case 16: return launch_bs<16>(a);
    case 32: return launch_bs<32>(a);
    case 64: return launch_bs<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}
