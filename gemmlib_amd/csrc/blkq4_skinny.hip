// M = 1..16 path (decode GEMV and small-batch GEMM) for gfx950.
//
// The work is a stream over the packed weights (K*N/2 bytes plus scales and zero-points) that has to
// run at HBM speed.  A workgroup of four waves owns 16 output columns and the whole K range:
//   - the waves split K in 128-deep slices, so every wave load is one 16-byte unit per lane,
//     16 columns x 4 consecutive k-units = four contiguous 256-byte runs of the packed layout;
//   - a lane keeps (column, 32 k) of weights and multiplies them with the matching 32 k of up to 16
//     activation rows through v_mfma_f32_16x16x32_f16 (the weights are the row operand, so a lane ends
//     up with 4 consecutive output columns of one activation row and writes them as one 8-byte store);
//   - the four partial tiles are summed through LDS by wave 0, so no atomics and no scratch buffer.
// Dequantization happens in registers (blkq4_dequant.h); accumulation is fp32.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_dequant.h"
#include "blkq4_device.h"

namespace {

using namespace blkq4;

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kUnroll = 4;  // k-slices whose loads a wave keeps in flight together

template <int BS, bool HAS_ZP>
__global__ __launch_bounds__(kThreads) void skinny_mfma_kernel(const uint16_t* __restrict__ A,
                                                               const uint4* __restrict__ W,
                                                               const uint16_t* __restrict__ S,
                                                               const uint8_t* __restrict__ Z,
                                                               uint16_t* __restrict__ C, int M, int N,
                                                               int K) {
  constexpr int kMeta = (BS == 16) ? 2 : 1;  // quantization blocks inside one 32-deep unit
  __shared__ float red[kWaves][64][4];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int nl = lane & 15;  // column inside the tile (weights operand) / activation row (other operand)
  const int g = lane >> 4;   // which of the 4 k-units of a slice
  const int n = blockIdx.x * 16 + nl;
  const int KS = K >> 5;                // 32-deep units along K
  const int slices = (KS + 3) >> 2;     // 128-deep slices (the last one may be half full)
  const bool row_ok = nl < M;
  const uint16_t* a_row = A + static_cast<size_t>(nl) * K;

  float4_t acc = {0.f, 0.f, 0.f, 0.f};

  for (int s0 = wave; s0 < slices; s0 += kWaves * kUnroll) {
    uint4 wq[kUnroll];
    uint4 av[kUnroll][4];
    uint32_t sc[kUnroll][kMeta];
    uint32_t zp[kUnroll][kMeta];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int ks = 4 * (s0 + u * kWaves) + g;
      const bool ok = ks < KS;  // also false for slices past the end
      wq[u] = make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int q = 0; q < kMeta; ++q) {
        sc[u][q] = 0;  // scale 0 makes an out-of-range unit contribute exactly 0
        zp[u][q] = 8;
      }
      if (ok) {
        wq[u] = W[static_cast<size_t>(ks) * N + n];
        const int b = (BS == 64) ? (ks >> 1) : (BS == 32) ? ks : (2 * ks);
#pragma unroll
        for (int q = 0; q < kMeta; ++q) {
          const size_t mi = static_cast<size_t>(b + q) * N + n;
          sc[u][q] = S[mi];
          if constexpr (HAS_ZP) zp[u][q] = Z[mi];
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) av[u][j] = make_uint4(0, 0, 0, 0);
      if (ok && row_ok) {
        const uint4* p = reinterpret_cast<const uint4*>(a_row + 32 * ks);
#pragma unroll
        for (int j = 0; j < 4; ++j) av[u][j] = p[j];
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      DequantConsts dc[kMeta];
#pragma unroll
      for (int q = 0; q < kMeta; ++q) dc[q] = make_dequant_consts(sc[u][q], zp[u][q]);
      const uint32_t words[4] = {wq[u].x, wq[u].y, wq[u].z, wq[u].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const half8_t wf = dequant_word(words[j], dc[(kMeta == 2) ? (j >> 1) : 0]);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, as_half8(av[u][j]), acc, 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int e = 0; e < 4; ++e) red[wave][lane][e] = acc[e];
  __syncthreads();
  if (wave == 0) {
    float r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = red[0][lane][e] + red[1][lane][e] + red[2][lane][e] + red[3][lane][e];
    if (row_ok) {
      // lane (row nl, group g) holds output columns 4g .. 4g+3 of the 16-column tile
      const uint32_t lo = float_to_half_bits(r[0]) | (static_cast<uint32_t>(float_to_half_bits(r[1])) << 16);
      const uint32_t hi = float_to_half_bits(r[2]) | (static_cast<uint32_t>(float_to_half_bits(r[3])) << 16);
      uint2* out = reinterpret_cast<uint2*>(C + static_cast<size_t>(nl) * N + blockIdx.x * 16 + 4 * g);
      *out = make_uint2(lo, hi);
    }
  }
}

template <int BS>
int launch_skinny(const blkq4_gemm_args* a) {
  const dim3 grid(a->n / 16);
  const dim3 block(kThreads);
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  const auto* A = static_cast<const uint16_t*>(a->a);
  const auto* W = static_cast<const uint4*>(a->packed_w);
  const auto* S = static_cast<const uint16_t*>(a->scales);
  const auto* Z = static_cast<const uint8_t*>(a->zero_points);
  auto* C = static_cast<uint16_t*>(a->c);
  if (Z) {
    hipLaunchKernelGGL((skinny_mfma_kernel<BS, true>), grid, block, 0, stream, A, W, S, Z, C, a->m, a->n, a->k);
  } else {
    hipLaunchKernelGGL((skinny_mfma_kernel<BS, false>), grid, block, 0, stream, A, W, S, Z, C, a->m, a->n, a->k);
  }
  return static_cast<int>(hipGetLastError());
}

}  // namespace

extern "C" int blkq4_dev_skinny(const blkq4_gemm_args* a) {
  if (a->m < 1 || a->m > 16 || (a->n % 16) != 0 || (a->k % 64) != 0) return static_cast<int>(hipErrorInvalidValue);
  switch (a->block_size) {
    case 16: return launch_skinny<16>(a);
    case 32: return launch_skinny<32>(a);
    case 64: return launch_skinny<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}
