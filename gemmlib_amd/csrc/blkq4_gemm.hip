// M > 16 path: fp16 MFMA GEMM with the 4-bit weights dequantized in registers (gfx950).
//
// Workgroup tile (32*RT) x 256 x 64 (M x N x K), four waves side by side along N, so a wave owns
// (32*RT) x 64 outputs and every packed weight is converted to fp16 by exactly one wave.
//   - activations: 16-byte global loads, staged through LDS (double buffered, XOR-swizzled 16-byte
//     columns so the MFMA-fragment reads of 32 different rows do not collide on banks);
//   - packed weights: a lane's MFMA operand for one 64-deep k tile is one 16-byte unit of the packed
//     layout (32 consecutive k of one column), loaded straight into registers: 32 lanes read 512
//     contiguous bytes.  The columns of a wave are private to it, so LDS staging would add a round
//     trip without any reuse;
//   - v_mfma_f32_32x32x16_f16 with the weights as the row operand: the accumulator of a lane then
//     holds 4 consecutive output columns of one activation row, written as 8-byte stores;
//   - the next k tile (activations into registers, weights/scales/zero-points into registers) is
//     requested before the current one is consumed.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_dequant.h"
#include "blkq4_device.h"

namespace {

using namespace blkq4;

constexpr int kThreads = 256;
constexpr int kBN = 256;
constexpr int kBK = 64;

template <int BS>
struct MetaRegs {
  static constexpr int kCount = (BS == 16) ? 2 : 1;  // quantization blocks inside a lane's 32-deep unit
  uint32_t scale[2][kCount];
  uint32_t zp[2][kCount];
};

template <int BS, bool HAS_ZP, int RT>
__global__ __launch_bounds__(kThreads) void gemm_mfma_kernel(const uint4* __restrict__ A,
                                                             const uint4* __restrict__ W,
                                                             const uint16_t* __restrict__ S,
                                                             const uint8_t* __restrict__ Z,
                                                             uint16_t* __restrict__ C, int M, int N, int K,
                                                             int m_tiles) {
  constexpr int BM = 32 * RT;
  constexpr int kMeta = MetaRegs<BS>::kCount;
  __shared__ uint4 a_lds[2][BM][8];  // [buffer][row][16-byte column ^ (row & 7)]

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int i = lane & 31;  // row of an activation fragment / column of a weight fragment
  const int h = lane >> 5;  // which 32-deep half of the 64-deep k tile this lane covers

  const int bm = blockIdx.x % m_tiles;
  const int bn = blockIdx.x / m_tiles;
  const int m0 = bm * BM;
  const int nw0 = bn * kBN + wave * 64;
  const bool tile_ok[2] = {nw0 < N, nw0 + 32 < N};  // N is a multiple of 32: 32-column tiles are whole

  const int ac = tid & 7;   // 16-byte column of the activation tile this thread copies
  const int ar = tid >> 3;  // its row (plus 32 per pass)
  const int KT = K / kBK;
  const size_t a_row_units = static_cast<size_t>(K) / 8;  // 16-byte units per activation row

  float16_t acc[RT][2];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[r][t][e] = 0.f;

  uint4 a_stage[RT];
  uint4 b_cur[2], b_nxt[2];
  MetaRegs<BS> m_cur, m_nxt;

  auto load_a = [&](int kt) {
#pragma unroll
    for (int it = 0; it < RT; ++it) {
      const int row = m0 + ar + 32 * it;
      a_stage[it] = make_uint4(0, 0, 0, 0);
      if (row < M) a_stage[it] = A[static_cast<size_t>(row) * a_row_units + kt * 8 + ac];
    }
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int it = 0; it < RT; ++it) a_lds[buf][ar + 32 * it][ac ^ (ar & 7)] = a_stage[it];
  };
  auto load_b = [&](int kt, uint4 (&b)[2], MetaRegs<BS>& mr) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      b[t] = make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int q = 0; q < kMeta; ++q) {
        mr.scale[t][q] = 0;
        mr.zp[t][q] = 8;
      }
      if (tile_ok[t]) {
        const int n = nw0 + 32 * t + i;
        const int ks = 2 * kt + h;
        b[t] = W[static_cast<size_t>(ks) * N + n];
        const int blk = (BS == 64) ? kt : (BS == 32) ? ks : (2 * ks);
#pragma unroll
        for (int q = 0; q < kMeta; ++q) {
          const size_t mi = static_cast<size_t>(blk + q) * N + n;
          mr.scale[t][q] = S[mi];
          if constexpr (HAS_ZP) mr.zp[t][q] = Z[mi];
        }
      }
    }
  };

  load_a(0);
  load_b(0, b_cur, m_cur);
  store_a(0);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    const bool more = (kt + 1) < KT;
    if (more) {
      load_a(kt + 1);
      load_b(kt + 1, b_nxt, m_nxt);
    }

    DequantConsts dc[2][kMeta];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int q = 0; q < kMeta; ++q) dc[t][q] = make_dequant_consts(m_cur.scale[t][q], m_cur.zp[t][q]);
    const uint32_t words[2][4] = {{b_cur[0].x, b_cur[0].y, b_cur[0].z, b_cur[0].w},
                                  {b_cur[1].x, b_cur[1].y, b_cur[1].z, b_cur[1].w}};

#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // k step j covers, for lane half h, k = 32*h + 8*j .. +7 of the tile: word j of the lane's unit
      half8_t af[RT];
#pragma unroll
      for (int r = 0; r < RT; ++r) af[r] = as_half8(a_lds[buf][32 * r + i][(4 * h + j) ^ (i & 7)]);
      half8_t wf[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) wf[t] = dequant_word(words[t][j], dc[t][(kMeta == 2) ? (j >> 1) : 0]);
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < 2; ++t)
          acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[t], af[r], acc[r][t], 0, 0, 0);
    }

    if (more) {
      store_a(buf ^ 1);
      b_cur[0] = b_nxt[0];
      b_cur[1] = b_nxt[1];
      m_cur = m_nxt;
    }
    __syncthreads();
  }

  // Epilogue.  Accumulator element 4*g + e of lane (i, h) is output row m0 + 32*r + i and column
  // nw0 + 32*t + 8*g + 4*h + e: four consecutive columns -> one 8-byte store.
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int m = m0 + 32 * r + i;
    if (m >= M) continue;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (!tile_ok[t]) continue;
      uint16_t* crow = C + static_cast<size_t>(m) * N + nw0 + 32 * t + 4 * h;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const uint32_t lo = float_to_half_bits(acc[r][t][4 * g + 0]) |
                            (static_cast<uint32_t>(float_to_half_bits(acc[r][t][4 * g + 1])) << 16);
        const uint32_t hi = float_to_half_bits(acc[r][t][4 * g + 2]) |
                            (static_cast<uint32_t>(float_to_half_bits(acc[r][t][4 * g + 3])) << 16);
        *reinterpret_cast<uint2*>(crow + 8 * g) = make_uint2(lo, hi);
      }
    }
  }
}

template <int BS, bool HAS_ZP, int RT>
int launch_one(const blkq4_gemm_args* a) {
  constexpr int BM = 32 * RT;
  const int m_tiles = (a->m + BM - 1) / BM;
  const int n_tiles = (a->n + kBN - 1) / kBN;
  const dim3 grid(static_cast<unsigned>(m_tiles) * n_tiles);
  hipLaunchKernelGGL((gemm_mfma_kernel<BS, HAS_ZP, RT>), grid, dim3(kThreads), 0,
                     static_cast<hipStream_t>(a->stream), static_cast<const uint4*>(a->a),
                     static_cast<const uint4*>(a->packed_w), static_cast<const uint16_t*>(a->scales),
                     static_cast<const uint8_t*>(a->zero_points), static_cast<uint16_t*>(a->c), a->m, a->n,
                     a->k, m_tiles);
  return static_cast<int>(hipGetLastError());
}

template <int BS, bool HAS_ZP>
int launch_rt(const blkq4_gemm_args* a) {
  // rows per workgroup: 128 unless the whole problem is shorter
  if (a->m <= 32) return launch_one<BS, HAS_ZP, 1>(a);
  if (a->m <= 64) return launch_one<BS, HAS_ZP, 2>(a);
  return launch_one<BS, HAS_ZP, 4>(a);
}

template <int BS>
int launch_bs(const blkq4_gemm_args* a) {
  return a->zero_points ? launch_rt<BS, true>(a) : launch_rt<BS, false>(a);
}

}  // namespace

extern "C" int blkq4_dev_gemm(const blkq4_gemm_args* a) {
  if (a->m < 1 || (a->n % 32) != 0 || (a->k % 64) != 0) return static_cast<int>(hipErrorInvalidValue);
  switch (a->block_size) {
    case 16: return launch_bs<16>(a);
    case 32: return launch_bs<32>(a);
    case 64: return launch_bs<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}
