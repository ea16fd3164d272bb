// GEMM for weights quantized with blocks along N (one k, BS consecutive columns), every M (gfx950).
//
// The packed weights are the same 16-byte units as for blocks along K; what changes is where a lane
// finds the scale and zero-point of a weight: they vary with k inside a lane's operand and are the
// same for the BS columns of a group.  The meta data keep the reference's packed order (reference:
// src/mickey/blk_q4/f16_quant_sm80.cuh:457-547): column-major [K][N/BS], and inside every group of
// 16 rows
//     scales       position 4t + {0,1,2,3} holds rows 2t + {0,1,8,9}
//     zero-points  position 4t + {0,1,2,3} holds rows 2t + {0,8,1,9}            (t = 0..3)
// That order is made for packed fp16 arithmetic: the 32-bit word 2t + hh of a scale group is the fp16
// pair of rows (8hh + 2t, 8hh + 2t + 1), and byte pair (w >> 8hh) & 0x00ff00ff of zero-point word t is
// the pair of zero-points of the same two rows, already one per 16-bit half.  A lane's MFMA operand for
// one 16-deep k step is 8 consecutive k = four such pairs, so the conversion is the same three packed
// instructions per pair as with blocks along K plus two that build the pair's constants.
//
// Workgroup: four waves side by side along N, tile (32*RT) x 128 x 64; activations are staged through
// LDS (double buffered, XOR swizzled), a lane's packed weights / scales / zero-points for the next k
// tile are fetched straight into registers while the current tile is multiplied (all lanes of a column
// group fetch the same meta words: one request per wave half).  v_mfma_f32_32x32x16_f16, weights as
// the row operand, fp32 accumulation, one rounding to fp16 at the end.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_dequant.h"
#include "blkq4_device.h"

namespace {

using namespace blkq4;

constexpr int kBK = 64;
constexpr int kBN = 128;

template <int BS, bool HAS_ZP, int RT>
__global__ __launch_bounds__(256) void gemm_rowwise_kernel(const uint8_t* __restrict__ A,
                                                            const uint8_t* __restrict__ W,
                                                            const uint8_t* __restrict__ S,
                                                            const uint8_t* __restrict__ Z,
                                                            uint16_t* __restrict__ C, int M, int N, int K) {
  constexpr int kBM = 32 * RT;
  constexpr int kTileBytes = kBM * 128;
  __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kTileBytes];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int i = lane & 31;  // row of an activation fragment / column of a weight fragment
  const int h = lane >> 5;  // which 32-deep half of the 64-deep k tile this lane covers
  const int m0 = blockIdx.x * kBM;
  const int nw0 = blockIdx.y * kBN + wave * 32;
  const bool live = nw0 < N;                 // N is a multiple of 32: a fragment is whole or absent
  const int n = min(nw0, N - 32) + i;        // absent fragments re-read the last one, nothing is stored
  const int KT = K / kBK;

  // activations: RT 16-byte units per thread and k tile
  const uint8_t* a_src[RT];
  uint32_t a_dst[RT];
#pragma unroll
  for (int p = 0; p < RT; ++p) {
    const int id = tid + 256 * p;
    const int row = id >> 3, unit = id & 7;
    a_src[p] = A + static_cast<size_t>(min(m0 + row, M - 1)) * K * 2 + unit * 16;
    a_dst[p] = row * 128 + ((unit ^ ((row >> 1) & 7)) * 16);
  }
  // packed weights: unit (2 kt + h, n); meta: 32 rows of column group n / BS starting at 64 kt + 32 h
  const uint8_t* w_src = W + (static_cast<size_t>(h) * N + n) * 16;
  const size_t w_step = static_cast<size_t>(N) * 32;
  const size_t meta0 = static_cast<size_t>(n / BS) * K + 32 * h;
  const uint8_t* s_src = S + meta0 * 2;
  const uint8_t* z_src = HAS_ZP ? Z + meta0 : nullptr;

  uint4 a_reg[RT];
  uint4 w_cur, w_nxt;
  uint4 s_cur[4], s_nxt[4];
  uint4 z_cur[2], z_nxt[2];

#define BLKQ4_FETCH(kt_)                                                                         \
  {                                                                                              \
    _Pragma("unroll") for (int p = 0; p < RT; ++p)                                               \
        a_reg[p] = *reinterpret_cast<const uint4*>(a_src[p] + static_cast<size_t>(kt_) * 128);   \
    w_nxt = *reinterpret_cast<const uint4*>(w_src + static_cast<size_t>(kt_) * w_step);          \
    _Pragma("unroll") for (int q = 0; q < 4; ++q)                                                \
        s_nxt[q] = *reinterpret_cast<const uint4*>(s_src + static_cast<size_t>(kt_) * 128 + q * 16); \
    if (HAS_ZP) {                                                                                \
      _Pragma("unroll") for (int q = 0; q < 2; ++q)                                              \
          z_nxt[q] = *reinterpret_cast<const uint4*>(z_src + static_cast<size_t>(kt_) * 64 + q * 16); \
    }                                                                                            \
  }
#define BLKQ4_STAGE(buf_)                                                                        \
  {                                                                                              \
    _Pragma("unroll") for (int p = 0; p < RT; ++p)                                               \
        *reinterpret_cast<uint4*>(lds + (buf_) * kTileBytes + a_dst[p]) = a_reg[p];              \
    w_cur = w_nxt;                                                                               \
    _Pragma("unroll") for (int q = 0; q < 4; ++q) s_cur[q] = s_nxt[q];                           \
    if (HAS_ZP) {                                                                                \
      _Pragma("unroll") for (int q = 0; q < 2; ++q) z_cur[q] = z_nxt[q];                         \
    }                                                                                            \
  }

  float16_t acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[r][e] = 0.f;

  BLKQ4_FETCH(0);
  BLKQ4_STAGE(0);
  __syncthreads();

  uint32_t a_rd[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) a_rd[j] = i * 128 + (((4 * h + j) ^ ((i >> 1) & 7)) * 16);

  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) BLKQ4_FETCH(kt + 1);
    const uint8_t* sa = lds + buf * kTileBytes;
    const uint32_t words[4] = {w_cur.x, w_cur.y, w_cur.z, w_cur.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // 16-row meta group j / 2 of the lane's 32 rows, rows 8 hh .. 8 hh + 7 of it
      const int hh = j & 1;
      const uint4 sg0 = s_cur[2 * (j >> 1)], sg1 = s_cur[2 * (j >> 1) + 1];
      const uint32_t sw[8] = {sg0.x, sg0.y, sg0.z, sg0.w, sg1.x, sg1.y, sg1.z, sg1.w};
      const uint4 zg = HAS_ZP ? z_cur[j >> 1] : make_uint4(0, 0, 0, 0);
      const uint32_t zw[4] = {zg.x, zg.y, zg.z, zg.w};
      const uint32_t w = words[j];
      const uint32_t wh = w >> 8;
      half2_t pr[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t zpair = HAS_ZP ? ((zw[t] >> (8 * hh)) & 0x00ff00ffu) : 0x00080008u;
        const half2_t s2 = as_half2(sw[2 * t + hh]);
        const uint32_t src = (t >= 2) ? wh : w;
        if ((t & 1) == 0) {
          pr[t] = (as_half2((src & 0x000f000fu) | 0x64006400u) + as_half2(0xE400E400u | zpair)) * s2;
        } else {
          pr[t] = (as_half2((src & 0x00f000f0u) | 0x54005400u) + as_half2(0xD400D400u | (zpair << 4))) * s2;
        }
      }
      half8_t wf;
      wf[0] = pr[0][0]; wf[1] = pr[0][1]; wf[2] = pr[1][0]; wf[3] = pr[1][1];
      wf[4] = pr[2][0]; wf[5] = pr[2][1]; wf[6] = pr[3][0]; wf[7] = pr[3][1];
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        const half8_t af = as_half8(*reinterpret_cast<const uint4*>(sa + a_rd[j] + r * 4096));
        acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf, af, acc[r], 0, 0, 0);
      }
    }
    if (kt + 1 < KT) BLKQ4_STAGE(buf ^ 1);
    __syncthreads();
  }
#undef BLKQ4_FETCH
#undef BLKQ4_STAGE

  // Accumulator element 4*g + e of lane (i, h) is output row m0 + 32*r + i, column nw0 + 8*g + 4*h + e.
  if (!live) return;
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int m = m0 + 32 * r + i;
    if (m >= M) continue;
    uint16_t* crow = C + static_cast<size_t>(m) * N + nw0 + 4 * h;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint32_t lo = float_to_half_bits(acc[r][4 * g + 0]) |
                          (static_cast<uint32_t>(float_to_half_bits(acc[r][4 * g + 1])) << 16);
      const uint32_t hi = float_to_half_bits(acc[r][4 * g + 2]) |
                          (static_cast<uint32_t>(float_to_half_bits(acc[r][4 * g + 3])) << 16);
      *reinterpret_cast<uint2*>(crow + 8 * g) = make_uint2(lo, hi);
    }
  }
}

template <int BS, bool HAS_ZP, int RT>
int launch_one(const blkq4_gemm_args* a) {
  const dim3 grid((a->m + 32 * RT - 1) / (32 * RT), (a->n + kBN - 1) / kBN);
  hipLaunchKernelGGL((gemm_rowwise_kernel<BS, HAS_ZP, RT>), grid, dim3(256), 0, static_cast<hipStream_t>(a->stream),
                     static_cast<const uint8_t*>(a->a), static_cast<const uint8_t*>(a->packed_w),
                     static_cast<const uint8_t*>(a->scales), static_cast<const uint8_t*>(a->zero_points),
                     static_cast<uint16_t*>(a->c), a->m, a->n, a->k);
  return static_cast<int>(hipGetLastError());
}

template <int BS, bool HAS_ZP>
int launch_rt(const blkq4_gemm_args* a) {
  if (a->m <= 32) return launch_one<BS, HAS_ZP, 1>(a);
  if (a->m <= 64) return launch_one<BS, HAS_ZP, 2>(a);
  return launch_one<BS, HAS_ZP, 4>(a);
}

template <int BS>
int launch_bs(const blkq4_gemm_args* a) {
  return a->zero_points ? launch_rt<BS, true>(a) : launch_rt<BS, false>(a);
}

}  // namespace

extern "C" int blkq4_dev_gemm_rowwise(const blkq4_gemm_args* a) {
  if (a->m < 1 || (a->n % 32) != 0 || a->n < 32 || (a->k % 64) != 0 || (a->n % a->block_size) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  // 16-byte loads of 32 consecutive meta rows: K is a multiple of 64, so the base alignment decides
  if ((reinterpret_cast<uintptr_t>(a->scales) & 15u) != 0 || (reinterpret_cast<uintptr_t>(a->zero_points) & 15u) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if ((a->n + kBN - 1) / kBN > 65535) return static_cast<int>(hipErrorInvalidValue);
  switch (a->block_size) {
    case 16: return launch_bs<16>(a);
    case 32: return launch_bs<32>(a);
    case 64: return launch_bs<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}
