// Decode kernel for gfx950: GEMV and GEMM with up to 16 activation rows and blocks along K (up to four rows with
// blocks along N), when a workgroup can request all of K at once.  The same arithmetic as the weight-streaming
// kernel (blkq4_skinny.hip), with as few instructions around it as the job allows.
//
// A compute unit issues one instruction per wave every four cycles, and the waves of a SIMD share one issue slot
// per instruction type, so at these sizes (a few microseconds, tens of kilobytes of weights per compute unit)
// the launch is bound by the instructions that stand between a wave's start and its first request, and between
// the arrival of its last weights and the end -- not by the weight stream.  Measured with timestamps inside the
// streaming kernel on M = 1, K = N = 4096: 1300 to 4000 cycles from a wave's start to its requests (250
// instructions of address arithmetic for cases this shape does not have, times four waves per SIMD), 1100 cycles
// waiting for the data, 1600 converting, 1800 at the barrier behind the slowest wave.  Hence:
//   - one pass: a wave owns D consecutive 128-deep slices of K (D or D - 1 when the slices do not divide evenly)
//     and requests all of them right away; nothing is refilled, so there is no ring, no loop and no address that
//     depends on a loop counter;
//   - every offset is 32 bits wide, relative to the kernel's own pointer arguments, and the lane's part of it is
//     computed once: a request is one instruction plus one addition;
//   - the arguments arrive in registers with the wave (kernel-argument preloading; the file is compiled with
//     -mllvm -amdgpu-kernarg-preload-count), all of them: a fetch of the bias pointer at the end cost 0.2 us;
//   - a slot's scales and zero-points are requested before its weights: requests complete in order, so whoever
//     has the weights has them too, and slot d is converted while slot d + 1 is still on its way;
//   - the activation rows of a wave's own slices are copied to LDS by the wave itself before its first weights
//     (asynchronous global_load_lds copies, laid out [pair of 32-deep units][row][128 bytes], 16-byte chunks
//     XOR-swizzled with bits 1..3 of the row: fragment reads without bank conflicts); its reads wait for the
//     first weights and need no barrier;
//   - one barrier: the waves' partial tiles meet in LDS and are summed in the order of the waves;
//   - neighbouring column tiles run on the same XCD at about the same time and share the cache lines of their
//     scales and zero-points (16 columns use 32 and 16 bytes of a row);
//   - blocks along N: a lane's 32 weights have a scale and a zero-point each, the same for the 16 columns of the
//     tile; a wave's slices have them in one contiguous run, which two or three copy instructions bring to LDS
//     (the streaming kernel fetches them with six loads per slot and lane).
// Dequantization is the streaming kernel's (blkq4_dequant.h: one rounding per weight), accumulation fp32 in
// v_mfma_f32_16x16x32_{f16,bf16} with the weights as the row operand.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_choose.h"
#include "blkq4_dequant.h"
#include "blkq4_device.h"
#include "blkq4_launch.h"
#include "blkq4_gemm_common.h"

// This file is compiled twice: as it is for fp16, and through blkq4_decode_bf16.hip, which defines
// BLKQ4_DECODE_BF16 before including it, for bf16 activations, scales and outputs.
#ifdef BLKQ4_DECODE_BF16
#define BLKQ4_DECODE_ENTRY blkq4_dev_decode_bf16
#else
#define BLKQ4_DECODE_ENTRY blkq4_dev_decode
#endif

namespace {

using namespace blkq4;

#ifdef BLKQ4_DECODE_BF16
constexpr bool kBF = true;
#else
constexpr bool kBF = false;
#endif

// Zero, available only once `loaded` -- the destination of a load -- has arrived: the compiler waits for the load
// before an asm statement that reads its destination, and what is computed from the result comes after that.
__device__ __forceinline__ uint32_t zero_once_loaded(uint32_t loaded) {
  uint32_t zero;
  asm volatile("v_and_b32 %0, 0, %1" : "=v"(zero) : "v"(loaded));
  return zero;
}

constexpr int log2_of(int v) { return v <= 1 ? 0 : 1 + log2_of(v / 2); }

// R: activation rows kept (a power of two, M <= R <= 16).  NT: 16-column tiles per workgroup that share the
// activation fragments.  kWaves waves split K; D: slices a wave requests (the last one may be missing).
// (BF repeats kBF so that the two compilations' kernels carry different names in a trace)
// ROW: quantization blocks run along N (one k, BS columns); S and Z are then in the packed order described in
// blkq4_device.h: a scale and a zero-point per k, the same for the 16 columns of a tile (NT = 1).
template <int BS, bool HAS_ZP, int R, int NT, int kWaves, int D, bool ROW = false, bool BF = kBF>
__global__ __launch_bounds__(64 * kWaves) void decode_mfma_kernel(const uint8_t* __restrict__ A,
                                                                const uint8_t* __restrict__ W,
                                                                const uint8_t* __restrict__ S,
                                                                const uint8_t* __restrict__ Z,
                                                                uint16_t* __restrict__ C,
                                                                const uint16_t* __restrict__ bias, uint32_t n_and_m,
                                                                int K) {
  constexpr int kMeta = (BS == 16) ? 2 : 1;      // quantization blocks inside one 32-deep unit
  constexpr int kLgR = log2_of(R);
  constexpr int kLgWaves = log2_of(kWaves);
  constexpr int kSliceBytes = 256 * R;           // a slice's rows in LDS: two pairs of units
  constexpr int kWaveBytes = D * kSliceBytes;    // a wave's rows
  constexpr int kCopies = (kWaveBytes + 1023) / 1024;
  // blocks along N: the scales (256 bytes) and zero-points (128 bytes) of a wave's slices, one after the other
  constexpr int kRowScaleBytes = ROW ? D * 256 : 0;
  constexpr int kRowMetaBytes = ROW ? D * 384 : 0;
  static_assert(!ROW || NT == 1, "blocks along N: one column tile per workgroup");
  // [wave][kWaveBytes] rows, then the partial tiles, then (blocks along N) [wave][kRowMetaBytes]
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  float* red = reinterpret_cast<float*>(smem + kWaves * kWaveBytes);

  // The arguments fill the 14 registers that can be preloaded (N and M - 1 share one: N < 2^28, M <= 16), so none
  // of them is fetched from memory, least of all at the end, where the bias pointer is first needed.  (Were they
  // not preloaded, this would fetch them all at once, up front: the compiler fetches every argument right before
  // its first use and waits for it there.)
  asm volatile("" ::"s"(A), "s"(W), "s"(S), "s"(Z), "s"(C), "s"(bias), "s"(n_and_m), "s"(K));
  const int N = static_cast<int>(n_and_m & 0x0fffffffu);
  const int M = static_cast<int>(n_and_m >> 28) + 1;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int nl = lane & 15;  // column inside the tile (weights operand) / activation row (other operand)
  const int g = lane >> 4;   // which of the 4 k-units of a slice
  const int slices = K >> 7;
  const int units = K >> 5;
  const int tiles = N >> 4;
  // Workgroup -> group of NT column tiles.  Consecutive workgroups go to consecutive XCDs (8 of them, each with an L2
  // of its own); an XCD's workgroups take eight neighbouring groups at a time, which share the cache lines of the
  // zero-point and scale rows, so that those are fetched from memory once.  The grid is rounded up to whole sets
  // of 64 groups.  (M = 1, K = N = 4096, one group per workgroup in launch order against two, four and eight
  // neighbours per XCD: 3.66, 3.64, 3.78, 3.62 us; with zero-points 4.05, 3.71, 3.86, 3.69; blocks of 16 with
  // zero-points 5.83, 4.80, 4.64, 4.52; no shape lost more than 2 %.)
  const uint32_t wg = blockIdx.x;
  const uint32_t cg = (((wg >> 3) >> 3) << 6) + ((wg & 7) << 3) + ((wg >> 3) & 7);
  if (cg >= static_cast<uint32_t>((tiles + NT - 1) / NT)) return;
  // this wave's slices: s0 .. s0 + mine - 1, mine = D or D - 1
  const int s0 = (wave * slices) >> kLgWaves;
  const int mine = (((wave + 1) * slices) >> kLgWaves) - s0;
  const bool last_ok = mine == D;  // wave-uniform

  // Rows.  A copy instruction fills 1 KiB of LDS, lane l the 16 bytes at 16 l: eight row-chunks e = (pair, row) of
  // 128 bytes, physical chunk l & 7 holding logical chunk (l & 7) ^ bits 1..3 of the row.
  // Up to four rows: all copies of the wave first (copy q fills bytes [1024 q, 1024 q + 1024) of the wave's part;
  // a slice has less than a copy's worth of rows).  Units past the end of K (the missing slot of the last wave)
  // fetch the last unit instead: any finite values do, they meet a zero scale.
  // Eight or sixteen rows: a slot's copies (two or four) go right before the slot's other requests, see below.
  constexpr bool kPerSlot = R >= 8;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)(smem)));
  const uint32_t wave_lds = lds0 + wave * kWaveBytes;
  // Blocks along N: the scales and zero-points of the wave's slices lie in one run each, [K] of the tile's column
  // block: copied first, 16 bytes per lane (the k range of a missing slot past the end of K fetches the last 16
  // bytes of the run instead)
  const uint32_t meta_lds = lds0 + kWaves * kWaveBytes + kWaves * NT * R * 64 + wave * kRowMetaBytes;
  if constexpr (ROW) {
    const uint32_t run = (cg * 16 / BS) * static_cast<uint32_t>(K) + static_cast<uint32_t>(s0) * 128u;  // elements
    const uint32_t run_end = (cg * 16 / BS + 1) * static_cast<uint32_t>(K);
#pragma unroll
    for (int c = 0; c * 1024 < kRowScaleBytes; ++c) {
      const uint32_t off = c * 1024 + lane * 16;
      if ((c + 1) * 1024 <= kRowScaleBytes || off < static_cast<uint32_t>(kRowScaleBytes)) {
        async_copy_16(meta_lds + c * 1024, S, min(run + off / 2, run_end - 8) * 2);
      }
    }
    if constexpr (HAS_ZP) {
      const uint32_t off = lane * 16;  // D * 128 <= 1024 bytes: one copy
      if (off < static_cast<uint32_t>(D * 128)) async_copy_16(meta_lds + kRowScaleBytes, Z, min(run + off, run_end - 16));
    }
  }
#pragma unroll
  for (int q = 0; q < (kPerSlot ? 0 : kCopies); ++q) {
    const uint32_t off = q * 1024 + lane * 16;
    const uint32_t e = off >> 7;
    const uint32_t r = e & (R - 1);
    const uint32_t pp = e >> kLgR;
    const uint32_t chunk = (lane & 7) ^ ((r >> 1) & 7);
    const uint32_t u = min(static_cast<uint32_t>(4 * s0) + 2 * pp + (chunk >> 2), static_cast<uint32_t>(units - 1));
    const uint32_t row = (R == 1) ? 0u : min(r, static_cast<uint32_t>(M - 1));
    if ((q + 1) * 1024 <= kWaveBytes || off < static_cast<uint32_t>(kWaveBytes)) {
      async_copy_16(wave_lds + q * 1024, A, (row * K + u * 32 + (chunk & 3) * 8) * 2);
    }
  }

  // Requests, slot by slot: scales and zero-points, then the weights.  Lane (nl, g) owns unit g of the slice for
  // column nl of each tile.  A tile past the end (last workgroup, when NT does not divide the tiles) re-reads
  // the last tile and is not stored.
  uint4 w[D][NT];
  uint32_t sc[D][NT][kMeta], zp[D][NT][kMeta];
  {
    // offsets of slot 0 (one multiplication each), the later slots a wave-uniform stride further
    const uint32_t unit0 = 4u * s0 + g;
    const uint32_t blk0 = (BS == 64) ? (unit0 >> 1) : (BS == 32) ? unit0 : 2 * unit0;
    const uint32_t w_stride = static_cast<uint32_t>(N) * 64u;               // bytes: 4 units of N columns
    const uint32_t m_stride = static_cast<uint32_t>(N) * (128u / BS);       // elements: the blocks of a slice
    const uint32_t last = static_cast<uint32_t>(min(D - 1, slices - 1 - s0));  // the missing slot asks for the last slice again
    // per-slot copies: copy h of a slot covers row-chunks 8 h .. 8 h + 7 of the slice; the lane's part of the
    // address never changes, the slice adds 256 bytes along K
    constexpr int kSlotCopies = kPerSlot ? R / 4 : 1;
    uint32_t a_off[kSlotCopies];
    if constexpr (kPerSlot) {
#pragma unroll
      for (int h = 0; h < kSlotCopies; ++h) {
        const uint32_t e = 8 * h + (lane >> 3);
        const uint32_t r = e & (R - 1);
        const uint32_t chunk = (lane & 7) ^ ((r >> 1) & 7);
        a_off[h] = (min(r, static_cast<uint32_t>(M - 1)) * K + (2 * (e >> kLgR) + (chunk >> 2)) * 32 + (chunk & 3) * 8) * 2 +
                   static_cast<uint32_t>(s0) * 256u;
      }
    }
    uint32_t w_off[NT], m_idx[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const uint32_t tile = (NT == 1) ? cg : min(cg * NT + t, static_cast<uint32_t>(tiles - 1));
      const uint32_t col = tile * 16 + nl;
      w_off[t] = (unit0 * N + col) * 16u;
      m_idx[t] = blk0 * N + col;
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const uint32_t dd = (d == D - 1) ? last : static_cast<uint32_t>(d);
      if constexpr (kPerSlot) {
#pragma unroll
        for (int h = 0; h < kSlotCopies; ++h) async_copy_16(wave_lds + d * kSliceBytes + h * 1024, A, a_off[h] + dd * 256u);
      }
      if constexpr (!ROW) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
#pragma unroll
          for (int q = 0; q < kMeta; ++q) {
            const uint32_t idx = m_idx[t] + dd * m_stride + (q == 0 ? 0u : static_cast<uint32_t>(N));
            sc[d][t][q] = *reinterpret_cast<const uint16_t*>(S + static_cast<size_t>(idx * 2u));
            zp[d][t][q] = HAS_ZP ? Z[static_cast<size_t>(idx)] : 8u;
          }
        }
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        // (read once per launch: non-temporal)
        const uint4_t v = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(W + static_cast<size_t>(w_off[t] + dd * w_stride)));
        w[d][t] = make_uint4(v[0], v[1], v[2], v[3]);
      }
      __builtin_amdgcn_sched_barrier(0);  // in this order
    }
  }

  const DequantMasks masks = DequantMasks::make();
  float4_t acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};

  // This lane's fragment addresses: row nl (rows past R - 1 read row R - 1: their sums are not stored), unit g =
  // half g & 1 of pair g >> 1.  The copies of a slot (of all slots, up to four rows) were requested before the
  // slot's weights (the first slot's) and requests complete in order: the reads wait for a word of those weights,
  // and with it for the rows.
  const uint32_t row = (R == 16) ? nl : min(nl, R - 1);
  // logical chunk 4 (g & 1) + j lies at physical chunk c0 ^ j; with one or two rows nothing is swizzled
  const uint32_t c0 = ((g & 1) * 4) ^ ((row >> 1) & 7);
  const uint32_t a_lane = (wave_lds + (g >> 1) * (128 * R) + row * 128) | (c0 << 4);
  auto fragments = [&](uint4 (&af)[4], int d, uint32_t arrived) {
    const uint32_t base = a_lane + arrived;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      af[j] = (R <= 2) ? lds_read_16(base, d * kSliceBytes + j * 16) : lds_read_16(base ^ (j << 4), d * kSliceBytes);
    }
  };

  // Blocks along N: the 32 scales (64 bytes) and zero-points (32 bytes) of the lane's unit, from the wave's copy
  auto row_meta = [&](uint4 (&rs)[4], uint4 (&rz)[2], int d, uint32_t arrived) {
    const uint32_t base = meta_lds + g * 64 + arrived;
#pragma unroll
    for (int q = 0; q < 4; ++q) rs[q] = lds_read_16(base, d * 256 + q * 16);
    if constexpr (HAS_ZP) {
      const uint32_t zbase = meta_lds + kRowScaleBytes + g * 32 + arrived;
#pragma unroll
      for (int q = 0; q < 2; ++q) rz[q] = lds_read_16(zbase, d * 128 + q * 16);
    }
  };

  // Slot by slot, while the later ones are on their way.  Up to four rows: the fragments of the next slot (and its
  // scales and zero-points, with blocks along N) are read while this one is converted (one read at a time right
  // before its MFMA leaves most of the LDS latency in the open).  More rows: a slot's fragments are there when its
  // weights are, and are read then.
  uint4 af[2][4];
  uint4 rs[2][4], rz[2][2];
  uint32_t arrived = 0;
  if constexpr (!kPerSlot || ROW) arrived = zero_once_loaded(w[0][0].x);
  if constexpr (!kPerSlot) fragments(af[0], 0, arrived);
  if constexpr (ROW) row_meta(rs[0], rz[0], 0, arrived);
#pragma unroll
  for (int d = 0; d < D; ++d) {
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kPerSlot) {
      fragments(af[d & 1], d, zero_once_loaded(w[d][0].x));
    } else {
      if (d + 1 < D) fragments(af[(d + 1) & 1], d + 1, arrived);
    }
    if constexpr (ROW) {
      if (d + 1 < D) row_meta(rs[(d + 1) & 1], rz[(d + 1) & 1], d + 1, arrived);
    }
    const uint32_t keep = (d < D - 1 || last_ok) ? 0xffffffffu : 0u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const uint32_t word = vec_word(w[d][t], j);
        const int q = (kMeta == 2) ? (j >> 1) : 0;
        if constexpr (ROW) {
          // word j is rows 8 hh .. 8 hh + 7 of 16-row group j / 2 of the unit: pair i has its scales in 32-bit word
          // 2 i + hh of the group and its zero-points in byte pair hh of word i (blkq4_skinny.hip has the same)
          const int hh = j & 1;
          const uint4 s0v = rs[d & 1][2 * (j >> 1)], s1v = rs[d & 1][2 * (j >> 1) + 1];
          const uint32_t sw[8] = {s0v.x, s0v.y, s0v.z, s0v.w, s1v.x, s1v.y, s1v.z, s1v.w};
          const uint4 zq = HAS_ZP ? rz[d & 1][j >> 1] : make_uint4(0, 0, 0, 0);
          const uint32_t zw[4] = {zq.x, zq.y, zq.z, zq.w};
          const uint32_t y = word >> 8;
          half2_t p[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t zpair = HAS_ZP ? ((zw[i] >> (8 * hh)) & 0x00ff00ffu) : 0x00080008u;
            const uint32_t src = (i >= 2) ? y : word;
            // q - zp of the pair, exact
            const half2_t dq = ((i & 1) == 0)
                ? as_half2((src & masks.lo_mask) | masks.magic_1024) + as_half2(0xE400E400u | zpair)
                : as_half2((src & masks.hi_mask) | masks.magic_64) + as_half2(0xD400D400u | (zpair << 4));
            if constexpr (BF) {
              p[i] = as_half2(row_pair_bf16(dq, sw[2 * i + hh] & keep));  // a bf16 pair in the same register
            } else {
              p[i] = dq * as_half2(sw[2 * i + hh] & keep);
            }
          }
          half8_t wf;
          wf[0] = p[0][0]; wf[1] = p[0][1]; wf[2] = p[1][0]; wf[3] = p[1][1];
          wf[4] = p[2][0]; wf[5] = p[2][1]; wf[6] = p[3][0]; wf[7] = p[3][1];
          if constexpr (BF) {
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, wf), as_bf16x8(af[d & 1][j]), acc[t], 0, 0, 0);
          } else {
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, as_half8(af[d & 1][j]), acc[t], 0, 0, 0);
          }
        } else if constexpr (BF) {
          const Bf16Consts bc = make_bf16_consts(sc[d][t][q] & keep, zp[d][t][q]);
          const bf16x8_t wf = dequant_word_bf16(word, bc, masks);
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, as_bf16x8(af[d & 1][j]), acc[t], 0, 0, 0);
        } else {
          const DequantConsts c = make_dequant_consts(sc[d][t][q] & keep, zp[d][t][q]);
          const uint32_t y = word >> 8;
          half2_t p[4];
          p[0] = dequant_pair(word, 0, c, masks);
          p[1] = dequant_pair(word, 1, c, masks);
          p[2] = dequant_pair(y, 2, c, masks);
          p[3] = dequant_pair(y, 3, c, masks);
          half8_t wf;
          wf[0] = p[0][0]; wf[1] = p[0][1]; wf[2] = p[1][0]; wf[3] = p[1][1];
          wf[4] = p[2][0]; wf[5] = p[2][1]; wf[6] = p[3][0]; wf[7] = p[3][1];
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, as_half8(af[d & 1][j]), acc[t], 0, 0, 0);
        }
      }
    }
  }

  // Partial tiles: [wave][tile t][row][16 columns] floats; lane (nl, g) holds columns 4 g .. 4 g + 3 of row nl.
  if (nl < R) {
#pragma unroll
    for (int t = 0; t < NT; ++t) *reinterpret_cast<float4_t*>(&red[(((wave * NT + t) << kLgR) + nl) * 16 + 4 * g]) = acc[t];
  }
  __syncthreads();
  constexpr int kPerWave = NT * R * 16;
  for (int v = tid; v < kPerWave; v += 64 * kWaves) {
    float sum = 0.f;
#pragma unroll
    for (int x = 0; x < kWaves; ++x) sum += red[x * kPerWave + v];
    const int c = v & 15, r = (v >> 4) & (R - 1), t = v >> (4 + kLgR);
    const int tile = static_cast<int>(cg) * NT + t;
    if (r < M && tile < tiles) {
      const int col = tile * 16 + c;
      uint32_t h = float_to_bits<BF>(sum);
      if (bias != nullptr) h = add_bias_bits_t<BF>(h, bias[col]);
      C[static_cast<size_t>(r) * N + col] = static_cast<uint16_t>(h);
    }
  }
}

template <auto kKernel>
hipError_t raise_lds_limit() {
  return raise_lds_limit_once(reinterpret_cast<const void*>(kKernel), kMaxLdsBytes, &lds_limit_flags<kKernel>());
}

// One instantiation with the geometry of the plan (blkq4_choose.h).  What the kernel assumes is checked here.
template <int BS, bool HAS_ZP, bool ROW, int R, int NT, int kWaves, int D>
int launch_kernel(const blkq4_gemm_args* a) {
  const blkq4_decode_plan& p = a->decode;
  if (a->launched_id != nullptr) *a->launched_id = decode_id(ROW, R, NT, kWaves, D);
  const int slices = a->k / 128;
  const size_t lds = decode_lds_bytes(ROW, R, NT, kWaves, D);
  if (a->m > R || slices > kWaves * D || slices <= kWaves * (D - 1) || lds > kMaxLdsBytes || p.lds_bytes != lds ||
      p.grid != decode_grid(a->n, NT)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (a->dry_run) return 0;  // the plan has passed every check a launch makes
  constexpr auto kernel = decode_mfma_kernel<BS, HAS_ZP, R, NT, kWaves, D, ROW>;
  if (lds > 64 * 1024) {
    if (hipError_t e = raise_lds_limit<kernel>(); e != hipSuccess) return static_cast<int>(e);
  }
  return static_cast<int>(launch_status(kernel, dim3(p.grid), dim3(64 * kWaves), lds, a->stream,
                                        static_cast<const uint8_t*>(a->a), static_cast<const uint8_t*>(a->packed_w),
                                        static_cast<const uint8_t*>(a->scales),
                                        static_cast<const uint8_t*>(a->zero_points), static_cast<uint16_t*>(a->c),
                                        static_cast<const uint16_t*>(a->bias),
                                        static_cast<uint32_t>(a->n) | static_cast<uint32_t>(a->m - 1) << 28, a->k));
}

// The shapes that exist, (R, NT, waves, D): what blkq4::decode_shape() may ask for.
#define BLKQ4_DECODE_DEPTHS(X, R_, NT_, W_) \
  X(R_, NT_, W_, 1) X(R_, NT_, W_, 2) X(R_, NT_, W_, 3) X(R_, NT_, W_, 4) X(R_, NT_, W_, 5) X(R_, NT_, W_, 6) \
  X(R_, NT_, W_, 7) X(R_, NT_, W_, 8)
#define BLKQ4_DECODE_DEPTHS_TO_4(X, R_, NT_, W_) X(R_, NT_, W_, 1) X(R_, NT_, W_, 2) X(R_, NT_, W_, 3) X(R_, NT_, W_, 4)
#define BLKQ4_DECODE_DEPTHS_9_TO_14(X, R_, NT_, W_) \
  X(R_, NT_, W_, 9) X(R_, NT_, W_, 10) X(R_, NT_, W_, 11) X(R_, NT_, W_, 12) X(R_, NT_, W_, 13) X(R_, NT_, W_, 14)
#define BLKQ4_DECODE_SHAPES(X)                                                                     \
  BLKQ4_DECODE_DEPTHS(X, 1, 1, 4) BLKQ4_DECODE_DEPTHS(X, 1, 1, 8) BLKQ4_DECODE_DEPTHS(X, 1, 1, 16) \
  BLKQ4_DECODE_DEPTHS(X, 4, 1, 4) BLKQ4_DECODE_DEPTHS(X, 4, 1, 8) BLKQ4_DECODE_DEPTHS(X, 4, 1, 16) \
  BLKQ4_DECODE_DEPTHS(X, 1, 2, 8) BLKQ4_DECODE_DEPTHS(X, 4, 2, 8)                                  \
  /* K up to 28672 with sixteen waves */                                                           \
  BLKQ4_DECODE_DEPTHS_9_TO_14(X, 1, 1, 16) BLKQ4_DECODE_DEPTHS_9_TO_14(X, 4, 1, 16)                \
  /* eight rows fit in LDS up to K = 8192, sixteen up to K = 4096 */                               \
  BLKQ4_DECODE_DEPTHS(X, 8, 1, 8) BLKQ4_DECODE_DEPTHS(X, 8, 2, 8) BLKQ4_DECODE_DEPTHS(X, 8, 3, 8)  \
  BLKQ4_DECODE_DEPTHS_TO_4(X, 16, 1, 8) BLKQ4_DECODE_DEPTHS_TO_4(X, 16, 2, 8) BLKQ4_DECODE_DEPTHS_TO_4(X, 16, 3, 8) BLKQ4_DECODE_DEPTHS_TO_4(X, 16, 4, 8)
// blocks along N: up to four rows, one tile, K up to 8192
#define BLKQ4_DECODE_ROW_SHAPES(X)                                                    \
  BLKQ4_DECODE_DEPTHS(X, 1, 1, 8) BLKQ4_DECODE_DEPTHS(X, 4, 1, 8)                     \
  X(1, 1, 4, 1) X(1, 1, 4, 2) X(1, 1, 4, 8) X(4, 1, 4, 1) X(4, 1, 4, 2) X(4, 1, 4, 8)

template <int BS, bool HAS_ZP, bool ROW>
int launch_plan(const blkq4_gemm_args* a) {
  const blkq4_decode_plan& p = a->decode;
#define BLKQ4_TRY(R_, NT_, W_, D_) \
  if (p.rows == R_ && p.nt == NT_ && p.waves == W_ && p.depth == D_) return launch_kernel<BS, HAS_ZP, ROW, R_, NT_, W_, D_>(a);
  if constexpr (ROW) {
    BLKQ4_DECODE_ROW_SHAPES(BLKQ4_TRY)
  } else {
    BLKQ4_DECODE_SHAPES(BLKQ4_TRY)
  }
#undef BLKQ4_TRY
  return static_cast<int>(hipErrorInvalidValue);  // a shape that does not exist
}

template <int BS>
int launch_bs(const blkq4_gemm_args* a) {
  if (a->column_wise) return a->zero_points ? launch_plan<BS, true, false>(a) : launch_plan<BS, false, false>(a);
  return a->zero_points ? launch_plan<BS, true, true>(a) : launch_plan<BS, false, true>(a);
}

}  // namespace

extern "C" int BLKQ4_DECODE_ENTRY(const blkq4_gemm_args* a) {
  // 32-bit offsets: the packed weights end below 4 GiB
  if (a->m < 1 || a->m > 16 || (a->n % 16) != 0 || (a->k % 128) != 0 ||
      static_cast<uint64_t>(a->k) * static_cast<uint64_t>(a->n) > (uint64_t{1} << 32)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (!a->column_wise) {
    // blocks along N: a 16-column tile lies inside one block, and the meta data are copied 16 bytes at a time
    if ((a->n % a->block_size) != 0 || (reinterpret_cast<uintptr_t>(a->scales) & 15u) != 0 ||
        (reinterpret_cast<uintptr_t>(a->zero_points) & 15u) != 0) {
      return static_cast<int>(hipErrorInvalidValue);
    }
  }
  switch (a->block_size) {
    case 16: return launch_bs<16>(a);
    case 32: return launch_bs<32>(a);
    case 64: return launch_bs<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}
