// M = 1..16 path (decode GEMV and small-batch GEMM) for gfx950.
//
// The work is a stream over the packed weights (K*N/2 bytes plus scales and zero-points) that has to
// run at HBM speed; everything else is arranged so that the stream is requested as early and as
// deeply as possible and nothing serialises behind it:
//   - a workgroup of four or eight waves owns 16, 32 or 48 output columns and the whole K range; the waves split K in
//     128-deep slices, so every wave load is one 16-byte unit per lane: 16 columns x 4 consecutive
//     k-units = four contiguous 256-byte runs of the packed layout;
//   - a wave keeps the weight units, scales and zero-points of kDepth slices in flight and refills a
//     slot as soon as it has consumed it (out-of-range slices wrap around to valid units and are
//     multiplied by a zero scale, so the loop has no divergent loads);
//   - the activation rows (at most 16 x K fp16) are copied once per workgroup into LDS by asynchronous
//     global_load_lds copies issued before the first weight request, laid out per 32-deep unit as
//     [unit][row][64 bytes] (16-byte chunks XOR-swizzled with bits 2..3 of the row so that a fragment
//     read is free of bank conflicts); when they do not fit (K too large) the lanes that carry a row
//     load their 64 bytes per slice straight from global memory (L2 resident) into the same ring;
//   - a lane multiplies its (column, 32 k) of weights with the matching 32 k of up to 16 activation
//     rows through v_mfma_f32_16x16x32_f16 (weights as the row operand: a lane ends up with 4
//     consecutive output columns of one activation row, one 8-byte store);
//   - the waves' partial tiles are summed through LDS by wave 0: no atomics, no scratch buffer.
// Dequantization happens in registers (blkq4_dequant.h); accumulation is fp32.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_dequant.h"
#include "blkq4_device.h"
#include "blkq4_gemm_common.h"

namespace {

using namespace blkq4;


// Where a wave finds its activation fragments.
constexpr int kRowsInRegisters = 0;  // each lane loads its rows' 64 bytes per slice into the ring of slots
constexpr int kRowsWholeInLds = 1;   // all rows, all of K, staged once per workgroup
constexpr int kRowsPerSlotInLds = 2; // 16 * MT rows x 128 k staged per slot, private to the wave

template <int BS, int NT, int MT, int AM>
struct Slot {
  static constexpr int kMeta = (BS == 16) ? 2 : 1;  // quantization blocks inside one 32-deep unit
  uint4 w[NT];
  uint32_t sc[NT][kMeta];
  uint32_t zp[NT][kMeta];
  uint4 a[AM == kRowsInRegisters ? 4 * MT : 1];  // 32 k of this lane's activation rows (unused when they are in LDS)
};

// kWaves: waves of the workgroup, which split K.  DEPTH: k slices (128 deep) a wave keeps in flight.  NT: 16-column tiles per wave that share one
// activation operand.  MT: 16-row tiles of activations (M <= 16 * MT) that share one conversion of the
// weights.  AM: where the activation rows are (see above).  kRowsWholeInLds: rows_log2 = log2 of the number
// of rows kept in LDS, a power of two >= M, and the dynamic LDS size is red_bytes + (K * 2 << rows_log2).
// kRowsPerSlotInLds: red_bytes + kWaves * DEPTH * 16 * MT * 256.
template <int BS, bool HAS_ZP, int DEPTH, int NT, int MT, int kWaves, int AM>
__global__ __launch_bounds__(64 * kWaves) void skinny_mfma_kernel(const uint16_t* __restrict__ A,
                                                               const uint4* __restrict__ W,
                                                               const uint16_t* __restrict__ S,
                                                               const uint8_t* __restrict__ Z,
                                                               uint16_t* __restrict__ C, int M, int N,
                                                               int K, int rows_log2) {
  constexpr int kMeta = Slot<BS, NT, MT, AM>::kMeta;
  constexpr bool A_LDS = AM == kRowsWholeInLds;
  constexpr int kLoads = NT * (1 + kMeta * (HAS_ZP ? 2 : 1));  // weight / scale / zero-point requests of a slot
  constexpr int kSlotRows = 16 * MT;                           // kRowsPerSlotInLds: rows staged per slot
  constexpr int kSlotBytes = kSlotRows * 256;
  constexpr int kRedFloats = kWaves * NT * MT * 64 * 4;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  float* red = reinterpret_cast<float*>(smem);
  const uint8_t* a_lds = smem + kRedFloats * 4;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int nl = lane & 15;  // column inside the tile (weights operand) / activation row (other operand)
  const int g = lane >> 4;   // which of the 4 k-units of a slice
  const int tiles = N >> 4;
  // column this lane loads for tile t; a tile past the end (last workgroup only, when NT does not
  // divide the tile count) re-reads the workgroup's first tile and is not stored
  int n[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int tile = blockIdx.x * NT + t;
    n[t] = ((tile < tiles) ? tile : blockIdx.x * NT) * 16 + nl;
  }
  const DequantMasks masks = DequantMasks::make();
  // lanes without a row (past M) re-read the last row: an output element depends on its own activation
  // row only, and the rows past M are never stored
  const uint8_t* a_row[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    a_row[mt] = reinterpret_cast<const uint8_t*>(A) + static_cast<size_t>(min(16 * mt + nl, M - 1)) * K * 2;
  }

  const int units = K >> 5;             // 32-deep units
  const int slices = (units + 3) >> 2;  // 128-deep slices (the last one may be half full)
  const int my_slices = (slices - wave + kWaves - 1) / kWaves;  // slices wave, wave + kWaves, ...

  const int wrap_mask = (1 << (31 - __builtin_clz(units))) - 1;  // any index & wrap_mask is < units

  float4_t acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = float4_t{0.f, 0.f, 0.f, 0.f};
  Slot<BS, NT, MT, AM> slot[DEPTH];

  // Rows to LDS: copy q fills LDS bytes [1024 q, 1024 q + 1024) of the [unit][row][64 B] layout, lane l
  // the 16 bytes at 16 l.  They are requested before anything else, so every later wait covers them.
  uint32_t a_rd = 0;  // LDS byte offset of this lane's row inside a unit, chunk 0
  uint32_t a_swz = 0;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                            (__attribute__((address_space(3))) uint8_t*)(smem))) + kRedFloats * 4;
  if (AM == kRowsPerSlotInLds) {
    // this wave's slots: DEPTH pieces of [4 units][kSlotRows rows][64 B]
    a_rd = (wave * DEPTH) * kSlotBytes + g * (kSlotRows * 64) + nl * 64;
    a_swz = (nl >> 2) & 3;
  }
  if (A_LDS) {
    const int rows = 1 << rows_log2;
    const int copies = ((K << rows_log2) + 511) >> 9;  // K * 2 * rows bytes in 1 KiB copies, the last one may be partial
    for (int q = wave; q < copies; q += kWaves) {
      const uint32_t off = q * 1024 + lane * 16;
      const int u = min(static_cast<int>(off >> (6 + rows_log2)), units - 1);  // past the end: any valid unit
      const int row = (off >> 6) & (rows - 1);
      const int chunk = (lane & 3) ^ ((row >> 2) & 3);
      async_copy_16(lds0 + q * 1024, A, (static_cast<uint32_t>(min(row, M - 1)) * K + u * 32 + chunk * 8) * 2);
    }
    const int row = min(nl, rows - 1);  // row tile mt: 16 mt rows further (same swizzle: bits 2..3 of the row)
    a_rd = row * 64;
    a_swz = (row >> 2) & 3;
  }
  // a slice past the end wraps around to valid units (so every slot always issues the same loads)
  // and gets a zero scale, which makes it contribute exactly 0
#define BLKQ4_LOAD_SLOT(dst_, d_, slice_)                                                        \
  {                                                                                            \
    const int ks_ = 4 * (slice_) + g;                                                          \
    const bool ok_ = ks_ < units;                                                              \
    const int ksg_ = ok_ ? ks_ : (ks_ & wrap_mask);                                            \
    const int b_ = (BS == 64) ? (ksg_ >> 1) : (BS == 32) ? ksg_ : (2 * ksg_);                  \
    if (AM == kRowsPerSlotInLds) {                                                             \
      /* copy q: LDS bytes [1024 q, 1024 q + 1024) of the slot, lane l the 16 bytes at 16 l; */ \
      /* requested before the slot's weights, so whoever has the weights has the rows        */ \
      _Pragma("unroll") for (int q = 0; q < 4 * MT; ++q) {                                     \
        const int rr_ = 16 * q + (lane >> 2);            /* (unit, row) index inside the slot */ \
        const int u_ = 4 * (slice_) + rr_ / kSlotRows;                                         \
        const int ug_ = (u_ < units) ? u_ : (u_ & wrap_mask);                                  \
        const int row_ = rr_ % kSlotRows;                                                      \
        const int chunk_ = (lane & 3) ^ ((row_ >> 2) & 3);                                     \
        async_copy_16(lds0 + (wave * DEPTH + (d_)) * kSlotBytes + q * 1024, A,                 \
                      (static_cast<uint32_t>(min(row_, M - 1)) * K + ug_ * 32 + chunk_ * 8) * 2); \
      }                                                                                        \
    }                                                                                          \
    _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                           \
      (dst_).w[t] = W[static_cast<size_t>(ksg_) * N + n[t]];                                  \
      _Pragma("unroll") for (int q = 0; q < kMeta; ++q) {                                      \
        const size_t mi_ = static_cast<size_t>(b_ + q) * N + n[t];                           \
        const uint32_t sc_ = S[mi_];                                                           \
        (dst_).sc[t][q] = ok_ ? sc_ : 0u;                                                      \
        (dst_).zp[t][q] = HAS_ZP ? static_cast<uint32_t>(Z[mi_]) : 8u;                         \
      }                                                                                        \
    }                                                                                          \
    if (AM == kRowsInRegisters) {                                                              \
      _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                      \
        const uint4* p_ = reinterpret_cast<const uint4*>(a_row[mt] + static_cast<size_t>(ksg_) * 64); \
        _Pragma("unroll") for (int j = 0; j < (AM == kRowsInRegisters ? 4 : 0); ++j) {         \
          (dst_).a[(AM == kRowsInRegisters) ? 4 * mt + j : 0] = p_[j];                         \
        }                                                                                      \
      }                                                                                        \
    }                                                                                          \
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) BLKQ4_LOAD_SLOT(slot[d], d, wave + d * kWaves);
  if (A_LDS) {
    // everything but the requests of the ring just issued has landed: this wave's share of the rows
    constexpr int kRing = DEPTH * kLoads;
    wait_vmcnt<(kRing < 63 ? kRing : 63)>();
    __syncthreads();
  }

  for (int i0 = 0; i0 < my_slices; i0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int li = i0 + d;  // local slice index; slice = wave + 4*li
      half8_t af[MT][4];
      if (A_LDS) {
        const int ks = 4 * (wave + kWaves * li) + g;
        const int ksg = (ks < units) ? ks : (ks & wrap_mask);
        const uint8_t* ap = a_lds + (static_cast<uint32_t>(ksg) << (6 + rows_log2)) + a_rd;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            af[mt][j] = as_half8(*reinterpret_cast<const uint4*>(ap + mt * 1024 + ((j ^ a_swz) * 16)));
          }
      } else if (AM == kRowsPerSlotInLds) {
        // the rows of this slot were requested before its weights; younger than them are those weights and
        // everything the other DEPTH - 1 slots have requested since
        constexpr int kYounger = kLoads + (DEPTH - 1) * (4 * MT + kLoads);
        wait_vmcnt<(kYounger < 63 ? kYounger : 63)>();
        const uint8_t* ap = a_lds + a_rd + d * kSlotBytes;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            af[mt][j] = as_half8(*reinterpret_cast<const uint4*>(ap + mt * 1024 + ((j ^ a_swz) * 16)));
          }
      } else {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int j = 0; j < 4; ++j) af[mt][j] = as_half8(slot[d].a[(AM == kRowsInRegisters) ? 4 * mt + j : 0]);
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        DequantConsts dc[kMeta];
#pragma unroll
        for (int q = 0; q < kMeta; ++q) dc[q] = make_dequant_consts(slot[d].sc[t][q], slot[d].zp[t][q]);
        const uint32_t words[4] = {slot[d].w[t].x, slot[d].w[t].y, slot[d].w[t].z, slot[d].w[t].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const DequantConsts& c = dc[(kMeta == 2) ? (j >> 1) : 0];
          const uint32_t y = words[j] >> 8;
          const half2_t p0 = dequant_pair(words[j], 0, c, masks), p1 = dequant_pair(words[j], 1, c, masks);
          const half2_t p2 = dequant_pair(y, 2, c, masks), p3 = dequant_pair(y, 3, c, masks);
          half8_t wf;
          wf[0] = p0[0]; wf[1] = p0[1]; wf[2] = p1[0]; wf[3] = p1[1];
          wf[4] = p2[0]; wf[5] = p2[1]; wf[6] = p3[0]; wf[7] = p3[1];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, af[mt][j], acc[t][mt], 0, 0, 0);
          }
        }
      }
      if (i0 + DEPTH < my_slices) BLKQ4_LOAD_SLOT(slot[d], d, wave + kWaves * (li + DEPTH));
    }
  }
#undef BLKQ4_LOAD_SLOT

  // cross-wave reduction through LDS
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int e = 0; e < 4; ++e) red[(((wave * NT + t) * MT + mt) * 64 + lane) * 4 + e] = acc[t][mt][e];
  __syncthreads();
  // value v = (tile t, row tile mt, lane L, element e) of the partial tiles: output row 16 mt + (L & 15),
  // column 4 (L >> 4) + e of tile t; every thread sums a few of them over the waves
  for (int v = tid; v < NT * MT * 256; v += 64 * kWaves) {
    float r = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) r += red[w * (NT * MT * 256) + v];
    const int t = v / (MT * 256), mt = (v >> 8) % MT, L = (v >> 2) & 63, e = v & 3;
    const int row = 16 * mt + (L & 15);
    if (row < M && blockIdx.x * NT + t < tiles) {
      C[static_cast<size_t>(row) * N + blockIdx.x * (16 * NT) + 16 * t + 4 * (L >> 4) + e] = float_to_half_bits(r);
    }
  }
}

// The kernel is bound by instruction issue as much as by the weight stream, so what matters is how
// evenly the workgroups fill the 256 compute units: with T column tiles per workgroup the busiest
// unit works through ceil(workgroups / 256) * T tiles.  Wider workgroups also re-read the activation
// rows less often, which weighs more the more rows there are.
constexpr size_t kMaxLdsBytes = 160 * 1024;
#ifndef BLKQ4_SKINNY_WAVES16
#define BLKQ4_SKINNY_WAVES16 1
#endif

void choose_shape(int m, int n, int* nt, int* depth) {
  constexpr int kComputeUnits = 256;
  const int tiles = n / 16;
  const float a_weight = (m > 4) ? 0.2f : 0.05f;  // cost of fetching the activations relative to one tile's work
  float best = 0.f;
  *nt = 1;
  for (int t = 1; t <= 3; ++t) {
    const int wgs = (tiles + t - 1) / t;
    const int rounds = (wgs + kComputeUnits - 1) / kComputeUnits;
    const float cost = static_cast<float>(rounds) * (static_cast<float>(t) + a_weight);
    if (t == 1 || cost < best) {
      best = cost;
      *nt = t;
    }
  }
  // one tile per workgroup: 8 slices in flight while at most two workgroups share a unit, else 4
  // (the deeper ring needs too many registers for more resident waves)
  *depth = (*nt == 1 && tiles <= 2 * kComputeUnits) ? 8 : 4;
}

// One kernel instantiation: raises its dynamic-LDS limit once, then launches.
template <int BS, bool HAS_ZP, int DEPTH, int NT, int MT, int kWaves, int AM>
int launch_kernel(const blkq4_gemm_args* a, int rows_log2) {
  constexpr int kRedBytes = kWaves * NT * MT * 64 * 4 * 4;
  constexpr size_t kPerSlotBytes = static_cast<size_t>(kWaves) * DEPTH * 16 * MT * 256;
  static_assert(AM != kRowsPerSlotInLds || kRedBytes + kPerSlotBytes <= kMaxLdsBytes, "slots do not fit in LDS");
  // the rows are copied 1 KiB at a time
  const size_t lds_bytes =
      kRedBytes + (AM == kRowsWholeInLds ? ((((static_cast<size_t>(a->k) * 2) << rows_log2) + 1023) & ~size_t{1023})
                   : AM == kRowsPerSlotInLds ? kPerSlotBytes
                                             : 0);
  auto* kernel = skinny_mfma_kernel<BS, HAS_ZP, DEPTH, NT, MT, kWaves, AM>;
  static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsBytes);
  if (attr != hipSuccess) return static_cast<int>(attr);
  hipLaunchKernelGGL(kernel, dim3((a->n / 16 + NT - 1) / NT), dim3(64 * kWaves), lds_bytes,
                     static_cast<hipStream_t>(a->stream), static_cast<const uint16_t*>(a->a),
                     static_cast<const uint4*>(a->packed_w), static_cast<const uint16_t*>(a->scales),
                     static_cast<const uint8_t*>(a->zero_points), static_cast<uint16_t*>(a->c), a->m, a->n, a->k,
                     rows_log2);
  return static_cast<int>(hipGetLastError());
}

template <int BS, bool HAS_ZP, int DEPTH, int NT>
int launch_waves(const blkq4_gemm_args* a) {
  // eight waves split K when there is enough of it: each wave has less to convert after its last
  // load has arrived, and more of that work overlaps the loads of the other waves
  int rows_log2 = 0;
  while ((1 << rows_log2) < a->m) ++rows_log2;
  const size_t a_bytes = (((static_cast<size_t>(a->k) * 2) << rows_log2) + 1023) & ~size_t{1023};
  if (a->k >= 4096 && BLKQ4_SKINNY_WAVES16) {
    constexpr int kD = 2;
    if (a_bytes + 16 * NT * 64 * 4 * 4 <= kMaxLdsBytes) {
      return launch_kernel<BS, HAS_ZP, kD, NT, 1, 16, kRowsWholeInLds>(a, rows_log2);
    }
  }
  if (a->k >= 1024) {
    constexpr int kD = DEPTH > 4 ? 4 : DEPTH;
    if (a_bytes + 8 * NT * 64 * 4 * 4 <= kMaxLdsBytes) {
      return launch_kernel<BS, HAS_ZP, kD, NT, 1, 8, kRowsWholeInLds>(a, rows_log2);
    }
    return launch_kernel<BS, HAS_ZP, kD, NT, 1, 8, kRowsPerSlotInLds>(a, rows_log2);  // 8 * 4 * 4 KiB of rows
  }
  return launch_kernel<BS, HAS_ZP, DEPTH, NT, 1, 4, kRowsWholeInLds>(a, rows_log2);  // K < 1024: at most 32 KiB of rows
}

// 16 < M <= 16 * MT: one conversion of the weights feeds MT row tiles; eight waves, NT column tiles.
template <int BS, bool HAS_ZP, int MT, int NT>
int launch_rows_nt(const blkq4_gemm_args* a) {
  int rows_log2 = 0;
  while ((1 << rows_log2) < a->m) ++rows_log2;
  const size_t a_bytes = (((static_cast<size_t>(a->k) * 2) << rows_log2) + 1023) & ~size_t{1023};
  if (a_bytes + 8 * NT * MT * 64 * 4 * 4 <= kMaxLdsBytes) {
    return launch_kernel<BS, HAS_ZP, 2, NT, MT, 8, kRowsWholeInLds>(a, rows_log2);
  }
  // 8 waves x 2 slots x 8 KiB of rows fit for 32 rows; 64 rows go through registers
  return launch_kernel<BS, HAS_ZP, 2, NT, MT, 8, (MT <= 2) ? kRowsPerSlotInLds : kRowsInRegisters>(a, rows_log2);
}

template <int BS, bool HAS_ZP, int MT>
int launch_rows(const blkq4_gemm_args* a) {
  // every workgroup fetches all the rows; two column tiles per workgroup halve that traffic as soon as
  // there are enough tiles for every compute unit to get a workgroup all the same
  if (MT == 2 && a->n / 16 >= 512) return launch_rows_nt<BS, HAS_ZP, MT, (MT == 2) ? 2 : 1>(a);
  return launch_rows_nt<BS, HAS_ZP, MT, 1>(a);
}

template <int BS, bool HAS_ZP>
int launch_shape(const blkq4_gemm_args* a) {
  if (a->m > 32) return launch_rows<BS, HAS_ZP, 4>(a);
  if (a->m > 16) return launch_rows<BS, HAS_ZP, 2>(a);
  int nt, depth;
  choose_shape(a->m, a->n, &nt, &depth);
  if (nt == 1 && depth == 8) return launch_waves<BS, HAS_ZP, 8, 1>(a);
  if (nt == 1) return launch_waves<BS, HAS_ZP, 4, 1>(a);
  if (nt == 2) return launch_waves<BS, HAS_ZP, 4, 2>(a);
  return launch_waves<BS, HAS_ZP, 4, 3>(a);
}

template <int BS>
int launch_skinny(const blkq4_gemm_args* a) {
  return a->zero_points ? launch_shape<BS, true>(a) : launch_shape<BS, false>(a);
}

}  // namespace

extern "C" int blkq4_dev_skinny(const blkq4_gemm_args* a) {
  if (a->m < 1 || a->m > 64 || (a->n % 16) != 0 || (a->k % 64) != 0) return static_cast<int>(hipErrorInvalidValue);
  switch (a->block_size) {
    case 16: return launch_skinny<16>(a);
    case 32: return launch_skinny<32>(a);
    case 64: return launch_skinny<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}
