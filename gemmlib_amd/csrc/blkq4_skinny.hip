// Weight-streaming kernel for gfx950: decode GEMV, small-batch GEMM and, in row groups of 32, every M
// for which streaming the weights once per row group beats the tile kernel.
//
// The work is a stream over the packed weights (K*N/2 bytes plus scales and zero-points) that has to
// run at HBM speed; everything else is arranged so that the stream is requested as early and as
// deeply as possible and nothing serialises behind it:
//   - a workgroup of 4, 8 or 16 waves owns 16 * NT output columns, 16 * MT rows and the whole K range; the
//     waves split K in 128-deep slices, so every wave load is one 16-byte unit per lane: 16 columns x 4
//     consecutive k-units = four contiguous 256-byte runs of the packed layout.  With enough column tiles for
//     every wave the chip holds (and few rows), the waves do not split K: each has column tiles of its own,
//     streams all of K, and stores its sums itself: no barrier after the rows have arrived;
//   - a wave keeps the weight units, scales and zero-points of DEPTH slices in flight and refills a
//     slot as soon as it has consumed it (a slot past the end asks for valid units once more and is
//     multiplied by a zero scale, so the loop has no divergent loads);
//   - the activation rows are copied into LDS by asynchronous global_load_lds copies, laid out per 32-deep
//     unit as [unit][row][64 bytes] (16-byte chunks XOR-swizzled with bits 2..3 of the row so that a
//     fragment read is free of bank conflicts): once per workgroup, before the first weight request, when
//     all of K fits; otherwise per slot, private to the wave and requested right before the slot's
//     weights, so that a wave that has its weights has its rows and no barrier is needed;
//   - a lane dequantizes its (column, 32 k) of weights once and multiplies them with the matching 32 k of
//     MT tiles of 16 activation rows through v_mfma_f32_16x16x32_f16 (weights as the row operand: a lane
//     ends up with 4 consecutive output columns of one activation row per tile);
//   - the waves' partial tiles are summed through LDS (the space of the activation rows, once every wave
//     is done with them) by all threads: no atomics, no scratch buffer;
//   - more than 32 rows: the grid has one workgroup per (row group of 32, column group); the row groups
//     of a column group run on the same XCD, so the weights they share are fetched into its L2 once;
//   - many more column groups than the chip holds workgroups: the grid is as large as the chip holds and a
//     workgroup walks over several column groups, requesting the first slices of the next one while it
//     finishes the current one.
// Dequantization happens in registers (blkq4_dequant.h), for blocks along K (a scale per column and block
// row) and along N (a scale per k, shared by BS columns, in the reference's packed order); accumulation
// is fp32.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_dequant.h"
#include "blkq4_device.h"
#include "blkq4_launch.h"
#include "blkq4_gemm_common.h"

// This file is compiled twice: as it is for fp16, and through blkq4_skinny_bf16.hip, which defines
// BLKQ4_SKINNY_BF16 before including it, for bf16 activations, scales and outputs.
#ifdef BLKQ4_SKINNY_BF16
#define BLKQ4_SKINNY_ENTRY blkq4_dev_skinny_bf16
#else
#define BLKQ4_SKINNY_ENTRY blkq4_dev_skinny
#endif

namespace {

using namespace blkq4;

// the packed weights are read once per launch: non-temporal
__device__ __forceinline__ uint4 BLKQ4_W_LOAD(const uint4_t* p) {
  const uint4_t v = __builtin_nontemporal_load(p);
  return make_uint4(v[0], v[1], v[2], v[3]);
}

#ifdef BLKQ4_SKINNY_BF16
constexpr bool kBF = true;
#else
constexpr bool kBF = false;
#endif

// Where a wave finds its activation fragments.
constexpr int kRowsWholeInLds = 1;   // all rows, all of K, staged once per workgroup
constexpr int kRowsPerSlotInLds = 2; // 16 * MT rows x 128 k staged per slot, private to the wave

template <int BS, int NT, int MT, int AM, bool ROW>
struct Slot {
  static constexpr int kMeta = (BS == 16) ? 2 : 1;  // quantization blocks inside one 32-deep unit
  uint4 w[NT];
  uint32_t sc[NT][ROW ? 1 : kMeta];
  uint32_t zp[NT][ROW ? 1 : kMeta];
  // blocks along N: a scale and a zero-point per k, 32 of each for the lane's unit, in the packed order of
  // the meta data (two 16-row groups of 32 + 16 bytes)
  uint4 rs[ROW ? NT : 1][4];
  uint4 rz[ROW ? NT : 1][2];
};

// kWaves: waves of the workgroup.  kSplit: how many of them split K: all (kSplit = kWaves; their partial tiles
// are summed through LDS) or none (kSplit = 1: every wave has NT column tiles of its own and all of K).
// DEPTH: k slices (128 deep) a wave keeps in flight.  NT: 16-column tiles per wave that share one activation
// operand.  MT: 16-row tiles of activations (M <= 16 * MT) that share one conversion of the weights.
// AM: where the activation rows are (see above).  kRowsWholeInLds: rows_log2 = log2 of the number of rows kept
// in LDS, a power of two >= M; kRowsPerSlotInLds: kWaves * DEPTH * 16 * MT * 256 bytes of slots.
// kRefill: false for one column group (NT * kWaves / kSplit tiles) per workgroup; true for workgroups that walk
// over the column groups cg, cg + cg_stride, ... (the partial tiles then live at red_offset, behind the rows,
// which stay) and for waves that do not split K.
// ROW: quantization blocks run along N (one k, BS columns); S and Z are then in the packed order
// described in blkq4_device.h and the lane's column group decides which 64 + 32 bytes it fetches per unit.
// (BF repeats kBF so that the two compilations' kernels carry different names in a trace)
template <int BS, bool HAS_ZP, int DEPTH, int NT, int MT, int kWaves, int AM, bool ROW, bool kRefill, int kSplit, bool BF = kBF>
__global__ __launch_bounds__(64 * kWaves) void skinny_mfma_kernel(const uint16_t* __restrict__ A,
                                                               const uint4* __restrict__ W,
                                                               const uint16_t* __restrict__ S,
                                                               const uint8_t* __restrict__ Z,
                                                               uint16_t* __restrict__ C,
                                                               const uint16_t* __restrict__ bias, int M_total, int N,
                                                               int K, int rows_log2, int row_groups,
                                                               int cg_stride, uint32_t red_offset) {
  constexpr int kMeta = Slot<BS, NT, MT, AM, ROW>::kMeta;
  constexpr bool A_LDS = AM == kRowsWholeInLds;
  // weight / scale / zero-point requests of a slot
  constexpr int kLoads = ROW ? NT * (1 + 4 + (HAS_ZP ? 2 : 0)) : NT * (1 + kMeta * (HAS_ZP ? 2 : 1));
  constexpr int kSlotRows = 16 * MT;                           // kRowsPerSlotInLds: rows staged per slot
  constexpr int kSlotBytes = kSlotRows * 256;
  // the partial tiles of the sums across waves reuse the LDS of the activation rows (red_offset = 0) or, when
  // the workgroup goes on to another column group and needs the rows again, lie behind them
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  float* red = reinterpret_cast<float*>(smem + red_offset);
  const uint8_t* a_lds = smem;

  // Workgroup -> (row group of 16 * MT rows, group of NT column tiles).  Consecutive workgroups go to
  // consecutive XCDs (8 of them).  An XCD's workgroups take, in this order: the row groups of a column
  // group (they share its weights), then the next of four neighbouring column groups (they share the 128-byte
  // lines of the scale and zero-point rows, and their weights are contiguous), so that what is shared is
  // fetched into that XCD's L2 once.
  static_assert(kSplit == kWaves || kSplit == 1, "the waves split K among all of them or not at all");
  constexpr int kTileWaves = kWaves / kSplit;  // waves (or sets of waves) with column tiles of their own
  const int col_groups = ((N >> 4) + NT * kTileWaves - 1) / (NT * kTileWaves);
  const int wg = blockIdx.x;
  const int q = wg >> 3;
  const int rg = q % row_groups;
  int cg = 4 * ((wg & 7) + 8 * ((q / row_groups) >> 2)) + ((q / row_groups) & 3);
  if (cg >= col_groups) return;  // the grid is rounded up to whole groups of 32 column groups
  const int m0 = rg * (16 * MT);
  const int M = min(16 * MT, M_total - m0);
  A += static_cast<size_t>(m0) * K;
  C += static_cast<size_t>(m0) * N;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int nl = lane & 15;  // column inside the tile (weights operand) / activation row (other operand)
  const int g = lane >> 4;   // which of the 4 k-units of a slice
  const int tiles = N >> 4;
  const DequantMasks masks = DequantMasks::make();
  const int units = K >> 5;             // 32-deep units
  const int slices = (units + 3) >> 2;  // 128-deep slices (the last one may be half full)
  const int ws = (kSplit == 1) ? 0 : wave;  // this wave's slices are ws, ws + kSplit, ...
  const int wt = (kSplit == 1) ? wave : 0;  // and its column tiles the wt-th NT of the column group
  const int my_slices = (slices - ws + kSplit - 1) / kSplit;

  const int wrap_mask = (1 << (31 - __builtin_clz(units))) - 1;  // any index & wrap_mask is < units

  // Addresses are a wave-uniform 64-bit part (slice and column tile: scalar arithmetic) plus a 32-bit part
  // of the lane that never changes: (k-unit of the slice g, column nl).  Only in the last slice, when it has
  // rem < 4 units, the lanes past the end ask for unit g % rem instead (their scales are zeroed when the slot
  // is consumed), and a slot past the wave's last slice asks for the last slice once more.
  constexpr int kBlocksPerSlice = (BS == 64) ? 2 : (BS == 32) ? 4 : 8;
  const int rem = units & 3;
  const int last_slice = slices - 1;
  const int g_alt = (rem == 0) ? g : (rem == 1) ? 0 : (rem == 2) ? (g & 1) : (g == 3 ? 0 : g);
  uint32_t w_lane[2], m_lane[2], a_lane[2];  // [1]: in a last slice that is not full
#pragma unroll
  for (int v = 0; v < 2; ++v) {
    const int gx = v ? g_alt : g;
    w_lane[v] = static_cast<uint32_t>(gx * N + nl) * 16u;  // bytes into the packed weights
    // elements into the scales and the zero-points
    m_lane[v] = ROW ? static_cast<uint32_t>(gx * 32)
                    : static_cast<uint32_t>(((BS == 64) ? (gx >> 1) : (BS == 32) ? gx : 2 * gx) * N + nl);
  }
  const uint32_t ok_last = (rem == 0 || g < rem) ? 0xffffffffu : 0u;

  float4_t acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = float4_t{0.f, 0.f, 0.f, 0.f};
  Slot<BS, NT, MT, AM, ROW> slot[DEPTH];

  // Rows to LDS: copy q fills LDS bytes [1024 q, 1024 q + 1024) of the [unit][row][64 B] layout, lane l
  // the 16 bytes at 16 l.  They are requested before anything else, so every later wait covers them.
  uint32_t a_rd = 0;  // LDS byte offset of this lane's row inside a unit, chunk 0
  uint32_t a_swz = 0;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                            (__attribute__((address_space(3))) uint8_t*)(smem)));
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
  a_lane[0] = (static_cast<uint32_t>(g) << (6 + rows_log2)) + a_rd;
  a_lane[1] = (static_cast<uint32_t>(g_alt) << (6 + rows_log2)) + a_rd;
  // a slot past the end asks for valid units (so every slot always issues the same loads); its scales are
  // zeroed when the slot is consumed (not here: that would wait for the load right after requesting it),
  // which makes it contribute exactly 0
#define BLKQ4_LOAD_SLOT(dst_, d_, cg_, slice_, keep_)                                                \
  {                                                                                            \
    const int sl_ = min((slice_), last_slice);                                                 \
    const bool alt_ = rem != 0 && sl_ == last_slice;                                           \
    const uint32_t wl_ = alt_ ? w_lane[1] : w_lane[0];                                         \
    const uint32_t ml_ = alt_ ? m_lane[1] : m_lane[0];                                         \
    const size_t keep64_ = static_cast<size_t>(static_cast<long long>(keep_));                 \
    if (AM == kRowsPerSlotInLds) {                                                             \
      /* copy q: LDS bytes [1024 q, 1024 q + 1024) of the slot, lane l the 16 bytes at 16 l; */ \
      /* requested before the slot's weights, so whoever has the weights has the rows        */ \
      _Pragma("unroll") for (int q = 0; q < 4 * MT; ++q) {                                     \
        const int rr_ = 16 * q + (lane >> 2);            /* (unit, row) index inside the slot */ \
        const int u_ = 4 * sl_ + rr_ / kSlotRows;                                              \
        const int ug_ = (u_ < units) ? u_ : (u_ & wrap_mask);                                  \
        const int row_ = rr_ % kSlotRows;                                                      \
        const int chunk_ = (lane & 3) ^ ((row_ >> 2) & 3);                                     \
        async_copy_16(__builtin_amdgcn_readfirstlane(lds0 + (wave * DEPTH + (d_)) * kSlotBytes + q * 1024), A, \
                      (static_cast<uint32_t>(min(row_, M - 1)) * K + ug_ * 32 + chunk_ * 8) * 2); \
      }                                                                                        \
    }                                                                                          \
    _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                           \
      /* tile t of column group cg_; a tile past the end (last column group only, when the group's */ \
      /* tile count does not divide the number of tiles) re-reads the group's first tile and is    */ \
      /* not stored                                                                                */ \
      const int tile_ = ((cg_) * kTileWaves + wt) * NT + t;                                    \
      const int tu_ = (tile_ < tiles) ? tile_ : (cg_) * (kTileWaves * NT);                     \
      const size_t wu_ = ((static_cast<size_t>(4 * sl_) * N + tu_ * 16) * 16) & keep64_;       \
      (dst_).w[t] = BLKQ4_W_LOAD(reinterpret_cast<const uint4_t*>(reinterpret_cast<const char*>(W) + wu_ + wl_)); \
      if (ROW) {                                                                               \
        const size_t mu_ = (static_cast<size_t>(tu_ * 16 / BS) * K + sl_ * 128) & keep64_;     \
        const char* sp_ = reinterpret_cast<const char*>(S) + mu_ * 2 + ml_ * 2;                \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                        \
          (dst_).rs[ROW ? t : 0][q] = reinterpret_cast<const uint4*>(sp_)[q];                  \
        }                                                                                      \
        if (HAS_ZP) {                                                                          \
          const char* zp_ = reinterpret_cast<const char*>(Z) + mu_ + ml_;                      \
          _Pragma("unroll") for (int q = 0; q < 2; ++q) {                                      \
            (dst_).rz[ROW ? t : 0][q] = reinterpret_cast<const uint4*>(zp_)[q];                \
          }                                                                                    \
        }                                                                                      \
      } else {                                                                                 \
        _Pragma("unroll") for (int q = 0; q < kMeta; ++q) {                                    \
          const size_t mu_ = (static_cast<size_t>(kBlocksPerSlice * sl_ + q) * N + tu_ * 16) & keep64_; \
          (dst_).sc[t][ROW ? 0 : q] =                                                          \
              *reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(S) + mu_ * 2 + ml_ * 2); \
          (dst_).zp[t][ROW ? 0 : q] =                                                          \
              HAS_ZP ? static_cast<uint32_t>(*(reinterpret_cast<const uint8_t*>(Z) + mu_ + ml_)) : 8u; \
        }                                                                                      \
      }                                                                                        \
    }                                                                                          \
  }
  // A wave's local slices are li = 0 .. my_slices - 1 (slice ws + kSplit * li), taken DEPTH at a time; the
  // slots past my_slices in the last round ask for the last slice once more and are zeroed.
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) BLKQ4_LOAD_SLOT(slot[d], d, cg, ws + kSplit * d, -1);
  if (A_LDS) {
    // everything but the requests of the ring just issued has landed: this wave's share of the rows
    constexpr int kRing = DEPTH * kLoads;
    wait_vmcnt<(kRing < 63 ? kRing : 63)>();
    __syncthreads();
  }

  // Sums the waves' partial tiles of column group `cgx` through LDS and stores the result: every wave is
  // done with the rows (when the partial tiles share their space) and with reading the partial tiles of
  // the column group before.
  auto flush = [&](int cgx) {
    if (kSplit == 1) {
      // a wave has whole sums: lane L holds columns 4 (L >> 4) .. + 3 of tile t, row 16 mt + (L & 15)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const int tile = (cgx * kTileWaves + wt) * NT + t;
          const int row = 16 * mt + nl;
          if (row < M && tile < tiles) {
            uint32_t lo = float_to_bits<kBF>(acc[t][mt][0]) | (float_to_bits<kBF>(acc[t][mt][1]) << 16);
            uint32_t hi = float_to_bits<kBF>(acc[t][mt][2]) | (float_to_bits<kBF>(acc[t][mt][3]) << 16);
            if (bias != nullptr) {
              const uint2 b = *reinterpret_cast<const uint2*>(bias + tile * 16 + 4 * g);
              lo = add_bias_pair_t<kBF>(lo, b.x);
              hi = add_bias_pair_t<kBF>(hi, b.y);
            }
            *reinterpret_cast<uint2*>(C + static_cast<size_t>(row) * N + tile * 16 + 4 * g) = make_uint2(lo, hi);
          }
          acc[t][mt] = float4_t{0.f, 0.f, 0.f, 0.f};
        }
      return;
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int e = 0; e < 4; ++e) red[(((wave * NT + t) * MT + mt) * 64 + lane) * 4 + e] = acc[t][mt][e];
        acc[t][mt] = float4_t{0.f, 0.f, 0.f, 0.f};
      }
    __syncthreads();
    // value v = (tile t, row tile mt, lane L, element e) of the partial tiles: output row 16 mt + (L & 15),
    // column 4 (L >> 4) + e of tile t; every thread sums a few of them over the waves
    for (int v = tid; v < NT * MT * 256; v += 64 * kWaves) {
      float r = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) r += red[w * (NT * MT * 256) + v];
      const int t = v / (MT * 256), mt = (v >> 8) % MT, L = (v >> 2) & 63, e = v & 3;
      const int row = 16 * mt + (L & 15);
      if (row < M && cgx * NT + t < tiles) {
        const int col = cgx * (16 * NT) + 16 * t + 4 * (L >> 4) + e;
        uint32_t h = float_to_bits<kBF>(r);
        if (bias != nullptr) h = add_bias_bits_t<kBF>(h, bias[col]);
        C[static_cast<size_t>(row) * N + col] = static_cast<uint16_t>(h);
      }
    }
  };

  // converts slot d, which holds local slice li, and multiplies it with the rows
  auto consume = [&](int d, int li) {
    const Slot<BS, NT, MT, AM, ROW>& cur = slot[d];
    const int slice = ws + kSplit * li;
    const int sl = min(slice, last_slice);
    const bool alt = rem != 0 && sl == last_slice;
    const uint32_t full = (slice < last_slice || (slice == last_slice && rem == 0)) ? 0xffffffffu : 0u;  // uniform
    const uint32_t okm = full | ((slice == last_slice) ? ok_last : 0u);
      uint4 af[MT][4];  // eight 16-bit activations each
      if (A_LDS) {
        const uint8_t* ap = a_lds + (static_cast<uint32_t>(4 * sl) << (6 + rows_log2)) + (alt ? a_lane[1] : a_lane[0]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            af[mt][j] = *reinterpret_cast<const uint4*>(ap + mt * 1024 + ((j ^ a_swz) * 16));
          }
      } else {
        // the rows of this slot were requested before its weights
        // (in-order completion: once one of the slot's weight words is here, so are the rows)
        asm volatile("" ::: "memory");
        const uint8_t* ap = a_lds + a_rd + d * kSlotBytes;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            af[mt][j] = *reinterpret_cast<const uint4*>(ap + mt * 1024 + ((j ^ a_swz) * 16));
          }
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const uint32_t words[4] = {cur.w[t].x, cur.w[t].y, cur.w[t].z, cur.w[t].w};
        if constexpr (kBF && !ROW) {
          Bf16Consts bc[kMeta];
#pragma unroll
          for (int q = 0; q < kMeta; ++q) bc[q] = make_bf16_consts(cur.sc[t][q] & okm, cur.zp[t][q]);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const bf16x8_t wf = dequant_word_bf16(words[j], bc[(kMeta == 2) ? (j >> 1) : 0], masks);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, as_bf16x8(af[mt][j]), acc[t][mt], 0, 0, 0);
            }
          }
          continue;
        }
        DequantConsts dc[kMeta];
        if (!ROW) {
#pragma unroll
          for (int q = 0; q < kMeta; ++q) dc[q] = make_dequant_consts(cur.sc[t][ROW ? 0 : q] & okm, cur.zp[t][ROW ? 0 : q]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t y = words[j] >> 8;
          half2_t p[4];
          if (ROW) {
            // word j is rows 8 hh .. 8 hh + 7 of 16-row group j / 2 of the unit: pair i has its scales in
            // 32-bit word 2 i + hh of the group and its zero-points in byte pair hh of word i
            constexpr int kRowSlot = ROW ? 1 : 0;
            const int hh = j & 1;
            const uint4 s0 = cur.rs[kRowSlot * t][2 * (j >> 1)], s1 = cur.rs[kRowSlot * t][2 * (j >> 1) + 1];
            const uint32_t sw[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
            const uint4 zq = HAS_ZP ? cur.rz[kRowSlot * t][j >> 1] : make_uint4(0, 0, 0, 0);
            const uint32_t zw[4] = {zq.x, zq.y, zq.z, zq.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const uint32_t zpair = HAS_ZP ? ((zw[i] >> (8 * hh)) & 0x00ff00ffu) : 0x00080008u;
              const uint32_t src = (i >= 2) ? y : words[j];
              const half2_t s2 = as_half2(sw[2 * i + hh] & okm);
              // q - zp of the pair, exact
              const half2_t d = ((i & 1) == 0)
                  ? as_half2((src & masks.lo_mask) | masks.magic_1024) + as_half2(0xE400E400u | zpair)
                  : as_half2((src & masks.hi_mask) | masks.magic_64) + as_half2(0xD400D400u | (zpair << 4));
              if constexpr (kBF) {
                p[i] = as_half2(row_pair_bf16(d, sw[2 * i + hh] & okm));  // a bf16 pair in the same register
              } else {
                p[i] = d * s2;
              }
            }
          } else {
            const DequantConsts& c = dc[(kMeta == 2) ? (j >> 1) : 0];
            p[0] = dequant_pair(words[j], 0, c, masks);
            p[1] = dequant_pair(words[j], 1, c, masks);
            p[2] = dequant_pair(y, 2, c, masks);
            p[3] = dequant_pair(y, 3, c, masks);
          }
          half8_t wf;
          wf[0] = p[0][0]; wf[1] = p[0][1]; wf[2] = p[1][0]; wf[3] = p[1][1];
          wf[4] = p[2][0]; wf[5] = p[2][1]; wf[6] = p[3][0]; wf[7] = p[3][1];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            if constexpr (kBF) {
              acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, wf), as_bf16x8(af[mt][j]),
                                                                  acc[t][mt], 0, 0, 0);
            } else {
              acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, as_half8(af[mt][j]), acc[t][mt], 0, 0, 0);
            }
          }
        }
      }
  };

  if (!kRefill) {
    // one column group per workgroup: a slot is refilled only while the wave has slices left
    for (int i0 = 0; i0 < my_slices; i0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        consume(d, i0 + d);
        if (i0 + DEPTH < my_slices) BLKQ4_LOAD_SLOT(slot[d], d, cg, ws + kSplit * (i0 + d + DEPTH), -1);
      }
    }
    flush(cg);
    return;
  }
  // A workgroup that walks over several column groups.  While a round is consumed, every slot is refilled
  // with the same slot of the round after it: the next one of this column group, else the first one of the
  // workgroup's next column group, else (nothing left) every lane asks for one and the same unit, unused.  So
  // every round issues the same requests in the same order and the compiler's waits are exact; behind a
  // conditional refill it waits for everything outstanding, the refills just issued included.
  const int rounds = (my_slices + DEPTH - 1) / DEPTH;
  while (cg < col_groups) {
    const int next_cg = cg + cg_stride;
    for (int r = 0; r < rounds; ++r) {
      const int i0 = r * DEPTH;
      const bool more = r + 1 < rounds;
      const bool next_group = !more && next_cg < col_groups;
      const int ld_cg = next_group ? next_cg : cg;
      const int ld_i0 = more ? i0 + DEPTH : next_group ? 0 : i0;
      const int keep = (more || next_group) ? -1 : 0;  // 0: every lane asks for the very first unit instead
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        consume(d, i0 + d);
        BLKQ4_LOAD_SLOT(slot[d], d, ld_cg, ws + kSplit * (ld_i0 + d), keep);
        // the refill is requested here, not together with the others at the end of the round
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    flush(cg);
    cg = next_cg;
  }
#undef BLKQ4_LOAD_SLOT
}

// The kernel is bound by instruction issue as much as by the weight stream, so what matters is how
// evenly the workgroups fill the 256 compute units: with T column tiles per workgroup the busiest
// unit works through ceil(workgroups / 256) * T tiles.  Wider workgroups also re-read the activation
// rows less often, which weighs more the more rows there are.
constexpr size_t kMaxLdsBytes = 160 * 1024;
constexpr int kStreamingMaxRows = 1024;
constexpr int kComputeUnits = 256;
constexpr int kPersistentFactor = 2;  // column groups per workgroup from which on workgroups walk


void choose_shape(int m, int n, int k, int* nt, int* depth) {
  const int tiles = n / 16;
  // cost of fetching the activation rows relative to one tile's work: small while they are staged once per
  // workgroup; when K is too long for that they are fetched again for every column group, 16 rows x 2 bytes
  // against a tile's 16 columns x 1/2 byte per k
  int rows = 1;
  while (rows < m) rows *= 2;
  const bool rows_fit = static_cast<size_t>(rows) * static_cast<size_t>(k) * 2 <= kMaxLdsBytes;
  const float a_weight = !rows_fit ? static_cast<float>(rows) / 4.0f : (m > 4) ? 0.2f : 0.05f;
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

// Raises a kernel's dynamic-LDS limit, once per kernel instantiation and device.
template <auto kKernel>
hipError_t raise_lds_limit() {
  return raise_lds_limit_once(reinterpret_cast<const void*>(kKernel), kMaxLdsBytes, &lds_limit_flags<kKernel>());
}

// One kernel instantiation: raises its dynamic-LDS limit, then launches `row_groups` row groups of
// 16 * MT rows each.
template <int BS, bool HAS_ZP, bool ROW, int DEPTH, int NT, int MT, int kWaves, int AM, int kSplit = kWaves>
int launch_kernel(const blkq4_gemm_args* a, int rows_log2, int row_groups = 1) {
  constexpr size_t kRedBytes = (kSplit == 1) ? 0 : static_cast<size_t>(kWaves) * NT * MT * 64 * 4 * 4;
  constexpr size_t kPerSlotBytes = static_cast<size_t>(kWaves) * DEPTH * 16 * MT * 256;
  static_assert(kRedBytes <= kMaxLdsBytes, "partial tiles do not fit in LDS");
  static_assert(AM != kRowsPerSlotInLds || kPerSlotBytes <= kMaxLdsBytes, "slots do not fit in LDS");
  // the rows are copied 1 KiB at a time; the partial tiles of the reduction reuse their space
  const size_t a_bytes = AM == kRowsWholeInLds ? ((((static_cast<size_t>(a->k) * 2) << rows_log2) + 1023) & ~size_t{1023})
                         : AM == kRowsPerSlotInLds ? kPerSlotBytes
                                                   : 0;
  constexpr int kGroupTiles = NT * (kWaves / kSplit);
  const int col_groups = (a->n / 16 + kGroupTiles - 1) / kGroupTiles;
  int cg_stride = (col_groups + 31) / 32 * 32;  // one column group per workgroup
  size_t lds_bytes = a_bytes > kRedBytes ? a_bytes : kRedBytes;
  size_t red_offset = 0;
  // Many more workgroups than the chip holds at once: a workgroup then walks over several column groups
  // (cg, cg + cg_stride, ...) and requests the first slices of the next one while it finishes the current
  // one, so only the first column group of a workgroup waits for its weights with nothing else to do.
  // The partial tiles then get LDS of their own: the rows stay where they are for the next column group.
  // (not the sixteen-wave kernel for blocks along N: its walking variant does not fit in 128 registers)
  constexpr bool kMayWalk = !(ROW && kWaves == 16);
  if (kMayWalk && a_bytes + kRedBytes <= kMaxLdsBytes) {
    const int by_lds = static_cast<int>(kMaxLdsBytes / (a_bytes + kRedBytes));
    const int by_waves = 32 / kWaves;
    const int resident = kComputeUnits * (by_lds < by_waves ? by_lds : by_waves);
    int stride = (resident / row_groups) / 32 * 32;
    if (stride < 32) stride = 32;
    if (cg_stride >= kPersistentFactor * stride) {
      cg_stride = stride;
      lds_bytes = a_bytes + kRedBytes;
      red_offset = a_bytes;
    }
  }
  const unsigned grid = static_cast<unsigned>(cg_stride) * static_cast<unsigned>(row_groups);
  // workgroups walk over several column groups, or waves stream all of K by themselves
  const bool refill = cg_stride < col_groups || kSplit == 1;
  auto launch = [&](auto* kernel, hipError_t attr) {
    if (attr != hipSuccess) return static_cast<int>(attr);
    // the launch's own status: a sticky error of an earlier, unrelated call stays where it is
    return static_cast<int>(launch_status(kernel, dim3(grid), dim3(64 * kWaves), lds_bytes, a->stream,
                                          static_cast<const uint16_t*>(a->a), static_cast<const uint4*>(a->packed_w),
                                          static_cast<const uint16_t*>(a->scales),
                                          static_cast<const uint8_t*>(a->zero_points), static_cast<uint16_t*>(a->c),
                                          static_cast<const uint16_t*>(a->bias), a->m, a->n, a->k, rows_log2,
                                          row_groups, cg_stride, static_cast<uint32_t>(red_offset)));
  };
  if (refill) {
    constexpr auto kernel = skinny_mfma_kernel<BS, HAS_ZP, DEPTH, NT, MT, kWaves, AM, ROW, true, kSplit>;
    return launch(kernel, raise_lds_limit<kernel>());
  }
  if constexpr (kSplit == 1) {
    return static_cast<int>(hipErrorInvalidValue);  // not reached
  } else {
    constexpr auto kernel = skinny_mfma_kernel<BS, HAS_ZP, DEPTH, NT, MT, kWaves, AM, ROW, false, kSplit>;
    return launch(kernel, raise_lds_limit<kernel>());
  }
}

// Slices that `waves` waves with rings of `depth` slices request for one column group: every wave asks for
// whole rings, also when it has fewer slices left.
int requested_slices(int k, int waves, int depth) {
  const int slices = (k / 32 + 3) / 4;
  int total = 0;
  for (int w = 0; w < waves; ++w) {
    const int mine = (slices - w + waves - 1) / waves;
    total += (mine + depth - 1) / depth * depth;
  }
  return total;
}

// M <= 16, enough column tiles to give every wave the chip can hold one of its own, and rows small enough for
// several workgroups per compute unit: the waves do not split K, each streams all of K for its own tile:
// no sums across waves, no barriers, and a ring that stays full from the first slice to the last.
template <int BS, bool HAS_ZP, bool ROW>
bool launch_independent_waves(const blkq4_gemm_args* a, int* status) {
  int rows_log2 = 0;
  while ((1 << rows_log2) < a->m) ++rows_log2;
  const size_t a_bytes = (((static_cast<size_t>(a->k) * 2) << rows_log2) + 1023) & ~size_t{1023};
  // measured break-even against workgroups that split K and walk (blocks along N gain more: their sixteen-wave
  // kernel has no walking variant)
  constexpr size_t kIndependentMaxRowBytes = (ROW ? 32 : 16) * 1024;
  // (from 832 tiles on when K is no multiple of what the splitting waves' rings hold, which then ask for a
  // fifth more slices than there are: K = 5120, N = 13824: 14.5 -> 12.7 us)
  const int slices = (a->k / 32 + 3) / 4;
  const bool rings_fit_k = 5 * requested_slices(a->k, 16, 2) < 6 * slices || 5 * requested_slices(a->k, 8, 4) < 6 * slices;
  const int kIndependentMinTiles = ROW ? 896 : rings_fit_k ? 2000 : 832;
  if (a->n / 16 < kIndependentMinTiles || a_bytes > kIndependentMaxRowBytes ||
      (reinterpret_cast<uintptr_t>(a->c) & 7u) != 0) {
    return false;
  }
  // four slices in flight per wave: with eight the kernel needs 90 registers and a SIMD holds five waves
  // instead of seven, which costs more than the deeper ring gains (52 against 55 us at N = 128256)
  *status = launch_kernel<BS, HAS_ZP, ROW, 4, 1, 1, 4, kRowsWholeInLds, 1>(a, rows_log2);
  return true;
}

// M <= 16: one row tile; the waves of a workgroup split K.
template <int BS, bool HAS_ZP, bool ROW, int DEPTH, int NT>
int launch_waves(const blkq4_gemm_args* a) {
  int rows_log2 = 0;
  while ((1 << rows_log2) < a->m) ++rows_log2;
  const size_t a_bytes = (((static_cast<size_t>(a->k) * 2) << rows_log2) + 1023) & ~size_t{1023};
  // sixteen waves when there is enough K: each wave has less to convert after its last load has arrived,
  // and more of that work overlaps the loads of the other waves.  With more workgroups than compute units,
  // eight waves: smaller workgroups fill the units more evenly (M = 1, K = 4096, N = 14336: 11.4 -> 9.5 us),
  // unless their rings would ask for many more slices than K has.
  if (a->k >= 4096 && a_bytes <= kMaxLdsBytes) {
    constexpr int kD8 = DEPTH > 4 ? 4 : DEPTH;
    const int col_groups = (a->n / 16 + NT - 1) / NT;
    if (!ROW && col_groups > kComputeUnits &&
        20 * requested_slices(a->k, 8, kD8) <= 21 * requested_slices(a->k, 16, 2)) {
      return launch_kernel<BS, HAS_ZP, ROW, kD8, NT, 1, 8, kRowsWholeInLds>(a, rows_log2);
    }
    return launch_kernel<BS, HAS_ZP, ROW, 2, NT, 1, 16, kRowsWholeInLds>(a, rows_log2);
  }
  if (a->k >= 1024) {
    constexpr int kD = DEPTH > 4 ? 4 : DEPTH;
    if (a_bytes <= kMaxLdsBytes) return launch_kernel<BS, HAS_ZP, ROW, kD, NT, 1, 8, kRowsWholeInLds>(a, rows_log2);
    return launch_kernel<BS, HAS_ZP, ROW, kD, NT, 1, 8, kRowsPerSlotInLds>(a, rows_log2);  // 8 * 4 * 4 KiB of rows
  }
  return launch_kernel<BS, HAS_ZP, ROW, DEPTH, NT, 1, 4, kRowsWholeInLds>(a, rows_log2);  // K < 1024: at most 32 KiB of rows
}

// M > 16: row groups of 32 rows (two row tiles share one conversion of the weights), NT column tiles per
// workgroup, eight waves.
template <int BS, bool HAS_ZP, bool ROW, int NT>
int launch_rows(const blkq4_gemm_args* a, int row_groups) {
  const size_t a_bytes = static_cast<size_t>(a->k) * 2 * 32;
  if (a_bytes <= kMaxLdsBytes) return launch_kernel<BS, HAS_ZP, ROW, 2, NT, 2, 8, kRowsWholeInLds>(a, 5, row_groups);
  return launch_kernel<BS, HAS_ZP, ROW, 2, NT, 2, 8, kRowsPerSlotInLds>(a, 5, row_groups);  // 8 * 2 * 8 KiB of rows
}

template <int BS, bool HAS_ZP, bool ROW>
int launch_shape(const blkq4_gemm_args* a) {
  if (a->m > 16) {
    // Every workgroup fetches the 32 rows of its group for all of K, so wide workgroups (more column tiles)
    // mean less activation traffic; but there should be a workgroup for most compute units (measured: four
    // tiles per workgroup from 160 workgroups of four on, two from 160 of two on).
    const int row_groups = (a->m + 31) / 32;
    const long tiles = static_cast<long>(a->n / 16) * row_groups;
    if (tiles >= 640) return launch_rows<BS, HAS_ZP, ROW, ROW ? 1 : 4>(a, row_groups);
    if (tiles >= 320) return launch_rows<BS, HAS_ZP, ROW, ROW ? 1 : 2>(a, row_groups);
    return launch_rows<BS, HAS_ZP, ROW, 1>(a, row_groups);
  }
  int status;
  if (launch_independent_waves<BS, HAS_ZP, ROW>(a, &status)) return status;
  if constexpr (!ROW) {
    // Wide N and more than four rows, or K too long for the rows to stay in LDS: the rows are staged per slice,
    // a workgroup takes four column tiles (the rows are fetched again for every column group) and a wave keeps
    // two slices in flight, so that the slots are small enough for several workgroups per compute unit: eight
    // waves from 832 column tiles on, four from 1536 on.  Measured against every other shape of workgroup:
    // M = 16, K = 8192: N = 14336 24.3 -> 17.6 us, N = 28672 43.1 -> 34.1 us; rows that would fit (M = 16,
    // K = 4096, N = 14336: 13.2 -> 11.1 us) gain less or nothing, never lose more than 3 %.
    int rows_log2 = 0;
    while ((1 << rows_log2) < a->m) ++rows_log2;
    const bool rows_fit = ((static_cast<size_t>(a->k) * 2) << rows_log2) <= kMaxLdsBytes;
    const int tiles = a->n / 16;
    if ((!rows_fit || a->m > 4) && a->k >= 1024) {
      if (tiles >= 1536) return launch_kernel<BS, HAS_ZP, ROW, 2, 4, 1, 4, kRowsPerSlotInLds>(a, rows_log2);
      if (tiles >= 832) return launch_kernel<BS, HAS_ZP, ROW, 2, 4, 1, 8, kRowsPerSlotInLds>(a, rows_log2);
    }
  }
  int nt, depth;
  choose_shape(a->m, a->n, a->k, &nt, &depth);
  if (ROW) {
    // blocks along N: 28 registers of packed weights, scales and zero-points per slot and tile, so one tile
    return (depth == 8) ? launch_waves<BS, HAS_ZP, ROW, 8, 1>(a) : launch_waves<BS, HAS_ZP, ROW, 4, 1>(a);
  }
  if (nt == 1 && depth == 8) return launch_waves<BS, HAS_ZP, ROW, 8, 1>(a);
  if (nt == 1) return launch_waves<BS, HAS_ZP, ROW, 4, 1>(a);
  if (nt == 2) return launch_waves<BS, HAS_ZP, ROW, 4, ROW ? 1 : 2>(a);
  return launch_waves<BS, HAS_ZP, ROW, 4, ROW ? 1 : 3>(a);
}

template <int BS>
int launch_skinny(const blkq4_gemm_args* a) {
  if (a->column_wise) return a->zero_points ? launch_shape<BS, true, false>(a) : launch_shape<BS, false, false>(a);
  return a->zero_points ? launch_shape<BS, true, true>(a) : launch_shape<BS, false, true>(a);
}

}  // namespace

extern "C" int BLKQ4_SKINNY_ENTRY(const blkq4_gemm_args* a) {
  if (a->m < 1 || a->m > kStreamingMaxRows || (a->n % 16) != 0 || (a->k % 64) != 0) return static_cast<int>(hipErrorInvalidValue);
  if (a->n > (1 << 26)) return static_cast<int>(hipErrorInvalidValue);  // a lane's offset inside a slice (up to 8 n rows of 16 bytes) is 32 bits wide
  if (!a->column_wise) {
    // blocks along N: a 16-column tile lies inside one block, and the meta data are fetched 16 bytes at a time
    if ((a->n % a->block_size) != 0 || (reinterpret_cast<uintptr_t>(a->scales) & 15u) != 0 ||
        (reinterpret_cast<uintptr_t>(a->zero_points) & 15u) != 0) {
      return static_cast<int>(hipErrorInvalidValue);
    }
  }
  switch (a->block_size) {
    case 16: return launch_skinny<16>(a);
    case 32: return launch_skinny<32>(a);
    case 64: return launch_skinny<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}
