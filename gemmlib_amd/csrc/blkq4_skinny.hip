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
//     fragment read is free of bank conflicts).  When all of K fits, a wave stages the rows of the slices it
//     will convert itself, once, before its first weight request; otherwise per slot, right before the slot's
//     weights.  Either way the rows a wave reads are rows it requested itself before the weights it multiplies
//     them with, requests complete in order, and no barrier is needed: a wave that has its weights has its rows.
//     (Waves that do not split K share out the copies of all rows and meet at one barrier.)
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

#include "blkq4_choose.h"
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

// Loads of the streamed operands at a byte offset from a base, for two kinds of base: the kernel's own
// restrict-qualified pointers (generic address space, global memory by inference) and pointers in the global
// address space whose origin the compiler cannot see (opaque_global).
typedef const __attribute__((address_space(1))) uint8_t* global_bytes_t;
typedef __attribute__((address_space(1))) const uint4_t* global_uint4_t;

// a pointer to global memory that is not restrict and not known to point to constant memory
__device__ __forceinline__ global_bytes_t opaque_global(const void* p) {
  asm volatile("" : "+s"(p));
  return (global_bytes_t)(p);
}
// the packed weights are read once per launch: non-temporal
__device__ __forceinline__ uint4 load_weights(const uint8_t* b, size_t off) {
  const uint4_t v = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(b + off));
  return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint4 load_weights(global_bytes_t b, size_t off) {
  const uint4_t v = __builtin_nontemporal_load((global_uint4_t)(b + off));
  return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint4 load_16(const uint8_t* b, size_t off) { return *reinterpret_cast<const uint4*>(b + off); }
__device__ __forceinline__ uint4 load_16(global_bytes_t b, size_t off) {
  const uint4_t v = *(global_uint4_t)(b + off);
  return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint32_t load_u16(const uint8_t* b, size_t off) { return *reinterpret_cast<const uint16_t*>(b + off); }
__device__ __forceinline__ uint32_t load_u16(global_bytes_t b, size_t off) {
  return *(__attribute__((address_space(1))) const uint16_t*)(b + off);
}
__device__ __forceinline__ uint32_t load_u8(const uint8_t* b, size_t off) { return b[off]; }
__device__ __forceinline__ uint32_t load_u8(global_bytes_t b, size_t off) { return b[off]; }

// Zero, available only once `loaded` -- the destination of a load -- has arrived: the compiler waits for the load
// before an asm statement that reads its destination, and what is computed from the result comes after that.
__device__ __forceinline__ uint32_t zero_once_loaded(uint32_t loaded) {
  uint32_t zero;
  asm volatile("v_and_b32 %0, 0, %1" : "=v"(zero) : "v"(loaded));
  return zero;
}

#ifdef BLKQ4_SKINNY_BF16
constexpr bool kBF = true;
#else
constexpr bool kBF = false;
#endif

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
  // fetched into that XCD's L2 once.  Column groups of four tiles or more hold whole lines by themselves and are
  // dealt out singly, which keeps the XCDs level when there are few of them.
  static_assert(kSplit == kWaves || kSplit == 1, "the waves split K among all of them or not at all");
  constexpr int kTileWaves = kWaves / kSplit;  // waves (or sets of waves) with column tiles of their own
  const int col_groups = ((N >> 4) + NT * kTileWaves - 1) / (NT * kTileWaves);
  const int wg = blockIdx.x;
  const int q = wg >> 3;
  const int rg = q % row_groups;
  constexpr int kNeighbours = streaming_neighbours(NT, kWaves, kSplit);
  const int cq = q / row_groups;
  int cg = kNeighbours * ((wg & 7) + 8 * (cq / kNeighbours)) + (cq % kNeighbours);
  if (cg >= col_groups) return;  // the grid is rounded up to whole groups of 8 * kNeighbours column groups
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

  // Addresses are a wave-uniform part (slice and column tile: scalar arithmetic) plus a part of the lane that
  // never changes, 32 bits each: (k-unit of the slice g, column nl).  Only in the last slice, when it has
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

  // Rows to LDS, requested before anything else.  Layout: [pair of 32-deep units][row][128 B], the eight 16-byte
  // chunks of a row's 128 bytes XOR-swizzled with bits 1..3 of the row (the 16 lanes of a fragment read touch 16
  // rows at the same logical chunk and land on 16 different 16-byte slots of the 256 bytes the banks span).  A copy
  // instruction moves 1 KiB = eight rows' 128 contiguous bytes each: whole 128-byte lines of the activations
  // (with 64 bytes per row and instruction the staging of 16 rows cost 1 us more on C3's shape).  The LDS side of
  // a copy is lane-linear, so the swizzle is applied to the global address a lane fetches.  A 128-deep slice is
  // two pairs = 256 * rows contiguous bytes.
  uint32_t a_rd = 0;   // LDS byte offset of this lane's row inside a pair
  uint32_t a_swz = 0;  // bits 1..3 of the row
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                            (__attribute__((address_space(3))) uint8_t*)(smem)));
  if (AM == kRowsPerSlotInLds) {
    // this wave's slots: DEPTH pieces of [2 pairs][kSlotRows rows][128 B]
    a_rd = (wave * DEPTH) * kSlotBytes + nl * 128;
    a_swz = (nl >> 1) & 7;
  }
  if (A_LDS) {
    const int rows = 1 << rows_log2;
    if (kSplit == 1) {
      // every wave needs all of K: the waves share out the copies (copy q fills LDS bytes [1024 q, 1024 q + 1024),
      // lane l the 16 bytes at 16 l) and meet at a barrier below
      const int copies = ((K << rows_log2) + 511) >> 9;  // K * 2 * rows bytes in 1 KiB copies, the last one may be partial
      for (int q = wave; q < copies; q += kWaves) {
        const uint32_t off = q * 1024 + lane * 16;
        const int e = off >> 7;
        const int row = e & (rows - 1);
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        const int u = min(2 * (e >> rows_log2) + (chunk >> 2), units - 1);  // past the end: any valid unit
        async_copy_16(lds0 + q * 1024, A, (static_cast<uint32_t>(min(row, M - 1)) * K + u * 32 + (chunk & 3) * 8) * 2);
      }
    } else {
      // The waves split K: a wave stages the rows of ITS slices, nobody else reads them, and no barrier is needed:
      // the copies are requested before the wave's first weights, requests complete in order, so a wave that has
      // its first weights has all its rows (consume() makes its first reads wait for a weight word).  With fewer
      // than four rows a copy moves less than its 1 KiB (the lanes past the slice, or past the end of K in the
      // last slice, are switched off: K is a multiple of 64, so a pair exists whole or not at all).
      const uint32_t slice_bytes = 256u << rows_log2;
      for (int li = 0; li < my_slices; ++li) {
        const int sl = ws + kSplit * li;
        for (uint32_t off0 = 0; off0 < slice_bytes; off0 += 1024) {
          const uint32_t off = off0 + lane * 16;
          const int e = off >> 7;
          const int row = e & (rows - 1);
          const int chunk = (lane & 7) ^ ((row >> 1) & 7);
          const int u = 4 * sl + 2 * (e >> rows_log2) + (chunk >> 2);
          if (off < slice_bytes && u < units) {  // (units past the end of K are not read, and lie outside the rows' LDS)
            async_copy_16(__builtin_amdgcn_readfirstlane(lds0 + (static_cast<uint32_t>(sl) << (8 + rows_log2)) + off0), A,
                          (static_cast<uint32_t>(min(row, M - 1)) * K + u * 32 + (chunk & 3) * 8) * 2);
          }
        }
      }
    }
    const int row = min(nl, rows - 1);  // row tile mt: 16 mt rows further (same swizzle: bits 1..3 of the row)
    a_rd = row * 128;
    a_swz = (row >> 1) & 7;
  }
  // unit g of a slice is half g & 1 of pair g >> 1 (a_lane: offset of the pair's row; a_half: which 64 bytes)
  const uint32_t pair_bytes = (AM == kRowsPerSlotInLds) ? kSlotRows * 128 : (128u << rows_log2);
  a_lane[0] = static_cast<uint32_t>(g >> 1) * pair_bytes + a_rd;
  a_lane[1] = static_cast<uint32_t>(g_alt >> 1) * pair_bytes + a_rd;
  const uint32_t a_half[2] = {static_cast<uint32_t>(g & 1) * 4, static_cast<uint32_t>(g_alt & 1) * 4};
  // a slot past the end asks for valid units (so every slot always issues the same loads); its scales are
  // zeroed when the slot is consumed (not here: that would wait for the load right after requesting it),
  // which makes it contribute exactly 0
  // Every offset is 32 bits wide (the launcher checks that the packed weights end below 4 GiB) and made of a part
  // of the lane that never changes and a part of the wave (slice, column tile: scalar arithmetic): a request costs
  // one vector addition.  (With 64-bit offsets the compiler keeps base + lane part in a register pair per operand and
  // adds the wave's part to it with 64-bit vector additions: 110 instructions of address arithmetic per slot of four
  // tiles against the 224 of its conversion.)
  const uint32_t m2_lane[2] = {m_lane[0] * 2, m_lane[1] * 2};
  // rows staged per slot: copy q fills LDS bytes [1024 q, 1024 q + 1024) of the slot, lane l the 16 bytes at 16 l;
  // a last slice with two units only fetches its first pair twice
  uint32_t a_copy[(AM == kRowsPerSlotInLds) ? 4 * MT : 1][2];
  if (AM == kRowsPerSlotInLds) {
#pragma unroll
    for (int q = 0; q < 4 * MT; ++q) {
      const int rr = 8 * q + (lane >> 3);  // (pair, row) index inside the slot
      const int row = rr % kSlotRows;
      const int chunk = (lane & 7) ^ ((row >> 1) & 7);
      const uint32_t in_pair = (static_cast<uint32_t>(min(row, M - 1)) * K + (chunk >> 2) * 32 + (chunk & 3) * 8) * 2;
      a_copy[q][0] = in_pair + (rr / kSlotRows) * 128;
      a_copy[q][1] = in_pair;
    }
  }
#define BLKQ4_LOAD_SLOT(dst_, d_, cg_, slice_, keep_, W_, S_, Z_)                                                \
  {                                                                                            \
    const int sl_ = min((slice_), last_slice);                                                 \
    const bool alt_ = rem != 0 && sl_ == last_slice;                                           \
    const uint32_t wl_ = alt_ ? w_lane[1] : w_lane[0];                                         \
    const uint32_t ml_ = alt_ ? m_lane[1] : m_lane[0];                                         \
    const uint32_t ml2_ = alt_ ? m2_lane[1] : m2_lane[0];                                      \
    const uint32_t keep32_ = static_cast<uint32_t>(keep_);                                     \
    if (AM == kRowsPerSlotInLds) {                                                             \
      /* requested before the slot's weights, so whoever has the weights has the rows */       \
      _Pragma("unroll") for (int q = 0; q < 4 * MT; ++q) {                                     \
        async_copy_16(__builtin_amdgcn_readfirstlane(lds0 + (wave * DEPTH + (d_)) * kSlotBytes + q * 1024), A, \
                      (alt_ ? a_copy[q][1] : a_copy[q][0]) + static_cast<uint32_t>(sl_) * 256u); \
      }                                                                                        \
    }                                                                                          \
    _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                           \
      /* tile t of column group cg_; a tile past the end (last column group only, when the group's */ \
      /* tile count does not divide the number of tiles) re-reads the group's first tile and is    */ \
      /* not stored                                                                                */ \
      const int tile_ = ((cg_) * kTileWaves + wt) * NT + t;                                    \
      const int tu_ = (tile_ < tiles) ? tile_ : (cg_) * (kTileWaves * NT);                     \
      const uint32_t wu_ = ((static_cast<uint32_t>(4 * sl_) * N + tu_ * 16) * 16u) & keep32_;  \
      (dst_).w[t] = load_weights(W_, static_cast<size_t>(wu_ + wl_));                          \
      if (ROW) {                                                                               \
        const uint32_t mu_ = (static_cast<uint32_t>(tu_ * 16 / BS) * K + sl_ * 128) & keep32_; \
        const uint32_t so_ = mu_ * 2 + ml2_;                                                   \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                        \
          (dst_).rs[ROW ? t : 0][q] = load_16(S_, static_cast<size_t>(so_) + 16 * q);          \
        }                                                                                      \
        if (HAS_ZP) {                                                                          \
          const uint32_t zo_ = mu_ + ml_;                                                      \
          _Pragma("unroll") for (int q = 0; q < 2; ++q) {                                      \
            (dst_).rz[ROW ? t : 0][q] = load_16(Z_, static_cast<size_t>(zo_) + 16 * q);        \
          }                                                                                    \
        }                                                                                      \
      } else {                                                                                 \
        _Pragma("unroll") for (int q = 0; q < kMeta; ++q) {                                    \
          const uint32_t mu_ = (static_cast<uint32_t>(kBlocksPerSlice * sl_ + q) * N + tu_ * 16) & keep32_; \
          (dst_).sc[t][ROW ? 0 : q] = load_u16(S_, static_cast<size_t>(mu_ * 2 + ml2_));       \
          (dst_).zp[t][ROW ? 0 : q] = HAS_ZP ? load_u8(Z_, static_cast<size_t>(mu_ + ml_)) : 8u; \
        }                                                                                      \
      }                                                                                        \
    }                                                                                          \
  }
  // A wave's local slices are li = 0 .. my_slices - 1 (slice ws + kSplit * li), taken DEPTH at a time; the
  // slots past my_slices in the last round ask for the last slice once more and are zeroed.
  // The first ring's requests go out right behind the copies of the rows and stay there: loads through the
  // restrict-qualified pointers to const are invariant to the compiler, which moves them across asm statements,
  // waits and barriers at will, while everything below counts on "rows requested before weights"; so these first
  // loads go through copies of the pointers whose origin it cannot see.  (All loads through unqualified pointers
  // cost the main loops too much: C3 9.3 -> 11.2 us.)
  const uint8_t* const wb = reinterpret_cast<const uint8_t*>(W);
  const uint8_t* const sb = reinterpret_cast<const uint8_t*>(S);
  const uint8_t* const zb = reinterpret_cast<const uint8_t*>(Z);
  {
    const global_bytes_t w0 = opaque_global(W), s0 = opaque_global(S), z0 = opaque_global(Z);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) BLKQ4_LOAD_SLOT(slot[d], d, cg, ws + kSplit * d, -1, w0, s0, z0);
  }
  if constexpr (A_LDS && kSplit == 1) {
    // everything but the requests of the ring just issued has landed: this wave's share of the rows; then
    // everybody's
    constexpr int kLoads = ROW ? NT * (1 + 4 + (HAS_ZP ? 2 : 0)) : NT * (1 + kMeta * (HAS_ZP ? 2 : 1));
    constexpr int kRing = DEPTH * kLoads;
    static_assert(kRing <= 63, "the counter of outstanding requests cannot tell the ring from the rows");
    wait_vmcnt<kRing>();
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
    // Only the rows that exist travel: lane L holds row 16 mt + (L & 15), and with one row tile the workgroup
    // keeps 1 << rows_log2 <= 16 rows.  Partial tiles: [wave][tile t][row tile mt][row][16 columns] floats.
    const int rows = (MT == 1) ? (1 << rows_log2) : 16;
    // the partial tiles share the rows' LDS (every wave must be done with the rows), or are written again for
    // the workgroup's next column group (every wave must be done reading the last ones)
    if (kRefill || red_offset == 0) __syncthreads();
    if (nl < rows) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          *reinterpret_cast<float4_t*>(&red[((((wave * NT + t) * MT + mt) * rows + nl) << 4) + 4 * g]) = acc[t][mt];
        }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[t][mt] = float4_t{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    // value v = (tile t, row tile mt, row, column) of the partial tiles; every thread sums a few of them over
    // the waves, in the order of the waves
    const int per_wave = NT * MT * rows * 16;
    for (int v = tid; v < per_wave; v += 64 * kWaves) {
      float r = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) r += red[w * per_wave + v];
      const int c = v & 15, row_in = (v >> 4) % rows, tm = (v >> 4) / rows;  // tm = t * MT + mt
      const int t = tm / MT, mt = tm % MT;
      const int row = 16 * mt + row_in;
      if (row < M && cgx * NT + t < tiles) {
        const int col = cgx * (16 * NT) + 16 * t + c;
        uint32_t h = float_to_bits<kBF>(r);
        if (bias != nullptr) h = add_bias_bits_t<kBF>(h, bias[col]);
        C[static_cast<size_t>(row) * N + col] = static_cast<uint16_t>(h);
      }
    }
  };

  bool own_rows_landed = false;  // wave-uniform
  // converts slot d, which holds local slice li, and multiplies it with the rows
  auto consume = [&](int d, int li) {
    const Slot<BS, NT, MT, AM, ROW>& cur = slot[d];
    const int slice = ws + kSplit * li;
    const int sl = min(slice, last_slice);
    const uint32_t full = (slice < last_slice || (slice == last_slice && rem == 0)) ? 0xffffffffu : 0u;  // uniform
    const uint32_t okm = full | ((slice == last_slice) ? ok_last : 0u);
      uint4 af[MT][4];  // eight 16-bit activations each
      // Rows staged by this wave itself were requested before the slot's weights and requests complete in
      // order: the reads below wait for one of the slot's weight words -- for every slot when the rows are staged
      // per slot, for the wave's first slot only when it staged the rows of all its slices up front (after that
      // they are all there, and the reads may run ahead of the weights again).  (Waiting for the copies by count
      // right behind the first ring's requests instead is slower: C2 4.55 -> 4.73 us.)
      uint32_t arrived = 0u;
      if (AM == kRowsPerSlotInLds) {
        arrived = zero_once_loaded(cur.w[0].x);
      } else if (kSplit != 1 && !own_rows_landed) {
        arrived = zero_once_loaded(cur.w[0].x);
        own_rows_landed = true;
      }
      if (A_LDS) {
        // (a slot past the wave's last slice holds the last slice's weights with zeroed scales; it is multiplied
        // with rows this wave has staged itself, those of its first slice: 0 times anything finite)
        const int sl_a = (kSplit == 1 || slice <= last_slice) ? sl : ws;
        const bool alt_a = rem != 0 && sl_a == last_slice;
        const uint8_t* ap = a_lds + (static_cast<uint32_t>(4 * sl_a) << (6 + rows_log2)) + (alt_a ? a_lane[1] : a_lane[0]) + arrived;
        const uint32_t half = alt_a ? a_half[1] : a_half[0];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            af[mt][j] = *reinterpret_cast<const uint4*>(ap + mt * 2048 + (((half + j) ^ a_swz) * 16));
          }
      } else {
        // (all four units of a slot hold valid rows, also past the end of K: the lane reads its own unit g)
        const uint8_t* ap = a_lds + a_lane[0] + d * kSlotBytes + arrived;
        const uint32_t half = a_half[0];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            af[mt][j] = *reinterpret_cast<const uint4*>(ap + mt * 2048 + (((half + j) ^ a_swz) * 16));
          }
      }
      // all fragment reads are requested before the conversion starts (left to itself the compiler puts each read
      // right before the MFMA that needs it, which then waits out the whole LDS latency)
      __builtin_amdgcn_sched_barrier(0);
      // the constants of the tile being converted (blocks along K)
      DequantConsts dc[kMeta];
      Bf16Consts bc[kMeta];
      // word j of tile t as the eight values of the MFMA's weight operand (for bf16: their bits)
      auto convert = [&](const int t, const int j) -> half8_t {
        const uint32_t word = vec_word(cur.w[t], j);
        if constexpr (kBF && !ROW) {
          if (j == 0) {
#pragma unroll
            for (int q = 0; q < kMeta; ++q) bc[q] = make_bf16_consts(cur.sc[t][q] & okm, cur.zp[t][q]);
          }
          return __builtin_bit_cast(half8_t, dequant_word_bf16(word, bc[(kMeta == 2) ? (j >> 1) : 0], masks));
        } else {
          if (!ROW && j == 0) {
#pragma unroll
            for (int q = 0; q < kMeta; ++q) dc[q] = make_dequant_consts(cur.sc[t][ROW ? 0 : q] & okm, cur.zp[t][ROW ? 0 : q]);
          }
          const uint32_t y = word >> 8;
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
              const uint32_t src = (i >= 2) ? y : word;
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
            p[0] = dequant_pair(word, 0, c, masks);
            p[1] = dequant_pair(word, 1, c, masks);
            p[2] = dequant_pair(y, 2, c, masks);
            p[3] = dequant_pair(y, 3, c, masks);
          }
          half8_t wf;
          wf[0] = p[0][0]; wf[1] = p[0][1]; wf[2] = p[1][0]; wf[3] = p[1][1];
          wf[4] = p[2][0]; wf[5] = p[2][1]; wf[6] = p[3][0]; wf[7] = p[3][1];
          return wf;
        }
      };
      // The next word is converted before this one's MFMAs are issued: a conversion's last instruction would otherwise
      // feed the MFMA right behind it, and the wait states that costs were an s_nop per word (21 of a slot's 355
      // instructions with four tiles).
      half8_t wf = convert(0, 0);
#pragma unroll
      for (int x = 0; x < 4 * NT; ++x) {
        const int t = x >> 2, j = x & 3;
        half8_t next = wf;
        if (x + 1 < 4 * NT) next = convert((x + 1) >> 2, (x + 1) & 3);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          if constexpr (kBF) {
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, wf), as_bf16x8(af[mt][j]),
                                                                acc[t][mt], 0, 0, 0);
          } else {
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, as_half8(af[mt][j]), acc[t][mt], 0, 0, 0);
          }
        }
        wf = next;
      }
  };

  if (!kRefill) {
    // one column group per workgroup: a slot is refilled only while the wave has slices left
    for (int i0 = 0; i0 < my_slices; i0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        consume(d, i0 + d);
        if (i0 + DEPTH < my_slices) BLKQ4_LOAD_SLOT(slot[d], d, cg, ws + kSplit * (i0 + d + DEPTH), -1, wb, sb, zb);
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
        BLKQ4_LOAD_SLOT(slot[d], d, ld_cg, ws + kSplit * (ld_i0 + d), keep, wb, sb, zb);
        // the refill is requested here, not together with the others at the end of the round
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    flush(cg);
    cg = next_cg;
  }
#undef BLKQ4_LOAD_SLOT
}

// Raises a kernel's dynamic-LDS limit, once per kernel instantiation and device.
template <auto kKernel>
hipError_t raise_lds_limit() {
  return raise_lds_limit_once(reinterpret_cast<const void*>(kKernel), kMaxLdsBytes, &lds_limit_flags<kKernel>());
}

// One kernel instantiation with the launch geometry of the plan (blkq4_choose.h): raises its dynamic-LDS limit,
// then launches.  What the kernel assumes about the plan is checked here.
template <int BS, bool HAS_ZP, bool ROW, int DEPTH, int NT, int MT, int kWaves, int AM, int kSplit>
int launch_kernel(const blkq4_gemm_args* a) {
  const blkq4_streaming_plan& p = a->streaming;
  // partial tiles of the sum across waves, rows that exist only
  const size_t red_rows = MT == 1 ? (size_t{1} << p.rows_log2) : 16;
  const size_t kRedBytes = (kSplit == 1) ? 0 : static_cast<size_t>(kWaves) * NT * MT * red_rows * 64;
  constexpr size_t kPerSlotBytes = static_cast<size_t>(kWaves) * DEPTH * 16 * MT * 256;
  static_assert(static_cast<size_t>(kWaves) * NT * MT * 16 * 64 <= kMaxLdsBytes, "partial tiles do not fit in LDS");
  static_assert(AM != kRowsPerSlotInLds || kPerSlotBytes <= kMaxLdsBytes, "slots do not fit in LDS");
  const bool refill = p.refill != 0;
  if (a->launched_id != nullptr) *a->launched_id = streaming_id(DEPTH, NT, MT, kWaves, AM, kSplit, refill);
  const size_t a_bytes = AM == kRowsWholeInLds ? ((((static_cast<size_t>(a->k) * 2) << p.rows_log2) + 1023) & ~size_t{1023})
                                               : kPerSlotBytes;
  constexpr int kGroupTiles = NT * (kWaves / kSplit);
  constexpr int kXcdRound = 8 * streaming_neighbours(NT, kWaves, kSplit);  // column groups dealt to the XCDs at a time
  const int col_groups = (a->n / 16 + kGroupTiles - 1) / kGroupTiles;
  if ((1 << p.rows_log2) * p.row_groups < a->m || (MT == 1 && (1 << p.rows_log2) > 16) || (MT == 2 && p.rows_log2 != 5) ||
      p.row_groups < 1 || p.cg_stride < kXcdRound || (p.cg_stride % kXcdRound) != 0 || p.lds_bytes > kMaxLdsBytes ||
      p.red_offset + kRedBytes > p.lds_bytes || a_bytes > p.lds_bytes || (p.red_offset != 0 && p.red_offset < a_bytes) ||
      (!refill && (p.cg_stride < col_groups || kSplit == 1)) ||
      p.grid != static_cast<uint32_t>(p.cg_stride) * static_cast<uint32_t>(p.row_groups) ||
      (kSplit == 1 && (reinterpret_cast<uintptr_t>(a->c) & 7u) != 0)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if constexpr (ROW && kWaves == 16) {
    if (refill) return static_cast<int>(hipErrorInvalidValue);  // this kernel has no walking variant
  }
  if (a->dry_run) return 0;  // the plan has passed every check a launch makes
  auto launch = [&](auto* kernel, hipError_t attr) {
    if (attr != hipSuccess) return static_cast<int>(attr);
    // the launch's own status: a sticky error of an earlier, unrelated call stays where it is
    return static_cast<int>(launch_status(kernel, dim3(p.grid), dim3(64 * kWaves), p.lds_bytes, a->stream,
                                          static_cast<const uint16_t*>(a->a), static_cast<const uint4*>(a->packed_w),
                                          static_cast<const uint16_t*>(a->scales),
                                          static_cast<const uint8_t*>(a->zero_points), static_cast<uint16_t*>(a->c),
                                          static_cast<const uint16_t*>(a->bias), a->m, a->n, a->k, p.rows_log2,
                                          p.row_groups, p.cg_stride, p.red_offset));
  };
  if (refill) {
    // (the sixteen-wave kernel for blocks along N has no walking variant: it does not fit in 128 registers)
    if constexpr (ROW && kWaves == 16) {
      return static_cast<int>(hipErrorInvalidValue);
    } else {
      constexpr auto kernel = skinny_mfma_kernel<BS, HAS_ZP, DEPTH, NT, MT, kWaves, AM, ROW, true, kSplit>;
      return launch(kernel, raise_lds_limit<kernel>());
    }
  }
  if constexpr (kSplit == 1) {
    return static_cast<int>(hipErrorInvalidValue);  // waves that do not split K exist in the walking form only
  } else {
    constexpr auto kernel = skinny_mfma_kernel<BS, HAS_ZP, DEPTH, NT, MT, kWaves, AM, ROW, false, kSplit>;
    return launch(kernel, raise_lds_limit<kernel>());
  }
}

// The shapes that exist, (DEPTH, NT, MT, waves, AM, split): what blkq4::choose() may ask for.  Blocks along N:
// those with one column tile per wave (28 registers of packed weights, scales and zero-points per slot and tile).
#define BLKQ4_W kRowsWholeInLds
#define BLKQ4_P kRowsPerSlotInLds
#define BLKQ4_STREAMING_SHAPES(X)                                                                          \
  /* row groups of 32 */                                                                                   \
  X(2, 1, 2, 8, BLKQ4_W, 8) X(2, 2, 2, 8, BLKQ4_W, 8) X(2, 4, 2, 8, BLKQ4_W, 8) X(2, 6, 2, 8, BLKQ4_W, 8)  \
  X(2, 8, 2, 8, BLKQ4_W, 8)                                                                                \
  X(2, 1, 2, 8, BLKQ4_P, 8) X(2, 2, 2, 8, BLKQ4_P, 8) X(2, 4, 2, 8, BLKQ4_P, 8) X(2, 6, 2, 8, BLKQ4_P, 8)  \
  X(2, 8, 2, 8, BLKQ4_P, 8)                                                                                \
  /* waves with column tiles of their own */                                                               \
  X(4, 1, 1, 4, BLKQ4_W, 1)                                                                                \
  /* wide layers, rows staged per slice */                                                                 \
  X(2, 4, 1, 4, BLKQ4_P, 4) X(2, 4, 1, 8, BLKQ4_P, 8)                                                      \
  X(2, 5, 1, 4, BLKQ4_P, 4) X(2, 6, 1, 4, BLKQ4_P, 4) X(2, 7, 1, 4, BLKQ4_P, 4)                            \
  X(2, 5, 1, 8, BLKQ4_P, 8) X(2, 6, 1, 8, BLKQ4_P, 8) X(2, 7, 1, 8, BLKQ4_P, 8)                            \
  /* up to 16 rows, the waves split K */                                                                   \
  X(4, 1, 1, 8, BLKQ4_W, 8) X(4, 2, 1, 8, BLKQ4_W, 8) X(4, 3, 1, 8, BLKQ4_W, 8) X(2, 1, 1, 8, BLKQ4_W, 8)  \
  X(2, 1, 1, 16, BLKQ4_W, 16) X(2, 2, 1, 16, BLKQ4_W, 16) X(2, 3, 1, 16, BLKQ4_W, 16)                      \
  X(4, 1, 1, 8, BLKQ4_P, 8) X(4, 2, 1, 8, BLKQ4_P, 8) X(4, 3, 1, 8, BLKQ4_P, 8)                            \
  X(8, 1, 1, 4, BLKQ4_W, 4) X(4, 1, 1, 4, BLKQ4_W, 4) X(4, 2, 1, 4, BLKQ4_W, 4) X(4, 3, 1, 4, BLKQ4_W, 4)

template <int BS, bool HAS_ZP, bool ROW>
int launch_plan(const blkq4_gemm_args* a) {
  const blkq4_streaming_plan& p = a->streaming;
#define BLKQ4_TRY(D_, NT_, MT_, W_, AM_, S_)                                                               \
  if (p.depth == D_ && p.nt == NT_ && p.mt == MT_ && p.waves == W_ && p.am == AM_ && p.split == S_) {      \
    if constexpr (ROW && NT_ > 1) {                                                                        \
      return static_cast<int>(hipErrorInvalidValue);                                                       \
    } else {                                                                                               \
      return launch_kernel<BS, HAS_ZP, ROW, D_, NT_, MT_, W_, AM_, S_>(a);                                 \
    }                                                                                                      \
  }
  BLKQ4_STREAMING_SHAPES(BLKQ4_TRY)
#undef BLKQ4_TRY
  return static_cast<int>(hipErrorInvalidValue);  // a shape that does not exist
}
#undef BLKQ4_W
#undef BLKQ4_P

template <int BS>
int launch_skinny(const blkq4_gemm_args* a) {
  if (a->column_wise) return a->zero_points ? launch_plan<BS, true, false>(a) : launch_plan<BS, false, false>(a);
  return a->zero_points ? launch_plan<BS, true, true>(a) : launch_plan<BS, false, true>(a);
}

}  // namespace

extern "C" int BLKQ4_SKINNY_ENTRY(const blkq4_gemm_args* a) {
  if (a->m < 1 || a->m > kStreamingMaxRows || (a->n % 16) != 0 || (a->k % 64) != 0) return static_cast<int>(hipErrorInvalidValue);
  // every offset is 32 bits wide: the packed weights (K N / 2 bytes) end below 4 GiB
  if (static_cast<uint64_t>(a->k) * static_cast<uint64_t>(a->n) >= kStreamingMaxWeights) return static_cast<int>(hipErrorInvalidValue);
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
