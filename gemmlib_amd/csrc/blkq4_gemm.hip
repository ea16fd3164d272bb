// M > 16 path: fp16 MFMA GEMM with the 4-bit weights dequantized in registers (gfx950).
//
// Workgroup tile (32*RT) x 128 x 64 (M x N x K), four waves side by side along N: a wave owns
// (32*RT) x 32 outputs, i.e. ONE 32-column weight fragment per 16-deep k step that it converts to
// fp16 once and feeds to RT MFMAs (RT = 8 for large M).  Measured on MI355X, a wave can issue about
// four VALU instructions in the shadow of one 32x32x16 MFMA; the tall wave tile keeps the
// conversion at 13 VALU instructions per 8 MFMAs.
//
// Data movement: everything the main loop consumes is copied HBM -> LDS by the asynchronous
// global_load_lds_dwordx4 / _dword instructions (no registers in between) into a ring of kStages
// k tiles, requested kDistance tiles ahead:
//   - activations: 16-byte units, XOR-swizzled inside each 128-byte row with bits 1..3 of the row
//     (LDS has 64 banks = 256 bytes, two rows; a 16-lane group of a fragment read touches 16
//     different rows at the same logical column and must land on 16 different 16-byte slots).  The
//     swizzle is applied to the global address a lane reads, because the LDS side of these loads is
//     lane-linear;
//   - packed weights: a lane's MFMA operand for one 64-deep k tile is exactly one 16-byte unit of
//     the packed layout (32 consecutive k of one column); 32 lanes request 512 contiguous bytes and
//     every lane later reads back the unit it requested;
//   - scales (and zero-points) of the tile: one 4-byte request per lane and quantization block row.
//
// Schedule of one k tile (four 16-deep steps, RT MFMAs each), written out in program order and
// pinned with scheduling barriers because the compiler's own schedule serialises LDS latency:
//   after MFMA r of step j come the LDS read of activation fragment r of step j+1 and one piece
//   (3-4 VALU instructions) of the next weight fragment's conversion, so that the issue slots in the
//   shadow of every MFMA are filled and nothing is consumed sooner than one step after its request.
//   After step 1 one s_waitcnt vmcnt + s_barrier publish the NEXT k tile, so that steps 2 and 3 can
//   already read its packed weights / scales and the fragments of its step 0: the MFMA pipe never
//   waits for the first LDS read of a tile.  The asynchronous copies for the tile kDistance ahead
//   are issued one per MFMA in steps 2 and 3 (a copy instruction can stall at issue while the
//   texture path drains; behind an MFMA that stall is hidden).
//
// Math: v_mfma_f32_32x32x16_f16 with the weights as the row operand, so the accumulator of a lane
// holds 4 consecutive output columns of one activation row (8-byte stores in the epilogue).
//
// Rows past M and 32-column tiles past N are handled by clamping the addresses that are read (the
// values computed from them are never stored), so the main loop has no branches.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_dequant.h"
#include "blkq4_device.h"

namespace {

using namespace blkq4;

constexpr int kWaves = 8;  // two per SIMD
constexpr int kThreads = 64 * kWaves;
constexpr int kBN = 32 * kWaves;
constexpr int kBK = 64;
constexpr int kStages = 4;    // LDS ring depth
constexpr int kDistance = 3;  // tiles requested ahead of the one being consumed

// Asynchronous copy: every active lane moves SIZE bytes from global address (base + offset) to
// LDS[lds_base + lane * SIZE].  lds_base and base are wave-uniform, offset is per lane.  The
// compiler does not see the LDS write (it is ordered by hand with wait_vmcnt + s_barrier below).
__device__ __forceinline__ void async_copy_16(uint32_t lds_base, const void* base, uint32_t offset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(offset), "s"(base)
               : "memory");
}
__device__ __forceinline__ void async_copy_4_flat(uint32_t lds_base, const void* gptr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_base), "v"(gptr) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// s_barrier that the compiler may not move LDS accesses across, in either direction
__device__ __forceinline__ void block_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
#define BLKQ4_PIN() __builtin_amdgcn_sched_barrier(0)

template <int BS, int RT>
struct Stage {
  static constexpr int kBlocks = kBK / BS;                   // quantization block rows per k tile
  static constexpr int kABytes = 32 * RT * 128;              // [row][8 x 16-byte units, swizzled]
  static constexpr int kBBytes = kWaves * 1024;              // [wave][lane] 16-byte units
  static constexpr int kMetaBytes = kWaves * kBlocks * 128;  // [wave][block][64 B scales | 32 B zps | pad]
  static constexpr int kBytes = kABytes + kBBytes + kMetaBytes;
  static constexpr int kAOps = (4 * RT + kWaves - 1) / kWaves;  // 8-row activation copies per wave and stage
  static constexpr int kOps = kAOps + 1 + kBlocks;              // async copies per wave and stage
};

template <int BS, bool HAS_ZP, int RT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_mfma_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ W, const uint8_t* __restrict__ S,
    const uint8_t* __restrict__ Z, uint16_t* __restrict__ C, int M, int N, int K, int m_tiles) {
  using St = Stage<BS, RT>;
  constexpr int kBlocks = St::kBlocks;
  constexpr int kOps = St::kOps;
  constexpr int kMeta = (BS == 16) ? 2 : 1;  // quantization blocks inside a lane's 32-deep unit
  static_assert(kStages * St::kBytes <= 160 * 1024, "LDS ring does not fit");
  static_assert(kDistance == kStages - 1, "the stage being refilled must be the one nobody reads");
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kStages * St::kBytes];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int i = lane & 31;  // row of an activation fragment / column of a weight fragment
  const int h = lane >> 5;  // which 32-deep half of the 64-deep k tile this lane covers

  const int bm = blockIdx.x % m_tiles;
  const int bn = blockIdx.x / m_tiles;
  const int m0 = bm * (32 * RT);
  const int nw0 = bn * kBN + wave * 32;
  // N is a multiple of 32, so 32-column tiles are whole; a tile past the end re-reads the last one
  const bool tile_ok = nw0 < N;
  const int nbase = min(nw0, N - 32);
  const int KT = K / kBK;

  // ---- per-lane byte offsets of the async copies inside k tile 0 ----
  constexpr int kAOps = St::kAOps;
  uint32_t a_off[kAOps];
  uint32_t a_dst[kAOps];  // LDS byte offset of the 8-row group inside the stage
#pragma unroll
  for (int p = 0; p < kAOps; ++p) {
    // 4*RT groups of 8 rows are shared out over the waves; with fewer groups than waves the extra
    // waves copy a group a second time (same bytes to the same place) so that every wave has the
    // same number of copies in flight
    const int group = (kWaves * p + wave) % (4 * RT);
    a_dst[p] = group * 1024;
    const int row = 8 * group + (lane >> 3);  // row inside the tile
    const int col = (lane & 7) ^ ((row >> 1) & 7);     // logical 16-byte column this lane fetches
    a_off[p] = static_cast<uint32_t>(min(m0 + row, M - 1)) * (static_cast<uint32_t>(K) * 2u) + col * 16;
  }
  const uint32_t b_off = (static_cast<uint32_t>(h) * N + nbase + i) * 16u;
  const uint32_t b_stride = static_cast<uint32_t>(N) * 32u;  // two 32-deep units per k tile
  // meta: lanes 0..15 fetch 2 scales each, lanes 16..23 fetch 4 zero-points each
  const bool meta_active = HAS_ZP ? (lane < 24) : (lane < 16);
  const bool meta_is_scale = lane < 16 || !HAS_ZP;
  const uint8_t* meta_ptr = (meta_is_scale ? S + static_cast<size_t>(nbase + 2 * (lane & 15)) * 2
                                           : Z + (nbase + 4 * (lane & 7)));
  const uint32_t meta_row_bytes = meta_is_scale ? static_cast<uint32_t>(N) * 2u : static_cast<uint32_t>(N);

  const uint32_t lds0 = static_cast<uint32_t>(
      reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)(&lds[0])));  // LDS byte address

  // Async copy number q (0 .. kOps-1) of k tile `tile_` into ring slot `stage_`:
  // q < kAOps: 8 activation rows; q == kAOps: this wave's packed weights; above: one scale/zero-point row.
#define BLKQ4_COPY_OP(q_, tile_, stage_)                                                                  \
  {                                                                                                       \
    const uint32_t sbase_ = lds0 + (stage_) * St::kBytes;                                                 \
    if ((q_) < kAOps) {                                                                                   \
      async_copy_16(sbase_ + a_dst[(q_) < kAOps ? (q_) : 0], A + static_cast<size_t>(tile_) * 128,       \
                    a_off[(q_) < kAOps ? (q_) : 0]);                                                      \
    } else if ((q_) == kAOps) {                                                                           \
      async_copy_16(sbase_ + St::kABytes + wave * 1024, W + static_cast<size_t>(tile_) * b_stride, b_off); \
    } else if (meta_active) {                                                                             \
      async_copy_4_flat(sbase_ + St::kABytes + St::kBBytes + (wave * kBlocks + ((q_) - kAOps - 1)) * 128,    \
                        meta_ptr + static_cast<size_t>((tile_) * kBlocks + ((q_) - kAOps - 1)) * meta_row_bytes); \
    }                                                                                                     \
  }

  float16_t acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[r][e] = 0.f;

  // ---- prologue: request tiles 0 .. kDistance-1, publish tile 0 ----
#pragma unroll
  for (int s = 0; s < kDistance; ++s) {
#pragma unroll
    for (int q = 0; q < kOps; ++q) BLKQ4_COPY_OP(q, min(s, KT - 1), s);
  }
  wait_vmcnt<(kDistance - 1) * kOps>();
  block_barrier();

  // ---- LDS byte offsets of this lane's reads inside a stage ----
  uint32_t a_rd[4];  // activation fragment of step j, row tile 0 (row tile r is 4096 bytes further)
#pragma unroll
  for (int j = 0; j < 4; ++j) a_rd[j] = static_cast<uint32_t>(i) * 128u + (((4 * h + j) ^ ((i >> 1) & 7)) * 16u);
  const uint32_t b_rd = St::kABytes + wave * 1024 + lane * 16;
  const uint32_t m_rd = St::kABytes + St::kBBytes + wave * kBlocks * 128;

  const DequantMasks masks = DequantMasks::make();

#define BLKQ4_READ_A(dst_, stage_ptr_, j_)                                                   \
  _Pragma("unroll") for (int r = 0; r < RT; ++r)(dst_)[r] =                                  \
      as_half8(*reinterpret_cast<const uint4*>((stage_ptr_) + a_rd[j_] + r * 4096))
#define BLKQ4_READ_A1(dst_, stage_ptr_, j_, r_) \
  (dst_)[r_] = as_half8(*reinterpret_cast<const uint4*>((stage_ptr_) + a_rd[j_] + (r_) * 4096))
#define BLKQ4_READ_B(words_, dc_, stage_ptr_)                                                \
  {                                                                                          \
    const uint4 u_ = *reinterpret_cast<const uint4*>((stage_ptr_) + b_rd);                   \
    (words_)[0] = u_.x;                                                                      \
    (words_)[1] = u_.y;                                                                      \
    (words_)[2] = u_.z;                                                                      \
    (words_)[3] = u_.w;                                                                      \
    _Pragma("unroll") for (int q = 0; q < kMeta; ++q) {                                      \
      const int blk_ = (BS == 64) ? 0 : (BS == 32) ? h : (2 * h + q);                        \
      const uint8_t* mb_ = (stage_ptr_) + m_rd + blk_ * 128;                                 \
      (dc_##_sc)[q] = *reinterpret_cast<const uint16_t*>(mb_ + i * 2);                       \
      (dc_##_zp)[q] = HAS_ZP ? static_cast<uint32_t>(mb_[64 + i]) : 8u;                      \
    }                                                                                        \
  }
  // piece p (0..3) of the conversion of `word_` into weight fragment slot `dst_`
#define BLKQ4_PIECE(dst_, word_, dc_, p_) \
  wp[dst_][p_] = dequant_pair(((p_) >= 2) ? ((word_) >> 8) : (word_), (p_), (dc_), masks)
#define BLKQ4_WFRAG(slot_) \
  __builtin_bit_cast(half8_t, half2x4_t{wp[slot_][0], wp[slot_][1], wp[slot_][2], wp[slot_][3]})

  struct half2x4_t {
    half2_t a, b, c, d;
  };

  half8_t af[2][RT];   // activation fragments, double buffered over the k steps
  half2_t wp[2][4];    // weight fragment (4 fp16 pairs), double buffered
  uint32_t words[4], nwords[4];
  uint32_t dc_sc[kMeta], dc_zp[kMeta], ndc_sc[kMeta], ndc_zp[kMeta];
  DequantConsts dc[kMeta], ndc[kMeta];

  {
    const uint8_t* s0 = lds;
    BLKQ4_READ_B(words, dc, s0);
#pragma unroll
    for (int q = 0; q < kMeta; ++q) dc[q] = make_dequant_consts(dc_sc[q], dc_zp[q]);
    BLKQ4_READ_A(af[0], s0, 0);
#pragma unroll
    for (int p = 0; p < 4; ++p) BLKQ4_PIECE(0, words[0], dc[0], p);
  }

  for (int kt = 0; kt < KT; ++kt) {
    const int stage = kt % kStages;
    const uint8_t* sa = lds + stage * St::kBytes;                         // tile kt
    const uint8_t* sn = lds + ((kt + 1) % kStages) * St::kBytes;          // tile kt + 1
    const int copy_tile = min(kt + kDistance, KT - 1);                    // clamped: re-fetches the last tile
    const int copy_stage = (kt + kDistance) % kStages;
    BLKQ4_PIN();

    // ---------------- step 0: uses af[0] / wp[0]; prepares step 1 ----------------
    {
      const half8_t wf = BLKQ4_WFRAG(0);
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf, af[0][r], acc[r], 0, 0, 0);
        BLKQ4_READ_A1(af[1], sa, 1, r);
        if (r < 4) BLKQ4_PIECE(1, words[1], dc[0], r);
        BLKQ4_PIN();
      }
#pragma unroll
      for (int p = RT; p < 4; ++p) BLKQ4_PIECE(1, words[1], dc[0], p);
    }
    // ---------------- step 1: uses af[1] / wp[1]; prepares step 2 ----------------
    {
      const half8_t wf = BLKQ4_WFRAG(1);
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf, af[1][r], acc[r], 0, 0, 0);
        BLKQ4_READ_A1(af[0], sa, 2, r);
        if (r < 4) BLKQ4_PIECE(0, words[2], dc[kMeta - 1], r);
        BLKQ4_PIN();
      }
#pragma unroll
      for (int p = RT; p < 4; ++p) BLKQ4_PIECE(0, words[2], dc[kMeta - 1], p);
    }
    // publish tile kt+1: this wave's copies for it have landed, then everybody's
    wait_vmcnt<kOps>();
    block_barrier();
    // ---------------- step 2: uses af[0] / wp[0]; prepares step 3, reads next tile's weights ----
    BLKQ4_READ_B(nwords, ndc, sn);
    BLKQ4_PIN();
    {
      const half8_t wf = BLKQ4_WFRAG(0);
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf, af[0][r], acc[r], 0, 0, 0);
        BLKQ4_READ_A1(af[1], sa, 3, r);
        if (r < 4) BLKQ4_PIECE(1, words[3], dc[kMeta - 1], r);
        if (r < kOps) BLKQ4_COPY_OP(r, copy_tile, copy_stage);
        BLKQ4_PIN();
      }
#pragma unroll
      for (int p = RT; p < 4; ++p) BLKQ4_PIECE(1, words[3], dc[kMeta - 1], p);
    }
    // ---------------- step 3: uses af[1] / wp[1]; prepares step 0 of tile kt+1 ----------------
#pragma unroll
    for (int q = 0; q < kMeta; ++q) ndc[q] = make_dequant_consts(ndc_sc[q], ndc_zp[q]);
    BLKQ4_PIN();
    {
      const half8_t wf = BLKQ4_WFRAG(1);
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf, af[1][r], acc[r], 0, 0, 0);
        BLKQ4_READ_A1(af[0], sn, 0, r);
        if (r < 4) BLKQ4_PIECE(0, nwords[0], ndc[0], r);
        if (RT + r < kOps) BLKQ4_COPY_OP(RT + r, copy_tile, copy_stage);
        BLKQ4_PIN();
      }
#pragma unroll
      for (int p = RT; p < 4; ++p) BLKQ4_PIECE(0, nwords[0], ndc[0], p);
#pragma unroll
      for (int q = 2 * RT; q < kOps; ++q) BLKQ4_COPY_OP(q, copy_tile, copy_stage);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) words[j] = nwords[j];
#pragma unroll
    for (int q = 0; q < kMeta; ++q) dc[q] = ndc[q];
  }
  wait_vmcnt<0>();  // the clamped re-fetches of the last tile are still in flight
#undef BLKQ4_COPY_OP
#undef BLKQ4_READ_A
#undef BLKQ4_READ_A1
#undef BLKQ4_READ_B
#undef BLKQ4_PIECE
#undef BLKQ4_WFRAG

  // Epilogue.  Accumulator element 4*g + e of lane (i, h) is output row m0 + 32*r + i and column
  // nw0 + 8*g + 4*h + e: four consecutive columns -> one 8-byte store.
  if (!tile_ok) return;
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
  constexpr int BM = 32 * RT;
  const int m_tiles = (a->m + BM - 1) / BM;
  const int n_tiles = (a->n + kBN - 1) / kBN;
  const dim3 grid(static_cast<unsigned>(m_tiles) * n_tiles);
  hipLaunchKernelGGL((gemm_mfma_kernel<BS, HAS_ZP, RT>), grid, dim3(kThreads), 0,
                     static_cast<hipStream_t>(a->stream), static_cast<const uint8_t*>(a->a),
                     static_cast<const uint8_t*>(a->packed_w), static_cast<const uint8_t*>(a->scales),
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
  if (a->m < 1 || (a->n % 32) != 0 || a->n < 32 || (a->k % 64) != 0) return static_cast<int>(hipErrorInvalidValue);
  // the async copies address A and W with 32-bit byte offsets from a per-tile base
  if (static_cast<uint64_t>(a->m) * a->k * 2 >= (1ull << 32) || static_cast<uint64_t>(a->k) * a->n / 2 >= (1ull << 32)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  switch (a->block_size) {
    case 16: return launch_bs<16>(a);
    case 32: return launch_bs<32>(a);
    case 64: return launch_bs<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}
