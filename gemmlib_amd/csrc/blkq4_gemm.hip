// Tile kernel: fp16 MFMA GEMM with the 4-bit weights dequantized in registers (gfx950), for the row
// counts the weight-streaming kernel does not take.
//
// A workgroup is WM x WN computing waves, each owning (32*RT) x (32*NT) outputs, plus PW producer waves
// that only issue copies (see blkq4_choose.h for the shapes in use: 256 x 256, 128 x 256, 128 x 128 and 64 x 128 tiles).
// A wave converts each of its NT 32-column weight fragments to fp16 once per 16-deep k step and feeds it
// to RT MFMAs; a wave can issue about five VALU instructions in the shadow of one 32x32x16 MFMA, and the
// conversion takes 13 per fragment and step.
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
//   - scales (and zero-points) of the tile: blocks along K, one 4-byte request per lane and
//     quantization block row; blocks along N (ROW), the 128 + 64 bytes per column group as they lie in
//     memory (the reference's packed order is made for packed fp16 arithmetic and is used as it is).
//
// Schedule of one k tile (four 16-deep steps, RT*NT MFMAs each), written out in program order and
// pinned with scheduling barriers because the compiler's own schedule serialises LDS latency:
//   behind every MFMA come the LDS read of an activation fragment of step j+1 and one stage of the
//   conversion of two pieces of the next weight fragments (two pieces interleaved: a packed instruction
//   that reads the result of the one before it costs a wait state), so that the issue slots in the
//   shadow of every MFMA are filled and nothing is consumed sooner than one step after its request.
//   After step 1 one s_waitcnt vmcnt + s_barrier publish the NEXT k tile, so that steps 2 and 3 can
//   already read its packed weights / scales and the fragments of its step 0: the MFMA pipe never
//   waits for the first LDS read of a tile.  The asynchronous copies for the tile kDistance ahead
//   are spread over the MFMAs of the steps after the barrier that frees their ring slot (a copy
//   instruction can stall at issue while the texture path drains; behind an MFMA that stall is hidden),
//   or left to the producer waves.
//
// Math: v_mfma_f32_32x32x16_f16 with the weights as the row operand, so the accumulator of a lane
// holds 4 consecutive output columns of one activation row; the epilogue transposes the tile through
// LDS and stores whole rows.
//
// Rows past M and 32-column tiles past N are handled by clamping the addresses that are read (the
// values computed from them are never stored), so the main loop has no branches.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include <type_traits>

#include "blkq4_choose.h"
#include "blkq4_dequant.h"
#include "blkq4_device.h"
#include "blkq4_launch.h"
#include "blkq4_gemm_common.h"

// This file is compiled twice: as it is for fp16, and through blkq4_gemm_bf16.hip, which defines BLKQ4_GEMM_BF16
// before including it, for bf16 activations, scales and outputs.
#ifdef BLKQ4_GEMM_BF16
#define BLKQ4_GEMM_ENTRY blkq4_dev_gemm_bf16
#else
#define BLKQ4_GEMM_ENTRY blkq4_dev_gemm
#endif

namespace {

using namespace blkq4;

#ifdef BLKQ4_GEMM_BF16
constexpr bool kBF = true;
#else
constexpr bool kBF = false;
#endif
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

constexpr int kBK = 64;

// MFMA slot (0 .. slots-1) after which copy y of the range [lo, hi) is issued: evenly spread
constexpr int copy_slot(int y, int lo, int hi, int slots) { return (hi > lo) ? (y - lo) * slots / (hi - lo) : -1; }
// MFMA slot in whose shadow stage u of conversion pair g (of `pairs`) is issued.  Stages: 0 = both and-or,
// 1 = first packed add, 2 = second packed add, 3 = both packed multiplies.  A pair has slots / pairs slots to
// itself: with three or more the stages go and-or | adds | multiplies, with two and-or + add | add +
// multiplies, with one everything in that order (dependent instructions are never adjacent).
constexpr int stage_slot(int g, int u, int pairs, int slots) {
  const int base = g * slots / pairs;
  const int span = slots / pairs;
  const int off = (span >= 3) ? ((u == 0) ? 0 : (u == 3) ? 2 : 1) : (span == 2) ? ((u <= 1) ? 0 : 1) : 0;
  return (base + off < slots) ? base + off : slots - 1;
}

// Shape of a workgroup: WM x WN waves, each owning (32*RT) rows x (32*NT) columns (the WM waves of a
// column group share its packed weights, scales and zero-points), plus PW producer waves that do
// nothing but issue the async copies.  With PW = 0 the computing waves issue the copies themselves.
// ROW: quantization blocks run along N (one k, BS columns).  The scales and zero-points of a k tile are
// then, per group of BS columns, 64 consecutive rows in the packed order described in blkq4_device.h:
// 128 + 64 bytes, copied as they are.
template <int BS, int RT, int NT, int WM, int WN, int PW, bool ROW, int KW = 1>
struct Stage {
  static constexpr int kCopiers = (PW > 0) ? PW : WM * WN;     // waves that share out the copies of a stage
  static constexpr int kBlocks = kBK / BS;                     // quantization block rows per k tile
  static constexpr int kABytes = 32 * RT * WM * 128;           // [row][8 x 16-byte units, swizzled]
  static constexpr int kBBytes = WN * NT * 1024;               // [column group][fragment][lane] 16-byte units
  // blocks along K: [column group][block][2 fragments][64 B scales | 32 B zps | pad]
  // blocks along N: [group of BS columns][128 B scales], then [group][64 B zero-points] (at least 256 B:
  // one copy instruction writes 256 B)
  static constexpr int kGroups = 32 * NT * WN / BS;            // column groups of a workgroup tile (ROW)
  static constexpr int kRowScaleOps = kGroups / 2;             // copies of 2 x 128 B
  static constexpr int kRowZpOps = (kGroups + 3) / 4;          // copies of 4 x 64 B
  static constexpr int kMetaBytes = ROW ? kGroups * 128 + kRowZpOps * 256 : WN * kBlocks * 256;
  static constexpr int kBytes = kABytes + kBBytes + kMetaBytes;
  // per copying wave and stage: 8-row activation groups, packed weight fragments, scale / zero-point rows
  static constexpr int kAOps = (4 * RT * WM + kCopiers - 1) / kCopiers;
  static constexpr int kBOps = (NT * WN + kCopiers - 1) / kCopiers;
  static constexpr int kMTotal = ROW ? kRowScaleOps + kRowZpOps : WN * kBlocks;
  static constexpr int kMOps = (kMTotal + kCopiers - 1) / kCopiers;
  static constexpr int kOps = kAOps + kBOps + kMOps;
  // Ring of k tiles in LDS, requested kDistance tiles ahead of the one being consumed.  A tile must have landed one
  // k tile before it is consumed (the barrier in the middle of the tile before publishes it), so with four slots a
  // request has two k tiles' time to complete: enough for the large tiles, whose k tile takes 0.6 us and more, not
  // for the small ones (0.3 us).  Eight slots for those: M = 300, K = N = 4096 21.2 -> 18.8 us, M = 64, N = 18432 23.3 ->
  // 19.6, M = 256 19.0 -> 18.3, M = 512 (256 workgroups: bound by what L2 delivers) 23.6 -> 23.2.  Six slots for the
  // 128 x 128 tiles change nothing (+- 2 %), eight for the 256-column tiles of one row tile lose 5 %.
  static constexpr bool kDeep = PW > 0 && (RT * NT <= 2 || KW > 1);  // (waves that split the k tile: 8 MFMAs or fewer per tile)
  static constexpr int kStages = (kDeep && 8 * kBytes <= 160 * 1024) ? 8 : (4 * kBytes <= 160 * 1024) ? 4 : 3;
  static constexpr int kDistance = kStages - 1;  // the slot being refilled is the one nobody reads
  static_assert((kDistance - 1) * kOps <= 63, "more copies in flight than the counter holds");
};

// (BF repeats kBF so that the two compilations' kernels carry different names in a trace)
// SK: the last `split_tiles` tiles of the tile order are computed by `split_k` workgroups each (workgroup
// whole_tiles + u: tile whole_tiles + u % split_tiles, part u / split_tiles of its k tiles).  Such a workgroup
// leaves its fp32 partial tile in `partials` and counts itself in the tile's arrival counter; the one that
// arrives last adds the parts up in the order 0, 1, ..., split_k - 1 (so the result does not depend on who
// that is), clears the counter for the next launch and runs the epilogue.  Nobody waits for anybody.
// KW = 4: the four computing waves share ONE (32*RT) x (32*NT) tile and split every 64-deep k tile between them, wave w
// owning its 16-deep step w (WM = WN = 1).  A weight fragment is then converted once per RT MFMAs whatever the
// tile's width, which is what small problems need: with tiles of 128 x 32 every compute unit of the chip has a tile at
// M = 256, N = 4096 and converts 3.25 instructions' worth per MFMA, where 64 x 128 tiles of four 64 x 32 waves convert
// 6.5 and occupy half the chip (same process: 16.5 against 19.0 us, 17.8 with those tiles split in two along K).  The
// waves' accumulators are added up through LDS in the epilogue, in wave order.  (Tiles of 128 x 64 of this kind were
// measured too and are not built: 20.8 us on that problem and no problem found where they are ahead.)
template <int BS, bool HAS_ZP, int RT, int NT, int WM, int WN, int PW, bool ROW, bool SK, int KW = 1, bool BF = kBF>
__global__ __launch_bounds__(64 * (WM * WN * KW + PW))
    __attribute__((amdgpu_waves_per_eu((WM * WN * KW + PW) / 4, (WM * WN * KW + PW) / 4))) void gemm_mfma_kernel(
        const uint8_t* __restrict__ A, const uint8_t* __restrict__ W, const uint8_t* __restrict__ S,
        const uint8_t* __restrict__ Z, uint16_t* __restrict__ C, const uint16_t* __restrict__ bias, int M, int N,
        int K, int m_tiles, int whole_tiles, int split_tiles, int split_k, float* __restrict__ partials,
        int* __restrict__ counters, int xcd_map) {
  using St = Stage<BS, RT, NT, WM, WN, PW, ROW, KW>;
  constexpr int kComputeWaves = WM * WN * KW;
  constexpr bool KS = KW > 1;
  constexpr int kAhead = KS ? 2 : 1;
  static_assert(KW == 1 || (KW == 4 && WM == 1 && WN == 1 && PW > 0 && !ROW && !SK),
                "waves that split the k tile: four of them, one tile, producer waves, blocks along K, no split tiles");
  static_assert(!ROW || St::kGroups % 2 == 0, "scale copies take two column groups at a time");
  constexpr int kCopiers = St::kCopiers;
  static_assert((WM * WN * KW + PW) % 4 == 0, "whole waves per SIMD");
  constexpr int kBlocks = St::kBlocks;
  constexpr int kOps = St::kOps;
  constexpr int kStages = St::kStages;
  constexpr int kDistance = St::kDistance;
  constexpr int kBN = 32 * NT * WN;
  constexpr int kBM = 32 * RT * WM;
  constexpr int kMeta = (BS == 16) ? 2 : 1;  // quantization blocks inside a lane's 32-deep unit
  constexpr int kMfmas = RT * NT;            // MFMAs of one 16-deep k step
  // 32-row tiles, and 64-row tiles of eight waves, are launched for problems of one row tile only: every packed
  // weight is then read once per launch
  constexpr bool kWeightsOnce = RT == 1 || (RT == 2 && WN == 8);
  static_assert(kStages * St::kBytes <= 160 * 1024, "LDS ring does not fit");
  static_assert(NT == 1 || NT == 2, "the scale / zero-point copy covers at most two fragments");
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kStages * St::kBytes];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = KS ? 0 : (wave / WN) % WM;  // position of the wave's tile inside the workgroup tile
  const int wn = KS ? 0 : wave % WN;
  const int cw = (PW > 0) ? max(wave - kComputeWaves, 0) : wave;  // index among the copying waves
  const int lane = tid & 63;
  const int i = lane & 31;  // row of an activation fragment / column of a weight fragment
  const int h = lane >> 5;  // which 32-deep half of the 64-deep k tile this lane covers

  int tile = blockIdx.x;
  int part = 0;      // which share of the k tiles, of `parts`
  int parts = 1;
  if (SK && tile >= whole_tiles) {
    const int u = tile - whole_tiles;
    tile = whole_tiles + u % split_tiles;
    part = u / split_tiles;
    parts = split_k;
  }
  int bm = tile % m_tiles;
  int bn = tile / m_tiles;
  if (xcd_map != 0 && tile < (whole_tiles & ~255)) {
    // A whole round of 256 unsplit tiles (256 / m_tiles tile columns): workgroup w of the round runs on XCD w % 8, and
    // the 32 tiles of an XCD are made a block of (1 << rp) tile rows x (32 >> rp) tile columns, so that its L2 fetches
    // fewer rows and weights than with every eighth tile of the column-major order (encoding: xcd_tile_map()).
    const int xm = xcd_map & 15, rp = (xcd_map >> 4) & 15, cl = (xcd_map >> 8) & 15;
    const int wl = tile & 255, x = wl & 7, j = wl >> 3;
    bm = ((x & ((1 << xm) - 1)) << rp) + (j & ((1 << rp) - 1));
    bn = ((tile >> 8) << cl) + ((x >> xm) << (5 - rp)) + (j >> rp);
  }
  const int m0 = bm * kBM;
  const int nw0 = bn * kBN + wn * (32 * NT);
  // N is a multiple of 32, so 32-column fragments are whole; a fragment past the end re-reads the last one
  int nbase[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) nbase[t] = min(nw0 + 32 * t, N - 32);
  // this workgroup's k tiles: [kt_first, kt_first + KT)
  const int kt_first = SK ? static_cast<int>(static_cast<long>(K / kBK) * part / parts) : 0;
  const int KT = SK ? static_cast<int>(static_cast<long>(K / kBK) * (part + 1) / parts) - kt_first : K / kBK;
  if (SK) {
    A += static_cast<size_t>(kt_first) * 128;
    W += static_cast<size_t>(kt_first) * (static_cast<size_t>(N) * 32u);
  }

  // ---- per-lane byte offsets of the async copies inside k tile 0 ----
  constexpr int kAOps = St::kAOps;
  uint32_t a_off[kAOps];
  uint32_t a_dst[kAOps];  // LDS byte offset of the 8-row group inside the stage
#pragma unroll
  for (int p = 0; p < kAOps; ++p) {
    // 4*RT*WM groups of 8 rows are shared out over the copying waves; when the division leaves a
    // remainder some waves copy a group a second time (same bytes to the same place) so that every
    // wave has the same number of copies in flight
    const int group = (kCopiers * p + cw) % (4 * RT * WM);
    a_dst[p] = group * 1024;
    const int row = 8 * group + (lane >> 3);  // row inside the tile
    const int col = (lane & 7) ^ ((row >> 1) & 7);     // logical 16-byte column this lane fetches
    a_off[p] = static_cast<uint32_t>(min(m0 + row, M - 1)) * (static_cast<uint32_t>(K) * 2u) + col * 16;
  }
  // the NT*WN weight fragments of the workgroup tile, shared out the same way
  constexpr int kBOps = St::kBOps;
  uint32_t b_off[kBOps];
  uint32_t b_dst[kBOps];
#pragma unroll
  for (int p = 0; p < kBOps; ++p) {
    const int f = (kCopiers * p + cw) % (NT * WN);  // fragment f: column group f / NT, fragment f % NT
    const int nb = min(bn * kBN + 32 * f, N - 32);
    b_off[p] = (static_cast<uint32_t>(h) * N + nb + i) * 16u;
    b_dst[p] = St::kABytes + f * 1024;
  }
  const uint32_t b_stride = static_cast<uint32_t>(N) * 32u;  // two 32-deep units per k tile
  // meta, blocks along K: one copy per (column group, block row).  Per 32-lane half (= fragment): lanes
  // 0..15 fetch 2 scales each, lanes 16..23 fetch 4 zero-points each.  The copy lands at 4 * lane inside a
  // 256-byte row, so the lanes with nothing to fetch write into padding; they re-read a scale so that the
  // copy needs no branch.
  // meta, blocks along N: the 128 bytes of scales of two column groups per copy (32 lanes each), then the
  // 64 bytes of zero-points of four column groups per copy (16 lanes each); a group past N re-reads the
  // last one.
  constexpr int kMOps = St::kMOps;
  const bool meta_is_scale = i < 16 || i >= 24 || !HAS_ZP;
  const uint32_t meta_row_bytes = meta_is_scale ? static_cast<uint32_t>(N) * 2u : static_cast<uint32_t>(N);
  const uint8_t* meta_ptr[kMOps];
  uint32_t meta_dst[kMOps];
  uint32_t meta_step[kMOps];  // bytes from one k tile to the next
#pragma unroll
  for (int p = 0; p < kMOps; ++p) {
    const int idx = (kCopiers * p + cw) % St::kMTotal;
    if (ROW) {
      const int last_group = N / BS - 1;
      const int group0 = bn * kBN / BS;
      if (idx < St::kRowScaleOps) {
        const int grp = min(group0 + 2 * idx + (lane >> 5), last_group);
        meta_ptr[p] = S + (static_cast<size_t>(grp) * K) * 2 + (lane & 31) * 4;
        meta_dst[p] = St::kABytes + St::kBBytes + idx * 256;
        meta_step[p] = 128;
      } else {
        const int z = idx - St::kRowScaleOps;
        const int grp = min(group0 + min(4 * z + (lane >> 4), St::kGroups - 1), last_group);
        meta_ptr[p] = (HAS_ZP ? Z + static_cast<size_t>(grp) * K : S) + (lane & 15) * 4;
        meta_dst[p] = St::kABytes + St::kBBytes + St::kGroups * 128 + z * 256;
        meta_step[p] = 64;
      }
    } else {
      // column group idx / kBlocks, block row idx % kBlocks
      const int nb = min(bn * kBN + (idx / kBlocks) * (32 * NT) + ((NT == 2) ? 32 * h : 0), N - 32);
      meta_ptr[p] = (meta_is_scale ? S + static_cast<size_t>(nb + 2 * (i & 15)) * 2 : Z + (nb + 4 * (i & 7))) +
                    static_cast<size_t>(idx % kBlocks) * meta_row_bytes;
      meta_dst[p] = St::kABytes + St::kBBytes + idx * 256;
      meta_step[p] = kBlocks * meta_row_bytes;
    }
    if (SK) meta_ptr[p] += static_cast<size_t>(kt_first) * meta_step[p];
  }

  const uint32_t lds0 = static_cast<uint32_t>(
      reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)(&lds[0])));  // LDS byte address

  // Async copy number q (0 .. kOps-1) of k tile `tile_` into ring slot `stage_`:
  // q < kAOps: 8 activation rows; the next kBOps: packed weight fragments; above: one
  // scale/zero-point row (all fragments of the column group).
#define BLKQ4_COPY_OP(q_, tile_, stage_)                                                                  \
  {                                                                                                       \
    const uint32_t sbase_ = lds0 + (stage_) * St::kBytes;                                                 \
    if ((q_) < kAOps) {                                                                                   \
      async_copy_16(sbase_ + a_dst[(q_) < kAOps ? (q_) : 0], A + static_cast<size_t>(tile_) * 128,       \
                    a_off[(q_) < kAOps ? (q_) : 0]);                                                      \
    } else if ((q_) < kAOps + kBOps) {                                                                    \
      const int p_ = ((q_) >= kAOps && (q_) < kAOps + kBOps) ? (q_) - kAOps : 0;                           \
      if constexpr (kWeightsOnce) {                                                                       \
        async_copy_16_once(sbase_ + b_dst[p_], W + static_cast<size_t>(tile_) * b_stride, b_off[p_]);     \
      } else {                                                                                            \
        async_copy_16(sbase_ + b_dst[p_], W + static_cast<size_t>(tile_) * b_stride, b_off[p_]);          \
      }                                                                                                   \
    } else {                                                                                              \
      const int p_ = ((q_) >= kAOps + kBOps) ? (q_) - kAOps - kBOps : 0;                                   \
      async_copy_4_flat(sbase_ + meta_dst[p_], meta_ptr[p_] + static_cast<size_t>(tile_) * meta_step[p_]); \
    }                                                                                                     \
  }

  if (PW > 0 && wave >= kComputeWaves) {
    // Producer wave: requests k tiles kDistance ahead and meets the computing waves at their barrier
    // once per tile, after its copies for the tile they are about to start reading have landed.
#pragma unroll
    for (int s = 0; s < kDistance; ++s) {
#pragma unroll
      for (int q = 0; q < kOps; ++q) BLKQ4_COPY_OP(q, min(s, KT - 1), s);
    }
    // kAhead: how many tiles past the one being multiplied the computing waves read after a tile's barrier (the
    // waves that split the k tile read two ahead: their tile is short, and a read issued behind the barrier would be
    // needed before it can have arrived)
    static_assert(kDistance - 1 - kAhead >= 0, "the ring is too short for reading that far ahead");
    wait_vmcnt<(kDistance - kAhead) * kOps>();
    block_barrier();
    for (int kt = 0; kt < KT; ++kt) {
      // tile kt+kAhead must have landed: everything but the kDistance-1-kAhead newest groups (near the end
      // fewer groups than that are in flight, then wait for all of them)
      if (kt + kDistance <= KT) {
        wait_vmcnt<(kDistance - 1 - kAhead) * kOps>();
      } else {
        wait_vmcnt<0>();
      }
      block_barrier();  // also: nobody reads the slot of tile kt-1 any more
      if (kt + kDistance < KT) {
        const int stage = (kt + kDistance) % kStages;
#pragma unroll
        for (int q = 0; q < kOps; ++q) BLKQ4_COPY_OP(q, kt + kDistance, stage);
      }
    }
    wait_vmcnt<0>();
    return;
  }

  float16_t acc[RT][NT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[r][t][e] = 0.f;

  // ---- prologue: request tiles 0 .. kDistance-1, publish tile 0 ----
  // (when a tile's copies are spread over four steps, the second half of the last of these tiles is
  // issued by steps 0 and 1 of the first loop iteration, like every later one)
  constexpr int kPrologueLast = (St::kStages >= 4) ? (kOps * 2 / 4) : kOps;
  if (PW == 0) {
#pragma unroll
    for (int s = 0; s < kDistance; ++s) {
#pragma unroll
      for (int q = 0; q < ((s == kDistance - 1) ? kPrologueLast : kOps); ++q) BLKQ4_COPY_OP(q, min(s, KT - 1), s);
    }
    wait_vmcnt<(kDistance - 2) * kOps + kPrologueLast>();
  }
  block_barrier();

  // ---- LDS byte offsets of this lane's reads inside a stage ----
  // (LDS addresses, so that a read costs one addition of the ring slot's offset and nothing else)
  uint32_t a_rd[4];  // activation fragment of step j, row tile 0 (row tile r is 4096 bytes further)
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    a_rd[j] = lds0 + static_cast<uint32_t>(wm * (32 * RT) + i) * 128u + (((4 * h + j) ^ ((i >> 1) & 7)) * 16u);
  }
  const uint32_t b_rd = lds0 + St::kABytes + wn * (NT * 1024) + lane * 16;
  const uint32_t m_rd = lds0 + St::kABytes + St::kBBytes + wn * kBlocks * 256;
  // blocks along N: the 16-row groups 2h and 2h + 1 of the column group of this lane's column, per fragment
  uint32_t msc_rd[NT], mzp_rd[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int gl = (wn * (32 * NT) + 32 * t + i) / BS;
    msc_rd[t] = lds0 + St::kABytes + St::kBBytes + gl * 128 + h * 64;
    mzp_rd[t] = lds0 + St::kABytes + St::kBBytes + St::kGroups * 128 + gl * 64 + h * 32;
  }

  const DequantMasks masks = DequantMasks::make();
  const RowMetaMasks rmasks = RowMetaMasks::make();

#define BLKQ4_READ_A1(dst_, stage_off_, j_, r_) (dst_)[r_] = as_half8(lds_read_16((stage_off_) + a_rd[j_], (r_) * 4096))
  // packed words, scales and zero-points of all the wave's fragments for one k tile
#define BLKQ4_READ_B(words_, dc_, stage_ptr_)                                                \
  _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                           \
    const uint4 u_ = lds_read_16((stage_ptr_) + b_rd, t * 1024);                             \
    (words_)[t][0] = u_.x;                                                                   \
    (words_)[t][1] = u_.y;                                                                   \
    (words_)[t][2] = u_.z;                                                                   \
    (words_)[t][3] = u_.w;                                                                   \
    if (!ROW) {                                                                              \
      _Pragma("unroll") for (int q = 0; q < kMeta; ++q) {                                    \
        const int blk_ = (BS == 64) ? 0 : (BS == 32) ? h : (2 * h + q);                      \
        const uint32_t mb_ = (stage_ptr_) + m_rd + blk_ * 256;                               \
        (dc_##_sc)[t][q] = lds_read_u16(mb_ + i * 2, t * 128);                               \
        (dc_##_zp)[t][q] = HAS_ZP ? lds_read_u8(mb_ + i, t * 128 + 64) : 8u;                 \
      }                                                                                      \
    }                                                                                        \
  }
#define BLKQ4_MAKE_CONSTS(dc_)                                                                      \
  if (!ROW) {                                                                                       \
    _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                                \
      _Pragma("unroll") for (int q = 0; q < kMeta; ++q) {                                           \
        if constexpr (kBF) {                                                                        \
          (b##dc_)[t][q] = make_bf16_consts((dc_##_sc)[t][q], (dc_##_zp)[t][q]);                    \
        } else {                                                                                    \
          (dc_)[t][q] = make_dequant_consts((dc_##_sc)[t][q], (dc_##_zp)[t][q]);                    \
        }                                                                                           \
      }                                                                                             \
    }                                                                                               \
  }
  // blocks along N: scales (2 x 16 bytes) and zero-points (16 bytes) of 16-row group 2h + jj_ of every
  // fragment's column group, as they lie in memory
#define BLKQ4_READ_ROW_META(jj_, stage_off_)                                                     \
  if (ROW) {                                                                                     \
    _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                             \
      mrow_s[jj_][t][0] = lds_read_16((stage_off_) + msc_rd[t], (jj_) * 32);                     \
      mrow_s[jj_][t][1] = lds_read_16((stage_off_) + msc_rd[t], (jj_) * 32 + 16);                \
      if (HAS_ZP) mrow_z[jj_][t] = lds_read_16((stage_off_) + mzp_rd[t], (jj_) * 16);            \
    }                                                                                            \
  }
  // Piece y (0 .. 4*NT-1) of the conversion of word `w_` of every fragment into fragment buffer `dst_` is fp16
  // pair y % 4 of fragment y / 4.  Its three instructions depend on each other (and a packed instruction
  // that reads the result of the one before it costs a wait state), so two pieces are converted together,
  // stage by stage: AO = v_and_or_b32, PA = v_pk_add_f16, PM = v_pk_mul_f16.
#define BLKQ4_PIECE_AO(words_, w_, y_)                                                                     \
  pt[y_] = as_half2((((((y_) % 4) >= 2) ? ((words_)[(y_) / 4][w_] >> 8) : (words_)[(y_) / 4][w_]) &      \
                     ((((y_) & 1) == 0) ? masks.lo_mask : masks.hi_mask)) |                               \
                    ((((y_) & 1) == 0) ? masks.magic_1024 : masks.magic_64))
  // Blocks along N: word w_ of a lane's unit is rows 8 hh .. 8 hh + 7 (hh = w_ & 1) of 16-row group w_ / 2 of
  // the lane's 32 rows; pair p has its zero-points in byte pair hh of zero-point word p and its scales in
  // word 2 p + hh of the group (see blkq4_device.h for the packed order).
  // bf16: PA is the two mixed-precision fmas of the pair (fp16 operand 1024 + q resp. 64 + q, fp32 scale and constant),
  // PM the packed conversion of their results to bf16.
#define BLKQ4_PIECE_PA(dc_, q_, w_, y_)                                                                       \
  {                                                                                                           \
    if constexpr (kBF && !ROW) {                                                                              \
      const Bf16Consts& bc_ = (b##dc_)[(y_) / 4][q_];                                                         \
      pf[y_][0] = __builtin_fmaf(static_cast<float>(pt[y_][0]), bc_.scale, (((y_) & 1) == 0) ? bc_.neg_c0 : bc_.neg_c1); \
      pf[y_][1] = __builtin_fmaf(static_cast<float>(pt[y_][1]), bc_.scale, (((y_) & 1) == 0) ? bc_.neg_c0 : bc_.neg_c1); \
    } else {                                                                                                  \
      pt[y_] = pt[y_] + (ROW ? row_neg_c<HAS_ZP>(vec_word(mrow_z[(w_) >> 1][(y_) / 4], (y_) % 4), (y_) % 4, (w_)&1, rmasks) \
                         : ((((y_) & 1) == 0) ? (dc_)[(y_) / 4][q_].neg_c0 : (dc_)[(y_) / 4][q_].neg_c1));   \
    }                                                                                                         \
  }
#define BLKQ4_PIECE_PM(dst_, dc_, q_, w_, y_)                                                                \
  {                                                                                                          \
    if constexpr (kBF && !ROW) {                                                                             \
      bf16x2_t v_;                                                                                           \
      v_[0] = static_cast<__bf16>(pf[y_][0]);                                                                \
      v_[1] = static_cast<__bf16>(pf[y_][1]);                                                                \
      wp[dst_][(y_) / 4][(y_) % 4] = __builtin_bit_cast(half2_t, v_);                                        \
    } else if constexpr (kBF) {                                                                              \
      /* blocks along N: pt holds q - zp of the pair, each weight has its own bf16 scale */                  \
      wp[dst_][(y_) / 4][(y_) % 4] = as_half2(row_pair_bf16(                                                 \
          pt[y_], vec_word(mrow_s[(w_) >> 1][(y_) / 4][(2 * ((y_) % 4) + ((w_)&1)) >> 2],                    \
                           (2 * ((y_) % 4) + ((w_)&1)) & 3)));                                               \
    } else {                                                                                                 \
      wp[dst_][(y_) / 4][(y_) % 4] =                                                                         \
          pt[y_] * (ROW ? as_half2(vec_word(mrow_s[(w_) >> 1][(y_) / 4][(2 * ((y_) % 4) + ((w_)&1)) >> 2],   \
                                            (2 * ((y_) % 4) + ((w_)&1)) & 3))                                \
                        : (dc_)[(y_) / 4][q_].scale2);                                                       \
    }                                                                                                        \
  }
#define BLKQ4_PIECE(dst_, words_, w_, dc_, q_, y_) \
  BLKQ4_PIECE_AO(words_, w_, y_);                  \
  BLKQ4_PIECE_PA(dc_, q_, w_, y_);                 \
  BLKQ4_PIECE_PM(dst_, dc_, q_, w_, y_)
#define BLKQ4_WFRAG(slot_, t_) \
  __builtin_bit_cast(half8_t, half2x4_t{wp[slot_][t_][0], wp[slot_][t_][1], wp[slot_][t_][2], wp[slot_][t_][3]})

  struct half2x4_t {
    half2_t a, b, c, d;
  };

  half8_t af[2][RT];      // activation fragments, double buffered over the k steps
  half2_t wp[2][NT][4];   // weight fragments (4 fp16 pairs each), double buffered
  half2_t pt[4 * NT];     // pieces of a fragment on their way through the conversion
  float pf[4 * NT][2];    // bf16: the pieces as fp32 pairs between the fmas and the packed conversion
  uint32_t words[NT][4], nwords[NT][4];
  uint32_t dc_sc[NT][kMeta], dc_zp[NT][kMeta], ndc_sc[NT][kMeta], ndc_zp[NT][kMeta];
  DequantConsts dc[NT][kMeta], ndc[NT][kMeta];
  Bf16Consts bdc[NT][kMeta], bndc[NT][kMeta];  // bf16: these instead
  uint4 mrow_s[2][NT][2], mrow_z[2][NT];  // blocks along N: meta of 16-row groups 2h (steps 0, 1) and 2h + 1 (steps 2, 3)

  if constexpr (!KS) {
    const uint32_t s0 = 0;
    BLKQ4_READ_B(words, dc, s0);
    BLKQ4_READ_ROW_META(0, s0);
    BLKQ4_MAKE_CONSTS(dc);
#pragma unroll
    for (int r = 0; r < RT; ++r) BLKQ4_READ_A1(af[0], s0, 0, r);
#pragma unroll
    for (int x = 0; x < 4 * NT; ++x) {
      BLKQ4_PIECE(0, words, 0, dc, 0, x);
    }
  }

  if constexpr (KS) {
    // ---- waves that split the k tile ----
    // Wave `wave` owns the 16-deep step `wave` of every k tile: the activation fragments of that step, word `wave`
    // of every lane's packed unit, the scale and zero-point of the block that word lies in.  One barrier per k
    // tile, as in the other loop: it publishes tile kt + 1 and retires the slot of tile kt - 1.  Behind it the
    // wave reads tile kt + 1 from LDS and converts its weights in the shadow of tile kt's MFMAs.
    const uint32_t ks_a_rd = lds0 + static_cast<uint32_t>(i) * 128u + (((4 * h + wave) ^ ((i >> 1) & 7)) * 16u);
    const uint32_t ks_w_rd = lds0 + St::kABytes + lane * 16 + 4 * wave;
    const int ks_blk = (BS == 64) ? 0 : (BS == 32) ? h : (2 * h + (wave >> 1));
    const uint32_t ks_m_rd = lds0 + St::kABytes + St::kBBytes + ks_blk * 256 + i;
    // Two tiles are read ahead: behind the barrier of tile kt the wave asks LDS for tile kt + 2 (fragments into one of
    // four buffers, packed words and scales into one of two), converts tile kt + 1 from what it asked for a tile ago,
    // and multiplies tile kt.
    uint32_t kw_words[2][NT][1];
    uint32_t kw_sc[2][NT], kw_zp[2][NT];
    DequantConsts kdc[NT][1];
    Bf16Consts bkdc[NT][1];
    half8_t kaf[4][RT];
#define BLKQ4_KS_READ(abuf_, wbuf_, so_)                                                               \
  {                                                                                                    \
    _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                                   \
      kw_words[wbuf_][t][0] = lds_read_u32((so_) + ks_w_rd, t * 1024);                                 \
      kw_sc[wbuf_][t] = lds_read_u16((so_) + ks_m_rd + i, t * 128);                                    \
      kw_zp[wbuf_][t] = HAS_ZP ? lds_read_u8((so_) + ks_m_rd, t * 128 + 64) : 8u;                      \
    }                                                                                                  \
    _Pragma("unroll") for (int r = 0; r < RT; ++r) kaf[abuf_][r] = as_half8(lds_read_16((so_) + ks_a_rd, r * 4096)); \
  }
#define BLKQ4_KS_CONSTS(wbuf_)                                                                         \
  _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                                     \
    if constexpr (kBF) {                                                                               \
      bkdc[t][0] = make_bf16_consts(kw_sc[wbuf_][t], kw_zp[wbuf_][t]);                                 \
    } else {                                                                                           \
      kdc[t][0] = make_dequant_consts(kw_sc[wbuf_][t], kw_zp[wbuf_][t]);                               \
    }                                                                                                  \
  }
    // MFMA slot behind which pair g2 (of 2 * NT) of the next tile's fragments is converted: spread over the tile
    auto ks_pair_slot = [](int g2) constexpr { return g2 * kMfmas / (2 * NT); };
    BLKQ4_KS_READ(0, 0, 0u);
    BLKQ4_KS_CONSTS(0);
#pragma unroll
    for (int x = 0; x < 4 * NT; ++x) {
      BLKQ4_PIECE(0, kw_words[0], 0, kdc, 0, x);
    }
    BLKQ4_KS_READ(1, 1, static_cast<uint32_t>(St::kBytes));
    auto ks_tile = [&](const uint32_t sn2, auto cur_tag) __attribute__((always_inline)) {
      constexpr int cur = decltype(cur_tag)::value;  // tile kt modulo 4
      constexpr int wcur = cur & 1, wnext = 1 - wcur;
      block_barrier();
      BLKQ4_KS_READ((cur + 2) & 3, wcur, sn2);
      BLKQ4_PIN();
      BLKQ4_KS_CONSTS(wnext);
      half8_t wf_[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) wf_[t] = BLKQ4_WFRAG(wcur, t);
#pragma unroll
      for (int r = 0; r < RT; ++r) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const int x_ = r * NT + t;
          if constexpr (kBF) {
            acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wf_[t]),
                                                               __builtin_bit_cast(bf16x8_t, kaf[cur][r]), acc[r][t], 0, 0, 0);
          } else {
            acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf_[t], kaf[cur][r], acc[r][t], 0, 0, 0);
          }
#pragma unroll
          for (int g2 = 0; g2 < 2 * NT; ++g2) {
            if (ks_pair_slot(g2) == x_) {
              BLKQ4_PIECE_AO(kw_words[wnext], 0, 2 * g2);
              BLKQ4_PIECE_AO(kw_words[wnext], 0, 2 * g2 + 1);
              BLKQ4_PIECE_PA(kdc, 0, 0, 2 * g2);
              BLKQ4_PIECE_PA(kdc, 0, 0, 2 * g2 + 1);
              BLKQ4_PIECE_PM(wnext, kdc, 0, 0, 2 * g2);
              BLKQ4_PIECE_PM(wnext, kdc, 0, 0, 2 * g2 + 1);
            }
          }
          BLKQ4_PIN();
        }
      }
    };
    // ring slot of tile kt + 2, as a byte offset; four tiles per trip so that the register buffers are constants
    uint32_t sn2 = (2 % kStages) * St::kBytes;
    auto advance = [&]() { sn2 = (sn2 + St::kBytes == kStages * St::kBytes) ? 0u : sn2 + St::kBytes; };
    for (int kt = 0; kt < KT; kt += 4) {
      ks_tile(sn2, std::integral_constant<int, 0>{});
      advance();
      if (kt + 1 < KT) {
        ks_tile(sn2, std::integral_constant<int, 1>{});
        advance();
      }
      if (kt + 2 < KT) {
        ks_tile(sn2, std::integral_constant<int, 2>{});
        advance();
      }
      if (kt + 3 < KT) {
        ks_tile(sn2, std::integral_constant<int, 3>{});
        advance();
      }
    }
#undef BLKQ4_KS_READ
#undef BLKQ4_KS_CONSTS
  }

  // One 16-deep k step: RT*NT MFMAs on fragment buffers `cur_`; in their shadow the LDS reads of the
  // next step's activation fragments (from `nstage_`, step `nj_`), the conversion of the next weight
  // fragments (word `nw_` of `nwords_`) and, in the second half of a tile, the async copies
  // lo_ .. hi_-1 of k tile ctile_ (into ring slot cstage_), spread evenly over the step.
#define BLKQ4_STEP(cur_, nstage_, nj_, nwords_, nw_, ndc_, nq_, lo_, hi_, ctile_, cstage_)         \
  {                                                                                                \
    half8_t wf_[NT];                                                                               \
    _Pragma("unroll") for (int t = 0; t < NT; ++t) wf_[t] = BLKQ4_WFRAG(cur_, t);                  \
    _Pragma("unroll") for (int r = 0; r < RT; ++r) {                                               \
      _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                             \
        const int x_ = r * NT + t;                                                                 \
        if constexpr (kBF) {                                                                       \
          acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wf_[t]),  \
              __builtin_bit_cast(bf16x8_t, af[cur_][r]), acc[r][t], 0, 0, 0);                        \
        } else {                                                                                   \
          acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf_[t], af[cur_][r], acc[r][t], 0, 0, 0); \
        }                                                                                          \
        if (t == NT - 1) BLKQ4_READ_A1(af[1 - (cur_)], nstage_, nj_, r);                           \
        _Pragma("unroll") for (int g2 = 0; g2 < 2 * NT; ++g2) {                                    \
          /* stage u of the pair's conversion is issued behind MFMA stage_slot(g2, u, ...) */      \
          if (stage_slot(g2, 0, 2 * NT, kMfmas) == x_) {                                           \
            BLKQ4_PIECE_AO(nwords_, nw_, 2 * g2);                                                  \
            BLKQ4_PIECE_AO(nwords_, nw_, 2 * g2 + 1);                                              \
          }                                                                                        \
          if (stage_slot(g2, 1, 2 * NT, kMfmas) == x_) BLKQ4_PIECE_PA(ndc_, nq_, nw_, 2 * g2);     \
          if (stage_slot(g2, 2, 2 * NT, kMfmas) == x_) BLKQ4_PIECE_PA(ndc_, nq_, nw_, 2 * g2 + 1); \
          if (stage_slot(g2, 3, 2 * NT, kMfmas) == x_) {                                           \
            BLKQ4_PIECE_PM(1 - (cur_), ndc_, nq_, nw_, 2 * g2);                                    \
            BLKQ4_PIECE_PM(1 - (cur_), ndc_, nq_, nw_, 2 * g2 + 1);                                \
          }                                                                                        \
        }                                                                                          \
        _Pragma("unroll") for (int y = (lo_); y < (hi_); ++y) {                                    \
          if (copy_slot(y, lo_, hi_, kMfmas) == x_) BLKQ4_COPY_OP(y, ctile_, cstage_);             \
        }                                                                                          \
        BLKQ4_PIN();                                                                               \
      }                                                                                            \
    }                                                                                              \
  }
  // The copies of one k tile are issued over the four steps that follow the barrier which frees
  // their ring slot (two steps when the ring has only three slots and the tile is needed sooner).
  constexpr int kCopySteps = (PW > 0) ? 0 : (kStages >= 4) ? 4 : 2;  // 0: the producer waves copy
  constexpr int kCut1 = (kCopySteps == 0) ? 0 : kOps * 1 / (kCopySteps == 0 ? 1 : kCopySteps);
  constexpr int kCut2 = (kCopySteps == 4) ? kOps * 2 / 4 : (kCopySteps == 2) ? kOps : 0;
  constexpr int kCut3 = kOps * 3 / 4;

  // One k tile, in ring slot `stage` (a compile-time constant: the loop below is unrolled by the ring's depth by
  // hand -- the compiler does not unroll a loop with barriers whose trip count it does not know -- so that the
  // slots' offsets are constants and the hand-over of the next tile's words and constants costs no copies).
  auto k_tile = [&](const int kt, auto stage_tag) __attribute__((always_inline)) {
    constexpr int stage = decltype(stage_tag)::value;
    constexpr uint32_t sa = stage * St::kBytes;                           // tile kt: offset of its ring slot
    constexpr uint32_t sn = ((stage + 1) % kStages) * St::kBytes;         // tile kt + 1
    const int copy_tile = min(kt + kDistance, KT - 1);                    // clamped: re-fetches the last tile
    constexpr int copy_stage = (stage + kDistance) % kStages;
    const int late_tile = min(kt + kDistance - 1, KT - 1);                // the group begun in the previous tile
    constexpr int late_stage = (stage + kDistance - 1) % kStages;
    BLKQ4_PIN();

    // step 0: uses buffers 0; prepares step 1
    BLKQ4_READ_ROW_META(1, sa);
    BLKQ4_STEP(0, sa, 1, words, 1, dc, 0, (kCopySteps == 4 ? kCut2 : 0), (kCopySteps == 4 ? kCut3 : 0), late_tile, late_stage);
    // step 1: uses buffers 1; prepares step 2
    BLKQ4_STEP(1, sa, 2, words, 2, dc, kMeta - 1, (kCopySteps == 4 ? kCut3 : 0), (kCopySteps == 4 ? kOps : 0), late_tile, late_stage);
    // publish tile kt+1: this wave's copies for it have landed, then everybody's
    if (PW == 0) wait_vmcnt<(kDistance - 2) * kOps>();
    block_barrier();
    // step 2: uses buffers 0; prepares step 3, reads the next tile's weights, starts the copies
    BLKQ4_READ_B(nwords, ndc, sn);
    BLKQ4_READ_ROW_META(0, sn);
    BLKQ4_PIN();
    BLKQ4_STEP(0, sa, 3, words, 3, dc, kMeta - 1, 0, kCut1, copy_tile, copy_stage);
    // step 3: uses buffers 1; prepares step 0 of tile kt+1, finishes the copies
    BLKQ4_MAKE_CONSTS(ndc);
    BLKQ4_PIN();
    BLKQ4_STEP(1, sn, 0, nwords, 0, ndc, 0, kCut1, kCut2, copy_tile, copy_stage);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int j = 0; j < 4; ++j) words[t][j] = nwords[t][j];
#pragma unroll
      for (int q = 0; q < kMeta; ++q) {
        if constexpr (kBF) bdc[t][q] = bndc[t][q];
        else dc[t][q] = ndc[t][q];
      }
    }
  };
  for (int kt0 = 0; !KS && kt0 < KT; kt0 += kStages) {
    k_tile(kt0, std::integral_constant<int, 0>{});
    if (kt0 + 1 < KT) k_tile(kt0 + 1, std::integral_constant<int, 1>{});
    if (kt0 + 2 < KT) k_tile(kt0 + 2, std::integral_constant<int, 2>{});
    if constexpr (kStages > 3) {
      if (kt0 + 3 < KT) k_tile(kt0 + 3, std::integral_constant<int, 3>{});
    }
    if constexpr (kStages > 4) {
      if (kt0 + 4 < KT) k_tile(kt0 + 4, std::integral_constant<int, 4>{});
      if (kt0 + 5 < KT) k_tile(kt0 + 5, std::integral_constant<int, 5>{});
    }
    if constexpr (kStages > 6) {
      if (kt0 + 6 < KT) k_tile(kt0 + 6, std::integral_constant<int, 6>{});
      if (kt0 + 7 < KT) k_tile(kt0 + 7, std::integral_constant<int, 7>{});
    }
    static_assert(kStages == 3 || kStages == 4 || kStages == 6 || kStages == 8, "unrolled by hand for these ring depths");
  }
  if (PW == 0) wait_vmcnt<0>();  // the clamped re-fetches of the last tile are still in flight
#undef BLKQ4_COPY_OP
#undef BLKQ4_READ_A1
#undef BLKQ4_READ_B
#undef BLKQ4_MAKE_CONSTS
#undef BLKQ4_READ_ROW_META
#undef BLKQ4_PIECE
#undef BLKQ4_PIECE_AO
#undef BLKQ4_PIECE_PA
#undef BLKQ4_PIECE_PM
#undef BLKQ4_WFRAG
#undef BLKQ4_STEP

  // Epilogue.  Accumulator element 4*g + e of lane (i, h), fragment t, is output row m0 + 32*r + i and
  // column nw0 + 32*t + 8*g + 4*h + e.  Stored straight from there, a wave's store instruction would touch
  // 32 rows with 16 bytes each; instead every wave transposes its tile through a private piece of the
  // (now unused) LDS ring, four row tiles at a time, and stores whole rows of its tile: 16 bytes per lane,
  // 64*NT contiguous bytes per row.
  block_barrier();  // nobody reads the ring any more
  if (SK && parts > 1) {
    // Partial tile of (split tile st, part): [wave][row tile][fragment][g][half][lane] pairs of floats -- a
    // wave's store or load instruction covers 512 consecutive bytes.  The partial tiles and the counters are
    // exchanged between workgroups on different XCDs, whose L2 caches do not see each other's lines.  So, per
    // workgroup and not per wave (the cache operations act on the XCD's whole L2, and every invalidate throws
    // away the operands the other workgroups of the XCD are working on): once all waves' stores have completed,
    // ONE thread writes the L2's dirty lines back (release) and counts the workgroup in; in the workgroup that
    // arrives last, ONE thread invalidates (acquire) before anybody reads the other parts.  The accesses
    // themselves are device-scope atomic accesses, which bypass the compute unit's own cache.  (A workspace in
    // uncached memory needs none of the cache operations; measured, that saves 1 us of 18 and is not used.)
    constexpr int kTilePairs = kComputeWaves * RT * NT * 8 * 64;  // 8-byte pairs per partial tile
    constexpr uint32_t kFlagOffset = kStages * St::kBytes - 64;   // behind the epilogue's staging area
    const int st = tile - whole_tiles;
    uint64_t* const tile_parts = reinterpret_cast<uint64_t*>(partials) + static_cast<size_t>(st) * parts * kTilePairs +
                                 (wm * WN + wn) * (RT * NT * 8 * 64) + lane;
    uint64_t* const mine = tile_parts + static_cast<size_t>(part) * kTilePairs;
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int g2 = 0; g2 < 8; ++g2) {
          // (the elements are copied out first: a bit cast applied to a vector element directly was compiled
          // into a read of element 0)
          const float lo = acc[r][t][2 * g2], hi = acc[r][t][2 * g2 + 1];
          const uint64_t v = static_cast<uint64_t>(__float_as_uint(lo)) | static_cast<uint64_t>(__float_as_uint(hi)) << 32;
          __hip_atomic_store(mine + ((r * NT + t) * 8 + g2) * 64, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    wait_vmcnt<0>();  // this wave's stores have completed
    block_barrier();  // every wave's have
    if (tid == 0) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
      const int arrived = __hip_atomic_fetch_add(&counters[st], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (arrived == parts - 1) {
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        // nobody else touches this counter any more in this launch: back to zero for the next one
        __hip_atomic_store(&counters[st], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      lds_write_8(lds0 + kFlagOffset, 0, static_cast<uint32_t>(arrived), 0u);
    }
    block_barrier();
    const int arrived = static_cast<int>(lds_read_16(lds0 + kFlagOffset).x);
    if (arrived != parts - 1) return;  // somebody else finishes this tile
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[r][t][e] = 0.f;
    constexpr int kPieces = RT * NT * 8;                   // pairs per lane
    constexpr int kChunk = kPieces < 32 ? kPieces : 32;    // loaded at a time (registers)
    for (int p = 0; p < parts; ++p) {  // fixed order, whoever arrived last: 0 + part 0 + part 1 + ...
      const uint64_t* src = tile_parts + static_cast<size_t>(p) * kTilePairs;
#pragma unroll
      for (int x0 = 0; x0 < kPieces; x0 += kChunk) {
        uint64_t v[kChunk];
#pragma unroll
        for (int x = 0; x < kChunk; ++x) {
          v[x] = __hip_atomic_load(src + (x0 + x) * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int x = 0; x < kChunk; ++x) {
          const int rt_ = (x0 + x) / 8, g2 = (x0 + x) % 8;
          acc[rt_ / NT][rt_ % NT][2 * g2] += __uint_as_float(static_cast<uint32_t>(v[x]));
          acc[rt_ / NT][rt_ % NT][2 * g2 + 1] += __uint_as_float(static_cast<uint32_t>(v[x] >> 32));
        }
      }
    }
  }
  if constexpr (KS) {
    // The four waves' accumulators as fp32 tiles [wave][row][32 * NT columns + 4 of padding] in the (by now unused)
    // ring; then all 256 threads add them up in wave order, 8 columns per thread, and store whole rows.
    constexpr int kRowWords = 32 * NT + 4;  // rows start 4 banks apart: 16 lanes write, or read, all 64 banks once
    constexpr uint32_t kPartBytes = 32 * RT * kRowWords * 4;
    static_assert(KW * kPartBytes <= kStages * St::kBytes, "the waves' partial tiles do not fit in the ring");
    const uint32_t mine = lds0 + static_cast<uint32_t>(wave) * kPartBytes + static_cast<uint32_t>(i * kRowWords + 4 * h) * 4u;
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const float e0 = acc[r][t][4 * g], e1 = acc[r][t][4 * g + 1], e2 = acc[r][t][4 * g + 2], e3 = acc[r][t][4 * g + 3];
          lds_write_16(mine, (32 * r * kRowWords + 32 * t + 8 * g) * 4, __float_as_uint(e0), __float_as_uint(e1),
                       __float_as_uint(e2), __float_as_uint(e3));
        }
    block_barrier();
    constexpr int kChunks = 4 * NT;              // 16-byte chunks of a row of the output tile
    constexpr int kRowsPerPass = 256 / kChunks;  // all 256 threads of the computing waves
    const int chunk = tid % kChunks, srow = tid / kChunks;
    const int col = nw0 + chunk * 8;
    uint4 bias8 = make_uint4(0, 0, 0, 0);
    if (bias != nullptr && col < N) bias8 = *reinterpret_cast<const uint4*>(bias + col);
    const uint32_t rd = lds0 + static_cast<uint32_t>(srow * kRowWords + chunk * 8) * 4u;
#pragma unroll
    for (int it = 0; it < 32 * RT / kRowsPerPass; ++it) {
      float sum[8];
#pragma unroll
      for (int p = 0; p < KW; ++p) {
        const uint4 lo = lds_read_16(rd, p * kPartBytes + it * kRowsPerPass * kRowWords * 4);
        const uint4 hi = lds_read_16(rd, p * kPartBytes + it * kRowsPerPass * kRowWords * 4 + 16);
        const float v[8] = {__uint_as_float(lo.x), __uint_as_float(lo.y), __uint_as_float(lo.z), __uint_as_float(lo.w),
                            __uint_as_float(hi.x), __uint_as_float(hi.y), __uint_as_float(hi.z), __uint_as_float(hi.w)};
#pragma unroll
        for (int e = 0; e < 8; ++e) sum[e] = (p == 0) ? v[e] : sum[e] + v[e];
      }
      uint4 v = make_uint4(float_to_bits<kBF>(sum[0]) | (float_to_bits<kBF>(sum[1]) << 16),
                           float_to_bits<kBF>(sum[2]) | (float_to_bits<kBF>(sum[3]) << 16),
                           float_to_bits<kBF>(sum[4]) | (float_to_bits<kBF>(sum[5]) << 16),
                           float_to_bits<kBF>(sum[6]) | (float_to_bits<kBF>(sum[7]) << 16));
      if (bias != nullptr) {
        v = make_uint4(add_bias_pair_t<kBF>(v.x, bias8.x), add_bias_pair_t<kBF>(v.y, bias8.y),
                       add_bias_pair_t<kBF>(v.z, bias8.z), add_bias_pair_t<kBF>(v.w, bias8.w));
      }
      const int m = m0 + it * kRowsPerPass + srow;
      if (m < M && col < N) {
        __builtin_nontemporal_store(uint4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<uint4_t*>(C + static_cast<size_t>(m) * N + col));
      }
    }
  } else {
    constexpr int kRowBytes = 64 * NT + 16;        // padded: consecutive rows start 4 (NT=2: 36) banks apart
    constexpr int kPassTiles = (RT < 4) ? RT : 4;  // row tiles staged at a time
    constexpr int kChunks = 4 * NT;                // 16-byte chunks per row
    constexpr int kRowsPerStore = 64 / kChunks;
    static_assert(kComputeWaves * 32 * kPassTiles * kRowBytes <= kStages * St::kBytes - 64, "staging area does not fit");
    const uint32_t region = lds0 + (wm * WN + wn) * (32 * kPassTiles * kRowBytes);
    const int srow = lane / kChunks, chunk = lane % kChunks;
    const int col = nw0 + chunk * 8;
    // the lane stores the same 8 columns of every row: their bias values are fetched once
    uint4 bias8 = make_uint4(0, 0, 0, 0);
    if (bias != nullptr && col < N) bias8 = *reinterpret_cast<const uint4*>(bias + col);
#pragma unroll
    for (int r0 = 0; r0 < RT; r0 += kPassTiles) {
#pragma unroll
      for (int r = r0; r < r0 + kPassTiles && r < RT; ++r) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const uint32_t lo = float_to_bits<kBF>(acc[r][t][4 * g + 0]) | (float_to_bits<kBF>(acc[r][t][4 * g + 1]) << 16);
            const uint32_t hi = float_to_bits<kBF>(acc[r][t][4 * g + 2]) | (float_to_bits<kBF>(acc[r][t][4 * g + 3]) << 16);
            lds_write_8(region + ((r - r0) * 32 + i) * kRowBytes + h * 8, t * 64 + g * 16, lo, hi);
          }
        }
      }
#pragma unroll
      for (int it = 0; it < 32 * kPassTiles / kRowsPerStore; ++it) {
        const int row = it * kRowsPerStore + srow;  // inside the pass
        uint4 v = lds_read_16(region + srow * kRowBytes + chunk * 16, it * kRowsPerStore * kRowBytes);
        if (bias != nullptr) {
          v = make_uint4(add_bias_pair_t<kBF>(v.x, bias8.x), add_bias_pair_t<kBF>(v.y, bias8.y),
                         add_bias_pair_t<kBF>(v.z, bias8.z), add_bias_pair_t<kBF>(v.w, bias8.w));
        }
        const int m = m0 + wm * (32 * RT) + r0 * 32 + row;
        if (m < M && col < N) {  // written once, not read again by this launch
          __builtin_nontemporal_store(uint4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<uint4_t*>(C + static_cast<size_t>(m) * N + col));
        }
      }
    }
  }
}

template <int BS, bool HAS_ZP, int RT, int NT, int WM, int WN, int PW, bool ROW, bool SK, int KW = 1>
int launch_one(const blkq4_gemm_args* a) {
  constexpr int BM = 32 * RT * WM;
  constexpr int kBN = 32 * NT * WN;
  const blkq4_tile_plan& t = a->tile;
  const int m_tiles = (a->m + BM - 1) / BM;
  const int n_tiles = (a->n + kBN - 1) / kBN;
  const int tiles = m_tiles * n_tiles;
  if (a->launched_id != nullptr) *a->launched_id = tile_id(RT, NT, WM, WN, PW, SK, KW);
  int whole = tiles, split_tiles = 0, split_k = 1;
  float* partials = nullptr;
  int* counters = nullptr;
  if (SK) {
    // what the kernel assumes about the workspace, checked here: counters first, then the partial tiles
    split_tiles = t.split_tiles;
    split_k = t.split_k;
    whole = tiles - split_tiles;
    const size_t need = kCounterBytes + static_cast<size_t>(split_tiles) * split_k * BM * kBN * 4;
    if (split_tiles < 1 || split_tiles > tiles || split_k < 2 || split_k > a->k / kBK ||
        static_cast<size_t>(split_tiles) * sizeof(int) > kCounterBytes || t.workspace_bytes != need) {
      return static_cast<int>(hipErrorInvalidValue);
    }
    if (a->dry_run) return 0;  // the plan has passed every check a launch makes but those of the buffer itself
    if (a->workspace == nullptr || a->workspace_bytes < need || (reinterpret_cast<uintptr_t>(a->workspace) & 255u) != 0) {
      return static_cast<int>(hipErrorInvalidValue);
    }
    counters = static_cast<int*>(a->workspace);
    partials = reinterpret_cast<float*>(static_cast<char*>(a->workspace) + kCounterBytes);
  }
  if (t.tiles != tiles) return static_cast<int>(hipErrorInvalidValue);
  // the tile order inside whole rounds: 0 (every eighth tile of the column-major order per XCD) or blocks
  int xcd_map = 0;
  if (t.xcd_rows != 0 && !xcd_tile_map(m_tiles, t.xcd_rows, &xcd_map)) return static_cast<int>(hipErrorInvalidValue);
  if (a->dry_run) return 0;
  const dim3 grid(static_cast<unsigned>(whole + split_tiles * split_k));
  // the launch's own status: a sticky error of an earlier, unrelated call stays where it is
  return static_cast<int>(launch_status(gemm_mfma_kernel<BS, HAS_ZP, RT, NT, WM, WN, PW, ROW, SK, KW>, grid,
                                        dim3(64 * (WM * WN * KW + PW)), 0, a->stream, static_cast<const uint8_t*>(a->a),
                                        static_cast<const uint8_t*>(a->packed_w),
                                        static_cast<const uint8_t*>(a->scales),
                                        static_cast<const uint8_t*>(a->zero_points), static_cast<uint16_t*>(a->c),
                                        static_cast<const uint16_t*>(a->bias), a->m, a->n, a->k, m_tiles, whole,
                                        split_tiles, split_k, partials, counters, xcd_map));
}

// The tile shapes that exist, (RT, NT, WM, WN, PW): what blkq4::choose() may ask for.  Those with whole rows
// of 32 or 64 (one row tile only) have no split form and no form for blocks along N.
#define BLKQ4_TILE_SHAPES(X) X(8, 2, 1, 4, 0) X(8, 1, 1, 4, 4) X(4, 2, 1, 4, 4) X(4, 1, 1, 4, 4) X(2, 1, 1, 4, 4)
#define BLKQ4_TILE_SHAPES_ONE_ROW_TILE(X) X(1, 1, 1, 4, 4) X(1, 1, 1, 8, 0) X(2, 1, 1, 8, 0)
// (RT, NT) of the tiles whose four computing waves split the k tile (one tile per workgroup, four producer waves);
// blocks along K, no split form
#define BLKQ4_TILE_SHAPES_K_SPLIT_WAVES(X) X(4, 1)

template <int BS, bool HAS_ZP>
int launch_plan(const blkq4_gemm_args* a) {
  const blkq4_tile_plan& t = a->tile;
  const bool sk = t.split_k > 1;
#define BLKQ4_TRY(RT_, NT_)                                                                            \
  if (t.kw == 4 && t.rt == RT_ && t.nt == NT_ && t.wm == 1 && t.wn == 1 && t.pw == 4 && a->column_wise && !sk) { \
    return launch_one<BS, HAS_ZP, RT_, NT_, 1, 1, 4, false, false, 4>(a);                               \
  }
  BLKQ4_TILE_SHAPES_K_SPLIT_WAVES(BLKQ4_TRY)
#undef BLKQ4_TRY
  if (t.kw != 1) return static_cast<int>(hipErrorInvalidValue);
#define BLKQ4_TRY(RT_, NT_, WM_, WN_, PW_)                                                              \
  if (t.rt == RT_ && t.nt == NT_ && t.wm == WM_ && t.wn == WN_ && t.pw == PW_) {                        \
    if (a->column_wise) {                                                                               \
      return sk ? launch_one<BS, HAS_ZP, RT_, NT_, WM_, WN_, PW_, false, true>(a)                       \
                : launch_one<BS, HAS_ZP, RT_, NT_, WM_, WN_, PW_, false, false>(a);                     \
    }                                                                                                   \
    return sk ? launch_one<BS, HAS_ZP, RT_, NT_, WM_, WN_, PW_, true, true>(a)                          \
              : launch_one<BS, HAS_ZP, RT_, NT_, WM_, WN_, PW_, true, false>(a);                        \
  }
  BLKQ4_TILE_SHAPES(BLKQ4_TRY)
#undef BLKQ4_TRY
#define BLKQ4_TRY(RT_, NT_, WM_, WN_, PW_)                                                              \
  if (t.rt == RT_ && t.nt == NT_ && t.wm == WM_ && t.wn == WN_ && t.pw == PW_ && a->column_wise && !sk) { \
    return launch_one<BS, HAS_ZP, RT_, NT_, WM_, WN_, PW_, false, false>(a);                            \
  }
  BLKQ4_TILE_SHAPES_ONE_ROW_TILE(BLKQ4_TRY)
#undef BLKQ4_TRY
  return static_cast<int>(hipErrorInvalidValue);  // a shape that does not exist
}

template <int BS>
int launch_bs(const blkq4_gemm_args* a) {
  return a->zero_points ? launch_plan<BS, true>(a) : launch_plan<BS, false>(a);
}

}  // namespace

extern "C" int BLKQ4_GEMM_ENTRY(const blkq4_gemm_args* a) {
  if (a->m < 1 || (a->n % 32) != 0 || a->n < 32 || (a->k % 64) != 0) return static_cast<int>(hipErrorInvalidValue);
  if (!a->column_wise && ((a->n % a->block_size) != 0 || (reinterpret_cast<uintptr_t>(a->scales) & 3u) != 0 ||
                          (reinterpret_cast<uintptr_t>(a->zero_points) & 3u) != 0)) {
    return static_cast<int>(hipErrorInvalidValue);  // the meta data are copied four bytes at a time
  }
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
