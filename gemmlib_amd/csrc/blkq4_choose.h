// Which kernel multiplies a given problem, and in which shape: the ONE place where the thresholds live.
// Host-only, plain C++ (no HIP headers): blkq4_api.cpp asks blkq4::choose(), hands the answer to the launchers
// inside blkq4_gemm_args, and the launchers (blkq4_gemm.hip, blkq4_skinny.hip) map it to a kernel instantiation
// without any threshold of their own.
//
// The reference switches kernels at m > 16 and knows two tile shapes (src/blkq4_f16_gemm_sm80.cu:343,
// src/mickey/blk_q4/f16_gemm_sm80.h:63-72); everything below is this library's own cost model, fitted to
// measurements on MI355X.

#pragma once

#include <stddef.h>
#include <stdint.h>

#include <initializer_list>

#include "blkq4_device.h"

namespace blkq4 {

constexpr int kComputeUnits = 256;
constexpr size_t kMaxLdsBytes = 160 * 1024;
constexpr int kStreamingMaxRows = 1024;

// Where the streaming kernel's waves find their activation fragments.
constexpr int kRowsWholeInLds = 1;    // all rows, all of K, staged once per workgroup
constexpr int kRowsPerSlotInLds = 2;  // 16 * MT rows x 128 k staged per slot, private to the wave

constexpr int kFamilyStreaming = 0;  // weight-streaming kernel (blkq4_skinny.hip)
constexpr int kFamilyTile = 1;       // MFMA tile kernel (blkq4_gemm.hip)
constexpr int kFamilyDecode = 2;     // decode kernel (blkq4_decode.hip)

using StreamingShape = blkq4_streaming_plan;  // see blkq4_device.h
using TileShape = blkq4_tile_plan;
using DecodeShape = blkq4_decode_plan;

struct Choice {
  int family;
  StreamingShape s;
  TileShape t;
  DecodeShape d;
};

// A kernel's identity as one number: what choose() picked and what a launcher started can be compared.
inline uint64_t streaming_id(int depth, int nt, int mt, int waves, int am, int split, bool refill) {
  return 1ull << 60 | static_cast<uint64_t>(depth) << 40 | static_cast<uint64_t>(nt) << 32 |
         static_cast<uint64_t>(mt) << 24 | static_cast<uint64_t>(waves) << 16 | static_cast<uint64_t>(am) << 12 |
         static_cast<uint64_t>(split) << 4 | (refill ? 1u : 0u);
}
inline uint64_t tile_id(int rt, int nt, int wm, int wn, int pw, bool split, int kw = 1) {
  return 2ull << 60 | static_cast<uint64_t>(rt) << 40 | static_cast<uint64_t>(nt) << 32 |
         static_cast<uint64_t>(wm) << 24 | static_cast<uint64_t>(wn) << 16 | static_cast<uint64_t>(pw) << 8 |
         static_cast<uint64_t>(kw) << 4 | (split ? 1u : 0u);
}
// the GEMV without MFMA (blkq4_gemv.hip; run only when asked for by name): rows kept (1, 2 or 4) and waves of a
// workgroup
inline int valu_gemv_rows(int m) { return m == 1 ? 1 : m == 2 ? 2 : 4; }
inline int valu_gemv_waves(int k) {
  // sixteen waves when every one of them gets at least two 128-deep slices, else eight, else four
  const int slices = (k / 32 + 3) / 4;
  return slices >= 32 ? 16 : slices >= 16 ? 8 : 4;
}
inline uint64_t valu_gemv_id(int rows, int waves) {
  return 3ull << 60 | static_cast<uint64_t>(rows) << 8 | static_cast<uint64_t>(waves);
}
inline uint64_t decode_id(bool row, int rows, int nt, int waves, int depth) {
  return 4ull << 60 | static_cast<uint64_t>(row ? 1 : 0) << 32 | static_cast<uint64_t>(rows) << 24 | static_cast<uint64_t>(nt) << 16 |
         static_cast<uint64_t>(waves) << 8 | static_cast<uint64_t>(depth);
}
inline uint64_t choice_id(const Choice& c) {
  if (c.family == kFamilyDecode) return decode_id(c.d.row != 0, c.d.rows, c.d.nt, c.d.waves, c.d.depth);
  return c.family == kFamilyStreaming
             ? streaming_id(c.s.depth, c.s.nt, c.s.mt, c.s.waves, c.s.am, c.s.split, c.s.refill != 0)
             : tile_id(c.t.rt, c.t.nt, c.t.wm, c.t.wn, c.t.pw, c.t.split_k > 1, c.t.kw);
}

// ---------------------------------------------------------------------------------------------------------
// Decode kernel
// ---------------------------------------------------------------------------------------------------------

constexpr int kDecodeMaxRows = 16;
constexpr int kDecodeMaxDepth = 8;
constexpr int kDecodeMaxDepthSixteenWaves = 14;  // up to four rows: K up to 28672

// LDS of a workgroup: the rows of every wave's slices (256 bytes per row and slice), then the waves' partial
// tiles (64 bytes per row and tile), then, with blocks along N, the scales and zero-points of every wave's slices
// (256 + 128 bytes per slice)
inline size_t decode_lds_bytes(bool row, int rows, int nt, int waves, int depth) {
  return static_cast<size_t>(waves) * depth * 256 * rows + static_cast<size_t>(waves) * nt * rows * 64 +
         (row ? static_cast<size_t>(waves) * depth * 384 : 0);
}

// Workgroups: one per group of nt column tiles, rounded up to whole sets of 64 groups (the kernel hands eight
// neighbouring groups to each of the 8 XCDs in turn)
inline uint32_t decode_grid(int n, int nt) {
  const int groups = (n / 16 + nt - 1) / nt;
  return static_cast<uint32_t>((groups + 63) / 64 * 64);
}

// Up to four rows on wide layers with long K: the streaming kernel's workgroups of four to seven tiles, all resident at
// once, beat the decode kernel's rounds of single tiles
//   - two to four rows, K >= 8192, 1376 to 3584 column tiles (same process, decode against streaming: M = 4, K = 8192:
//     N = 28672 27.6 -> 26.7 us, N = 57344 58.2 -> 52.2, blocks of 16 with zero-points, N = 24576 31.0 -> 25.9; the worst
//     case found, M = 3, N = 22016 without zero-points, 19.7 -> 20.5; one row: 23.1 against 24.3, stays);
//   - one to four rows, K > 8192 (where the decode kernel needs sixteen waves), 832 to 1792 column tiles (M = 1:
//     K = 16384, N = 28672 51.1 -> 45.5 us, N = 13312 29.7 -> 25.1; K = N = 28672 87.0 -> 75.8; K = 8256, N = 13312 18.4 ->
//     14.9; K = 11008, N = 28672 with zero-points 42.6 -> 37.7, N = 14336 without 19.0 -> 20.6, the one loss found; on
//     wider layers the decode kernel is ahead again: K = 11008, N = 36864 41.4 against 44.0).
// At K = 4096 and on wider layers the decode kernel wins.
// (The first case later, against the decode kernel's eight waves with eight slices each and one tile per workgroup:
// with blocks of 32 or 64 two and three rows are 2 - 7 % faster in the decode kernel up to 1792 tiles -- M = 2, K = 8192,
// N = 22016 21.3 against 23.0 us, N = 28672 26.0 against 27.7 -- four rows level, N = 57344 level to 8 % behind; with blocks
// of 16 the streaming kernel is 10 - 15 % ahead throughout, N = 24576, M = 4 28.9 against 33.1.)
inline bool streaming_takes_few_rows(int m, int n, int k, int block_size = 64) {
  const int tiles = n / 16;
  if (m > 4) return false;
  if (k > 8192 && tiles >= 832 && tiles <= 1792) return true;
  if (m >= 2 && k >= 8192 && tiles >= 1376 && tiles <= 3584) return block_size < 32 || m == 4 || tiles > 1792;
  return false;
}

// The decode kernel's shape for m rows, or false when it has none or the streaming kernel is expected to be
// faster: blocks along K, at most kDecodeMaxRows rows, K in whole 128-deep slices, few enough of them for the waves
// to request them all at once and for the rows to fit in LDS, and packed weights that 32-bit offsets reach.
//
// Waves.  Eight by default (measured on M = 1, rotating weights, against 4 and 16 waves: K = 2048, N = 2048: 2.62
// against 2.74 and 2.68 us; K = 4096, N = 11008: 6.54 against 6.64 and 7.06; N = 128256: 49.1 against 50.2 and 58.3;
// K = 8192, N = 4096: 5.41 against 16 waves' 5.40), four for short K, sixteen when eight would have to request more
// than eight slices each (up to four rows only).  (Four waves with eight slices each for one workgroup per compute
// unit, K = N = 4096, were the rule once: without zero-points the two are level, 3.71 against 3.70 us; with zero-points
// eight waves take 3.70 against 3.86, in bf16 3.91 against 4.07.)
//
// Column tiles per workgroup.  The busiest compute unit works through ceil(workgroups / 256) workgroups of nt
// tiles each, and every workgroup costs a fraction of a tile's work on top: staging the rows, the instructions
// before the first request, the sum across the waves.  That fraction, fitted to sweeps over N = 4096 .. 28672 at
// K = 4096 and 8192: 0.1 for one row, 0.5 for more.  Two tiles with more than six slices per wave take a tenth
// longer than that (registers: fewer workgroups fit a compute unit), with five or six a twenty-fifth (M = 2 ... 4, K = 5120,
// N = 27648: two tiles 15.5 - 16.1 us, one 16.6 - 17.6), and with eight two fifths longer when they need more than one
// round (K = 8192, M = 2: N = 14336 17.8 us against 15.2 with one tile, N = 28672 34.5 against 26.0; with seven slices,
// K = 7168, N = 32768, M = 3, two tiles take 24.2 us and one 27.6).
//
// Eight and sixteen rows keep 64 to 128 KiB of rows per workgroup, so one or two workgroups fit a compute unit and a
// second round of them starts from nothing; once there are more rounds than that the streaming kernel, whose
// workgroups keep their rows and walk over the column tiles, is faster (M = 16, K = 4096, N = 28672: 17.2 against
// 20.9 us; M = 8, K = 8192, N = 14336: 15.5 against 18.4; but M = 16, K = 4096, N = 11008: 9.2 against 7.9).  Sixteen rows
// take up to four tiles per workgroup (all of LDS at K = 4096), which keeps layers of 12304 ... 16384 columns in one round:
// M = 9 ... 16, K = 4096, N = 14336 9.1 - 9.9 us against the streaming kernel's 10.4 - 10.9, N = 16384 10.1 against 11.1 (at
// N = 11008 three tiles stay ahead, 8.7 against 9.4); with eight rows a fourth tile gains nothing (N = 14336 8.6 against
// 8.7 with two, N = 16384 9.6 against 9.0).
inline bool decode_shape(bool column_wise, int m, int n, int k, DecodeShape* d, int block_size = 64) {
  if (m < 1 || m > kDecodeMaxRows || (k % 128) != 0 || (n % 16) != 0 ||
      static_cast<uint64_t>(k) * static_cast<uint64_t>(n) > (uint64_t{1} << 32)) {
    return false;
  }
  if (!column_wise) {
    // Blocks along N: up to four rows, one column tile per workgroup, eight waves with up to eight slices each
    // (four waves for short K and, with one row, for one workgroup per compute unit at most with eight slices each); the scales
    // and zero-points of a wave's slices, one of each per k, come through LDS.  (M = 1, K = N = 4096: 4.3 against
    // the streaming kernel's 5.3 us.)
    const int slices = k / 128;
    const int tiles = n / 16;
    if (m > 4 || slices > 8 * kDecodeMaxDepth) return false;
    // (two to four rows: eight waves there too, M = 4, K = N = 4096 4.67 against 5.02 us; one row: level, 4.57 and 4.62)
    const int waves = (slices <= 8 || (m == 1 && slices > 28 && slices <= 32 && tiles <= kComputeUnits)) ? 4 : 8;
    d->row = 1;
    d->rows = m == 1 ? 1 : 4;
    d->nt = 1;
    d->waves = waves;
    d->depth = (slices + waves - 1) / waves;
    d->grid = decode_grid(n, 1);
    d->lds_bytes = static_cast<uint32_t>(decode_lds_bytes(true, d->rows, 1, waves, d->depth));
    return true;
  }
  const int slices = k / 128;
  const int tiles = n / 16;
  if (streaming_takes_few_rows(m, n, k, block_size)) return false;
  const int rows = m == 1 ? 1 : m <= 4 ? 4 : m <= 8 ? 8 : 16;
  int waves = 8;
  if (rows <= 4) {
    if (slices <= 8) waves = 4;
    if (slices > 8 * kDecodeMaxDepth) waves = 16;
    if (slices > 16 * kDecodeMaxDepthSixteenWaves) return false;
    // K = N = 8192 (512 tiles, 64 slices): sixteen waves with four slices each, two such workgroups per compute unit
    // and all 512 resident at once, against two rounds of eight waves with eight or one round of two tiles
    // (M = 1 8.53 against 8.84 us, M = 2 8.88 against 9.99, M = 4 9.38 against 9.78; with 320 ... 448 tiles, N = 5120 ... 7168,
    // the eight waves stay 0 - 8 % ahead, and so they do with blocks of 16, whose scales are four times as many:
    // M = 3 11.2 us with two tiles against 12.4)
    if (waves == 8 && block_size >= 32 && slices > 56 && slices <= 64 && tiles > 448 && tiles <= 2 * kComputeUnits) waves = 16;
  }
  const int depth = (slices + waves - 1) / waves;
  if (depth > ((rows == 16) ? 4 : (rows <= 4 && waves == 16) ? kDecodeMaxDepthSixteenWaves : kDecodeMaxDepth)) return false;
  const int max_nt = rows == 16 ? 4 : rows == 8 ? 3 : (waves == 8 ? 2 : 1);  // the instantiations that exist
  const float per_workgroup = rows == 1 ? 0.1f : 0.5f;
  int nt = 1;
  float best = 0.f;
  for (int t = 1; t <= max_nt; ++t) {
    if (decode_lds_bytes(false, rows, t, waves, depth) > kMaxLdsBytes) break;
    const int wgs = (tiles + t - 1) / t;
    float cost = static_cast<float>((wgs + kComputeUnits - 1) / kComputeUnits) * (static_cast<float>(t) + per_workgroup);
    if (rows <= 4 && t == 2 && depth > 4) cost *= depth <= 6 ? 1.04f : (depth < 8 || wgs <= kComputeUnits) ? 1.1f : 1.4f;
    if (t == 1 || cost < best) {
      best = cost;
      nt = t;
    }
  }
  d->row = 0;
  d->rows = rows;
  d->nt = nt;
  d->waves = waves;
  d->depth = depth;
  d->grid = decode_grid(n, nt);
  d->lds_bytes = static_cast<uint32_t>(decode_lds_bytes(false, rows, nt, waves, depth));
  if (d->lds_bytes > kMaxLdsBytes) return false;
  if (rows >= 8) {
    const int per_unit = static_cast<size_t>(d->lds_bytes) * 2 <= kMaxLdsBytes ? 2 : 1;  // workgroups a compute unit holds
    const int rounds = ((tiles + nt - 1) / nt + kComputeUnits * per_unit - 1) / (kComputeUnits * per_unit);
    // (eight rows: two rounds of one workgroup per unit still win while a wave requests five slices: M = 6 ... 8, K = 5120,
    // N = 13824 and 15360 11.4 - 12.1 us against 12.7 - 13.5, the streaming kernel's rings asking for a fifth more
    // slices than K = 5120 has; with six, K = 6144, N = 14336 and 16384, 13.8 - 14.7 against 13.0 - 14.1)
    if (rounds > per_unit && !(rounds == 2 && rows == 8 && depth == 5)) return false;
  }
  return true;
}

// ---------------------------------------------------------------------------------------------------------
// Streaming kernel
// ---------------------------------------------------------------------------------------------------------

// Slices that `waves` waves with rings of `depth` slices request for one column group: every wave asks for
// whole rings, also when it has fewer slices left.
inline int requested_slices(int k, int waves, int depth) {
  const int slices = (k / 32 + 3) / 4;
  int total = 0;
  for (int w = 0; w < waves; ++w) {
    const int mine = (slices - w + waves - 1) / waves;
    total += (mine + depth - 1) / depth * depth;
  }
  return total;
}

// The kernel is bound by instruction issue as much as by the weight stream, so what matters is how
// evenly the workgroups fill the 256 compute units: with T column tiles per workgroup the busiest
// unit works through ceil(workgroups / 256) * T tiles.  Wider workgroups also re-read the activation
// rows less often, which weighs more the more rows there are.
inline void streaming_tiles_per_workgroup(int m, int n, int k, int* nt, int* depth) {
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

// Neighbouring column groups that the streaming kernel gives to one XCD one after the other: four while a column
// group is narrower than a 128-byte line of scales (16 columns a tile), so that the line is fetched into one L2; one
// from four tiles per group on, which deals the column groups to the eight XCDs evenly also when there are few of them
// (80 groups of four tiles, three row groups: in fours XCDs 0 - 3 get 36 workgroups for their 32 compute units and the
// others 24, and the launch takes two rounds, 28.9 us at M = 96, K = N = 5120; singly every XCD gets 30).
constexpr int streaming_neighbours(int nt, int waves, int split) { return (split == waves && nt >= 4) ? 1 : 4; }
// Workgroups on the busiest XCD (the first one, which gets most of what is left over), one column group each; and
// those per compute unit of it, rounded up: the rounds a launch of resident workgroups takes.
inline long streaming_busiest_xcd(int row_groups, int col_groups, int neighbours) {
  const int deal = 8 * neighbours;
  const int rest = col_groups % deal;
  const long busiest = static_cast<long>(neighbours) * (col_groups / deal) + (rest < neighbours ? rest : neighbours);
  return busiest * row_groups;
}
inline long streaming_rounds(int row_groups, int col_groups, int neighbours) {
  return (streaming_busiest_xcd(row_groups, col_groups, neighbours) + kComputeUnits / 8 - 1) / (kComputeUnits / 8);
}

// Launch geometry of one instantiation.  Many more workgroups than the chip holds at once: a workgroup then
// walks over several column groups (cg, cg + cg_stride, ...) and requests the first slices of the next one
// while it finishes the current one, so only the first column group of a workgroup waits for its weights with
// nothing else to do.  The partial tiles then get LDS of their own: the rows stay where they are for the next
// column group.  (not the sixteen-wave kernel for blocks along N: its walking variant does not fit in 128
// registers)
inline void streaming_geometry(StreamingShape* s, bool row, int n, int k) {
  constexpr int kPersistentFactor = 2;  // column groups per workgroup from which on workgroups walk
  // partial tiles of the sum across waves: [wave][tile][row tile][row][16 columns] floats, rows that exist only
  const size_t rows = s->mt == 1 ? (size_t{1} << s->rows_log2) : 16;
  const size_t red_bytes = (s->split == 1) ? 0 : static_cast<size_t>(s->waves) * s->nt * s->mt * rows * 64;
  const size_t per_slot_bytes = static_cast<size_t>(s->waves) * s->depth * 16 * s->mt * 256;
  // the rows are copied 1 KiB at a time
  const size_t a_bytes = s->am == kRowsWholeInLds
                             ? ((((static_cast<size_t>(k) * 2) << s->rows_log2) + 1023) & ~size_t{1023})
                             : per_slot_bytes;
  const int group_tiles = s->nt * (s->waves / s->split);
  const int col_groups = (n / 16 + group_tiles - 1) / group_tiles;
  const int per_xcd_round = 8 * streaming_neighbours(s->nt, s->waves, s->split);
  int cg_stride = (col_groups + per_xcd_round - 1) / per_xcd_round * per_xcd_round;  // one column group per workgroup
  // The partial tiles lie behind the rows when both fit (one barrier less: nobody has to wait until every wave
  // is done with the rows), else they reuse the rows' space.
  const bool separate = a_bytes + red_bytes <= kMaxLdsBytes;
  size_t lds_bytes = separate ? a_bytes + red_bytes : (a_bytes > red_bytes ? a_bytes : red_bytes);
  size_t red_offset = separate ? a_bytes : 0;
  const bool may_walk = !(row && s->waves == 16);
  if (may_walk && separate) {
    const int by_lds = static_cast<int>(kMaxLdsBytes / (a_bytes + red_bytes));
    const int by_waves = 32 / s->waves;
    const int resident = kComputeUnits * (by_lds < by_waves ? by_lds : by_waves);
    int stride = (resident / s->row_groups) / 32 * 32;
    if (stride < 32) stride = 32;
    if (cg_stride >= kPersistentFactor * stride) cg_stride = stride;
  }
  s->cg_stride = cg_stride;
  s->grid = static_cast<uint32_t>(cg_stride) * static_cast<uint32_t>(s->row_groups);
  s->lds_bytes = static_cast<uint32_t>(lds_bytes);
  s->red_offset = static_cast<uint32_t>(red_offset);
  // workgroups walk over several column groups, or waves stream all of K by themselves
  s->refill = (cg_stride < col_groups || s->split == 1) ? 1 : 0;
}

inline StreamingShape streaming_shape(bool row, int m, int n, int k, int block_size = 64) {
  StreamingShape s{};
  auto set = [&](int depth, int nt, int mt, int waves, int am, int split) {
    s.depth = depth; s.nt = nt; s.mt = mt; s.waves = waves; s.am = am; s.split = split;
  };
  s.row_groups = 1;
  if (m > 16) {
    // Row groups of 32 rows (two row tiles share one conversion of the weights), eight waves.  A workgroup's time
    // grows with its column tiles -- measured at K = 4096: 3.0 + 1.73 us per tile (M = 128, N = 4096 with 4, 6 and 8
    // tiles: 11.6, 15.2, 18.5 us) -- and an XCD with more workgroups than compute units takes longer than their number
    // says: 1.45 x workgroups per unit x one workgroup's time, at least the busiest unit's whole number of them
    // (M = 96, K = N = 4096: 3 per unit of one tile, 4.7 us each by that line, take 19.9 us, 1.5 per unit of two tiles,
    // 6.5 us each, 14.5; N = 5152: 1.97 per unit of two tiles 20.1).  As many tiles per workgroup (1, 2, 4, 6, 8) as make
    // that smallest (M = 64, N = 11008: 344 workgroups of four tiles 21.8 us, 230 of six 15.9; M = 96, N = 5152: two tiles
    // 20.1, six 15.5).  Blocks along N: 28 registers of packed weights, scales and zero-points per slot and tile, so one
    // tile.
    s.row_groups = (m + 31) / 32;
    s.rows_log2 = 5;
    int nt = 1;
    if (!row) {
      double best = 0.0;
      for (const int t : {1, 2, 4, 6, 8}) {
        const double per_unit = static_cast<double>(streaming_busiest_xcd(s.row_groups, (n / 16 + t - 1) / t, streaming_neighbours(t, 8, 8))) /
                                (kComputeUnits / 8);
        const double whole = static_cast<double>(static_cast<long>(per_unit + 0.999));  // the busiest unit's workgroups
        const double cost = (per_unit <= 1.0 ? 1.0 : (1.45 * per_unit > whole ? 1.45 * per_unit : whole)) * (3.0 + 1.73 * t);
        if (t == 1 || cost < best) {
          best = cost;
          nt = t;
        }
      }
    }
    // the rows whole in LDS only while they are a small part of it: at K = 2048 (128 KB) staging them slice by slice is
    // a tenth faster (M = 80 ... 128, N = 4096: 7.4 - 7.6 against 8.2 - 8.3 us), at K = 1024 they are level
    // (blocks along K; with blocks along N whole rows stay ahead, M = 24 ... 96, K = 2048: 8.1 - 11.6 against 9.8 - 15.7 us)
    const bool rows_fit = static_cast<size_t>(k) * 2 * 32 <= kMaxLdsBytes && (row || k <= 1536);
    set(2, nt, 2, 8, rows_fit ? kRowsWholeInLds : kRowsPerSlotInLds, 8);
    streaming_geometry(&s, row, n, k);
    return s;
  }
  while ((1 << s.rows_log2) < m) ++s.rows_log2;
  const size_t a_bytes = (((static_cast<size_t>(k) * 2) << s.rows_log2) + 1023) & ~size_t{1023};
  const bool rows_fit = a_bytes <= kMaxLdsBytes;
  const int tiles = n / 16;
  const int slices = (k / 32 + 3) / 4;
  auto done = [&]() {
    streaming_geometry(&s, row, n, k);
    return s;
  };
  {
    // Enough column tiles to give every wave the chip can hold one of its own, and rows small enough for
    // several workgroups per compute unit: the waves do not split K, each streams all of K for its own tile:
    // no sums across waves, no barriers, and a ring that stays full from the first slice to the last.
    // Break-even measured against workgroups that split K and walk (blocks along N gain more: their
    // sixteen-wave kernel has no walking variant); from 832 tiles on when K is no multiple of what the
    // splitting waves' rings hold, which then ask for a fifth more slices than there are (K = 5120,
    // N = 13824: 14.5 -> 12.7 us).  Four slices in flight per wave: with eight the kernel needs 90 registers
    // and a SIMD holds five waves instead of seven (52 against 55 us at N = 128256).
    // (blocks along N with more than four rows: whatever fits, one or two workgroups per compute unit -- M = 16, K = 4096,
    // N = 14336 16.7 against 20.2 us with waves that split K)
    // N = 14336 16.7 against 20.2 us with waves that split K -- as long as all workgroups are resident at once: with
    // N = 28672 and two rounds of them 31.6 against 26.2)
    size_t max_row_bytes = row ? 32 * 1024 : 16 * 1024;
    if (row && m > 4 && a_bytes <= kMaxLdsBytes &&
        (tiles + 3) / 4 <= kComputeUnits * static_cast<int>(kMaxLdsBytes / a_bytes)) {
      max_row_bytes = kMaxLdsBytes;
    }
    const bool rings_fit_k =
        5 * requested_slices(k, 16, 2) < 6 * slices || 5 * requested_slices(k, 8, 4) < 6 * slices;
    const int min_tiles = row ? 896 : rings_fit_k ? 2000 : 832;
    if (tiles >= min_tiles && a_bytes <= max_row_bytes) {
      set(4, 1, 1, 4, kRowsWholeInLds, 1);
      return done();
    }
  }
  if (!row && (!rows_fit || m > 4 || streaming_takes_few_rows(m, n, k, block_size)) && k >= 1024) {
    // Wide N and more than four rows, or K too long for the rows to stay in LDS: the rows are staged per
    // slice, a workgroup takes four column tiles (the rows are fetched again for every column group) and a
    // wave keeps two slices in flight, so that the slots are small enough for several workgroups per compute
    // unit: eight waves from 832 column tiles on, four from 1536 on.  Measured against every other shape of
    // workgroup: M = 16, K = 8192: N = 14336 24.3 -> 17.6 us, N = 28672 43.1 -> 34.1 us; rows that would fit
    // (M = 16, K = 4096, N = 14336: 13.2 -> 11.1 us) gain less or nothing, never lose more than 3 %.
    //
    // Tiles per workgroup and waves: every workgroup is resident from the start (no second round, no walking), and
    // the launch takes as long as the busiest compute unit, which has ceil(workgroups / 256) workgroups of nt
    // tiles each; a unit with four waves only hides a twelfth less of the latency, one with eight a fifteenth
    // (M = 16, K = 8192: N = 28672, 448 workgroups of four tiles and four waves 30.2 us, 256 of seven tiles and
    // eight waves 28.5, and four waves 29.6; N = 57344, 896 of four tiles 60.9, 512 of seven 52.1; N = 14336, 224
    // of four tiles and eight waves 17.3, and four waves 19.7, 128 of seven tiles 24.4).  Four tiles (four waves
    // from 1536 column tiles on, else eight) unless another shape promises 3 % less.
    if (tiles >= 832) {
      const size_t red_rows = size_t{1} << s.rows_log2;
      auto busiest = [&](int nt, int waves, bool all_resident) -> double {
        const size_t lds = static_cast<size_t>(waves) * 2 * 4096 + static_cast<size_t>(waves) * nt * red_rows * 64;
        const long by_lds = static_cast<long>(kMaxLdsBytes / lds), by_waves = 32 / waves;
        const long resident = by_lds < by_waves ? by_lds : by_waves;
        const long per_unit = ((tiles + nt - 1) / nt + kComputeUnits - 1) / kComputeUnits;
        if (all_resident && per_unit > resident) return -1.0;
        const long on_unit = per_unit * waves;
        return static_cast<double>(per_unit * nt) * (on_unit <= 4 ? 1.12 : on_unit <= 8 ? 1.07 : 1.0);
      };
      int nt = 4, waves = tiles >= 1536 ? 4 : 8;
      const double usual = busiest(nt, waves, false);
      double best = usual;
      for (const int w : {8, 4}) {
        for (const int t : {5, 6, 7}) {
          const double cost = busiest(t, w, true);
          if (cost > 0.0 && cost < best && cost < 0.97 * usual) {
            best = cost;
            nt = t;
            waves = w;
          }
        }
      }
      set(2, nt, 1, waves, kRowsPerSlotInLds, waves);
      return done();
    }
  }
  int nt, depth;
  streaming_tiles_per_workgroup(m, n, k, &nt, &depth);
  if (row) nt = 1;
  if (nt > 1) depth = 4;
  if (k >= 4096 && rows_fit) {
    // sixteen waves when there is enough K: each wave has less to convert after its last load has arrived,
    // and more of that work overlaps the loads of the other waves.  With more workgroups than compute units,
    // eight waves: smaller workgroups fill the units more evenly (M = 1, K = 4096, N = 14336: 11.4 -> 9.5 us),
    // unless their rings would ask for many more slices than K has.
    const int d8 = depth > 4 ? 4 : depth;
    const int col_groups = (tiles + nt - 1) / nt;
    if (!row && col_groups > kComputeUnits && 20 * requested_slices(k, 8, d8) <= 21 * requested_slices(k, 16, 2)) {
      set(d8, nt, 1, 8, kRowsWholeInLds, 8);
    } else if (row && m > 4 && k <= 8192) {
      // blocks along N, five to sixteen rows: eight waves with four slices in flight and the rows staged per slice
      // (measured against the sixteen-wave shape: M = 16, K = N = 4096 6.6 against 7.2 us, M = 8, N = 11008 15.8
      // against 16.9)
      set(4, 1, 1, 8, kRowsPerSlotInLds, 8);
    } else {
      set(2, nt, 1, 16, kRowsWholeInLds, 16);
    }
    return done();
  }
  if (k >= 1024) {
    // a wave asks for whole rings: rings of two slices when rings of four would ask for slices that do not exist
    // (K = 2048: 16 slices, eight waves with rings of four ask for 32)
    // (then one column tile per workgroup too: K = 2048, N = 8192: 5.9 -> 4.9 us)
    int d = depth > 4 ? 4 : depth;
    if (rows_fit && requested_slices(k, 8, 2) < requested_slices(k, 8, 4)) {
      d = 2;
      nt = 1;
    }
    set(d, nt, 1, 8, rows_fit ? kRowsWholeInLds : kRowsPerSlotInLds, 8);  // 8 * 4 * 4 KiB of rows
    return done();
  }
  set(depth, nt, 1, 4, kRowsWholeInLds, 4);  // K < 1024: at most 32 KiB of rows
  return done();
}

// ---------------------------------------------------------------------------------------------------------
// Tile kernel
// ---------------------------------------------------------------------------------------------------------

inline long ceil_div(long a, long b) { return (a + b - 1) / b; }

// The tile shapes, (rt, nt, wm, wn, pw): 64 x 128, 128 x 128 and 128 x 256 tiles of four computing waves
// (64 x 32, 128 x 32, 128 x 64 each) plus four producer waves that only issue copies, and 256 x 256 tiles of
// four waves of 256 x 64 (every register of a SIMD belongs to the one wave, which leaves no room for producer
// waves).  Larger tiles convert fewer weights per MFMA; smaller ones fill the chip with smaller problems.
constexpr int kTileShapes[4][5] = {{2, 1, 1, 4, 4}, {4, 1, 1, 4, 4}, {4, 2, 1, 4, 4}, {8, 2, 1, 4, 0}};

// Arrival counters first (one per split tile), then the fp32 partial tiles of the split tiles.
constexpr size_t kCounterBytes = 16 * 1024;  // room for 4096 split tiles
constexpr int kMinKTilesPerPart = 4;         // a part of a split tile is at least this many 64-deep k tiles
constexpr int kMaxSplit = 4;                 // the workgroup that arrives last reads all the parts by itself

inline size_t tile_workspace_bytes(const TileShape& t) {
  if (t.split_k <= 1) return 0;
  const size_t tile_elems = static_cast<size_t>(32 * t.rt * t.wm) * (32 * t.nt * t.wn);
  return kCounterBytes + static_cast<size_t>(t.split_tiles) * t.split_k * tile_elems * 4;
}

// Tile order inside a whole round of 256 unsplit tiles.  Workgroup w of a round runs on XCD w % 8 (round-robin
// dispatch), each XCD with an L2 of its own.  In the column-major tile order an XCD gets every eighth tile: with 8 or
// more tile rows that is m_tiles / 8 rows x ALL the round's columns.  xcd_rows = 1, 2, 4 or 8 cuts the round's
// m_tiles x (256 / m_tiles) rectangle into xcd_rows row bands x (8 / xcd_rows) column bands instead, one block per
// XCD.  Needs m_tiles to be a power of two between xcd_rows and 32 * xcd_rows.  The kernel's argument: log2 of
// xcd_rows, of the block's rows and of the round's columns, 4 bits each.
inline int log2_exact(int v) {
  int l = 0;
  while ((1 << l) < v) ++l;
  return (1 << l) == v ? l : -1;
}
inline bool xcd_tile_map(int m_tiles, int xcd_rows, int* map) {
  const int ml = log2_exact(m_tiles), xl = log2_exact(xcd_rows);
  if (ml < 0 || xl < 0 || ml > 8 || xl > 3 || xl > ml || ml - xl > 5) return false;
  *map = xl | (ml - xl) << 4 | (8 - ml) << 8 | 1 << 12;
  return true;
}

// Which cut to use: per k, the 32 tiles of an XCD make its L2 fetch (block rows) x 2 BM + (block columns) x BN / 2
// bytes.  Blocks are used when they fetch at most 0.8 of what every-eighth-tile fetches (the large tiles' time does
// not depend on it, the traffic through the fabric does: C4 fetches 66 instead of 83 MB).  Measured with forced plans
// (same process, us; 0 = every eighth tile, else xcd_rows): M = 512, K = N = 4096 in 64 x 128 tiles (8 tile rows: a whole
// row of 32 tiles per XCD, 71 MB through the fabric; 2 row bands make it 33 MB) 23.4 | 1: 22.6, 2: 21.6, 4: 22.3, 8: 23.0;
// nothing else moves by more than 1 %: M = 1024 in 128 x 128 tiles 33.6 | 33.5 - 33.9, C4 58.0 | 58.2 - 59.0,
// M = 512, N = 11008 in 128 x 128 tiles 53.9 | 53.1 - 54.2, M = 1024, K = N = 8192 114.0 | 112.6 - 114.0, C5 1500 - 1527 |
// 1500 - 1516.
inline int xcd_rows_for(const TileShape& t, int m) {
  const int bm = 32 * t.rt * t.wm, bn = 32 * t.nt * t.wn;
  const int m_tiles = static_cast<int>(ceil_div(m, bm));
  const int ml = log2_exact(m_tiles);
  if (ml < 0 || ml > 8 || t.tiles - t.split_tiles < kComputeUnits) return 0;
  auto fetched = [&](int xcd_rows) {
    const int rows = m_tiles / xcd_rows;
    return rows * bm * 4 + (32 / rows) * bn;
  };
  const int as_is = fetched(m_tiles < 8 ? m_tiles : 8);
  int best = 0, best_bytes = as_is;
  for (int xr = 1; xr <= 8 && xr <= m_tiles; xr *= 2) {
    if (m_tiles / xr > 32) continue;
    if (fetched(xr) < best_bytes) {
      best = xr;
      best_bytes = fetched(xr);
    }
  }
  return best_bytes * 10 <= as_is * 8 ? best : 0;
}

// Measured microseconds per 64-deep k tile of one workgroup when `busy` workgroups share the chip (fp16, blocks
// of 64 along K, K = 4096 ... 14336, N = 4096 ... 28672): flat while half the compute units idle, then rising with the
// load on the memory system and the clock the chip holds -- 64 x 128: 0.29 (<= 192 workgroups) to 0.33 (256),
// 128 x 128: 0.32 (<= 128) to 0.51, 128 x 256: 0.65 (<= 128) to 0.89, 256 x 256: 1.07 (<= 128) to 1.63 --
// and what a workgroup spends outside its main loop.  (Refitted after the loops were unrolled and the tiles dealt to
// the XCDs in blocks: 128 x 128 had been 0.37 to 0.575 and lost M = 384 ... 512 at K = 11008 to slower plans by 10 %.)
struct TileCost {
  double step_idle, step_slope, fixed;
  int flat_until;
};
// The constants were fitted on fp16 with blocks of 64 along K.  The other forms convert with more instructions per
// weight, which counts where the conversion is what a workgroup waits for; measured against that form, every plan, a k
// step takes, up to half a chip busy and on a full chip:
//   bf16 (50 shapes, M = 128 ... 1024): 64 x 128 tiles 1.30 and 1.14 x, 128 x 128 1.30 and 1.12, 128 x 256 1.16 and 1.04,
//     256 x 256 1.09 and 1.00; the 128 x 32 tiles whose waves split the k tile 0.99; the streaming kernel 1.06;
//   blocks along N (36 shapes, M = 128 ... 512): 1.24 and 1.15, 1.11 and 1.085, 1.02, 1.01 and 1.00;
//   blocks of 16 (36 shapes): 1.16 and 1.13, 1.14 and 1.09, 1.11 and 1.06, 1.075 and 1.04 (blocks of 32: as 64).
// Where several apply the factors multiply: bf16 with blocks of 16 measures 1.50 and 1.29, 1.39 and 1.20, 1.31 and 1.11,
// 1.20 (products: 1.51 and 1.29, 1.48 and 1.22, 1.29 and 1.10, 1.17), bf16 with blocks along N 1.72 and 1.41, 1.53 and
// 1.27, 1.31 and 1.10, 1.10 (1.61 and 1.31, 1.44 and 1.22, 1.18 and 1.06, 1.10; 24 shapes each).
// With fp16's constants for all, a copy of tile_plan() fed with the measured times of every plan picks a plan more than
// 5 % behind the best one for 4 of the 50, 3 of the 36 and 3 of the 36 shapes (up to 30 %: 128 x 128 tiles on half the
// chip where a split or a larger tile wins) and, with bf16's factors alone, for 7 and 3 of the 24 + 24 shapes of the
// combinations; with the factors as they are here for 1, 1, 0, 0 and 0.
enum TileCostRow { kCostPlain = 0, kCostBf16 = 1, kCostBlocksAlongN = 2, kCostBlocksOf16 = 4 };  // bits
inline int tile_cost_row(bool column_wise, bool bf16, int block_size) {
  return (bf16 ? kCostBf16 : 0) | (!column_wise ? kCostBlocksAlongN : 0) | (block_size == 16 ? kCostBlocksOf16 : 0);
}
inline TileCost tile_cost(const TileShape& t, int row = kCostPlain) {
  // 64 x 128, 128 x 128, 128 x 256, 256 x 256
  static constexpr TileCost kPlain[4] = {{0.29, 0.00065, 1.0, 192}, {0.32, 0.0015, 2.0, 128}, {0.65, 0.0019, 2.0, 128}, {1.07, 0.0044, 3.0, 128}};
  // factors on the k step of (up to flat_until workgroups, 256 workgroups) for bf16, blocks along N, blocks of 16
  static constexpr double kFactor[3][4][2] = {{{1.30, 1.14}, {1.30, 1.12}, {1.16, 1.04}, {1.09, 1.00}},
                                              {{1.24, 1.15}, {1.11, 1.085}, {1.02, 1.02}, {1.01, 1.00}},
                                              {{1.16, 1.13}, {1.14, 1.09}, {1.11, 1.06}, {1.075, 1.04}}};
  const int shape = t.rt == 8 ? 3 : (t.rt == 4 && t.nt == 2) ? 2 : t.rt == 4 ? 1 : (t.rt == 2 && t.wn == 4) ? 0 : -1;
  if (shape < 0) return {0.55, 0.0, 0.0, 256};  // tiles of one row tile (up to 64 rows)
  TileCost c = kPlain[shape];
  if (row == kCostPlain) return c;
  double idle = c.step_idle, full = c.step_idle + (kComputeUnits - c.flat_until) * c.step_slope;
  for (int bit = 0; bit < 3; ++bit) {
    if (row & (1 << bit)) {
      idle *= kFactor[bit][shape][0];
      full *= kFactor[bit][shape][1];
    }
  }
  c.step_idle = idle;
  c.step_slope = full > idle ? (full - idle) / (kComputeUnits - c.flat_until) : 0.0;
  return c;
}
inline double tile_round_us(const TileShape& t, int k_tiles, long busy, int row = kCostPlain) {
  const TileCost c = tile_cost(t, row);
  const long b = busy < kComputeUnits ? busy : kComputeUnits;
  return c.fixed + k_tiles * (c.step_idle + (b > c.flat_until ? (b - c.flat_until) * c.step_slope : 0.0));
}

// Tiles of 128 x 32 whose four computing waves split the k tile (kw = 4): only when one round of them covers the
// problem.  Fitted to measurements with 256 of them on the chip (fp16, blocks of 64, N = 4096 or 8192): K = 2048 10.3 us,
// 4096 16.4 - 16.9, 6144 24.7, 8192 30.2 -- 3.2 us outside the main loop (the sum of the four waves' accumulators
// through LDS is part of it) and 0.215 us per 64-deep k tile.  Against the other plans' estimates that hands them
// M = 129 ... 256 at N = 4096 up to K of about 5000 (same process, M = 256, K = N = 4096: 16.5 us against 19.0 in 64 x 128
// tiles, 17.8 with those split in two along K, 17.5 streaming; K = 6144: 24.7 against 23.4 split, which keeps it).
inline double k_split_waves_estimate_us(const TileShape& t, int k) {
  (void)t;
  return 3.2 + (k / 64) * 0.215;
}

// Estimated time of the tile kernel with shape t (split or not) on k: whole rounds of unsplit tiles, a last
// round of what is left of them, then one round of parts: their share of the k tiles, the partial tile
// written once and all parts read by the workgroup that arrives last (about 100 GB/s) plus 5 us for the cache
// write-back and invalidate and the two extra barriers (measured: 64 x 128 in 2 parts 17.7 - 19.1 us against
// 18.7 unsplit at M = 256, K = N = 4096; 128 x 128 in 3 parts 32.7 against 44.6 us at K = 11008).  Partial tiles of more
// than 24 MB in all no longer stay in the eight L2s (32 MB) until they are summed: 128 x 256 tiles in 4 parts on every
// compute unit (33.5 MB) take 7 us longer than the rest of the formula says (M = 512, N = 4096, K = 11008: 57.7 us, in
// 3 parts 56.2, 128 x 128 tiles in 2 parts 52.5).
inline double tile_estimate_us(const TileShape& t, int k, int row = kCostPlain) {
  if (t.kw > 1) return k_split_waves_estimate_us(t, k);
  const int kt = k / 64;
  const long whole = t.tiles - (t.split_k > 1 ? t.split_tiles : 0);
  double us = static_cast<double>(whole / kComputeUnits) * tile_round_us(t, kt, kComputeUnits, row);
  if (whole % kComputeUnits) us += tile_round_us(t, kt, whole % kComputeUnits, row);
  if (t.split_k > 1) {
    const long units = static_cast<long>(t.split_tiles) * t.split_k;
    const double tile_bytes = 4.0 * (32 * t.rt * t.wm) * (32 * t.nt * t.wn);
    // (256 x 256: the accumulators fill the registers and the workgroup that adds the parts up has one request in
    // flight at a time, 30 us per part -- by timestamps 118.6 us for four parts where a 128 x 256 tile's take 7.6;
    // M = 1280, N = 14336, K = 8192 in 256 x 256 tiles with the last 24 in 4 parts 366 us, unsplit 331, in 128 x 256 tiles
    // with the last 48 in 4 parts 260)
    const double bytes_per_us = t.rt == 8 ? 9e3 : 100e3;
    us += static_cast<double>(ceil_div(units, kComputeUnits)) *
          (tile_round_us(t, static_cast<int>(ceil_div(kt, t.split_k)), units, row) + 5.0 + (1 + t.split_k) * tile_bytes / bytes_per_us);
    const double partial_bytes = static_cast<double>(units) * tile_bytes;
    if (partial_bytes > 24e6) us += (partial_bytes - 24e6) / 1.36e6;
  }
  return us;
}

// Tiles of one row tile (up to 64 rows, blocks along K): a workgroup walks through K at a pace set by latency, not
// by the chip's load.  Measured over N = 2048 ... 32768 (16 -> 256 workgroups of 128 columns, four waves and four
// producer waves): K = 1024 (16 k tiles) 6.5 -> 7.3 us with up to 32 rows, 7.3 -> 9.5 with up to 64; K = 2048 10.0 ->
// 12.1 and 11.0 -> 15.8; K = 4096 17.5 -> 20.5 and 19.4 -> 27.4; 256 columns with eight waves 28.6 -> 31.7 us at
// K = 4096.  Whole rounds of 256 workgroups.
inline double one_row_tile_estimate_us(const TileShape& t, int k, int row = kCostPlain) {
  const long busy = t.tiles < kComputeUnits ? t.tiles : kComputeUnits;
  double step, fixed;
  if (t.wn != 4) {
    step = 0.40 + 0.0003 * busy;
    fixed = 2.9;
  } else if (t.rt == 1) {
    step = 0.22 + 0.0002 * busy;
    fixed = 2.85;
  } else {
    step = 0.25 + (busy > 128 ? (busy - 128) * 0.00097 : 0.0);
    fixed = 3.3;
    // the 64 x 128 tile of the general kernel: bf16 and blocks of 16 cost it what they cost there (bf16, M = 48,
    // N = 14336, K = 4096: 24.4 us unsplit where fp16 takes 19.4, 21.0 against 18.9 in 2 parts)
    if (row != kCostPlain) step *= tile_cost(t, row).step_idle / tile_cost(t, kCostPlain).step_idle;
  }
  return static_cast<double>(ceil_div(t.tiles, kComputeUnits)) * (fixed + (k / 64) * step);
}

// The 64 x 128 tile on 33 to 64 rows, unsplit or every tile in parts.  Split, no two workgroups share a weight and
// the chip's load counts for more than the general estimate says once more than 160 workgroups run: measured minus
// estimated (fp16, blocks of 64) 0 ... -1.3 us at 128 workgroups (N = 4096, K = 4096 ... 14336 in 4 parts), 0.7 at 160,
// 1.0 ... 1.5 at 172 ... 192 (16 ... 32 k tiles a part), 2.2 ... 2.9 at 216 ... 240, 3.0 and 4.5 at 256 (64 and 112 k
// tiles a part).
inline double few_rows_tile_estimate_us(const TileShape& t, int k, int row = kCostPlain) {
  if (t.split_k == 1) return one_row_tile_estimate_us(t, k, row);
  const long units = static_cast<long>(t.split_tiles) * t.split_k;
  double us = tile_estimate_us(t, k, row);
  if (units > 160) us += 1.5 + 0.023 * static_cast<double>(ceil_div(k / 64, t.split_k)) * static_cast<double>(units - 160) / 96.0;
  return us;
}

// The tile kernel's plan: the shape with the smallest estimate; when its last round of tiles would leave most
// of the chip idle and the estimate says it pays, those last `split_tiles` tiles are each shared out over
// split_k workgroups.  Up to 64 rows with blocks along K: tiles of one row tile, which fetch every packed
// weight once (128 columns with four waves and four producer waves, or 256 columns with eight waves, whichever
// one_row_tile_estimate_us() expects to be faster: the narrow ones up to one round of them, N = 32768).
inline TileShape tile_plan(bool column_wise, int m, int n, int k, size_t workspace_capacity, int row = kCostPlain) {
  TileShape best{};
  auto shape = [&](int rt, int nt, int wm, int wn, int pw) {
    TileShape t{};
    t.rt = rt; t.nt = nt; t.wm = wm; t.wn = wn; t.pw = pw;
    t.kw = 1;
    t.split_k = 1;
    t.tiles = static_cast<int>(ceil_div(m, 32 * rt * wm) * ceil_div(n, 32 * nt * wn));
    return t;
  };
  const int kt = k / 64;
  if (column_wise && m <= 64) {
    const int rt = m <= 32 ? 1 : 2;
    const TileShape narrow = shape(rt, 1, 1, 4, 4), wide = shape(rt, 1, 1, 8, 0);
    // (up to 32 rows the estimates of the tile and of the streaming kernel are those of fp16 with blocks of 64 for
    // every form)
    TileShape one = one_row_tile_estimate_us(narrow, k) <= one_row_tile_estimate_us(wide, k) ? narrow : wide;
    if (rt == 2) {
      // 33 to 64 rows on a layer that does not fill the chip: the 64 x 128 tile, which is the narrow shape here, has
      // a split form (M = 64, N = 5120, K = 13824: 23.0 us in 4 parts, 30.3 streaming, 55 unsplit; N = 8192, K = 28672:
      // 48.8, 62.9 and 110; N = 16384, K = 8192: 31.8 in 2 parts, 36.0 and 35.2)
      const double unsplit_us = one_row_tile_estimate_us(one, k, row);
      double best_us = unsplit_us;
      TileShape t = narrow;
      for (int split = 2; split <= kMaxSplit; ++split) {
        if (t.tiles * split > kComputeUnits || kt / split < kMinKTilesPerPart) break;
        if (split == 4 && t.tiles * 4 > 224 && kt < 128) continue;  // (as for more rows, below)
        t.split_k = split;
        t.split_tiles = t.tiles;
        t.workspace_bytes = tile_workspace_bytes(t);
        if (t.workspace_bytes > workspace_capacity || static_cast<size_t>(t.tiles) * sizeof(int) > kCounterBytes) continue;
        const double us = few_rows_tile_estimate_us(t, k, row);
        if (us < 0.95 * unsplit_us && us < best_us) {
          one = t;
          best_us = us;
        }
      }
    }
    return one;
  }
  double best_us = 0.0, best_unsplit_us = 0.0;
  for (const auto& sh : kTileShapes) {
    const TileShape t = shape(sh[0], sh[1], sh[2], sh[3], sh[4]);
    const double us = tile_estimate_us(t, k, row);
    if (best.rt == 0 || us < best_us) {
      best = t;
      best_us = us;
    }
  }
  best_unsplit_us = best_us;
  if (column_wise) {
    // 128 x 32 tiles of four waves that split the k tile, when one round of them covers the problem
    TileShape t = shape(4, 1, 1, 1, 4);
    t.kw = 4;
    if (t.tiles <= kComputeUnits) {
      const double us = k_split_waves_estimate_us(t, k);
      if (us < best_us) {  // (the bar a split plan has to clear stays that of the other unsplit shapes)
        best = t;
        best_us = us;
      }
    }
  }
  for (const auto& sh : kTileShapes) {
    TileShape t = shape(sh[0], sh[1], sh[2], sh[3], sh[4]);
    const int rem = t.tiles % kComputeUnits;
    if (rem == 0) continue;
    for (int split = 2; split <= kMaxSplit; ++split) {
      if (rem * split > kComputeUnits || kt / split < kMinKTilesPerPart) break;
      // A fourth part that fills the chip pays only with a long K: of 86 problems measured with 64 tiles in 4 parts, three
      // parts are faster for most below K = 8192 (median 6 %), four by 3 - 13 % at K = 11008; and with every compute unit
      // busy the last workgroups' invalidates hit the others' operands (M = 256, K = N = 4096, blocks along N, 128 x 128
      // tiles: 25 - 27 us in 4 parts on one box of the pool, 20.6 on the others, 20.2 in 3 parts on all).
      if (split == 4 && rem * 4 > 224 && kt < 128) continue;
      t.split_k = split;
      t.split_tiles = rem;
      t.workspace_bytes = tile_workspace_bytes(t);
      if (t.workspace_bytes > workspace_capacity || static_cast<size_t>(rem) * sizeof(int) > kCounterBytes) continue;
      const double us = tile_estimate_us(t, k, row);
      // a split has to promise a twentieth less than the best unsplit shape: its estimate is the less certain one
      if (us < 0.95 * best_unsplit_us && us < best_us) {
        best = t;
        best_us = us;
      }
    }
  }
  best.xcd_rows = xcd_rows_for(best, m);
  return best;
}

// Which kernel multiplies m rows.  The reference switches at m > 16 (src/blkq4_f16_gemm_sm80.cu:343,
// f16_gemm_sm80.h:63-72).  Here the weight-streaming kernel keeps going, in row groups of 32, for as long as
// it is expected to be faster than the tile kernel, whose grid cannot fill the chip when m is small.
// The streaming kernel's time grows with row groups x n x k (2.8 us per row group at n = k = 4096) and, once
// it has more workgroups than compute units, with whole rounds of them.
constexpr uint64_t kStreamingMaxWeights = uint64_t{1} << 33;

inline bool streaming_kernel_takes(bool column_wise, int m, int n, int k, const StreamingShape& s, double tile_us, int row = kCostPlain) {
  // its offsets into the packed weights (K N / 2 bytes) are 32 bits wide (so are the other kernels': the entry points
  // refuse such problems before any kernel is chosen)
  if (static_cast<uint64_t>(k) * static_cast<uint64_t>(n) >= kStreamingMaxWeights) return false;
  if (m <= 16) return true;
  if (m > kStreamingMaxRows) return false;
  const long row_groups = s.row_groups;
  const long streaming_groups = row_groups * ceil_div(n / 16, s.nt);
  // (row groups of 32: the waves split K, a column group is s.nt tiles)
  const long col_groups = ceil_div(n / 16, s.nt);
  const long rounds = s.cg_stride >= col_groups
                          ? streaming_rounds(s.row_groups, static_cast<int>(col_groups), streaming_neighbours(s.nt, s.waves, s.split))
                          : ceil_div(streaming_groups, kComputeUnits);
  if (column_wise && (m <= 64 || k < 4096)) {
    // (More row groups with a short K too: the product further down has no fixed part and said 5.6 us for M = 256,
    // K = 1024, N = 4096, which takes 11.3 -- and the 128 x 32 tiles whose waves split the k tile 6.7; this line says 12.1.
    // Of 63 shapes with M = 80 ... 384, K = 1024 ... 3072 sixteen went to the streaming kernel and lost 8 - 70 % by it.)
    // One or two row groups of 32, blocks along K: rounds of 256 workgroups, a workgroup's time growing with its
    // column tiles and K.  Least squares over 142 measurements (M = 24 ... 64, K = 1024 ... 4096, N = 2048 ... 32768;
    // within 15 % of all but a few, and of M = 128, K = N = 4096 and M = 40 ... 64, K = 8192, N = 16384 ... 18432, which
    // were not among them); against the tile kernel's estimate it picks the slower kernel for 0.2 % of the time
    // on them.  (M = 64, N = 18432: K = 4096 29.8 us streaming, 19.6 in tiles; K = 1024 17.2 and 8.7.  With the same
    // formula for three and four row groups M = 96, N = 8192 went to the tile kernel and took 20.1 instead of 19.4 us.)
    // Beyond K = 8192 a column tile costs more per k than that: with four of them and two row groups K = 8192 takes
    // 20.5 us (18.2 by the line above), 13824 30.2 (26.4), 28672 61 ... 63 (47.8), hence the square.
    const double kk = static_cast<double>(k) / 1024.0;
    double streaming_us = 3.2 + static_cast<double>(rounds) * (0.44 + s.nt * (0.69 + 0.37 * kk));
    if (kk > 8.0) streaming_us += static_cast<double>(rounds) * s.nt * 0.0075 * (kk - 8.0) * (kk - 8.0);
    // (33 to 64 rows, where the tile's estimate knows the form: the streaming kernel takes 1.06 x as long in bf16, 1.13 x
    // with blocks of 16 and 1.19 x with both as with fp16 and blocks of 64, same plans)
    if (m > 32) streaming_us *= ((row & kCostBf16) ? 1.06 : 1.0) * ((row & kCostBlocksOf16) ? 1.13 : 1.0);
    return streaming_us < tile_us;
  }
  if (!column_wise && k < 4096) {
    // Blocks along N with a short K: one column tile per workgroup, so row groups x N / 16 workgroups, and the time grows
    // with their number per compute unit: measured 2.5 us + (row groups x N / 4096) x 2.5 (K = 1024) or 2.8 (K = 2048)
    // with the rows whole in LDS (M = 24 ... 96, N = 4096 and 8192: 5.0 ... 17.4 and 5.3 ... 18.4 us), 6 at K = 4096 where they
    // are staged per slice.  (The product below said 5.6 us for M = 48, N = 8192, K = 1024, which takes 12.6; tiles 8.2.)
    // The tiles' estimate is the less certain one at this size: the streaming kernel keeps what it wins by less than 15 %.
    const double x = static_cast<double>(row_groups) * (static_cast<double>(n) / 4096.0);
    const double kk = static_cast<double>(k) / 1024.0;
    const double streaming_us = 2.5 + x * (k <= 2560 ? 2.2 + 0.3 * kk : 1.5 * kk);
    return streaming_us < 1.15 * tile_us;
  }
  // more row groups, and blocks along N (from 17 rows on: M = 32, K = 8192, N = 28672 with blocks along N takes 80 us
  // streaming and 50 in 64 x 128 tiles), where the streaming kernel converts with 23 instead of 13 instructions per 8
  // weights
  double streaming_us = (column_wise ? 2.8 : 5.6) * static_cast<double>(row_groups) * (static_cast<double>(n) / 4096.0) *
                        (static_cast<double>(k) / 4096.0);
  if (streaming_groups > kComputeUnits) {
    streaming_us *= static_cast<double>(rounds) / (static_cast<double>(streaming_groups) / kComputeUnits);
  }
  if (row & kCostBf16) streaming_us *= 1.06;
  return streaming_us < tile_us;
}

// The whole decision.  workspace_capacity: bytes of workspace the caller could hand to a split tile kernel
// (0: none, no split).
inline Choice choose(bool column_wise, bool bf16, int m, int n, int k, size_t workspace_capacity, int block_size = 64) {
  Choice c{};
  // few rows, blocks along K, a K that a workgroup can request at once: the decode kernel
  if (decode_shape(column_wise, m, n, k, &c.d, block_size)) {
    c.family = kFamilyDecode;
    return c;
  }
  if (m <= kStreamingMaxRows) c.s = streaming_shape(!column_wise, m, n, k, block_size);
  const int row = tile_cost_row(column_wise, bf16, block_size);
  c.t = tile_plan(column_wise, m, n, k, workspace_capacity, row);
  const double tile_us = (column_wise && m <= 64) ? few_rows_tile_estimate_us(c.t, k, m > 32 ? row : kCostPlain) : tile_estimate_us(c.t, k, row);
  c.family = streaming_kernel_takes(column_wise, m, n, k, c.s, tile_us, row) ? kFamilyStreaming : kFamilyTile;
  return c;
}

}  // namespace blkq4
