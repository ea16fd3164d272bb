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


template <int BS, int NT, bool A_LDS>
struct Slot {
  static constexpr int kMeta = (BS == 16) ? 2 : 1;  // quantization blocks inside one 32-deep unit
  uint4 w[NT];
  uint32_t sc[NT][kMeta];
  uint32_t zp[NT][kMeta];
  uint4 a[A_LDS ? 1 : 4];  // 32 k of this lane's activation row (unused when the rows are in LDS)
};

// kWaves: waves of the workgroup, which split K.  DEPTH: k slices (128 deep) a wave keeps in flight.  NT: 16-column tiles per wave that share one
// activation operand.  A_LDS: the activation rows are staged in LDS (rows_log2 = log2 of the number of rows
// kept there, a power of two >= M); the dynamic LDS size is red_bytes + (K * 2 << rows_log2).
template <int BS, bool HAS_ZP, int DEPTH, int NT, int kWaves, bool A_LDS>
__global__ __launch_bounds__(64 * kWaves) void skinny_mfma_kernel(const uint16_t* __restrict__ A,
                                                               const uint4* __restrict__ W,
                                                               const uint16_t* __restrict__ S,
                                                               const uint8_t* __restrict__ Z,
                                                               uint16_t* __restrict__ C, int M, int N,
                                                               int K, int rows_log2) {
  constexpr int kMeta = Slot<BS, NT, A_LDS>::kMeta;
  constexpr int kRedFloats = kWaves * NT * 64 * 4;
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
  const bool row_ok = nl < M;
  const DequantMasks masks = DequantMasks::make();
  // lanes without a row load nothing and feed whatever their registers hold to the MFMA: an output
  // element depends on its own activation row only, and the rows past M are never stored
  const uint8_t* a_row = reinterpret_cast<const uint8_t*>(A) + static_cast<size_t>(min(nl, M - 1)) * K * 2;

  const int units = K >> 5;             // 32-deep units
  const int slices = (units + 3) >> 2;  // 128-deep slices (the last one may be half full)
  const int my_slices = (slices - wave + kWaves - 1) / kWaves;  // slices wave, wave + kWaves, ...

  const int wrap_mask = (1 << (31 - __builtin_clz(units))) - 1;  // any index & wrap_mask is < units

  float4_t acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
  Slot<BS, NT, A_LDS> slot[DEPTH];

  // Rows to LDS: copy q fills LDS bytes [1024 q, 1024 q + 1024) of the [unit][row][64 B] layout, lane l
  // the 16 bytes at 16 l.  They are requested before anything else, so every later wait covers them.
  uint32_t a_rd = 0;  // LDS byte offset of this lane's row inside a unit, chunk 0
  uint32_t a_swz = 0;
  if (A_LDS) {
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                              (__attribute__((address_space(3))) uint8_t*)(smem))) + kRedFloats * 4;
    const int rows = 1 << rows_log2;
    const int copies = ((K << rows_log2) + 511) >> 9;  // K * 2 * rows bytes in 1 KiB copies, the last one may be partial
    for (int q = wave; q < copies; q += kWaves) {
      const uint32_t off = q * 1024 + lane * 16;
      const int u = min(static_cast<int>(off >> (6 + rows_log2)), units - 1);  // past the end: any valid unit
      const int row = (off >> 6) & (rows - 1);
      const int chunk = (lane & 3) ^ ((row >> 2) & 3);
      async_copy_16(lds0 + q * 1024, A, (static_cast<uint32_t>(min(row, M - 1)) * K + u * 32 + chunk * 8) * 2);
    }
    const int row = min(nl, rows - 1);
    a_rd = row * 64;
    a_swz = (row >> 2) & 3;
  }
  // a slice past the end wraps around to valid units (so every slot always issues the same loads)
  // and gets a zero scale, which makes it contribute exactly 0
#define BLKQ4_LOAD_SLOT(dst_, slice_)                                                          \
  {                                                                                            \
    const int ks_ = 4 * (slice_) + g;                                                          \
    const bool ok_ = ks_ < units;                                                              \
    const int ksg_ = ok_ ? ks_ : (ks_ & wrap_mask);                                            \
    const int b_ = (BS == 64) ? (ksg_ >> 1) : (BS == 32) ? ksg_ : (2 * ksg_);                  \
    _Pragma("unroll") for (int t = 0; t < NT; ++t) {                                           \
      (dst_).w[t] = W[static_cast<size_t>(ksg_) * N + n[t]];                                  \
      _Pragma("unroll") for (int q = 0; q < kMeta; ++q) {                                      \
        const size_t mi_ = static_cast<size_t>(b_ + q) * N + n[t];                           \
        const uint32_t sc_ = S[mi_];                                                           \
        (dst_).sc[t][q] = ok_ ? sc_ : 0u;                                                      \
        (dst_).zp[t][q] = HAS_ZP ? static_cast<uint32_t>(Z[mi_]) : 8u;                         \
      }                                                                                        \
    }                                                                                          \
    if (!A_LDS) {                                                                              \
      const uint4* p_ = reinterpret_cast<const uint4*>(a_row + static_cast<size_t>(ksg_) * 64);\
      if (row_ok) {                                                                            \
        _Pragma("unroll") for (int j = 0; j < (A_LDS ? 1 : 4); ++j)(dst_).a[j] = p_[j];        \
      }                                                                                        \
    }                                                                                          \
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) BLKQ4_LOAD_SLOT(slot[d], wave + d * kWaves);
  if (A_LDS) {
    // everything but the requests of the ring just issued has landed: this wave's share of the rows
    constexpr int kRing = DEPTH * NT * (1 + kMeta * (HAS_ZP ? 2 : 1));
    wait_vmcnt<(kRing < 63 ? kRing : 63)>();
    __syncthreads();
  }

  for (int i0 = 0; i0 < my_slices; i0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int li = i0 + d;  // local slice index; slice = wave + 4*li
      half8_t af[4];
      if (A_LDS) {
        const int ks = 4 * (wave + kWaves * li) + g;
        const int ksg = (ks < units) ? ks : (ks & wrap_mask);
        const uint8_t* ap = a_lds + (static_cast<uint32_t>(ksg) << (6 + rows_log2)) + a_rd;
#pragma unroll
        for (int j = 0; j < 4; ++j) af[j] = as_half8(*reinterpret_cast<const uint4*>(ap + ((j ^ a_swz) * 16)));
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) af[j] = as_half8(slot[d].a[j < (A_LDS ? 1 : 4) ? j : 0]);
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
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, af[j], acc[t], 0, 0, 0);
        }
      }
      if (i0 + DEPTH < my_slices) BLKQ4_LOAD_SLOT(slot[d], wave + kWaves * (li + DEPTH));
    }
  }
#undef BLKQ4_LOAD_SLOT

  // cross-wave reduction through LDS
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) red[((wave * NT + t) * 64 + lane) * 4 + e] = acc[t][e];
  __syncthreads();
  // value v = (tile t, lane L, element e) of the partial tiles: output row L & 15, column 4 (L >> 4) + e
  // of tile t; every thread sums a few of them over the waves
  for (int v = tid; v < NT * 256; v += 64 * kWaves) {
    float r = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) r += red[w * (NT * 256) + v];
    const int t = v >> 8, L = (v >> 2) & 63, e = v & 3;
    const int row = L & 15;
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
template <int BS, bool HAS_ZP, int DEPTH, int NT, int kWaves, bool A_LDS>
int launch_kernel(const blkq4_gemm_args* a, int rows_log2) {
  constexpr int kRedBytes = kWaves * NT * 64 * 4 * 4;
  // the rows are copied 1 KiB at a time
  const size_t lds_bytes = kRedBytes + (A_LDS ? ((((static_cast<size_t>(a->k) * 2) << rows_log2) + 1023) & ~size_t{1023}) : 0);
  auto* kernel = skinny_mfma_kernel<BS, HAS_ZP, DEPTH, NT, kWaves, A_LDS>;
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
    if (a_bytes + 16 * NT * 64 * 4 * 4 <= kMaxLdsBytes) return launch_kernel<BS, HAS_ZP, kD, NT, 16, true>(a, rows_log2);
    return launch_kernel<BS, HAS_ZP, kD, NT, 16, false>(a, rows_log2);
  }
  if (a->k >= 1024) {
    constexpr int kD = DEPTH > 4 ? 4 : DEPTH;
    if (a_bytes + 8 * NT * 64 * 4 * 4 <= kMaxLdsBytes) return launch_kernel<BS, HAS_ZP, kD, NT, 8, true>(a, rows_log2);
    return launch_kernel<BS, HAS_ZP, kD, NT, 8, false>(a, rows_log2);
  }
  return launch_kernel<BS, HAS_ZP, DEPTH, NT, 4, true>(a, rows_log2);  // K < 1024: at most 32 KiB of rows
}

template <int BS, bool HAS_ZP>
int launch_shape(const blkq4_gemm_args* a) {
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
  if (a->m < 1 || a->m > 16 || (a->n % 16) != 0 || (a->k % 64) != 0) return static_cast<int>(hipErrorInvalidValue);
  switch (a->block_size) {
    case 16: return launch_skinny<16>(a);
    case 32: return launch_skinny<32>(a);
    case 64: return launch_skinny<64>(a);
    default: return static_cast<int>(hipErrorInvalidValue);
  }
}
