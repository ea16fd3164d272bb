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
//   - the lanes that carry an activation row load their 64 bytes per slice straight from global
//     memory (L2 resident) into the same ring, so every request of a slice is issued together and
//     the compiler's in-order vmcnt waits let slice i be consumed while slices i+1.. are in flight;
//   - a lane multiplies its (column, 32 k) of weights with the matching 32 k of up to 16 activation
//     rows through v_mfma_f32_16x16x32_f16 (weights as the row operand: a lane ends up with 4
//     consecutive output columns of one activation row, one 8-byte store);
//   - the waves' partial tiles are summed through LDS by wave 0: no atomics, no scratch buffer.
// Dequantization happens in registers (blkq4_dequant.h); accumulation is fp32.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "blkq4_dequant.h"
#include "blkq4_device.h"

namespace {

using namespace blkq4;


template <int BS, int NT>
struct Slot {
  static constexpr int kMeta = (BS == 16) ? 2 : 1;  // quantization blocks inside one 32-deep unit
  uint4 w[NT];
  uint32_t sc[NT][kMeta];
  uint32_t zp[NT][kMeta];
  uint4 a[4];  // 32 k of this lane's activation row
};

// kWaves: waves of the workgroup, which split K.  DEPTH: k slices (128 deep) a wave keeps in flight.  NT: 16-column tiles per wave that share one
// activation operand.
template <int BS, bool HAS_ZP, int DEPTH, int NT, int kWaves>
__global__ __launch_bounds__(64 * kWaves) void skinny_mfma_kernel(const uint16_t* __restrict__ A,
                                                               const uint4* __restrict__ W,
                                                               const uint16_t* __restrict__ S,
                                                               const uint8_t* __restrict__ Z,
                                                               uint16_t* __restrict__ C, int M, int N,
                                                               int K) {
  constexpr int kMeta = Slot<BS, NT>::kMeta;
  __shared__ float red[kWaves * NT * 64 * 4];

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
  Slot<BS, NT> slot[DEPTH];
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
    const uint4* p_ = reinterpret_cast<const uint4*>(a_row + static_cast<size_t>(ksg_) * 64);  \
    if (row_ok) {                                                                              \
      _Pragma("unroll") for (int j = 0; j < 4; ++j)(dst_).a[j] = p_[j];                        \
    }                                                                                          \
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) BLKQ4_LOAD_SLOT(slot[d], wave + d * kWaves);

  for (int i0 = 0; i0 < my_slices; i0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int li = i0 + d;  // local slice index; slice = wave + 4*li
      half8_t af[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) af[j] = as_half8(slot[d].a[j]);
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
  if (wave == 0) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float r[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        r[e] = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) r[e] += red[((w * NT + t) * 64 + lane) * 4 + e];
      }
      if (row_ok && blockIdx.x * NT + t < tiles) {
        // lane (row nl, group g) holds output columns 4g .. 4g+3 of 16-column tile t
        const uint32_t lo = float_to_half_bits(r[0]) | (static_cast<uint32_t>(float_to_half_bits(r[1])) << 16);
        const uint32_t hi = float_to_half_bits(r[2]) | (static_cast<uint32_t>(float_to_half_bits(r[3])) << 16);
        uint2* out = reinterpret_cast<uint2*>(C + static_cast<size_t>(nl) * N + blockIdx.x * (16 * NT) + 16 * t + 4 * g);
        *out = make_uint2(lo, hi);
      }
    }
  }
}

// The kernel is bound by instruction issue as much as by the weight stream, so what matters is how
// evenly the workgroups fill the 256 compute units: with T column tiles per workgroup the busiest
// unit works through ceil(workgroups / 256) * T tiles.  Wider workgroups also re-read the activation
// rows less often, which weighs more the more rows there are.
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

template <int BS>
int launch_skinny(const blkq4_gemm_args* a) {
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  const auto* A = static_cast<const uint16_t*>(a->a);
  const auto* W = static_cast<const uint4*>(a->packed_w);
  const auto* S = static_cast<const uint16_t*>(a->scales);
  const auto* Z = static_cast<const uint8_t*>(a->zero_points);
  auto* C = static_cast<uint16_t*>(a->c);
#define BLKQ4_LAUNCH(ZP_, DEPTH_, NT_)                                                                  \
  if (waves == 8)                                                                                       \
    hipLaunchKernelGGL((skinny_mfma_kernel<BS, ZP_, (DEPTH_ > 4 ? 4 : DEPTH_), NT_, 8>),                \
                       dim3((a->n / 16 + NT_ - 1) / NT_), dim3(512), 0, stream, A, W, S, Z, C, a->m, a->n, a->k); \
  else                                                                                                  \
    hipLaunchKernelGGL((skinny_mfma_kernel<BS, ZP_, DEPTH_, NT_, 4>), dim3((a->n / 16 + NT_ - 1) / NT_), \
                       dim3(256), 0, stream, A, W, S, Z, C, a->m, a->n, a->k)
  int nt, depth;
  choose_shape(a->m, a->n, &nt, &depth);
  // eight waves split K when there is enough of it: each wave has less to convert after its last
  // load has arrived, and more of that work overlaps the loads of the other waves
  const int waves = (a->k >= 1024) ? 8 : 4;
#define BLKQ4_LAUNCH_ZP(ZP_)                   \
  if (nt == 1 && depth == 8) { BLKQ4_LAUNCH(ZP_, 8, 1); } \
  else if (nt == 1) { BLKQ4_LAUNCH(ZP_, 4, 1); }   \
  else if (nt == 2) { BLKQ4_LAUNCH(ZP_, 4, 2); }   \
  else { BLKQ4_LAUNCH(ZP_, 4, 3); }
  if (Z) { BLKQ4_LAUNCH_ZP(true); } else { BLKQ4_LAUNCH_ZP(false); }
#undef BLKQ4_LAUNCH_ZP
#undef BLKQ4_LAUNCH
  return static_cast<int>(hipGetLastError());
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
