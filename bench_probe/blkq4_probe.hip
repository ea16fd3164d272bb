// Measurement aids for bench.py (their own small library, not part of the product's ABI): an empty
// kernel, a kernel that issues the weight-streaming kernel's memory requests and nothing else, and a kernel
// that does nothing but fp16 MFMAs.  They give what the figures are read against: what a graph node costs
// when it does nothing, what reading the packed weights and scales costs with this access pattern, and the
// MFMA rate the chip sustains on real operands (the clock it holds depends on the operands' bits).

#include <hip/hip_runtime.h>

#include <stdint.h>

namespace {

__global__ void empty_kernel(unsigned* out) {
  if (threadIdx.x == 0xffffffffu) out[0] = 1;
}

// Same requests as the streaming kernel for M <= 16, blocks of 64 along K: a workgroup of WAVES waves owns 16
// columns and all of K; lane (nl, g) of wave w reads unit (4 (w + WAVES d) + g, 16 b + nl) for d = 0, 1, ...
// and, with SCALES, the fp16 scale of that unit's block.
template <int WAVES, bool SCALES>
__global__ __launch_bounds__(64 * WAVES) void stream_kernel(const uint4* __restrict__ W,
                                                            const uint16_t* __restrict__ S, unsigned* out, int N,
                                                            int K) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nl = lane & 15, g = lane >> 4;
  const int units = K >> 5;
  unsigned a = 0;
  for (int ks0 = 4 * wave; ks0 < units; ks0 += 4 * WAVES * 4) {
    uint4 v[4];
    unsigned sc[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int ks = min(ks0 + 4 * WAVES * d + g, units - 1);
      v[d] = W[static_cast<size_t>(ks) * N + blockIdx.x * 16 + nl];
      sc[d] = SCALES ? S[static_cast<size_t>(ks >> 1) * N + blockIdx.x * 16 + nl] : 0u;
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) a ^= v[d].x ^ v[d].y ^ v[d].z ^ v[d].w ^ sc[d];
  }
  if (a == 0x12345678u) out[blockIdx.x] = a;  // keeps the loads alive, (almost) never stores
}

// The decode kernel's requests for M = 1, blocks of 64 along K: a workgroup of WAVES waves owns 16 columns, wave w
// the D consecutive slices from w D on, all requested at once with 32-bit offsets (scale first, then the unit).
template <int WAVES, int D>
__global__ __launch_bounds__(64 * WAVES) void decode_requests_kernel(const uint8_t* __restrict__ W,
                                                                     const uint8_t* __restrict__ S, unsigned* out,
                                                                     int N) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nl = lane & 15, g = lane >> 4;
  const unsigned unit0 = 4u * (wave * D) + g;
  const unsigned col = blockIdx.x * 16 + nl;
  uint4 v[D];
  unsigned sc[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    sc[d] = *reinterpret_cast<const uint16_t*>(S + (((unit0 >> 1) + 2u * d) * N + col) * 2u);
    v[d] = *reinterpret_cast<const uint4*>(W + ((unit0 + 4u * d) * N + col) * 16u);
  }
  unsigned a = 0;
#pragma unroll
  for (int d = 0; d < D; ++d) a ^= v[d].x ^ v[d].y ^ v[d].z ^ v[d].w ^ sc[d];
  if (a == 0x12345678u) out[blockIdx.x] = a;  // keeps the loads alive, (almost) never stores
}

// The quantizer's memory traffic and nothing else: the tile, the loads, the trip through LDS and the stores of the
// product's kernel for blocks of BS along K with zero-points (32 columns x 256 rows per workgroup, four 16-byte
// non-temporal loads per lane, packed words 16 bytes per lane, scales 8 and zero-points 4 bytes per lane), with an
// exclusive-or in place of the arithmetic.  What it takes is what the quantizer cannot go below without moving
// its bytes differently.
typedef unsigned probe_u32x4 __attribute__((ext_vector_type(4)));
template <int BS>
__global__ __launch_bounds__(256) void prepack_traffic_kernel(const uint16_t* __restrict__ src, int K, int N, int ld,
                                                             uint4* __restrict__ packed_w, uint16_t* __restrict__ scales,
                                                             uint8_t* __restrict__ zps, unsigned k_tiles) {
  constexpr int kTileN = 32, kTileK = 256, kBlocksPerTile = kTileK / BS;
  __shared__ uint32_t w_lds[kTileK / 32][kTileN][4];
  __shared__ __attribute__((aligned(8))) uint16_t s_lds[kBlocksPerTile][kTileN];
  __shared__ __attribute__((aligned(4))) uint8_t z_lds[kBlocksPerTile][kTileN];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int k0 = static_cast<int>(blockIdx.x % k_tiles) * kTileK, n0 = static_cast<int>(blockIdx.x / k_tiles) * kTileN;
  const int kl = (lane & 31) * 8;
  probe_u32x4 raw[4];
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int nl = wave * 8 + it * 2 + (lane >> 5);
    raw[it] = __builtin_nontemporal_load(reinterpret_cast<const probe_u32x4*>(
        src + static_cast<size_t>(min(n0 + nl, N - 1)) * ld + min(k0 + kl, K - 8)));
  }
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int nl = wave * 8 + it * 2 + (lane >> 5);
    const uint32_t word = raw[it][0] ^ raw[it][1] ^ raw[it][2] ^ raw[it][3];
    w_lds[kl >> 5][nl][(kl >> 3) & 3] = word;
    if ((kl % BS) == 0) {
      s_lds[kl / BS][nl] = static_cast<uint16_t>(word);
      z_lds[kl / BS][nl] = static_cast<uint8_t>(word >> 16);
    }
  }
  __syncthreads();
  {
    const int ksl = tid / kTileN, nl = tid % kTileN;
    const int k = k0 + ksl * 32, n = n0 + nl;
    if (k < K && n < N) {
      const uint4 v = *reinterpret_cast<const uint4*>(&w_lds[ksl][nl][0]);
      __builtin_nontemporal_store(probe_u32x4{v.x, v.y, v.z, v.w},
                                  reinterpret_cast<probe_u32x4*>(&packed_w[static_cast<size_t>(k >> 5) * N + n]));
    }
  }
  for (int u = tid; u < kBlocksPerTile * kTileN / 4; u += 256) {
    const int bl = u / (kTileN / 4), nl = (u % (kTileN / 4)) * 4;
    const int k = k0 + bl * BS, n = n0 + nl;
    if (k < K && n < N) {
      const size_t idx = static_cast<size_t>(k / BS) * N + n;
      *reinterpret_cast<uint2*>(scales + idx) = *reinterpret_cast<const uint2*>(&s_lds[bl][nl]);
      *reinterpret_cast<uint32_t*>(zps + idx) = *reinterpret_cast<const uint32_t*>(&z_lds[bl][nl]);
    }
  }
}

typedef _Float16 probe_half8 __attribute__((ext_vector_type(8)));
typedef float probe_float16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ unsigned mix_bits(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// One wave per SIMD, eight independent accumulators, back-to-back v_mfma_f32_32x32x16_f16 and nothing else.
// RANDOM: operands are fp16 values of either sign in [0.125, 0.5) with random mantissas; otherwise zeros.
template <bool RANDOM>
__global__ __launch_bounds__(256) void mfma_kernel(float* out, int iters) {
  probe_half8 a[8], b[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const unsigned r = mix_bits(threadIdx.x * 64 + s * 8 + e + blockIdx.x * 7919u);
      a[s][e] = __builtin_bit_cast(_Float16, static_cast<unsigned short>(RANDOM ? (0x3000u | (r & 0x8fffu)) : 0u));
      b[s][e] = __builtin_bit_cast(_Float16, static_cast<unsigned short>(RANDOM ? (0x3000u | ((r >> 16) & 0x8fffu)) : 0u));
    }
  }
  probe_float16 acc[8];
#pragma unroll
  for (int n = 0; n < 8; ++n)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[n][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < 8; ++n) acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[n], b[(3 * n + 1) & 7], acc[n], 0, 0, 0);
  }
  float sum = 0.f;
#pragma unroll
  for (int n = 0; n < 8; ++n)
#pragma unroll
    for (int e = 0; e < 16; ++e) sum += acc[n][e];
  out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
}


// What a wave's own instruction stream costs: `iters` rounds of four independent MFMAs (32 x 32 x 16, fp16), each
// followed by N independent packed vector instructions.  Every wave leaves its cycle count (s_memtime) per MFMA in
// cycles[wave]; with one workgroup the waves' figures show how waves of one SIMD share it.
typedef _Float16 probe_half8_t __attribute__((ext_vector_type(8)));
typedef float probe_float16_t __attribute__((ext_vector_type(16)));
template <int N>
__global__ __launch_bounds__(1024) void issue_kernel(unsigned long long* cycles, int iters, unsigned seed) {
  probe_half8_t a, b;
  for (int e = 0; e < 8; ++e) {
    a[e] = static_cast<_Float16>(static_cast<float>((threadIdx.x + e + seed) & 7));
    b[e] = static_cast<_Float16>(static_cast<float>((e * 3 + seed) & 7));
  }
  probe_float16_t acc[4];
  for (int g = 0; g < 4; ++g)
    for (int e = 0; e < 16; ++e) acc[g][e] = 0.f;
  unsigned x[8];
  for (int j = 0; j < 8; ++j) x[j] = seed + j + threadIdx.x;
  const unsigned c = seed * 3 + 1;
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      acc[g] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[g], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < N; ++j) asm volatile("v_pk_add_f16 %0, %0, %1" : "+v"(x[(g * N + j) % 8]) : "v"(c));
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  float s = 0;
  for (int g = 0; g < 4; ++g)
    for (int e = 0; e < 16; ++e) s += acc[g][e];
  unsigned y = 0;
  for (int j = 0; j < 8; ++j) y ^= x[j];
  if ((threadIdx.x & 63) == 0 && blockIdx.x == 0) cycles[threadIdx.x >> 6] = (t1 - t0) / (4ull * iters);
  if (s == 12345.678f && y == 77) cycles[63] = 1;  // keeps the work alive, (almost) never stores
}

}  // namespace

#define PROBE_EXPORT extern "C" __attribute__((visibility("default")))

PROBE_EXPORT int blkq4_probe_empty(void* scratch, void* stream) {
  hipLaunchKernelGGL(empty_kernel, dim3(256), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<unsigned*>(scratch));
  return static_cast<int>(hipGetLastError());
}

// an empty kernel of any launch shape (what a graph node costs depends on how many waves have to be started)
PROBE_EXPORT int blkq4_probe_empty_shape(int grid, int block, int lds_bytes, void* scratch, void* stream) {
  hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), lds_bytes, static_cast<hipStream_t>(stream),
                     static_cast<unsigned*>(scratch));
  return static_cast<int>(hipGetLastError());
}

// packed_w: uint8[K/32][N][16]; scales: fp16 [K/64][N] or NULL; scratch: at least N / 16 * 4 bytes
PROBE_EXPORT int blkq4_probe_stream(const void* packed_w, const void* scales, int n, int k, void* scratch,
                                    void* stream) {
  if (n % 16 != 0 || k % 64 != 0) return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid(n / 16), block(64 * 8);
  if (scales) {
    hipLaunchKernelGGL((stream_kernel<8, true>), grid, block, 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(packed_w), static_cast<const uint16_t*>(scales),
                       static_cast<unsigned*>(scratch), n, k);
  } else {
    hipLaunchKernelGGL((stream_kernel<8, false>), grid, block, 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(packed_w), static_cast<const uint16_t*>(nullptr),
                       static_cast<unsigned*>(scratch), n, k);
  }
  return static_cast<int>(hipGetLastError());
}

// the same requests from workgroups of sixteen waves (the product's shape for C2)
PROBE_EXPORT int blkq4_probe_stream16(const void* packed_w, const void* scales, int n, int k, void* scratch,
                                      void* stream) {
  if (n % 16 != 0 || k % 64 != 0) return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid(n / 16), block(64 * 16);
  if (scales) {
    hipLaunchKernelGGL((stream_kernel<16, true>), grid, block, 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(packed_w), static_cast<const uint16_t*>(scales),
                       static_cast<unsigned*>(scratch), n, k);
  } else {
    hipLaunchKernelGGL((stream_kernel<16, false>), grid, block, 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(packed_w), static_cast<const uint16_t*>(nullptr),
                       static_cast<unsigned*>(scratch), n, k);
  }
  return static_cast<int>(hipGetLastError());
}

// the decode kernel's requests: eight waves with four slices each (k = 4096)
PROBE_EXPORT int blkq4_probe_decode_requests(const void* packed_w, const void* scales, int n, int k, void* scratch,
                                             void* stream) {
  if (n % 16 != 0 || k != 4096) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL((decode_requests_kernel<8, 4>), dim3(n / 16), dim3(512), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint8_t*>(packed_w), static_cast<const uint8_t*>(scales),
                     static_cast<unsigned*>(scratch), n);
  return static_cast<int>(hipGetLastError());
}

// 256 workgroups of four waves, `iters` x 8 MFMAs per wave: 256 * 4 * iters * 8 * 32768 flop.
// scratch: at least 256 * 256 * 4 bytes
PROBE_EXPORT int blkq4_probe_mfma(int random_operands, int iters, void* scratch, void* stream) {
  if (random_operands) {
    hipLaunchKernelGGL(mfma_kernel<true>, dim3(256), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<float*>(scratch), iters);
  } else {
    hipLaunchKernelGGL(mfma_kernel<false>, dim3(256), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<float*>(scratch), iters);
  }
  return static_cast<int>(hipGetLastError());
}

// src: fp16 [n][ld]; packed_w k n / 2 bytes, scales (k / 16) n fp16 (8-byte aligned), zps (k / 16) n bytes (4-byte
// aligned): the buffers of the quantizer for blocks of 16 along K; k a multiple of 64, n of 32
PROBE_EXPORT int blkq4_probe_prepack_traffic(const void* src, int k, int n, int ld, void* packed_w, void* scales, void* zps,
                                             void* stream) {
  if (k % 64 != 0 || n % 32 != 0) return static_cast<int>(hipErrorInvalidValue);
  const unsigned k_tiles = (k + 255) / 256;
  hipLaunchKernelGGL(prepack_traffic_kernel<16>, dim3(k_tiles * (n / 32)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(src), k, n, ld, static_cast<uint4*>(packed_w),
                     static_cast<uint16_t*>(scales), static_cast<uint8_t*>(zps), k_tiles);
  return static_cast<int>(hipGetLastError());
}

// `workgroups` workgroups of `threads` threads (64 ... 1024), 4 * iters MFMAs per wave, each followed by
// vector_per_mfma (0, 2, 4, 6, 8, 12 or 16) independent vector instructions; cycles: 64 x 8 bytes of device memory
// that receive workgroup 0's cycles per MFMA, wave by wave.  Flop of the launch: workgroups * threads / 64 * iters * 4 * 32768.
PROBE_EXPORT int blkq4_probe_issue(int vector_per_mfma, int workgroups, int threads, int iters, void* cycles, void* stream) {
  if (threads < 64 || threads > 1024 || threads % 64 != 0 || workgroups < 1 || iters < 1) return static_cast<int>(hipErrorInvalidValue);
#define PROBE_ISSUE_CASE(N_)                                                                                          \
  case N_:                                                                                                            \
    hipLaunchKernelGGL(issue_kernel<N_>, dim3(workgroups), dim3(threads), 0, static_cast<hipStream_t>(stream),        \
                       static_cast<unsigned long long*>(cycles), iters, 1u);                                          \
    break;
  switch (vector_per_mfma) {
    PROBE_ISSUE_CASE(0) PROBE_ISSUE_CASE(2) PROBE_ISSUE_CASE(4) PROBE_ISSUE_CASE(6) PROBE_ISSUE_CASE(8) PROBE_ISSUE_CASE(12)
    PROBE_ISSUE_CASE(16)
    default: return static_cast<int>(hipErrorInvalidValue);
  }
#undef PROBE_ISSUE_CASE
  return static_cast<int>(hipGetLastError());
}
