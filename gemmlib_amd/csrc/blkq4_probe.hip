// Measurement aids for bench.py (their own small library, not part of the product's ABI): an empty
// kernel, and a kernel that issues the weight-streaming kernel's memory requests and nothing else.  They
// give the two floors that the GEMV figures are read against: what a graph node costs when it does
// nothing, and what reading the packed weights and scales costs with this access pattern.

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

}  // namespace

#define PROBE_EXPORT extern "C" __attribute__((visibility("default")))

PROBE_EXPORT int blkq4_probe_empty(void* scratch, void* stream) {
  hipLaunchKernelGGL(empty_kernel, dim3(256), dim3(256), 0, static_cast<hipStream_t>(stream),
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
