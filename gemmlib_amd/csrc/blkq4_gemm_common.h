// Pieces shared by the MFMA GEMM kernels: the asynchronous HBM -> LDS copy instructions, the manual
// counter waits that order them, and the barrier wrapper.

#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace blkq4 {

// Asynchronous copy: every active lane moves 16 (4) bytes from global memory to
// LDS[lds_base + lane * 16 (4)].  lds_base and base are wave-uniform, offset is per lane.  The
// compiler does not see the LDS write; it is ordered by hand with wait_vmcnt + s_barrier.
__device__ __forceinline__ void async_copy_16(uint32_t lds_base, const void* base, uint32_t offset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(offset), "s"(base)
               : "memory");
}
__device__ __forceinline__ void async_copy_4_flat(uint32_t lds_base, const void* gptr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_base), "v"(gptr) : "memory");
}
// the same with lanes 0..31 only (the other lanes must be active when this is called)
__device__ __forceinline__ void async_copy_4_flat_lo32(uint32_t lds_base, const void* gptr) {
  uint64_t saved;
  asm volatile(
      "s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xffffffff\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
      "global_load_lds_dword %2, off\n\ts_mov_b64 exec, %0"
      : "=&s"(saved)
      : "s"(lds_base), "v"(gptr)
      : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// s_barrier that the compiler may not move LDS accesses across, in either direction
__device__ __forceinline__ void block_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

}  // namespace blkq4

#define BLKQ4_PIN() __builtin_amdgcn_sched_barrier(0)
