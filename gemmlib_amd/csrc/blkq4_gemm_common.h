// Pieces shared by the MFMA GEMM kernels: the asynchronous HBM -> LDS copy instructions, the manual
// counter waits that order them, and the barrier wrapper.

#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace blkq4 {

// Asynchronous copy: every active lane moves 16 (4) bytes from global memory to
// LDS[lds_base + lane * 16 (4)].  lds_base and base are wave-uniform, offset is per lane.  The
// compiler does not see the LDS write; it is ordered by hand with wait_vmcnt + s_barrier.
// M0 is named as clobbered so that the compiler never carries a value of its own in it across these
// statements (it warns that M0 is a reserved register; the clobber is recorded all the same).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void async_copy_16(uint32_t lds_base, const void* base, uint32_t offset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(offset), "s"(base)
               : "memory", "m0");
}
// the same with the non-temporal hint, for data that this launch reads once
__device__ __forceinline__ void async_copy_16_once(uint32_t lds_base, const void* base, uint32_t offset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_base), "v"(offset), "s"(base)
               : "memory", "m0");
}
__device__ __forceinline__ void async_copy_4_flat(uint32_t lds_base, const void* gptr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_base), "v"(gptr) : "memory", "m0");
}
#pragma clang diagnostic pop
// LDS reads at byte address `addr` + `imm`.  `imm` is a compile-time constant applied as a pointer offset,
// which the compiler folds into the instruction's offset field (it will not do that for an integer addition,
// which may wrap); `addr` costs whatever the caller spends on it and nothing more.
typedef uint32_t lds_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 lds_read_16(uint32_t addr, int imm = 0) {
  const auto* p = reinterpret_cast<const __attribute__((address_space(3))) uint8_t*>(addr) + imm;
  const lds_u32x4_t v = *reinterpret_cast<const __attribute__((address_space(3))) lds_u32x4_t*>(p);
  return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint32_t lds_read_u16(uint32_t addr, int imm = 0) {
  const auto* p = reinterpret_cast<const __attribute__((address_space(3))) uint8_t*>(addr) + imm;
  return *reinterpret_cast<const __attribute__((address_space(3))) uint16_t*>(p);
}
__device__ __forceinline__ uint32_t lds_read_u8(uint32_t addr, int imm = 0) {
  return *(reinterpret_cast<const __attribute__((address_space(3))) uint8_t*>(addr) + imm);
}
__device__ __forceinline__ uint32_t lds_read_u32(uint32_t addr, int imm = 0) {
  const auto* p = reinterpret_cast<const __attribute__((address_space(3))) uint8_t*>(addr) + imm;
  return *reinterpret_cast<const __attribute__((address_space(3))) uint32_t*>(p);
}
__device__ __forceinline__ void lds_write_16(uint32_t addr, int imm, uint32_t x, uint32_t y, uint32_t z, uint32_t w) {
  auto* p = reinterpret_cast<__attribute__((address_space(3))) uint8_t*>(addr) + imm;
  *reinterpret_cast<__attribute__((address_space(3))) lds_u32x4_t*>(p) = lds_u32x4_t{x, y, z, w};
}
typedef uint32_t lds_u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void lds_write_8(uint32_t addr, int imm, uint32_t lo, uint32_t hi) {
  auto* p = reinterpret_cast<__attribute__((address_space(3))) uint8_t*>(addr) + imm;
  *reinterpret_cast<__attribute__((address_space(3))) lds_u32x2_t*>(p) = lds_u32x2_t{lo, hi};
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

}  // namespace blkq4

#define BLKQ4_PIN() __builtin_amdgcn_sched_barrier(0)
