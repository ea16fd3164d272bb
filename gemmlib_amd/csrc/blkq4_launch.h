// Host-side launch helpers shared by the kernel files.

#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <tuple>

namespace blkq4 {

// Launches `kernel` and returns the launch's own status.  (hipGetLastError() after a <<<>>> launch would
// also return, and clear, a sticky error that an earlier, unrelated call left on this thread.)
template <class... KArgs, class... Args>
inline hipError_t launch_status(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, void* stream,
                                Args... args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "one argument per kernel parameter");
  std::tuple<KArgs...> values(static_cast<KArgs>(args)...);
  return std::apply(
      [&](auto&... v) {
        void* ptrs[] = {static_cast<void*>(&v)...};
        return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds_bytes,
                               static_cast<hipStream_t>(stream));
      },
      values);
}

// Sets a kernel's dynamic-LDS limit unless `done` says this device has it already: one bit per device index
// below 64 (the attribute belongs to the device's copy of the code).  `done` must belong to this kernel alone.
inline hipError_t raise_lds_limit_once(const void* kernel, size_t bytes, std::atomic<uint64_t>* done) {
  int device = 0;
  if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return e;
  if (device < 64 && ((done->load(std::memory_order_acquire) >> device) & 1u) != 0) return hipSuccess;
  const hipError_t e =
      hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
  if (e == hipSuccess && device < 64) done->fetch_or(uint64_t{1} << device, std::memory_order_release);
  return e;
}


// The flags of kernel `kKernel`.  The kernel is a template VALUE: every instantiation of a kernel template has
// flags of its own (instantiations share their function type, so a template over the type would share one set).
template <auto kKernel>
inline std::atomic<uint64_t>& lds_limit_flags() {
  static std::atomic<uint64_t> done{0};
  return done;
}

}  // namespace blkq4
