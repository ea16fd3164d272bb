// Workspace of the split tile kernels (arrival counters + fp32 partial tiles): where it comes from.
//
//   blkq4_dev_workspace: one buffer per (device, stream), owned by the library, allocated on the first call
//     that needs one and kept until the process ends.  Calls on one stream run in order, so they can share a
//     buffer; calls on different streams may overlap, so they cannot.  A call that is being recorded into a graph
//     may allocate too (the allocation is no stream operation; the thread's capture mode is set to relaxed around
//     it, as tensor libraries do for their own allocations during capture).  A recorded call keeps using the
//     buffer of the stream it was recorded on, whatever stream the graph is launched on later.
//
// The kernels leave the arrival counters at zero (the workgroup that arrives last clears its tile's counter), so
// they are cleared once, when the buffer is allocated, by a small kernel on a stream of the allocation's own.

#include <hip/hip_runtime.h>

#include <stdint.h>

#include <mutex>

#include "blkq4_choose.h"
#include "blkq4_device.h"
#include "blkq4_launch.h"

namespace {

constexpr size_t kPoolBytes = blkq4::kCounterBytes + (size_t{32} << 20);
constexpr int kMaxSlots = 16;  // streams with a buffer of their own; later ones run unsplit kernels

__global__ void clear_counters(int* counters) {
  for (unsigned i = threadIdx.x; i < blkq4::kCounterBytes / sizeof(int); i += blockDim.x) counters[i] = 0;
}

struct Slot {
  int device;
  hipStream_t stream;
  void* ptr;
};
std::mutex g_mutex;
Slot g_slots[kMaxSlots];
int g_slot_count = 0;

}  // namespace

extern "C" size_t blkq4_dev_workspace_capacity(void) { return kPoolBytes; }

extern "C" int blkq4_dev_workspace(void* stream_ptr, void** ptr) {
  *ptr = nullptr;
  hipStream_t stream = static_cast<hipStream_t>(stream_ptr);
  int device = 0;
  if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return static_cast<int>(e);
  std::lock_guard<std::mutex> lock(g_mutex);
  for (int i = 0; i < g_slot_count; ++i) {
    if (g_slots[i].device == device && g_slots[i].stream == stream) {
      *ptr = g_slots[i].ptr;
      return 0;
    }
  }
  if (g_slot_count == kMaxSlots) return 0;  // no workspace for this stream: unsplit kernels
  // An allocation is allowed while this or another thread records a graph only in relaxed mode.  The counters
  // are cleared on a stream of this function's own and waited for, so they are zero when this returns, whether
  // the caller's stream is executing or being recorded.
  hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
  if (hipError_t e = hipThreadExchangeStreamCaptureMode(&mode); e != hipSuccess) return static_cast<int>(e);
  void* p = nullptr;
  hipStream_t own = nullptr;
  hipError_t e = hipMalloc(&p, kPoolBytes);
  if (e == hipSuccess) {
    e = hipStreamCreateWithFlags(&own, hipStreamNonBlocking);
    if (e == hipSuccess) {
      e = blkq4::launch_status(clear_counters, dim3(1), dim3(1024), 0, own, static_cast<int*>(p));
      if (e == hipSuccess) e = hipStreamSynchronize(own);
      (void)hipStreamDestroy(own);
    }
    if (e != hipSuccess) (void)hipFree(p);
  }
  (void)hipThreadExchangeStreamCaptureMode(&mode);
  if (e == hipErrorOutOfMemory) {
    (void)hipGetLastError();  // not an error of the call: run unsplit
    return 0;
  }
  if (e != hipSuccess) return static_cast<int>(e);
  g_slots[g_slot_count++] = Slot{device, stream, p};
  *ptr = p;
  return 0;
}
