// Workspace of the split tile kernels (arrival counters + fp32 partial tiles): where it comes from.
//
//   blkq4_dev_workspace: one buffer per (device, stream), owned by the library, allocated on the first call
//     that needs one and kept until the process ends.  Calls on one stream run in order, so they can share a
//     buffer; calls on different streams may overlap, so they cannot.  A call that is being recorded into a graph
//     may allocate too (the allocation is no stream operation; the thread's capture mode is set to relaxed around
//     it, as tensor libraries do for their own allocations during capture).  A recorded call keeps using the
//     buffer of the stream it was recorded on, whatever stream the graph is launched on later.
//
//   blkq4_dev_static_workspace: a buffer inside the library's device image, for callers that must not allocate
//     (code recorded into a graph by a harness that forbids it, tight serving loops).  Nothing is ever allocated;
//     every GPU the library runs on holds its copy until the process ends.  One per device, shared by all of its
//     streams: calls that overlap on one device race.  Its counters are zero when the image is loaded.
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
constexpr size_t kStaticBytes = blkq4::kCounterBytes + (size_t{16} << 20);
constexpr int kMaxDevices = 64;

// Host code never uses this name as an address (it is a host-side stand-in for the symbol): it asks
// hipGetSymbolAddress for the array's device address, once per device, and works with that.
static __device__ __align__(256) unsigned char scratch[kStaticBytes];
void* g_static_ptr[kMaxDevices];  // each GPU holds its own copy of the array at its own address

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

extern "C" size_t blkq4_dev_static_workspace_capacity(void) { return kStaticBytes; }

extern "C" int blkq4_dev_static_workspace(void** ptr) {
  *ptr = nullptr;
  int device = 0;
  if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return static_cast<int>(e);
  if (device < 0 || device >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_static_ptr[device] == nullptr) {
    // set-up, once per device, with that device current
    void* p = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)); e != hipSuccess) return static_cast<int>(e);
    if (p == nullptr || (reinterpret_cast<uintptr_t>(p) & 255u) != 0) return static_cast<int>(hipErrorInvalidSymbol);
    g_static_ptr[device] = p;
  }
  *ptr = g_static_ptr[device];
  return 0;
}
