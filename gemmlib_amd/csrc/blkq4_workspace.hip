// Workspace of the split tile kernels (arrival counters + fp32 partial tiles): where it comes from.
//
//   blkq4_dev_workspace: buffers owned by the library, one per (device, stream, recording) -- see
//     blkq4_workspace_table.h for why that is the key -- allocated by the first call that needs one and kept until
//     blkq4_dev_workspace_release or the end of the process.  A call that is being recorded into a graph may
//     allocate too (the allocation is no stream operation; the thread's capture mode is set to relaxed around it,
//     as tensor libraries do for their own allocations during capture); the graph keeps using that buffer whatever
//     stream it is launched on later, and nothing else ever uses it.  hipStreamPerThread names a different stream
//     in every host thread, so the handle identifies nothing: such calls get no buffer (unsplit kernels).
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
#include "blkq4_workspace_table.h"

namespace {

constexpr size_t kPoolBytes = blkq4::kCounterBytes + (size_t{32} << 20);
constexpr size_t kStaticBytes = blkq4::kCounterBytes + (size_t{16} << 20);
constexpr int kMaxDevices = 64;

// Host code never uses this name as an address (it is a host-side stand-in for the symbol): it asks
// hipGetSymbolAddress for the array's device address, once per device, and works with that.
static __device__ __align__(256) unsigned char scratch[kStaticBytes];
void* g_static_ptr[kMaxDevices];  // each GPU holds its own copy of the array at its own address

__global__ void clear_counters(int* counters) {
  for (unsigned i = threadIdx.x; i < blkq4::kCounterBytes / sizeof(int); i += blockDim.x) counters[i] = 0;
}

std::mutex g_mutex;
blkq4::WorkspaceTable g_table;

// (device, stream, recording) of a call on `stream` made now; false: calls on this stream get no buffer
bool key_of(hipStream_t stream, blkq4::WorkspaceKey* key, hipError_t* error) {
  *error = hipSuccess;
  if (stream == hipStreamPerThread) return false;
  int device = 0;
  if ((*error = hipGetDevice(&device)) != hipSuccess) return false;
  unsigned long long capture = 0;
  if (stream != nullptr && stream != hipStreamLegacy) {  // the legacy default stream cannot record
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    if ((*error = hipStreamGetCaptureInfo(stream, &status, &id)) != hipSuccess) return false;
    if (status == hipStreamCaptureStatusActive) capture = id + 1;  // never 0 for a recording
  }
  *key = blkq4::WorkspaceKey{device, stream, capture};
  return true;
}

}  // namespace

extern "C" size_t blkq4_dev_workspace_capacity(void) { return kPoolBytes; }

extern "C" int blkq4_dev_workspace(void* stream_ptr, void** ptr) {
  *ptr = nullptr;
  blkq4::WorkspaceKey key{};
  hipError_t e = hipSuccess;
  if (!key_of(static_cast<hipStream_t>(stream_ptr), &key, &e)) return static_cast<int>(e);
  std::lock_guard<std::mutex> lock(g_mutex);
  if (void* have = g_table.find(key)) {
    *ptr = have;
    return 0;
  }
  if (!g_table.has_room(key.capture != 0)) return 0;  // no workspace for this call: unsplit kernels
  // An allocation is allowed while this or another thread records a graph only in relaxed mode.  The counters
  // are cleared on a stream of this function's own and waited for, so they are zero when this returns, whether
  // the caller's stream is executing or being recorded.
  hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
  if (e = hipThreadExchangeStreamCaptureMode(&mode); e != hipSuccess) return static_cast<int>(e);
  void* p = nullptr;
  hipStream_t own = nullptr;
  e = hipMalloc(&p, kPoolBytes);
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
  g_table.add(key, p);
  *ptr = p;
  return 0;
}

// What a split GEMM issued on `stream` now would find: *state = 1 the call has a buffer, 0 it would allocate one,
// -1 it would run the unsplit plan (no room for another buffer, or hipStreamPerThread).
extern "C" int blkq4_dev_workspace_info(void* stream_ptr, int* state, int* in_use, int* capacity) {
  blkq4::WorkspaceKey key{};
  hipError_t e = hipSuccess;
  const bool keyed = key_of(static_cast<hipStream_t>(stream_ptr), &key, &e);
  if (e != hipSuccess) return static_cast<int>(e);
  std::lock_guard<std::mutex> lock(g_mutex);
  *state = !keyed ? -1 : g_table.find(key) != nullptr ? 1 : g_table.has_room(key.capture != 0) ? 0 : -1;
  *in_use = g_table.in_use();
  *capacity = blkq4::WorkspaceTable::capacity();
  return 0;
}

// Frees every buffer.  The caller promises that no GEMM of this library is executing or queued and that no graph
// holding one will be launched again.
extern "C" int blkq4_dev_workspace_release(void) {
  std::lock_guard<std::mutex> lock(g_mutex);
  int current = 0;
  hipError_t first = hipGetDevice(&current);
  if (first != hipSuccess) return static_cast<int>(first);
  g_table.release_all([&](int device, void* p) {
    hipError_t e = hipSetDevice(device);
    if (e == hipSuccess) e = hipFree(p);
    if (e != hipSuccess && first == hipSuccess) first = e;
  });
  (void)hipSetDevice(current);
  return static_cast<int>(first);
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
