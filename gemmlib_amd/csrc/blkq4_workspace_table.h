// Who owns which workspace of the split tile kernels: the bookkeeping, host-only and free of HIP calls so that it
// can be compiled and tested on a machine without a GPU.  blkq4_workspace.hip does the allocating.
//
// A workspace (arrival counters + fp32 partial tiles) may be used by one split GEMM at a time.  Calls that are
// ordered with respect to each other can share one, calls that may overlap cannot.  What orders two calls:
//   - eager calls on the same stream of the same device;
//   - calls recorded on the same stream during the same capture (the graph keeps them in that order).
// A graph can be launched on any stream at any later time, so a recording never shares a buffer with eager calls
// or with another recording: the key is (device, stream handle, capture id), capture id 0 meaning "not recording".
//
// The number of buffers is bounded (each is 32 MiB and is kept until blkq4_gemm_workspace_release_sm80 or the end
// of the process): a call that finds no buffer and no room for a new one runs the unsplit plan, which needs none.

#pragma once

#include <stddef.h>

namespace blkq4 {

struct WorkspaceKey {
  int device;
  const void* stream;
  unsigned long long capture;  // 0: the stream is executing, not recording
};

constexpr int kMaxEagerWorkspaces = 16;     // streams with a buffer of their own for eager calls
constexpr int kMaxCapturedWorkspaces = 16;  // recordings with a buffer of their own

class WorkspaceTable {
 public:
  // the buffer of `key`, or nullptr
  void* find(const WorkspaceKey& key) const {
    for (int i = 0; i < count_; ++i) {
      if (slots_[i].key.device == key.device && slots_[i].key.stream == key.stream &&
          slots_[i].key.capture == key.capture) {
        return slots_[i].ptr;
      }
    }
    return nullptr;
  }
  // whether a key of this kind (recording or not) could still get a buffer
  bool has_room(bool captured) const {
    return captured ? captured_ < kMaxCapturedWorkspaces : count_ - captured_ < kMaxEagerWorkspaces;
  }
  // false when there is no room (nothing changes then) or the key has a buffer already
  bool add(const WorkspaceKey& key, void* ptr) {
    const bool captured = key.capture != 0;
    if (ptr == nullptr || !has_room(captured) || find(key) != nullptr) return false;
    slots_[count_].key = key;
    slots_[count_].ptr = ptr;
    ++count_;
    if (captured) ++captured_;
    return true;
  }
  int in_use() const { return count_; }
  int in_use_by_recordings() const { return captured_; }
  static constexpr int capacity() { return kMaxEagerWorkspaces + kMaxCapturedWorkspaces; }
  // hands every buffer to `free_buffer(device, ptr)` and forgets it
  template <class Free>
  void release_all(Free&& free_buffer) {
    for (int i = 0; i < count_; ++i) free_buffer(slots_[i].key.device, slots_[i].ptr);
    count_ = 0;
    captured_ = 0;
  }

 private:
  struct Slot {
    WorkspaceKey key;
    void* ptr;
  };
  Slot slots_[kMaxEagerWorkspaces + kMaxCapturedWorkspaces] = {};
  int count_ = 0;
  int captured_ = 0;
};

}  // namespace blkq4
