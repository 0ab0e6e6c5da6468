// Ids handed over in pageable host memory (csrc/core/preprocess.cu:98-99 of the reference copies them with one
// cudaMemcpyAsync): the copy to the device, through a pinned staging buffer filled by several threads, with the
// transfers of the pieces that are ready issued behind them.  The runtime's own path for pageable memory stages with one
// thread; at 13.6 MB of ids per batch that copy is as long as the rest of the training step.
#pragma once
#include "common.h"

namespace hctr {

class HostStager {
 public:
  HostStager() = default;
  ~HostStager();
  HostStager(const HostStager &) = delete;
  HostStager &operator=(const HostStager &) = delete;

  // Enqueues on `s` the transfer of `bytes` bytes at pageable `src` to device memory `dst` and returns once `src` has
  // been read (the caller may reuse it).  The staging buffer is reused by the next call on this object, which first
  // waits for the transfers enqueued here.
  // narrow_ids: `src` holds 64-bit ids and `dst` receives bytes / 2 bytes of 32-bit ones, half the bytes on the bus;
  // an id that does not fit (a negative one too) arrives as 0xffffffff.
  void copy(void *dst, const void *src, size_t bytes, hipStream_t s, bool narrow_ids = false);

 private:
  unsigned char *pinned_ = nullptr;
  size_t cap_ = 0;
  hipEvent_t sent_ = nullptr; // behind the last transfer out of the staging buffer
};

// threads that fill staging buffers, the calling one included; HETUCTR_COPY_THREADS (1..64), default 8
int host_copy_threads();

} // namespace hctr
