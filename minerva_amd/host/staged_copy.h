// Host-to-device copy out of pageable memory through a pinned staging area in two
// alternating halves: the CPU fills one while the DMA engine drains the other (left to the
// runtime, such a copy runs at a fraction of the link's rate: 4 against 27 GB/s measured for
// the 158 MB batch of the AlexNet shape).  Synchronises `stream` before it returns, so the
// host buffer may go away.  Used by the ArrayLoader operator (reference cuda.cpp:592-598) and
// by the batch prefetch.
#pragma once
#include <cstddef>
#include <cstring>

#include "mnv_hip.h"

namespace minerva {

inline int StagedHostToDevice(void* dst_device, const void* src_host, size_t bytes, void* stream,
                              void* staging, size_t staging_bytes) {
  const char* src = static_cast<const char*>(src_host);
  char* dst = static_cast<char*>(dst_device);
  const size_t half = staging_bytes / 2;
  if (!staging || half == 0 || bytes <= half) {
    int rc = mnv_memcpy_h2d(dst, src, bytes, stream);
    const int rs = mnv_stream_sync(stream);
    return rc != MNV_OK ? rc : rs;
  }
  char* stage = static_cast<char*>(staging);
  void* drained[2] = {nullptr, nullptr};
  int rc = mnv_event_create_ordering(&drained[0]);
  if (rc == MNV_OK) rc = mnv_event_create_ordering(&drained[1]);
  size_t off = 0;
  for (int i = 0; off < bytes && rc == MNV_OK; ++i, off += half) {
    const int b = i & 1;
    const size_t n = bytes - off < half ? bytes - off : half;
    if (i >= 2) rc = mnv_event_sync(drained[b]);  // this half has left for the device
    if (rc != MNV_OK) break;
    std::memcpy(stage + b * half, src + off, n);
    rc = mnv_memcpy_h2d(dst + off, stage + b * half, n, stream);
    if (rc == MNV_OK) rc = mnv_event_record(drained[b], stream);
  }
  const int rs = mnv_stream_sync(stream);
  if (drained[0]) mnv_event_destroy(drained[0]);
  if (drained[1]) mnv_event_destroy(drained[1]);
  return rc != MNV_OK ? rc : rs;
}

}  // namespace minerva
