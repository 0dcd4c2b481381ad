// Process-wide plumbing shared by the C ABI translation units: the library's own
// stream, counted allocation wrappers (hot-path allocation audit) and the
// fail-closed result helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include "nerva_hip_api.h"

namespace nv {

// True when at least one HIP device is usable; otherwise *hip_error is set to
// NERVA_HIP_ERROR_NO_DEVICE (mirrors the reference's stub build: native_stubs.rs:5-33).
bool device_ready(int32_t *hip_error);
hipStream_t library_stream();
hipStream_t library_stream_if_created();   // null before the first library_stream() call: creates nothing
hipStream_t resolve_stream(void *stream);

hipError_t counted_malloc(void **ptr, size_t bytes);
hipError_t counted_host_malloc(void **ptr, size_t bytes);
uint64_t allocation_count();

// memset(out, 0); status = -1. Returns false when out is null.
template <typename Result>
inline bool begin_result(Result *out) {
  if (out == nullptr) return false;
  memset(out, 0, sizeof(*out));
  out->status = -1;
  return true;
}

inline uint64_t fnv1a_bytes(const void *data, size_t bytes) {
  const uint8_t *p = static_cast<const uint8_t *>(data);
  uint64_t hash = 0xcbf29ce484222325ull;
  for (size_t i = 0; i < bytes; ++i) {
    hash ^= p[i];
    hash *= 0x00000100000001b3ull;
  }
  return hash;
}

}  // namespace nv
