// Shared host-side helpers of libmfsdp_hip: error reporting and device queries.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/mfsdp_hip.h"

namespace mfsdp {

// Stores a printf-style message for mfsdp_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Number of compute units of the current device (cached per device).
int device_cu_count();

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

#define MFSDP_HIP_TRY(expr)                                                                          \
  do {                                                                                               \
    hipError_t err__ = (expr);                                                                       \
    if (err__ != hipSuccess)                                                                         \
      return ::mfsdp::fail(MFSDP_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(err__), \
                           __FILE__, __LINE__);                                                      \
  } while (0)

// Launch errors (bad configuration) surface through hipGetLastError right after the launch.
#define MFSDP_CHECK_LAUNCH(name)                                                                  \
  do {                                                                                            \
    hipError_t err__ = hipGetLastError();                                                         \
    if (err__ != hipSuccess)                                                                      \
      return ::mfsdp::fail(MFSDP_ERR_HIP, "launch of %s failed: %s", name, hipGetErrorString(err__)); \
  } while (0)

}  // namespace mfsdp
