// Error plumbing of the C ABI: a status code plus a thread-local message (include/dsgx.h).
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/dsgx.h"

namespace dsgx {
// records the message for dsgx_last_error() and returns `code`
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
inline size_t align256(size_t b) { return (b + 255) / 256 * 256; }
int num_cus_cached();
// Raises a kernel's dynamic-LDS limit when `lds` needs it; remembered per kernel, so that a launch inside a stream
// capture (after one eager launch of the same shape) makes no attribute call.
int allow_dynamic_lds(const void* kern, size_t lds);
}  // namespace dsgx

#define DSGX_HIP(x)                                                                                          \
  do {                                                                                                       \
    hipError_t e_ = (x);                                                                                     \
    if (e_ != hipSuccess) return ::dsgx::fail(DSGX_EHIP, "%s:%d: %s: %s", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
  } while (0)
