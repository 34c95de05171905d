// Host-side helpers of the C ABI: status/error plumbing and argument checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/xllm_hip_paged_kv.h"

namespace xllm_hip {

// Thread-local message of the last failure; read through xllm_hip_last_error().
char* last_error_buffer();

inline int fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return status;
}

#define XLLM_HIP_REQUIRE(cond, ...)                                     \
  do {                                                                  \
    if (!(cond)) return ::xllm_hip::fail(XLLM_HIP_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    return fail(XLLM_HIP_RUNTIME_ERROR, "%s: %s", what, hipGetErrorString(e));
  }
  return XLLM_HIP_OK;
}

inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
inline int ilog2(int64_t v) {
  int r = 0;
  while ((int64_t(1) << (r + 1)) <= v) ++r;
  return r;
}

}  // namespace xllm_hip
