// Shared host-side helpers of the C ABI: thread-local error text, argument
// checks, launch checks.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/blksprs_amd.h"

namespace bsa {

char *error_buffer();
int fail(int code, const char *fmt, ...);

inline hipStream_t as_stream(bsa_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Checks the launch that was just enqueued.
inline int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(BSA_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return BSA_OK;
}

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }

}  // namespace bsa

#define BSA_REQUIRE(cond, ...)                                  \
  do {                                                          \
    if (!(cond)) return ::bsa::fail(BSA_EINVAL, __VA_ARGS__);   \
  } while (0)

#define BSA_HIP(call)                                                                         \
  do {                                                                                        \
    hipError_t e_ = (call);                                                                   \
    if (e_ != hipSuccess) return ::bsa::fail(BSA_ELAUNCH, "%s: %s", #call, hipGetErrorString(e_)); \
  } while (0)
