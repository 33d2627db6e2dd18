// Shared by the translation units of libmist_search.so: error reporting.
#pragma once
#include <hip/hip_runtime.h>

namespace mist {
// Records a printf-style message for mist_last_error() (per thread) and returns `code`.
int fail(int code, const char *fmt, ...);
}  // namespace mist

#define MIST_HIP_CHECK(expr)                                                                \
  do {                                                                                      \
    hipError_t err__ = (expr);                                                              \
    if (err__ != hipSuccess)                                                                \
      return mist::fail(MIST_E_HIP, "%s failed: %s", #expr, hipGetErrorString(err__));      \
  } while (0)
