// Shared by every translation unit of libdkernel_hip.so: error reporting that
// never lets a C++ exception cross the C ABI, and small host helpers.
#pragma once

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/dkernel_hip.h"

namespace dk {

// Stores a printf-style message for dk_last_error() on this thread and
// returns `code`, so call sites read `return fail(DK_ERR_INVALID, "...")`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

#define DK_REQUIRE(cond, ...)                                   \
  do {                                                          \
    if (!(cond)) return ::dk::fail(DK_ERR_INVALID, __VA_ARGS__); \
  } while (0)

#define DK_HIP_CHECK(expr)                                                              \
  do {                                                                                  \
    hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess)                                                               \
      return ::dk::fail(DK_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));     \
  } while (0)

inline int cdiv(int a, int b) { return (a + b - 1) / b; }
inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }

}  // namespace dk
