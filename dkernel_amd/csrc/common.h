// Shared by every translation unit of libdkernel_hip.so: error reporting that
// never lets a C++ exception cross the C ABI, and small host helpers.
#pragma once

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/dkernel_hip.h"

namespace dk {

// Stores a printf-style message for dk_last_error() on this thread and
// returns `code`, so call sites read `return fail(DK_ERR_INVALID, "...")`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

// Names of the kernels that the current forward / backward call has launched on this thread
// (dk_last_kernels()): `kernel` plus the template arguments of the launcher that chose it, taken
// from its __PRETTY_FUNCTION__.  Tests and the benchmark use it to tell which path ran.
void note_kernel(const char *kernel, const char *launcher_signature);
void clear_kernels();
#define DK_NOTE_KERNEL(kernel) ::dk::note_kernel(kernel, __PRETTY_FUNCTION__)

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

// Raises a kernel's dynamic LDS limit once per device: the attribute belongs to the current
// device's copy of the kernel, so a process that uses several GPUs has to set it on each.
// `done` holds one bit per device ordinal; a race between threads only repeats the call.
#define DK_ALLOW_DYNAMIC_LDS(kernel, bytes)                                                          \
  do {                                                                                               \
    static std::atomic<uint64_t> done_{0};                                                           \
    int dev_ = 0;                                                                                    \
    DK_HIP_CHECK(hipGetDevice(&dev_));                                                               \
    const uint64_t bit_ = 1ull << (dev_ & 63);                                                       \
    if (!(done_.load(std::memory_order_relaxed) & bit_)) {                                           \
      DK_HIP_CHECK(hipFuncSetAttribute((const void *)(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (bytes))); \
      done_.fetch_or(bit_, std::memory_order_relaxed);                                               \
    }                                                                                                \
  } while (0)

inline int cdiv(int a, int b) { return (a + b - 1) / b; }
inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }

}  // namespace dk
