// Shared host-side helpers for the C ABI: last-error string and HIP status checks.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <mutex>
#include <set>
#include <utility>

namespace stir {

// Thread-local message returned by stir_last_error(); the same convention as
// TVMAPISetLastError / TVMGetLastError (include/tvm/runtime/c_runtime_api.h:181-190
// in the reference): an entry point returns -1 after recording why.
void set_error(const char* fmt, ...);
const char* get_error();

inline int fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
inline int fail(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  set_error("%s", buf);
  return -1;
}

}  // namespace stir

#define STIR_HIP(expr)                                                                     \
  do {                                                                                     \
    hipError_t _e = (expr);                                                                \
    if (_e != hipSuccess)                                                                  \
      return stir::fail("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__,   \
                        __LINE__);                                                         \
  } while (0)

#define STIR_REQUIRE(cond, ...)                   \
  do {                                            \
    if (!(cond)) return stir::fail(__VA_ARGS__);  \
  } while (0)

#define STIR_LAUNCH_CHECK() STIR_HIP(hipGetLastError())

namespace stir {
constexpr int kWave = 64;
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }

// Compute units of the current device (asked once per device and thread; 0 on failure).
inline int compute_units() {
  static thread_local int cached_dev = -1, cached = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev != cached_dev) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached_dev = dev, cached = cus;
  }
  return cached;
}

// LDS a workgroup may ask for on the current device (0 on failure)
inline size_t lds_bytes_per_workgroup() {
  static thread_local int cached_dev = -1;
  static thread_local size_t cached = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev != cached_dev) {
    int bytes = 0;
    if (hipDeviceGetAttribute(&bytes, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) return 0;
    cached_dev = dev, cached = (size_t)bytes;
  }
  return cached;
}

// Kernels that use more than 64 KB of dynamic LDS have to be told so once per device.
inline int allow_lds(const void* fn) {
  static std::mutex mu;
  static std::set<std::pair<int, const void*>> done;
  int dev = 0;
  STIR_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  if (done.count({dev, fn})) return 0;
  STIR_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes_per_workgroup()));
  done.insert({dev, fn});
  return 0;
}
}  // namespace stir
