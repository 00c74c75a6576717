// Shared host-side helpers of libkfac_hip: error reporting and device tables.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../include/kfac_hip.h"

namespace kfac {

// Last error of the calling thread, returned by kfac_last_error_string().
char *error_buffer();

inline int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

#define KFAC_HIP_CHECK(expr)                                                   \
  do {                                                                         \
    hipError_t e_ = (expr);                                                    \
    if (e_ != hipSuccess)                                                      \
      return ::kfac::fail(KFAC_EHIP, "%s failed: %s (%s:%d)", #expr,           \
                          hipGetErrorString(e_), __FILE__, __LINE__);          \
  } while (0)

#define KFAC_REQUIRE(cond, ...)                                                \
  do {                                                                         \
    if (!(cond)) return ::kfac::fail(KFAC_EINVAL, __VA_ARGS__);                \
  } while (0)

// A device array mirrored by a host shadow.  set() uploads only when the
// contents changed; the (rare) upload waits for `stream` first so that work
// already enqueued against the old contents is not disturbed.
class DevTable {
 public:
  DevTable() = default;
  DevTable(const DevTable &) = delete;
  DevTable &operator=(const DevTable &) = delete;
  ~DevTable() {
    if (dev_) (void)hipFree(dev_);
  }
  int set(const void *host, size_t bytes, hipStream_t stream) {
    if (bytes == shadow_.size() && dev_ &&
        (bytes == 0 || memcmp(host, shadow_.data(), bytes) == 0))
      return KFAC_OK;
    KFAC_HIP_CHECK(hipStreamSynchronize(stream));
    if (bytes > capacity_) {
      if (dev_) KFAC_HIP_CHECK(hipFree(dev_));
      dev_ = nullptr;
      capacity_ = 0;
      KFAC_HIP_CHECK(hipMalloc(&dev_, bytes ? bytes : 4));
      capacity_ = bytes ? bytes : 4;
    }
    if (bytes) KFAC_HIP_CHECK(hipMemcpy(dev_, host, bytes, hipMemcpyHostToDevice));
    shadow_.assign(static_cast<const char *>(host),
                   static_cast<const char *>(host) + bytes);
    return KFAC_OK;
  }
  template <typename T>
  T *as() const {
    return static_cast<T *>(dev_);
  }

 private:
  void *dev_ = nullptr;
  size_t capacity_ = 0;
  std::vector<char> shadow_;
};

inline hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }

// Brackets one kernel launch with HIP events while benchmark timing is on.
bool timing_on();
void timing_begin(int family, hipStream_t stream);
void timing_end(hipStream_t stream);

struct TimedLaunch {
  hipStream_t stream;
  bool on;
  TimedLaunch(int family, hipStream_t s) : stream(s), on(timing_on()) {
    if (on) timing_begin(family, s);
  }
  ~TimedLaunch() {
    if (on) timing_end(stream);
  }
};

template <typename T>
inline T ceil_div(T a, T b) {
  return (a + b - 1) / b;
}

}  // namespace kfac
