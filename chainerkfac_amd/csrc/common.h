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
  bool matches(const void *host, size_t bytes) const {
    return bytes == shadow_.size() && dev_ &&
           (bytes == 0 || memcmp(host, shadow_.data(), bytes) == 0);
  }
  int set(const void *host, size_t bytes, hipStream_t stream) {
    if (matches(host, bytes)) return KFAC_OK;
    // an upload waits for the stream and copies synchronously: impossible while the
    // stream is being captured into a graph (and it would invalidate the capture)
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cs) != hipSuccess) {
      (void)hipGetLastError();
      cs = hipStreamCaptureStatusActive;
    }
    if (cs != hipStreamCaptureStatusNone)
      return ::kfac::fail(KFAC_EINVAL,
                          "a device table would have to be uploaded during stream capture: call once "
                          "with the same arguments before capturing");
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

// A few device copies of a table whose contents alternate between a small number
// of versions (e.g. the pointer / scale table of a grouped launch with beta = 0
// on the first micro-batch and beta = 1 afterwards): a version that is resident
// is used as it is, a new one replaces the least recently used copy.  A HIP
// graph captured over a call keeps replaying against the copy it saw.
class DevTableRing {
 public:
  static constexpr int kSlots = 4;
  int set(const void *host, size_t bytes, hipStream_t stream, const void **dev_out) {
    ++clock_;
    int lru = 0;
    for (int i = 0; i < kSlots; ++i) {
      if (slots_[i].matches(host, bytes)) {
        stamp_[i] = clock_;
        *dev_out = slots_[i].as<const void>();
        return KFAC_OK;
      }
      if (stamp_[i] < stamp_[lru]) lru = i;
    }
    if (int rc = slots_[lru].set(host, bytes, stream)) return rc;
    stamp_[lru] = clock_;
    *dev_out = slots_[lru].as<const void>();
    return KFAC_OK;
  }

 private:
  DevTable slots_[kSlots];
  unsigned long long stamp_[kSlots] = {};
  unsigned long long clock_ = 0;
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
