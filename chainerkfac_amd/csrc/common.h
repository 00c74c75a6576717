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

// Host-only mode (option host_only = 1): no call reaches the HIP runtime.  Plans are
// built, arguments checked, task tables filled and every launch site passed with its
// grid computed, but nothing is allocated, copied or launched: the planners and their
// index arithmetic then run on a machine without a GPU, under a host sanitizer.
bool host_only();

#define KFAC_HIP_CHECK(expr)                                                   \
  do {                                                                         \
    if (!::kfac::host_only()) {                                                \
      hipError_t e_ = (expr);                                                  \
      if (e_ != hipSuccess)                                                    \
        return ::kfac::fail(KFAC_EHIP, "%s failed: %s (%s:%d)", #expr,         \
                            hipGetErrorString(e_), __FILE__, __LINE__);        \
    }                                                                          \
  } while (0)

// Every kernel launch of the library goes through here.
#define KFAC_LAUNCH(...)                                                       \
  do {                                                                         \
    if (!::kfac::host_only()) hipLaunchKernelGGL(__VA_ARGS__);                 \
  } while (0)

#define KFAC_REQUIRE(cond, ...)                                                \
  do {                                                                         \
    if (!(cond)) return ::kfac::fail(KFAC_EINVAL, __VA_ARGS__);                \
  } while (0)

// A device array mirrored by a host shadow.  set() uploads only when the contents
// changed, and then without stopping the host: the new contents go to a pinned
// staging buffer and from there to the device with a copy ordered on `stream`
// (behind the launches already queued there that read the old contents; launches
// that read a table on another stream must have been joined into `stream` before
// the next set(), as the library's own side streams and the callers' lanes are).
// The staging buffer is reused only after its previous copy has finished (an
// event the host waits for; in steady state it is long past).
class DevTable {
 public:
  DevTable() = default;
  DevTable(const DevTable &) = delete;
  DevTable &operator=(const DevTable &) = delete;
  ~DevTable() {
    if (dev_ == &host_only_address_) dev_ = nullptr;
    if (dev_) (void)hipFree(dev_);
    if (staging_) (void)hipHostFree(staging_);
    if (copied_) (void)hipEventDestroy(copied_);
  }
  bool matches(const void *host, size_t bytes) const {
    return bytes == shadow_.size() && dev_ &&
           (bytes == 0 || memcmp(host, shadow_.data(), bytes) == 0);
  }
  // true once a call made while `stream` was being captured has used these contents:
  // a graph replays against them, so they must never change again
  bool pinned() const { return pinned_; }
  int set(const void *host, size_t bytes, hipStream_t stream) {
    if (host_only()) return set_sync(host, bytes);
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cs) != hipSuccess) {
      (void)hipGetLastError();
      cs = hipStreamCaptureStatusActive;
    }
    const bool capturing = cs != hipStreamCaptureStatusNone;
    if (matches(host, bytes)) {
      if (capturing) pinned_ = true;
      // the contents may still be on their way, queued on another stream: this one waits for them
      // (a capture starts after the device has been synchronised, so nothing is pending then)
      if (copy_pending_ && !capturing) {
        if (hipEventQuery(copied_) == hipSuccess)
          copy_pending_ = false;
        else if (stream != upload_stream_)
          KFAC_HIP_CHECK(hipStreamWaitEvent(stream, copied_, 0));
        (void)hipGetLastError();   // hipErrorNotReady of the query is not an error
      }
      return KFAC_OK;
    }
    // an upload cannot be part of a capture (its source is gone by the time of a replay)
    if (capturing)
      return ::kfac::fail(KFAC_EINVAL,
                          "a device table would have to be uploaded during stream capture: call once "
                          "with the same arguments before capturing");
    if (pinned_)
      return ::kfac::fail(KFAC_EINVAL,
                          "a device table that a captured graph replays against would have to change: "
                          "use another plan for other arguments");
    if (!copied_) KFAC_HIP_CHECK(hipEventCreateWithFlags(&copied_, hipEventDisableTiming));
    if (copy_pending_) {
      KFAC_HIP_CHECK(hipEventSynchronize(copied_));
      copy_pending_ = false;
    }
    if (bytes > capacity_) {
      // (hipFree waits for the device: nothing still reads the old array)
      if (dev_) KFAC_HIP_CHECK(hipFree(dev_));
      if (staging_) KFAC_HIP_CHECK(hipHostFree(staging_));
      dev_ = staging_ = nullptr;
      capacity_ = 0;
      const size_t cap = bytes + bytes / 2 + 64;
      KFAC_HIP_CHECK(hipMalloc(&dev_, cap));
      capacity_ = cap;
    }
    if (!dev_) {   // an empty table still has an address
      KFAC_HIP_CHECK(hipMalloc(&dev_, 64));
      capacity_ = 64;
    }
    if (bytes) {
      if (!staging_) KFAC_HIP_CHECK(hipHostMalloc(&staging_, capacity_, hipHostMallocDefault));
      memcpy(staging_, host, bytes);
      KFAC_HIP_CHECK(hipMemcpyAsync(dev_, staging_, bytes, hipMemcpyHostToDevice, stream));
      KFAC_HIP_CHECK(hipEventRecord(copied_, stream));
      copy_pending_ = true;
      upload_stream_ = stream;
    }
    shadow_.assign(static_cast<const char *>(host),
                   static_cast<const char *>(host) + bytes);
    return KFAC_OK;
  }
  // Upload that has finished when the call returns (plan creation: the tables are read by
  // launches on whatever streams the plan is used on later).
  int set_sync(const void *host, size_t bytes) {
    if (host_only()) {   // the contents only: nothing lives on a device
      shadow_.assign(static_cast<const char *>(host), static_cast<const char *>(host) + bytes);
      if (!dev_) dev_ = &host_only_address_;
      return KFAC_OK;
    }
    if (matches(host, bytes)) return KFAC_OK;
    if (pinned_)
      return ::kfac::fail(KFAC_EINVAL, "a device table that a captured graph replays against would have to change");
    if (copy_pending_) {
      KFAC_HIP_CHECK(hipEventSynchronize(copied_));
      copy_pending_ = false;
    }
    if (bytes > capacity_ || !dev_) {
      if (dev_) KFAC_HIP_CHECK(hipFree(dev_));
      if (staging_) KFAC_HIP_CHECK(hipHostFree(staging_));
      dev_ = staging_ = nullptr;
      capacity_ = 0;
      KFAC_HIP_CHECK(hipMalloc(&dev_, bytes ? bytes : 64));
      capacity_ = bytes ? bytes : 64;
    }
    if (bytes) KFAC_HIP_CHECK(hipMemcpy(dev_, host, bytes, hipMemcpyHostToDevice));
    shadow_.assign(static_cast<const char *>(host), static_cast<const char *>(host) + bytes);
    return KFAC_OK;
  }
  template <typename T>
  T *as() const {
    return static_cast<T *>(dev_);
  }

 private:
  void *dev_ = nullptr;
  void *staging_ = nullptr;
  size_t capacity_ = 0;
  std::vector<char> shadow_;
  hipEvent_t copied_ = nullptr;
  hipStream_t upload_stream_ = nullptr;
  bool copy_pending_ = false, pinned_ = false;
  char host_only_address_ = 0;   // what as<T>() returns in host-only mode (never dereferenced)
  // the contents last set, for checks of the tables on the host
 public:
  const std::vector<char> &shadow() const { return shadow_; }
};

// A few device copies of a table whose contents alternate between a small number
// of versions (e.g. the pointer / scale table of a grouped launch with beta = 0
// on the first micro-batch and beta = 1 afterwards, or gradient arrays that move
// from step to step): a version that is resident is used as it is, a new one
// replaces the least recently used copy that no captured graph replays against.
class DevTableRing {
 public:
  static constexpr int kSlots = 4;
  int set(const void *host, size_t bytes, hipStream_t stream, const void **dev_out) {
    ++clock_;
    int lru = -1;
    for (int i = 0; i < kSlots; ++i) {
      if (slots_[i].matches(host, bytes)) {
        if (int rc = slots_[i].set(host, bytes, stream)) return rc;   // pins it under capture
        stamp_[i] = clock_;
        *dev_out = slots_[i].as<const void>();
        return KFAC_OK;
      }
      if (!slots_[i].pinned() && (lru < 0 || stamp_[i] < stamp_[lru])) lru = i;
    }
    if (lru < 0)
      return ::kfac::fail(KFAC_EINVAL,
                          "every copy of this device table belongs to a captured graph: use another "
                          "plan for other arguments");
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

// Brackets one kernel launch (or a run of launches on one stream) with HIP events
// while benchmark timing is on.  Brackets may nest.
bool timing_on();
int timing_begin(int family, hipStream_t stream);   // index of the bracket, -1: none
void timing_end(int index, hipStream_t stream);

struct TimedLaunch {
  hipStream_t stream;
  int index;
  TimedLaunch(int family, hipStream_t s) : stream(s), index(timing_on() ? timing_begin(family, s) : -1) {}
  ~TimedLaunch() {
    if (index >= 0) timing_end(index, stream);
  }
  TimedLaunch(const TimedLaunch &) = delete;
  TimedLaunch &operator=(const TimedLaunch &) = delete;
};

// Tuning options of the library (kfac_option_set / kfac_option_get; the environment
// variable KFAC_<NAME IN CAPITALS> gives a starting value and is read once per process).
// An option that was never set leaves the built-in choice in force.
enum Option : int {
  kOptSyrkBm64Max,        // single-factor SYRK: largest side that takes 64-tiles
  kOptSyrkSplits,         // single-factor SYRK: forced number of k-slices
  kOptConvRows,           // 0: k x k convolutions skip the compile-time rows kernels
  kOptRowsWm,             // rows kernels: 1 = 64-tiles, 2 = 128-tiles
  kOptShiftSlices5,       // shifted correlations: k-slices of the five-shift groups
  kOptShiftSlices3,       //                       ... of the three-shift group (both must be set)
  kOptConvShift,          // shifted correlations: 0 = off, else the least channel count
  kOptConvShiftStrict,    // 1: a workspace too small for that route is an error, not a fallback
  kOptGroupBm64Max,       // grouped covariances: largest side that takes 64-tiles
  kOptGroupMacro,         // grouped covariances: 1 = macro-tile kernel for slabs of several 128-tiles
  kOptGroupPanels,        // grouped launches: panel units per workgroup
  kOptGroupMacroTasks,    // macro-tile launches: workgroups per launch
  kOptGroupGraded,        // grouped covariances: 0 = equal slices, n >= 2: the last n-th is halved
  kOptGroupSideStream,    // grouped covariances: 0 = every launch on the caller's stream
  kOptInverseGroup,       // inverse: block columns per trailing update
  kOptInverseBorder,      // inverse: 0 = matrices of 128 m + 1 rows are tiled whole
  kOptInverseLookahead,   // inverse: 0 = everything on the caller's stream
  kOptInverseRestLds,     // inverse: bytes of LDS the trailing update asks for
  kOptInverseAlign,       // inverse: 0 = sweeps start together ... 100 = end together
  kOptPrecondTasks,       // grouped preconditioning: workgroups per launch
  kOptBnStatsLoop,        // 1: batch-norm statistics always by the looping kernel
  kOptHostOnly,           // 1: host-only mode: plan, check and count, never touch a GPU
  kOptCount
};
bool option_is_set(Option o);
double option_value(Option o, double unset_value);
inline int option_int(Option o, int unset_value) { return (int)option_value(o, (double)unset_value); }

template <typename T>
inline T ceil_div(T a, T b) {
  return (a + b - 1) / b;
}

}  // namespace kfac
