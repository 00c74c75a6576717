// Small bandwidth-bound helpers of the K-FAC step: axpby (moving average and
// unfused accumulation), diagonal damping and the momentum update rule.
#include "common.h"

namespace kfac {
char *error_buffer() {
  static thread_local char buf[512] = "";
  return buf;
}
}  // namespace kfac

namespace kfac {
namespace {
struct TimedRec {
  int family;
  hipEvent_t start, stop;
};
bool g_timing = false;
std::vector<TimedRec> g_open;
long long g_launches[KFAC_TIMED_FAMILIES];
double g_total_ms[KFAC_TIMED_FAMILIES];
}  // namespace

bool timing_on() { return g_timing; }

void timing_begin(int family, hipStream_t stream) {
  TimedRec r;
  r.family = family;
  if (hipEventCreate(&r.start) != hipSuccess) return;
  if (hipEventCreate(&r.stop) != hipSuccess) {
    (void)hipEventDestroy(r.start);
    return;
  }
  (void)hipEventRecord(r.start, stream);
  g_open.push_back(r);
}

void timing_end(hipStream_t stream) {
  if (!g_open.empty()) (void)hipEventRecord(g_open.back().stop, stream);
}

static void timing_collect() {
  for (auto &r : g_open) {
    float ms = 0.f;
    if (hipEventSynchronize(r.stop) == hipSuccess &&
        hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
      g_launches[r.family] += 1;
      g_total_ms[r.family] += ms;
    }
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  g_open.clear();
}
}  // namespace kfac

extern "C" int kfac_timing_enable(int on) {
  kfac::timing_collect();
  if (on) {
    for (int i = 0; i < KFAC_TIMED_FAMILIES; ++i) {
      kfac::g_launches[i] = 0;
      kfac::g_total_ms[i] = 0.0;
    }
  }
  kfac::g_timing = on != 0;
  return KFAC_OK;
}

extern "C" int kfac_timing_read(int family, int64_t *launches, double *total_ms) {
  KFAC_REQUIRE(family >= 0 && family < KFAC_TIMED_FAMILIES, "bad kernel family %d", family);
  KFAC_REQUIRE(launches && total_ms, "null pointer");
  kfac::timing_collect();
  *launches = kfac::g_launches[family];
  *total_ms = kfac::g_total_ms[family];
  return KFAC_OK;
}

extern "C" int kfac_abi_version(void) { return KFAC_ABI_VERSION; }
extern "C" const char *kfac_last_error_string(void) { return kfac::error_buffer(); }

namespace {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void axpby_kernel(
    const float *__restrict__ x, float *__restrict__ y, long long n, float a, float b) {
  long long i = (long long)blockIdx.x * kThreads + threadIdx.x;
  const long long stride = (long long)gridDim.x * kThreads;
  // b == 0 overwrites: y is not read (it may be uninitialised memory holding NaN)
  if (b == 0.f) {
    for (; i < n; i += stride) y[i] = a * x[i];
  } else {
    for (; i < n; i += stride) y[i] = a * x[i] + b * y[i];
  }
}

__global__ __launch_bounds__(kThreads) void add_diag_kernel(
    float *__restrict__ M, int d, int split, double v0, double v1) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < d) {
    const long long at = (long long)i * d + i;
    M[at] = (float)((double)M[at] + (i < split ? v0 : v1));
  }
}

__global__ __launch_bounds__(kThreads) void momentum_kernel(
    float *__restrict__ p, float *__restrict__ v, const float *__restrict__ g,
    long long n, float lr, float momentum) {
  long long i = (long long)blockIdx.x * kThreads + threadIdx.x;
  const long long stride = (long long)gridDim.x * kThreads;
  for (; i < n; i += stride) {
    const float nv = momentum * v[i] - lr * g[i];
    v[i] = nv;
    p[i] += nv;
  }
}

int grid_for(long long n) {
  long long g = kfac::ceil_div<long long>(n, kThreads);
  const long long cap = 256LL * 32;
  return (int)(g < cap ? g : cap);
}

}  // namespace

extern "C" int kfac_axpby_f32(const float *x, float *y, int64_t nelems, float a,
                              float b, void *stream) {
  KFAC_REQUIRE(nelems >= 0, "nelems < 0");
  if (nelems == 0) return KFAC_OK;
  KFAC_REQUIRE(x && y, "null pointer");
  hipLaunchKernelGGL(axpby_kernel, dim3(grid_for(nelems)), dim3(kThreads), 0,
                     kfac::as_stream(stream), x, y, (long long)nelems, a, b);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

extern "C" int kfac_add_diag_f32(float *M, int d, int split, double v0, double v1,
                                 void *stream) {
  KFAC_REQUIRE(d >= 0, "d < 0");
  if (d == 0) return KFAC_OK;
  KFAC_REQUIRE(M != nullptr, "M is null");
  hipLaunchKernelGGL(add_diag_kernel, dim3(kfac::ceil_div(d, kThreads)), dim3(kThreads),
                     0, kfac::as_stream(stream), M, d, split, v0, v1);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

extern "C" int kfac_momentum_update_f32(float *param, float *v, const float *grad,
                                        int64_t nelems, float lr, float momentum,
                                        void *stream) {
  KFAC_REQUIRE(nelems >= 0, "nelems < 0");
  if (nelems == 0) return KFAC_OK;
  KFAC_REQUIRE(param && v && grad, "null pointer");
  hipLaunchKernelGGL(momentum_kernel, dim3(grid_for(nelems)), dim3(kThreads), 0,
                     kfac::as_stream(stream), param, v, grad, (long long)nelems, lr,
                     momentum);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}
