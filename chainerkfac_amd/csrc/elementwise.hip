// Small bandwidth-bound helpers of the K-FAC step: axpby (moving average and
// unfused accumulation), diagonal damping and the momentum update rule.
#include <new>
#include <vector>

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

struct DiagItem {
  float *M;
  int d, split;
  double v0, v1;
};

// blockIdx.y = matrix, blockIdx.x = chunk of its diagonal
__global__ __launch_bounds__(kThreads) void add_diag_batched_kernel(const DiagItem *__restrict__ items) {
  const DiagItem it = items[blockIdx.y];
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < it.d) {
    const long long at = (long long)i * it.d + i;
    it.M[at] = (float)((double)it.M[at] + (i < it.split ? it.v0 : it.v1));
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

struct kfac_diag_batch {
  std::vector<DiagItem> host;
  kfac::DevTableRing table;
};

extern "C" int kfac_diag_batch_create(kfac_diag_batch_t *out) {
  KFAC_REQUIRE(out != nullptr, "batch_out is null");
  *out = new (std::nothrow) kfac_diag_batch;
  if (!*out) return kfac::fail(KFAC_ENOMEM, "out of host memory");
  return KFAC_OK;
}

extern "C" int kfac_diag_batch_destroy(kfac_diag_batch_t batch) {
  delete batch;
  return KFAC_OK;
}

extern "C" int kfac_add_diag_batched_f32(kfac_diag_batch_t batch, int count, float *const *mats,
                                         const int32_t *dims, const int32_t *splits,
                                         const double *v0, const double *v1, void *stream) {
  KFAC_REQUIRE(batch != nullptr, "batch is null");
  KFAC_REQUIRE(count >= 0, "count < 0");
  if (count == 0) return KFAC_OK;
  KFAC_REQUIRE(mats && dims && splits && v0 && v1, "null table");
  KFAC_REQUIRE(count <= 65535, "more than 65535 matrices");
  batch->host.resize(count);
  int max_d = 0;
  for (int i = 0; i < count; ++i) {
    KFAC_REQUIRE(dims[i] >= 0 && (dims[i] == 0 || mats[i]), "matrix %d: bad dimension or null pointer", i);
    batch->host[i] = DiagItem{mats[i], dims[i], splits[i], v0[i], v1[i]};
    max_d = dims[i] > max_d ? dims[i] : max_d;
  }
  if (max_d == 0) return KFAC_OK;
  hipStream_t s = kfac::as_stream(stream);
  const void *dev = nullptr;
  if (int rc = batch->table.set(batch->host.data(), sizeof(DiagItem) * (size_t)count, s, &dev)) return rc;
  hipLaunchKernelGGL(add_diag_batched_kernel, dim3(kfac::ceil_div(max_d, kThreads), count), dim3(kThreads),
                     0, s, static_cast<const DiagItem *>(dev));
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
