// Small bandwidth-bound helpers of the K-FAC step: axpby (moving average and
// unfused accumulation), diagonal damping and the momentum update rule.
#include <cctype>
#include <cstdlib>
#include <mutex>
#include <new>
#include <string>
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

int timing_begin(int family, hipStream_t stream) {
  TimedRec r;
  r.family = family;
  if (hipEventCreate(&r.start) != hipSuccess) return -1;
  if (hipEventCreate(&r.stop) != hipSuccess) {
    (void)hipEventDestroy(r.start);
    return -1;
  }
  (void)hipEventRecord(r.start, stream);
  g_open.push_back(r);
  return (int)g_open.size() - 1;
}

void timing_end(int index, hipStream_t stream) {
  if (index >= 0 && index < (int)g_open.size()) (void)hipEventRecord(g_open[index].stop, stream);
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

namespace kfac {
namespace {
const char *const kOptionNames[kOptCount] = {
    "syrk_bm64_max",   "syrk_splits",      "conv_rows",       "rows_wm",          "shift_slices5",
    "shift_slices3",   "conv_shift",       "conv_shift_strict", "group_bm64_max", "group_macro",
    "group_panels",    "group_macro_tasks", "group_graded",   "group_side_stream", "inverse_group",  "inverse_border",
    "inverse_lookahead", "inverse_rest_lds", "inverse_align", "precond_tasks",    "bn_stats_loop",
    "host_only"};
struct OptionState {
  bool set[kOptCount] = {};
  double value[kOptCount] = {};
};
OptionState &option_state() {
  static OptionState st;
  static std::once_flag once;
  std::call_once(once, [] {
    for (int i = 0; i < kOptCount; ++i) {
      std::string env = "KFAC_";
      for (const char *c = kOptionNames[i]; *c; ++c) env += (char)toupper((unsigned char)*c);
      if (const char *v = getenv(env.c_str())) {
        char *end = nullptr;
        const double x = strtod(v, &end);
        if (end != v) {
          st.set[i] = true;
          st.value[i] = x;
        }
      }
    }
  });
  return st;
}
int option_index(const char *name) {
  if (name)
    for (int i = 0; i < kOptCount; ++i)
      if (strcmp(name, kOptionNames[i]) == 0) return i;
  return -1;
}
}  // namespace
bool option_is_set(Option o) { return option_state().set[o]; }
bool host_only() {
  const OptionState &st = option_state();
  return st.set[kOptHostOnly] && st.value[kOptHostOnly] != 0.0;
}
double option_value(Option o, double unset_value) {
  const OptionState &st = option_state();
  return st.set[o] ? st.value[o] : unset_value;
}
}  // namespace kfac

extern "C" int kfac_option_set(const char *name, double value) {
  const int i = kfac::option_index(name);
  KFAC_REQUIRE(i >= 0, "unknown option '%s'", name ? name : "(null)");
  kfac::OptionState &st = kfac::option_state();
  st.set[i] = true;
  st.value[i] = value;
  return KFAC_OK;
}

extern "C" int kfac_option_unset(const char *name) {
  const int i = kfac::option_index(name);
  KFAC_REQUIRE(i >= 0, "unknown option '%s'", name ? name : "(null)");
  kfac::option_state().set[i] = false;
  return KFAC_OK;
}

extern "C" int kfac_option_get(const char *name, double *value, int *is_set) {
  const int i = kfac::option_index(name);
  KFAC_REQUIRE(i >= 0, "unknown option '%s'", name ? name : "(null)");
  KFAC_REQUIRE(value && is_set, "null pointer");
  const kfac::OptionState &st = kfac::option_state();
  *is_set = st.set[i] ? 1 : 0;
  *value = st.set[i] ? st.value[i] : 0.0;
  return KFAC_OK;
}

extern "C" int kfac_option_count(void) { return kfac::kOptCount; }

extern "C" const char *kfac_option_name(int index) {
  return index >= 0 && index < kfac::kOptCount ? kfac::kOptionNames[index] : nullptr;
}

extern "C" int kfac_abi_version(void) { return KFAC_ABI_VERSION; }
extern "C" const char *kfac_last_error_string(void) { return kfac::error_buffer(); }

namespace {

constexpr int kThreads = 256;

// a x + b y: the one expression of the single and of the batched kernel (so that
// both round alike)
__device__ __forceinline__ float axpby_value(float x, float y, float a, float b) { return a * x + b * y; }

__global__ __launch_bounds__(kThreads) void axpby_kernel(
    const float *__restrict__ x, float *__restrict__ y, long long n, float a, float b) {
  long long i = (long long)blockIdx.x * kThreads + threadIdx.x;
  const long long stride = (long long)gridDim.x * kThreads;
  // b == 0 overwrites: y is not read (it may be uninitialised memory holding NaN)
  if (b == 0.f) {
    for (; i < n; i += stride) y[i] = a * x[i];
  } else {
    for (; i < n; i += stride) y[i] = axpby_value(x[i], y[i], a, b);
  }
}

// Work of the batched elementwise kernels: a unit is kBatchUnit consecutive
// elements of one array pair; `owner` gives a workgroup its entry with one load.
constexpr int kBatchQuads = 1;                             // 16-byte accesses per thread
constexpr int kBatchUnit = kThreads * 4 * kBatchQuads;     // elements per workgroup
typedef float floatx4a __attribute__((ext_vector_type(4)));

struct AxpbyEntry {
  const float *x;
  float *y;
  long long n;
  int unit0;     // first unit of this entry
  int aligned;   // both arrays start on 16-byte boundaries
};

// MODE 0: y = a x + b y; 1: y = a x (y is not read); 2: y = x / a (an IEEE division)
template <int MODE>
__global__ __launch_bounds__(kThreads) void axpby_batched_kernel(
    const AxpbyEntry *__restrict__ entries, const int *__restrict__ owner, float a, float b) {
  const AxpbyEntry t = entries[owner[blockIdx.x]];
  const long long base = (long long)((int)blockIdx.x - t.unit0) * kBatchUnit;
#pragma unroll
  for (int q = 0; q < kBatchQuads; ++q) {
    const long long i = base + ((long long)q * kThreads + threadIdx.x) * 4;
    if (i >= t.n) continue;
    if (t.aligned && i + 4 <= t.n) {
      const floatx4a x = *reinterpret_cast<const floatx4a *>(t.x + i);
      floatx4a y;
      if (MODE == 1) {
        y = a * x;
      } else if (MODE == 2) {
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = x[e] / a;
      } else {
        y = *reinterpret_cast<const floatx4a *>(t.y + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = axpby_value(x[e], y[e], a, b);
      }
      *reinterpret_cast<floatx4a *>(t.y + i) = y;
    } else {
      const long long end = i + 4 < t.n ? i + 4 : t.n;
      for (long long j = i; j < end; ++j)
        t.y[j] = MODE == 1 ? a * t.x[j] : MODE == 2 ? t.x[j] / a : axpby_value(t.x[j], t.y[j], a, b);
    }
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

// v = momentum * v - lr * g; p += v: the one expression of the single and of the
// batched kernel (so that both round alike).
__device__ __forceinline__ void momentum_step(float &p, float &v, float g, float lr, float momentum) {
  const float nv = momentum * v - lr * g;
  v = nv;
  p += nv;
}

__global__ __launch_bounds__(kThreads) void momentum_kernel(
    float *__restrict__ p, float *__restrict__ v, const float *__restrict__ g,
    long long n, float lr, float momentum) {
  long long i = (long long)blockIdx.x * kThreads + threadIdx.x;
  const long long stride = (long long)gridDim.x * kThreads;
  for (; i < n; i += stride) momentum_step(p[i], v[i], g[i], lr, momentum);
}

// The momentum rule of many parameters in one launch.  A unit is kMomentumUnit
// consecutive elements of one parameter; `owner` gives a workgroup its entry
// with one load.
constexpr int kMomentumQuads = kBatchQuads;
constexpr int kMomentumUnit = kBatchUnit;
constexpr int kEntryGradF16 = 1, kEntryWriteBack = 2, kEntryAligned = 4;

struct MomentumEntry {
  float *param;               // float32 values that are updated (the master copy of a float16 parameter)
  float *v;
  void *grad;                 // float32, or float16 with kEntryGradF16
  unsigned short *param_f16;  // float16 parameter that receives the rounded result, or null
  long long n;
  int unit0;                  // first unit of this entry
  int flags;
};

typedef _Float16 halfx4a __attribute__((ext_vector_type(4)));

template <bool SCALE>
__device__ __forceinline__ float scaled_grad(float g, float loss_scale) {
  return SCALE ? g / loss_scale : g;   // an IEEE division, as the reference's in-place `/=`
}

template <bool SCALE>
__global__ __launch_bounds__(kThreads) void momentum_batched_kernel(
    const MomentumEntry *__restrict__ entries, const int *__restrict__ owner, float lr,
    float momentum, float loss_scale) {
  const MomentumEntry t = entries[owner[blockIdx.x]];
  const long long base = (long long)((int)blockIdx.x - t.unit0) * kMomentumUnit;
  const bool g16 = t.flags & kEntryGradF16;
  const bool wb = SCALE && (t.flags & kEntryWriteBack) && !g16;
#pragma unroll
  for (int q = 0; q < kMomentumQuads; ++q) {
    const long long i = base + ((long long)q * kThreads + threadIdx.x) * 4;
    if (i >= t.n) continue;
    if ((t.flags & kEntryAligned) && i + 4 <= t.n) {
      floatx4a p = *reinterpret_cast<floatx4a *>(t.param + i);
      floatx4a v = *reinterpret_cast<floatx4a *>(t.v + i);
      floatx4a g;
      if (g16) {
        const halfx4a h = *reinterpret_cast<const halfx4a *>(static_cast<const _Float16 *>(t.grad) + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) g[e] = (float)h[e];
      } else {
        g = *reinterpret_cast<const floatx4a *>(static_cast<const float *>(t.grad) + i);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float ge = scaled_grad<SCALE>(g[e], loss_scale);
        float pe = p[e], ve = v[e];
        momentum_step(pe, ve, ge, lr, momentum);
        g[e] = ge;
        p[e] = pe;
        v[e] = ve;
      }
      if (wb) *reinterpret_cast<floatx4a *>(static_cast<float *>(t.grad) + i) = g;
      *reinterpret_cast<floatx4a *>(t.v + i) = v;
      *reinterpret_cast<floatx4a *>(t.param + i) = p;
      if (t.param_f16) {
        halfx4a h;
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = (_Float16)p[e];
        *reinterpret_cast<halfx4a *>(reinterpret_cast<_Float16 *>(t.param_f16) + i) = h;
      }
    } else {
      const long long end = i + 4 < t.n ? i + 4 : t.n;
      for (long long j = i; j < end; ++j) {
        float g = g16 ? (float)static_cast<const _Float16 *>(t.grad)[j] : static_cast<const float *>(t.grad)[j];
        g = scaled_grad<SCALE>(g, loss_scale);
        float p = t.param[j], v = t.v[j];
        momentum_step(p, v, g, lr, momentum);
        if (wb) static_cast<float *>(t.grad)[j] = g;
        t.v[j] = v;
        t.param[j] = p;
        if (t.param_f16) reinterpret_cast<_Float16 *>(t.param_f16)[j] = (_Float16)p;
      }
    }
  }
}

// M[r][c] = 0 for r != c: 16-byte stores over whole rows where the row allows, the
// diagonal entry kept.
__global__ __launch_bounds__(kThreads) void keep_diag_kernel(float *__restrict__ M, int d) {
  const long long total = (long long)d * d;
  for (long long i = (long long)blockIdx.x * kThreads + threadIdx.x; i < total;
       i += (long long)gridDim.x * kThreads) {
    const long long r = i / d;
    if (i - r * d != r) M[i] = 0.f;
  }
}

// out[i] = 1 / (x[i] + (i < split ? v0 : v1)), the sum and the quotient in float64
__global__ __launch_bounds__(kThreads) void recip_add_kernel(const float *__restrict__ x, long long split,
                                                             double v0, double v1, float *__restrict__ out,
                                                             long long n) {
  for (long long i = (long long)blockIdx.x * kThreads + threadIdx.x; i < n; i += (long long)gridDim.x * kThreads)
    out[i] = (float)(1.0 / ((double)x[i] + (i < split ? v0 : v1)));
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
  KFAC_LAUNCH(axpby_kernel, dim3(grid_for(nelems)), dim3(kThreads), 0,
                     kfac::as_stream(stream), x, y, (long long)nelems, a, b);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

extern "C" int kfac_add_diag_f32(float *M, int d, int split, double v0, double v1,
                                 void *stream) {
  KFAC_REQUIRE(d >= 0, "d < 0");
  if (d == 0) return KFAC_OK;
  KFAC_REQUIRE(M != nullptr, "M is null");
  KFAC_LAUNCH(add_diag_kernel, dim3(kfac::ceil_div(d, kThreads)), dim3(kThreads),
                     0, kfac::as_stream(stream), M, d, split, v0, v1);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

extern "C" int kfac_keep_diag_f32(float *M, int d, void *stream) {
  KFAC_REQUIRE(d >= 0 && d <= 46340, "bad dimension %d", d);
  if (d == 0) return KFAC_OK;
  KFAC_REQUIRE(M != nullptr, "M is null");
  KFAC_LAUNCH(keep_diag_kernel, dim3(grid_for((long long)d * d)), dim3(kThreads), 0,
                     kfac::as_stream(stream), M, d);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

extern "C" int kfac_recip_add_f32(const float *x, int64_t split, double v0, double v1, float *out,
                                  int64_t nelems, void *stream) {
  KFAC_REQUIRE(nelems >= 0, "nelems < 0");
  if (nelems == 0) return KFAC_OK;
  KFAC_REQUIRE(x && out, "null pointer");
  KFAC_LAUNCH(recip_add_kernel, dim3(grid_for(nelems)), dim3(kThreads), 0, kfac::as_stream(stream),
                     x, (long long)split, v0, v1, out, (long long)nelems);
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
  KFAC_LAUNCH(add_diag_batched_kernel, dim3(kfac::ceil_div(max_d, kThreads), count), dim3(kThreads),
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
  KFAC_LAUNCH(momentum_kernel, dim3(grid_for(nelems)), dim3(kThreads), 0,
                     kfac::as_stream(stream), param, v, grad, (long long)nelems, lr,
                     momentum);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

struct kfac_momentum_batch {
  std::vector<MomentumEntry> entries;
  std::vector<int> owner;
  kfac::DevTableRing entry_table, owner_table;
};

extern "C" int kfac_momentum_batch_create(kfac_momentum_batch_t *out) {
  KFAC_REQUIRE(out != nullptr, "batch_out is null");
  *out = new (std::nothrow) kfac_momentum_batch;
  if (!*out) return kfac::fail(KFAC_ENOMEM, "out of host memory");
  return KFAC_OK;
}

extern "C" int kfac_momentum_batch_destroy(kfac_momentum_batch_t batch) {
  delete batch;
  return KFAC_OK;
}

extern "C" int kfac_momentum_update_batched_f32(kfac_momentum_batch_t batch, int count,
                                                float *const *params, float *const *vs,
                                                void *const *grads, const int64_t *nelems,
                                                const int32_t *flags, void *const *params_f16,
                                                float lr, float momentum, float loss_scale,
                                                void *stream) {
  KFAC_REQUIRE(batch != nullptr, "batch is null");
  KFAC_REQUIRE(count >= 0, "count < 0");
  if (count == 0) return KFAC_OK;
  KFAC_REQUIRE(params && vs && grads && nelems, "null table");
  KFAC_REQUIRE(loss_scale == loss_scale && loss_scale != 0.f, "loss_scale must be a non-zero number (1 = none)");
  batch->entries.clear();
  batch->owner.clear();
  long long units = 0;
  for (int i = 0; i < count; ++i) {
    KFAC_REQUIRE(nelems[i] >= 0, "parameter %d: nelems < 0", i);
    if (nelems[i] == 0) continue;
    KFAC_REQUIRE(params[i] && vs[i] && grads[i], "parameter %d: null pointer", i);
    const int f = flags ? flags[i] : 0;
    KFAC_REQUIRE((f & ~(KFAC_MOMENTUM_GRAD_F16 | KFAC_MOMENTUM_WRITE_BACK_GRAD)) == 0,
                 "parameter %d: unknown flag bits %d", i, f);
    MomentumEntry e;
    memset(&e, 0, sizeof(e));   // the table is compared bytewise with the uploaded one
    e.param = params[i];
    e.v = vs[i];
    e.grad = grads[i];
    e.param_f16 = params_f16 ? static_cast<unsigned short *>(params_f16[i]) : nullptr;
    e.n = nelems[i];
    e.unit0 = (int)units;
    e.flags = ((f & KFAC_MOMENTUM_GRAD_F16) ? kEntryGradF16 : 0) |
              ((f & KFAC_MOMENTUM_WRITE_BACK_GRAD) ? kEntryWriteBack : 0);
    const uintptr_t bits = reinterpret_cast<uintptr_t>(e.param) | reinterpret_cast<uintptr_t>(e.v) |
                           ((f & KFAC_MOMENTUM_GRAD_F16) ? 2 * reinterpret_cast<uintptr_t>(e.grad)
                                                         : reinterpret_cast<uintptr_t>(e.grad)) |
                           2 * reinterpret_cast<uintptr_t>(e.param_f16);
    if (bits % 16 == 0) e.flags |= kEntryAligned;
    const long long u = kfac::ceil_div<long long>(e.n, kMomentumUnit);
    units += u;
    KFAC_REQUIRE(units < 0x7fffffffLL, "too many elements");
    batch->owner.insert(batch->owner.end(), (size_t)u, (int)batch->entries.size());
    batch->entries.push_back(e);
  }
  if (units == 0) return KFAC_OK;
  hipStream_t s = kfac::as_stream(stream);
  const void *d_entries = nullptr, *d_owner = nullptr;
  if (int rc = batch->entry_table.set(batch->entries.data(), sizeof(MomentumEntry) * batch->entries.size(), s,
                                      &d_entries))
    return rc;
  if (int rc = batch->owner_table.set(batch->owner.data(), sizeof(int) * batch->owner.size(), s, &d_owner))
    return rc;
  if (loss_scale != 1.f)
    KFAC_LAUNCH(momentum_batched_kernel<true>, dim3((unsigned)units), dim3(kThreads), 0, s,
                       static_cast<const MomentumEntry *>(d_entries), static_cast<const int *>(d_owner), lr,
                       momentum, loss_scale);
  else
    KFAC_LAUNCH(momentum_batched_kernel<false>, dim3((unsigned)units), dim3(kThreads), 0, s,
                       static_cast<const MomentumEntry *>(d_entries), static_cast<const int *>(d_owner), lr,
                       momentum, loss_scale);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

struct kfac_axpby_batch {
  std::vector<AxpbyEntry> entries;
  std::vector<int> owner;
  kfac::DevTableRing entry_table, owner_table;
};

extern "C" int kfac_axpby_batch_create(kfac_axpby_batch_t *out) {
  KFAC_REQUIRE(out != nullptr, "batch_out is null");
  *out = new (std::nothrow) kfac_axpby_batch;
  if (!*out) return kfac::fail(KFAC_ENOMEM, "out of host memory");
  return KFAC_OK;
}

extern "C" int kfac_axpby_batch_destroy(kfac_axpby_batch_t batch) {
  delete batch;
  return KFAC_OK;
}

namespace {
int run_axpby_batch(kfac_axpby_batch_t batch, int count, const float *const *xs, float *const *ys,
                    const int64_t *nelems, float a, float b, bool divide, void *stream) {
  KFAC_REQUIRE(batch != nullptr, "batch is null");
  KFAC_REQUIRE(count >= 0, "count < 0");
  if (count == 0) return KFAC_OK;
  KFAC_REQUIRE(xs && ys && nelems, "null table");
  batch->entries.clear();
  batch->owner.clear();
  long long units = 0;
  for (int i = 0; i < count; ++i) {
    KFAC_REQUIRE(nelems[i] >= 0, "pair %d: nelems < 0", i);
    if (nelems[i] == 0) continue;
    KFAC_REQUIRE(xs[i] && ys[i], "pair %d: null pointer", i);
    AxpbyEntry e;
    memset(&e, 0, sizeof(e));   // the table is compared bytewise with the uploaded one
    e.x = xs[i];
    e.y = ys[i];
    e.n = nelems[i];
    e.unit0 = (int)units;
    e.aligned = (reinterpret_cast<uintptr_t>(e.x) | reinterpret_cast<uintptr_t>(e.y)) % 16 == 0;
    const long long u = kfac::ceil_div<long long>(e.n, kBatchUnit);
    units += u;
    KFAC_REQUIRE(units < 0x7fffffffLL, "too many elements");
    batch->owner.insert(batch->owner.end(), (size_t)u, (int)batch->entries.size());
    batch->entries.push_back(e);
  }
  if (units == 0) return KFAC_OK;
  hipStream_t s = kfac::as_stream(stream);
  const void *d_entries = nullptr, *d_owner = nullptr;
  if (int rc = batch->entry_table.set(batch->entries.data(), sizeof(AxpbyEntry) * batch->entries.size(), s,
                                      &d_entries))
    return rc;
  if (int rc = batch->owner_table.set(batch->owner.data(), sizeof(int) * batch->owner.size(), s, &d_owner))
    return rc;
  if (divide)
    KFAC_LAUNCH(axpby_batched_kernel<2>, dim3((unsigned)units), dim3(kThreads), 0, s,
                       static_cast<const AxpbyEntry *>(d_entries), static_cast<const int *>(d_owner), a, b);
  else if (b == 0.f)
    KFAC_LAUNCH(axpby_batched_kernel<1>, dim3((unsigned)units), dim3(kThreads), 0, s,
                       static_cast<const AxpbyEntry *>(d_entries), static_cast<const int *>(d_owner), a, b);
  else
    KFAC_LAUNCH(axpby_batched_kernel<0>, dim3((unsigned)units), dim3(kThreads), 0, s,
                       static_cast<const AxpbyEntry *>(d_entries), static_cast<const int *>(d_owner), a, b);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}
}  // namespace

extern "C" int kfac_axpby_batched_f32(kfac_axpby_batch_t batch, int count, const float *const *xs,
                                      float *const *ys, const int64_t *nelems, float a, float b,
                                      void *stream) {
  return run_axpby_batch(batch, count, xs, ys, nelems, a, b, false, stream);
}

extern "C" int kfac_div_batched_f32(kfac_axpby_batch_t batch, int count, float *const *arrays,
                                    const int64_t *nelems, float divisor, void *stream) {
  KFAC_REQUIRE(divisor == divisor && divisor != 0.f, "the divisor must be a non-zero number");
  return run_axpby_batch(batch, count, arrays, arrays, nelems, divisor, 0.f, true, stream);
}
