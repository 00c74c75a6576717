// Trace-norm pi and in-place damping of (A, G) factor pairs, all layers in one
// launch.  Follows chainerkfac/optimizers/fisher_block.py:23-42 (pi),
// fisher_blocks/connection.py:66-77 (diagonal values) and the fill_diagonal of
// fisher_block.py:175: pi is a float32, 1/pi is formed in float32, the added
// values pi*rW and (1/pi)*rW are float64 and the damped diagonal is rounded to
// float32 when stored.
#include "common.h"

namespace {

constexpr int kThreads = 256;

struct DampTables {
  float *const *A;
  float *const *G;
  const int *dA;
  const int *dG;
  const double *rW;
};

__device__ double block_sum(double v, double *sh) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  return sh[0] + sh[1] + sh[2] + sh[3];
}

__global__ __launch_bounds__(kThreads) void pi_damp_kernel(DampTables tb, int use_pi,
                                                           float *__restrict__ pi_out) {
  __shared__ double sh[4];
  const int l = blockIdx.x;
  float *__restrict__ A = tb.A[l];
  float *__restrict__ G = tb.G[l];
  const int dA = tb.dA[l], dG = tb.dG[l];
  float pi = 1.0f;
  if (use_pi) {
    double ta = 0.0, tg = 0.0;
    for (int i = threadIdx.x; i < dA; i += kThreads) ta += (double)A[(long long)i * dA + i];
    for (int i = threadIdx.x; i < dG; i += kThreads) tg += (double)G[(long long)i * dG + i];
    const float trA = (float)block_sum(ta, sh);
    const float trG = (float)block_sum(tg, sh);
    const float lnorm = trA * (float)dG;
    const float rnorm = trG * (float)dA;
    pi = sqrtf(lnorm / rnorm);
  }
  const double rW = tb.rW[l];
  const double addA = (double)pi * rW;
  const double addG = (double)(1.0f / pi) * rW;
  for (int i = threadIdx.x; i < dA; i += kThreads) {
    const long long at = (long long)i * dA + i;
    A[at] = (float)((double)A[at] + addA);
  }
  for (int i = threadIdx.x; i < dG; i += kThreads) {
    const long long at = (long long)i * dG + i;
    G[at] = (float)((double)G[at] + addG);
  }
  if (pi_out && threadIdx.x == 0) pi_out[l] = pi;
}

}  // namespace

struct kfac_damp_plan {
  int count = 0;
  std::vector<void *> a, g;
  kfac::DevTable d_A, d_G, d_dA, d_dG, d_rW;
};

extern "C" int kfac_damp_plan_create(int count, const int32_t *dimsA, const int32_t *dimsG,
                                     kfac_damp_plan_t *plan_out) {
  KFAC_REQUIRE(plan_out != nullptr, "plan_out is null");
  *plan_out = nullptr;
  KFAC_REQUIRE(count >= 0, "count < 0");
  KFAC_REQUIRE(count == 0 || (dimsA && dimsG), "null table");
  for (int i = 0; i < count; ++i)
    KFAC_REQUIRE(dimsA[i] > 0 && dimsG[i] > 0, "layer %d: bad dimension", i);
  auto *p = new (std::nothrow) kfac_damp_plan;
  if (!p) return kfac::fail(KFAC_ENOMEM, "out of host memory");
  p->count = count;
  int rc = p->d_dA.set_sync(dimsA, sizeof(int) * count);
  if (rc == KFAC_OK) rc = p->d_dG.set_sync(dimsG, sizeof(int) * count);
  if (rc != KFAC_OK) {
    delete p;
    return rc;
  }
  *plan_out = p;
  return KFAC_OK;
}

extern "C" int kfac_damp_plan_destroy(kfac_damp_plan_t plan) {
  delete plan;
  return KFAC_OK;
}

extern "C" int kfac_pi_damp_batched_f32(kfac_damp_plan_t plan, float *const *A_ptrs,
                                        float *const *G_ptrs, const double *rW, int use_pi,
                                        float *pi_out_dev, void *stream) {
  KFAC_REQUIRE(plan != nullptr, "plan is null");
  if (plan->count == 0) return KFAC_OK;
  KFAC_REQUIRE(A_ptrs && G_ptrs && rW, "null table");
  for (int i = 0; i < plan->count; ++i)
    KFAC_REQUIRE(A_ptrs[i] && G_ptrs[i], "layer %d: null pointer", i);
  hipStream_t s = kfac::as_stream(stream);
  int rc = plan->d_A.set(A_ptrs, sizeof(void *) * plan->count, s);
  if (rc == KFAC_OK) rc = plan->d_G.set(G_ptrs, sizeof(void *) * plan->count, s);
  if (rc == KFAC_OK) rc = plan->d_rW.set(rW, sizeof(double) * plan->count, s);
  if (rc != KFAC_OK) return rc;
  DampTables tb;
  tb.A = plan->d_A.as<float *const>();
  tb.G = plan->d_G.as<float *const>();
  tb.dA = plan->d_dA.as<const int>();
  tb.dG = plan->d_dG.as<const int>();
  tb.rW = plan->d_rW.as<const double>();
  KFAC_LAUNCH(pi_damp_kernel, dim3(plan->count), dim3(kThreads), 0, s, tb, use_pi,
                     pi_out_dev);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}
