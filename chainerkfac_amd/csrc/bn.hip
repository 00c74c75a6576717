// Per-sample gradient matrix of a batch-normalisation layer,
//   U[s] = [ sum_hw gy'[s] * h[s] | sum_hw gy'[s] ],   h = (x - mean) / sqrt(var + eps),
// with the batch mean and biased variance recomputed from x (two passes, as
// numpy's mean/var do), gy' = gy * gy_scale.  The activation and its gradient
// are each read from HBM once more than strictly needed (x twice, gy once) and
// nothing of their size is written.  One wave owns one (sample, channel) slab.
// Replaces chainerkfac/optimizers/fisher_blocks/normalizations/
// batch_normalization.py:86-119.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

__device__ __forceinline__ float wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
  return __shfl(v, 0, 64);
}

// s1[slab] = sum x
__global__ __launch_bounds__(kThreads) void bn_sum_kernel(const float *__restrict__ x,
                                                          int nslab, int hw,
                                                          float *__restrict__ s1) {
  const int slab = blockIdx.x * kWaves + (threadIdx.x >> 6);
  if (slab >= nslab) return;
  const int lane = threadIdx.x & 63;
  const float *p = x + (long long)slab * hw;
  float acc = 0.f;
  if ((hw & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    const float4 *p4 = reinterpret_cast<const float4 *>(p);
    for (int i = lane; i < hw / 4; i += 64) {
      const float4 v = p4[i];
      acc += (v.x + v.y) + (v.z + v.w);
    }
  } else {
    for (int i = lane; i < hw; i += 64) acc += p[i];
  }
  acc = wave_sum(acc);
  if (lane == 0) s1[slab] = acc;
}

// per slab: ss = sum (x-mean)^2, sg = sum gy, sgx = sum gy (x-mean)
__global__ __launch_bounds__(kThreads) void bn_moments_kernel(
    const float *__restrict__ x, const float *__restrict__ gy, int n, int c, int hw,
    const float *__restrict__ s1, float *__restrict__ ss, float *__restrict__ sg,
    float *__restrict__ sgx) {
  const int nslab = n * c;
  const int slab = blockIdx.x * kWaves + (threadIdx.x >> 6);
  if (slab >= nslab) return;
  const int lane = threadIdx.x & 63;
  const int ch = slab % c;
  float tot = 0.f;
  for (int s = lane; s < n; s += 64) tot += s1[s * c + ch];
  const float mean = wave_sum(tot) / ((float)n * (float)hw);
  const float *px = x + (long long)slab * hw;
  const float *pg = gy + (long long)slab * hw;
  float a = 0.f, b = 0.f, g = 0.f;
  if ((hw & 3) == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gy)) & 15) == 0) {
    const float4 *x4 = reinterpret_cast<const float4 *>(px);
    const float4 *g4 = reinterpret_cast<const float4 *>(pg);
    for (int i = lane; i < hw / 4; i += 64) {
      const float4 xv = x4[i];
      const float4 gv = g4[i];
      const float d0 = xv.x - mean, d1 = xv.y - mean, d2 = xv.z - mean, d3 = xv.w - mean;
      a += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
      b += (gv.x + gv.y) + (gv.z + gv.w);
      g += (gv.x * d0 + gv.y * d1) + (gv.z * d2 + gv.w * d3);
    }
  } else {
    for (int i = lane; i < hw; i += 64) {
      const float dv = px[i] - mean;
      const float gv = pg[i];
      a += dv * dv;
      b += gv;
      g += gv * dv;
    }
  }
  a = wave_sum(a);
  b = wave_sum(b);
  g = wave_sum(g);
  if (lane == 0) {
    ss[slab] = a;
    sg[slab] = b;
    sgx[slab] = g;
  }
}

// U[s][ch] = gy_scale * rstd[ch] * sgx ; U[s][off_beta + ch] = gy_scale * sg
__global__ __launch_bounds__(kThreads) void bn_finish_kernel(
    int n, int c, int hw, float eps, float gy_scale, int has_gamma, int has_beta,
    const float *__restrict__ ss, const float *__restrict__ sg, const float *__restrict__ sgx,
    float *__restrict__ U) {
  const int idx = blockIdx.x * kThreads + threadIdx.x;
  if (idx >= n * c) return;
  const int ch = idx % c, s = idx / c;
  const int width = c * (has_gamma + has_beta);
  if (has_gamma) {
    float tot = 0.f;
    for (int t = 0; t < n; ++t) tot += ss[t * c + ch];
    const float var = tot / ((float)n * (float)hw);
    const float rstd = 1.0f / sqrtf(var + eps);
    U[(long long)s * width + ch] = gy_scale * (sgx[idx] * rstd);
  }
  if (has_beta) U[(long long)s * width + (has_gamma ? c : 0) + ch] = gy_scale * sg[idx];
}

}  // namespace

extern "C" size_t kfac_bn_workspace_bytes(int n, int c) {
  if (n <= 0 || c <= 0) return 0;
  return (size_t)4 * n * c * sizeof(float);
}

extern "C" int kfac_bn_grad_matrix_f32(const float *x, const float *gy, int n, int c, int hw,
                                       float eps, float gy_scale, int has_gamma, int has_beta,
                                       float *U, void *ws, size_t ws_bytes, void *stream) {
  KFAC_REQUIRE(n > 0 && c > 0 && hw > 0, "bad shape n=%d c=%d hw=%d", n, c, hw);
  KFAC_REQUIRE((long long)n * c < 0x7fffffffLL, "too many (sample, channel) slabs");
  KFAC_REQUIRE(has_gamma || has_beta, "gamma and beta are both absent");
  KFAC_REQUIRE(x && gy && U, "null pointer");
  if (ws == nullptr || ws_bytes < kfac_bn_workspace_bytes(n, c))
    return kfac::fail(KFAC_ENOMEM, "batch-norm workspace too small: %zu < %zu bytes", ws_bytes,
                      kfac_bn_workspace_bytes(n, c));
  hipStream_t s = kfac::as_stream(stream);
  const int nslab = n * c;
  float *s1 = static_cast<float *>(ws);
  float *ss = s1 + nslab, *sg = ss + nslab, *sgx = sg + nslab;
  const int grid = kfac::ceil_div(nslab, kWaves);
  hipLaunchKernelGGL(bn_sum_kernel, dim3(grid), dim3(kThreads), 0, s, x, nslab, hw, s1);
  hipLaunchKernelGGL(bn_moments_kernel, dim3(grid), dim3(kThreads), 0, s, x, gy, n, c, hw, s1, ss,
                     sg, sgx);
  hipLaunchKernelGGL(bn_finish_kernel, dim3(kfac::ceil_div(nslab, kThreads)), dim3(kThreads), 0, s,
                     n, c, hw, eps, gy_scale, has_gamma ? 1 : 0, has_beta ? 1 : 0, ss, sg, sgx, U);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}
