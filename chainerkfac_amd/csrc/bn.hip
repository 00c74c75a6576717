// Per-sample gradient matrix of a batch-normalisation layer,
//   U[s] = [ sum_hw gy'[s] * h[s] | sum_hw gy'[s] ],   h = (x - mean) / sqrt(var + eps),
// with the batch mean and biased variance recomputed from x (centred second
// moments, as numpy's var computes them), gy' = gy * gy_scale.  The activation
// and its gradient are each read from HBM once and nothing of their size is
// written.  One wave owns one (sample, channel) slab.
// Replaces chainerkfac/optimizers/fisher_blocks/normalizations/
// batch_normalization.py:86-119.
#include <cstdlib>
#include <new>
#include <vector>

#include "common.h"

namespace {

constexpr int kThreads = 256;

// Sum over a group of LPS consecutive lanes, delivered to every lane of the group.
template <int LPS>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int o = LPS / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, LPS);
  return v;
}

// LPS lanes (a wave, or a quarter wave for small images) per (sample, channel)
// slab of hw pixels: the slab's mean, its
// centred second moment, sum gy and sum gy (x - slab mean).  The second sweep
// over the slab hits cache; per-channel batch statistics are assembled from
// these exactly (pairwise combination of means and centred moments), so x and
// gy are each read from HBM once.
template <int LPS>
__global__ __launch_bounds__(kThreads) void bn_stats_kernel(
    const float *__restrict__ x, const float *__restrict__ gy, int nslab, int hw,
    float *__restrict__ smean, float *__restrict__ sm2, float *__restrict__ sg,
    float *__restrict__ sgx) {
  // idle groups of the last workgroup redo the last slab, so that every lane
  // takes part in the shuffles
  int slab = (blockIdx.x * kThreads + threadIdx.x) / LPS;
  if (slab >= nslab) slab = nslab - 1;
  const int lane = threadIdx.x % LPS;
  const float *px = x + (long long)slab * hw;
  const float *pg = gy + (long long)slab * hw;
  const bool vec =
      (hw & 3) == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gy)) & 15) == 0;
  float acc = 0.f;
  if (vec) {
    const float4 *x4 = reinterpret_cast<const float4 *>(px);
    for (int i = lane; i < hw / 4; i += LPS) {
      const float4 v = x4[i];
      acc += (v.x + v.y) + (v.z + v.w);
    }
  } else {
    for (int i = lane; i < hw; i += LPS) acc += px[i];
  }
  const float mean = group_sum<LPS>(acc) / (float)hw;
  float a = 0.f, b = 0.f, g = 0.f;
  if (vec) {
    const float4 *x4 = reinterpret_cast<const float4 *>(px);
    const float4 *g4 = reinterpret_cast<const float4 *>(pg);
    for (int i = lane; i < hw / 4; i += LPS) {
      const float4 xv = x4[i];
      const float4 gv = g4[i];
      const float d0 = xv.x - mean, d1 = xv.y - mean, d2 = xv.z - mean, d3 = xv.w - mean;
      a += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
      b += (gv.x + gv.y) + (gv.z + gv.w);
      g += (gv.x * d0 + gv.y * d1) + (gv.z * d2 + gv.w * d3);
    }
  } else {
    for (int i = lane; i < hw; i += LPS) {
      const float dv = px[i] - mean;
      const float gv = pg[i];
      a += dv * dv;
      b += gv;
      g += gv * dv;
    }
  }
  a = group_sum<LPS>(a);
  b = group_sum<LPS>(b);
  g = group_sum<LPS>(g);
  if (lane == 0) {
    smean[slab] = mean;
    sm2[slab] = a;
    sg[slab] = b;
    sgx[slab] = g;
  }
}

// The same for slabs of at most 4 * LPS * Q pixels whose rows are 16-byte aligned:
// the lane's Q quads of x stay in registers between the two sweeps (x is loaded
// once, all loads of a sweep are in flight together), and so do those of gy.
template <int LPS, int Q>
__global__ __launch_bounds__(kThreads) void bn_stats_reg_kernel(
    const float *__restrict__ x, const float *__restrict__ gy, int nslab, int hw,
    float *__restrict__ smean, float *__restrict__ sm2, float *__restrict__ sg,
    float *__restrict__ sgx) {
  int slab = (blockIdx.x * kThreads + threadIdx.x) / LPS;
  if (slab >= nslab) slab = nslab - 1;
  const int lane = threadIdx.x % LPS;
  const float4 *x4 = reinterpret_cast<const float4 *>(x + (long long)slab * hw);
  const float4 *g4 = reinterpret_cast<const float4 *>(gy + (long long)slab * hw);
  const int nq = hw / 4;
  float4 xv[Q], gv[Q];
#pragma unroll
  for (int k = 0; k < Q; ++k) {
    const int i = lane + k * LPS;
    xv[k] = i < nq ? x4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int k = 0; k < Q; ++k) {
    const int i = lane + k * LPS;
    gv[k] = i < nq ? g4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float acc = 0.f;
#pragma unroll
  for (int k = 0; k < Q; ++k) acc += (xv[k].x + xv[k].y) + (xv[k].z + xv[k].w);
  const float mean = group_sum<LPS>(acc) / (float)hw;
  float a = 0.f, b = 0.f, g = 0.f;
#pragma unroll
  for (int k = 0; k < Q; ++k) {
    if (lane + k * LPS < nq) {
      const float d0 = xv[k].x - mean, d1 = xv[k].y - mean, d2 = xv[k].z - mean, d3 = xv[k].w - mean;
      a += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
      b += (gv[k].x + gv[k].y) + (gv[k].z + gv[k].w);
      g += (gv[k].x * d0 + gv[k].y * d1) + (gv[k].z * d2 + gv[k].w * d3);
    }
  }
  a = group_sum<LPS>(a);
  b = group_sum<LPS>(b);
  g = group_sum<LPS>(g);
  if (lane == 0) {
    smean[slab] = mean;
    sm2[slab] = a;
    sg[slab] = b;
    sgx[slab] = g;
  }
}

// 64 channels per workgroup (lanes on consecutive channels, so every access is
// coalesced), the samples dealt to the 4 waves: batch mean and variance of the
// channel from the slab statistics, then the channel's column(s) of U.
//   sum_hw gy (x - mean_c) = sgx_s + (mean_s - mean_c) sg_s
__device__ __forceinline__ void bn_finish_block(
    int block, int n, int c, int hw, float eps, float gy_scale, int has_gamma, int has_beta,
    const float *__restrict__ smean, const float *__restrict__ sm2, const float *__restrict__ sg,
    const float *__restrict__ sgx, float *__restrict__ U) {
  __shared__ float part[2][4][64];
  const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
  const int ch = block * 64 + lane;
  const bool live = ch < c;
  const int width = c * (has_gamma + has_beta);
  float mean = 0.f, rstd = 0.f;
  if (has_gamma) {
    float tot = 0.f;
    if (live) {
#pragma unroll 8
      for (int s = grp; s < n; s += 4) tot += smean[s * c + ch];
    }
    part[0][grp][lane] = tot;
    __syncthreads();
    mean = ((part[0][0][lane] + part[0][1][lane]) + (part[0][2][lane] + part[0][3][lane])) / (float)n;
    float m2 = 0.f, dev = 0.f;
    if (live) {
#pragma unroll 8
      for (int s = grp; s < n; s += 4) {
        const float dm = smean[s * c + ch] - mean;
        m2 += sm2[s * c + ch];
        dev += dm * dm;
      }
    }
    part[1][grp][lane] = m2 + (float)hw * dev;
    __syncthreads();
    const float var = ((part[1][0][lane] + part[1][1][lane]) + (part[1][2][lane] + part[1][3][lane])) /
                      ((float)n * (float)hw);
    rstd = 1.0f / sqrtf(var + eps);
  }
  if (!live) return;
#pragma unroll 8
  for (int s = grp; s < n; s += 4) {
    const int idx = s * c + ch;
    const float b = sg[idx];
    if (has_gamma) {
      const float g = sgx[idx] + (smean[idx] - mean) * b;
      U[(long long)s * width + ch] = gy_scale * (g * rstd);
    }
    if (has_beta) U[(long long)s * width + (has_gamma ? c : 0) + ch] = gy_scale * b;
  }
}

__global__ __launch_bounds__(256) void bn_finish_kernel(
    int n, int c, int hw, float eps, float gy_scale, int has_gamma, int has_beta,
    const float *__restrict__ smean, const float *__restrict__ sm2, const float *__restrict__ sg,
    const float *__restrict__ sgx, float *__restrict__ U) {
  bn_finish_block(blockIdx.x, n, c, hw, eps, gy_scale, has_gamma, has_beta, smean, sm2, sg, sgx, U);
}

// The finish step of many layers in one launch: a unit is 64 channels of one layer.
struct BnFinishItem {
  const float *stats;   // [4][n][c]: slab mean, centred second moment, sum gy, sum gy (x - slab mean)
  float *U;
  int n, c, hw, has_gamma, has_beta;
  float eps, gy_scale;
};

__global__ __launch_bounds__(256) void bn_finish_batched_kernel(const BnFinishItem *__restrict__ items,
                                                                const int2 *__restrict__ units) {
  const int2 u = units[blockIdx.x];
  const BnFinishItem it = items[u.x];
  const long long nslab = (long long)it.n * it.c;
  bn_finish_block(u.y, it.n, it.c, it.hw, it.eps, it.gy_scale, it.has_gamma, it.has_beta, it.stats,
                  it.stats + nslab, it.stats + 2 * nslab, it.stats + 3 * nslab, it.U);
}

// The slab statistics of one layer (the kernel is chosen from the slab size and alignment).
void launch_stats(const float *x, const float *gy, int nslab, int hw, float *smean, float *sm2, float *sg,
                  float *sgx, hipStream_t s) {
  const bool vec =
      (hw & 3) == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gy)) & 15) == 0;
  const bool stats_loop = kfac::option_int(kfac::kOptBnStatsLoop, 0) != 0;   // tuning override
  if (vec && hw <= 4 * 16 * 4 && !stats_loop)
    KFAC_LAUNCH((bn_stats_reg_kernel<16, 4>), dim3(kfac::ceil_div(nslab, kThreads / 16)),
                       dim3(kThreads), 0, s, x, gy, nslab, hw, smean, sm2, sg, sgx);
  else if (vec && hw > 256 && hw <= 4 * 64 * 13 && !stats_loop)
    KFAC_LAUNCH((bn_stats_reg_kernel<64, 13>), dim3(kfac::ceil_div(nslab, kThreads / 64)),
                       dim3(kThreads), 0, s, x, gy, nslab, hw, smean, sm2, sg, sgx);
  else if (hw <= 256)
    KFAC_LAUNCH(bn_stats_kernel<16>, dim3(kfac::ceil_div(nslab, kThreads / 16)),
                       dim3(kThreads), 0, s, x, gy, nslab, hw, smean, sm2, sg, sgx);
  else
    KFAC_LAUNCH(bn_stats_kernel<64>, dim3(kfac::ceil_div(nslab, kThreads / 64)),
                       dim3(kThreads), 0, s, x, gy, nslab, hw, smean, sm2, sg, sgx);
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
  float *smean = static_cast<float *>(ws);
  float *sm2 = smean + nslab, *sg = sm2 + nslab, *sgx = sg + nslab;
  kfac::TimedLaunch timed(KFAC_TIMED_BN, s);
  launch_stats(x, gy, nslab, hw, smean, sm2, sg, sgx, s);
  KFAC_LAUNCH(bn_finish_kernel, dim3(kfac::ceil_div(c, 64)), dim3(256), 0, s, n, c, hw, eps,
                     gy_scale, has_gamma ? 1 : 0, has_beta ? 1 : 0, smean, sm2, sg, sgx, U);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

extern "C" int kfac_bn_stats_f32(const float *x, const float *gy, int n, int c, int hw, float *stats,
                                 size_t stats_bytes, void *stream) {
  KFAC_REQUIRE(n > 0 && c > 0 && hw > 0, "bad shape n=%d c=%d hw=%d", n, c, hw);
  KFAC_REQUIRE((long long)n * c < 0x7fffffffLL, "too many (sample, channel) slabs");
  KFAC_REQUIRE(x && gy, "null pointer");
  if (stats == nullptr || stats_bytes < kfac_bn_workspace_bytes(n, c))
    return kfac::fail(KFAC_ENOMEM, "batch-norm statistics buffer too small: %zu < %zu bytes", stats_bytes,
                      kfac_bn_workspace_bytes(n, c));
  hipStream_t s = kfac::as_stream(stream);
  const int nslab = n * c;
  kfac::TimedLaunch timed(KFAC_TIMED_BN, s);
  launch_stats(x, gy, nslab, hw, stats, stats + nslab, stats + 2 * (size_t)nslab, stats + 3 * (size_t)nslab, s);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

struct kfac_bn_finish_batch {
  std::vector<BnFinishItem> items;
  std::vector<int2> units;
  kfac::DevTableRing item_table;
  kfac::DevTable unit_table;
};

extern "C" int kfac_bn_finish_batch_create(kfac_bn_finish_batch_t *batch_out) {
  KFAC_REQUIRE(batch_out != nullptr, "batch_out is null");
  *batch_out = new (std::nothrow) kfac_bn_finish_batch;
  return *batch_out ? KFAC_OK : kfac::fail(KFAC_ENOMEM, "out of host memory");
}

extern "C" int kfac_bn_finish_batch_destroy(kfac_bn_finish_batch_t batch) {
  delete batch;
  return KFAC_OK;
}

extern "C" int kfac_bn_finish_batched_f32(kfac_bn_finish_batch_t batch, int count, const float *const *stats,
                                          float *const *U, const int32_t *n, const int32_t *c,
                                          const int32_t *hw, const float *eps, const float *gy_scale,
                                          const int32_t *has_gamma, const int32_t *has_beta, void *stream) {
  KFAC_REQUIRE(batch != nullptr, "batch is null");
  KFAC_REQUIRE(count >= 0, "count < 0");
  if (count == 0) return KFAC_OK;
  KFAC_REQUIRE(stats && U && n && c && hw && eps && gy_scale && has_gamma && has_beta, "null table");
  batch->items.resize(count);
  batch->units.clear();
  for (int i = 0; i < count; ++i) {
    KFAC_REQUIRE(n[i] > 0 && c[i] > 0 && hw[i] > 0, "layer %d: bad shape n=%d c=%d hw=%d", i, n[i], c[i], hw[i]);
    KFAC_REQUIRE((long long)n[i] * c[i] < 0x7fffffffLL, "layer %d: too many (sample, channel) slabs", i);
    KFAC_REQUIRE(has_gamma[i] || has_beta[i], "layer %d: gamma and beta are both absent", i);
    KFAC_REQUIRE(stats[i] && U[i], "layer %d: null pointer", i);
    batch->items[i] = BnFinishItem{stats[i], U[i],           n[i],         c[i], hw[i], has_gamma[i] ? 1 : 0,
                                   has_beta[i] ? 1 : 0, eps[i], gy_scale[i]};
    for (int b = 0; b < kfac::ceil_div(c[i], 64); ++b) batch->units.push_back(make_int2(i, b));
  }
  hipStream_t s = kfac::as_stream(stream);
  const void *d_items = nullptr;
  if (int rc = batch->item_table.set(batch->items.data(), sizeof(BnFinishItem) * (size_t)count, s, &d_items))
    return rc;
  if (int rc = batch->unit_table.set(batch->units.data(), sizeof(int2) * batch->units.size(), s)) return rc;
  kfac::TimedLaunch timed(KFAC_TIMED_BN, s);
  KFAC_LAUNCH(bn_finish_batched_kernel, dim3((unsigned)batch->units.size()), dim3(256), 0, s,
                     static_cast<const BnFinishItem *>(d_items), batch->unit_table.as<const int2>());
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}
