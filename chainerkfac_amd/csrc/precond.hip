// Gradient preconditioning  kf = (G^-1 . [dW | db]) . A^-1  as two FP32 MFMA
// GEMMs, and the batch-norm block's  kf = F^-1 . [dgamma ; dbeta]  as a GEMV
// with the NaN fallback.  The [dW | db] concatenation is folded into the
// operand loader of the first product and the kfgrad split into the epilogue
// of the second, so no concatenated or sliced copy is made.
// Replaces compute_kfgrads / update_kfgrads of
// chainerkfac/optimizers/fisher_blocks/connections/{linear,convolution_2d}.py,
// fisher_blocks/connection.py:51-61 and normalizations/batch_normalization.py:159-191.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "common.h"
#include "mma_core.h"

namespace {

using namespace kfac::mma;

// D[i][j] = sum_k Aop(i,k) Bop(j,k), i < M, j < N, over this workgroup's slice
// of k.  Without split-K (partial == nullptr) column j < n_main goes to
// C0[i*ld0 + j] and column n_main (if any) to C1[i]; with split-K the raw tile
// goes to the workspace and gemm_finish_kernel adds the slices up.
template <int W, class LA, class LB>
__global__ __launch_bounds__(THREADS, 2) void gemm_kernel(LA la_in, LB lb_in, int M, int N, int K,
                                                          long long klen, int tiles_n, int ntiles,
                                                          float *__restrict__ partial,
                                                          float *__restrict__ C0, long long ld0,
                                                          int n_main, float *__restrict__ C1) {
  constexpr int BM = 64 * W;
  __shared__ float ldsA[Panel<BM>::kFloats];
  __shared__ float ldsB[Panel<BM>::kFloats];
  // Workgroup i of a launch runs on XCD i % 8 (each XCD has its own L2): every XCD gets a
  // contiguous run of the work list, which walks the tile rows of one tile column and
  // k-slice first, so that the workgroups that read the same B panels share an L2.
  const int total = (int)gridDim.x;
  const int xcd = blockIdx.x % 8, idx = blockIdx.x / 8;
  const int base = total / 8, rem = total % 8;
  const int w = xcd * base + (xcd < rem ? xcd : rem) + idx;
  const int tiles_m = ntiles / tiles_n;
  const int split = w / ntiles;
  const int q = w - split * ntiles;
  const int tj = q / tiles_m, ti = q - tj * tiles_m;
  const int tile = ti * tiles_n + tj;
  LA la = la_in;
  LB lb = lb_in;
  la.init(nullptr, ti * BM);
  lb.init(nullptr, tj * BM);
  const long long kbeg = (long long)split * klen;
  long long kend = kbeg + klen;
  if (kend > K) kend = K;
  floatx16 acc[W][W];
  zero_acc<W, W>(acc);
  mainloop<W, W, false>(la, lb, ti * BM, tj * BM, kbeg, kend, ldsA, ldsB, acc);
  if (partial) {
    float *out = partial + ((long long)split * ntiles + tile) * (BM * BM);
    for_each_acc<W, W>(acc, [&](int r, int c, float v) { out[r * BM + c] = v; });
  } else {
    for_each_acc<W, W>(acc, [&](int r, int c, float v) {
      const int i = ti * BM + r, j = tj * BM + c;
      if (i < M && j < N) {
        if (j < n_main)
          C0[(long long)i * ld0 + j] = v;
        else
          C1[i] = v;
      }
    });
  }
}

__global__ __launch_bounds__(256) void gemm_finish_kernel(const float *__restrict__ partial,
                                                          int nsplit, int ntiles, int tiles_n,
                                                          int bm, int M, int N,
                                                          float *__restrict__ C0, long long ld0,
                                                          int n_main, float *__restrict__ C1) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)M * N) return;
  const int i = (int)(idx / N), j = (int)(idx - (long long)i * N);
  const int tile = (i / bm) * tiles_n + j / bm;
  const float *p = partial + (long long)tile * bm * bm + (i % bm) * bm + (j % bm);
  const long long stride = (long long)ntiles * bm * bm;
  float sum = 0.f;
  for (int s = 0; s < nsplit; ++s) sum += p[s * stride];
  if (j < n_main)
    C0[(long long)i * ld0 + j] = sum;
  else
    C1[i] = sum;
}

struct GemmPlan {
  int w;        // 1: 64x64 tiles, 2: 128x128 tiles
  int tm, tn;
  int nsplit;
  long long klen;
  size_t partial_floats() const {
    return nsplit > 1 ? (size_t)nsplit * tm * tn * (64 * w) * (64 * w) : 0;
  }
};

// 128x128 tiles with enough k-slices to put ~1000 workgroups in flight; 64x64
// tiles when even that leaves most CUs idle (small products).
GemmPlan plan_gemm(int M, int N, int K) {
  const long long nk = kfac::ceil_div(K, KT);
  auto splits = [&](long long tiles) {
    long long ns = kfac::ceil_div<long long>(1024, tiles);
    const long long max_ns = nk >= 6 ? nk / 6 : 1;
    if (ns > max_ns) ns = max_ns;
    return ns < 1 ? 1 : ns;
  };
  GemmPlan p;
  p.w = 2;
  p.tm = kfac::ceil_div(M, 128);
  p.tn = kfac::ceil_div(N, 128);
  long long ns = splits((long long)p.tm * p.tn);
  if ((long long)p.tm * p.tn * ns < 256) {
    p.w = 1;
    p.tm = kfac::ceil_div(M, 64);
    p.tn = kfac::ceil_div(N, 64);
    ns = splits((long long)p.tm * p.tn);
  }
  const long long per = kfac::ceil_div(nk, ns);
  p.nsplit = (int)kfac::ceil_div(nk, per);
  p.klen = per * KT;
  return p;
}

// 16-byte loads need rows that start on 16-byte boundaries (the reduction length
// is free: the loader takes a quad cut by the end of the range element by element)
bool kc_aligned(const float *base, long long ld) {
  return (ld % 4 == 0) && (reinterpret_cast<uintptr_t>(base) % 16 == 0);
}

bool ks_aligned(const float *base, long long ld) {
  return (ld % 4 == 0) && (reinterpret_cast<uintptr_t>(base) % 16 == 0);
}

template <int ROWS, bool VEC>
LoaderKC<ROWS, VEC> rowmajor_kc(const float *base, int rows, int K, long long ld) {
  LoaderKC<ROWS, VEC> l;
  l.base = base;
  l.sample_stride = 0;
  l.row_stride = (unsigned)ld;
  l.L = (unsigned)K;
  l.rows_valid = rows;
  return l;
}

template <int ROWS, bool VEC>
LoaderKS<ROWS, VEC> colop_ks(const float *base, long long ld, int rows_valid, const float *extra) {
  LoaderKS<ROWS, VEC> l;
  l.base = base;
  l.extra = extra;
  l.ld = (unsigned)ld;
  l.rows_valid = rows_valid;
  l.has_extra = extra != nullptr;
  return l;
}

// Row `row` of y = F g with g = [g0 ; g1], by one wave (the result is valid in lane 0).
__device__ __forceinline__ float gemv_row(const float *__restrict__ F, int d, int row,
                                          const float *__restrict__ g0, int n0,
                                          const float *__restrict__ g1) {
  const int lane = threadIdx.x & 63;
  const float *fr = F + (long long)row * d;
  float acc = 0.f;
  const bool vec = ((d | n0) & 3) == 0 &&
                   ((reinterpret_cast<uintptr_t>(F) | reinterpret_cast<uintptr_t>(g0) |
                     reinterpret_cast<uintptr_t>(g1)) & 15) == 0;
  if (vec) {
    // float4 loads, four independent partial sums per lane
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    const float4 *f4 = reinterpret_cast<const float4 *>(fr);
    const float4 *g04 = reinterpret_cast<const float4 *>(g0);
    const float4 *g14 = reinterpret_cast<const float4 *>(g1);
    const int q0 = n0 / 4, q = d / 4;
#pragma unroll 4
    for (int j = lane; j < q; j += 64) {
      const float4 f = f4[j];
      const float4 g = j < q0 ? g04[j] : g14[j - q0];
      a0 += f.x * g.x;
      a1 += f.y * g.y;
      a2 += f.z * g.z;
      a3 += f.w * g.w;
    }
    acc = (a0 + a1) + (a2 + a3);
  } else {
    for (int j = lane; j < d; j += 64) acc += fr[j] * (j < n0 ? g0[j] : g1[j - n0]);
  }
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o, 64);
  return acc;
}

// y = F g with g = [g0 ; g1]; one wave per row.
__global__ __launch_bounds__(256) void gemv_kernel(const float *__restrict__ F, int d,
                                                   const float *__restrict__ g0, int n0,
                                                   const float *__restrict__ g1,
                                                   float *__restrict__ y) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= d) return;
  const float acc = gemv_row(F, d, row, g0, n0, g1);
  if ((threadIdx.x & 63) == 0) y[row] = acc;
}

// One workgroup: if any y is NaN the outputs are the raw gradients.
__device__ __forceinline__ void bn_select(const float *__restrict__ y, int d,
                                          const float *__restrict__ g0, int n0,
                                          const float *__restrict__ g1, float *__restrict__ k0,
                                          float *__restrict__ k1, int *__restrict__ flag) {
  __shared__ int any;
  if (threadIdx.x == 0) any = 0;
  __syncthreads();
  int mine = 0;
  for (int i = threadIdx.x; i < d; i += 1024) mine |= (y[i] != y[i]);
  if (mine) any = 1;
  __syncthreads();
  const int bad = any;
  for (int i = threadIdx.x; i < d; i += 1024) {
    if (i < n0)
      k0[i] = bad ? g0[i] : y[i];
    else
      k1[i - n0] = bad ? g1[i - n0] : y[i];
  }
  if (flag && threadIdx.x == 0) *flag = bad;
}

__global__ __launch_bounds__(1024) void bn_select_kernel(const float *__restrict__ y, int d,
                                                         const float *__restrict__ g0, int n0,
                                                         const float *__restrict__ g1,
                                                         float *__restrict__ k0,
                                                         float *__restrict__ k1,
                                                         int *__restrict__ flag) {
  bn_select(y, d, g0, n0, g1, k0, k1, flag);
}

// The same two kernels over a list of batch-norm blocks: a unit is four rows of
// one block's product (one wave per row, the single-block kernel's arithmetic),
// the selection takes one workgroup per block.
struct BnPreItem {
  const float *F, *g0, *g1;
  float *k0, *k1;
  int *flag;
  long long y_off;   // floats from the workspace base
  int d, n0;
};

__global__ __launch_bounds__(256) void gemv_batched_kernel(const BnPreItem *__restrict__ items,
                                                           const int2 *__restrict__ units,
                                                           float *__restrict__ ws) {
  const int2 u = units[blockIdx.x];   // (item, first row)
  const BnPreItem it = items[u.x];
  const int row = u.y + (threadIdx.x >> 6);
  if (row >= it.d) return;
  const float acc = gemv_row(it.F, it.d, row, it.g0, it.n0, it.g1);
  if ((threadIdx.x & 63) == 0) ws[it.y_off + row] = acc;
}

__global__ __launch_bounds__(1024) void bn_select_batched_kernel(const BnPreItem *__restrict__ items,
                                                                 const float *__restrict__ ws) {
  const BnPreItem it = items[blockIdx.x];
  bn_select(ws + it.y_off, it.d, it.g0, it.n0, it.g1, it.k0, it.k1, it.flag);
}

template <class LA64, class LB64, class LA128, class LB128>
int launch_gemm(const LA64 &a64, const LB64 &b64, const LA128 &a128, const LB128 &b128, int M,
                int N, int K, float *partial, float *C0, long long ld0, int n_main, float *C1,
                hipStream_t stream) {
  const GemmPlan p = plan_gemm(M, N, K);
  const int ntiles = p.tm * p.tn;
  float *part = p.nsplit > 1 ? partial : nullptr;
  {
    kfac::TimedLaunch timed(KFAC_TIMED_GEMM, stream);
    if (p.w == 2)
      KFAC_LAUNCH((gemm_kernel<2, LA128, LB128>), dim3(ntiles * p.nsplit), dim3(THREADS), 0,
                         stream, a128, b128, M, N, K, p.klen, p.tn, ntiles, part, C0, ld0, n_main,
                         C1);
    else
      KFAC_LAUNCH((gemm_kernel<1, LA64, LB64>), dim3(ntiles * p.nsplit), dim3(THREADS), 0,
                         stream, a64, b64, M, N, K, p.klen, p.tn, ntiles, part, C0, ld0, n_main, C1);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  if (part) {
    const long long total = (long long)M * N;
    kfac::TimedLaunch timed(KFAC_TIMED_GEMM_AUX, stream);
    KFAC_LAUNCH(gemm_finish_kernel, dim3((unsigned)kfac::ceil_div<long long>(total, 256)),
                       dim3(256), 0, stream, part, p.nsplit, ntiles, p.tn, 64 * p.w, M, N, C0, ld0,
                       n_main, C1);
    KFAC_HIP_CHECK(hipGetLastError());
  }
  return KFAC_OK;
}

size_t align_floats(size_t n) { return (n + 63) & ~(size_t)63; }

}  // namespace

// Leading dimension of the intermediate product T = Ginv . grad: rows start on
// 16-byte boundaries whatever dA is, so that the second product reads T with
// 16-byte loads.
int padded_ld(int dA) { return (dA + 3) & ~3; }

extern "C" size_t kfac_precond_conn_workspace_bytes(int dG, int dA) {
  if (dG <= 0 || dA <= 0) return 0;
  const size_t p1 = plan_gemm(dG, dA, dG).partial_floats();
  const size_t p2 = plan_gemm(dG, dA, dA).partial_floats();
  return (align_floats((size_t)dG * padded_ld(dA)) + (p1 > p2 ? p1 : p2)) * sizeof(float) + 256;
}

extern "C" int kfac_precond_conn_f32(const float *Ginv, int dG, const float *Ainv, int dA,
                                     const float *gradW, const float *gradb, float *kfW,
                                     float *kfb, void *ws, size_t ws_bytes, void *stream) {
  KFAC_REQUIRE(dG > 0 && dA > 0, "bad dimensions dG=%d dA=%d", dG, dA);
  KFAC_REQUIRE(Ginv && Ainv && gradW && kfW, "null pointer");
  KFAC_REQUIRE((gradb == nullptr) == (kfb == nullptr), "gradb and kfb must both be given or both null");
  const int hb = gradb ? 1 : 0;
  KFAC_REQUIRE(dA - hb > 0, "dA too small");
  KFAC_REQUIRE((long long)dG * dA < 0x40000000LL && (long long)dA * dA < 0x40000000LL &&
                   (long long)dG * dG < 0x40000000LL,
               "factor too large");
  if (ws == nullptr || ws_bytes < kfac_precond_conn_workspace_bytes(dG, dA))
    return kfac::fail(KFAC_ENOMEM, "preconditioning workspace too small: %zu < %zu bytes",
                      ws_bytes, kfac_precond_conn_workspace_bytes(dG, dA));
  hipStream_t s = kfac::as_stream(stream);
  float *T = reinterpret_cast<float *>((reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255);
  const int dW = dA - hb;
  const int ldT = padded_ld(dA);
  float *partial = T + align_floats((size_t)dG * ldT);
  // T (dG x dA) = Ginv (dG x dG) . [gradW | gradb] (dG x dA); float4 loads when
  // both operands are aligned, scalar loads otherwise
  int rc;
  if (kc_aligned(Ginv, dG) && ks_aligned(gradW, dW))
    rc = launch_gemm(rowmajor_kc<64, true>(Ginv, dG, dG, dG), colop_ks<64, true>(gradW, dW, dW, gradb),
                     rowmajor_kc<128, true>(Ginv, dG, dG, dG),
                     colop_ks<128, true>(gradW, dW, dW, gradb), dG, dA, dG, partial, T, ldT, dA,
                     nullptr, s);
  else
    rc = launch_gemm(rowmajor_kc<64, false>(Ginv, dG, dG, dG),
                     colop_ks<64, false>(gradW, dW, dW, gradb),
                     rowmajor_kc<128, false>(Ginv, dG, dG, dG),
                     colop_ks<128, false>(gradW, dW, dW, gradb), dG, dA, dG, partial, T, ldT, dA,
                     nullptr, s);
  if (rc != KFAC_OK) return rc;
  // kf (dG x dA) = T . Ainv (symmetric: column j of Ainv is its row j); T is read with
  // 16-byte loads, Ainv too when its rows are aligned (dA a multiple of 4)
  if (kc_aligned(Ainv, dA))
    return launch_gemm(rowmajor_kc<64, true>(T, dG, dA, ldT), rowmajor_kc<64, true>(Ainv, dA, dA, dA),
                       rowmajor_kc<128, true>(T, dG, dA, ldT),
                       rowmajor_kc<128, true>(Ainv, dA, dA, dA), dG, dA, dA, partial, kfW, dW, dW,
                       kfb, s);
  return launch_gemm(rowmajor_kc<64, true>(T, dG, dA, ldT), rowmajor_kc<64, false>(Ainv, dA, dA, dA),
                     rowmajor_kc<128, true>(T, dG, dA, ldT),
                     rowmajor_kc<128, false>(Ainv, dA, dA, dA), dG, dA, dA, partial, kfW, dW, dW,
                     kfb, s);
}

// ---------------------------------------------------------------------------
// kfac_precond_bn_static_f32: the batch-norm preconditioning with its staging
// vector (the product F^-1 g before the NaN selection) in a device array that
// is part of the library image, for callers that cannot allocate.
// ---------------------------------------------------------------------------
static __device__ __align__(256) float scratch[KFAC_PRECOND_BN_STATIC_MAX_D];

namespace {

constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
float *scratch_ptr[kMaxDevices];   // device address of `scratch` on each GPU, null until resolved

// Every GPU holds its own copy of `scratch` at its own address; the name of the
// array is only a host-side handle.  Resolved once per device, with that device
// current, and kept.
int scratch_of_current_device(float **out) {
  int dev = -1;
  KFAC_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices)
    return kfac::fail(KFAC_EINVAL, "device index %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void *p = nullptr;
    KFAC_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (p == nullptr) return kfac::fail(KFAC_EHIP, "hipGetSymbolAddress returned a null address");
    scratch_ptr[dev] = static_cast<float *>(p);
  }
  *out = scratch_ptr[dev];
  return KFAC_OK;
}

}  // namespace

extern "C" int kfac_precond_bn_static_f32(const float *Finv, int d, const float *g_gamma,
                                          int n_gamma, const float *g_beta, int n_beta,
                                          float *kf_gamma, float *kf_beta,
                                          int32_t *nan_flag_dev, void *stream) {
  KFAC_REQUIRE(d > 0 && n_gamma >= 0 && n_beta >= 0 && n_gamma + n_beta == d,
               "sizes %d + %d do not match d = %d", n_gamma, n_beta, d);
  if (d > KFAC_PRECOND_BN_STATIC_MAX_D)
    return kfac::fail(KFAC_EINVAL,
                      "d = %d exceeds the built-in scratch array (at most %d); use "
                      "kfac_precond_bn_f32 with a caller workspace",
                      d, KFAC_PRECOND_BN_STATIC_MAX_D);
  KFAC_REQUIRE(Finv != nullptr, "Finv is null");
  KFAC_REQUIRE(n_gamma == 0 || (g_gamma && kf_gamma), "gamma pointers are null");
  KFAC_REQUIRE(n_beta == 0 || (g_beta && kf_beta), "beta pointers are null");
  float *y = nullptr;
  if (int rc = scratch_of_current_device(&y)) return rc;
  hipStream_t s = kfac::as_stream(stream);
  // y[0, d) is written in full by the product before the selection reads it, so
  // nothing of an earlier call's contents is ever seen and nothing needs clearing
  kfac::TimedLaunch timed(KFAC_TIMED_GEMM_AUX, s);
  KFAC_LAUNCH(gemv_kernel, dim3(kfac::ceil_div(d, 4)), dim3(256), 0, s, Finv, d, g_gamma,
                     n_gamma, g_beta, y);
  KFAC_LAUNCH(bn_select_kernel, dim3(1), dim3(1024), 0, s, y, d, g_gamma, n_gamma, g_beta,
                     kf_gamma, kf_beta, nan_flag_dev);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

extern "C" size_t kfac_precond_bn_workspace_bytes(int d) {
  return d > 0 ? (size_t)d * sizeof(float) : 0;
}

extern "C" int kfac_precond_bn_f32(const float *Finv, int d, const float *g_gamma, int n_gamma,
                                   const float *g_beta, int n_beta, float *kf_gamma,
                                   float *kf_beta, int32_t *nan_flag_dev, void *ws,
                                   size_t ws_bytes, void *stream) {
  KFAC_REQUIRE(d > 0 && n_gamma >= 0 && n_beta >= 0 && n_gamma + n_beta == d,
               "sizes %d + %d do not match d = %d", n_gamma, n_beta, d);
  KFAC_REQUIRE(Finv != nullptr, "Finv is null");
  KFAC_REQUIRE(n_gamma == 0 || (g_gamma && kf_gamma), "gamma pointers are null");
  KFAC_REQUIRE(n_beta == 0 || (g_beta && kf_beta), "beta pointers are null");
  if (ws == nullptr || ws_bytes < kfac_precond_bn_workspace_bytes(d))
    return kfac::fail(KFAC_ENOMEM, "batch-norm preconditioning workspace too small");
  hipStream_t s = kfac::as_stream(stream);
  float *y = static_cast<float *>(ws);
  kfac::TimedLaunch timed(KFAC_TIMED_GEMM_AUX, s);
  KFAC_LAUNCH(gemv_kernel, dim3(kfac::ceil_div(d, 4)), dim3(256), 0, s, Finv, d, g_gamma,
                     n_gamma, g_beta, y);
  KFAC_LAUNCH(bn_select_kernel, dim3(1), dim3(1024), 0, s, y, d, g_gamma, n_gamma, g_beta,
                     kf_gamma, kf_beta, nan_flag_dev);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

struct kfac_precond_bn_batch {
  std::vector<BnPreItem> items;
  std::vector<int2> units;
  kfac::DevTableRing item_table;
  kfac::DevTable unit_table;
};

extern "C" int kfac_precond_bn_batch_create(kfac_precond_bn_batch_t *batch_out) {
  KFAC_REQUIRE(batch_out != nullptr, "batch_out is null");
  *batch_out = new (std::nothrow) kfac_precond_bn_batch;
  return *batch_out ? KFAC_OK : kfac::fail(KFAC_ENOMEM, "out of host memory");
}

extern "C" int kfac_precond_bn_batch_destroy(kfac_precond_bn_batch_t batch) {
  delete batch;
  return KFAC_OK;
}

extern "C" size_t kfac_precond_bn_batched_workspace_bytes(int count, const int32_t *dims) {
  size_t floats = 0;
  for (int i = 0; i < count; ++i)
    if (dims && dims[i] > 0) floats += ((size_t)dims[i] + 3) / 4 * 4;
  return floats * sizeof(float);
}

extern "C" int kfac_precond_bn_batched_f32(kfac_precond_bn_batch_t batch, int count,
                                           const float *const *Finv, const int32_t *dims,
                                           const float *const *g_gamma, const int32_t *n_gamma,
                                           const float *const *g_beta, float *const *kf_gamma,
                                           float *const *kf_beta, int32_t *const *nan_flags,
                                           void *ws, size_t ws_bytes, void *stream) {
  KFAC_REQUIRE(batch != nullptr, "batch is null");
  KFAC_REQUIRE(count >= 0, "count < 0");
  if (count == 0) return KFAC_OK;
  KFAC_REQUIRE(Finv && dims && g_gamma && n_gamma && g_beta && kf_gamma && kf_beta, "null table");
  if (ws == nullptr || ws_bytes < kfac_precond_bn_batched_workspace_bytes(count, dims))
    return kfac::fail(KFAC_ENOMEM, "batch-norm preconditioning workspace too small");
  batch->items.resize(count);
  batch->units.clear();
  long long off = 0;
  for (int i = 0; i < count; ++i) {
    const int d = dims[i], n0 = n_gamma[i];
    KFAC_REQUIRE(d > 0 && n0 >= 0 && n0 <= d, "block %d: sizes %d of %d", i, n0, d);
    KFAC_REQUIRE(Finv[i] != nullptr, "block %d: Finv is null", i);
    KFAC_REQUIRE(n0 == 0 || (g_gamma[i] && kf_gamma[i]), "block %d: gamma pointers are null", i);
    KFAC_REQUIRE(n0 == d || (g_beta[i] && kf_beta[i]), "block %d: beta pointers are null", i);
    batch->items[i] = BnPreItem{Finv[i],     g_gamma[i], g_beta[i], kf_gamma[i],
                                kf_beta[i],  nan_flags ? nan_flags[i] : nullptr,
                                off,         d,          n0};
    off += ((long long)d + 3) / 4 * 4;
    for (int r = 0; r < d; r += 4) batch->units.push_back(make_int2(i, r));
  }
  hipStream_t s = kfac::as_stream(stream);
  const void *d_items = nullptr;
  if (int rc = batch->item_table.set(batch->items.data(), sizeof(BnPreItem) * (size_t)count, s, &d_items))
    return rc;
  if (int rc = batch->unit_table.set(batch->units.data(), sizeof(int2) * batch->units.size(), s)) return rc;
  kfac::TimedLaunch timed(KFAC_TIMED_GEMM_AUX, s);
  KFAC_LAUNCH(gemv_batched_kernel, dim3((unsigned)batch->units.size()), dim3(256), 0, s,
                     static_cast<const BnPreItem *>(d_items), batch->unit_table.as<const int2>(),
                     static_cast<float *>(ws));
  KFAC_LAUNCH(bn_select_batched_kernel, dim3(count), dim3(1024), 0, s,
                     static_cast<const BnPreItem *>(d_items), static_cast<const float *>(ws));
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

// ---------------------------------------------------------------------------
// Grouped launch: the preconditioning products of all connection layers of a
// network.  Most layers' products are far too small to fill the GPU (a launch
// each, two to four launches per layer with their split-K finishes): a group
// cuts the first product of every layer into (layer, tile, k-slice) tasks of
// about equal length and runs them from one task table, then the same for the
// second product: a few launches per phase (one per tile size and loader kind)
// for the whole network.
// ---------------------------------------------------------------------------
namespace {

struct PreStatic {
  int dG, dA, dW, hb, ldT, w;     // w: 1 = 64-tiles, 2 = 128-tiles
  int tm, tn;
  int nsplit[2];
  long long klen[2];
  long long t_off, part_off;      // floats from the workspace base: T, partial tiles
};

struct PreDyn {
  const float *Ginv, *Ainv, *gradW, *gradb;
  float *kfW, *kfb;
};

// task = (item, tile-and-slice index in the order (slice, tile column, tile row))
template <int W, int PHASE, bool VA, bool VB>
__global__ __launch_bounds__(THREADS, 2) void gemm_group_kernel(const PreStatic *__restrict__ st,
                                                                const PreDyn *__restrict__ dy,
                                                                const int2 *__restrict__ tasks,
                                                                float *__restrict__ ws) {
  constexpr int BM = 64 * W;
  __shared__ float ldsA[Panel<BM>::kFloats];
  __shared__ float ldsB[Panel<BM>::kFloats];
  const int2 task = tasks[blockIdx.x];
  const PreStatic s = st[task.x];
  const PreDyn v = dy[task.x];
  const int ntiles = s.tm * s.tn;
  const int split = task.y / ntiles;
  const int q = task.y - split * ntiles;
  const int tj = q / s.tm, ti = q - tj * s.tm;
  const int tile = ti * s.tn + tj;
  float *T = ws + s.t_off;
  float *partial = ws + s.part_off;
  const int K = PHASE == 0 ? s.dG : s.dA;
  const long long kbeg = (long long)split * s.klen[PHASE];
  long long kend = kbeg + s.klen[PHASE];
  if (kend > K) kend = K;
  floatx16 acc[W][W];
  zero_acc<W, W>(acc);
  if (PHASE == 0) {
    // T = Ginv . [gradW | gradb]
    LoaderKC<BM, VA> la;
    la.base = v.Ginv;
    la.sample_stride = 0;
    la.row_stride = (unsigned)s.dG;
    la.L = (unsigned)s.dG;
    la.rows_valid = s.dG;
    LoaderKS<BM, VB> lb;
    lb.base = v.gradW;
    lb.extra = v.gradb;
    lb.ld = (unsigned)s.dW;
    lb.rows_valid = s.dW;
    lb.has_extra = s.hb;
    la.init(nullptr, ti * BM);
    lb.init(nullptr, tj * BM);
    mainloop<W, W, false>(la, lb, ti * BM, tj * BM, kbeg, kend, ldsA, ldsB, acc);
  } else {
    // kf = T . Ainv
    LoaderKC<BM, VA> la;
    la.base = T;
    la.sample_stride = 0;
    la.row_stride = (unsigned)s.ldT;
    la.L = (unsigned)s.dA;
    la.rows_valid = s.dG;
    LoaderKC<BM, VB> lb;
    lb.base = v.Ainv;
    lb.sample_stride = 0;
    lb.row_stride = (unsigned)s.dA;
    lb.L = (unsigned)s.dA;
    lb.rows_valid = s.dA;
    la.init(nullptr, ti * BM);
    lb.init(nullptr, tj * BM);
    mainloop<W, W, false>(la, lb, ti * BM, tj * BM, kbeg, kend, ldsA, ldsB, acc);
  }
  if (s.nsplit[PHASE] > 1) {
    float *out = partial + ((long long)split * ntiles + tile) * (BM * BM);
    for_each_acc<W, W>(acc, [&](int r, int c, float val) { out[r * BM + c] = val; });
    return;
  }
  const int M = s.dG, N = s.dA;
  for_each_acc<W, W>(acc, [&](int r, int c, float val) {
    const int i = ti * BM + r, j = tj * BM + c;
    if (i < M && j < N) {
      if (PHASE == 0)
        T[(long long)i * s.ldT + j] = val;
      else if (j < s.dW)
        v.kfW[(long long)i * s.dW + j] = val;
      else
        v.kfb[i] = val;
    }
  });
}

// task = (item, block of 256 output elements): sums the item's k-slices
template <int PHASE>
__global__ __launch_bounds__(256) void gemm_group_finish_kernel(const PreStatic *__restrict__ st,
                                                                const PreDyn *__restrict__ dy,
                                                                const int2 *__restrict__ tasks,
                                                                float *__restrict__ ws) {
  const int2 task = tasks[blockIdx.x];
  const PreStatic s = st[task.x];
  const PreDyn v = dy[task.x];
  const int M = s.dG, N = s.dA;
  const long long idx = (long long)task.y * 256 + threadIdx.x;
  if (idx >= (long long)M * N) return;
  const int i = (int)(idx / N), j = (int)(idx - (long long)i * N);
  const int bm = 64 * s.w;
  const int ntiles = s.tm * s.tn;
  const int tile = (i / bm) * s.tn + j / bm;
  const float *p = ws + s.part_off + (long long)tile * bm * bm + (i % bm) * bm + (j % bm);
  const long long stride = (long long)ntiles * bm * bm;
  // eight slices' loads in flight at a time (the sum stays in slice order)
  float sum = 0.f;
  int k = 0;
  for (; k + 8 <= s.nsplit[PHASE]; k += 8) {
    float x[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) x[q] = p[(k + q) * stride];
#pragma unroll
    for (int q = 0; q < 8; ++q) sum += x[q];
  }
  for (; k < s.nsplit[PHASE]; ++k) sum += p[k * stride];
  if (PHASE == 0)
    (ws + s.t_off)[(long long)i * s.ldT + j] = sum;
  else if (j < s.dW)
    v.kfW[(long long)i * s.dW + j] = sum;
  else
    v.kfb[i] = sum;
}

void deal_tasks_to_xcds(std::vector<int2> &table, const std::vector<int2> &natural) {
  const size_t n = natural.size();
  const size_t chunk = (n + 7) / 8;
  for (size_t p = 0; p < chunk; ++p)
    for (size_t x = 0; x < 8; ++x) {
      const size_t i = x * chunk + p;
      if (i < n) table.push_back(natural[i]);
    }
}

// launches of one phase: {64-tiles, 128-tiles} x {both operands with 16-byte loads,
// A only (phase 2: T is always aligned), neither}
constexpr int kPreKinds = 6;

}  // namespace

struct kfac_precond_group {
  int count = 0;
  std::vector<PreStatic> items;
  std::vector<PreDyn> dyn;
  std::vector<int> kind[2];         // per phase, per item
  size_t ws_floats = 0;
  int task0[2][kPreKinds] = {}, ntask[2][kPreKinds] = {};
  int ftask0[2] = {0, 0}, nftask[2] = {0, 0};
  double kind_work[2][kPreKinds] = {};   // matrix work of each launch
  kfac::DevTable d_items, d_tasks;
  kfac::DevTableRing d_dyn;
  // The launches of a phase are independent of each other: the longest stays on the
  // caller's stream, the others run beside it on a stream of the group's own (each
  // launch ends on a partly empty GPU; side by side they fill each other's tails).
  hipStream_t side = nullptr;
  hipEvent_t ev_fork[2] = {nullptr, nullptr}, ev_join[2] = {nullptr, nullptr};
  bool capture_origin = false;   // see kfac_precond_group_set_capture_origin
  ~kfac_precond_group() {
    for (hipEvent_t e : {ev_fork[0], ev_fork[1], ev_join[0], ev_join[1]})
      if (e) (void)hipEventDestroy(e);
    if (side) (void)hipStreamDestroy(side);
  }
};

extern "C" int kfac_precond_group_create(int count, const int32_t *dG, const int32_t *dA,
                                         const int32_t *has_bias, kfac_precond_group_t *out) {
  KFAC_REQUIRE(out != nullptr, "group_out is null");
  *out = nullptr;
  KFAC_REQUIRE(count >= 0 && (count == 0 || (dG && dA && has_bias)), "bad item list");
  auto *g = new (std::nothrow) kfac_precond_group;
  if (!g) return kfac::fail(KFAC_ENOMEM, "out of host memory");
  g->count = count;
  g->items.resize(count);
  g->dyn.resize(count);
  g->kind[0].resize(count);
  g->kind[1].resize(count);
  double work[2][kPreKinds] = {};
  std::vector<long long> nk[2];
  nk[0].resize(count);
  nk[1].resize(count);
  size_t off = 0;
  for (int i = 0; i < count; ++i) {
    PreStatic &s = g->items[i];
    memset(&s, 0, sizeof(s));
    const int hb = has_bias[i] ? 1 : 0;
    if (dG[i] <= 0 || dA[i] - hb <= 0 || (long long)dG[i] * dA[i] >= 0x40000000LL ||
        (long long)dA[i] * dA[i] >= 0x40000000LL || (long long)dG[i] * dG[i] >= 0x40000000LL) {
      delete g;
      return kfac::fail(KFAC_EINVAL, "item %d: bad dimensions dG=%d dA=%d", i, dG[i], dA[i]);
    }
    s.dG = dG[i];
    s.dA = dA[i];
    s.hb = hb;
    s.dW = dA[i] - hb;
    s.ldT = padded_ld(dA[i]);
    // 128-tiles unless they would be mostly padding
    s.w = (s.dG >= 96 && s.dA >= 96) ? 2 : 1;
    const int bm = 64 * s.w;
    s.tm = kfac::ceil_div(s.dG, bm);
    s.tn = kfac::ceil_div(s.dA, bm);
    nk[0][i] = kfac::ceil_div(s.dG, KT);
    nk[1][i] = kfac::ceil_div(s.dA, KT);
    // loader kinds: 16-byte loads need aligned rows (the pointers are checked at run time)
    const bool va0 = s.dG % 4 == 0, vb0 = s.dW % 4 == 0;
    g->kind[0][i] = (s.w == 1 ? 0 : 3) + ((va0 && vb0) ? 0 : 2);
    g->kind[1][i] = (s.w == 1 ? 0 : 3) + (s.dA % 4 == 0 ? 0 : 1);
    for (int p = 0; p < 2; ++p)
      work[p][g->kind[p][i]] += (double)s.tm * s.tn * (double)nk[p][i] * (s.w == 1 ? 1.0 : 4.0);
    s.t_off = (long long)off;
    off += align_floats((size_t)s.dG * s.ldT);
  }
  std::vector<int2> natural[2][kPreKinds], fin[2];
  for (int p = 0; p < 2; ++p) {
    double per_wg[kPreKinds];
    for (int k = 0; k < kPreKinds; ++k) {
      // ~4096 workgroups per launch: five rounds of 3 x 256.  Measured on ResNet-50 (kernel
      // time of the six launches / whole phase with its finish launches): 2304 tasks 1.89 /
      // 2.04 ms, 3072 1.69 / 1.95, 4608 1.61 / 1.97, 6144 1.60 / 2.02, 9216 1.61 / 2.11: shorter
      // tasks shorten the tail of a launch, more k-slices lengthen the finish.
      // Option precond_tasks is a tuning override.
      const double ntasks = std::max(1.0, kfac::option_value(kfac::kOptPrecondTasks, 4096.0));
      per_wg[k] = work[p][k] / ntasks;
      if (per_wg[k] < 32.0) per_wg[k] = 32.0;
      {   // tuning override
        const double val = kfac::option_value(kfac::kOptGroupPanels, 0.0);
        if (val >= 1.0) per_wg[k] = val;
      }
    }
    for (int i = 0; i < count; ++i) {
      PreStatic &s = g->items[i];
      long long ns = (long long)((double)nk[p][i] * (s.w == 1 ? 1.0 : 4.0) / per_wg[g->kind[p][i]] + 0.5);
      if (ns < 1) ns = 1;
      if (ns > 64) ns = 64;
      if (ns > nk[p][i]) ns = nk[p][i];
      const long long per = kfac::ceil_div(nk[p][i], ns);
      s.nsplit[p] = (int)kfac::ceil_div(nk[p][i], per);
      s.klen[p] = per * KT;
      const int ntiles = s.tm * s.tn;
      for (int w = 0; w < ntiles * s.nsplit[p]; ++w) natural[p][g->kind[p][i]].push_back(make_int2(i, w));
      if (s.nsplit[p] > 1) {
        const long long blocks = kfac::ceil_div<long long>((long long)s.dG * s.dA, 256);
        for (long long b = 0; b < blocks; ++b) fin[p].push_back(make_int2(i, (int)b));
      }
    }
  }
  for (int p = 0; p < 2; ++p)
    for (int k = 0; k < kPreKinds; ++k) g->kind_work[p][k] = work[p][k];
  // partial tiles: one area per item, shared by the two phases
  for (int i = 0; i < count; ++i) {
    PreStatic &s = g->items[i];
    const int bm = 64 * s.w;
    const int ns = std::max(s.nsplit[0], s.nsplit[1]);
    s.part_off = (long long)off;
    if (ns > 1) off += (size_t)ns * s.tm * s.tn * bm * bm;
  }
  g->ws_floats = off;
  std::vector<int2> tasks;
  for (int p = 0; p < 2; ++p)
    for (int k = 0; k < kPreKinds; ++k) {
      g->task0[p][k] = (int)tasks.size();
      g->ntask[p][k] = (int)natural[p][k].size();
      deal_tasks_to_xcds(tasks, natural[p][k]);
    }
  for (int p = 0; p < 2; ++p) {
    g->ftask0[p] = (int)tasks.size();
    g->nftask[p] = (int)fin[p].size();
    tasks.insert(tasks.end(), fin[p].begin(), fin[p].end());
  }
  if (tasks.empty()) tasks.push_back(make_int2(0, 0));
  int rc = g->d_items.set_sync(g->items.data(), sizeof(PreStatic) * (size_t)count);
  if (rc == KFAC_OK) rc = g->d_tasks.set_sync(tasks.data(), sizeof(int2) * tasks.size());
  if (rc != KFAC_OK) {
    delete g;
    return rc;
  }
  *out = g;
  return KFAC_OK;
}

extern "C" size_t kfac_precond_group_workspace_bytes(kfac_precond_group_t group) {
  return group ? group->ws_floats * sizeof(float) + 256 : 0;
}

extern "C" int kfac_precond_group_destroy(kfac_precond_group_t group) {
  delete group;
  return KFAC_OK;
}

extern "C" int kfac_precond_group_set_capture_origin(kfac_precond_group_t group, int is_origin) {
  KFAC_REQUIRE(group != nullptr, "group is null");
  group->capture_origin = is_origin != 0;
  return KFAC_OK;
}

extern "C" int kfac_precond_group_run_f32(kfac_precond_group_t group, const float *const *Ginv,
                                          const float *const *Ainv, const float *const *gradW,
                                          const float *const *gradb, float *const *kfW,
                                          float *const *kfb, void *ws, size_t ws_bytes,
                                          void *stream) {
  KFAC_REQUIRE(group != nullptr, "group is null");
  const int count = group->count;
  if (count == 0) return KFAC_OK;
  KFAC_REQUIRE(Ginv && Ainv && gradW && gradb && kfW && kfb, "null table");
  if (ws == nullptr || ws_bytes < kfac_precond_group_workspace_bytes(group))
    return kfac::fail(KFAC_ENOMEM, "preconditioning group workspace too small: %zu < %zu bytes",
                      ws_bytes, kfac_precond_group_workspace_bytes(group));
  auto aligned16 = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  for (int i = 0; i < count; ++i) {
    const PreStatic &s = group->items[i];
    KFAC_REQUIRE(Ginv[i] && Ainv[i] && gradW[i] && kfW[i], "item %d: null pointer", i);
    KFAC_REQUIRE((s.hb != 0) == (gradb[i] != nullptr) && (s.hb != 0) == (kfb[i] != nullptr),
                 "item %d: bias pointers do not match the group's description", i);
    // plans assume what torch allocations give; a misaligned view must use the single call
    KFAC_REQUIRE(aligned16(Ginv[i]) && aligned16(Ainv[i]) && aligned16(gradW[i]),
                 "item %d: factor and gradient pointers must be 16-byte aligned", i);
    group->dyn[i] = PreDyn{Ginv[i], Ainv[i], gradW[i], gradb[i], kfW[i], kfb[i]};
  }
  hipStream_t s = kfac::as_stream(stream);
  const void *dyn_dev = nullptr;
  if (int rc = group->d_dyn.set(group->dyn.data(), sizeof(PreDyn) * (size_t)count, s, &dyn_dev)) return rc;
  float *base = reinterpret_cast<float *>((reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255);
  const PreStatic *st = group->d_items.as<const PreStatic>();
  const PreDyn *dy = static_cast<const PreDyn *>(dyn_dev);
  const int2 *tasks = group->d_tasks.as<const int2>();
  using Kern = void (*)(const PreStatic *, const PreDyn *, const int2 *, float *);
  static const Kern kerns[2][kPreKinds] = {
      {gemm_group_kernel<1, 0, true, true>, nullptr, gemm_group_kernel<1, 0, false, false>,
       gemm_group_kernel<2, 0, true, true>, nullptr, gemm_group_kernel<2, 0, false, false>},
      {gemm_group_kernel<1, 1, true, true>, gemm_group_kernel<1, 1, true, false>, nullptr,
       gemm_group_kernel<2, 1, true, true>, gemm_group_kernel<2, 1, true, false>, nullptr}};
  // side stream: not while launches are timed one by one, not in host-only mode, and under
  // stream capture only from the stream the capture began on (the caller says so)
  bool may_fork = kfac::option_int(kfac::kOptGroupSideStream, 1) != 0 && !kfac::timing_on() && !kfac::host_only();
  if (may_fork && !group->capture_origin) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cs) != hipSuccess) {
      (void)hipGetLastError();
      may_fork = false;
    } else if (cs != hipStreamCaptureStatusNone) {
      may_fork = false;
    }
  }
  for (int p = 0; p < 2; ++p) {
    int nlaunch = 0, longest = -1;
    for (int k = 0; k < kPreKinds; ++k) {
      if (group->ntask[p][k] == 0) continue;
      if (!kerns[p][k]) return kfac::fail(KFAC_EINVAL, "internal: no kernel for kind %d", k);
      ++nlaunch;
      if (longest < 0 || group->kind_work[p][k] > group->kind_work[p][longest]) longest = k;
    }
    const bool fork = may_fork && nlaunch >= 2;
    if (fork) {
      if (!group->side) KFAC_HIP_CHECK(hipStreamCreateWithFlags(&group->side, hipStreamNonBlocking));
      if (!group->ev_fork[p]) {
        KFAC_HIP_CHECK(hipEventCreateWithFlags(&group->ev_fork[p], hipEventDisableTiming));
        KFAC_HIP_CHECK(hipEventCreateWithFlags(&group->ev_join[p], hipEventDisableTiming));
      }
      KFAC_HIP_CHECK(hipEventRecord(group->ev_fork[p], s));
      KFAC_HIP_CHECK(hipStreamWaitEvent(group->side, group->ev_fork[p], 0));
    }
    // (the longest first: its workgroups are placed before the others fill in)
    for (int pass = 0; pass < 2; ++pass)
      for (int k = 0; k < kPreKinds; ++k) {
        if (group->ntask[p][k] == 0 || (pass == 0) != (k == longest)) continue;
        hipStream_t st_k = fork && k != longest ? group->side : s;
        kfac::TimedLaunch timed(KFAC_TIMED_GEMM, st_k);
        KFAC_LAUNCH(kerns[p][k], dim3(group->ntask[p][k]), dim3(THREADS), 0, st_k, st, dy,
                    tasks + group->task0[p][k], base);
      }
    KFAC_HIP_CHECK(hipGetLastError());
    if (fork) {
      KFAC_HIP_CHECK(hipEventRecord(group->ev_join[p], group->side));
      KFAC_HIP_CHECK(hipStreamWaitEvent(s, group->ev_join[p], 0));
    }
    if (group->nftask[p] > 0) {
      kfac::TimedLaunch timed(KFAC_TIMED_GEMM_AUX, s);
      if (p == 0)
        KFAC_LAUNCH(gemm_group_finish_kernel<0>, dim3(group->nftask[p]), dim3(256), 0, s, st, dy,
                           tasks + group->ftask0[p], base);
      else
        KFAC_LAUNCH(gemm_group_finish_kernel<1>, dim3(group->nftask[p]), dim3(256), 0, s, st, dy,
                           tasks + group->ftask0[p], base);
      KFAC_HIP_CHECK(hipGetLastError());
    }
  }
  return KFAC_OK;
}
