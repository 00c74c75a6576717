// Kronecker-factor construction:  C = beta*C + alpha * P^T P  for the patch /
// activation / gradient matrix P of one layer, never materialised.
//
// syrk_kernel: each workgroup owns one lower-triangle tile (I >= J) of C and one
// slice of the reduction index (split-K: the reduction runs over samples x
// pixels and is far longer than C is wide for most layers).
//   one slice        the tile is scaled and written straight from registers;
//   more slices      every workgroup stores its raw partial tile; reduce_kernel
//                    (more than 8 slices: folds them to 8 slots in parallel)
//                    and finish_kernel (one workgroup per 64x64 block of C, a
//                    fixed summation order, so deterministic) write C.
// Tiles are written as C[I,J] plus the mirror C[J,I] through an LDS transpose,
// so C is exactly symmetric and every store is a contiguous row segment.
//
// Replaces the im2col + transpose + column_stack + GEMM + scale chain of
// chainerkfac/optimizers/fisher_blocks/connections/{linear,convolution_2d}.py
// and the batch-norm block's grad^T grad.
#include <cstdlib>

#include "common.h"
#include "mma_core.h"

namespace {

using namespace kfac::mma;

struct SyrkPlan {
  int bm;          // tile side: 64 or 128
  int tiles;       // per side
  int ntile;       // lower-triangle tiles
  int nsplit;
  long long klen;  // reduction length per split (multiple of KT)
  int nreduced;    // slots after the pre-reduction (0 = none)
};

constexpr int kFinishSplits = 8;

SyrkPlan plan_syrk(int d, long long rows) {
  SyrkPlan p;
  p.bm = d <= 320 ? 64 : 128;
  p.tiles = kfac::ceil_div(d, p.bm);
  p.ntile = p.tiles * (p.tiles + 1) / 2;
  const long long nk = kfac::ceil_div<long long>(rows > 0 ? rows : 1, KT);
  // Measured on MI355X: a launch runs best with a few thousand workgroups in
  // flight-order (several per CU, refilled as they retire), as long as each
  // keeps at least ~6 panels of work to amortise its prologue and the partial
  // tile it writes.  Sweeps over ResNet-50 shapes are flat between ~700 and
  // ~4000 workgroups; aim for 1536.
  const long long target = 1536;
  long long ns = kfac::ceil_div<long long>(target, p.ntile);
  const long long max_ns = nk >= 6 ? nk / 6 : 1;
  if (ns > max_ns) ns = max_ns;
  if (ns < 1) ns = 1;
  // tuning override: KFAC_SYRK_SPLITS=<n> forces the split count
  if (const char *env = getenv("KFAC_SYRK_SPLITS")) {
    const long long forced = atoll(env);
    if (forced >= 1) ns = forced < nk ? forced : nk;
  }
  const long long per = kfac::ceil_div(nk, ns);
  p.nsplit = (int)kfac::ceil_div(nk, per);
  p.klen = per * KT;
  // partials are pre-reduced to at most kFinishSplits slots before finishing
  p.nreduced = p.nsplit > kFinishSplits ? kFinishSplits : 0;
  return p;
}

size_t syrk_ws_floats(const SyrkPlan &p) {
  return (size_t)(p.nsplit + p.nreduced) * p.ntile * p.bm * p.bm;
}

// Sums groups of splits: out slot g = sum of splits [g*per, (g+1)*per).
__global__ __launch_bounds__(256) void reduce_kernel(const float4 *__restrict__ partial,
                                                     float4 *__restrict__ out, int nsplit,
                                                     int per, long long slot4) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= slot4) return;
  const int g = blockIdx.y;
  int s = g * per;
  const int send = (s + per < nsplit) ? s + per : nsplit;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (; s < send; ++s) {
    const float4 v = partial[(long long)s * slot4 + i];
    acc.x += v.x;
    acc.y += v.y;
    acc.z += v.z;
    acc.w += v.w;
  }
  out[(long long)g * slot4 + i] = acc;
}

__device__ __forceinline__ void tri_decode(int t, int &I, int &J) {
  int r = (int)((sqrtf(8.f * (float)t + 1.f) - 1.f) * 0.5f);
  while (r * (r + 1) / 2 > t) --r;
  while ((r + 1) * (r + 2) / 2 <= t) ++r;
  I = r;
  J = t - r * (r + 1) / 2;
}

// Writes the finished tile: C[I,J] = alpha*acc + beta*C[I,J] and, for I != J,
// the mirror C[J,I], 64x64 quadrant by quadrant through an LDS transpose so
// that every global access is a contiguous row segment.
template <int WM>
__device__ __forceinline__ void write_tile(floatx16 (&acc)[WM][WM], float *lds, int I, int J,
                                           int d, float alpha, float beta,
                                           float *__restrict__ C) {
  constexpr int BM = 64 * WM;
  float(*t)[65] = reinterpret_cast<float(*)[65]>(lds);
  const int lc = threadIdx.x & 63, lr0 = threadIdx.x >> 6;
  for (int q = 0; q < WM * WM; ++q) {
    const int qm = q / WM, qn = q % WM;
    __syncthreads();
    for_each_acc<WM, WM>(acc, [&](int r, int c, float v) {
      if (r / 64 == qm && c / 64 == qn) t[r % 64][c % 64] = v;
    });
    __syncthreads();
    const int r0 = I * BM + qm * 64, c0 = J * BM + qn * 64;
#pragma unroll 4
    for (int p = 0; p < 16; ++p) {
      const int lr = lr0 + 4 * p;
      const int r = r0 + lr, c = c0 + lc;
      float v = alpha * t[lr][lc];
      const bool ok = r < d && c < d;
      if (ok) {
        if (beta != 0.f) v += beta * C[(long long)r * d + c];
        C[(long long)r * d + c] = v;
      }
      if (beta != 0.f && I != J) t[lr][lc] = v;   // mirror gets the same value
    }
    if (I != J) {
      if (beta != 0.f) __syncthreads();
#pragma unroll 4
      for (int p = 0; p < 16; ++p) {
        const int lr = lr0 + 4 * p;
        const int mr = c0 + lr, mc = r0 + lc;   // row of the mirrored quadrant = column here
        if (mr < d && mc < d) C[(long long)mr * d + mc] = (beta != 0.f) ? t[lc][lr] : alpha * t[lc][lr];
      }
    }
  }
}

// With a single k-slice (direct != 0) the tile is scaled and written straight
// from registers; otherwise the raw partial tile goes to the workspace.
template <int WM, class Loader>
__global__ __launch_bounds__(THREADS, 3) void syrk_kernel(Loader ld, long long K,
                                                          long long klen, int ntile, int direct,
                                                          int d, float alpha,
                                                          float beta, float *__restrict__ partial,
                                                          float *__restrict__ C) {
  constexpr int BM = 64 * WM;
  __shared__ float lds[2 * Panel<BM>::kFloats];
  __shared__ int2 tabA[BM];
  __shared__ int2 tabB[BM];
  float *ldsA = lds, *ldsB = lds + Panel<BM>::kFloats;
  static_assert(2 * Panel<BM>::kFloats >= 64 * 65, "LDS too small for the epilogue transpose");
  const int tile = blockIdx.x % ntile;
  const int split = blockIdx.x / ntile;
  int I, J;
  tri_decode(tile, I, J);
  Loader la = ld, lb = ld;
  la.init(reinterpret_cast<float *>(tabA), I * BM);
  lb.init(reinterpret_cast<float *>(tabB), J * BM);
  __syncthreads();
  const long long kbeg = (long long)split * klen;
  long long kend = kbeg + klen;
  if (kend > K) kend = K;
  floatx16 acc[WM][WM];
  zero_acc<WM, WM>(acc);
  if (I == J)
    mainloop<WM, WM, true>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB, acc);
  else
    mainloop<WM, WM, false>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB, acc);
  if (direct) {
    write_tile<WM>(acc, lds, I, J, d, alpha, beta, C);
    return;
  }
  float *out = partial + ((long long)split * ntile + tile) * (BM * BM);
  for_each_acc<WM, WM>(acc, [&](int r, int c, float v) { out[r * BM + c] = v; });
}

// One workgroup per 64x64 sub-block (si >= sj) of C.
__global__ __launch_bounds__(256) void finish_kernel(const float *__restrict__ partial,
                                                     int nsplit, int ntile, int bm, int d,
                                                     float alpha, float beta,
                                                     float *__restrict__ C) {
  __shared__ float tile[64][65];
  int si, sj;
  tri_decode(blockIdx.x, si, sj);
  const int per = bm / 64;  // sub-blocks per tile side
  const int I = si / per, J = sj / per;
  const int t = I * (I + 1) / 2 + J;
  const int r_in = (si - I * per) * 64, c_in = (sj - J * per) * 64;
  const int lc = threadIdx.x & 63, lr0 = threadIdx.x >> 6;
  const long long tile_stride = (long long)bm * bm;
  const float *p0 = partial + (long long)t * tile_stride + (long long)r_in * bm + c_in;
  float sum[16];
#pragma unroll
  for (int p = 0; p < 16; ++p) sum[p] = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float *ps = p0 + (long long)s * ntile * tile_stride;
#pragma unroll
    for (int p = 0; p < 16; ++p) sum[p] += ps[(lr0 + 4 * p) * bm + lc];
  }
#pragma unroll
  for (int p = 0; p < 16; ++p) {
    const int lr = lr0 + 4 * p;
    const int r = si * 64 + lr, c = sj * 64 + lc;
    float v = alpha * sum[p];
    if (beta != 0.f && r < d && c < d) v += beta * C[(long long)r * d + c];
    tile[lr][lc] = v;
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 16; ++p) {
    const int lr = lr0 + 4 * p;
    const int r = si * 64 + lr, c = sj * 64 + lc;
    if (si == sj) {
      if (r < d && c < d) C[(long long)r * d + c] = (lc <= lr) ? tile[lr][lc] : tile[lc][lr];
    } else {
      if (r < d && c < d) C[(long long)r * d + c] = tile[lr][lc];
      const int mr = sj * 64 + lr, mc = si * 64 + lc;
      if (mr < d && mc < d) C[(long long)mr * d + mc] = tile[lc][lr];
    }
  }
}

template <class L64, class L128>
int run_syrk(const L64 &l64, const L128 &l128, int d, long long K, float alpha, float beta,
             float *C, void *ws, size_t ws_bytes, hipStream_t stream) {
  const SyrkPlan p = plan_syrk(d, K);
  const size_t need = syrk_ws_floats(p) * sizeof(float);
  if (ws_bytes < need || ws == nullptr)
    return kfac::fail(KFAC_ENOMEM, "covariance workspace too small: %zu < %zu bytes",
                      ws_bytes, need);
  float *partial = static_cast<float *>(ws);
  const int grid = p.ntile * p.nsplit;
  const int direct = p.nsplit == 1 ? 1 : 0;
  {
    kfac::TimedLaunch timed(KFAC_TIMED_SYRK, stream);
    if (p.bm == 64)
      hipLaunchKernelGGL((syrk_kernel<1, L64>), dim3(grid), dim3(THREADS), 0, stream, l64, K,
                         p.klen, p.ntile, direct, d, alpha, beta, partial, C);
    else
      hipLaunchKernelGGL((syrk_kernel<2, L128>), dim3(grid), dim3(THREADS), 0, stream, l128, K,
                         p.klen, p.ntile, direct, d, alpha, beta, partial, C);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  if (direct) return KFAC_OK;
  const float *fin = partial;
  int nfin = p.nsplit;
  if (p.nreduced) {
    const long long slot4 = (long long)p.ntile * p.bm * p.bm / 4;
    float *red = partial + (size_t)p.nsplit * p.ntile * p.bm * p.bm;
    const int per = kfac::ceil_div(p.nsplit, p.nreduced);
    nfin = kfac::ceil_div(p.nsplit, per);
    hipLaunchKernelGGL(reduce_kernel, dim3((unsigned)kfac::ceil_div<long long>(slot4, 256), nfin),
                       dim3(256), 0, stream, reinterpret_cast<const float4 *>(partial),
                       reinterpret_cast<float4 *>(red), p.nsplit, per, slot4);
    KFAC_HIP_CHECK(hipGetLastError());
    fin = red;
  }
  const int sub = kfac::ceil_div(d, 64);
  hipLaunchKernelGGL(finish_kernel, dim3(sub * (sub + 1) / 2), dim3(256), 0, stream, fin, nfin,
                     p.ntile, p.bm, d, alpha, beta, C);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

template <int ROWS>
LoaderKC<ROWS> make_kc(const float *base, long long sample_stride, long long row_stride, int L,
                       int rows_valid, int ones_row) {
  LoaderKC<ROWS> l;
  l.base = base;
  l.sample_stride = (unsigned)sample_stride;
  l.row_stride = (unsigned)row_stride;
  l.L = (unsigned)L;
  l.rows_valid = rows_valid;
  l.ones_row = ones_row;
  l.vec = (sample_stride % 4 == 0) && (row_stride % 4 == 0) && (L % 4 == 0) &&
          (reinterpret_cast<uintptr_t>(base) % 16 == 0);
  return l;
}

template <int ROWS>
LoaderKS<ROWS> make_ks(const float *base, long long ld, int rows_valid, int has_extra,
                       const float *extra) {
  LoaderKS<ROWS> l;
  l.base = base;
  l.extra = extra;
  l.ld = (unsigned)ld;
  l.rows_valid = rows_valid;
  l.has_extra = has_extra;
  l.vec = (ld % 4 == 0) && (reinterpret_cast<uintptr_t>(base) % 16 == 0);
  return l;
}

template <int ROWS>
LoaderIM<ROWS> make_im(const float *x, int c, int h, int w, int kh, int kw, int sy, int sx,
                       int ph, int pw, int ho, int wo, int append_ones) {
  LoaderIM<ROWS> l;
  l.base = x;
  l.C = c;
  l.H = h;
  l.W = w;
  l.kh = kh;
  l.kw = kw;
  l.sy = sy;
  l.sx = sx;
  l.ph = ph;
  l.pw = pw;
  l.ho = ho;
  l.wo = wo;
  l.d_patch = c * kh * kw;
  l.append_ones = append_ones;
  l.table = nullptr;
  return l;
}

}  // namespace

extern "C" size_t kfac_cov_workspace_bytes(int d, int64_t rows) {
  if (d <= 0) return 0;
  return syrk_ws_floats(plan_syrk(d, rows)) * sizeof(float);
}

extern "C" int kfac_cov_linear_f32(const float *x, int n, int d_in, int append_ones,
                                   float alpha, float beta, float *C, void *ws,
                                   size_t ws_bytes, void *stream) {
  KFAC_REQUIRE(n > 0 && d_in > 0, "bad shape n=%d d_in=%d", n, d_in);
  KFAC_REQUIRE((long long)n * d_in < 0x7fffffffLL, "input too large");
  KFAC_REQUIRE(x && C, "null pointer");
  const int d = d_in + (append_ones ? 1 : 0);
  return run_syrk(make_ks<64>(x, d_in, d_in, append_ones, nullptr),
                  make_ks<128>(x, d_in, d_in, append_ones, nullptr), d, n, alpha, beta, C, ws,
                  ws_bytes, kfac::as_stream(stream));
}

extern "C" int kfac_cov_conv_g_f32(const float *gy, int n, int c, int howo, float alpha,
                                   float beta, float *C, void *ws, size_t ws_bytes,
                                   void *stream) {
  KFAC_REQUIRE(n > 0 && c > 0 && howo > 0, "bad shape n=%d c=%d howo=%d", n, c, howo);
  KFAC_REQUIRE((long long)n * c * howo < 0x7fffffffLL, "input too large");
  KFAC_REQUIRE(gy && C, "null pointer");
  const long long K = (long long)n * howo;
  return run_syrk(make_kc<64>(gy, (long long)c * howo, howo, howo, c, -1),
                  make_kc<128>(gy, (long long)c * howo, howo, howo, c, -1), c, K, alpha, beta,
                  C, ws, ws_bytes, kfac::as_stream(stream));
}

extern "C" int kfac_cov_conv_a_f32(const float *x, int n, int c, int h, int w, int kh, int kw,
                                   int sy, int sx, int ph, int pw, int append_ones,
                                   float alpha, float beta, float *C, void *ws,
                                   size_t ws_bytes, void *stream) {
  KFAC_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0, "bad input shape");
  KFAC_REQUIRE(kh > 0 && kw > 0 && sy > 0 && sx > 0 && ph >= 0 && pw >= 0, "bad geometry");
  KFAC_REQUIRE(kh < 32768 && kw < 65536, "kernel too large");
  KFAC_REQUIRE(h + 2 * ph >= kh && w + 2 * pw >= kw, "kernel larger than padded input");
  KFAC_REQUIRE(x && C, "null pointer");
  const int ho = (h + 2 * ph - kh) / sy + 1;
  const int wo = (w + 2 * pw - kw) / sx + 1;
  const long long dl = (long long)c * kh * kw + (append_ones ? 1 : 0);
  KFAC_REQUIRE(dl < 46340, "factor dimension %lld too large", dl);
  KFAC_REQUIRE((long long)n * c * h * w < 0x7fffffffLL, "input too large");
  const int d = (int)dl;
  const long long K = (long long)n * ho * wo;
  hipStream_t s = kfac::as_stream(stream);
  if (kh == 1 && kw == 1 && sy == 1 && sx == 1 && ph == 0 && pw == 0) {
    // 1x1 convolution: the patch matrix is the NCHW tensor itself
    const int hw = h * w;
    const int ones = append_ones ? c : -1;
    return run_syrk(make_kc<64>(x, (long long)c * hw, hw, hw, c, ones),
                    make_kc<128>(x, (long long)c * hw, hw, hw, c, ones), d, K, alpha, beta, C,
                    ws, ws_bytes, s);
  }
  return run_syrk(make_im<64>(x, c, h, w, kh, kw, sy, sx, ph, pw, ho, wo, append_ones),
                  make_im<128>(x, c, h, w, kh, kw, sy, sx, ph, pw, ho, wo, append_ones), d, K,
                  alpha, beta, C, ws, ws_bytes, s);
}
