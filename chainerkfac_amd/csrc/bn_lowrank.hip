// Damped inverse of batch-norm Fisher blocks from their low-rank form.
//
// A batch-norm block's factor is F = U^T U / n with U the (n x w) per-sample
// gradient matrix (n = batch size, w = 2C): rank <= n.  Its damped inverse
//     (F + D)^-1,  D = diag(d_gamma ... d_gamma, d_beta ... d_beta),
// is, by the Woodbury identity with  Uh = U D^-1/2 / sqrt(n)  (n x w),
//     S = I_n + Uh Uh^T  (n x n, SPD),   S = L L^T,
//     V = L^-1 Uh D^-1/2  (n x w),       (F + D)^-1 = D^-1 - V^T V:
// an n x n Cholesky and two thin products instead of a w^3 factorisation
// (w = 4096 for the last stage of ResNet-50; the batch-norm blocks are 43 % of
// that network's dense inversion work).  The result is the same dense
// symmetric matrix the dense path returns, to rounding.
//
// All blocks of a plan go through four launches together:
//   gram    partial n x n Gram matrices of Uh over chunks of 256 columns
//   factor  per block: S = I + sum of its partials (fixed order), Cholesky and
//           L^-1 of the 32 x 32 matrix by one wave (rows >= n are identity)
//   apply   V = L^-1 Uh D^-1/2
//   outer   out = D^-1 - V^T V on 64 x 64 tiles (HBM-bound: writes w^2 floats)
// Everything up to V is float64: S = I + (entries up to lambda_max / damping)
// loses its small eigenvalues to float32 rounding, and the difference
// D^-1 - V^T V cancels; with V exact to float32 rounding the result is as
// accurate as the dense float32 inverse.  The float64 work is O(n^2 w), small.
// Supported for n <= 32; both damping values must be positive.
//
// Replaces, for such blocks, the dense path of update_invs
// (chainerkfac/optimizers/fisher_block.py:165-179 with
// optimizers/cholesky_inverse.py:16-102) applied to the factor of
// normalizations/batch_normalization.py:121-131.
#include <vector>

#include "chol32.h"
#include "common.h"

namespace {

constexpr int NMAX = kfac::kChol32;   // largest batch size
constexpr int CHUNK = 128;            // columns per gram / apply workgroup
constexpr int SLS = NMAX + 1;         // LDS row stride of the n x n matrix
constexpr int TILE = 64;              // output tile of the outer product
typedef float floatx16 __attribute__((ext_vector_type(16)));

struct LrTables {
  const float *const *U;    // [count] (n x w), row-major
  float *const *out;        // [count] (w x w)
  const int *w;             // [count]
  const int *split;         // [count] columns below split take d_gamma
  const float *dg;          // [count]
  const float *db;          // [count]
  const int *chunk_cs;      // [count+1] cumulative chunk counts
  const int *tile_cs;       // [count+1] cumulative tile counts (tiles per side squared)
  const int *tile_owner;    // [tiles] block of every output tile (one load instead of a search)
  const long long *v_off;   // [count] float offset of V in the workspace
  double *part;             // [chunks][NMAX*NMAX]
  double *winv;             // [count][NMAX*NMAX]  U32 = (L^-1)^T
  float *V;                 // concatenated (NMAX x w) matrices
  int *info;
};

__device__ __forceinline__ int find_slot(const int *__restrict__ cs, int n, int idx) {
  int lo = 0, hi = n - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cs[mid] <= idx)
      lo = mid;
    else
      hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float damp_of(const LrTables &tb, int l, int col) {
  return col < tb.split[l] ? tb.dg[l] : tb.db[l];
}

// part[chunk] = Uh[:, chunk] Uh[:, chunk]^T
__global__ __launch_bounds__(256) void lr_gram_kernel(LrTables tb, int count, int n) {
  __shared__ double X[NMAX][CHUNK + 1];
  const int l = find_slot(tb.chunk_cs, count, blockIdx.x);
  const int c0 = (blockIdx.x - tb.chunk_cs[l]) * CHUNK;
  const int w = tb.w[l];
  const float *__restrict__ U = tb.U[l];
  for (int e = threadIdx.x; e < NMAX * CHUNK; e += 256) {
    const int i = e / CHUNK, c = e % CHUNK;
    const int col = c0 + c;
    double v = 0.0;
    if (i < n && col < w) v = (double)U[(long long)i * w + col] / sqrt((double)n * (double)damp_of(tb, l, col));
    X[i][c] = v;
  }
  __syncthreads();
  double *__restrict__ dst = tb.part + (long long)blockIdx.x * (NMAX * NMAX);
#pragma unroll
  for (int q = 0; q < NMAX * NMAX / 256; ++q) {
    const int e = threadIdx.x + 256 * q;
    const int a = e / NMAX, b = e % NMAX;   // a is uniform over 32 lanes, b = lane
    double acc = 0.0;
#pragma unroll 8
    for (int j = 0; j < CHUNK; ++j) acc += X[a][j] * X[b][j];
    dst[e] = acc;
  }
}

// One workgroup per block: S (all waves sum the chunks' partial Gram matrices,
// several loads in flight per thread), its Cholesky factor (wave 0) and
// winv = (L^-1)^T.
constexpr int kFactorThreads = 256;
__global__ __launch_bounds__(kFactorThreads) void lr_factor_kernel(LrTables tb) {
  __shared__ double S[NMAX * SLS];
  const int l = blockIdx.x;
  const int c_lo = tb.chunk_cs[l], c_hi = tb.chunk_cs[l + 1];
#pragma unroll
  for (int q = 0; q < NMAX * NMAX / kFactorThreads; ++q) {
    const int e = threadIdx.x + kFactorThreads * q;
    const int a = e / NMAX, b = e % NMAX;
    const double *__restrict__ src = tb.part + (long long)c_lo * (NMAX * NMAX) + e;
    // in chunk order, whatever the unrolling: the sum does not depend on it
    double acc = a == b ? 1.0 : 0.0;
    int c = c_lo;
    for (; c + 8 <= c_hi; c += 8, src += 8 * NMAX * NMAX) {
      double v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = src[(long long)u * (NMAX * NMAX)];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; c < c_hi; ++c, src += NMAX * NMAX) acc += *src;
    S[a * SLS + b] = acc;
  }
  __syncthreads();
  int bad = 0;
  if (threadIdx.x < 64) bad = kfac::chol_inv_32<SLS>(S, 0);
  __syncthreads();
  if (threadIdx.x == 0) tb.info[l] = bad;
  double *__restrict__ dst = tb.winv + (long long)l * (NMAX * NMAX);
#pragma unroll
  for (int q = 0; q < NMAX * NMAX / kFactorThreads; ++q) {
    const int e = threadIdx.x + kFactorThreads * q;
    const int m = e / NMAX, r = e % NMAX;
    dst[e] = r >= m ? S[m * SLS + r] : 0.0;   // winv[m][r] = (L^-1)[r][m]
  }
}

// V[r][col] = (sum_{i <= r} Linv[r][i] U[i][col]) / (sqrt(n) d_col), one thread per column.
__global__ __launch_bounds__(CHUNK) void lr_apply_kernel(LrTables tb, int count, int n) {
  __shared__ double Wt[NMAX * NMAX];   // Wt[i * NMAX + r] = Linv[r][i]
  const int l = find_slot(tb.chunk_cs, count, blockIdx.x);
  const int col = (blockIdx.x - tb.chunk_cs[l]) * CHUNK + threadIdx.x;
  const int w = tb.w[l];
  for (int e = threadIdx.x; e < NMAX * NMAX; e += CHUNK) Wt[e] = tb.winv[(long long)l * (NMAX * NMAX) + e];
  __syncthreads();
  if (col >= w) return;
  const float *__restrict__ U = tb.U[l];
  double x[NMAX];
#pragma unroll
  for (int i = 0; i < NMAX; ++i) x[i] = i < n ? (double)U[(long long)i * w + col] : 0.0;
  const double s = 1.0 / (sqrt((double)n) * (double)damp_of(tb, l, col));
  float *__restrict__ V = tb.V + tb.v_off[l];
#pragma unroll
  for (int r = 0; r < NMAX; ++r) {
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i <= r; ++i) acc += Wt[i * NMAX + r] * x[i];
    V[(long long)r * w + col] = (float)(acc * s);
  }
}

// out tile = D^-1 - V[:, rows]^T V[:, cols]
__global__ __launch_bounds__(256) void lr_outer_kernel(LrTables tb, int count) {
  __shared__ float Vi[NMAX][TILE + 4];
  __shared__ float Vj[NMAX][TILE + 4];
  const int l = tb.tile_owner[blockIdx.x];
  const int w = tb.w[l];
  const int tiles = (w + TILE - 1) / TILE;
  const int t = blockIdx.x - tb.tile_cs[l];
  const int i0 = (t / tiles) * TILE, j0 = (t % tiles) * TILE;
  const float *__restrict__ V = tb.V + tb.v_off[l];
  for (int e = threadIdx.x; e < NMAX * TILE; e += 256) {
    const int k = e / TILE, c = e % TILE;
    Vi[k][c] = i0 + c < w ? V[(long long)k * w + i0 + c] : 0.f;
    Vj[k][c] = j0 + c < w ? V[(long long)k * w + j0 + c] : 0.f;
  }
  __syncthreads();
  // four waves, one 32 x 32 quadrant each: 16 matrix instructions over the NMAX rows of V.
  // v_mfma_f32_32x32x2_f32 takes A[i][k] and B[k][j] with i, j = lane % 32, k = lane / 32
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 31, lk = lane >> 5;
  floatx16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
  for (int kk = 0; kk < NMAX / 2; ++kk)
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(Vi[2 * kk + lk][wm * 32 + li], Vj[2 * kk + lk][wn * 32 + li], acc,
                                               0, 0, 0);
  // accumulator element v of a lane: row 8 (v / 4) + 4 (lane / 32) + v % 4, column lane % 32
  float *__restrict__ out = tb.out[l];
  const int c = j0 + wn * 32 + li;
  // D^-1 only meets the quadrants on the diagonal (a wave-uniform test): the others are
  // stored as they are, without a division per element
  const float dinv = (i0 + wm * 32 == j0 + wn * 32 && c < w) ? 1.0f / damp_of(tb, l, c) : 0.f;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int r = i0 + wm * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
    if (r < w && c < w) out[(long long)r * w + c] = (r == c ? dinv : 0.f) - acc[v];
  }
}

}  // namespace

struct kfac_bn_lowrank_plan {
  int count = 0;
  int n = 0;
  std::vector<int> w, split;
  int chunks = 0, tiles = 0;
  size_t v_floats = 0;
  std::vector<const void *> u_host, out_host;
  std::vector<float> dg_host, db_host;
  kfac::DevTable d_u, d_out, d_w, d_split, d_dg, d_db, d_chunk, d_tile, d_tile_owner, d_voff;
};

extern "C" int kfac_bn_lowrank_plan_create(int count, int n, const int32_t *widths,
                                           const int32_t *splits,
                                           kfac_bn_lowrank_plan_t *plan_out) {
  KFAC_REQUIRE(plan_out != nullptr, "plan_out is null");
  *plan_out = nullptr;
  KFAC_REQUIRE(count >= 0, "count < 0");
  KFAC_REQUIRE(n >= 1 && n <= NMAX, "batch size %d is outside 1..%d", n, NMAX);
  KFAC_REQUIRE(count == 0 || (widths && splits), "null table");
  for (int i = 0; i < count; ++i)
    KFAC_REQUIRE(widths[i] > 0 && widths[i] <= 46340 && splits[i] >= 0 && splits[i] <= widths[i],
                 "block %d: bad width %d / split %d", i, widths[i], splits[i]);
  auto *p = new (std::nothrow) kfac_bn_lowrank_plan;
  if (!p) return kfac::fail(KFAC_ENOMEM, "out of host memory");
  p->count = count;
  p->n = n;
  p->w.assign(widths, widths + count);
  p->split.assign(splits, splits + count);
  std::vector<int> chunk_cs(count + 1, 0), tile_cs(count + 1, 0);
  std::vector<long long> voff(count, 0);
  long long tiles_total = 0;
  for (int i = 0; i < count; ++i) {
    chunk_cs[i + 1] = chunk_cs[i] + kfac::ceil_div(widths[i], CHUNK);
    const long long t = kfac::ceil_div(widths[i], TILE);
    tiles_total += t * t;
    if (tiles_total > 0x7fffffffLL) {
      delete p;
      return kfac::fail(KFAC_EINVAL, "too many output tiles");
    }
    tile_cs[i + 1] = (int)tiles_total;
    voff[i] = (long long)p->v_floats;
    p->v_floats += (size_t)NMAX * widths[i];
  }
  p->chunks = chunk_cs[count];
  p->tiles = tile_cs[count];
  int rc = KFAC_OK;
  auto up = [&](kfac::DevTable &t, const void *h, size_t b) {
    if (rc == KFAC_OK) rc = t.set_sync(h, b);
  };
  up(p->d_w, p->w.data(), sizeof(int) * count);
  up(p->d_split, p->split.data(), sizeof(int) * count);
  up(p->d_chunk, chunk_cs.data(), sizeof(int) * (count + 1));
  up(p->d_tile, tile_cs.data(), sizeof(int) * (count + 1));
  {
    std::vector<int> owner((size_t)p->tiles);
    for (int i = 0; i < count; ++i) std::fill(owner.begin() + tile_cs[i], owner.begin() + tile_cs[i + 1], i);
    up(p->d_tile_owner, owner.data(), sizeof(int) * owner.size());
  }
  up(p->d_voff, voff.data(), sizeof(long long) * count);
  if (rc != KFAC_OK) {
    delete p;
    return rc;
  }
  *plan_out = p;
  return KFAC_OK;
}

extern "C" size_t kfac_bn_lowrank_workspace_bytes(kfac_bn_lowrank_plan_t plan) {
  if (!plan) return 0;
  const size_t doubles = (size_t)plan->chunks * NMAX * NMAX + (size_t)plan->count * NMAX * NMAX;
  return doubles * sizeof(double) + plan->v_floats * sizeof(float) + 256;
}

extern "C" int kfac_bn_lowrank_plan_destroy(kfac_bn_lowrank_plan_t plan) {
  delete plan;
  return KFAC_OK;
}

extern "C" int kfac_bn_lowrank_inverse_batched_f32(kfac_bn_lowrank_plan_t plan,
                                                   const float *const *U_ptrs,
                                                   float *const *out_ptrs,
                                                   const double *d_gamma, const double *d_beta,
                                                   int32_t *info_dev, void *ws, size_t ws_bytes,
                                                   void *stream) {
  KFAC_REQUIRE(plan != nullptr, "plan is null");
  const int count = plan->count;
  if (count == 0) return KFAC_OK;
  KFAC_REQUIRE(U_ptrs && out_ptrs && d_gamma && d_beta && info_dev, "null table");
  if (ws == nullptr || ws_bytes < kfac_bn_lowrank_workspace_bytes(plan))
    return kfac::fail(KFAC_ENOMEM, "low-rank inverse workspace too small: %zu < %zu bytes",
                      ws_bytes, kfac_bn_lowrank_workspace_bytes(plan));
  plan->u_host.resize(count);
  plan->out_host.resize(count);
  plan->dg_host.resize(count);
  plan->db_host.resize(count);
  for (int i = 0; i < count; ++i) {
    KFAC_REQUIRE(U_ptrs[i] && out_ptrs[i], "block %d: null pointer", i);
    // a half without columns needs no damping value
    const bool need_g = plan->split[i] > 0, need_b = plan->split[i] < plan->w[i];
    KFAC_REQUIRE((!need_g || d_gamma[i] > 0.0) && (!need_b || d_beta[i] > 0.0),
                 "block %d: the damping values must be positive", i);
    plan->u_host[i] = U_ptrs[i];
    plan->out_host[i] = out_ptrs[i];
    plan->dg_host[i] = need_g ? (float)d_gamma[i] : 1.f;
    plan->db_host[i] = need_b ? (float)d_beta[i] : 1.f;
  }
  hipStream_t s = kfac::as_stream(stream);
  int rc = plan->d_u.set(plan->u_host.data(), sizeof(void *) * count, s);
  if (rc == KFAC_OK) rc = plan->d_out.set(plan->out_host.data(), sizeof(void *) * count, s);
  if (rc == KFAC_OK) rc = plan->d_dg.set(plan->dg_host.data(), sizeof(float) * count, s);
  if (rc == KFAC_OK) rc = plan->d_db.set(plan->db_host.data(), sizeof(float) * count, s);
  if (rc != KFAC_OK) return rc;
  LrTables tb;
  tb.U = plan->d_u.as<const float *const>();
  tb.out = plan->d_out.as<float *const>();
  tb.w = plan->d_w.as<const int>();
  tb.split = plan->d_split.as<const int>();
  tb.dg = plan->d_dg.as<const float>();
  tb.db = plan->d_db.as<const float>();
  tb.chunk_cs = plan->d_chunk.as<const int>();
  tb.tile_cs = plan->d_tile.as<const int>();
  tb.tile_owner = plan->d_tile_owner.as<const int>();
  tb.v_off = plan->d_voff.as<const long long>();
  uintptr_t base = (reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255;
  tb.part = reinterpret_cast<double *>(base);
  tb.winv = tb.part + (size_t)plan->chunks * NMAX * NMAX;
  tb.V = reinterpret_cast<float *>(tb.winv + (size_t)count * NMAX * NMAX);
  tb.info = info_dev;
  KFAC_LAUNCH(lr_gram_kernel, dim3(plan->chunks), dim3(256), 0, s, tb, count, plan->n);
  KFAC_LAUNCH(lr_factor_kernel, dim3(count), dim3(kFactorThreads), 0, s, tb);
  KFAC_LAUNCH(lr_apply_kernel, dim3(plan->chunks), dim3(CHUNK), 0, s, tb, count, plan->n);
  KFAC_LAUNCH(lr_outer_kernel, dim3(plan->tiles), dim3(256), 0, s, tb, count);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}
