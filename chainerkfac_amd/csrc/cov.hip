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
// A bias ("ones") column is kept out of the tile grid: d = 9C + 1 would pay a
// whole extra tile row for it.  Its row of C is the vector of row sums of the
// operand, which the diagonal tiles' workgroups accumulate on the side from the
// operand values they feed to the matrix cores anyway, and its corner entry is
// the reduction length.
//
// Replaces the im2col + transpose + column_stack + GEMM + scale chain of
// chainerkfac/optimizers/fisher_blocks/connections/{linear,convolution_2d}.py
// and the batch-norm block's grad^T grad.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "common.h"
#include "conv_halo.h"
#include "conv_rows.h"
#include "conv_shift.h"
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

// No plan uses more k-slices than this (every planner clamps to it, and the
// workspace bound of kfac_cov_workspace_bytes is computed from it): about
// kMaxWorkgroups workgroups per launch.
constexpr long long kMaxWorkgroups = 3072;
long long max_splits(int ntile) {
  const long long m = kfac::ceil_div<long long>(kMaxWorkgroups, ntile);
  return m < 1 ? 1 : m;
}

SyrkPlan plan_syrk_panels(int d, long long nk, int panel_len) {
  SyrkPlan p;
  int bm64_max = 520;   // measured: 64-tiles win up to d = 512 (more workgroups, 4x smaller partial tiles)
  bm64_max = kfac::option_int(kfac::kOptSyrkBm64Max, bm64_max);   // tuning override
  p.bm = d <= bm64_max ? 64 : 128;
  // A short reduction (batch-norm blocks: K = batch size) is all output traffic:
  // 64-tiles spread the stores over four times as many workgroups.
  if (panel_len == KT && nk <= 4 && kfac::ceil_div(d, 128) <= 32) p.bm = 64;
  p.tiles = kfac::ceil_div(d, p.bm);
  p.ntile = p.tiles * (p.tiles + 1) / 2;
  if (nk < 1) nk = 1;
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
  if (panel_len != KT) {
    // Region kernel (panel = one step of <= 64 pixels): its workgroups are all
    // alike and 2 fit a CU, so a launch runs in rounds of 512 and a round that
    // is nearly empty still costs a full workgroup.  Pick the slice count with
    // the least rounds x (steps per slice + fixed cost), near the target above.
    const long long slots = 512;
    double best = 0;
    long long best_ns = ns;
    for (long long c = 1; c <= max_ns && c <= 4 * ns && c <= max_splits(p.ntile); ++c) {
      const long long per = kfac::ceil_div(nk, c);
      const long long eff = kfac::ceil_div(nk, per);
      const long long rounds = kfac::ceil_div(p.ntile * eff, slots);
      const double cost = (double)rounds * ((double)per + 3.0) + 0.25 * (double)eff;
      if (c == 1 || cost < best) {
        best = cost;
        best_ns = c;
      }
    }
    ns = best_ns;
  }
  // tuning override: option syrk_splits forces the split count
  if (kfac::option_is_set(kfac::kOptSyrkSplits)) {
    const long long forced = (long long)kfac::option_value(kfac::kOptSyrkSplits, 0);
    if (forced >= 1) ns = forced < nk ? forced : nk;
  }
  if (ns > max_splits(p.ntile)) ns = max_splits(p.ntile);
  const long long per = kfac::ceil_div(nk, ns);
  p.nsplit = (int)kfac::ceil_div(nk, per);
  p.klen = per * panel_len;
  // partials are pre-reduced to at most kFinishSplits slots before finishing
  p.nreduced = p.nsplit > kFinishSplits ? kFinishSplits : 0;
  return p;
}

// Plan for the compile-time-geometry convolution kernel: 128-tiles, `steps`
// reduction steps of `step_us` microseconds of matrix-core time each, `occ`
// workgroups resident per CU.  The hardware deals workgroups to the 256 CUs as
// slots free up, so a launch takes about ceil(workgroups / 256) workgroups' time
// on the busiest CU; each workgroup also pays a fixed prologue / epilogue, each
// extra slice a partial tile that is written and read back, and fewer
// workgroups than CUs x occ leave matrix pipes without a second wave to hide
// the staging phases.
SyrkPlan plan_rows(int d, int bm, long long steps, double step_us, int occ) {
  SyrkPlan p;
  p.bm = bm;
  p.tiles = kfac::ceil_div(d, p.bm);
  p.ntile = p.tiles * (p.tiles + 1) / 2;
  if (steps < 1) steps = 1;
  const double fixed_us = 6.0, partial_us = 0.05, finish_us = 8.0;
  long long best_c = 1;
  double best = 0;
  const long long cmax = std::min<long long>(steps, max_splits(p.ntile));
  for (long long c = 1; c <= cmax; ++c) {
    const long long per = kfac::ceil_div(steps, c);
    const long long eff = kfac::ceil_div(steps, per);
    if (eff != c) continue;
    const long long wgs = (long long)p.ntile * eff;
    const long long deep = kfac::ceil_div<long long>(wgs, 256);
    double cost = (double)deep * ((double)per * step_us + fixed_us);
    // measured: a CU with one resident workgroup runs its steps ~25 % slower than one with three
    const double per_cu = std::min((double)occ, (double)wgs / 256.0);
    if (per_cu < 3.0) cost *= 1.0 + 0.14 * (3.0 - per_cu);
    if (eff > 1) cost += finish_us + partial_us * (double)wgs;
    if (c == 1 || cost < best) {
      best = cost;
      best_c = c;
    }
  }
  if (kfac::option_is_set(kfac::kOptSyrkSplits)) {   // tuning override
    const long long forced = (long long)kfac::option_value(kfac::kOptSyrkSplits, 0);
    if (forced >= 1) best_c = std::min(forced, cmax);
  }
  const long long per = kfac::ceil_div(steps, best_c);
  p.nsplit = (int)kfac::ceil_div(steps, per);
  p.klen = per;
  p.nreduced = p.nsplit > kFinishSplits ? kFinishSplits : 0;
  return p;
}

SyrkPlan plan_syrk(int d, long long rows) {
  return plan_syrk_panels(d, kfac::ceil_div<long long>(rows > 0 ? rows : 1, KT), KT);
}

// Floats of one k-slice in the workspace: the partial tiles, then one row-sum
// slot per tile row (used when there is a ones column).
size_t syrk_slot_floats(const SyrkPlan &p) {
  return (size_t)p.ntile * p.bm * p.bm + (size_t)p.tiles * p.bm;
}

size_t syrk_ws_floats(const SyrkPlan &p) {
  return (size_t)(p.nsplit + p.nreduced) * syrk_slot_floats(p);
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
#pragma unroll 4
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

// Ones column of a diagonal tile's rows.  rs[im] holds this lane's half of the
// row sums (see the main loops); after adding the other half, lanes 0..31 of the
// waves with wave_n == 0 own row (wave_m * WM + im) * 32 + lane of the tile.
// direct: C[d-1, row] = C[row, d-1] = alpha * sum + beta * C[d-1, row], and the
// first tile also writes the corner alpha * count + beta * C[d-1, d-1];
// otherwise the sums go to the k-slice's row-sum slot.
// rowmask: bit im set = row block im of this wave is its to write.
template <int WM>
__device__ __forceinline__ void write_rowsums(float (&rs)[WM], int I, int dt, int d, int direct,
                                              float count, float alpha, float beta,
                                              float *__restrict__ vec, float *__restrict__ C,
                                              int wave = threadIdx.x >> 6, unsigned rowmask = 0xffffffffu) {
  constexpr int BM = 64 * WM;
  const int lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
  for (int im = 0; im < WM; ++im) {
    const float tot = rs[im] + __shfl_xor(rs[im], 32, 64);
    if (wn != 0 || lane >= 32 || !((rowmask >> im) & 1u)) continue;
    const int row = I * BM + (wm * WM + im) * 32 + lane;
    if (!direct) {
      vec[row] = tot;
    } else if (row < dt) {
      float v = alpha * tot;
      if (beta != 0.f) v += beta * C[(long long)(d - 1) * d + row];
      C[(long long)(d - 1) * d + row] = v;
      C[(long long)row * d + d - 1] = v;
    }
  }
  if (direct && I == 0 && wave == 0 && (rowmask & 1u) && lane == 0) {
    float v = alpha * count;
    if (beta != 0.f) v += beta * C[(long long)(d - 1) * d + d - 1];
    C[(long long)(d - 1) * d + d - 1] = v;
  }
}

// With a single k-slice (direct != 0) the tile is scaled and written straight
// from registers; otherwise the raw partial tile goes to the workspace.
// Workgroup -> (tile, k-slice).  Hardware deals consecutive workgroup ids
// round-robin to the 8 XCDs, each with its own L2.  Every XCD therefore gets a
// contiguous chunk of the work list, ordered so that the ~100 workgroups an
// XCD runs at a time share operand panels: one k-slice at a time, tiles in
// super-rows of 8 tile rows walked column by column (8 tiles share a J panel,
// the whole super-row shares 8 I panels).
constexpr int kXcds = 8;
constexpr int kSuperRows = 8;

__device__ __forceinline__ void work_decode(int bid, int total, int ntile, int tiles, int &split,
                                            int &tile, int &I, int &J) {
  const int xcd = bid % kXcds, idx = bid / kXcds;
  const int base = total / kXcds, rem = total % kXcds;
  const int w = xcd * base + (xcd < rem ? xcd : rem) + idx;
  split = w / ntile;
  const int q = w - split * ntile;
  int row, dummy;
  tri_decode(q, row, dummy);
  const int r = row / kSuperRows;
  const int I0 = r * kSuperRows;
  int I1 = I0 + kSuperRows - 1;
  if (I1 > tiles - 1) I1 = tiles - 1;
  const int h = I1 - I0 + 1;
  int qq = q - I0 * (I0 + 1) / 2;
  if (qq < (I0 + 1) * h) {
    J = qq / h;
    I = I0 + (qq - J * h);
  } else {
    qq -= (I0 + 1) * h;
    J = I0 + 1;
    while (qq >= I1 - J + 1) {
      qq -= I1 - J + 1;
      ++J;
    }
    I = J + qq;
  }
  tile = I * (I + 1) / 2 + J;
}

template <int WM, class Loader>
__global__ __launch_bounds__(THREADS, 3) void syrk_kernel(Loader ld, long long K,
                                                          long long klen, int ntile, int nsplit,
                                                          int direct, int d, int ones,
                                                          float alpha, float beta,
                                                          float *__restrict__ partial,
                                                          float *__restrict__ C) {
  constexpr int BM = 64 * WM;
  __shared__ float lds[2 * Panel<BM>::kFloats];
  __shared__ int2 tabA[BM];
  __shared__ int2 tabB[BM];
  float *ldsA = lds, *ldsB = lds + Panel<BM>::kFloats;
  static_assert(2 * Panel<BM>::kFloats >= 64 * 65, "LDS too small for the epilogue transpose");
  const int dt = d - ones;   // rows of the tile grid
  const int tiles = (dt + BM - 1) / BM;
  int split, tile, I, J;
  work_decode(blockIdx.x, ntile * nsplit, ntile, tiles, split, tile, I, J);
  Loader la = ld, lb = ld;
  la.init(reinterpret_cast<float *>(tabA), I * BM);
  lb.init(reinterpret_cast<float *>(tabB), J * BM);
  __syncthreads();
  const long long kbeg = (long long)split * klen;
  long long kend = kbeg + klen;
  if (kend > K) kend = K;
  floatx16 acc[WM][WM];
  zero_acc<WM, WM>(acc);
  float rs[WM];
#pragma unroll
  for (int im = 0; im < WM; ++im) rs[im] = 0.f;
  const int wave = threadIdx.x >> 6;
  const bool active = syrk_wave_active<WM>(I * BM, J * BM, dt, wave);
  if (I == J)
    mainloop_rowsum<WM, WM, true>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB, acc, rs, active,
                                  wave);
  else
    mainloop<WM, WM, false>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB, acc, active, wave);
  const long long slot = (long long)ntile * (BM * BM) + (long long)tiles * BM;
  float *mine = partial + split * slot;
  if (ones && I == J)
    write_rowsums<WM>(rs, I, dt, d, direct, (float)K, alpha, beta, mine + (long long)ntile * (BM * BM), C,
                      wave);
  if (direct) {
    write_tile<WM>(acc, lds, I, J, dt, d, alpha, beta, C, wave);
    return;
  }
  float *out = mine + (long long)tile * (BM * BM);
  for_each_acc<WM, WM>(acc, [&](int r, int c, float v) { out[r * BM + c] = v; }, wave);
}

// Convolution A factor through the LDS halo region (conv_halo.h); `klen` counts
// reduction steps, not k-values.
template <int WM, int NKK, bool MASK>
__global__ __launch_bounds__(THREADS, 2) void syrk_conv_kernel(ConvGeom g, long long total_steps,
                                                               long long klen, int ntile,
                                                               int nsplit, int direct, int d,
                                                               int ones, float count,
                                                               float alpha, float beta,
                                                               float *__restrict__ partial,
                                                               float *__restrict__ C) {
  constexpr int BM = 64 * WM;
  extern __shared__ float smem[];
  const int region = halo_region_floats(g);
  const int regA = 0, regB = region;
  int *koff_tbl = reinterpret_cast<int *>(smem + 2 * region);
  const int dt = d - ones;   // rows of the tile grid
  const int tiles = (dt + BM - 1) / BM;
  int split, tile, I, J;
  work_decode(blockIdx.x, ntile * nsplit, ntile, tiles, split, tile, I, J);
  // zero plane of both regions and the k -> offset table
  for (int e = threadIdx.x; e < g.Rsz; e += THREADS) {
    smem[regA + g.CH * g.Rsz + e] = 0.f;
    smem[regB + g.CH * g.Rsz + e] = 0.f;
  }
  for (int k = threadIdx.x; k < kHaloMaxK; k += THREADS) {
    int off = 0;
    if (k < g.RT * g.WS) {
      const int orow = k / g.WS, ocol = k - orow * g.WS;
      off = orow * g.sy * g.Wr + ocol * g.sx;
    }
    koff_tbl[k] = off;
  }
  __syncthreads();
  const long long sbeg = (long long)split * klen;
  long long send = sbeg + klen;
  if (send > total_steps) send = total_steps;
  floatx16 acc[WM][WM];
  zero_acc<WM, WM>(acc);
  float rs[WM];
#pragma unroll
  for (int im = 0; im < WM; ++im) rs[im] = 0.f;
  if (I == J)
    halo_mainloop<WM, NKK, true, MASK>(g, I * BM, J * BM, sbeg, send, smem, regA, regB, koff_tbl, acc, rs);
  else
    halo_mainloop<WM, NKK, false, MASK>(g, I * BM, J * BM, sbeg, send, smem, regA, regB, koff_tbl, acc, rs);
  const long long slot = (long long)ntile * (BM * BM) + (long long)tiles * BM;
  float *mine = partial + split * slot;
  if (ones && I == J)
    write_rowsums<WM>(rs, I, dt, d, direct, count, alpha, beta, mine + (long long)ntile * (BM * BM), C);
  if (direct) {
    write_tile<WM>(acc, smem, I, J, dt, d, alpha, beta, C);
    return;
  }
  float *out = mine + (long long)tile * (BM * BM);
  for_each_acc<WM, WM>(acc, [&](int r, int c, float v) { out[r * BM + c] = v; });
}

// Convolution A factor through the compile-time row geometry of conv_rows.h;
// `klen` counts reduction steps (RT output rows of a pair of samples each).
template <class Cfg>
__global__ __launch_bounds__(THREADS, 2) void syrk_rows_kernel(RowsGeom g, long long total_steps,
                                                               long long klen, int ntile,
                                                               int nsplit, int direct, int d,
                                                               int ones, float count,
                                                               float alpha, float beta,
                                                               float *__restrict__ partial,
                                                               float *__restrict__ C) {
  constexpr int WM = Cfg::WM;
  constexpr int BM = 64 * WM;
  extern __shared__ float smem[];
  const int dt = d - ones;   // rows of the tile grid
  const int tiles = (dt + BM - 1) / BM;
  int split, tile, I, J;
  work_decode(blockIdx.x, ntile * nsplit, ntile, tiles, split, tile, I, J);
  // padding columns, the planes of zeros and everything else not staged later
  for (int e = threadIdx.x; e < Cfg::lds_floats(false); e += THREADS) smem[e] = 0.f;
  __syncthreads();
  const long long sbeg = (long long)split * klen;
  long long send = sbeg + klen;
  if (send > total_steps) send = total_steps;
  floatx16 acc[WM][WM];
  zero_acc<WM, WM>(acc);
  float rs[WM];
#pragma unroll
  for (int im = 0; im < WM; ++im) rs[im] = 0.f;
  const int wave = threadIdx.x >> 6;
  if (I == J)
    rows_mainloop<Cfg, true>(g, I * BM, J * BM, sbeg, send, smem, acc, rs, wave);
  else
    rows_mainloop<Cfg, false>(g, I * BM, J * BM, sbeg, send, smem, acc, rs, wave);
  const long long slot = (long long)ntile * (BM * BM) + (long long)tiles * BM;
  float *mine = partial + split * slot;
  if (ones && I == J)
    write_rowsums<WM>(rs, I, dt, d, direct, count, alpha, beta, mine + (long long)ntile * (BM * BM), C,
                      wave);
  if (direct) {
    write_tile<WM>(acc, smem, I, J, dt, d, alpha, beta, C, wave);
    return;
  }
  float *out = mine + (long long)tile * (BM * BM);
  for_each_acc<WM, WM>(acc, [&](int r, int c, float v) { out[r * BM + c] = v; }, wave);
}

// One workgroup per 64x64 sub-block (si >= sj) of C.  The number of slices is a
// compile-time constant so that all loads of a thread are issued before the
// first sum needs one (with a run-time loop every slice costs a trip to memory).
template <int NS>
__global__ __launch_bounds__(256) void finish_kernel(const float *__restrict__ partial, int ntile,
                                                     int bm, long long slot, int dt, int d,
                                                     int ones, float count, float alpha,
                                                     float beta, float *__restrict__ C) {
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
  for (int p = 0; p < 16; ++p) {
    float a = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s) a += p0[s * slot + (lr0 + 4 * p) * bm + lc];
    sum[p] = a;
  }
  // ones column: the diagonal sub-blocks finish their 64 row sums
  if (ones && si == sj && threadIdx.x < 64) {
    const int row = si * 64 + threadIdx.x;
    const float *v0 = partial + (long long)ntile * tile_stride + row;
    float a = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s) a += v0[s * slot];
    if (row < dt) {
      float v = alpha * a;
      if (beta != 0.f) v += beta * C[(long long)(d - 1) * d + row];
      C[(long long)(d - 1) * d + row] = v;
      C[(long long)row * d + d - 1] = v;
    }
    if (row == 0) {
      float v = alpha * count;
      if (beta != 0.f) v += beta * C[(long long)(d - 1) * d + d - 1];
      C[(long long)(d - 1) * d + d - 1] = v;
    }
  }
#pragma unroll
  for (int p = 0; p < 16; ++p) {
    const int lr = lr0 + 4 * p;
    const int r = si * 64 + lr, c = sj * 64 + lc;
    float v = alpha * sum[p];
    if (beta != 0.f && r < dt && c < dt) v += beta * C[(long long)r * d + c];
    tile[lr][lc] = v;
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 16; ++p) {
    const int lr = lr0 + 4 * p;
    const int r = si * 64 + lr, c = sj * 64 + lc;
    if (si == sj) {
      if (r < dt && c < dt) C[(long long)r * d + c] = (lc <= lr) ? tile[lr][lc] : tile[lc][lr];
    } else {
      if (r < dt && c < dt) C[(long long)r * d + c] = tile[lr][lc];
      const int mr = sj * 64 + lr, mc = si * 64 + lc;
      if (mr < dt && mc < dt) C[(long long)mr * d + mc] = tile[lc][lr];
    }
  }
}

// reduce_kernel (more than 8 slices) + finish_kernel on the partial tiles.
// d is the dimension of C, ones = 1 if its last row/column is the ones column,
// count the reduction length (the corner entry).
int finish_partials(const SyrkPlan &p, int d, int ones, float count, float alpha, float beta,
                    float *C, float *partial, hipStream_t stream) {
  const float *fin = partial;
  int nfin = p.nsplit;
  const long long slot = (long long)syrk_slot_floats(p);
  kfac::TimedLaunch timed(KFAC_TIMED_COV_AUX, stream);
  if (p.nreduced) {
    const long long slot4 = slot / 4;
    float *red = partial + (size_t)p.nsplit * slot;
    const int per = kfac::ceil_div(p.nsplit, p.nreduced);
    nfin = kfac::ceil_div(p.nsplit, per);
    KFAC_LAUNCH(reduce_kernel, dim3((unsigned)kfac::ceil_div<long long>(slot4, 256), nfin),
                       dim3(256), 0, stream, reinterpret_cast<const float4 *>(partial),
                       reinterpret_cast<float4 *>(red), p.nsplit, per, slot4);
    KFAC_HIP_CHECK(hipGetLastError());
    fin = red;
  }
  const int dt = d - ones;
  const int sub = kfac::ceil_div(dt, 64);
  using Kern = void (*)(const float *, int, int, long long, int, int, int, float, float, float,
                        float *);
  static const Kern kerns[kFinishSplits] = {finish_kernel<1>, finish_kernel<2>, finish_kernel<3>,
                                            finish_kernel<4>, finish_kernel<5>, finish_kernel<6>,
                                            finish_kernel<7>, finish_kernel<8>};
  if (nfin < 1 || nfin > kFinishSplits) return kfac::fail(KFAC_EINVAL, "bad slice count %d", nfin);
  KFAC_LAUNCH(kerns[nfin - 1], dim3(sub * (sub + 1) / 2), dim3(256), 0, stream, fin, p.ntile,
                     p.bm, slot, dt, d, ones, count, alpha, beta, C);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

int check_ws(const SyrkPlan &p, void *ws, size_t ws_bytes) {
  const size_t need = syrk_ws_floats(p) * sizeof(float);
  if (ws_bytes < need || ws == nullptr)
    return kfac::fail(KFAC_ENOMEM, "covariance workspace too small: %zu < %zu bytes", ws_bytes,
                      need);
  return KFAC_OK;
}

// d: dimension of C; ones = 1 if its last row/column is a ones column, which
// the loaders must then not supply (their rows end at d - 1).
template <class L64, class L128>
int run_syrk(const L64 &l64, const L128 &l128, int d, int ones, long long K, float alpha,
             float beta, float *C, void *ws, size_t ws_bytes, hipStream_t stream) {
  if (d - ones == 0) return kfac::fail(KFAC_EINVAL, "empty factor");
  const SyrkPlan p = plan_syrk(d - ones, K);
  if (int rc = check_ws(p, ws, ws_bytes)) return rc;
  float *partial = static_cast<float *>(ws);
  const int grid = p.ntile * p.nsplit;
  const int direct = p.nsplit == 1 ? 1 : 0;
  {
    kfac::TimedLaunch timed(KFAC_TIMED_SYRK, stream);
    if (p.bm == 64)
      KFAC_LAUNCH((syrk_kernel<1, L64>), dim3(grid), dim3(THREADS), 0, stream, l64, K,
                         p.klen, p.ntile, p.nsplit, direct, d, ones, alpha, beta, partial, C);
    else
      KFAC_LAUNCH((syrk_kernel<2, L128>), dim3(grid), dim3(THREADS), 0, stream, l128, K,
                         p.klen, p.ntile, p.nsplit, direct, d, ones, alpha, beta, partial, C);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  if (direct) return KFAC_OK;
  return finish_partials(p, d, ones, (float)K, alpha, beta, C, partial, stream);
}

// Fills the fields of g that depend on the step shape (WS output columns x RT
// output rows); false if that shape does not fit the kernel's limits.
bool halo_step_shape(ConvGeom &g, int WS, int RT) {
  const int khkw = g.kh * g.kw;
  if (WS < 1 || RT < 1 || g.wo % WS != 0) return false;   // ragged column segments are not handled
  g.WS = WS;
  g.RT = RT;
  g.segs = g.wo / WS;
  g.rgroups = kfac::ceil_div(g.ho, RT);
  // k-values per step: one of the compiled loop lengths (2 * 25, 28 or 32);
  // the slots past RT*WS are masked
  const int span = RT * WS;
  if (span < 40 || span > kHaloMaxK) return false;   // too few pixels per step do not pay off
  g.nk = span <= 50 ? 50 : (span <= 56 ? 56 : 64);
  g.Rin = (RT - 1) * g.sy + g.kh;
  g.Win = (WS - 1) * g.sx + g.kw;
  if (g.Rin > 255 || g.Win > 255) return false;
  auto round_mod32 = [](int at_least, int residue) {
    return at_least + ((residue - at_least) % 32 + 32) % 32;
  };
  g.Wr = round_mod32(g.Win, g.kw % 32);
  g.Rsz = round_mod32(g.Rin * g.Wr, khkw % 32);
  g.CH = 127 / khkw + 2;   // 128 consecutive patch rows touch at most this many channels
  g.LPR = 16;
  while (g.LPR < g.Win) g.LPR *= 2;
  if (g.LPR > THREADS) return false;
  g.CPP = THREADS / g.LPR;
  g.passes = kfac::ceil_div(g.CH, g.CPP);
  g.nq = g.passes * g.Rin;
  if (g.nq > kHaloMaxQ) return false;
  g.rep = 0;
  for (int p = 0; p < g.passes; ++p) g.rep |= 1u << (p * g.Rin);
  return true;
}

// Geometry of the LDS halo kernel for one convolution; false when the shape
// does not fit its limits (the element-wise im2col loader is used instead).
// Among the step shapes that fit, the one with the fewest k-slots per sample
// (padding of a step to its loop length and row groups hanging over the bottom
// edge both cost matrix-core work), then the fewest steps.
bool make_halo_geom(const float *x, int n, int c, int h, int w, int kh, int kw, int sy, int sx, int ph,
                    int pw, int ho, int wo, ConvGeom *out) {
  ConvGeom g;
  g.x = x;
  g.C = c; g.H = h; g.W = w; g.kh = kh; g.kw = kw; g.sy = sy; g.sx = sx; g.ph = ph; g.pw = pw;
  g.ho = ho; g.wo = wo;
  g.d_patch = c * kh * kw;
  const int khkw = kh * kw;
  if (khkw < 2 || khkw > 127) return false;
  // the staging loads address x through a 32-bit byte offset whose top bit
  // marks elements outside the image
  const long long x_bytes = (long long)n * c * h * w * (long long)sizeof(float);
  if (x_bytes >= (1ll << 31)) return false;
  g.x_bytes = (unsigned)x_bytes;
  bool found = false;
  long long best_slots = 0, best_steps = 0;
  for (int segs = 1; segs <= wo; ++segs) {
    if (wo % segs != 0) continue;
    const int WS = wo / segs;
    if (WS > kHaloMaxK) continue;
    const int rt_max = std::min(ho, kHaloMaxK / WS);
    for (int RT = 1; RT <= rt_max; ++RT) {
      ConvGeom t = g;
      if (!halo_step_shape(t, WS, RT)) continue;
      const long long steps = (long long)t.segs * t.rgroups;
      const long long slots = steps * t.nk;
      if (!found || slots < best_slots || (slots == best_slots && steps < best_steps)) {
        found = true;
        best_slots = slots;
        best_steps = steps;
        *out = t;
      }
    }
  }
  return found;
}

size_t halo_lds_bytes(const ConvGeom &g) {
  size_t floats = 2 * (size_t)halo_region_floats(g) + kHaloMaxK;
  if (floats < 64 * 65) floats = 64 * 65;   // the epilogue transposes through the same memory
  return floats * sizeof(float);
}

int run_conv_halo(const ConvGeom &g, int n, int d, int ones, float alpha, float beta, float *C,
                  void *ws, size_t ws_bytes, hipStream_t stream) {
  const long long total_steps = (long long)n * g.segs * g.rgroups;
  const float count = (float)((long long)n * g.ho * g.wo);
  SyrkPlan p = plan_syrk_panels(d - ones, total_steps, 1);
  if (p.bm != 128) return 1;   // small factors stay on the generic kernel
  if (int rc = check_ws(p, ws, ws_bytes)) return rc;
  const size_t lds = halo_lds_bytes(g);
  // the masked variants zero operands of k-values past the image's bottom edge
  // or past the end of a step; most shapes do not need them
  const bool mask = (g.RT * g.WS != g.nk) || (g.ho % g.RT != 0);
  using Kern = void (*)(ConvGeom, long long, long long, int, int, int, int, int, float, float,
                        float, float *, float *);
  static const Kern kerns[3][2] = {
      {syrk_conv_kernel<2, 25, false>, syrk_conv_kernel<2, 25, true>},
      {syrk_conv_kernel<2, 28, false>, syrk_conv_kernel<2, 28, true>},
      {syrk_conv_kernel<2, 32, false>, syrk_conv_kernel<2, 32, true>}};
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [] {
    if (kfac::host_only()) return;
    for (int i = 0; i < 3; ++i)
      for (int j = 0; j < 2; ++j) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kerns[i][j]),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 160 * 1024);
        if (e != hipSuccess) attr_rc = e;
      }
  });
  KFAC_HIP_CHECK(attr_rc);
  float *partial = static_cast<float *>(ws);
  const int direct = p.nsplit == 1 ? 1 : 0;
  const dim3 grid(p.ntile * p.nsplit), block(THREADS);
  const Kern kern = kerns[g.nk == 50 ? 0 : (g.nk == 56 ? 1 : 2)][mask ? 1 : 0];
  {
    kfac::TimedLaunch timed(KFAC_TIMED_SYRK, stream);
    KFAC_LAUNCH(kern, grid, block, lds, stream, g, total_steps, p.klen, p.ntile, p.nsplit,
                       direct, d, ones, count, alpha, beta, partial, C);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  if (direct) return KFAC_OK;
  return finish_partials(p, d, ones, count, alpha, beta, C, partial, stream);
}

// The compile-time-geometry kernel (conv_rows.h) for one of its instantiations.
template <class Cfg>
int run_conv_rows(const float *x, int n, int c, int h, int w, int ho, int d, int ones, float alpha,
                  float beta, float *C, void *ws, size_t ws_bytes, hipStream_t stream) {
  RowsGeom g;
  g.x = x;
  g.n = n; g.C = c; g.H = h; g.W = w;
  g.ho = ho;
  g.rgroups = ho / Cfg::RT;
  g.d_patch = c * Cfg::KK;
  g.x_bytes = (unsigned)((long long)n * c * h * w * (long long)sizeof(float));
  const long long total_steps = (long long)(n / 2) * g.rgroups;
  const float count = (float)((long long)n * ho * Cfg::WS);
  // small factors: 64-tiles of the general kernel (a 7x7 kernel has 49 taps per channel: 3
  // channels are a factor of 147 rows, and the element gather it would otherwise take is slow)
  if (d - ones <= (Cfg::K == 7 ? 128 : 256)) return 1;
  constexpr size_t lds = (size_t)Cfg::lds_floats(false) * sizeof(float);
  constexpr int occ = (160 * 1024) / lds >= 3 ? 3 : (int)((160 * 1024) / lds);
  const SyrkPlan p = plan_rows(d - ones, 64 * Cfg::WM, total_steps, Cfg::NK * Cfg::WM * Cfg::WM * 64 / 2400.0, occ);
  if (int rc = check_ws(p, ws, ws_bytes)) return rc;
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [] {
    if (kfac::host_only()) return;
    attr_rc = hipFuncSetAttribute(reinterpret_cast<const void *>(syrk_rows_kernel<Cfg>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  });
  KFAC_HIP_CHECK(attr_rc);
  float *partial = static_cast<float *>(ws);
  const int direct = p.nsplit == 1 ? 1 : 0;
  {
    kfac::TimedLaunch timed(KFAC_TIMED_SYRK, stream);
    KFAC_LAUNCH((syrk_rows_kernel<Cfg>), dim3(p.ntile * p.nsplit), dim3(THREADS), lds, stream,
                       g, total_steps, p.klen, p.ntile, p.nsplit, direct, d, ones, count, alpha, beta,
                       partial, C);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  if (direct) return KFAC_OK;
  return finish_partials(p, d, ones, count, alpha, beta, C, partial, stream);
}

// Picks the instantiation of the compile-time-geometry kernel that matches the
// convolution; 1 when there is none (the caller then takes a general kernel).
int try_conv_rows(const float *x, int n, int c, int h, int w, int kh, int kw, int sy, int sx, int ph,
                  int pw, int ho, int wo, int d, int ones, float alpha, float beta, float *C,
                  void *ws, size_t ws_bytes, hipStream_t stream) {
  if (kfac::option_int(kfac::kOptConvRows, 1) == 0) return 1;   // tuning override: the general kernels only
  if (n % 2 != 0 || kh != kw || sy != sx || ph != pw) return 1;
  if ((long long)n * c * h * w * (long long)sizeof(float) >= (1ll << 31)) return 1;
  // 128-tiles feed the matrix cores with half the LDS traffic of 64-tiles, but a
  // factor whose side is not a multiple of 128 pays for the padded part of its last
  // tile row and every diagonal tile for its upper half: take 64-tiles when they
  // save more than the ~15 % their main loop is slower by (576 rows: 45 tiles of
  // 64 against 15 of 128, i.e. 45 against 60 units of matrix-core work).
  const int dt = d - ones;
  const long long t64 = kfac::ceil_div(dt, 64), t128 = kfac::ceil_div(dt, 128);
  bool small_tiles = 1.15 * (double)(t64 * (t64 + 1) / 2) < 4.0 * (double)(t128 * (t128 + 1) / 2);
  if (kfac::option_is_set(kfac::kOptRowsWm)) small_tiles = kfac::option_int(kfac::kOptRowsWm, 2) == 1;   // tuning override
#define KFAC_ROWS_CASE(K, S, P, WS, RT, PAD)                                                      \
  if (kh == K && sy == S && ph == P && wo == WS && ho % RT == 0) {                                \
    if (small_tiles)                                                                              \
      return run_conv_rows<RowsCfg<1, K, S, P, WS, RT, PAD>>(x, n, c, h, w, ho, d, ones, alpha,   \
                                                             beta, C, ws, ws_bytes, stream);      \
    return run_conv_rows<RowsCfg<2, K, S, P, WS, RT, PAD>>(x, n, c, h, w, ho, d, ones, alpha,     \
                                                           beta, C, ws, ws_bytes, stream);        \
  }
  // (kernel, stride, padding, output width, output rows per step, plane padding: the
  // smallest that leaves the 32 operand rows of a block on 32 different banks of 64)
  KFAC_ROWS_CASE(3, 1, 1, 56, 1, 0)
  KFAC_ROWS_CASE(3, 1, 1, 28, 2, 1)
  KFAC_ROWS_CASE(3, 1, 1, 14, 7, 3)
  KFAC_ROWS_CASE(3, 1, 1, 7, 7, 9)
  // the strided 3x3 convolutions of ResNet-D (56 -> 28, 28 -> 14) and its 112-wide stem.  (14 -> 7
  // with the whole 7x7 output per step needs 65 KB of LDS, two workgroups per CU, and was
  // measured slower than the halo-region kernel: 443 against 364 us for 512 channels.)
  KFAC_ROWS_CASE(3, 2, 1, 28, 1, 1)
  KFAC_ROWS_CASE(3, 2, 1, 14, 2, 6)
  KFAC_ROWS_CASE(3, 1, 1, 112, 1, 1)
  // the 7x7 stride-2 stem of ResNet at 224 x 224
  KFAC_ROWS_CASE(7, 2, 3, 112, 1, 0)
  // CIFAR-sized images
  KFAC_ROWS_CASE(3, 1, 1, 32, 2, 0)
  KFAC_ROWS_CASE(3, 1, 1, 16, 4, 8)
  KFAC_ROWS_CASE(3, 1, 1, 8, 8, 11)
#undef KFAC_ROWS_CASE
  return 1;
}

// Slices of the whole-image groups of the shifted-correlation route: the workgroups
// of a launch run two to a CU, 512 at a time (three with 64 first-operand channels),
// and a group of ns shifts does ns tile products per panel.  Among the slice counts
// (s5 for the two groups of five shifts, s3 for the group of three) the pair with
// the least rounds x longest item, plus what an item costs besides its panels
// (prologue, partial tiles written and summed).  ntab: tile pairs per product, nk:
// panels of the whole reduction.
struct ShiftSlices {
  long long s5, s3;
  double longest;   // shift-panels of the longest item
};
constexpr long long kShiftMaxItems = 1024;

ShiftSlices plan_shift_slices(int wm, int ntab, long long nk) {
  long long best_s5 = 1, best_s3 = 1;
  double best_cost = 0.0, best_longest = (double)(5 * nk);
  for (long long s5 = 1; s5 <= nk && ntab * (2 * s5 + 1) <= kShiftMaxItems; ++s5) {
    const long long len5 = kfac::ceil_div(nk, s5);
    if (kfac::ceil_div(nk, len5) != s5) continue;
    // the slice count of the three-shift group whose items are no longer than these
    long long len3 = std::min(nk, std::max<long long>(1, 5 * len5 / 3));
    const long long s3 = kfac::ceil_div(nk, len3);
    len3 = kfac::ceil_div(nk, s3);
    const long long items = ntab * (2 * s5 + s3);
    if (items > kShiftMaxItems) continue;
    const double longest = (double)std::max(5 * len5, 3 * len3);
    const double rounds = (double)kfac::ceil_div<long long>(items, wm == 1 ? 768 : 512);
    // an item's fixed cost in units of one shift-panel
    const double cost = rounds * (longest + 6.0) + 0.004 * (double)items;
    if (best_cost == 0.0 || cost < best_cost) {
      best_cost = cost;
      best_s5 = s5;
      best_s3 = s3;
      best_longest = longest;
    }
  }
  if (kfac::option_is_set(kfac::kOptShiftSlices5) && kfac::option_is_set(kfac::kOptShiftSlices3)) {   // tuning override
    const long long a = (long long)kfac::option_value(kfac::kOptShiftSlices5, 0);
    const long long b = (long long)kfac::option_value(kfac::kOptShiftSlices3, 0);
    if (a >= 1 && b >= 1) {
      best_s5 = std::min(a, nk);
      best_s3 = std::min(b, nk);
      best_longest = (double)std::max(5 * kfac::ceil_div(nk, best_s5), 3 * kfac::ceil_div(nk, best_s3));
    }
  }
  return ShiftSlices{best_s5, best_s3, best_longest};
}

// Stacked groups (one tile pair, two groups of three column offsets): equal slices,
// about 720 items in all for the 768 slots of three workgroups per CU.
ShiftSlices plan_stacked_slices(long long nk) {
  const long long want = std::max<long long>(1, std::min<long long>(360, nk / 8));
  const long long len = kfac::ceil_div(nk, want);
  const long long ns = kfac::ceil_div(nk, len);
  return ShiftSlices{ns, ns, (double)(3 * len)};
}

// Slices of a strip or corner group of gk panels: items about as long as the others'.
long long shift_strip_slices(long long gk, double longest) {
  return kfac::ceil_div<long long>(3 * gk, std::max<long long>(3, (long long)longest));
}

// 64-row first-operand tiles unless 128 rows waste no more on the channel count
int shift_wm(int c) {
  const long long t64 = kfac::ceil_div(c, 64), t128 = kfac::ceil_div(c, 128);
  return 1.15 * (double)(t64 * t64) < 4.0 * (double)(t128 * t128) ? 1 : 2;
}

// Layers of 28..32 channels take the route with stacked operand tiles (conv_shift.h).
bool shift_stacked(int c) { return c >= 28 && c <= 32; }

bool shift_route_takes(int c, int h, int w) {
  int min_c = 64;
  bool stacked_on = true;
  if (kfac::option_is_set(kfac::kOptConvShift)) {   // tuning override: 0 = off, else the least channel count
    min_c = kfac::option_int(kfac::kOptConvShift, min_c);
    if (min_c <= 0) return false;
    stacked_on = min_c <= 32;
  }
  return (c >= min_c || (stacked_on && shift_stacked(c))) && h >= 4 && w >= 4 && h <= 32767 && w <= 32767;
}

// Upper bound of the workspace floats the route takes for c channels and `rows` =
// samples x pixels (the image's sides are not known here: at least 4 each).
size_t shift_ws_floats_bound(int c, long long rows) {
  const int wm = shift_wm(c), bm = 64 * wm;
  const int ntab = kfac::ceil_div(c, bm) * kfac::ceil_div(c, 64);
  const long long nk = kfac::ceil_div<long long>(rows, KT);
  const bool stacked = shift_stacked(c);
  const ShiftSlices sl = stacked ? plan_stacked_slices(nk) : plan_shift_slices(wm, ntab, nk);
  size_t floats = stacked ? (size_t)(sl.s5 + sl.s3) * 3 * bm * 64
                          : (size_t)ntab * (size_t)(2 * sl.s5 * 5 + sl.s3 * 3) * bm * 64;
  // 8 strip / corner groups of three shifts; a strip has at most rows / 4 k-values
  const long long strip =
      shift_strip_slices(kfac::ceil_div<long long>(kfac::ceil_div<long long>(rows, 4), KT), sl.longest);
  floats += (size_t)8 * ntab * (size_t)std::max(1ll, strip) * 3 * bm * 64;
  floats += (size_t)kfac::shift::kArrays * c * c;
  floats += (size_t)1024 * kfac::shift::kChannelSums + (size_t)c * 16;   // sums: at most 1024 (chunk, channel) pairs
  floats += (size_t)c * (size_t)kfac::ceil_div<long long>(rows, 2);      // border columns: 2 n c h, h <= rows / (4 n)
  return floats + 256;
}

// The shifted-correlation route (conv_shift.h) for a 3x3, stride-1, padding-1
// convolution: 1 when the shape is left to the patch-product kernels (few
// channels, tiny images, workspace too small).
template <int WM>
int run_conv_shift(kfac::shift::Plan &pl, int d, int ones, float alpha, float beta, float *C, void *ws,
                   size_t ws_bytes, hipStream_t stream) {
  using namespace kfac::shift;
  constexpr int BM = 64 * WM;
  const int c = pl.C, h = pl.H, w = pl.W, n = pl.n;
  pl.tiles_a = kfac::ceil_div(c, BM);
  pl.tiles_b = kfac::ceil_div(c, 64);
  const int ntab = pl.tiles_a * pl.tiles_b;
  // workspace: [partial tiles | arrays | channel sums | border columns]; the last two
  // have sizes known up front and are placed from the end
  const int nchunk = std::max(1, std::min(n, 1024 / c));
  const size_t array_floats = (size_t)kArrays * c * c;
  const size_t sums_floats = (size_t)nchunk * c * kChannelSums;
  const size_t edge_floats = (size_t)2 * n * c * h;
  const size_t tail_floats = array_floats + sums_floats + edge_floats + 64;
  // a workspace smaller than the route needs sends the factor to the patch-product
  // kernels (option conv_shift_strict: an error instead, for the test of the workspace query)
  auto too_small = [&](size_t need_floats) {
    if (kfac::option_int(kfac::kOptConvShiftStrict, 0) != 0)
      return kfac::fail(KFAC_ENOMEM, "shifted-correlation workspace too small: %zu < %zu bytes", ws_bytes,
                        need_floats * sizeof(float));
    return 1;
  };
  if (ws == nullptr || ws_bytes < tail_floats * sizeof(float)) return too_small(tail_floats);
  float *partial = static_cast<float *>(ws);
  float *arrays = partial + (ws_bytes / sizeof(float) - tail_floats) / 4 * 4;
  float *sums = arrays + array_floats;
  float *edges = sums + sums_floats;
  // groups: whole image (di = 0, 1, 2), first / last row, first / last column, corners
  auto group = [&](int gi, const float *base, long long sample_stride, int row_stride, int line_stride, int L,
                   int mem_line, int vline, int di, int dj0, int ns, int amax) {
    ShiftGroup &g = pl.grp[gi];
    g.base = base;
    g.sample_stride = (unsigned)sample_stride; g.row_stride = (unsigned)row_stride;
    g.line_stride = (unsigned)line_stride;
    g.L = (unsigned)L; g.mem_line = (unsigned)mem_line; g.vline = (unsigned)vline;
    g.di = (short)di; g.dj0 = (short)dj0; g.ns = (short)ns; g.amax = (short)amax;
    g.stacked = 0;
    g.K = n * L;
  };
  const long long xs = (long long)c * h * w, es = (long long)c * h;
  const bool stacked = shift_stacked(c);
  if (stacked) {
    // row shifts 0 and 1 from one group (both halves of the first operand), row shift 2 from another
    group(0, pl.x, xs, h * w, w, h * w, h * w, w, 0, -2, 3, h);
    group(1, pl.x, xs, h * w, w, h * w, h * w, w, 2, -2, 3, h);
    group(2, pl.x, xs, h * w, w, h * w, h * w, w, 2, -2, 3, h);   // no items
    pl.grp[0].stacked = 2;
    pl.grp[1].stacked = 1;
  } else {
    group(0, pl.x, xs, h * w, w, h * w, h * w, w, 0, 0, 3, h);
    group(1, pl.x, xs, h * w, w, h * w, h * w, w, 1, -2, 5, h);
    group(2, pl.x, xs, h * w, w, h * w, h * w, w, 2, -2, 5, h);
  }
  for (int last = 0; last < 2; ++last) {
    group(3 + last, pl.x + (last ? (h - 1) * w : 0), xs, h * w, w, w, w, w, 0, 0, 3, 1);
    const float *col = edges + (size_t)last * n * c * h;
    group(5 + last, col, es, h, h, h, h, h, 0, 0, 3, 1);
  }
  for (int lr = 0; lr < 2; ++lr)
    for (int lc = 0; lc < 2; ++lc)
      group(7 + 2 * lr + lc, edges + (size_t)lc * n * c * h + (lr ? h - 1 : 0), es, h, h, 1, 1, 1, 0, 0, 3, 1);
  const long long nk = kfac::ceil_div(n * h * w, KT);
  const ShiftSlices sl = stacked ? plan_stacked_slices(nk) : plan_shift_slices(WM, ntab, nk);
  const long long best_s5 = sl.s5, best_s3 = sl.s3;
  const double best_longest = sl.longest;
  // items: strips and corners first (block order), then the whole-image groups
  size_t partial_floats = 0;
  int total = 0;
  auto slice = [&](int gi, long long ns) {
    ShiftGroup &g = pl.grp[gi];
    const long long gk = kfac::ceil_div(g.K, KT);
    const long long len = kfac::ceil_div(gk, std::max(1ll, std::min(ns, gk)));
    g.nsplit = (int)kfac::ceil_div(gk, len);
    g.klen = (int)len * KT;
    g.task0 = total;
    g.part_off = (unsigned)partial_floats;
    total += ntab * g.nsplit;
    partial_floats += (size_t)ntab * g.nsplit * g.ns * BM * 64;
  };
  for (int gi = 3; gi < kGroups; ++gi) {
    const long long gk = kfac::ceil_div(pl.grp[gi].K, KT);
    slice(gi, shift_strip_slices(gk, best_longest));
  }
  pl.nsmall = total;
  slice(0, best_s3);
  slice(1, best_s5);
  if (stacked) {
    ShiftGroup &g = pl.grp[2];   // empty
    g.nsplit = 0;
    g.klen = KT;
    g.task0 = total;
    g.part_off = (unsigned)partial_floats;
  } else {
    slice(2, best_s5);
  }
  pl.total = total;
  // products -> (group, shift)
  int np = 0;
  auto product = [&](int gi, int e, int out, int out_t) {
    const ShiftGroup &g = pl.grp[gi];
    Product &p = pl.prod[np++];
    p.nsplit = g.nsplit;
    p.tile_stride = (unsigned)(g.ns * BM * 64);
    p.split_stride = (unsigned)ntab * p.tile_stride;
    p.part_off = g.part_off + (unsigned)((e - g.dj0) * BM * 64);
    p.out = (short)out;
    p.out_t = (short)out_t;
  };
  for (int di = 0; di <= 2; ++di)
    for (int dj = (di == 0 ? 0 : -2); dj <= 2; ++dj) {
      if (!stacked) {
        product(di, dj, (di + 2) * 5 + dj + 2, (2 - di) * 5 + 2 - dj);
        continue;
      }
      // block (a, b) of the stacked tile at column offset e: row shift di0 + a, column shift -2 + 3 b + e
      const int gi = di == 2 ? 1 : 0, a = di == 2 ? 0 : di, b = (dj + 2) / 3, e = (dj + 2) % 3;
      product(gi, -2 + e, (di + 2) * 5 + dj + 2, (2 - di) * 5 + 2 - dj);
      pl.prod[np - 1].part_off += (unsigned)(a * 32 * 64 + b * 32);
    }
  for (int last = 0; last < 2; ++last)
    for (int dj = 0; dj <= 2; ++dj) product(3 + last, dj, 25 + 5 * last + dj + 2, 25 + 5 * last + 2 - dj);
  for (int last = 0; last < 2; ++last)
    for (int di = 0; di <= 2; ++di) product(5 + last, di, 35 + 5 * last + di + 2, 35 + 5 * last + 2 - di);
  for (int lr = 0; lr < 2; ++lr)
    for (int lc = 0; lc < 2; ++lc) product(7 + 2 * lr + lc, 0, 45 + 2 * lr + lc, 45 + 2 * lr + lc);
  if (np != kProducts) return kfac::fail(KFAC_EINVAL, "internal: %d products", np);
  if (partial_floats >= (1ull << 32)) return 1;
  if (partial + partial_floats > arrays) return too_small(partial_floats + tail_floats + 4);
  {
    kfac::TimedLaunch timed(KFAC_TIMED_COV_AUX, stream);
    KFAC_LAUNCH(edge_sums_kernel, dim3(c, nchunk), dim3(256), 0, stream, pl, sums, edges);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  {
    kfac::TimedLaunch timed(KFAC_TIMED_SYRK, stream);
    KFAC_LAUNCH((corr_kernel<WM>), dim3(pl.total), dim3(THREADS), 0, stream, pl, partial);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  int max_split = 1;
  for (int i = 0; i < np; ++i) max_split = std::max(max_split, pl.prod[i].nsplit);
  kfac::TimedLaunch timed_post(KFAC_TIMED_COV_AUX, stream);   // the two launches that follow
  if (max_split >= 32 && c <= 128) {
    const int nb = kfac::ceil_div(c, 16);
    KFAC_LAUNCH((corr_finish_kernel<4, WM>), dim3(kProducts * nb * nb), dim3(256), 0, stream, pl, partial,
                       arrays);
  } else {
    const int nb = kfac::ceil_div(c, 32);
    KFAC_LAUNCH((corr_finish_kernel<1, WM>), dim3(kProducts * nb * nb), dim3(256), 0, stream, pl, partial,
                       arrays);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  KFAC_LAUNCH(assemble_kernel, dim3(c, kfac::ceil_div(c, 64), c <= 128 ? 3 : 1), dim3(256), 0, stream, pl, arrays, sums,
                     nchunk, d, ones, (float)((long long)n * h * w), alpha, beta, C);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

int try_conv_shift(const float *x, int n, int c, int h, int w, int kh, int kw, int sy, int sx, int ph,
                   int pw, int d, int ones, float alpha, float beta, float *C, void *ws, size_t ws_bytes,
                   hipStream_t stream) {
  if (kh != 3 || kw != 3 || sy != 1 || sx != 1 || ph != 1 || pw != 1) return 1;
  if (!shift_route_takes(c, h, w)) return 1;
  kfac::shift::Plan pl;
  memset(&pl, 0, sizeof(pl));
  pl.x = x;
  pl.sample_stride = (unsigned)((long long)c * h * w);
  pl.row_stride = (unsigned)(h * w);
  pl.C = c; pl.H = h; pl.W = w; pl.n = n;
  if (shift_wm(c) == 1) return run_conv_shift<1>(pl, d, ones, alpha, beta, C, ws, ws_bytes, stream);
  return run_conv_shift<2>(pl, d, ones, alpha, beta, C, ws, ws_bytes, stream);
}

bool kc_vec_ok(const float *base, long long sample_stride, long long row_stride, int L) {
  return (sample_stride % 4 == 0) && (row_stride % 4 == 0) && (L % 4 == 0) &&
         (reinterpret_cast<uintptr_t>(base) % 16 == 0);
}

template <int ROWS, bool VEC>
LoaderKC<ROWS, VEC> make_kc(const float *base, long long sample_stride, long long row_stride, int L,
                            int rows_valid) {
  LoaderKC<ROWS, VEC> l;
  l.base = base;
  l.sample_stride = (unsigned)sample_stride;
  l.row_stride = (unsigned)row_stride;
  l.L = (unsigned)L;
  l.rows_valid = rows_valid;
  return l;
}

bool ks_vec_ok(const float *base, long long ld) {
  return (ld % 4 == 0) && (reinterpret_cast<uintptr_t>(base) % 16 == 0);
}

template <int ROWS, bool VEC>
LoaderKS<ROWS, VEC> make_ks(const float *base, long long ld, int rows_valid, int has_extra,
                            const float *extra) {
  LoaderKS<ROWS, VEC> l;
  l.base = base;
  l.extra = extra;
  l.ld = (unsigned)ld;
  l.rows_valid = rows_valid;
  l.has_extra = has_extra;
  return l;
}

template <int ROWS>
LoaderIM<ROWS> make_im(const float *x, int c, int h, int w, int kh, int kw, int sy, int sx,
                       int ph, int pw, int ho, int wo) {
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
  l.table = nullptr;
  return l;
}

}  // namespace

extern "C" size_t kfac_cov_workspace_bytes(int d, int64_t rows) {
  if (d <= 0) return 0;
  // upper bound over every kernel and reduction length: no plan uses more than
  // max_splits(tiles) k-slices (plus the slots of the pre-reduction), with 64- or
  // 128-tiles, with or without a ones column (the tile grid then covers d - 1 rows)
  size_t need = 0;
  for (int dt = d > 1 ? d - 1 : d; dt <= d; ++dt)
    for (int bm = 64; bm <= 128; bm *= 2) {
      SyrkPlan p;
      p.bm = bm;
      p.tiles = kfac::ceil_div(dt, bm);
      p.ntile = p.tiles * (p.tiles + 1) / 2;
      p.nsplit = (int)max_splits(p.ntile);
      p.nreduced = p.nsplit > kFinishSplits ? kFinishSplits : 0;
      need = std::max(need, syrk_ws_floats(p));
    }
  // the shifted-correlation route of a 3x3 convolution's A factor (d = 9 c or 9 c + 1)
  for (int ones = 0; ones <= 1 && rows > 0; ++ones)
    if ((d - ones) % 9 == 0 && shift_route_takes((d - ones) / 9, 4, 4))
      need = std::max(need, shift_ws_floats_bound((d - ones) / 9, rows));
  return need * sizeof(float);
}

extern "C" int kfac_cov_linear_f32(const float *x, int n, int d_in, int append_ones,
                                   float alpha, float beta, float *C, void *ws,
                                   size_t ws_bytes, void *stream) {
  KFAC_REQUIRE(n > 0 && d_in > 0, "bad shape n=%d d_in=%d", n, d_in);
  KFAC_REQUIRE((long long)n * d_in < 0x40000000LL, "input too large");
  KFAC_REQUIRE(x && C, "null pointer");
  const int ones = append_ones ? 1 : 0;
  const int d = d_in + ones;
  if (ks_vec_ok(x, d_in))
    return run_syrk(make_ks<64, true>(x, d_in, d_in, 0, nullptr),
                    make_ks<128, true>(x, d_in, d_in, 0, nullptr), d, ones, n, alpha, beta, C, ws,
                    ws_bytes, kfac::as_stream(stream));
  return run_syrk(make_ks<64, false>(x, d_in, d_in, 0, nullptr),
                  make_ks<128, false>(x, d_in, d_in, 0, nullptr), d, ones, n, alpha, beta, C, ws,
                  ws_bytes, kfac::as_stream(stream));
}

extern "C" int kfac_cov_conv_g_f32(const float *gy, int n, int c, int howo, float alpha,
                                   float beta, float *C, void *ws, size_t ws_bytes,
                                   void *stream) {
  KFAC_REQUIRE(n > 0 && c > 0 && howo > 0, "bad shape n=%d c=%d howo=%d", n, c, howo);
  KFAC_REQUIRE((long long)n * c * howo < 0x40000000LL, "input too large");
  KFAC_REQUIRE(gy && C, "null pointer");
  const long long K = (long long)n * howo;
  if (kc_vec_ok(gy, (long long)c * howo, howo, howo))
    return run_syrk(make_kc<64, true>(gy, (long long)c * howo, howo, howo, c),
                    make_kc<128, true>(gy, (long long)c * howo, howo, howo, c), c, 0, K, alpha,
                    beta, C, ws, ws_bytes, kfac::as_stream(stream));
  return run_syrk(make_kc<64, false>(gy, (long long)c * howo, howo, howo, c),
                  make_kc<128, false>(gy, (long long)c * howo, howo, howo, c), c, 0, K, alpha,
                  beta, C, ws, ws_bytes, kfac::as_stream(stream));
}

namespace {
thread_local int last_conv_route = -1;
}

extern "C" int kfac_cov_conv_a_last_route(void) { return last_conv_route; }

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
  KFAC_REQUIRE((long long)n * c * h * w < 0x40000000LL, "input too large");
  const int d = (int)dl;
  const int ones = append_ones ? 1 : 0;
  const long long K = (long long)n * ho * wo;
  hipStream_t s = kfac::as_stream(stream);
  last_conv_route = KFAC_CONV_ROUTE_SLAB;
  if (kh == 1 && kw == 1 && sy == 1 && sx == 1 && ph == 0 && pw == 0) {
    // 1x1 convolution: the patch matrix is the NCHW tensor itself
    const int hw = h * w;
    if (kc_vec_ok(x, (long long)c * hw, hw, hw))
      return run_syrk(make_kc<64, true>(x, (long long)c * hw, hw, hw, c),
                      make_kc<128, true>(x, (long long)c * hw, hw, hw, c), d, ones, K, alpha,
                      beta, C, ws, ws_bytes, s);
    return run_syrk(make_kc<64, false>(x, (long long)c * hw, hw, hw, c),
                    make_kc<128, false>(x, (long long)c * hw, hw, hw, c), d, ones, K, alpha,
                    beta, C, ws, ws_bytes, s);
  }
  if (kh == 1 && kw == 1 && ph == 0 && pw == 0) {
    // strided 1x1 convolution: the same slab, every sx-th pixel of every sy-th line
    auto l64 = make_kc<64, false>(x, (long long)c * h * w, (long long)h * w, ho * wo, c);
    auto l128 = make_kc<128, false>(x, (long long)c * h * w, (long long)h * w, ho * wo, c);
    l64.line_len = l128.line_len = (unsigned)wo;
    l64.line_stride = l128.line_stride = (unsigned)(sy * w);
    l64.px_stride = l128.px_stride = (unsigned)sx;
    return run_syrk(l64, l128, d, ones, K, alpha, beta, C, ws, ws_bytes, s);
  }
  {
    last_conv_route = KFAC_CONV_ROUTE_SHIFT;
    const int rc = try_conv_shift(x, n, c, h, w, kh, kw, sy, sx, ph, pw, d, ones, alpha, beta, C, ws,
                                  ws_bytes, s);
    if (rc <= 0) return rc;   // 1 = shape left to the patch-product kernels
  }
  {
    last_conv_route = KFAC_CONV_ROUTE_ROWS;
    const int rc = try_conv_rows(x, n, c, h, w, kh, kw, sy, sx, ph, pw, ho, wo, d, ones, alpha, beta, C,
                                 ws, ws_bytes, s);
    if (rc <= 0) return rc;   // 1 = no instantiation for this shape
  }
  ConvGeom geom;
  if (make_halo_geom(x, n, c, h, w, kh, kw, sy, sx, ph, pw, ho, wo, &geom)) {
    last_conv_route = KFAC_CONV_ROUTE_HALO;
    const int rc = run_conv_halo(geom, n, d, ones, alpha, beta, C, ws, ws_bytes, s);
    if (rc <= 0) return rc;   // 1 = shape left to the generic kernel
  }
  last_conv_route = KFAC_CONV_ROUTE_GATHER;
  return run_syrk(make_im<64>(x, c, h, w, kh, kw, sy, sx, ph, pw, ho, wo),
                  make_im<128>(x, c, h, w, kh, kw, sy, sx, ph, pw, ho, wo), d, ones, K, alpha,
                  beta, C, ws, ws_bytes, s);
}

// ---------------------------------------------------------------------------
// Grouped launch: the factors of many small layers in a handful of launches.
//
// A network has dozens of factors whose SYRK is far too small to fill the GPU
// (a few tiles, or a few hundred reduction panels): launched one by one each
// costs a launch whose workgroups run two to six panels between a prologue and
// an epilogue.  A group takes a list of such factors, cuts all of them into
// (factor, tile, k-slice) tasks of about equal length (so a long reduction over
// one tile and a short one over thousands of tiles end up in workgroups of
// similar duration, ~100 panels where the work allows it) and runs the tasks of
// all factors from one task table: one launch per loader kind, one for the
// split-K finish.  All grouped factors use 64-tiles.
// ---------------------------------------------------------------------------
namespace {

struct GroupItemStatic {
  int d, ones, bm, tiles, ntile, nsplit, direct;
  long long K, klen;      // reduction length; per k-slice (a multiple of KT)
  // graded slices: the first nfull slices have klen k-values, the others klen2
  // (half of it: short tasks for the end of a launch)
  int nfull;
  long long klen2;
  long long part_off;     // floats from the workspace base to this item's partial slots
  float count;            // reduction length as a float: the corner entry of a ones column
  int kind;               // KFAC_COV_LINEAR / KFAC_COV_SLAB
  int vec;                // float4 loader
  unsigned sample_stride, row_stride, L;   // slab: (sample, row, l) strides; l values per sample
  unsigned line_len, line_stride, px_stride;
  unsigned ld;            // linear: leading dimension
  int rows_valid;
};

struct GroupItemDyn {
  const float *in;
  float *out;
  float alpha, beta;
};

template <class Loader>
struct GroupLoader;

template <int ROWS, bool VEC>
struct GroupLoader<LoaderKC<ROWS, VEC>> {
  static __device__ __forceinline__ LoaderKC<ROWS, VEC> make(const GroupItemStatic &s, const float *in) {
    LoaderKC<ROWS, VEC> l;
    l.base = in;
    l.sample_stride = s.sample_stride;
    l.row_stride = s.row_stride;
    l.L = s.L;
    l.rows_valid = s.rows_valid;
    if constexpr (!VEC) {
      l.line_len = s.line_len;
      l.line_stride = s.line_stride;
      l.px_stride = s.px_stride;
    }
    return l;
  }
};

template <int ROWS, bool VEC>
struct GroupLoader<LoaderKS<ROWS, VEC>> {
  static __device__ __forceinline__ LoaderKS<ROWS, VEC> make(const GroupItemStatic &s, const float *in) {
    LoaderKS<ROWS, VEC> l;
    l.base = in;
    l.extra = nullptr;
    l.ld = s.ld;
    l.rows_valid = s.rows_valid;
    l.has_extra = 0;
    return l;
  }
};

// task = (item, tile + ntile * k-slice); WM = 1: items with 64-tiles, 2: 128-tiles
template <int WM, class Loader>
__global__ __launch_bounds__(THREADS, 3) void syrk_group_kernel(const GroupItemStatic *__restrict__ st,
                                                                const GroupItemDyn *__restrict__ dy,
                                                                const int2 *__restrict__ tasks,
                                                                float *__restrict__ ws) {
  constexpr int BM = 64 * WM;
  __shared__ float lds[2 * Panel<BM>::kFloats];
  static_assert(2 * Panel<BM>::kFloats >= 64 * 65, "LDS too small for the epilogue transpose");
  float *ldsA = lds, *ldsB = lds + Panel<BM>::kFloats;
  const int2 task = tasks[blockIdx.x];
  if (task.x < 0) return;   // padding of a shorter XCD run
  const GroupItemStatic s = st[task.x];
  const GroupItemDyn v = dy[task.x];
  const int split = task.y / s.ntile;
  const int tile = task.y - split * s.ntile;
  int I, J;
  tri_decode(tile, I, J);
  const int dt = s.d - s.ones;
  Loader la = GroupLoader<Loader>::make(s, v.in), lb = la;
  la.init(nullptr, I * BM);
  lb.init(nullptr, J * BM);
  const long long kbeg = split < s.nfull ? (long long)split * s.klen
                                         : (long long)s.nfull * s.klen + (long long)(split - s.nfull) * s.klen2;
  long long kend = kbeg + (split < s.nfull ? s.klen : s.klen2);
  if (kend > s.K) kend = s.K;
  floatx16 acc[WM][WM];
  zero_acc<WM, WM>(acc);
  float rs[WM];
#pragma unroll
  for (int im = 0; im < WM; ++im) rs[im] = 0.f;
  int wave = threadIdx.x >> 6;
  const bool active = syrk_wave_active<WM>(I * BM, J * BM, dt, wave);
  unsigned store = 0xfu, rowmask = 0x3u;
  if (I != J) {
    mainloop<WM, WM, false>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB, acc, active, wave);
  } else if (WM == 2 && (I + 1) * BM <= dt) {
    // a whole diagonal 128-tile: all four waves share its ten blocks
    const DiagRole role = diag_tile_role(wave);
    wave = role.role;
    store = role.compute == 0xdu ? 0xfu : role.store;
    rowmask = role.compute == 0xdu ? 0x3u : (role.compute == 0x3u ? 0x1u : 0x2u);
    if (role.compute == 0xdu)
      mainloop_impl<WM, WM, true, true, Loader, Loader, 0xdu>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB,
                                                             acc, rs, true, wave);
    else if (role.compute == 0x3u)
      mainloop_impl<WM, WM, true, true, Loader, Loader, 0x3u>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB,
                                                             acc, rs, true, wave);
    else
      mainloop_impl<WM, WM, true, true, Loader, Loader, 0xcu>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB,
                                                             acc, rs, true, wave);
  } else {
    mainloop_rowsum<WM, WM, true>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB, acc, rs, active,
                                  wave);
  }
  const long long slot = (long long)s.ntile * (BM * BM) + (long long)s.tiles * BM;
  float *mine = ws + s.part_off + split * slot;
  if (s.ones && I == J)
    write_rowsums<WM>(rs, I, dt, s.d, s.direct, s.count, v.alpha, v.beta,
                      mine + (long long)s.ntile * (BM * BM), v.out, wave, rowmask);
  if (s.direct) {
    write_tile<WM>(acc, lds, I, J, dt, s.d, v.alpha, v.beta, v.out, wave, store);
    return;
  }
  float *out = mine + (long long)tile * (BM * BM);
  for_each_acc_masked<WM, WM>(acc, store, [&](int r, int c, float val) { out[r * BM + c] = val; }, wave);
}

// Macro-tile variant for 128-tile slab items with several k-slices: a workgroup
// of four teams (4 x 256 threads) computes the 2 x 2 tiles (2 MI + a, 2 MJ + b)
// of one k-slice from four operand panels staged once.  Tiles that share an
// operand panel only share it in L2 when they run within a microsecond of each
// other (an XCD's workgroups stream 3 MB through its 4 MB L2 per panel step), and
// as separate workgroups they do not: the grouped launch of 128-tiles fetched
// its inputs 2.2 - 2.5 times (hardware counters).  Here team t stages panel t
// (rows 2 MI, 2 MI + 1, 2 MJ, 2 MJ + 1; a macro-tile on the diagonal has only the
// first two) with the same loader code as a 256-thread workgroup, and team
// (a, b) multiplies tile (2 MI + a, 2 MJ + b) out of panels a and 2 + b.  Every
// barrier is reached by all 1024 threads: a team without a tile or a panel (above
// the diagonal, past a ragged end) skips the work, never the barrier.
// task = (item, macro-tile + nmacro * k-slice); partial tiles go to the same
// slots as syrk_group_kernel's, so the finish launch is shared.
constexpr int kMacroThreads = 4 * THREADS;
constexpr size_t kMacroLdsBytes = 4 * Panel<128>::kFloats * sizeof(float);

template <class Loader>
__global__ __launch_bounds__(kMacroThreads, 1) void syrk_macro_kernel(
    const GroupItemStatic *__restrict__ st, const GroupItemDyn *__restrict__ dy,
    const int2 *__restrict__ tasks, float *__restrict__ ws) {
  constexpr int BM = 128, WM = 2;
  constexpr int PF = Panel<BM>::kFloats;
  extern __shared__ float lds[];
  const int team = threadIdx.x >> 8;
  const int ta = team >> 1, tb = team & 1;
  const int wave = (threadIdx.x >> 6) & 3;
  const int lane = threadIdx.x & 63;
  const int2 task = tasks[blockIdx.x];
  if (task.x < 0) return;   // padding of a shorter XCD run
  const GroupItemStatic s = st[task.x];
  const GroupItemDyn v = dy[task.x];
  const int mtiles = (s.tiles + 1) / 2;
  const int nmacro = mtiles * (mtiles + 1) / 2;
  const int split = task.y / nmacro;
  int MI, MJ;
  tri_decode(task.y - split * nmacro, MI, MJ);
  const bool on_diag = MI == MJ;
  const int I = 2 * MI + ta, J = 2 * MJ + tb;
  const int dt = s.d - s.ones;
  // this team's tile and this team's panel
  const bool has_tile = I < s.tiles && J <= I;
  const int prow = (team < 2 ? 2 * MI : 2 * MJ) + (team & 1);
  const bool stages = prow < s.tiles && !(on_diag && team >= 2);
  float *mine_panel = lds + team * PF;
  const float *pa = lds + ta * PF;
  const float *pb = lds + (on_diag ? tb : 2 + tb) * PF;
  Loader ld = GroupLoader<Loader>::make(s, v.in);
  ld.init(nullptr, stages ? prow * BM : 0);
  const long long kbeg = split < s.nfull ? (long long)split * s.klen
                                         : (long long)s.nfull * s.klen + (long long)(split - s.nfull) * s.klen2;
  long long kend = kbeg + (split < s.nfull ? s.klen : s.klen2);
  if (kend > s.K) kend = s.K;
  floatx16 acc[WM][WM];
  zero_acc<WM, WM>(acc);
  float rs[WM] = {0.f, 0.f};
  const bool active = has_tile && syrk_wave_active<WM>(I * BM, J * BM, dt, wave);
  const bool sums = active && I == J;   // diagonal tile: also the row sums (the ones column)
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane & 31, lk = lane >> 5;
  typename Loader::Regs r;
  if (stages && kbeg < kend) ld.load(r, prow * BM, kbeg, kend);
  for (long long k0 = kbeg; k0 < kend; k0 += KT) {
    if (stages) ld.store(r, mine_panel);
    __syncthreads();
    if (stages && k0 + KT < kend) ld.load(r, prow * BM, k0 + KT, kend);
    if (active) {
#pragma unroll
      for (int kk = 0; kk < KT / 2; ++kk) {
        float a[WM], b[WM];
#pragma unroll
        for (int im = 0; im < WM; ++im)
          a[im] = fetch<BM, Loader::kKRow>(pa, (wm * WM + im) * 32 + lrow, 2 * kk + lk);
        if (sums) {
#pragma unroll
          for (int im = 0; im < WM; ++im) rs[im] += a[im];
        }
#pragma unroll
        for (int in = 0; in < WM; ++in)
          b[in] = fetch<BM, Loader::kKRow>(pb, (wn * WM + in) * 32 + lrow, 2 * kk + lk);
#pragma unroll
        for (int im = 0; im < WM; ++im)
#pragma unroll
          for (int in = 0; in < WM; ++in)
            acc[im][in] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[im], b[in], acc[im][in], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  if (!has_tile) return;
  const long long slot = (long long)s.ntile * (BM * BM) + (long long)s.tiles * BM;
  float *mine = ws + s.part_off + split * slot;
  if (s.ones && I == J)
    write_rowsums<WM>(rs, I, dt, s.d, 0, s.count, v.alpha, v.beta, mine + (long long)s.ntile * (BM * BM),
                      v.out, wave);
  float *out = mine + (long long)(I * (I + 1) / 2 + J) * (BM * BM);
  for_each_acc<WM, WM>(acc, [&](int rr, int cc, float val) { out[rr * BM + cc] = val; }, wave);
}

// task = (item, 64 x 64 block of the lower triangle); sums the item's k-slices
// in a fixed order and writes the block and its mirror image.
__global__ __launch_bounds__(256) void finish_group_kernel(const GroupItemStatic *__restrict__ st,
                                                           const GroupItemDyn *__restrict__ dy,
                                                           const int2 *__restrict__ tasks,
                                                           const float *__restrict__ ws) {
  __shared__ float tile[64][65];
  const int2 task = tasks[blockIdx.x];
  const GroupItemStatic s = st[task.x];
  const GroupItemDyn v = dy[task.x];
  int si, sj;
  tri_decode(task.y, si, sj);
  const int dt = s.d - s.ones, d = s.d;
  const int lc = threadIdx.x & 63, lr0 = threadIdx.x >> 6;
  const int bm = s.bm, per = bm / 64;   // 64-blocks per tile side
  const int I = si / per, J = sj / per;
  const int t = I * (I + 1) / 2 + J;
  const int r_in = (si - I * per) * 64, c_in = (sj - J * per) * 64;
  const long long tile_stride = (long long)bm * bm;
  const long long slot = (long long)s.ntile * tile_stride + (long long)s.tiles * bm;
  const float *p0 = ws + s.part_off + (long long)t * tile_stride + (long long)r_in * bm + c_in;
  float sum[16];
#pragma unroll
  for (int p = 0; p < 16; ++p) sum[p] = 0.f;
  // four slices' loads in flight at a time (the sums stay in slice order)
  int k = 0;
  for (; k + 4 <= s.nsplit; k += 4) {
    float x[4][16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float *pk = p0 + (k + q) * slot;
#pragma unroll
      for (int p = 0; p < 16; ++p) x[q][p] = pk[(lr0 + 4 * p) * bm + lc];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int p = 0; p < 16; ++p) sum[p] += x[q][p];
  }
  for (; k < s.nsplit; ++k) {
    const float *pk = p0 + k * slot;
#pragma unroll
    for (int p = 0; p < 16; ++p) sum[p] += pk[(lr0 + 4 * p) * bm + lc];
  }
  float *C = v.out;
  const float alpha = v.alpha, beta = v.beta;
  if (s.ones && si == sj && threadIdx.x < 64) {
    const int row = si * 64 + threadIdx.x;
    const float *v0 = ws + s.part_off + (long long)s.ntile * tile_stride + row;
    float a = 0.f;
    for (int k = 0; k < s.nsplit; ++k) a += v0[k * slot];
    if (row < dt) {
      float val = alpha * a;
      if (beta != 0.f) val += beta * C[(long long)(d - 1) * d + row];
      C[(long long)(d - 1) * d + row] = val;
      C[(long long)row * d + d - 1] = val;
    }
    if (row == 0) {
      float val = alpha * s.count;
      if (beta != 0.f) val += beta * C[(long long)(d - 1) * d + d - 1];
      C[(long long)(d - 1) * d + d - 1] = val;
    }
  }
#pragma unroll
  for (int p = 0; p < 16; ++p) {
    const int lr = lr0 + 4 * p;
    const int r = si * 64 + lr, c = sj * 64 + lc;
    float val = alpha * sum[p];
    if (beta != 0.f && r < dt && c < dt) val += beta * C[(long long)r * d + c];
    tile[lr][lc] = val;
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 16; ++p) {
    const int lr = lr0 + 4 * p;
    const int r = si * 64 + lr, c = sj * 64 + lc;
    if (si == sj) {
      if (r < dt && c < dt) C[(long long)r * d + c] = (lc <= lr) ? tile[lr][lc] : tile[lc][lr];
    } else {
      if (r < dt && c < dt) C[(long long)r * d + c] = tile[lr][lc];
      const int mr = sj * 64 + lr, mc = si * 64 + lc;
      if (mr < dt && mc < dt) C[(long long)mr * d + mc] = tile[lc][lr];
    }
  }
}

// Emits `natural` dealt so that each XCD (workgroup i of a launch runs on XCD
// i % 8) receives one contiguous run of it, the runs cut at equal shares of the
// total weight (the time a task takes: its reduction length, three quarters of it
// for a whole diagonal 128-tile); shorter runs are padded with empty tasks (item
// -1).  Measured on ResNet-50's grouped launch of 128-tiles before this: runs of
// equal task counts left the XCDs with 21 400 .. 25 500 panel steps of work, and the
// launch lasted as long as the slowest of them.
// `tail`: short tasks that every XCD runs last (its share of them, again a contiguous
// run by weight), so that a launch ends on short tasks everywhere.
void deal_to_xcds(std::vector<int2> &table, const std::vector<int2> &natural,
                  const std::vector<double> &weight, const std::vector<int2> &tail = {},
                  const std::vector<double> &tail_weight = {}) {
  std::vector<int2> queue[kXcds];
  auto deal = [&](const std::vector<int2> &list, const std::vector<double> &wts) {
    double total = 0.0;
    for (double w : wts) total += w;
    double cum = 0.0;
    for (size_t i = 0; i < list.size(); ++i) {
      // the run in which the middle of the task falls
      int x = total > 0.0 ? (int)((cum + 0.5 * wts[i]) * kXcds / total) : 0;
      if (x >= kXcds) x = kXcds - 1;
      queue[x].push_back(list[i]);
      cum += wts[i];
    }
  };
  deal(natural, weight);
  deal(tail, tail_weight);
  size_t longest = 0;
  for (const auto &q : queue) longest = std::max(longest, q.size());
  for (size_t p = 0; p < longest; ++p)
    for (size_t x = 0; x < (size_t)kXcds; ++x)
      table.push_back(p < queue[x].size() ? queue[x][p] : make_int2(-1, 0));
}

// {64-tiles, 128-tiles} x {slab float4, slab scalar, linear float4, linear scalar},
// then the macro-tile launches {slab float4, slab scalar}
constexpr int kGroupKinds = 10;
constexpr int kMacroKind0 = 8;

}  // namespace

struct kfac_cov_group {
  int count = 0;
  std::vector<GroupItemStatic> items;
  std::vector<GroupItemDyn> dyn;
  size_t ws_floats = 0;
  int task0[kGroupKinds] = {}, ntask[kGroupKinds] = {};
  int ftask0 = 0, nftask = 0;
  double kind_work[kGroupKinds] = {};   // matrix work of each launch (panels of a 64-tile)
  kfac::DevTable d_items, d_tasks;
  kfac::DevTableRing d_dyn;
  // The launches of a group are independent of each other.  Each ends with the GPU
  // draining (the last round of workgroups of a launch runs on a part of the CUs), so
  // the longest launch stays on the caller's stream and the others run beside it on a
  // stream of the group's own, filling each other's tails.
  hipStream_t side = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  bool capture_origin = false;   // see kfac_cov_group_set_capture_origin
  ~kfac_cov_group() {
    if (ev_fork) (void)hipEventDestroy(ev_fork);
    if (ev_join) (void)hipEventDestroy(ev_join);
    if (side) (void)hipStreamDestroy(side);
  }
};

extern "C" int kfac_cov_group_create(int count, const kfac_cov_item *items, kfac_cov_group_t *out) {
  KFAC_REQUIRE(out != nullptr, "group_out is null");
  *out = nullptr;
  KFAC_REQUIRE(count >= 0 && (count == 0 || items), "bad item list");
  auto *g = new (std::nothrow) kfac_cov_group;
  if (!g) return kfac::fail(KFAC_ENOMEM, "out of host memory");
  g->count = count;
  g->items.resize(count);
  g->dyn.resize(count);
  std::vector<long long> nk(count);
  std::vector<int> kind_of(count);
  double work[kGroupKinds] = {};   // per launch, in panels of a 64-tile
  for (int i = 0; i < count; ++i) {
    const kfac_cov_item &it = items[i];
    GroupItemStatic &s = g->items[i];
    memset(&s, 0, sizeof(s));
    auto bad = [&](const char *what) {
      delete g;
      return kfac::fail(KFAC_EINVAL, "item %d: %s", i, what);
    };
    if (it.kind != KFAC_COV_LINEAR && it.kind != KFAC_COV_SLAB) return bad("unknown kind");
    if (it.n <= 0 || it.c <= 0) return bad("bad shape");
    s.kind = it.kind;
    s.ones = it.append_ones ? 1 : 0;
    if (it.kind == KFAC_COV_LINEAR) {
      // x (n, c) row-major
      if ((long long)it.n * it.c >= 0x40000000LL) return bad("input too large");
      s.K = it.n;
      s.ld = (unsigned)it.c;
      s.rows_valid = it.c;
      s.vec = (it.aligned && it.c % 4 == 0) ? 1 : 0;
    } else {
      // (n, c, h, w) tensor; every sy-th line and sx-th pixel of it when subsampled
      if (it.h <= 0 || it.w <= 0 || it.sy <= 0 || it.sx <= 0) return bad("bad shape");
      if ((long long)it.n * it.c * it.h * it.w >= 0x40000000LL) return bad("input too large");
      const int ho = (it.h - 1) / it.sy + 1, wo = (it.w - 1) / it.sx + 1;
      const int hw = it.h * it.w;
      s.K = (long long)it.n * ho * wo;
      s.sample_stride = (unsigned)((long long)it.c * hw);
      s.row_stride = (unsigned)hw;
      s.L = (unsigned)(ho * wo);
      s.rows_valid = it.c;
      if (it.sy != 1 || it.sx != 1) {
        s.line_len = (unsigned)wo;
        s.line_stride = (unsigned)(it.sy * it.w);
        s.px_stride = (unsigned)it.sx;
        s.vec = 0;
      } else {
        s.px_stride = 1;
        s.vec = (it.aligned && hw % 4 == 0) ? 1 : 0;
      }
    }
    s.d = it.c + s.ones;
    s.count = (float)s.K;
    nk[i] = kfac::ceil_div<long long>(s.K, KT);
    // 128-tiles feed the matrix cores with half the LDS and load instructions of
    // 64-tiles and, in a grouped launch, need not be many to fill the GPU; 64-tiles for
    // narrow factors (padding) and for short reductions over many tiles (all output
    // traffic: smaller tiles spread the stores over more workgroups).
    // Option group_bm64_max is a tuning override.
    const int bm64_max = kfac::option_int(kfac::kOptGroupBm64Max, 160);
    s.bm = (it.c <= bm64_max || nk[i] <= 4) ? 64 : 128;
    s.tiles = kfac::ceil_div(it.c, s.bm);
    s.ntile = s.tiles * (s.tiles + 1) / 2;
    kind_of[i] = (s.bm == 64 ? 0 : 4) + (s.kind == KFAC_COV_SLAB ? 0 : 2) + (s.vec ? 0 : 1);
    // Slabs of several 128-tiles with a reduction long enough to cut into slices can take
    // the macro-tile kernel, option group_macro = 1.  Off by default: on ResNet-50 it cuts the
    // HBM fetch of the grouped launches by 30 % (the launches' total traffic from 1.77 to
    // 1.58 times the algorithmic bytes) at the same kernel time, but its workgroups own a
    // CU each, so they need more and shorter k-slices to balance, and the extra partial
    // tiles make the finish launch 70 us longer: 1 % of a step.
    const bool macro_on = kfac::option_int(kfac::kOptGroupMacro, 0) != 0;
    if (macro_on && s.bm == 128 && s.kind == KFAC_COV_SLAB && s.tiles >= 2 && nk[i] >= 16) {
      kind_of[i] = kMacroKind0 + (s.vec ? 0 : 1);
      const int mt = (s.tiles + 1) / 2;
      work[kind_of[i]] += (double)(mt * (mt + 1) / 2) * (double)nk[i];
    } else {
      work[kind_of[i]] += (double)s.ntile * (double)nk[i] * (s.bm == 64 ? 1.0 : 4.0);
    }
  }
  // k-slices: every launch (one per loader kind and tile size) is cut into workgroups
  // of about equal length (a panel of a 128-tile counts four times a panel of a
  // 64-tile), ~2300 of them when the work allows it, none shorter than 32 panel units
  // (unless the whole reduction is) and at most 256 per factor
  double per_wg[kGroupKinds];
  for (int k = 0; k < kGroupKinds; ++k) {
    per_wg[k] = work[k] / 2304.0;
    if (per_wg[k] < 32.0) per_wg[k] = 32.0;
    {   // tuning override: panel units per workgroup
      const double v = kfac::option_value(kfac::kOptGroupPanels, 0.0);
      if (v >= 1.0) per_wg[k] = v;
    }
  }
  // a macro-tile workgroup has a CU to itself: ~6 rounds of 256 (measured: fewer, longer
  // workgroups balance worse, more gain nothing), at least 8 panels each
  // (work counted in panels per macro-tile; option group_macro_tasks is a tuning override)
  for (int k = kMacroKind0; k < kGroupKinds; ++k) {
    const double ntasks = std::max(1.0, kfac::option_value(kfac::kOptGroupMacroTasks, 1536.0));
    per_wg[k] = std::max(8.0, work[k] / ntasks);
  }
  // A launch of several rounds of workgroups ends with the GPU draining: the last
  // tasks of every XCD start one after the other and all take a full task's time
  // (measured on ResNet-50's launch of 128-tiles: 2.4 of 3 workgroup slots occupied on
  // average, the last 300-500 us of 1.9 ms on a half-empty GPU).  So the last third of
  // every factor's reduction is cut into slices of half the length, and those tasks go
  // to the end of every XCD's run.  Option group_graded = 0 switches this off.
  bool graded_on = true;
  int graded_part = 3;   // the last 1 / graded_part of a reduction is halved
  if (kfac::option_is_set(kfac::kOptGroupGraded)) {   // tuning override: 0 = off, n >= 2: the last n-th
    const int v = kfac::option_int(kfac::kOptGroupGraded, 1);
    graded_on = v != 0;
    if (v >= 2) graded_part = v;
  }
  double ntasks_kind[kGroupKinds] = {};
  for (int i = 0; i < count; ++i) {
    const GroupItemStatic &s = g->items[i];
    const int k = kind_of[i];
    if (k < kMacroKind0)
      ntasks_kind[k] += (double)s.ntile * (double)nk[i] * (s.bm == 64 ? 1.0 : 4.0) / per_wg[k];
  }
  size_t off = 0;
  std::vector<int2> natural[kGroupKinds], tail[kGroupKinds], fin;
  std::vector<double> weight[kGroupKinds], tail_weight[kGroupKinds];
  for (int i = 0; i < count; ++i) {
    GroupItemStatic &s = g->items[i];
    const bool macro = kind_of[i] >= kMacroKind0;
    long long ns = (long long)((double)nk[i] * (macro ? 1.0 : s.bm == 64 ? 1.0 : 4.0) / per_wg[kind_of[i]] + 0.5);
    if (ns < 1) ns = 1;
    if (ns > 256) ns = 256;
    if (ns > nk[i]) ns = nk[i];
    const long long per = kfac::ceil_div(nk[i], ns);
    s.nsplit = (int)kfac::ceil_div(nk[i], per);
    s.klen = per * KT;
    s.nfull = s.nsplit;
    s.klen2 = s.klen;
    // graded: launches of at least two rounds (768 workgroups each), slices of at least 16 panels
    if (graded_on && !macro && ntasks_kind[kind_of[i]] >= 1536.0 && per >= 16 && s.nsplit >= graded_part) {
      const int nhalved = s.nsplit / graded_part;       // full slices that become two half slices each
      const long long per2 = kfac::ceil_div<long long>(per, 2);
      s.nfull = s.nsplit - nhalved;
      const long long rest = nk[i] - (long long)s.nfull * per;   // panels left for the half slices
      s.klen2 = per2 * KT;
      s.nsplit = s.nfull + (int)kfac::ceil_div(rest, per2);
    }
    s.direct = (s.nsplit == 1 && !macro) ? 1 : 0;   // the macro-tile kernel always writes partial tiles
    s.part_off = (long long)off;
    const size_t slot = (size_t)s.ntile * s.bm * s.bm + (size_t)s.tiles * s.bm;
    if (!s.direct) off += (size_t)s.nsplit * slot;
    const int mt = (s.tiles + 1) / 2;
    const int per_slice = macro ? mt * (mt + 1) / 2 : s.ntile;
    for (int w = 0; w < per_slice * s.nsplit; ++w) {
      // the task's panel steps; a whole diagonal 128-tile takes three quarters of the time
      const int split = w / per_slice, tile = w - split * per_slice;
      const bool half = split >= s.nfull;
      const long long per2 = s.klen2 / KT;
      const long long k0 = half ? (long long)s.nfull * per + (long long)(split - s.nfull) * per2 : (long long)split * per;
      const long long k1 = std::min<long long>(k0 + (half ? per2 : per), nk[i]);
      (half ? tail : natural)[kind_of[i]].push_back(make_int2(i, w));
      std::vector<double> &wlist = (half ? tail_weight : weight)[kind_of[i]];
      double wt = (double)(k1 - k0);
      if (!macro && s.bm == 128) {
        int I = (int)((std::sqrt(8.0 * tile + 1.0) - 1.0) * 0.5);
        while (I * (I + 1) / 2 > tile) --I;
        while ((I + 1) * (I + 2) / 2 <= tile) ++I;
        const int J = tile - I * (I + 1) / 2;
        if (I == J && (I + 1) * 128 <= items[i].c) wt *= 0.75;
      }
      wlist.push_back(wt);
    }
    if (!s.direct) {
      const int sub = kfac::ceil_div(items[i].c, 64);
      for (int b = 0; b < sub * (sub + 1) / 2; ++b) fin.push_back(make_int2(i, b));
    }
  }
  g->ws_floats = off;
  for (int k = 0; k < kGroupKinds; ++k) g->kind_work[k] = work[k];
  std::vector<int2> tasks;
  for (int k = 0; k < kGroupKinds; ++k) {
    g->task0[k] = (int)tasks.size();
    deal_to_xcds(tasks, natural[k], weight[k], tail[k], tail_weight[k]);
    g->ntask[k] = (int)tasks.size() - g->task0[k];
  }
  g->ftask0 = (int)tasks.size();
  g->nftask = (int)fin.size();
  tasks.insert(tasks.end(), fin.begin(), fin.end());
  if (tasks.empty()) tasks.push_back(make_int2(0, 0));
  int rc = g->d_items.set_sync(g->items.data(), sizeof(GroupItemStatic) * (size_t)count);
  if (rc == KFAC_OK) rc = g->d_tasks.set_sync(tasks.data(), sizeof(int2) * tasks.size());
  if (rc != KFAC_OK) {
    delete g;
    return rc;
  }
  *out = g;
  return KFAC_OK;
}

extern "C" size_t kfac_cov_group_workspace_bytes(kfac_cov_group_t group) {
  return group ? group->ws_floats * sizeof(float) + 256 : 0;
}

extern "C" int kfac_cov_group_destroy(kfac_cov_group_t group) {
  delete group;
  return KFAC_OK;
}

extern "C" int kfac_cov_group_set_capture_origin(kfac_cov_group_t group, int is_origin) {
  KFAC_REQUIRE(group != nullptr, "group is null");
  group->capture_origin = is_origin != 0;
  return KFAC_OK;
}

extern "C" int kfac_cov_group_run_f32(kfac_cov_group_t group, const float *const *inputs,
                                      float *const *outputs, const float *alpha,
                                      const float *beta, void *ws, size_t ws_bytes, void *stream) {
  KFAC_REQUIRE(group != nullptr, "group is null");
  const int count = group->count;
  if (count == 0) return KFAC_OK;
  KFAC_REQUIRE(inputs && outputs && alpha && beta, "null table");
  if (ws == nullptr || ws_bytes < kfac_cov_group_workspace_bytes(group))
    return kfac::fail(KFAC_ENOMEM, "covariance group workspace too small: %zu < %zu bytes", ws_bytes,
                      kfac_cov_group_workspace_bytes(group));
  for (int i = 0; i < count; ++i) {
    KFAC_REQUIRE(inputs[i] && outputs[i], "item %d: null pointer", i);
    KFAC_REQUIRE(!group->items[i].vec || reinterpret_cast<uintptr_t>(inputs[i]) % 16 == 0,
                 "item %d was declared 16-byte aligned and is not", i);
    group->dyn[i] = GroupItemDyn{inputs[i], outputs[i], alpha[i], beta[i]};
  }
  hipStream_t s = kfac::as_stream(stream);
  const void *dyn_dev = nullptr;
  if (int rc = group->d_dyn.set(group->dyn.data(), sizeof(GroupItemDyn) * (size_t)count, s, &dyn_dev))
    return rc;
  float *base = reinterpret_cast<float *>((reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255);
  const GroupItemStatic *st = group->d_items.as<const GroupItemStatic>();
  const GroupItemDyn *dy = static_cast<const GroupItemDyn *>(dyn_dev);
  const int2 *tasks = group->d_tasks.as<const int2>();
  using Kern = void (*)(const GroupItemStatic *, const GroupItemDyn *, const int2 *, float *);
  static const Kern kerns[kMacroKind0] = {
      syrk_group_kernel<1, LoaderKC<64, true>>,   syrk_group_kernel<1, LoaderKC<64, false>>,
      syrk_group_kernel<1, LoaderKS<64, true>>,   syrk_group_kernel<1, LoaderKS<64, false>>,
      syrk_group_kernel<2, LoaderKC<128, true>>,  syrk_group_kernel<2, LoaderKC<128, false>>,
      syrk_group_kernel<2, LoaderKS<128, true>>,  syrk_group_kernel<2, LoaderKS<128, false>>};
  // The launch with the most work stays on `s`, the others go to the group's side stream
  // (not while launches are being timed one by one, not in host-only mode, and under stream
  // capture only when the caller has declared `s` the capture's origin: a fork of a forked
  // stream has crashed the runtime).
  int nlaunch = 0, longest = -1;
  for (int k = 0; k < kGroupKinds; ++k) {
    if (group->ntask[k] == 0) continue;
    ++nlaunch;
    if (longest < 0 || group->kind_work[k] > group->kind_work[longest]) longest = k;
  }
  bool fork = nlaunch >= 2 && kfac::option_int(kfac::kOptGroupSideStream, 1) != 0 && !kfac::timing_on() &&
              !kfac::host_only();
  if (fork && !group->capture_origin) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cs) != hipSuccess) {
      (void)hipGetLastError();
      fork = false;
    } else if (cs != hipStreamCaptureStatusNone) {
      fork = false;
    }
  }
  if (fork && !group->side) {
    KFAC_HIP_CHECK(hipStreamCreateWithFlags(&group->side, hipStreamNonBlocking));
    KFAC_HIP_CHECK(hipEventCreateWithFlags(&group->ev_fork, hipEventDisableTiming));
    KFAC_HIP_CHECK(hipEventCreateWithFlags(&group->ev_join, hipEventDisableTiming));
  }
  if (fork) {
    KFAC_HIP_CHECK(hipEventRecord(group->ev_fork, s));
    KFAC_HIP_CHECK(hipStreamWaitEvent(group->side, group->ev_fork, 0));
  }
  auto stream_of = [&](int k) { return fork && k != longest ? group->side : s; };
  // (the longest first: its workgroups are placed before the others fill in)
  if (longest >= 0 && longest < kMacroKind0) {
    kfac::TimedLaunch timed(KFAC_TIMED_SYRK, s);
    KFAC_LAUNCH(kerns[longest], dim3(group->ntask[longest]), dim3(THREADS), 0, s, st, dy,
                tasks + group->task0[longest], base);
  }
  for (int k = 0; k < kMacroKind0; ++k) {
    if (group->ntask[k] == 0 || k == longest) continue;
    kfac::TimedLaunch timed(KFAC_TIMED_SYRK, stream_of(k));
    KFAC_LAUNCH(kerns[k], dim3(group->ntask[k]), dim3(THREADS), 0, stream_of(k), st, dy,
                       tasks + group->task0[k], base);
  }
  static const Kern macro_kerns[2] = {syrk_macro_kernel<LoaderKC<128, true>>,
                                      syrk_macro_kernel<LoaderKC<128, false>>};
  static std::once_flag macro_attr;
  static hipError_t macro_attr_rc = hipSuccess;
  std::call_once(macro_attr, [&] {
    if (kfac::host_only()) return;
    for (Kern f : macro_kerns) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(f),
                                               hipFuncAttributeMaxDynamicSharedMemorySize,
                                               (int)kMacroLdsBytes);
      if (e != hipSuccess) macro_attr_rc = e;
    }
  });
  KFAC_HIP_CHECK(macro_attr_rc);
  for (int k = kMacroKind0; k < kGroupKinds; ++k) {
    if (group->ntask[k] == 0) continue;
    kfac::TimedLaunch timed(KFAC_TIMED_SYRK, stream_of(k));
    KFAC_LAUNCH(macro_kerns[k - kMacroKind0], dim3(group->ntask[k]), dim3(kMacroThreads),
                       kMacroLdsBytes, stream_of(k), st, dy, tasks + group->task0[k], base);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  if (fork) {
    KFAC_HIP_CHECK(hipEventRecord(group->ev_join, group->side));
    KFAC_HIP_CHECK(hipStreamWaitEvent(s, group->ev_join, 0));
  }
  if (group->nftask > 0) {
    kfac::TimedLaunch timed(KFAC_TIMED_COV_AUX, s);
    KFAC_LAUNCH(finish_group_kernel, dim3(group->nftask), dim3(256), 0, s, st, dy,
                       tasks + group->ftask0, base);
    KFAC_HIP_CHECK(hipGetLastError());
  }
  return KFAC_OK;
}
