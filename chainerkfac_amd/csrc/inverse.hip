// Batched damped inverse of SPD Kronecker factors: blocked Cholesky (potrf)
// followed by the triangular inverse and L^-T L^-1 (potri), FP32 MFMA.
//
// All matrices of a batch advance together.  Each is copied (lower tiles
// only) into a zero/identity padded workspace of NB x NB tiles (NB = 128) and
// swept once, block column k = 0 .. T-1, with three launches per step that
// cover every matrix that still has a block column k:
//
//   diag(k)    one workgroup per matrix: Cholesky of the updated diagonal
//              tile, its inverse W = L_kk^-1 and Z = W^T W (= A_kk^-1), all
//              inside LDS on 32x32 MFMA blocks.
//   panel(k)   L(m,k) = A(m,k) W^T                     (m > k)   "trsm"
//              X^T(k,m) = -Z A(m,k)^T                  (m > k)   trtri seed
//              U(n,k) = X^T(n,k) W^T                   (n < k)   trtri row finish
//   update(k)  A(m,n) -= L(m,k) L(n,k)^T               (k < n <= m)  potrf
//              X^T(n,m) -= U(n,k) L(m,k)^T             (n < k < m)   trtri
//
// The strictly lower tiles hold L, the upper tiles hold U = L^-T (the running
// right-looking triangular inverse, stored transposed), so potrf and trtri
// share one sweep and every product is a k-contiguous "NT" tile GEMM.  A final
// launch forms  out(i,j) = sum_{k >= i} U(i,k) U(j,k)^T  (lauum) and writes the
// full symmetric inverse.  Tasks of a launch are found with one wave-uniform
// binary search over per-step cumulative tables built once per plan.
//
// Replaces chainerkfac/optimizers/cholesky_inverse.py:16-102 (potrf + potrs
// against the identity, one matrix at a time).
#include <algorithm>
#include <numeric>

#include "common.h"
#include "mma_core.h"

namespace {

using namespace kfac::mma;

constexpr int NB = 128;
constexpr int SB = 32;
constexpr int LS = NB + 1;  // LDS row stride of the diagonal-tile kernel

struct InvTables {
  const float *const *in;    // [count] sorted slot -> input matrix
  float *const *out;         // [count]
  const int *orig;           // [count] slot -> caller index
  const int *dim;            // [count]
  const int *nt;             // [count] tiles per side
  const long long *ws_off;   // [count] float offset of the padded matrix
  const int *tile_cs;        // [count+1] cumulative lower-tile counts
  const int *panel_cs;       // [count+1] cumulative (nt-1)
  const int *update_cs;      // flat per-step cumulative update-task counts
  float *ws;                 // padded matrices
  float *side;               // per slot: W (NB*NB) then Z (NB*NB)
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

__device__ __forceinline__ void tri_decode(int t, int &I, int &J) {
  int r = (int)((sqrtf(8.f * (float)t + 1.f) - 1.f) * 0.5f);
  while (r * (r + 1) / 2 > t) --r;
  while ((r + 1) * (r + 2) / 2 <= t) ++r;
  I = r;
  J = t - r * (r + 1) / 2;
}

// ---------------------------------------------------------------------------
// copy-in: lower tiles of in -> padded workspace (identity on the padding)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void copy_in_kernel(InvTables tb, int count) {
  const int s = find_slot(tb.tile_cs, count, blockIdx.x);
  int I, J;
  tri_decode(blockIdx.x - tb.tile_cs[s], I, J);
  const int d = tb.dim[s];
  const long long ld = (long long)tb.nt[s] * NB;
  const float *__restrict__ src = tb.in[s];
  float *__restrict__ dst = tb.ws + tb.ws_off[s];
  const int c4 = (threadIdx.x & 31) * 4;
  const int r0 = threadIdx.x >> 5;
#pragma unroll 4
  for (int p = 0; p < NB / 8; ++p) {
    const int r = I * NB + r0 + 8 * p;
    const int c = J * NB + c4;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int ce = c + e;
      float x = (r == ce) ? 1.f : 0.f;
      if (r < d && ce < d) x = src[(long long)r * d + ce];
      v[e] = x;
    }
    *reinterpret_cast<float4 *>(dst + (long long)r * ld + c) = make_float4(v[0], v[1], v[2], v[3]);
  }
}

// ---------------------------------------------------------------------------
// diagonal tile: Cholesky + inverse + Z inside LDS
// ---------------------------------------------------------------------------

// acc += A(32 x K) * B^T, A at a[row*LS + k]; B at b[row*LS + k] or, when BT,
// at b[k*LS + row].
template <bool BT>
__device__ __forceinline__ floatx16 wave_gemm(const float *a, const float *b, int K,
                                              floatx16 acc) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  for (int k = 0; k < K; k += 2) {
    const float av = a[r * LS + k + h];
    const float bv = BT ? b[(k + h) * LS + r] : b[r * LS + k + h];
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
  }
  return acc;
}

template <class F>
__device__ __forceinline__ void wave_visit(const floatx16 &acc, F f) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int v = 0; v < 16; ++v) f(8 * (v >> 2) + 4 * (lane >> 5) + (v & 3), lane & 31, acc[v]);
}

__device__ __forceinline__ float lane_bcast(float x, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), lane));
}

// Wave 0: factor the 32x32 block at S[b0.., b0..] (lower) in registers, then
// overwrite the block with U32 = (L32^-1)^T (upper triangular, zeros below).
// Returns 0 or 1 + the local index of the first non-positive pivot.
__device__ __forceinline__ int chol_inv_32(float *S, int b0) {
  const int lane = threadIdx.x & 63;
  const int i = lane & 31;
  float a[SB];
#pragma unroll
  for (int c = 0; c < SB; ++c) a[c] = S[(b0 + i) * LS + b0 + c];
  int bad = 0;
#pragma unroll
  for (int j = 0; j < SB; ++j) {
    const float piv = lane_bcast(a[j], j);
    if (!(piv > 0.f) && bad == 0) bad = j + 1;
    const float root = sqrtf(piv);
    const float rinv = 1.0f / root;
    a[j] = (i == j) ? root : a[j] * rinv;
#pragma unroll
    for (int c = j + 1; c < SB; ++c) {
      const float lcj = lane_bcast(a[j], c);
      a[c] -= a[j] * lcj;
    }
  }
  // lane c solves L w = e_c: w[i] = (delta_ic - sum_{k<i} l_ik w_k) / l_ii
  float w[SB];
#pragma unroll
  for (int r = 0; r < SB; ++r) {
    float s = (r == i) ? 1.f : 0.f;
#pragma unroll
    for (int k = 0; k < r; ++k) s -= lane_bcast(a[k], r) * w[k];
    w[r] = s / lane_bcast(a[r], r);
  }
  // lane c holds column c of W = row c of U; entries with r < c are exact zeros
  if (lane < SB) {
#pragma unroll
    for (int r = 0; r < SB; ++r) S[(b0 + i) * LS + b0 + r] = w[r];
  }
  return bad;
}

__global__ __launch_bounds__(256) void diag_kernel(InvTables tb, int k) {
  extern __shared__ float smem[];
  float *S = smem;                      // NB x LS working tile
  float *scratch = smem + NB * LS;      // 4 waves x SB x LS
  const int s = blockIdx.x;
  const int d = tb.dim[s];
  const long long ld = (long long)tb.nt[s] * NB;
  float *tile = tb.ws + tb.ws_off[s] + (long long)k * NB * ld + (long long)k * NB;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  {
    const int c4 = (threadIdx.x & 31) * 4, r0 = threadIdx.x >> 5;
#pragma unroll 4
    for (int p = 0; p < NB / 8; ++p) {
      const int r = r0 + 8 * p;
      const float4 v = *reinterpret_cast<const float4 *>(tile + (long long)r * ld + c4);
      S[r * LS + c4 + 0] = v.x;
      S[r * LS + c4 + 1] = v.y;
      S[r * LS + c4 + 2] = v.z;
      S[r * LS + c4 + 3] = v.w;
    }
  }
  __syncthreads();
  floatx16 zero;
#pragma unroll
  for (int v = 0; v < 16; ++v) zero[v] = 0.f;

  // ---- potrf on 32x32 blocks
  for (int jb = 0; jb < NB / SB; ++jb) {
    if (wave == 0) {
      const int bad = chol_inv_32(S, jb * SB);
      if (lane == 0) {
        int *pinfo = &tb.info[tb.orig[s]];
        if (k == 0 && jb == 0) *pinfo = 0;
        const int col = k * NB + jb * SB + bad - 1;
        if (bad && col < d && *pinfo == 0) *pinfo = col + 1;
      }
    }
    __syncthreads();
    // panel: L(ib,jb) = A(ib,jb) U32(jb), one block per wave
    for (int ib = jb + 1 + wave; ib < NB / SB; ib += 4) {
      float *blk = S + (ib * SB) * LS + jb * SB;
      const floatx16 acc = wave_gemm<true>(blk, S + (jb * SB) * LS + jb * SB, SB, zero);
      wave_visit(acc, [&](int r, int c, float v) { blk[r * LS + c] = v; });
    }
    __syncthreads();
    // trailing update: A(ib,cb) -= L(ib,jb) L(cb,jb)^T for jb < cb <= ib
    const int rem = NB / SB - jb - 1;
    for (int t = wave; t < rem * (rem + 1) / 2; t += 4) {
      int a, b;
      tri_decode(t, a, b);
      const int ib = jb + 1 + a, cb = jb + 1 + b;
      float *blk = S + (ib * SB) * LS + cb * SB;
      const floatx16 acc = wave_gemm<false>(S + (ib * SB) * LS + jb * SB,
                                            S + (cb * SB) * LS + jb * SB, SB, zero);
      wave_visit(acc, [&](int r, int c, float v) { blk[r * LS + c] -= v; });
    }
    __syncthreads();
  }

  // ---- trtri: U(jb,ib) = -[sum_kb U(jb,kb) L(ib,kb)^T] U32(ib), by distance
  float *P = scratch + wave * SB * LS;
  for (int dd = 1; dd < NB / SB; ++dd) {
    for (int jb = wave; jb + dd < NB / SB; jb += 4) {
      const int ib = jb + dd;
      const floatx16 p = wave_gemm<false>(S + (jb * SB) * LS + jb * SB,
                                          S + (ib * SB) * LS + jb * SB, dd * SB, zero);
      wave_visit(p, [&](int r, int c, float v) { P[r * LS + c] = v; });
      // the same wave re-reads P: LDS accesses of one wave execute in order
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      const floatx16 u = wave_gemm<true>(P, S + (ib * SB) * LS + ib * SB, SB, zero);
      float *blk = S + (jb * SB) * LS + ib * SB;
      wave_visit(u, [&](int r, int c, float v) { blk[r * LS + c] = -v; });
    }
    __syncthreads();
  }

  // ---- outputs
  float *Wg = tb.side + (long long)s * 2 * NB * NB;
  float *Zg = Wg + NB * NB;
  {
    // U -> diagonal tile of the workspace (zeros below the diagonal);
    // W = U^T -> side buffer (zeros above the diagonal)
    const int c = threadIdx.x & 127;
    const int r0 = threadIdx.x >> 7;
    for (int p = 0; p < NB / 2; ++p) {
      const int r = r0 + 2 * p;
      const bool up = (c / SB > r / SB) || (c / SB == r / SB && c >= r);
      tile[(long long)r * ld + c] = up ? S[r * LS + c] : 0.f;
      const bool lo = (r / SB > c / SB) || (c / SB == r / SB && r >= c);
      Wg[r * NB + c] = lo ? S[c * LS + r] : 0.f;
    }
  }
  // Z = U U^T on lower blocks, mirrored
  for (int t = wave; t < 10; t += 4) {
    int bi, bj;
    tri_decode(t, bi, bj);
    const floatx16 z = wave_gemm<false>(S + (bi * SB) * LS + bi * SB,
                                        S + (bj * SB) * LS + bi * SB, NB - bi * SB, zero);
    wave_visit(z, [&](int r, int c, float v) {
      Zg[(bi * SB + r) * NB + bj * SB + c] = v;
      if (bi != bj) Zg[(bj * SB + c) * NB + bi * SB + r] = v;
    });
  }
}

// ---------------------------------------------------------------------------
// panel and update: 128x128x128 tile products through the shared main loop
// ---------------------------------------------------------------------------
__device__ __forceinline__ LoaderKC<NB, true> tile_loader(const float *base, long long ld) {
  LoaderKC<NB, true> l;
  l.base = base;
  l.sample_stride = 0;
  l.row_stride = (unsigned)ld;
  l.L = NB;
  l.rows_valid = NB;
  l.ones_row = -1;
  l.init(nullptr, 0);
  return l;
}

__global__ __launch_bounds__(THREADS, 2) void panel_kernel(InvTables tb, int k, int nactive) {
  __shared__ float ldsA[Panel<NB>::kFloats];
  __shared__ float ldsB[Panel<NB>::kFloats];
  const int s = find_slot(tb.panel_cs, nactive, blockIdx.x);
  const int local = blockIdx.x - tb.panel_cs[s];
  const int T = tb.nt[s];
  const long long ld = (long long)T * NB;
  float *M = tb.ws + tb.ws_off[s];
  const float *Wg = tb.side + (long long)s * 2 * NB * NB;
  const float *Zg = Wg + NB * NB;
  const int r = T - k - 1;
  floatx16 acc[2][2];
  zero_acc<2, 2>(acc);
  if (local < r) {
    const int m = k + 1 + local;
    float *Amk = M + (long long)m * NB * ld + (long long)k * NB;   // lower slot (m,k)
    float *Xkm = M + (long long)k * NB * ld + (long long)m * NB;   // upper slot (k,m)
    // X^T(k,m) = -Z A(m,k)^T
    mainloop<2, 2, false>(tile_loader(Zg, NB), tile_loader(Amk, ld), 0, 0, 0, NB, ldsA, ldsB, acc);
    for_each_acc<2, 2>(acc, [&](int rr, int cc, float v) { Xkm[(long long)rr * ld + cc] = -v; });
    // L(m,k) = A(m,k) W^T, in place
    zero_acc<2, 2>(acc);
    mainloop<2, 2, false>(tile_loader(Amk, ld), tile_loader(Wg, NB), 0, 0, 0, NB, ldsA, ldsB, acc);
    for_each_acc<2, 2>(acc, [&](int rr, int cc, float v) { Amk[(long long)rr * ld + cc] = v; });
  } else {
    const int n = local - r;
    float *Unk = M + (long long)n * NB * ld + (long long)k * NB;   // upper slot (n,k)
    // U(n,k) = X^T(n,k) W^T, in place
    mainloop<2, 2, false>(tile_loader(Unk, ld), tile_loader(Wg, NB), 0, 0, 0, NB, ldsA, ldsB, acc);
    for_each_acc<2, 2>(acc, [&](int rr, int cc, float v) { Unk[(long long)rr * ld + cc] = v; });
  }
}

__global__ __launch_bounds__(THREADS, 2) void update_kernel(InvTables tb, int k, int nactive,
                                                            int cs_off) {
  __shared__ float ldsA[Panel<NB>::kFloats];
  __shared__ float ldsB[Panel<NB>::kFloats];
  const int *cs = tb.update_cs + cs_off;
  const int s = find_slot(cs, nactive, blockIdx.x);
  const int local = blockIdx.x - cs[s];
  const int T = tb.nt[s];
  const long long ld = (long long)T * NB;
  float *M = tb.ws + tb.ws_off[s];
  const int r = T - k - 1;
  const int ntri = r * (r + 1) / 2;
  floatx16 acc[2][2];
  zero_acc<2, 2>(acc);
  float *C;
  if (local < ntri) {
    int a, b;
    tri_decode(local, a, b);
    const int m = k + 1 + a, n = k + 1 + b;
    const float *Lm = M + (long long)m * NB * ld + (long long)k * NB;
    const float *Ln = M + (long long)n * NB * ld + (long long)k * NB;
    C = M + (long long)m * NB * ld + (long long)n * NB;
    if (m == n)
      mainloop<2, 2, true>(tile_loader(Lm, ld), tile_loader(Ln, ld), 0, 0, 0, NB, ldsA, ldsB, acc);
    else
      mainloop<2, 2, false>(tile_loader(Lm, ld), tile_loader(Ln, ld), 0, 0, 0, NB, ldsA, ldsB, acc);
  } else {
    const int q = local - ntri;
    const int a = q / k, n = q - a * k;
    const int m = k + 1 + a;
    const float *Unk = M + (long long)n * NB * ld + (long long)k * NB;
    const float *Lm = M + (long long)m * NB * ld + (long long)k * NB;
    C = M + (long long)n * NB * ld + (long long)m * NB;  // upper slot (n,m)
    mainloop<2, 2, false>(tile_loader(Unk, ld), tile_loader(Lm, ld), 0, 0, 0, NB, ldsA, ldsB, acc);
  }
  for_each_acc<2, 2>(acc, [&](int rr, int cc, float v) { C[(long long)rr * ld + cc] -= v; });
}

// out(i,j) = sum_{k >= i} U(i,k) U(j,k)^T for i >= j, written with its mirror.
__global__ __launch_bounds__(THREADS, 2) void lauum_kernel(InvTables tb, int count) {
  __shared__ float ldsA[Panel<NB>::kFloats];
  __shared__ float ldsB[Panel<NB>::kFloats];
  const int s = find_slot(tb.tile_cs, count, blockIdx.x);
  int I, J;
  tri_decode(blockIdx.x - tb.tile_cs[s], I, J);
  const int T = tb.nt[s];
  const int d = tb.dim[s];
  const long long ld = (long long)T * NB;
  const float *M = tb.ws + tb.ws_off[s];
  const int K = (T - I) * NB;
  LoaderKC<NB, true> la = tile_loader(M + (long long)I * NB * ld + (long long)I * NB, ld);
  LoaderKC<NB, true> lb = tile_loader(M + (long long)J * NB * ld + (long long)I * NB, ld);
  la.L = K;
  lb.L = K;
  floatx16 acc[2][2];
  zero_acc<2, 2>(acc);
  if (I == J)
    mainloop<2, 2, true>(la, lb, 0, 0, 0, K, ldsA, ldsB, acc);
  else
    mainloop<2, 2, false>(la, lb, 0, 0, 0, K, ldsA, ldsB, acc);
  float *__restrict__ out = tb.out[s];
  for_each_acc<2, 2>(acc, [&](int rr, int cc, float v) {
    const int r = I * NB + rr, c = J * NB + cc;
    if (r < d && c < d) {
      out[(long long)r * d + c] = v;
      if (I != J) out[(long long)c * d + r] = v;
    }
  });
}

constexpr size_t kDiagLds = (size_t)(NB * LS + 4 * SB * LS) * sizeof(float);

}  // namespace

struct kfac_inverse_plan {
  int count = 0;
  int max_t = 0;
  std::vector<int> order;          // slot -> caller index
  std::vector<int> nt;             // per slot
  std::vector<int> nactive;        // per step
  std::vector<int> panel_total;    // per step
  std::vector<int> update_total;   // per step
  std::vector<int> update_off;     // per step offset into update_cs
  int total_tiles = 0;
  size_t ws_floats = 0;            // padded matrices
  size_t side_floats = 0;
  std::vector<const void *> in_sorted, out_sorted;
  kfac::DevTable d_in, d_out, d_orig, d_dim, d_nt, d_off, d_tile, d_panel, d_update;
  bool attr_set = false;
};

extern "C" int kfac_inverse_plan_create(int count, const int32_t *dims,
                                        kfac_inverse_plan_t *plan_out) {
  KFAC_REQUIRE(plan_out != nullptr, "plan_out is null");
  *plan_out = nullptr;
  KFAC_REQUIRE(count >= 0, "count < 0");
  KFAC_REQUIRE(count == 0 || dims != nullptr, "dims is null");
  for (int i = 0; i < count; ++i)
    KFAC_REQUIRE(dims[i] > 0 && dims[i] <= 46340, "matrix %d: bad dimension %d", i, dims[i]);
  auto *p = new (std::nothrow) kfac_inverse_plan;
  if (!p) return kfac::fail(KFAC_ENOMEM, "out of host memory");
  p->count = count;
  p->order.resize(count);
  std::iota(p->order.begin(), p->order.end(), 0);
  std::stable_sort(p->order.begin(), p->order.end(),
                   [&](int a, int b) { return dims[a] > dims[b]; });
  std::vector<int> dim(count), tile_cs(count + 1, 0), panel_cs(count + 1, 0);
  std::vector<long long> off(count);
  p->nt.resize(count);
  size_t total = 0;
  for (int s = 0; s < count; ++s) {
    dim[s] = dims[p->order[s]];
    const int T = kfac::ceil_div(dim[s], NB);
    p->nt[s] = T;
    off[s] = (long long)total;
    total += (size_t)T * NB * T * NB;
    tile_cs[s + 1] = tile_cs[s] + T * (T + 1) / 2;
    panel_cs[s + 1] = panel_cs[s] + (T - 1);
  }
  p->ws_floats = total;
  p->side_floats = (size_t)count * 2 * NB * NB;
  p->total_tiles = tile_cs[count];
  p->max_t = count ? p->nt[0] : 0;
  std::vector<int> update_cs;
  for (int k = 0; k < p->max_t; ++k) {
    int na = 0;
    while (na < count && p->nt[na] > k) ++na;
    p->nactive.push_back(na);
    p->panel_total.push_back(panel_cs[na]);
    p->update_off.push_back((int)update_cs.size());
    int run = 0;
    update_cs.push_back(0);
    for (int s = 0; s < na; ++s) {
      const int r = p->nt[s] - k - 1;
      run += r * (r + 1) / 2 + r * k;
      update_cs.push_back(run);
    }
    p->update_total.push_back(run);
  }
  if (update_cs.empty()) update_cs.push_back(0);
  int rc = KFAC_OK;
  auto up = [&](kfac::DevTable &t, const void *h, size_t b) {
    if (rc == KFAC_OK) rc = t.set(h, b, nullptr);
  };
  up(p->d_orig, p->order.data(), sizeof(int) * count);
  up(p->d_dim, dim.data(), sizeof(int) * count);
  up(p->d_nt, p->nt.data(), sizeof(int) * count);
  up(p->d_off, off.data(), sizeof(long long) * count);
  up(p->d_tile, tile_cs.data(), sizeof(int) * (count + 1));
  up(p->d_panel, panel_cs.data(), sizeof(int) * (count + 1));
  up(p->d_update, update_cs.data(), sizeof(int) * update_cs.size());
  if (rc != KFAC_OK) {
    delete p;
    return rc;
  }
  *plan_out = p;
  return KFAC_OK;
}

extern "C" size_t kfac_inverse_plan_workspace_bytes(kfac_inverse_plan_t plan) {
  if (!plan) return 0;
  return (plan->ws_floats + plan->side_floats) * sizeof(float) + 256;
}

extern "C" int kfac_inverse_plan_destroy(kfac_inverse_plan_t plan) {
  delete plan;
  return KFAC_OK;
}

extern "C" int kfac_spd_inverse_batched_f32(kfac_inverse_plan_t plan,
                                            const float *const *in_ptrs,
                                            float *const *out_ptrs, int32_t *info_dev,
                                            void *ws, size_t ws_bytes, void *stream) {
  KFAC_REQUIRE(plan != nullptr, "plan is null");
  const int count = plan->count;
  if (count == 0) return KFAC_OK;
  KFAC_REQUIRE(in_ptrs && out_ptrs && info_dev, "null table");
  if (ws == nullptr || ws_bytes < kfac_inverse_plan_workspace_bytes(plan))
    return kfac::fail(KFAC_ENOMEM, "inverse workspace too small: %zu < %zu bytes", ws_bytes,
                      kfac_inverse_plan_workspace_bytes(plan));
  hipStream_t s = kfac::as_stream(stream);
  plan->in_sorted.resize(count);
  plan->out_sorted.resize(count);
  for (int i = 0; i < count; ++i) {
    KFAC_REQUIRE(in_ptrs[plan->order[i]] && out_ptrs[plan->order[i]], "matrix %d: null pointer",
                 plan->order[i]);
    KFAC_REQUIRE(in_ptrs[plan->order[i]] != out_ptrs[plan->order[i]],
                 "matrix %d: in-place inversion is not supported", plan->order[i]);
    plan->in_sorted[i] = in_ptrs[plan->order[i]];
    plan->out_sorted[i] = out_ptrs[plan->order[i]];
  }
  int rc = plan->d_in.set(plan->in_sorted.data(), sizeof(void *) * count, s);
  if (rc != KFAC_OK) return rc;
  rc = plan->d_out.set(plan->out_sorted.data(), sizeof(void *) * count, s);
  if (rc != KFAC_OK) return rc;
  if (!plan->attr_set) {
    KFAC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(diag_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)kDiagLds));
    plan->attr_set = true;
  }
  InvTables tb;
  tb.in = plan->d_in.as<const float *const>();
  tb.out = plan->d_out.as<float *const>();
  tb.orig = plan->d_orig.as<const int>();
  tb.dim = plan->d_dim.as<const int>();
  tb.nt = plan->d_nt.as<const int>();
  tb.ws_off = plan->d_off.as<const long long>();
  tb.tile_cs = plan->d_tile.as<const int>();
  tb.panel_cs = plan->d_panel.as<const int>();
  tb.update_cs = plan->d_update.as<const int>();
  uintptr_t base = (reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255;
  tb.ws = reinterpret_cast<float *>(base);
  tb.side = tb.ws + plan->ws_floats;
  tb.info = info_dev;

  hipLaunchKernelGGL(copy_in_kernel, dim3(plan->total_tiles), dim3(256), 0, s, tb, count);
  KFAC_HIP_CHECK(hipGetLastError());
  for (int k = 0; k < plan->max_t; ++k) {
    const int na = plan->nactive[k];
    hipLaunchKernelGGL(diag_kernel, dim3(na), dim3(256), kDiagLds, s, tb, k);
    if (plan->panel_total[k] > 0)
      hipLaunchKernelGGL(panel_kernel, dim3(plan->panel_total[k]), dim3(THREADS), 0, s, tb, k, na);
    if (plan->update_total[k] > 0) {
      kfac::TimedLaunch timed(KFAC_TIMED_INV_UPDATE, s);
      hipLaunchKernelGGL(update_kernel, dim3(plan->update_total[k]), dim3(THREADS), 0, s, tb, k,
                         na, plan->update_off[k]);
    }
  }
  KFAC_HIP_CHECK(hipGetLastError());
  {
    kfac::TimedLaunch timed(KFAC_TIMED_INV_LAUUM, s);
    hipLaunchKernelGGL(lauum_kernel, dim3(plan->total_tiles), dim3(THREADS), 0, s, tb, count);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}
