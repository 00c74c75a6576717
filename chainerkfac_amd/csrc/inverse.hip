// Batched damped inverse of SPD Kronecker factors: blocked Cholesky (potrf)
// followed by the triangular inverse and L^-T L^-1 (potri), FP32 MFMA.
//
// All matrices of a batch advance together.  Each is copied (lower tiles
// only) into a zero/identity padded workspace of NB x NB tiles (NB = 128),
// stored tile by tile (tile (I,J) of a T x T grid is the contiguous 64 KB block
// number I*T + J), so that every operand panel and every tile that is read and
// written back is one dense block instead of 128 short rows a matrix row apart.
// The strictly lower tiles end up holding L, the upper tiles U = L^-T (the
// triangular inverse, stored transposed), the diagonal tiles U_kk = L_kk^-T.
// With M(a,j) the tile in slot (a,j), every product of the sweep has one form,
//
//     C(a,b) -= sum_{j = j_lo .. j_hi} M(a,j) M(b,j)^T                   (*)
//
//   a >= b   potrf:  A(a,b) -= sum_j L(a,j) L(b,j)^T                (j < b)
//   a <  b   trtri:  X^T(a,b) = -sum_j U(a,j) L(b,j)^T         (a <= j < b)
//            followed by U(a,b) = X^T(a,b) L_bb^-T once the sum is complete,
//
// both k-contiguous "NT" tile GEMMs over row slabs of the workspace.  Block
// columns are processed in groups of kGroup (2): inside a group the sweep is
// left-looking (column k receives the products of the group's earlier columns
// just before it is factored, K up to (kGroup-1)*NB), and after a group every
// column to its right receives the whole group at once (K = kGroup*NB), which
// reads and writes each trailing tile once per group instead of once per
// column.  Per block column k, two dependent launches:
//
//   step(k)    one workgroup per matrix gives the diagonal tile the products it
//              is still owed, then does its Cholesky and U_kk = L_kk^-T inside
//              LDS on 32x32 MFMA blocks; the other workgroups of the launch
//              apply (*) to the rest of column k (inside a group: the group's
//              earlier columns; on a group's first column: the previous group,
//              for both columns of this group)
//   panel(k)   M(x,k) = M(x,k) U_kk for x != k  (L(x,k) below, U(x,k) above)
//
// and after a group's last column, on a second stream beside the next group's
// sweep, rest(g): (*) for all tiles right of the next group.  A final launch
// forms  out(i,j) = sum_{k >= i} U(i,k) U(j,k)^T  (lauum) and writes the full
// symmetric inverse.  Matrices of different sizes end their sweeps together (a
// matrix of T tiles joins at step max_T - T).  The tiles of every launch are
// listed in a task table built once per plan.
//
// Replaces chainerkfac/optimizers/cholesky_inverse.py:16-102 (potrf + potrs
// against the identity, one matrix at a time).
#include <cstdlib>
#include <algorithm>
#include <numeric>

#include "chol32.h"
#include "common.h"
#include "mma_core.h"

namespace {

using namespace kfac::mma;

constexpr int NB = 128;
constexpr int SB = 32;
constexpr int LS = NB + 1;  // LDS row stride of the diagonal-tile kernel
constexpr int PS = SB + 1;  // row stride of a wave's private 32x32 block

struct InvTables {
  const float *const *in;    // [count] sorted slot -> input matrix
  float *const *out;         // [count]
  const int *orig;           // [count] slot -> caller index
  const int *dim;            // [count]
  const int *nt;             // [count] tiles per side
  const int *shift;          // [count] sweep step at which the matrix starts
  const long long *ws_off;   // [count] float offset of the padded matrix
  const int *tile_cs;        // [count+1] cumulative lower-tile counts
  const int *panel_cs;       // [count+1] cumulative (nt-1)
  const int2 *tasks;         // update tasks of all launches: {slot, a | b << 16}
  float *ws;                 // padded matrices
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

__device__ __forceinline__ float *tile_ptr(const InvTables &tb, int s, int I, int J) {
  return tb.ws + tb.ws_off[s] + ((long long)I * tb.nt[s] + J) * (NB * NB);
}

// Operand loader of the shared main loop for a run of consecutive tiles of one
// tile row: k-value k is column k % NB of tile k / NB.  A 128 x 32 panel is
// 128 rows of 128 contiguous bytes inside one tile; no edge masks are needed
// (the workspace is padded).
typedef float vfloat4 __attribute__((ext_vector_type(4)));   // register arrays of HIP's float4 struct can end up in scratch

struct LoaderTile {
  static constexpr bool kKRow = false;
  struct Regs {
    vfloat4 v[NB / 32];
  };
  const float *base;   // first tile of the run
  __device__ __forceinline__ void load(Regs &r, int, long long k0, long long) const {
    const unsigned k = (unsigned)k0 + (threadIdx.x & 7) * 4;
    const float *p = base + (size_t)(k / NB) * (NB * NB) + (k % NB) + (threadIdx.x >> 3) * NB;
#pragma unroll
    for (int i = 0; i < NB / 32; ++i) r.v[i] = *reinterpret_cast<const vfloat4 *>(p + 32 * i * NB);
  }
  __device__ __forceinline__ void store(const Regs &r, float *lds) const {
    const int kq = (threadIdx.x & 7) * 4;
    const int rr = threadIdx.x >> 3;
#pragma unroll
    for (int i = 0; i < NB / 32; ++i) {
      float *p = lds + (rr + 32 * i) * Panel<NB>::kRowKStride + kq;
      p[0] = r.v[i].x;
      p[1] = r.v[i].y;
      p[2] = r.v[i].z;
      p[3] = r.v[i].w;
    }
  }
};

// The same tile read as its transpose: operand row c, k-value q is element
// (q, c).  Rows of the tile are contiguous in c, so the panel goes to LDS in the
// k-major layout.
struct LoaderTileT {
  static constexpr bool kKRow = true;
  struct Regs {
    vfloat4 v[KT / 8];
  };
  const float *base;
  __device__ __forceinline__ void load(Regs &r, int, long long k0, long long) const {
    const float *p = base + ((int)k0 + (threadIdx.x >> 5)) * NB + (threadIdx.x & 31) * 4;
#pragma unroll
    for (int i = 0; i < KT / 8; ++i) r.v[i] = *reinterpret_cast<const vfloat4 *>(p + 8 * i * NB);
  }
  __device__ __forceinline__ void store(const Regs &r, float *lds) const {
    float *p = lds + (threadIdx.x >> 5) * Panel<NB>::kKRowStride + (threadIdx.x & 31) * 4;
#pragma unroll
    for (int i = 0; i < KT / 8; ++i)
      *reinterpret_cast<vfloat4 *>(p + 8 * i * Panel<NB>::kKRowStride) = r.v[i];
  }
};

// Main loop of the tile kernels: the shared loop with 64 k-values (two LDS
// panels per operand) per pass instead of 32.  The products of this file are
// short (K = 128 .. 512) and often one workgroup per CU, so what counts is how
// many loads are in flight and how few barrier-to-barrier round trips a product
// needs: K = 128 takes two passes instead of four.  K must be a multiple of 64.
// lds: 4 panels (A0, A1, B0, B1) of Panel<NB>::kFloats.
constexpr int kTileLdsFloats = 4 * Panel<NB>::kFloats;
constexpr size_t kTileLdsBytes = kTileLdsFloats * sizeof(float);

template <bool SAME, int D, class LA, class LB>
__device__ __forceinline__ void tile_mainloop(const LA &la, const LB &lb, int K, float *lds,
                                              floatx16 (&acc)[2][2]) {
  constexpr int PF = Panel<NB>::kFloats;
  // D: passes of 64 k-values held in registers ahead of the one in LDS.  With
  // one, a third of the passes of a full GPU wait 2-4 us for their operands
  // (measured with time stamps); two cover that where the registers allow it.
  float *ldsA = lds, *ldsB = lds + 2 * PF;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane & 31, lk = lane >> 5;
  typename LA::Regs ra[D][2];
  typename LB::Regs rb[D][2];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    if (d * 2 * KT < K) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        la.load(ra[d][h], 0, d * 2 * KT + KT * h, K);
        if (!SAME) lb.load(rb[d][h], 0, d * 2 * KT + KT * h, K);
      }
    }
  }
  for (int kb = 0; kb < K; kb += D * 2 * KT) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int k0 = kb + d * 2 * KT;
      if (k0 < K) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        la.store(ra[d][h], ldsA + h * PF);
        if (!SAME) lb.store(rb[d][h], ldsB + h * PF);
      }
      __syncthreads();
      if (k0 + D * 2 * KT < K) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          la.load(ra[d][h], 0, k0 + D * 2 * KT + KT * h, K);
          if (!SAME) lb.load(rb[d][h], 0, k0 + D * 2 * KT + KT * h, K);
        }
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float *pa = ldsA + h * PF;
        const float *pb = SAME ? pa : ldsB + h * PF;
#pragma unroll
        for (int kk = 0; kk < KT / 2; ++kk) {
          float a[2], b[2];
#pragma unroll
          for (int im = 0; im < 2; ++im)
            a[im] = fetch<NB, LA::kKRow>(pa, (wm * 2 + im) * 32 + lrow, 2 * kk + lk);
#pragma unroll
          for (int in = 0; in < 2; ++in) {
            if (SAME)
              b[in] = fetch<NB, LA::kKRow>(pb, (wn * 2 + in) * 32 + lrow, 2 * kk + lk);
            else
              b[in] = fetch<NB, LB::kKRow>(pb, (wn * 2 + in) * 32 + lrow, 2 * kk + lk);
          }
#pragma unroll
          for (int im = 0; im < 2; ++im)
#pragma unroll
            for (int in = 0; in < 2; ++in)
              acc[im][in] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[im], b[in], acc[im][in], 0, 0, 0);
        }
      }
      __syncthreads();
      }
    }
  }
}

// ---------------------------------------------------------------------------
// copy-in: lower tiles of in -> padded workspace (identity on the padding)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void copy_in_kernel(InvTables tb, int count) {
  const int s = find_slot(tb.tile_cs, count, blockIdx.x);
  int I, J;
  tri_decode(blockIdx.x - tb.tile_cs[s], I, J);
  const int d = tb.dim[s];
  const float *__restrict__ src = tb.in[s];
  float *__restrict__ dst = tile_ptr(tb, s, I, J);
  const int c4 = (threadIdx.x & 31) * 4;
  const int r0 = threadIdx.x >> 5;
#pragma unroll 4
  for (int p = 0; p < NB / 8; ++p) {
    const int rl = r0 + 8 * p;
    const int r = I * NB + rl;
    const int c = J * NB + c4;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int ce = c + e;
      float x = (r == ce) ? 1.f : 0.f;
      if (r < d && ce < d) x = src[(long long)r * d + ce];
      v[e] = x;
    }
    *reinterpret_cast<float4 *>(dst + rl * NB + c4) = make_float4(v[0], v[1], v[2], v[3]);
  }
}

// ---------------------------------------------------------------------------
// diagonal tile: Cholesky + triangular inverse inside LDS
// ---------------------------------------------------------------------------

// acc += A(32 x K) * B^T, A at a[row*AS + k]; B at b[row*LS + k] or, when BT,
// at b[k*LS + row].
template <bool BT, int AS = LS>
__device__ __forceinline__ floatx16 wave_gemm(const float *a, const float *b, int K,
                                              floatx16 acc) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  for (int k = 0; k < K; k += 2) {
    const float av = a[r * AS + k + h];
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

// Diagonal tile (k,k) of matrix s: first the products it is still owed,
//   C(k,k) -= sum_{j = lo .. hi} M(k,j) M(k,j)^T        (nothing when hi < lo),
// through the shared main loop (the other tiles of the column receive theirs
// from the update workgroups of the same launch), then the factorisation.
__device__ __forceinline__ void diag_role(const InvTables &tb, int s, int k, int lo, int hi,
                                          float *smem) {
  float *S = smem;                      // NB x LS working tile
  float *scratch = smem + NB * LS;      // 3 waves x SB x PS
  const int d = tb.dim[s];
  constexpr int ld = NB;
  float *tile = tile_ptr(tb, s, k, k);
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  if (hi >= lo) {
    floatx16 acc[2][2];
    fill_acc<2, 2>(acc, [&](int rr, int cc) { return -tile[rr * NB + cc]; });
    const LoaderTile la{tile_ptr(tb, s, k, lo)};
    tile_mainloop<true, 1>(la, la, (hi - lo + 1) * NB, smem, acc);   // ends with a barrier
    for_each_acc<2, 2>(acc, [&](int rr, int cc, float v) { S[rr * LS + cc] = -v; });
  } else {
    const int c4 = (threadIdx.x & 31) * 4, r0 = threadIdx.x >> 5;
#pragma unroll 4
    for (int p = 0; p < NB / 8; ++p) {
      const int r = r0 + 8 * p;
      const float4 v = *reinterpret_cast<const float4 *>(tile + r * ld + c4);
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
      const int bad = kfac::chol_inv_32<LS>(S, jb * SB);
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
  float *P = scratch + wave * SB * PS;
  for (int dd = 1; dd < NB / SB; ++dd) {
    for (int jb = wave; jb + dd < NB / SB; jb += 4) {
      const int ib = jb + dd;
      const floatx16 p = wave_gemm<false>(S + (jb * SB) * LS + jb * SB,
                                          S + (ib * SB) * LS + jb * SB, dd * SB, zero);
      wave_visit(p, [&](int r, int c, float v) { P[r * PS + c] = v; });
      // the same wave re-reads P: LDS accesses of one wave execute in order
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      const floatx16 u = wave_gemm<true, PS>(P, S + (ib * SB) * LS + ib * SB, SB, zero);
      float *blk = S + (jb * SB) * LS + ib * SB;
      wave_visit(u, [&](int r, int c, float v) { blk[r * LS + c] = -v; });
    }
    __syncthreads();
  }

  // ---- outputs
  // U -> diagonal tile of the workspace, exact zeros below the diagonal
  {
    const int c4 = (threadIdx.x & 31) * 4, r0 = threadIdx.x >> 5;
#pragma unroll 4
    for (int p = 0; p < NB / 8; ++p) {
      const int r = r0 + 8 * p;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int c = c4 + e;
        const bool up = (c / SB > r / SB) || (c / SB == r / SB && c >= r);
        v[e] = up ? S[r * LS + c] : 0.f;
      }
      *reinterpret_cast<float4 *>(tile + r * ld + c4) = make_float4(v[0], v[1], v[2], v[3]);
    }
  }
}

// ---------------------------------------------------------------------------
// panel and update: 128x128x128 tile products through the shared main loop
// ---------------------------------------------------------------------------
// M(x,k) = M(x,k) W^T = M(x,k) U_kk in place for every x != k; the operand
// W^T is the diagonal tile itself, read transposed.
__global__ __launch_bounds__(THREADS, 2) void panel_kernel(InvTables tb, int step, int nactive) {
  extern __shared__ float lds[];
  const int s = find_slot(tb.panel_cs, nactive, blockIdx.x);
  const int k = step - tb.shift[s];
  const int local = blockIdx.x - tb.panel_cs[s];
  const int x = local < k ? local : local + 1;
  float *tile = tile_ptr(tb, s, x, k);
  floatx16 acc[2][2];
  zero_acc<2, 2>(acc);
  tile_mainloop<false, 1>(LoaderTile{tile}, LoaderTileT{tile_ptr(tb, s, k, k)}, NB, lds, acc);
  for_each_acc<2, 2>(acc, [&](int rr, int cc, float v) { tile[rr * NB + cc] = v; });
}

// One task of (*): tile (a,b) of matrix `slot`, products over the block
// columns [k0, k1] clipped to the tile's own range.  The accumulators start
// from -C, so the tile is read while the first operand panels are in flight and
// the epilogue is a plain store.  An upper tile whose row lies inside [k0, k1]
// receives its first product here and is overwritten (it holds stale data).
template <int D>
__device__ __forceinline__ void update_role(const InvTables &tb, int2 task, int k0, int k1,
                                            float *lds) {
  const int s = task.x;
  const int a = task.y & 0xffff, b = task.y >> 16;
  const bool upper = a < b;
  const int j_lo = upper && a > k0 ? a : k0;
  const int j_hi = upper && b - 1 < k1 ? b - 1 : k1;
  const int K = (j_hi - j_lo + 1) * NB;
  const bool first = upper && a >= k0;
  float *C = tile_ptr(tb, s, a, b);
  floatx16 acc[2][2];
  if (first)
    zero_acc<2, 2>(acc);
  else
    fill_acc<2, 2>(acc, [&](int rr, int cc) { return -C[rr * NB + cc]; });
  const LoaderTile la{tile_ptr(tb, s, a, j_lo)}, lb{tile_ptr(tb, s, b, j_lo)};
  if (a == b)
    tile_mainloop<true, D>(la, lb, K, lds, acc);
  else
    tile_mainloop<false, D>(la, lb, K, lds, acc);
  for_each_acc<2, 2>(acc, [&](int rr, int cc, float v) { C[rr * NB + cc] = -v; });
}

// The group's block columns [step0, step1] in matrix s's own numbering (a
// matrix that starts inside the group has a shorter first group).
__device__ __forceinline__ void local_range(const InvTables &tb, int s, int step0, int step1,
                                            int &k0, int &k1) {
  const int shift = tb.shift[s];
  k0 = step0 > shift ? step0 - shift : 0;
  k1 = step1 - shift;
}

// One launch per sweep step: workgroups [0, ndiag) factor the diagonal tile of
// their matrix (after giving it the products of columns [step0, step1]), the
// others apply the same columns to the tiles the next panel step reads.  The
// diagonal workgroups come first in launch order, so the serial part starts at
// once and the updates fill the rest of the GPU beside it.
__global__ __launch_bounds__(THREADS, 2) void step_kernel(InvTables tb, int step, int ndiag,
                                                          int task0, int step0, int step1) {
  extern __shared__ float lds[];
  if ((int)blockIdx.x < ndiag) {
    const int s = blockIdx.x;
    int k0, k1;
    local_range(tb, s, step0, step1, k0, k1);
    diag_role(tb, s, step - tb.shift[s], k0, k1, lds);
  } else {
    const int2 task = tb.tasks[task0 + blockIdx.x - ndiag];
    int k0, k1;
    local_range(tb, task.x, step0, step1, k0, k1);
    update_role<1>(tb, task, k0, k1, lds);
  }
}

// The part of a trailing update that the next group's sweep does not read.
__global__ __launch_bounds__(THREADS, 2) void update_kernel(InvTables tb, int task0, int step0,
                                                            int step1) {
  extern __shared__ float lds[];
  const int2 task = tb.tasks[task0 + blockIdx.x];
  int k0, k1;
  local_range(tb, task.x, step0, step1, k0, k1);
  update_role<1>(tb, task, k0, k1, lds);
}

// out(i,j) = sum_{k >= i} U(i,k) U(j,k)^T for i >= j, written with its mirror.
// One task per tile; the table deals whole tile rows to XCDs (see the plan).
__global__ __launch_bounds__(THREADS, 2) void lauum_kernel(InvTables tb, int task0) {
  extern __shared__ float lds[];
  const int2 task = tb.tasks[task0 + blockIdx.x];
  const int s = task.x;
  if (s < 0) return;   // padding of an XCD's shorter list
  const int I = task.y & 0xffff, J = task.y >> 16;
  const int T = tb.nt[s];
  const int d = tb.dim[s];
  const int K = (T - I) * NB;
  const LoaderTile la{tile_ptr(tb, s, I, I)}, lb{tile_ptr(tb, s, J, I)};
  floatx16 acc[2][2];
  zero_acc<2, 2>(acc);
  if (I == J)
    tile_mainloop<true, 2>(la, lb, K, lds, acc);
  else
    tile_mainloop<false, 2>(la, lb, K, lds, acc);
  // through an LDS transpose, so that the mirror is written in row segments too
  write_tile<2>(acc, lds, I, J, d, d, 1.f, 0.f, tb.out[s]);
}

// Dynamic LDS of the step kernel: the diagonal role's working tile and three
// private blocks (at most three waves are busy in a pass of the triangular
// inverse), 77 KB, so that two workgroups share a CU like the other tile kernels.
constexpr size_t kDiagLds = (size_t)(NB * LS + 3 * SB * PS) * sizeof(float);
constexpr size_t kStepLds = kDiagLds > kTileLdsBytes ? kDiagLds : kTileLdsBytes;
static_assert(2 * kStepLds <= 160 * 1024, "two step workgroups must fit a CU");
constexpr size_t kRestLdsBytes = 81 * 1024;
static_assert(2 * kRestLdsBytes > 160 * 1024 && kRestLdsBytes + kStepLds <= 160 * 1024,
              "one rest workgroup per CU, with room for a step workgroup");

}  // namespace

struct UpdateLaunch {
  int task0 = 0, count = 0;   // range in the task table
  int k0 = 0, k1 = 0;         // block columns whose products are applied
};

struct kfac_inverse_plan {
  int count = 0;
  int max_t = 0;
  int group = 2;                   // block columns per trailing update (measured best of 1..8)
  std::vector<int> order;          // slot -> caller index
  std::vector<int> nt;             // per slot
  std::vector<int> nactive;        // per step
  std::vector<int> panel_total;    // per step
  // per step: the update tasks that share the launch with the diagonal tiles:
  // inside a group the left-looking update of column k, on a group's first
  // column the previous group's trailing update of this group's columns
  std::vector<UpdateLaunch> with_diag;
  // per step, set on the last column of a group: its trailing update of
  // everything right of the next group
  std::vector<UpdateLaunch> rest;
  // The rest of a trailing update touches nothing the next group's sweep needs,
  // so it runs on a second stream beside that sweep.
  bool lookahead = true;
  // Under stream capture the fork onto `side` is only safe from the stream the
  // capture began on (a fork of a forked stream has crashed the runtime), which
  // the library cannot find out by itself: the caller says so.
  bool capture_origin = false;
  size_t rest_lds = 0;
  hipStream_t side = nullptr;
  std::vector<hipEvent_t> ev_main, ev_side;   // per step
  ~kfac_inverse_plan() {
    for (hipEvent_t e : ev_main) (void)hipEventDestroy(e);
    for (hipEvent_t e : ev_side) (void)hipEventDestroy(e);
    if (side) (void)hipStreamDestroy(side);
  }
  int total_tiles = 0;
  int lauum_task0 = 0, lauum_count = 0;
  size_t ws_floats = 0;            // padded matrices
  std::vector<const void *> in_sorted, out_sorted;
  kfac::DevTable d_in, d_out, d_orig, d_dim, d_nt, d_shift, d_off, d_tile, d_panel, d_tasks;
  bool attr_set = false;
};

namespace {

// Workgroup i of a launch runs on XCD i % 8.  Deal the tasks out so that each
// XCD receives one contiguous run of the natural order (neighbouring tasks
// share operand row slabs, which then stay in that XCD's L2).
void append_tasks(std::vector<int2> &table, const std::vector<int2> &natural) {
  const size_t n = natural.size();
  const size_t chunk = (n + 7) / 8;
  std::vector<int2> dealt;
  dealt.reserve(n);
  // position p of XCD x holds natural[x * chunk + p]; emit in launch order
  // (p major, x minor) and skip the holes of a ragged last chunk
  for (size_t p = 0; p < chunk; ++p)
    for (size_t x = 0; x < 8; ++x) {
      const size_t i = x * chunk + p;
      if (i < n) dealt.push_back(natural[i]);
    }
  table.insert(table.end(), dealt.begin(), dealt.end());
}

}  // namespace

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
  if (const char *e = getenv("KFAC_INVERSE_GROUP")) {   // tuning override
    const int g = atoi(e);
    if (g >= 1 && g <= 64) p->group = g;
  }
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
  p->total_tiles = tile_cs[count];
  p->max_t = count ? p->nt[0] : 0;
  std::vector<int2> tasks, natural;
  p->with_diag.resize(p->max_t);
  p->rest.resize(p->max_t);
  if (const char *e = getenv("KFAC_INVERSE_LOOKAHEAD")) p->lookahead = atoi(e) != 0;
  // The rest asks for more LDS than it uses, 81 KB: then one of its workgroups
  // fits a CU, not two, and a step or panel workgroup always finds room beside
  // it instead of queueing behind the rest for a slot (measured: the rest alone
  // loses 14 %, the sweep as a whole gains).  KFAC_INVERSE_REST_LDS overrides.
  p->rest_lds = kRestLdsBytes;
  if (const char *e = getenv("KFAC_INVERSE_REST_LDS")) {
    const long v = atol(e);
    if (v >= (long)kTileLdsBytes && v <= 160 * 1024) p->rest_lds = (size_t)v;
  }
  auto pack = [](int s, int a, int b) { return make_int2(s, a | (b << 16)); };
  // Matrix s joins the sweep at step shift[s] and runs nt[s] steps.  Aligning
  // the ends (shift = max_t - nt) puts the short sweeps of the small matrices
  // beside the late steps of the largest ones, which on their own leave most of
  // the GPU idle (few tiles, one dependent launch after another); aligning the
  // starts piles all matrices onto the early steps, which are the ones that are
  // already throughput-bound.  KFAC_INVERSE_ALIGN=<percent> (0 = starts, 100 =
  // ends) is a tuning override.
  int align = 100;
  if (const char *e = getenv("KFAC_INVERSE_ALIGN")) align = std::min(100, std::max(0, atoi(e)));
  std::vector<int> shift(count);
  for (int s = 0; s < count; ++s) shift[s] = (p->max_t - p->nt[s]) * align / 100;
  // Tiles right of the source group [s0, s1] (sweep steps) that receive its
  // products: the columns of the following group when `next`, otherwise
  // everything right of those.  The upper tiles whose row lies inside the source
  // group have shorter sums and go to `tail`.  The following group's first
  // diagonal tile is left to its diagonal workgroup.
  auto trailing = [&](bool next, int s0, int s1, std::vector<int2> &body, std::vector<int2> &tail) {
    for (int s = 0; s < count; ++s) {
      const int T = p->nt[s];
      const int k1 = s1 - shift[s];
      if (k1 < 0 || k1 >= T) continue;   // not in the sweep during the source group
      const int k0 = std::max(s0 - shift[s], 0);
      const int ku = k1 + p->group;
      const int c_lo = next ? k1 + 1 : ku + 1;
      const int c_hi = next ? std::min(ku, T - 1) : T - 1;
      for (int n = c_lo; n <= c_hi; ++n)
        for (int m = n; m < T; ++m)
          if (!(next && m == c_lo)) body.push_back(pack(s, m, n));
      for (int a = 0; a < k0; ++a)
        for (int b = c_lo; b <= c_hi; ++b) body.push_back(pack(s, a, b));
      for (int a = k0; a <= k1; ++a)
        for (int b = c_lo; b <= c_hi; ++b) tail.push_back(pack(s, a, b));
    }
  };
  for (int g = 0; g < p->max_t; ++g) {
    // active matrices: shift <= g < shift + nt; a prefix of the sorted order
    // (shift grows and shift + nt shrinks with the slot number)
    int na = 0;
    while (na < count && shift[na] <= g && g < shift[na] + p->nt[na]) ++na;
    p->nactive.push_back(na);
    p->panel_total.push_back(panel_cs[na]);
    const int g0 = g / p->group * p->group;
    const int g1 = std::min(g0 + p->group - 1, p->max_t - 1);
    UpdateLaunch &w = p->with_diag[g];
    std::vector<int2> tail;
    natural.clear();
    if (g > g0) {
      // column g - shift of every active matrix: products of the group's earlier
      // columns (the diagonal tile takes its own inside the diagonal workgroup)
      w.k0 = g0;
      w.k1 = g - 1;
      for (int s = 0; s < na; ++s) {
        const int k = g - shift[s], k0 = std::max(g0 - shift[s], 0);
        if (k <= k0) continue;
        for (int m = k + 1; m < p->nt[s]; ++m) natural.push_back(pack(s, m, k));
        for (int a = 0; a < k; ++a) natural.push_back(pack(s, a, k));
      }
    } else {
      // first column of a group: the previous group's products for this group's columns
      w.k0 = g0 - p->group;
      w.k1 = g0 - 1;
      if (g > 0) trailing(true, w.k0, w.k1, natural, tail);
    }
    w.task0 = (int)tasks.size();
    w.count = (int)(natural.size() + tail.size());
    append_tasks(tasks, natural);
    append_tasks(tasks, tail);
    if (g == g1 && g1 + 1 < p->max_t) {
      natural.clear();
      tail.clear();
      trailing(false, g0, g1, natural, tail);
      UpdateLaunch &u = p->rest[g];
      u.task0 = (int)tasks.size();
      u.count = (int)(natural.size() + tail.size());
      u.k0 = g0;
      u.k1 = g1;
      append_tasks(tasks, natural);
      append_tasks(tasks, tail);
    }
  }
  // Final products out(I,J) = sum_k U(I,k) U(J,k)^T: the I + 1 tiles of tile row I
  // all read the row U(I, I..T-1).  A whole row goes to one XCD (workgroup i of a
  // launch runs on XCD i % 8), so that the row stays in that XCD's L2 while its
  // tiles stream the U(J, .) rows; rows are dealt longest first to the XCD with
  // the least work, and each XCD runs its long-K rows first.
  {
    struct Row { int s, I; double cost; };
    std::vector<Row> rows;
    for (int s = 0; s < count; ++s)
      for (int I = 0; I < p->nt[s]; ++I)
        rows.push_back({s, I, (double)(I + 1) * (p->nt[s] - I) + 0.5 * (I + 1)});
    std::stable_sort(rows.begin(), rows.end(), [](const Row &a, const Row &b) { return a.cost > b.cost; });
    std::vector<Row> mine[8];
    double load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (const Row &r : rows) {
      int x = 0;
      for (int i = 1; i < 8; ++i)
        if (load[i] < load[x]) x = i;
      mine[x].push_back(r);
      load[x] += r.cost;
    }
    std::vector<int2> list[8];
    size_t longest = 0;
    for (int x = 0; x < 8; ++x) {
      std::stable_sort(mine[x].begin(), mine[x].end(), [&](const Row &a, const Row &b) {
        return p->nt[a.s] - a.I > p->nt[b.s] - b.I;
      });
      for (const Row &r : mine[x])
        for (int J = 0; J <= r.I; ++J) list[x].push_back(pack(r.s, r.I, J));
      longest = std::max(longest, list[x].size());
    }
    p->lauum_task0 = (int)tasks.size();
    for (size_t i = 0; i < longest; ++i)
      for (int x = 0; x < 8; ++x)
        tasks.push_back(i < list[x].size() ? list[x][i] : make_int2(-1, 0));
    p->lauum_count = (int)(longest * 8);
  }
  if (tasks.empty()) tasks.push_back(make_int2(0, 0));
  int rc = KFAC_OK;
  auto up = [&](kfac::DevTable &t, const void *h, size_t b) {
    if (rc == KFAC_OK) rc = t.set(h, b, nullptr);
  };
  up(p->d_orig, p->order.data(), sizeof(int) * count);
  up(p->d_dim, dim.data(), sizeof(int) * count);
  up(p->d_nt, p->nt.data(), sizeof(int) * count);
  up(p->d_shift, shift.data(), sizeof(int) * count);
  up(p->d_off, off.data(), sizeof(long long) * count);
  up(p->d_tile, tile_cs.data(), sizeof(int) * (count + 1));
  up(p->d_panel, panel_cs.data(), sizeof(int) * (count + 1));
  up(p->d_tasks, tasks.data(), sizeof(int2) * tasks.size());
  if (rc == KFAC_OK && p->lookahead && p->max_t > p->group) {
    bool ok = hipStreamCreateWithFlags(&p->side, hipStreamNonBlocking) == hipSuccess;
    for (int g = 0; ok && g < p->max_t; ++g) {
      hipEvent_t a = nullptr, b = nullptr;
      ok = hipEventCreateWithFlags(&a, hipEventDisableTiming) == hipSuccess;
      if (ok) p->ev_main.push_back(a);
      ok = ok && hipEventCreateWithFlags(&b, hipEventDisableTiming) == hipSuccess;
      if (ok && b) p->ev_side.push_back(b);
    }
    if (!ok) rc = kfac::fail(KFAC_EHIP, "cannot create the look-ahead stream or its events");
  } else {
    p->lookahead = false;
  }
  if (rc != KFAC_OK) {
    delete p;
    return rc;
  }
  *plan_out = p;
  return KFAC_OK;
}

extern "C" size_t kfac_inverse_plan_workspace_bytes(kfac_inverse_plan_t plan) {
  if (!plan) return 0;
  return plan->ws_floats * sizeof(float) + 256;
}

extern "C" int kfac_inverse_plan_set_capture_origin(kfac_inverse_plan_t plan, int is_origin) {
  KFAC_REQUIRE(plan != nullptr, "plan is null");
  plan->capture_origin = is_origin != 0;
  return KFAC_OK;
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
  // The trailing updates fork onto the plan's own stream.  While `s` is being
  // captured into a graph that is done only if the caller has declared `s` the
  // capture's origin; otherwise everything stays on `s`, in program order.
  bool lookahead = plan->lookahead;
  if (lookahead && !plan->capture_origin) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cs) != hipSuccess) {
      (void)hipGetLastError();   // e.g. the null stream beside a global-mode capture
      lookahead = false;
    } else if (cs != hipStreamCaptureStatusNone) {
      lookahead = false;
    }
  }
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
    KFAC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(step_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)kStepLds));
    for (const void *f : {reinterpret_cast<const void *>(panel_kernel),
                          reinterpret_cast<const void *>(lauum_kernel)})
      KFAC_HIP_CHECK(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)kTileLdsBytes));
    KFAC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(update_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    plan->attr_set = true;
  }
  InvTables tb;
  tb.in = plan->d_in.as<const float *const>();
  tb.out = plan->d_out.as<float *const>();
  tb.orig = plan->d_orig.as<const int>();
  tb.dim = plan->d_dim.as<const int>();
  tb.nt = plan->d_nt.as<const int>();
  tb.shift = plan->d_shift.as<const int>();
  tb.ws_off = plan->d_off.as<const long long>();
  tb.tile_cs = plan->d_tile.as<const int>();
  tb.panel_cs = plan->d_panel.as<const int>();
  tb.tasks = plan->d_tasks.as<const int2>();
  uintptr_t base = (reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255;
  tb.ws = reinterpret_cast<float *>(base);
  tb.info = info_dev;

  hipLaunchKernelGGL(copy_in_kernel, dim3(plan->total_tiles), dim3(256), 0, s, tb, count);
  KFAC_HIP_CHECK(hipGetLastError());
  // Side stream: after the last column of a group, the rest of its trailing
  // update.  It is queued just after the next step's launch, so that the step's
  // workgroups (the serial part of the sweep) are placed first and the rest
  // fills the GPU around them.
  int pending = -1;    // step of the latest work queued on the side stream
  int deferred = -1;   // step whose rest is still to be queued
  auto queue_rest = [&]() -> int {
    if (deferred < 0) return KFAC_OK;
    const UpdateLaunch &r = plan->rest[deferred];
    hipStream_t st = s;
    if (lookahead) {
      KFAC_HIP_CHECK(hipStreamWaitEvent(plan->side, plan->ev_main[deferred], 0));
      st = plan->side;
    }
    {
      kfac::TimedLaunch timed(KFAC_TIMED_INV_UPDATE, st);
      hipLaunchKernelGGL(update_kernel, dim3(r.count), dim3(THREADS), plan->rest_lds, st, tb,
                         r.task0, r.k0, r.k1);
    }
    if (lookahead) {
      KFAC_HIP_CHECK(hipEventRecord(plan->ev_side[deferred], plan->side));
      pending = deferred;
    }
    deferred = -1;
    return KFAC_OK;
  };
  for (int k = 0; k < plan->max_t; ++k) {
    const int na = plan->nactive[k];
    const UpdateLaunch &w = plan->with_diag[k];
    // A group's first step applies the previous group to this group's columns,
    // tiles that the rest of the group before that one (two back) also updated.
    // The rest of the previous group itself only touches columns further right
    // and runs beside this group's sweep.
    const int two_back = k - 1 - plan->group;
    if (lookahead && k % plan->group == 0 && two_back >= 0 && plan->rest[two_back].count > 0)
      KFAC_HIP_CHECK(hipStreamWaitEvent(s, plan->ev_side[two_back], 0));
    if (!lookahead)
      if (int rc2 = queue_rest()) return rc2;   // one stream: keep the program order
    {
      kfac::TimedLaunch timed(KFAC_TIMED_INV_UPDATE, s);
      hipLaunchKernelGGL(step_kernel, dim3(na + w.count), dim3(THREADS), kStepLds, s, tb, k, na,
                         w.task0, w.k0, w.k1);
    }
    if (int rc2 = queue_rest()) return rc2;
    if (plan->panel_total[k] > 0)
      hipLaunchKernelGGL(panel_kernel, dim3(plan->panel_total[k]), dim3(THREADS), kTileLdsBytes, s,
                         tb, k, na);
    if (plan->rest[k].count == 0) continue;
    if (lookahead) KFAC_HIP_CHECK(hipEventRecord(plan->ev_main[k], s));
    deferred = k;
  }
  if (int rc2 = queue_rest()) return rc2;
  if (pending >= 0) KFAC_HIP_CHECK(hipStreamWaitEvent(s, plan->ev_side[pending], 0));
  KFAC_HIP_CHECK(hipGetLastError());
  {
    kfac::TimedLaunch timed(KFAC_TIMED_INV_LAUUM, s);
    hipLaunchKernelGGL(lauum_kernel, dim3(plan->lauum_count), dim3(THREADS), kTileLdsBytes, s, tb,
                       plan->lauum_task0);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

