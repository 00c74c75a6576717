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
// column.  Per block column k, three launches:
//
//   diag(k)    one workgroup per matrix gives the diagonal tile the products it
//              is still owed, then does its Cholesky and U_kk = L_kk^-T inside
//              LDS on 32x32 MFMA blocks
//   column(k)  beside diag(k), on a stream of its own: (*) for the rest of
//              column k (inside a group: the group's earlier columns; on a
//              group's first column: the previous group, for both columns of
//              this group)
//   panel(k)   after both: M(x,k) = M(x,k) U_kk for x != k  (L(x,k) below,
//              U(x,k) above)
//
// and after a group's last column, on a further stream beside the next group's
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

// One tile product, resolved on the host when the plan is built: a workgroup
// reads its record (one scalar load) and can issue its operand loads at once,
// instead of walking the per-matrix tables first (three dependent round trips
// of 1-2 us each on a busy GPU, on the critical path of every launch of the
// sweep).  Offsets are float offsets into the workspace.
struct TileTask {
  long long c_off;   // tile that is updated / written; lauum: the slot of the matrix
  long long a_off;   // first tile of the A operand's run
  long long b_off;   // first tile of the B operand's run; diagonal task: caller index | dimension << 32
  int K;             // reduction length; 0: nothing to do (diagonal task: no products owed)
  int flags;         // update: kFirst | kSame; diagonal task: block column k; lauum: I | J << 16
};
constexpr int kFirst = 1;   // the accumulators start from zero (first product of an upper tile)
constexpr int kSame = 2;    // both operands are the same run

struct BorderTask;
struct InvTables {
  const float *const *in;    // [count] sorted slot -> input matrix
  float *const *out;         // [count]
  const int *dim;            // [count]
  const int *core;           // [count] rows of the tiled part: dim, or dim - 1 for a bordered matrix
  const int *orig;           // [count] sorted slot -> caller index
  const long long *vec_off;  // [count] bordered matrix: float offset of its vectors a | y | w (core floats
                             // each) and the scalars alpha, S, 1/S behind them; -1 otherwise
  const int *nt;             // [count] tiles per side
  const long long *ws_off;   // [count] float offset of the padded matrix
  const int *tile_cs;        // [count+1] cumulative lower-tile counts (copy-in)
  const int2 *tile_owner;    // [tiles] copy-in: (slot, I | J << 16) of every lower tile, one load instead of a search
  const TileTask *tasks;     // the tile tasks of all launches
  const BorderTask *btasks;  // the vector tasks of the bordered matrices
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

// ---------------------------------------------------------------------------
// The tile product  acc(128 x 128) += A(128 x K) B(128 x K)^T  of this file
// ---------------------------------------------------------------------------
// Operands are runs of consecutive workspace tiles (k-value k is column k % NB
// of tile k / NB: 128 rows of 128 contiguous bytes per panel of KT k-values, no
// edge masks, the workspace is padded) or one tile read as its transpose.
//
// Everything around the matrix instructions is kept off the vector ALU and
// placed between them by hand: the products are short (K = 128 .. 512) and run
// one or two workgroups per CU, so instructions that the compiler leaves in one
// block (the LDS stores and the global loads of the next panels, 90 instructions
// per pass with their address arithmetic) stall the matrix pipe with nothing
// else to fill it.
//   * global loads: wave-uniform base (scalar registers, advanced per pass) plus
//     a per-lane 32-bit offset that never changes;
//   * LDS: row-major panels with a row stride of KT + 4 floats, written and read
//     16 bytes at a time.  v_mfma_f32_32x32x2_f32 takes two k-values per
//     instruction, one from each half of the wave; which two does not matter as
//     long as both operands agree, so the lanes of half h read the four k-values
//     8g + 4h .. 8g + 4h + 3 of their row in one instruction and feed them to
//     four consecutive MFMAs (k pairs {8g + j, 8g + 4 + j});
//   * the LDS panels are double-buffered: one barrier per pass, and the stores
//     and loads for the passes ahead are dealt out one per group of four MFMAs.
// The global loads run PD passes ahead of the LDS stores (with less than two
// passes of 64 k-values in flight, a third of the passes of a full GPU waited
// 2-4 us for their operands, measured with time stamps).
typedef float vfloat4 __attribute__((ext_vector_type(4)));   // register arrays of HIP's float4 struct can end up in scratch

constexpr int RS = KT + 4;      // row stride of a row-major LDS panel (16-byte aligned rows; 8 lanes
                                // of a 16-byte access then cover all 32 banks)
constexpr int TS = NB + 4;      // k-row stride of a transposed LDS panel
constexpr int PF = NB * RS;     // floats per LDS panel
static_assert(KT * TS <= PF, "a transposed panel must fit the same buffer");
constexpr int kTileLdsFloats = 4 * PF;   // A even / odd pass, B even / odd pass
constexpr size_t kTileLdsBytes = kTileLdsFloats * sizeof(float);

// States that a pointer is the same in every lane, so that it is kept in scalar
// registers (the compiler cannot always see this through the table lookups).
__device__ __forceinline__ const float *wave_uniform(const float *p) {
  const unsigned long long v = reinterpret_cast<unsigned long long>(p);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  return reinterpret_cast<const float *>(((unsigned long long)hi << 32) | lo);
}

__device__ __forceinline__ vfloat4 gload16(const float *base, unsigned byte_off) {
  return *(const KFAC_GLOBAL_AS vfloat4 *)((const KFAC_GLOBAL_AS char *)base + byte_off);
}

__device__ __forceinline__ void gstore1(float *base, unsigned byte_off, float v) {
  *(KFAC_GLOBAL_AS float *)((KFAC_GLOBAL_AS char *)base + byte_off) = v;
}

// The accumulators <-> a row-major NB x NB tile at a wave-uniform address, as
// scalar base + one lane offset per group of eight elements + immediates (no
// 64-bit address per element).
__device__ __forceinline__ unsigned acc_lane_offset() {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row0 = (wave >> 1) * 64 + 4 * (lane >> 5), col0 = (wave & 1) * 64 + (lane & 31);
  return (unsigned)((row0 * NB + col0) * sizeof(float));
}
// acc = -C
__device__ __forceinline__ void load_neg_tile(const float *C, floatx16 (&acc)[2][2]) {
  const unsigned lane_off = acc_lane_offset();
#pragma unroll
  for (int im = 0; im < 2; ++im)
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      const unsigned o = lane_off + (unsigned)((im * 32 + 8 * vq) * NB * sizeof(float));
#pragma unroll
      for (int vr = 0; vr < 4; ++vr)
#pragma unroll
        for (int in = 0; in < 2; ++in)
          acc[im][in][vq * 4 + vr] = -gload1(C, o + (unsigned)((vr * NB + in * 32) * sizeof(float)));
    }
}
// C = -acc
__device__ __forceinline__ void store_neg_tile(float *C, const floatx16 (&acc)[2][2]) {
  const unsigned lane_off = acc_lane_offset();
#pragma unroll
  for (int im = 0; im < 2; ++im)
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      const unsigned o = lane_off + (unsigned)((im * 32 + 8 * vq) * NB * sizeof(float));
#pragma unroll
      for (int vr = 0; vr < 4; ++vr)
#pragma unroll
        for (int in = 0; in < 2; ++in)
          gstore1(C, o + (unsigned)((vr * NB + in * 32) * sizeof(float)), -acc[im][in][vq * 4 + vr]);
    }
}

// k along the rows of a run of consecutive tiles
struct OperandRows {
  const float *base;   // first tile of the run
  __device__ __forceinline__ static unsigned lane_offset() {
    return (unsigned)(((threadIdx.x >> 3) * NB + (threadIdx.x & 7) * 4) * sizeof(float));
  }
  __device__ __forceinline__ void load(vfloat4 (&r)[4], unsigned off, int pass) const {
    const int k = pass * KT;
    const float *b = wave_uniform(base + (size_t)(k / NB) * (NB * NB) + (k % NB));
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = gload16(b, off + i * (32 * NB * (unsigned)sizeof(float)));
  }
  __device__ __forceinline__ static void store1(const vfloat4 (&r)[4], int i, float *panel) {
    float *p = panel + (threadIdx.x >> 3) * RS + (threadIdx.x & 7) * 4;
    *reinterpret_cast<vfloat4 *>(p + 32 * i * RS) = r[i];
  }
  // the four k-values 8g + 4h .. + 3 of operand row `row`
  __device__ __forceinline__ static vfloat4 fetch4(const float *panel, int row, int g, int h) {
    return *reinterpret_cast<const vfloat4 *>(panel + row * RS + 8 * g + 4 * h);
  }
};

// one tile read as its transpose: operand row c, k-value q is element (q, c)
struct OperandCols {
  const float *base;
  __device__ __forceinline__ static unsigned lane_offset() {
    return (unsigned)(((threadIdx.x >> 5) * NB + (threadIdx.x & 31) * 4) * sizeof(float));
  }
  __device__ __forceinline__ void load(vfloat4 (&r)[4], unsigned off, int pass) const {
    const float *b = wave_uniform(base + pass * (KT * NB));
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = gload16(b, off + i * (8 * NB * (unsigned)sizeof(float)));
  }
  __device__ __forceinline__ static void store1(const vfloat4 (&r)[4], int i, float *panel) {
    float *p = panel + (threadIdx.x >> 5) * TS + (threadIdx.x & 31) * 4;
    *reinterpret_cast<vfloat4 *>(p + 8 * i * TS) = r[i];
  }
  __device__ __forceinline__ static vfloat4 fetch4(const float *panel, int row, int g, int h) {
    const float *p = panel + (8 * g + 4 * h) * TS + row;
    vfloat4 v;
    v.x = p[0];
    v.y = p[TS];
    v.z = p[2 * TS];
    v.w = p[3 * TS];
    return v;
  }
};

// One pass of KT k-values from the LDS panels `pa` / `pb` (both `pa` when SAME),
// ending with a barrier.  Beside the MFMAs it writes the register set `ra` /
// `rb` (the pass after this one) to the panels `na` / `nb`, then calls
// `refill_a()` / `refill_b()`, which load that register set again.
template <bool SAME, class LA, class LB, class FA, class FB>
__device__ __forceinline__ void tile_pass(const float *pa, const float *pb, float *na, float *nb,
                                          vfloat4 (&ra)[4], vfloat4 (&rb)[4],
                                          floatx16 (&acc)[2][2], FA refill_a, FB refill_b) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane & 31, lk = lane >> 5;
  vfloat4 fa[2], fb[2];
#pragma unroll
  for (int im = 0; im < 2; ++im) fa[im] = LA::fetch4(pa, (wm * 2 + im) * 32 + lrow, 0, lk);
#pragma unroll
  for (int in = 0; in < 2; ++in)
    fb[in] = SAME ? LA::fetch4(pa, (wn * 2 + in) * 32 + lrow, 0, lk)
                  : LB::fetch4(pb, (wn * 2 + in) * 32 + lrow, 0, lk);
#pragma unroll
  for (int g = 0; g < KT / 8; ++g) {
    vfloat4 ga[2], gb[2];
    if (g + 1 < KT / 8) {
#pragma unroll
      for (int im = 0; im < 2; ++im) ga[im] = LA::fetch4(pa, (wm * 2 + im) * 32 + lrow, g + 1, lk);
#pragma unroll
      for (int in = 0; in < 2; ++in)
        gb[in] = SAME ? LA::fetch4(pa, (wn * 2 + in) * 32 + lrow, g + 1, lk)
                      : LB::fetch4(pb, (wn * 2 + in) * 32 + lrow, g + 1, lk);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int im = 0; im < 2; ++im)
#pragma unroll
        for (int in = 0; in < 2; ++in)
          acc[im][in] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[im][j], fb[in][j], acc[im][in], 0, 0, 0);
      // slot 4g + j of 16: one LDS store at most (the last pass of a product stores what it
      // holds as well, into the buffer nobody reads any more: cheaper than a branch per store)
      const int slot = 4 * g + j;
      if (slot >= 1 && slot < 5) LA::store1(ra, slot - 1, na);
      if (!SAME && slot >= 5 && slot < 9) LB::store1(rb, slot - 5, nb);
    }
    if (g == 1) refill_a();               // after its stores (slots 1 .. 4)
    if (!SAME && g == 2) refill_b();      // slots 5 .. 8
    if (g + 1 < KT / 8) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[i] = ga[i];
        fb[i] = gb[i];
      }
    }
  }
  __syncthreads();
}

// K must be a multiple of 4 * KT.  lds: kTileLdsFloats.  Ends with a barrier.
template <bool SAME, int PD, class LA, class LB>
__device__ __forceinline__ void tile_mainloop(const LA &la, const LB &lb, int K, float *lds,
                                              floatx16 (&acc)[2][2]) {
  constexpr int UNROLL = PD % 2 == 0 ? PD : 2 * PD;   // register set and LDS buffer of a pass are static
  float *ldsA = lds, *ldsB = lds + 2 * PF;
  const int P = K / KT;
  const unsigned offA = LA::lane_offset(), offB = LB::lane_offset();
  vfloat4 ra[PD][4];
  vfloat4 rb[SAME ? 1 : PD][4];
#pragma unroll
  for (int q = 0; q < PD; ++q) {
    if (q < P) {
      la.load(ra[q], offA, q);
      if (!SAME) lb.load(rb[q], offB, q);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    LA::store1(ra[0], i, ldsA);
    if (!SAME) LB::store1(rb[0], i, ldsB);
  }
  if (PD < P) {
    la.load(ra[0], offA, PD);
    if (!SAME) lb.load(rb[0], offB, PD);
  }
  __syncthreads();
  for (int pb = 0; pb < P; pb += UNROLL) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int p = pb + u;
      if (UNROLL > 4 && p >= P) break;   // P is a multiple of 4
      const int r = (u + 1) % PD;            // register set of pass p + 1 (static once unrolled)
      const bool ahead = p + 1 + PD < P;     // which then takes pass p + 1 + PD
      tile_pass<SAME, LA, LB>(
          ldsA + (u & 1) * PF, ldsB + (u & 1) * PF, ldsA + ((u + 1) & 1) * PF, ldsB + ((u + 1) & 1) * PF,
          ra[r], rb[SAME ? 0 : r], acc,
          [&]() { if (ahead) la.load(ra[r], offA, p + 1 + PD); },
          [&]() { if (ahead) lb.load(rb[SAME ? 0 : r], offB, p + 1 + PD); });
    }
  }
}

// ---------------------------------------------------------------------------
// copy-in: lower tiles of in -> padded workspace (identity on the padding)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void copy_in_kernel(InvTables tb, int count, int tile0) {
  const int2 owner = tb.tile_owner[(int)blockIdx.x + tile0];
  const int s = owner.x, I = owner.y & 0xffff, J = owner.y >> 16;
  const int d = tb.dim[s], dc = tb.core[s];
  const float *__restrict__ src = tb.in[s];
  float *__restrict__ dst = tile_ptr(tb, s, I, J);
  const int c4 = (threadIdx.x & 31) * 4;
  const int r0 = threadIdx.x >> 5;
  // 16-byte loads at float granularity (the rows of an odd-sized matrix do not start on
  // 16-byte boundaries); the quads cut by the edge of the matrix go element by element
  typedef float floatx4u __attribute__((ext_vector_type(4), aligned(4)));
#pragma unroll 8
  for (int p = 0; p < NB / 8; ++p) {
    const int rl = r0 + 8 * p;
    const int r = I * NB + rl;
    const int c = J * NB + c4;
    float v[4];
    if (r < dc && c + 3 < dc) {
      const floatx4u x = *reinterpret_cast<const floatx4u *>(src + (long long)r * d + c);
      v[0] = x.x;
      v[1] = x.y;
      v[2] = x.z;
      v[3] = x.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int ce = c + e;
        float x = (r == ce) ? 1.f : 0.f;
        if (r < dc && ce < dc) x = src[(long long)r * d + ce];
        v[e] = x;
      }
    }
    *reinterpret_cast<float4 *>(dst + rl * NB + c4) = make_float4(v[0], v[1], v[2], v[3]);
  }
  // a bordered matrix: its last column and corner go beside the tiles
  const long long vo = tb.vec_off[s];
  if (vo >= 0 && I == J) {
    float *vec = tb.ws + vo;
    if (threadIdx.x < NB) vec[I * NB + threadIdx.x] = src[(long long)(I * NB + threadIdx.x) * d + d - 1];
    if (I == 0 && threadIdx.x == 0) vec[3 * (long long)dc] = src[(long long)(d - 1) * d + d - 1];   // scal[0]
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

// Diagonal tile (k,k) of a matrix: first the products it is still owed,
//   C(k,k) -= sum_{j = lo .. hi} M(k,j) M(k,j)^T        (nothing when K = 0),
// through the shared main loop (the other tiles of the column receive theirs
// from the update workgroups of the same launch), then the factorisation.
__device__ __forceinline__ void diag_role(const InvTables &tb, const TileTask &t, float *smem) {
  float *S = smem;                      // NB x LS working tile
  float *scratch = smem + NB * LS;      // 3 waves x SB x PS
  const int d = (int)(t.b_off >> 32);
  const int k = t.flags;
  constexpr int ld = NB;
  float *tile = tb.ws + t.c_off;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  if (t.K > 0) {
    floatx16 acc[2][2];
    fill_acc<2, 2>(acc, [&](int rr, int cc) { return -tile[rr * NB + cc]; });
    const OperandRows la{tb.ws + t.a_off};
    tile_mainloop<true, 2>(la, la, t.K, smem, acc);   // ends with a barrier
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
        int *pinfo = &tb.info[(int)(t.b_off & 0xffffffffLL)];
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
// Bordered matrices.  The Kronecker factor of a layer with a bias has d = 9C + 1
// or C + 1 rows: one more than a multiple of the tile size for every
// power-of-two C, which as a tiled matrix pays a whole extra tile row and column
// (4609 -> 37 tiles instead of 36; 11 % of the tile products of ResNet-50's
// factors).  Such a matrix M = [A a; a^T alpha] keeps its last row out of the
// tiles: the sweep factors the leading block A = L L^T, and the last row of M's
// Cholesky factor, l = L^-1 a, follows it as a vector, by the same block forward
// substitution that a tile row would go through,
//     l_k = U_kk^T (a_k - sum_{j<k} L(k,j) l_j),
// as do the last column of the triangular inverse and the last pivot,
//     w = U l = A^-1 a  (w_i = sum_{k >= i} U(i,k) l_k),   S = alpha - l^T l,
//     M^-1 = [A^-1 + w w^T / S, -w / S; -w^T / S, 1 / S].
// These are tile-by-vector products, a few workgroups per step that ride in the
// launches of the sweep: beside the diagonal tiles of step k the partial sums of
// sum_{j<k} L(k,j) l_j (chunks of kBorderChunk tiles) and w += U(.,k-1) l_{k-1},
// beside the panel step l_k itself.  (Forming l = U^T a from the finished inverse
// instead loses a factor of cond(L) in accuracy against the substitution.)  The
// rank-1 term is added to the accumulators of the final product.
// ---------------------------------------------------------------------------
constexpr int kBorderChunk = 6;
constexpr int kBorderSum = 0;     // part[j] = sum_{c in chunk j} L(i,c) l_c          (i = k, j = chunk)
constexpr int kBorderSolve = 1;   // l_i = U_ii^T (a_i - sum of the partial vectors)
constexpr int kBorderW = 2;       // w_i (+)= U(i,j) l_j, the first term (j = i) overwrites
constexpr int kBorderPivot = 3;   // S = alpha - l^T l in float64, 1 / S, info
struct BorderTask {
  int s, kind, i, j;
};
constexpr int kBorderLdsFloats = NB + NB * 33;

// vectors of a bordered matrix in the workspace: a | l | w | scalars (64) | partial vectors
struct BorderVecs {
  float *a, *y, *w, *scal, *part;
  int dc;
};
__device__ __forceinline__ BorderVecs border_vecs(const InvTables &tb, int s) {
  BorderVecs v;
  v.dc = tb.core[s];
  v.a = tb.ws + tb.vec_off[s];
  v.y = v.a + v.dc;
  v.w = v.y + v.dc;
  v.scal = v.w + v.dc;
  v.part = v.scal + 64;
  return v;
}

// p[r] += sum_{c in the thread's 4 columns} M[rg * 16 + r][c] x[c] for one NB x NB tile; x in LDS
__device__ __forceinline__ void border_rows_acc(const float *tile, const float *xs, float (&p)[16]) {
  const int c4 = (threadIdx.x & 31) * 4, rg = threadIdx.x >> 5;
  const float4 x = *reinterpret_cast<const float4 *>(xs + c4);
  const float *m = tile + (rg * 16) * NB + c4;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float4 u = *reinterpret_cast<const float4 *>(m + r * NB);
    p[r] += u.x * x.x + u.y * x.y + u.z * x.z + u.w * x.w;
  }
}
// the row sums of p over the 32 threads of a row group, in a fixed order; valid in threads < NB
__device__ __forceinline__ float border_rows_reduce(const float (&p)[16], float *red) {
  const int q = threadIdx.x & 31, rg = threadIdx.x >> 5;
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 16; ++r) red[(rg * 16 + r) * 33 + q] = p[r];
  __syncthreads();
  float t = 0.f;
  if (threadIdx.x < NB) {
#pragma unroll
    for (int i = 0; i < 32; ++i) t += red[threadIdx.x * 33 + i];
  }
  return t;
}

__device__ __forceinline__ void border_role(const InvTables &tb, const BorderTask t, float *lds) {
  float *xs = lds;         // NB floats
  float *red = lds + NB;   // NB x 33
  const BorderVecs v = border_vecs(tb, t.s);
  if (t.kind == kBorderSum) {
    float p[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) p[r] = 0.f;
    const int j_end = min((t.j + 1) * kBorderChunk, t.i);
    for (int j = t.j * kBorderChunk; j < j_end; ++j) {
      __syncthreads();
      if (threadIdx.x < NB) xs[threadIdx.x] = v.y[j * NB + threadIdx.x];
      __syncthreads();
      border_rows_acc(tile_ptr(tb, t.s, t.i, j), xs, p);
    }
    const float sum = border_rows_reduce(p, red);
    if (threadIdx.x < NB) v.part[t.j * NB + threadIdx.x] = sum;
  } else if (t.kind == kBorderSolve) {
    if (threadIdx.x < NB) {
      float x = v.a[t.i * NB + threadIdx.x];
      const int nch = (t.i + kBorderChunk - 1) / kBorderChunk;
      for (int ch = 0; ch < nch; ++ch) x -= v.part[ch * NB + threadIdx.x];
      xs[threadIdx.x] = x;
    }
    __syncthreads();
    // l_k[c] = sum_r U_kk[r][c] x[r]
    const int c4 = (threadIdx.x & 31) * 4, rg = threadIdx.x >> 5;
    const float *U = tile_ptr(tb, t.s, t.i, t.i) + (rg * 16) * NB + c4;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float4 u = *reinterpret_cast<const float4 *>(U + r * NB);
      const float xv = xs[rg * 16 + r];
      acc.x += u.x * xv;
      acc.y += u.y * xv;
      acc.z += u.z * xv;
      acc.w += u.w * xv;
    }
    *reinterpret_cast<float4 *>(red + rg * NB + c4) = acc;
    __syncthreads();
    if (threadIdx.x < NB) {
      float l = 0.f;
#pragma unroll
      for (int g = 0; g < 8; ++g) l += red[g * NB + threadIdx.x];
      v.y[t.i * NB + threadIdx.x] = l;
    }
  } else if (t.kind == kBorderW) {
    float p[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) p[r] = 0.f;
    if (threadIdx.x < NB) xs[threadIdx.x] = v.y[t.j * NB + threadIdx.x];
    __syncthreads();
    border_rows_acc(tile_ptr(tb, t.s, t.i, t.j), xs, p);
    const float sum = border_rows_reduce(p, red);
    if (threadIdx.x < NB) {
      float *w = v.w + t.i * NB + threadIdx.x;
      *w = t.j == t.i ? sum : *w + sum;
    }
  } else {
    double *dred = reinterpret_cast<double *>(lds);
    double sum = 0.0;
    for (int j = threadIdx.x; j < v.dc; j += THREADS) sum += (double)v.y[j] * (double)v.y[j];
    dred[threadIdx.x] = sum;
    __syncthreads();
    for (int w = THREADS / 2; w > 0; w >>= 1) {
      if ((int)threadIdx.x < w) dred[threadIdx.x] += dred[threadIdx.x + w];
      __syncthreads();
    }
    if (threadIdx.x == 0) {
      const double S = (double)v.scal[0] - dred[0];
      v.scal[1] = (float)S;
      v.scal[2] = (float)(1.0 / S);
      int *pinfo = &tb.info[tb.orig[t.s]];
      if (!(S > 0.0) && *pinfo == 0) *pinfo = tb.dim[t.s];
    }
  }
}

// the border tasks that follow the last step of the sweep
__global__ __launch_bounds__(THREADS) void border_kernel(InvTables tb, int btask0) {
  __shared__ __align__(16) float lds[kBorderLdsFloats];
  border_role(tb, tb.btasks[btask0 + blockIdx.x], lds);
}

// ---------------------------------------------------------------------------
// panel and update: 128x128x128 tile products through the shared main loop
// ---------------------------------------------------------------------------
// M(x,k) = M(x,k) W^T = M(x,k) U_kk in place for every x != k; the operand
// W^T is the diagonal tile itself, read transposed.
__global__ __launch_bounds__(THREADS, 2) void panel_kernel(InvTables tb, int task0, int ntask, int btask0) {
  extern __shared__ float lds[];
  if ((int)blockIdx.x >= ntask) {   // bordered matrices: l_k of this step
    border_role(tb, tb.btasks[btask0 + blockIdx.x - ntask], lds);
    return;
  }
  const TileTask t = tb.tasks[task0 + blockIdx.x];
  float *tile = tb.ws + t.c_off;
  floatx16 acc[2][2];
  zero_acc<2, 2>(acc);
  tile_mainloop<false, 2>(OperandRows{tile}, OperandCols{tb.ws + t.b_off}, NB, lds, acc);
  for_each_acc<2, 2>(acc, [&](int rr, int cc, float v) { tile[rr * NB + cc] = v; });
}

// One task of (*): tile (a,b) of a matrix, products over the block columns of
// the launch clipped to the tile's own range (resolved in the task record).  The
// accumulators start from -C, so the tile is read while the first operand panels
// are in flight and the epilogue is a plain store.  An upper tile whose row lies
// inside the source columns receives its first product here and is overwritten
// (it holds stale data): kFirst.
template <int D>
__device__ __forceinline__ void update_role(const InvTables &tb, const TileTask &t, float *lds) {
  float *C = const_cast<float *>(wave_uniform(tb.ws + t.c_off));
  floatx16 acc[2][2];
  if (t.flags & kFirst)
    zero_acc<2, 2>(acc);
  else
    load_neg_tile(C, acc);
  const OperandRows la{tb.ws + t.a_off}, lb{tb.ws + t.b_off};
  if (t.flags & kSame)
    tile_mainloop<true, D>(la, lb, t.K, lds, acc);
  else
    tile_mainloop<false, D>(la, lb, t.K, lds, acc);
  store_neg_tile(C, acc);
}

// One workgroup per active matrix: the diagonal tile of sweep step `step`
// (after it has received the products of columns [step0, step1]).  This is the
// serial part of the sweep, and most of it is one wave's dependent chain of
// vector instructions.  It runs at a third of its speed when its waves share
// their SIMDs with those of a trailing update (measured: 20 us against 60-80 us
// for the 128 x 128 factorisation), so the kernel asks for more LDS than fits
// beside a workgroup of the trailing update (kDiagKernelLds): it waits for a CU
// without one, at most the few microseconds until the next of them retires, and
// keeps the following ones away from that CU while it runs.
__global__ __launch_bounds__(THREADS, 2) void diag_kernel(InvTables tb, int task0, int ntask, int btask0) {
  extern __shared__ float lds[];
  if ((int)blockIdx.x >= ntask) {   // bordered matrices: the vector work this step can start with
    border_role(tb, tb.btasks[btask0 + blockIdx.x - ntask], lds);
    return;
  }
  const TileTask t = tb.tasks[task0 + blockIdx.x];
  diag_role(tb, t, lds);
}

// A list of tasks of (*): the column updates of a sweep step (the tiles the next
// panel step reads; beside the diagonal kernel) or the part of a trailing update
// that the next group's sweep does not read.
__global__ __launch_bounds__(THREADS, 2) void update_kernel(InvTables tb, int task0) {
  extern __shared__ float lds[];
  const TileTask t = tb.tasks[task0 + blockIdx.x];
  update_role<2>(tb, t, lds);
}

// out(i,j) = sum_{k >= i} U(i,k) U(j,k)^T for i >= j, written with its mirror.
// One task per tile; the table deals whole tile rows to XCDs (see the plan).
__global__ __launch_bounds__(THREADS, 2) void lauum_kernel(InvTables tb, int task0) {
  extern __shared__ float lds[];
  const TileTask t = tb.tasks[task0 + blockIdx.x];
  if (t.K == 0) return;   // padding of an XCD's shorter list
  const int s = (int)t.c_off;
  const int I = t.flags & 0xffff, J = t.flags >> 16;
  const int d = tb.dim[s], dc = tb.core[s];
  const long long vo = tb.vec_off[s];
  float *out = tb.out[s];
  const OperandRows la{tb.ws + t.a_off}, lb{tb.ws + t.b_off};
  floatx16 acc[2][2];
  zero_acc<2, 2>(acc);
  if (I == J)
    tile_mainloop<true, 4>(la, lb, t.K, lds, acc);
  else
    tile_mainloop<false, 4>(la, lb, t.K, lds, acc);
  if (vo >= 0) {
    // bordered matrix: + w w^T / S on the leading block, -w / S in the last row and column
    const BorderVecs bv = border_vecs(tb, s);
    const float sigma = bv.scal[2];
    const float *wi = bv.w + I * NB, *wj = bv.w + J * NB;
#pragma unroll
    for (int im = 0; im < 2; ++im)
#pragma unroll
      for (int in = 0; in < 2; ++in)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
          const int row = ((wave >> 1) * 2 + im) * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
          const int col = ((wave & 1) * 2 + in) * 32 + (lane & 31);
          acc[im][in][v] += sigma * wi[row] * wj[col];
        }
    if (I == J && threadIdx.x < NB) {
      const float b = -sigma * wi[threadIdx.x];
      out[(long long)(d - 1) * d + I * NB + threadIdx.x] = b;
      out[(long long)(I * NB + threadIdx.x) * d + d - 1] = b;
      if (I == 0 && threadIdx.x == 0) out[(long long)(d - 1) * d + d - 1] = sigma;
    }
  }
  // through LDS, so that the mirror is written in row segments too
  static_assert(kWholeTileLdsFloats <= kTileLdsFloats, "the tile must fit the panels' LDS");
  write_whole_tile(acc, lds, I, J, dc, d, out);
}

// Dynamic LDS.  The trailing update ("rest") asks for 81 KB although it uses 74:
// then one of its workgroups fits a CU, not two, and a column or panel workgroup
// of the sweep (74 KB) always finds room beside it instead of queueing behind
// the rest for a slot.  The diagonal kernel needs 77 KB (its working tile and
// three private blocks: at most three waves are busy in a pass of the triangular
// inverse) and asks for 80: two of its workgroups share a CU, but none shares
// one with a workgroup of the rest.
constexpr size_t kDiagLds = (size_t)(NB * LS + 3 * SB * PS) * sizeof(float);
constexpr size_t kRestLdsBytes = 81 * 1024;
constexpr size_t kDiagKernelLds = 80 * 1024;
static_assert(kDiagLds <= kDiagKernelLds && kTileLdsBytes <= kDiagKernelLds, "diagonal role's LDS");
static_assert(2 * kDiagKernelLds <= 160 * 1024 && kDiagKernelLds + kRestLdsBytes > 160 * 1024 &&
                  kDiagKernelLds + kTileLdsBytes <= 160 * 1024,
              "a diagonal workgroup shares a CU with another or with a column workgroup, not with the rest");
static_assert(2 * kRestLdsBytes > 160 * 1024 && kRestLdsBytes + kTileLdsBytes <= 160 * 1024,
              "one rest workgroup per CU, with room for a column or panel workgroup");

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
  std::vector<int> diag_task0, panel_task0;   // per step: first record of the launch
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
  // The column updates of a step are independent of its diagonal tiles: they run
  // on a third stream beside the diagonal kernel.
  hipStream_t col = nullptr;
  std::vector<hipEvent_t> ev_main, ev_side, ev_fork, ev_col;   // per step
  // The matrices that join the sweep at its first step are copied in on the caller's
  // stream; the others (they join later) on the side stream, beside the first step.
  int first_tiles = 0;
  hipEvent_t ev_copy_fork = nullptr, ev_copy = nullptr;
  ~kfac_inverse_plan() {
    for (hipEvent_t e : {ev_copy_fork, ev_copy})
      if (e) (void)hipEventDestroy(e);
    for (auto *v : {&ev_main, &ev_side, &ev_fork, &ev_col})
      for (hipEvent_t e : *v)
        if (e) (void)hipEventDestroy(e);
    if (side) (void)hipStreamDestroy(side);
    if (col) (void)hipStreamDestroy(col);
  }
  int total_tiles = 0;
  int lauum_task0 = 0, lauum_count = 0;
  // bordered matrices: their vector tasks per step (beside the diagonal tiles, beside the
  // panel step) and after the sweep
  int nborder = 0;
  std::vector<int> bdiag_task0, bdiag_count, bpanel_task0, bpanel_count;
  int bfinal_task0 = 0, bfinal_count = 0;
  kfac::DevTable d_core, d_orig, d_vec, d_btasks;
  size_t ws_floats = 0;            // padded matrices
  std::vector<const void *> in_sorted, out_sorted;
  kfac::DevTable d_in, d_out, d_dim, d_nt, d_off, d_tile, d_tile_owner, d_tasks;
  bool attr_set = false;
};

namespace {

// Workgroup i of a launch runs on XCD i % 8.  Deal the tasks out so that each
// XCD receives one contiguous run of the natural order (neighbouring tasks
// share operand row slabs, which then stay in that XCD's L2).
template <class T>
void append_tasks(std::vector<T> &table, const std::vector<T> &natural) {
  const size_t n = natural.size();
  const size_t chunk = (n + 7) / 8;
  std::vector<T> dealt;
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
  {   // tuning override
    const int g = kfac::option_int(kfac::kOptInverseGroup, p->group);
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
  // matrices of 128 m + 1 rows are inverted from their leading 128 m x 128 m block
  // (option inverse_border = 0 tiles them whole, for comparisons)
  const bool border_on = kfac::option_int(kfac::kOptInverseBorder, 1) != 0;
  std::vector<int> core(count);
  std::vector<long long> vec_off(count, -1);
  std::vector<int> border_slots;
  for (int s = 0; s < count; ++s) {
    dim[s] = dims[p->order[s]];
    core[s] = (border_on && dim[s] > NB && dim[s] % NB == 1) ? dim[s] - 1 : dim[s];
    const int T = kfac::ceil_div(core[s], NB);
    p->nt[s] = T;
    off[s] = (long long)total;
    total += (size_t)T * NB * T * NB;
    tile_cs[s + 1] = tile_cs[s] + T * (T + 1) / 2;
    panel_cs[s + 1] = panel_cs[s] + (T - 1);
  }
  for (int s = 0; s < count; ++s) {
    if (core[s] == dim[s]) continue;
    vec_off[s] = (long long)total;
    const int nch = (p->nt[s] - 1) / kBorderChunk + 1;
    total += (size_t)3 * core[s] + 64 + (size_t)nch * NB;
    border_slots.push_back(s);
  }
  p->nborder = (int)border_slots.size();
  p->ws_floats = total;
  p->total_tiles = tile_cs[count];
  p->first_tiles = tile_cs[count];   // set once the steps are known
  // copy-in: the lower tiles of every matrix in row-major order, slot by slot
  std::vector<int2> tile_owner;
  tile_owner.reserve((size_t)p->total_tiles);
  for (int s = 0; s < count; ++s)
    for (int I = 0; I < p->nt[s]; ++I)
      for (int J = 0; J <= I; ++J) tile_owner.push_back(make_int2(s, I | (J << 16)));
  p->max_t = count ? p->nt[0] : 0;
  std::vector<TileTask> tasks;
  std::vector<int2> natural;
  p->with_diag.resize(p->max_t);
  p->rest.resize(p->max_t);
  p->lookahead = kfac::option_int(kfac::kOptInverseLookahead, 1) != 0;
  // The rest asks for more LDS than it uses, 81 KB: then one of its workgroups
  // fits a CU, not two, and a step or panel workgroup always finds room beside
  // it instead of queueing behind the rest for a slot (measured: the rest alone
  // loses 14 %, the sweep as a whole gains).  Option inverse_rest_lds overrides.
  p->rest_lds = kRestLdsBytes;
  {
    const long v = (long)kfac::option_value(kfac::kOptInverseRestLds, 0.0);
    if (v >= (long)kTileLdsBytes && v <= 160 * 1024) p->rest_lds = (size_t)v;
  }
  auto pack = [](int s, int a, int b) { return make_int2(s, a | (b << 16)); };
  // Matrix s joins the sweep at step shift[s] and runs nt[s] steps.  Aligning
  // the ends (shift = max_t - nt) puts the short sweeps of the small matrices
  // beside the late steps of the largest ones, which on their own leave most of
  // the GPU idle (few tiles, one dependent launch after another); aligning the
  // starts piles all matrices onto the early steps, which are the ones that are
  // already throughput-bound.  Option inverse_align = <percent> (0 = starts, 100 =
  // ends) is a tuning override.
  int align = 100;
  align = std::min(100, std::max(0, kfac::option_int(kfac::kOptInverseAlign, align)));
  std::vector<int> shift(count);
  for (int s = 0; s < count; ++s) shift[s] = (p->max_t - p->nt[s]) * align / 100;
  std::vector<BorderTask> btasks;
  // step g, bordered matrix s at its block column k = g - shift: beside the diagonal tiles the
  // chunks of sum_{j<k} L(k,j) l_j and w_i (+)= U(i,k-1) l_{k-1} (k = nt: only the latter);
  // beside the panel step l_k
  for (int g = 0; g <= p->max_t; ++g) {
    const int first = (int)btasks.size();
    for (int s : border_slots) {
      const int k = g - shift[s], T = p->nt[s];
      if (k < 1 || k > T) continue;
      if (k < T)
        for (int ch = 0; ch * kBorderChunk < k; ++ch) btasks.push_back(BorderTask{s, kBorderSum, k, ch});
      for (int i = 0; i < k; ++i) btasks.push_back(BorderTask{s, kBorderW, i, k - 1});
    }
    if (g < p->max_t) {
      p->bdiag_task0.push_back(first);
      p->bdiag_count.push_back((int)btasks.size() - first);
      const int pfirst = (int)btasks.size();
      for (int s : border_slots) {
        const int k = g - shift[s];
        if (k >= 0 && k < p->nt[s]) btasks.push_back(BorderTask{s, kBorderSolve, k, 0});
      }
      p->bpanel_task0.push_back(pfirst);
      p->bpanel_count.push_back((int)btasks.size() - pfirst);
    } else {
      // after the sweep: the last terms of w and the pivots
      for (int s : border_slots) btasks.push_back(BorderTask{s, kBorderPivot, 0, 0});
      p->bfinal_task0 = first;
      p->bfinal_count = (int)btasks.size() - first;
    }
  }
  if (btasks.empty()) btasks.push_back(BorderTask{0, 0, 0, 0});
  auto tile_off = [&](int s, int I, int J) {
    return off[s] + ((long long)I * p->nt[s] + J) * (long long)(NB * NB);
  };
  // tile (a,b) of a matrix receives the products of the sweep steps [step0, step1]: those of
  // them that are block columns of this matrix (one that starts inside the range has fewer)
  // and lie inside the tile's own range
  auto resolve = [&](const std::vector<int2> &list, int step0, int step1) {
    std::vector<TileTask> out;
    out.reserve(list.size());
    for (const int2 &t : list) {
      const int s = t.x, a = t.y & 0xffff, b = t.y >> 16;
      const int k0 = step0 > shift[s] ? step0 - shift[s] : 0, k1 = step1 - shift[s];
      const bool upper = a < b;
      const int j_lo = upper && a > k0 ? a : k0;
      const int j_hi = upper && b - 1 < k1 ? b - 1 : k1;
      TileTask r;
      r.c_off = tile_off(s, a, b);
      r.a_off = tile_off(s, a, j_lo);
      r.b_off = tile_off(s, b, j_lo);
      r.K = (j_hi - j_lo + 1) * NB;
      r.flags = (upper && a >= k0 ? kFirst : 0) | (a == b ? kSame : 0);
      out.push_back(r);
    }
    return out;
  };
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
    if (g == 0) p->first_tiles = tile_cs[na];
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
    append_tasks(tasks, resolve(natural, w.k0, w.k1));
    append_tasks(tasks, resolve(tail, w.k0, w.k1));
    // the diagonal tiles of the step, which take the same columns' products themselves
    p->diag_task0.push_back((int)tasks.size());
    for (int s = 0; s < na; ++s) {
      const int k = g - shift[s];
      const int k0 = w.k0 > shift[s] ? w.k0 - shift[s] : 0, k1 = w.k1 - shift[s];
      TileTask r;
      r.c_off = tile_off(s, k, k);
      r.a_off = tile_off(s, k, k0);
      r.b_off = (long long)p->order[s] | ((long long)core[s] << 32);
      r.K = k1 >= k0 ? (k1 - k0 + 1) * NB : 0;
      r.flags = k;
      tasks.push_back(r);
    }
    // and the panel step: every other tile of block column k times U_kk
    p->panel_task0.push_back((int)tasks.size());
    {
      std::vector<TileTask> panel;
      for (int s = 0; s < na; ++s) {
        const int k = g - shift[s];
        for (int x = 0; x < p->nt[s]; ++x) {
          if (x == k) continue;
          TileTask r;
          r.c_off = r.a_off = tile_off(s, x, k);
          r.b_off = tile_off(s, k, k);
          r.K = NB;
          r.flags = 0;
          panel.push_back(r);
        }
      }
      tasks.insert(tasks.end(), panel.begin(), panel.end());
    }
    if (g == g1 && g1 + 1 < p->max_t) {
      natural.clear();
      tail.clear();
      trailing(false, g0, g1, natural, tail);
      UpdateLaunch &u = p->rest[g];
      u.task0 = (int)tasks.size();
      u.count = (int)(natural.size() + tail.size());
      u.k0 = g0;
      u.k1 = g1;
      append_tasks(tasks, resolve(natural, u.k0, u.k1));
      append_tasks(tasks, resolve(tail, u.k0, u.k1));
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
    std::vector<TileTask> list[8];
    size_t longest = 0;
    for (int x = 0; x < 8; ++x) {
      std::stable_sort(mine[x].begin(), mine[x].end(), [&](const Row &a, const Row &b) {
        return p->nt[a.s] - a.I > p->nt[b.s] - b.I;
      });
      for (const Row &r : mine[x])
        for (int J = 0; J <= r.I; ++J) {
          TileTask t;
          t.c_off = r.s;
          t.a_off = tile_off(r.s, r.I, r.I);
          t.b_off = tile_off(r.s, J, r.I);
          t.K = (p->nt[r.s] - r.I) * NB;
          t.flags = r.I | (J << 16);
          list[x].push_back(t);
        }
      longest = std::max(longest, list[x].size());
    }
    p->lauum_task0 = (int)tasks.size();
    for (size_t i = 0; i < longest; ++i)
      for (int x = 0; x < 8; ++x)
        tasks.push_back(i < list[x].size() ? list[x][i] : TileTask{0, 0, 0, 0, 0});
    p->lauum_count = (int)(longest * 8);
  }
  if (tasks.empty()) tasks.push_back(TileTask{0, 0, 0, 0, 0});
  int rc = KFAC_OK;
  auto up = [&](kfac::DevTable &t, const void *h, size_t b) {
    if (rc == KFAC_OK) rc = t.set_sync(h, b);
  };
  up(p->d_dim, dim.data(), sizeof(int) * count);
  up(p->d_core, core.data(), sizeof(int) * count);
  up(p->d_orig, p->order.data(), sizeof(int) * count);
  up(p->d_vec, vec_off.data(), sizeof(long long) * count);
  up(p->d_btasks, btasks.data(), sizeof(BorderTask) * btasks.size());
  up(p->d_nt, p->nt.data(), sizeof(int) * count);
  up(p->d_off, off.data(), sizeof(long long) * count);
  up(p->d_tile, tile_cs.data(), sizeof(int) * (count + 1));
  up(p->d_tile_owner, tile_owner.data(), sizeof(int2) * tile_owner.size());
  up(p->d_tasks, tasks.data(), sizeof(TileTask) * tasks.size());
  if (rc == KFAC_OK && p->lookahead && p->max_t > p->group) {
    const bool real = !kfac::host_only();   // host-only mode: null handles that nothing ever uses
    bool ok = !real || (hipStreamCreateWithFlags(&p->side, hipStreamNonBlocking) == hipSuccess &&
                        hipStreamCreateWithFlags(&p->col, hipStreamNonBlocking) == hipSuccess);
    for (int g = 0; ok && g < p->max_t; ++g)
      for (auto *v : {&p->ev_main, &p->ev_side, &p->ev_fork, &p->ev_col}) {
        hipEvent_t e = nullptr;
        ok = ok && (!real || hipEventCreateWithFlags(&e, hipEventDisableTiming) == hipSuccess);
        if (ok) v->push_back(e);
      }
    for (hipEvent_t *e : {&p->ev_copy_fork, &p->ev_copy})
      ok = ok && (!real || hipEventCreateWithFlags(e, hipEventDisableTiming) == hipSuccess);
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
  if (lookahead && !plan->capture_origin && !kfac::host_only()) {
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
    KFAC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(diag_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)kDiagKernelLds));
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
  tb.dim = plan->d_dim.as<const int>();
  tb.core = plan->d_core.as<const int>();
  tb.orig = plan->d_orig.as<const int>();
  tb.vec_off = plan->d_vec.as<const long long>();
  tb.nt = plan->d_nt.as<const int>();
  tb.ws_off = plan->d_off.as<const long long>();
  tb.tile_cs = plan->d_tile.as<const int>();
  tb.tile_owner = plan->d_tile_owner.as<const int2>();
  tb.tasks = plan->d_tasks.as<const TileTask>();
  tb.btasks = plan->d_btasks.as<const BorderTask>();
  uintptr_t base = (reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255;
  tb.ws = reinterpret_cast<float *>(base);
  tb.info = info_dev;

  kfac::TimedLaunch timed_call(KFAC_TIMED_INV_CALL, s);   // copy-in to the final product (the side streams rejoin `s`)
  // copy-in: what the first step needs on `s`, the rest beside it on the side stream
  const int late_tiles = lookahead ? plan->total_tiles - plan->first_tiles : 0;
  if (late_tiles > 0) {
    KFAC_HIP_CHECK(hipEventRecord(plan->ev_copy_fork, s));
    KFAC_HIP_CHECK(hipStreamWaitEvent(plan->side, plan->ev_copy_fork, 0));
    KFAC_LAUNCH(copy_in_kernel, dim3(late_tiles), dim3(256), 0, plan->side, tb, count, plan->first_tiles);
    KFAC_HIP_CHECK(hipEventRecord(plan->ev_copy, plan->side));
  }
  if (plan->total_tiles - late_tiles > 0)
    KFAC_LAUNCH(copy_in_kernel, dim3(plan->total_tiles - late_tiles), dim3(256), 0, s, tb, count, 0);
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
      KFAC_LAUNCH(update_kernel, dim3(r.count), dim3(THREADS), plan->rest_lds, st, tb,
                         r.task0);
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
    // the matrices that join from the second step on have been copied in by then
    if (k == 1 && late_tiles > 0) KFAC_HIP_CHECK(hipStreamWaitEvent(s, plan->ev_copy, 0));
    // A group's first step applies the previous group to this group's columns,
    // tiles that the rest of the group before that one (two back) also updated.
    // The rest of the previous group itself only touches columns further right
    // and runs beside this group's sweep.
    const int two_back = k - 1 - plan->group;
    if (lookahead && k % plan->group == 0 && two_back >= 0 && plan->rest[two_back].count > 0)
      KFAC_HIP_CHECK(hipStreamWaitEvent(s, plan->ev_side[two_back], 0));
    if (!lookahead)
      if (int rc2 = queue_rest()) return rc2;   // one stream: keep the program order
    // the diagonal tiles on `s`, the column updates beside them
    hipStream_t cs = s;
    if (lookahead && w.count > 0) {
      KFAC_HIP_CHECK(hipEventRecord(plan->ev_fork[k], s));
      KFAC_HIP_CHECK(hipStreamWaitEvent(plan->col, plan->ev_fork[k], 0));
      cs = plan->col;
    }
    KFAC_LAUNCH(diag_kernel, dim3(na + plan->bdiag_count[k]), dim3(THREADS), kDiagKernelLds, s, tb,
                       plan->diag_task0[k], na, plan->bdiag_task0[k]);
    if (w.count > 0) {
      kfac::TimedLaunch timed(KFAC_TIMED_INV_UPDATE, cs);
      KFAC_LAUNCH(update_kernel, dim3(w.count), dim3(THREADS), kTileLdsBytes, cs, tb, w.task0);
    }
    if (cs != s) {
      KFAC_HIP_CHECK(hipEventRecord(plan->ev_col[k], cs));
      KFAC_HIP_CHECK(hipStreamWaitEvent(s, plan->ev_col[k], 0));
    }
    if (int rc2 = queue_rest()) return rc2;
    if (plan->panel_total[k] + plan->bpanel_count[k] > 0)
      KFAC_LAUNCH(panel_kernel, dim3(plan->panel_total[k] + plan->bpanel_count[k]), dim3(THREADS),
                         kTileLdsBytes, s, tb, plan->panel_task0[k], plan->panel_total[k],
                         plan->bpanel_task0[k]);
    if (plan->rest[k].count == 0) continue;
    if (lookahead) KFAC_HIP_CHECK(hipEventRecord(plan->ev_main[k], s));
    deferred = k;
  }
  if (int rc2 = queue_rest()) return rc2;
  if (pending >= 0) KFAC_HIP_CHECK(hipStreamWaitEvent(s, plan->ev_side[pending], 0));
  KFAC_HIP_CHECK(hipGetLastError());
  if (plan->bfinal_count > 0) {
    KFAC_LAUNCH(border_kernel, dim3(plan->bfinal_count), dim3(THREADS), 0, s, tb, plan->bfinal_task0);
    KFAC_HIP_CHECK(hipGetLastError());
  }
  {
    kfac::TimedLaunch timed(KFAC_TIMED_INV_LAUUM, s);
    KFAC_LAUNCH(lauum_kernel, dim3(plan->lauum_count), dim3(THREADS), kTileLdsBytes, s, tb,
                       plan->lauum_task0);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

