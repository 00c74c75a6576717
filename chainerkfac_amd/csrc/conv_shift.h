// The A factor of a 3x3, stride-1, padding-1 convolution from shifted
// correlations of the input instead of a product of patch matrices.
//
// With X zero outside the image and rows (c, i, j) of the patch matrix,
//   A[(c,i,j), (c',i',j')] = sum_{n, y, x} X(c, y+i-1, x+j-1) X(c', y+i'-1, x+j'-1)
//                          = sum_{n} sum_{u in U_i, v in V_j} X(c, u, v) X(c', u+di, v+dj),
// di = i'-i, dj = j'-j, where u = y+i-1 runs over U_i = all image rows but one at
// the border (i = 0: not the last row, i = 2: not the first, i = 1: all), and V_j
// likewise for the columns.  So every entry is a shifted correlation over the
// whole image,
//   S(di,dj)[c,c'] = sum_{n,u,v} X(c, u, v) X(c', u+di, v+dj),
// minus what the excluded row and column contribute (inclusion - exclusion).  The
// excluded row is the first or last of the image and its partner row u+di lies
// outside the image unless di = 0 (the same for columns), so the corrections are
//   i = 2, di = 0:  - R_first(dj)      i = 0, di = 0:  - R_last(dj)
//   j = 2, dj = 0:  - C_first(di)      j = 0, dj = 0:  - C_last(di)
//   di = dj = 0 and both excluded:     + the corner pixel's product,
// with R_u0(dj)[c,c'] = sum_{n,v} X(c,u0,v) X(c',u0,v+dj) over one image row and
// C_v0(di) over one image column.  S(-d) = S(d)^T, R(-dj) = R(dj)^T, C(-di) =
// C(di)^T: 13 + 6 + 6 + 4 = 29 products of C x C, of which the 13 over whole images
// carry the work: 26 C^2 M flop instead of the 81 C^2 M of the patch product
// (M = n H W).  The ones column follows from per-channel sums the same way.
// Reference semantics: chainerkfac/optimizers/fisher_blocks/connections/convolution_2d.py:19-56
// (im2col, A = col^T col / n, the ones column of _bias).
#pragma once

#include "mma_core.h"

namespace kfac {
namespace mma {

// First operand of a group of products: rows = channels, k = (sample, p), p < L
// running over the group's domain (a whole image, one image row, one border column
// or one pixel):
//   element = base[sample * sample_stride + row * row_stride + (p / line_len) * line_stride + p % line_len],
// 0 for rows >= rows_valid and k past the end of the slice.  Dword loads, the 32
// lanes of a half-wave on 32 consecutive k of one row (the layout of LoaderKC's
// scalar variant).
template <int ROWS>
struct LoaderDomain {
  static constexpr bool kKRow = false;
  static constexpr int NR = ROWS / 8;   // rows per thread
  struct Regs {
    float v[NR];
    bool kvalid;
  };
  const float *base;
  unsigned sample_stride, row_stride;
  unsigned L, line_len, line_stride;
  int rows_valid;
  int first_row;
  unsigned last_off;

  __device__ __forceinline__ void init(int row0) {
    first_row = row0 + (team_tid() >> 5);
    last_off = (unsigned)(rows_valid > 0 ? rows_valid - 1 : 0) * row_stride;
  }

  __device__ __forceinline__ void load(Regs &r, long long k0, long long k_end) const {
    const long long kg = k0 + (team_tid() & 31);
    r.kvalid = kg < k_end;
    const unsigned kc = r.kvalid ? (unsigned)kg : 0u;
    const unsigned s = kc / L;
    const unsigned p = kc - s * L;
    const unsigned a = p / line_len;
    const unsigned koff = s * sample_stride + a * line_stride + (p - a * line_len);
    int fr = first_row;
    asm volatile("" : "+v"(fr));   // keep the NR row offsets out of registers (see LoaderKC)
    const unsigned off0 = (unsigned)fr * row_stride;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const unsigned off = off0 + (unsigned)(8 * i) * row_stride;
      r.v[i] = gload1(base, (koff + (off < last_off ? off : last_off)) * 4u);
    }
  }

  __device__ __forceinline__ void store(const Regs &r, float *lds) const {
    float *p = lds + (team_tid() >> 5) * Panel<ROWS>::kRowKStride + (team_tid() & 31);
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = first_row + 8 * i;
      p[8 * i * Panel<ROWS>::kRowKStride] = (r.kvalid && row < rows_valid) ? r.v[i] : 0.f;
    }
  }
};

}  // namespace mma
}  // namespace kfac

namespace kfac {
namespace shift {

using namespace kfac::mma;

// Arrays of C x C that the assembly kernel reads, every one stored both ways
// round (offset d and offset -d = its transpose) so that a row of the factor
// only reads rows of them:
//   [0, 25)   S(di, dj), index (di + 2) * 5 + dj + 2
//   [25, 35)  R_first(dj), R_last(dj): 25 + 5 * last + dj + 2
//   [35, 45)  C_first(di), C_last(di): 35 + 5 * last + di + 2
//   [45, 49)  corner pixels: 45 + 2 * (last row) + (last column)
constexpr int kArrays = 49;
constexpr int kProducts = 29;
constexpr int kGroups = 11;
constexpr int kChannelSums = 9;   // whole image, first / last row, first / last column, 4 corners

// Products that share their first operand and differ in the second operand's
// shift along the domain are computed together, ns (3 or 5) at a time.  A domain
// is a set of pixels per sample, numbered p < L: the whole image (three groups,
// one per row shift di: column shifts 0..2 for di = 0, whose negative ones are
// transposes, and -2..2 for di = 1, 2), the first or last image row (column shifts
// 0..2), the first or last image column (row shifts 0..2, which move along the
// column) or one corner pixel.
//   memory:  pixel p of sample s, channel c at
//            base[s * sample_stride + c * row_stride + (p / mem_line) * line_stride + p % mem_line]
//   shift e (= dj0 + 0 .. ns - 1) of row shift di:  p -> p + di * vline + e, inside the
//   domain if  p / vline + di < amax  and  0 <= p % vline + e < vline
// The whole image and its first / last row are read from the input tensor; the
// first / last column and the corners from a compact copy of the two border columns
// ([2][n][C][H], written by edge_sums_kernel), where a column is contiguous.
// Layers of at most 32 channels would fill a quarter of a 64 x 64 tile.  Their
// whole-image groups are `stacked`: the 64 first-operand rows are the channels at
// row shift 0 and, 32 rows on, the same channels one image row up (X(c, u - 1, v):
// against a second operand at row shift di that is the product of row shift di + 1),
// the 64 second-operand rows the channels and, 32 rows on, the same channels three
// columns on -- so the four 32 x 32 blocks of a tile and its three column offsets
// are the products of row shifts di, di + 1 and column shifts dj0 .. dj0 + 5.
// stacked = 2: both first-operand halves; 1: only the first (the waves of the
// second issue no matrix instructions); 0: plain rows = channels.
struct ShiftGroup {
  const float *base;
  unsigned sample_stride, row_stride, line_stride;
  unsigned L, mem_line, vline;
  short di, dj0, ns, amax;
  int stacked;
  int K;               // reduction length: samples * L
  int klen, nsplit;    // k-values per slice (a multiple of KT), slices
  int task0;           // first work item of the group
  unsigned part_off;   // its partial tiles: [item][shift][rows of the A tile][64]
};

// Where the slices of one product's partial sums lie in the workspace, element
// (row, col) of slice s at  part_off + s * split_stride
//   + ((row / tile_rows) * tiles_j + col / 64) * tile_stride + (row % tile_rows) * 64 + col % 64,
// and the arrays it becomes.
struct Product {
  unsigned part_off, split_stride, tile_stride;
  int nsplit;
  short out, out_t;    // array written as it is / transposed (equal: symmetric product)
};

struct Plan {
  const float *x;
  unsigned sample_stride, row_stride;   // C H W, H W
  int C, H, W, n;
  int tiles_a, tiles_b;     // tile grid: 64 * WM first-operand channels x 64 second-operand channels
  int nsmall, total;        // work items of the groups 3.. (strips and corners), and of all groups
  ShiftGroup grp[kGroups];
  Product prod[kProducts];
};

// Consecutive workgroup ids go round-robin to the 8 XCDs; each XCD takes a
// contiguous run of the item list, in which the tiles of one slice of one group
// follow each other (they share operand panels).
__device__ __forceinline__ int item_of_block(int bid, int total) {
  const int xcd = bid % 8, idx = bid / 8;
  const int base = total / 8, rem = total % 8;
  return xcd * base + (xcd < rem ? xcd : rem) + idx;
}

// k runs over (sample, pixel of the domain).  The workgroup stages 32 k-values of
// its 64 * WM first-operand channels and the 36 values from di * vline - 2 places on
// of its 64 second-operand channels; the NS shifts read the latter at NS
// consecutive offsets.  Where a shifted pixel falls outside the domain is the same
// for all channels: one 32-bit mask per shift and panel, applied to the operand
// values as they are read (as 64-bit lane masks in scalar registers: one select
// per value).  Per panel a wave issues 16 * WM * NS matrix instructions for
// (8 * WM + 9) global loads of its lanes; one product at a time (WM * WM
// instructions for 16 * WM loads per step) is bound by the loads.
constexpr int kShiftCols = 36;
constexpr int kShiftStride = 37;   // odd: the 32 rows of an operand read on 32 banks

template <int WM, int NS, bool STACKED = false>
__device__ __forceinline__ void corr_shifts_body(const Plan &pl, const ShiftGroup &g, int q, float *lds,
                                                 float *__restrict__ partial) {
  static_assert(!STACKED || WM == 1, "stacked groups use 64-row tiles");
  constexpr int BMA = 64 * WM;
  float *ldsA = lds, *ldsB = lds + Panel<BMA>::kFloats;
  const int ntile = pl.tiles_a * pl.tiles_b;
  const int split = q / ntile, tile = q - split * ntile;
  const int I = tile / pl.tiles_b, J = tile - I * pl.tiles_b;
  const unsigned L = g.L, mem_line = g.mem_line, vline = g.vline;
  const int K = g.K;
  LoaderDomain<BMA> la;
  la.base = g.base;
  la.sample_stride = g.sample_stride;
  la.row_stride = g.row_stride;
  la.L = L;
  la.line_len = mem_line;
  la.line_stride = g.line_stride;
  la.rows_valid = pl.C;
  la.init(I * BMA);
  if (STACKED) {   // all of a thread's rows are rows of one half: channel = row % 32
    la.first_row = team_tid() >> 5;
    la.rows_valid = pl.C;
  }
  const int tid = team_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane & 31, lk = lane >> 5;
  // second operand: 32 columns x 8 row passes, then 4 columns x 64 rows
  const int jm = tid & 31, rm = tid >> 5;
  const int je = 32 + (tid & 3), re = tid >> 2;
  const int shift = g.di * (int)vline - 2;
  unsigned rowoff[8];
  unsigned rowok = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = STACKED ? (rm + 8 * i) & 31 : J * 64 + rm + 8 * i;
    rowoff[i] = (unsigned)(row < pl.C ? row : pl.C - 1) * g.row_stride;
    if (row < pl.C) rowok |= 1u << i;
  }
  const int rowe = STACKED ? re & 31 : J * 64 + re;
  const unsigned rowoff_e = (unsigned)(rowe < pl.C ? rowe : pl.C - 1) * g.row_stride;
  const long long kbeg = (long long)split * g.klen;
  long long kend = kbeg + g.klen;
  if (kend > K) kend = K;
  floatx16 acc[NS][WM];
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int im = 0; im < WM; ++im)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[s][im][v] = 0.f;
  typename LoaderDomain<BMA>::Regs ra;
  float rb[9];
  auto load_b = [&](long long k0) {
    auto offset_of = [&](int j) {
      long long kk = k0 + shift + j;
      kk = kk < 0 ? 0 : (kk >= K ? K - 1 : kk);   // any element of the tensor will do: masked when read
      const unsigned ku = (unsigned)kk, s = ku / L, p = ku - s * L;
      const unsigned line = p / mem_line;
      return s * g.sample_stride + line * g.line_stride + (p - line * mem_line);
    };
    const unsigned om = offset_of(jm), oe = offset_of(je + (STACKED && re >= 32 ? 3 : 0));
    const unsigned om1 = STACKED ? offset_of(jm + 3) : om;   // rows 32..: three columns on
#pragma unroll
    for (int i = 0; i < 8; ++i) rb[i] = gload1(g.base, ((STACKED && i >= 4 ? om1 : om) + rowoff[i]) * 4u);
    rb[8] = gload1(g.base, (oe + rowoff_e) * 4u);
  };
  // first operand of a stacked group: rows 32.. are the channels one image row up
  auto load_a = [&](long long k0) {
    if (!STACKED) {
      la.load(ra, k0, kend);
      return;
    }
    const long long kg = k0 + jm;
    ra.kvalid = kg < kend;
    const long long kc = ra.kvalid ? kg : 0;
    auto offset_at = [&](long long kk) {
      const unsigned ku = (unsigned)(kk < 0 ? 0 : kk), s = ku / L, p = ku - s * L;
      return s * g.sample_stride + p;   // whole images: pixels are contiguous
    };
    const unsigned o0 = offset_at(kc), o1 = offset_at(kc - (long long)vline);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = (rm + 8 * i) & 31;
      ra.v[i] = gload1(g.base, ((i >= 4 ? o1 : o0) + (unsigned)(row < pl.C ? row : pl.C - 1) * g.row_stride) * 4u);
    }
  };
  auto store_a = [&]() {
    if (!STACKED) {
      la.store(ra, ldsA);
      return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
      ldsA[(rm + 8 * i) * Panel<BMA>::kRowKStride + jm] = (ra.kvalid && ((rm + 8 * i) & 31) < pl.C) ? ra.v[i] : 0.f;
  };
  if (kbeg < kend) {
    load_a(kbeg);
    load_b(kbeg);
  }
  for (long long k0 = kbeg; k0 < kend; k0 += KT) {
    store_a();
#pragma unroll
    for (int i = 0; i < 8; ++i) ldsB[(rm + 8 * i) * kShiftStride + jm] = ((rowok >> i) & 1u) ? rb[i] : 0.f;
    ldsB[re * kShiftStride + je] = rowe < pl.C ? rb[8] : 0.f;
    __syncthreads();
    if (k0 + KT < kend) {
      load_a(k0 + KT);
      load_b(k0 + KT);
    }
    // validity of the NS shifted pixels of this panel's 32 k-values: bit k of m[s]
    unsigned m[NS];
    {
      const long long kg = k0 + (lane & 31);
      const unsigned kc = kg < kend ? (unsigned)kg : 0u;
      const unsigned pix = kc % L;
      const unsigned a = pix / vline, b = pix - a * vline;
      // stacked: this wave's blocks are row shift di + wm (first operand one row up:
      // not for the first image row) and column shifts dj0 + 3 wn + s
      const bool row_in = kg < kend && (int)a + g.di < g.amax && (!STACKED || (int)a >= wm);
      const int dj_first = g.dj0 + (STACKED ? 3 * wn : 0);
#pragma unroll
      for (int s = 0; s < NS; ++s)
        m[s] = __builtin_amdgcn_readfirstlane(
            (unsigned)__ballot(row_in && (unsigned)((int)b + dj_first + s) < vline));
    }
    const bool active = !STACKED || wm < g.stacked;
    const float *pa = ldsA + (wm * WM * 32 + lrow) * Panel<BMA>::kRowKStride + lk;
    const float *pb = ldsB + (wn * 32 + lrow) * kShiftStride + lk + 2 + g.dj0;
    // operands of step kk + 1 are read from LDS before the matrix instructions of
    // step kk issue (the scheduling barriers keep the compiler from sinking the
    // reads to their first use, which would expose the LDS latency in every step)
    float a[2][WM], b[2][NS];
#pragma unroll
    for (int im = 0; im < WM; ++im) a[0][im] = pa[im * 32 * Panel<BMA>::kRowKStride];
#pragma unroll
    for (int s = 0; s < NS; ++s) b[0][s] = pb[s];
    if (active) {
#pragma unroll
    for (int kk = 0; kk < KT / 2; ++kk) {
      const int cur = kk & 1, nxt = cur ^ 1;
      if (kk + 1 < KT / 2) {
#pragma unroll
        for (int im = 0; im < WM; ++im) a[nxt][im] = pa[im * 32 * Panel<BMA>::kRowKStride + 2 * kk + 2];
#pragma unroll
        for (int s = 0; s < NS; ++s) b[nxt][s] = pb[2 * kk + 2 + s];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        // lanes 0..31 hold k = 2 kk, lanes 32..63 k = 2 kk + 1: the lane mask of the
        // valid ones, built from two bits of the panel's mask in scalar registers
        const unsigned lo = 0u - ((m[s] >> (2 * kk)) & 1u), hi = 0u - ((m[s] >> (2 * kk + 1)) & 1u);
        const unsigned long long lanes = ((unsigned long long)hi << 32) | lo;
        const float v = __builtin_amdgcn_inverse_ballot_w64(lanes) ? b[cur][s] : 0.f;
#pragma unroll
        for (int im = 0; im < WM; ++im)
          acc[s][im] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][im], v, acc[s][im], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    }
    __syncthreads();
  }
  float *out = partial + g.part_off + (long long)q * (NS * BMA * 64);
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int im = 0; im < WM; ++im)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = (wm * WM + im) * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        out[(s * BMA + row) * 64 + wn * 32 + (lane & 31)] = acc[s][im][v];
      }
}

// The strips and corners first (few items, bound by latency: they start early and
// run beside the rest), then the whole-image groups.
template <int WM>
__global__ __launch_bounds__(THREADS, 2) void corr_kernel(Plan pl, float *__restrict__ partial) {
  __shared__ float lds[Panel<64 * WM>::kFloats + 64 * kShiftStride];
  int w = blockIdx.x;
  if (w >= pl.nsmall) w = pl.nsmall + item_of_block(w - pl.nsmall, pl.total - pl.nsmall);
  int gi = 0;
  if (w >= pl.nsmall) {
    gi = w >= pl.grp[2].task0 ? 2 : (w >= pl.grp[1].task0 ? 1 : 0);
  } else {
    gi = 3;
    while (gi + 1 < kGroups && pl.grp[gi + 1].task0 <= w) ++gi;
  }
  const ShiftGroup &g = pl.grp[gi];
  if constexpr (WM == 1) {
    if (g.stacked) {
      corr_shifts_body<1, 3, true>(pl, g, w - g.task0, lds, partial);
      return;
    }
  }
  if (g.ns == 3)
    corr_shifts_body<WM, 3>(pl, g, w - g.task0, lds, partial);
  else
    corr_shifts_body<WM, 5>(pl, g, w - g.task0, lds, partial);
}

// One pass over the input before the products: the per-channel sums that make the
// ones column, over the samples of chunk blockIdx.y (a contiguous range),
//   sums[chunk][c][0..8] = whole image, first row, last row, first column, last
//   column, corners (first,first) (first,last) (last,first) (last,last),
// and the compact copy of the first and last image column, edges[last][s][c][u].
__global__ __launch_bounds__(256) void edge_sums_kernel(Plan pl, float *__restrict__ sums,
                                                        float *__restrict__ edges) {
  __shared__ float red[4][kChannelSums];
  const int c = blockIdx.x, chunk = blockIdx.y, nchunk = gridDim.y;
  const int H = pl.H, W = pl.W, HW = H * W;
  const int per = (pl.n + nchunk - 1) / nchunk;
  const int s0 = chunk * per, s1 = s0 + per < pl.n ? s0 + per : pl.n;
  float acc[kChannelSums];
#pragma unroll
  for (int e = 0; e < kChannelSums; ++e) acc[e] = 0.f;
  const float *base = pl.x + (long long)c * pl.row_stride;
  float *e0 = edges + (long long)c * H, *e1 = e0 + (long long)pl.n * pl.C * H;
  if (W % 4 == 0 && (reinterpret_cast<uintptr_t>(pl.x) & 15) == 0) {
    // four pixels of one image row at a time
    const int Q = HW / 4;
    for (int e = s0 * Q + (int)threadIdx.x; e < s1 * Q; e += 256) {
      const int s = e / Q, p = (e - s * Q) * 4;
      const float4 v = *reinterpret_cast<const float4 *>(base + (long long)s * pl.sample_stride + p);
      const int u = p / W, q = p - u * W;
      const bool r0 = u == 0, r1 = u == H - 1, c0 = q == 0, c1 = q + 4 == W;
      const float t = (v.x + v.y) + (v.z + v.w);
      acc[0] += t;
      if (r0) acc[1] += t;
      if (r1) acc[2] += t;
      if (c0) {
        acc[3] += v.x;
        e0[(long long)s * pl.C * H + u] = v.x;
        if (r0) acc[5] += v.x;
        if (r1) acc[7] += v.x;
      }
      if (c1) {
        acc[4] += v.w;
        e1[(long long)s * pl.C * H + u] = v.w;
        if (r0) acc[6] += v.w;
        if (r1) acc[8] += v.w;
      }
    }
  } else {
    for (int e = s0 * HW + (int)threadIdx.x; e < s1 * HW; e += 256) {
      const int s = e / HW, p = e - s * HW;
      const float v = base[(long long)s * pl.sample_stride + p];
      const int u = p / W, q = p - u * W;
      const bool r0 = u == 0, r1 = u == H - 1, c0 = q == 0, c1 = q == W - 1;
      acc[0] += v;
      if (r0) acc[1] += v;
      if (r1) acc[2] += v;
      if (c0) {
        acc[3] += v;
        e0[(long long)s * pl.C * H + u] = v;
      }
      if (c1) {
        acc[4] += v;
        e1[(long long)s * pl.C * H + u] = v;
      }
      if (r0 && c0) acc[5] += v;
      if (r0 && c1) acc[6] += v;
      if (r1 && c0) acc[7] += v;
      if (r1 && c1) acc[8] += v;
    }
  }
#pragma unroll
  for (int e = 0; e < kChannelSums; ++e) {
    float v = acc[e];
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6][e] = v;
  }
  __syncthreads();
  if (threadIdx.x < kChannelSums)
    sums[((long long)chunk * pl.C + c) * kChannelSums + threadIdx.x] =
        red[0][threadIdx.x] + red[1][threadIdx.x] + red[2][threadIdx.x] + red[3][threadIdx.x];
}

// Sums the slices of one block of one product and writes it to the product's
// array and, transposed, to the array of the opposite offset.  A symmetric
// product (offset zero) is written from its lower triangle.  G = 1: blocks of 32 x
// 32, every thread sums all slices of its four elements; G = 4 (many slices, few
// blocks): blocks of 16 x 16, four threads share an element's slices (s = g, g +
// 4, ...) and their sums are added in a fixed order.
template <int G, int WM>
__global__ __launch_bounds__(256) void corr_finish_kernel(Plan pl, const float *__restrict__ partial,
                                                          float *__restrict__ arrays) {
  constexpr int B = G == 1 ? 32 : 16;
  constexpr int tile_rows = 64 * WM;
  __shared__ float t[G][B][B + 1];
  const int blk = blockIdx.x;
  const int nb = (pl.C + B - 1) / B;
  const int p = blk / (nb * nb);
  const int b = blk - p * (nb * nb);
  const int bi = b / nb, bj = b - bi * nb;
  const Product &pr = pl.prod[p];
  const bool sym = pr.out == pr.out_t;
  if (sym && bi < bj) return;
  const int tid = threadIdx.x % (256 / G), grp = threadIdx.x / (256 / G);
  const int r = tid / (B / 4), c4 = (tid % (B / 4)) * 4;
  const int row = bi * B + r, col = bj * B + c4;
  const int ti = row / tile_rows, tj = col / 64;
  const float4 *src = reinterpret_cast<const float4 *>(
      partial + pr.part_off + (long long)(ti * pl.tiles_b + tj) * pr.tile_stride +
      (row - ti * tile_rows) * 64 + (col - tj * 64));
  const long long step4 = pr.split_stride / 4;
  float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
  int s = grp;
  for (; s + 7 * G < pr.nsplit; s += 8 * G) {
    float4 v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = src[(s + e * G) * step4];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a.x += v[e].x;
      a.y += v[e].y;
      a.z += v[e].z;
      a.w += v[e].w;
    }
  }
  for (; s < pr.nsplit; s += G) {
    const float4 v = src[s * step4];
    a.x += v.x;
    a.y += v.y;
    a.z += v.z;
    a.w += v.w;
  }
  t[grp][r][c4] = a.x;
  t[grp][r][c4 + 1] = a.y;
  t[grp][r][c4 + 2] = a.z;
  t[grp][r][c4 + 3] = a.w;
  __syncthreads();
  const int C = pl.C;
  float *o = arrays + (long long)pr.out * C * C;
  float *ot = arrays + (long long)pr.out_t * C * C;
  const int lc = threadIdx.x % B, lr0 = threadIdx.x / B;
  auto total = [&](int i, int j) {
    float v = t[0][i][j];
#pragma unroll
    for (int g = 1; g < G; ++g) v += t[g][i][j];
    return v;
  };
#pragma unroll
  for (int e = 0; e < B * B / 256; ++e) {
    const int lr = lr0 + (256 / B) * e;
    const int gr = bi * B + lr, gc = bj * B + lc;
    if (sym && bi == bj) {
      if (gr < C && gc < C) o[(long long)gr * C + gc] = lc <= lr ? total(lr, lc) : total(lc, lr);
      continue;
    }
    if (gr < C && gc < C) o[(long long)gr * C + gc] = total(lr, lc);
    const int tr = bj * B + lr, tc = bi * B + lc;   // block (bj, bi) of the transposed array
    if (tr < C && tc < C) ot[(long long)tr * C + tc] = total(lc, lr);
  }
}

// Entry ((c,i,j), (c',i',j')) of the factor from the arrays' values at [c][c'],
// staged in LDS as arr[array][c' - first c' of the chunk].
template <int CHUNK>
__device__ __forceinline__ float assemble(const float (*arr)[CHUNK], int cl, int i, int j, int i2, int j2) {
  const int di = i2 - i, dj = j2 - j;
  float v = arr[(di + 2) * 5 + dj + 2][cl];
  if (di == 0 && i != 1) v -= arr[25 + (i == 0 ? 5 : 0) + dj + 2][cl];
  if (dj == 0 && j != 1) v -= arr[35 + (j == 0 ? 5 : 0) + di + 2][cl];
  if (di == 0 && dj == 0 && i != 1 && j != 1) v += arr[45 + (i == 0 ? 2 : 0) + (j == 0 ? 1 : 0)][cl];
  return v;
}

// Writes the 9 rows of channel blockIdx.x (a third of them per blockIdx.z when the
// grid has three layers), columns of the 64 channels of chunk blockIdx.y: out =
// alpha * value + beta * out.  The workgroups of chunk 0 also
// write the ones column and row of their 9 rows (and the first of them the corner).
__global__ __launch_bounds__(256) void assemble_kernel(Plan pl, const float *__restrict__ arrays,
                                                        const float *__restrict__ sums, int nchunk_sums,
                                                        int d, int ones, float count, float alpha,
                                                        float beta, float *__restrict__ out) {
  constexpr int CHUNK = 64;
  __shared__ float arr[kArrays][CHUNK];
  __shared__ float cs[kChannelSums];
  const int C = pl.C;
  const int c = blockIdx.x, c0 = blockIdx.y * CHUNK;
  const int width = (C - c0 < CHUNK) ? C - c0 : CHUNK;
  // all of a thread's loads in flight before the first is stored
  constexpr int kPer = (kArrays * CHUNK + 255) / 256;
  float stage[kPer];
#pragma unroll
  for (int k = 0; k < kPer; ++k) {
    const int e = threadIdx.x + 256 * k;
    const int a = e / CHUNK, cl = e - a * CHUNK;
    stage[k] = (a < kArrays && cl < width) ? arrays[((long long)a * C + c) * C + c0 + cl] : 0.f;
  }
#pragma unroll
  for (int k = 0; k < kPer; ++k) {
    const int e = threadIdx.x + 256 * k;
    const int a = e / CHUNK, cl = e - a * CHUNK;
    if (a < kArrays) arr[a][cl] = stage[k];
  }
  if (ones && blockIdx.y == 0 && threadIdx.x < kChannelSums) {
    float v = 0.f;
    for (int k = 0; k < nchunk_sums; ++k) v += sums[((long long)k * C + c) * kChannelSums + threadIdx.x];
    cs[threadIdx.x] = v;
  }
  __syncthreads();
  const int ncol = width * 9;
  const int rows_per = 9 / gridDim.z;   // gridDim.z = 1 or 3: a small factor is spread over more workgroups
  for (int ij = blockIdx.z * rows_per; ij < (int)(blockIdx.z + 1) * rows_per; ++ij) {
    const int i = ij / 3, j = ij - 3 * i;
    float *dst = out + (long long)(c * 9 + ij) * d + c0 * 9;
#pragma unroll
    for (int t = threadIdx.x; t < CHUNK * 9; t += 256) {
      if (t >= ncol) break;
      const int cl = t / 9, ij2 = t - 9 * cl;
      const int i2 = ij2 / 3, j2 = ij2 - 3 * i2;
      float v = alpha * assemble<CHUNK>(arr, cl, i, j, i2, j2);
      if (beta != 0.f) v += beta * dst[t];
      dst[t] = v;
    }
  }
  if (ones && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x < 9) {
    const int ij = threadIdx.x, i = ij / 3, j = ij - 3 * i;
    float v = cs[0];
    if (i != 1) v -= cs[i == 0 ? 2 : 1];
    if (j != 1) v -= cs[j == 0 ? 4 : 3];
    if (i != 1 && j != 1) v += cs[5 + (i == 0 ? 2 : 0) + (j == 0 ? 1 : 0)];
    const int row = c * 9 + ij;
    v *= alpha;
    if (beta != 0.f) v += beta * out[(long long)(d - 1) * d + row];
    out[(long long)(d - 1) * d + row] = v;
    out[(long long)row * d + d - 1] = v;
    if (c == 0 && ij == 0) {
      float k = alpha * count;
      if (beta != 0.f) k += beta * out[(long long)(d - 1) * d + d - 1];
      out[(long long)(d - 1) * d + d - 1] = k;
    }
  }
}

}  // namespace shift
}  // namespace kfac
