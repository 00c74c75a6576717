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

// Operand of one product: rows = channels, k = (sample, p), p < L running over the
// product's domain (a whole image, one image row, one image column or one pixel);
//   p -> (a, b) = (p / line_len, p % line_len),
//   element = base[sample * sample_stride + row * row_stride + (a + da) * line_stride + (b + db)]
// if 0 <= a + da < amax and 0 <= b + db < bmax, else 0.  Dword loads, the 32 lanes
// of a half-wave on 32 consecutive k of one row (the layout of LoaderKC's scalar
// variant).
template <int ROWS>
struct LoaderShift {
  static constexpr bool kKRow = false;
  static constexpr int NR = ROWS / 8;   // rows per thread
  struct Regs {
    float v[NR];
    bool kvalid;
  };
  const float *base;
  unsigned sample_stride, row_stride;
  unsigned L, line_len, line_stride;
  int da, db, amax, bmax;
  int rows_valid;
  int first_row;
  unsigned last_off;

  __device__ __forceinline__ void init(float *, int row0) {
    first_row = row0 + (team_tid() >> 5);
    last_off = (unsigned)(rows_valid > 0 ? rows_valid - 1 : 0) * row_stride;
  }

  __device__ __forceinline__ void load(Regs &r, int, long long k0, long long k_end) const {
    const long long kg = k0 + (team_tid() & 31);
    const bool kin = kg < k_end;
    const unsigned kc = kin ? (unsigned)kg : 0u;
    const unsigned s = kc / L;
    const unsigned p = kc - s * L;
    const unsigned a0 = p / line_len;
    const int a = (int)a0 + da, b = (int)(p - a0 * line_len) + db;
    r.kvalid = kin && (unsigned)a < (unsigned)amax && (unsigned)b < (unsigned)bmax;
    const unsigned koff = r.kvalid ? s * sample_stride + (unsigned)a * line_stride + (unsigned)b : 0u;
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
constexpr int kChannelSums = 9;   // whole image, first / last row, first / last column, 4 corners

struct Product {
  unsigned base_off;   // first element of the domain within an image plane
  unsigned L;          // k-values per sample: pixels of the domain
  unsigned line_len;   // p -> (a, b) = (p / line_len, p % line_len)
  short da, db;        // the second operand's shift
  short amax, bmax;    // bounds of a + da, b + db
  int K;               // reduction length: samples * L
  int klen;            // k-values per slice (a multiple of KT)
  int nsplit;
  int task0;           // first work item; the item's index is also its partial tile's
  short out, out_t;    // array written as it is / transposed (equal: symmetric product)
};

struct Plan {
  const float *x;
  unsigned sample_stride, row_stride, line_stride;   // C H W, H W, W
  int C, H, W, n;
  int tiles;    // per side
  int total;    // work items
  Product prod[kProducts];
};

// Work item -> (product, tile, slice).  Consecutive workgroup ids go round-robin
// to the 8 XCDs; each XCD takes a contiguous run of the item list, in which the
// tiles of one slice of one product follow each other (they share operand panels).
__device__ __forceinline__ int item_of_block(int bid, int total) {
  const int xcd = bid % 8, idx = bid / 8;
  const int base = total / 8, rem = total % 8;
  return xcd * base + (xcd < rem ? xcd : rem) + idx;
}

template <int WM>
__global__ __launch_bounds__(THREADS, 3) void corr_kernel(Plan pl, float *__restrict__ partial) {
  constexpr int BM = 64 * WM;
  __shared__ float lds[2 * Panel<BM>::kFloats];
  float *ldsA = lds, *ldsB = lds + Panel<BM>::kFloats;
  const int w = item_of_block(blockIdx.x, pl.total);
  int p = 0;
  while (p + 1 < kProducts && pl.prod[p + 1].task0 <= w) ++p;
  const Product &pr = pl.prod[p];
  const int ntile = pl.tiles * pl.tiles;
  const int q = w - pr.task0;
  const int split = q / ntile, tile = q - split * ntile;
  const int I = tile / pl.tiles, J = tile - I * pl.tiles;
  LoaderShift<BM> la, lb;
  la.base = lb.base = pl.x + pr.base_off;
  la.sample_stride = lb.sample_stride = pl.sample_stride;
  la.row_stride = lb.row_stride = pl.row_stride;
  la.L = lb.L = pr.L;
  la.line_len = lb.line_len = pr.line_len;
  la.line_stride = lb.line_stride = pl.line_stride;
  la.amax = lb.amax = pr.amax;
  la.bmax = lb.bmax = pr.bmax;
  la.rows_valid = lb.rows_valid = pl.C;
  la.da = la.db = 0;
  lb.da = pr.da;
  lb.db = pr.db;
  la.init(nullptr, I * BM);
  lb.init(nullptr, J * BM);
  const long long kbeg = (long long)split * pr.klen;
  long long kend = kbeg + pr.klen;
  if (kend > pr.K) kend = pr.K;
  floatx16 acc[WM][WM];
  zero_acc<WM, WM>(acc);
  mainloop<WM, WM, false>(la, lb, I * BM, J * BM, kbeg, kend, ldsA, ldsB, acc);
  float *out = partial + (long long)w * (BM * BM);
  for_each_acc<WM, WM>(acc, [&](int r, int c, float v) { out[r * BM + c] = v; });
}

// Sums the slices of one 32 x 32 block of one product and writes it to the
// product's array and, transposed, to the array of the opposite offset.  A
// symmetric product (offset zero) is written from its lower triangle.
template <int WM>
__global__ __launch_bounds__(256) void corr_finish_kernel(Plan pl, const float *__restrict__ partial,
                                                          float *__restrict__ arrays) {
  constexpr int BM = 64 * WM;
  __shared__ float t[32][33];
  const int nb = (pl.C + 31) / 32;
  const int p = blockIdx.x / (nb * nb);
  const int b = blockIdx.x - p * (nb * nb);
  const int bi = b / nb, bj = b - bi * nb;
  const Product &pr = pl.prod[p];
  const bool sym = pr.out == pr.out_t;
  if (sym && bi < bj) return;
  const int ntile = pl.tiles * pl.tiles;
  const int r = threadIdx.x >> 3, c4 = (threadIdx.x & 7) * 4;
  const int row = bi * 32 + r, col = bj * 32 + c4;
  const int tile = (row / BM) * pl.tiles + col / BM;
  const float4 *src = reinterpret_cast<const float4 *>(
      partial + ((long long)pr.task0 + tile) * (BM * BM) + (row % BM) * BM + col % BM);
  const long long step4 = (long long)ntile * (BM * BM) / 4;
  float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
  int s = 0;
  for (; s + 8 <= pr.nsplit; s += 8) {
    float4 v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = src[(s + e) * step4];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a.x += v[e].x;
      a.y += v[e].y;
      a.z += v[e].z;
      a.w += v[e].w;
    }
  }
  for (; s < pr.nsplit; ++s) {
    const float4 v = src[s * step4];
    a.x += v.x;
    a.y += v.y;
    a.z += v.z;
    a.w += v.w;
  }
  t[r][c4] = a.x;
  t[r][c4 + 1] = a.y;
  t[r][c4 + 2] = a.z;
  t[r][c4 + 3] = a.w;
  __syncthreads();
  const int C = pl.C;
  float *o = arrays + (long long)pr.out * C * C;
  float *ot = arrays + (long long)pr.out_t * C * C;
  const int lc = threadIdx.x & 31, lr0 = threadIdx.x >> 5;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int lr = lr0 + 8 * e;
    const int gr = bi * 32 + lr, gc = bj * 32 + lc;
    if (sym && bi == bj) {
      if (gr < C && gc < C) o[(long long)gr * C + gc] = lc <= lr ? t[lr][lc] : t[lc][lr];
      continue;
    }
    if (gr < C && gc < C) o[(long long)gr * C + gc] = t[lr][lc];
    const int tr = bj * 32 + lr, tc = bi * 32 + lc;   // block (bj, bi) of the transposed array
    if (tr < C && tc < C) ot[(long long)tr * C + tc] = t[lc][lr];
  }
}

// Per-channel sums over the samples of chunk blockIdx.y (every gridDim.y-th
// sample): sums[chunk][c][0..8] = whole image, first row, last row, first column,
// last column, corners (first,first) (first,last) (last,first) (last,last).
__global__ __launch_bounds__(256) void channel_sums_kernel(Plan pl, float *__restrict__ sums) {
  __shared__ float red[4][kChannelSums];
  const int c = blockIdx.x;
  const int H = pl.H, W = pl.W, HW = H * W;
  float acc[kChannelSums];
#pragma unroll
  for (int e = 0; e < kChannelSums; ++e) acc[e] = 0.f;
  for (int s = blockIdx.y; s < pl.n; s += gridDim.y) {
    const float *plane = pl.x + (long long)s * pl.sample_stride + (long long)c * pl.row_stride;
    for (int p = threadIdx.x; p < HW; p += 256) {
      const float v = plane[p];
      const int u = p / W, q = p - u * W;
      const bool r0 = u == 0, r1 = u == H - 1, c0 = q == 0, c1 = q == W - 1;
      acc[0] += v;
      if (r0) acc[1] += v;
      if (r1) acc[2] += v;
      if (c0) acc[3] += v;
      if (c1) acc[4] += v;
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
    sums[((long long)blockIdx.y * pl.C + c) * kChannelSums + threadIdx.x] =
        red[0][threadIdx.x] + red[1][threadIdx.x] + red[2][threadIdx.x] + red[3][threadIdx.x];
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

// Writes the 9 rows of channel blockIdx.x, columns of the 64 channels of chunk
// blockIdx.y: out = alpha * value + beta * out.  The workgroups of chunk 0 also
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
  for (int e = threadIdx.x; e < kArrays * CHUNK; e += 256) {
    const int a = e / CHUNK, cl = e - a * CHUNK;
    arr[a][cl] = cl < width ? arrays[((long long)a * C + c) * C + c0 + cl] : 0.f;
  }
  if (ones && blockIdx.y == 0 && threadIdx.x < kChannelSums) {
    float v = 0.f;
    for (int k = 0; k < nchunk_sums; ++k) v += sums[((long long)k * C + c) * kChannelSums + threadIdx.x];
    cs[threadIdx.x] = v;
  }
  __syncthreads();
  const int ncol = width * 9;
  for (int ij = 0; ij < 9; ++ij) {
    const int i = ij / 3, j = ij - 3 * i;
    float *dst = out + (long long)(c * 9 + ij) * d + c0 * 9;
    for (int t = threadIdx.x; t < ncol; t += 256) {
      const int cl = t / 9, ij2 = t - 9 * cl;
      const int i2 = ij2 / 3, j2 = ij2 - 3 * i2;
      float v = alpha * assemble<CHUNK>(arr, cl, i, j, i2, j2);
      if (beta != 0.f) v += beta * dst[t];
      dst[t] = v;
    }
  }
  if (ones && blockIdx.y == 0 && threadIdx.x < 9) {
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
