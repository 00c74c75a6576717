// FP32 MFMA tile engine shared by the covariance (SYRK), preconditioning (GEMM)
// and inverse kernels.
//
// A workgroup of 256 threads (4 waves, 2 x 2) computes a (64*WM) x (64*WN)
// tile of  D[i][j] = sum_k Aop(i, k) * Bop(j, k)  with v_mfma_f32_32x32x2_f32;
// each wave owns WM x WN accumulator blocks of 32 x 32.  Operand panels
// (rows x 32 k-values) are staged through LDS by "loaders" that know how an
// operand is laid out in memory:
//
//   LoaderKC  k is the contiguous index:  (sample, row, l) tensors such as an
//             NCHW activation viewed as rows = channel, k = (sample, pixel),
//             and plain row-major matrices used as the k-contiguous operand.
//   LoaderKS  row is the contiguous index: a row-major (k, row) matrix, e.g.
//             the (batch, features) input of a Linear layer or the right-hand
//             operand of an NN product; an optional extra row supplies the
//             bias column (ones, or a second array).
//   LoaderIM  implicit im2col: row = (c, kh, kw) [+ ones], k = (sample, y, x);
//             the patch matrix is gathered straight from the NCHW tensor.
//
// LDS panel layouts: "RowK" (row-major, stride 33, used by KC/IM) and "KRow"
// (k-major, stride rows+4, used by KS); both give conflict-free MFMA operand
// reads.  The main loop keeps one LDS buffer and prefetches the next panel
// into registers while the current one feeds the matrix cores.
#pragma once

#include <hip/hip_runtime.h>

namespace kfac {
namespace mma {

constexpr int KT = 32;        // k-values per LDS panel
constexpr int THREADS = 256;  // 4 waves
typedef float floatx16 __attribute__((ext_vector_type(16)));

// Loads from global memory at a wave-uniform base plus a 32-bit byte offset per
// lane: the form of the load instruction that takes the base from scalar
// registers, so that no 64-bit address is formed per lane and per load.  The
// tensors read this way are smaller than 4 GiB (checked on the host).
typedef float floatx4 __attribute__((ext_vector_type(4), aligned(4)));
#define KFAC_GLOBAL_AS __attribute__((address_space(1)))
__device__ __forceinline__ float4 gload4(const float *base, unsigned byte_off) {
  const floatx4 t = *(const KFAC_GLOBAL_AS floatx4 *)((const KFAC_GLOBAL_AS char *)base + byte_off);
  return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ float gload1(const float *base, unsigned byte_off) {
  return *(const KFAC_GLOBAL_AS float *)((const KFAC_GLOBAL_AS char *)base + byte_off);
}

// Thread index inside a team of THREADS threads.  The workgroups of this engine
// have THREADS threads, except those of the macro-tile covariance kernel, whose
// four teams each stage and multiply like one such workgroup.
__device__ __forceinline__ int team_tid() { return (int)(threadIdx.x & (THREADS - 1)); }

template <int ROWS>
struct Panel {
  static constexpr int kRowKStride = KT + 1;
  static constexpr int kKRowStride = ROWS + 4;
  static constexpr int kFloats =
      (ROWS * kRowKStride > KT * kKRowStride) ? ROWS * kRowKStride : KT * kKRowStride;
};

// Loader protocol: init() fixes the panel (first row) and precomputes what
// does not change along k (row offsets, row validity); load() issues the
// global loads of one panel; store() writes it to LDS.  Interior panels (all
// rows and all k valid: a workgroup-uniform test) take a path without any
// per-element selects; edge panels load from clamped (always valid) addresses
// and apply validity masks when storing.  Nothing between load() and store()
// touches the loaded registers, so the loads stay in flight while the matrix
// cores work on the previous panel.  Offsets are 32-bit element offsets from
// the tensor base (tensors hold fewer than 2^30 elements, 4 GiB; checked on the host).

// ---------------------------------------------------------------------------
// LoaderKC: element (row, kg) at base + (kg / L) * sample_stride
//                                     + row * row_stride + (kg % L)
// rows >= rows_valid read as 0.
// ---------------------------------------------------------------------------
// VEC: 16-byte loads of four consecutive k-values of a row; for tensors whose
// rows start on 16-byte boundaries (base, row and sample strides multiples of 4
// floats: misaligned 16-byte loads work but were measured slower than the
// scalar variant below).  A quad that is cut by the end of the range, or that
// runs from one sample into the next, is loaded element by element by the
// lanes concerned, so the reduction length is free.  A compile-time choice so
// that this common case carries no code or registers of the scalar variant.
// The primary template is this one.
template <int ROWS, bool VEC>
struct LoaderKC {
  static_assert(VEC, "the scalar variant is the specialisation below");
  static constexpr bool kKRow = false;
  static constexpr int NV = ROWS / 32;
  struct Regs {
    float4 v[NV];
    unsigned kmask;  // bit e: k-value e of this thread's quad is inside the range
    bool fast;       // interior panel: no masks needed
  };
  const float *base;
  unsigned sample_stride;
  unsigned row_stride;
  unsigned L;      // k-values per sample
  int rows_valid;
  // per-thread panel state
  unsigned rowoff[NV];
  unsigned rowvalid;  // bit i: row i of this thread is a data row
  bool full_rows;

  __device__ __forceinline__ void init(float *, int row0) {
    const int rr = team_tid() >> 3;
    rowvalid = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int row = row0 + rr + 32 * i;
      const bool ok = row < rows_valid;
      rowoff[i] = (ok ? (unsigned)row : 0u) * row_stride;
      if (ok) rowvalid |= 1u << i;
    }
    full_rows = row0 + ROWS <= rows_valid;
  }

  __device__ __forceinline__ void load(Regs &r, int, long long k0, long long k_end) const {
    const unsigned kq = (team_tid() & 7) * 4;
    const long long kgl = k0 + kq;
    const bool full_k = k0 + KT <= k_end;
    r.fast = full_rows && full_k;
    const bool whole = full_k || kgl + 3 < k_end;
    const long long left = k_end - kgl;   // valid k-values from kg on
    r.kmask = whole ? 0xfu : (left > 0 ? (1u << (int)left) - 1u : 0u);
    const unsigned kc = left > 0 ? (unsigned)kgl : 0u;
    unsigned koff = kc, rem = kc;
    if (L < (unsigned)k_end) {  // more than one sample
      const unsigned s = kc / L;
      rem = kc - s * L;
      koff = s * sample_stride + rem;
    }
    if (whole && rem + 3 < L) {
#pragma unroll
      for (int i = 0; i < NV; ++i) r.v[i] = gload4(base, (koff + rowoff[i]) * 4u);
    } else {
      // element by element: k-values past the range read k = 0 of the row (masked when
      // stored), k-values past the end of the sample continue in the next sample
      unsigned off[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool in = (r.kmask >> e) & 1u;
        off[e] = in ? koff + e + (rem + e >= L ? sample_stride - L : 0u) : 0u;
      }
#pragma unroll
      for (int i = 0; i < NV; ++i)
        r.v[i] = make_float4(gload1(base, (off[0] + rowoff[i]) * 4u), gload1(base, (off[1] + rowoff[i]) * 4u),
                             gload1(base, (off[2] + rowoff[i]) * 4u), gload1(base, (off[3] + rowoff[i]) * 4u));
    }
  }

  __device__ __forceinline__ void store(const Regs &r, float *lds) const {
    const int kq = (team_tid() & 7) * 4;
    const int rr = team_tid() >> 3;
    if (r.fast) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        float *p = lds + (rr + 32 * i) * Panel<ROWS>::kRowKStride + kq;
        p[0] = r.v[i].x;
        p[1] = r.v[i].y;
        p[2] = r.v[i].z;
        p[3] = r.v[i].w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        float *p = lds + (rr + 32 * i) * Panel<ROWS>::kRowKStride + kq;
        const float t[4] = {r.v[i].x, r.v[i].y, r.v[i].z, r.v[i].w};
        const bool rv = (rowvalid >> i) & 1u;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const bool kv = (r.kmask >> e) & 1u;
          p[e] = (kv && rv) ? t[e] : 0.f;
        }
      }
    }
  }
};

// Scalar variant: dword loads with the 32 lanes of a half-wave on 32 consecutive
// k-values of one row.  It is the one that can subsample (line_len > 0).
template <int ROWS>
struct LoaderKC<ROWS, false> {
  static constexpr bool kKRow = false;
  static constexpr int NR = ROWS / 8;   // rows per thread
  struct Regs {
    float v[NR];
    bool kvalid;   // this thread's k-value is inside the range
  };
  const float *base;
  unsigned sample_stride;
  unsigned row_stride;
  unsigned L;      // k-values per sample
  int rows_valid;
  // Subsampled rows (a strided 1x1 convolution reads every sx-th pixel of every
  // sy-th image line): k-value p of a sample is pixel (p / line_len) *
  // line_stride + (p % line_len) * px_stride of the row.  line_len = 0: k-values
  // are consecutive elements.
  unsigned line_len = 0, line_stride = 0, px_stride = 1;
  // per-thread panel state: row i of the thread is first_row + 8 i; rows past
  // the end load from the last data row (masked when stored)
  int first_row;
  unsigned last_off;

  __device__ __forceinline__ void init(float *, int row0) {
    first_row = row0 + (team_tid() >> 5);
    last_off = (unsigned)(rows_valid > 0 ? rows_valid - 1 : 0) * row_stride;
  }

  __device__ __forceinline__ void load(Regs &r, int, long long k0, long long k_end) const {
    const long long kg = k0 + (team_tid() & 31);
    r.kvalid = kg < k_end;
    const unsigned kc = r.kvalid ? (unsigned)kg : 0u;
    unsigned koff = kc;
    if (L < (unsigned)k_end || line_len) {  // more than one sample, or subsampled rows
      const unsigned s = kc / L;
      unsigned pix = kc - s * L;
      if (line_len) {
        const unsigned line = pix / line_len;
        pix = line * line_stride + (pix - line * line_len) * px_stride;
      }
      koff = s * sample_stride + pix;
    }
    // The row offsets are cheap to recompute and expensive to keep: hide the
    // row from the optimiser so that it does not hoist NR offsets per operand
    // out of the k loop (which spills under a 3-workgroup register budget).
    int fr = first_row;
    asm volatile("" : "+v"(fr));
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

// ---------------------------------------------------------------------------
// LoaderKS: element (row, kg) at base + kg * ld + row for row < rows_valid;
// row == rows_valid reads extra[kg] (or 1 when extra is null) if has_extra.
// ---------------------------------------------------------------------------
template <int ROWS, bool VEC>
struct LoaderKS {
  static constexpr bool kKRow = true;
  static constexpr int RQ = ROWS / 4;          // row quads per k
  static constexpr int KPP = THREADS / RQ;     // k-values per pass
  static constexpr int NV = KT / KPP;
  struct Regs {
    float4 v[NV];
    unsigned kmask;  // bit i: k-value of pass i is inside the range
    bool fast;
  };
  const float *base;
  const float *extra;
  unsigned ld;
  int rows_valid;
  int has_extra;
  // per-thread panel state
  int row;          // first of this thread's four rows
  bool quad_ok;     // all four rows are data rows and float4 loads are allowed
  bool full_rows;

  __device__ __forceinline__ void init(float *, int row0) {
    row = row0 + (team_tid() % RQ) * 4;
    quad_ok = VEC && row + 3 < rows_valid;
    full_rows = VEC && row0 + ROWS <= rows_valid;
  }

  __device__ __forceinline__ void load(Regs &r, int, long long k0, long long k_end) const {
    const int kk = team_tid() / RQ;
    const bool full_k = k0 + KT <= k_end;
    r.fast = full_rows && full_k;
    r.kmask = 0;
    if (quad_ok) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const long long kg = k0 + kk + KPP * i;
        const bool kok = full_k || kg < k_end;
        if (kok) r.kmask |= 1u << i;
        r.v[i] = gload4(base, ((unsigned)(kok ? kg : 0) * ld + (unsigned)row) * 4u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const long long kg = k0 + kk + KPP * i;
        const bool kok = kg < k_end;
        if (kok) r.kmask |= 1u << i;
        const unsigned kc = (unsigned)(kok ? kg : 0);
        float t[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int re = row + e;
          const float *q = base + kc * ld + (unsigned)(re < rows_valid ? re : 0);
          if (re == rows_valid && has_extra && extra) q = extra + kc;
          t[e] = *q;
        }
        r.v[i] = make_float4(t[0], t[1], t[2], t[3]);
      }
    }
  }

  __device__ __forceinline__ void store(const Regs &r, float *lds) const {
    const int rq = (team_tid() % RQ) * 4;
    const int kk = team_tid() / RQ;
    if (r.fast) {
#pragma unroll
      for (int i = 0; i < NV; ++i)
        *reinterpret_cast<float4 *>(lds + (kk + KPP * i) * Panel<ROWS>::kKRowStride + rq) = r.v[i];
    } else {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const float t[4] = {r.v[i].x, r.v[i].y, r.v[i].z, r.v[i].w};
        const bool kv = (r.kmask >> i) & 1u;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int re = row + e;
          float val = 0.f;
          if (re < rows_valid)
            val = t[e];
          else if (re == rows_valid && has_extra)
            val = extra ? t[e] : 1.f;
          o[e] = kv ? val : 0.f;
        }
        *reinterpret_cast<float4 *>(lds + (kk + KPP * i) * Panel<ROWS>::kKRowStride + rq) =
            make_float4(o[0], o[1], o[2], o[3]);
      }
    }
  }
};

// ---------------------------------------------------------------------------
// LoaderIM: implicit im2col over an NCHW tensor.
//   row = (c * kh + i) * kw + j  for row < d_patch (rows past it read as 0);
//   kg = (sample * ho + oy) * wo + ox.
// ---------------------------------------------------------------------------
template <int ROWS>
struct LoaderIM {
  static constexpr bool kKRow = false;
  static constexpr int NV = ROWS / 8;
  struct Regs {
    float v[NV];
    unsigned use;
  };
  const float *base;
  int C, H, W, kh, kw, sy, sx, ph, pw, ho, wo;
  int d_patch;
  int2 *table;  // LDS, ROWS entries: {offset inside a sample, (i << 16) | j}; y = -1: row past the end

  // Build the per-row table for panel rows [row0, row0 + ROWS).
  __device__ __forceinline__ void init(float *lds_table, int row0) {
    table = reinterpret_cast<int2 *>(lds_table);
    for (int t = team_tid(); t < ROWS; t += THREADS) {
      const int row = row0 + t;
      int2 e;
      if (row < d_patch) {
        const int c = row / (kh * kw);
        const int rem = row - c * (kh * kw);
        const int i = rem / kw;
        const int j = rem - i * kw;
        e.x = (c * H + i) * W + j;
        e.y = (i << 16) | j;
      } else {
        e.x = 0;
        e.y = -1;
      }
      table[t] = e;
    }
  }

  __device__ __forceinline__ void load(Regs &r, int, long long k0, long long k_end) const {
    const int k = team_tid() & 31;
    const int rr = team_tid() >> 5;
    const long long kg = k0 + k;
    const bool kok = kg < k_end;
    const unsigned kc = kok ? (unsigned)kg : 0u;
    const unsigned howo = (unsigned)(ho * wo);
    const unsigned s = kc / howo;
    const unsigned rem = kc - s * howo;
    const int oy = (int)(rem / (unsigned)wo);
    const int ox = (int)rem - oy * wo;
    const int iy0 = oy * sy - ph;
    const int ix0 = ox * sx - pw;
    const long long idx0 = ((long long)s * C * H + iy0) * (long long)W + ix0;
    r.use = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int2 e = table[rr + 8 * i];
      const int iy = iy0 + (e.y >> 16);
      const int ix = ix0 + (e.y & 0xffff);
      const bool ok = kok && e.y >= 0 && (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
      r.v[i] = base[ok ? idx0 + e.x : 0];
      if (ok) r.use |= 1u << i;
    }
  }

  __device__ __forceinline__ void store(const Regs &r, float *lds) const {
    const int k = team_tid() & 31;
    const int rr = team_tid() >> 5;
#pragma unroll
    for (int i = 0; i < NV; ++i)
      lds[(rr + 8 * i) * Panel<ROWS>::kRowKStride + k] = ((r.use >> i) & 1u) ? r.v[i] : 0.f;
  }
};

// Operand fetch for one MFMA: lane l supplies element (row = l % 32, k = l / 32).
template <int ROWS, bool KROW>
__device__ __forceinline__ float fetch(const float *lds, int row, int k) {
  if (KROW)
    return lds[k * Panel<ROWS>::kKRowStride + row];
  else
    return lds[row * Panel<ROWS>::kRowKStride + k];
}

// Main loop.  acc[im][in] accumulates the 32x32 block at rows
// (wave_m * WM + im) * 32 of the A panel and (wave_n * WN + in) * 32 of the B
// panel.  With SAME the B operand is read from the A panel (diagonal tile of a
// SYRK) and lb is not used.  ldsA / ldsB hold Panel<64*WM> / Panel<64*WN>
// floats.  Operands of step kk+1 are fetched from LDS before the MFMAs of step
// kk issue, so LDS latency hides behind the matrix pipeline.
// With RS the lane also sums the A operand values it feeds to the matrix cores:
// rs[im] ends as the sum over this lane's k-values (k = lane / 32 mod 2) of row
// (wave_m * WM + im) * 32 + lane % 32, i.e. half of that row's sum.
// A wave with `active` false stages panels like the others but feeds nothing to
// the matrix cores (its block of the tile is not needed: above the diagonal of a
// symmetric product, or past the end of the matrix); its accumulators stay as
// they are.
// MASK: bit im * WN + in set = this wave computes block (im, in) of its 2 x 2
// (compile time, so that a wave that owns fewer blocks carries no test per MFMA).
template <int WM, int WN, bool SAME, bool RS, class LA, class LB, unsigned MASK = 0xffffffffu>
__device__ __forceinline__ void mainloop_impl(const LA &la, const LB &lb, int rowA0, int rowB0,
                                              long long kbeg, long long kend, float *ldsA,
                                              float *ldsB, floatx16 (&acc)[WM][WN], float *rs,
                                              bool active = true, int wave = threadIdx.x >> 6) {
  constexpr int RA = 64 * WM, RB = 64 * WN;
  const int lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane & 31, lk = lane >> 5;
  typename LA::Regs ra;
  typename LB::Regs rb;
  if (kbeg < kend) {
    la.load(ra, rowA0, kbeg, kend);
    if (!SAME) lb.load(rb, rowB0, kbeg, kend);
  }
  for (long long k0 = kbeg; k0 < kend; k0 += KT) {
    la.store(ra, ldsA);
    if (!SAME) lb.store(rb, ldsB);
    __syncthreads();
    if (k0 + KT < kend) {
      la.load(ra, rowA0, k0 + KT, kend);
      if (!SAME) lb.load(rb, rowB0, k0 + KT, kend);
    }
    if (active) {
#pragma unroll
    for (int kk = 0; kk < KT / 2; ++kk) {
      float a[WM], b[WN];
#pragma unroll
      for (int im = 0; im < WM; ++im)
        a[im] = fetch<RA, LA::kKRow>(ldsA, (wm * WM + im) * 32 + lrow, 2 * kk + lk);
      if (RS) {
#pragma unroll
        for (int im = 0; im < WM; ++im) rs[im] += a[im];
      }
#pragma unroll
      for (int in = 0; in < WN; ++in) {
        if (SAME)
          b[in] = fetch<RA, LA::kKRow>(ldsA, (wn * WN + in) * 32 + lrow, 2 * kk + lk);
        else
          b[in] = fetch<RB, LB::kKRow>(ldsB, (wn * WN + in) * 32 + lrow, 2 * kk + lk);
      }
#pragma unroll
      for (int im = 0; im < WM; ++im)
#pragma unroll
        for (int in = 0; in < WN; ++in)
          if (MASK & (1u << (im * WN + in)))
            acc[im][in] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[im], b[in], acc[im][in], 0, 0, 0);
    }
    }
    __syncthreads();
  }
}

template <int WM, int WN, bool SAME, class LA, class LB>
__device__ __forceinline__ void mainloop(const LA &la, const LB &lb, int rowA0, int rowB0,
                                         long long kbeg, long long kend, float *ldsA,
                                         float *ldsB, floatx16 (&acc)[WM][WN], bool active = true,
                                         int wave = threadIdx.x >> 6) {
  mainloop_impl<WM, WN, SAME, false>(la, lb, rowA0, rowB0, kbeg, kend, ldsA, ldsB, acc, nullptr,
                                     active, wave);
}

template <int WM, int WN, bool SAME, class LA, class LB>
__device__ __forceinline__ void mainloop_rowsum(const LA &la, const LB &lb, int rowA0, int rowB0,
                                                long long kbeg, long long kend, float *ldsA,
                                                float *ldsB, floatx16 (&acc)[WM][WN],
                                                float (&rs)[WM], bool active = true,
                                                int wave = threadIdx.x >> 6) {
  mainloop_impl<WM, WN, SAME, true>(la, lb, rowA0, rowB0, kbeg, kend, ldsA, ldsB, acc, rs, active,
                                    wave);
}

// Whether this wave's block of a symmetric product's tile (first rows row0A /
// row0B, dt rows in all) is needed: it is not when it lies entirely above the
// diagonal (the epilogues take those entries from the mirrored block) or past
// the end of the matrix.
template <int WM>
__device__ __forceinline__ bool syrk_wave_active(int row0A, int row0B, int dt,
                                                 int wave = threadIdx.x >> 6) {
  const int ra = row0A + (wave >> 1) * WM * 32, rb = row0B + (wave & 1) * WM * 32;
  return ra + WM * 32 > rb && ra < dt && rb < dt;
}

// The diagonal 128-tile of a symmetric product needs 10 of its 16 blocks of 32 x
// 32 (the lower triangle).  Dealt by 64 x 64 quadrant, three waves compute four
// blocks each (two of them above the diagonal) and the fourth wave nothing; here
// the wave of the unused quadrant takes over the lower block row of quadrant
// (1, 0) and the diagonal quadrants skip their upper block: 3, 2, 2 and 3 blocks,
// three quarters of the time.
//   role     the wave index (2 x 2 layout) whose accumulator coordinates this wave uses
//   compute  bit im * 2 + in: block (im, in) is multiplied out
//   store    bit im * 2 + in: block (im, in) is this wave's to write (a block that
//            is not computed but stored holds zeros)
struct DiagRole {
  int role;
  unsigned compute, store;
};
__device__ __forceinline__ DiagRole diag_tile_role(int wave) {
  switch (wave) {
    case 0: return DiagRole{0, 0xdu, 0xfu};    // quadrant (0,0): blocks (0,0) (1,0) (1,1)
    case 3: return DiagRole{3, 0xdu, 0xfu};    // quadrant (1,1)
    case 2: return DiagRole{2, 0x3u, 0x3u};    // quadrant (1,0), upper block row
    default: return DiagRole{2, 0xcu, 0xcu};   // the wave of quadrant (0,1): quadrant (1,0), lower block row
  }
}

// Set every accumulator element of this lane to f(row, col), row / col relative
// to the workgroup tile.
template <int WM, int WN, class F>
__device__ __forceinline__ void fill_acc(floatx16 (&acc)[WM][WN], F f, int wave = threadIdx.x >> 6) {
  const int lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
  for (int im = 0; im < WM; ++im)
#pragma unroll
    for (int in = 0; in < WN; ++in)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = (wm * WM + im) * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        const int col = (wn * WN + in) * 32 + (lane & 31);
        acc[im][in][v] = f(row, col);
      }
}

// Visit every accumulator element of this lane: f(row, col, value) with row /
// col relative to the workgroup tile.
template <int WM, int WN, class F>
__device__ __forceinline__ void for_each_acc(floatx16 (&acc)[WM][WN], F f,
                                             int wave = threadIdx.x >> 6) {
  const int lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
  for (int im = 0; im < WM; ++im)
#pragma unroll
    for (int in = 0; in < WN; ++in)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = (wm * WM + im) * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        const int col = (wn * WN + in) * 32 + (lane & 31);
        f(row, col, acc[im][in][v]);
      }
}

// for_each_acc over the blocks whose bit (im * WN + in) is set in `mask`
template <int WM, int WN, class F>
__device__ __forceinline__ void for_each_acc_masked(floatx16 (&acc)[WM][WN], unsigned mask, F f, int wave) {
  const int lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
  for (int im = 0; im < WM; ++im)
#pragma unroll
    for (int in = 0; in < WN; ++in) {
      if (!(mask & (1u << (im * WN + in)))) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = (wm * WM + im) * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        const int col = (wn * WN + in) * 32 + (lane & 31);
        f(row, col, acc[im][in][v]);
      }
    }
}

template <int WM, int WN>
__device__ __forceinline__ void zero_acc(floatx16 (&acc)[WM][WN]) {
#pragma unroll
  for (int im = 0; im < WM; ++im)
#pragma unroll
    for (int in = 0; in < WN; ++in)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[im][in][v] = 0.f;
}

// Writes the finished tile: C[I,J] = alpha*acc + beta*C[I,J] and its mirror
// image C[J,I], 64x64 quadrant by quadrant through an LDS transpose so that
// every global access is a contiguous row segment.  Only entries on or below
// the diagonal of C are taken from the accumulators: a quadrant above the
// diagonal of a diagonal tile is skipped (it is the mirror of the one below),
// and a quadrant on the diagonal writes its upper triangle from its lower one.
// Rows and columns below dt (the tiled part); d is the leading dimension of C.
// `store`: the blocks of this wave's 2 x 2 that are its to write (see DiagRole).
template <int WM>
__device__ __forceinline__ void write_tile(floatx16 (&acc)[WM][WM], float *lds, int I, int J,
                                           int dt, int d, float alpha, float beta,
                                           float *__restrict__ C, int wave = threadIdx.x >> 6,
                                           unsigned store = 0xffffffffu) {
  constexpr int BM = 64 * WM;
  float(*t)[65] = reinterpret_cast<float(*)[65]>(lds);
  const int lc = threadIdx.x & 63, lr0 = threadIdx.x >> 6;
  for (int q = 0; q < WM * WM; ++q) {
    const int qm = q / WM, qn = q % WM;
    if (I == J && qm < qn) continue;
    const bool diag = I == J && qm == qn;
    __syncthreads();
    for_each_acc_masked<WM, WM>(acc, store, [&](int r, int c, float v) {
      if (r / 64 == qm && c / 64 == qn) t[r % 64][c % 64] = v;
    }, wave);
    __syncthreads();
    const int r0 = I * BM + qm * 64, c0 = J * BM + qn * 64;
#pragma unroll 4
    for (int p = 0; p < 16; ++p) {
      const int lr = lr0 + 4 * p;
      const int r = r0 + lr, c = c0 + lc;
      float v = alpha * t[lr][lc];
      const bool ok = r < dt && c < dt && (!diag || lc <= lr);
      if (ok) {
        if (beta != 0.f) v += beta * C[(long long)r * d + c];
        C[(long long)r * d + c] = v;
      }
      if (beta != 0.f) t[lr][lc] = v;   // the mirror gets the same value
    }
    if (beta != 0.f) __syncthreads();
#pragma unroll 4
    for (int p = 0; p < 16; ++p) {
      const int lr = lr0 + 4 * p;
      const float v = (beta != 0.f) ? t[lc][lr] : alpha * t[lc][lr];
      if (diag) {
        const int r = r0 + lr, c = c0 + lc;     // upper triangle of the quadrant itself
        if (lc > lr && r < dt && c < dt) C[(long long)r * d + c] = v;
      } else {
        const int mr = c0 + lr, mc = r0 + lc;   // row of the mirrored quadrant = column here
        if (mr < dt && mc < dt) C[(long long)mr * d + mc] = v;
      }
    }
  }
}

// The finished 128 x 128 tile (I, J), I >= J, and its mirror image written to C
// (leading dimension d, rows and columns below dt) in one go: the whole tile is
// laid out in LDS (128 x 129 floats) once, then every thread stores 16 bytes at
// a time (at float granularity: rows of an odd-sized matrix do not start on
// 16-byte boundaries), rows of the tile and rows of the mirrored tile alike.
// For C = acc (no scaling, no accumulation); ends without a barrier.
constexpr int kWholeTileLdsFloats = 128 * 129;
__device__ __forceinline__ void write_whole_tile(floatx16 (&acc)[2][2], float *lds, int I, int J, int dt,
                                                 int d, float *__restrict__ C) {
  typedef float floatx4u __attribute__((ext_vector_type(4), aligned(4)));
  constexpr int LD = 129;
  __syncthreads();   // the main loop's last LDS reads
  for_each_acc<2, 2>(acc, [&](int r, int c, float v) { lds[r * LD + c] = v; });
  __syncthreads();
  const int q = (threadIdx.x & 31) * 4;    // four columns
  const int r0 = threadIdx.x >> 5;         // 8 rows per pass
  const int row0 = I * 128, col0 = J * 128;
  const bool diag = I == J;
#pragma unroll 4
  for (int p = 0; p < 16; ++p) {
    const int lr = r0 + 8 * p;
    const int r = row0 + lr, c = col0 + q;
    if (r >= dt) continue;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (!diag || q + e <= lr) ? lds[lr * LD + q + e] : lds[(q + e) * LD + lr];
    float *dst = C + (long long)r * d + c;
    if (c + 3 < dt) {
      floatx4u o;
      o.x = v[0];
      o.y = v[1];
      o.z = v[2];
      o.w = v[3];
      *reinterpret_cast<floatx4u *>(dst) = o;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (c + e < dt) dst[e] = v[e];
    }
  }
  if (diag) return;
  // mirrored tile (J, I): its row lr is column lr of the tile
#pragma unroll 4
  for (int p = 0; p < 16; ++p) {
    const int lr = r0 + 8 * p;
    const int r = col0 + lr, c = row0 + q;
    if (r >= dt) continue;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = lds[(q + e) * LD + lr];
    float *dst = C + (long long)r * d + c;
    if (c + 3 < dt) {
      floatx4u o;
      o.x = v[0];
      o.y = v[1];
      o.z = v[2];
      o.w = v[3];
      *reinterpret_cast<floatx4u *>(dst) = o;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (c + e < dt) dst[e] = v[e];
    }
  }
}

}  // namespace mma
}  // namespace kfac
