// Covariance of convolution patches (the A factor of a k x k convolution,
// k > 1) without forming patches anywhere: the workgroup stages the raw input
// region ("halo") that a block of output pixels needs -- a few input rows of up
// to 16 channels -- in LDS once, and every MFMA operand
//     P[(c, i, j), (oy, ox)] = x[c, oy*sy - ph + i, ox*sx - pw + j]
// is read straight from that region at address rowoff(c, i, j) + koff(oy, ox).
// A 3x3 patch row re-reads each staged input element nine times from LDS, so
// global loads and their address arithmetic drop ~9x compared with gathering
// the patch matrix element by element; zero padding is written into the region
// when it is staged, the ones column is a constant plane next to it.
//
// Region layout per panel (128 rows of (c,i,j)): plane ch (input channel
// c_lo + ch) at ch*Rsz, element (ry, rx) at ry*Wr + rx, with Wr = kw and
// Rsz = kh*kw (mod 32): the 32 consecutive patch rows an MFMA operand fetch
// touches then fall into 32 different LDS banks.  Two extra planes hold ones
// (bias column) and zeros (rows past the end of the factor).
//
// One "step" of the reduction covers RT output rows x WS output columns of one
// sample (RT*WS <= 64, rounded up to even for the 2-deep MFMA).
#pragma once

#include "mma_core.h"

namespace kfac {
namespace mma {

struct ConvGeom {
  const float *x;
  int C, H, W, kh, kw, sy, sx, ph, pw, ho, wo;
  int d_patch;      // C*kh*kw
  int append_ones;
  int WS, RT;       // output columns / rows per step
  int segs;         // column segments per output row
  int rgroups;      // row groups per sample
  int nk;           // k-values per step (even)
  int Rin, Win;     // staged input rows / columns per step
  int Wr, Rsz;      // LDS row stride / plane stride
  int CH;           // staged channel planes per panel
  // staging: thread t handles column t % LPR of channel t / LPR (+ CPP per
  // pass) for every staged row; element e of a thread is (pass, row) =
  // (nibble e of e_pass, nibble e of e_row)
  int LPR, CPP, passes, nq;
  unsigned long long e_pass, e_row;
  int goffE[16];    // element e: offset inside the sample, (pass*CPP*H + row) * W
  int loffE[16];    // element e: offset inside the region, pass*CPP*Rsz + row*Wr
};

constexpr int kHaloMaxQ = 16;   // staged elements per thread and panel
constexpr int kHaloMaxK = 64;   // k-values per step

struct HaloPanel {
  float v[kHaloMaxQ];
  unsigned okmask;     // bit e: element e of this step is inside the image
  // thread constants of the panel
  int rx;
  bool rx_in;
  unsigned g_thread;   // chq*H*W + rx
  unsigned l_thread;   // chq*Rsz + rx
  unsigned chreal;     // bit p: channel of pass p exists in the input
  unsigned chlive;     // bit p: channel of pass p has a plane in the region
  int c_lo;

  __device__ __forceinline__ void init(const ConvGeom &g, int row0) {
    c_lo = row0 / (g.kh * g.kw);
    const int chq = threadIdx.x / g.LPR;
    rx = threadIdx.x - chq * g.LPR;
    rx_in = rx < g.Win;
    g_thread = (unsigned)(chq * g.H * g.W + rx);
    l_thread = (unsigned)(chq * g.Rsz + rx);
    chreal = 0;
    chlive = 0;
    for (int p = 0; p < g.passes; ++p) {
      const int ch = p * g.CPP + chq;
      if (ch < g.CH) chlive |= 1u << p;
      if (ch < g.CH && c_lo + ch < g.C) chreal |= 1u << p;
    }
  }

  // Issue the loads of the region for the step whose first tap is input pixel
  // (iy0, ix0) of the sample at `sample_base`.  Element offsets are uniform
  // across the workgroup apart from the per-thread base.
  __device__ __forceinline__ void load(const ConvGeom &g, long long sample_base, int iy0, int ix0) {
    const float *p = g.x + sample_base + (long long)c_lo * g.H * g.W + (long long)iy0 * g.W + ix0 +
                     g_thread;
    const bool col_ok = rx_in && (unsigned)(ix0 + rx) < (unsigned)g.W;
    okmask = 0;
#pragma unroll
    for (int e = 0; e < kHaloMaxQ; ++e) {
      const int ps = (int)((g.e_pass >> (4 * e)) & 15), ry = (int)((g.e_row >> (4 * e)) & 15);
      const bool ok = e < g.nq && col_ok && ((chreal >> ps) & 1u) &&
                      (unsigned)(iy0 + ry) < (unsigned)g.H;
      const float *addr = ok ? p + g.goffE[e] : g.x;   // always valid
      v[e] = *addr;
      if (ok) okmask |= 1u << e;
    }
  }

  __device__ __forceinline__ void store(const ConvGeom &g, float *region) const {
#pragma unroll
    for (int e = 0; e < kHaloMaxQ; ++e) {
      const int ps = (int)((g.e_pass >> (4 * e)) & 15);
      if (e < g.nq && rx_in && ((chlive >> ps) & 1u))
        region[l_thread + g.loffE[e]] = ((okmask >> e) & 1u) ? v[e] : 0.f;
    }
  }
};

// LDS floats: two regions of (CH + 2) planes, the koff table, the row tables.
__host__ __device__ inline int halo_region_floats(const ConvGeom &g) { return (g.CH + 2) * g.Rsz; }

// NKK = k-values per step / 2, a compile-time constant so that the MFMA loop is
// fully unrolled and the per-lane k offsets live in registers.
template <int WM, int NKK, bool SAME>
__device__ __forceinline__ void halo_mainloop(const ConvGeom &g, int row0A, int row0B,
                                              long long sbeg, long long send, float *regA,
                                              float *regB, const int *koff_tbl,
                                              floatx16 (&acc)[WM][WM]) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane & 31, lk = lane >> 5;
  const int khkw = g.kh * g.kw;
  const int steps_per_sample = g.segs * g.rgroups;

  // operand row offsets of this lane (floats): plane of the row's channel + tap
  auto row_offset = [&](int row0, int r) {
    const int grow = row0 + r;
    const int c_lo = row0 / khkw;
    if (grow < g.d_patch) {
      const int c = grow / khkw;
      const int rem = grow - c * khkw;
      const int i = rem / g.kw;
      const int j = rem - i * g.kw;
      return (c - c_lo) * g.Rsz + i * g.Wr + j;
    }
    if (grow == g.d_patch && g.append_ones) return g.CH * g.Rsz;   // ones plane
    return (g.CH + 1) * g.Rsz;                                     // zero plane
  };
  int offA[WM], offB[WM];
#pragma unroll
  for (int im = 0; im < WM; ++im) {
    offA[im] = row_offset(row0A, (wm * WM + im) * 32 + lrow);
    offB[im] = row_offset(row0B, (wn * WM + im) * 32 + lrow);
  }
  const float *opB = SAME ? regA : regB;
  // per-lane k offsets (k = 2t + lk)
  int ko[NKK];
#pragma unroll
  for (int t = 0; t < NKK; ++t) ko[t] = koff_tbl[2 * t + lk];

  HaloPanel pa, pb;
  pa.init(g, row0A);
  if (!SAME) pb.init(g, row0B);

  auto decode = [&](long long s, long long &sample_base, int &iy0, int &ix0, int &orow0, int &ocol0) {
    const long long smp = s / steps_per_sample;
    const int rem = (int)(s - smp * steps_per_sample);
    const int rg = rem / g.segs;
    const int sg = rem - rg * g.segs;
    orow0 = rg * g.RT;
    ocol0 = sg * g.WS;
    iy0 = orow0 * g.sy - g.ph;
    ix0 = ocol0 * g.sx - g.pw;
    sample_base = smp * (long long)g.C * g.H * g.W;
  };

  long long sample_base;
  int iy0, ix0, orow0, ocol0;
  if (sbeg < send) {
    decode(sbeg, sample_base, iy0, ix0, orow0, ocol0);
    pa.load(g, sample_base, iy0, ix0);
    if (!SAME) pb.load(g, sample_base, iy0, ix0);
  }
  for (long long s = sbeg; s < send; ++s) {
    pa.store(g, regA);
    if (!SAME) pb.store(g, regB);
    // k-values at or past kcut lie below the image (row group hanging over the
    // bottom edge) or past the end of the step; their A operand is zeroed
    int kcut = (g.ho - orow0) * g.WS;
    if (kcut > g.RT * g.WS) kcut = g.RT * g.WS;
    __syncthreads();
    if (s + 1 < send) {
      decode(s + 1, sample_base, iy0, ix0, orow0, ocol0);
      pa.load(g, sample_base, iy0, ix0);
      if (!SAME) pb.load(g, sample_base, iy0, ix0);
    }
    // Opaque copies of the operand row offsets: without them the compiler
    // hoists all NKK * 2 * WM operand addresses out of the step loop and
    // spills.  (Offsets, not pointers, so the reads stay LDS instructions.)
    int qA[WM], qB[WM];
#pragma unroll
    for (int im = 0; im < WM; ++im) {
      qA[im] = offA[im];
      qB[im] = offB[im];
      asm volatile("" : "+v"(qA[im]), "+v"(qB[im]));
    }
#pragma unroll
    for (int t = 0; t < NKK; ++t) {
      float a[WM], b[WM];
#pragma unroll
      for (int im = 0; im < WM; ++im) {
        const float x = regA[qA[im] + ko[t]];
        a[im] = (2 * t + lk < kcut) ? x : 0.f;
      }
#pragma unroll
      for (int in = 0; in < WM; ++in) b[in] = opB[qB[in] + ko[t]];
#pragma unroll
      for (int im = 0; im < WM; ++im)
#pragma unroll
        for (int in = 0; in < WM; ++in)
          acc[im][in] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[im], b[in], acc[im][in], 0, 0, 0);
    }
    __syncthreads();
  }
}

}  // namespace mma
}  // namespace kfac
