// Covariance of convolution patches (the A factor of a k x k convolution,
// k > 1) without forming patches anywhere: the workgroup stages the raw input
// region ("halo") that a block of output pixels needs -- a few input rows of up
// to 16 channels -- in LDS once, and every MFMA operand
//     P[(c, i, j), (oy, ox)] = x[c, oy*sy - ph + i, ox*sx - pw + j]
// is read straight from that region at address rowoff(c, i, j) + koff(oy, ox).
// A 3x3 patch row re-reads each staged input element nine times from LDS, so
// global loads and their address arithmetic drop ~9x compared with gathering
// the patch matrix element by element; zero padding is written into the region
// when it is staged.  (A bias column never reaches this loop: the caller takes
// it from the row sums the diagonal tiles accumulate.)
//
// Region layout per panel (128 rows of (c,i,j)): plane ch (input channel
// c_lo + ch) at ch*Rsz, element (ry, rx) at ry*Wr + rx, with Wr = kw and
// Rsz = kh*kw (mod 32): the 32 consecutive patch rows an MFMA operand fetch
// touches then fall into 32 different LDS banks.  One extra plane holds zeros
// (rows past the end of the factor).
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
  int WS, RT;       // output columns / rows per step
  int segs;         // column segments per output row
  int rgroups;      // row groups per sample
  int nk;           // k-values per step (even)
  int Rin, Win;     // staged input rows / columns per step
  int Wr, Rsz;      // LDS row stride / plane stride
  int CH;           // staged channel planes per panel
  // staging: thread t handles column t % LPR of channel t / LPR (+ CPP per
  // pass) for every staged row; element e of a thread is (pass, row) =
  // (e / Rin, e % Rin), nq = passes * Rin of them
  int LPR, CPP, passes, nq;
  unsigned rep;      // sum over passes of 1 << (pass * Rin)
  unsigned x_bytes;  // size of x in bytes (below 2^31)
};

constexpr int kHaloMaxQ = 16;   // staged elements per thread and panel
constexpr int kHaloMaxK = 64;   // k-values per step
constexpr int kHaloDump = 32;   // floats after each region that absorb stores of idle threads

// LDS floats of one region: CH channel planes, the zero plane and the dump slots.
__host__ __device__ inline int halo_region_floats(const ConvGeom &g) {
  return (g.CH + 1) * g.Rsz + kHaloDump;
}

// NKK = k-values per step / 2, a compile-time constant so that the MFMA loop is
// fully unrolled and the per-lane k offsets live in registers.
//
// Staging is branch-free per element: the input is read through a raw buffer
// descriptor, and an element outside the image (zero padding, a channel past
// the end of the input) gets bit 31 set in its byte offset, which puts it past
// the descriptor's size so that the load returns 0 without touching memory.
// Everything about an element that does not change from step to step (its
// offset inside a sample, its LDS slot, whether its channel and column exist)
// is computed once per workgroup and kept in registers.
// With SAME (diagonal tile) the lane also sums the A operand values it feeds to
// the matrix cores into rs[im] (half of the row sum of row (wave_m * WM + im) *
// 32 + lane % 32: the other half is in lane ^ 32).
template <int WM, int NKK, bool SAME, bool MASK>
__device__ __forceinline__ void halo_mainloop(const ConvGeom &g, int row0A, int row0B,
                                              long long sbeg, long long send, float *smem,
                                              int regA, int regB, const int *koff_tbl,
                                              floatx16 (&acc)[WM][WM], float (&rs)[WM]) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane & 31, lk = lane >> 5;
  const int khkw = g.kh * g.kw;
  const int HW = g.H * g.W;

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
    return g.CH * g.Rsz;   // zero plane
  };
  int offA[WM], offB[WM];
#pragma unroll
  for (int im = 0; im < WM; ++im) {
    offA[im] = regA + row_offset(row0A, (wm * WM + im) * 32 + lrow);
    offB[im] = (SAME ? regA : regB) + row_offset(row0B, (wn * WM + im) * 32 + lrow);
  }
  // per-lane k offsets (k = 2t + lk)
  int ko[NKK];
#pragma unroll
  for (int t = 0; t < NKK; ++t) ko[t] = koff_tbl[2 * t + lk];

  // ---- per-thread staging constants
  const int c_loA = row0A / khkw, c_loB = row0B / khkw;
  const int chq = tid / g.LPR;
  const int rx = tid - chq * g.LPR;
  int goff[kHaloMaxQ];   // byte offset of the element inside a sample, from channel c_lo
  int loff[kHaloMaxQ];   // float offset of its LDS slot inside a region
  unsigned tmaskA = 0, tmaskB = 0;
  {
    const int dump = (g.CH + 1) * g.Rsz + (tid & (kHaloDump - 1));
    int ps = 0, ry = 0;
#pragma unroll
    for (int e = 0; e < kHaloMaxQ; ++e) {
      const int ch = ps * g.CPP + chq;
      const bool live = e < g.nq && rx < g.Win && ch < g.CH;
      goff[e] = (ch * HW + ry * g.W + rx) * 4;
      loff[e] = live ? ch * g.Rsz + ry * g.Wr + rx : dump;
      if (live && c_loA + ch < g.C) tmaskA |= 1u << e;
      if (live && c_loB + ch < g.C) tmaskB |= 1u << e;
      if (++ry == g.Rin) { ry = 0; ++ps; }
    }
  }
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(g.x), (short)0, (int)g.x_bytes, 0x00020000);

  // ---- step state (uniform): position inside the sample and byte offset of the sample
  const int steps_per_sample = g.segs * g.rgroups;
  const long long smp0 = sbeg / steps_per_sample;
  int rg, sg;
  {
    const int rem = (int)(sbeg - smp0 * steps_per_sample);
    rg = rem / g.segs;
    sg = rem - rg * g.segs;
  }
  int sample4 = (int)(smp0 * g.C * HW * 4);
  const int sample_stride4 = g.C * HW * 4;

  float va[kHaloMaxQ], vb[kHaloMaxQ];
  auto issue = [&](float (&v)[kHaloMaxQ], unsigned tmask, int c_lo) {
    const int iy0 = rg * g.RT * g.sy - g.ph, ix0 = sg * g.WS * g.sx - g.pw;
    // rows of the region inside the image: [rlo, rhi)
    const int rlo = iy0 < 0 ? -iy0 : 0;
    int rhi = g.H - iy0;
    if (rhi > g.Rin) rhi = g.Rin;
    const unsigned rowbits = rhi > rlo ? (1u << rhi) - (1u << rlo) : 0u;
    const unsigned emask = rowbits * g.rep;
    const bool col_ok = (unsigned)(ix0 + rx) < (unsigned)g.W;
    const unsigned ninv = col_ok ? ~(tmask & emask) : ~0u;
    const int step4 = sample4 + (c_lo * HW + iy0 * g.W + ix0) * 4;
#pragma unroll
    for (int e0 = 0; e0 < kHaloMaxQ; e0 += 4) {
      if (e0 < g.nq) {
#pragma unroll
        for (int e = e0; e < e0 + 4; ++e) {
          const unsigned bad = ninv << (31 - e);
          const unsigned voff = ((unsigned)(goff[e] + step4) & 0x7fffffffu) | (bad & 0x80000000u);
          v[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)voff, 0, 0));
        }
      }
    }
  };
  auto stash = [&](const float (&v)[kHaloMaxQ], int reg) {
#pragma unroll
    for (int e0 = 0; e0 < kHaloMaxQ; e0 += 4) {
      if (e0 < g.nq) {
#pragma unroll
        for (int e = e0; e < e0 + 4; ++e) smem[reg + loff[e]] = v[e];
      }
    }
  };
  auto advance = [&]() {
    if (++sg == g.segs) {
      sg = 0;
      if (++rg == g.rgroups) {
        rg = 0;
        sample4 += sample_stride4;
      }
    }
  };

  if (sbeg < send) {
    issue(va, tmaskA, c_loA);
    if (!SAME) issue(vb, tmaskB, c_loB);
  }
  for (long long s = sbeg; s < send; ++s) {
    stash(va, regA);
    if (!SAME) stash(vb, regB);
    // k-values at or past kcut lie below the image (row group hanging over the
    // bottom edge) or past the end of the step; their A operand is zeroed
    int kcut = (g.ho - rg * g.RT) * g.WS;
    if (kcut > g.RT * g.WS) kcut = g.RT * g.WS;
    __syncthreads();
    if (s + 1 < send) {
      advance();
      issue(va, tmaskA, c_loA);
      if (!SAME) issue(vb, tmaskB, c_loB);
    }
    // Opaque copies of the operand row offsets: without them the compiler
    // hoists all NKK * 2 * WM operand addresses out of the step loop and
    // spills.
    int qA[WM], qB[WM];
#pragma unroll
    for (int im = 0; im < WM; ++im) {
      qA[im] = offA[im];
      qB[im] = offB[im];
      asm volatile("" : "+v"(qA[im]), "+v"(qB[im]));
    }
    // two-stage software pipeline: the operands of step t+1 are fetched from
    // LDS before the MFMAs of step t issue
    float a[2][WM], b[2][WM];
    auto fetch_t = [&](int t, int buf) {
      const bool kv = !MASK || lk < kcut - 2 * t;
#pragma unroll
      for (int im = 0; im < WM; ++im) {
        const float x = smem[qA[im] + ko[t]];
        a[buf][im] = kv ? x : 0.f;
      }
#pragma unroll
      for (int in = 0; in < WM; ++in) b[buf][in] = smem[qB[in] + ko[t]];
    };
    fetch_t(0, 0);
#pragma unroll
    for (int t = 0; t < NKK; ++t) {
      const int cur = t & 1;
      if (t + 1 < NKK) fetch_t(t + 1, cur ^ 1);
      // keep the scheduler from sinking those reads below the MFMAs (it does,
      // to save three registers, and then every MFMA waits for its operand)
      __builtin_amdgcn_sched_barrier(0);
      if (SAME) {
#pragma unroll
        for (int im = 0; im < WM; ++im) rs[im] += a[cur][im];
      }
#pragma unroll
      for (int im = 0; im < WM; ++im)
#pragma unroll
        for (int in = 0; in < WM; ++in)
          acc[im][in] =
              __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][im], b[cur][in], acc[im][in], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  }
}

}  // namespace mma
}  // namespace kfac
