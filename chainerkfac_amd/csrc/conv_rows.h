// Covariance of convolution patches for the common case of a k x k convolution
// whose output rows are at most 64 pixels wide: a kernel whose geometry is a
// compile-time constant, so that nothing in its inner loop needs a vector ALU
// instruction next to the matrix instructions.
//
// One reduction "step" covers RT whole output rows of a PAIR of samples.  The
// workgroup stages the input rows those output rows need (RIN = (RT-1)*S + K
// full-width rows of up to CH channels, zero padding included) for both samples
// in LDS, and every MFMA operand
//     P[(c, i, j), (oy, ox)] = x[c, oy*S - P + i, ox*S - P + j]
// is read at   rowoff(c, i, j) + sample * REGION + (oy*S*WR + ox*S),
// where the last term is an instruction immediate: the two halves of a wave
// (which supply the two k-values of v_mfma_f32_32x32x2_f32) take the same pixel
// of the two samples, so both use the same immediate and differ only in their
// base register.  Loads of neighbouring pixels merge into ds_read2_b32.
//
// Staging needs no vector ALU work either.  A wave's load instruction covers 64
// (channel, column) pairs of ONE input row: the per-lane part of the address
// (channel, column) is the same for every row and every step and lives in a few
// registers, the row / sample / step part is wave-uniform and goes into the
// scalar offset of the buffer load, and a row outside the image is read through
// a descriptor of size zero (the hardware then returns 0), chosen with scalar
// selects.  The LDS slot of a loaded element is a per-lane constant plus an
// immediate.
#pragma once

#include "mma_core.h"

namespace kfac {
namespace mma {

struct RowsGeom {
  const float *x;
  int n, C, H, W;       // NCHW input
  int ho;               // output rows (the output width is the template's WS)
  int rgroups;          // ho / RT
  int d_patch;          // C * K * K
  unsigned x_bytes;     // size of x in bytes (below 2^31)
};

// PAD_: floats added to the stride between channel planes.  The 32 lanes of an
// operand fetch read 32 consecutive patch rows (c, i, j), at plane stride * c +
// WR * i + j; the pad is chosen per shape so that these fall into different LDS
// banks as far as possible.
template <int WM_, int K_, int S_, int P_, int WS_, int RT_, int PAD_>
struct RowsCfg {
  static constexpr int WM = WM_, K = K_, S = S_, P = P_, WS = WS_, RT = RT_;
  static constexpr int BM = 64 * WM;
  static constexpr int KK = K * K;
  static constexpr int CH = (BM - 1) / KK + 2;    // channel planes a panel of BM patch rows can touch
  static constexpr int RIN = (RT - 1) * S + K;    // staged input rows per step
  static constexpr int WIN = (WS - 1) * S + K;    // staged columns per row, padding included
  static constexpr int NCOL = WIN - P;            // columns that can hold input (ix = 0 .. NCOL-1)
  static constexpr int WR = WIN;                  // LDS row stride
  static constexpr int RSZ = RIN * WR + PAD_;     // plane stride
  // CH planes, a plane of zeros, and a tail that absorbs the stores of lanes without a pair
  // (their slot is TAIL0 + lane, to which the row immediate ry * WR is added like to any other);
  // the two samples' regions are 32 banks apart
  static constexpr int TAIL0 = (CH + 1) * RSZ;
  static constexpr int REGION = (TAIL0 + RIN * WR + 64 + 31) / 64 * 64 + 32;
  static constexpr int PAIRS = CH * NCOL;         // (channel, column) pairs of one staged row
  static constexpr int PARTS = (PAIRS + THREADS - 1) / THREADS;
  static constexpr int NK = RT * WS;              // pixels per sample and step = MFMA k-steps
  // regions: operand A sample 0 / 1, operand B sample 0 / 1
  static constexpr int lds_floats(bool same) {
    const int f = (same ? 2 : 4) * REGION;
    return f > 64 * 65 ? f : 64 * 65;             // the epilogue transposes through the same memory
  }
  static constexpr int imm(int t) { return (t / WS) * S * WR + (t % WS) * S; }
};

// SAME: diagonal tile (B operand = A panel); the lane then also sums the A
// operand values it feeds to the matrix cores into rs[im]: rs ends as the sum
// over this lane's sample of row (wave_m * WM + im) * 32 + lane % 32; the other
// sample's half is in lane ^ 32.
template <class Cfg, bool SAME>
__device__ __forceinline__ void rows_mainloop(const RowsGeom &g, int row0A, int row0B,
                                              long long sbeg, long long send, float *smem,
                                              floatx16 (&acc)[Cfg::WM][Cfg::WM],
                                              float (&rs)[Cfg::WM], int wave) {
  constexpr int WM = Cfg::WM, KK = Cfg::KK, K = Cfg::K, S = Cfg::S, P = Cfg::P;
  constexpr int RIN = Cfg::RIN, WR = Cfg::WR, RSZ = Cfg::RSZ, REGION = Cfg::REGION;
  constexpr int PARTS = Cfg::PARTS, NK = Cfg::NK, CH = Cfg::CH, NCOL = Cfg::NCOL;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane & 31, lk = lane >> 5;
  const int HW = g.H * g.W;
  constexpr int regA = 0, regB = SAME ? 0 : 2 * REGION;

  // ---- operand base offsets of this lane: region of its sample + plane of the row's channel + tap
  const int c_loA = row0A / KK, c_loB = row0B / KK;
  auto row_offset = [&](int row0, int c_lo, int r) {
    const int grow = row0 + r;
    if (grow < g.d_patch) {
      const int c = grow / KK;
      const int rem = grow - c * KK;
      const int i = rem / K;
      return (c - c_lo) * RSZ + i * WR + (rem - i * K);
    }
    return CH * RSZ;   // plane of zeros
  };
  int qA[WM], qB[WM];
#pragma unroll
  for (int im = 0; im < WM; ++im) {
    qA[im] = regA + lk * REGION + row_offset(row0A, c_loA, (wm * WM + im) * 32 + lrow);
    qB[im] = regB + lk * REGION + row_offset(row0B, c_loB, (wn * WM + im) * 32 + lrow);
  }

  // ---- staging constants of this lane: pair m = (part * 4 + wave) * 64 + lane -> (channel, column)
  int voffA[PARTS], voffB[PARTS], lslot[PARTS];
#pragma unroll
  for (int p = 0; p < PARTS; ++p) {
    const int m = (p * 4 + wave) * 64 + lane;
    const int ch = m / NCOL, ix = m - ch * NCOL;
    const bool pair_ok = m < Cfg::PAIRS;
    const bool col_ok = pair_ok && ix < g.W;
    const int off = (ch * HW + ix) * 4;
    // an offset with bit 31 set lies past the end of the descriptor: the load returns 0
    voffA[p] = (col_ok && c_loA + ch < g.C) ? off : (int)0x80000000u;
    voffB[p] = (col_ok && c_loB + ch < g.C) ? off : (int)0x80000000u;
    lslot[p] = pair_ok ? ch * RSZ + ix + P : Cfg::TAIL0 + lane;
  }

  // ---- step state (wave-uniform): sample pair and row group
  long long pair_idx = sbeg / g.rgroups;
  int rg = (int)(sbeg - pair_idx * g.rgroups);
  const int sample_bytes = g.C * HW * 4;
  int pair4 = (int)(pair_idx * 2) * sample_bytes;   // byte offset of the pair's first sample

  float va[2][RIN * PARTS], vb[SAME ? 1 : 2][SAME ? 1 : RIN * PARTS];
  auto issue = [&]() {
    const int iy0 = rg * (Cfg::RT * S) - P;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int ry = 0; ry < RIN; ++ry) {
        const int iy = iy0 + ry;
        // a row outside the image is read through a descriptor of size zero: every lane gets 0
        const bool row_ok = (unsigned)iy < (unsigned)g.H;
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(g.x), (short)0, row_ok ? (int)g.x_bytes : 0, 0x00020000);
        const int row4 = pair4 + s * sample_bytes + iy * g.W * 4;
#pragma unroll
        for (int p = 0; p < PARTS; ++p) {
          va[s][ry * PARTS + p] = __builtin_bit_cast(
              float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voffA[p],
                                                          row4 + c_loA * HW * 4, 0));
          if (!SAME)
            vb[s][ry * PARTS + p] = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voffB[p],
                                                            row4 + c_loB * HW * 4, 0));
        }
      }
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int ry = 0; ry < RIN; ++ry)
#pragma unroll
        for (int p = 0; p < PARTS; ++p) {
          smem[regA + s * REGION + ry * WR + lslot[p]] = va[s][ry * PARTS + p];
          if (!SAME) smem[regB + s * REGION + ry * WR + lslot[p]] = vb[s][ry * PARTS + p];
        }
  };
  auto advance = [&]() {
    if (++rg == g.rgroups) {
      rg = 0;
      pair4 += 2 * sample_bytes;
    }
  };

  // a wave whose 64 x 64 block lies above the diagonal or past the end of the
  // factor stages like the others but leaves the matrix cores to them
  const bool active = syrk_wave_active<WM>(row0A, row0B, g.d_patch, wave);
  if (sbeg < send) issue();
  for (long long s = sbeg; s < send; ++s) {
    stash();
    __syncthreads();
    if (s + 1 < send) {
      advance();
      issue();
    }
    if (active) {
    // Opaque copies of the operand bases: without them the compiler folds base +
    // immediate for every k-step into registers of their own and spills.
    int pA[WM], pB[WM];
#pragma unroll
    for (int im = 0; im < WM; ++im) {
      pA[im] = qA[im];
      pB[im] = qB[im];
      asm volatile("" : "+v"(pA[im]), "+v"(pB[im]));
    }
    // software pipeline in stages of two k-steps: the operands of stage u+1 are
    // fetched from LDS before the MFMAs of stage u issue
    constexpr int NST = (NK + 1) / 2;
    float a[2][2][WM], b[2][2][WM];
    auto fetch = [&](int u, int buf) {
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int t = 2 * u + e;
        if (t < NK) {
#pragma unroll
          for (int im = 0; im < WM; ++im) a[buf][e][im] = smem[pA[im] + Cfg::imm(t)];
#pragma unroll
          for (int in = 0; in < WM; ++in) b[buf][e][in] = smem[pB[in] + Cfg::imm(t)];
        }
      }
    };
    fetch(0, 0);
#pragma unroll
    for (int u = 0; u < NST; ++u) {
      const int cur = u & 1;
      if (u + 1 < NST) fetch(u + 1, cur ^ 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        if (2 * u + e < NK) {
          if (SAME) {
#pragma unroll
            for (int im = 0; im < WM; ++im) rs[im] += a[cur][e][im];
          }
#pragma unroll
          for (int im = 0; im < WM; ++im)
#pragma unroll
            for (int in = 0; in < WM; ++in)
              acc[im][in] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][e][im], b[cur][e][in],
                                                                 acc[im][in], 0, 0, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    }
    __syncthreads();
  }
}

}  // namespace mma
}  // namespace kfac
