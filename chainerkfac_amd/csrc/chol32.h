// Cholesky factorisation and triangular inverse of a 32x32 SPD block by one
// wave, in registers.  Shared by the batched inverse (diagonal tiles) and the
// low-rank batch-norm inverse.
#pragma once

#include <hip/hip_runtime.h>

namespace kfac {

constexpr int kChol32 = 32;

__device__ __forceinline__ float lane_bcast(float x, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), lane));
}

__device__ __forceinline__ double lane_bcast(double x, int lane) {
  const long long b = __double_as_longlong(x);
  const int lo = __builtin_amdgcn_readlane((int)(b & 0xffffffffLL), lane);
  const int hi = __builtin_amdgcn_readlane((int)(b >> 32), lane);
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// 1 / sqrt(x): the hardware estimate plus one Newton step in float32, the
// correctly rounded operations in float64.
__device__ __forceinline__ float inv_sqrt(float x) {
  const float r = __builtin_amdgcn_rsqf(x);
  return r * (1.5f - 0.5f * x * r * r);
}

__device__ __forceinline__ double inv_sqrt(double x) { return 1.0 / sqrt(x); }

// Wave 0: factor the 32x32 block at S[b0.., b0..] (lower) in registers and
// overwrite it with U32 = (L32^-1)^T (upper triangular, zeros below).
//
// Lanes 0..31 hold the rows of A, lanes 32..63 the columns of the identity: the
// column operations of the right-looking Cholesky (scale column j by
// 1/sqrt(pivot), subtract l_cj times it from column c) turn the first into L
// and, applied to the identity with the same multipliers, are exactly the
// forward substitution that turns the second into the columns of L^-1.  One
// broadcast of l_cj feeds both halves in the same instruction.
// Returns 0 or 1 + the local index of the first non-positive pivot.
template <int LS, class T>
__device__ __forceinline__ int chol_inv_32(T *S, int b0) {
  const int lane = threadIdx.x & 63;
  const int i = lane & 31;
  const bool chol = lane < kChol32;
  T x[kChol32];
#pragma unroll
  for (int c = 0; c < kChol32; ++c) {
    const T a = S[(b0 + i) * LS + b0 + c];
    x[c] = chol ? a : (c == i ? T(1) : T(0));
  }
  int bad = 0;
#pragma unroll
  for (int j = 0; j < kChol32; ++j) {
    const T piv = lane_bcast(x[j], j);
    if (!(piv > T(0)) && bad == 0) bad = j + 1;
    const T rinv = inv_sqrt(piv);
    x[j] *= rinv;
#pragma unroll
    for (int c = j + 1; c < kChol32; ++c) x[c] -= x[j] * lane_bcast(x[j], c);
  }
  // lane 32 + m holds column m of W = row m of U; entries with r < m are exact zeros
  if (!chol) {
#pragma unroll
    for (int r = 0; r < kChol32; ++r) S[(b0 + i) * LS + b0 + r] = x[r];
  }
  return bad;
}

}  // namespace kfac
