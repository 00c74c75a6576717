// Triangular pack / unpack of a list of arrays into one flat float32 buffer:
// the wire format of the reference communicator
// (chainerkfac/communicators/pure_nccl_communicator.py:221-463).
//
// Layout: arrays are concatenated in list order; a triangular array of side n
// takes n(n+1)/2 slots, slot r(r+1)/2 + c holding M[r, c] for c <= r; any
// other array is copied flat.
//
// Both kernels are bandwidth bound.  Work is cut into units that a workgroup
// finds with one wave-uniform binary search over a small cumulative table
// (the reference searches once per *element*):
//   pack    unit = 4096 consecutive packed slots of one array.  Packed slots
//           are walked linearly, so stores are fully coalesced and loads are
//           contiguous along each matrix row; the upper triangle is never
//           touched.
//   unpack  unit = one 64x64 tile (I >= J) of a triangular array: the tile's
//           row segments are read once from the buffer, written to M[I, J]
//           directly and to M[J, I] through an LDS transpose, so every global
//           access is a contiguous 256-byte run per wave.  Flat arrays use
//           4096-element chunks.
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kChunk = 4096;           // packed slots per pack unit
constexpr int kPerThread = kChunk / kThreads;
constexpr int kTile = 64;              // unpack tile side

struct PackTables {
  const float *const *ptrs;   // [n] array base pointers
  const int *tri;             // [n] side if triangular else 0
  const int *rank;            // [n]
  const long long *nel;       // [n] packed slots of the array
  const long long *buf_off;   // [n] first slot in the buffer
  const int *pack_csum;       // [n+1] cumulative pack units
  const int *unpack_csum;     // [n+1] cumulative unpack units
  int n;
};

// Index j with csum[j] <= unit < csum[j+1]; `unit` is wave-uniform so the
// search runs on the scalar unit.
__device__ __forceinline__ int find_array(const int *__restrict__ csum, int n,
                                          int unit) {
  int lo = 0, hi = n - 1;
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (csum[mid] <= unit)
      lo = mid;
    else
      hi = mid - 1;
  }
  return lo;
}

// Row of packed slot t: the largest r with r(r+1)/2 <= t.
__device__ __forceinline__ int tri_row(long long t) {
  long long r = (long long)((sqrt(8.0 * (double)t + 1.0) - 1.0) * 0.5);
  while (r * (r + 1) / 2 > t) --r;
  while ((r + 1) * (r + 2) / 2 <= t) ++r;
  return (int)r;
}

// Element type of the packed buffer: float, or __half for the float16 wire
// format (the arrays stay float32).  Conversions follow the reference kernels:
// pack stores (half)value, round to nearest even; unpack divides in the
// buffer's type, half / (half)divisor rounded to half, then widens.
__device__ __forceinline__ void to_buf(float v, float &out) { out = v; }
__device__ __forceinline__ void to_buf(float v, __half &out) { out = __float2half_rn(v); }

__device__ __forceinline__ float from_buf(float v, int divisor) {
  return divisor != 1 ? v / (float)divisor : v;
}
__device__ __forceinline__ float from_buf(__half v, int divisor) {
  // the float quotient of two halves rounds to the correctly rounded half quotient
  return __half2float(__float2half_rn(__half2float(v) / __half2float(__int2half_rn(divisor))));
}

// Workgroup i of a launch runs on XCD i % 8, each XCD with an L2 of its own.
// Every XCD takes one contiguous run of the unit list: neighbouring units touch
// neighbouring memory (the cache lines at the seams of two tiles or chunks), and
// a line that two workgroups each write half of is completed inside one L2
// instead of being written back twice as partial lines.
__device__ __forceinline__ int xcd_contiguous_unit(int total) {
  const int xcd = blockIdx.x % 8, idx = blockIdx.x / 8;
  const int base = total / 8, rem = total % 8;
  return xcd * base + (xcd < rem ? xcd : rem) + idx;
}

template <class B>
__global__ __launch_bounds__(kThreads) void pack_kernel(PackTables tb, B *__restrict__ buf,
                                                        int target) {
  const int unit = xcd_contiguous_unit(gridDim.x);
  const int j = find_array(tb.pack_csum, tb.n, unit);
  if (target >= 0 && tb.rank[j] != target) return;
  const long long nel = tb.nel[j];
  const long long t0 = (long long)(unit - tb.pack_csum[j]) * kChunk + threadIdx.x;
  const float *__restrict__ src = tb.ptrs[j];
  B *__restrict__ dst = buf + tb.buf_off[j];
  const int d = tb.tri[j];
  float val[kPerThread];
  if (d > 0) {
    int r = 0, c = 0;
    if (t0 < nel) {
      r = tri_row(t0);
      c = (int)(t0 - (long long)r * (r + 1) / 2);
    }
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const long long t = t0 + (long long)i * kThreads;
      val[i] = (t < nel) ? src[(long long)r * d + c] : 0.f;
      c += kThreads;
      while (c > r) {
        c -= r + 1;
        ++r;
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const long long t = t0 + (long long)i * kThreads;
      val[i] = (t < nel) ? src[t] : 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < kPerThread; ++i) {
    const long long t = t0 + (long long)i * kThreads;
    if (t < nel) to_buf(val[i], dst[t]);
  }
}

template <class B>
__global__ __launch_bounds__(kThreads) void unpack_kernel(PackTables tb, const B *__restrict__ buf,
                                                          int target, int divisor) {
  __shared__ float tile[kTile][kTile + 1];
  const int unit = xcd_contiguous_unit(gridDim.x);
  const int j = find_array(tb.unpack_csum, tb.n, unit);
  if (target >= 0 && tb.rank[j] != target) return;
  const int local = unit - tb.unpack_csum[j];
  float *__restrict__ dst = const_cast<float *>(tb.ptrs[j]);
  const B *__restrict__ src = buf + tb.buf_off[j];
  const int d = tb.tri[j];
  if (d == 0) {
    const long long nel = tb.nel[j];
    const long long t0 = (long long)local * kChunk + threadIdx.x;
    B val[kPerThread];
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const long long t = t0 + (long long)i * kThreads;
      if (t < nel) val[i] = src[t];
    }
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const long long t = t0 + (long long)i * kThreads;
      if (t < nel) dst[t] = from_buf(val[i], divisor);
    }
    return;
  }
  // tile (I, J), I >= J, from the unit index in row-major lower order
  const int I = tri_row(local);
  const int J = local - I * (I + 1) / 2;
  const int lc = threadIdx.x % kTile;   // column inside the tile
  const int lr0 = threadIdx.x / kTile;  // 0..3
  constexpr int kRowsPerPass = kThreads / kTile;
  constexpr int kPasses = kTile / kRowsPerPass;
  B val[kPasses];
  bool have[kPasses];
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int lr = lr0 + p * kRowsPerPass;
    const int r = I * kTile + lr;
    const int c = J * kTile + lc;
    have[p] = r < d && c <= r;
    if (have[p]) val[p] = src[(long long)r * (r + 1) / 2 + c];
  }
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int lr = lr0 + p * kRowsPerPass;
    tile[lr][lc] = have[p] ? from_buf(val[p], divisor) : 0.f;
  }
  __syncthreads();
  if (I == J) {
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int lr = lr0 + p * kRowsPerPass;
      const int r = I * kTile + lr;
      const int c = J * kTile + lc;
      if (r < d && c < d)
        dst[(long long)r * d + c] = (lc <= lr) ? tile[lr][lc] : tile[lc][lr];
    }
  } else {
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int lr = lr0 + p * kRowsPerPass;
      const int r = I * kTile + lr;
      const int c = J * kTile + lc;
      if (r < d) dst[(long long)r * d + c] = tile[lr][lc];  // c < r < d
      // mirrored tile (J, I): row J*64 + lr, column I*64 + lc
      const int mr = J * kTile + lr;
      const int mc = I * kTile + lc;
      if (mc < d) dst[(long long)mr * d + mc] = tile[lc][lr];  // mr < I*64 < d
    }
  }
}

}  // namespace

struct kfac_pack_plan {
  int n = 0;
  long long total_packed = 0;
  int pack_units = 0;
  int unpack_units = 0;
  std::vector<const void *> ptrs;
  kfac::DevTable d_ptrs, d_tri, d_rank, d_nel, d_off, d_pcs, d_ucs;
  PackTables tables() const {
    PackTables t;
    t.ptrs = d_ptrs.as<const float *const>();
    t.tri = d_tri.as<const int>();
    t.rank = d_rank.as<const int>();
    t.nel = d_nel.as<const long long>();
    t.buf_off = d_off.as<const long long>();
    t.pack_csum = d_pcs.as<const int>();
    t.unpack_csum = d_ucs.as<const int>();
    t.n = n;
    return t;
  }
};

extern "C" int64_t kfac_packed_nelems(int n_arrays, const int64_t *sizes,
                                      const int32_t *triangle_size) {
  int64_t total = 0;
  for (int i = 0; i < n_arrays; ++i) {
    const int64_t t = triangle_size[i];
    if (t > 0) {
      if (sizes[i] != t * t) {
        kfac::fail(KFAC_EINVAL, "array %d: size %lld is not triangle_size^2 (%lld)",
                   i, (long long)sizes[i], (long long)t);
        return -1;
      }
      total += t * (t + 1) / 2;
    } else {
      total += sizes[i];
    }
  }
  return total;
}

extern "C" int kfac_pack_plan_create(int n_arrays, const void *const *ptrs,
                                     const int64_t *sizes,
                                     const int32_t *triangle_size,
                                     const int32_t *rank_of,
                                     kfac_pack_plan_t *plan_out) {
  KFAC_REQUIRE(plan_out != nullptr, "plan_out is null");
  *plan_out = nullptr;
  KFAC_REQUIRE(n_arrays >= 0, "n_arrays < 0");
  KFAC_REQUIRE(n_arrays == 0 || (ptrs && sizes && triangle_size && rank_of),
               "null table");
  std::vector<int> tri(n_arrays), rank(n_arrays), pcs(n_arrays + 1), ucs(n_arrays + 1);
  std::vector<long long> nel(n_arrays), off(n_arrays);
  long long total = 0, punits = 0, uunits = 0;
  pcs[0] = ucs[0] = 0;
  for (int i = 0; i < n_arrays; ++i) {
    const long long t = triangle_size[i];
    KFAC_REQUIRE(sizes[i] >= 0 && t >= 0, "array %d: negative size", i);
    KFAC_REQUIRE(sizes[i] == 0 || ptrs[i] != nullptr, "array %d: null pointer", i);
    long long packed;
    if (t > 0) {
      KFAC_REQUIRE(sizes[i] == t * t, "array %d: size %lld is not triangle_size^2",
                   i, (long long)sizes[i]);
      packed = t * (t + 1) / 2;
      const long long tt = kfac::ceil_div<long long>(t, kTile);
      uunits += tt * (tt + 1) / 2;
    } else {
      packed = sizes[i];
      uunits += kfac::ceil_div<long long>(packed, kChunk);
    }
    punits += kfac::ceil_div<long long>(packed, kChunk);
    KFAC_REQUIRE(punits < 0x7fffffffLL && uunits < 0x7fffffffLL, "too many work units");
    tri[i] = (int)t;
    rank[i] = rank_of[i];
    nel[i] = packed;
    off[i] = total;
    total += packed;
    pcs[i + 1] = (int)punits;
    ucs[i + 1] = (int)uunits;
  }
  auto *p = new (std::nothrow) kfac_pack_plan;
  if (!p) return kfac::fail(KFAC_ENOMEM, "out of host memory");
  p->n = n_arrays;
  p->total_packed = total;
  p->pack_units = (int)punits;
  p->unpack_units = (int)uunits;
  p->ptrs.assign(ptrs, ptrs + n_arrays);
  int rc = KFAC_OK;
  hipStream_t s = nullptr;
  auto up = [&](kfac::DevTable &t, const void *h, size_t b) {
    if (rc == KFAC_OK) rc = t.set(h, b, s);
  };
  up(p->d_ptrs, p->ptrs.data(), sizeof(void *) * n_arrays);
  up(p->d_tri, tri.data(), sizeof(int) * n_arrays);
  up(p->d_rank, rank.data(), sizeof(int) * n_arrays);
  up(p->d_nel, nel.data(), sizeof(long long) * n_arrays);
  up(p->d_off, off.data(), sizeof(long long) * n_arrays);
  up(p->d_pcs, pcs.data(), sizeof(int) * (n_arrays + 1));
  up(p->d_ucs, ucs.data(), sizeof(int) * (n_arrays + 1));
  if (rc != KFAC_OK) {
    delete p;
    return rc;
  }
  *plan_out = p;
  return KFAC_OK;
}

extern "C" int kfac_pack_plan_set_ptrs(kfac_pack_plan_t plan,
                                       const void *const *ptrs, void *stream) {
  KFAC_REQUIRE(plan != nullptr, "plan is null");
  KFAC_REQUIRE(plan->n == 0 || ptrs != nullptr, "ptrs is null");
  plan->ptrs.assign(ptrs, ptrs + plan->n);
  return plan->d_ptrs.set(plan->ptrs.data(), sizeof(void *) * plan->n,
                          kfac::as_stream(stream));
}

extern "C" int64_t kfac_pack_plan_nelems(kfac_pack_plan_t plan) {
  return plan ? plan->total_packed : -1;
}

extern "C" int kfac_pack_plan_destroy(kfac_pack_plan_t plan) {
  delete plan;
  return KFAC_OK;
}

namespace {

template <class B>
int run_pack(kfac_pack_plan_t plan, B *buf, int64_t buf_nelems, int target_rank, void *stream) {
  KFAC_REQUIRE(plan != nullptr, "plan is null");
  KFAC_REQUIRE(buf_nelems >= plan->total_packed,
               "buffer holds %lld elements, %lld needed", (long long)buf_nelems,
               plan->total_packed);
  if (plan->pack_units == 0) return KFAC_OK;
  KFAC_REQUIRE(buf != nullptr, "buf is null");
  kfac::TimedLaunch timed(KFAC_TIMED_PACK, kfac::as_stream(stream));
  hipLaunchKernelGGL(pack_kernel<B>, dim3(plan->pack_units), dim3(kThreads), 0,
                     kfac::as_stream(stream), plan->tables(), buf, target_rank);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

template <class B>
int run_unpack(kfac_pack_plan_t plan, const B *buf, int64_t buf_nelems, int target_rank,
               int divisor, void *stream) {
  KFAC_REQUIRE(plan != nullptr, "plan is null");
  KFAC_REQUIRE(divisor != 0, "divisor is 0");
  KFAC_REQUIRE(buf_nelems >= plan->total_packed,
               "buffer holds %lld elements, %lld needed", (long long)buf_nelems,
               plan->total_packed);
  if (plan->unpack_units == 0) return KFAC_OK;
  KFAC_REQUIRE(buf != nullptr, "buf is null");
  kfac::TimedLaunch timed(KFAC_TIMED_UNPACK, kfac::as_stream(stream));
  hipLaunchKernelGGL(unpack_kernel<B>, dim3(plan->unpack_units), dim3(kThreads), 0,
                     kfac::as_stream(stream), plan->tables(), buf, target_rank, divisor);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

}  // namespace

namespace {

// Plain streaming copy, 16 bytes per lane and load, four loads in flight per
// lane: the yardstick for the bandwidth-bound kernels of this file.
__global__ __launch_bounds__(kThreads) void stream_copy_kernel(const float4 *__restrict__ src,
                                                               float4 *__restrict__ dst,
                                                               long long n4) {
  const long long base = (long long)blockIdx.x * (kThreads * 4) + threadIdx.x;
  float4 v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long long t = base + (long long)i * kThreads;
    if (t < n4) v[i] = src[t];
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long long t = base + (long long)i * kThreads;
    if (t < n4) dst[t] = v[i];
  }
}

__global__ __launch_bounds__(kThreads) void stream_copy_tail_kernel(const float *__restrict__ src,
                                                                    float *__restrict__ dst,
                                                                    long long from, long long n) {
  const long long t = from + threadIdx.x;
  if (t < n) dst[t] = src[t];
}

}  // namespace

extern "C" int kfac_stream_copy_f32(float *dst, const float *src, int64_t nelems, void *stream) {
  KFAC_REQUIRE(nelems >= 0, "nelems < 0");
  if (nelems == 0) return KFAC_OK;
  KFAC_REQUIRE(dst && src, "null pointer");
  KFAC_REQUIRE(((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) == 0,
               "pointers must be 16-byte aligned");
  hipStream_t s = kfac::as_stream(stream);
  const long long n4 = nelems / 4;
  {
    kfac::TimedLaunch timed(KFAC_TIMED_COPY, s);
    if (n4 > 0)
      hipLaunchKernelGGL(stream_copy_kernel, dim3((unsigned)kfac::ceil_div<long long>(n4, kThreads * 4)),
                         dim3(kThreads), 0, s, reinterpret_cast<const float4 *>(src),
                         reinterpret_cast<float4 *>(dst), n4);
    if (n4 * 4 < nelems)
      hipLaunchKernelGGL(stream_copy_tail_kernel, dim3(1), dim3(kThreads), 0, s, src, dst, n4 * 4,
                         (long long)nelems);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

extern "C" int kfac_pack_f32(kfac_pack_plan_t plan, float *buf, int64_t buf_nelems,
                             int target_rank, void *stream) {
  return run_pack(plan, buf, buf_nelems, target_rank, stream);
}

extern "C" int kfac_unpack_f32(kfac_pack_plan_t plan, const float *buf, int64_t buf_nelems,
                               int target_rank, int divisor, void *stream) {
  return run_unpack(plan, buf, buf_nelems, target_rank, divisor, stream);
}

extern "C" int kfac_pack_f16(kfac_pack_plan_t plan, void *buf, int64_t buf_nelems,
                             int target_rank, void *stream) {
  return run_pack(plan, static_cast<__half *>(buf), buf_nelems, target_rank, stream);
}

extern "C" int kfac_unpack_f16(kfac_pack_plan_t plan, const void *buf, int64_t buf_nelems,
                               int target_rank, int divisor, void *stream) {
  return run_unpack(plan, static_cast<const __half *>(buf), buf_nelems, target_rank, divisor,
                    stream);
}
