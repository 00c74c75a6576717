// Triangular pack / unpack of a list of arrays into one flat float32 buffer:
// the wire format of the reference communicator
// (chainerkfac/communicators/pure_nccl_communicator.py:221-463).
//
// Layout: arrays are concatenated in list order; a triangular array of side n
// takes n(n+1)/2 slots, slot r(r+1)/2 + c holding M[r, c] for c <= r; any
// other array is copied flat.
//
// Both kernels are bandwidth bound and move 16 bytes per lane and access, at
// float granularity (neither the packed rows nor the rows of an odd-sized matrix
// start on 16-byte boundaries).  Work is cut into units; a per-unit owner table
// tells a workgroup its array with one load (the reference searches once per
// *element*):
//   pack    unit = 512 aligned quads of buffer slots (2048 slots) of one array, a
//           thread fills two of them: packed slots are walked linearly, so stores
//           are aligned and fully coalesced and loads are contiguous along each
//           matrix row; the upper triangle is never touched.  Units are dealt
//           round-robin to the XCDs, stores are streaming (non-temporal) stores.
//   unpack  unit = one 64x64 tile (I >= J) of a triangular array: the tile's
//           row segments are read once from the buffer, written to M[I, J]
//           directly and to M[J, I] through an LDS transpose, so every global
//           access is a contiguous 256-byte run per 16 lanes.  Flat arrays use
//           4096-element chunks.  Units of matrices whose rows start on cache
//           lines (sides that are multiples of 32) are dealt round-robin too; of
//           the others every XCD takes a contiguous run, so that a line two
//           neighbouring tiles each write a part of is completed inside one L2.
// Measured on an MI355X (ResNet-50-D factor list, 0.53 GB packed): pack 5.7 TB/s,
// unpack 5.5 TB/s; a kernel that only reads n and writes 2 n bytes (unpack's mix)
// reaches 6.0 TB/s, a plain copy 6.2 - 6.6 TB/s.  What did not help: streaming
// loads (slower for unpack), streaming stores in unpack (rows that are not
// line-aligned then never merge in L2), more than two quads per thread.
#include <hip/hip_fp16.h>

#include <algorithm>

#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kChunk = 4096;           // packed slots per pack unit
constexpr int kTile = 64;              // unpack tile side
constexpr int kPackU = 2;              // quads of buffer slots per thread of the pack kernel
constexpr int kUnpackThreads = 512;    // threads of an unpack workgroup (two passes over a tile)
constexpr int kPackQuads = kThreads * kPackU;

struct PackTables {
  const float *const *ptrs;   // [n] array base pointers
  const int *tri;             // [n] side if triangular else 0
  const int *rank;            // [n]
  const long long *nel;       // [n] packed slots of the array
  const long long *buf_off;   // [n] first slot in the buffer
  const int *pack_csum;       // [n+1] cumulative pack units
  const int *unpack_csum;     // [n+1] cumulative unpack units
  const int *pack_owner;      // [pack units] array of each unit (one load instead of a search)
  const int2 *unpack_sched;   // [unpack workgroups] {unit, array}; unit < 0: nothing to do
  int n;
};

// Row of packed slot t: the largest r with r(r+1)/2 <= t.  t < 2^30 (a triangle of
// side <= 46340), so 32-bit arithmetic holds every r(r+1)/2 that is compared; the
// float estimate is off by one at most and the two loops correct it.
__device__ __forceinline__ int tri_row(unsigned t) {
  int r = (int)((__builtin_sqrtf(8.f * (float)t + 1.f) - 1.f) * 0.5f);
  while ((unsigned)r * (unsigned)(r + 1) / 2u > t) --r;
  while ((unsigned)(r + 1) * (unsigned)(r + 2) / 2u <= t) ++r;
  return r;
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

// Four consecutive buffer slots as one access.
typedef float floatx4u __attribute__((ext_vector_type(4), aligned(4)));   // 16-byte load at any float address
typedef float floatx4a __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_quad(float *p, const float (&v)[4]) {
  floatx4a o;
  o.x = v[0];
  o.y = v[1];
  o.z = v[2];
  o.w = v[3];
  // streamed: the buffer is next read by another kernel (or the network), not by this one
  __builtin_nontemporal_store(o, reinterpret_cast<floatx4a *>(p));
}
__device__ __forceinline__ floatx4u load_quad(const float *p) {
  return *reinterpret_cast<const floatx4u *>(p);
}
__device__ __forceinline__ void store_quad(__half *p, const float (&v)[4]) {
  __half2 lo = __halves2half2(__float2half_rn(v[0]), __float2half_rn(v[1]));
  __half2 hi = __halves2half2(__float2half_rn(v[2]), __float2half_rn(v[3]));
  uint2 u;
  u.x = *reinterpret_cast<unsigned *>(&lo);
  u.y = *reinterpret_cast<unsigned *>(&hi);
  *reinterpret_cast<uint2 *>(p) = u;
}

// pack: a thread fills one aligned quad of buffer slots (slots 4q .. 4q + 3 of the
// whole buffer, so that the store is one aligned 16-byte access whatever the
// array's offset in the buffer) from four consecutive elements of a matrix row
// (one 16-byte load; a quad that runs over the end of a row, or that the array
// only partly owns at its first or last slot, goes element by element).  U quads
// per thread, 256 U quads per unit.
template <class B, int U>
__global__ __launch_bounds__(kThreads) void pack_kernel(PackTables tb, B *__restrict__ buf,
                                                        int target) {
  const int unit = blockIdx.x;
  const int j = tb.pack_owner[unit];
  if (target >= 0 && tb.rank[j] != target) return;
  const long long nel = tb.nel[j];
  const long long off = tb.buf_off[j];
  const float *__restrict__ src = tb.ptrs[j];
  const int d = tb.tri[j];
  const long long q0 = (long long)(unit - tb.pack_csum[j]) * (kThreads * U) + threadIdx.x;
  float val[U][4];
  long long t[U];
#pragma unroll
  for (int i = 0; i < U; ++i) {
    // first slot of the quad relative to the array: -3 .. nel - 1
    t[i] = ((off >> 2) + q0 + (long long)i * kThreads) * 4 - off;
    const long long tq = t[i];
    if (tq >= nel) continue;
    if (d > 0) {
      const unsigned tc = tq > 0 ? (unsigned)tq : 0u;
      int r = tri_row(tc);
      int c = (int)(tc - (unsigned)r * (unsigned)(r + 1) / 2u);
      if (tq >= 0 && tq + 3 < nel && c + 3 <= r) {
        const floatx4u v = load_quad(src + (long long)r * d + c);
        val[i][0] = v.x;
        val[i][1] = v.y;
        val[i][2] = v.z;
        val[i][3] = v.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const long long te = tq + e;
          val[i][e] = 0.f;
          if (te >= 0 && te < nel) {
            val[i][e] = src[(long long)r * d + c];
            if (++c > r) {
              c = 0;
              ++r;
            }
          }
        }
      }
    } else if (tq >= 0 && tq + 3 < nel) {
      const floatx4u v = load_quad(src + tq);
      val[i][0] = v.x;
      val[i][1] = v.y;
      val[i][2] = v.z;
      val[i][3] = v.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const long long te = tq + e;
        val[i][e] = (te >= 0 && te < nel) ? src[te] : 0.f;
      }
    }
  }
  B *__restrict__ dst = buf + off;
#pragma unroll
  for (int i = 0; i < U; ++i) {
    const long long tq = t[i];
    if (tq >= nel) continue;
    if (tq >= 0 && tq + 3 < nel) {
      store_quad(dst + tq, val[i]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (tq + e >= 0 && tq + e < nel) to_buf(val[i][e], dst[tq + e]);
    }
  }
}

// Four consecutive buffer elements, scaled: one 16-byte load for a float buffer.
__device__ __forceinline__ void load_scaled4(const float *p, int divisor, float (&o)[4]) {
  const floatx4u v = load_quad(p);
  o[0] = from_buf(v.x, divisor);
  o[1] = from_buf(v.y, divisor);
  o[2] = from_buf(v.z, divisor);
  o[3] = from_buf(v.w, divisor);
}
__device__ __forceinline__ void load_scaled4(const __half *p, int divisor, float (&o)[4]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = from_buf(p[e], divisor);
}
// Four consecutive floats of an array at any float address, as one 16-byte store.
__device__ __forceinline__ void store_row4(float *p, const float (&v)[4]) {
  floatx4u o;
  o.x = v[0];
  o.y = v[1];
  o.z = v[2];
  o.w = v[3];
  *reinterpret_cast<floatx4u *>(p) = o;
}

// unpack: a thread moves four consecutive elements of a row at a time (16-byte
// accesses at float granularity: neither the packed rows nor the rows of an
// odd-sized matrix start on 16-byte boundaries).
template <class B, int TH>
__global__ __launch_bounds__(TH) void unpack_kernel(PackTables tb, const B *__restrict__ buf,
                                                    int target, int divisor) {
  __shared__ float tile[kTile][kTile + 1];
  const int2 sched = tb.unpack_sched[blockIdx.x];
  const int unit = sched.x, j = sched.y;
  if (unit < 0) return;
  if (target >= 0 && tb.rank[j] != target) return;
  const int local = unit - tb.unpack_csum[j];
  float *__restrict__ dst = const_cast<float *>(tb.ptrs[j]);
  const B *__restrict__ src = buf + tb.buf_off[j];
  const int d = tb.tri[j];
  if (d == 0) {
    const long long nel = tb.nel[j];
    const long long t0 = (long long)local * kChunk + 4 * threadIdx.x;
    constexpr int kQuads = kChunk / (4 * TH);   // per thread
    float val[kQuads][4];
#pragma unroll
    for (int i = 0; i < kQuads; ++i) {
      const long long t = t0 + (long long)i * (4 * TH);
      if (t + 3 < nel) {
        load_scaled4(src + t, divisor, val[i]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (t + e < nel) val[i][e] = from_buf(src[t + e], divisor);
      }
    }
#pragma unroll
    for (int i = 0; i < kQuads; ++i) {
      const long long t = t0 + (long long)i * (4 * TH);
      if (t + 3 < nel) {
        store_row4(dst + t, val[i]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (t + e < nel) dst[t + e] = val[i][e];
      }
    }
    return;
  }
  // tile (I, J), I >= J, from the unit index in row-major lower order
  const int I = tri_row((unsigned)local);
  const int J = local - I * (I + 1) / 2;
  const int lc = (threadIdx.x % (kTile / 4)) * 4;   // first of the thread's four columns
  const int lr0 = threadIdx.x / (kTile / 4);        // 0..15
  constexpr int kRowsPerPass = TH / (kTile / 4);
  constexpr int kPasses = kTile / kRowsPerPass;
  float val[kPasses][4];
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int lr = lr0 + p * kRowsPerPass;
    const int r = I * kTile + lr;
    const int c = J * kTile + lc;
    const long long row0 = (long long)r * (r + 1) / 2;
    if (r < d && c + 3 <= r) {
      load_scaled4(src + row0 + c, divisor, val[p]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) val[p][e] = (r < d && c + e <= r) ? from_buf(src[row0 + c + e], divisor) : 0.f;
    }
  }
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int lr = lr0 + p * kRowsPerPass;
#pragma unroll
    for (int e = 0; e < 4; ++e) tile[lr][lc + e] = val[p][e];
  }
  __syncthreads();
  if (I == J) {
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int lr = lr0 + p * kRowsPerPass;
      const int r = I * kTile + lr;
      const int c = J * kTile + lc;
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (lc + e <= lr) ? tile[lr][lc + e] : tile[lc + e][lr];
      if (r < d && c + 3 < d) {
        store_row4(dst + (long long)r * d + c, o);
      } else if (r < d) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (c + e < d) dst[(long long)r * d + c + e] = o[e];
      }
    }
  } else {
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int lr = lr0 + p * kRowsPerPass;
      const int r = I * kTile + lr;
      const int c = J * kTile + lc;
      if (r < d) store_row4(dst + (long long)r * d + c, val[p]);   // c + 3 < I * 64 <= r < d
      // mirrored tile (J, I): row J*64 + lr (< I*64 < d), columns I*64 + lc ..
      const int mr = J * kTile + lr;
      const int mc = I * kTile + lc;
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = tile[lc + e][lr];
      if (mc + 3 < d) {
        store_row4(dst + (long long)mr * d + mc, o);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (mc + e < d) dst[(long long)mr * d + mc + e] = o[e];
      }
    }
  }
}

}  // namespace

struct kfac_pack_plan {
  int n = 0;
  long long total_packed = 0;
  int pack_units = 0;
  int unpack_units = 0;
  int unpack_blocks = 0;   // workgroups of an unpack launch (>= unpack_units, see the schedule)
  std::vector<const void *> ptrs;
  kfac::DevTable d_ptrs, d_tri, d_rank, d_nel, d_off, d_pcs, d_ucs, d_pown, d_uown;
  PackTables tables() const {
    PackTables t;
    t.ptrs = d_ptrs.as<const float *const>();
    t.tri = d_tri.as<const int>();
    t.rank = d_rank.as<const int>();
    t.nel = d_nel.as<const long long>();
    t.buf_off = d_off.as<const long long>();
    t.pack_csum = d_pcs.as<const int>();
    t.unpack_csum = d_ucs.as<const int>();
    t.pack_owner = d_pown.as<const int>();
    t.unpack_sched = d_uown.as<const int2>();
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
    KFAC_REQUIRE(t <= 46340, "array %d: triangle side %lld exceeds 46340", i, t);
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
    // pack: units of kPackQuads aligned quads of buffer slots
    if (packed > 0)
      punits += kfac::ceil_div<long long>(kfac::ceil_div<long long>(total + packed, 4) - total / 4, kPackQuads);
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
  auto up = [&](kfac::DevTable &t, const void *h, size_t b) {
    if (rc == KFAC_OK) rc = t.set_sync(h, b);
  };
  up(p->d_ptrs, p->ptrs.data(), sizeof(void *) * n_arrays);
  up(p->d_tri, tri.data(), sizeof(int) * n_arrays);
  up(p->d_rank, rank.data(), sizeof(int) * n_arrays);
  up(p->d_nel, nel.data(), sizeof(long long) * n_arrays);
  up(p->d_off, off.data(), sizeof(long long) * n_arrays);
  up(p->d_pcs, pcs.data(), sizeof(int) * (n_arrays + 1));
  up(p->d_ucs, ucs.data(), sizeof(int) * (n_arrays + 1));
  std::vector<int> pown((size_t)punits + 1, 0);
  for (int i = 0; i < n_arrays; ++i) std::fill(pown.begin() + pcs[i], pown.begin() + pcs[i + 1], i);
  up(p->d_pown, pown.data(), sizeof(int) * pown.size());
  // The unpack schedule: workgroup b (which runs on XCD b % 8, each XCD with an L2
  // of its own) takes entry b / 8 of its XCD's queue.  The tiles of matrices whose rows do not start on cache lines
  // (side not a multiple of 32) go to the queues as eight contiguous runs; all
  // other units are dealt round-robin behind them.
  {
    std::vector<int2> queue[8];
    std::vector<int2> ragged, even;
    for (int i = 0; i < n_arrays; ++i)
      for (int u = ucs[i]; u < ucs[i + 1]; ++u)
        (tri[i] > 0 && tri[i] % 32 != 0 ? ragged : even).push_back(make_int2(u, i));
    const size_t chunk = (ragged.size() + 7) / 8;
    for (size_t k = 0; k < ragged.size(); ++k) queue[k / (chunk ? chunk : 1)].push_back(ragged[k]);
    for (size_t k = 0; k < even.size(); ++k) {
      // to the shortest queue, first the one whose turn it is
      size_t best = k % 8;
      for (size_t x = 0; x < 8; ++x)
        if (queue[x].size() + 1 < queue[best].size()) best = x;
      queue[best].push_back(even[k]);
    }
    size_t longest = 0;
    for (auto &q : queue) longest = std::max(longest, q.size());
    std::vector<int2> sched(std::max<size_t>(longest * 8, 1), make_int2(-1, 0));
    for (size_t x = 0; x < 8; ++x)
      for (size_t k = 0; k < queue[x].size(); ++k) sched[k * 8 + x] = queue[x][k];
    p->unpack_blocks = (int)(longest * 8);
    up(p->d_uown, sched.data(), sizeof(int2) * sched.size());
  }
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
  KFAC_REQUIRE(reinterpret_cast<uintptr_t>(buf) % (4 * sizeof(B)) == 0,
               "the buffer must be aligned to four of its elements (%zu bytes)", 4 * sizeof(B));
  kfac::TimedLaunch timed(KFAC_TIMED_PACK, kfac::as_stream(stream));
  KFAC_LAUNCH((pack_kernel<B, kPackU>), dim3(plan->pack_units), dim3(kThreads), 0,
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
  KFAC_LAUNCH((unpack_kernel<B, kUnpackThreads>), dim3(plan->unpack_blocks), dim3(kUnpackThreads), 0,
                     kfac::as_stream(stream), plan->tables(), buf, target_rank, divisor);
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

}  // namespace

namespace {

// Plain streaming copy, the yardstick for the bandwidth-bound kernels of this
// file: one 16-byte streaming load and store per lane, 4 KB per workgroup (the
// fastest of the structures measured on an MI355X: 6.6 TB/s; two, four or eight
// accesses per lane, grid-stride loops and per-XCD contiguous ranges reach 4.3 -
// 6.3 TB/s, hipMemcpyAsync 5.3 TB/s).
__global__ __launch_bounds__(kThreads) void stream_copy_kernel(const floatx4a *__restrict__ src,
                                                               floatx4a *__restrict__ dst,
                                                               long long n4) {
  const long long t = (long long)blockIdx.x * kThreads + threadIdx.x;
  if (t < n4) __builtin_nontemporal_store(__builtin_nontemporal_load(src + t), dst + t);
}

// The same with unpack's mix of traffic: every element read once and written twice.
__global__ __launch_bounds__(kThreads) void stream_fanout_kernel(const floatx4a *__restrict__ src,
                                                                 floatx4a *__restrict__ dst0,
                                                                 floatx4a *__restrict__ dst1, long long n4) {
  const long long t = (long long)blockIdx.x * kThreads + threadIdx.x;
  if (t < n4) {
    const floatx4a v = __builtin_nontemporal_load(src + t);
    __builtin_nontemporal_store(v, dst0 + t);
    __builtin_nontemporal_store(v, dst1 + t);
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
      KFAC_LAUNCH(stream_copy_kernel, dim3((unsigned)kfac::ceil_div<long long>(n4, kThreads)),
                         dim3(kThreads), 0, s, reinterpret_cast<const floatx4a *>(src),
                         reinterpret_cast<floatx4a *>(dst), n4);
    if (n4 * 4 < nelems)
      KFAC_LAUNCH(stream_copy_tail_kernel, dim3(1), dim3(kThreads), 0, s, src, dst, n4 * 4,
                         (long long)nelems);
  }
  KFAC_HIP_CHECK(hipGetLastError());
  return KFAC_OK;
}

extern "C" int kfac_stream_fanout_f32(float *dst0, float *dst1, const float *src, int64_t nelems, void *stream) {
  KFAC_REQUIRE(nelems >= 0 && nelems % 4 == 0, "nelems must be a non-negative multiple of 4");
  if (nelems == 0) return KFAC_OK;
  KFAC_REQUIRE(dst0 && dst1 && src, "null pointer");
  KFAC_REQUIRE(((reinterpret_cast<uintptr_t>(dst0) | reinterpret_cast<uintptr_t>(dst1) |
                 reinterpret_cast<uintptr_t>(src)) & 15) == 0,
               "pointers must be 16-byte aligned");
  hipStream_t s = kfac::as_stream(stream);
  const long long n4 = nelems / 4;
  {
    kfac::TimedLaunch timed(KFAC_TIMED_COPY, s);
    KFAC_LAUNCH(stream_fanout_kernel, dim3((unsigned)kfac::ceil_div<long long>(n4, kThreads)), dim3(kThreads), 0, s,
                reinterpret_cast<const floatx4a *>(src), reinterpret_cast<floatx4a *>(dst0),
                reinterpret_cast<floatx4a *>(dst1), n4);
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
