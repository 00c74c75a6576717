// The pack / unpack descriptor: unit tables and the unpack schedule.
#include "../../chainerkfac_amd/csrc/pack.hip"

#include <map>

#include "check.h"

namespace {

void check_list(const std::vector<long long> &sizes, const std::vector<int> &tri, const char *what) {
  const int n = (int)sizes.size();
  std::vector<const void *> ptrs(n);
  std::vector<int64_t> sz(sizes.begin(), sizes.end());
  std::vector<int32_t> rank(n);
  for (int i = 0; i < n; ++i) {
    ptrs[i] = fake_ptr(i);
    rank[i] = i % 3;
  }
  kfac_pack_plan_t plan = nullptr;
  int rc = kfac_pack_plan_create(n, ptrs.data(), sz.data(), tri.data(), rank.data(), &plan);
  EXPECT(rc == KFAC_OK && plan, "%s: plan_create failed: %s", what, kfac_last_error_string());
  if (rc != KFAC_OK || !plan) return;
  const long long total = kfac_packed_nelems(n, sz.data(), tri.data());
  EXPECT(total == kfac_pack_plan_nelems(plan), "%s: packed length", what);
  const int *pcs = reinterpret_cast<const int *>(plan->d_pcs.shadow().data());
  const int *ucs = reinterpret_cast<const int *>(plan->d_ucs.shadow().data());
  const int *pown = reinterpret_cast<const int *>(plan->d_pown.shadow().data());
  const long long *off = reinterpret_cast<const long long *>(plan->d_off.shadow().data());
  const long long *nel = reinterpret_cast<const long long *>(plan->d_nel.shadow().data());
  const int2 *sched = reinterpret_cast<const int2 *>(plan->d_uown.shadow().data());
  const size_t nsched = plan->d_uown.shadow().size() / sizeof(int2);
  EXPECT(plan->d_pown.shadow().size() >= sizeof(int) * (size_t)plan->pack_units, "%s: pack owner table", what);
  long long slot = 0;
  for (int i = 0; i < n; ++i) {
    EXPECT(off[i] == slot, "%s: array %d offset", what, i);
    const long long packed = tri[i] > 0 ? (long long)tri[i] * (tri[i] + 1) / 2 : sizes[i];
    EXPECT(nel[i] == packed, "%s: array %d packed size", what, i);
    // pack units: aligned quads of buffer slots that overlap the array, kPackQuads per unit
    const long long q0 = slot / 4, q1 = (slot + packed + 3) / 4;
    const long long units = packed > 0 ? (q1 - q0 + kPackQuads - 1) / kPackQuads : 0;
    EXPECT(pcs[i + 1] - pcs[i] == units, "%s: array %d pack units %d, expected %lld", what, i, pcs[i + 1] - pcs[i], units);
    for (int u = pcs[i]; u < pcs[i + 1]; ++u) EXPECT(pown[u] == i, "%s: pack unit %d owner", what, u);
    const long long tt = (tri[i] + kTile - 1) / kTile;
    const long long uu = tri[i] > 0 ? tt * (tt + 1) / 2 : (packed + kChunk - 1) / kChunk;
    EXPECT(ucs[i + 1] - ucs[i] == uu, "%s: array %d unpack units", what, i);
    slot += packed;
  }
  EXPECT(pcs[n] == plan->pack_units && ucs[n] == plan->unpack_units, "%s: unit totals", what);
  // the unpack schedule holds every unit once, with its array
  EXPECT(nsched >= (size_t)plan->unpack_blocks && plan->unpack_blocks >= plan->unpack_units, "%s: schedule size", what);
  std::map<int, int> seen;
  for (int b = 0; b < plan->unpack_blocks; ++b) {
    if (sched[b].x < 0) continue;
    const int u = sched[b].x, j = sched[b].y;
    EXPECT(u < plan->unpack_units && j >= 0 && j < n && u >= ucs[j] && u < ucs[j + 1], "%s: schedule entry %d = (%d, %d)", what, b,
           u, j);
    ++seen[u];
  }
  EXPECT((int)seen.size() == plan->unpack_units, "%s: schedule holds %zu of %d units", what, seen.size(), plan->unpack_units);
  for (const auto &kv : seen) EXPECT(kv.second == 1, "%s: unpack unit %d scheduled %d times", what, kv.first, kv.second);
  // the entry points
  const long long buf_n = total + 8;
  for (int target : {-1, 1}) {
    rc = kfac_pack_f32(plan, fake_ptr(700000), buf_n, target, nullptr);
    EXPECT(rc == KFAC_OK, "%s: pack: %s", what, kfac_last_error_string());
    rc = kfac_unpack_f32(plan, fake_ptr(700000), buf_n, target, 2, nullptr);
    EXPECT(rc == KFAC_OK, "%s: unpack: %s", what, kfac_last_error_string());
    rc = kfac_pack_f16(plan, fake_ptr(700000), buf_n, target, nullptr);
    EXPECT(rc == KFAC_OK, "%s: pack f16: %s", what, kfac_last_error_string());
    rc = kfac_unpack_f16(plan, fake_ptr(700000), buf_n, target, 1, nullptr);
    EXPECT(rc == KFAC_OK, "%s: unpack f16: %s", what, kfac_last_error_string());
  }
  if (total > 0) {
    rc = kfac_pack_f32(plan, fake_ptr(700000), total - 1, -1, nullptr);
    EXPECT(rc != KFAC_OK, "%s: a buffer one slot short was accepted", what);
  }
  std::vector<const void *> other(n);
  for (int i = 0; i < n; ++i) other[i] = fake_ptr(1000 + i);
  rc = kfac_pack_plan_set_ptrs(plan, other.data(), nullptr);
  EXPECT(rc == KFAC_OK, "%s: set_ptrs: %s", what, kfac_last_error_string());
  kfac_pack_plan_destroy(plan);
}

}  // namespace

int check_pack(const std::vector<Workload> &workloads) {
  const int before = g_failures;
  for (const Workload &w : workloads) {
    // the communicator's list: per layer the gradients (flat) then the factors (triangular)
    std::vector<long long> sizes;
    std::vector<int> tri;
    for (const ConvShape &c : w.convs) {
      sizes.push_back((long long)c.c_out * c.c * c.k * c.k);
      tri.push_back(0);
      if (c.bias) {
        sizes.push_back(c.c_out);
        tri.push_back(0);
      }
    }
    for (int d : w.factor_dims) {
      sizes.push_back((long long)d * d);
      tri.push_back(d);
    }
    check_list(sizes, tri, w.name.c_str());
  }
  check_list({}, {}, "empty list");
  Rng rng(3);
  for (int it = 0; it < 200; ++it) {
    const int n = rng.range(1, 14);
    std::vector<long long> sizes(n);
    std::vector<int> tri(n);
    for (int i = 0; i < n; ++i) {
      if (rng.range(0, 1)) {
        tri[i] = rng.range(1, rng.range(0, 4) ? 200 : 1500);
        sizes[i] = (long long)tri[i] * tri[i];
      } else {
        tri[i] = 0;
        sizes[i] = rng.range(0, rng.range(0, 3) ? 5000 : 300000);
      }
    }
    char name[64];
    std::snprintf(name, sizeof(name), "random list %d", it);
    check_list(sizes, tri, name);
  }
  return g_failures - before;
}
