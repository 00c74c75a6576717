// The covariance planners: grouped launches replayed on the host, and every single-factor
// entry point walked in host-only mode over the configurations' layer shapes.
#include "../../chainerkfac_amd/csrc/cov.hip"

#include <map>

#include "check.h"

namespace {

void check_group(const std::vector<kfac_cov_item> &items, const char *what) {
  const int count = (int)items.size();
  kfac_cov_group_t g = nullptr;
  int rc = kfac_cov_group_create(count, items.data(), &g);
  EXPECT(rc == KFAC_OK && g, "%s: group_create failed: %s", what, kfac_last_error_string());
  if (rc != KFAC_OK || !g) return;
  const size_t ws_bytes = kfac_cov_group_workspace_bytes(g);
  const auto &raw = g->d_tasks.shadow();
  const int2 *tasks = reinterpret_cast<const int2 *>(raw.data());
  const int ntasks = (int)(raw.size() / sizeof(int2));
  // every (item, tile, k-slice) exactly once over the main launches; its k range and partial slot
  std::vector<std::map<int, int>> seen(count);
  for (int k = 0; k < kGroupKinds; ++k) {
    EXPECT(g->task0[k] >= 0 && g->task0[k] + g->ntask[k] <= ntasks, "%s: launch %d range", what, k);
    for (int i = 0; i < g->ntask[k]; ++i) {
      const int2 t = tasks[g->task0[k] + i];
      if (t.x < 0) continue;   // padding of a shorter XCD run
      EXPECT(t.x < count, "%s: launch %d task %d item %d", what, k, i, t.x);
      if (t.x >= count) continue;
      const GroupItemStatic &s = g->items[t.x];
      const bool macro = k >= kMacroKind0;
      const int mt = (s.tiles + 1) / 2;
      const int per_slice = macro ? mt * (mt + 1) / 2 : s.ntile;
      const int split = t.y / per_slice;
      EXPECT(t.y >= 0 && split < s.nsplit, "%s: item %d task %d slice %d of %d", what, t.x, t.y, split, s.nsplit);
      EXPECT((s.bm == 64) == (k < 4) || macro, "%s: item %d with %d-tiles in launch %d", what, t.x, s.bm, k);
      ++seen[t.x][t.y];
      // the slice's part of the reduction, as the kernel computes it
      const long long kbeg = split < s.nfull ? (long long)split * s.klen
                                             : (long long)s.nfull * s.klen + (long long)(split - s.nfull) * s.klen2;
      EXPECT(kbeg < s.K && kbeg % KT == 0, "%s: item %d slice %d starts at %lld of %lld", what, t.x, split, kbeg, s.K);
      if (!s.direct) {
        const long long slot = (long long)s.ntile * s.bm * s.bm + (long long)s.tiles * s.bm;
        const long long end = s.part_off + (long long)(split + 1) * slot;
        EXPECT(s.part_off >= 0 && (size_t)end <= g->ws_floats, "%s: item %d slice %d partial tiles outside the workspace", what,
               t.x, split);
      }
    }
  }
  for (int i = 0; i < count; ++i) {
    const GroupItemStatic &s = g->items[i];
    EXPECT(s.d == items[i].c + (items[i].append_ones ? 1 : 0) && s.tiles == (items[i].c + s.bm - 1) / s.bm &&
               s.ntile == s.tiles * (s.tiles + 1) / 2,
           "%s: item %d geometry", what, i);
    // the slices cover the reduction exactly: full slices, then the half-length ones
    const long long covered = (long long)s.nfull * s.klen + (long long)(s.nsplit - s.nfull) * s.klen2;
    const long long last = covered - (s.nsplit > s.nfull ? s.klen2 : s.klen);
    EXPECT(covered >= s.K && last < s.K && s.nfull >= 0 && s.nfull <= s.nsplit && s.nsplit >= 1,
           "%s: item %d: %d + %d slices of %lld / %lld cover %lld of %lld", what, i, s.nfull, s.nsplit - s.nfull, s.klen,
           s.klen2, covered, s.K);
    const bool macro = seen[i].size() && false;
    (void)macro;
    // which launch kind the item went to decides how many tasks a slice has
    size_t want = 0;
    for (int k = 0; k < kGroupKinds; ++k)
      for (int j = 0; j < g->ntask[k]; ++j)
        if (tasks[g->task0[k] + j].x == i) {
          const int mt = (s.tiles + 1) / 2;
          want = (size_t)(k >= kMacroKind0 ? mt * (mt + 1) / 2 : s.ntile) * s.nsplit;
          k = kGroupKinds;
          break;
        }
    EXPECT(seen[i].size() == want, "%s: item %d has %zu of %zu tasks", what, i, seen[i].size(), want);
    for (const auto &kv : seen[i]) EXPECT(kv.second == 1, "%s: item %d task %d %d times", what, i, kv.first, kv.second);
  }
  // finish launch: every 64 x 64 block of the lower triangle of every item with partial tiles, once
  std::vector<std::map<int, int>> fin(count);
  EXPECT(g->ftask0 >= 0 && g->ftask0 + g->nftask <= ntasks, "%s: finish range", what);
  for (int i = 0; i < g->nftask; ++i) {
    const int2 t = tasks[g->ftask0 + i];
    EXPECT(t.x >= 0 && t.x < count, "%s: finish task %d", what, i);
    if (t.x < 0 || t.x >= count) continue;
    const int sub = (items[t.x].c + 63) / 64;
    EXPECT(!g->items[t.x].direct && t.y >= 0 && t.y < sub * (sub + 1) / 2, "%s: finish task %d of item %d", what, t.y, t.x);
    ++fin[t.x][t.y];
  }
  for (int i = 0; i < count; ++i) {
    const int sub = (items[i].c + 63) / 64;
    EXPECT(fin[i].size() == (g->items[i].direct ? 0u : (size_t)(sub * (sub + 1) / 2)), "%s: item %d finish blocks", what, i);
  }
  // one run through the entry point
  std::vector<const float *> in(count);
  std::vector<float *> out(count);
  std::vector<float> alpha(count, 0.5f), beta(count, 0.f);
  for (int i = 0; i < count; ++i) {
    in[i] = fake_ptr(2 * i);
    out[i] = fake_ptr(2 * i + 1);
  }
  if (count) {
    rc = kfac_cov_group_run_f32(g, in.data(), out.data(), alpha.data(), beta.data(), fake_ptr(800000), ws_bytes, nullptr);
    EXPECT(rc == KFAC_OK, "%s: run failed: %s", what, kfac_last_error_string());
    rc = kfac_cov_group_run_f32(g, in.data(), out.data(), alpha.data(), beta.data(), fake_ptr(800000), ws_bytes - 1, nullptr);
    EXPECT(rc == KFAC_ENOMEM, "%s: a workspace one byte short was accepted", what);
  }
  kfac_cov_group_destroy(g);
}

void check_single(const Workload &w) {
  const char *what = w.name.c_str();
  for (const ConvShape &c : w.convs) {
    const int ho = (c.h + 2 * c.p - c.k) / c.s + 1, wo = (c.w + 2 * c.p - c.k) / c.s + 1;
    const int d = c.c * c.k * c.k + c.bias;
    const long long rows = (long long)c.n * ho * wo;
    const size_t ws = kfac_cov_workspace_bytes(d, rows);
    for (int beta = 0; beta < 2; ++beta) {
      int rc = kfac_cov_conv_a_f32(fake_ptr(1), c.n, c.c, c.h, c.w, c.k, c.k, c.s, c.s, c.p, c.p, c.bias, 1.f / c.n,
                                   (float)beta, fake_ptr(2), fake_ptr(3), ws, nullptr);
      EXPECT(rc == KFAC_OK, "%s: conv A %dx%d/%d %d ch @%d: %s", what, c.k, c.k, c.s, c.c, c.h, kfac_last_error_string());
    }
    const size_t wsg = kfac_cov_workspace_bytes(c.c_out, rows);
    int rc = kfac_cov_conv_g_f32(fake_ptr(1), c.n, c.c_out, ho * wo, 1.f, 0.f, fake_ptr(2), fake_ptr(3), wsg, nullptr);
    EXPECT(rc == KFAC_OK, "%s: conv G %d ch @%d: %s", what, c.c_out, ho, kfac_last_error_string());
  }
  for (const LinShape &l : w.linears) {
    int rc = kfac_cov_linear_f32(fake_ptr(1), l.n, l.d_in, l.bias, 1.f / l.n, 0.f, fake_ptr(2), fake_ptr(3),
                                 kfac_cov_workspace_bytes(l.d_in + l.bias, l.n), nullptr);
    EXPECT(rc == KFAC_OK, "%s: linear A %d: %s", what, l.d_in, kfac_last_error_string());
    rc = kfac_cov_linear_f32(fake_ptr(1), l.n, l.d_out, 0, 1.f, 0.f, fake_ptr(2), fake_ptr(3),
                             kfac_cov_workspace_bytes(l.d_out, l.n), nullptr);
    EXPECT(rc == KFAC_OK, "%s: linear G %d: %s", what, l.d_out, kfac_last_error_string());
  }
}

// the factors a step defers to the grouped launch (at most 8 GFLOP each), as the hooks would list them
std::vector<kfac_cov_item> group_items(const Workload &w) {
  std::vector<kfac_cov_item> items;
  auto small = [](long long rows, int d) { return (double)rows * d * (d + 1) <= 8e9; };
  for (const ConvShape &c : w.convs) {
    const int ho = (c.h + 2 * c.p - c.k) / c.s + 1, wo = (c.w + 2 * c.p - c.k) / c.s + 1;
    const long long rows = (long long)c.n * ho * wo;
    if (c.k == 1 && c.p == 0 && small(rows, c.c + c.bias))
      items.push_back(kfac_cov_item{KFAC_COV_SLAB, c.n, c.c, c.h, c.w, c.s, c.s, c.bias, 1});
    if (small(rows, c.c_out)) items.push_back(kfac_cov_item{KFAC_COV_SLAB, c.n, c.c_out, ho, wo, 1, 1, 0, 1});
  }
  for (const LinShape &l : w.linears) {
    items.push_back(kfac_cov_item{KFAC_COV_LINEAR, l.n, l.d_in, 1, 1, 1, 1, l.bias, 1});
    items.push_back(kfac_cov_item{KFAC_COV_LINEAR, l.n, l.d_out, 1, 1, 1, 1, 0, 1});
  }
  for (const BnShape &b : w.bns) items.push_back(kfac_cov_item{KFAC_COV_LINEAR, b.n, 2 * b.c, 1, 1, 1, 1, 0, 1});
  return items;
}

}  // namespace

int check_cov(const std::vector<Workload> &workloads) {
  const int before = g_failures;
  for (const Workload &w : workloads) {
    check_single(w);
    check_group(group_items(w), w.name.c_str());
    kfac_option_set("group_macro", 1);
    check_group(group_items(w), (w.name + " (macro tiles)").c_str());
    kfac_option_unset("group_macro");
    kfac_option_set("group_graded", 0);
    check_group(group_items(w), (w.name + " (equal slices)").c_str());
    kfac_option_unset("group_graded");
  }
  check_group({}, "empty group");
  Rng rng(5);
  for (int it = 0; it < 150; ++it) {
    std::vector<kfac_cov_item> items(rng.range(1, 12));
    for (kfac_cov_item &x : items) {
      x.kind = rng.range(0, 1);
      x.n = rng.range(1, 40);
      x.c = rng.range(1, rng.range(0, 3) ? 300 : 2100);
      x.h = x.kind == KFAC_COV_SLAB ? rng.range(1, 30) : 1;
      x.w = x.kind == KFAC_COV_SLAB ? rng.range(1, 30) : 1;
      x.sy = x.sx = x.kind == KFAC_COV_SLAB ? rng.range(1, 2) : 1;
      x.append_ones = rng.range(0, 1);
      x.aligned = rng.range(0, 1);
    }
    char name[64];
    std::snprintf(name, sizeof(name), "random group %d", it);
    check_group(items, name);
  }
  // random convolution geometries through the single-factor entry point (all kernel routes)
  Workload r;
  r.name = "random convolutions";
  for (int it = 0; it < 300; ++it) {
    ConvShape c;
    c.k = rng.range(0, 3) ? 3 : (rng.range(0, 1) ? 1 : rng.range(2, 7));
    c.s = rng.range(1, 2);
    c.p = rng.range(0, c.k / 2);
    c.n = rng.range(1, 8) * (rng.range(0, 1) + 1);
    c.c = rng.range(1, rng.range(0, 2) ? 96 : 520);
    c.h = rng.range(c.k, 40);
    c.w = rng.range(c.k, 40);
    c.bias = rng.range(0, 1);
    c.c_out = rng.range(1, 300);
    if ((long long)c.c * c.k * c.k >= 40000) continue;
    r.convs.push_back(c);
  }
  for (int it = 0; it < 100; ++it) r.linears.push_back(LinShape{rng.range(1, 300), rng.range(1, 5000), rng.range(1, 1200), rng.range(0, 1)});
  check_single(r);
  return g_failures - before;
}
