// The grouped preconditioning plan, and the single-layer and batch-norm entry points.
#include "../../chainerkfac_amd/csrc/precond.hip"

#include <map>

#include "check.h"

namespace {

void check_group(const std::vector<int> &dG, const std::vector<int> &dA, const std::vector<int> &hb, const char *what) {
  const int count = (int)dG.size();
  kfac_precond_group_t g = nullptr;
  int rc = kfac_precond_group_create(count, dG.data(), dA.data(), hb.data(), &g);
  EXPECT(rc == KFAC_OK && g, "%s: group_create failed: %s", what, kfac_last_error_string());
  if (rc != KFAC_OK || !g) return;
  const size_t ws_bytes = kfac_precond_group_workspace_bytes(g);
  const int2 *tasks = reinterpret_cast<const int2 *>(g->d_tasks.shadow().data());
  const int ntasks = (int)(g->d_tasks.shadow().size() / sizeof(int2));
  for (int p = 0; p < 2; ++p) {
    std::vector<std::map<int, int>> seen(count);
    for (int k = 0; k < kPreKinds; ++k) {
      EXPECT(g->task0[p][k] >= 0 && g->task0[p][k] + g->ntask[p][k] <= ntasks, "%s: phase %d launch %d range", what, p, k);
      for (int i = 0; i < g->ntask[p][k]; ++i) {
        const int2 t = tasks[g->task0[p][k] + i];
        EXPECT(t.x >= 0 && t.x < count, "%s: phase %d task item %d", what, p, t.x);
        if (t.x < 0 || t.x >= count) continue;
        const PreStatic &s = g->items[t.x];
        EXPECT(g->kind[p][t.x] == k, "%s: item %d in launch %d, kind %d", what, t.x, k, g->kind[p][t.x]);
        const int ntiles = s.tm * s.tn;
        const int split = t.y / ntiles;
        EXPECT(t.y >= 0 && split < s.nsplit[p], "%s: phase %d item %d slice %d of %d", what, p, t.x, split, s.nsplit[p]);
        const int K = p == 0 ? s.dG : s.dA;
        EXPECT((long long)split * s.klen[p] < K && s.klen[p] % KT == 0, "%s: phase %d item %d slice %d starts past K", what, p, t.x,
               split);
        if (s.nsplit[p] > 1) {
          const int bm = 64 * s.w;
          const long long end = s.part_off + (long long)(split + 1) * ntiles * bm * bm;
          EXPECT((size_t)end <= g->ws_floats, "%s: phase %d item %d partial tiles outside the workspace", what, p, t.x);
        }
        ++seen[t.x][t.y];
      }
    }
    for (int i = 0; i < count; ++i) {
      const PreStatic &s = g->items[i];
      const int K = p == 0 ? s.dG : s.dA;
      EXPECT((long long)s.nsplit[p] * s.klen[p] >= K && (long long)(s.nsplit[p] - 1) * s.klen[p] < K,
             "%s: phase %d item %d: %d slices of %lld for K = %d", what, p, i, s.nsplit[p], s.klen[p], K);
      EXPECT((int)seen[i].size() == s.tm * s.tn * s.nsplit[p], "%s: phase %d item %d has %zu of %d tasks", what, p, i,
             seen[i].size(), s.tm * s.tn * s.nsplit[p]);
      for (const auto &kv : seen[i]) EXPECT(kv.second == 1, "%s: phase %d item %d task %d %d times", what, p, i, kv.first, kv.second);
      EXPECT(s.t_off >= 0 && (size_t)(s.t_off + (long long)s.dG * s.ldT) <= g->ws_floats && s.ldT >= s.dA && s.ldT % 4 == 0,
             "%s: item %d intermediate outside the workspace", what, i);
    }
    // finish: every 256-element block of the outputs of the items with partial tiles
    std::vector<long long> blocks(count, 0);
    EXPECT(g->ftask0[p] >= 0 && g->ftask0[p] + g->nftask[p] <= ntasks, "%s: phase %d finish range", what, p);
    for (int i = 0; i < g->nftask[p]; ++i) {
      const int2 t = tasks[g->ftask0[p] + i];
      EXPECT(t.x >= 0 && t.x < count && g->items[t.x].nsplit[p] > 1, "%s: phase %d finish task %d", what, p, i);
      if (t.x >= 0 && t.x < count) {
        EXPECT(t.y == blocks[t.x], "%s: phase %d finish blocks of item %d out of order", what, p, t.x);
        ++blocks[t.x];
      }
    }
    for (int i = 0; i < count; ++i) {
      const PreStatic &s = g->items[i];
      const long long want = s.nsplit[p] > 1 ? ((long long)s.dG * s.dA + 255) / 256 : 0;
      EXPECT(blocks[i] == want, "%s: phase %d item %d finish blocks %lld of %lld", what, p, i, blocks[i], want);
    }
  }
  if (count) {
    std::vector<const float *> Gi(count), Ai(count), gW(count), gb(count);
    std::vector<float *> kW(count), kb(count);
    for (int i = 0; i < count; ++i) {
      Gi[i] = fake_ptr(6 * i);
      Ai[i] = fake_ptr(6 * i + 1);
      gW[i] = fake_ptr(6 * i + 2);
      gb[i] = hb[i] ? fake_ptr(6 * i + 3) : nullptr;
      kW[i] = fake_ptr(6 * i + 4);
      kb[i] = hb[i] ? fake_ptr(6 * i + 5) : nullptr;
    }
    rc = kfac_precond_group_run_f32(g, Gi.data(), Ai.data(), gW.data(), gb.data(), kW.data(), kb.data(), fake_ptr(800000),
                                    ws_bytes, nullptr);
    EXPECT(rc == KFAC_OK, "%s: run failed: %s", what, kfac_last_error_string());
    rc = kfac_precond_group_run_f32(g, Gi.data(), Ai.data(), gW.data(), gb.data(), kW.data(), kb.data(), fake_ptr(800000),
                                    ws_bytes - 1, nullptr);
    EXPECT(rc == KFAC_ENOMEM, "%s: a workspace one byte short was accepted", what);
    for (int i = 0; i < count; ++i) {
      rc = kfac_precond_conn_f32(Gi[i], dG[i], Ai[i], dA[i], gW[i], gb[i], kW[i], kb[i], fake_ptr(800000),
                                 kfac_precond_conn_workspace_bytes(dG[i], dA[i]), nullptr);
      EXPECT(rc == KFAC_OK, "%s: single layer %d x %d: %s", what, dG[i], dA[i], kfac_last_error_string());
    }
  }
  kfac_precond_group_destroy(g);
}

void check_bn(const std::vector<int> &widths, const char *what) {
  const int count = (int)widths.size();
  kfac_precond_bn_batch_t b = nullptr;
  EXPECT(kfac_precond_bn_batch_create(&b) == KFAC_OK && b, "%s: batch_create", what);
  if (!b) return;
  std::vector<const float *> F(count), gg(count), gb(count);
  std::vector<float *> kg(count), kb(count);
  std::vector<int32_t *> flags(count);
  std::vector<int32_t> n0(count);
  for (int i = 0; i < count; ++i) {
    F[i] = fake_ptr(6 * i);
    n0[i] = widths[i] / 2;
    gg[i] = n0[i] ? fake_ptr(6 * i + 1) : nullptr;
    kg[i] = n0[i] ? fake_ptr(6 * i + 2) : nullptr;
    gb[i] = fake_ptr(6 * i + 3);
    kb[i] = fake_ptr(6 * i + 4);
    flags[i] = reinterpret_cast<int32_t *>(fake_ptr(6 * i + 5));
  }
  const size_t ws = kfac_precond_bn_batched_workspace_bytes(count, widths.data());
  int rc = kfac_precond_bn_batched_f32(b, count, F.data(), widths.data(), gg.data(), n0.data(), gb.data(), kg.data(),
                                       kb.data(), flags.data(), fake_ptr(800000), ws, nullptr);
  EXPECT(rc == KFAC_OK, "%s: batched call: %s", what, kfac_last_error_string());
  if (count) {
    long long off = 0;
    for (int i = 0; i < count; ++i) {
      EXPECT(b->items[i].y_off == off && b->items[i].d == widths[i], "%s: block %d staging offset", what, i);
      off += (widths[i] + 3) / 4 * 4;
    }
    EXPECT((size_t)off * sizeof(float) <= ws, "%s: staging vectors outside the workspace", what);
    size_t units = 0;
    for (int d : widths) units += (d + 3) / 4;
    EXPECT(b->units.size() == units, "%s: units", what);
    for (const int2 &u : b->units) EXPECT(u.x >= 0 && u.x < count && u.y >= 0 && u.y < widths[u.x] && u.y % 4 == 0, "%s: unit", what);
    if (ws > 0) {
      rc = kfac_precond_bn_batched_f32(b, count, F.data(), widths.data(), gg.data(), n0.data(), gb.data(), kg.data(),
                                       kb.data(), flags.data(), fake_ptr(800000), ws - 1, nullptr);
      EXPECT(rc == KFAC_ENOMEM, "%s: a workspace one byte short was accepted", what);
    }
  }
  kfac_precond_bn_batch_destroy(b);
}

}  // namespace

int check_precond(const std::vector<Workload> &workloads) {
  const int before = g_failures;
  for (const Workload &w : workloads) {
    std::vector<int> dG, dA, hb, widths;
    for (const ConvShape &c : w.convs) {
      dG.push_back(c.c_out);
      dA.push_back(c.c * c.k * c.k + c.bias);
      hb.push_back(c.bias);
    }
    for (const LinShape &l : w.linears) {
      dG.push_back(l.d_out);
      dA.push_back(l.d_in + l.bias);
      hb.push_back(l.bias);
    }
    for (const BnShape &b : w.bns) widths.push_back(2 * b.c);
    check_group(dG, dA, hb, w.name.c_str());
    check_bn(widths, w.name.c_str());
  }
  check_group({}, {}, {}, "empty group");
  check_bn({}, "no batch-norm blocks");
  Rng rng(9);
  for (int it = 0; it < 150; ++it) {
    const int n = rng.range(1, 10);
    std::vector<int> dG(n), dA(n), hb(n), widths(n);
    for (int i = 0; i < n; ++i) {
      hb[i] = rng.range(0, 1);
      dG[i] = rng.range(1, rng.range(0, 3) ? 300 : 2100);
      dA[i] = rng.range(1 + hb[i], rng.range(0, 3) ? 700 : 4700);
      widths[i] = rng.range(1, 600);
    }
    char name[64];
    std::snprintf(name, sizeof(name), "random group %d", it);
    check_group(dG, dA, hb, name);
    check_bn(widths, name);
  }
  return g_failures - before;
}
