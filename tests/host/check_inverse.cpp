// The batched inverse's plan: every tile product of the sweep, replayed on the host.
#include "../../chainerkfac_amd/csrc/inverse.hip"

#include <map>

#include "check.h"

namespace {

struct Located {
  int s, I, J;
};

// the tile a workspace offset names: which matrix, which tile row and column
bool locate(const std::vector<long long> &off, const std::vector<int> &nt, long long o, Located *out) {
  for (size_t s = 0; s < off.size(); ++s) {
    const long long size = (long long)nt[s] * nt[s] * NB * NB;
    if (o >= off[s] && o < off[s] + size) {
      const long long t = o - off[s];
      if (t % (NB * NB)) return false;
      out->s = (int)s;
      out->I = (int)(t / (NB * NB) / nt[s]);
      out->J = (int)(t / (NB * NB) % nt[s]);
      return true;
    }
  }
  return false;
}

void check_dims(const std::vector<int> &dims, const char *what) {
  const int count = (int)dims.size();
  kfac_inverse_plan_t plan = nullptr;
  int rc = kfac_inverse_plan_create(count, dims.data(), &plan);
  EXPECT(rc == KFAC_OK && plan, "%s: plan_create failed: %s", what, kfac_last_error_string());
  if (rc != KFAC_OK || !plan) return;
  const size_t ws_bytes = kfac_inverse_plan_workspace_bytes(plan);
  // the tables the kernels would read
  const auto &raw = plan->d_tasks.shadow();
  const TileTask *tasks = reinterpret_cast<const TileTask *>(raw.data());
  const int ntasks = (int)(raw.size() / sizeof(TileTask));
  const long long *off = reinterpret_cast<const long long *>(plan->d_off.shadow().data());
  const int *core = reinterpret_cast<const int *>(plan->d_core.shadow().data());
  const int *dim = reinterpret_cast<const int *>(plan->d_dim.shadow().data());
  const long long *vec = reinterpret_cast<const long long *>(plan->d_vec.shadow().data());
  std::vector<long long> offs(off, off + count);
  long long tiles_end = 0;
  for (int s = 0; s < count; ++s) {
    EXPECT(plan->nt[s] == (core[s] + NB - 1) / NB, "%s: slot %d tile count", what, s);
    EXPECT(core[s] == dim[s] || (core[s] == dim[s] - 1 && dim[s] % NB == 1), "%s: slot %d core %d of %d", what, s,
           core[s], dim[s]);
    EXPECT(offs[s] == tiles_end, "%s: slot %d offset", what, s);
    tiles_end += (long long)plan->nt[s] * plan->nt[s] * NB * NB;
    EXPECT((vec[s] >= 0) == (core[s] != dim[s]), "%s: slot %d border vectors", what, s);
    if (vec[s] >= 0)
      EXPECT(vec[s] >= tiles_end - (long long)plan->nt[s] * plan->nt[s] * NB * NB &&
                 (size_t)(vec[s] + 3LL * core[s] + 64) * sizeof(float) <= ws_bytes,
             "%s: slot %d vectors outside the workspace", what, s);
  }
  EXPECT((size_t)tiles_end * sizeof(float) <= ws_bytes, "%s: tiles outside the workspace", what);
  {
    // copy-in: one workgroup per lower tile, told its matrix and tile by the owner table
    const auto &own_raw = plan->d_tile_owner.shadow();
    const int2 *own = reinterpret_cast<const int2 *>(own_raw.data());
    const long long nown = (long long)(own_raw.size() / sizeof(int2));
    EXPECT(nown == plan->total_tiles, "%s: owner table has %lld entries for %d tiles", what, nown, plan->total_tiles);
    long long at = 0;
    for (int s = 0; s < count && at <= nown; ++s)
      for (int I = 0; I < plan->nt[s]; ++I)
        for (int J = 0; J <= I; ++J, ++at)
          if (at < nown)
            EXPECT(own[at].x == s && (own[at].y & 0xffff) == I && (own[at].y >> 16) == J, "%s: owner of tile %lld", what, at);
    EXPECT(at == nown, "%s: owner table does not cover every lower tile once", what);
    EXPECT(plan->first_tiles >= 0 && plan->first_tiles <= plan->total_tiles, "%s: first_tiles", what);
  }

  // applied[s][(a, b)][j] = how often column j's product reached tile (a, b)
  std::vector<std::map<std::pair<int, int>, std::vector<int>>> applied(count);
  std::vector<int> next_col(count, 0);   // columns factored so far
  auto apply = [&](const TileTask &t, const char *launch, int step) {
    if (t.K == 0) return;
    Located c, a, b;
    const bool ok = locate(offs, plan->nt, t.c_off, &c) && locate(offs, plan->nt, t.a_off, &a) &&
                    locate(offs, plan->nt, t.b_off, &b);
    EXPECT(ok, "%s: step %d %s: offset outside the tiles", what, step, launch);
    if (!ok) return;
    EXPECT(t.K > 0 && t.K % (4 * KT) == 0, "%s: step %d %s: K = %d", what, step, launch, t.K);
    const int nj = t.K / NB;
    EXPECT(a.s == c.s && b.s == c.s && a.I == c.I && b.I == c.J && a.J == b.J, "%s: step %d %s: operands (%d,%d) (%d,%d) of tile (%d,%d)",
           what, step, launch, a.I, a.J, b.I, b.J, c.I, c.J);
    EXPECT(a.J + nj <= plan->nt[c.s], "%s: step %d %s: operand run leaves its tile row", what, step, launch);
    EXPECT(((t.flags & kSame) != 0) == (c.I == c.J), "%s: step %d %s: kSame on tile (%d,%d)", what, step, launch, c.I, c.J);
    auto &cnt = applied[c.s][{c.I, c.J}];
    if (cnt.empty()) cnt.assign(plan->nt[c.s], 0);
    bool first = true;
    for (int v : cnt) first = first && v == 0;
    if (c.I < c.J)
      EXPECT(((t.flags & kFirst) != 0) == first, "%s: step %d %s: kFirst on upper tile (%d,%d)", what, step, launch, c.I, c.J);
    else
      EXPECT((t.flags & kFirst) == 0, "%s: step %d %s: kFirst on a lower tile", what, step, launch);
    for (int j = a.J; j < a.J + nj && j < plan->nt[c.s]; ++j) {
      // the operand tiles (., j) must be final: column j's panel step has run
      EXPECT(j < next_col[c.s], "%s: step %d %s: reads column %d of slot %d before its panel step", what, step, launch, j, c.s);
      ++cnt[j];
    }
  };
  const int max_t = plan->max_t;
  EXPECT((int)plan->nactive.size() == max_t && (int)plan->with_diag.size() == max_t, "%s: per-step tables", what);
  for (int k = 0; k < max_t; ++k) {
    const UpdateLaunch &w = plan->with_diag[k];
    EXPECT(w.task0 >= 0 && w.task0 + w.count <= ntasks, "%s: step %d column launch range", what, k);
    for (int i = 0; i < w.count; ++i) apply(tasks[w.task0 + i], "column", k);
    const int na = plan->nactive[k];
    EXPECT(plan->diag_task0[k] + na <= ntasks, "%s: step %d diagonal range", what, k);
    for (int i = 0; i < na; ++i) {
      const TileTask &t = tasks[plan->diag_task0[k] + i];
      Located c;
      const bool ok = locate(offs, plan->nt, t.c_off, &c);
      EXPECT(ok && c.I == c.J && c.I == t.flags, "%s: step %d diagonal task %d", what, k, i);
      if (!ok) continue;
      EXPECT((int)(t.b_off & 0xffffffffLL) == plan->order[c.s] && (int)(t.b_off >> 32) == core[c.s],
             "%s: step %d diagonal task %d: caller index / size", what, k, i);
      EXPECT(c.I == next_col[c.s], "%s: step %d: slot %d factors column %d, expected %d", what, k, c.s, c.I, next_col[c.s]);
      if (t.K > 0) {
        TileTask u = t;
        u.b_off = t.a_off;
        u.flags = kSame;
        apply(u, "diagonal", k);
      }
      // every product of the earlier columns must have reached the diagonal tile by now
      auto &cnt = applied[c.s][{c.I, c.I}];
      for (int j = 0; j < c.I; ++j)
        EXPECT(!cnt.empty() && cnt[j] == 1, "%s: step %d: slot %d diagonal tile %d has column %d %d times", what, k, c.s, c.I,
               j, cnt.empty() ? 0 : cnt[j]);
    }
    // panel step: every other tile of the column must be complete, then the column is final
    const int np = plan->panel_total[k];
    EXPECT(plan->panel_task0[k] + np <= ntasks, "%s: step %d panel range", what, k);
    std::vector<int> rows_seen(count, 0);
    for (int i = 0; i < np; ++i) {
      const TileTask &t = tasks[plan->panel_task0[k] + i];
      Located c, b;
      const bool ok = locate(offs, plan->nt, t.c_off, &c) && locate(offs, plan->nt, t.b_off, &b);
      EXPECT(ok && t.a_off == t.c_off && t.K == NB && b.s == c.s && b.I == b.J && b.I == c.J && c.I != c.J &&
                 c.J == next_col[c.s],
             "%s: step %d panel task %d", what, k, i);
      if (!ok) continue;
      ++rows_seen[c.s];
      auto &cnt = applied[c.s][{c.I, c.J}];
      const int lo = c.I < c.J ? c.I : 0;   // upper tile (a, b): columns a .. b - 1; lower: 0 .. b - 1
      for (int j = 0; j < plan->nt[c.s]; ++j) {
        const int want = (j >= lo && j < c.J) ? 1 : 0;
        const int got = cnt.empty() ? 0 : cnt[j];
        EXPECT(got == want, "%s: step %d: slot %d tile (%d,%d) has column %d %d times, expected %d", what, k, c.s, c.I, c.J, j,
               got, want);
      }
    }
    for (int s = 0; s < na; ++s) {
      EXPECT(rows_seen[s] == plan->nt[s] - 1, "%s: step %d: slot %d panel tiles %d of %d", what, k, s, rows_seen[s],
             plan->nt[s] - 1);
      ++next_col[s];
    }
    const UpdateLaunch &r = plan->rest[k];
    EXPECT(r.task0 >= 0 && r.task0 + r.count <= ntasks, "%s: step %d trailing launch range", what, k);
    for (int i = 0; i < r.count; ++i) apply(tasks[r.task0 + i], "trailing", k);
    // border tasks of the step
    const BorderTask *bt = reinterpret_cast<const BorderTask *>(plan->d_btasks.shadow().data());
    const int nbt = (int)(plan->d_btasks.shadow().size() / sizeof(BorderTask));
    for (int pass = 0; pass < 2; ++pass) {
      const int t0 = pass ? plan->bpanel_task0[k] : plan->bdiag_task0[k];
      const int n = pass ? plan->bpanel_count[k] : plan->bdiag_count[k];
      EXPECT(t0 >= 0 && t0 + n <= nbt, "%s: step %d border range", what, k);
      for (int i = 0; i < n && t0 + i < nbt; ++i) {
        const BorderTask &b = bt[t0 + i];
        EXPECT(b.s >= 0 && b.s < count && vec[b.s] >= 0 && b.i >= 0 && b.i < plan->nt[b.s] &&
                   b.j >= 0 && b.j < plan->nt[b.s],
               "%s: step %d border task (%d,%d,%d,%d)", what, k, b.s, b.kind, b.i, b.j);
      }
    }
  }
  for (int s = 0; s < count; ++s) EXPECT(next_col[s] == plan->nt[s], "%s: slot %d factored %d of %d columns", what, s, next_col[s], plan->nt[s]);
  // the final products: every lower tile of every matrix once, K = the rest of its tile row
  std::vector<std::map<std::pair<int, int>, int>> final_seen(count);
  EXPECT(plan->lauum_task0 + plan->lauum_count <= ntasks, "%s: final launch range", what);
  for (int i = 0; i < plan->lauum_count; ++i) {
    const TileTask &t = tasks[plan->lauum_task0 + i];
    if (t.K == 0) continue;
    const int s = (int)t.c_off, I = t.flags & 0xffff, J = t.flags >> 16;
    EXPECT(s >= 0 && s < count && J <= I && I < plan->nt[s], "%s: final task %d", what, i);
    if (!(s >= 0 && s < count)) continue;
    Located a, b;
    const bool ok = locate(offs, plan->nt, t.a_off, &a) && locate(offs, plan->nt, t.b_off, &b);
    EXPECT(ok && a.s == s && b.s == s && a.I == I && a.J == I && b.I == J && b.J == I && t.K == (plan->nt[s] - I) * NB,
           "%s: final task %d operands", what, i);
    ++final_seen[s][{I, J}];
  }
  for (int s = 0; s < count; ++s)
    for (int I = 0; I < plan->nt[s]; ++I)
      for (int J = 0; J <= I; ++J) EXPECT(final_seen[s][std::make_pair(I, J)] == 1, "%s: slot %d final tile (%d,%d)", what, s, I, J);

  // and one run through the entry point: argument checks, launch grids, event bookkeeping
  std::vector<const float *> in(count);
  std::vector<float *> out(count);
  for (int i = 0; i < count; ++i) {
    in[i] = fake_ptr(2 * i);
    out[i] = fake_ptr(2 * i + 1);
  }
  rc = kfac_spd_inverse_batched_f32(plan, in.data(), out.data(), reinterpret_cast<int32_t *>(fake_ptr(900000)),
                                    fake_ptr(900001), ws_bytes, nullptr);
  EXPECT(rc == KFAC_OK, "%s: run failed: %s", what, kfac_last_error_string());
  if (count > 0) {
    rc = kfac_spd_inverse_batched_f32(plan, in.data(), out.data(), reinterpret_cast<int32_t *>(fake_ptr(900000)),
                                      fake_ptr(900001), ws_bytes - 1, nullptr);
    EXPECT(rc == KFAC_ENOMEM, "%s: a workspace one byte short was accepted", what);
  }
  kfac_inverse_plan_destroy(plan);
}

}  // namespace

int check_inverse(const std::vector<Workload> &workloads) {
  const int before = g_failures;
  for (const Workload &w : workloads) check_dims(w.factor_dims, w.name.c_str());
  check_dims({}, "empty");
  check_dims({1}, "one");
  // random size lists, with the sizes around the tile size and the bordered form over-represented
  Rng rng(11);
  for (int it = 0; it < 120; ++it) {
    std::vector<int> dims(rng.range(1, 9));
    for (int &d : dims) {
      const int kind = rng.range(0, 5);
      const int m = rng.range(1, kind == 0 ? 12 : 5);
      d = kind <= 1 ? 128 * m + 1 : kind == 2 ? 128 * m : kind == 3 ? 128 * m + rng.range(-2, 2) : rng.range(1, 700);
      if (d < 1) d = 1;
    }
    char name[64];
    std::snprintf(name, sizeof(name), "random list %d", it);
    check_dims(dims, name);
  }
  // the schedule options
  const struct { const char *name; double v; } opts[] = {{"inverse_group", 1}, {"inverse_group", 3}, {"inverse_group", 4},
                                                         {"inverse_align", 0},  {"inverse_align", 50}, {"inverse_border", 0},
                                                         {"inverse_lookahead", 0}};
  for (const auto &o : opts) {
    kfac_option_set(o.name, o.v);
    char name[64];
    std::snprintf(name, sizeof(name), "%s=%g", o.name, o.v);
    check_dims({900, 641, 640, 385, 300, 129, 128, 40, 3}, name);
    check_dims({2305, 1153, 1025, 577, 513, 257}, name);
    kfac_option_unset(o.name);
  }
  return g_failures - before;
}
