// Argument checks and table building of the remaining entry points, in host-only mode:
// batch-norm statistics, damping, batched elementwise launches, low-rank inverse plans.
#include "check.h"
#include "../../include/kfac_hip.h"

int check_elementwise(const std::vector<Workload> &workloads) {
  const int before = g_failures;
  for (const Workload &w : workloads) {
    const char *what = w.name.c_str();
    for (const BnShape &b : w.bns) {
      int rc = kfac_bn_grad_matrix_f32(fake_ptr(1), fake_ptr(2), b.n, b.c, b.h * b.w, 2e-5f, (float)b.n, 1, 1, fake_ptr(3),
                                       fake_ptr(4), kfac_bn_workspace_bytes(b.n, b.c), nullptr);
      EXPECT(rc == KFAC_OK, "%s: batch-norm statistics %d ch @%d: %s", what, b.c, b.h, kfac_last_error_string());
    }
    {
      // the same in two parts: statistics per layer, one finish launch for all layers
      const int nb = (int)w.bns.size();
      std::vector<const float *> stats(nb);
      std::vector<float *> U(nb);
      std::vector<int32_t> bn_n(nb), bn_c(nb), bn_hw(nb), yes(nb, 1), no(nb, 0);
      std::vector<float> eps(nb, 2e-5f), scale(nb);
      for (int i = 0; i < nb; ++i) {
        const BnShape &b = w.bns[i];
        stats[i] = fake_ptr(10 + 2 * i);
        U[i] = fake_ptr(11 + 2 * i);
        bn_n[i] = b.n, bn_c[i] = b.c, bn_hw[i] = b.h * b.w, scale[i] = (float)b.n;
        int rc = kfac_bn_stats_f32(fake_ptr(1), fake_ptr(2), b.n, b.c, b.h * b.w, fake_ptr(10 + 2 * i),
                                   kfac_bn_workspace_bytes(b.n, b.c), nullptr);
        EXPECT(rc == KFAC_OK, "%s: batch-norm statistics alone %d ch @%d: %s", what, b.c, b.h, kfac_last_error_string());
        rc = kfac_bn_stats_f32(fake_ptr(1), fake_ptr(2), b.n, b.c, b.h * b.w, fake_ptr(10 + 2 * i),
                               kfac_bn_workspace_bytes(b.n, b.c) - 1, nullptr);
        EXPECT(rc == KFAC_ENOMEM, "%s: a statistics buffer one byte short was accepted", what);
      }
      kfac_bn_finish_batch_t fb = nullptr;
      EXPECT(kfac_bn_finish_batch_create(&fb) == KFAC_OK && fb, "%s: bn finish batch", what);
      for (int rep = 0; rep < 2; ++rep)
        EXPECT(kfac_bn_finish_batched_f32(fb, nb, stats.data(), U.data(), bn_n.data(), bn_c.data(), bn_hw.data(), eps.data(),
                                          scale.data(), yes.data(), yes.data(), nullptr) == KFAC_OK,
               "%s: batched finish: %s", what, kfac_last_error_string());
      if (nb) {
        EXPECT(kfac_bn_finish_batched_f32(fb, nb, stats.data(), U.data(), bn_n.data(), bn_c.data(), bn_hw.data(), eps.data(),
                                          scale.data(), no.data(), no.data(), nullptr) == KFAC_EINVAL,
               "%s: layers with neither gamma nor beta accepted", what);
        U[nb - 1] = nullptr;
        EXPECT(kfac_bn_finish_batched_f32(fb, nb, stats.data(), U.data(), bn_n.data(), bn_c.data(), bn_hw.data(), eps.data(),
                                          scale.data(), yes.data(), no.data(), nullptr) == KFAC_EINVAL,
               "%s: a null output accepted", what);
      }
      kfac_bn_finish_batch_destroy(fb);
    }
    const int n = (int)w.factor_dims.size();
    std::vector<float *> mats(n);
    std::vector<const float *> xs(n);
    std::vector<int64_t> nel(n);
    std::vector<int32_t> dims(n), splits(n);
    std::vector<double> v0(n, 1e-3), v1(n, 2e-3);
    for (int i = 0; i < n; ++i) {
      mats[i] = fake_ptr(2 * i);
      xs[i] = fake_ptr(2 * i + 1);
      dims[i] = w.factor_dims[i];
      splits[i] = dims[i] / 2;
      nel[i] = (int64_t)dims[i] * dims[i];
    }
    kfac_axpby_batch_t ab = nullptr;
    EXPECT(kfac_axpby_batch_create(&ab) == KFAC_OK, "%s: axpby batch", what);
    EXPECT(kfac_axpby_batched_f32(ab, n, xs.data(), mats.data(), nel.data(), 0.99f, 0.01f, nullptr) == KFAC_OK, "%s: axpby: %s",
           what, kfac_last_error_string());
    EXPECT(kfac_axpby_batched_f32(ab, n, xs.data(), mats.data(), nel.data(), 0.5f, 0.f, nullptr) == KFAC_OK, "%s: axpby b=0", what);
    EXPECT(kfac_div_batched_f32(ab, n, mats.data(), nel.data(), 128.f, nullptr) == KFAC_OK, "%s: div", what);
    EXPECT(kfac_div_batched_f32(ab, n, mats.data(), nel.data(), 0.f, nullptr) == KFAC_EINVAL, "%s: division by zero accepted", what);
    kfac_axpby_batch_destroy(ab);
    kfac_diag_batch_t db = nullptr;
    EXPECT(kfac_diag_batch_create(&db) == KFAC_OK, "%s: diag batch", what);
    EXPECT(kfac_add_diag_batched_f32(db, n, mats.data(), dims.data(), splits.data(), v0.data(), v1.data(), nullptr) == KFAC_OK,
           "%s: add_diag: %s", what, kfac_last_error_string());
    kfac_diag_batch_destroy(db);
    kfac_momentum_batch_t mb = nullptr;
    EXPECT(kfac_momentum_batch_create(&mb) == KFAC_OK, "%s: momentum batch", what);
    std::vector<void *> grads(n);
    std::vector<float *> vs(n);
    for (int i = 0; i < n; ++i) {
      grads[i] = fake_ptr(5000 + i);
      vs[i] = fake_ptr(9000 + i);
    }
    EXPECT(kfac_momentum_update_batched_f32(mb, n, mats.data(), vs.data(), grads.data(), nel.data(), nullptr, nullptr, 1e-3f,
                                            0.9f, 1.f, nullptr) == KFAC_OK,
           "%s: momentum: %s", what, kfac_last_error_string());
    kfac_momentum_batch_destroy(mb);
    // low-rank inverses of the batch-norm blocks
    if (!w.bns.empty()) {
      const int nb = (int)w.bns.size();
      std::vector<int32_t> widths(nb), half(nb);
      std::vector<const float *> U(nb);
      std::vector<float *> out(nb);
      std::vector<double> dg(nb, 4e-3), dbeta(nb, 4e-3);
      for (int i = 0; i < nb; ++i) {
        widths[i] = 2 * w.bns[i].c;
        half[i] = w.bns[i].c;
        U[i] = fake_ptr(2 * i);
        out[i] = fake_ptr(2 * i + 1);
      }
      kfac_bn_lowrank_plan_t lp = nullptr;
      const int batch = w.bns[0].n <= 32 ? w.bns[0].n : 32;
      int rc = kfac_bn_lowrank_plan_create(nb, batch, widths.data(), half.data(), &lp);
      EXPECT(rc == KFAC_OK && lp, "%s: low-rank plan: %s", what, kfac_last_error_string());
      if (lp) {
        rc = kfac_bn_lowrank_inverse_batched_f32(lp, U.data(), out.data(), dg.data(), dbeta.data(),
                                                 reinterpret_cast<int32_t *>(fake_ptr(700000)), fake_ptr(700001),
                                                 kfac_bn_lowrank_workspace_bytes(lp), nullptr);
        EXPECT(rc == KFAC_OK, "%s: low-rank inverse: %s", what, kfac_last_error_string());
        kfac_bn_lowrank_plan_destroy(lp);
      }
    }
    // trace-norm damping of the connection layers
    std::vector<int32_t> dAs, dGs;
    for (const ConvShape &c : w.convs) {
      dAs.push_back(c.c * c.k * c.k + c.bias);
      dGs.push_back(c.c_out);
    }
    for (const LinShape &l : w.linears) {
      dAs.push_back(l.d_in + l.bias);
      dGs.push_back(l.d_out);
    }
    kfac_damp_plan_t dp = nullptr;
    const int nc = (int)dAs.size();
    int rc = kfac_damp_plan_create(nc, dAs.data(), dGs.data(), &dp);
    EXPECT(rc == KFAC_OK, "%s: damp plan: %s", what, kfac_last_error_string());
    if (dp) {
      std::vector<float *> A(nc), G(nc);
      std::vector<double> rW(nc, 0.0158);
      for (int i = 0; i < nc; ++i) {
        A[i] = fake_ptr(2 * i);
        G[i] = fake_ptr(2 * i + 1);
      }
      rc = kfac_pi_damp_batched_f32(dp, A.data(), G.data(), rW.data(), 1, fake_ptr(600000), nullptr);
      EXPECT(rc == KFAC_OK, "%s: pi damping: %s", what, kfac_last_error_string());
      kfac_damp_plan_destroy(dp);
    }
  }
  return g_failures - before;
}
