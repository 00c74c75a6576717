"""Parity of the HIP damped inverse with the oracle (rel 1e-3, needs the GPU)."""
import numpy as np
import pytest
import torch

from oracle import kfac_oracle as O

pytestmark = pytest.mark.gpu

RTOL = 1e-3   # inverse tolerance of the north-star spec


def spd(d, seed):
    r = np.random.default_rng(seed)
    X = r.standard_normal((2 * d, d)).astype(np.float32)
    return (X.T @ X / np.float32(2 * d) + np.float32(1e-3) * np.eye(d, dtype=np.float32)).astype(np.float32)


def check_inverse(M, inv):
    d = M.shape[0]
    ref = O.inverse(M.copy())
    ref64 = np.linalg.inv(M.astype(np.float64))
    nrm = np.linalg.norm(ref64)
    assert np.linalg.norm(inv - ref) / nrm < RTOL
    # no worse than a small multiple of the reference formula's own float32 error
    err_ref = np.linalg.norm(ref - ref64) / nrm
    err_hip = np.linalg.norm(inv - ref64) / nrm
    assert err_hip < max(4 * err_ref, 1e-5)
    resid = np.linalg.norm(M.astype(np.float64) @ inv - np.eye(d)) / np.sqrt(d)
    assert resid < RTOL
    assert np.array_equal(inv, inv.T), 'inverse must be exactly symmetric'


DIMS = [1, 2, 7, 31, 32, 33, 64, 65, 127, 128, 129, 200, 257, 384, 577, 1000, 1025]


def test_batched_inverse_mixed_sizes():
    from chainerkfac_amd import ops
    mats = [spd(d, 100 + d) for d in DIMS]
    dev = [torch.from_numpy(m).cuda() for m in mats]
    outs, info = ops.spd_inverse_batched(dev)
    torch.cuda.synchronize()
    assert info.cpu().tolist() == [0] * len(DIMS)
    for m, m_dev, o in zip(mats, dev, outs):
        assert np.array_equal(m_dev.cpu().numpy(), m), 'input must not be modified'
        check_inverse(m, o.cpu().numpy())


@pytest.mark.parametrize('opts,extra', [({'inverse_align': 0}, 3), ({'inverse_align': 50}, 4),
                                        ({'inverse_group': 3}, 5), ({'inverse_group': 1}, 6),
                                        ({'inverse_lookahead': 0}, 8),
                                        ({'inverse_group': 4, 'inverse_align': 30}, 9)])
def test_schedule_overrides_do_not_change_results(opts, extra):
    """The tuning options (where a matrix joins the sweep, block columns per
    group, second stream) only reorder launches.  A plan reads them when it is
    created; `extra` makes the size list, and with it the plan, unique to the case."""
    from chainerkfac_amd import _lib, ops
    with _lib.options(**opts):
        _run_schedule_case(ops, extra)


def _run_schedule_case(ops, extra):
    dims = [900, 641, 640, 385, 300, 129, 128, 40, extra]
    mats = [spd(d, 200 + d) for d in dims]
    outs, info = ops.spd_inverse_batched([torch.from_numpy(m).cuda() for m in mats])
    torch.cuda.synchronize()
    assert info.cpu().tolist() == [0] * len(dims)
    for m, o in zip(mats, outs):
        check_inverse(m, o.cpu().numpy())


@pytest.mark.parametrize('d', [10, 148, 2305])
def test_single_inverse_free_function(d):
    from chainerkfac_amd.optimizers.cholesky_inverse import inverse
    M = spd(d, d)
    inv = inverse(torch.from_numpy(M).cuda())
    check_inverse(M, inv.cpu().numpy())


def test_special_cases():
    from chainerkfac_amd import ops
    diag = np.diag(np.array([1.0, 4.0, 0.5, 2.0, 8.0], dtype=np.float32))
    one = np.array([[4.0]], dtype=np.float32)
    ident = np.eye(130, dtype=np.float32)
    outs, info = ops.spd_inverse_batched([torch.from_numpy(a).cuda() for a in (diag, one, ident)])
    np.testing.assert_allclose(outs[0].cpu().numpy(), np.diag([1.0, 0.25, 2.0, 0.5, 0.125]), rtol=1e-6)
    np.testing.assert_allclose(outs[1].cpu().numpy(), [[0.25]], rtol=1e-6)
    assert np.array_equal(outs[2].cpu().numpy(), ident)
    assert info.cpu().tolist() == [0, 0, 0]
    outs, info = ops.spd_inverse_batched([])
    assert outs == []


def test_non_spd_and_nan_are_flagged_per_matrix():
    """The reference GPU path never reads cuSOLVER's dev_info; here every matrix
    gets its own code: 1 + index of the first non-positive pivot."""
    from chainerkfac_amd import ops
    good = spd(40, 1)
    bad = np.array([[1.0, 2.0], [2.0, 1.0]], dtype=np.float32)          # pivot 1 is -3
    late = spd(200, 2); late[150, 150] = -5.0                             # fails at column 150
    nan = spd(33, 3); nan[0, 0] = np.nan
    outs, info = ops.spd_inverse_batched([torch.from_numpy(a).cuda() for a in (good, bad, late, nan)])
    info = info.cpu().tolist()
    assert info[0] == 0 and info[1] == 2 and info[2] == 151 and info[3] == 1
    check_inverse(good, outs[0].cpu().numpy())
    with pytest.raises(np.linalg.LinAlgError):
        O.inverse(bad)


def test_bordered_matrices():
    """Matrices of 128 m + 1 rows (a layer with a bias) are inverted from their leading
    block plus a border; the result equals the whole-matrix path (option inverse_border = 0) to
    rounding, a non-positive last pivot is reported as info = d, and sizes around the rule
    (128 m, 128 m + 2, 129) take their own paths."""
    from chainerkfac_amd import ops
    dims = [129, 257, 513, 641, 130, 256, 258, 1153]
    mats = [spd(d, 300 + d) for d in dims]
    dev = [torch.from_numpy(m).cuda() for m in mats]
    outs, info = ops.spd_inverse_batched(dev)
    torch.cuda.synchronize()
    assert info.cpu().tolist() == [0] * len(dims)
    for m, o in zip(mats, outs):
        check_inverse(m, o.cpu().numpy())
    # the same through the whole-matrix path (a plan reads the switch when it is created)
    from chainerkfac_amd import _lib
    with _lib.options(inverse_border=0):
        whole, info = ops.spd_inverse_batched(dev + [torch.from_numpy(spd(3, 1)).cuda()])
    for m, o, w in zip(mats, outs, whole):
        ref64 = np.linalg.inv(m.astype(np.float64))
        assert np.linalg.norm(o.cpu().numpy() - w.cpu().numpy()) <= 2e-4 * np.linalg.norm(ref64)
    # last pivot not positive: SPD leading block, corner too small
    bad = spd(257, 9).astype(np.float64)
    a = bad[:256, 256]
    bad[256, 256] = a @ np.linalg.solve(bad[:256, :256], a) * 0.5
    early = spd(385, 10)
    early[100, 100] = -1.0
    outs, info = ops.spd_inverse_batched([torch.from_numpy(bad.astype(np.float32)).cuda(),
                                          torch.from_numpy(early).cuda(),
                                          torch.from_numpy(spd(257, 11)).cuda()])
    assert info.cpu().tolist() == [257, 101, 0]
    check_inverse(spd(257, 11), outs[2].cpu().numpy())


def test_repeated_calls_reuse_plan_and_workspace():
    from chainerkfac_amd import ops
    mats = [torch.from_numpy(spd(d, d)).cuda() for d in (300, 50)]
    outs = [torch.empty_like(m) for m in mats]
    for _ in range(3):
        ops.spd_inverse_batched(mats, outs=outs)
    for m, o in zip(mats, outs):
        check_inverse(m.cpu().numpy(), o.cpu().numpy())


def test_pi_damp_matches_oracle():
    from chainerkfac_amd import ops
    layers = [(6, 4), (785, 1000), (1001, 10), (28, 64)]
    As = [spd(a, a) for a, _ in layers]
    Gs = [(spd(g, 7 * g) * np.float32(0.01)) for _, g in layers]
    dampings = [1e-3, 1e-3, 2.5e-4, 0.03]
    refA = [a.copy() for a in As]; refG = [g.copy() for g in Gs]
    pis = []
    for a, g, dmp in zip(refA, refG, dampings):
        (dA, dG), pi = O.connection_diagvals(a, g, dmp)
        O.damp_inplace(a, dA); O.damp_inplace(g, dG)
        pis.append(float(pi))
    dA = [torch.from_numpy(a).cuda() for a in As]; dG = [torch.from_numpy(g).cuda() for g in Gs]
    pi = ops.pi_damp_batched(dA, dG, [d ** 0.5 for d in dampings])
    np.testing.assert_allclose(pi.cpu().numpy(), pis, rtol=1e-5)
    for got, ref in zip(dA + dG, refA + refG):
        got = got.cpu().numpy()
        off = ~np.eye(ref.shape[0], dtype=bool)
        assert np.array_equal(got[off], ref[off])
        np.testing.assert_allclose(np.diagonal(got), np.diagonal(ref), rtol=2e-6)
    # pi_type other than tracenorm: pi = 1
    a = torch.from_numpy(As[0]).cuda(); g = torch.from_numpy(Gs[0]).cuda()
    pi = ops.pi_damp_batched([a], [g], [0.1], use_pi=False)
    assert pi.cpu().tolist() == [1.0]
    np.testing.assert_allclose(np.diagonal(a.cpu().numpy()), np.diagonal(As[0]) + 0.1, rtol=1e-6)


def test_add_diag_batch_norm_halves():
    from chainerkfac_amd import ops
    F = spd(10, 4)
    ref = F.copy()
    (dv,) = O.bn_diagvals(6, 4, damping=2.5e-4, stab_coeff=16.0, l2_beta=0.5)
    O.damp_inplace(ref, dv)
    got = ops.add_diag(torch.from_numpy(F).cuda(), dv[0], dv[-1], split=6).cpu().numpy()
    assert np.array_equal(got, ref)


@pytest.mark.gpu
def test_add_diag_batched_matches_the_single_calls():
    """One launch for the damping of many blocks (ragged sizes, gamma+beta, one half only):
    bit-identical to the oracle's in-place damping and to a second call with other values."""
    from chainerkfac_amd import ops
    sizes = [(10, 6), (1, 1), (300, 150), (64, 64), (513, 0)]
    mats, refs, v0s, v1s, splits = [], [], [], [], []
    for i, (d, split) in enumerate(sizes):
        F = spd(d, 20 + i)
        (dv,) = O.bn_diagvals(max(split, 1), max(d - split, 1), damping=2.5e-4 * (i + 1), stab_coeff=16.0, l2_beta=0.5)
        v0, v1 = float(dv[0]), float(dv[-1])
        ref = F.copy()
        diag = np.where(np.arange(d) < split, v0, v1)
        O.damp_inplace(ref, diag)
        mats.append(torch.from_numpy(F).cuda())
        refs.append(ref)
        v0s.append(v0)
        v1s.append(v1)
        splits.append(split)
    ops.add_diag_batched(mats, v0s, v1s, splits)
    for M, ref in zip(mats, refs):
        assert np.array_equal(M.cpu().numpy(), ref)
    # the same matrices again with other values: the argument table is replaced
    ops.add_diag_batched(mats, [1.0] * len(mats))
    for M, ref in zip(mats, refs):
        want = ref.copy()
        O.damp_inplace(want, np.ones(ref.shape[0]))
        assert np.array_equal(M.cpu().numpy(), want)
    assert ops.add_diag_batched([], []) == []


@pytest.mark.gpu
@pytest.mark.parametrize('n', [32, 7, 1])
def test_bn_lowrank_inverse_matches_dense_oracle(n):
    """(U^T U / n + D)^-1 by the Woodbury identity against the dense float64 inverse and the
    float32 oracle formula, for gamma+beta, gamma-only and beta-only blocks of ragged widths."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(40 + n)
    widths = [128, 600, 2, 257, 64]
    splits = [64, 300, 1, 257, 0]          # 257: gamma only, 0: beta only
    d_gamma = [4e-3, 1e-2, 0.5, 2e-3, None]
    d_beta = [4e-3, 3e-3, 0.25, None, 1e-3]
    Us = [(r.standard_normal((n, w)) * r.uniform(0.1, 3.0, size=w)).astype(np.float32) for w in widths]
    outs, info = ops.bn_lowrank_inverse_batched([torch.from_numpy(U).cuda() for U in Us], splits, d_gamma, d_beta)
    assert int((info != 0).sum()) == 0
    for U, w, sp, dg, db, out in zip(Us, widths, splits, d_gamma, d_beta, outs):
        diag = np.concatenate([np.full(sp, dg if dg is not None else 0.0), np.full(w - sp, db if db is not None else 0.0)])
        F = U.astype(np.float64).T @ U.astype(np.float64) / n + np.diag(diag)
        ref64 = np.linalg.inv(F)
        got = out.cpu().numpy()
        assert np.array_equal(got, got.T)
        err = np.linalg.norm(got - ref64) / np.linalg.norm(ref64)
        ref32 = O.inverse(F.astype(np.float32)).astype(np.float64)
        err_ref = np.linalg.norm(ref32 - ref64) / np.linalg.norm(ref64)
        assert err < 1e-3 and err <= 4 * err_ref + 1e-6, (w, err, err_ref)
        # residual no worse than a small multiple of the reference formula's own (both grow with
        # the condition number lambda_max / damping of these rank-deficient factors)
        resid = np.linalg.norm(F @ got - np.eye(w)) / np.sqrt(w)
        resid_ref = np.linalg.norm(F @ ref32 - np.eye(w)) / np.sqrt(w)
        assert resid < max(4 * resid_ref, 1e-4), (w, resid, resid_ref)


@pytest.mark.gpu
def test_bn_lowrank_rejects_bad_arguments():
    from chainerkfac_amd import ops, _lib
    U = torch.zeros(40, 8, device='cuda')
    with pytest.raises(_lib.KfacHipError):
        ops.bn_lowrank_inverse_batched([U], [4], [1e-3], [1e-3])       # batch larger than 32
    U = torch.zeros(4, 8, device='cuda')
    with pytest.raises(_lib.KfacHipError):
        ops.bn_lowrank_inverse_batched([U], [4], [0.0], [1e-3])        # non-positive damping


def test_capture_on_a_forked_stream_keeps_the_inverse_on_that_stream():
    """Captured into a HIP graph from a stream that is itself a fork of the
    capture (a lane), the batched inverse must not fork again onto its own side
    stream: the plan is told it is not on the capture's origin and keeps every
    launch on the given stream.  The replayed results equal the eager ones bit for
    bit, on every replay."""
    from chainerkfac_amd import device, ops
    dims = [700, 300, 129]           # 6 block columns: a plan with the look-ahead stream
    mats = [torch.from_numpy(spd(d, 300 + d)).cuda() for d in dims]
    eager, info_e = ops.spd_inverse_batched(mats)
    torch.cuda.synchronize()
    outs = [torch.zeros_like(m) for m in mats]
    info = torch.zeros(len(dims), dtype=torch.int32, device='cuda')
    lanes = device.Lanes(2)

    def work():
        lanes.run(lambda: ops.spd_inverse_batched(mats, outs=outs, info=info), mats)
        lanes.join()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()                        # plans, tables and lane workspaces exist before the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for o, e in zip(outs, eager):
        assert torch.equal(o, e)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        work()
    for _ in range(3):
        for o in outs:
            o.zero_()                 # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert info.cpu().tolist() == [0, 0, 0]
        for o, e in zip(outs, eager):
            assert torch.equal(o, e)


def test_update_invs_with_a_diagonal_factor():
    """A factor kept as a vector is inverted entry by entry, 1 / (cov + diagvals), beside the dense
    inverse of the block's other factor, with pi taken from the vector's sum (reference
    fisher_block.py:23-42, :165-179); the batched path of the optimizer hands such blocks to it."""
    from chainerkfac_amd import links as L
    from chainerkfac_amd.optimizers import KFAC
    from chainerkfac_amd.optimizers import fisher_blocks as FB
    r = np.random.default_rng(40)
    lin = L.Linear(50, 30, device='cuda')
    fb = FB.FisherBlockLinear('/fc', lin, cov_ema_decay=1.0, damping=1e-2)
    a = (r.random(51) + 0.1).astype(np.float32)
    G = spd(30, 77)
    fb.cov_emas = [torch.from_numpy(a).cuda(), torch.from_numpy(G).cuda()]
    fb.update_invs()
    ref_emas = [a.copy(), G.copy()]
    diagvals, _ = O.connection_diagvals(ref_emas[0], ref_emas[1], 1e-2)
    ref = O.update_invs(ref_emas, diagvals)
    assert fb.invs[0].shape == (51,) and fb.invs[1].shape == (30, 30)
    np.testing.assert_allclose(fb.invs[0].cpu().numpy(), ref[0], rtol=1e-5)
    assert np.linalg.norm(fb.invs[1].cpu().numpy() - ref[1]) < 1e-3 * np.linalg.norm(ref[1])
    # the damped matrix is left in cov_emas, the vector untouched (as in the reference)
    np.testing.assert_allclose(fb.cov_emas[1].cpu().numpy(), ref_emas[1], rtol=1e-6)
    assert np.array_equal(fb.cov_emas[0].cpu().numpy(), a)
    # through the optimizer's batched path, next to an ordinary block
    model = L.Chain()
    model.a = L.Linear(50, 30, device='cuda')
    model.b = L.Linear(30, 8, device='cuda')
    opt = KFAC(damping=1e-2, cov_ema_decay=1.0).setup(model)
    fa, fbb = opt.fblocks
    A2, G2 = spd(31, 5), spd(8, 6)
    fa.cov_emas = [torch.from_numpy(a).cuda(), torch.from_numpy(G).cuda()]
    fbb.cov_emas = [torch.from_numpy(A2).cuda(), torch.from_numpy(G2).cuda()]
    opt.update_invs_batched(opt.fblocks)
    np.testing.assert_allclose(fa.invs[0].cpu().numpy(), ref[0], rtol=1e-5)
    refb = [A2.copy(), G2.copy()]
    dv, _ = O.connection_diagvals(refb[0], refb[1], 1e-2)
    refb = O.update_invs(refb, dv)
    for got, want in zip(fbb.invs, refb):
        assert np.linalg.norm(got.cpu().numpy() - want) < 1e-3 * np.linalg.norm(want)
