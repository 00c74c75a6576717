"""Pins for the oracle's damping, inverse, preconditioning and update rule (no GPU)."""
import numpy as np
import pytest
import scipy.linalg.lapack as lapack

from oracle import kfac_oracle as O


def spd(d, seed, dtype=np.float32):
    r = np.random.default_rng(seed)
    X = r.standard_normal((2 * d, d))
    return (X.T @ X / (2 * d) + 1e-3 * np.eye(d)).astype(dtype)


def test_pi_closed_form_scaled_identities():
    A = (4.0 * np.eye(5)).astype(np.float32)
    G = (0.25 * np.eye(3)).astype(np.float32)
    pi = O.compute_pi_tracenorm(A, G)
    assert pi.dtype == np.float32
    assert pi == pytest.approx(4.0)           # sqrt(a/g)
    assert O.compute_pi(A, G, 'other') == 1.0
    # general: sqrt((trA/dimA)/(trG/dimG))
    A = spd(6, 1); G = spd(4, 2)
    ref = np.sqrt((np.trace(A.astype(np.float64)) / 6) / (np.trace(G.astype(np.float64)) / 4))
    assert O.compute_pi_tracenorm(A, G) == pytest.approx(ref, rel=1e-6)
    # 1-D (diagonal) factors use the sum
    assert O.compute_pi_tracenorm(np.full(5, 4.0, np.float32), np.full(3, 0.25, np.float32)) == pytest.approx(4.0)


def test_connection_diagvals_and_damping_rounding():
    A = spd(6, 3); G = spd(4, 4)
    (dA, dG), pi = O.connection_diagvals(A, G, damping=1e-3)
    assert dA.dtype == np.float64 and dG.dtype == np.float64
    rW = 1e-3 ** 0.5
    np.testing.assert_allclose(dA, float(pi) * rW, rtol=1e-12)
    np.testing.assert_allclose(dG, rW / float(pi), rtol=1e-6)
    # product of the two damping values is the damping itself
    np.testing.assert_allclose(dA[0] * dG[0], 1e-3, rtol=1e-6)
    # l2_coef larger than damping wins
    (dA2, _), _ = O.connection_diagvals(A, G, damping=1e-3, l2_coef=4e-2)
    np.testing.assert_allclose(dA2, float(pi) * 0.2, rtol=1e-12)
    A0 = A.copy()
    O.damp_inplace(A, dA)
    off = ~np.eye(6, dtype=bool)
    assert np.array_equal(A[off], A0[off])
    expect = (np.diagonal(A0).astype(np.float64) + dA).astype(np.float32)
    assert np.array_equal(np.diagonal(A), expect)


def test_bn_diagvals_no_sqrt_no_pi():
    (d,) = O.bn_diagvals(3, 3, damping=2.5e-4, stab_coeff=16.0)
    np.testing.assert_allclose(d, 4e-3)
    assert d.shape == (6,)
    (d,) = O.bn_diagvals(3, None, damping=1e-3, stab_coeff=2.0)
    assert d.shape == (3,)
    (d,) = O.bn_diagvals(3, 3, damping=1e-3, stab_coeff=2.0, l2_beta=1.0)
    np.testing.assert_allclose(d, [2e-3] * 3 + [2.0] * 3)
    with pytest.raises(RuntimeError):
        O.bn_diagvals(None, None, 1e-3, 1.0)


@pytest.mark.parametrize('d', [1, 2, 7, 64, 200])
def test_inverse_against_lapack_and_float64(d):
    M = spd(d, d)
    inv = O.inverse(M.copy())
    assert inv.dtype == np.float32
    ref64 = np.linalg.inv(M.astype(np.float64))
    assert np.linalg.norm(inv - ref64) / np.linalg.norm(ref64) < 1e-4
    resid = np.linalg.norm(M.astype(np.float64) @ inv - np.eye(d)) / np.sqrt(d)
    assert resid < 1e-3
    np.testing.assert_allclose(inv, inv.T, rtol=1e-5, atol=1e-5)
    # LAPACK potrf + potri (lower) is the library special case
    c, info = lapack.spotrf(M, lower=1)
    assert info == 0
    pi_, info = lapack.spotri(c, lower=1)
    full = np.tril(pi_) + np.tril(pi_, -1).T
    assert np.linalg.norm(inv - full) / np.linalg.norm(full) < 1e-4


def test_inverse_diagonal_matrix_and_nonspd():
    Dg = np.diag(np.array([1.0, 4.0, 0.5], dtype=np.float32))
    np.testing.assert_allclose(O.inverse(Dg), np.diag([1.0, 0.25, 2.0]), rtol=1e-6)
    with pytest.raises(np.linalg.LinAlgError):
        O.inverse(np.array([[1.0, 2.0], [2.0, 1.0]], dtype=np.float32))


def test_update_invs_mutates_and_handles_1d():
    M = spd(5, 9)
    v = np.array([1.0, 3.0], dtype=np.float32)
    M0 = M.copy()
    invs = O.update_invs([M, v], [np.full(5, 0.5), np.full(2, 1.0)])
    assert np.allclose(np.diagonal(M), np.diagonal(M0) + 0.5)
    ref = np.linalg.inv(M0.astype(np.float64) + 0.5 * np.eye(5))
    np.testing.assert_allclose(invs[0], ref, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(invs[1], [0.5, 0.25])


def test_precondition_kronecker_identity():
    r = np.random.default_rng(5)
    dG, c, k = 3, 2, 2
    dA = c * k * k + 1
    A_inv = np.linalg.inv(spd(dA, 1).astype(np.float64)).astype(np.float32)
    G_inv = np.linalg.inv(spd(dG, 2).astype(np.float64)).astype(np.float32)
    gW = r.standard_normal((dG, c, k, k)).astype(np.float32)
    gb = r.standard_normal(dG).astype(np.float32)
    kW, kb = O.precondition_conn(A_inv, G_inv, gW, gb)
    assert kW.shape == gW.shape and kb.shape == gb.shape and kW.dtype == np.float32
    g = np.column_stack([gW.reshape(dG, -1), gb]).astype(np.float64)
    # column-major vec: vec(G^-1 g A^-1) = (A^-1 (x) G^-1) vec(g)
    K = np.kron(A_inv.astype(np.float64), G_inv.astype(np.float64))
    ref = (K @ g.reshape(-1, order='F')).reshape(dG, dA, order='F')
    np.testing.assert_allclose(np.column_stack([kW.reshape(dG, -1), kb]), ref, rtol=1e-4, atol=1e-5)
    # identity inverses return the gradient; no-bias path keeps the shape
    kW2, kb2 = O.precondition_conn(np.eye(dA - 1, dtype=np.float32), np.eye(dG, dtype=np.float32), gW, None)
    assert kb2 is None and np.array_equal(kW2, gW)


def test_precondition_bn_split_and_nan_fallback():
    r = np.random.default_rng(6)
    C = 3
    F_inv = np.linalg.inv(spd(2 * C, 3).astype(np.float64)).astype(np.float32)
    gg = r.standard_normal(C).astype(np.float32)
    gb = r.standard_normal(C).astype(np.float32)
    kg, kb, nan = O.precondition_bn(F_inv, gg, gb)
    assert not nan
    ref = F_inv.astype(np.float64) @ np.concatenate([gg, gb])
    np.testing.assert_allclose(np.concatenate([kg, kb]), ref, rtol=1e-4, atol=1e-6)
    F_bad = F_inv.copy(); F_bad[1, 1] = np.nan
    kg, kb, nan = O.precondition_bn(F_bad, gg, gb)
    assert nan and kg is gg and kb is gb


def test_momentum_update_two_steps():
    p = np.ones(3, dtype=np.float32); v = np.zeros(3, dtype=np.float32)
    g = np.full(3, 2.0, dtype=np.float32)
    O.momentum_update(p, v, g, lr=0.1, momentum=0.9)
    np.testing.assert_allclose(v, -0.2); np.testing.assert_allclose(p, 0.8)
    O.momentum_update(p, v, g, lr=0.1, momentum=0.9)
    np.testing.assert_allclose(v, -0.38, rtol=1e-6); np.testing.assert_allclose(p, 0.42, rtol=1e-6)
    # adjust_momentum scales momentum by lr/lr_pre when lr dropped
    p = np.ones(1, np.float32); v = np.full(1, 1.0, np.float32)
    O.momentum_update(p, v, np.zeros(1, np.float32), lr=0.05, momentum=0.9, lr_pre=0.1, adjust_momentum=True)
    np.testing.assert_allclose(v, 0.45, rtol=1e-6)
