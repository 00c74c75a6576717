"""Pins for the oracle's Kronecker-factor construction (no GPU).

The reference holds no tests or vectors for these functions, so each is pinned
by something independent of the oracle's own formula: float64 closed forms,
brute-force patch extraction, torch's CPU unfold / conv2d autograd /
batch_norm, and structural identities a dropped term or transposed operand
would break.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

from oracle import kfac_oracle as O


def rng(seed):
    return np.random.default_rng(seed)


def test_linear_A_closed_form_and_invariants():
    x = rng(0).random((16, 7), dtype=np.float32)
    A = O.linear_A(x, has_bias=True)
    xe = np.concatenate([x.astype(np.float64), np.ones((16, 1))], axis=1)
    ref = np.einsum('ni,nj->ij', xe, xe) / 16
    assert A.dtype == np.float32 and A.shape == (8, 8)
    np.testing.assert_allclose(A, ref, rtol=1e-5)
    assert np.array_equal(A, A.T)
    assert A[-1, -1] == pytest.approx(1.0)
    np.testing.assert_allclose(A[-1, :-1], x.mean(axis=0), rtol=1e-5)
    A0 = O.linear_A(x, has_bias=False)
    np.testing.assert_allclose(A0, ref[:-1, :-1], rtol=1e-5)


def test_linear_G_scale():
    gy = rng(1).standard_normal((8, 5)).astype(np.float32)
    G = O.linear_G(gy)
    ref = 8 * gy.astype(np.float64).T @ gy.astype(np.float64)
    np.testing.assert_allclose(G, ref, rtol=1e-5)
    G2 = O.linear_G(gy, loss_scale=4.0)
    np.testing.assert_allclose(G2, ref / 16, rtol=1e-5)


def _patches_bruteforce(x, k, s, p, has_bias):
    n, c, h, w = x.shape
    ho = (h + 2 * p - k) // s + 1
    wo = (w + 2 * p - k) // s + 1
    d = c * k * k + (1 if has_bias else 0)
    P = np.zeros((n * ho * wo, d), dtype=np.float64)
    for i in range(n):
        for y in range(ho):
            for xx in range(wo):
                r = (i * ho + y) * wo + xx
                for ci in range(c):
                    for a in range(k):
                        for b in range(k):
                            yy = y * s - p + a
                            xw = xx * s - p + b
                            if 0 <= yy < h and 0 <= xw < w:
                                P[r, (ci * k + a) * k + b] = x[i, ci, yy, xw]
                if has_bias:
                    P[r, -1] = 1.0
    return P, ho, wo


@pytest.mark.parametrize('k,s,p,h,w', [(3, 1, 1, 6, 5), (3, 2, 1, 7, 7), (1, 1, 0, 4, 4),
                                        (1, 2, 0, 6, 6), (5, 1, 0, 8, 8), (7, 2, 3, 12, 12),
                                        (3, 2, 0, 8, 8)])
def test_conv_A_bruteforce_and_unfold(k, s, p, h, w):
    x = rng(k * 10 + s).standard_normal((3, 2, h, w)).astype(np.float32)
    P, ho, wo = _patches_bruteforce(x, k, s, p, True)
    A = O.conv_A(x, k, s, p, has_bias=True)
    ref = P.T @ P / 3
    np.testing.assert_allclose(A, ref, rtol=2e-5, atol=1e-6)
    assert np.array_equal(A, A.T)
    assert A[-1, -1] == pytest.approx(ho * wo)
    # torch unfold gives (n, c*k*k, L) with the same channel-major row order
    u = TF.unfold(torch.from_numpy(x), k, padding=p, stride=s).numpy()
    col = O.im2col(x, k, s, p).reshape(3, -1, ho * wo)
    assert np.array_equal(col, u)


def test_conv_A_1x1_reduces_to_outer_products():
    x = rng(5).standard_normal((4, 6, 3, 3)).astype(np.float32)
    A = O.conv_A(x, 1, 1, 0, has_bias=False)
    xs = x.astype(np.float64).reshape(4, 6, 9)
    ref = np.einsum('ncl,ndl->cd', xs, xs) / 4
    np.testing.assert_allclose(A, ref, rtol=1e-5)


def test_conv_factor_ordering_matches_weight_gradient():
    """dW.reshape(c_out,-1) == gy_mat^T x_mat ties the (c,kh,kw) column order
    of A and the row order of G to the weight layout."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 3, 7, 6, generator=g)
    W = torch.randn(4, 3, 3, 3, generator=g, requires_grad=True)
    y = TF.conv2d(x, W, None, stride=2, padding=1)
    gy = torch.randn(y.shape, generator=g)
    y.backward(gy)
    col, n, ho, wo = O.conv_patch_matrix(x.numpy(), 3, 2, 1, False)
    gy_mat = gy.numpy().transpose(0, 2, 3, 1).reshape(n * ho * wo, -1)
    np.testing.assert_allclose(W.grad.numpy().reshape(4, -1), gy_mat.T @ col,
                               rtol=1e-4, atol=1e-5)


def test_conv_G_closed_form():
    gy = rng(7).standard_normal((4, 5, 3, 2)).astype(np.float32)
    G = O.conv_G(gy)
    g = gy.astype(np.float64)
    ref = np.einsum('nchw,ndhw->cd', g, g) * (4 ** 2) / (4 * 3 * 2)
    np.testing.assert_allclose(G, ref, rtol=1e-5, atol=1e-5)
    assert np.array_equal(G, G.T)
    np.testing.assert_allclose(O.conv_G(gy, loss_scale=8.0), ref / 64, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize('shape', [(6, 4, 5, 3), (8, 5)])
def test_bn_F_against_torch_batch_norm(shape):
    r = rng(11)
    x = (r.standard_normal(shape) * 2 + 0.7).astype(np.float32)
    gy = r.standard_normal(shape).astype(np.float32)
    eps = 2e-5
    n, C = shape[0], shape[1]
    xt = torch.from_numpy(x).double()
    gamma = torch.ones(C, dtype=torch.double, requires_grad=True)
    beta = torch.zeros(C, dtype=torch.double, requires_grad=True)
    h = TF.batch_norm(xt, None, None, gamma, beta, training=True, eps=eps)
    np.testing.assert_allclose(O.batch_normalize(x, eps), h.detach().numpy(), rtol=1e-4, atol=1e-5)
    # per-sample gradient matrix, built independently with torch in float64
    gyt = torch.from_numpy(gy).double() * n
    hd = h.detach()
    if len(shape) == 4:
        U = torch.cat([(gyt * hd).sum((2, 3)), gyt.sum((2, 3))], 1).numpy()
    else:
        U = torch.cat([gyt * hd, gyt], 1).numpy()
    F = O.bn_F(x, gy, eps)
    assert F.shape == (2 * C, 2 * C)
    np.testing.assert_allclose(F, U.T @ U / n, rtol=2e-4, atol=1e-4)
    # sum over samples of the per-sample rows equals n * (dgamma, dbeta)
    h.backward(torch.from_numpy(gy).double())
    Um = O.bn_grad_matrix(x, gy, eps)
    np.testing.assert_allclose(Um[:, :C].sum(0), n * gamma.grad.numpy(), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(Um[:, C:].sum(0), n * beta.grad.numpy(), rtol=1e-4, atol=1e-4)
    # halves
    Fg = O.bn_F(x, gy, eps, has_beta=False)
    Fb = O.bn_F(x, gy, eps, has_gamma=False)
    np.testing.assert_allclose(Fg, F[:C, :C], rtol=1e-6)
    np.testing.assert_allclose(Fb, F[C:, C:], rtol=1e-6)


def test_bn_rejects_other_ranks():
    x = np.zeros((2, 3, 4), dtype=np.float32)
    with pytest.raises(RuntimeError):
        O.bn_F(x, x, 1e-5)


def test_accumulate_is_mean_of_covs():
    r = rng(2)
    covs = [[r.standard_normal((4, 4)).astype(np.float32), r.standard_normal((3, 3)).astype(np.float32)]
            for _ in range(4)]
    acc = None
    for c in covs:
        acc = O.accumulate_covs(acc, c, 4)
    np.testing.assert_allclose(acc[0], np.mean([c[0] for c in covs], axis=0), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(acc[1], np.mean([c[1] for c in covs], axis=0), rtol=1e-5, atol=1e-6)
    g = None
    grads = [r.standard_normal(5).astype(np.float32) for _ in range(4)]
    for gg in grads:
        g = O.accumulate_grad(g, gg, 4)
    np.testing.assert_allclose(g, np.mean(grads, axis=0), rtol=1e-5, atol=1e-6)


def test_ema_weights_new_cov_by_decay_and_aliases_first():
    a = np.full((2, 2), 2.0, dtype=np.float32)
    first = O.update_cov_emas([a], None, 0.99)
    assert first[0] is a            # shallow copy: same array
    same = O.update_cov_emas([a], [np.zeros((2, 2), np.float32)], 1.0)
    assert same[0] is a
    ema = O.update_cov_emas([a], [np.zeros((2, 2), np.float32)], 0.75)
    np.testing.assert_allclose(ema[0], 1.5)   # 0.75 * new + 0.25 * old


def test_diagonal_branches_are_the_diagonals_of_the_full_factors():
    """The ``diagonalize`` / ``link.diag`` branches (linear.py:25,43-44, convolution_2d.py:56-70,
    batch_normalization.py:121-124) against the diagonal of the float64 Gram matrix written out
    independently: a vector for the linear A factor, matrices with zero off-diagonals elsewhere."""
    r = rng(20)
    x = r.standard_normal((6, 5)).astype(np.float32)
    xe = np.concatenate([x.astype(np.float64), np.ones((6, 1))], axis=1)
    A = O.linear_A(x, True, diagonalize=True)
    assert A.shape == (6,)
    np.testing.assert_allclose(A, np.einsum('ni,ni->i', xe, xe) / 6, rtol=1e-5)
    gy = (r.standard_normal((6, 4)) / 6).astype(np.float32)
    G = O.linear_G(gy, diagonalize=True)
    g64 = gy.astype(np.float64)
    assert G.shape == (4, 4) and np.count_nonzero(G - np.diag(np.diag(G))) == 0
    np.testing.assert_allclose(np.diag(G), 6 * np.einsum('ni,ni->i', g64, g64), rtol=1e-5)
    gyc = (r.standard_normal((3, 4, 5, 5)) / 3).astype(np.float32)
    full = O.conv_G(gyc).astype(np.float64)
    for kw in ({'diag': True}, {'diagonalize': True}):
        Gc = O.conv_G(gyc, **kw)
        assert Gc.shape == (4, 4) and np.count_nonzero(Gc - np.diag(np.diag(Gc))) == 0
        np.testing.assert_allclose(np.diag(Gc), np.diag(full), rtol=1e-5)
        m = gyc.astype(np.float64).transpose(0, 2, 3, 1).reshape(-1, 4)
        np.testing.assert_allclose(np.diag(Gc), 3.0 ** 2 / 75 * np.einsum('ni,ni->i', m, m), rtol=1e-5)
    xb = r.standard_normal((4, 3, 5, 5)).astype(np.float32)
    gb = (r.standard_normal((4, 3, 5, 5)) / 4).astype(np.float32)
    F = O.bn_F(xb, gb, 2e-5, diagonalize=True)
    assert F.shape == (6, 6) and np.count_nonzero(F - np.diag(np.diag(F))) == 0
    np.testing.assert_allclose(np.diag(F), np.diag(O.bn_F(xb, gb, 2e-5)), rtol=1e-5)
