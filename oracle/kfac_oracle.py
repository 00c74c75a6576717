"""CPU oracle for the K-FAC per-layer hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, in NumPy, the arithmetic that tyohei/chainerkfac performs
on its ``--no_cuda`` (NumPy) path.  It is the checker that the HIP kernels are
compared against and the CPU baseline that ``bench.py`` times.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it; nothing in ``chainerkfac_amd`` does.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  The reference ships no tests, golden vectors or fixtures,
so each function is pinned by an independent check in ``tests/test_oracle_*``:

  linear_A / linear_G / conv_G   float64 einsum closed form, exact symmetry,
                                 A[-1,-1] == 1 (linear) / ho*wo (conv)
  im2col / conv_A                brute-force 6-loop patch extraction,
                                 torch.nn.functional.unfold, and the weight-
                                 gradient ordering identity
                                 dW.reshape(c_out,-1) == gy_mat.T @ x_mat
  bn_F                           torch.nn.functional.batch_norm, and the
                                 identities sum_n gyh == n * dgamma etc.
  accumulate / ema               linear-algebra identities (mean of covs,
                                 reversed EMA weights)
  pi / diagvals / damp           closed form for A=aI, G=gI
  inverse                        scipy.linalg.lapack spotrf/spotri, float64
                                 numpy.linalg.inv, residual ||M Minv - I||
  precondition_*                 Kronecker identity
                                 vec(Ginv g Ainv) = (Ainv (x) Ginv) vec(g)
  pack / unpack / get_nelems     numpy.tril_indices order, brute-force loops
                                 and the C restatement in pack_oracle.c
  momentum_update                closed form after two steps

Third-party arithmetic the reference delegates to Chainer (``F.im2col``,
``F.batch_normalization``; version unpinned in the reference's setup.py:9) is
restated from Chainer's documented behaviour: im2col with ``cover_all=False``
and channel-major (c, kh, kw) rows; batch normalisation with the biased batch
variance and ``eps`` inside the square root.
"""

import numpy as np

NCCL_FLOAT16 = 6
NCCL_FLOAT32 = 7

PI_TYPE_TRACENORM = 'tracenorm'


# --------------------------------------------------------------------------
# Kronecker-factor construction
# --------------------------------------------------------------------------

def linear_A(x, has_bias=True, diagonalize=False):
    """chainerkfac/optimizers/fisher_blocks/connections/linear.py:14-27.  With
    ``diagonalize`` the factor is a vector (:25)."""
    n = x.shape[0]
    if has_bias:
        ones = np.ones(n, dtype=x.dtype)
        x = np.column_stack((x, ones))
    if x.dtype == np.float16:
        x = x.astype(np.float32)
    return (x * x).mean(axis=0) if diagonalize else x.T.dot(x) * (1 / n)


def linear_G(gy, loss_scale=None, diagonalize=False):
    """linear.py:29-46.  With ``diagonalize`` a diagonal matrix (:43-44)."""
    n = gy.shape[0]
    gy_scale = n
    if loss_scale is not None:
        gy_scale *= 1.0 / loss_scale
    if gy.dtype == np.float16:
        gy = gy_scale * gy.astype(np.float32)
    else:
        gy = gy_scale * gy
    return np.diag((gy * gy).mean(axis=0)) if diagonalize else gy.T.dot(gy) * (1 / n)


def conv_out_size(size, k, s, p):
    """Chainer get_conv_outsize with cover_all=False, dilation 1."""
    return (size + 2 * p - k) // s + 1


def im2col(x, ksize, stride, pad):
    """Chainer ``F.im2col(x, ksize, stride, pad)`` as called at
    fisher_blocks/connections/convolution_2d.py:25: returns
    (n, c*kh*kw, out_h, out_w), rows ordered channel-major then kh, kw,
    zero padding, cover_all=False.  Written as the strided (kh, kw) loop
    Chainer's CPU im2col uses."""
    n, c, h, w = x.shape
    kh = kw = ksize
    ho = conv_out_size(h, kh, stride, pad)
    wo = conv_out_size(w, kw, stride, pad)
    xp = np.pad(x, ((0, 0), (0, 0), (pad, pad + stride - 1),
                    (pad, pad + stride - 1)), mode='constant')
    col = np.zeros((n, c, kh, kw, ho, wo), dtype=x.dtype)
    for j in range(kh):
        jlim = j + stride * ho
        for i in range(kw):
            ilim = i + stride * wo
            col[:, :, j, i, :, :] = xp[:, :, j:jlim:stride, i:ilim:stride]
    return col.reshape(n, c * kh * kw, ho, wo)


def conv_patch_matrix(x, ksize, stride, pad, has_bias):
    """convolution_2d.py:25-32: im2col -> NHWC -> (n*ho*wo, c*k*k) with the
    ones column appended last when the link has a bias."""
    col = im2col(x, ksize, stride, pad)
    col = col.transpose(0, 2, 3, 1)
    n, ho, wo, _ = col.shape
    col = col.reshape(n * ho * wo, -1)
    if has_bias:
        ones = np.ones(col.shape[0], dtype=col.dtype)
        col = np.column_stack((col, ones))
    return col, n, ho, wo


def conv_A(x, ksize, stride, pad, has_bias=True):
    """convolution_2d.py:19-41.  Note the scale is 1/n, not 1/(n*ho*wo)."""
    col, n, _, _ = conv_patch_matrix(x, ksize, stride, pad, has_bias)
    A_scale = 1 / n
    if col.dtype == np.float16:
        col = col.astype(np.float32)
    return col.T.dot(col) * A_scale


def conv_G(gy, loss_scale=None, diag=False, diagonalize=False):
    """convolution_2d.py:43-72.  ``diagonalize`` is the block's own switch (:57-62),
    ``diag`` the link attribute (:68-70); both return a matrix."""
    gy = gy.transpose(0, 2, 3, 1)
    n, ho, wo, _ = gy.shape
    gy = gy.reshape(n * ho * wo, -1)
    gy_scale = n
    if loss_scale is not None:
        gy_scale *= 1.0 / loss_scale
    if diagonalize:
        if gy.dtype == np.float16:
            gy = gy_scale * gy.astype(np.float32)
        else:
            gy = gy_scale * gy
        return np.diag((gy * gy).mean(axis=0))
    G_scale = 1 / (n * ho * wo) * (gy_scale ** 2)
    if gy.dtype == np.float16:
        gy = gy.astype(np.float32)
    G = gy.T.dot(gy) * G_scale
    if diag:
        G = np.diag(np.diag(G))
    return G


def batch_normalize(x, eps):
    """Chainer ``F.batch_normalization(x, 1, 0, eps)`` in training mode:
    per-channel batch mean and biased variance over every axis but 1."""
    axes = (0,) + tuple(range(2, x.ndim))
    shape = [1, x.shape[1]] + [1] * (x.ndim - 2)
    mean = x.mean(axis=axes)
    var = x.var(axis=axes)
    std = np.sqrt(var + x.dtype.type(eps), dtype=x.dtype)
    return (x - mean.reshape(shape)) / std.reshape(shape)


def bn_grad_matrix(x, gy, eps, loss_scale=None, has_gamma=True, has_beta=True):
    """normalizations/batch_normalization.py:78-119: the (n, 2C) per-sample
    gradient matrix [sum_hw gy*h | sum_hw gy], gamma part first."""
    ndim = x.ndim
    if ndim not in (2, 4):
        raise RuntimeError(
            'len(x.shape) must be 2 or 4, not {}.'.format(ndim))
    n = x.shape[0]
    gy_scale = n
    if loss_scale is not None:
        gy_scale *= 1.0 / loss_scale
    h = batch_normalize(x, eps)
    if ndim == 2:
        gy = gy_scale * gy
        gyh = gy * h
    else:
        h = h.transpose(0, 2, 3, 1)
        gy = gy.transpose(0, 2, 3, 1)
        gy = gy * gy_scale
        gyh = gy * h
        gyh = gyh.sum(axis=(1, 2))
        gy = gy.sum(axis=(1, 2))
    if not has_beta:
        grad = gyh
    elif not has_gamma:
        grad = gy
    else:
        grad = np.hstack((gyh, gy))
    return grad.astype(x.dtype, copy=False)


def bn_F(x, gy, eps, loss_scale=None, has_gamma=True, has_beta=True, diagonalize=False):
    """batch_normalization.py:78-131 (``diagonalize``: :121-124)."""
    grad = bn_grad_matrix(x, gy, eps, loss_scale, has_gamma, has_beta)
    n = x.shape[0]
    if diagonalize:
        if grad.dtype == np.float16:
            grad = grad.astype(np.float32)
        return np.diag((grad * grad).mean(axis=0))
    F_scale = 1 / n
    if grad.dtype == np.float16:
        grad = grad.astype(np.float32)
    return grad.T.dot(grad) * F_scale


# --------------------------------------------------------------------------
# Accumulation over acc_iters and the moving average
# --------------------------------------------------------------------------

def accumulate_covs(acc_covs, covs, acc_iters):
    """optimizers/kfac.py:294-304.  Returns the new accumulator list."""
    new_covs = [cov * (1 / acc_iters) for cov in covs]
    if acc_covs is None:
        return new_covs
    for acc_cov, new_cov in zip(acc_covs, new_covs):
        acc_cov += new_cov
    return acc_covs


def accumulate_grad(acc_grad, grad, acc_iters):
    """optimizers/kfac.py:286-292."""
    new_grad = grad * (1 / acc_iters)
    if acc_grad is None:
        return new_grad
    acc_grad += new_grad
    return acc_grad


def update_cov_emas(covs, cov_emas, decay):
    """optimizers/fisher_block.py:155-163.  The first call, or decay == 1.0,
    returns a *shallow* list copy (the same arrays); otherwise the new
    covariance is weighted by ``decay`` and the old average by 1-decay."""
    r = decay
    if r == 1.0 or cov_emas is None:
        return list(covs)
    return [r * cov + (1 - r) * cov_ema for cov, cov_ema in zip(covs, cov_emas)]


# --------------------------------------------------------------------------
# Damping
# --------------------------------------------------------------------------

def get_diagval(l2_coef, damping):
    """optimizers/fisher_block.py:14-20 (param present)."""
    r = l2_coef if l2_coef is not None else 0.0
    return max(r, damping)


def compute_pi_tracenorm(lcov, rcov):
    """optimizers/fisher_block.py:23-42."""
    def compute_trace(cov):
        return cov.sum() if cov.ndim == 1 else cov.trace()
    lnorm = compute_trace(lcov) * rcov.shape[0]
    rnorm = compute_trace(rcov) * lcov.shape[0]
    return np.sqrt(lnorm / rnorm, dtype=np.float32)


def compute_pi(lcov, rcov, pi_type=PI_TYPE_TRACENORM):
    """optimizers/fisher_block.py:45-49."""
    if pi_type == PI_TYPE_TRACENORM:
        return compute_pi_tracenorm(lcov, rcov)
    return 1.0


def connection_diagvals(A, G, damping, l2_coef=0.0, pi_type=PI_TYPE_TRACENORM):
    """fisher_blocks/connection.py:66-77.  The returned vectors are float64
    (``xp.ones`` default dtype) scaled by a float32 pi."""
    rW = get_diagval(l2_coef, damping) ** 0.5
    diagvalsA = rW * np.ones(A.shape[0])
    diagvalsG = rW * np.ones(G.shape[0])
    pi = compute_pi(A, G, pi_type)
    return [pi * diagvalsA, (1 / pi) * diagvalsG], pi


def bn_diagvals(n_gamma, n_beta, damping, stab_coeff, l2_gamma=0.0, l2_beta=0.0):
    """normalizations/batch_normalization.py:133-157.  ``n_gamma``/``n_beta``
    are the parameter sizes, or None where the parameter is absent."""
    if n_gamma is None and n_beta is None:
        raise RuntimeError('gamma and beta must not be None as the same time')
    d_gamma = None if n_gamma is None else get_diagval(l2_gamma, damping) * stab_coeff
    d_beta = None if n_beta is None else get_diagval(l2_beta, damping) * stab_coeff
    if d_beta is None:
        return [d_gamma * np.ones(n_gamma)]
    if d_gamma is None:
        return [d_beta * np.ones(n_beta)]
    return [np.hstack((d_gamma * np.ones(n_gamma), d_beta * np.ones(n_beta)))]


def damp_inplace(cov_ema, diagvals):
    """optimizers/fisher_block.py:175: the float64 sum is rounded to the
    factor's dtype when written back into its diagonal, in place."""
    np.fill_diagonal(cov_ema, np.diagonal(cov_ema) + diagvals)
    return cov_ema


# --------------------------------------------------------------------------
# Inverse
# --------------------------------------------------------------------------

def inverse(a, use_cholesky=True):
    """optimizers/cholesky_inverse.py:16-25 (NumPy branch)."""
    if use_cholesky:
        la = np.linalg.cholesky(a)
        la_inv = np.linalg.inv(la)
        return np.matmul(la_inv.T, la_inv)
    return np.linalg.inv(a)


def update_invs(cov_emas, diagvals_list):
    """optimizers/fisher_block.py:165-179."""
    invs = []
    for cov_ema, diagvals in zip(cov_emas, diagvals_list):
        if cov_ema.ndim == 1:
            inv = 1 / (cov_ema + diagvals)
        else:
            damp_inplace(cov_ema, diagvals)
            inv = inverse(cov_ema, True)
        invs.append(inv)
    return invs


# --------------------------------------------------------------------------
# Preconditioning
# --------------------------------------------------------------------------

def precondition_conn(A_inv, G_inv, gW, gb=None):
    """connections/convolution_2d.py:74-90, connections/linear.py:48-61 and the
    split of fisher_blocks/connection.py:51-61.  Returns (W.kfgrad, b.kfgrad)."""
    grad = gW.reshape(gW.shape[0], -1)
    if gb is not None:
        grad = np.column_stack([grad, gb])
    out_dtype = grad.dtype
    if A_inv.dtype != grad.dtype:
        grad = grad.astype(A_inv.dtype)
    kfgrad = np.dot(np.dot(G_inv, grad), A_inv).astype(out_dtype)
    if gb is not None:
        return kfgrad[:, :-1].reshape(gW.shape), kfgrad[:, -1].reshape(gb.shape)
    return kfgrad.reshape(gW.shape), None


def precondition_bn(F_inv, g_gamma, g_beta):
    """normalizations/batch_normalization.py:159-191 incl. the NaN fallback of
    :21-33.  Returns (gamma.kfgrad, beta.kfgrad, nan_detected)."""
    if g_beta is None:
        grad = g_gamma
    elif g_gamma is None:
        grad = g_beta
    else:
        grad = np.hstack((g_gamma, g_beta))
    out_dtype = grad.dtype
    if F_inv.dtype != grad.dtype:
        grad = grad.astype(F_inv.dtype)
    kfgrads = np.dot(F_inv, grad).astype(out_dtype)
    if np.any(np.isnan(kfgrads)):
        return g_gamma, g_beta, True
    if g_beta is None:
        return kfgrads, None, False
    if g_gamma is None:
        return None, kfgrads, False
    return kfgrads[:len(g_gamma)], kfgrads[len(g_gamma):], False


def momentum_update(param, v, grad, lr, momentum, lr_pre=None, adjust_momentum=False):
    """optimizers/kfac.py:87-99, in place on ``param`` and ``v``."""
    if lr_pre is None:
        lr_pre = lr
    if adjust_momentum and lr < lr_pre:
        momentum *= lr / lr_pre
    v *= momentum
    v -= lr * grad
    param += v


# --------------------------------------------------------------------------
# Communicator buffer layout: triangular pack / unpack
# --------------------------------------------------------------------------

def get_nelems(arrays):
    """communicators/_utility.py:72-83."""
    nelems = 0
    for local_arrays in arrays:
        for array, triangular in local_arrays:
            if triangular:
                if array.shape[0] != array.shape[1]:
                    raise RuntimeError('get_nelems: not a square matrix')
                nelems += array.shape[0] * (array.shape[0] + 1) // 2
            else:
                nelems += array.size
    return nelems


class ArraysInfo(object):
    """communicators/pure_nccl_communicator.py:221-279: the descriptor tables
    (host side only; ``dptr`` is left to the caller)."""

    def __init__(self, arrays):
        n_arrays = sum(len(local_arrays) for local_arrays in arrays)
        self.rank = np.empty(n_arrays, dtype=np.int32)
        self.dtype = np.empty(n_arrays, dtype=np.int32)
        self.triangle_size = np.empty(n_arrays, dtype=np.int32)
        self.size_csum = np.empty(n_arrays + 1, dtype=np.int32)
        self.buf_size_csum = np.empty(n_arrays + 1, dtype=np.int32)
        self.size_csum[0] = 0
        self.buf_size_csum[0] = 0
        self.flat = []
        i = 0
        for rank, local_arrays in enumerate(arrays):
            for array, triangular in local_arrays:
                self.rank[i] = rank
                if array.dtype not in [np.float16, np.float32]:
                    raise ValueError('dtype must be float16 or float32.')
                self.dtype[i] = (NCCL_FLOAT16 if array.dtype == np.float16
                                 else NCCL_FLOAT32)
                if triangular:
                    _len = array.shape[0]
                    self.triangle_size[i] = _len
                    nelems = _len * (_len + 1) // 2
                else:
                    self.triangle_size[i] = 0
                    nelems = array.size
                self.size_csum[i + 1] = self.size_csum[i] + array.size
                self.buf_size_csum[i + 1] = self.buf_size_csum[i] + nelems
                self.flat.append(array)
                i += 1
        assert n_arrays == i
        self.n_arrays = n_arrays
        self.size_total = int(self.size_csum[n_arrays])
        self.buf_size_total = int(self.buf_size_csum[n_arrays])


def pack_bruteforce(arrays, buf, target=-1):
    """pure_nccl_communicator.py:300-377 evaluated thread by thread: one loop
    iteration per source element (``tid``).  Small inputs only."""
    info = ArraysInfo(arrays)
    for j in range(info.n_arrays):
        if target >= 0 and info.rank[j] != target:
            continue
        src = info.flat[j].reshape(-1)
        dst = buf[info.buf_size_csum[j]:info.buf_size_csum[j + 1]]
        m = int(info.triangle_size[j])
        for src_idx in range(src.size):
            if m > 0:
                row_idx = src_idx // m
                col_idx = src_idx % m
                if col_idx > row_idx:
                    continue
                dst_idx = (row_idx * (row_idx + 1) // 2) + col_idx
            else:
                dst_idx = src_idx
            dst[dst_idx] = src[src_idx]
    return buf


def unpack_bruteforce(arrays, buf, target=-1, divisor=1):
    """pure_nccl_communicator.py:380-463 evaluated thread by thread."""
    info = ArraysInfo(arrays)
    for j in range(info.n_arrays):
        if target >= 0 and info.rank[j] != target:
            continue
        dst = info.flat[j].reshape(-1)
        src = buf[info.buf_size_csum[j]:info.buf_size_csum[j + 1]]
        m = int(info.triangle_size[j])
        for dst_idx in range(dst.size):
            if m > 0:
                row_idx = dst_idx // m
                col_idx = dst_idx % m
                if row_idx >= col_idx:
                    src_idx = (row_idx * (row_idx + 1) // 2) + col_idx
                else:
                    src_idx = (col_idx * (col_idx + 1) // 2) + row_idx
            else:
                src_idx = dst_idx
            src_val = src[src_idx] / src.dtype.type(divisor)
            dst[dst_idx] = src_val
    return arrays


def pack(arrays, buf, target=-1):
    """Vectorised form of :func:`pack_bruteforce` (``numpy.tril_indices`` order
    equals slot ``r(r+1)/2 + c``)."""
    info = ArraysInfo(arrays)
    for j in range(info.n_arrays):
        if target >= 0 and info.rank[j] != target:
            continue
        a = info.flat[j]
        dst = buf[info.buf_size_csum[j]:info.buf_size_csum[j + 1]]
        m = int(info.triangle_size[j])
        if m > 0:
            dst[:] = a[np.tril_indices(m)]
        else:
            dst[:] = a.reshape(-1)
    return buf


def unpack(arrays, buf, target=-1, divisor=1):
    """Vectorised form of :func:`unpack_bruteforce`."""
    info = ArraysInfo(arrays)
    for j in range(info.n_arrays):
        if target >= 0 and info.rank[j] != target:
            continue
        a = info.flat[j]
        src = buf[info.buf_size_csum[j]:info.buf_size_csum[j + 1]]
        val = (src / src.dtype.type(divisor)).astype(a.dtype)
        m = int(info.triangle_size[j])
        if m > 0:
            r, c = np.tril_indices(m)
            a[r, c] = val
            a[c, r] = val
        else:
            a.reshape(-1)[:] = val
    return arrays
