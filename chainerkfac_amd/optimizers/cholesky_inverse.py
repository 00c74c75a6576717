"""``inverse(a, use_cholesky=True)``: the free function of the reference
(chainerkfac/optimizers/cholesky_inverse.py:16-102) on the HIP path."""
import torch

from chainerkfac_amd import device as _dev
from chainerkfac_amd import ops


def inverse(a, use_cholesky=True):
    """Dense inverse of the SPD float32 matrix ``a`` (a GPU tensor) through a
    blocked Cholesky factorisation and potri.  Returns a new tensor; ``a`` is
    left untouched (the reference's GPU branch overwrites it with its Cholesky
    factor, its NumPy branch does not).

    Only the Cholesky branch exists: ``use_cholesky=False`` (the reference's LU
    path) raises.
    """
    if not use_cholesky:
        raise NotImplementedError(
            'only the Cholesky inverse is implemented (use_cholesky=True)')
    _dev.require_gpu_tensor(a, 'a')
    if a.ndim != 2 or a.shape[0] != a.shape[1]:
        raise ValueError('a must be a square matrix')
    outs, _ = ops.spd_inverse_batched([a])
    return outs[0]
