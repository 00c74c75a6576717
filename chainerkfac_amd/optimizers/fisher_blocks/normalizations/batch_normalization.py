"""Fisher block of a BatchNormalization layer: one full (2C x 2C) factor built
from the per-sample gradients of (gamma, beta).  Counterpart of
chainerkfac/optimizers/fisher_blocks/normalizations/batch_normalization.py."""
import warnings

import torch

from chainerkfac_amd import links
from chainerkfac_amd import ops
from chainerkfac_amd.optimizers.fisher_block import FisherBlock
from chainerkfac_amd.optimizers.fisher_block import as_float32


def _same_array(a, b):
    return a is not None and b is not None and a is b


class FisherBlockBatchNormalization(FisherBlock):

    #: largest batch size the low-rank inverse handles (one 32 x 32 Cholesky per block)
    LOWRANK_MAX_BATCH = 32

    def __init__(self, *args, **kwargs):
        self._F = None
        self._U = None
        self._covs = None
        self._own_factor = False
        self._ema_is_single_factor = False
        #: cleared by whoever replaces ``covs`` by something that is not this
        #: process's own single-batch factor (e.g. an average over ranks)
        self.factor_is_local = True
        self.nan_flag = None
        super(FisherBlockBatchNormalization, self).__init__(*args, **kwargs)

    @property
    def funcclass(self):
        return links.BatchNormalizationFunction

    # ``covs`` assigned by anyone but ``backward_preprocess`` (accumulation,
    # an average over ranks, a caller's own factor) no longer is U^T U / n of
    # the kept gradient matrix: forget U, so that the inverse is taken of the
    # factor actually stored and not of the stale low-rank form.
    @property
    def covs(self):
        return self._covs

    @covs.setter
    def covs(self, value):
        self._covs = value
        if not self._own_factor:
            self._U = None

    @property
    def cov_forward(self):
        return None

    @property
    def cov_backward(self):
        return self.covs[0]

    @property
    def inv_forward(self):
        return None

    @property
    def inv_backward(self):
        return self.invs[0]

    def is_mine(self, func, in_data, out_grad_data=None):
        if not isinstance(func, self.funcclass):
            return False
        gamma, beta = self.link.gamma, self.link.beta
        if not _same_array(in_data[1], None if gamma is None else gamma.data) and \
                not _same_array(in_data[2], None if beta is None else beta.data):
            return False
        return True

    def forward_postprocess(self, func, in_data):
        pass   # F needs the output gradient

    def backward_preprocess(self, func, in_data, out_grad_data):
        self._F = self.compute_F(in_data, out_grad_data)
        self._own_factor = True
        try:
            self.covs = [self._F]
        finally:
            self._own_factor = False

    def compute_F(self, in_data, out_grad_data):
        x = as_float32(in_data[0])
        gy = as_float32(out_grad_data[0])
        if x.ndim not in (2, 4):
            raise RuntimeError('len(x.shape) must be 2 or 4, not {}.'.format(x.ndim))
        n = x.shape[0]
        gy_scale = float(n)
        if self._loss_scale is not None:
            gy_scale *= 1.0 / self._loss_scale
        has_gamma = self.link.gamma is not None
        has_beta = self.link.beta is not None
        width = x.shape[1] * (int(has_gamma) + int(has_beta))
        U = self._buffer('U', (n, width), x.device)
        self._U = U
        out, alpha, beta = self._cov_target('F', (width, width), x.device, 1.0 / n)
        eps = self.link.eps

        def stats():
            ops.bn_grad_matrix(x, gy, eps, gy_scale, has_gamma, has_beta, out=U)

        if self.diagonalize:
            # F = diag(mean(grad^2)): diag(diag(F)), a matrix (reference batch_normalization.py:121-124)
            def diagonal_factor():
                stats()
                ops.cov_linear(U, False, alpha, beta, out)
                ops.keep_diag(out)
            self._on_lane(diagonal_factor, (x, gy))
            return out
        if self.pending_covs is not None and self.pending_covs.accepts(n, width):
            # the pass over x and gy now, on a lane; U from the statistics with all other layers'
            # in one launch, right before the grouped launch that reads it
            slabs = self._buffer('bn_stats', (4, n, x.shape[1]), x.device)
            if torch.cuda.is_current_stream_capturing():
                self._on_lane(lambda: ops.bn_stats(x, gy, out=slabs), (x, gy))
            else:
                # Launched from the host, the statistics stay on the caller's stream: the fork onto
                # a lane (an event on one stream, a wait on the other) costs the GPU 10-17 us, as
                # much as the kernel (7-16 us), and its inputs come from that stream anyway
                # (measured on the ResNet-50 update: 31.5 -> 30.7 ms).  In a captured graph the
                # edge is free and the kernel runs beside the other layers' factors.
                ops.bn_stats(x, gy, out=slabs)
                if self.lanes is not None:
                    self.lanes.skip()   # the other layers' pieces keep their lanes
            hw = 1 if x.ndim == 2 else x.shape[2] * x.shape[3]
            self.pending_covs.add_bn_finish(slabs, U, n, x.shape[1], hw, eps, gy_scale, has_gamma, has_beta)
            self._defer_cov(ops.COV_LINEAR, U, False, n, out, alpha, beta)
            return out

        def stats_and_factor():
            stats()
            ops.cov_linear(U, False, alpha, beta, out)

        self._on_lane(stats_and_factor, (x, gy))
        return out

    def update_cov_emas(self):
        first = self.cov_emas is None
        super(FisherBlockBatchNormalization, self).update_cov_emas()
        self._ema_is_single_factor = first or self.cov_ema_decay == 1.0

    def cov_ema_pairs(self):
        pairs = super(FisherBlockBatchNormalization, self).cov_ema_pairs()
        if pairs is not None:
            self._ema_is_single_factor = False   # the average now has history
        return pairs

    def lowrank_inverse_args(self):
        """``(U, split, d_gamma, d_beta)`` when the damped moving average is exactly
        ``U^T U / n + diag(d_gamma | d_beta)`` with U this step's per-sample
        gradient matrix, so that its inverse can be taken by the Woodbury identity
        (an n x n Cholesky) instead of a dense factorisation; ``None`` otherwise
        (accumulation over micro-batches, a moving average with history, factors
        that were averaged over ranks, batches larger than LOWRANK_MAX_BATCH)."""
        U = self._U
        if U is None or not self._ema_is_single_factor or not self.factor_is_local or self.diagonalize:
            return None
        if self.acc_state[0] != 1 or U.shape[0] > self.LOWRANK_MAX_BATCH:
            return None
        if self.cov_emas is None or self.cov_emas[0].shape[0] != U.shape[1]:
            return None
        d_gamma, d_beta = self._diag_pair()
        for d in (d_gamma, d_beta):
            if d is not None and not d > 0.0:
                return None
        split = 0 if self.link.gamma is None else self.link.gamma.size
        return U, split, d_gamma, d_beta

    def _diag_pair(self):
        gamma, beta = self.link.gamma, self.link.beta
        if gamma is None and beta is None:
            raise RuntimeError('gamma and beta must not be None as the same time')
        d_gamma = self.get_diagval('gamma')
        d_beta = self.get_diagval('beta')
        if d_gamma is not None:
            d_gamma *= self.stab_coeff
        if d_beta is not None:
            d_beta *= self.stab_coeff
        return d_gamma, d_beta

    def get_diagvals(self):
        import numpy as np
        d_gamma, d_beta = self._diag_pair()
        setattr(self, 'diag_val_backward', d_gamma)
        gamma, beta = self.link.gamma, self.link.beta
        if d_beta is None:
            return [d_gamma * np.ones(gamma.size)]
        if d_gamma is None:
            return [d_beta * np.ones(beta.size)]
        return [np.hstack((d_gamma * np.ones(gamma.size), d_beta * np.ones(beta.size)))]

    def damp_args(self):
        """``(F, v0, v1, split)``: the damping adds v0 to the first ``split`` diagonal
        entries of F and v1 to the others."""
        d_gamma, d_beta = self._diag_pair()
        F = self.cov_emas[0]
        if d_beta is None:
            return F, d_gamma, d_gamma, F.shape[0]
        if d_gamma is None:
            return F, d_beta, d_beta, F.shape[0]
        return F, d_gamma, d_beta, self.link.gamma.size

    def damp(self):
        F, v0, v1, split = self.damp_args()
        ops.add_diag(F, v0, v1, split=split)

    def kfgrad_operands(self):
        """``(F_inv, g_gamma, g_beta, kf_gamma, kf_beta, nan_flag)`` of the preconditioning
        product, with the output buffers this block keeps."""
        self.check_attr('invs')
        gamma, beta = self.link.gamma, self.link.beta

        def grad_of(param):
            if param is None:
                return None
            g = as_float32(param.grad)
            return g if g.is_contiguous() else g.contiguous()

        kg = None if gamma is None else self._buffer('kf_gamma', gamma.shape, gamma.data.device)
        kb = None if beta is None else self._buffer('kf_beta', beta.shape, beta.data.device)
        if self.nan_flag is None:
            import torch
            self.nan_flag = torch.zeros(1, dtype=torch.int32, device=self.invs[0].device)
        return self.invs[0], grad_of(gamma), grad_of(beta), kg, kb, self.nan_flag

    def finish_kfgrads(self):
        """After the product: ``kfgrad`` in the gradient's own type (reference
        batch_normalization.py:185-193)."""
        gamma, beta = self.link.gamma, self.link.beta
        kg, kb = self._bufs.get('kf_gamma'), self._bufs.get('kf_beta')
        if gamma is not None:
            gamma.kfgrad = kg if gamma.grad.dtype == kg.dtype else kg.to(gamma.grad.dtype)
        if beta is not None:
            beta.kfgrad = kb if beta.grad.dtype == kb.dtype else kb.to(beta.grad.dtype)
        # The reference warns on the spot (batch_normalization.py:21-33), which
        # costs a device->host read per block; here the flag stays on the device
        # and KFAC.check_numerics() reads all of them together at the start of the
        # next step.  ``link.debug`` asks for the immediate warning.
        if self.debug():
            self.warn_if_nan()

    def update_kfgrads(self):
        # NaN anywhere in F^-1 grad makes the kernel hand back the raw gradients
        ops.precond_bn(*self.kfgrad_operands())
        self.finish_kfgrads()

    def warn_if_nan(self):
        if self.nan_flag is not None and int(self.nan_flag.item()):
            warnings.warn('Detected NaN in the kfgrads of the batch normalization layer {}; '
                          '``grad`` was substituted for ``kfgrad``'.format(self.linkname))
            return True
        return False

    def extract_for_reduce_scatter_v(self):
        arrays = self.extract_attr_from_params('grad')
        arrays.append((self.cov_backward, True))
        return arrays
