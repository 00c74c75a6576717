"""Fisher-block base class on the HIP path.

Mirrors the object contract of the reference
(chainerkfac/optimizers/fisher_block.py:52-216): attributes ``covs``,
``cov_emas``, ``invs``, ``acc_covs``, ``diagonalize``, ``linkname``, ``link``,
``xp``; methods ``is_mine``, ``forward_postprocess``, ``backward_preprocess``,
``update_cov_emas``, ``update_invs``, ``update_kfgrads``, ``get_diagvals``,
``check_attr`` and the ``extract_for_*`` buffer-order helpers.  Arrays are
float32 torch-ROCm tensors and every numerical step runs in libkfac_hip.

Differences that follow from running on persistent device buffers:
  * factors, their moving averages and inverses live in buffers owned by the
    block and are overwritten each step (stable device pointers);
  * with ``cov_ema_decay != 1`` the first moving average is a copy of the
    covariance, not an alias of the same array, so the in-place damping of
    ``update_invs`` does not show up in ``covs``;
  * the damping scalars (pi) stay on the device; ``get_diagvals`` copies them
    to the host only when it is called explicitly.
"""
import torch

from chainerkfac_amd import ops

PI_TYPE_TRACENORM = 'tracenorm'


def get_diagval(link, attrname, damping):
    """max(param.l2_coef, damping), or None when the link lacks the parameter
    (reference fisher_block.py:14-20)."""
    param = getattr(link, attrname, None)
    if param is None:
        return None
    r = getattr(param, 'l2_coef', 0.0)
    return max(r, damping)


def compute_pi_tracenorm(lcov, rcov):
    """sqrt((tr(l)/dim(l)) / (tr(r)/dim(r))) as a float32 (reference
    fisher_block.py:23-42); evaluated with torch reductions, host result."""
    def tr(c):
        return c.sum() if c.ndim == 1 else torch.diagonal(c).sum()
    lnorm = tr(lcov).float() * rcov.shape[0]
    rnorm = tr(rcov).float() * lcov.shape[0]
    return torch.sqrt(lnorm / rnorm)


def compute_pi(lcov, rcov, pi_type=PI_TYPE_TRACENORM):
    if pi_type == PI_TYPE_TRACENORM:
        return compute_pi_tracenorm(lcov, rcov)
    return 1.0


def as_float32(t):
    """float16 activations and gradients enter the factor and preconditioning kernels as
    float32, like the reference's cast before its GEMMs (linear.py:22-23, 38-39,
    convolution_2d.py:35-37, 57-66, batch_normalization.py:122-129)."""
    import torch
    if t is not None and t.dtype == torch.float16:
        return t.float()
    return t


class FisherBlock(object):

    def __init__(self, linkname, link, cov_ema_decay, damping,
                 communicate_after_forward=False, pi_type=PI_TYPE_TRACENORM,
                 use_cholesky=True, stab_coeff=64.0, loss_scale=None):
        if not use_cholesky:
            raise NotImplementedError('only the Cholesky inverse exists on the HIP path')
        self._link = link
        self._linkname = linkname
        self._linkclass = link.__class__
        self._communicate_after_forward = communicate_after_forward
        self._pi_type = pi_type
        self._use_cholesky = use_cholesky
        self._loss_scale = loss_scale
        self.cov_ema_decay = cov_ema_decay
        self.damping = damping
        self.stab_coeff = stab_coeff
        self.xp = torch
        self.covs = None
        self.invs = None
        self.cov_emas = None
        self.acc_covs = None
        self.diagonalize = False
        # (acc_iters, index of the current micro-batch); set by the optimizer
        self.acc_state = (1, 0)
        #: ops.PendingCovs of the optimizer, or None: where the factors of small
        #: layers wait for one grouped launch instead of being computed on the spot
        self.pending_covs = None
        #: device.Lanes of the optimizer, or None: side streams for the kernels this
        #: block launches on its own (they are independent of other layers' work)
        self.lanes = None
        self._bufs = {}

    # ---- identity -------------------------------------------------------
    @property
    def linkname(self):
        return self._linkname

    @property
    def link(self):
        return self._link

    @property
    def funcclass(self):
        raise NotImplementedError

    @property
    def cov_forward(self):
        raise NotImplementedError

    @property
    def cov_backward(self):
        raise NotImplementedError

    @property
    def inv_forward(self):
        raise NotImplementedError

    @property
    def inv_backward(self):
        raise NotImplementedError

    def debug(self):
        return getattr(self._link, 'debug', False)

    def is_mine(self, func, in_data, out_grad_data=None):
        raise NotImplementedError

    def forward_postprocess(self, func, in_data):
        raise NotImplementedError

    def backward_preprocess(self, func, in_data, out_grad_data):
        raise NotImplementedError

    def check_attr(self, name):
        if getattr(self, name) is None:
            raise RuntimeError('{} is None:\nlinkname: {}\nlinkclass: {}'.format(
                name, self._linkname, self._linkclass))

    def get_diagval(self, attr):
        return get_diagval(self._link, attr, self.damping)

    # ---- buffers --------------------------------------------------------
    def _buffer(self, key, shape, device):
        buf = self._bufs.get(key)
        if buf is None or tuple(buf.shape) != tuple(shape) or buf.device != device:
            buf = self._bufs[key] = torch.empty(shape, dtype=torch.float32, device=device)
        return buf

    def _cov_target(self, key, shape, device, scale):
        """Where a covariance of this step goes and with which alpha / beta.

        With accumulation (acc_iters > 1) the kernel adds scale/acc_iters times
        the new covariance onto the running buffer (beta = 1 after the first
        micro-batch), which is the sum KFAC.accumulate_covs forms in the
        reference (optimizers/kfac.py:294-304)."""
        acc_iters, acc_index = self.acc_state
        if acc_iters > 1:
            return (self._buffer('acc_' + key, shape, device), scale / acc_iters,
                    0.0 if acc_index == 0 else 1.0)
        return self._buffer(key, shape, device), scale, 0.0

    def _on_lane(self, fn, tensors=()):
        """Runs ``fn`` (kernel launches that read ``tensors``) on the next side stream."""
        if self.lanes is None:
            return fn()
        return self.lanes.run(fn, tensors)

    def _defer_cov(self, kind, x, ones, rows, out, alpha, beta, stride=1):
        """Hands a factor to the grouped launch if there is one and the factor
        is small; True when it did (``out`` is then filled at the flush)."""
        pending = self.pending_covs
        if pending is None or not pending.accepts(rows, out.shape[0]):
            return False
        pending.add(kind, x, ones, out, alpha, beta, stride)
        return True

    # ---- moving average ---------------------------------------------------
    def update_cov_emas(self):
        self.check_attr('covs')
        r = self.cov_ema_decay
        if r == 1.0:
            self.cov_emas = list(self.covs)
        elif self.cov_emas is None:
            self.cov_emas = []
            for i, cov in enumerate(self.covs):
                ema = self._buffer('ema{}'.format(i), cov.shape, cov.device)
                ema.copy_(cov)
                self.cov_emas.append(ema)
        else:
            for cov, cov_ema in self.cov_ema_pairs():
                ops.axpby(cov, cov_ema, r, 1 - r)

    def cov_ema_pairs(self):
        """The (covariance, moving average) pairs of a step that does average
        (not the first one, decay != 1), else None: what ``KFAC.update_cov_emas``
        hands to one launch for all blocks."""
        if self.cov_ema_decay == 1.0 or self.cov_emas is None:
            return None
        self.check_attr('covs')
        return list(zip(self.covs, self.cov_emas))

    # ---- damping + inverse ------------------------------------------------
    def _inv_buffers(self):
        return [self._buffer('inv{}'.format(i), c.shape, c.device)
                for i, c in enumerate(self.cov_emas)]

    def damp(self):
        """Add the damping to the diagonals of ``cov_emas`` in place."""
        raise NotImplementedError

    def has_diagonal_factor(self):
        """True when a factor is kept as its diagonal only (a 1-D array)."""
        return self.cov_emas is not None and any(c.ndim == 1 for c in self.cov_emas)

    def update_invs(self):
        self.check_attr('cov_emas')
        if not self.has_diagonal_factor():
            self.damp()
            self.invs, self.inv_info = ops.spd_inverse_batched(self.cov_emas, outs=self._inv_buffers())
            return
        # A factor kept as a 1-D array is inverted entry by entry, 1 / (cov + diagvals)
        # (reference fisher_block.py:165-179); the damping values come to the host here
        # (get_diagvals), which the all-matrix path above avoids.
        import numpy as np
        invs, dense, dense_at = [], [], []
        for i, (c, vals) in enumerate(zip(self.cov_emas, self.get_diagvals())):
            vals = np.asarray(vals, dtype=np.float64).reshape(-1)
            changes = np.nonzero(vals != vals[0])[0]
            split = int(changes[0]) if changes.size else vals.size
            if not np.all(vals[split:] == vals[-1]):
                raise ValueError('the damping of a factor must take at most two values')
            if c.ndim == 1:
                invs.append(ops.recip_add(c, vals[0], vals[-1], split,
                                          out=self._buffer('inv{}'.format(i), c.shape, c.device)))
            elif c.ndim == 2:
                ops.add_diag(c, vals[0], vals[-1], split=split)
                dense.append(c)
                dense_at.append(i)
                invs.append(None)
            else:
                raise ValueError('a factor must be a vector or a square matrix')
        self.inv_info = None
        if dense:
            outs, self.inv_info = ops.spd_inverse_batched(
                dense, outs=[self._buffer('inv{}'.format(i), self.cov_emas[i].shape, self.cov_emas[i].device)
                             for i in dense_at])
            for i, o in zip(dense_at, outs):
                invs[i] = o
        self.invs = invs

    def get_diagvals(self):
        raise NotImplementedError

    def update_kfgrads(self):
        raise NotImplementedError

    # ---- communicator buffer order -----------------------------------------
    def extract_attr_from_params(self, attrname, triangular=False):
        arrays = []
        for _, param in sorted(self.link.namedparams()):
            x = getattr(param, attrname, None)
            if x is not None:
                arrays.append((x, triangular))
        return arrays

    def extract_for_reduce_scatter_v_after_forward(self):
        if self._communicate_after_forward:
            return [(self.cov_forward, True)]
        return []

    def extract_for_reduce_scatter_v(self):
        arrays = self.extract_attr_from_params('grad')
        if not self._communicate_after_forward:
            arrays.append((self.cov_forward, True))
        arrays.append((self.cov_backward, True))
        return arrays

    def extract_for_all_gather_v(self, target='kfgrad'):
        return self.extract_attr_from_params(target)
