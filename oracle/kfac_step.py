"""One K-FAC optimizer step restated on the CPU.  TEST INFRASTRUCTURE ONLY.

Follows KFAC.update / accumulate / update_kfgrads of the reference
(chainerkfac/optimizers/kfac.py:222-310) on recorded per-layer tensors: for
every layer, in sorted link-name order, moving average -> damping -> inverse ->
preconditioning (fisher_block.py:155-179, fisher_blocks/connection.py:51-77,
normalizations/batch_normalization.py:133-191), then the momentum rule
(kfac.py:87-99).  State that the reference keeps across steps (cov_emas, the
in-place damped diagonals of the NumPy path, momentum buffers, accumulators) is
kept here the same way.

Pinned by tests/test_oracle_step.py against an independent float64 restatement
(torch unfold / explicit batch statistics, numpy.linalg.inv, an explicit
Kronecker-product solve): one and three steps with the damped diagonal carried
inside the moving average, decay 1, accumulation over two micro-batches, and a
loss scale that must cancel.
"""
import numpy as np

from . import kfac_oracle as O


class LayerRecord(object):
    """What the function hooks see for one layer in one micro-batch."""

    def __init__(self, kind, name, x, gy, params, grads, **attrs):
        self.kind = kind          # 'linear' | 'conv' | 'bn'
        self.name = name
        self.x = x
        self.gy = gy
        self.params = params      # dict name -> ndarray (updated in place)
        self.grads = grads        # dict name -> ndarray
        self.attrs = attrs        # ksize/stride/pad or eps


class OracleKFAC(object):

    def __init__(self, lr=0.001, momentum=0.9, cov_ema_decay=0.99, damping=0.03, stab_coeff=16.0,
                 pi_type='tracenorm', loss_scale=None, acc_iters=1):
        self.lr = lr
        self.momentum = momentum
        self.decay = cov_ema_decay
        self.damping = damping
        self.stab_coeff = stab_coeff
        self.pi_type = pi_type
        self.loss_scale = loss_scale
        self.acc_iters = acc_iters
        self.acc_count = 0
        self.cov_emas = {}
        self.acc_covs = {}
        self.acc_grads = {}
        self.v = {}
        self.invs = {}
        self.kfgrads = {}

    def covs_of(self, rec):
        if rec.kind == 'linear':
            return [O.linear_A(rec.x, 'b' in rec.params), O.linear_G(rec.gy, self.loss_scale)]
        if rec.kind == 'conv':
            a = rec.attrs
            return [O.conv_A(rec.x, a['ksize'], a['stride'], a['pad'], 'b' in rec.params),
                    O.conv_G(rec.gy, self.loss_scale, diag=a.get('diag', False))]
        return [O.bn_F(rec.x, rec.gy, rec.attrs['eps'], self.loss_scale,
                       'gamma' in rec.params, 'beta' in rec.params)]

    def step(self, records):
        """records: list of LayerRecord of one micro-batch.  Returns True when
        the parameters were updated (last micro-batch of an accumulation)."""
        records = sorted(records, key=lambda r: r.name)
        covs = {r.name: self.covs_of(r) for r in records}
        grads = {(r.name, k): g for r in records for k, g in r.grads.items()}
        if self.acc_iters > 1:
            if self.acc_count == 0:
                self.acc_covs = {}
                self.acc_grads = {}
            for name, c in covs.items():
                self.acc_covs[name] = O.accumulate_covs(self.acc_covs.get(name), c, self.acc_iters)
            for key, g in grads.items():
                self.acc_grads[key] = O.accumulate_grad(self.acc_grads.get(key), g, self.acc_iters)
            self.acc_count += 1
            if self.acc_count < self.acc_iters:
                return False
            self.acc_count = 0
            covs = self.acc_covs
            grads = self.acc_grads
        for r in records:
            emas = O.update_cov_emas(covs[r.name], self.cov_emas.get(r.name), self.decay)
            self.cov_emas[r.name] = emas
            if r.kind == 'bn':
                ng = r.params['gamma'].size if 'gamma' in r.params else None
                nb = r.params['beta'].size if 'beta' in r.params else None
                diagvals = O.bn_diagvals(ng, nb, self.damping, self.stab_coeff)
            else:
                diagvals, _ = O.connection_diagvals(emas[0], emas[1], self.damping, 0.0, self.pi_type)
            invs = O.update_invs(emas, diagvals)
            self.invs[r.name] = invs
            if r.kind == 'bn':
                kg, kb, _ = O.precondition_bn(invs[0], grads.get((r.name, 'gamma')), grads.get((r.name, 'beta')))
                kf = {'gamma': kg, 'beta': kb}
            else:
                kW, kb = O.precondition_conn(invs[0], invs[1], grads[(r.name, 'W')], grads.get((r.name, 'b')))
                kf = {'W': kW, 'b': kb}
            for pname, p in r.params.items():
                g = kf[pname]
                # gradients of a scaled loss carry the scale; the update rule
                # divides the preconditioned gradient back (kfac.py:72-78)
                if self.loss_scale is not None:
                    g = g / np.float32(self.loss_scale)
                self.kfgrads[(r.name, pname)] = g
                key = (r.name, pname)
                if key not in self.v:
                    self.v[key] = np.zeros_like(p)
                O.momentum_update(p, self.v[key], g, self.lr, self.momentum)
        return True
