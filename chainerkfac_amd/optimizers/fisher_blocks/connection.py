"""Fisher block of a connection layer (Linear / Convolution2D): two Kronecker
factors A (inputs) and G (output gradients).  Counterpart of the reference's
chainerkfac/optimizers/fisher_blocks/connection.py."""
from chainerkfac_amd import ops
from chainerkfac_amd.optimizers.fisher_block import FisherBlock
from chainerkfac_amd.optimizers.fisher_block import as_float32
from chainerkfac_amd.optimizers.fisher_block import PI_TYPE_TRACENORM


class FisherBlockConnection(FisherBlock):

    def __init__(self, *args, **kwargs):
        self._A = None
        self._G = None
        self.pi = None
        super(FisherBlockConnection, self).__init__(*args, **kwargs)

    @property
    def cov_forward(self):
        return self.covs[0]

    @property
    def cov_backward(self):
        return self.covs[1]

    @property
    def inv_forward(self):
        return self.invs[0]

    @property
    def inv_backward(self):
        return self.invs[1]

    def is_mine(self, func, in_data, out_grad_data=None):
        if not isinstance(func, self.funcclass):
            return False
        if in_data[1] is not self.link.W.data:
            return False
        return True

    def forward_postprocess(self, func, in_data):
        self._A = self.compute_A(in_data)
        self.covs = [self._A, self._G]

    def backward_preprocess(self, func, in_data, out_grad_data):
        self._G = self.compute_G(in_data, out_grad_data)
        self.covs = [self._A, self._G]

    def compute_A(self, in_data):
        raise NotImplementedError

    def compute_G(self, in_data, out_grad_data):
        raise NotImplementedError

    def gy_scale(self, n):
        """Factor that undoes the 1/n of a mean-reduced loss (and the loss scale)."""
        s = float(n)
        if self._loss_scale is not None:
            s *= 1.0 / self._loss_scale
        return s

    # damping: pi * sqrt(r) on A, sqrt(r) / pi on G (reference connection.py:66-77)
    def _rW(self):
        return self.get_diagval('W') ** 0.5

    def damp(self):
        A, G = self.cov_emas
        self.pi = ops.pi_damp_batched([A], [G], [self._rW()],
                                      use_pi=self._pi_type == PI_TYPE_TRACENORM)

    def get_diagvals(self):
        """The two float64 diagonal vectors the damping adds, evaluated from the
        current (undamped) ``cov_emas``; copies pi to the host."""
        import numpy as np
        from chainerkfac_amd.optimizers.fisher_block import compute_pi
        A, G = self.cov_emas
        rW = self._rW()
        pi = compute_pi(A, G, self._pi_type)
        pi = np.float32(pi.item() if hasattr(pi, 'item') else pi)
        setattr(self, 'diag_val_forward', pi * rW)
        setattr(self, 'diag_val_backward', (1 / pi) * rW)
        return [pi * (rW * np.ones(A.shape[0])), (1 / pi) * (rW * np.ones(G.shape[0]))]

    def kfgrad_operands(self):
        """``(G_inv, A_inv, gradW, gradb, kfW, kfb)`` of the preconditioning products, with
        the output buffers this block keeps; publishes them as ``W.kfgrad`` / ``b.kfgrad``."""
        self.check_attr('invs')
        W = self.link.W
        b = self.link.b
        A_inv, G_inv = self.invs
        kfW = self._buffer('kfW', W.shape, W.data.device)
        kfb = None if b is None else self._buffer('kfb', b.shape, b.data.device)
        W.kfgrad = kfW
        if b is not None:
            b.kfgrad = kfb
        gW = as_float32(W.grad)
        gW = gW if gW.is_contiguous() else gW.contiguous()
        gb = None if b is None else as_float32(b.grad)
        gb = None if gb is None else (gb if gb.is_contiguous() else gb.contiguous())
        return G_inv, A_inv, gW, gb, kfW, kfb

    def finish_kfgrads(self):
        """After the products: ``kfgrad`` in the gradient's own type when that is
        float16 (reference linear.py:55-61, convolution_2d.py:84-90)."""
        for param in (self.link.W, self.link.b):
            if param is not None and param.kfgrad is not None and param.kfgrad.dtype != param.grad.dtype:
                param.kfgrad = param.kfgrad.to(param.grad.dtype)

    def update_kfgrads(self):
        ops.precond_conn(*self.kfgrad_operands())
        self.finish_kfgrads()

    def compute_kfgrads(self, W, b, invs):
        """(G^-1 [dW | db]) A^-1 as one (c_out, dA) matrix, for callers that want
        the unsplit result like the reference's compute_kfgrads."""
        import torch
        A_inv, G_inv = invs
        kfW, kfb = ops.precond_conn(G_inv, A_inv, W.grad, None if b is None else b.grad)
        kf = kfW.reshape(kfW.shape[0], -1)
        return kf if kfb is None else torch.cat([kf, kfb[:, None]], dim=1)
