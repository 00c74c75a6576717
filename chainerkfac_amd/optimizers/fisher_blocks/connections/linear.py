"""Fisher block of a Linear layer: A = [x, 1]^T [x, 1] / n, G = n * gy^T gy.
Counterpart of chainerkfac/optimizers/fisher_blocks/connections/linear.py."""
from chainerkfac_amd import links
from chainerkfac_amd import ops
from chainerkfac_amd.optimizers.fisher_block import as_float32
from chainerkfac_amd.optimizers.fisher_blocks.connection import FisherBlockConnection


class FisherBlockLinear(FisherBlockConnection):

    @property
    def funcclass(self):
        return links.LinearFunction

    def compute_A(self, in_data):
        x = as_float32(in_data[0])
        n, d_in = x.shape
        has_b = self.link.b is not None
        d = d_in + (1 if has_b else 0)
        out, alpha, beta = self._cov_target('A', (d, d), x.device, 1.0 / n)
        if self.diagonalize:
            # A = mean(x^2, axis 0), a vector (reference linear.py:25): the diagonal of the
            # matrix factor (with accumulation the matrix buffer carries the running sum)
            vec = self._buffer('A_diag', (d,), x.device)

            def diagonal_factor():
                ops.cov_linear(x, has_b, alpha, beta, out)
                vec.copy_(out.diagonal())
            self._on_lane(diagonal_factor, (x,))
            return vec
        if self._defer_cov(ops.COV_LINEAR, x, has_b, n, out, alpha, beta):
            return out
        return self._on_lane(lambda: ops.cov_linear(x, has_b, alpha, beta, out), (x,))

    def compute_G(self, in_data, out_grad_data):
        gy = as_float32(out_grad_data[0])
        n, d_out = gy.shape
        scale = self.gy_scale(n) ** 2 / n
        out, alpha, beta = self._cov_target('G', (d_out, d_out), gy.device, scale)
        if self.diagonalize:
            # G = diag(mean(gy'^2, axis 0)), a matrix (reference linear.py:43-44)
            def diagonal_factor():
                ops.cov_linear(gy, False, alpha, beta, out)
                ops.keep_diag(out)
            self._on_lane(diagonal_factor, (gy,))
            return out
        if self._defer_cov(ops.COV_LINEAR, gy, False, n, out, alpha, beta):
            return out
        return self._on_lane(lambda: ops.cov_linear(gy, False, alpha, beta, out), (gy,))
