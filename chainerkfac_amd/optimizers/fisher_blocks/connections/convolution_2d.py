"""Fisher block of a Convolution2D layer.  A is the Gram matrix of the im2col
patches (columns (c, kh, kw) then ones), scaled by 1/n; G the Gram matrix of the
output gradients over samples and pixels.  The patch matrix is formed inside
the SYRK kernel.  Counterpart of
chainerkfac/optimizers/fisher_blocks/connections/convolution_2d.py."""
from chainerkfac_amd import links
from chainerkfac_amd import ops
from chainerkfac_amd.optimizers.fisher_block import as_float32
from chainerkfac_amd.optimizers.fisher_blocks.connection import FisherBlockConnection


class FisherBlockConvolution2D(FisherBlockConnection):

    @property
    def funcclass(self):
        return links.Convolution2DFunction

    def compute_A(self, in_data):
        x = as_float32(in_data[0])
        link = self.link
        ksize, stride, pad = link.ksize, link.stride[0], link.pad[0]
        n, c = x.shape[0], x.shape[1]
        has_b = link.b is not None
        d = c * ksize * ksize + (1 if has_b else 0)
        out, alpha, beta = self._cov_target('A', (d, d), x.device, 1.0 / n)
        if ksize == 1 and pad == 0:
            # a 1x1 convolution's patch matrix is the (subsampled) NCHW tensor itself
            ho, wo = (x.shape[2] - 1) // stride + 1, (x.shape[3] - 1) // stride + 1
            if self._defer_cov(ops.COV_SLAB, x, has_b, n * ho * wo, out, alpha, beta, stride):
                return out
        return self._on_lane(lambda: ops.cov_conv_a(x, ksize, stride, pad, has_b, alpha, beta, out), (x,))

    def compute_G(self, in_data, out_grad_data):
        gy = as_float32(out_grad_data[0])
        n, c, ho, wo = gy.shape
        scale = self.gy_scale(n) ** 2 / (n * ho * wo)
        out, alpha, beta = self._cov_target('G', (c, c), gy.device, scale)
        if self.diagonalize or getattr(self.link, 'diag', False):
            # G = diag(diag(G)), still a c x c matrix (reference convolution_2d.py:57-62, :68-70)
            def diagonal_factor():
                ops.cov_conv_g(gy, alpha, beta, out)
                ops.keep_diag(out)
            self._on_lane(diagonal_factor, (gy,))
            return out
        if self._defer_cov(ops.COV_SLAB, gy, False, n * ho * wo, out, alpha, beta):
            return out
        return self._on_lane(lambda: ops.cov_conv_g(gy, alpha, beta, out), (gy,))
