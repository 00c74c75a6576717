"""Parity of the HIP covariance kernels with the oracle (rel 1e-4, needs the GPU)."""
import numpy as np
import pytest
import torch

from oracle import kfac_oracle as O

pytestmark = pytest.mark.gpu

RTOL = 1e-4   # covariance tolerance of the north-star spec


def rel_err(a, ref):
    """Norm-wise relative error against a float64 reference."""
    ref = ref.astype(np.float64)
    return np.linalg.norm(a.astype(np.float64) - ref) / max(np.linalg.norm(ref), 1e-30)


def check(out, ref):
    out = out.cpu().numpy()
    assert out.shape == ref.shape
    assert rel_err(out, ref) < RTOL
    # element-wise, scaled by the largest entry (cancelling entries can be tiny)
    assert np.max(np.abs(out - ref)) <= RTOL * np.max(np.abs(ref))
    assert np.array_equal(out, out.T), 'factor must be exactly symmetric'


@pytest.mark.parametrize('n,d_in,bias', [(128, 784, True), (128, 1000, True), (32, 2048, True), (7, 5, True),
                                         (1, 3, False), (33, 64, False), (128, 10, False), (40, 321, True),
                                         (128, 4096, True)])
def test_linear_A(n, d_in, bias):
    from chainerkfac_amd import ops
    x = np.random.default_rng(n + d_in).random((n, d_in), dtype=np.float32)
    A = ops.cov_linear(torch.from_numpy(x).cuda(), bias, 1.0 / n)
    check(A, O.linear_A(x, bias))


@pytest.mark.parametrize('n,d_out', [(128, 1000), (128, 10), (32, 1000), (5, 130)])
def test_linear_G(n, d_out):
    from chainerkfac_amd import ops
    gy = (np.random.default_rng(n * d_out).standard_normal((n, d_out)) / n).astype(np.float32)
    G = ops.cov_linear(torch.from_numpy(gy).cuda(), False, float(n) ** 2 / n)
    check(G, O.linear_G(gy))


CONV_CASES = [
    # n, c, h, w, k, s, p, bias
    (2, 3, 8, 8, 3, 1, 1, True),
    (3, 2, 7, 6, 3, 2, 1, True),
    (2, 4, 9, 9, 1, 1, 0, True),        # 1x1: NCHW slab path, 81 pixels (scalar loads)
    (2, 8, 8, 8, 1, 1, 0, False),       # 1x1, vector loads
    (2, 5, 8, 8, 1, 2, 0, True),        # strided 1x1: the slab, subsampled
    (3, 70, 9, 7, 1, 2, 0, True),       # strided 1x1, odd sizes (5x4 outputs), two 64-tiles
    (2, 600, 6, 6, 1, 2, 0, True),      # strided 1x1, 128-tiles
    (2, 40, 9, 9, 1, 3, 0, False),      # stride 3
    (2, 3, 12, 12, 7, 2, 3, True),      # stem-like
    (2, 3, 10, 10, 5, 1, 0, False),
    (4, 3, 32, 32, 3, 1, 1, True),      # CIFAR conv1 shape (28)
    (8, 64, 16, 16, 3, 1, 1, True),     # 577
    (4, 128, 8, 8, 3, 1, 1, True),      # 1153
    (2, 40, 6, 6, 3, 1, 1, False),      # 360: six 64-tiles, the last ragged
    (2, 70, 6, 6, 3, 1, 1, False),      # 630: 128-tiles, ragged fifth, element-gather loader
    (1, 2, 3, 3, 3, 1, 1, True),        # fewer pixels than a panel
    # shapes that take the LDS-staged input-region kernel (d > 520, >= 40 pixels per step)
    (2, 64, 29, 29, 3, 2, 1, True),     # stride 2, 15x15 outputs: 4-row steps hang over the bottom edge
    (2, 24, 14, 14, 5, 1, 2, True),     # 5x5 taps, 14-wide rows, ragged last row group
    (1, 64, 56, 56, 3, 1, 1, True),     # one 56-wide output row per step, four staging passes
    (2, 64, 28, 28, 3, 1, 1, False),    # two 28-wide rows per step, no bias row
    (4, 64, 7, 7, 3, 1, 1, True),       # whole 7x7 image per step (49 of 50 k slots used)
    (1, 60, 20, 112, 3, 1, 1, True),    # rows wider than a step: two column segments
    (2, 12, 38, 38, 7, 2, 3, True),     # 7x7 stride 2, 19x19 outputs
    (3, 130, 9, 9, 3, 1, 0, True),      # no padding, 7x7 outputs, last panel past the channel count
    # shapes that take the compile-time row-geometry kernel (3x3, pad 1, even batch, 56/28/14/7-wide outputs)
    (2, 64, 56, 56, 3, 1, 1, True),     # one output row of a sample pair per step
    (2, 40, 14, 14, 3, 1, 1, True),     # 361: seven rows per step, three tile rows with a ragged last one
    (4, 37, 7, 7, 3, 1, 1, False),      # 333: channel count that ends inside a panel
    (2, 150, 7, 7, 3, 1, 1, True),      # 1351: eleven tile rows, panels that start mid-channel
    (6, 64, 14, 14, 3, 1, 1, True),     # three sample pairs
    (2, 48, 28, 28, 3, 1, 1, True),     # 433
    # the same kernel's other geometries: 112-wide rows, stride 2 (28/14/7-wide outputs), CIFAR widths
    (2, 32, 112, 112, 3, 1, 1, False),  # 288: the stem of ResNet-D, 64-tiles with a ragged fifth
    (2, 30, 112, 112, 3, 1, 1, True),   # 271
    (2, 64, 56, 56, 3, 2, 1, False),    # stride 2, 28-wide outputs, one row per step
    (2, 40, 28, 28, 3, 2, 1, True),     # stride 2, 14-wide outputs, two rows per step
    (4, 64, 14, 14, 3, 2, 1, False),    # stride 2, 7-wide outputs (halo-region kernel)
    (2, 64, 32, 32, 3, 1, 1, True),     # 32-wide rows, two per step
    (2, 3, 224, 224, 7, 2, 3, True),    # 148: the ImageNet stem, 112-wide outputs
]


def takes_shift_route(c, h, w, k, s, p):
    """3x3 / stride 1 / padding 1 with at least 64 channels (or 28..32, with stacked operand tiles):
    computed from shifted correlations of the input unless the option conv_shift = 0 leaves it to
    the patch-product kernels."""
    return k == 3 and s == 1 and p == 1 and (c >= 64 or 28 <= c <= 32) and h >= 4 and w >= 4


@pytest.fixture
def lib_options():
    """Sets tuning options of the library for one test and restores the defaults afterwards."""
    from chainerkfac_amd import _lib
    touched = []

    def set_option(name, value):
        touched.append(name)
        _lib.set_option(name, value)
    yield set_option
    for name in touched:
        _lib.set_option(name, None)


@pytest.fixture
def patch_product_route(lib_options):
    def switch(on):
        lib_options('conv_shift', 0 if on else None)
    return switch


@pytest.mark.parametrize('n,c,h,w,k,s,p,bias', CONV_CASES)
def test_conv_A(n, c, h, w, k, s, p, bias, patch_product_route):
    from chainerkfac_amd import ops
    x = np.random.default_rng(c * h + k).standard_normal((n, c, h, w)).astype(np.float32)
    ref = O.conv_A(x, k, s, p, bias)
    A = ops.cov_conv_a(torch.from_numpy(x).cuda(), k, s, p, bias, 1.0 / n)
    check(A, ref)
    if takes_shift_route(c, h, w, k, s, p):
        # the same shape through the patch-product kernels
        patch_product_route(True)
        B = ops.cov_conv_a(torch.from_numpy(x).cuda(), k, s, p, bias, 1.0 / n)
        patch_product_route(False)
        check(B, ref)
        assert rel_err(A.cpu().numpy(), B.cpu().numpy()) < 1e-5


SHIFT_CASES = [
    # n, c, h, w, bias: 3x3 / 1 / 1 shapes of the shifted-correlation route
    (1, 64, 4, 4, True),        # the smallest image it takes: border strips are half the image
    (3, 64, 5, 9, True),        # odd batch, H != W
    (2, 96, 12, 10, False),     # one 128-tile, a quarter of it padding
    (2, 200, 6, 7, True),       # two 128-tiles per side, the second ragged
    (1, 64, 20, 112, True),     # long image rows
    (2, 64, 56, 56, False),     # 3136 pixels: k-slices that start inside an image
    (2, 256, 14, 14, True),     # four tiles per product
    (5, 130, 7, 7, True),       # channel count just past a tile
    (2, 64, 1000, 4, True),     # tall and narrow: column strips of 1000 pixels
    (2, 1024, 5, 4, False),     # 8 x 16 tiles per product, a reduction shorter than one panel
    # 28..32 channels: stacked tiles (two row shifts x two column offsets of the same 32 channels)
    (2, 32, 112, 112, False),   # ResNet-50-D's stem
    (3, 32, 9, 7, True),        # odd sizes, odd batch
    (2, 30, 16, 16, True),      # fewer than 32 channels
    (1, 28, 4, 4, True),
]


@pytest.mark.parametrize('n,c,h,w,bias', SHIFT_CASES)
def test_conv_A_shift_route(n, c, h, w, bias):
    from chainerkfac_amd import ops
    assert takes_shift_route(c, h, w, 3, 1, 1)
    x = np.random.default_rng(c + h * w).standard_normal((n, c, h, w)).astype(np.float32)
    x += 0.5    # non-zero mean: the ones column is not just noise
    A = ops.cov_conv_a(torch.from_numpy(x).cuda(), 3, 1, 1, bias, 1.0 / n)
    check(A, O.conv_A(x, 3, 1, 1, bias))


def test_conv_A_shift_route_unaligned_input_and_accumulation():
    """An input that starts one float past a 16-byte boundary (a view into a larger buffer), and
    beta = 1 accumulation onto an existing factor with its ones row and column."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(11)
    n, c, h, w = 2, 64, 8, 12
    buf = torch.zeros(n * c * h * w + 1, device='cuda')
    xs = [r.standard_normal((n, c, h, w)).astype(np.float32) + 0.25 for _ in range(2)]
    out = None
    acc = None
    for i, x in enumerate(xs):
        buf[1:].copy_(torch.from_numpy(x).reshape(-1))
        xv = buf[1:].view(n, c, h, w)
        assert xv.data_ptr() % 16 == 4
        out = ops.cov_conv_a(xv, 3, 1, 1, True, (1.0 / n) / 2, beta=0.0 if i == 0 else 1.0, out=out)
        acc = O.accumulate_covs(acc, [O.conv_A(x, 3, 1, 1, True)], 2)
    check(out, acc[0])


@pytest.mark.parametrize('n,c,h,w', [(32, 64, 56, 56), (32, 128, 28, 28), (8, 256, 14, 14), (4, 512, 7, 7),
                                     (2, 64, 4, 200), (3, 96, 9, 5)])
def test_workspace_query_covers_the_shift_route(n, c, h, w, lib_options):
    """A workspace of exactly kfac_cov_workspace_bytes(d, rows) is enough for the shifted-correlation
    route (with the option conv_shift_strict a workspace that is too small for it is an error instead
    of a silent change of route)."""
    from chainerkfac_amd import _lib, device as _dev
    lib = _lib.load()
    lib_options('conv_shift_strict', 1)
    d = 9 * c + 1
    nbytes = lib.kfac_cov_workspace_bytes(d, n * h * w)
    ws = torch.empty(nbytes, dtype=torch.uint8, device='cuda')
    x = torch.randn(n, c, h, w, device='cuda')
    out = torch.empty(d, d, device='cuda')
    _lib.check(lib.kfac_cov_conv_a_f32(x.data_ptr(), n, c, h, w, 3, 3, 1, 1, 1, 1, 1, 1.0 / n, 0.0, out.data_ptr(),
                                       ws.data_ptr(), nbytes, _dev.stream_handle(None)))
    torch.cuda.synchronize()
    # and one byte less than the route's tail is refused in strict mode
    with pytest.raises(Exception):
        _lib.check(lib.kfac_cov_conv_a_f32(x.data_ptr(), n, c, h, w, 3, 3, 1, 1, 1, 1, 1, 1.0 / n, 0.0,
                                           out.data_ptr(), ws.data_ptr(), 1024, _dev.stream_handle(None)))


def test_conv_A_shift_route_random_shapes():
    """Seeded random geometries of the shifted-correlation route (both tile modes, ragged channel
    counts, images from 4 x 4 up, reductions shorter and longer than a panel, with and without the
    ones column) against the oracle."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(2024)
    for _ in range(40):
        c = int(r.integers(28, 33)) if r.random() < 0.3 else int(r.integers(64, 200))
        n, h, w = int(r.integers(1, 6)), int(r.integers(4, 24)), int(r.integers(4, 24))
        bias = bool(r.integers(0, 2))
        assert takes_shift_route(c, h, w, 3, 1, 1)
        x = (r.standard_normal((n, c, h, w)) + r.standard_normal()).astype(np.float32)
        A = ops.cov_conv_a(torch.from_numpy(x).cuda(), 3, 1, 1, bias, 1.0 / n)
        try:
            check(A, O.conv_A(x, 3, 1, 1, bias))
        except AssertionError as e:
            raise AssertionError('shape n={} c={} h={} w={} bias={}: {}'.format(n, c, h, w, bias, e))


def test_conv_A_shift_route_border_terms():
    """An input that is zero except on the image border and corners: every entry of the factor is
    then made of the border corrections (row / column strips and corner pixels) alone."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(3)
    x = np.zeros((2, 64, 6, 8), np.float32)
    x[:, :, 0, :] = r.standard_normal((2, 64, 8))
    x[:, :, -1, :] = r.standard_normal((2, 64, 8))
    x[:, :, :, 0] = r.standard_normal((2, 64, 6))
    x[:, :, :, -1] = r.standard_normal((2, 64, 6))
    A = ops.cov_conv_a(torch.from_numpy(x).cuda(), 3, 1, 1, True, 0.5)
    check(A, O.conv_A(x, 3, 1, 1, True))


@pytest.mark.parametrize('n,c,ho,wo', [(2, 5, 3, 3), (4, 64, 16, 16), (3, 130, 7, 7), (2, 256, 4, 4),
                                       (128, 64, 32, 32), (2, 700, 2, 2)])
def test_conv_G(n, c, ho, wo):
    from chainerkfac_amd import ops
    gy = (np.random.default_rng(c + ho).standard_normal((n, c, ho, wo)) / n).astype(np.float32)
    G = ops.cov_conv_g(torch.from_numpy(gy).cuda(), float(n) ** 2 / (n * ho * wo))
    check(G, O.conv_G(gy))


def test_running_accumulation_matches_mean_of_covs():
    """beta = 1, alpha = scale/acc_iters reproduces KFAC.accumulate_covs."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(0)
    acc_iters = 4
    xs = [r.standard_normal((2, 6, 8, 8)).astype(np.float32) for _ in range(acc_iters)]
    acc = None
    out = None
    for i, x in enumerate(xs):
        acc = O.accumulate_covs(acc, [O.conv_A(x, 3, 1, 1, True)], acc_iters)
        out = ops.cov_conv_a(torch.from_numpy(x).cuda(), 3, 1, 1, True, (1.0 / 2) / acc_iters,
                             beta=0.0 if i == 0 else 1.0, out=out)
    check(out, acc[0])


@pytest.mark.parametrize('shape', ['conv3x3_region', 'conv1x1_slab', 'linear'])
def test_accumulation_with_ones_column(shape):
    """beta != 0 on the ones row/column and the corner entry, for the kernels that keep the ones column
    outside the tile grid (k-sliced and single-slice epilogues)."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(5)
    acc = None
    out = None
    for i in range(3):
        if shape == 'conv3x3_region':      # d = 577, 2048 pixels: several k-slices + finish kernel
            x = r.standard_normal((8, 64, 16, 16)).astype(np.float32)
            ref = O.conv_A(x, 3, 1, 1, True)
            run = lambda b, o: ops.cov_conv_a(torch.from_numpy(x).cuda(), 3, 1, 1, True, (1.0 / 8) / 3, beta=b, out=o)
        elif shape == 'conv1x1_slab':      # d = 41, odd pixel count: scalar slab loader
            x = r.standard_normal((4, 40, 7, 7)).astype(np.float32)
            ref = O.conv_A(x, 1, 1, 0, True)
            run = lambda b, o: ops.cov_conv_a(torch.from_numpy(x).cuda(), 1, 1, 0, True, (1.0 / 4) / 3, beta=b, out=o)
        else:                              # one 32-row panel: written straight from registers
            x = r.random((16, 200), dtype=np.float32)
            ref = O.linear_A(x, True)
            run = lambda b, o: ops.cov_linear(torch.from_numpy(x).cuda(), True, (1.0 / 16) / 3, b, o)
        acc = O.accumulate_covs(acc, [ref], 3)
        out = run(0.0 if i == 0 else 1.0, out)
    check(out, acc[0])
    got = out.cpu().numpy()
    assert np.array_equal(got, got.T)
    assert abs(got[-1, -1] - acc[0][-1, -1]) <= 1e-6 * abs(acc[0][-1, -1])


def test_grouped_launch_matches_the_single_calls():
    """One grouped launch for a mixed list of small factors (convolution G, 1x1 convolution A
    with and without a ones column, strided 1x1, odd pixel counts, linear layers, a batch-norm
    gradient matrix; with and without accumulation onto an existing factor) against the
    oracle, and against the single-call entry points."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(17)

    def t(*shape):
        return torch.from_numpy(r.standard_normal(shape).astype(np.float32)).cuda()

    cases = [
        # kind, input, ones, stride, alpha, beta
        (ops.COV_SLAB, t(4, 64, 14, 14), False, 1, 0.25, 0.0),      # G, 64: one tile, float4 loads
        (ops.COV_SLAB, t(4, 65, 14, 14), True, 1, 0.25, 0.0),       # 1x1 A with ones, 66: ragged second tile
        (ops.COV_SLAB, t(2, 130, 7, 7), True, 1, 0.5, 0.0),         # 49 pixels: scalar loads
        (ops.COV_SLAB, t(2, 96, 9, 7), True, 2, 0.5, 0.0),          # strided 1x1: every 2nd line / pixel
        (ops.COV_SLAB, t(3, 200, 6, 6), False, 1, 1.0, 1.0),        # accumulates onto an existing factor
        (ops.COV_SLAB, t(8, 32, 56, 56), False, 1, 0.125, 0.0),     # long reduction: several k-slices
        (ops.COV_LINEAR, t(32, 256), False, 1, 1 / 32, 0.0),        # batch-norm gradient matrix
        (ops.COV_LINEAR, t(16, 101), True, 1, 1 / 16, 1.0),         # linear A with ones, odd width
        (ops.COV_LINEAR, t(128, 10), False, 1, 128.0, 0.0),         # linear G
        (ops.COV_SLAB, t(4, 600, 8, 8), False, 1, 0.25, 0.0),       # 128-tiles, float4 loads
        (ops.COV_SLAB, t(6, 530, 7, 7), True, 1, 0.5, 1.0),         # 128-tiles, scalar loads, ones, accumulation
        (ops.COV_LINEAR, t(200, 600), True, 1, 0.005, 0.0),         # 128-tiles, linear with ones
    ]
    pending = ops.PendingCovs()
    outs, refs, singles = [], [], []
    for kind, x, ones, stride, alpha, beta in cases:
        d = x.shape[1] + int(ones)
        prev = t(d, d)
        prev = (prev + prev.T).contiguous()
        out = prev.clone()
        xs = x.cpu().numpy()
        if kind == ops.COV_SLAB:
            sub = xs[:, :, ::stride, ::stride]
            P = sub.transpose(0, 2, 3, 1).reshape(-1, xs.shape[1]).astype(np.float64)
            single = ops.cov_conv_a(x, 1, stride, 0, ones, alpha, beta, prev.clone())
        else:
            P = xs.astype(np.float64)
            single = ops.cov_linear(x, ones, alpha, beta, prev.clone())
        if ones:
            P = np.concatenate([P, np.ones((P.shape[0], 1))], axis=1)
        refs.append(alpha * (P.T @ P) + beta * prev.cpu().numpy().astype(np.float64))
        pending.add(kind, x, ones, out, alpha, beta, stride)
        outs.append(out)
        singles.append(single)
    assert [o.shape[0] for o in outs] == [64, 66, 131, 97, 200, 32, 256, 102, 10, 600, 531, 601]
    pending.flush()
    torch.cuda.synchronize()
    assert pending.items == []
    for out, ref, single in zip(outs, refs, singles):
        got = out.cpu().numpy()
        assert np.linalg.norm(got - ref) <= 1e-4 * np.linalg.norm(ref)
        assert np.array_equal(got, got.T)
        assert np.linalg.norm(got - single.cpu().numpy()) <= 1e-5 * np.linalg.norm(ref)
    # the oracle's own functions on two of them
    x = cases[1][1].cpu().numpy()
    np.testing.assert_allclose(outs[1].cpu().numpy(), O.conv_A(x, 1, 1, 0, True) * (0.25 * 4), rtol=1e-4, atol=1e-4)
    gy = cases[0][1].cpu().numpy()
    np.testing.assert_allclose(outs[0].cpu().numpy(), O.conv_G(gy) * (0.25 * 14 * 14 / 4), rtol=1e-4, atol=1e-4)


def test_grouped_launch_macro_tiles(lib_options):
    """With the option group_macro = 1 (read when a group is created), slabs of several 128-tiles with
    a long reduction take the macro-tile kernel (four teams
    per workgroup, 2 x 2 tiles from four panels staged once): an even and an odd number of
    tiles, a ragged last tile, 16-byte and scalar loads, a ones column, accumulation; against
    float64 and the single-call entry point."""
    from chainerkfac_amd import ops
    lib_options('group_macro', 1)
    r = np.random.default_rng(29)

    def t(*shape):
        return torch.from_numpy(r.standard_normal(shape).astype(np.float32)).cuda()

    cases = [
        # input, ones, stride, alpha, beta
        (t(8, 256, 28, 28), False, 1, 1.0 / 8, 0.0),     # 2 tiles: one macro-tile on the diagonal
        (t(4, 384, 28, 28), True, 1, 0.25, 0.0),         # 3 tiles: ragged last macro row, ones column
        (t(6, 500, 20, 20), True, 1, 0.5, 1.0),          # 4 tiles, ragged last tile, accumulation
        (t(8, 272, 15, 15), True, 1, 0.125, 0.0),        # 225 pixels: scalar loads
        (t(4, 300, 30, 30), False, 2, 0.25, 0.0),        # strided 1x1: scalar loads, 3 tiles
        (t(2, 1024, 16, 16), False, 1, 0.5, 0.0),        # 8 tiles: 10 macro-tiles per slice
    ]
    pending = ops.PendingCovs()
    outs, refs, singles = [], [], []
    for x, ones, stride, alpha, beta in cases:
        d = x.shape[1] + int(ones)
        prev = t(d, d)
        prev = (prev + prev.T).contiguous()
        out = prev.clone()
        sub = x.cpu().numpy()[:, :, ::stride, ::stride]
        P = sub.transpose(0, 2, 3, 1).reshape(-1, x.shape[1]).astype(np.float64)
        if ones:
            P = np.concatenate([P, np.ones((P.shape[0], 1))], axis=1)
        refs.append(alpha * (P.T @ P) + beta * prev.cpu().numpy().astype(np.float64))
        singles.append(ops.cov_conv_a(x, 1, stride, 0, ones, alpha, beta, prev.clone()))
        pending.add(ops.COV_SLAB, x, ones, out, alpha, beta, stride)
        outs.append(out)
    pending.flush()
    torch.cuda.synchronize()
    for out, ref, single in zip(outs, refs, singles):
        got = out.cpu().numpy()
        assert np.isfinite(got).all()
        assert np.linalg.norm(got - ref) <= 1e-4 * np.linalg.norm(ref)
        assert np.array_equal(got, got.T)
        assert np.linalg.norm(got - single.cpu().numpy()) <= 1e-5 * np.linalg.norm(ref)


def test_grouped_launch_alternating_arguments_under_capture():
    """Accumulation calls one group with beta = 0, then beta = 1: both argument tables stay
    resident, so a graph can be captured over the pair after one eager pass, and every
    replay gives the eager result.  An argument set that is not resident is refused inside a
    capture instead of silently uploading."""
    from chainerkfac_amd import _lib, ops
    r = np.random.default_rng(23)
    xs = [torch.from_numpy(r.standard_normal(s).astype(np.float32)).cuda()
          for s in [(4, 64, 14, 14), (16, 101)]]
    items = [(ops.COV_SLAB, 4, 64, 14, 14, 1, 1, 0, 1), (ops.COV_LINEAR, 16, 101, 1, 1, 1, 1, 1, 1)]
    outs = [torch.empty(64, 64, device='cuda'), torch.empty(102, 102, device='cuda')]
    group = ops.CovGroup(items)

    def pair():
        group.run(xs, outs, [0.5, 0.25], [0.0, 0.0])
        group.run(xs, outs, [0.5, 0.25], [1.0, 1.0])

    pair()
    torch.cuda.synchronize()
    want = [o.clone() for o in outs]
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            pair()
    for _ in range(3):
        for o in outs:
            o.fill_(float('nan'))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for o, w in zip(outs, want):
            assert torch.equal(o, w)
    P = xs[1].cpu().numpy().astype(np.float64)
    P = np.concatenate([P, np.ones((16, 1))], axis=1)
    np.testing.assert_allclose(outs[1].cpu().numpy(), 0.5 * (P.T @ P), rtol=1e-4, atol=1e-4)
    # a table the group has not seen cannot be uploaded while capturing
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph2, stream=side):
            with pytest.raises(_lib.KfacHipError):
                group.run(xs, outs, [0.125, 0.25], [0.0, 0.0])
            group.run(xs, outs, [0.5, 0.25], [0.0, 0.0])
    graph2.replay()
    torch.cuda.synchronize()
    np.testing.assert_allclose(outs[1].cpu().numpy(), 0.25 * (P.T @ P), rtol=1e-4, atol=1e-4)


def test_grouped_launch_argument_checks():
    from chainerkfac_amd import _lib, ops
    with pytest.raises(_lib.KfacHipError):
        ops.CovGroup([(7, 2, 3, 1, 1, 1, 1, 0, 1)])            # unknown kind
    g = ops.CovGroup([(ops.COV_LINEAR, 4, 8, 1, 1, 1, 1, 0, 1)])
    x = torch.zeros(4, 8, device='cuda')
    with pytest.raises(ValueError):
        g.run([x], [torch.zeros(9, 9, device='cuda')], [1.0], [0.0])
    assert ops.CovGroup([]).run([], [], [], []) == []


def test_workspace_too_small_is_reported():
    import ctypes
    from chainerkfac_amd import _lib
    lib = _lib.load()
    x = torch.zeros(4, 8, device='cuda')
    C = torch.zeros(8, 8, device='cuda')
    rc = lib.kfac_cov_linear_f32(x.data_ptr(), 4, 8, 0, 1.0, 0.0, C.data_ptr(), None, 0, None)
    assert rc == -3 and b'workspace' in lib.kfac_last_error_string()
    rc = lib.kfac_cov_linear_f32(x.data_ptr(), 0, 8, 0, 1.0, 0.0, C.data_ptr(), None, 0, None)
    assert rc == -1


def _conv_block(c_in, c_out, k, diag=False, diagonalize=False):
    from chainerkfac_amd import links as L
    from chainerkfac_amd.optimizers import fisher_blocks as FB
    link = L.Convolution2D(c_in, c_out, k, 1, k // 2, device='cuda')
    if diag:
        link.diag = True
    fb = FB.FisherBlockConvolution2D('/conv', link, cov_ema_decay=1.0, damping=1e-3)
    fb.diagonalize = diagonalize
    return link, fb


@pytest.mark.parametrize('kw', [{'diag': True}, {'diagonalize': True}])
def test_conv_G_diagonal_branches(kw):
    """``link.diag`` and the block's ``diagonalize``: G = diag(diag(G)), still a matrix, also when
    the factor is accumulated over micro-batches (reference convolution_2d.py:56-70)."""
    from chainerkfac_amd import links as L
    r = np.random.default_rng(31)
    link, fb = _conv_block(6, 40, 3, **kw)
    x = torch.from_numpy(r.standard_normal((4, 6, 9, 9)).astype(np.float32)).cuda()
    gys = [(r.standard_normal((4, 40, 9, 9)) / 4).astype(np.float32) for _ in range(2)]
    func = L.Convolution2DFunction()
    fb.forward_postprocess(func, (x, link.W.data, link.b.data))
    fb.backward_preprocess(func, (x, link.W.data, link.b.data), (torch.from_numpy(gys[0]).cuda(),))
    G = fb.covs[1].cpu().numpy()
    assert G.shape == (40, 40) and np.count_nonzero(G - np.diag(np.diag(G))) == 0
    np.testing.assert_allclose(G, O.conv_G(gys[0], **kw), rtol=1e-4, atol=1e-7)
    # two micro-batches: the mean of the two diagonal factors
    acc = None
    for i, gy in enumerate(gys):
        fb.acc_state = (2, i)
        fb.backward_preprocess(func, (x, link.W.data, link.b.data), (torch.from_numpy(gy).cuda(),))
        acc = O.accumulate_covs(acc, [O.conv_G(gy, **kw)], 2)
    G = fb.covs[1].cpu().numpy()
    assert np.count_nonzero(G - np.diag(np.diag(G))) == 0
    np.testing.assert_allclose(G, acc[0], rtol=1e-4, atol=1e-7)


def test_linear_and_batchnorm_diagonalize():
    """``diagonalize`` on the other blocks: the linear A factor becomes a vector, G and the
    batch-norm factor diagonal matrices (reference linear.py:25,43-44, batch_normalization.py:121-124),
    and the batch-norm block no longer offers its low-rank inverse."""
    from chainerkfac_amd import links as L
    from chainerkfac_amd.optimizers import fisher_blocks as FB
    r = np.random.default_rng(32)
    lin = L.Linear(33, 20, device='cuda')
    fb = FB.FisherBlockLinear('/fc', lin, cov_ema_decay=1.0, damping=1e-3)
    fb.diagonalize = True
    x = r.standard_normal((16, 33)).astype(np.float32)
    gy = (r.standard_normal((16, 20)) / 16).astype(np.float32)
    func = L.LinearFunction()
    in_data = (torch.from_numpy(x).cuda(), lin.W.data, lin.b.data)
    fb.forward_postprocess(func, in_data)
    fb.backward_preprocess(func, in_data, (torch.from_numpy(gy).cuda(),))
    A, G = (c.cpu().numpy() for c in fb.covs)
    assert A.shape == (34,) and G.shape == (20, 20)
    np.testing.assert_allclose(A, O.linear_A(x, True, diagonalize=True), rtol=1e-4)
    np.testing.assert_allclose(G, O.linear_G(gy, diagonalize=True), rtol=1e-4, atol=1e-7)
    bn = L.BatchNormalization(12, device='cuda')
    fbn = FB.FisherBlockBatchNormalization('/bn', bn, cov_ema_decay=1.0, damping=1e-3)
    fbn.diagonalize = True
    xb = r.standard_normal((8, 12, 5, 5)).astype(np.float32)
    gb = (r.standard_normal((8, 12, 5, 5)) / 8).astype(np.float32)
    fbn.backward_preprocess(L.BatchNormalizationFunction(), (torch.from_numpy(xb).cuda(), bn.gamma.data, bn.beta.data),
                            (torch.from_numpy(gb).cuda(),))
    F = fbn.covs[0].cpu().numpy()
    assert np.count_nonzero(F - np.diag(np.diag(F))) == 0
    np.testing.assert_allclose(F, O.bn_F(xb, gb, bn.eps, diagonalize=True), rtol=1e-4, atol=1e-7)
    fbn.update_cov_emas()
    assert fbn.lowrank_inverse_args() is None


@pytest.mark.parametrize('n,c,h,w', [(32, 64, 56, 56), (32, 128, 28, 28), (32, 256, 14, 14), (32, 512, 7, 7),
                                     (32, 32, 112, 112)])
def test_resnet_3x3_shapes_take_the_shift_route(n, c, h, w):
    """The 3x3 convolutions of ResNet-50 (and the 32-channel stem convolution of ResNet-50-D, with
    stacked tiles) are computed from shifted correlations when called the way the benchmark calls
    them: through ``ops.cov_conv_a`` with the workspace ``kfac_cov_workspace_bytes`` reports.  A
    workspace that is too small sends them to the patch-product kernels without an error, so the
    route is read back from the library."""
    from chainerkfac_amd import _lib, ops
    lib = _lib.load()
    x = torch.randn(n, c, h, w, device='cuda')
    A = ops.cov_conv_a(x, 3, 1, 1, True, 1.0 / n)
    assert lib.kfac_cov_conv_a_last_route() == 1      # KFAC_CONV_ROUTE_SHIFT
    assert torch.equal(A, A.T)
    # the same call with the route switched off lands on the rows kernels
    with _lib.options(conv_shift=0):
        ops.cov_conv_a(x, 3, 1, 1, True, 1.0 / n)
    assert lib.kfac_cov_conv_a_last_route() == 2      # KFAC_CONV_ROUTE_ROWS
    # other geometries report their own routes
    ops.cov_conv_a(torch.randn(2, 16, 9, 9, device='cuda'), 1, 1, 0, True, 0.5)
    assert lib.kfac_cov_conv_a_last_route() == 0      # KFAC_CONV_ROUTE_SLAB
    torch.cuda.synchronize()
