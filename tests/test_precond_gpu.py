"""Parity of preconditioning, batch-norm statistics and the update rule with the oracle (GPU)."""
import numpy as np
import pytest
import torch

from oracle import kfac_oracle as O

pytestmark = pytest.mark.gpu

RTOL = 1e-3   # preconditioned-gradient tolerance of the north-star spec


def sym(d, seed):
    r = np.random.default_rng(seed)
    X = r.standard_normal((d, d)).astype(np.float32)
    return ((X + X.T) / np.float32(2 * np.sqrt(d))).astype(np.float32)


def rel(a, b):
    return np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30)


@pytest.mark.parametrize('dG,wshape,bias', [(10, (10, 1000), True), (1000, (1000, 784), True), (64, (64, 3, 3, 3), True),
                                             (128, (128, 64, 3, 3), True), (256, (256, 128, 1, 1), False),
                                             (5, (5, 3), True), (1, (1, 1), False), (130, (130, 70), False),
                                             (512, (512, 64, 3, 3), False)])
def test_precondition_connection(dG, wshape, bias):
    from chainerkfac_amd import ops
    r = np.random.default_rng(dG)
    dA = int(np.prod(wshape[1:])) + (1 if bias else 0)
    Ainv = sym(dA, 1); Ginv = sym(dG, 2)
    gW = r.standard_normal(wshape).astype(np.float32)
    gb = r.standard_normal(dG).astype(np.float32) if bias else None
    kW, kb = O.precondition_conn(Ainv, Ginv, gW, gb)
    hW, hb = ops.precond_conn(torch.from_numpy(Ginv).cuda(), torch.from_numpy(Ainv).cuda(),
                              torch.from_numpy(gW).cuda(), None if gb is None else torch.from_numpy(gb).cuda())
    assert tuple(hW.shape) == wshape
    assert rel(hW.cpu().numpy(), kW) < RTOL
    ref64 = (Ginv.astype(np.float64) @ np.column_stack([gW.reshape(dG, -1)] + ([gb] if bias else [])).astype(np.float64)
             @ Ainv.astype(np.float64))
    got = np.column_stack([hW.cpu().numpy().reshape(dG, -1)] + ([hb.cpu().numpy()] if bias else []))
    assert rel(got, ref64) < 1e-5
    if bias:
        assert hb.shape == (dG,) and rel(hb.cpu().numpy(), kb) < RTOL
    else:
        assert hb is None


def test_precondition_identity_returns_gradient():
    from chainerkfac_amd import ops
    g = torch.randn(7, 12, device='cuda'); b = torch.randn(7, device='cuda')
    kW, kb = ops.precond_conn(torch.eye(7, device='cuda'), torch.eye(13, device='cuda'), g, b)
    assert torch.equal(kW, g) and torch.equal(kb, b)


@pytest.mark.parametrize('C', [3, 64, 1024])
def test_precondition_bn_and_nan_fallback(C):
    from chainerkfac_amd import ops
    r = np.random.default_rng(C)
    Finv = sym(2 * C, 5)
    gg = r.standard_normal(C).astype(np.float32); gb = r.standard_normal(C).astype(np.float32)
    kg, kb, _ = O.precondition_bn(Finv, gg, gb)
    hg, hb, flag = ops.precond_bn(torch.from_numpy(Finv).cuda(), torch.from_numpy(gg).cuda(), torch.from_numpy(gb).cuda())
    assert flag.item() == 0
    assert rel(hg.cpu().numpy(), kg) < RTOL and rel(hb.cpu().numpy(), kb) < RTOL
    Fbad = Finv.copy(); Fbad[1, 2] = np.nan
    hg, hb, flag = ops.precond_bn(torch.from_numpy(Fbad).cuda(), torch.from_numpy(gg).cuda(), torch.from_numpy(gb).cuda())
    assert flag.item() == 1
    assert np.array_equal(hg.cpu().numpy(), gg) and np.array_equal(hb.cpu().numpy(), gb)
    # gamma only
    kg, _, _ = O.precondition_bn(Finv[:C, :C].copy(), gg, None)
    hg, hb, _ = ops.precond_bn(torch.from_numpy(Finv[:C, :C].copy()).cuda(), torch.from_numpy(gg).cuda(), None)
    assert hb is None and rel(hg.cpu().numpy(), kg) < RTOL


@pytest.mark.parametrize('shape', [(6, 4, 5, 3), (8, 5), (32, 64, 8, 8), (4, 130, 7, 7), (16, 1000)])
def test_bn_factor(shape):
    from chainerkfac_amd import ops
    r = np.random.default_rng(sum(shape))
    x = (r.standard_normal(shape) * 2 + 0.7).astype(np.float32)
    gy = (r.standard_normal(shape) / shape[0]).astype(np.float32)
    eps = 2e-5
    n = shape[0]
    U = ops.bn_grad_matrix(torch.from_numpy(x).cuda(), torch.from_numpy(gy).cuda(), eps, float(n))
    Uref = O.bn_grad_matrix(x, gy, eps)
    assert rel(U.cpu().numpy(), Uref) < 1e-4
    F = ops.cov_linear(U, False, 1.0 / n)
    Fref = O.bn_F(x, gy, eps)
    assert rel(F.cpu().numpy(), Fref) < 1e-4
    assert np.max(np.abs(F.cpu().numpy() - Fref)) <= 1e-4 * np.max(np.abs(Fref))
    Ug = ops.bn_grad_matrix(torch.from_numpy(x).cuda(), torch.from_numpy(gy).cuda(), eps, float(n), has_beta=False)
    assert rel(Ug.cpu().numpy(), O.bn_grad_matrix(x, gy, eps, has_beta=False)) < 1e-4
    Ub = ops.bn_grad_matrix(torch.from_numpy(x).cuda(), torch.from_numpy(gy).cuda(), eps, float(n), has_gamma=False)
    assert rel(Ub.cpu().numpy(), O.bn_grad_matrix(x, gy, eps, has_gamma=False)) < 1e-4


def test_bn_factor_in_two_parts_for_many_layers():
    """The statistics pass per layer and the finish of all layers in one launch give,
    bit for bit, what the one-layer entry point gives (the same arithmetic), against
    the oracle, for every combination of gamma / beta, channel counts that are not
    multiples of the 64-channel unit, 2-D inputs and different scales per layer."""
    from chainerkfac_amd import ops
    cases = [((6, 4, 5, 3), True, True, 6.0), ((8, 5), True, True, 8.0), ((32, 64, 8, 8), True, False, 1.0),
             ((4, 130, 7, 7), False, True, 4.0), ((16, 1000), True, True, 0.25), ((3, 65, 16, 16), True, True, 3.0)]
    r = np.random.default_rng(41)
    layers, singles, refs = [], [], []
    for shape, has_gamma, has_beta, scale in cases:
        x = (r.standard_normal(shape) * 2 + 0.7).astype(np.float32)
        gy = (r.standard_normal(shape) / shape[0]).astype(np.float32)
        eps = 2e-5
        n, c = shape[0], shape[1]
        hw = int(np.prod(shape[2:])) if len(shape) == 4 else 1
        xd, gd = torch.from_numpy(x).cuda(), torch.from_numpy(gy).cuda()
        singles.append(ops.bn_grad_matrix(xd, gd, eps, scale, has_gamma, has_beta))
        refs.append(O.bn_grad_matrix(x, gy, eps, has_gamma=has_gamma, has_beta=has_beta) * (scale / n))
        stats = ops.bn_stats(xd, gd)
        assert tuple(stats.shape) == (4, n, c)
        U = torch.full((n, c * (int(has_gamma) + int(has_beta))), float('nan'), device='cuda')
        layers.append((stats, U, n, c, hw, eps, scale, has_gamma, has_beta))
    for _ in range(2):   # the second call finds its tables in place
        ops.bn_finish_batched(layers)
    for layer, single, ref in zip(layers, singles, refs):
        assert torch.equal(layer[1], single), layer[2:]
        assert rel(single.cpu().numpy(), ref) < 1e-4
    ops.bn_finish_batched([])
    with pytest.raises(ValueError):
        ops.bn_finish_batched([(layers[0][0], layers[1][1]) + layers[0][2:]])


def test_bn_rejects_other_ranks():
    from chainerkfac_amd import ops
    x = torch.zeros(2, 3, 4, device='cuda')
    with pytest.raises(RuntimeError):
        ops.bn_grad_matrix(x, x, 1e-5, 1.0)


def test_axpby_and_momentum_update():
    from chainerkfac_amd import ops
    r = np.random.default_rng(0)
    x = r.standard_normal(100003).astype(np.float32); y = r.standard_normal(100003).astype(np.float32)
    got = ops.axpby(torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda(), 0.99, 0.01).cpu().numpy()
    np.testing.assert_allclose(got, np.float32(0.99) * x + np.float32(0.01) * y, rtol=1e-6, atol=1e-7)
    # b == 0 overwrites without reading y (the accumulators start from uninitialised buffers)
    ynan = torch.full((100003,), float('nan'), device='cuda')
    got0 = ops.axpby(torch.from_numpy(x).cuda(), ynan, 0.5, 0.0).cpu().numpy()
    assert np.array_equal(got0, np.float32(0.5) * x)
    p = r.standard_normal(1000).astype(np.float32); v = r.standard_normal(1000).astype(np.float32)
    g = r.standard_normal(1000).astype(np.float32)
    pd, vd = torch.from_numpy(p).cuda(), torch.from_numpy(v).cuda()
    ops.momentum_update(pd, vd, torch.from_numpy(g).cuda(), 0.1, 0.9)
    O.momentum_update(p, v, g, 0.1, 0.9)
    np.testing.assert_allclose(vd.cpu().numpy(), v, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(pd.cpu().numpy(), p, rtol=1e-6, atol=1e-7)


def test_axpby_batched():
    """y = a x + b y for many array pairs in one launch: ragged sizes around the unit size,
    empty arrays, arrays that start off a 16-byte boundary; bit-exact against the single-pair
    kernel, and b == 0 overwrites without reading y."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(5)
    sizes = [0, 1, 7, 2047, 2048, 2049, 100003, 3 * 4096, 65 * 65, 4609]
    xs, ys, singles = [], [], []
    for k, n in enumerate(sizes):
        off = k % 3
        x = torch.from_numpy(r.standard_normal(n + 3).astype(np.float32)).cuda()[off:off + n]
        yoff = (off + (k // 3) % 2) % 3   # both aligned, one aligned, none aligned
        y = torch.from_numpy(r.standard_normal(n + 3).astype(np.float32)).cuda()[yoff:yoff + n]
        xs.append(x); ys.append(y)
        singles.append(ops.axpby(x.contiguous(), y.clone(), 0.99, 0.01) if n else y.clone())
    expect = [np.float32(0.99) * x.cpu().numpy() + np.float32(0.01) * y.cpu().numpy() for x, y in zip(xs, ys)]
    ops.axpby_batched(xs, ys, 0.99, 0.01)
    torch.cuda.synchronize()
    for y, single, e in zip(ys, singles, expect):
        assert torch.equal(y, single)
        np.testing.assert_allclose(y.cpu().numpy(), e, rtol=1e-6, atol=1e-7)
    nans = [torch.full_like(y, float('nan')) for y in ys]
    ops.axpby_batched(xs, nans, 0.5, 0.0)
    torch.cuda.synchronize()
    for x, y in zip(xs, nans):
        assert np.array_equal(y.cpu().numpy(), np.float32(0.5) * x.cpu().numpy())
    with pytest.raises(ValueError):
        ops.axpby_batched(xs[:2], ys[:1], 1.0, 1.0)
    with pytest.raises(ValueError):
        ops.axpby_batched([xs[2]], [ys[3]], 1.0, 1.0)


@pytest.mark.parametrize('loss_scale', [None, 128.0, 3.0])
def test_momentum_update_batched(loss_scale):
    """One launch for the rule of many parameters (optimizers/kfac.py:63-116): ragged sizes
    around the unit size, empty arrays, arrays that start off a 16-byte boundary, float16
    gradients and float16 parameters behind a float32 master copy, with and without a loss
    scale.  Against the oracle's rule on the divided gradients, bit-exact against the
    single-parameter kernel, and the divided gradient is stored where it is asked for."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(11)
    sizes = [0, 1, 5, 2047, 2048, 2049, 100003, 3 * 4096, 777, 6144]
    lr, momentum = 0.05, 0.9
    params, vs, grads, wbs, halves, expect = [], [], [], [], [], []
    for k, n in enumerate(sizes):
        off = k % 3   # views that start 0, 4 or 8 bytes past an aligned address
        p = torch.from_numpy(r.standard_normal(n + 3).astype(np.float32)).cuda()[off:off + n]
        v = torch.from_numpy(r.standard_normal(n + 3).astype(np.float32)).cuda()[off:off + n]
        g16 = k % 4 == 1
        g = torch.from_numpy(r.standard_normal(n + 3).astype(np.float16 if g16 else np.float32)).cuda()[off:off + n]
        h = torch.zeros(n + 3, dtype=torch.float16, device='cuda')[off:off + n] if k % 4 in (1, 2) else None
        wb = (not g16) and k % 2 == 0
        pe, ve, ge = p.cpu().numpy().copy(), v.cpu().numpy().copy(), g.cpu().numpy().astype(np.float32)
        if loss_scale is not None:
            ge = ge / np.float32(loss_scale)
        single = None
        if n:
            # the single-parameter kernel on copies (divided by a device scalar: a true division)
            ps, vs1 = p.clone(), v.clone()
            gs = g.float() if loss_scale is None else g.float() / torch.tensor(loss_scale, device='cuda')
            ops.momentum_update(ps, vs1, gs.contiguous(), lr, momentum)
            single = (ps, vs1)
        O.momentum_update(pe, ve, ge, lr, momentum)
        params.append(p); vs.append(v); grads.append(g); wbs.append(wb); halves.append(h)
        expect.append((pe, ve, ge, single, g.clone()))
    ops.momentum_update_batched(params, vs, grads, lr, momentum, loss_scale, wbs, halves)
    torch.cuda.synchronize()
    for p, v, g, wb, h, (pe, ve, ge, single, g0) in zip(params, vs, grads, wbs, halves, expect):
        np.testing.assert_allclose(v.cpu().numpy(), ve, rtol=1e-6, atol=1e-6)
        np.testing.assert_allclose(p.cpu().numpy(), pe, rtol=1e-6, atol=1e-6)
        if single is not None:
            assert torch.equal(p, single[0]) and torch.equal(v, single[1])
        if wb and loss_scale is not None:
            assert np.array_equal(g.cpu().numpy(), ge)
        else:
            assert torch.equal(g, g0)
        if h is not None:
            assert torch.equal(h, p.half())
    # the same call again goes through the cached tables; a changed list rewrites them
    ops.momentum_update_batched(params, vs, grads, lr, momentum, loss_scale, wbs, halves)
    ops.momentum_update_batched(params[3:6], vs[3:6], grads[3:6], lr, momentum)
    torch.cuda.synchronize()
    with pytest.raises(ValueError):
        ops.momentum_update_batched(params[:2], vs[:1], grads[:2], lr, momentum)
    with pytest.raises(ValueError):
        ops.momentum_update_batched([params[1]], [vs[1]], [grads[1]], lr, momentum, 2.0, [True])


def test_grouped_preconditioning_matches_the_single_calls():
    """All layers' products in one grouped call: 64- and 128-tiles, with and without bias,
    aligned and odd dimensions, several k-slices; against float64 and the single calls."""
    from chainerkfac_amd import ops
    r = np.random.default_rng(23)

    def spd(d):
        X = r.standard_normal((2 * d, d)).astype(np.float32)
        return torch.from_numpy((X.T @ X / (2 * d) + 0.1 * np.eye(d, dtype=np.float32)).astype(np.float32)).cuda()

    shapes = [(64, 577, True), (10, 785, True), (256, 64, False), (130, 1153, True), (1000, 2049, True),
              (96, 96, False), (7, 28, True), (512, 1024, False)]
    ops_in = []
    for dG, dA, hb in shapes:
        gW = torch.from_numpy(r.standard_normal((dG, dA - int(hb))).astype(np.float32)).cuda()
        gb = torch.from_numpy(r.standard_normal(dG).astype(np.float32)).cuda() if hb else None
        ops_in.append((spd(dG), spd(dA), gW, gb, torch.full_like(gW, float('nan')),
                       torch.full_like(gb, float('nan')) if hb else None))
    group = ops.precond_group(shapes)
    group.run(*[[o[i] for o in ops_in] for i in range(6)])
    torch.cuda.synchronize()
    for (dG, dA, hb), (G, A, gW, gb, kW, kb) in zip(shapes, ops_in):
        grad = gW.double() if not hb else torch.cat([gW.double(), gb.double()[:, None]], dim=1)
        ref = (G.double() @ grad @ A.double()).cpu().numpy()
        got = kW.cpu().numpy() if not hb else np.column_stack([kW.cpu().numpy(), kb.cpu().numpy()])
        assert rel(got, ref) < 1e-5, (dG, dA, hb)
        sW, sb = ops.precond_conn(G, A, gW, gb)
        single = sW.cpu().numpy() if not hb else np.column_stack([sW.cpu().numpy(), sb.cpu().numpy()])
        assert rel(got, single) < 1e-5, (dG, dA, hb)
    with pytest.raises(ValueError):
        group.run(*[[o[i] for o in ops_in[:-1]] for i in range(6)])
