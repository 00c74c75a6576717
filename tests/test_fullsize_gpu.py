"""Full-size cases of the ResNet-50 batch-32 workload (the sizes the benchmark is quoted on).

The NumPy oracle needs minutes at these sizes, so the checks are against float64 PyTorch on the
GPU (``unfold`` + GEMM for the patch covariance, ``linalg.inv`` for the inverses) and against
properties that hold at any size: exact symmetry, the ones row equals the column means of the
patch matrix, M M^-1 = I.
"""
import numpy as np
import pytest
import torch

from oracle import kfac_oracle as O

pytestmark = pytest.mark.gpu


def rel(a, b):
    return float((a.double() - b).norm() / b.norm())


def patch_cov64(x, k, s, p, bias):
    n = x.shape[0]
    P = torch.nn.functional.unfold(x.double(), k, padding=p, stride=s)     # (n, c*k*k, L)
    P = P.permute(0, 2, 1).reshape(-1, P.shape[1])
    if bias:
        P = torch.cat([P, torch.ones(P.shape[0], 1, dtype=P.dtype, device=P.device)], dim=1)
    return P.T @ P / n, P


@pytest.mark.parametrize('c,hw,k,s,p', [(64, 56, 3, 1, 1),      # d = 577, 100 352 patches
                                         (128, 28, 3, 1, 1),     # d = 1153
                                         (256, 14, 3, 1, 1),     # d = 2305
                                         (512, 7, 3, 1, 1),      # d = 4609
                                         (3, 224, 7, 2, 3),      # stem: d = 148, 401 408 patches
                                         (256, 56, 1, 1, 0),     # 1x1 slab, d = 257
                                         (1024, 14, 1, 2, 0)])   # strided 1x1, d = 1025
def test_conv_A_full_size(c, hw, k, s, p):
    from chainerkfac_amd import ops
    g = torch.Generator(device='cuda').manual_seed(c + hw)
    x = torch.randn(32, c, hw, hw, device='cuda', generator=g)
    A = ops.cov_conv_a(x, k, s, p, True, 1.0 / 32)
    ref, P = patch_cov64(x, k, s, p, True)
    assert rel(A, ref) < 1e-4
    assert torch.equal(A, A.T)
    # ones row = column sums of the patch matrix / n; corner = patches per sample
    assert rel(A[-1, :-1], P[:, :-1].sum(0) / 32) < 1e-5
    assert abs(float(A[-1, -1]) - P.shape[0] / 32) <= 1e-6 * P.shape[0] / 32


@pytest.mark.parametrize('c,hw', [(64, 112), (256, 56), (2048, 7)])
def test_conv_G_full_size(c, hw):
    from chainerkfac_amd import ops
    g = torch.Generator(device='cuda').manual_seed(c)
    gy = torch.randn(32, c, hw, hw, device='cuda', generator=g) / 32
    G = ops.cov_conv_g(gy, 32.0 ** 2 / (32 * hw * hw))
    M = gy.double().permute(0, 2, 3, 1).reshape(-1, c)
    ref = M.T @ M * (32.0 ** 2 / (32 * hw * hw))
    assert rel(G, ref) < 1e-4
    assert torch.equal(G, G.T)


def test_inverse_of_all_161_factor_sizes():
    """The inverse-only configuration: 161 SPD matrices of ResNet-50's factor sizes, 27^2 .. 4609^2
    (the list the benchmark's c4 builds)."""
    import bench
    from chainerkfac_amd import ops
    dims = bench.inverse_dims()
    assert len(dims) == 161 and max(dims) == 4609 and min(dims) == 27
    g = torch.Generator(device='cuda').manual_seed(4)
    mats = []
    for d in dims:
        X = torch.randn(2 * d, d, device='cuda', generator=g)
        mats.append(X.T @ X / (2 * d) + 1e-3 * torch.eye(d, device='cuda'))
        del X
    outs, info = ops.spd_inverse_batched(mats)
    assert int((info != 0).sum()) == 0
    for d, M, inv in zip(dims, mats, outs):
        assert torch.equal(inv, inv.T)
    # residual on one matrix of every distinct size, float64 inverse on the largest
    seen = set()
    for d, M, inv in zip(dims, mats, outs):
        if d in seen:
            continue
        seen.add(d)
        resid = float((M.double() @ inv.double() - torch.eye(d, device='cuda', dtype=torch.float64)).norm()) / d ** 0.5
        assert resid < 1e-3, (d, resid)
    i = dims.index(4609)
    assert rel(outs[i].cpu(), torch.linalg.inv(mats[i].double().cpu())) < 1e-3   # LAPACK on the host


def test_bn_lowrank_inverse_full_size():
    from chainerkfac_amd import ops
    g = torch.Generator(device='cuda').manual_seed(9)
    widths = [128, 512, 1024, 2048, 4096]
    Us = [torch.randn(32, w, device='cuda', generator=g) * 0.05 for w in widths]
    d = 16 * 2.5e-4
    outs, info = ops.bn_lowrank_inverse_batched(Us, [w // 2 for w in widths], [d] * 5, [d] * 5)
    assert int((info != 0).sum()) == 0
    for U, w, out in zip(Us, widths, outs):
        F = U.double().T @ U.double() / 32 + d * torch.eye(w, device='cuda', dtype=torch.float64)
        assert rel(out.cpu(), torch.linalg.inv(F.cpu())) < 1e-3   # LAPACK on the host
        assert torch.equal(out, out.T)


def test_precondition_largest_layer():
    from chainerkfac_amd import ops
    g = torch.Generator(device='cuda').manual_seed(11)
    dG, dA = 512, 4609

    def spd(d):
        X = torch.randn(2 * d, d, device='cuda', generator=g)
        return X.T @ X / (2 * d) + 0.1 * torch.eye(d, device='cuda')
    Ginv, Ainv = spd(dG), spd(dA)
    gW = torch.randn(dG, 512, 3, 3, device='cuda', generator=g)
    gb = torch.randn(dG, device='cuda', generator=g)
    kW, kb = ops.precond_conn(Ginv, Ainv, gW, gb)
    grad = torch.cat([gW.reshape(dG, -1), gb[:, None]], dim=1).double()
    ref = Ginv.double() @ grad @ Ainv.double()
    assert rel(kW.reshape(dG, -1), ref[:, :-1]) < 1e-3
    assert rel(kb, ref[:, -1]) < 1e-3


@pytest.mark.parametrize('c,hw', [(64, 112), (256, 56), (2048, 7)])
def test_bn_grad_matrix_full_size(c, hw):
    """The batch-norm statistics pass at the activation sizes of ResNet-50 batch 32
    (stem, a stage-2 output, a stage-5 output) against float64 batch statistics."""
    from chainerkfac_amd import ops
    g = torch.Generator(device='cuda').manual_seed(c + hw)
    n, eps = 32, 2e-5
    x = torch.randn(n, c, hw, hw, device='cuda', generator=g) * 1.7 + 0.4
    gy = torch.randn(n, c, hw, hw, device='cuda', generator=g) / (n * hw)
    U = ops.bn_grad_matrix(x, gy, eps, float(n))
    xd, gd = x.double(), gy.double() * n
    mean = xd.mean(dim=(0, 2, 3), keepdim=True)
    var = ((xd - mean) ** 2).mean(dim=(0, 2, 3), keepdim=True)
    h = (xd - mean) / torch.sqrt(var + eps)
    ref = torch.cat([(gd * h).sum(dim=(2, 3)), gd.sum(dim=(2, 3))], dim=1)
    assert U.shape == (n, 2 * c)
    assert rel(U, ref) < 1e-4
    F = ops.cov_linear(U, False, 1.0 / n)
    assert rel(F, ref.T @ ref / n) < 1e-4
    assert torch.equal(F, F.T)
    # the identities that tie U to the parameter gradients: sum_n U = n * (dgamma | dbeta)
    xl = x.clone().requires_grad_(True)
    gamma = torch.ones(c, device='cuda', requires_grad=True)
    beta = torch.zeros(c, device='cuda', requires_grad=True)
    y = torch.nn.functional.batch_norm(xl, None, None, gamma, beta, True, 0.1, eps)
    y.backward(gy)
    assert rel(U[:, :c].sum(0) / n, gamma.grad.double()) < 1e-3
    assert rel(U[:, c:].sum(0) / n, beta.grad.double()) < 1e-4


def _inv64(M):
    return torch.linalg.inv(M.double().cpu()).cuda()   # LAPACK on the host


def test_resnet50d_accumulation_pack_inverse_precondition():
    """The large-batch accumulation configuration at ResNet-50-D's own shapes: 16
    micro-batches of synthetic activations / gradients accumulated by the
    covariance kernels' running sum (beta = 1, alpha = scale / 16), the factors and
    gradients packed into one flat buffer in the reference's order and unpacked
    (bit-exact round trip), then damped inverse and preconditioning.  Layers: the
    biased 3->32 stride-2 stem (d = 28), a 288, a strided 3x3 (1152), a 2304 and a
    4608 factor, a 1x1 slab and a batch-norm block."""
    import bench
    from chainerkfac_amd import workloads as W
    from chainerkfac_amd.communicators import ArrayPacker
    from chainerkfac_amd.optimizers import KFAC
    from chainerkfac_amd.optimizers.kfac import extract
    table = {l['name']: l for l in W.resnet50_d()}
    layers = [table[k] for k in ('conv1_1', 'conv1_2', 'res2/0/conv1', 'res3/0/conv2', 'res4/1/conv2',
                                 'res5/1/conv2', 'res4/1/bn2')]
    assert [W.factor_dims(l) for l in layers] == [(28, 32), (288, 32), (64, 64), (1152, 128), (2304, 256),
                                                  (4608, 512), (512,)]
    n, iters, damping = 32, 16, 2.5e-4
    dev = torch.device('cuda:0')
    gen = torch.Generator(device=dev).manual_seed(5)
    model, calls = bench.build_model(layers, dev, gen)
    opt = KFAC(damping=damping, stab_coeff=16.0, cov_ema_decay=1.0, acc_iters=iters).setup(model)
    by_link = {id(fb.link): fb for fb in opt.fblocks}
    fbs = [by_link[id(getattr(model, name))] for name, _, _, _ in calls]
    ref_covs = [None] * len(calls)
    ref_grads = {}
    for it in range(iters):
        for fb in opt.fblocks:
            fb.acc_state = (iters, it)
        for i, (name, func, in_data, _) in enumerate(calls):
            layer = layers[i]
            x = torch.randn(in_data[0].shape, device=dev, generator=gen)
            gy_shape = (n, layer['c'], layer['h'], layer['w']) if layer['kind'] == 'bn' else \
                (n, layer['c_out']) + (W.conv_out(layer['h'], layer['k'], layer['s'], layer['p']),) * 2
            gy = torch.randn(gy_shape, device=dev, generator=gen) / (n * gy_shape[-1])
            data = (x,) + tuple(in_data[1:])
            opt.kfhook.forward_postprocess(func, data)
            opt.kfhook.backward_preprocess(func, data, (gy,))
            if layer['kind'] == 'conv':
                A64, _ = patch_cov64(x, layer['k'], layer['s'], layer['p'], layer['bias'])
                g64 = gy.double().permute(0, 2, 3, 1).reshape(-1, gy.shape[1])
                G64 = g64.T @ g64 * (float(n) ** 2 / g64.shape[0])
                new = [A64, G64]
            else:
                xd, gd = x.double(), gy.double() * n
                mean = xd.mean(dim=(0, 2, 3), keepdim=True)
                h = (xd - mean) / torch.sqrt(((xd - mean) ** 2).mean(dim=(0, 2, 3), keepdim=True) + 2e-5)
                U = torch.cat([(gd * h).sum(dim=(2, 3)), gd.sum(dim=(2, 3))], dim=1)
                new = [U.T @ U / n]
            ref_covs[i] = new if ref_covs[i] is None else [a + b for a, b in zip(ref_covs[i], new)]
            del x, gy, new
        for pname, p in model.namedparams():
            p.grad = torch.randn(p.shape, device=dev, generator=gen)
            ref_grads[pname] = ref_grads.get(pname, 0) + p.grad.double() / iters
        opt.finish_covs()
        go_on = opt.accumulate()
        assert go_on == (it < iters - 1)
    # accumulated factors and gradients = means over the micro-batches
    for i, fb in enumerate(fbs):
        for got, want in zip(fb.covs, ref_covs[i]):
            assert rel(got, want / iters) < 1e-4, (layers[i]['name'], got.shape)
            assert torch.equal(got, got.T)
    for pname, p in model.namedparams():
        assert rel(p.grad, ref_grads[pname]) < 1e-5, pname
    # wire format: grads, A, G per block in the reference's order; bit-exact round trip
    arrays = extract(opt.fblocks, [range(len(opt.fblocks))], lambda b: b.extract_for_reduce_scatter_v())
    assert sum(1 for _, tri in arrays[0] if tri) == 13 and sum(1 for _, tri in arrays[0] if not tri) == 9
    packer = ArrayPacker()
    nel = packer.get_nelems(arrays)
    assert nel == sum(a.shape[0] * (a.shape[0] + 1) // 2 if tri else a.numel() for a, tri in arrays[0])
    buf = torch.empty(nel, dtype=torch.float32, device=dev)
    packer._pack_arrays_to_buffer(arrays, buf)
    before = [a.clone() for a, _ in arrays[0]]
    for a, _ in arrays[0]:
        a.fill_(float('nan'))
    packer._unpack_arrays_from_buffer(arrays, buf)
    for (a, _), b in zip(arrays[0], before):
        assert torch.equal(a, b)
    # damped inverse + preconditioning of the accumulated factors
    opt.reallocate_cleared_grads()
    opt.update_kfgrads(opt.fblocks)
    torch.cuda.synchronize()
    assert int((opt.inv_info != 0).sum()) == 0
    for i, fb in enumerate(fbs):
        layer = layers[i]
        for M, inv in zip(fb.cov_emas, fb.invs):        # cov_emas now hold the damped factors
            d = M.shape[0]
            resid = float((M.double() @ inv.double() - torch.eye(d, device=dev, dtype=torch.float64)).norm()) / d ** 0.5
            assert resid < 1e-3, (layer['name'], d, resid)
        if layer['kind'] == 'conv':
            Ainv, Ginv = _inv64(fb.cov_emas[0]), _inv64(fb.cov_emas[1])
            assert rel(fb.invs[0], Ainv) < 1e-3 and rel(fb.invs[1], Ginv) < 1e-3, layer['name']
            link = fb.link
            grad = link.W.grad.double().reshape(link.W.shape[0], -1)
            if link.b is not None:
                grad = torch.cat([grad, link.b.grad.double()[:, None]], dim=1)
            kf = Ginv @ grad @ Ainv
            got = link.W.kfgrad.reshape(link.W.shape[0], -1)
            if link.b is not None:
                assert rel(link.b.kfgrad, kf[:, -1]) < 1e-3, layer['name']
                kf = kf[:, :-1]
            assert rel(got, kf) < 1e-3, layer['name']
        else:
            Finv = _inv64(fb.cov_emas[0])
            g = torch.cat([fb.link.gamma.grad, fb.link.beta.grad]).double()
            kf = Finv @ g
            c = layer['c']
            assert rel(fb.link.gamma.kfgrad, kf[:c]) < 1e-3 and rel(fb.link.beta.kfgrad, kf[c:]) < 1e-3


def test_resnet50_assembled_step_all_161_factors():
    """One whole K-FAC step of the ResNet-50 batch-32 workload assembled the way the
    benchmark runs it (all 161 factors through the hook calls, then moving average
    -> damping -> inverse -> preconditioning): every block's inverse against its
    damped factor, and the preconditioned gradients of a sample of layers against
    float64."""
    import bench
    from chainerkfac_amd import workloads as W
    from chainerkfac_amd.optimizers import KFAC
    from chainerkfac_amd.optimizers import fisher_blocks as FB
    dev = torch.device('cuda:0')
    gen = torch.Generator(device=dev).manual_seed(3)
    layers = W.resnet50_v1()
    model, calls = bench.build_model(layers, dev, gen)
    opt = KFAC(damping=bench.DAMPING, stab_coeff=bench.STAB_COEFF, cov_ema_decay=1.0).setup(model)
    assert len(opt.fblocks) == 107 and sum(len(W.factor_dims(l)) for l in layers) == 161
    for _, func, in_data, gy in calls:
        opt.kfhook.forward_postprocess(func, in_data)
        opt.kfhook.backward_preprocess(func, in_data, (gy,))
    opt.update_kfgrads(opt.fblocks)
    torch.cuda.synchronize()
    assert opt.check_numerics() == []
    n_factors = 0
    for fb in opt.fblocks:
        for M, inv in zip(fb.cov_emas, fb.invs):
            d = M.shape[0]
            n_factors += 1
            assert torch.equal(inv, inv.T)
            resid = float((M.double() @ inv.double() - torch.eye(d, device=dev, dtype=torch.float64)).norm()) / d ** 0.5
            assert resid < 1e-3, (fb.linkname, d, resid)
    assert n_factors == 161
    by_link = {id(fb.link): fb for fb in opt.fblocks}
    sample = ('conv1', 'res2/0/conv2', 'res3/1/conv3', 'res4/0/conv4', 'res4/2/conv2', 'res5/0/conv1', 'fc',
              'bn1', 'res3/0/bn3', 'res5/2/bn3')
    for i, layer in enumerate(layers):
        if layer['name'] not in sample:
            continue
        fb = by_link[id(getattr(model, calls[i][0]))]
        if isinstance(fb, FB.FisherBlockConnection):
            Ainv, Ginv = _inv64(fb.cov_emas[0]), _inv64(fb.cov_emas[1])
            link = fb.link
            grad = torch.cat([link.W.grad.double().reshape(link.W.shape[0], -1), link.b.grad.double()[:, None]], dim=1)
            kf = Ginv @ grad @ Ainv
            assert rel(link.W.kfgrad.reshape(link.W.shape[0], -1), kf[:, :-1]) < 1e-3, layer['name']
            assert rel(link.b.kfgrad, kf[:, -1]) < 1e-3, layer['name']
        else:
            c = layer['c']
            kf = _inv64(fb.cov_emas[0]) @ torch.cat([fb.link.gamma.grad, fb.link.beta.grad]).double()
            assert rel(fb.link.gamma.kfgrad, kf[:c]) < 1e-3 and rel(fb.link.beta.kfgrad, kf[c:]) < 1e-3, layer['name']


@pytest.mark.timeout(900)
def test_resnet50_real_network_one_update():
    """ResNet-50 (bottleneck v1, bias, 1000-way) built from the link classes, one
    ``KFAC.update`` at batch 32 @ 224: the function hooks of a real forward /
    backward pass feed all 107 Fisher blocks (161 factors).  A second hook records
    what a sample of layers saw, and their factors and preconditioned gradients
    are checked against float64."""
    import torch.nn.functional as TF
    from chainerkfac_amd import links as L
    from chainerkfac_amd import workloads as W
    from chainerkfac_amd.optimizers import KFAC
    dev = torch.device('cuda:0')
    gen = torch.Generator(device=dev).manual_seed(3)
    model = W.build_resnet50_v1(device=dev, generator=gen)
    opt = KFAC(lr=1e-3, damping=2.5e-4, stab_coeff=16.0, cov_ema_decay=1.0).setup(model)
    assert len(opt.fblocks) == 107
    assert [fb.linkname for fb in opt.fblocks] == sorted(fb.linkname for fb in opt.fblocks)
    x = torch.randn(32, 3, 224, 224, device=dev, generator=gen)
    t = torch.randint(0, 1000, (32,), device=dev, generator=gen)
    watch = {'/conv1': model.conv1, '/res2/0/conv2': model.res2[0].conv2, '/res4/3/conv1': model.res4[3].conv1,
             '/res5/0/conv4': model.res5[0].conv4, '/fc': model.fc}
    owner = {id(l.W.data): name for name, l in watch.items()}
    seen = {}

    class Recorder(L.FunctionHook):
        def forward_postprocess(self, function, in_data):
            name = owner.get(id(in_data[1]))
            if name:
                seen.setdefault(name, {})['x'] = in_data[0].clone()

        def backward_preprocess(self, function, in_data, out_grad_data):
            name = owner.get(id(in_data[1]))
            if name:
                seen[name]['gy'] = out_grad_data[0].clone()

    before = {name: p.data.clone() for name, p in model.namedparams()}
    with Recorder():
        opt.update(lambda: TF.cross_entropy(model(x), t))
    torch.cuda.synchronize()
    dims = sorted(c.shape[0] for fb in opt.fblocks for c in fb.covs)
    assert dims == sorted(W.all_factor_dims(W.resnet50_v1()))
    assert opt.t == 1
    for name, p in model.namedparams():
        assert bool(torch.isfinite(p.data).all()), name
        assert not torch.equal(p.data, before[name]), name
    by_name = {fb.linkname: fb for fb in opt.fblocks}
    assert sorted(seen) == sorted(watch)
    for name, link in watch.items():
        fb = by_name[name]
        xs, gy = seen[name]['x'], seen[name]['gy']
        if isinstance(link, L.Linear):
            xe = torch.cat([xs.double(), torch.ones(32, 1, device=dev, dtype=torch.float64)], dim=1)
            A64 = xe.T @ xe / 32
            G64 = gy.double().T @ gy.double() * 32
        else:
            A64, _ = patch_cov64(xs, link.ksize, link.stride[0], link.pad[0], True)
            g64 = gy.double().permute(0, 2, 3, 1).reshape(-1, gy.shape[1])
            G64 = g64.T @ g64 * (32.0 ** 2 / g64.shape[0])
        # decay 1: cov_emas are the factors of this step with the damping on their diagonals
        A, G = fb.cov_emas
        offA = A - torch.diag(torch.diagonal(A))
        offG = G - torch.diag(torch.diagonal(G))
        assert rel(offA, A64 - torch.diag(torch.diagonal(A64))) < 1e-4, name
        assert rel(offG, G64 - torch.diag(torch.diagonal(G64))) < 1e-4, name
        pi = float(fb.pi)
        want_pi = float(torch.sqrt(torch.trace(A64) * G64.shape[0] / (torch.trace(G64) * A64.shape[0])))
        assert abs(pi - want_pi) < 1e-4 * want_pi, name
        assert rel(torch.diagonal(A), torch.diagonal(A64) + want_pi * 2.5e-4 ** 0.5) < 1e-4, name
        assert rel(torch.diagonal(G), torch.diagonal(G64) + 2.5e-4 ** 0.5 / want_pi) < 1e-4, name
        # the preconditioned gradient against float64 on the same damped factors.  Factors of a
        # real network are far worse conditioned than synthetic ones (post-ReLU activations have a
        # large mean component), so the bound is the float64 result: no further from it than 4x
        # the NumPy formula of the reference (float32 Cholesky, inv, matmul) on the same inputs.
        grad = torch.cat([link.W.grad.double().reshape(link.W.shape[0], -1), link.b.grad.double()[:, None]], dim=1)
        kf = _inv64(G) @ grad @ _inv64(A)
        got = torch.cat([link.W.kfgrad.reshape(link.W.shape[0], -1), link.b.kfgrad[:, None]], dim=1)
        kW, kb = O.precondition_conn(O.inverse(A.cpu().numpy()), O.inverse(G.cpu().numpy()),
                                     link.W.grad.cpu().numpy(), link.b.grad.cpu().numpy())
        ref32 = np.column_stack([kW.reshape(kW.shape[0], -1), kb])
        err_hip = rel(got, kf)
        err_ref = rel(torch.from_numpy(ref32).cuda(), kf)
        assert err_hip < max(4 * err_ref, 1e-3), (name, err_hip, err_ref)
        # the update itself: p1 = p0 - lr * kfgrad (the momentum buffer starts at zero)
        p0 = before[[k for k, p in model.namedparams() if p is link.W][0]]
        want = p0 - 1e-3 * link.W.kfgrad
        assert float((link.W.data - want).abs().max()) <= 2e-7 * float(p0.abs().max()) + 1e-12, name
