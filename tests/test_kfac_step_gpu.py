"""End-to-end parity of the KFAC optimizer (hooks, phase order, scales, state)
with the CPU oracle on the same seeded model and batches (needs the GPU).

The model's forward/backward is not part of the K-FAC path: it runs through
torch autograd on both sides (GPU for the product, CPU for the oracle), with a
recording hook on the CPU side that captures what the reference's function
hooks would see."""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

from oracle import kfac_oracle as O
from oracle.kfac_step import LayerRecord, OracleKFAC

pytestmark = pytest.mark.gpu


def rel(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def build_mlp(L, device, gen):
    class MLP(L.Chain):
        def __init__(self):
            super(MLP, self).__init__()
            self.l1 = L.Linear(784, 1000, device=device, generator=gen)
            self.l2 = L.Linear(1000, 1000, device=device, generator=gen)
            self.l3 = L.Linear(1000, 10, device=device, generator=gen)

        def __call__(self, x):
            return self.l3(TF.relu(self.l2(TF.relu(self.l1(x)))))
    return MLP()


def build_cnn(L, device, gen):
    class CNN(L.Chain):
        def __init__(self):
            super(CNN, self).__init__()
            self.conv1 = L.Convolution2D(3, 16, 3, 1, 1, device=device, generator=gen)
            self.bn1 = L.BatchNormalization(16, device=device)
            self.conv2 = L.Convolution2D(16, 24, 3, 2, 1, nobias=True, device=device, generator=gen)
            self.bn2 = L.BatchNormalization(24, device=device)
            self.conv3 = L.Convolution2D(24, 32, 1, 1, 0, device=device, generator=gen)
            self.fc = L.Linear(32 * 4 * 4, 10, device=device, generator=gen)

        def __call__(self, x):
            h = TF.relu(self.bn1(self.conv1(x)))
            h = TF.max_pool2d(h, 2)
            h = TF.relu(self.bn2(self.conv2(h)))
            h = TF.relu(self.conv3(h))
            return self.fc(h)
    return CNN()


def build_cifar_cnn(L, device, gen):
    """The CIFAR-shaped CNN of the benchmark's second configuration: three 3x3
    convolutions (3->64->128->256, pad 1, bias) with ReLU and 2x2 max-pooling,
    then a 4096->10 fully connected layer: A factors 28, 577, 1153, 4097."""
    class CifarCNN(L.Chain):
        def __init__(self):
            super(CifarCNN, self).__init__()
            self.conv1 = L.Convolution2D(3, 64, 3, 1, 1, device=device, generator=gen)
            self.conv2 = L.Convolution2D(64, 128, 3, 1, 1, device=device, generator=gen)
            self.conv3 = L.Convolution2D(128, 256, 3, 1, 1, device=device, generator=gen)
            self.fc = L.Linear(4096, 10, device=device, generator=gen)

        def __call__(self, x):
            h = TF.max_pool2d(TF.relu(self.conv1(x)), 2)
            h = TF.max_pool2d(TF.relu(self.conv2(h)), 2)
            h = TF.max_pool2d(TF.relu(self.conv3(h)), 2)
            return self.fc(h)
    return CifarCNN()


def copy_params(src, dst):
    for (n1, p1), (n2, p2) in zip(sorted(src.namedparams()), sorted(dst.namedparams())):
        assert n1 == n2
        with torch.no_grad():
            p2.tensor.copy_(p1.tensor.to(p2.tensor.device))


class Recorder(object):
    """CPU-side hook: collects (x, gy) per link-function call."""

    def __init__(self, L, model):
        self.L = L
        self.owner = {}
        for name, link in model.namedlinks():
            for key in link._params:           # parameters the link itself owns
                p = getattr(link, key)
                if p is not None:
                    self.owner[id(p.data)] = (name, link)
        self.calls = {}

    def hook(self):
        L = self.L
        rec = self

        class H(L.FunctionHook):
            def forward_postprocess(self, function, in_data):
                name, link = rec.owner[id(next(a for a in in_data[1:] if a is not None))]
                rec.calls[name] = {'link': link, 'x': in_data[0].numpy().copy()}

            def backward_preprocess(self, function, in_data, out_grad_data):
                name, link = rec.owner[id(next(a for a in in_data[1:] if a is not None))]
                rec.calls[name]['gy'] = out_grad_data[0].numpy().copy()
        return H()

    def records(self):
        L = self.L
        out = []
        for name, c in self.calls.items():
            link = c['link']
            params = {k.lstrip('/'): p.data.numpy() for k, p in link.namedparams()}
            grads = {k.lstrip('/'): p.grad.numpy().copy() for k, p in link.namedparams()}
            if isinstance(link, L.Linear):
                out.append(LayerRecord('linear', name, c['x'], c['gy'], params, grads))
            elif isinstance(link, L.Convolution2D):
                out.append(LayerRecord('conv', name, c['x'], c['gy'], params, grads, ksize=link.ksize,
                                       stride=link.stride[0], pad=link.pad[0], diag=getattr(link, 'diag', False)))
            else:
                out.append(LayerRecord('bn', name, c['x'], c['gy'], params, grads, eps=link.eps))
        return out


def run_case(build, batches, after_first_update=None, prepare=None, **hyper):
    """``after_first_update(model, ref_model, opt, oracle)`` is called once both sides have made
    their first parameter update (the only one whose inputs are bit-identical on both sides);
    ``prepare(model)`` is applied to both models before the optimizers are set up."""
    from chainerkfac_amd import links as L
    from chainerkfac_amd.optimizers import KFAC
    gen = torch.Generator(device='cpu').manual_seed(7)
    ref_model = build(L, 'cpu', gen)
    model = build(L, 'cuda', None)
    copy_params(ref_model, model)
    if prepare is not None:
        prepare(model)
        prepare(ref_model)
    opt = KFAC(**hyper).setup(model)
    oracle = OracleKFAC(**hyper)

    def lossfun(m, x, t):
        return TF.cross_entropy(m(x), t)

    updates = 0
    for x, t in batches:
        opt.update(lossfun, model, torch.from_numpy(x).cuda(), torch.from_numpy(t).cuda())
        rec = Recorder(L, ref_model)
        ref_model.cleargrads()
        with rec.hook():
            loss = lossfun(ref_model, torch.from_numpy(x), torch.from_numpy(t))
            loss.backward()
        # updates ref_model's parameters in place (shared memory); False inside an accumulation
        updates += bool(oracle.step(rec.records()))
        if updates == 1 and after_first_update is not None:
            torch.cuda.synchronize()
            after_first_update(model, ref_model, opt, oracle)
            after_first_update = None
    torch.cuda.synchronize()
    return model, ref_model, opt, oracle


def compare(model, ref_model, opt, oracle, tol_param=1e-3, tol_kf=1e-3, loose=None):
    """Factors 1e-4, inverses 1e-3, preconditioned gradients ``tol_kf``, parameters ``tol_param``;
    ``loose`` maps a parameter path ('/fc/b') to its own (tol_param, tol_kf)."""
    loose = loose or {}
    by_name = {fb.linkname: fb for fb in opt.fblocks}
    assert [fb.linkname for fb in opt.fblocks] == sorted(by_name)
    for name, invs in oracle.invs.items():
        fb = by_name[name]
        for got, ref in zip(fb.invs, invs):
            assert rel(got.cpu().numpy(), ref) < 1e-3, name
        for got, ref in zip(fb.cov_emas, oracle.cov_emas[name]):
            assert rel(got.cpu().numpy(), ref) < 1e-4, name
    for (lname, pname), ref in oracle.kfgrads.items():
        got = getattr(by_name[lname].link, pname).kfgrad.cpu().numpy()
        assert got.shape == ref.shape
        tol = loose.get(lname + '/' + pname, (tol_param, tol_kf))[1]
        assert rel(got, ref) < tol, (lname, pname, rel(got, ref))
    for (n1, p1), (n2, p2) in zip(sorted(model.namedparams()), sorted(ref_model.namedparams())):
        tol = loose.get(n1, (tol_param, tol_kf))[0]
        assert rel(p1.data.cpu().numpy(), p2.data.numpy()) < tol, (n1, rel(p1.data.cpu().numpy(), p2.data.numpy()))
    assert int((opt.inv_info != 0).sum()) == 0


def mnist_batches(n_batches, bs=128, seed=1):
    r = np.random.default_rng(seed)
    return [(r.random((bs, 784), dtype=np.float32), r.integers(0, 10, bs).astype(np.int64))
            for _ in range(n_batches)]


def cnn_batches(n_batches, bs=16, seed=2):
    r = np.random.default_rng(seed)
    return [(r.standard_normal((bs, 3, 16, 16)).astype(np.float32), r.integers(0, 10, bs).astype(np.int64))
            for _ in range(n_batches)]


def test_mlp_one_step_config1():
    """MLP 784-1000-1000-10, batch 128, damping 1e-3: one full optimizer step."""
    out = run_case(build_mlp, mnist_batches(1), lr=1e-3, momentum=0.9, cov_ema_decay=0.99, damping=1e-3)
    compare(*out)
    opt = out[2]
    assert opt.t == 1 and opt.acc_aware_iterations == 1
    assert [tuple(c.shape) for fb in opt.fblocks for c in fb.covs] == \
        [(785, 785), (1000, 1000), (1001, 1001), (1000, 1000), (1001, 1001), (10, 10)]


def test_mlp_three_steps_moving_average_and_momentum():
    """After the first step the two sides no longer see identical inputs (the
    models' own forward/backward round differently on GPU and CPU and the
    parameters drift apart by ~1e-6), and the damped inverse of the nearly
    singular softmax-gradient factor amplifies that; the 1e-3 bound of the
    single-step tests is therefore relaxed to 5e-3 for the later steps."""
    out = run_case(build_mlp, mnist_batches(3, bs=32), after_first_update=compare,
                   lr=1e-2, momentum=0.9, cov_ema_decay=0.9, damping=1e-2)   # first step: 1e-3
    compare(*out, tol_param=2e-3, tol_kf=5e-3)
    shadow_check(*out)


def test_cnn_with_batchnorm_two_steps():
    out = run_case(build_cnn, cnn_batches(2), after_first_update=compare,
                   lr=1e-2, momentum=0.9, cov_ema_decay=1.0, damping=1e-2, stab_coeff=16.0)   # first step: 1e-3
    compare(*out, tol_param=2e-3, tol_kf=5e-3)
    shadow_check(*out)


def test_cnn_with_diagonal_G_factor():
    """``link.diag = True`` on a convolution (a user-settable attribute the reference reads at
    convolution_2d.py:68-70): G = diag(diag(G)) goes through damping, inverse and preconditioning
    like any other factor; one step against the oracle."""
    def prepare(model):
        model.conv1.diag = True
        model.conv3.diag = True
    out = run_case(build_cnn, cnn_batches(1), prepare=prepare, lr=1e-2, momentum=0.9, cov_ema_decay=1.0,
                   damping=1e-2, stab_coeff=16.0)
    compare(*out)
    opt = out[2]
    for name in ('/conv1', '/conv3'):
        G = {fb.linkname: fb for fb in opt.fblocks}[name].covs[1].cpu().numpy()
        assert np.count_nonzero(G - np.diag(np.diag(G))) == 0


def kfgrad_errors_vs_float64(A_damped, G_damped, gW, gb, kW, kb):
    """Relative error of a float32 preconditioned gradient against the float64
    product of the float64 inverses of the same (float32, damped) factors."""
    grad = gW.reshape(gW.shape[0], -1).astype(np.float64)
    if gb is not None:
        grad = np.column_stack([grad, gb.astype(np.float64)])
    kf = np.linalg.inv(G_damped.astype(np.float64)) @ grad @ np.linalg.inv(A_damped.astype(np.float64))
    got = kW.reshape(kW.shape[0], -1)
    if kb is not None:
        got = np.column_stack([got, kb])
    return rel(got, kf)


def shadow_check(model, ref_model, opt, oracle, floor=1e-3):
    """Second criterion for steps whose float32 results cannot agree to 1e-3 (factors that
    are nearly singular before damping, inputs that already differ in the last bits after an
    earlier step): on each side the preconditioned gradients are compared with the float64
    product of the float64 inverses of that side's own damped factors and gradients.  The HIP
    path must be no further from float64 than 4x what the NumPy formula of the reference is."""
    ref_links = dict(ref_model.namedlinks())
    for fb in opt.fblocks:
        name = fb.linkname
        rl = ref_links[name]
        if hasattr(fb.link, 'W'):
            W, b = fb.link.W, fb.link.b
            err_hip = kfgrad_errors_vs_float64(
                fb.cov_emas[0].cpu().numpy(), fb.cov_emas[1].cpu().numpy(), W.grad.cpu().numpy(),
                None if b is None else b.grad.cpu().numpy(), W.kfgrad.cpu().numpy(),
                None if b is None else b.kfgrad.cpu().numpy())
            err_ref = kfgrad_errors_vs_float64(
                oracle.cov_emas[name][0], oracle.cov_emas[name][1], rl.W.grad.numpy(),
                None if rl.b is None else rl.b.grad.numpy(), oracle.kfgrads[(name, 'W')],
                None if rl.b is None else oracle.kfgrads[(name, 'b')])
        else:
            def bn_err(F, g_gamma, g_beta, k_gamma, k_beta):
                kf = np.linalg.inv(F.astype(np.float64)) @ np.concatenate([g_gamma, g_beta]).astype(np.float64)
                return rel(np.concatenate([k_gamma, k_beta]), kf)
            gm, bt = fb.link.gamma, fb.link.beta
            err_hip = bn_err(fb.cov_emas[0].cpu().numpy(), gm.grad.cpu().numpy(), bt.grad.cpu().numpy(),
                             gm.kfgrad.cpu().numpy(), bt.kfgrad.cpu().numpy())
            err_ref = bn_err(oracle.cov_emas[name][0], rl.gamma.grad.numpy(), rl.beta.grad.numpy(),
                             oracle.kfgrads[(name, 'gamma')], oracle.kfgrads[(name, 'beta')])
        assert err_hip < max(4 * err_ref, floor), (name, err_hip, err_ref)


def test_cifar_cnn_one_step_config2():
    """Small CIFAR-shaped CNN, batch 128, input (128,3,32,32) ~ N(0,1), damping 1e-3:
    one full optimizer step (factors 28/577/1153/4097 and 64/128/256/10).

    The 4097x4097 factor of the last layer has rank 128 plus the damping (a
    condition number near 1e6), so two float32 evaluations of G^-1 g A^-1 agree to
    ~1e-3..1e-2 only; the bound there is the float64 result: the HIP path must be
    no further from it than 4x the NumPy formula is."""
    r = np.random.default_rng(2)
    batches = [(r.standard_normal((128, 3, 32, 32)).astype(np.float32), r.integers(0, 10, 128).astype(np.int64))]
    model, ref_model, opt, oracle = run_case(build_cifar_cnn, batches, lr=1e-3, momentum=0.9,
                                             cov_ema_decay=0.99, damping=1e-3)
    # The three convolutions meet rel 1e-3 against the oracle.  The last layer's 4097 x 4097 factor
    # is where two float32 evaluations part: 1e-2 for its weights; its bias row rides on the last
    # column of that inverse, which the NumPy formula itself gets right to 0.7 % only, so 2e-2
    # between the two float32 results there (a bias starts at 0, so after one step it is the update
    # itself) and the float64 criterion below for the bias on its own.
    compare(model, ref_model, opt, oracle, tol_param=1e-3, tol_kf=1e-3,
            loose={'/fc/W': (1e-3, 1e-2), '/fc/b': (2e-2, 2e-2)})
    assert [tuple(c.shape) for fb in opt.fblocks for c in fb.covs] == \
        [(28, 28), (64, 64), (577, 577), (128, 128), (1153, 1153), (256, 256), (4097, 4097), (10, 10)]
    ref_links = dict(ref_model.namedlinks())
    for fb in opt.fblocks:
        W, b = fb.link.W, fb.link.b
        err_hip = kfgrad_errors_vs_float64(
            fb.cov_emas[0].cpu().numpy(), fb.cov_emas[1].cpu().numpy(), W.grad.cpu().numpy(), b.grad.cpu().numpy(),
            W.kfgrad.cpu().numpy(), b.kfgrad.cpu().numpy())
        rl = ref_links[fb.linkname]
        name = fb.linkname
        err_ref = kfgrad_errors_vs_float64(
            oracle.cov_emas[name][0], oracle.cov_emas[name][1], rl.W.grad.numpy(), rl.b.grad.numpy(),
            oracle.kfgrads[(name, 'W')], oracle.kfgrads[(name, 'b')])
        assert err_hip < max(4 * err_ref, 1e-3), (name, err_hip, err_ref)
        # the bias column on its own (it is a 4097th of the block above)
        A64 = np.linalg.inv(fb.cov_emas[0].cpu().numpy().astype(np.float64))
        G64 = np.linalg.inv(fb.cov_emas[1].cpu().numpy().astype(np.float64))
        g = np.column_stack([W.grad.cpu().numpy().reshape(W.grad.shape[0], -1), b.grad.cpu().numpy()])
        kb64 = (G64 @ g.astype(np.float64) @ A64)[:, -1]
        rA64 = np.linalg.inv(oracle.cov_emas[name][0].astype(np.float64))
        rG64 = np.linalg.inv(oracle.cov_emas[name][1].astype(np.float64))
        rg = np.column_stack([rl.W.grad.numpy().reshape(g.shape[0], -1), rl.b.grad.numpy()])
        rkb64 = (rG64 @ rg.astype(np.float64) @ rA64)[:, -1]
        err_hip_b = rel(b.kfgrad.cpu().numpy(), kb64)
        err_ref_b = rel(oracle.kfgrads[(name, 'b')], rkb64)
        assert err_hip_b < max(1.25 * err_ref_b, 2e-4), (name, err_hip_b, err_ref_b)
    # the bordered-matrix path of the inverse (d = 128 m + 1: 577, 1153, 4097) against the path that
    # tiles such matrices whole, on this step's damped factors: what separates the two HIP results
    # is rounding, not the border formula
    from chainerkfac_amd import _lib, ops
    mats = [c.clone() for fb in opt.fblocks for c in fb.cov_emas]
    bordered, _ = ops.spd_inverse_batched(mats)
    with _lib.options(inverse_border=0):
        whole, _ = ops.spd_inverse_batched(mats + [torch.eye(3, device='cuda')])
    for M, a, b in zip(mats, bordered, whole):
        ref64 = np.linalg.inv(M.cpu().numpy().astype(np.float64))
        ea, eb = rel(a.cpu().numpy(), ref64), rel(b.cpu().numpy(), ref64)
        assert ea < max(2 * eb, 1e-5), (M.shape, ea, eb)


def test_accumulation_over_micro_batches():
    batches = cnn_batches(4, bs=8, seed=3)
    model, ref_model, opt, oracle = run_case(build_cnn, batches, lr=1e-2, momentum=0.0, cov_ema_decay=1.0,
                                             damping=1e-2, acc_iters=2)
    compare(model, ref_model, opt, oracle, tol_param=2e-3, tol_kf=5e-3)
    shadow_check(model, ref_model, opt, oracle)
    assert opt.t == 2 and opt.acc_aware_iterations == 2 and opt.acc_count == 0


def test_loss_scale_cancels_end_to_end():
    """KFAC(loss_scale=128): the backward pass runs on 128 * loss, the factors undo the scale
    through gy_scale and the update rule divides the preconditioned gradients back
    (reference kfac.py:72-78), so the step is that of the unscaled loss: judged against the
    oracle run WITHOUT a loss scale on the same model and batch."""
    from chainerkfac_amd import links as L
    from chainerkfac_amd.optimizers import KFAC
    hyper = dict(lr=1e-2, momentum=0.9, cov_ema_decay=1.0, damping=1e-2)
    gen = torch.Generator(device='cpu').manual_seed(7)
    ref_model = build_cnn(L, 'cpu', gen)
    model = build_cnn(L, 'cuda', None)
    copy_params(ref_model, model)
    # a convolution without a Fisher block of its own would take the plain-gradient path;
    # here every parameter has a block, so every update goes through kfgrad
    opt = KFAC(loss_scale=128.0, **hyper).setup(model)
    oracle = OracleKFAC(**hyper)

    def lossfun(m, x, t):
        return TF.cross_entropy(m(x), t)

    for x, t in cnn_batches(2):
        opt.update(lossfun, model, torch.from_numpy(x).cuda(), torch.from_numpy(t).cuda())
        rec = Recorder(L, ref_model)
        ref_model.cleargrads()
        with rec.hook():
            lossfun(ref_model, torch.from_numpy(x), torch.from_numpy(t)).backward()
        oracle.step(rec.records())
    torch.cuda.synchronize()
    for p in model.params():
        assert p._loss_scale == 128.0
    by_name = {fb.linkname: fb for fb in opt.fblocks}
    for name, emas in oracle.cov_emas.items():
        for got, ref in zip(by_name[name].cov_emas, emas):
            assert rel(got.cpu().numpy(), ref) < 1e-4, name
    # kfgrads were divided by the scale in place (reference kfac.py:76-78) and so were the
    # gradients (Chainer's UpdateRule.update, which the reference's rule calls next)
    for (lname, pname), ref in oracle.kfgrads.items():
        got = getattr(by_name[lname].link, pname).kfgrad.cpu().numpy()
        assert rel(got, ref) < 5e-3, (lname, pname)
    ref_params = dict(ref_model.namedparams())
    for name, p in model.namedparams():
        # (the bias of conv1 feeds a batch normalisation: its gradient is zero up to rounding noise)
        if name != '/conv1/b':
            assert rel(p.grad.cpu().numpy(), ref_params[name].grad.numpy()) < 1e-4, name
        assert rel(p.data.cpu().numpy(), ref_params[name].data.numpy()) < 2e-3, name


def test_plain_gradient_path_divides_by_loss_scale():
    """A parameter without a Fisher block is updated from ``grad`` (reference kfac.py:88); with
    a loss scale that gradient is divided back first, as Chainer's UpdateRule.update does."""
    from chainerkfac_amd import links as L
    from chainerkfac_amd.optimizers import KFAC

    class Scale(L.Link):
        def __init__(self):
            super(Scale, self).__init__()
            self.w = L.Parameter(torch.ones(5, device='cuda'))

        def __call__(self, x):
            return x * self.w.tensor

    class Net(L.Chain):
        def __init__(self):
            super(Net, self).__init__()
            self.fc = L.Linear(5, 3, device='cuda', generator=None)
            self.scale = Scale()

        def __call__(self, x):
            return self.fc(self.scale(x))

    torch.manual_seed(0)
    x = torch.randn(4, 5, device='cuda')
    t = torch.tensor([0, 1, 2, 1], device='cuda')
    nets = []
    for ls in (None, 64.0):
        torch.manual_seed(1)
        net = Net()
        opt = KFAC(lr=0.1, momentum=0.0, damping=1e-2, cov_ema_decay=1.0, loss_scale=ls).setup(net)
        assert [fb.linkname for fb in opt.fblocks] == ['/fc']
        opt.update(lambda: TF.cross_entropy(net(x), t))
        nets.append(net)
    torch.cuda.synchronize()
    a, b = nets
    assert not torch.equal(a.scale.w.data, torch.ones(5, device='cuda'))
    assert rel(b.scale.w.data.cpu().numpy(), a.scale.w.data.cpu().numpy()) < 1e-5
    assert rel(b.fc.W.data.cpu().numpy(), a.fc.W.data.cpu().numpy()) < 1e-4


@pytest.mark.parametrize('loss_scale', [None, 64.0])
def test_batched_parameter_updates_match_the_per_parameter_rule(loss_scale):
    """KFAC.batch_param_updates and batch_elementwise: one momentum launch over all parameters
    (and one moving-average launch over all factors) leaves the same
    parameters, velocities, (divided) gradients and step counts as one rule call per
    parameter (momentum and lr_pre exercised over three steps, adjust_momentum on)."""
    from chainerkfac_amd import links as L
    from chainerkfac_amd.optimizers import KFAC

    def lossfun(m, x, t):
        return TF.cross_entropy(m(x), t)

    nets = []
    for batched in (True, False):
        gen = torch.Generator(device='cpu').manual_seed(7)
        src = build_cnn(L, 'cpu', gen)
        model = build_cnn(L, 'cuda', None)
        copy_params(src, model)
        opt = KFAC(lr=1e-2, momentum=0.9, cov_ema_decay=0.9, damping=1e-2, loss_scale=loss_scale,
                   adjust_momentum=True).setup(model)
        opt.batch_param_updates = opt.batch_elementwise = batched
        for step, (x, t) in enumerate(cnn_batches(3)):
            if step == 2:
                opt.hyperparam.lr_pre, opt.hyperparam.lr = opt.hyperparam.lr, 0.5 * opt.hyperparam.lr
            opt.update(lossfun, model, torch.from_numpy(x).cuda(), torch.from_numpy(t).cuda())
        torch.cuda.synchronize()
        nets.append(model)
    a, b = nets
    pb = dict(b.namedparams())
    # (two runs of the same configuration already differ in the last bits: the backward pass
    # of the network is not run-to-run deterministic; that the two kernels round alike is
    # tested on fixed arrays in test_precond_gpu.py)
    for name, p in a.namedparams():
        q = pb[name]
        assert rel(p.data.cpu().numpy(), q.data.cpu().numpy()) < 1e-3, name
        assert rel(p.update_rule.state['v'].cpu().numpy(), q.update_rule.state['v'].cpu().numpy()) < 1e-3, name
        assert p.update_rule.t == q.update_rule.t == 3
        for attr in ('grad', 'kfgrad'):
            ga, gb = getattr(p, attr, None), getattr(q, attr, None)
            assert (ga is None) == (gb is None)
            if ga is not None and name != '/conv1/b':   # (a zero gradient up to rounding noise)
                assert rel(ga.cpu().numpy(), gb.cpu().numpy()) < 1e-3, (name, attr)


def test_side_streams_do_not_change_results(monkeypatch):
    """The per-layer kernels dealt onto side streams are the same launches on the
    same data: factors, inverses and preconditioned gradients are bit-identical to
    the one-stream run.  (Driven through the hook calls on fixed tensors: the
    network's own backward pass is not bit-reproducible from run to run.)"""
    import bench
    from chainerkfac_amd.optimizers import KFAC
    layers = [
        dict(kind='conv', name='c1', c_in=3, c_out=16, k=3, s=1, p=1, bias=True, h=16, w=16),
        dict(kind='bn', name='b1', c=16, h=16, w=16),
        dict(kind='conv', name='c2', c_in=16, c_out=72, k=1, s=1, p=0, bias=True, h=16, w=16),
        dict(kind='bn', name='b2', c=72, h=16, w=16),
        dict(kind='conv', name='c3', c_in=72, c_out=40, k=3, s=2, p=1, bias=False, h=16, w=16),
        dict(kind='conv', name='c4', c_in=40, c_out=40, k=1, s=2, p=0, bias=True, h=8, w=8),
        dict(kind='linear', name='fc', d_in=640, d_out=10, bias=True),
    ]
    outs = []
    for lanes in (0, 3, 2):
        monkeypatch.setattr(KFAC, 'lanes', lanes)
        gen = torch.Generator(device='cuda').manual_seed(11)
        model, calls = bench.build_model(layers, torch.device('cuda:0'), gen)
        opt = KFAC(damping=1e-2, cov_ema_decay=0.9).setup(model)
        assert opt._lanes.n == lanes
        for _ in range(2):   # the second pass runs the moving average
            for _, func, in_data, gy in calls:
                opt.kfhook.forward_postprocess(func, in_data)
                opt.kfhook.backward_preprocess(func, in_data, (gy,))
            opt.reallocate_cleared_grads()
            opt.update_kfgrads(opt.fblocks)
        torch.cuda.synchronize()
        got = []
        for fb in opt.fblocks:
            got += [(fb.linkname, 'cov', c.cpu().numpy()) for c in fb.cov_emas]
            got += [(fb.linkname, 'inv', c.cpu().numpy()) for c in fb.invs]
        got += [(n, 'kfgrad', p.kfgrad.cpu().numpy()) for n, p in sorted(model.namedparams())]
        outs.append(got)
    for other in outs[1:]:
        assert len(other) == len(outs[0])
        for (n0, k0, a0), (n1, k1, a1) in zip(outs[0], other):
            assert (n0, k0) == (n1, k1)
            assert np.array_equal(a0, a1), (n0, k0)


@pytest.mark.parametrize('decay', [1.0, 0.9])
def test_step_replayed_from_a_hip_graph_matches_the_eager_step(monkeypatch, decay):
    """The benchmark times the step as a HIP-graph replay with four lanes (and the
    library's own side streams forked inside the capture).  Every replay must leave
    exactly what the eager step leaves: two optimizers built from the same seed run
    in lockstep, one eagerly and one replaying its captured step, with unrelated
    eager work and synchronisations between the replays.  decay 1: every step is a
    first step (factors aliased, rank-n batch-norm inverses); decay 0.9: the moving
    average carries history from replay to replay."""
    import bench
    from chainerkfac_amd.optimizers import KFAC
    layers = [
        dict(kind='conv', name='c0', c_in=3, c_out=64, k=3, s=1, p=1, bias=True, h=14, w=14),
        dict(kind='bn', name='b0', c=64, h=14, w=14),
        dict(kind='conv', name='c1', c_in=64, c_out=64, k=3, s=1, p=1, bias=True, h=14, w=14),   # shifted correlations, d = 577
        dict(kind='bn', name='b1', c=64, h=14, w=14),
        dict(kind='conv', name='c2', c_in=64, c_out=136, k=1, s=1, p=0, bias=True, h=14, w=14),
        dict(kind='conv', name='c3', c_in=136, c_out=40, k=3, s=2, p=1, bias=False, h=14, w=14),
        dict(kind='conv', name='c4', c_in=40, c_out=256, k=1, s=1, p=0, bias=True, h=7, w=7),   # d = 257: bordered inverse
        dict(kind='linear', name='fc', d_in=640, d_out=10, bias=True),
    ]
    monkeypatch.setattr(KFAC, 'lanes', 4)
    dev = torch.device('cuda:0')

    def make():
        gen = torch.Generator(device='cuda').manual_seed(23)
        model, calls = bench.build_model(layers, dev, gen, 8)
        opt = KFAC(damping=1e-2, cov_ema_decay=decay).setup(model)
        assert opt._lanes.n == 4

        def step():
            for _, func, in_data, gy in calls:
                opt.kfhook.forward_postprocess(func, in_data)
                opt.kfhook.backward_preprocess(func, in_data, (gy,))
            opt.finish_covs()
            opt.update_cov_emas(opt.fblocks)
            opt.update_invs_batched(opt.fblocks)
            opt.precondition(opt.fblocks)
        opt.reallocate_cleared_grads()
        return model, opt, step

    def state(model, opt):
        torch.cuda.synchronize()
        got = []
        for fb in opt.fblocks:
            got += [(fb.linkname, 'cov', c.cpu().numpy()) for c in fb.cov_emas]
            got += [(fb.linkname, 'inv', c.cpu().numpy()) for c in fb.invs]
        got += [(n, 'kfgrad', p.kfgrad.cpu().numpy()) for n, p in sorted(model.namedparams())]
        return got

    eager_model, eager_opt, eager_step = make()
    graph_model, graph_opt, graph_step = make()
    for _ in range(2):   # plans, device tables and lane workspaces exist before the capture
        eager_step()
        graph_step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        graph_step()
    scratch = torch.randn(512, 512, device=dev)
    for replay in range(3):
        eager_step()
        graph.replay()
        a, b = state(eager_model, eager_opt), state(graph_model, graph_opt)
        assert len(a) == len(b) and len(a) > 30
        for (n0, k0, x0), (n1, k1, x1) in zip(a, b):
            assert (n0, k0) == (n1, k1)
            assert np.isfinite(x0).all(), (replay, n0, k0)
            assert np.array_equal(x0, x1), (replay, n0, k0)
        # the program's own eager work between the replays
        scratch = torch.tanh(scratch @ scratch)
        assert not eager_opt.check_numerics() and not graph_opt.check_numerics()
        torch.cuda.synchronize()


def test_constructor_defaults_and_plugin_seam():
    from chainerkfac_amd import links as L
    from chainerkfac_amd.optimizers import KFAC, fblock_constructor
    from chainerkfac_amd.optimizers import fisher_blocks as FB
    opt = KFAC()
    assert (opt.lr, opt.momentum, opt.cov_ema_decay, opt.damping, opt.stab_coeff) == (0.001, 0.9, 0.99, 0.03, 16.0)
    assert set(opt.constructor_kwargs) == {'cov_ema_decay', 'damping', 'use_cholesky', 'pi_type', 'stab_coeff',
                                           'loss_scale'}
    seen = []

    def constructor(name, link, **kw):
        seen.append(name)
        return fblock_constructor(name, link, **kw)

    model = build_cnn(L, 'cuda', None)
    opt = KFAC(constructor=constructor).setup(model)
    assert seen == sorted(seen) and seen[0] == '/'
    kinds = [type(fb) for fb in opt.fblocks]
    assert kinds == [FB.FisherBlockBatchNormalization, FB.FisherBlockBatchNormalization, FB.FisherBlockConvolution2D,
                     FB.FisherBlockConvolution2D, FB.FisherBlockConvolution2D, FB.FisherBlockLinear]
    with pytest.raises(RuntimeError):
        opt.fblocks[0].check_attr('covs')
    bn = L.BatchNormalization(4, use_gamma=False, use_beta=False)
    assert fblock_constructor('/bn', bn, **opt.constructor_kwargs) is None
    with pytest.raises(AssertionError):
        KFAC(acc_iters=0)


def test_buffer_order_of_extract_helpers():
    """grads in sorted parameter-name order, then A, then G (BN: grads, then F)."""
    out = run_case(build_cnn, cnn_batches(1), damping=1e-2, cov_ema_decay=1.0)
    opt = out[2]
    by_name = {fb.linkname: fb for fb in opt.fblocks}
    conv = by_name['/conv1']
    arrays = conv.extract_for_reduce_scatter_v()
    assert [t for _, t in arrays] == [False, False, True, True]
    assert arrays[0][0] is conv.link.W.grad and arrays[1][0] is conv.link.b.grad
    assert arrays[2][0] is conv.cov_forward and arrays[3][0] is conv.cov_backward
    bn = by_name['/bn1']
    arrays = bn.extract_for_reduce_scatter_v()
    assert [t for _, t in arrays] == [False, False, True]
    assert arrays[0][0] is bn.link.beta.grad and arrays[1][0] is bn.link.gamma.grad   # '/beta' < '/gamma'
    assert [a.shape for a, _ in conv.extract_for_all_gather_v('kfgrad')] == [conv.link.W.shape, conv.link.b.shape]


def test_extract_builds_the_per_rank_lists_the_packer_consumes():
    """``extract(blocks, indices, extractor)`` (reference kfac.py:456-464) defines the wire
    order: per rank, the owned blocks in index order, each block's arrays in its own order.
    Its output goes straight into the packer; unpacking into fresh arrays restores every
    gradient and both triangles of every factor bit for bit, and a rank-filtered pack
    fills exactly that rank's segment of the buffer."""
    from chainerkfac_amd.communicators import ArrayPacker
    from chainerkfac_amd.optimizers.kfac import extract
    out = run_case(build_cnn, cnn_batches(1), damping=1e-2, cov_ema_decay=1.0)
    opt = out[2]
    n = len(opt.fblocks)
    indices = [list(range(0, 2)), list(range(2, n))]      # two "ranks", contiguous runs of blocks
    arrays = extract(opt.fblocks, indices, lambda b: b.extract_for_reduce_scatter_v())
    assert len(arrays) == 2
    flat = [a for fb in opt.fblocks for a in fb.extract_for_reduce_scatter_v()]
    assert [id(a) for local in arrays for a, _ in local] == [id(a) for a, _ in flat]
    assert [len(local) for local in arrays] == [sum(len(fb.extract_for_reduce_scatter_v()) for fb in opt.fblocks[:2]),
                                                sum(len(fb.extract_for_reduce_scatter_v()) for fb in opt.fblocks[2:])]
    packer = ArrayPacker()
    nel = packer.get_nelems(arrays)
    host = [[(a.cpu().numpy(), t) for a, t in local] for local in arrays]
    assert nel == O.get_nelems(host)
    buf = torch.zeros(nel, dtype=torch.float32, device='cuda')
    packer._pack_arrays_to_buffer(arrays, buf)
    ref = np.zeros(nel, np.float32)
    O.pack(host, ref)
    assert np.array_equal(buf.cpu().numpy(), ref)
    back = [[(torch.full_like(a, float('nan')), t) for a, t in local] for local in arrays]
    packer._unpack_arrays_from_buffer(back, buf)
    for local, local_back in zip(arrays, back):
        for (a, _), (b, _) in zip(local, local_back):
            assert torch.equal(a, b)
    # rank 1 only: the first rank's segment stays untouched
    buf1 = torch.full_like(buf, -7.0)
    packer._pack_arrays_to_buffer(arrays, buf1, target=1)
    n0 = O.get_nelems([host[0]])
    assert bool((buf1[:n0] == -7.0).all()) and np.array_equal(buf1[n0:].cpu().numpy(), ref[n0:])
    assert extract(opt.fblocks, [[], [1]], lambda b: b.extract_for_all_gather_v('kfgrad'))[0] == []


def test_float16_activations_and_gradients_are_cast_up():
    """float16 activations / output gradients give the factors of their float32 values, and a
    float16 gradient is preconditioned in float32 and handed back as float16 (reference
    linear.py:22-23, 38-39, 55-61; convolution_2d.py:35-37, 57-66; batch_normalization.py:122-129)."""
    from chainerkfac_amd import links
    from chainerkfac_amd.optimizers import fisher_blocks as FB
    g = torch.Generator(device='cuda').manual_seed(5)

    def rnd(*shape):
        return torch.randn(*shape, device='cuda', generator=g)

    kw = dict(cov_ema_decay=1.0, damping=1e-2)
    lin = links.Linear(24, 12, generator=g)
    fb = FB.FisherBlockLinear('/l', lin, **kw)
    x16, gy16 = rnd(16, 24).half(), rnd(16, 12).half()
    a16 = fb.compute_A((x16, lin.W.data, lin.b.data)).clone()
    a32 = fb.compute_A((x16.float(), lin.W.data, lin.b.data)).clone()
    g16 = fb.compute_G((x16,), (gy16,)).clone()
    g32 = fb.compute_G((x16,), (gy16.float(),)).clone()
    assert torch.equal(a16, a32) and torch.equal(g16, g32)

    conv = links.Convolution2D(6, 8, 3, pad=1, generator=g)
    fc = FB.FisherBlockConvolution2D('/c', conv, **kw)
    xc, gc = rnd(4, 6, 8, 8).half(), rnd(4, 8, 8, 8).half()
    assert torch.equal(fc.compute_A((xc, conv.W.data, conv.b.data)).clone(),
                       fc.compute_A((xc.float(), conv.W.data, conv.b.data)).clone())
    assert torch.equal(fc.compute_G((xc,), (gc,)).clone(), fc.compute_G((xc,), (gc.float(),)).clone())

    bn = links.BatchNormalization(8)
    fbn = FB.FisherBlockBatchNormalization('/bn', bn, **kw)
    xb, gb = rnd(4, 8, 5, 5).half(), rnd(4, 8, 5, 5).half()
    f16 = fbn.compute_F((xb, bn.gamma.data, bn.beta.data), (gb,)).clone()
    f32 = fbn.compute_F((xb.float(), bn.gamma.data, bn.beta.data), (gb.float(),)).clone()
    assert torch.equal(f16, f32)

    # preconditioning of float16 gradients: float32 products of the cast gradients, float16 result
    fb.forward_postprocess(None, (x16, lin.W.data, lin.b.data))
    fb.backward_preprocess(None, (x16,), (gy16,))
    fb.update_cov_emas()
    fb.update_invs()
    gw, gbias = rnd(12, 24).half(), rnd(12).half()

    class Half(object):
        def __init__(self, p, grad):
            self.p, self.grad, self.kfgrad = p, grad, None
            self.shape, self.data = p.shape, p.data

    lin.W, lin.b = Half(lin.W, gw), Half(lin.b, gbias)
    fb.update_kfgrads()
    assert lin.W.kfgrad.dtype == torch.float16 and lin.b.kfgrad.dtype == torch.float16
    A_inv, G_inv = [m.double() for m in fb.invs]
    full = G_inv @ torch.cat([gw.double(), gbias.double()[:, None]], dim=1) @ A_inv
    got = torch.cat([lin.W.kfgrad.double(), lin.b.kfgrad.double()[:, None]], dim=1)
    assert (got - full).norm() <= 2e-3 * full.norm()


@pytest.mark.parametrize('batched', [False, True])
def test_float16_parameter_is_updated_through_a_float32_master_copy(batched):
    """reference kfac.py:64-85: the update runs on a float32 copy; the float16 parameter follows.
    ``batched``: through the rule's job for the one launch that takes all parameters."""
    from chainerkfac_amd import ops
    from chainerkfac_amd.optimizers.kfac import KFACUpdateRule, Hyperparameter

    class P(object):
        pass

    g = torch.Generator(device='cuda').manual_seed(6)
    p = P()
    p.data = torch.randn(257, device='cuda', generator=g).half()
    p.grad = None
    p._loss_scale = 8.0
    hp = Hyperparameter()
    hp.lr, hp.lr_pre, hp.momentum = 0.01, 0.01, 0.9
    rule = KFACUpdateRule(hp)
    master = p.data.double()
    v = torch.zeros_like(master)
    for _ in range(3):
        p.kfgrad = (torch.randn(257, device='cuda', generator=g) * 8.0).half()
        kf = p.kfgrad.double() / 8.0
        kf16 = p.kfgrad.clone()
        if batched:
            job = rule.batched_job(p)
            lr, momentum, loss_scale = job['key']
            ops.momentum_update_batched([job['param']], [job['v']], [job['grad']], lr, momentum, loss_scale,
                                        [job['write_back']], [job['param_f16']])
        else:
            rule.update(p)
        assert torch.equal(p.kfgrad, kf16)   # divided in a float32 copy, not in place
        v = 0.9 * v - 0.01 * kf
        master = master + v
        assert p.data.dtype == torch.float16
        # the float16 parameter is the rounded master copy, not an accumulation of rounded steps
        assert torch.equal(p.data, rule._fp32_param.half())
        assert (rule._fp32_param.double() - master).abs().max() <= 1e-5


def test_float32_parameter_with_float16_gradients_and_both_divisions():
    """A float32 parameter whose gradients arrive in float16 (the batched launch does not take the
    pair and hands it to the per-parameter rule, which casts up), and the two in-place divisions of
    a scaled loss: ``kfgrad`` by the reference's rule (kfac.py:76-78), ``grad`` by Chainer's
    UpdateRule.update, also on the batched path."""
    from chainerkfac_amd import links as L
    from chainerkfac_amd.optimizers import KFAC
    from chainerkfac_amd.optimizers.kfac import KFACUpdateRule, Hyperparameter

    class P(object):
        pass

    g = torch.Generator(device='cuda').manual_seed(8)
    hp = Hyperparameter()
    hp.lr, hp.lr_pre, hp.momentum = 0.1, 0.1, 0.0
    p = P()
    p.data = torch.randn(100, device='cuda', generator=g)
    before = p.data.clone()
    p.grad = torch.randn(100, device='cuda', generator=g).half()
    p.kfgrad = p.grad.clone()
    p._loss_scale = None
    rule = KFACUpdateRule(hp)
    assert rule.batched_job(p) is NotImplemented
    rule.t = 0
    rule.update(p)
    assert torch.allclose(p.data, before - 0.1 * p.kfgrad.float(), rtol=1e-6, atol=1e-7)
    # both arrays of a float32 parameter are divided by the loss scale
    for batched in (False, True):
        model = L.Chain()
        model.fc = L.Linear(6, 4, device='cuda')
        opt = KFAC(lr=0.1, momentum=0.0, loss_scale=4.0).setup(model)
        opt.batch_param_updates = batched
        for q in model.params():
            q.grad = torch.full(q.data.shape, 8.0, device='cuda')
            q.kfgrad = torch.full(q.data.shape, 2.0, device='cuda')
            q._loss_scale = 4.0
        start = [q.data.clone() for q in model.params()]
        opt.update_params()
        torch.cuda.synchronize()
        for q, s0 in zip(model.params(), start):
            assert torch.equal(q.grad, torch.full_like(q.grad, 2.0))
            assert torch.equal(q.kfgrad, torch.full_like(q.kfgrad, 0.5))
            assert torch.allclose(q.data, s0 - 0.1 * 0.5)
