"""Pins for the oracle's optimizer-step chain (oracle/kfac_step.py), no GPU.

``OracleKFAC.step`` is what every end-to-end GPU test is judged against, so it
is itself checked here against an independent float64 restatement of the
reference's step (chainerkfac/optimizers/kfac.py:222-310,
fisher_block.py:155-179, fisher_blocks/connection.py:51-77,
normalizations/batch_normalization.py:78-191) that shares no code with the
oracle: factors from ``torch.nn.functional.unfold`` / explicit batch statistics,
``numpy.linalg.inv`` instead of the Cholesky formula, the preconditioned
gradient from an explicit Kronecker-product solve, and the state the reference
carries from step to step (moving average with the weight on the new factor,
the damped diagonal left inside the moving average, momentum, accumulation)
written out by hand.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

from oracle.kfac_step import LayerRecord, OracleKFAC

EPS = 2e-5


def rel(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300)


# ---------------------------------------------------------------------------
# a tiny Conv(bias) -> BN -> ReLU -> Conv(stride 2, no bias) -> Linear(bias) net
# ---------------------------------------------------------------------------

def init_params(seed=0):
    g = torch.Generator().manual_seed(seed)
    return {
        'c1': {'W': torch.randn(3, 2, 3, 3, generator=g) * 0.4, 'b': torch.randn(3, generator=g) * 0.1},
        'bn': {'gamma': 1 + 0.1 * torch.randn(3, generator=g), 'beta': 0.1 * torch.randn(3, generator=g)},
        'c2': {'W': torch.randn(4, 3, 3, 3, generator=g) * 0.3},
        'fc': {'W': torch.randn(5, 36, generator=g) * 0.2, 'b': torch.randn(5, generator=g) * 0.1},
    }


def forward_backward(params, x, t, loss_scale=None):
    """One forward/backward of the net; returns per layer what the reference's
    function hooks see: the layer input, the gradient of the (scaled) loss with
    respect to the layer output, and the parameter gradients."""
    leaves = {ln: {pn: p.clone().requires_grad_(True) for pn, p in ps.items()} for ln, ps in params.items()}
    seen = {}

    def tap(name, inp, out):
        out.retain_grad()
        seen[name] = (inp.detach(), out)
        return out

    h0 = x
    h1 = tap('c1', h0, TF.conv2d(h0, leaves['c1']['W'], leaves['c1']['b'], 1, 1))
    h2 = tap('bn', h1, TF.batch_norm(h1, None, None, leaves['bn']['gamma'], leaves['bn']['beta'], True, 0.1, EPS))
    h3 = TF.relu(h2)
    h4 = tap('c2', h3, TF.conv2d(h3, leaves['c2']['W'], None, 2, 1))
    h5 = TF.relu(h4).reshape(x.shape[0], -1)
    h6 = tap('fc', h5, TF.linear(h5, leaves['fc']['W'], leaves['fc']['b']))
    loss = TF.cross_entropy(h6, t)
    (loss * loss_scale if loss_scale is not None else loss).backward()
    out = {}
    for name, (inp, o) in seen.items():
        out[name] = {'x': inp.numpy().copy(), 'gy': o.grad.numpy().copy(),
                     'grads': {pn: p.grad.numpy().copy() for pn, p in leaves[name].items()}}
    return out


KINDS = {'c1': ('conv', dict(ksize=3, stride=1, pad=1)), 'bn': ('bn', dict(eps=EPS)),
         'c2': ('conv', dict(ksize=3, stride=2, pad=1)), 'fc': ('linear', {})}


def batches(n, bs=6, seed=5):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(bs, 2, 6, 6, generator=g), torch.randint(0, 5, (bs,), generator=g)) for _ in range(n)]


# ---------------------------------------------------------------------------
# independent float64 restatement of the reference's step
# ---------------------------------------------------------------------------

class Float64KFAC(object):

    def __init__(self, lr, momentum, decay, damping, stab_coeff=16.0, loss_scale=None, acc_iters=1,
                 leak_damping_into_ema=True):
        self.lr, self.mu, self.decay, self.damping = lr, momentum, decay, damping
        self.stab, self.ls, self.acc_iters = stab_coeff, loss_scale, acc_iters
        self.leak = leak_damping_into_ema
        self.ema = {}
        self.v = {}
        self.acc = []
        self.kf = {}
        self.inv = {}

    def factors(self, name, x, gy):
        kind, attrs = KINDS[name]
        x = torch.from_numpy(x).double()
        gy = torch.from_numpy(gy).double()
        n = x.shape[0]
        s = n / (self.ls if self.ls is not None else 1.0)      # undoes the mean reduction and the loss scale
        if kind == 'linear':
            xe = torch.cat([x, torch.ones(n, 1, dtype=torch.float64)], 1)
            return [(xe.T @ xe / n).numpy(), ((gy * s).T @ (gy * s) / n).numpy()]
        if kind == 'conv':
            cols = TF.unfold(x, attrs['ksize'], padding=attrs['pad'], stride=attrs['stride'])   # (n, c*k*k, L)
            P = cols.permute(0, 2, 1).reshape(-1, cols.shape[1])
            if name == 'c1':                                   # the layer with a bias
                P = torch.cat([P, torch.ones(P.shape[0], 1, dtype=torch.float64)], 1)
            A = P.T @ P / n
            g = gy.permute(0, 2, 3, 1).reshape(-1, gy.shape[1])
            G = g.T @ g * s * s / g.shape[0]
            return [A.numpy(), G.numpy()]
        mean = x.mean(dim=(0, 2, 3), keepdim=True)
        var = ((x - mean) ** 2).mean(dim=(0, 2, 3), keepdim=True)
        h = (x - mean) / torch.sqrt(var + attrs['eps'])
        U = torch.cat([(gy * s * h).sum(dim=(2, 3)), (gy * s).sum(dim=(2, 3))], 1)   # gamma half first
        return [(U.T @ U / n).numpy()]

    def step(self, fb, params):
        """fb: output of forward_backward; params: dict of float64 arrays, updated in place."""
        covs = {name: self.factors(name, d['x'], d['gy']) for name, d in fb.items()}
        grads = {(name, pn): g.astype(np.float64) for name, d in fb.items() for pn, g in d['grads'].items()}
        if self.acc_iters > 1:
            self.acc.append((covs, grads))
            if len(self.acc) < self.acc_iters:
                return False
            covs = {name: [sum(c[0][name][i] for c in self.acc) / self.acc_iters for i in range(len(covs[name]))]
                    for name in covs}
            grads = {k: sum(c[1][k] for c in self.acc) / self.acc_iters for k in grads}
            self.acc = []
        for name in sorted(covs):
            kind, _ = KINDS[name]
            if self.decay == 1.0 or name not in self.ema:
                ema = [c.copy() for c in covs[name]]
            else:                                              # weight `decay` on the NEW factor
                ema = [self.decay * c + (1 - self.decay) * e for c, e in zip(covs[name], self.ema[name])]
            if kind == 'bn':
                damped = [ema[0] + self.stab * self.damping * np.eye(ema[0].shape[0])]
            else:
                A, G = ema
                pi = np.sqrt((np.trace(A) * G.shape[0]) / (np.trace(G) * A.shape[0]))
                r = np.sqrt(self.damping)
                damped = [A + pi * r * np.eye(A.shape[0]), G + r / pi * np.eye(G.shape[0])]
            # the reference adds the damping to the moving average in place, so it is still in
            # there when the next step mixes in the new factor
            self.ema[name] = damped if self.leak else ema
            invs = [np.linalg.inv(m) for m in damped]
            self.inv[name] = invs
            if kind == 'bn':
                g = np.concatenate([grads[(name, 'gamma')], grads[(name, 'beta')]])
                k = np.linalg.solve(damped[0], g)
                kf = {'gamma': k[:3], 'beta': k[3:]}
            else:
                gW = grads[(name, 'W')]
                g = gW.reshape(gW.shape[0], -1)
                if (name, 'b') in grads:
                    g = np.column_stack([g, grads[(name, 'b')]])
                # (A (x) G) vec(K) = vec(g), vec = column stacking  <=>  G K A = g
                K = np.linalg.solve(np.kron(damped[0], damped[1]), g.flatten('F')).reshape(g.shape, order='F')
                kf = {'W': K[:, :gW[0].size].reshape(gW.shape)}
                if (name, 'b') in grads:
                    kf['b'] = K[:, -1]
            for pn, k in kf.items():
                if self.ls is not None:
                    k = k / self.ls
                self.kf[(name, pn)] = k
                v = self.v.setdefault((name, pn), np.zeros_like(params[name][pn]))
                v *= self.mu
                v -= self.lr * k
                params[name][pn] += v
        return True


def run_both(n_steps, bs=6, loss_scale=None, acc_iters=1, leak=True, **hyper):
    """Drives the float32 oracle and the float64 restatement with the same
    recorded layer tensors (taken from the oracle's float32 parameters)."""
    p32 = {ln: {pn: p.numpy().copy() for pn, p in ps.items()} for ln, ps in init_params().items()}
    p64 = {ln: {pn: p.astype(np.float64) for pn, p in ps.items()} for ln, ps in p32.items()}
    oracle = OracleKFAC(lr=hyper['lr'], momentum=hyper['momentum'], cov_ema_decay=hyper['decay'],
                        damping=hyper['damping'], stab_coeff=16.0, loss_scale=loss_scale, acc_iters=acc_iters)
    ref = Float64KFAC(hyper['lr'], hyper['momentum'], hyper['decay'], hyper['damping'], 16.0, loss_scale,
                      acc_iters, leak_damping_into_ema=leak)
    for x, t in batches(n_steps, bs):
        fb = forward_backward({ln: {pn: torch.from_numpy(p) for pn, p in ps.items()} for ln, ps in p32.items()},
                              x, t, loss_scale)
        records = [LayerRecord(KINDS[name][0], name, d['x'], d['gy'], p32[name], d['grads'], **KINDS[name][1])
                   for name, d in fb.items()]
        updated = oracle.step(records)
        assert updated == ref.step(fb, p64)
    return oracle, ref, p32, p64


def check(oracle, ref, p32, p64, tol=2e-5):
    for name, invs in ref.inv.items():
        for got, want in zip(oracle.invs[name], invs):
            assert got.dtype == np.float32
            assert rel(got, want) < tol, name
    for key, want in ref.kf.items():
        assert rel(oracle.kfgrads[key], want) < tol, key
    for ln in p64:
        for pn in p64[ln]:
            assert rel(p32[ln][pn], p64[ln][pn]) < tol, (ln, pn)


HYPER = dict(lr=1e-2, momentum=0.9, decay=0.9, damping=1e-2)


def test_one_step_matches_float64_closed_form():
    out = run_both(1, **HYPER)
    check(*out)
    oracle = out[0]
    # block order is the sorted link-name order and every parameter got a kfgrad
    assert sorted(oracle.kfgrads) == [('bn', 'beta'), ('bn', 'gamma'), ('c1', 'W'), ('c1', 'b'), ('c2', 'W'),
                                      ('fc', 'W'), ('fc', 'b')]
    # p1 = p0 - lr * kfgrad on the first step (v starts at 0)
    p0 = {ln: {pn: p.numpy() for pn, p in ps.items()} for ln, ps in init_params().items()}
    for (ln, pn), k in oracle.kfgrads.items():
        np.testing.assert_allclose(out[2][ln][pn], p0[ln][pn] - 1e-2 * k, rtol=1e-5, atol=1e-7)


def test_three_steps_moving_average_keeps_the_damped_diagonal():
    """With decay != 1 the reference's in-place damping stays inside the moving
    average (fisher_block.py:162-175): the oracle must follow the restatement
    that carries the damped matrix forward, and must differ from the one that
    does not by much more than the tolerance."""
    oracle, ref, p32, p64 = run_both(3, **HYPER)
    check(oracle, ref, p32, p64)
    for name, emas in ref.ema.items():
        for got, want in zip(oracle.cov_emas[name], emas):
            assert rel(got, want) < 1e-5, name
    _, clean, _, q64 = run_both(3, leak=False, **HYPER)
    gaps = [rel(clean.inv[name][i], ref.inv[name][i]) for name in ref.inv for i in range(len(ref.inv[name]))]
    assert min(gaps) > 1e-3, gaps          # every factor's inverse shows the leak
    worst = max(rel(oracle.invs[name][i], clean.inv[name][i]) for name in ref.inv for i in range(len(ref.inv[name])))
    assert worst > 1e-3


def test_decay_one_has_no_history():
    """decay == 1: the moving average is the current factor every step."""
    oracle, ref, p32, p64 = run_both(2, lr=1e-2, momentum=0.5, decay=1.0, damping=1e-2)
    check(oracle, ref, p32, p64)


def test_accumulation_is_the_mean_over_micro_batches():
    """acc_iters = 2 (kfac.py:259-304): factors and gradients are the means over
    the micro-batches, parameters move only on the second one, and the
    accumulators start afresh afterwards."""
    oracle, ref, p32, p64 = run_both(4, acc_iters=2, **HYPER)
    check(oracle, ref, p32, p64)
    assert oracle.acc_count == 0
    # first micro-batch alone changes nothing
    o1, r1, q32, q64 = run_both(1, acc_iters=2, **HYPER)
    p0 = init_params()
    for ln in q32:
        for pn in q32[ln]:
            assert np.array_equal(q32[ln][pn], p0[ln][pn].numpy())
    assert o1.kfgrads == {} and o1.acc_count == 1


def test_loss_scale_cancels():
    """Gradients of loss * s carry s; the factors undo it through gy * n / s
    (connections/linear.py:34-41) and the update rule divides the preconditioned
    gradient by s (kfac.py:72-78): the step is that of the unscaled loss."""
    plain = run_both(2, **HYPER)
    scaled = run_both(2, loss_scale=128.0, **HYPER)
    check(*scaled)
    for ln in plain[2]:
        for pn in plain[2][ln]:
            assert rel(scaled[2][ln][pn], plain[2][ln][pn]) < 1e-5, (ln, pn)
    # and the unscaled kfgrads the two oracles keep agree as well
    for key, k in plain[0].kfgrads.items():
        assert rel(scaled[0].kfgrads[key], k) < 1e-4, key
