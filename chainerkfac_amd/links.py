"""Minimal link / parameter / function-hook layer standing in for the parts of
Chainer that the K-FAC optimizer touches.

The reference is a Chainer plug-in: it walks ``link.namedlinks()``, reads
``link.W / b / gamma / beta / ksize / stride / pad / eps / avg_mean`` and is
driven by Chainer function hooks (``forward_postprocess(function, in_data)`` /
``backward_preprocess(function, in_data, out_grad)``).  Chainer is not
available here, so this module supplies objects with those attributes on top of
torch-ROCm tensors; the model's own forward/backward runs through torch
autograd and is not part of the K-FAC path.
"""
import math
import threading

import torch
import torch.nn.functional as TF


class Parameter(object):
    """A named array with ``data``, ``grad`` and (set by K-FAC) ``kfgrad``."""

    def __init__(self, tensor, name=None):
        self._t = tensor.detach().clone().requires_grad_(True)
        self._data = self._t.detach()   # stable alias used for identity checks
        self.name = name
        self.update_rule = None
        self._loss_scale = None

    @property
    def data(self):
        return self._data

    array = data

    @property
    def tensor(self):
        """The autograd leaf used when the link is called."""
        return self._t

    @property
    def grad(self):
        return self._t.grad

    @grad.setter
    def grad(self, value):
        self._t.grad = value

    @property
    def shape(self):
        return tuple(self._t.shape)

    @property
    def dtype(self):
        return self._t.dtype

    @property
    def size(self):
        return self._t.numel()

    def cleargrad(self):
        self._t.grad = None

    def update(self):
        if self.update_rule is not None:
            self.update_rule.update(self)


class Link(object):
    """Container of parameters and child links (attribute order = registration order)."""

    def __init__(self):
        object.__setattr__(self, '_params', [])
        object.__setattr__(self, '_children', [])
        self.name = None

    def __setattr__(self, key, value):
        if isinstance(value, Parameter):
            if key not in self._params:
                self._params.append(key)
            value.name = key
        elif isinstance(value, Link) and key != 'link':
            if key not in self._children:
                self._children.append(key)
            value.name = key
        object.__setattr__(self, key, value)

    @property
    def xp(self):
        return torch

    def params(self, include_uninit=True):
        for _, p in self.namedparams(include_uninit):
            yield p

    def namedparams(self, include_uninit=True):
        for key in self._params:
            p = getattr(self, key)
            if p is not None:
                yield '/' + key, p
        for key in self._children:
            prefix = '/' + key
            for path, p in getattr(self, key).namedparams(include_uninit):
                yield prefix + path, p

    def namedlinks(self, skipself=False):
        if not skipself:
            yield '/', self
        for key in self._children:
            child = getattr(self, key)
            prefix = '/' + key
            yield prefix, child
            for path, link in child.namedlinks(True):
                yield prefix + path, link

    def links(self, skipself=False):
        for _, l in self.namedlinks(skipself):
            yield l

    def cleargrads(self):
        for p in self.params():
            p.cleargrad()

    def zerograds(self):
        for p in self.params():
            if p.grad is not None:
                p.grad.zero_()


class Chain(Link):
    pass


class ChainList(Link):
    def __init__(self, *links):
        super(ChainList, self).__init__()
        self._list = []
        for l in links:
            self.add_link(l)

    def add_link(self, link):
        setattr(self, str(len(self._list)), link)
        self._list.append(link)

    def __iter__(self):
        return iter(self._list)

    def __len__(self):
        return len(self._list)

    def __getitem__(self, i):
        return self._list[i]


# ---------------------------------------------------------------------------
# function hooks
# ---------------------------------------------------------------------------

_local = threading.local()


def _active_hooks():
    hooks = getattr(_local, 'hooks', None)
    if hooks is None:
        hooks = _local.hooks = []
    return hooks


class FunctionHook(object):
    """``with hook:`` makes the hook receive every link-function call."""

    def __enter__(self):
        _active_hooks().append(self)
        return self

    def __exit__(self, *exc):
        _active_hooks().remove(self)

    def forward_postprocess(self, function, in_data):
        pass

    def backward_preprocess(self, function, in_data, out_grad_data):
        pass


class LinearFunction(object):
    pass


class Convolution2DFunction(object):
    pass


class BatchNormalizationFunction(object):
    pass


def _dispatch(function, in_data, y):
    hooks = list(_active_hooks())
    if not hooks:
        return y
    for h in hooks:
        h.forward_postprocess(function, in_data)
    if y.requires_grad:
        def _on_grad(gy):
            for h in hooks:
                h.backward_preprocess(function, in_data, (gy.contiguous(),))
        y.register_hook(_on_grad)
    return y


def _he_normal(shape, fan_in, device, generator):
    return torch.randn(shape, device=device, generator=generator) * math.sqrt(2.0 / fan_in)


class Linear(Link):
    def __init__(self, in_size, out_size, nobias=False, device='cuda', generator=None):
        super(Linear, self).__init__()
        self.W = Parameter(_he_normal((out_size, in_size), in_size, device, generator))
        self.b = None if nobias else Parameter(torch.zeros(out_size, device=device))

    def __call__(self, x):
        if x.ndim > 2:
            x = x.reshape(x.shape[0], -1)
        x = x.contiguous()
        b = self.b
        y = TF.linear(x, self.W.tensor, None if b is None else b.tensor)
        in_data = (x.detach(), self.W.data) + (() if b is None else (b.data,))
        return _dispatch(LinearFunction(), in_data, y)


class Convolution2D(Link):
    def __init__(self, in_channels, out_channels, ksize, stride=1, pad=0, nobias=False,
                 device='cuda', generator=None):
        super(Convolution2D, self).__init__()
        self.ksize = ksize
        self.stride = (stride, stride) if isinstance(stride, int) else tuple(stride)
        self.pad = (pad, pad) if isinstance(pad, int) else tuple(pad)
        fan_in = in_channels * ksize * ksize
        self.W = Parameter(_he_normal((out_channels, in_channels, ksize, ksize), fan_in, device, generator))
        self.b = None if nobias else Parameter(torch.zeros(out_channels, device=device))

    def __call__(self, x):
        x = x.contiguous()
        b = self.b
        y = TF.conv2d(x, self.W.tensor, None if b is None else b.tensor, self.stride, self.pad)
        in_data = (x.detach(), self.W.data) + (() if b is None else (b.data,))
        return _dispatch(Convolution2DFunction(), in_data, y)


class BatchNormalization(Link):
    def __init__(self, size, decay=0.9, eps=2e-5, use_gamma=True, use_beta=True, device='cuda'):
        super(BatchNormalization, self).__init__()
        self.gamma = Parameter(torch.ones(size, device=device)) if use_gamma else None
        self.beta = Parameter(torch.zeros(size, device=device)) if use_beta else None
        self.avg_mean = torch.zeros(size, device=device)
        self.avg_var = torch.ones(size, device=device)
        self.eps = eps
        self.decay = decay

    def __call__(self, x):
        x = x.contiguous()
        g = None if self.gamma is None else self.gamma.tensor
        b = None if self.beta is None else self.beta.tensor
        y = TF.batch_norm(x, None, None, g, b, training=True, eps=self.eps)
        in_data = (x.detach(), None if self.gamma is None else self.gamma.data,
                   None if self.beta is None else self.beta.data)
        return _dispatch(BatchNormalizationFunction(), in_data, y)
