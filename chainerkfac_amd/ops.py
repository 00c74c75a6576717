"""Thin tensor-level wrappers over the C ABI (one function per entry point).

Inputs and outputs are float32 torch-ROCm tensors; all work is enqueued on
torch's current stream (or the ``stream`` given).  These functions allocate
outputs and workspace, check shapes and call libkfac_hip -- they do not
compute anything themselves.
"""
import ctypes

import torch

from . import _lib
from . import device as _dev


def _out(out, shape, like):
    if out is None:
        return torch.empty(shape, dtype=torch.float32, device=like.device)
    _dev.require_gpu_tensor(out, 'out')
    if tuple(out.shape) != tuple(shape):
        raise ValueError('out has shape {}, expected {}'.format(tuple(out.shape), tuple(shape)))
    return out


def _cov_ws(d, rows, device):
    lib = _lib.load()
    nbytes = lib.kfac_cov_workspace_bytes(int(d), int(rows))
    return _dev.workspace('cov', nbytes, device), nbytes


def cov_linear(x, append_ones, alpha, beta=0.0, out=None, stream=None):
    """out = beta*out + alpha * [x, 1]^T [x, 1] for x of shape (n, d_in)."""
    _dev.require_gpu_tensor(x, 'x')
    if x.ndim != 2:
        raise ValueError('x must be 2-D')
    n, d_in = x.shape
    d = d_in + (1 if append_ones else 0)
    if out is None and beta != 0.0:
        raise ValueError('beta != 0 needs an existing out')
    out = _out(out, (d, d), x)
    ws, nbytes = _cov_ws(d, n, x.device)
    _lib.check(_lib.load().kfac_cov_linear_f32(
        x.data_ptr(), n, d_in, int(bool(append_ones)), alpha, beta, out.data_ptr(),
        ws.data_ptr(), ws.numel(), _dev.stream_handle(stream)))
    return out


def cov_conv_a(x, ksize, stride, pad, append_ones, alpha, beta=0.0, out=None, stream=None):
    """out = beta*out + alpha * P^T P, P the im2col patch matrix of NCHW x
    (columns (c, kh, kw) then ones)."""
    _dev.require_gpu_tensor(x, 'x')
    if x.ndim != 4:
        raise ValueError('x must be NCHW')
    kh, kw = (ksize, ksize) if isinstance(ksize, int) else ksize
    sy, sx = (stride, stride) if isinstance(stride, int) else stride
    ph, pw = (pad, pad) if isinstance(pad, int) else pad
    n, c, h, w = x.shape
    ho = (h + 2 * ph - kh) // sy + 1
    wo = (w + 2 * pw - kw) // sx + 1
    d = c * kh * kw + (1 if append_ones else 0)
    if out is None and beta != 0.0:
        raise ValueError('beta != 0 needs an existing out')
    out = _out(out, (d, d), x)
    ws, nbytes = _cov_ws(d, n * ho * wo, x.device)
    _lib.check(_lib.load().kfac_cov_conv_a_f32(
        x.data_ptr(), n, c, h, w, kh, kw, sy, sx, ph, pw, int(bool(append_ones)), alpha, beta,
        out.data_ptr(), ws.data_ptr(), ws.numel(), _dev.stream_handle(stream)))
    return out


def cov_conv_g(gy, alpha, beta=0.0, out=None, stream=None):
    """out = beta*out + alpha * gy_mat^T gy_mat for NCHW gy viewed as (n*ho*wo, c)."""
    _dev.require_gpu_tensor(gy, 'gy')
    if gy.ndim != 4:
        raise ValueError('gy must be NCHW')
    n, c, ho, wo = gy.shape
    if out is None and beta != 0.0:
        raise ValueError('beta != 0 needs an existing out')
    out = _out(out, (c, c), gy)
    ws, nbytes = _cov_ws(c, n * ho * wo, gy.device)
    _lib.check(_lib.load().kfac_cov_conv_g_f32(
        gy.data_ptr(), n, c, ho * wo, alpha, beta, out.data_ptr(), ws.data_ptr(), ws.numel(),
        _dev.stream_handle(stream)))
    return out


COV_LINEAR, COV_SLAB = 0, 1


class _CovItem(ctypes.Structure):
    _fields_ = [(name, ctypes.c_int32) for name in
                ('kind', 'n', 'c', 'h', 'w', 'sy', 'sx', 'append_ones', 'aligned')]


class CovGroup(object):
    """The covariances of a fixed list of small layers as one grouped launch.
    ``items``: tuples ``(kind, n, c, h, w, sy, sx, append_ones, aligned)``."""

    def __init__(self, items):
        self.items = tuple(tuple(int(v) for v in it) for it in items)
        lib = _lib.load()
        arr = (_CovItem * max(len(self.items), 1))()
        for dst, it in zip(arr, self.items):
            (dst.kind, dst.n, dst.c, dst.h, dst.w, dst.sy, dst.sx, dst.append_ones, dst.aligned) = it
        plan = ctypes.c_void_p()
        _lib.check(lib.kfac_cov_group_create(len(self.items), ctypes.cast(arr, ctypes.c_void_p),
                                             ctypes.byref(plan)))
        self._plan = plan
        self.workspace_bytes = lib.kfac_cov_group_workspace_bytes(plan)

    def __del__(self):
        try:
            plan, self._plan = self._plan, None
            if plan is not None:
                _lib._lib.kfac_cov_group_destroy(plan)
        except Exception:   # interpreter shutdown: the library may be gone
            pass

    def run(self, inputs, outputs, alphas, betas, stream=None):
        if len(inputs) != len(self.items) or len(outputs) != len(self.items):
            raise ValueError('expected {} items'.format(len(self.items)))
        if not self.items:
            return outputs
        for it, x, out in zip(self.items, inputs, outputs):
            _dev.require_gpu_tensor(x, 'input')
            _dev.require_gpu_tensor(out, 'out')
            d = it[2] + it[7]
            want = it[1] * it[2] * (it[3] * it[4] if it[0] == COV_SLAB else 1)
            if x.numel() != want or tuple(out.shape) != (d, d):
                raise ValueError('item {} does not match its tensors'.format(it))
        ws = _dev.workspace('cov_group', self.workspace_bytes, inputs[0].device)
        # (under HIP-graph capture the group may fork only from the stream the capture began on)
        origin = stream is None and _dev.current_lane() is None
        _lib.check(_lib.load().kfac_cov_group_set_capture_origin(self._plan, int(origin)))
        _lib.check(_lib.load().kfac_cov_group_run_f32(
            self._plan, _lib.ptr_array([x.data_ptr() for x in inputs]),
            _lib.ptr_array([o.data_ptr() for o in outputs]),
            ctypes.cast(_lib.f32_array(alphas), ctypes.c_void_p),
            ctypes.cast(_lib.f32_array(betas), ctypes.c_void_p),
            ws.data_ptr(), ws.numel(), _dev.stream_handle(stream)))
        return outputs


_cov_groups = None


def cov_group(items):
    """Cached ``CovGroup`` for a list of item descriptors."""
    global _cov_groups
    if _cov_groups is None:
        _cov_groups = _PlanCache(32)
    key = tuple(tuple(int(v) for v in it) for it in items)
    return _cov_groups.get(key, lambda: CovGroup(key))


class PendingCovs(object):
    """Collects the factor computations of layers that are too small to fill
    the GPU on their own; ``flush`` runs all of them as one grouped launch.
    The tensors are kept alive until then."""

    #: a factor is deferred when its SYRK has at most this many flops (rows * d * (d+1));
    #: larger ones (the k x k convolutions of a deep network) fill the GPU on their own
    max_flops = 8e9

    def __init__(self):
        self.items, self.inputs, self.outputs, self.alphas, self.betas = [], [], [], [], []
        self.bn_finishes = []

    def accepts(self, rows, d):
        return float(rows) * d * (d + 1) <= self.max_flops

    def add(self, kind, x, ones, out, alpha, beta, stride=1):
        if kind == COV_LINEAR:
            n, c = x.shape
            h = w = 1
        else:
            n, c, h, w = x.shape
        self.items.append((kind, n, c, h, w, stride, stride, int(bool(ones)), int(x.data_ptr() % 16 == 0)))
        self.inputs.append(x)
        self.outputs.append(out)
        self.alphas.append(alpha)
        self.betas.append(beta)

    def add_bn_finish(self, stats, U, n, c, hw, eps, gy_scale, has_gamma, has_beta):
        """The second part of a batch-norm layer's gradient matrix (``bn_stats`` has been
        queued): all layers' finishes run as one launch at ``flush``, before the factors."""
        self.bn_finishes.append((stats, U, n, c, hw, eps, gy_scale, has_gamma, has_beta))

    def flush(self, stream=None):
        if not self.items and not self.bn_finishes:
            return
        try:
            if self.bn_finishes:
                bn_finish_batched(self.bn_finishes, stream)
            if self.items:
                cov_group(self.items).run(self.inputs, self.outputs, self.alphas, self.betas, stream)
        finally:
            self.__init__()


def bn_grad_matrix(x, gy, eps, gy_scale, has_gamma=True, has_beta=True, out=None, stream=None):
    """(n, 2C) matrix [sum_hw gy'*h | sum_hw gy'] of a batch-norm layer."""
    _dev.require_gpu_tensor(x, 'x')
    _dev.require_gpu_tensor(gy, 'gy')
    if x.ndim not in (2, 4):
        raise RuntimeError('len(x.shape) must be 2 or 4, not {}.'.format(x.ndim))
    if x.shape != gy.shape:
        raise ValueError('x and gy shapes differ')
    n, c = x.shape[0], x.shape[1]
    hw = 1 if x.ndim == 2 else x.shape[2] * x.shape[3]
    width = c * (int(bool(has_gamma)) + int(bool(has_beta)))
    if width == 0:
        raise RuntimeError('gamma and beta must not be None as the same time')
    out = _out(out, (n, width), x)
    lib = _lib.load()
    nbytes = lib.kfac_bn_workspace_bytes(n, c)
    ws = _dev.workspace('bn', nbytes, x.device)
    _lib.check(lib.kfac_bn_grad_matrix_f32(
        x.data_ptr(), gy.data_ptr(), n, c, hw, eps, gy_scale, int(bool(has_gamma)),
        int(bool(has_beta)), out.data_ptr(), ws.data_ptr(), ws.numel(), _dev.stream_handle(stream)))
    return out


def bn_stats(x, gy, out=None, stream=None):
    """First part of ``bn_grad_matrix``: the per (sample, channel) statistics of one layer,
    a (4, n, C) array that ``bn_finish_batched`` turns into the gradient matrix."""
    _dev.require_gpu_tensor(x, 'x')
    _dev.require_gpu_tensor(gy, 'gy')
    if x.ndim not in (2, 4):
        raise RuntimeError('len(x.shape) must be 2 or 4, not {}.'.format(x.ndim))
    if x.shape != gy.shape:
        raise ValueError('x and gy shapes differ')
    n, c = x.shape[0], x.shape[1]
    hw = 1 if x.ndim == 2 else x.shape[2] * x.shape[3]
    out = _out(out, (4, n, c), x)
    _lib.check(_lib.load().kfac_bn_stats_f32(x.data_ptr(), gy.data_ptr(), n, c, hw, out.data_ptr(),
                                             out.numel() * 4, _dev.stream_handle(stream)))
    return out


class _BnFinishBatch(object):
    def __init__(self):
        h = ctypes.c_void_p()
        _lib.check(_lib.load().kfac_bn_finish_batch_create(ctypes.byref(h)))
        self._h = h

    def __del__(self):
        try:
            h, self._h = self._h, None
            if h is not None:
                _lib._lib.kfac_bn_finish_batch_destroy(h)
        except Exception:   # interpreter shutdown: the library may be gone
            pass


_bn_finish_batches = None


def bn_finish_batched(layers, stream=None):
    """Second part of ``bn_grad_matrix`` for a list of layers in one launch.  Every entry is
    ``(stats, U, n, c, hw, eps, gy_scale, has_gamma, has_beta)`` with ``stats`` from
    ``bn_stats`` and ``U`` the (n, width) output."""
    global _bn_finish_batches
    if not layers:
        return
    if _bn_finish_batches is None:
        _bn_finish_batches = _PlanCache(16)
    # one batch object per list of buffers (persistent per layer), so that its tables are written once
    key = tuple(l[0].data_ptr() for l in layers) + tuple(l[1].data_ptr() for l in layers)
    batch = _bn_finish_batches.get(key, _BnFinishBatch)
    described = tuple(l[2:] for l in layers)
    if getattr(batch, 'described', None) != described:
        for stats, U, n, c, hw, eps, gy_scale, has_gamma, has_beta in layers:
            _dev.require_gpu_tensor(stats, 'stats')
            _dev.require_gpu_tensor(U, 'U')
            width = c * (int(bool(has_gamma)) + int(bool(has_beta)))
            if width == 0:
                raise RuntimeError('gamma and beta must not be None as the same time')
            if stats.numel() != 4 * n * c or U.numel() != n * width:
                raise ValueError('stats {} / U {} do not match n={} c={}'.format(
                    tuple(stats.shape), tuple(U.shape), n, c))
        # the argument arrays of a list that comes back every step are built once
        batch.arrays = (
            _lib.ptr_array([l[0].data_ptr() for l in layers]), _lib.ptr_array([l[1].data_ptr() for l in layers]),
            _lib.i32_array([l[2] for l in layers]), _lib.i32_array([l[3] for l in layers]),
            _lib.i32_array([l[4] for l in layers]), _lib.f32_array([l[5] for l in layers]),
            _lib.f32_array([l[6] for l in layers]), _lib.i32_array([int(bool(l[7])) for l in layers]),
            _lib.i32_array([int(bool(l[8])) for l in layers]))
        batch.described = described
    _lib.check(_lib.load().kfac_bn_finish_batched_f32(batch._h, len(layers), *batch.arrays,
                                                      _dev.stream_handle(stream)))


def axpby(x, y, a, b, stream=None):
    """y = a*x + b*y in place."""
    _dev.require_gpu_tensor(x, 'x')
    _dev.require_gpu_tensor(y, 'y')
    if x.numel() != y.numel():
        raise ValueError('size mismatch')
    _lib.check(_lib.load().kfac_axpby_f32(x.data_ptr(), y.data_ptr(), x.numel(), a, b,
                                          _dev.stream_handle(stream)))
    return y


class _AxpbyBatch(object):
    def __init__(self):
        h = ctypes.c_void_p()
        _lib.check(_lib.load().kfac_axpby_batch_create(ctypes.byref(h)))
        self._h = h

    def __del__(self):
        try:
            h, self._h = self._h, None
            if h is not None:
                _lib._lib.kfac_axpby_batch_destroy(h)
        except Exception:   # interpreter shutdown: the library may be gone
            pass


_axpby_batches = None


def axpby_batched(xs, ys, a, b, stream=None):
    """ys[i] = a*xs[i] + b*ys[i] for a list of array pairs in one launch (in place)."""
    global _axpby_batches
    if len(xs) != len(ys):
        raise ValueError('one y per x')
    if not xs:
        return ys
    for x, y in zip(xs, ys):
        _dev.require_gpu_tensor(x, 'x')
        _dev.require_gpu_tensor(y, 'y')
        if x.numel() != y.numel():
            raise ValueError('size mismatch')
    if _axpby_batches is None:
        _axpby_batches = _PlanCache(16)
    # one batch object per list of destinations (they persist; the sources of a gradient
    # accumulation need not, and the object keeps its last few tables)
    xp, yp = tuple(x.data_ptr() for x in xs), tuple(y.data_ptr() for y in ys)
    batch = _axpby_batches.get(yp, _AxpbyBatch)
    _lib.check(_lib.load().kfac_axpby_batched_f32(
        batch._h, len(xs), _lib.ptr_array(xp), _lib.ptr_array(yp),
        _lib.i64_array([x.numel() for x in xs]), a, b, _dev.stream_handle(stream)))
    return ys


_div_batches = None


def div_batched(arrays, divisor, stream=None):
    """arrays[i] /= divisor in place for a list of float32 arrays in one launch."""
    global _div_batches
    if not arrays:
        return arrays
    for a in arrays:
        _dev.require_gpu_tensor(a, 'array')
    if _div_batches is None:
        _div_batches = _PlanCache(4)
    # one batch object per number of arrays (gradient arrays may be new ones every step; the
    # object keeps its last few tables)
    batch = _div_batches.get(len(arrays), _AxpbyBatch)
    _lib.check(_lib.load().kfac_div_batched_f32(
        batch._h, len(arrays), _lib.ptr_array([a.data_ptr() for a in arrays]),
        _lib.i64_array([a.numel() for a in arrays]), float(divisor), _dev.stream_handle(stream)))
    return arrays


def add_diag(M, v0, v1=None, split=None, stream=None):
    """diag(M)[i] += v0 for i < split else v1 (float64 sum, float32 store)."""
    _dev.require_gpu_tensor(M, 'M')
    d = M.shape[0]
    if M.ndim != 2 or M.shape[1] != d:
        raise ValueError('M must be square')
    if split is None:
        split, v1 = d, v0
    _lib.check(_lib.load().kfac_add_diag_f32(M.data_ptr(), d, int(split), float(v0), float(v1),
                                             _dev.stream_handle(stream)))
    return M


def keep_diag(M, stream=None):
    """M = diag(diag(M)) in place."""
    _dev.require_gpu_tensor(M, 'M')
    if M.ndim != 2 or M.shape[0] != M.shape[1]:
        raise ValueError('M must be square')
    _lib.check(_lib.load().kfac_keep_diag_f32(M.data_ptr(), M.shape[0], _dev.stream_handle(stream)))
    return M


def recip_add(x, v0, v1=None, split=None, out=None, stream=None):
    """1 / (x[i] + (v0 if i < split else v1)) elementwise (float64 arithmetic, float32 result)."""
    _dev.require_gpu_tensor(x, 'x')
    out = _out(out, tuple(x.shape), x)
    if split is None:
        split, v1 = x.numel(), v0
    _lib.check(_lib.load().kfac_recip_add_f32(x.data_ptr(), int(split), float(v0), float(v1), out.data_ptr(),
                                              x.numel(), _dev.stream_handle(stream)))
    return out


class _DiagBatch(object):
    def __init__(self):
        h = ctypes.c_void_p()
        _lib.check(_lib.load().kfac_diag_batch_create(ctypes.byref(h)))
        self._h = h

    def __del__(self):
        try:
            h, self._h = self._h, None
            if h is not None:
                _lib._lib.kfac_diag_batch_destroy(h)
        except Exception:   # interpreter shutdown: the library may be gone
            pass


_diag_batches = None


def add_diag_batched(mats, v0s, v1s=None, splits=None, stream=None):
    """``add_diag`` for a list of square matrices in one launch: diag(M_i)[j] += v0s[i] for
    j < splits[i] else v1s[i]."""
    global _diag_batches
    if not mats:
        return mats
    dims = []
    for M in mats:
        _dev.require_gpu_tensor(M, 'M')
        if M.ndim != 2 or M.shape[0] != M.shape[1]:
            raise ValueError('M must be square')
        dims.append(M.shape[0])
    if v1s is None:
        v1s, splits = v0s, dims
    if not (len(v0s) == len(v1s) == len(splits) == len(mats)):
        raise ValueError('one value pair and one split per matrix')
    if _diag_batches is None:
        _diag_batches = _PlanCache(16)
    ptrs = tuple(M.data_ptr() for M in mats)
    batch = _diag_batches.get(ptrs, _DiagBatch)
    _lib.check(_lib.load().kfac_add_diag_batched_f32(
        batch._h, len(mats), _lib.ptr_array(ptrs), _lib.i32_array(dims), _lib.i32_array(splits),
        _lib.f64_array(v0s), _lib.f64_array(v1s), _dev.stream_handle(stream)))
    return mats


class InversePlan(object):
    """Schedule for inverting a fixed list of SPD matrix sizes together."""

    def __init__(self, dims):
        self.dims = tuple(int(d) for d in dims)
        lib = _lib.load()
        plan = ctypes.c_void_p()
        _lib.check(lib.kfac_inverse_plan_create(len(self.dims), _lib.i32_array(self.dims),
                                                ctypes.byref(plan)))
        self._plan = plan
        self.workspace_bytes = lib.kfac_inverse_plan_workspace_bytes(plan)

    def __del__(self):
        try:
            plan, self._plan = self._plan, None
            if plan is not None:
                _lib._lib.kfac_inverse_plan_destroy(plan)
        except Exception:   # interpreter shutdown: the library may be gone
            pass

    def run(self, mats, outs=None, info=None, stream=None):
        if len(mats) != len(self.dims):
            raise ValueError('expected {} matrices'.format(len(self.dims)))
        for m, d in zip(mats, self.dims):
            _dev.require_gpu_tensor(m, 'matrix')
            if tuple(m.shape) != (d, d):
                raise ValueError('matrix shape {} != ({}, {})'.format(tuple(m.shape), d, d))
        if not mats:
            return [], info
        dev = mats[0].device
        if outs is None:
            outs = [torch.empty_like(m) for m in mats]
        for o, d in zip(outs, self.dims):
            _dev.require_gpu_tensor(o, 'out')
            if tuple(o.shape) != (d, d):
                raise ValueError('out shape mismatch')
        if info is None:
            info = torch.empty(len(mats), dtype=torch.int32, device=dev)
        ws = _dev.workspace('inverse', self.workspace_bytes, dev)
        # Under HIP-graph capture the plan may fork its trailing updates onto its
        # own stream only from the stream the capture began on: torch's current
        # stream when the call is not inside a lane (a lane is itself a fork).
        origin = stream is None and _dev.current_lane() is None
        _lib.check(_lib.load().kfac_inverse_plan_set_capture_origin(self._plan, int(origin)))
        _lib.check(_lib.load().kfac_spd_inverse_batched_f32(
            self._plan, _lib.ptr_array([m.data_ptr() for m in mats]),
            _lib.ptr_array([o.data_ptr() for o in outs]), info.data_ptr(), ws.data_ptr(),
            ws.numel(), _dev.stream_handle(stream)))
        return outs, info


class _PlanCache(object):
    """Least-recently-used cache of plans.

    A plan keeps its device-side pointer tables between calls and rewrites them
    (stream synchronisation + blocking copy) when it is called with other
    buffers.  Callers that pass persistent buffers -- the Fisher blocks do --
    therefore get one plan per (shapes, buffers): equal-shaped layers do not
    evict each other's tables, no call after the first touches the host-device
    link, and a HIP graph captured over a call keeps replaying against tables
    nobody rewrites.  Calls that let the wrapper allocate fresh outputs share
    one plan per shape list instead (their pointers change every time)."""

    def __init__(self, limit=1024):
        from collections import OrderedDict
        self._plans = OrderedDict()
        self._limit = limit

    def get(self, key, make):
        plan = self._plans.get(key)
        if plan is None:
            while len(self._plans) >= self._limit:
                self._plans.popitem(last=False)
            plan = self._plans[key] = make()
        else:
            self._plans.move_to_end(key)
        return plan

    def __len__(self):
        return len(self._plans)


def _ptr_key(tensors):
    return None if tensors is None else tuple(t.data_ptr() for t in tensors)


_inverse_plans = _PlanCache()


def inverse_plan(dims, bound_to=None):
    """Plan for a list of matrix sizes; ``bound_to`` (any hashable, normally the
    buffers' device pointers) gives callers with persistent buffers a plan of
    their own."""
    dims = tuple(int(d) for d in dims)
    return _inverse_plans.get((dims, bound_to), lambda: InversePlan(dims))


def spd_inverse_batched(mats, outs=None, info=None, stream=None):
    """Inverses of a list of SPD matrices (potrf + potri on the GPU)."""
    bound = None if outs is None else (_ptr_key(mats), _ptr_key(outs))
    return inverse_plan([m.shape[0] for m in mats], bound).run(mats, outs, info, stream)


class BnLowrankPlan(object):
    """Schedule for the low-rank damped inverses of a fixed list of batch-norm blocks."""

    def __init__(self, n, widths, splits):
        self.n = int(n)
        self.widths = tuple(int(w) for w in widths)
        self.splits = tuple(int(v) for v in splits)
        lib = _lib.load()
        plan = ctypes.c_void_p()
        _lib.check(lib.kfac_bn_lowrank_plan_create(
            len(self.widths), self.n, _lib.i32_array(self.widths), _lib.i32_array(self.splits),
            ctypes.byref(plan)))
        self._plan = plan
        self.workspace_bytes = lib.kfac_bn_lowrank_workspace_bytes(plan)

    def __del__(self):
        try:
            plan, self._plan = self._plan, None
            if plan is not None:
                _lib._lib.kfac_bn_lowrank_plan_destroy(plan)
        except Exception:   # interpreter shutdown: the library may be gone
            pass

    def run(self, Us, d_gamma, d_beta, outs=None, info=None, stream=None):
        if len(Us) != len(self.widths):
            raise ValueError('expected {} gradient matrices'.format(len(self.widths)))
        for U, w in zip(Us, self.widths):
            _dev.require_gpu_tensor(U, 'U')
            if tuple(U.shape) != (self.n, w):
                raise ValueError('U shape {} != ({}, {})'.format(tuple(U.shape), self.n, w))
        if not Us:
            return [], info
        dev = Us[0].device
        if outs is None:
            outs = [torch.empty((w, w), dtype=torch.float32, device=dev) for w in self.widths]
        for o, w in zip(outs, self.widths):
            _dev.require_gpu_tensor(o, 'out')
            if tuple(o.shape) != (w, w):
                raise ValueError('out shape mismatch')
        if info is None:
            info = torch.empty(len(Us), dtype=torch.int32, device=dev)
        ws = _dev.workspace('bn_lowrank', self.workspace_bytes, dev)
        _lib.check(_lib.load().kfac_bn_lowrank_inverse_batched_f32(
            self._plan, _lib.ptr_array([U.data_ptr() for U in Us]),
            _lib.ptr_array([o.data_ptr() for o in outs]),
            _lib.f64_array([0.0 if v is None else v for v in d_gamma]),
            _lib.f64_array([0.0 if v is None else v for v in d_beta]),
            info.data_ptr(), ws.data_ptr(), ws.numel(), _dev.stream_handle(stream)))
        return outs, info


_bn_lowrank_plans = _PlanCache()


def bn_lowrank_inverse_batched(Us, splits, d_gamma, d_beta, outs=None, info=None, stream=None):
    """(U^T U / n + diag(d_gamma | d_beta))^-1 for a list of (n, w) gradient matrices."""
    key = (Us[0].shape[0], tuple(U.shape[1] for U in Us), tuple(int(v) for v in splits))
    bound = None if outs is None else (_ptr_key(Us), _ptr_key(outs))
    plan = _bn_lowrank_plans.get(key + (bound,), lambda: BnLowrankPlan(*key))
    return plan.run(Us, d_gamma, d_beta, outs, info, stream)


class DampPlan(object):
    def __init__(self, dimsA, dimsG):
        self.dimsA = tuple(int(d) for d in dimsA)
        self.dimsG = tuple(int(d) for d in dimsG)
        plan = ctypes.c_void_p()
        _lib.check(_lib.load().kfac_damp_plan_create(
            len(self.dimsA), _lib.i32_array(self.dimsA), _lib.i32_array(self.dimsG),
            ctypes.byref(plan)))
        self._plan = plan

    def __del__(self):
        try:
            plan, self._plan = self._plan, None
            if plan is not None:
                _lib._lib.kfac_damp_plan_destroy(plan)
        except Exception:   # interpreter shutdown: the library may be gone
            pass

    def run(self, As, Gs, rW, use_pi=True, pi_out=None, stream=None):
        for t in list(As) + list(Gs):
            _dev.require_gpu_tensor(t, 'factor')
        if pi_out is None:
            pi_out = torch.empty(len(As), dtype=torch.float32, device=As[0].device)
        _lib.check(_lib.load().kfac_pi_damp_batched_f32(
            self._plan, _lib.ptr_array([a.data_ptr() for a in As]),
            _lib.ptr_array([g.data_ptr() for g in Gs]), _lib.f64_array(rW), int(bool(use_pi)),
            pi_out.data_ptr(), _dev.stream_handle(stream)))
        return pi_out


_damp_plans = _PlanCache()


def pi_damp_batched(As, Gs, rW, use_pi=True, pi_out=None, stream=None):
    """In-place trace-norm damping of (A, G) pairs; returns the device vector of pi."""
    key = (tuple(a.shape[0] for a in As), tuple(g.shape[0] for g in Gs))
    # the factors are damped in place, so their buffers identify the caller
    plan = _damp_plans.get(key + (_ptr_key(As), _ptr_key(Gs)), lambda: DampPlan(*key))
    return plan.run(As, Gs, rW, use_pi, pi_out, stream)


def precond_conn(Ginv, Ainv, gradW, gradb=None, kfW=None, kfb=None, stream=None):
    """(Ginv . [gradW | gradb]) . Ainv split back into the shapes of gradW / gradb."""
    for t, nm in ((Ginv, 'Ginv'), (Ainv, 'Ainv'), (gradW, 'gradW')):
        _dev.require_gpu_tensor(t, nm)
    dG, dA = Ginv.shape[0], Ainv.shape[0]
    has_b = gradb is not None
    if gradW.shape[0] != dG or gradW.numel() != dG * (dA - int(has_b)):
        raise ValueError('gradW shape {} does not match factors ({}, {})'.format(
            tuple(gradW.shape), dG, dA))
    if has_b:
        _dev.require_gpu_tensor(gradb, 'gradb')
        if gradb.numel() != dG:
            raise ValueError('gradb size mismatch')
    kfW = torch.empty_like(gradW) if kfW is None else _dev.require_gpu_tensor(kfW, 'kfW')
    if has_b:
        kfb = torch.empty_like(gradb) if kfb is None else _dev.require_gpu_tensor(kfb, 'kfb')
    lib = _lib.load()
    nbytes = lib.kfac_precond_conn_workspace_bytes(dG, dA)
    ws = _dev.workspace('precond', nbytes, Ginv.device)
    _lib.check(lib.kfac_precond_conn_f32(
        Ginv.data_ptr(), dG, Ainv.data_ptr(), dA, gradW.data_ptr(), _dev.ptr(gradb),
        kfW.data_ptr(), _dev.ptr(kfb) if has_b else 0, ws.data_ptr(), ws.numel(),
        _dev.stream_handle(stream)))
    return kfW, (kfb if has_b else None)


class PrecondGroup(object):
    """``precond_conn`` for a fixed list of layers ``(dG, dA, has_bias)`` as one grouped call."""

    def __init__(self, shapes):
        self.shapes = tuple((int(a), int(b), int(bool(c))) for a, b, c in shapes)
        lib = _lib.load()
        plan = ctypes.c_void_p()
        _lib.check(lib.kfac_precond_group_create(
            len(self.shapes), _lib.i32_array([s[0] for s in self.shapes]),
            _lib.i32_array([s[1] for s in self.shapes]), _lib.i32_array([s[2] for s in self.shapes]),
            ctypes.byref(plan)))
        self._plan = plan
        self.workspace_bytes = lib.kfac_precond_group_workspace_bytes(plan)

    def __del__(self):
        try:
            plan, self._plan = self._plan, None
            if plan is not None:
                _lib._lib.kfac_precond_group_destroy(plan)
        except Exception:   # interpreter shutdown: the library may be gone
            pass

    def run(self, Ginvs, Ainvs, gradWs, gradbs, kfWs, kfbs, stream=None):
        n = len(self.shapes)
        if not (len(Ginvs) == len(Ainvs) == len(gradWs) == len(gradbs) == len(kfWs) == len(kfbs) == n):
            raise ValueError('expected {} layers'.format(n))
        if n == 0:
            return
        for (dG, dA, hb), G, A, gW, gb, kW, kb in zip(self.shapes, Ginvs, Ainvs, gradWs, gradbs, kfWs, kfbs):
            for t, nm in ((G, 'Ginv'), (A, 'Ainv'), (gW, 'gradW'), (kW, 'kfW')):
                _dev.require_gpu_tensor(t, nm)
            if tuple(G.shape) != (dG, dG) or tuple(A.shape) != (dA, dA) or gW.numel() != dG * (dA - hb) \
                    or kW.numel() != gW.numel():
                raise ValueError('layer ({}, {}, {}) does not match its tensors'.format(dG, dA, hb))
            if bool(hb) != (gb is not None) or bool(hb) != (kb is not None):
                raise ValueError('bias arrays do not match the group')
            if hb:
                _dev.require_gpu_tensor(gb, 'gradb')
                _dev.require_gpu_tensor(kb, 'kfb')
        ws = _dev.workspace('precond_group', self.workspace_bytes, Ginvs[0].device)
        origin = stream is None and _dev.current_lane() is None
        _lib.check(_lib.load().kfac_precond_group_set_capture_origin(self._plan, int(origin)))
        _lib.check(_lib.load().kfac_precond_group_run_f32(
            self._plan, _lib.ptr_array([t.data_ptr() for t in Ginvs]),
            _lib.ptr_array([t.data_ptr() for t in Ainvs]), _lib.ptr_array([t.data_ptr() for t in gradWs]),
            _lib.ptr_array([_dev.ptr(t) for t in gradbs]), _lib.ptr_array([t.data_ptr() for t in kfWs]),
            _lib.ptr_array([_dev.ptr(t) for t in kfbs]), ws.data_ptr(), ws.numel(),
            _dev.stream_handle(stream)))


_precond_groups = None


def precond_group(shapes, bound_to=None):
    """Cached ``PrecondGroup``; ``bound_to`` (the buffers' device pointers) gives callers
    with persistent buffers a plan whose pointer table is never rewritten."""
    global _precond_groups
    if _precond_groups is None:
        _precond_groups = _PlanCache(16)
    key = tuple((int(a), int(b), int(bool(c))) for a, b, c in shapes)
    return _precond_groups.get((key, bound_to), lambda: PrecondGroup(key))


def precond_bn(Finv, g_gamma, g_beta, kf_gamma=None, kf_beta=None, nan_flag=None, stream=None):
    """Finv . [g_gamma ; g_beta] with the NaN fallback to the raw gradients."""
    _dev.require_gpu_tensor(Finv, 'Finv')
    d = Finv.shape[0]
    ng = 0 if g_gamma is None else g_gamma.numel()
    nb = 0 if g_beta is None else g_beta.numel()
    if ng + nb != d:
        raise ValueError('gradient sizes {}+{} do not match Finv ({})'.format(ng, nb, d))
    if g_gamma is not None:
        _dev.require_gpu_tensor(g_gamma, 'g_gamma')
        kf_gamma = torch.empty_like(g_gamma) if kf_gamma is None else kf_gamma
    if g_beta is not None:
        _dev.require_gpu_tensor(g_beta, 'g_beta')
        kf_beta = torch.empty_like(g_beta) if kf_beta is None else kf_beta
    if nan_flag is None:
        nan_flag = torch.empty(1, dtype=torch.int32, device=Finv.device)
    lib = _lib.load()
    ws = _dev.workspace('precond_bn', lib.kfac_precond_bn_workspace_bytes(d), Finv.device)
    _lib.check(lib.kfac_precond_bn_f32(
        Finv.data_ptr(), d, _dev.ptr(g_gamma), ng, _dev.ptr(g_beta), nb, _dev.ptr(kf_gamma),
        _dev.ptr(kf_beta), nan_flag.data_ptr(), ws.data_ptr(), ws.numel(),
        _dev.stream_handle(stream)))
    return kf_gamma, kf_beta, nan_flag


class _PrecondBnBatch(object):
    def __init__(self):
        h = ctypes.c_void_p()
        _lib.check(_lib.load().kfac_precond_bn_batch_create(ctypes.byref(h)))
        self._h = h

    def __del__(self):
        try:
            h, self._h = self._h, None
            if h is not None:
                _lib._lib.kfac_precond_bn_batch_destroy(h)
        except Exception:   # interpreter shutdown: the library may be gone
            pass


_precond_bn_batches = None


def precond_bn_batched(Finvs, g_gammas, g_betas, kf_gammas, kf_betas, nan_flags, stream=None):
    """``precond_bn`` for a list of batch-norm blocks in two launches.  Every list has one
    entry per block; gradient / output entries may be None where a block has no gamma or
    no beta; ``nan_flags`` entries are one-element int32 tensors."""
    global _precond_bn_batches
    n = len(Finvs)
    if not (len(g_gammas) == len(g_betas) == len(kf_gammas) == len(kf_betas) == len(nan_flags) == n):
        raise ValueError('one entry per block in every list')
    if n == 0:
        return
    dims, n0s = [], []
    for F, g, b, kg, kb, flag in zip(Finvs, g_gammas, g_betas, kf_gammas, kf_betas, nan_flags):
        _dev.require_gpu_tensor(F, 'Finv')
        d = F.shape[0]
        ng = 0 if g is None else g.numel()
        nb = 0 if b is None else b.numel()
        if F.ndim != 2 or F.shape[1] != d or ng + nb != d:
            raise ValueError('gradient sizes {}+{} do not match Finv {}'.format(ng, nb, tuple(F.shape)))
        for t, out, nm in ((g, kg, 'gamma'), (b, kb, 'beta')):
            if t is not None:
                _dev.require_gpu_tensor(t, 'g_' + nm)
                _dev.require_gpu_tensor(out, 'kf_' + nm)
                if out.numel() != t.numel():
                    raise ValueError('kf_{} does not match its gradient'.format(nm))
        if flag is not None:
            _dev.require_gpu_tensor(flag, 'nan_flag', dtype=torch.int32)
        dims.append(d)
        n0s.append(ng)
    if _precond_bn_batches is None:
        _precond_bn_batches = _PlanCache(16)
    # one batch object per list of inverses and outputs (persistent); gradient arrays may move
    key = tuple(t.data_ptr() for t in Finvs) + tuple(_dev.ptr(t) for t in kf_gammas) + \
        tuple(_dev.ptr(t) for t in kf_betas)
    batch = _precond_bn_batches.get(key, _PrecondBnBatch)
    lib = _lib.load()
    dims_arr = _lib.i32_array(dims)
    ws = _dev.workspace('precond_bn', lib.kfac_precond_bn_batched_workspace_bytes(n, dims_arr), Finvs[0].device)
    _lib.check(lib.kfac_precond_bn_batched_f32(
        batch._h, n, _lib.ptr_array([t.data_ptr() for t in Finvs]), dims_arr,
        _lib.ptr_array([_dev.ptr(t) for t in g_gammas]), _lib.i32_array(n0s),
        _lib.ptr_array([_dev.ptr(t) for t in g_betas]), _lib.ptr_array([_dev.ptr(t) for t in kf_gammas]),
        _lib.ptr_array([_dev.ptr(t) for t in kf_betas]), _lib.ptr_array([_dev.ptr(t) for t in nan_flags]),
        ws.data_ptr(), ws.numel(), _dev.stream_handle(stream)))


def momentum_update(param, v, grad, lr, momentum, stream=None):
    """v = momentum*v - lr*grad; param += v (in place)."""
    for t in (param, v, grad):
        _dev.require_gpu_tensor(t, 'tensor')
    _lib.check(_lib.load().kfac_momentum_update_f32(
        param.data_ptr(), v.data_ptr(), grad.data_ptr(), param.numel(), lr, momentum,
        _dev.stream_handle(stream)))


class _MomentumBatch(object):
    def __init__(self):
        h = ctypes.c_void_p()
        _lib.check(_lib.load().kfac_momentum_batch_create(ctypes.byref(h)))
        self._h = h

    def __del__(self):
        try:
            h, self._h = self._h, None
            if h is not None:
                _lib._lib.kfac_momentum_batch_destroy(h)
        except Exception:   # interpreter shutdown: the library may be gone
            pass


_momentum_batches = None


def momentum_update_batched(params, vs, grads, lr, momentum, loss_scale=None, write_back=None,
                            params_f16=None, stream=None):
    """The momentum rule of a list of parameters in one launch (in place).

    ``params`` and ``vs`` are float32; ``grads`` float32 or float16.  With a
    ``loss_scale`` every gradient is divided by it first, and where
    ``write_back[i]`` is true (float32 gradients only) the quotient replaces the
    gradient.  ``params_f16[i]`` (or None) is a float16 array that receives the
    rounded new values of ``params[i]``."""
    global _momentum_batches
    n = len(params)
    if not (len(vs) == len(grads) == n):
        raise ValueError('one velocity and one gradient per parameter')
    if n == 0:
        return
    write_back = [False] * n if write_back is None else list(write_back)
    params_f16 = [None] * n if params_f16 is None else list(params_f16)
    if not (len(write_back) == len(params_f16) == n):
        raise ValueError('one flag and one float16 array (or None) per parameter')
    flags = []
    for p, v, g, wb, h in zip(params, vs, grads, write_back, params_f16):
        for t, nm in ((p, 'param'), (v, 'v')):
            _dev.require_gpu_tensor(t, nm)
        if g.dtype not in (torch.float32, torch.float16) or not g.is_cuda or not g.is_contiguous():
            raise ValueError('grad must be a contiguous float32 or float16 GPU tensor')
        if v.numel() != p.numel() or g.numel() != p.numel():
            raise ValueError('param, v and grad differ in size')
        if h is not None and (h.dtype != torch.float16 or not h.is_cuda or not h.is_contiguous()
                              or h.numel() != p.numel()):
            raise ValueError('params_f16 entries must be contiguous float16 GPU tensors of the parameter\'s size')
        if wb and g.dtype != torch.float32:
            raise ValueError('only a float32 gradient can receive the divided values')
        flags.append((1 if g.dtype == torch.float16 else 0) | (2 if wb else 0))
    if _momentum_batches is None:
        _momentum_batches = _PlanCache(16)
    # one batch object per list of parameters (gradient arrays may be new ones every step;
    # the object keeps its last few tables)
    batch = _momentum_batches.get(tuple(p.data_ptr() for p in params), _MomentumBatch)
    _lib.check(_lib.load().kfac_momentum_update_batched_f32(
        batch._h, n, _lib.ptr_array([p.data_ptr() for p in params]),
        _lib.ptr_array([v.data_ptr() for v in vs]), _lib.ptr_array([g.data_ptr() for g in grads]),
        _lib.i64_array([p.numel() for p in params]), _lib.i32_array(flags),
        _lib.ptr_array([_dev.ptr(h) for h in params_f16]), lr, momentum,
        1.0 if loss_scale is None else float(loss_scale), _dev.stream_handle(stream)))
