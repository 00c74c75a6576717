"""Triangular pack / unpack of Kronecker factors and gradients into one flat
float32 buffer: the single-GPU half of the reference communicator
(chainerkfac/communicators/pure_nccl_communicator.py:110-148, :221-279).

``arrays`` is a list (one entry per owning rank) of lists of
``(array, triangular)`` pairs, exactly what ``chainerkfac.optimizers.kfac.extract``
produces; arrays are float32 torch-ROCm tensors.  The collectives that sit
between pack and unpack in the reference are not part of this package.
"""
import ctypes

import numpy as np
import torch

from .. import _lib
from .. import device as _dev
from . import _utility


class _ArraysInfo(object):
    """Descriptor of ``arrays`` in buffer order (reference ``_ArraysInfo``,
    pure_nccl_communicator.py:221-279).  The tables live on the device inside a
    plan of the C library and are uploaded once."""

    def __init__(self, arrays):
        flat, ranks, tris = [], [], []
        for rank, local_arrays in enumerate(arrays):
            for array, triangular in local_arrays:
                if isinstance(array, torch.Tensor) and array.dtype not in (torch.float16, torch.float32):
                    raise ValueError('dtype must be float16 or float32.')
                if isinstance(array, torch.Tensor) and array.dtype == torch.float16:
                    raise NotImplementedError('float16 arrays are not supported (float32 arrays, float32 or '
                                              'float16 buffer)')
                _dev.require_gpu_tensor(array, 'array')
                if triangular:
                    if array.ndim != 2 or array.shape[0] != array.shape[1]:
                        raise RuntimeError('triangular array must be a square matrix')
                    tris.append(array.shape[0])
                else:
                    tris.append(0)
                flat.append(array)
                ranks.append(rank)
        self.arrays = flat
        self.n_arrays = len(flat)
        self.rank = np.asarray(ranks, dtype=np.int32)
        self.triangle_size = np.asarray(tris, dtype=np.int32)
        sizes = np.asarray([a.numel() for a in flat], dtype=np.int64)
        buf_sizes = np.where(self.triangle_size > 0,
                             self.triangle_size.astype(np.int64) * (self.triangle_size + 1) // 2, sizes)
        self.size_csum = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        self.buf_size_csum = np.concatenate([[0], np.cumsum(buf_sizes)]).astype(np.int64)
        self.size_total = int(self.size_csum[-1])
        self.buf_size_total = int(self.buf_size_csum[-1])
        self.key = tuple((a.data_ptr(), a.numel(), t, r) for a, t, r in zip(flat, tris, ranks))
        lib = _lib.load()
        plan = ctypes.c_void_p()
        _lib.check(lib.kfac_pack_plan_create(
            self.n_arrays, _lib.ptr_array([a.data_ptr() for a in flat]),
            _lib.i64_array(sizes), _lib.i32_array(tris), _lib.i32_array(ranks),
            ctypes.byref(plan)))
        self._plan = plan
        assert lib.kfac_pack_plan_nelems(plan) == self.buf_size_total

    @property
    def plan(self):
        return self._plan

    def __del__(self):
        try:
            plan, self._plan = self._plan, None
            if plan is not None:
                _lib._lib.kfac_pack_plan_destroy(plan)
        except Exception:   # interpreter shutdown: the library may be gone
            pass

    def show(self):
        print('# ainfo: n_arrays: {}'.format(self.n_arrays))
        print('# ainfo: size_total: {}'.format(self.size_total))
        print('# ainfo: buf_size_total: {}'.format(self.buf_size_total))
        for i in range(self.n_arrays):
            print('# ainfo[{}], rank:{}, dptr:{}, size:{}, buf_size:{}, triangle_size:{}'.format(
                i, self.rank[i], self.arrays[i].data_ptr(),
                self.size_csum[i + 1] - self.size_csum[i],
                self.buf_size_csum[i + 1] - self.buf_size_csum[i], self.triangle_size[i]))


def _key_of(arrays):
    return tuple((a.data_ptr(), a.numel(), bool(t), r)
                 for r, local in enumerate(arrays) for a, t in local)


class ArrayPacker(object):
    """Holds the pack/unpack entry points of the reference communicator with
    their signatures (``_pack_arrays_to_buffer`` / ``_unpack_arrays_from_buffer``,
    pure_nccl_communicator.py:110-148).  Descriptors are cached per distinct
    list of arrays, so steady-state calls upload nothing."""

    def __init__(self, rank=0, max_cached=8):
        self.rank = rank
        self._cache = {}
        self._max_cached = max_cached

    def _info(self, arrays, stream=None):
        key = _key_of(arrays)
        info = self._cache.pop(key, None)
        if info is None:
            info = self._rebind(key, arrays, stream)
        if info is None:
            if len(self._cache) >= self._max_cached:
                self._cache.pop(next(iter(self._cache)))
            info = _ArraysInfo(arrays)
        self._cache[key] = info      # most recently used last
        return info

    def _rebind(self, key, arrays, stream):
        """A cached descriptor of the same layout pointed at other arrays (gradient arrays
        move from step to step): only the pointer table is uploaded again.  The two most
        recent descriptors of a layout are left alone (lists that alternate keep theirs),
        and so is one that a captured HIP graph replays against (the library refuses to
        change it)."""
        layout = tuple(k[1:] for k in key)
        same = [k for k in self._cache if tuple(e[1:] for e in k) == layout]
        if len(same) < 2:
            return None
        flat = [_dev.require_gpu_tensor(a, 'array') for local in arrays for a, _ in local]
        for old_key in same[:-1]:
            info = self._cache[old_key]
            try:
                _lib.check(_lib.load().kfac_pack_plan_set_ptrs(
                    info.plan, _lib.ptr_array([a.data_ptr() for a in flat]), _dev.stream_handle(stream)))
            except _lib.KfacHipError:
                continue
            del self._cache[old_key]
            info.arrays = flat
            info.key = key
            return info
        return None

    def get_nelems(self, arrays):
        return _utility.get_nelems(arrays)

    @staticmethod
    def _check_buf(gpu_buf, buf_dtype, need):
        """Returns 'f32' or 'f16': the element type of the wire buffer.  The
        arrays themselves are float32; float16 is the reference's optional
        communication dtype (pure_nccl_communicator.py:32-33)."""
        dt = np.dtype(np.float32 if buf_dtype is None else buf_dtype)
        if dt == np.float32:
            kind, tdtype = 'f32', torch.float32
        elif dt == np.float16:
            kind, tdtype = 'f16', torch.float16
        else:
            raise ValueError('the buffer must be float32 or float16, not {}'.format(buf_dtype))
        _dev.require_gpu_tensor(gpu_buf, 'gpu_buf', dtype=tdtype)
        if gpu_buf.numel() < need:
            raise ValueError('gpu_buf holds {} elements, {} needed'.format(gpu_buf.numel(), need))
        return kind

    def _pack_arrays_to_buffer(self, arrays, gpu_buf, buf_dtype=np.float32, target=-1,
                               stream=None, debug=False):
        info = self._info(arrays, stream)
        if debug and self.rank == 0:
            info.show()
        kind = self._check_buf(gpu_buf, buf_dtype, info.buf_size_total)
        lib = _lib.load()
        fn = lib.kfac_pack_f16 if kind == 'f16' else lib.kfac_pack_f32
        _lib.check(fn(info.plan, gpu_buf.data_ptr(), gpu_buf.numel(), int(target),
                      _dev.stream_handle(stream)))

    def _unpack_arrays_from_buffer(self, arrays, gpu_buf, buf_dtype=np.float32, target=-1,
                                   divisor=1, stream=None, debug=False):
        info = self._info(arrays, stream)
        if debug and self.rank == 0:
            info.show()
        kind = self._check_buf(gpu_buf, buf_dtype, info.buf_size_total)
        lib = _lib.load()
        fn = lib.kfac_unpack_f16 if kind == 'f16' else lib.kfac_unpack_f32
        _lib.check(fn(info.plan, gpu_buf.data_ptr(), gpu_buf.numel(), int(target), int(divisor),
                      _dev.stream_handle(stream)))
