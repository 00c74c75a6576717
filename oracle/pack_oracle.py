"""ctypes front end of the C pack/unpack oracle.  TEST INFRASTRUCTURE ONLY.

Runs the sequential restatement in ``pack_oracle.c`` of the reference kernels
(chainerkfac/communicators/pure_nccl_communicator.py:300-463) on NumPy arrays.
"""
import ctypes
import os

import numpy as np

from . import kfac_oracle

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def _lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, 'libpack_oracle.so')
        if not os.path.exists(path):
            raise RuntimeError(
                'oracle/libpack_oracle.so is not built; run '
                '`make -C oracle` or __graft_entry__.build()')
        _LIB = ctypes.CDLL(path)
        ip = ctypes.POINTER(ctypes.c_int)
        up = ctypes.POINTER(ctypes.c_uint64)
        fp = ctypes.POINTER(ctypes.c_float)
        _LIB.oracle_pack_f32.argtypes = [fp, ip, up, ip, ip, ip, ctypes.c_int,
                                         ctypes.c_int, ctypes.c_int]
        _LIB.oracle_pack_f32.restype = None
        _LIB.oracle_unpack_f32.argtypes = [up, ip, fp, ip, ip, ip, ctypes.c_int,
                                           ctypes.c_int, ctypes.c_int,
                                           ctypes.c_int]
        _LIB.oracle_unpack_f32.restype = None
    return _LIB


def _tables(arrays):
    info = kfac_oracle.ArraysInfo(arrays)
    for a in info.flat:
        if a.dtype != np.float32 or not a.flags.c_contiguous:
            raise ValueError('C oracle handles C-contiguous float32 arrays')
    dptr = np.array([a.ctypes.data for a in info.flat], dtype=np.uint64)
    return info, dptr


def _p(a, t):
    return a.ctypes.data_as(ctypes.POINTER(t))


def pack(arrays, buf, target=-1):
    info, dptr = _tables(arrays)
    assert buf.dtype == np.float32 and buf.size >= info.buf_size_total
    _lib().oracle_pack_f32(
        _p(buf, ctypes.c_float), _p(info.buf_size_csum, ctypes.c_int),
        _p(dptr, ctypes.c_uint64), _p(info.size_csum, ctypes.c_int),
        _p(info.triangle_size, ctypes.c_int), _p(info.rank, ctypes.c_int),
        int(target), info.size_total, info.n_arrays)
    return buf


def unpack(arrays, buf, target=-1, divisor=1):
    info, dptr = _tables(arrays)
    assert buf.dtype == np.float32 and buf.size >= info.buf_size_total
    _lib().oracle_unpack_f32(
        _p(dptr, ctypes.c_uint64), _p(info.size_csum, ctypes.c_int),
        _p(buf, ctypes.c_float), _p(info.buf_size_csum, ctypes.c_int),
        _p(info.triangle_size, ctypes.c_int), _p(info.rank, ctypes.c_int),
        int(target), int(divisor), info.size_total, info.n_arrays)
    return arrays
