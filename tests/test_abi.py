"""The C-ABI library loads and exports every symbol include/kfac_hip.h declares (no GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, 'include', 'kfac_hip.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(kfac_[a-z0-9_]+)\s*\(', text)))


def test_header_symbols_exported_and_bound():
    from chainerkfac_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail('libkfac_hip.so is not built; run __graft_entry__.build()')
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), 'missing export ' + n
    assert sorted(_lib.PROTOTYPES) == names
    assert _lib.load().kfac_abi_version() == 1


def test_host_only_entry_points():
    from chainerkfac_amd import _lib
    lib = _lib.load()
    sizes = _lib.i64_array([6, 16, 49])
    tri = _lib.i32_array([0, 4, 7])
    assert lib.kfac_packed_nelems(3, sizes, tri) == 6 + 10 + 28
    bad = _lib.i64_array([6, 15, 49])
    assert lib.kfac_packed_nelems(3, bad, tri) == -1
    assert b'triangle_size' in lib.kfac_last_error_string()


def test_missing_library_fails_loudly(monkeypatch):
    from chainerkfac_amd import _lib
    monkeypatch.setattr(_lib, '_lib', None)
    monkeypatch.setattr(_lib, 'LIB_PATH', '/nonexistent/libkfac_hip.so')
    with pytest.raises(_lib.KfacHipError):
        _lib.load()


def test_cpu_tensor_is_rejected():
    import torch
    from chainerkfac_amd import _lib
    from chainerkfac_amd.communicators import ArrayPacker
    with pytest.raises(_lib.KfacHipError):
        ArrayPacker()._pack_arrays_to_buffer([[(torch.zeros(3, 3), True)]], torch.zeros(6))
