"""Pins for the oracle's communicator buffer layout (no GPU).

Three independent statements of the same index map must agree bit for bit:
the pure-Python per-thread loop, numpy.tril_indices, and the C restatement of
the reference kernels.
"""
import numpy as np
import pytest

from oracle import kfac_oracle as O


def make_arrays(seed, spec):
    """spec: list (per rank) of lists of ('t', d) | ('f', shape)."""
    r = np.random.default_rng(seed)
    out = []
    for local in spec:
        la = []
        for kind, s in local:
            if kind == 't':
                la.append((r.standard_normal((s, s)).astype(np.float32), True))
            else:
                la.append((r.standard_normal(s).astype(np.float32), False))
        out.append(la)
    return out


SPEC = [[('f', (3, 2)), ('t', 4), ('t', 1)], [('f', (5,)), ('t', 7), ('f', (2, 2, 2)), ('t', 3)], [], [('t', 5)]]


def test_get_nelems_closed_form():
    arrays = make_arrays(0, SPEC)
    assert O.get_nelems(arrays) == 6 + 10 + 1 + 5 + 28 + 8 + 6 + 15
    with pytest.raises(RuntimeError):
        O.get_nelems([[(np.zeros((2, 3), np.float32), True)]])
    info = O.ArraysInfo(arrays)
    assert info.size_total == 6 + 16 + 1 + 5 + 49 + 8 + 9 + 25
    assert info.buf_size_total == O.get_nelems(arrays)
    assert list(info.rank) == [0, 0, 0, 1, 1, 1, 1, 3]
    assert list(info.triangle_size) == [0, 4, 1, 0, 7, 0, 3, 5]
    with pytest.raises(ValueError):
        O.ArraysInfo([[(np.zeros(3, np.float64), False)]])


def test_tril_indices_order_is_slot_formula():
    for m in (1, 2, 5, 33):
        r, c = np.tril_indices(m)
        assert np.array_equal(r * (r + 1) // 2 + c, np.arange(m * (m + 1) // 2))


@pytest.mark.parametrize('target', [-1, 0, 1, 3])
def test_pack_three_ways(pack_oracle_c, target):
    arrays = make_arrays(1, SPEC)
    n = O.get_nelems(arrays)
    b1 = np.full(n, -7.0, np.float32); b2 = b1.copy(); b3 = b1.copy()
    O.pack_bruteforce(arrays, b1, target)
    O.pack(arrays, b2, target)
    pack_oracle_c.pack(arrays, b3, target)
    assert np.array_equal(b1, b2) and np.array_equal(b1, b3)
    if target == -1:
        assert not np.any(b1 == -7.0)
    # slot check straight from the formula for one triangular array
    M = arrays[1][1][0]
    off = 6 + 10 + 1 + 5
    if target in (-1, 1):
        assert b1[off + 5 * 6 // 2 + 2] == M[5, 2]


@pytest.mark.parametrize('target,divisor', [(-1, 1), (1, 1), (-1, 4), (0, 3)])
def test_unpack_three_ways_and_symmetry(pack_oracle_c, target, divisor):
    arrays = make_arrays(2, SPEC)
    n = O.get_nelems(arrays)
    buf = np.random.default_rng(3).standard_normal(n).astype(np.float32)
    outs = []
    for fn in (O.unpack_bruteforce, O.unpack, pack_oracle_c.unpack):
        dst = [[(np.full_like(a, 9.0), t) for a, t in la] for la in arrays]
        fn(dst, buf, target, divisor)
        outs.append(dst)
    for la1, la2, la3 in zip(*outs):
        for (a1, t), (a2, _), (a3, _) in zip(la1, la2, la3):
            assert np.array_equal(a1, a2) and np.array_equal(a1, a3)
            if t and not np.any(a1 == 9.0):
                assert np.array_equal(a1, a1.T)
    M = outs[0][1][1][0]
    if target in (-1, 1):
        off = 6 + 10 + 1 + 5
        assert M[2, 5] == np.float32(buf[off + 5 * 6 // 2 + 2] / np.float32(divisor))
    else:
        assert np.all(M == 9.0)


def test_round_trip_bit_exact_for_symmetric(pack_oracle_c):
    r = np.random.default_rng(4)
    mats = []
    for d in (1, 2, 17, 64, 65):
        X = r.standard_normal((d, d)).astype(np.float32)
        mats.append(X + X.T)
    arrays = [[(m, True) for m in mats] + [(r.standard_normal(11).astype(np.float32), False)]]
    buf = np.zeros(O.get_nelems(arrays), np.float32)
    pack_oracle_c.pack(arrays, buf)
    dst = [[(np.zeros_like(a), t) for a, t in arrays[0]]]
    pack_oracle_c.unpack(dst, buf)
    for (a, _), (b, _) in zip(arrays[0], dst[0]):
        assert np.array_equal(a, b)
