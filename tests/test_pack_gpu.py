"""Parity of the HIP pack/unpack with the oracle, bit for bit (needs the GPU)."""
import numpy as np
import pytest
import torch

from oracle import kfac_oracle as O

pytestmark = pytest.mark.gpu


def to_dev(arrays):
    return [[(torch.from_numpy(a).cuda(), t) for a, t in la] for la in arrays]


def make(seed, spec, symmetric=False):
    r = np.random.default_rng(seed)
    out = []
    for local in spec:
        la = []
        for kind, s in local:
            if kind == 't':
                m = r.standard_normal((s, s)).astype(np.float32)
                la.append(((m + m.T) if symmetric else m, True))
            else:
                la.append((r.standard_normal(s).astype(np.float32), False))
        out.append(la)
    return out


RAGGED = [[('f', (3, 2)), ('t', 4), ('t', 1)], [('f', (5,)), ('t', 7), ('f', (2, 2, 2)), ('t', 3)], [],
          [('t', 5)], [('t', 63), ('t', 64), ('t', 65), ('f', (4097,)), ('t', 129), ('f', (4096,)), ('t', 200)]]


@pytest.mark.parametrize('target', [-1, 0, 1, 2, 4])
def test_pack_matches_oracle(pack_oracle_c, target):
    from chainerkfac_amd.communicators import ArrayPacker
    host = make(1, RAGGED)
    dev = to_dev(host)
    n = O.get_nelems(host)
    ref = np.full(n, -3.0, np.float32)
    pack_oracle_c.pack(host, ref, target)
    ref2 = np.full(n, -3.0, np.float32)
    O.pack(host, ref2, target)
    assert np.array_equal(ref, ref2)
    buf = torch.full((n,), -3.0, dtype=torch.float32, device='cuda')
    p = ArrayPacker()
    assert p.get_nelems(dev) == n
    p._pack_arrays_to_buffer(dev, buf, np.float32, target, None)
    torch.cuda.synchronize()
    assert np.array_equal(buf.cpu().numpy(), ref)


@pytest.mark.parametrize('target,divisor', [(-1, 1), (4, 1), (-1, 4), (1, 3), (2, 2)])
def test_unpack_matches_oracle(pack_oracle_c, target, divisor):
    from chainerkfac_amd.communicators import ArrayPacker
    host = make(2, RAGGED)
    n = O.get_nelems(host)
    bufh = np.random.default_rng(3).standard_normal(n).astype(np.float32)
    ref = [[(np.full_like(a, 9.0), t) for a, t in la] for la in host]
    pack_oracle_c.unpack(ref, bufh, target, divisor)
    dev = [[(torch.full(a.shape, 9.0, dtype=torch.float32, device='cuda'), t) for a, t in la] for la in host]
    ArrayPacker()._unpack_arrays_from_buffer(dev, torch.from_numpy(bufh).cuda(), np.float32, target, divisor, None)
    torch.cuda.synchronize()
    for la, lr in zip(dev, ref):
        for (a, _), (b, _) in zip(la, lr):
            assert np.array_equal(a.cpu().numpy(), b)


def test_empty_lists():
    from chainerkfac_amd.communicators import ArrayPacker
    p = ArrayPacker()
    buf = torch.zeros(4, device='cuda')
    p._pack_arrays_to_buffer([[], []], buf)
    p._unpack_arrays_from_buffer([[], []], buf)
    p._pack_arrays_to_buffer([], buf)
    torch.cuda.synchronize()
    assert p.get_nelems([[], []]) == 0


def test_buffer_too_small_is_an_error():
    from chainerkfac_amd.communicators import ArrayPacker
    a = torch.zeros(8, 8, device='cuda')
    with pytest.raises(ValueError):
        ArrayPacker()._pack_arrays_to_buffer([[(a, True)]], torch.zeros(35, device='cuda'))
    with pytest.raises(RuntimeError):
        ArrayPacker().get_nelems([[(torch.zeros(2, 3, device='cuda'), True)]])


def test_resnet50d_factor_list_round_trip_bit_exact(pack_oracle_c):
    """All 167 factors of ResNet-50-D plus its parameter gradients in the
    reference's buffer order (grads, A, G per layer): pack against the C
    oracle on the four largest layers' worth of data, and the full list
    through the round trip (pack -> unpack reproduces every symmetric factor
    bit for bit)."""
    from chainerkfac_amd import workloads as W
    from chainerkfac_amd.communicators import ArrayPacker
    g = torch.Generator(device='cuda').manual_seed(5)
    arrays = []
    for layer in W.resnet50_d():
        dims = W.factor_dims(layer)
        if len(dims) == 2:
            grads = [torch.randn(dims[1], dims[0] - (1 if layer.get('bias') else 0), device='cuda', generator=g)]
            if layer.get('bias'):
                grads.append(torch.randn(dims[1], device='cuda', generator=g))
        else:
            grads = [torch.randn(dims[0] // 2, device='cuda', generator=g) for _ in range(2)]
        for t in grads:
            arrays.append((t, False))
        for d in dims:
            m = torch.randn(d, d, device='cuda', generator=g)
            arrays.append((torch.triu(m) + torch.triu(m, 1).T, True))
    arrays = [arrays]
    p = ArrayPacker()
    n = p.get_nelems(arrays)
    assert n == 133489867 + sum(a.numel() for a, t in arrays[0] if not t)
    buf = torch.empty(n, device='cuda')
    p._pack_arrays_to_buffer(arrays, buf)
    out = [[(torch.full_like(a, float('nan')), t) for a, t in arrays[0]]]
    p._unpack_arrays_from_buffer(out, buf)
    torch.cuda.synchronize()
    for (a, _), (b, _) in zip(arrays[0], out[0]):
        assert torch.equal(a, b)
    # oracle check of the packed bytes on a slice of the list (the last 12 arrays
    # include 4096^2 and 2049^2 factors)
    tail = arrays[0][-12:]
    host = [[(a.cpu().numpy(), t) for a, t in tail]]
    ref = np.zeros(O.get_nelems(host), np.float32)
    pack_oracle_c.pack(host, ref)
    assert np.array_equal(buf[n - ref.size:].cpu().numpy(), ref)


def _half_stress_values(n, seed):
    """float32 values that exercise float16 rounding: ties, subnormals, overflow, signed zeros."""
    r = np.random.default_rng(seed)
    v = (r.standard_normal(n) * np.exp(r.uniform(-12, 12, n))).astype(np.float32)
    special = np.array([0.0, -0.0, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65504.0, 65520.0, 65519.9, 1e6, -1e6,
                        2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25, 6.1e-5, -5.96e-8, 2049.0, 2051.0], np.float32)
    v[:special.size] = special[:min(special.size, n)]
    return v


@pytest.mark.parametrize('target', [-1, 1, 4])
def test_pack_float16_buffer_matches_oracle(target):
    """Round to nearest even into a half buffer (pure_nccl_communicator.py:354-363)."""
    from chainerkfac_amd.communicators import ArrayPacker
    host = make(5, RAGGED)
    for la in host:
        for a, _ in la:
            a.reshape(-1)[:] = _half_stress_values(a.size, a.size)
    dev = to_dev(host)
    n = O.get_nelems(host)
    ref = np.full(n, -3.0, np.float16)
    with np.errstate(over='ignore'):
        O.pack(host, ref, target)
    small = [[la[0]] if la else [] for la in host]
    assert np.array_equal(O.pack(small, np.zeros(O.get_nelems(small), np.float16)).view(np.uint16),
                          O.pack_bruteforce(small, np.zeros(O.get_nelems(small), np.float16)).view(np.uint16))
    buf = torch.full((n,), -3.0, dtype=torch.float16, device='cuda')
    ArrayPacker()._pack_arrays_to_buffer(dev, buf, np.float16, target, None)
    got = buf.cpu().numpy()
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize('target,divisor', [(-1, 1), (-1, 4), (1, 3), (-1, 7), (4, 2048)])
def test_unpack_float16_buffer_matches_oracle(target, divisor):
    """buf[i] / (half)divisor in half precision, then widened (pure_nccl_communicator.py:438-449)."""
    from chainerkfac_amd.communicators import ArrayPacker
    host = make(6, RAGGED)
    n = O.get_nelems(host)
    with np.errstate(over='ignore'):
        bufh = _half_stress_values(n, 8).astype(np.float16)   # values past 65504 become inf on purpose
    ref = [[(np.full_like(a, 9.0), t) for a, t in la] for la in host]
    O.unpack(ref, bufh, target, divisor)
    dev = [[(torch.full_like(torch.from_numpy(a), 9.0).cuda(), t) for a, t in la] for la in host]
    ArrayPacker()._unpack_arrays_from_buffer(dev, torch.from_numpy(bufh).cuda(), np.float16, target, divisor, None)
    for lr, ld in zip(ref, dev):
        for (a, _), (b, _) in zip(lr, ld):
            assert np.array_equal(a.view(np.uint32), b.cpu().numpy().view(np.uint32))


def test_float16_arrays_and_wrong_buffer_dtype_are_rejected():
    from chainerkfac_amd.communicators import ArrayPacker
    p = ArrayPacker()
    with pytest.raises(NotImplementedError):
        p._pack_arrays_to_buffer([[(torch.zeros(4, dtype=torch.float16, device='cuda'), False)]],
                                 torch.zeros(4, device='cuda'))
    with pytest.raises(ValueError):
        p._pack_arrays_to_buffer([[(torch.zeros(4, device='cuda'), False)]],
                                 torch.zeros(4, device='cuda'), np.float16)   # float32 tensor, float16 declared
    with pytest.raises(ValueError):
        p._pack_arrays_to_buffer([[(torch.zeros(4, device='cuda'), False)]],
                                 torch.zeros(4, dtype=torch.float64, device='cuda'), np.float64)
