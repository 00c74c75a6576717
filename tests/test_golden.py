"""The committed fixtures of tests/golden/ (inputs and the oracle's outputs for
every stage of the path): the oracle still reproduces them, and the HIP path
matches them to the tolerances of the north-star spec (bit-exact wire format,
rel 1e-4 factors, rel 1e-3 inverses and preconditioned gradients)."""
import os

import numpy as np
import pytest

from oracle import kfac_oracle as O

GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'kfac_small.npz'))


def rel(a, b):
    b = b.astype(np.float64)
    return np.linalg.norm(a.astype(np.float64) - b) / max(np.linalg.norm(b), 1e-30)


def test_fixture_generator_is_deterministic_and_oracle_unchanged():
    """Regenerating the fixtures gives the committed values (to BLAS rounding:
    a different host may sum a dot product in another order)."""
    import importlib.util
    spec = importlib.util.spec_from_file_location(
        'make_golden', os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'make_golden.py'))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh = mod.build()
    assert sorted(fresh) == sorted(GOLDEN.files)
    for k in GOLDEN.files:
        assert fresh[k].shape == GOLDEN[k].shape and fresh[k].dtype == GOLDEN[k].dtype, k
        if k.startswith(('lin_x', 'lin_gy', 'conv_x', 'conv_gy', 'bn_x', 'bn_gy', 'pre_g', 'bn_gg', 'bn_gbeta')):
            assert np.array_equal(fresh[k], GOLDEN[k]), k   # inputs: bit-exact
        else:
            assert rel(fresh[k], GOLDEN[k]) < 1e-5, k


def test_packed_fixture_is_the_lower_triangle_row_major():
    """Independent of the oracle: numpy.tril_indices order, flat arrays copied."""
    A, gb, G = GOLDEN['lin_A'], GOLDEN['pre_gb'], GOLDEN['conv_G']
    expect = np.concatenate([A[np.tril_indices(A.shape[0])], gb, G[np.tril_indices(G.shape[0])]])
    assert np.array_equal(GOLDEN['pack_buf'], expect)


@pytest.mark.gpu
def test_hip_covariances_match_fixtures():
    import torch
    from chainerkfac_amd import ops
    g = GOLDEN
    dev = lambda k: torch.from_numpy(g[k]).cuda()
    cases = [
        (ops.cov_linear(dev('lin_x'), True, 1.0 / 12), 'lin_A'),
        (ops.cov_linear(dev('lin_gy'), False, 12.0), 'lin_G'),
        (ops.cov_conv_a(dev('conv_x'), 3, 1, 1, True, 1.0 / 3), 'conv_A_k3s1p1'),
        (ops.cov_conv_a(dev('conv_x'), 1, 2, 0, False, 1.0 / 3), 'conv_A_k1s2p0'),
        (ops.cov_conv_a(dev('conv_x'), 3, 2, 1, True, 1.0 / 3), 'conv_A_k3s2p1'),
        (ops.cov_conv_g(dev('conv_gy'), 9.0 / (3 * 9 * 8)), 'conv_G'),
    ]
    for got, key in cases:
        got = got.cpu().numpy()
        assert got.shape == g[key].shape, key
        assert rel(got, g[key]) < 1e-4, key
        assert np.array_equal(got, got.T), key
    U = ops.bn_grad_matrix(dev('bn_x'), dev('bn_gy'), 2e-5, 6.0)
    assert rel(U.cpu().numpy(), g['bn_grad']) < 1e-4
    F = ops.cov_linear(U, False, 1.0 / 6)
    assert rel(F.cpu().numpy(), g['bn_F']) < 1e-4


@pytest.mark.gpu
def test_hip_damping_inverse_precondition_match_fixtures():
    import torch
    from chainerkfac_amd import ops
    g = GOLDEN
    dev = lambda k: torch.from_numpy(g[k].copy()).cuda()
    A, G = dev('damp_A_in'), dev('damp_G_in')
    pi = ops.pi_damp_batched([A], [G], [1e-2 ** 0.5])
    want = float(g['damp_pi'].item())
    assert abs(float(pi[0].item()) - want) < 1e-5 * want
    assert rel(A.cpu().numpy(), g['damp_A_out']) < 1e-6 and rel(G.cpu().numpy(), g['damp_G_out']) < 1e-6
    (Ainv, Ginv), info = ops.spd_inverse_batched([A, G])
    assert info.cpu().tolist() == [0, 0]
    assert rel(Ainv.cpu().numpy(), g['inv_A']) < 1e-3 and rel(Ginv.cpu().numpy(), g['inv_G']) < 1e-3
    kW, kb = ops.precond_conn(dev('inv_G'), dev('inv_A'), dev('pre_gW'), dev('pre_gb'))
    assert rel(kW.cpu().numpy(), g['pre_kW']) < 1e-3 and rel(kb.cpu().numpy(), g['pre_kb']) < 1e-3
    kg, kbeta, nan = ops.precond_bn(dev('bn_Finv'), dev('bn_gg'), dev('bn_gbeta'))
    assert int(nan[0]) == 0
    assert rel(kg.cpu().numpy(), g['bn_kg']) < 1e-3 and rel(kbeta.cpu().numpy(), g['bn_kbeta']) < 1e-3


@pytest.mark.gpu
def test_hip_pack_matches_fixture_bit_for_bit():
    import torch
    from chainerkfac_amd.communicators import ArrayPacker
    g = GOLDEN
    arrays = [[(torch.from_numpy(g['lin_A']).cuda(), True), (torch.from_numpy(g['pre_gb']).cuda(), False),
               (torch.from_numpy(g['conv_G']).cuda(), True)]]
    packer = ArrayPacker()
    buf = torch.zeros(packer.get_nelems(arrays), dtype=torch.float32, device='cuda')
    packer._pack_arrays_to_buffer(arrays, buf)
    assert np.array_equal(buf.cpu().numpy(), g['pack_buf'])
    outs = [[(torch.zeros_like(a), t) for a, t in arrays[0]]]
    packer._unpack_arrays_from_buffer(outs, buf)
    for (a, _), (o, _) in zip(arrays[0], outs[0]):
        assert np.array_equal(o.cpu().numpy(), a.cpu().numpy())   # symmetric inputs: exact round trip
