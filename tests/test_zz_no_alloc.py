"""The entry point that allocates nothing (kfac_precond_bn_static_f32) against the
workspace-taking kfac_precond_bn_f32, through the C ABI (needs the GPU).

Both run the same kernels, so the outputs must be identical bit for bit; two
calls in a row, the second on a smaller block, because every call on a GPU
shares the one built-in scratch array and finds the previous call's contents
in it."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call_both(lib, d, n_gamma, seed, poison=None):
    from chainerkfac_amd import _lib
    g = torch.Generator(device='cuda').manual_seed(seed)
    X = torch.randn(d + 8, d, device='cuda', generator=g)
    Finv = (X.T @ X / (d + 8) + 0.1 * torch.eye(d, device='cuda')).contiguous()
    if poison is not None:
        Finv[poison] = float('nan')
    grad = torch.randn(d, device='cuda', generator=g)
    n_beta = d - n_gamma
    gg, gb = grad[:n_gamma].contiguous(), grad[n_gamma:].contiguous()
    stream = torch.cuda.current_stream().cuda_stream

    def ptr(t):
        return t.data_ptr() if t.numel() else 0

    outs = []
    for static in (False, True):
        kg = torch.full((n_gamma,), -3.0, device='cuda')
        kb = torch.full((n_beta,), -3.0, device='cuda')
        flag = torch.full((1,), 7, dtype=torch.int32, device='cuda')
        if static:
            _lib.check(lib.kfac_precond_bn_static_f32(Finv.data_ptr(), d, ptr(gg), n_gamma, ptr(gb), n_beta,
                                                      ptr(kg), ptr(kb), flag.data_ptr(), stream))
        else:
            ws = torch.empty(lib.kfac_precond_bn_workspace_bytes(d), dtype=torch.uint8, device='cuda')
            _lib.check(lib.kfac_precond_bn_f32(Finv.data_ptr(), d, ptr(gg), n_gamma, ptr(gb), n_beta,
                                               ptr(kg), ptr(kb), flag.data_ptr(), ws.data_ptr(), ws.numel(),
                                               stream))
        torch.cuda.synchronize()
        outs.append((kg.cpu().numpy(), kb.cpu().numpy(), int(flag.item())))
    (kg0, kb0, f0), (kg1, kb1, f1) = outs
    assert np.array_equal(kg0, kg1) and np.array_equal(kb0, kb1) and f0 == f1
    # and the result is the product itself (float64 reference), not just self-consistent
    if poison is None:
        ref = Finv.double() @ grad.double()
        got = np.concatenate([kg1, kb1])
        assert f1 == 0
        assert np.linalg.norm(got - ref.cpu().numpy()) <= 1e-5 * np.linalg.norm(ref.cpu().numpy())
    else:
        assert f1 == 1
        assert np.array_equal(kg1, gg.cpu().numpy()) and np.array_equal(kb1, gb.cpu().numpy())


def test_static_scratch_entry_point_matches_workspace_entry_point():
    from chainerkfac_amd import _lib
    lib = _lib.load()
    _call_both(lib, 4096, 2048, seed=1)          # the largest batch-norm block of ResNet-50
    _call_both(lib, 130, 65, seed=2)             # right after it, a smaller one: stale scratch beyond d
    _call_both(lib, 130, 130, seed=3)            # gamma only
    _call_both(lib, 64, 32, seed=4, poison=(3, 5))   # NaN fallback
    _call_both(lib, 8192, 4096, seed=5)          # the maximum size


def test_static_scratch_entry_point_rejects_sizes_beyond_its_array():
    from chainerkfac_amd import _lib
    lib = _lib.load()
    d = 8193
    z = torch.zeros(d, device='cuda')
    rc = lib.kfac_precond_bn_static_f32(z.data_ptr(), d, z.data_ptr(), d, 0, 0, z.data_ptr(), 0, 0,
                                        torch.cuda.current_stream().cuda_stream)
    assert rc == -1
    assert b'8192' in lib.kfac_last_error_string()
    with pytest.raises(_lib.KfacHipError):
        _lib.check(rc)
