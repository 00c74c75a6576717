"""Full-size cases of the ResNet-50 batch-32 workload (the sizes the benchmark is quoted on).

The NumPy oracle needs minutes at these sizes, so the checks are against float64 PyTorch on the
GPU (``unfold`` + GEMM for the patch covariance, ``linalg.inv`` for the inverses) and against
properties that hold at any size: exact symmetry, the ones row equals the column means of the
patch matrix, M M^-1 = I.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def rel(a, b):
    return float((a.double() - b).norm() / b.norm())


def patch_cov64(x, k, s, p, bias):
    n = x.shape[0]
    P = torch.nn.functional.unfold(x.double(), k, padding=p, stride=s)     # (n, c*k*k, L)
    P = P.permute(0, 2, 1).reshape(-1, P.shape[1])
    if bias:
        P = torch.cat([P, torch.ones(P.shape[0], 1, dtype=P.dtype, device=P.device)], dim=1)
    return P.T @ P / n, P


@pytest.mark.parametrize('c,hw,k,s,p', [(64, 56, 3, 1, 1),      # d = 577, 100 352 patches
                                         (256, 14, 3, 1, 1),     # d = 2305
                                         (512, 7, 3, 1, 1),      # d = 4609
                                         (3, 224, 7, 2, 3),      # stem: d = 148, 401 408 patches
                                         (256, 56, 1, 1, 0),     # 1x1 slab, d = 257
                                         (1024, 14, 1, 2, 0)])   # strided 1x1, d = 1025
def test_conv_A_full_size(c, hw, k, s, p):
    from chainerkfac_amd import ops
    g = torch.Generator(device='cuda').manual_seed(c + hw)
    x = torch.randn(32, c, hw, hw, device='cuda', generator=g)
    A = ops.cov_conv_a(x, k, s, p, True, 1.0 / 32)
    ref, P = patch_cov64(x, k, s, p, True)
    assert rel(A, ref) < 1e-4
    assert torch.equal(A, A.T)
    # ones row = column sums of the patch matrix / n; corner = patches per sample
    assert rel(A[-1, :-1], P[:, :-1].sum(0) / 32) < 1e-5
    assert abs(float(A[-1, -1]) - P.shape[0] / 32) <= 1e-6 * P.shape[0] / 32


@pytest.mark.parametrize('c,hw', [(64, 112), (256, 56), (2048, 7)])
def test_conv_G_full_size(c, hw):
    from chainerkfac_amd import ops
    g = torch.Generator(device='cuda').manual_seed(c)
    gy = torch.randn(32, c, hw, hw, device='cuda', generator=g) / 32
    G = ops.cov_conv_g(gy, 32.0 ** 2 / (32 * hw * hw))
    M = gy.double().permute(0, 2, 3, 1).reshape(-1, c)
    ref = M.T @ M * (32.0 ** 2 / (32 * hw * hw))
    assert rel(G, ref) < 1e-4
    assert torch.equal(G, G.T)


def test_inverse_of_all_161_factor_sizes():
    """The inverse-only configuration: one SPD matrix per factor of ResNet-50 (64 .. 4609)."""
    from chainerkfac_amd import ops, workloads as W
    dims = W.all_factor_dims(W.resnet50_v1())
    assert len(dims) == 161 and max(dims) == 4609
    g = torch.Generator(device='cuda').manual_seed(4)
    mats = []
    for d in dims:
        X = torch.randn(2 * d, d, device='cuda', generator=g)
        mats.append(X.T @ X / (2 * d) + 1e-3 * torch.eye(d, device='cuda'))
        del X
    outs, info = ops.spd_inverse_batched(mats)
    assert int((info != 0).sum()) == 0
    for d, M, inv in zip(dims, mats, outs):
        assert torch.equal(inv, inv.T)
    # residual on one matrix of every distinct size, float64 inverse on the largest
    seen = set()
    for d, M, inv in zip(dims, mats, outs):
        if d in seen:
            continue
        seen.add(d)
        resid = float((M.double() @ inv.double() - torch.eye(d, device='cuda', dtype=torch.float64)).norm()) / d ** 0.5
        assert resid < 1e-3, (d, resid)
    i = dims.index(4609)
    assert rel(outs[i].cpu(), torch.linalg.inv(mats[i].double().cpu())) < 1e-3   # LAPACK on the host


def test_bn_lowrank_inverse_full_size():
    from chainerkfac_amd import ops
    g = torch.Generator(device='cuda').manual_seed(9)
    widths = [128, 512, 1024, 2048, 4096]
    Us = [torch.randn(32, w, device='cuda', generator=g) * 0.05 for w in widths]
    d = 16 * 2.5e-4
    outs, info = ops.bn_lowrank_inverse_batched(Us, [w // 2 for w in widths], [d] * 5, [d] * 5)
    assert int((info != 0).sum()) == 0
    for U, w, out in zip(Us, widths, outs):
        F = U.double().T @ U.double() / 32 + d * torch.eye(w, device='cuda', dtype=torch.float64)
        assert rel(out.cpu(), torch.linalg.inv(F.cpu())) < 1e-3   # LAPACK on the host
        assert torch.equal(out, out.T)


def test_precondition_largest_layer():
    from chainerkfac_amd import ops
    g = torch.Generator(device='cuda').manual_seed(11)
    dG, dA = 512, 4609

    def spd(d):
        X = torch.randn(2 * d, d, device='cuda', generator=g)
        return X.T @ X / (2 * d) + 0.1 * torch.eye(d, device='cuda')
    Ginv, Ainv = spd(dG), spd(dA)
    gW = torch.randn(dG, 512, 3, 3, device='cuda', generator=g)
    gb = torch.randn(dG, device='cuda', generator=g)
    kW, kb = ops.precond_conn(Ginv, Ainv, gW, gb)
    grad = torch.cat([gW.reshape(dG, -1), gb[:, None]], dim=1).double()
    ref = Ginv.double() @ grad @ Ainv.double()
    assert rel(kW.reshape(dG, -1), ref[:, :-1]) < 1e-3
    assert rel(kb, ref[:, -1]) < 1e-3
