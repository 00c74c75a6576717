"""Host-side logic that needs no GPU: the lanes helper with side streams switched
off, the block grouping of the optimizer set-up, and the workload tables bench.py
measures (factor dimensions and algorithmic work of ResNet-50 at batch 32)."""
import pytest


def test_lanes_disabled_runs_inline():
    from chainerkfac_amd.device import Lanes, current_lane
    lanes = Lanes(0)
    seen = []
    out = lanes.run(lambda: seen.append(current_lane()) or 'done')
    assert out == 'done' and seen == [None]
    lanes.join()   # nothing to wait for


def test_resnet50_workload_totals():
    from chainerkfac_amd import workloads as W
    layers = W.resnet50_v1()
    dims = W.all_factor_dims(layers)
    assert len(dims) == 161 and max(dims) == 4609 and min(dims) == 64
    fl = W.flops(layers, 32)
    assert abs(fl['cov'] / 1e9 - 790.0) < 0.5
    assert abs(fl['inverse'] / 1e9 - 802.3) < 0.5
    assert abs(fl['precondition'] / 1e9 - 156.5) < 0.5
    # factors as full matrices: 1067 MB, lower triangles 534 MB
    full = sum(d * d for d in dims) * 4
    tri = sum(d * (d + 1) // 2 for d in dims) * 4
    assert abs(full / 1e6 - 1067) < 2 and abs(tri / 1e6 - 534) < 2


def test_issued_covariance_work():
    """The multiply-adds the covariance kernels issue: equal to M d (d+1) where no layer takes the
    shifted-correlation route, about a third of it for a 3x3 stride-1 convolution that does, and
    between the two for the networks."""
    from chainerkfac_amd import workloads as W
    mlp = W.mlp_mnist()
    assert W.cov_flops_executed(mlp, 128) == W.flops(mlp, 128)['cov']
    conv = [dict(kind='conv', name='c', c_in=256, c_out=256, k=3, s=1, p=1, h=14, w=14, bias=False)]
    assert W.takes_shift_route(conv[0])
    a_work = 32 * 14 * 14 * 2304 * 2305                      # the A factor as a patch product
    g_work = 32 * 14 * 14 * 256 * 257
    issued = W.cov_flops_executed(conv, 32) - g_work
    assert 0.30 < issued / a_work < 0.36                      # 13 of 40.5 products, plus border strips
    strided = [dict(conv[0], s=2)]
    assert not W.takes_shift_route(strided[0])
    assert W.cov_flops_executed(strided, 32) == W.flops(strided, 32)['cov']
    stem = [dict(conv[0], c_in=32, h=112, w=112)]             # stacked tiles: 18 blocks of 32 x 32
    assert W.takes_shift_route(stem[0])
    for layers in (W.resnet50_v1(), W.resnet50_d(), W.cifar_cnn()):
        total, done = W.flops(layers, 32)['cov'], W.cov_flops_executed(layers, 32)
        assert 0.4 * total < done < total


def test_bench_rejects_more_than_one_gpu():
    import subprocess, sys, os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--gpus', '2'], capture_output=True, text=True)
    assert p.returncode != 0 and 'single-GPU' in (p.stderr + p.stdout)
