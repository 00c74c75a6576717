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


def test_bench_rejects_more_than_one_gpu():
    import subprocess, sys, os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--gpus', '2'], capture_output=True, text=True)
    assert p.returncode != 0 and 'single-GPU' in (p.stderr + p.stdout)
