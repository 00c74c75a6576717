"""The library's planners on the host, under AddressSanitizer and UndefinedBehaviorSanitizer (no GPU).

``build/plan_check`` (tests/host, built by ``__graft_entry__.build_host_check``) is every source of
the library compiled for the host alone.  With the option ``host_only`` no call reaches the GPU:
plans are built, arguments checked and launch grids computed, nothing is allocated or launched.
The program replays each task table against what it must cover -- every tile product of the
inverse's sweep exactly once and only from finished columns, every (factor, tile, k-slice) of the
grouped covariance and preconditioning launches once with its partial tiles inside the workspace the
``*_workspace_bytes`` query reports, every pack / unpack unit once -- over the layer shapes of the
five benchmark configurations and a few hundred random lists.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _write_workloads(path):
    import bench
    from chainerkfac_amd import workloads as W
    cfgs = bench.configs()
    with open(path, 'w') as f:
        for name in ('c1', 'c2', 'c3', 'c4', 'c5'):
            cfg = cfgs[name]
            f.write('workload {}\n'.format(name))
            if cfg['layers'] is None:
                for d in bench.inverse_dims():
                    f.write('dim {}\n'.format(d))
                continue
            n = cfg['batch']
            for layer in cfg['layers']:
                if layer['kind'] == 'conv':
                    f.write('conv {} {} {} {} {} {} {} {} {}\n'.format(
                        n, layer['c_in'], layer['h'], layer['w'], layer['k'], layer['s'], layer['p'],
                        int(layer['bias']), layer['c_out']))
                elif layer['kind'] == 'linear':
                    f.write('linear {} {} {} {}\n'.format(n, layer['d_in'], layer['d_out'], int(layer['bias'])))
                else:
                    f.write('bn {} {} {} {}\n'.format(n, layer['c'], layer['h'], layer['w']))
            for d in W.all_factor_dims(cfg['layers']):
                f.write('dim {}\n'.format(d))


@pytest.fixture(scope='module')
def plan_check():
    import __graft_entry__ as entry
    if not os.path.exists(entry.HOST_CHECK):
        entry.build_host_check()
    return entry.HOST_CHECK


@pytest.mark.parametrize('part', ['inverse', 'covariance', 'precondition', 'pack', 'elementwise'])
def test_planners_under_sanitizers(plan_check, part, tmp_path):
    shapes = tmp_path / 'workloads.txt'
    _write_workloads(str(shapes))
    env = dict(os.environ, ASAN_OPTIONS='detect_leaks=0:abort_on_error=0:verify_asan_link_order=0', UBSAN_OPTIONS='print_stacktrace=1')
    proc = subprocess.run([plan_check, str(shapes), part], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                          timeout=600, env=env)
    out = proc.stdout.decode() + proc.stderr.decode()
    assert proc.returncode == 0, out[-6000:]
    assert '5 workloads, 0 failures' in out, out[-2000:]
