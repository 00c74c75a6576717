#!/usr/bin/env python
"""Benchmark of the K-FAC per-layer hot path on one MI355X.

Workload (BASELINE.json configs[2]): ResNet-50 (bottleneck v1, 1000-way FC, all
convs with bias) K-FAC step on one GPU's share, batch 32 at 224x224, fp32:
for all 161 Kronecker factors, covariance (fused im2col SYRK) + pi-damped
Cholesky inverse + gradient preconditioning.  Per-layer activations, output
gradients and parameter gradients are synthetic N(0,1) tensors of the real
shapes (output gradients scaled by 1/(batch*sqrt(pixels)), the size a
mean-reduced loss gives them, which keeps the rank-32 batch-norm factors
positive definite in float32), resident in HBM before the timed region.  The step is driven through
the drop-in host classes (FisherBlock*.forward_postprocess /
backward_preprocess, KFAC.update_kfgrads).  The 53 batch-norm blocks, whose
factor is the rank-32 matrix U^T U / 32 of this batch, are inverted through
their Woodbury form (the same dense damped inverse as the Cholesky path, which
--dense-bn-inverse forces); the JSON states which path ran and reports the
inverse rate both against the reference's 161 dense inversions and against
the dense work actually executed.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-graph] [--no-cpu]

prints ONE JSON line: ms per K-FAC step, per-phase TFLOP/s, the roofline of the
dominant kernel family (covariance SYRK, timed live with HIP events inside the
library) and the CPU baseline (the NumPy oracle on a bounded sample of layers).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3   # MI355X dense FP32 matrix peak
HBM_PEAK_GBPS = 8000.0           # MI355X HBM3E peak
# HBM bytes per covariance SYRK launch (average over the 161 launches of a step):
# hardware counters FETCH_SIZE and WRITE_SIZE collected with `rocprofv3 --pmc` on
# this script (--no-graph --calibrate-copy), each scaled by what it reads for the
# 256 MiB calibration copy; the counter summary is kept under profiles/.
SYRK_HBM_BYTES_PER_LAUNCH = 41.4e6
BATCH = 32
DAMPING = 2.5e-4
STAB_COEFF = 16.0


def build_model(layers, device, gen):
    """Links with the layer table's shapes plus synthetic per-layer tensors."""
    import torch
    from chainerkfac_amd import links as L
    from chainerkfac_amd import workloads as W
    model = L.Chain()
    calls = []
    for i, layer in enumerate(layers):
        name = 'l{:03d}_{}'.format(i, layer['name'].replace('/', '_'))
        if layer['kind'] == 'conv':
            link = L.Convolution2D(layer['c_in'], layer['c_out'], layer['k'], layer['s'], layer['p'],
                                   nobias=not layer['bias'], device=device, generator=gen)
            ho = W.conv_out(layer['h'], layer['k'], layer['s'], layer['p'])
            x = torch.randn(BATCH, layer['c_in'], layer['h'], layer['w'], device=device, generator=gen)
            gy = torch.randn(BATCH, layer['c_out'], ho, ho, device=device, generator=gen) / (BATCH * ho)
            func = L.Convolution2DFunction()
            in_data = (x, link.W.data) + ((link.b.data,) if layer['bias'] else ())
        elif layer['kind'] == 'linear':
            link = L.Linear(layer['d_in'], layer['d_out'], nobias=not layer['bias'], device=device, generator=gen)
            x = torch.randn(BATCH, layer['d_in'], device=device, generator=gen)
            gy = torch.randn(BATCH, layer['d_out'], device=device, generator=gen) / BATCH
            func = L.LinearFunction()
            in_data = (x, link.W.data) + ((link.b.data,) if layer['bias'] else ())
        else:
            link = L.BatchNormalization(layer['c'], device=device)
            x = torch.randn(BATCH, layer['c'], layer['h'], layer['w'], device=device, generator=gen)
            gy = torch.randn(BATCH, layer['c'], layer['h'], layer['w'], device=device, generator=gen) / (BATCH * layer['h'])
            func = L.BatchNormalizationFunction()
            in_data = (x, link.gamma.data, link.beta.data)
        setattr(model, name, link)
        for p in link.params():
            p.grad = torch.randn(p.shape, device=device, generator=gen)
        calls.append((name, func, in_data, gy))
    return model, calls


def run_gpu(args):
    import torch
    from chainerkfac_amd import _lib
    from chainerkfac_amd import workloads as W
    from chainerkfac_amd.optimizers import KFAC

    lib = _lib.load()
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(3)
    if args.calibrate_copy:
        src = torch.ones(64 << 20, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.add(src, 0.0, out=dst)   # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    layers = W.resnet50_v1()
    flops = W.flops(layers, BATCH)
    model, calls = build_model(layers, dev, gen)
    opt = KFAC(damping=DAMPING, stab_coeff=STAB_COEFF, cov_ema_decay=1.0)
    opt.bn_lowrank_inverse = not args.dense_bn_inverse
    opt.lanes = args.lanes
    opt = opt.setup(model)
    work = [(func, in_data, (gy,)) for _, func, in_data, gy in calls]
    assert len(opt.fblocks) == len(layers)
    hook = opt.kfhook

    # the calls the function hooks make during forward/backward, then KFAC.update_kfgrads in its three parts
    def cov_phase():
        for func, in_data, gy in work:
            hook.forward_postprocess(func, in_data)
            hook.backward_preprocess(func, in_data, gy)
        opt.finish_covs()

    def inv_phase():
        opt.update_cov_emas(opt.fblocks)
        opt.update_invs_batched(opt.fblocks)

    def pre_phase():
        opt.precondition(opt.fblocks)

    def step():
        cov_phase()
        inv_phase()
        pre_phase()

    for _ in range(max(args.warmup, 1)):
        step()
    torch.cuda.synchronize()

    def capture(fn):
        """The launches of ``fn`` as one HIP graph (fixed sequence, fixed buffers):
        the host then pays for a single launch per replay."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        g.replay()
        torch.cuda.synchronize()
        return g.replay

    run = step if args.no_graph else capture(step)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # per-phase split: each phase launched the same way as the step (its own graph), timed with events
    def timed(fn, reps=3):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    phases = {'cov': cov_phase, 'inverse': inv_phase, 'precondition': pre_phase}
    phase_ms = {k: timed(fn if args.no_graph else capture(fn)) for k, fn in phases.items()}

    # wire format of the factors (outside the step: what a communicator would do with them): pack the
    # lower triangles of all 161 factors into one buffer and unpack them again, HBM-bound
    from chainerkfac_amd.communicators import ArrayPacker
    packer = ArrayPacker()
    arrays = [[(cov, True) for fb in opt.fblocks for cov in fb.covs]]
    nel = packer.get_nelems(arrays)
    wire = torch.empty(nel, dtype=torch.float32, device=dev)
    full = sum(c.numel() for c, _ in arrays[0])
    packer._pack_arrays_to_buffer(arrays, wire)
    packer._unpack_arrays_from_buffer(arrays, wire)
    pack_ms = timed(lambda: packer._pack_arrays_to_buffer(arrays, wire), reps=10)
    unpack_ms = timed(lambda: packer._unpack_arrays_from_buffer(arrays, wire), reps=10)
    wire_stats = {
        'pack': {'ms': round(pack_ms, 4), 'GBps': round(8.0 * nel / pack_ms / 1e6, 1),
                 'frac_of_hbm_peak': round(8.0 * nel / pack_ms / 1e6 / HBM_PEAK_GBPS, 3)},
        'unpack': {'ms': round(unpack_ms, 4), 'GBps': round(4.0 * (nel + full) / unpack_ms / 1e6, 1),
                   'frac_of_hbm_peak': round(4.0 * (nel + full) / unpack_ms / 1e6 / HBM_PEAK_GBPS, 3)},
        'packed_MB': round(4.0 * nel / 1e6, 1), 'full_MB': round(4.0 * full / 1e6, 1),
    }

    # dominant kernel family, timed launch by launch inside the library
    # (one stream: with lanes, launches overlap and the time between a launch's events is shared with others)
    opt._lanes.n = 0
    _lib.check(lib.kfac_timing_enable(1))
    step()
    torch.cuda.synchronize()
    opt._lanes.n = args.lanes
    fam = {}
    for name, fid in (('syrk', 0), ('inv_update', 1), ('inv_lauum', 2), ('gemm', 3)):
        n = ctypes.c_int64()
        ms = ctypes.c_double()
        _lib.check(lib.kfac_timing_read(fid, ctypes.byref(n), ctypes.byref(ms)))
        fam[name] = (n.value, ms.value)
    _lib.check(lib.kfac_timing_enable(0))
    info_bad = int((opt.inv_info != 0).sum().item())
    lowrank = [fb for fb in opt.fblocks if getattr(fb, 'lowrank_inverse_args', lambda: None)() is not None] \
        if opt.bn_lowrank_inverse else []
    info_bad += sum(int((fb.inv_info != 0).sum().item()) for fb in lowrank)
    # d^3 of the factors that went through the dense Cholesky path (the reference inverts all 161 densely)
    dense_inverse_flops = flops['inverse'] - sum(float(fb.cov_emas[0].shape[0]) ** 3 for fb in lowrank)

    # What a pair of events adds to the launch it brackets (the time between an
    # event and the neighbouring kernel's edge): bracket nothing, many times.
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(200)]
    torch.cuda.synchronize()
    for e0, e1 in pairs:
        e0.record()
        e1.record()
    torch.cuda.synchronize()
    bracket_ms = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)[len(pairs) // 2]

    syrk_n, syrk_raw_ms = fam['syrk']
    syrk_ms = max(syrk_raw_ms - syrk_n * bracket_ms, 1e-9)
    achieved = flops['cov'] / (syrk_ms * 1e-3) / 1e12 if syrk_n > 0 else 0.0
    total_flops = flops['cov'] + flops['inverse'] + flops['precondition']
    executed_flops = flops['cov'] + dense_inverse_flops + flops['precondition']
    result = {
        'metric': 'ms per K-FAC step, ResNet-50 bs32/GPU; cov+inv TFLOP/s vs FP32 MFMA peak',
        'value': round(ms_per_step, 4),
        'unit': 'ms/step',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': round(ms_per_step, 4),
        'higher_is_better': False,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f32',
        'data': 'synthetic',
        'config': {'workload': 'ResNet-50 v1 (bias, 1000-way) K-FAC step, batch 32 @224: 161 factors, '
                               'cov + damped Cholesky inverse + precondition',
                   'batch': BATCH, 'factors': len(W.all_factor_dims(layers)), 'damping': DAMPING,
                   'hip_graph': not args.no_graph,
            'lanes': args.lanes,
                   'bn_inverse': 'woodbury rank-32 ({} blocks)'.format(len(lowrank)) if lowrank else 'dense'},
        # rates use the flops actually executed; the *_reference_work entries divide the work of the
        # reference's algorithm (all 161 factors inverted densely) by the same times
        'tflops': {
            'step': round(executed_flops / ms_per_step / 1e9, 2),
            'cov_inv': round((flops['cov'] + dense_inverse_flops) / ((phase_ms['cov'] + phase_ms['inverse'])) / 1e9, 2),
            'cov': round(flops['cov'] / phase_ms['cov'] / 1e9, 2),
            'inverse': round(dense_inverse_flops / phase_ms['inverse'] / 1e9, 2),
            'precondition': round(flops['precondition'] / phase_ms['precondition'] / 1e9, 2),
            'frac_of_fp32_mfma_peak': round(executed_flops / ms_per_step / 1e9 / FP32_MFMA_PEAK_TFLOPS, 4),
            'step_reference_work': round(total_flops / ms_per_step / 1e9, 2),
            'inverse_reference_work': round(flops['inverse'] / phase_ms['inverse'] / 1e9, 2),
        },
        'phase_ms': {k: round(v, 3) for k, v in phase_ms.items()},
        'gflop': dict({k: round(v / 1e9, 1) for k, v in flops.items()},
                      inverse_executed=round(dense_inverse_flops / 1e9, 1)),
        'kernel_ms': {k: {'launches': n, 'total_ms': round(ms, 3)} for k, (n, ms) in fam.items()},
        'inverse_info_nonzero': info_bad,
        'wire_format': wire_stats,
        'roofline': {
            'kernel': 'syrk_kernel (covariance, all loaders)',
            'bound': 'mfma',
            'achieved': round(achieved, 2),
            'peak': FP32_MFMA_PEAK_TFLOPS,
            'unit': 'TFLOP/s',
            'frac': round(achieved / FP32_MFMA_PEAK_TFLOPS, 4),
            'launches': syrk_n,
            'avg_launch_ms': round(syrk_ms / max(syrk_n, 1), 4),
            'avg_launch_ms_with_event_bracket': round(syrk_raw_ms / max(syrk_n, 1), 4),
            'event_bracket_ms': round(bracket_ms, 4),
            'timed': 'launches on one stream (--lanes 0 for this pass), HIP events around each launch, empty bracket subtracted',
            'traffic': SYRK_HBM_BYTES_PER_LAUNCH,
            'traffic_unit': 'bytes/launch',
        },
    }
    return result, layers


def write_per_layer(path, layers):
    """Per-layer roofline table of the covariance kernels (markdown): every distinct
    convolution / linear shape of the workload, its A and G factor timed alone on one
    stream (HIP events inside the library around the SYRK launch, empty bracket
    subtracted), against min(FP32 MFMA peak, arithmetic intensity x HBM peak)."""
    import torch
    from chainerkfac_amd import _lib, ops
    from chainerkfac_amd import workloads as W
    lib = _lib.load()
    dev = torch.device('cuda:0')

    def bracket_ms():
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(100)]
        torch.cuda.synchronize()
        for e0, e1 in pairs:
            e0.record()
            e1.record()
        torch.cuda.synchronize()
        return sorted(e0.elapsed_time(e1) for e0, e1 in pairs)[50]

    empty = bracket_ms()

    def syrk_ms(fn, iters=10):
        fn()
        torch.cuda.synchronize()
        _lib.check(lib.kfac_timing_enable(1))
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        n = ctypes.c_int64()
        ms = ctypes.c_double()
        _lib.check(lib.kfac_timing_read(0, ctypes.byref(n), ctypes.byref(ms)))
        _lib.check(lib.kfac_timing_enable(0))
        return max(ms.value / max(n.value, 1) - empty, 1e-6)

    rows = []
    seen = set()
    for layer in layers:
        if layer['kind'] == 'conv':
            key = ('conv', layer['c_in'], layer['c_out'], layer['k'], layer['s'], layer['h'])
        elif layer['kind'] == 'linear':
            key = ('linear', layer['d_in'], layer['d_out'])
        else:
            continue
        count = sum(1 for other in layers if other['kind'] == layer['kind'] and all(
            other.get(f) == layer.get(f) for f in ('c_in', 'c_out', 'k', 's', 'h', 'd_in', 'd_out')))
        if key in seen:
            continue
        seen.add(key)
        dA, dG = W.factor_dims(layer)
        M = W.cov_rows(layer, BATCH)
        if layer['kind'] == 'conv':
            ho = W.conv_out(layer['h'], layer['k'], layer['s'], layer['p'])
            x = torch.randn(BATCH, layer['c_in'], layer['h'], layer['w'], device=dev)
            gy = torch.randn(BATCH, layer['c_out'], ho, ho, device=dev)
            ta = syrk_ms(lambda: ops.cov_conv_a(x, layer['k'], layer['s'], layer['p'], layer['bias'], 1.0 / BATCH))
            tg = syrk_ms(lambda: ops.cov_conv_g(gy, 1.0))
            desc = 'conv {}x{}/{} {}->{} @{}'.format(layer['k'], layer['k'], layer['s'], layer['c_in'], layer['c_out'],
                                                   layer['h'])
        else:
            x = torch.randn(BATCH, layer['d_in'], device=dev)
            gy = torch.randn(BATCH, layer['d_out'], device=dev)
            ta = syrk_ms(lambda: ops.cov_linear(x, layer['bias'], 1.0 / BATCH))
            tg = syrk_ms(lambda: ops.cov_linear(gy, False, float(BATCH)))
            desc = 'linear {}->{}'.format(layer['d_in'], layer['d_out'])
        in_a, in_g = x.numel() * 4.0, gy.numel() * 4.0
        for fac, d, t, in_bytes in (('A', dA, ta, in_a), ('G', dG, tg, in_g)):
            flop = float(M) * d * (d + 1)
            ai = flop / (in_bytes + 4.0 * d * d)
            cap = min(FP32_MFMA_PEAK_TFLOPS, ai * HBM_PEAK_GBPS / 1e3)
            rows.append((desc, count, fac, d, M, flop / 1e9, t * 1e3, flop / t / 1e9, ai, cap, flop / t / 1e9 / cap))
        del x, gy
    with open(path, 'w') as f:
        f.write('| layer (x count) | factor | d | rows M | GFLOP | SYRK kernel us | TFLOP/s | flop/B | roofline cap TFLOP/s '
                '| fraction of cap |\n|---|---|---:|---:|---:|---:|---:|---:|---:|---:|\n')
        for desc, count, fac, d, M, gf, us, tf, ai, cap, frac in rows:
            f.write('| {} (x{}) | {} | {} | {} | {:.2f} | {:.1f} | {:.1f} | {:.0f} | {:.1f} | {:.2f} |\n'.format(
                desc, count, fac, d, M, gf, us, tf, ai, cap, frac))


def run_cpu_baseline(layers, budget_s=20.0):
    """The NumPy oracle (the restatement of the reference's --no_cuda arithmetic)
    on a bounded sample of the workload's layers, scaled to the whole step by
    algorithmic FLOPs."""
    import numpy as np
    from chainerkfac_amd import workloads as W
    from oracle import kfac_oracle as O
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get('num_threads', 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count()
    rng = np.random.default_rng(3)
    total = W.flops(layers, BATCH)
    total_f = sum(total.values())
    # one bottleneck of every stage plus the FC (every kernel kind and every factor size class), in an
    # order that puts the big stage-5 factors last, where the time budget cuts the sample off
    sample = []
    for prefix in ('res3/1/', 'res4/1/', 'fc', 'res2/1/', 'res5/1/', 'res4/2/', 'res5/2/', 'res3/2/'):
        sample += [l for l in layers if l['name'].startswith(prefix) or l['name'] == prefix]
    done_f = 0
    names = []
    t_used = 0.0
    for layer in sample:
        f = sum(W.flops([layer], BATCH).values())
        t0 = time.perf_counter()
        if layer['kind'] == 'conv':
            ho = W.conv_out(layer['h'], layer['k'], layer['s'], layer['p'])
            x = rng.standard_normal((BATCH, layer['c_in'], layer['h'], layer['w']), dtype=np.float32)
            gy = rng.standard_normal((BATCH, layer['c_out'], ho, ho), dtype=np.float32) / (BATCH * ho)
            gW = rng.standard_normal((layer['c_out'], layer['c_in'], layer['k'], layer['k']), dtype=np.float32)
            gb = rng.standard_normal(layer['c_out'], dtype=np.float32) if layer['bias'] else None
            t0 = time.perf_counter()
            A = O.conv_A(x, layer['k'], layer['s'], layer['p'], layer['bias'])
            G = O.conv_G(gy)
        elif layer['kind'] == 'linear':
            x = rng.standard_normal((BATCH, layer['d_in']), dtype=np.float32)
            gy = rng.standard_normal((BATCH, layer['d_out']), dtype=np.float32) / BATCH
            gW = rng.standard_normal((layer['d_out'], layer['d_in']), dtype=np.float32)
            gb = rng.standard_normal(layer['d_out'], dtype=np.float32)
            t0 = time.perf_counter()
            A = O.linear_A(x, True)
            G = O.linear_G(gy)
        else:
            x = rng.standard_normal((BATCH, layer['c'], layer['h'], layer['w']), dtype=np.float32)
            gy = rng.standard_normal((BATCH, layer['c'], layer['h'], layer['w']), dtype=np.float32) / (BATCH * layer['h'])
            gg = rng.standard_normal(layer['c'], dtype=np.float32)
            gb = rng.standard_normal(layer['c'], dtype=np.float32)
            t0 = time.perf_counter()
            F = O.bn_F(x, gy, 2e-5)
        if layer['kind'] == 'bn':
            (dv,) = O.bn_diagvals(layer['c'], layer['c'], DAMPING, STAB_COEFF)
            (Finv,) = O.update_invs([F], [dv])
            O.precondition_bn(Finv, gg, gb)
        else:
            dv, _ = O.connection_diagvals(A, G, DAMPING)
            Ainv, Ginv = O.update_invs([A, G], dv)
            O.precondition_conn(Ainv, Ginv, gW, gb)
        t_used += time.perf_counter() - t0
        done_f += f
        names.append(layer['name'])
        if t_used > budget_s:
            break
    est_ms = t_used * 1e3 * total_f / done_f
    return {
        'value': round(est_ms, 1),
        'unit': 'ms/step',
        'cores': int(threads),
        'kind': 'port',
        'sample': 'NumPy oracle (cov + damped inverse + precondition) on layers {} = {:.1f} of {:.1f} GFLOP '
                  'in {:.1f} s, scaled by FLOPs'.format(','.join(names), done_f / 1e9, total_f / 1e9, t_used),
    }


def main():
    import faulthandler
    faulthandler.enable()   # a crash inside a native call still names the Python line it came from
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=3)
    ap.add_argument('--no-graph', action='store_true', help='launch every kernel from the host each step')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    ap.add_argument('--dense-bn-inverse', action='store_true',
                    help='invert the batch-norm blocks with the dense Cholesky path as well (default: their '
                         'rank-32 Woodbury form, which yields the same dense inverse)')
    ap.add_argument('--lanes', type=int, default=3,
                    help='side streams for the per-layer factor and preconditioning kernels (0 = one stream)')
    ap.add_argument('--per-layer', metavar='PATH', default=None,
                    help='also time the covariance kernels of every distinct layer shape alone and write a '
                         'markdown roofline table to PATH')
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='first run one 256 MiB device-to-device elementwise copy (a kernel of known traffic, '
                         'the reference point for hardware byte counters collected under rocprofv3 --pmc)')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py measures the single-GPU K-FAC hot path: inter-GPU collectives are outside this '
                 'build, so --gpus must be 1 (got {})'.format(args.gpus))
    result, layers = run_gpu(args)
    if args.per_layer:
        write_per_layer(args.per_layer, layers)
    if not args.no_cpu:
        result['cpu_baseline'] = run_cpu_baseline(layers)
    print(json.dumps(result))


if __name__ == '__main__':
    main()
