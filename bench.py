#!/usr/bin/env python
"""Benchmark of the K-FAC per-layer hot path on one MI355X.

    python bench.py [--config c3] [--gpus 1] [--steps K] [--warmup W] [--no-graph] [--no-cpu]

Headline workload (--config c3, the default): ResNet-50 (bottleneck v1, 1000-way
FC, all convs with bias) K-FAC step on one GPU's share, batch 32 at 224x224,
fp32: for all 161 Kronecker factors, covariance (fused im2col SYRK) + pi-damped
Cholesky inverse + gradient preconditioning.  Per-layer activations, output
gradients and parameter gradients are synthetic N(0,1) tensors of the real
shapes (output gradients scaled by 1/(batch*sqrt(pixels)), the size a
mean-reduced loss gives them, which keeps the rank-32 batch-norm factors
positive definite in float32), resident in HBM before the timed region.  The
step is driven through the drop-in host classes (the function hook's
forward_postprocess / backward_preprocess calls, KFAC.update_kfgrads).

The other configurations of the benchmark definition run the same way:
  c1  MLP 784-1000-1000-10, batch 128, damping 1e-3 (6 factors)
  c2  CIFAR-shaped CNN, batch 128, damping 1e-3 (8 factors, up to 4097^2)
  c4  inverse only: 161 SPD matrices of ResNet-50's factor sizes (27^2 .. 4609^2)
  c5  ResNet-50-D shapes, batch 32, acc_iters = 16: 16 micro-batches accumulated by
      the covariance kernels, then triangular pack and unpack of all factors and
      gradients, damped inverse, preconditioning

Prints ONE JSON line: ms per step (a step = one pass of the configuration's hot
path), per-phase TFLOP/s, the roofline of the dominant kernel family (timed
live with HIP events inside the library) and the CPU baseline (the NumPy oracle
on a bounded sample of the same workload).
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
# HBM bytes per launch of the covariance SYRK family, written by
# `bench.py --summarize-traffic` from two `rocprofv3 --pmc` runs (FETCH_SIZE, WRITE_SIZE)
TRAFFIC_FILE = os.path.join(ROOT, 'profiles', 'syrk_hbm_traffic.json')
BATCH = 32
DAMPING = 2.5e-4
STAB_COEFF = 16.0
METRIC = 'ms per K-FAC step, ResNet-50 bs32/GPU; cov+inv TFLOP/s vs FP32 MFMA peak'


def configs():
    from chainerkfac_amd import workloads as W
    return {
        'c1': dict(layers=W.mlp_mnist(), batch=128, damping=1e-3, decay=0.99, acc_iters=1,
                   workload='MLP 784-1000-1000-10 (bias) K-FAC step, batch 128: 6 factors, '
                            'cov + damped Cholesky inverse + precondition'),
        'c2': dict(layers=W.cifar_cnn(), batch=128, damping=1e-3, decay=0.99, acc_iters=1,
                   workload='CIFAR-shaped CNN (3 conv3x3 + FC 4096->10) K-FAC step, batch 128: 8 factors '
                            'up to 4097^2, cov + damped Cholesky inverse + precondition'),
        'c3': dict(layers=W.resnet50_v1(), batch=BATCH, damping=DAMPING, decay=1.0, acc_iters=1,
                   workload='ResNet-50 v1 (bias, 1000-way) K-FAC step, batch 32 @224: 161 factors, '
                            'cov + damped Cholesky inverse + precondition'),
        'c4': dict(layers=None, batch=0, damping=1e-3, decay=1.0, acc_iters=1,
                   workload='inverse only: 161 SPD fp32 matrices of ResNet-50 factor sizes (27^2 .. 4609^2), '
                            'X^T X / n + 1e-3 I, damped Cholesky inverse of all of them'),
        'c5': dict(layers=W.resnet50_d(), batch=BATCH, damping=DAMPING, decay=1.0, acc_iters=16,
                   workload='ResNet-50-D shapes, batch 32, acc_iters 16: covariances of 16 micro-batches '
                            'accumulated (167 factors), triangular pack + unpack of factors and gradients, '
                            'damped inverse, precondition'),
    }


def build_model(layers, device, gen, batch=None):
    """Links with the layer table's shapes plus synthetic per-layer tensors."""
    import torch
    from chainerkfac_amd import links as L
    from chainerkfac_amd import workloads as W
    batch = BATCH if batch is None else batch
    model = L.Chain()
    calls = []
    for i, layer in enumerate(layers):
        name = 'l{:03d}_{}'.format(i, layer['name'].replace('/', '_'))
        if layer['kind'] == 'conv':
            link = L.Convolution2D(layer['c_in'], layer['c_out'], layer['k'], layer['s'], layer['p'],
                                   nobias=not layer['bias'], device=device, generator=gen)
            ho = W.conv_out(layer['h'], layer['k'], layer['s'], layer['p'])
            x = torch.randn(batch, layer['c_in'], layer['h'], layer['w'], device=device, generator=gen)
            gy = torch.randn(batch, layer['c_out'], ho, ho, device=device, generator=gen) / (batch * ho)
            func = L.Convolution2DFunction()
            in_data = (x, link.W.data) + ((link.b.data,) if layer['bias'] else ())
        elif layer['kind'] == 'linear':
            link = L.Linear(layer['d_in'], layer['d_out'], nobias=not layer['bias'], device=device, generator=gen)
            x = torch.randn(batch, layer['d_in'], device=device, generator=gen)
            gy = torch.randn(batch, layer['d_out'], device=device, generator=gen) / batch
            func = L.LinearFunction()
            in_data = (x, link.W.data) + ((link.b.data,) if layer['bias'] else ())
        else:
            link = L.BatchNormalization(layer['c'], device=device)
            x = torch.randn(batch, layer['c'], layer['h'], layer['w'], device=device, generator=gen)
            gy = torch.randn(batch, layer['c'], layer['h'], layer['w'], device=device, generator=gen) / (batch * layer['h'])
            func = L.BatchNormalizationFunction()
            in_data = (x, link.gamma.data, link.beta.data)
        setattr(model, name, link)
        for p in link.params():
            p.grad = torch.randn(p.shape, device=device, generator=gen)
        calls.append((name, func, in_data, gy))
    return model, calls


def _events(n):
    import torch
    return [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]


def bracket_ms():
    """What a pair of events adds to the launch it brackets (the time between an event and
    the neighbouring kernel's edge): bracket nothing, many times, take the median."""
    import torch
    pairs = _events(200)
    torch.cuda.synchronize()
    for e0, e1 in pairs:
        e0.record()
        e1.record()
    torch.cuda.synchronize()
    return sorted(e0.elapsed_time(e1) for e0, e1 in pairs)[len(pairs) // 2]


def capture(fn):
    """The launches of ``fn`` as one HIP graph (fixed sequence, fixed buffers): the host then
    pays for a single launch per replay."""
    import torch
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


def timed_steps(run, steps):
    """EXACTLY ``steps`` calls of ``run`` between two synchronisations: (mean ms over the
    wall clock, median ms over per-call event pairs)."""
    import torch
    pairs = _events(steps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for e0, e1 in pairs:
        e0.record()
        run()
        e1.record()
    torch.cuda.synchronize()
    mean = (time.perf_counter() - t0) * 1e3 / steps
    each = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)
    return mean, each[len(each) // 2]


def timed(fn, reps=11):
    import torch
    pairs = _events(reps)
    torch.cuda.synchronize()
    for e0, e1 in pairs:
        e0.record()
        fn()
        e1.record()
    torch.cuda.synchronize()
    return sorted(e0.elapsed_time(e1) for e0, e1 in pairs)[reps // 2]


FAMILY_IDS = (('syrk', 0), ('inv_update', 1), ('inv_lauum', 2), ('gemm', 3), ('pack', 4), ('unpack', 5), ('copy', 6),
              ('cov_aux', 7), ('bn_stats', 8), ('inv_call', 9), ('gemm_aux', 10))


def family_times(lib):
    """(launches, summed ms between the HIP events) of every timed kernel family since timing was enabled."""
    from chainerkfac_amd import _lib
    fam = {}
    for name, fid in FAMILY_IDS:
        n = ctypes.c_int64()
        ms = ctypes.c_double()
        _lib.check(lib.kfac_timing_read(fid, ctypes.byref(n), ctypes.byref(ms)))
        fam[name] = (n.value, ms.value)
    return fam


def family_roofline(label, kernels, flop, members, fam, empty, note, reference_flop=None):
    """Roofline entry of one kernel family: `flop` is the work its kernels are given (issued
    multiply-adds x 2), the time is the sum of the event brackets of `members` (each bracket less
    what an empty bracket measures)."""
    n = sum(fam[m][0] for m in members)
    ms = sum(max(fam[m][1] - fam[m][0] * empty, 0.0) for m in members)
    rate = flop / (ms * 1e-3) / 1e12 if ms > 0 else 0.0
    out = {'kernel': kernels, 'bound': 'mfma', 'achieved': round(rate, 2), 'peak': FP32_MFMA_PEAK_TFLOPS,
           'unit': 'TFLOP/s', 'frac': round(rate / FP32_MFMA_PEAK_TFLOPS, 4),
           'gflop_per_step': round(flop / 1e9, 1), 'kernel_ms_per_step': round(ms, 4), 'brackets': n,
           'avg_bracket_ms': round(ms / max(n, 1), 4), 'timed': note}
    if reference_flop is not None and ms > 0:
        # the work of the reference's algorithm for the same result over the same time: a labelled
        # extra, not a utilisation (it exceeds the peak where this build issues fewer flops)
        out['reference_work_gflop_per_step'] = round(reference_flop / 1e9, 1)
        out['reference_work_rate'] = round(reference_flop / (ms * 1e-3) / 1e12, 2)
    return out


def read_traffic():
    """The record `bench.py --summarize-traffic` wrote from two counter runs, or None."""
    try:
        with open(TRAFFIC_FILE) as f:
            return json.load(f)
    except (OSError, ValueError):
        return None


def wire_format(arrays, dev, lib):
    """Triangular pack / unpack of ``arrays`` (bandwidth-bound), beside a plain streaming copy
    of the same number of bytes through the library's own copy kernel."""
    import torch
    from chainerkfac_amd import _lib
    from chainerkfac_amd.communicators import ArrayPacker
    packer = ArrayPacker()
    nel = packer.get_nelems(arrays)
    wire = torch.empty(nel, dtype=torch.float32, device=dev)
    full = sum(a.numel() for a, _ in arrays[0])
    packer._pack_arrays_to_buffer(arrays, wire)
    packer._unpack_arrays_from_buffer(arrays, wire)
    pack_ms = timed(lambda: packer._pack_arrays_to_buffer(arrays, wire), reps=11)
    unpack_ms = timed(lambda: packer._unpack_arrays_from_buffer(arrays, wire), reps=11)
    n_copy = (nel + full) // 2 // 4 * 4     # moves as many bytes as the unpack
    src = torch.ones(n_copy, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    stream = torch.cuda.current_stream().cuda_stream
    copy_ms = timed(lambda: _lib.check(lib.kfac_stream_copy_f32(dst.data_ptr(), src.data_ptr(), n_copy, stream)),
                    reps=11)
    # and a copy with the unpack's mix: n elements read, 2 n written, the same number of bytes
    n_fan = (nel + full) // 3 // 4 * 4
    dst2 = torch.empty(n_fan, dtype=torch.float32, device=dev)
    fan_ms = timed(lambda: _lib.check(lib.kfac_stream_fanout_f32(dst.data_ptr(), dst2.data_ptr(), src.data_ptr(), n_fan,
                                                                 stream)), reps=11)
    del src, dst, dst2
    copy_gbps = 8.0 * n_copy / copy_ms / 1e6
    fan_gbps = 12.0 * n_fan / fan_ms / 1e6
    out = {
        'arrays': len(arrays[0]), 'triangular': sum(1 for _, t in arrays[0] if t),
        'pack': {'ms': round(pack_ms, 4), 'GBps': round(8.0 * nel / pack_ms / 1e6, 1)},
        'unpack': {'ms': round(unpack_ms, 4), 'GBps': round(4.0 * (nel + full) / unpack_ms / 1e6, 1)},
        'stream_copy': {'ms': round(copy_ms, 4), 'GBps': round(copy_gbps, 1), 'bytes': 8 * n_copy},
        # one read, two writes per element: the traffic mix of the unpack
        'stream_fanout': {'ms': round(fan_ms, 4), 'GBps': round(fan_gbps, 1), 'bytes': 12 * n_fan},
        'packed_MB': round(4.0 * nel / 1e6, 1), 'full_MB': round(4.0 * full / 1e6, 1),
    }
    for k in ('pack', 'unpack', 'stream_copy', 'stream_fanout'):
        out[k]['frac_of_hbm_peak'] = round(out[k]['GBps'] / HBM_PEAK_GBPS, 3)
    for k in ('pack', 'unpack'):
        out[k]['frac_of_stream_copy'] = round(out[k]['GBps'] / copy_gbps, 3)
    out['unpack']['frac_of_stream_fanout'] = round(out['unpack']['GBps'] / fan_gbps, 3)
    return out, wire


def run_step_config(args, name, cfg, host=None):
    """c1, c2, c3, c5: cov (x acc_iters) [+ pack/unpack] + inverse + precondition."""
    import torch
    from chainerkfac_amd import _lib
    from chainerkfac_amd import workloads as W
    from chainerkfac_amd.optimizers import KFAC
    from chainerkfac_amd.optimizers.kfac import extract

    lib = _lib.load()
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(3)
    if args.calibrate_copy:
        from chainerkfac_amd import _lib
        src = torch.ones(64 << 20, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        # stream_copy_kernel: reads 256 MiB, writes 256 MiB
        _lib.check(_lib.load().kfac_stream_copy_f32(dst.data_ptr(), src.data_ptr(), src.numel(), None))
        torch.cuda.synchronize()
        del src, dst
    layers, batch, acc_iters = cfg['layers'], cfg['batch'], cfg['acc_iters']
    flops = W.flops(layers, batch)
    flops['cov'] *= acc_iters
    model, calls = build_model(layers, dev, gen, batch)
    opt = KFAC(damping=cfg['damping'], stab_coeff=STAB_COEFF, cov_ema_decay=cfg['decay'], acc_iters=acc_iters)
    opt.bn_lowrank_inverse = not args.dense_bn_inverse
    opt.lanes = args.lanes
    opt = opt.setup(model)
    work = [(func, in_data, (gy,)) for _, func, in_data, gy in calls]
    assert len(opt.fblocks) == len(layers)
    hook = opt.kfhook

    # the calls the function hooks make during forward/backward (per micro-batch), then
    # KFAC.update_kfgrads in its three parts
    def cov_phase():
        for it in range(acc_iters):
            for fb in opt.fblocks:
                fb.acc_state = (acc_iters, it)
            for func, in_data, gy in work:
                hook.forward_postprocess(func, in_data)
                hook.backward_preprocess(func, in_data, gy)
            opt.finish_covs()
            if acc_iters > 1:
                opt.accumulate_covs()

    wire_state = {}

    def wire_phase():
        # what the communicator does with a rank's factors and gradients (configuration c5):
        # pack into one flat buffer in the reference's order, unpack again
        if 'arrays' not in wire_state:
            from chainerkfac_amd.communicators import ArrayPacker
            arrays = extract(opt.fblocks, [range(len(opt.fblocks))], lambda b: b.extract_for_reduce_scatter_v())
            packer = ArrayPacker()
            wire_state.update(arrays=arrays, packer=packer,
                              buf=torch.empty(packer.get_nelems(arrays), dtype=torch.float32, device=dev))
        wire_state['packer']._pack_arrays_to_buffer(wire_state['arrays'], wire_state['buf'])
        wire_state['packer']._unpack_arrays_from_buffer(wire_state['arrays'], wire_state['buf'])

    def inv_phase():
        opt.update_cov_emas(opt.fblocks)
        opt.update_invs_batched(opt.fblocks)

    def pre_phase():
        opt.precondition(opt.fblocks)

    with_wire = name == 'c5'

    def step():
        cov_phase()
        if with_wire:
            wire_phase()
        inv_phase()
        pre_phase()

    if args.host_launch_child:
        # no lane exists before the brackets have been read (the pool of streams is made on first use)
        opt._lanes.n = 0
        _lib.set_option('group_side_stream', 0)
    for _ in range(max(args.warmup, 1)):
        step()
    torch.cuda.synchronize()

    def host_launched():
        """Every kernel family timed bracket by bracket inside the library, on one stream (with
        lanes, launches overlap and the time between a launch's events is shared with others);
        then the step launched kernel by kernel from the host with the lanes back on: what a
        caller of the drop-in classes gets without capturing a graph of its own."""
        opt._lanes.n = 0
        _lib.set_option('group_side_stream', 0)
        step()
        torch.cuda.synchronize()
        _lib.check(lib.kfac_timing_enable(1))
        step()
        torch.cuda.synchronize()
        fam = family_times(lib)
        _lib.check(lib.kfac_timing_enable(0))
        empty = bracket_ms()
        opt._lanes.n = args.lanes
        _lib.set_option('group_side_stream', None if args.lanes else 0)
        for _ in range(3):
            step()
        eager, _ = timed_steps(step, max(args.steps, 5))
        # how long the host takes to queue a step (no synchronisation until the last one is queued)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            step()
        queued = (time.perf_counter() - t0) * 1e3 / 5
        torch.cuda.synchronize()
        return {'eager_ms_per_step': eager, 'host_ms_to_queue_a_step': queued, 'lanes': args.lanes, 'fam': fam,
                'empty': empty, 'info_bad': len(opt.check_numerics())}

    if args.host_launch_child:
        return host_launched()
    run = step if args.no_graph else capture(step)
    ms_per_step, ms_median = timed_steps(run, args.steps)
    replay_equals_eager = None
    if not args.no_graph:
        # the timed replays must have computed what the eager step computes: every factor inverse
        # and every preconditioned gradient, bit for bit (a step of these configurations has no
        # history, so the eager step afterwards starts from the same inputs)
        def results():
            return [t.clone() for fb in opt.fblocks for t in fb.invs] + \
                   [p.kfgrad.clone() for _, p in sorted(model.namedparams()) if getattr(p, 'kfgrad', None) is not None]
        replayed = results()
        step()
        torch.cuda.synchronize()
        eager = results()
        replay_equals_eager = len(eager) == len(replayed) and all(torch.equal(a, b) for a, b in zip(replayed, eager))
        del replayed, eager

    # per-phase split: each phase launched the same way as the step (its own graph), timed with events
    phases = {'cov': cov_phase, 'inverse': inv_phase, 'precondition': pre_phase}
    if with_wire:
        phases['pack_unpack'] = wire_phase
    phase_ms = {k: timed(fn if args.no_graph else capture(fn)) for k, fn in phases.items()}

    # wire format of the factors (and, for c5, of the gradients too): outside the step for the
    # configurations whose step has no communication
    if with_wire:
        arrays = wire_state['arrays']
    else:
        arrays = [[(cov, True) for fb in opt.fblocks for cov in fb.covs]]
    wire_stats, _ = wire_format(arrays, dev, lib)

    extras = {}
    if not args.no_extras:
        # the momentum rule over all parameters (the reference's next call after the preconditioning,
        # optimizers/kfac.py:250-252): not part of `value`, timed the same way as the phases
        def update_phase():
            opt.update_params()

        update_ms = {}
        for label, batched in (('batched', True), ('per_parameter', False)):
            opt.batch_param_updates = batched
            update_phase()
            update_ms[label] = timed(update_phase if args.no_graph else capture(update_phase))
        opt.batch_param_updates = True
        n_param_arrays = len(list(model.params()))
        n_params = sum(p.data.numel() for p in model.params())

        # the moving average of all factors in a step that has history (cov_ema_decay = 0.99, the
        # reference's default; the first step, which `value` times for c3 - c5, only aliases)
        for fb in opt.fblocks:
            fb.cov_ema_decay, fb.cov_emas = 0.99, None

        def ema_phase():
            opt.update_cov_emas(opt.fblocks)

        ema_phase()   # the first call copies
        ema_ms = {}
        for label, batched in (('batched', True), ('per_array', False)):
            opt.batch_elementwise = batched
            ema_phase()
            ema_ms[label] = timed(ema_phase if args.no_graph else capture(ema_phase))
        opt.batch_elementwise = True
        n_factor_arrays = sum(len(fb.covs) for fb in opt.fblocks)
        n_factor_elems = sum(c.numel() for fb in opt.fblocks for c in fb.covs)
        for fb in opt.fblocks:
            fb.cov_ema_decay, fb.cov_emas = cfg['decay'], None
        inv_phase()   # back to this configuration's own averages and inverses
        extras = {
            # v = momentum v - lr kfgrad; param += v over every parameter: 20 bytes per element
            'param_update': {'parameters': n_params, 'arrays': n_param_arrays,
                             'one_launch_ms': round(update_ms['batched'], 4),
                             'launch_per_parameter_ms': round(update_ms['per_parameter'], 4),
                             'one_launch_tb_s': round(20.0 * n_params / (update_ms['batched'] * 1e-3) / 1e12, 3),
                             'frac_of_hbm_peak': round(20.0 * n_params / (update_ms['batched'] * 1e-3) / 1e12 / 8.0, 3),
                             'in_value': False},
            # ema = 0.99 cov + 0.01 ema over every factor: 12 bytes per element
            'moving_average': {'elements': n_factor_elems, 'arrays': n_factor_arrays,
                               'one_launch_ms': round(ema_ms['batched'], 4),
                               'launch_per_array_ms': round(ema_ms['per_array'], 4),
                               'one_launch_tb_s': round(12.0 * n_factor_elems / (ema_ms['batched'] * 1e-3) / 1e12, 3),
                               'frac_of_hbm_peak': round(12.0 * n_factor_elems / (ema_ms['batched'] * 1e-3) / 1e12 / 8.0, 3),
                               'in_value': False}}

    # Launches made from the host: the per-family event brackets and the eager step time, measured
    # here when the caller has not already measured them in a process of their own (see main).
    if host is None:
        host = host_launched()
    real_network = host.pop('real_network', None)
    eager_ms, eager_lanes = host['eager_ms_per_step'], host['lanes']
    fam = {k: tuple(v) for k, v in host['fam'].items()}
    empty = host['empty']
    info_bad = host['info_bad']
    lowrank = [fb for fb in opt.fblocks if getattr(fb, 'lowrank_inverse_args', lambda: None)() is not None] \
        if opt.bn_lowrank_inverse else []
    # d^3 of the factors that went through the dense Cholesky path (the reference inverts all of them densely)
    dense_inverse_flops = flops['inverse'] - sum(float(fb.cov_emas[0].shape[0]) ** 3 for fb in lowrank)

    # what the matrix cores are actually given: 3x3 stride-1 convolutions compute their A factor from
    # shifted correlations, about a third of the multiply-adds of the patch product
    cov_executed = float(W.cov_flops_executed(layers, batch)) * acc_iters
    executed_flops = cov_executed + dense_inverse_flops + flops['precondition']
    total_flops = flops['cov'] + flops['inverse'] + flops['precondition']
    one_stream = 'launches on one stream (--lanes 0 for this pass), HIP events around each launch, empty bracket subtracted'
    families = {
        'cov_syrk': family_roofline(
            'cov_syrk', 'covariance SYRK family: shift::corr_kernel, syrk_rows_kernel, syrk_group_kernel, syrk_kernel, '
            'syrk_conv_kernel and the kernels around them (edge_sums, corr_finish, assemble, finish_group, finish, reduce)',
            cov_executed, ('syrk', 'cov_aux'), fam, empty, one_stream, reference_flop=flops['cov']),
        'inverse_tiles': family_roofline(
            'inverse_tiles', 'batched dense inverse: copy_in, diag, update, panel, border, lauum kernels',
            dense_inverse_flops, ('inv_call',), fam, empty,
            'd^3 flop of the densely inverted factors over the time between the first and the last launch of the '
            'batched call (its kernels overlap on three streams, so their durations do not add up)',
            reference_flop=flops['inverse']),
        'precond_gemm': family_roofline(
            'precond_gemm', 'preconditioning GEMMs: gemm_group_kernel (both phases), gemm_group_finish_kernel, '
            'gemv_kernel + bn_select_kernel of the batch-norm blocks',
            flops['precondition'], ('gemm', 'gemm_aux'), fam, empty, one_stream),
    }
    main_syrk = family_roofline('', '', cov_executed, ('syrk',), fam, empty, '')
    families['cov_syrk']['main_kernels_only'] = {
        'launches': main_syrk['brackets'], 'kernel_ms_per_step': main_syrk['kernel_ms_per_step'],
        'achieved': main_syrk['achieved'], 'frac': main_syrk['frac']}
    # HBM bytes per step of every family, from hardware counters of an earlier profiling run of this
    # configuration (profiles/), beside the bytes the algorithm has to move
    record = read_traffic() if name == 'c3' else None
    factor_bytes = 4.0 * sum(float(c.numel()) for fb in opt.fblocks for c in fb.covs)
    input_bytes = 4.0 * sum(float(in_data[0].numel()) + float(gy[0].numel()) for _, in_data, gy in work)
    dense_bytes = 4.0 * sum(float(c.numel()) for fb in opt.fblocks if fb not in lowrank for c in fb.cov_emas)
    grad_bytes = 4.0 * sum(float(p.data.numel()) for p in model.params())
    algorithmic = {'cov_syrk': (input_bytes + factor_bytes) * acc_iters,   # inputs read, factors written
                   'inverse_tiles': 2.0 * dense_bytes,                         # factors read, inverses written
                   'precond_gemm': factor_bytes + 2.0 * grad_bytes}            # inverses and gradients read, kfgrads written
    for fam_name, fam_entry in families.items():
        measured = None if record is None else record.get('families', {}).get(fam_name, {}).get('bytes_per_step')
        fam_entry['traffic'] = None if measured is None else round(measured / max(fam_entry['brackets'], 1), 1)
        fam_entry['traffic_unit'] = 'HBM bytes per bracket (the family\'s bytes per step over its brackets per step)'
        fam_entry['traffic_bytes_per_step'] = measured
        fam_entry['algorithmic_bytes_per_step'] = algorithmic[fam_name]
    families['cov_syrk']['traffic_main_kernels_per_launch'] = None if record is None else record.get('bytes_per_launch')
    dominant = max(families, key=lambda k: families[k]['kernel_ms_per_step'])
    roofline = dict(families[dominant])
    roofline['family'] = dominant
    roofline['event_bracket_ms'] = round(empty, 4)
    roofline['families'] = families
    result = {
        'metric': METRIC,
        'value': round(ms_per_step, 4),
        'unit': 'ms/step',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': round(ms_per_step, 4),
        'ms_per_step_median': round(ms_median, 4),
        'higher_is_better': False,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f32',
        'data': 'synthetic',
        'config': {'workload': cfg['workload'], 'name': name, 'batch': batch,
                   'factors': len(W.all_factor_dims(layers)), 'damping': cfg['damping'], 'acc_iters': acc_iters,
                   'cov_ema_decay': cfg['decay'],
                   'hip_graph': not args.no_graph, 'lanes': args.lanes, 'macro_tiles': bool(args.macro_tiles),
                   'bn_inverse': 'woodbury rank-{} ({} blocks)'.format(batch, len(lowrank)) if lowrank else 'dense'},
        # rates use the flops actually executed; the *_reference_work entries divide the work of the
        # reference's algorithm (every factor a patch / activation product, every factor inverted densely)
        # by the same times
        'tflops': {
            'step': round(executed_flops / ms_per_step / 1e9, 2),
            'cov_inv': round((cov_executed + dense_inverse_flops) / ((phase_ms['cov'] + phase_ms['inverse'])) / 1e9, 2),
            'cov': round(cov_executed / phase_ms['cov'] / 1e9, 2),
            'cov_reference_work': round(flops['cov'] / phase_ms['cov'] / 1e9, 2),
            'inverse': round(dense_inverse_flops / phase_ms['inverse'] / 1e9, 2),
            'precondition': round(flops['precondition'] / phase_ms['precondition'] / 1e9, 2),
            'frac_of_fp32_mfma_peak': round(executed_flops / ms_per_step / 1e9 / FP32_MFMA_PEAK_TFLOPS, 4),
            'step_reference_work': round(total_flops / ms_per_step / 1e9, 2),
            'inverse_reference_work': round(flops['inverse'] / phase_ms['inverse'] / 1e9, 2),
        },
        'phase_ms': {k: round(v, 3) for k, v in phase_ms.items()},
        'phase_ms_timed': 'each phase as its own HIP graph, median of 11 replays',
        'gflop': dict({k: round(v / 1e9, 1) for k, v in flops.items()},
                      inverse_executed=round(dense_inverse_flops / 1e9, 1), cov_executed=round(cov_executed / 1e9, 1)),
        'kernel_ms': {k: {'launches': n, 'total_ms': round(ms - n * empty, 3)} for k, (n, ms) in fam.items() if n},
        'inverse_info_nonzero': info_bad,
        'wire_format': wire_stats,
        'roofline': roofline,
    }
    if replay_equals_eager is not None:
        result['graph_replay_equals_eager_step'] = replay_equals_eager
    result['eager_ms_per_step'] = round(eager_ms, 4)
    result['eager_lanes'] = eager_lanes
    result['eager_host_ms_to_queue_a_step'] = round(host['host_ms_to_queue_a_step'], 3)
    if real_network is not None:
        result['real_network'] = real_network
    result.update(extras)
    if name == 'c3' and lowrank and not args.no_dense_field:
        # the reference's algorithm inverts the batch-norm blocks densely as well: the same step with
        # the Woodbury shortcut switched off, as a second figure
        opt.bn_lowrank_inverse = False
        for _ in range(2):
            step()
        torch.cuda.synchronize()
        run_dense = step if args.no_graph else capture(step)
        dense_ms, dense_median = timed_steps(run_dense, max(args.steps // 2, 5))
        inv_dense = timed(inv_phase if args.no_graph else capture(inv_phase))
        result['dense_bn_inverse'] = {
            'ms_per_step': round(dense_ms, 4), 'ms_per_step_median': round(dense_median, 4),
            'inverse_ms': round(inv_dense, 3),
            'inverse_tflops': round(flops['inverse'] / inv_dense / 1e9, 2),
            'step_tflops': round(total_flops / dense_ms / 1e9, 2)}
        # a step with history: cov_ema_decay = 0.99 (the reference's default), so every factor is averaged
        # into its moving average (one launch over all factors) and every batch-norm block is inverted
        # densely (its moving average is no longer this step's rank-n matrix)
        opt.bn_lowrank_inverse = True
        for fb in opt.fblocks:
            fb.cov_ema_decay, fb.cov_emas = 0.99, None
        for _ in range(2):
            step()      # the first call copies, the second averages
        torch.cuda.synchronize()
        run_steady = step if args.no_graph else capture(step)
        steady_ms, steady_median = timed_steps(run_steady, max(args.steps // 2, 5))
        result['steady_state'] = {
            'cov_ema_decay': 0.99, 'bn_inverse': 'dense', 'ms_per_step': round(steady_ms, 4),
            'ms_per_step_median': round(steady_median, 4),
            'step_tflops_reference_work': round(total_flops / steady_ms / 1e9, 2)}
        for fb in opt.fblocks:
            fb.cov_ema_decay, fb.cov_emas = cfg['decay'], None
    return result


def host_launch_child(args, name, real_network=False):
    """Runs this script again, in a process of its own, for the measurements of launches made
    from the host (see run_step_config) and returns what it printed."""
    import subprocess
    from chainerkfac_amd.optimizers import KFAC
    cmd = [sys.executable, os.path.abspath(__file__), '--config', name, '--host-launch-child', '--no-graph',
           '--no-cpu', '--lanes', str(min(args.lanes, KFAC.lanes)), '--steps', str(max(min(args.steps, 20), 5)),
           '--warmup', str(max(args.warmup, 1))]
    if args.dense_bn_inverse:
        cmd.append('--dense-bn-inverse')
    if args.macro_tiles:
        cmd.append('--macro-tiles')
    if real_network:
        cmd.append('--real-network')
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
    lines = [l for l in proc.stdout.decode().splitlines() if l.startswith('{')]
    if proc.returncode != 0 or not lines:
        raise RuntimeError('the host-launch measurement failed:\n' + proc.stderr.decode()[-3000:])
    return json.loads(lines[-1])


def inverse_dims():
    """The 161 factor sizes of ResNet-50 with the 3x3 no-bias stem of the reference's own model
    file (27 instead of 148): the stated range 27^2 .. 4609^2."""
    from chainerkfac_amd import workloads as W
    dims = W.all_factor_dims(W.resnet50_v1())
    dims[dims.index(148)] = 27
    return dims


def run_inverse_config(args, name, cfg):
    """c4: damped Cholesky inverse of 161 SPD matrices."""
    import torch
    from chainerkfac_amd import _lib, ops
    lib = _lib.load()
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(4)
    dims = inverse_dims()
    mats = []
    for d in dims:
        X = torch.randn(2 * d, d, device=dev, generator=gen)
        mats.append(X.T @ X / (2 * d) + 1e-3 * torch.eye(d, device=dev))
        del X
    outs = [torch.empty_like(m) for m in mats]
    info = torch.zeros(len(mats), dtype=torch.int32, device=dev)

    def step():
        ops.spd_inverse_batched(mats, outs=outs, info=info)

    for _ in range(max(args.warmup, 1)):
        step()
    torch.cuda.synchronize()

    run = step if args.no_graph else capture(step)
    ms_per_step, ms_median = timed_steps(run, args.steps)
    _lib.check(lib.kfac_timing_enable(1))
    step()
    torch.cuda.synchronize()
    fam = family_times(lib)
    _lib.check(lib.kfac_timing_enable(0))
    empty = bracket_ms()
    worst = 0.0
    seen = set()
    for d, M, inv in zip(dims, mats, outs):
        if d in seen:
            continue
        seen.add(d)
        resid = float((M.double() @ inv.double() - torch.eye(d, device=dev, dtype=torch.float64)).norm()) / d ** 0.5
        worst = max(worst, resid)
    flop = float(sum(d ** 3 for d in dims))
    achieved = flop / ms_per_step / 1e9
    return {
        'metric': METRIC, 'value': round(ms_per_step, 4), 'unit': 'ms/step', 'n_gpus': 1, 'steps': args.steps,
        'warmup': args.warmup, 'ms_per_step': round(ms_per_step, 4), 'ms_per_step_median': round(ms_median, 4),
        'higher_is_better': False, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': cfg['workload'], 'name': name, 'factors': len(dims), 'hip_graph': not args.no_graph},
        'tflops': {'inverse': round(achieved, 2)},
        'gflop': {'inverse': round(flop / 1e9, 1)},
        'kernel_ms': {k: {'launches': n, 'total_ms': round(ms - n * empty, 3)} for k, (n, ms) in fam.items() if n},
        'inverse_info_nonzero': int((info != 0).sum().item()),
        'max_residual': worst,      # max over sizes of ||M M^-1 - I||_F / sqrt(d); the bound is 1e-3
        'roofline': {
            'family': 'inverse_tiles',
            'kernel': 'batched dense inverse: copy_in, diag, update, panel, border, lauum kernels', 'bound': 'mfma',
            'achieved': round(achieved, 2), 'peak': FP32_MFMA_PEAK_TFLOPS, 'unit': 'TFLOP/s',
            'frac': round(achieved / FP32_MFMA_PEAK_TFLOPS, 4),
            'timed': 'd^3 flop per matrix over the wall time of the whole batched call (its kernels overlap on two '
                     'streams, so their durations do not add up)',
            'traffic': None},
    }, dims


def run_real_network(steps=10, warmup=5, lanes=None):
    """``KFAC.update(lossfun)`` on the ResNet-50 built from the link classes (batch 32 @ 224): a
    real forward and backward pass under the function hooks, then moving average, damped inverse,
    preconditioning and the momentum rule, launched from the host with no HIP graph.  Gradient and
    activation buffers are whatever torch's autograd hands out each step."""
    import torch
    import torch.nn.functional as TF
    from chainerkfac_amd import workloads as W
    from chainerkfac_amd.optimizers import KFAC
    dev = torch.device('cuda:0')
    gen = torch.Generator(device=dev).manual_seed(3)
    model = W.build_resnet50_v1(device=dev, generator=gen)
    x = torch.randn(BATCH, 3, 224, 224, device=dev, generator=gen)
    t = torch.randint(0, 1000, (BATCH,), device=dev, generator=gen)

    def lossfun():
        return TF.cross_entropy(model(x), t)

    def wall(fn, n):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / n

    def plain():
        model.cleargrads()
        lossfun().backward()

    for _ in range(warmup):
        plain()
    plain_ms = min(wall(plain, steps) for _ in range(3))
    opt = KFAC(lr=1e-3, damping=DAMPING, stab_coeff=STAB_COEFF, cov_ema_decay=1.0)
    if lanes is not None:
        opt.lanes = lanes
    opt = opt.setup(model)
    for _ in range(warmup):
        opt.update(lossfun)
    update_ms = min(wall(lambda: opt.update(lossfun), steps) for _ in range(3))
    return {'workload': 'KFAC.update(lossfun) on the link-built ResNet-50 v1 (bias), batch 32 @224, 161 factors, '
                        'eager (no HIP graph), torch autograd for the forward / backward pass',
            'steps': steps, 'timed': 'best of 3 runs of {} updates'.format(steps), 'lanes': opt.lanes, 'ms_per_update': round(update_ms, 3),
            'forward_backward_only_ms': round(plain_ms, 3),
            'kfac_part_ms': round(update_ms - plain_ms, 3), 'in_value': False}


def compact(result):
    """The few figures of another configuration's line that go into the default line."""
    roof = result['roofline']
    out = {'workload': result['config']['workload'], 'ms_per_step': result['value'], 'steps': result['steps'],
           'roofline': {k: roof.get(k) for k in ('family', 'kernel', 'achieved', 'unit', 'frac') if k in roof}}
    if 'phase_ms' in result:
        out['phase_ms'] = result['phase_ms']
    if 'families' in roof:
        out['family_frac'] = {k: v['frac'] for k, v in roof['families'].items()}
    if result['config'].get('name') == 'c5':
        w = result['wire_format']
        out['wire_format'] = {'arrays': w['arrays'], 'triangular': w['triangular'],
                              'pack': w['pack'], 'unpack': w['unpack'], 'stream_copy': w['stream_copy'],
                              'stream_fanout': w['stream_fanout']}
    if 'max_residual' in result:
        out['max_residual'] = result['max_residual']
    return out


def write_per_layer(path, layers, config='c3'):
    """Per-layer roofline table of the covariance kernels (markdown): every distinct
    convolution / linear shape of the workload, its A and G factor timed alone on one
    stream (HIP events inside the library around the SYRK launch, empty bracket
    subtracted), against min(FP32 MFMA peak, arithmetic intensity x HBM peak)."""
    import torch
    from chainerkfac_amd import _lib, ops
    from chainerkfac_amd import workloads as W
    lib = _lib.load()
    dev = torch.device('cuda:0')
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
            issued = flop
            if fac == 'A' and W.takes_shift_route(layer):   # shifted correlations: fewer multiply-adds than M d (d+1)
                issued = float(W.cov_flops_executed([layer], BATCH)) - float(M) * dG * (dG + 1)
            ai = flop / (in_bytes + 4.0 * d * d)
            cap = min(FP32_MFMA_PEAK_TFLOPS, ai * HBM_PEAK_GBPS / 1e3)
            rows.append((desc, count, fac, d, M, flop / 1e9, issued / 1e9, t * 1e3, flop / t / 1e9, issued / t / 1e9,
                         ai, cap, issued / t / 1e9 / cap))
        del x, gy
    with open(path, 'w') as f:
        f.write('# Covariance kernels layer by layer (every distinct convolution / linear shape of the workload)\n\n'
                'Command (one MI355X, repository root):\n\n```\npython3 bench.py --config {} --no-cpu --no-dense-field '
                '--no-extras --steps 5 --per-layer {}\n```\n\n'
                'Each factor is computed alone, by the single-factor entry point, on one stream; "SYRK kernel us" is '
                'the duration of its SYRK launch (HIP events inside the library around the launch, 10 repetitions, the '
                '{:.1f} us an empty event bracket measures subtracted); the kernels that sum split-K partial tiles are '
                'not in it. In a K-FAC step the small factors (at most 8 GFLOP: most 1x1 convolutions, linear and '
                'batch-norm layers) do not run alone but in a handful of grouped launches, so their rows here show the '
                'latency floor of a single launch, not their cost in the step. GFLOP = M d (d+1), the work of the '
                'patch / activation product; "issued" is what the kernel gives the matrix cores, which is less for the A '
                'factor of a 3x3 stride-1 convolution (29 shifted correlations of C x C instead of a 9C x 9C product); '
                'flop/B = M d (d+1) over the bytes of the input tensor read once plus the factor written once; roofline '
                'cap = min(157.3 TFLOP/s FP32 MFMA, flop/B x 8 TB/s); the last column is the issued rate over the cap.'
                '\n\n'.format(config, path, empty * 1e3))
        f.write('| layer (x count) | factor | d | rows M | GFLOP | GFLOP issued | SYRK kernel us | TFLOP/s (M d (d+1)) | '
                'TFLOP/s issued | flop/B | roofline cap TFLOP/s | issued / cap |\n'
                '|---|---|---:|---:|---:|---:|---:|---:|---:|---:|---:|---:|\n')
        for desc, count, fac, d, M, gf, gi, us, tf, ti, ai, cap, frac in rows:
            f.write('| {} (x{}) | {} | {} | {} | {:.2f} | {:.2f} | {:.1f} | {:.1f} | {:.1f} | {:.0f} | {:.1f} | {:.2f} |\n'.format(
                desc, count, fac, d, M, gf, gi, us, tf, ti, ai, cap, frac))


def _cpu_threads():
    try:
        from threadpoolctl import threadpool_info
        return int(max([p.get('num_threads', 1) for p in threadpool_info()] or [1]))
    except Exception:
        return os.cpu_count()


def _cpu_layer(O, rng, layer, batch, damping):
    """One layer through the NumPy oracle (cov + damped inverse + precondition); seconds."""
    import numpy as np
    from chainerkfac_amd import workloads as W
    if layer['kind'] == 'conv':
        ho = W.conv_out(layer['h'], layer['k'], layer['s'], layer['p'])
        x = rng.standard_normal((batch, layer['c_in'], layer['h'], layer['w']), dtype=np.float32)
        gy = rng.standard_normal((batch, layer['c_out'], ho, ho), dtype=np.float32) / (batch * ho)
        gW = rng.standard_normal((layer['c_out'], layer['c_in'], layer['k'], layer['k']), dtype=np.float32)
        gb = rng.standard_normal(layer['c_out'], dtype=np.float32) if layer['bias'] else None
        t0 = time.perf_counter()
        A = O.conv_A(x, layer['k'], layer['s'], layer['p'], layer['bias'])
        G = O.conv_G(gy)
    elif layer['kind'] == 'linear':
        x = rng.standard_normal((batch, layer['d_in']), dtype=np.float32)
        gy = rng.standard_normal((batch, layer['d_out']), dtype=np.float32) / batch
        gW = rng.standard_normal((layer['d_out'], layer['d_in']), dtype=np.float32)
        gb = rng.standard_normal(layer['d_out'], dtype=np.float32) if layer['bias'] else None
        t0 = time.perf_counter()
        A = O.linear_A(x, layer['bias'])
        G = O.linear_G(gy)
    else:
        x = rng.standard_normal((batch, layer['c'], layer['h'], layer['w']), dtype=np.float32)
        gy = rng.standard_normal((batch, layer['c'], layer['h'], layer['w']), dtype=np.float32) / (batch * layer['h'])
        gg = rng.standard_normal(layer['c'], dtype=np.float32)
        gb = rng.standard_normal(layer['c'], dtype=np.float32)
        t0 = time.perf_counter()
        F = O.bn_F(x, gy, 2e-5)
    if layer['kind'] == 'bn':
        (dv,) = O.bn_diagvals(layer['c'], layer['c'], damping, STAB_COEFF)
        (Finv,) = O.update_invs([F], [dv])
        O.precondition_bn(Finv, gg, gb)
    else:
        dv, _ = O.connection_diagvals(A, G, damping)
        Ainv, Ginv = O.update_invs([A, G], dv)
        O.precondition_conn(Ainv, Ginv, gW, gb)
    return time.perf_counter() - t0


def run_cpu_baseline(name, cfg, budget_s=20.0):
    """The NumPy oracle (the restatement of the reference's --no_cuda arithmetic) on a
    bounded sample of the configuration's work, scaled to the whole step by algorithmic FLOPs."""
    import numpy as np
    from chainerkfac_amd import workloads as W
    from oracle import kfac_oracle as O
    threads = _cpu_threads()
    rng = np.random.default_rng(3)
    if name == 'c4':
        dims = inverse_dims()
        total_f = float(sum(d ** 3 for d in dims))
        done_f, t_used, used = 0.0, 0.0, []
        for d in sorted(set(dims)):
            X = rng.standard_normal((2 * d, d), dtype=np.float32)
            M = (X.T @ X / np.float32(2 * d) + np.float32(1e-3) * np.eye(d, dtype=np.float32)).astype(np.float32)
            t0 = time.perf_counter()
            O.inverse(M)
            t_used += time.perf_counter() - t0
            done_f += float(d) ** 3
            used.append(d)
            if t_used > budget_s:
                break
        return {'value': round(t_used * 1e3 * total_f / done_f, 1), 'unit': 'ms/step', 'cores': threads, 'kind': 'port',
                'sample': 'NumPy oracle inverse (cholesky, inv, matmul) of one matrix of each size {} = {:.1f} of '
                          '{:.1f} GFLOP in {:.1f} s, scaled by d^3'.format(used, done_f / 1e9, total_f / 1e9, t_used)}
    layers, batch, acc_iters = cfg['layers'], cfg['batch'], cfg['acc_iters']
    total = W.flops(layers, batch)
    total['cov'] *= acc_iters
    total_f = sum(total.values())
    if name in ('c1', 'c2'):
        sample = list(layers)                   # the whole step
    else:
        # one bottleneck of every stage plus the FC (every kernel kind and every factor size class), in an
        # order that puts the big stage-5 factors last, where the time budget cuts the sample off
        sample = []
        for prefix in ('res3/1/', 'res4/1/', 'fc', 'res2/1/', 'res5/1/', 'res4/2/', 'res5/2/', 'res3/2/'):
            sample += [l for l in layers if l['name'].startswith(prefix) or l['name'] == prefix]
    done_f, t_used, names = 0.0, 0.0, []
    for layer in sample:
        # (with accumulation the oracle repeats the covariance acc_iters times: one micro-batch is timed
        # and counted, the scaling by FLOPs accounts for the rest)
        t_used += _cpu_layer(O, rng, layer, batch, cfg['damping'])
        done_f += sum(W.flops([layer], batch).values())
        names.append(layer['name'])
        if t_used > budget_s:
            break
    whole = len(names) == len(layers) and acc_iters == 1
    return {
        'value': round(t_used * 1e3 * (1.0 if whole else total_f / done_f), 1),
        'unit': 'ms/step', 'cores': threads, 'kind': 'port',
        'sample': ('NumPy oracle (cov + damped inverse + precondition), the whole step: {:.1f} s'.format(t_used)
                   if whole else
                   'NumPy oracle (cov + damped inverse + precondition) on layers {} = {:.1f} of {:.1f} GFLOP '
                   'in {:.1f} s, scaled by FLOPs'.format(','.join(names), done_f / 1e9, total_f / 1e9, t_used)),
    }


def _short_kernel_name(name):
    for junk in ('void ', '(anonymous namespace)::', 'kfac::mma::', 'kfac::'):
        name = name.replace(junk, '')
    depth, out = 0, []
    for ch in name:          # drop the argument list, keep the template arguments
        if ch == '(' and depth == 0:
            break
        depth += ch == '<'
        depth -= ch == '>'
        out.append(ch)
    name = ''.join(out)
    return name if len(name) <= 90 else name[:87] + '...'


def _csv_rows(directory, suffix):
    import csv
    import glob
    for f in sorted(glob.glob(os.path.join(directory, '**', '*' + suffix), recursive=True)):
        with open(f) as fh:
            for r in csv.DictReader(fh):
                yield r


# (first match wins: the finish kernels of the GEMMs and of the batch-norm statistics carry their
# own family's prefix and must not fall to the covariances' 'finish_')
KERNEL_FAMILIES = (
    ('covariance SYRK family', ('syrk_', 'shift::corr_kernel')),
    ('preconditioning GEMMs (with their split-K finish and the batch-norm GEMV)', ('gemm_', 'gemv_', 'bn_select')),
    ('batch-norm statistics and finish', ('bn_',)),
    ('batch-norm rank-n inverses', ('lr_',)),
    ('split-K finish, edge sums and assembly of the covariances', ('finish_', 'reduce_kernel', 'shift::assemble',
                                                                  'shift::edge_sums')),
    ('inverse tile kernels', ('diag_kernel', 'update_kernel', 'lauum_kernel', 'panel_kernel', 'copy_in', 'copy_out',
                              'border_kernel', 'trtri', 'potrf', 'small_inverse')),
    ('damping', ('pi_damp', 'add_diag')),
    ('pack / unpack / copy', ('pack_kernel', 'unpack_kernel', 'stream_copy', 'stream_fanout')),
)


def _family_of(name):
    for fam, keys in KERNEL_FAMILIES:
        if any(k in name for k in keys):
            return fam
    return None


def _own_kernel(name):
    return not name.startswith('at::') and 'at::native' not in name and 'hiprand' not in name


def summarize_kernel_trace(trace_dir, out_path, command):
    """Markdown summary (per kernel and per kernel family) of the kernel trace a
    `rocprofv3 --kernel-trace --stats` run of this script wrote under ``trace_dir``."""
    agg = {}
    for r in _csv_rows(trace_dir, 'kernel_trace.csv'):
        name = _short_kernel_name(r['Kernel_Name'])
        dur = int(r['End_Timestamp']) - int(r['Start_Timestamp'])
        a = agg.setdefault(name, [0, 0, 1 << 62, 0])
        a[0] += 1
        a[1] += dur
        a[2] = min(a[2], dur)
        a[3] = max(a[3], dur)
    if not agg:
        raise SystemExit('no kernel_trace.csv under ' + trace_dir)
    total = float(sum(a[1] for a in agg.values()))
    # elapsed time of every batched inverse: first copy_in after the previous call's lauum .. end of lauum
    # (only calls with the whole sweep in between: the three-matrix inverses of other runs are left out)
    spans, begin, inside = [], None, 0
    ordered = sorted((int(r['Start_Timestamp']), int(r['End_Timestamp']), r['Kernel_Name'])
                     for r in _csv_rows(trace_dir, 'kernel_trace.csv'))
    for t0, t1, name in ordered:
        if 'copy_in_kernel' in name and begin is None:
            begin, inside = t0, 0
        elif begin is not None and ('diag_kernel' in name or 'update_kernel' in name):
            inside += 1
        elif 'lauum_kernel' in name and begin is not None:
            spans.append((t1 - begin, inside))
            begin = None
    most = max((n for _, n in spans), default=0)
    spans = sorted(d for d, n in spans if n == most)
    lines = ['# Kernel time by kernel: ' + os.path.basename(out_path)[:-3].replace('_', ' '), '',
             'Command (one MI355X, repository root; raw output stays outside the repository):', '', '```',
             command, '```', '',
             'All launches of the run are counted (warm-up, timed steps, the phase split and the pass that times '
             'every launch with HIP events), so "launches" is a multiple of the per-step count. Durations are '
             'summed per kernel: the kernels of the batched inverse run side by side on three streams (diagonal '
             'tiles and panels, column updates, trailing updates), so their sum is about 1.7 times the time the '
             'inverse takes (what `roofline.families.inverse_tiles` of the bench line divides by is the time '
             'between the first and the last launch of the call), and "share" is a share of summed kernel time, '
             'not of elapsed time.', '',
             '| family | launches | total ms | avg us / launch | share of summed kernel time |', '|---|---:|---:|---:|---:|']
    fam = {}
    for name, a in agg.items():
        f = _family_of(name)
        if f:
            t = fam.setdefault(f, [0, 0])
            t[0] += a[0]
            t[1] += a[1]
    for f, _ in KERNEL_FAMILIES:
        if f in fam:
            n, t = fam[f]
            lines.append('| {} | {} | {:.3f} | {:.1f} | {:.1f} % |'.format(f, n, t / 1e6, t / n / 1e3, 100 * t / total))
    if spans:
        lines += ['', 'Elapsed time of a batched inverse (start of its first `copy_in_kernel` to the end of its '
                  '`lauum_kernel`, {} calls with the full sweep): median {:.3f} ms, min {:.3f}, max {:.3f}.'.format(
                      len(spans), spans[len(spans) // 2] / 1e6, spans[0] / 1e6, spans[-1] / 1e6)]
    lines += ['', '| kernel | launches | total ms | avg us | min us | max us | share |', '|---|---:|---:|---:|---:|---:|---:|']
    for name, a in sorted(agg.items(), key=lambda kv: -kv[1][1])[:40]:
        if a[1] / total < 0.001:
            break
        lines.append('| `{}` | {} | {:.3f} | {:.1f} | {:.1f} | {:.1f} | {:.1f} % |'.format(
            name, a[0], a[1] / 1e6, a[1] / a[0] / 1e3, a[2] / 1e3, a[3] / 1e3, 100 * a[1] / total))
    with open(out_path, 'w') as f:
        f.write('\n'.join(lines) + '\n')
    print('\n'.join(lines[:24]))


def summarize_mfma(pmc_dir, out_path, command):
    """Matrix-pipe utilisation per kernel from a `rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES
    GRBM_GUI_ACTIVE` run of this script.  SQ_VALU_MFMA_BUSY_CYCLES adds up, over the
    chip's 1024 SIMDs, the cycles in which the SIMD's matrix pipe was busy;
    GRBM_GUI_ACTIVE adds up the 8 XCDs' active cycles: busy fraction =
    MFMA_BUSY / (GUI_ACTIVE / 8 * 1024)."""
    disp = {}
    for r in _csv_rows(pmc_dir, 'counter_collection.csv'):
        d = disp.setdefault(r['Dispatch_Id'], {'name': _short_kernel_name(r['Kernel_Name'])})
        d[r['Counter_Name']] = d.get(r['Counter_Name'], 0.0) + float(r['Counter_Value'])
    agg = {}
    for d in disp.values():
        if 'SQ_VALU_MFMA_BUSY_CYCLES' not in d or 'GRBM_GUI_ACTIVE' not in d or not _own_kernel(d['name']):
            continue
        a = agg.setdefault(d['name'], [0, 0.0, 0.0])
        a[0] += 1
        a[1] += d['SQ_VALU_MFMA_BUSY_CYCLES']
        a[2] += d['GRBM_GUI_ACTIVE']
    if not agg:
        raise SystemExit('no SQ_VALU_MFMA_BUSY_CYCLES / GRBM_GUI_ACTIVE rows under ' + pmc_dir)
    lines = ['# FP32 matrix-pipe utilisation by kernel: ' + os.path.basename(out_path)[:-3].replace('_', ' '), '',
             'Command (one MI355X, repository root; every kernel launched from the host on one stream so that each '
             'dispatch has its own counter record):', '', '```', command, '```', '',
             '`SQ_VALU_MFMA_BUSY_CYCLES` sums, over the 1024 SIMDs, the cycles in which a SIMD\'s matrix pipe was '
             'busy; `GRBM_GUI_ACTIVE` sums the active cycles of the 8 XCDs.  busy = MFMA_BUSY / (GUI_ACTIVE / 8 x '
             '1024): the share of all matrix-pipe cycles of the launch (ramp-up, tail and padding work included) '
             'in which an MFMA was executing.  Only `v_mfma_f32_32x32x2_f32` is used, so busy x 157.3 TFLOP/s is '
             'the rate of executed (padded) matrix work.', '',
             '| family | launches | matrix pipe busy |', '|---|---:|---:|']
    fam = {}
    for name, a in agg.items():
        f = _family_of(name)
        if f:
            t = fam.setdefault(f, [0, 0.0, 0.0])
            for i in range(3):
                t[i] += a[i]
    for f, _ in KERNEL_FAMILIES:
        if f in fam and fam[f][1] > 0:
            n, busy, act = fam[f]
            lines.append('| {} | {} | {:.1f} % |'.format(f, n, 100 * busy / (act / 8 * 1024)))
    lines += ['', '| kernel | launches | active Mcycles / launch | matrix pipe busy |', '|---|---:|---:|---:|']
    for name, a in sorted(agg.items(), key=lambda kv: -kv[1][2]):
        if a[1] == 0:
            continue
        lines.append('| `{}` | {} | {:.3f} | {:.1f} % |'.format(name, a[0], a[2] / 8 / a[0] / 1e6,
                                                              100 * a[1] / (a[2] / 8 * 1024)))
    with open(out_path, 'w') as f:
        f.write('\n'.join(lines) + '\n')
    print('\n'.join(lines[12:40]))


TRAFFIC_FAMILIES = (
    # family, kernels of the family, the kernel whose launches count the steps of the run
    ('cov_syrk', ('syrk_', 'shift::corr_kernel', 'finish_group_kernel', 'finish_kernel', 'reduce_kernel',
                  'shift::assemble', 'shift::edge_sums', 'shift::corr_finish'), 'finish_group_kernel'),
    ('inverse_tiles', ('copy_in_kernel', 'diag_kernel', 'update_kernel', 'panel_kernel', 'border_kernel',
                       'lauum_kernel'), 'lauum_kernel'),
    ('precond_gemm', ('gemm_group', 'gemv_', 'bn_select'), 'gemm_group_finish_kernel<1>'),
)


def summarize_traffic(fetch_dir, write_dir, out_path, command):
    """Reads the per-dispatch FETCH_SIZE / WRITE_SIZE counters (KiB) of two
    `rocprofv3 --pmc` runs of this script with --calibrate-copy, scales each by what it
    reads for the 256 MiB calibration copy (stream_copy_kernel), and writes the HBM bytes
    of every kernel family per step, and per launch of the covariance SYRK main kernels,
    to ``out_path`` (JSON, read back as roofline.traffic) and a per-kernel table next to
    it (markdown)."""
    def load(d, counter):
        rows = {}
        for r in _csv_rows(d, 'counter_collection.csv'):
            if r.get('Counter_Name') == counter:
                key = (r['Dispatch_Id'], _short_kernel_name(r['Kernel_Name']))
                rows[key] = rows.get(key, 0.0) + float(r['Counter_Value'])
        return [(k[1], v) for k, v in sorted(rows.items(), key=lambda kv: int(kv[0][0]))]

    out = {'families': {}}
    total = 0.0
    per_kernel = {}
    for d, counter, key in ((fetch_dir, 'FETCH_SIZE', 'fetch'), (write_dir, 'WRITE_SIZE', 'write')):
        rows = load(d, counter)
        syrk = [v for k, v in rows if 'syrk_' in k or 'shift::corr_kernel' in k]
        cal = [v for k, v in rows if 'stream_copy_kernel' in k]
        if not syrk or not cal:
            raise SystemExit('no {} rows for the SYRK family or the calibration copy under {}'.format(counter, d))
        # the calibration copy is the run's first launch of the copy kernel
        scale = (256.0 * 1024.0) / cal[0]       # counter KiB -> true KiB
        out[key + '_counter_for_256MiB_copy'] = cal[0]
        out[key + '_scale'] = round(scale, 4)
        out[key + '_bytes_per_launch'] = sum(syrk) / len(syrk) * 1024.0 * scale
        out['launches'] = len(syrk)
        total += out[key + '_bytes_per_launch']
        for fam, keys, marker in TRAFFIC_FAMILIES:
            steps = sum(1 for k, _ in rows if marker in k)
            # (the finish kernels of the GEMMs and of the batch-norm statistics are not the covariances')
            kib = sum(v for k, v in rows if any(x in k for x in keys)
                      and (fam != 'cov_syrk' or not any(x in k for x in ('gemm_', 'bn_'))))
            f = out['families'].setdefault(fam, {'steps_in_run': steps})
            f[key + '_bytes_per_step'] = kib * 1024.0 * scale / max(steps, 1)
        for k, v in rows:
            if _own_kernel(k):
                a = per_kernel.setdefault(k, {'fetch': [0, 0.0], 'write': [0, 0.0]})[key]
                a[0] += 1
                a[1] += v * scale
    out['bytes_per_launch'] = total
    for f in out['families'].values():
        f['bytes_per_step'] = f.get('fetch_bytes_per_step', 0.0) + f.get('write_bytes_per_step', 0.0)
    with open(out_path, 'w') as f:
        json.dump(out, f, indent=1)
        f.write('\n')
    lines = ['# HBM traffic per launch (hardware counters)', '',
             'Two counter runs on one MI355X from the repository root (raw output stays outside the repository); '
             'every kernel is launched from the host on one stream so that each dispatch has its own counter record, '
             'and `--calibrate-copy` first runs `stream_copy_kernel` over 256 MiB (reads 256 MiB, writes 256 MiB):',
             '', '```', command, '```', '',
             'Calibration: for the 262144 KiB copy FETCH_SIZE reads {:.1f} and WRITE_SIZE reads {:.1f}, so the '
             'counters are scaled by {:.3f} and {:.3f} to get KiB.'.format(
                 out['fetch_counter_for_256MiB_copy'], out['write_counter_for_256MiB_copy'],
                 out['fetch_scale'], out['write_scale']), '',
             'Covariance SYRK main kernels (`syrk_*` and `shift::corr_kernel`, {} launches in the run): **fetch {:.1f} MiB + write {:.1f} MiB = '
             '{:.1f} MiB per launch** ({:.4g} bytes).'.format(
                 out['launches'], out['fetch_bytes_per_launch'] / 2 ** 20, out['write_bytes_per_launch'] / 2 ** 20,
                 total / 2 ** 20, total), '',
             'Kernel families, all their kernels, per step (the `roofline.traffic` figures of bench.py):', '',
             '| family | steps in the run | fetch MiB / step | write MiB / step | total MiB / step |', '|---|---:|---:|---:|---:|']
    for fam, _, _ in TRAFFIC_FAMILIES:
        f = out['families'][fam]
        lines.append('| {} | {} | {:.1f} | {:.1f} | {:.1f} |'.format(
            fam, f['steps_in_run'], f.get('fetch_bytes_per_step', 0) / 2 ** 20, f.get('write_bytes_per_step', 0) / 2 ** 20,
            f['bytes_per_step'] / 2 ** 20))
    lines += ['', '| kernel | launches | fetch MiB/launch | write MiB/launch |', '|---|---:|---:|---:|']

    def tot(v):
        return v['fetch'][1] + v['write'][1]
    for k, v in sorted(per_kernel.items(), key=lambda kv: -tot(kv[1]))[:24]:
        n = max(v['fetch'][0], v['write'][0], 1)
        lines.append('| `{}` | {} | {:.2f} | {:.2f} |'.format(k, n, v['fetch'][1] / n / 1024, v['write'][1] / n / 1024))
    md = out_path[:-5] + '.md'
    with open(md, 'w') as f:
        f.write('\n'.join(lines) + '\n')
    print(json.dumps(out))


def main():
    import faulthandler
    faulthandler.enable()   # a crash inside a native call still names the Python line it came from
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=3)
    ap.add_argument('--config', default='c3', choices=['c1', 'c2', 'c3', 'c4', 'c5'],
                    help='benchmark configuration (default: c3, the headline ResNet-50 batch-32 step)')
    ap.add_argument('--no-graph', action='store_true', help='launch every kernel from the host each step')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    ap.add_argument('--dense-bn-inverse', action='store_true',
                    help='invert the batch-norm blocks with the dense Cholesky path as well (default: their '
                         'rank-32 Woodbury form, which yields the same dense inverse)')
    ap.add_argument('--no-dense-field', action='store_true',
                    help='skip the second measurement of c3 with all batch-norm blocks inverted densely')
    ap.add_argument('--no-extras', action='store_true',
                    help='skip the measurements beside the step (momentum rule of all parameters, moving average '
                         'of all factors): profiling runs')
    ap.add_argument('--host-launch-child', action='store_true', help=argparse.SUPPRESS)
    ap.add_argument('--in-process', action='store_true',
                    help='measure the eager step and the per-family brackets in this process instead of '
                         'a fresh one (chosen by itself under rocprofv3: a profiled process must not start others)')
    ap.add_argument('--real-network', action='store_true', help=argparse.SUPPRESS)
    ap.add_argument('--no-other-configs', action='store_true',
                    help='c3 only: skip the short runs of c1, c2, c4 and c5 and the real-network step that the '
                         'default line carries beside its own figures')
    ap.add_argument('--lanes', type=int, default=4,
                    help='side streams for the per-layer factor and preconditioning kernels (0 = one stream, also for '
                         'the grouped launches)')
    ap.add_argument('--macro-tiles', action='store_true',
                    help='grouped covariance launches use the macro-tile kernel for slabs of several 128-tiles '
                         '(library option group_macro = 1: less HBM traffic, about 1 %% slower)')
    ap.add_argument('--per-layer', metavar='PATH', default=None,
                    help='also time the covariance kernels of every distinct layer shape alone and write a '
                         'markdown roofline table to PATH')
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='first run one 256 MiB device-to-device elementwise copy (a kernel of known traffic, '
                         'the reference point for hardware byte counters collected under rocprofv3 --pmc)')
    ap.add_argument('--summarize-traffic', nargs=2, metavar=('FETCH_DIR', 'WRITE_DIR'), default=None,
                    help='no benchmark: turn the counter files of two rocprofv3 --pmc runs of this script into '
                         'profiles/syrk_hbm_traffic.json (read back as roofline.traffic) and a table beside it')
    ap.add_argument('--summarize-trace', nargs=2, metavar=('TRACE_DIR', 'OUT_MD'), default=None,
                    help='no benchmark: per-kernel / per-family table of a rocprofv3 --kernel-trace run')
    ap.add_argument('--summarize-mfma', nargs=2, metavar=('PMC_DIR', 'OUT_MD'), default=None,
                    help='no benchmark: matrix-pipe utilisation per kernel from a rocprofv3 --pmc '
                         'SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE run')
    ap.add_argument('--profiled-command', default='(not recorded)',
                    help='the profiling command line, copied into the summary that --summarize-* writes')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py measures the single-GPU K-FAC hot path: inter-GPU collectives are outside this '
                 'build, so --gpus must be 1 (got {})'.format(args.gpus))
    if args.summarize_traffic:
        summarize_traffic(args.summarize_traffic[0], args.summarize_traffic[1], TRAFFIC_FILE, args.profiled_command)
        return
    if args.summarize_trace:
        summarize_kernel_trace(args.summarize_trace[0], args.summarize_trace[1], args.profiled_command)
        return
    if args.summarize_mfma:
        summarize_mfma(args.summarize_mfma[0], args.summarize_mfma[1], args.profiled_command)
        return
    # Launches made from the host (eager step time, per-family event brackets, the step on a real
    # network) are measured in processes of their own, with the drop-in's default number of lanes,
    # when this one replays graphs: a process that has captured the step with four lanes holds more
    # streams than the GPU gives one process hardware queues, and independent launches from the host
    # then wait behind each other (the batched inverse took a fifth longer that way).  They run
    # first, before this process has touched the GPU.
    with_others = args.config == 'c3' and not args.no_other_configs
    host = {}
    # (a process started under rocprofv3 must not start others: the profiler's library has touched
    # the GPU before main() runs; such a run measures everything in this process, like --in-process)
    profiled = any(k.startswith(('ROCPROF', 'ROCP_')) for k in os.environ) or \
        'rocprof' in os.environ.get('LD_PRELOAD', '')
    if profiled and not args.no_graph and args.lanes > 0:
        # the kernel tracer crashes in the replay of a graph with forked streams
        print('bench.py: running under rocprofv3: graphs are captured on one stream (--lanes 0)', file=sys.stderr)
        args.lanes = 0
    if not args.no_graph and not args.host_launch_child and not args.in_process and not profiled:
        # (a child that cannot run leaves its measurements to this process: figures taken in a
        # process that also replays graphs are somewhat pessimistic, but the line is still printed)
        for name in [args.config] + (['c1', 'c2', 'c5'] if with_others else []):
            if name == 'c4':
                continue
            try:
                host[name] = host_launch_child(args, name)
            except Exception as e:   # noqa: BLE001
                print('bench.py: {}: measured in this process instead ({})'.format(name, str(e)[-300:]), file=sys.stderr)
        if with_others and args.config in host:
            try:
                host[args.config]['real_network'] = host_launch_child(args, args.config, real_network=True)
            except Exception as e:   # noqa: BLE001
                print('bench.py: real network: measured in this process instead ({})'.format(str(e)[-300:]), file=sys.stderr)
    if args.macro_tiles:
        from chainerkfac_amd import _lib
        _lib.set_option('group_macro', 1)
    if args.lanes == 0:
        # one stream everywhere: the grouped launches keep to the caller's stream as well (profiling
        # runs, where kernels that run side by side would share their durations)
        from chainerkfac_amd import _lib
        _lib.set_option('group_side_stream', 0)
    cfg = configs()[args.config]
    if args.host_launch_child:
        print(json.dumps(run_real_network(lanes=args.lanes) if args.real_network else run_step_config(args, args.config, cfg)))
        return
    if args.config == 'c4':
        result, _ = run_inverse_config(args, args.config, cfg)
    else:
        result = run_step_config(args, args.config, cfg, host.get(args.config))
        if args.per_layer:
            write_per_layer(args.per_layer, cfg['layers'], args.config)
    if with_others:
        # the other configurations of the benchmark definition, shorter runs of the same code paths
        # (their full lines: --config c1 | c2 | c4 | c5), and the drop-in step on a real network
        import copy
        import gc
        import torch
        others = {}
        for name, steps in (('c1', 50), ('c2', 50), ('c4', 20), ('c5', 5)):
            gc.collect()
            torch.cuda.empty_cache()
            sub = copy.copy(args)
            sub.config, sub.steps, sub.warmup = name, steps, 1
            sub.no_extras = sub.no_dense_field = True
            sub.per_layer = None
            sub_cfg = configs()[name]
            if name == 'c4':
                line, _ = run_inverse_config(sub, name, sub_cfg)
            else:
                line = run_step_config(sub, name, sub_cfg, host.get(name))
            others[name] = compact(line)
        result['other_configs'] = others
        if 'real_network' not in result:
            gc.collect()
            torch.cuda.empty_cache()
            result['real_network'] = run_real_network()
    if not args.no_cpu:
        result['cpu_baseline'] = run_cpu_baseline(args.config, cfg)
    print(json.dumps(result))


if __name__ == '__main__':
    main()
