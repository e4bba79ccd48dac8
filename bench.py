'''Benchmark of the vkJAX hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload resnet50] [--batch 64]

A step is one forward pass of the workload through the interpreter's recorded launch sequence
with all inputs (images and weights) already resident in HBM. The default workload is the one
the headline metric is quoted on: ResNet-50, batch 64, 224x224x3, fp32. Prints ONE JSON line.

`roofline` describes the dominant kernel family of the workload (the fp32-MFMA implicit-GEMM
convolution for ResNet-50): algorithmic FLOPs (or bytes) of its launches divided by their
summed durations, measured with HIP events on the launch stream. `kernels` gives the same
figures for every kernel family in the sequence. `cpu_baseline` times the CPU oracle on a
bounded sample of the same workload on this machine's host cores.
'''
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS          = 8000.0

UNITS = {'resnet50': ('images/sec', 'batch'), 'mlp': ('samples/sec', 'batch'), 'conv_block': ('images/sec', 'batch'),
         'affine': ('calls/sec', None), 'rng_uniform': ('Gsamples/sec', None), 'gather_scatter': ('Grows/sec', None),
         'mlp_train': ('samples/sec', 'batch'), 'convnet_train': ('images/sec', 'batch'), 'resnet50_train': ('images/sec', 'batch')}
BATCHED = ('resnet50', 'mlp', 'conv_block', 'mlp_train', 'convnet_train', 'resnet50_train')


def kernel_family(name: str) -> str:
    for prefix in ('conv_gemm', 'wgrad_gemm', 'softmax_rows', 'ew_chain', 'threefry2x32', 'gather_rows', 'pool', 'reduce_rows', 'reduce_cols', 'scatter_rows',
                   'select_window', 'scatter_selected', 'pad_nd', 'scale_relu_backward', 'scale_backward', 'transpose_tiled'):
        if name.startswith(prefix):
            return prefix
    return name


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--workload', default='resnet50', choices=list(UNITS))
    ap.add_argument('--batch', type=int, default=None)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-fuse', action='store_true')
    ap.add_argument('--end-to-end', action='store_true',
                    help='also time whole calls through wrap() (uploads, launches, downloads, Python), median of 5')
    ap.add_argument('--graph', action='store_true', help='replay the launches as one captured HIP graph')
    ap.add_argument('--profile-iters', type=int, default=3)
    ap.add_argument('--dump-launches', default=None, help='write one line per launch (kernel, grid, FLOP, bytes, ms) to this file')
    ap.add_argument('--calibration-copy', action='store_true',
                    help='also launch one plain 256 MiB -> 256 MiB copy (kernel ew_chain_v4_s2, the only dispatch with a 16777216-block '
                         'grid), so that a hardware-counter run of this command holds a dispatch of known HBM traffic')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py measures one GPU: the hot path runs on a single MI355X and nothing here shards '
              'across devices; run with --gpus 1', file=sys.stderr)
        sys.exit(2)

    import vkjax_amd
    from vkjax_amd import hip, minijax as mj, workloads as W
    from vkjax_amd.minijax import tree_util

    fn, make_inputs = W.WORKLOADS[args.workload]
    kwargs = {}
    if args.batch is not None and UNITS[args.workload][1]:
        kwargs['batch'] = args.batch
    inputs = make_inputs(**kwargs)
    dev    = hip.Device.get()
    props  = dev.get_device_properties()

    t0 = time.perf_counter()
    wrapped = vkjax_amd.wrap(fn, frontend='minijax', fuse=not args.no_fuse, graph=args.graph)
    interp, _ = wrapped._get_or_create_jaxpr_interpreter(tuple(inputs))
    build_s = time.perf_counter() - t0
    interp.upload_inputs(*inputs)

    if args.calibration_copy:
        n = 64 * 1024 * 1024
        copy = vkjax_amd.wrap(lambda x: x + 0.0, frontend='minijax')
        ci, _ = copy._get_or_create_jaxpr_interpreter((np.zeros(n, np.float32),))
        ci.replay(1)
        dev.sync()

    for _ in range(args.warmup):
        interp.replay(1)
    dev.sync()
    t0 = time.perf_counter()
    device_ms = 0.0
    for _ in range(args.steps):
        device_ms += interp.replay(1)
    dev.sync()
    wall_s = time.perf_counter() - t0
    ms_per_step = wall_s * 1e3 / args.steps

    leaves = tree_util.tree_leaves(inputs)
    if args.workload in BATCHED:
        units_per_step = leaves[-1].shape[0]
    elif args.workload == 'rng_uniform':
        units_per_step = 4096 * 4096 / 1e9
    elif args.workload == 'gather_scatter':
        units_per_step = 2 * inputs[1].size / 1e9
    else:
        units_per_step = 1
    value = units_per_step / (ms_per_step / 1e3)

    #per-launch durations: a second sequence of the same program with an event after every launch
    from vkjax_amd.jaxpr_interpreter import JaxprInterpreter
    prof = JaxprInterpreter(interp.jaxpr, interp.static_argnums, profiling=True, fuse=interp.fuse)
    prof.upload_inputs(*inputs)
    fam = {}
    per_launch = np.zeros(len(prof.launches))
    for it in range(args.profile_iters + 1):
        prof.sequence.eval([None] * prof.sequence.n_slots, flags=hip.EVAL_SKIP_UPLOADS | hip.EVAL_SKIP_DOWNLOADS)
        if it == 0:
            continue                                            #warm-up
        stamps = prof.sequence.get_timestamps()
        durs   = np.diff(stamps)[1:1 + len(prof.launches)]      #[uploads | launches ... | downloads]
        per_launch += durs
        for launch, ms in zip(prof.launches, durs):
            f = fam.setdefault(kernel_family(launch.kernel), dict(launches=0, ms=0.0, flops=0, bytes=0))
            f['launches'] += 1; f['ms'] += float(ms); f['flops'] += launch.flops; f['bytes'] += launch.bytes_moved
    if args.dump_launches:
        with open(args.dump_launches, 'w') as fh:
            for op, launch, ms in zip(prof.all_ops, prof.launches, per_launch / max(args.profile_iters, 1)):
                rate = f'{launch.flops / ms / 1e9:7.1f} TFLOP/s' if launch.flops else f'{launch.bytes_moved / ms / 1e6:7.0f} GB/s'
                fh.write(f'{launch.kernel:28s} grid {launch.grid[0]:6d} {launch.flops / 1e9:8.3f} GFLOP {launch.bytes_moved / 1e6:8.1f} MB '
                         f'{ms * 1e3:8.1f} us {rate}  {op.equation!r:.60s}\n')
    kernels = {}
    for name, f in fam.items():
        n = args.profile_iters
        entry = dict(launches=f['launches'] // n, ms=round(f['ms'] / n, 4))
        if f['flops']:
            entry['tflops'] = round(f['flops'] / f['ms'] / 1e9, 3)
            entry['frac_mfma_peak'] = round(entry['tflops'] / PEAK_FP32_MFMA_TFLOPS, 4)
        entry['gbs'] = round(f['bytes'] / f['ms'] / 1e6, 1)
        entry['frac_hbm_peak'] = round(entry['gbs'] / PEAK_HBM_GBS, 4)
        kernels[name] = entry
    dominant = max(fam, key=lambda k: fam[k]['ms'])
    d = fam[dominant]
    if d['flops']:
        achieved = d['flops'] / d['ms'] / 1e9
        roofline = dict(bound='mfma', kernel=dominant, achieved=round(achieved, 3), peak=PEAK_FP32_MFMA_TFLOPS, unit='TFLOP/s',
                        frac=round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), traffic=None,
                        launches_per_step=d['launches'] // args.profile_iters,
                        avg_launch_ms=round(d['ms'] / d['launches'], 5))
    else:
        achieved = d['bytes'] / d['ms'] / 1e6
        roofline = dict(bound='hbm', kernel=dominant, achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit='GB/s',
                        frac=round(achieved / PEAK_HBM_GBS, 4), traffic=None,
                        launches_per_step=d['launches'] // args.profile_iters,
                        avg_launch_ms=round(d['ms'] / d['launches'], 5))

    roofline['traffic'] = measured_hbm_traffic(args.workload, dominant)

    #end-to-end calls through wrap(): host arrays in, host arrays out, uploads and Python included;
    #once copying every argument per call (what the reference does), once with the weights resident
    end_to_end = {}
    if args.end_to_end:
        import statistics
        for label, kw in (('all_arguments_copied_ms', {}), ('weights_resident_ms', dict(resident_argnums=(0,)))):
            if label == 'weights_resident_ms' and not isinstance(inputs[0], dict):
                continue
            f = vkjax_amd.wrap(fn, frontend='minijax', fuse=not args.no_fuse, **kw)
            f(*inputs)
            times = []
            for _ in range(5):
                t0 = time.perf_counter()
                f(*inputs)
                times.append((time.perf_counter() - t0) * 1e3)
            end_to_end[label] = round(statistics.median(times), 3)
            if label == 'weights_resident_ms':
                #the same calls through Function.stream: each upload overlaps the step before it
                n = 40
                results = f.stream([tuple(inputs)] * (n + 1))
                next(results)
                t0 = time.perf_counter()
                for _ in results:
                    pass
                end_to_end['weights_resident_streamed_ms'] = round((time.perf_counter() - t0) * 1e3 / n, 3)

    cpu_baseline = None
    if not args.no_cpu_baseline:
        cpu_baseline = time_cpu_baseline(args.workload, fn, make_inputs, kwargs)

    out = {
        'metric': 'ResNet-50 bs64 fp32 images/sec' if args.workload == 'resnet50' else f'{args.workload} throughput',
        'value': round(value, 3), 'unit': UNITS[args.workload][0], 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': round(ms_per_step, 4), 'device_ms_per_step': round(device_ms / args.steps, 4),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': args.workload, 'input_shape': list(leaves[-1].shape) if hasattr(leaves[-1], 'shape') else None,
                   'launches_per_step': len(interp.launches), 'fused': interp.fuse, 'inputs_resident_in_hbm': True,
                   'device': props['device_name'], 'arch': props['arch'], 'compute_units': props['compute_units'],
                   'hbm_bytes_allocated': interp.bufferpool.total_device_bytes(), 'build_seconds': round(build_s, 2),
                   **({'end_to_end_call': end_to_end} if end_to_end else {})},
        'roofline': roofline, 'kernels': kernels, 'cpu_baseline': cpu_baseline,
    }
    print(json.dumps(out))


def measured_hbm_traffic(workload, family):
    '''HBM bytes per launch of the dominant kernel family from the hardware-counter passes
    (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, each scaled by what the counter reads for a plain
    copy of known size), as recorded in the committed summary of that profile; None if there is none.
    Counters cannot be collected from inside this process.'''
    import glob, re
    here = os.path.dirname(os.path.abspath(__file__))
    #summaries are named <kernels>_<workload>.txt (the headline one: <kernels>_resnet50_bs64.txt)
    paths = glob.glob(os.path.join(here, 'profiles', f'*_{workload}.txt')) + glob.glob(os.path.join(here, 'profiles', f'*_{workload}_bs64.txt'))
    for path in sorted(paths):
        m = re.search(rf'^hbm_traffic_bytes_per_launch {re.escape(family)} (\d+)', open(path).read(), re.M)
        if m:
            return int(m.group(1))
    return None


def time_cpu_baseline(workload, fn, make_inputs, kwargs):
    '''The CPU oracle (numpy restatement of the same program) on a bounded sample, on this host.'''
    from vkjax_amd import minijax as mj
    from vkjax_amd.minijax import tree_util
    from oracle.eval_jaxpr import eval_closed_jaxpr
    sample_kwargs = dict(kwargs)
    sample = 'same shapes as the GPU run'
    if workload == 'resnet50':
        sample_kwargs['batch'] = 4
        sample = 'batch 4 of the same 224x224x3 ResNet-50 forward'
    if workload == 'resnet50_train':
        sample_kwargs['batch'] = 1
        sample = 'batch 1 of the same training step'
    if workload == 'convnet_train':
        sample_kwargs['batch'] = 1
        sample = 'batch 1 of the same training step (the pooling gradient of the oracle is a python loop)'
    inputs = make_inputs(**sample_kwargs)
    closed = mj.make_jaxpr(fn)(*inputs)
    leaves = tree_util.tree_leaves(inputs)
    reps, t_total = 0, 0.0
    while reps < 1 or (t_total < 10.0 and reps < 20):
        t0 = time.perf_counter()
        eval_closed_jaxpr(closed, *leaves)
        t_total += time.perf_counter() - t0
        reps += 1
    per_call = t_total / reps
    if workload in BATCHED:
        units = leaves[-1].shape[0]
    elif workload == 'rng_uniform':
        units = 4096 * 4096 / 1e9
    elif workload == 'gather_scatter':
        units = 2 * inputs[1].size / 1e9
    else:
        units = 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count()
    jax_note = 'jax not importable on this machine'
    try:
        import jax    # noqa: F401
        jax_note = 'jax importable (not used for this figure)'
    except ImportError:
        pass
    return dict(value=round(units / per_call, 4), unit=UNITS[workload][0], cores=cores, kind='port',
                sample=f'{sample}; {reps} evaluation(s) of the numpy oracle (float64 accumulation, BLAS threads = host cores), '
                       f'{per_call:.2f} s each; {jax_note}')


if __name__ == '__main__':
    main()
