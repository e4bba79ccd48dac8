'''Benchmark of the vkJAX hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload resnet50] [--batch 64]

A step is one forward pass of the workload through the interpreter's recorded launch sequence
with all inputs (images and weights) already resident in HBM ("device-only, inputs resident").
The default workload is the one the headline metric is quoted on: ResNet-50, batch 64,
224x224x3, fp32. Prints ONE JSON line.

`roofline` describes the dominant kernel family of the workload (the fp32-MFMA implicit-GEMM
convolution for ResNet-50): algorithmic FLOPs (or bytes) of its launches divided by the time they
take in a timed step. That time is measured in two parts: the whole step between two HIP events
on the launch stream, launches back to back (`device_ms_per_step`), and the share of each launch
in a step from a second sequence of the same program with an event after every launch. An event
after every launch costs a few microseconds per launch, so the per-launch figures add up to more
than a step; they are scaled to `device_ms_per_step` (`stamped_ms` keeps the unscaled sum).
`kernels` gives the same figures for every kernel family in the sequence.

`config.end_to_end_call` times whole calls through wrap(): host arrays in, host arrays out,
uploads, Python and downloads included. `configs` repeats the measurement for the other
workloads of the metric (affine layer, MLP, conv block, RNG draw, gather + scatter-add).
`cpu_baseline` times the same program on this machine's host cores: jax's CPU backend where jax
is importable, otherwise an fp32 torch-CPU graph of the same layers as a substitute; its result
is also what the GPU result of the timed interpreter is compared with (`output_check`).
'''
import argparse
import json
import os
import statistics
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
#the other workloads the metric names ("per-primitive HBM GB/s / MFMA util"), measured after the headline one
OTHER_CONFIGS = ('affine', 'mlp', 'conv_block', 'rng_uniform', 'gather_scatter')


#kernel families whose launches compute their results from their operands alone, so that replaying one changes nothing
REPEATABLE = ('conv_gemm', 'dense_rows', 'softmax_rows', 'ew_chain', 'ew_affine', 'threefry2x32', 'gather_rows', 'pool', 'reduce_rows',
              'reduce_cols', 'transpose_tiled', 'pad_nd')


def kernel_family(name: str) -> str:
    for prefix in ('conv_gemm', 'wgrad_gemm', 'dense_rows', 'softmax_rows', 'ew_chain', 'ew_affine', 'threefry2x32', 'gather_rows', 'pool', 'reduce_rows', 'reduce_cols', 'scatter_rows',
                   'select_window', 'scatter_selected', 'pad_nd', 'scale_relu_backward', 'scale_backward', 'transpose_tiled'):
        if name.startswith(prefix):
            return prefix
    return name


def units_per_step(workload, inputs, leaves):
    if workload in BATCHED:
        return leaves[-1].shape[0]
    if workload == 'rng_uniform':
        return 4096 * 4096 / 1e9
    if workload == 'gather_scatter':
        return 2 * inputs[1].size / 1e9
    return 1


def measure(workload, steps, warmup, batch=None, fuse=True, graph=False, profile_iters=3, end_to_end=True,
            dump_launches=None, calibration_copy=False, per_launch=True):
    '''Builds the workload's interpreter, times `steps` replays with resident inputs, then the per-launch shares
    and whole calls. Returns (result dict, wrapped function, inputs).'''
    import vkjax_amd
    from vkjax_amd import hip, workloads as W
    from vkjax_amd.minijax import tree_util
    from vkjax_amd.jaxpr_interpreter import JaxprInterpreter

    fn, make_inputs = W.WORKLOADS[workload]
    kwargs = {}
    if batch is not None and UNITS[workload][1]:
        kwargs['batch'] = batch
    inputs = make_inputs(**kwargs)
    dev    = hip.Device.get()

    t0 = time.perf_counter()
    wrapped = vkjax_amd.wrap(fn, frontend='minijax', fuse=fuse, graph=graph)
    interp, _ = wrapped._get_or_create_jaxpr_interpreter(tuple(inputs))
    build_s = time.perf_counter() - t0
    interp.upload_inputs(*inputs)

    if calibration_copy:
        n = 64 * 1024 * 1024
        copy = vkjax_amd.wrap(lambda x: x + 0.0, frontend='minijax')
        ci, _ = copy._get_or_create_jaxpr_interpreter((np.zeros(n, np.float32),))
        ci.replay(1)
        dev.sync()

    for _ in range(warmup):
        interp.replay(1)
    dev.sync()
    t0 = time.perf_counter()
    device_ms = 0.0
    for _ in range(steps):
        device_ms += interp.replay(1)
    dev.sync()
    wall_s = time.perf_counter() - t0
    ms_per_step        = wall_s * 1e3 / steps
    device_ms_per_step = device_ms / steps

    leaves = tree_util.tree_leaves(inputs)
    units  = units_per_step(workload, inputs, leaves)
    result = dict(workload=workload, value=round(units / (ms_per_step / 1e3), 3), unit=UNITS[workload][0],
                  ms_per_step=round(ms_per_step, 4), device_ms_per_step=round(device_ms_per_step, 4), steps=steps, warmup=warmup,
                  input_shape=list(leaves[-1].shape) if hasattr(leaves[-1], 'shape') else None,
                  launches_per_step=len(interp.launches), fused=interp.fuse,
                  hbm_bytes_allocated=interp.bufferpool.total_device_bytes(), build_seconds=round(build_s, 2))

    if per_launch:
        #per-launch shares: a second sequence of the same program with an event after every launch
        prof = JaxprInterpreter(interp.jaxpr, interp.static_argnums, profiling=True, fuse=interp.fuse)
        prof.upload_inputs(*inputs)
        stamped = np.zeros(len(prof.launches))
        for it in range(profile_iters + 1):
            prof.sequence.eval([None] * prof.sequence.n_slots, flags=hip.EVAL_SKIP_UPLOADS | hip.EVAL_SKIP_DOWNLOADS)
            if it == 0:
                continue                                            #warm-up
            stamps = prof.sequence.get_timestamps()
            stamped += np.diff(stamps)[1:1 + len(prof.launches)]    #[uploads | launches ... | downloads]
        stamped /= max(profile_iters, 1)
        scale = device_ms_per_step / float(stamped.sum()) if stamped.sum() > 0 else 1.0
        #Launches of less than 20 us: the event after every launch and the gaps between launches are a large part of
        #the stamped figure. Such a launch is also replayed ALONE, 200 times back to back on the buffers as the step
        #left them (`repeated_ms`: one launch without event and with one launch-to-launch gap; its operands may come
        #from the last-level cache, as they mostly do behind the launch that produced them). Only kernels that read
        #their inputs and write their outputs anew each time are repeated; the index passes of the sorted scatter-add
        #count in place and are left out.
        repeated = [None] * len(prof.launches)
        for k, (launch, ms) in enumerate(zip(prof.launches, stamped * scale)):
            if ms < 0.02 and kernel_family(launch.kernel) in REPEATABLE:
                single = dev.sequence()
                prof.record_launch(single, launch)
                single.replay(20)
                repeated[k] = single.replay(200) / 200
                single.destroy()
        fam = {}
        for launch, ms, rep in zip(prof.launches, stamped, repeated):
            f = fam.setdefault(kernel_family(launch.kernel), dict(launches=0, stamped_ms=0.0, flops=0, bytes=0, repeated_ms=0.0, repeated=0))
            f['launches'] += 1; f['stamped_ms'] += float(ms); f['flops'] += launch.flops; f['bytes'] += launch.bytes_moved
            if rep is not None:
                f['repeated'] += 1; f['repeated_ms'] += rep
        if dump_launches:
            with open(dump_launches, 'w') as fh:
                for op, launch, ms in zip(prof.all_ops, prof.launches, stamped * scale):
                    rate = f'{launch.flops / ms / 1e9:7.1f} TFLOP/s' if launch.flops else f'{launch.bytes_moved / ms / 1e6:7.0f} GB/s'
                    fh.write(f'{launch.kernel:28s} grid {launch.grid[0]:6d} {launch.flops / 1e9:8.3f} GFLOP {launch.bytes_moved / 1e6:8.1f} MB '
                             f'{ms * 1e3:8.1f} us {rate}  {op.equation!r:.60s}\n')
        kernels = {}
        for name, f in fam.items():
            ms = f['stamped_ms'] * scale
            entry = dict(launches=f['launches'], ms=round(ms, 5), stamped_ms=round(f['stamped_ms'], 5))
            if f['flops']:
                entry['gflop'] = round(f['flops'] / 1e9, 3)
                entry['tflops'] = round(f['flops'] / ms / 1e9, 3)
                entry['frac_mfma_peak'] = round(entry['tflops'] / PEAK_FP32_MFMA_TFLOPS, 4)
            entry['mbytes'] = round(f['bytes'] / 1e6, 3)
            entry['gbs'] = round(f['bytes'] / ms / 1e6, 1)
            entry['frac_hbm_peak'] = round(entry['gbs'] / PEAK_HBM_GBS, 4)
            if f['repeated'] == f['launches'] and f['repeated_ms'] > 0:
                #every launch of the family is a short one: the family's time without events and gaps
                entry['repeated_ms'] = round(f['repeated_ms'], 5)
                entry['repeated_gbs'] = round(f['bytes'] / f['repeated_ms'] / 1e6, 1)
                entry['repeated_frac_hbm_peak'] = round(entry['repeated_gbs'] / PEAK_HBM_GBS, 4)
                if f['flops']:
                    entry['repeated_tflops'] = round(f['flops'] / f['repeated_ms'] / 1e9, 3)
            kernels[name] = entry
        dominant = max(fam, key=lambda k: fam[k]['stamped_ms'])
        d, ms = fam[dominant], fam[dominant]['stamped_ms'] * scale
        #(dense_rows_n16 multiplies on the vector ALUs: a few rows of a small batch, priced by the bytes it moves)
        if d['flops'] and dominant != 'dense_rows':
            achieved = d['flops'] / ms / 1e9
            roofline = dict(bound='mfma', kernel=dominant, achieved=round(achieved, 3), peak=PEAK_FP32_MFMA_TFLOPS, unit='TFLOP/s',
                            frac=round(achieved / PEAK_FP32_MFMA_TFLOPS, 4))
        else:
            achieved = d['bytes'] / ms / 1e6
            roofline = dict(bound='hbm', kernel=dominant, achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit='GB/s',
                            frac=round(achieved / PEAK_HBM_GBS, 4))
        roofline.update(traffic=measured_hbm_traffic(workload, dominant), launches_per_step=d['launches'],
                        avg_launch_ms=round(ms / d['launches'], 5), stamped_avg_launch_ms=round(d['stamped_ms'] / d['launches'], 5))
        if dominant == 'threefry2x32':
            #the draw is bound by the integer ALUs, not by its stores: 68 vector instructions per Threefry block of two
            #words (20 rounds of add / rotate / xor, five key injections, counters, the uniform chain), 16 lanes per
            #SIMD and clock; the time below is that floor at the device's nominal clock
            props   = hip.Device.get().get_device_properties()
            blocks  = sum(l.bytes_moved for l in prof.launches if kernel_family(l.kernel) == dominant) / 8
            floor   = blocks * 68 / (props['compute_units'] * 4 * 16 * props['clock_khz'] * 1e3) * 1e3
            longest = max(m for l, m in zip(prof.launches, stamped * scale) if kernel_family(l.kernel) == dominant)
            roofline.update(valu_floor_ms=round(floor, 5), longest_launch_ms=round(float(longest), 5),
                            frac_of_valu_floor=round(floor / float(longest), 4))
        result.update(roofline=roofline, kernels=kernels)

    if end_to_end:
        result['end_to_end_call'] = time_whole_calls(fn, inputs, fuse)
        if workload == 'resnet50':
            result['steps_in_flight'] = time_steps_in_flight(interp, inputs, units)
    return result, wrapped, inputs


def time_steps_in_flight(interp, inputs, units, lanes=3, steps=20, warm=3):
    '''Throughput of independent steps with `lanes` of them on the device at a time: the program is recorded once per
    lane, each on a device context (streams, buffers) of its own with its inputs resident, and every lane replays
    `steps` steps from a thread of its own; the clock runs from a common start until the last lane is through. The
    launches of one step still run in order on one stream - what the GPU gains is that the start and the tail of one
    lane's launches are covered by the other lanes' work. This is NOT the headline `value` (one in-order stream).'''
    import threading
    from vkjax_amd import hip
    from vkjax_amd.jaxpr_interpreter import JaxprInterpreter
    index = hip.Device.get().index
    programs = [JaxprInterpreter(interp.jaxpr, interp.static_argnums, fuse=interp.fuse, device=hip.Device(index)) for _ in range(lanes)]
    for program in programs:
        program.upload_inputs(*inputs)
        program.replay(warm)
    gate = threading.Barrier(lanes + 1)
    def run(program):
        gate.wait()
        program.replay(steps)
    threads = [threading.Thread(target=run, args=(program,)) for program in programs]
    for t in threads:
        t.start()
    gate.wait()
    t0 = time.perf_counter()
    for t in threads:
        t.join()
    ms = (time.perf_counter() - t0) * 1e3 / (lanes * steps)
    return dict(lanes=lanes, steps=lanes * steps, ms_per_step=round(ms, 4), value=round(units / (ms / 1e3), 3))


def measure_primitives(iters=30, warm=10, only=None):
    '''Single primitives at sizes where HBM bandwidth is the bound (vkjax_amd.workloads.PRIMITIVES): each program is
    built, its inputs are made resident, and its launches are replayed `iters` times back to back between two HIP
    events on the launch stream (after `warm` untimed replays). `bytes` is the ALGORITHMIC traffic of one evaluation
    - every operand read once, every result written once - so `gbs` is what the caller of the primitive sees;
    gaps between the launches of a program (one to five launches) are inside the time.'''
    import gc
    import vkjax_amd
    from vkjax_amd import hip, workloads as W
    dev, rows = hip.Device.get(), []
    for name, (fn, make_inputs, algorithmic_bytes) in W.PRIMITIVES.items():
        if only and not any(o in name for o in only):
            continue
        inputs  = make_inputs()
        wrapped = vkjax_amd.wrap(fn, frontend='minijax')
        interp, _ = wrapped._get_or_create_jaxpr_interpreter(tuple(inputs))
        interp.upload_inputs(*inputs)
        interp.replay(warm)
        ms = statistics.median(interp.replay(iters) for _ in range(3)) / iters
        nbytes = int(algorithmic_bytes(inputs))
        gbs = nbytes / ms / 1e6
        rows.append(dict(primitive=name, kernels=[l.kernel for l in interp.launches], mbytes=round(nbytes / 1e6, 3), ms=round(ms, 5),
                         gbs=round(gbs, 1), frac_hbm_peak=round(gbs / PEAK_HBM_GBS, 4)))
        del interp, wrapped, inputs
        gc.collect()
        dev.sync()
    return rows


def time_whole_calls(fn, inputs, fuse):
    '''Whole calls through wrap(): host arrays in, host arrays out, uploads and Python included; once copying every
    argument per call (what the reference does, vkjax/kompute_jaxpr_interpreter.py:66-81), once with the weights
    resident, once streamed (each call's upload overlaps the call before it), once streamed with two calls on the device at
    a time. Median of 9 / mean of 40 (80) after 4 (8).'''
    import vkjax_amd
    from vkjax_amd.minijax import tree_util
    out = {}
    def frozen(a):
        a = a.copy()
        a.flags.writeable = False
        return a
    #read_only_weights_ms: plain wrap(f)(params, x), nothing declared, with a parameter tree of read-only arrays, which
    #stay in HBM by themselves; weights_resident_ms: writeable parameters declared resident (each looked at for changes)
    for label, kw in (('all_arguments_copied_ms', {}), ('read_only_weights_ms', {}), ('weights_resident_ms', dict(resident_argnums=(0,)))):
        if label != 'all_arguments_copied_ms' and not isinstance(inputs[0], dict):
            continue
        f = vkjax_amd.wrap(fn, frontend='minijax', fuse=fuse, **kw)
        call_inputs = [tree_util.tree_map(frozen, inputs[0])] + list(inputs[1:]) if label == 'read_only_weights_ms' else inputs
        f(*call_inputs)
        f(*call_inputs)
        times = []
        for _ in range(9):
            t0 = time.perf_counter()
            f(*call_inputs)
            times.append((time.perf_counter() - t0) * 1e3)
        out[label] = round(statistics.median(times), 3)
        if label == 'weights_resident_ms':
            n, warm = 40, 4                  #(the first streamed calls allocate their landing buffers and find the clocks low)
            results = f.stream([tuple(inputs)] * (n + warm))
            for _ in range(warm):
                next(results)
            t0 = time.perf_counter()
            for _ in results:
                pass
            out['weights_resident_streamed_ms'] = round((time.perf_counter() - t0) * 1e3 / n, 3)
            #the same with two and with three batches on the device at a time, each on a context of its own
            #(Function.stream(in_flight=...)). The lanes run up to four tuples each ahead of the consumer, so results that
            #were finished before the clock starts must not count: the rate is taken between arrivals that the consumer
            #had to wait for
            for lanes, label_lanes in ((2, 'two'), (3, 'three')):
                ahead = 4 * lanes
                arrivals = []
                for _ in f.stream([tuple(inputs)] * (2 * n + 2 * warm + ahead), in_flight=lanes):
                    arrivals.append(time.perf_counter())
                first = 2 * warm + ahead - 1
                out[f'weights_resident_streamed_{label_lanes}_in_flight_ms'] = round(
                    (arrivals[-1] - arrivals[first]) * 1e3 / (len(arrivals) - 1 - first), 3)
    return out


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


# ------------------------------------------------------------------ CPU baseline

def host_cores():
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    for name in ('OMP_NUM_THREADS',):                #the share of the machine this process was given
        if os.environ.get(name, '').isdigit():
            n = min(n, int(os.environ[name]))
    return max(n, 1)


def torch_cpu_graph(workload, inputs):
    '''The workload as an fp32 torch graph on the CPU: returns a function without arguments that evaluates it once
    and returns its results as numpy arrays (same order as the traced function's), or None for workloads torch has
    no counterpart of (the threefry draw).'''
    import torch
    import torch.nn.functional as F
    from vkjax_amd.workloads import RESNET50_STAGES, _same_pads
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))

    def conv_bn(p, x, stride=1, pads=None, relu=True, residual=None):
        kh, kw = p['w_oihw'].shape[2], p['w_oihw'].shape[3]
        if pads is None:
            pads = (_same_pads(x.shape[2], kh, stride), _same_pads(x.shape[3], kw, stride))
        if pads[0][0] == pads[0][1] and pads[1][0] == pads[1][1]:
            y = F.conv2d(x, p['w_oihw'], stride=stride, padding=(pads[0][0], pads[1][0]))
        else:
            y = F.conv2d(F.pad(x, (pads[1][0], pads[1][1], pads[0][0], pads[0][1])), p['w_oihw'], stride=stride)
        y = (y - p['mean']) * p['inv'] + p['shift']
        if residual is not None:
            y = y + residual
        return F.relu(y) if relu else y

    def prepared(p):
        c = lambda v: t(v).reshape(1, -1, 1, 1)
        return dict(w_oihw=t(p['w']).permute(3, 2, 0, 1).contiguous(memory_format=torch.channels_last),
                    inv=c(p['scale']) * torch.rsqrt(c(p['var']) + 1e-5), shift=c(p['shift']), mean=c(p['mean']))

    def max_pool_3x3_s2(y):
        ph, pw = _same_pads(y.shape[2], 3, 2), _same_pads(y.shape[3], 3, 2)
        return F.max_pool2d(F.pad(y, (pw[0], pw[1], ph[0], ph[1]), value=float('-inf')), 3, 2)

    if workload == 'affine':
        x, W, b = map(t, inputs)
        return lambda: [(x @ W + b).numpy()]
    if workload == 'mlp':
        p, x = {k: t(v) for k, v in inputs[0].items()}, t(inputs[1])
        def run():
            h = F.relu(x @ p['w1'] + p['b1'])
            h = F.relu(h @ p['w2'] + p['b2'])
            probs = F.softmax(h @ p['w3'] + p['b3'], dim=-1)
            return [probs.numpy(), probs.argmax(dim=1).to(torch.int32).numpy()]
        return run
    if workload == 'conv_block':
        p = prepared(inputs[0])
        x = t(inputs[1]).permute(0, 3, 1, 2).contiguous(memory_format=torch.channels_last)
        def run():
            y = conv_bn(p, x, pads=((1, 1), (1, 1)))
            y = F.max_pool2d(F.pad(y, (0, 1, 0, 1), value=float('-inf')), 3, 2)
            return [y.permute(0, 2, 3, 1).contiguous().numpy()]
        return run
    if workload == 'resnet50':
        params = inputs[0]
        stem   = prepared(params['stem'])
        stages = [[{k: prepared(v) for k, v in params[f'stage{s}'][f'block{b}'].items()} for b in range(blocks)]
                  for s, (blocks, _, _) in enumerate(RESNET50_STAGES)]
        fc_w, fc_b = t(params['fc']['w']), t(params['fc']['b'])
        x = t(inputs[1]).permute(0, 3, 1, 2).contiguous(memory_format=torch.channels_last)
        def run():
            y = conv_bn(stem, x, stride=2, pads=((3, 3), (3, 3)))
            y = max_pool_3x3_s2(y)
            for s, (blocks, _, stride) in enumerate(RESNET50_STAGES):
                for b in range(blocks):
                    p  = stages[s][b]
                    st = stride if b == 0 else 1
                    shortcut = conv_bn(p['proj'], y, stride=st, relu=False) if 'proj' in p else y
                    z = conv_bn(p['conv1'], y)
                    z = conv_bn(p['conv2'], z, stride=st)
                    y = conv_bn(p['conv3'], z, relu=True, residual=shortcut)
            logits = y.mean(dim=(2, 3)) @ fc_w + fc_b
            return [logits.numpy(), logits.argmax(dim=1).to(torch.int32).numpy()]
        return run
    if workload == 'gather_scatter':
        table, idx, updates = t(inputs[0]), t(inputs[1]).to(torch.int64), t(inputs[2])
        flat_idx, flat_upd = idx.reshape(-1), updates.reshape(-1, updates.shape[-1])
        def run():
            rows = table[idx]
            acc  = torch.zeros_like(table).index_add_(0, flat_idx, flat_upd)
            return [rows.numpy(), acc.numpy()]
        return run
    return None


def time_cpu_baseline(workload, fn, inputs, budget_s=12.0):
    '''The same program on this machine's host cores. jax's CPU backend is the reference's ground truth; where jax
    is not importable, the fp32 torch-CPU graph above stands in for it (the numpy oracle for the threefry draw).
    Returns (record, results of one evaluation as numpy arrays, or None).'''
    from vkjax_amd.minijax import tree_util
    cores  = host_cores()
    leaves = tree_util.tree_leaves(inputs)
    units  = units_per_step(workload, inputs, leaves)
    sample = 'the same inputs and shapes as the GPU run'
    run, kind, note = None, None, ''
    try:
        import jax                                    # noqa: F401
        #the workloads are written against the stand-in front-end; a jax.numpy graph of them is not part of this file
        note = 'jax importable on this machine but not used for this figure; '
    except ImportError:
        pass
    try:
        import torch
        torch.set_num_threads(cores)
        run = torch_cpu_graph(workload, inputs)
        if run is not None:
            kind = 'substitute: torch-cpu fp32, jax not installed'
            note += f'torch {torch.__version__}, {torch.get_num_threads()} intra-op threads'
    except ImportError:
        run = None
    if run is None:
        from vkjax_amd import minijax as mj
        from oracle.eval_jaxpr import eval_closed_jaxpr
        closed = mj.make_jaxpr(fn)(*inputs)
        run    = lambda: eval_closed_jaxpr(closed, *leaves)
        kind   = 'port'
        note  += 'numpy oracle of the same program (float64 accumulation, BLAS threads = host cores)'
    results = run()                                   #warm-up, and the values the GPU result is compared with
    reps, t_total = 0, 0.0
    while reps < 3 or (t_total < budget_s and reps < 20):
        t0 = time.perf_counter()
        run()
        t_total += time.perf_counter() - t0
        reps += 1
        if t_total > 3 * budget_s:
            break
    per_call = t_total / reps
    record = dict(value=round(units / per_call, 4), unit=UNITS[workload][0], cores=cores, kind=kind,
                  ms_per_step=round(per_call * 1e3, 3),
                  sample=f'{sample}; {reps} evaluations after one warm-up, {per_call:.3f} s each; {note}')
    return record, [np.asarray(r) for r in results]


def check_outputs(got, expected, rtol):
    '''Largest deviation of the GPU results from the CPU baseline's, per result. Float results: |a - b| against
    rtol * |b| + 1e-5 * max|b| (values that cross zero have no meaningful relative error); integer results
    (arg-max labels): fraction that agree.'''
    report = []
    for a, b in zip(got, expected):
        a, b = np.asarray(a), np.asarray(b)
        if a.shape != b.shape:
            report.append(dict(ok=False, reason=f'shape {a.shape} vs {b.shape}'))
        elif np.issubdtype(b.dtype, np.floating):
            scale = float(np.abs(b).max()) or 1.0
            err   = np.abs(a.astype(np.float64) - b.astype(np.float64))
            ok    = bool((err <= rtol * np.abs(b) + 1e-5 * scale).all())
            report.append(dict(ok=ok, max_abs_err=float(err.max()), max_abs_value=scale, rtol=rtol))
        else:
            report.append(dict(ok=bool((a == b).mean() > 0.98), agree=float((a == b).mean())))
    return dict(ok=all(r['ok'] for r in report), against='cpu_baseline results', results=report)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--workload', default='resnet50', choices=list(UNITS))
    ap.add_argument('--batch', type=int, default=None)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-fuse', action='store_true')
    ap.add_argument('--no-configs', action='store_true', help='measure only the named workload, not the other configurations of the metric')
    ap.add_argument('--no-end-to-end', action='store_true', help='skip the whole-call timings through wrap()')
    ap.add_argument('--replays-only', action='store_true',
                    help='warm-up and timed replays only (no per-launch sequence, whole calls, other configurations or CPU baseline): '
                         'under a kernel trace every dispatch after the first warmup x launches_per_step then belongs to a timed step')
    ap.add_argument('--graph', action='store_true', help='replay the launches as one captured HIP graph')
    ap.add_argument('--no-primitives', action='store_true', help='skip the single-primitive bandwidth measurements')
    ap.add_argument('--primitives-only', nargs='*', default=None, metavar='NAME',
                    help='measure only the single primitives (those whose name contains one of the given words; all if none is given)')
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

    from vkjax_amd import hip, workloads as W
    props = hip.Device.get().get_device_properties()
    lean  = args.replays_only
    if args.primitives_only is not None:
        if args.calibration_copy:
            import vkjax_amd
            copy = vkjax_amd.wrap(lambda x: x + 0.0, frontend='minijax')
            ci, _ = copy._get_or_create_jaxpr_interpreter((np.zeros(64 * 1024 * 1024, np.float32),))
            ci.replay(1)                                   #the first dispatch of the run: 256 MiB read, 256 MiB written
            hip.Device.get().sync()
            del ci, copy
        print(json.dumps({'metric': 'per-primitive HBM GB/s', 'unit': 'GB/s', 'n_gpus': 1, 'dtype': 'f32', 'data': 'synthetic',
                          'peak_hbm_gbs': PEAK_HBM_GBS, 'replays_per_primitive': {'warm': 10, 'timed': 90},
                          'primitives': measure_primitives(only=args.primitives_only)}))
        return

    head, wrapped, inputs = measure(args.workload, args.steps, args.warmup, batch=args.batch, fuse=not args.no_fuse, graph=args.graph,
                                    profile_iters=args.profile_iters, end_to_end=not (lean or args.no_end_to_end),
                                    dump_launches=args.dump_launches, calibration_copy=args.calibration_copy, per_launch=not lean)

    cpu_baseline, output_check = None, None
    if not (args.no_cpu_baseline or lean):
        cpu_baseline, expected = time_cpu_baseline(args.workload, W.WORKLOADS[args.workload][0], inputs)
        from vkjax_amd.minijax import tree_util
        got = tree_util.tree_leaves(wrapped(*inputs))            #the timed interpreter, this time with uploads and downloads
        rtol = 1e-3 if args.workload.startswith('resnet50') else 1e-4
        if expected is not None and len(expected) == len(got):
            output_check = check_outputs(got, expected, rtol)

    configs = []
    if args.workload == 'resnet50' and args.batch in (None, 64) and not (args.no_configs or lean):
        for name in OTHER_CONFIGS:
            c, _, _ = measure(name, steps=100, warmup=10, fuse=not args.no_fuse, profile_iters=args.profile_iters,
                              end_to_end=not args.no_end_to_end)
            configs.append(c)

    primitives = None
    if args.workload == 'resnet50' and args.batch in (None, 64) and not (args.no_configs or args.no_primitives or lean):
        primitives = measure_primitives()

    out = {
        'metric': 'ResNet-50 bs64 fp32 images/sec' if args.workload == 'resnet50' else f'{args.workload} throughput',
        'value': head['value'], 'unit': head['unit'], 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': head['ms_per_step'], 'device_ms_per_step': head['device_ms_per_step'],
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'timed_region': 'device-only replay of the recorded launches, inputs and weights resident in HBM; whole calls through wrap() '
                        'are in config.end_to_end_call, the throughput of independent steps with three on the device at a time in config.steps_in_flight',
        'config': {'workload': args.workload, 'input_shape': head['input_shape'],
                   'launches_per_step': head['launches_per_step'], 'fused': head['fused'], 'inputs_resident_in_hbm': True,
                   'device': props['device_name'] or props['arch'], 'arch': props['arch'], 'compute_units': props['compute_units'],
                   'hbm_bytes_allocated': head['hbm_bytes_allocated'], 'build_seconds': head['build_seconds'],
                   **({'end_to_end_call': head['end_to_end_call']} if 'end_to_end_call' in head else {}),
                   **({'steps_in_flight': head['steps_in_flight']} if 'steps_in_flight' in head else {})},
        'roofline': head.get('roofline'), 'kernels': head.get('kernels'), 'cpu_baseline': cpu_baseline, 'output_check': output_check,
        'configs': configs, 'primitives': primitives,
    }
    print(json.dumps(out))


if __name__ == '__main__':
    main()
