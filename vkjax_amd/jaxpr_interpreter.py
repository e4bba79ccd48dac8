'''The jaxpr interpreter: analyses a closed jaxpr once into device ops and buffers, records
them into one replayable sequence, and runs it with one native call per invocation.

Same structure and public surface as the reference's JaxprInterpreter
(vkjax/kompute_jaxpr_interpreter.py:14-102): constructor arguments `(jaxpr, static_argnums,
profiling, reuse_buffers)`, `.run(*X, return_all=False)`, `.get_profiling_info()`, attributes
`.jaxpr .static_argnums .bufferpool .all_ops .sequence`. The Kompute manager / tensors /
sequence are replaced by the HIP runtime behind include/vkjax_hip.h.
'''
import os
import typing as tp

import numpy as np

from . import fusion
from . import hip
from . import kernels as K
from . import lanes
from . import ops
from .buffers import BufferPool, PlanOnlyDevice, to_device_words, view_or_convert_from_32bit
from .minijax import core, tree_util


class JaxprInterpreter:
    def __init__(self, jaxpr, static_argnums: tp.Tuple[int, ...] = (), profiling: bool = False,
                 reuse_buffers: bool = True, fuse: bool = True, plan_only: bool = False, graph: bool = False,
                 resident_argnums: tp.Tuple[int, ...] = (), two_lanes: bool = False, device: tp.Optional['hip.Device'] = None):
        self.jaxpr          = jaxpr
        #Which argument leaves stay in HBM between calls instead of being copied on every call, as the reference
        #does (vkjax/kompute_jaxpr_interpreter.py:72-75):
        # * leaves that cannot change under the caller's feet - numpy arrays that are not writeable (nor views of
        #   writeable ones) and jax arrays - without being asked: such a leaf is uploaded when the object passed for
        #   it is not the one uploaded last;
        # * every leaf of the arguments named in resident_argnums (weights, tables), writeable or not. A writeable
        #   one that is changed in place is noticed only when its first or last 64 bytes change; pass a new array
        #   (or a read-only one) for a new value.
        #All other leaves are copied on every call.
        self.resident_argnums = tuple(resident_argnums)
        self._resident_leaves = {}
        #two_lanes: launches that do not depend on the ones before them run beside them on a second stream
        #(vkjax_amd/lanes.py). Off by default: on this GPU a dependency between two streams costs about 12 us, more
        #than the launches it would let overlap (see the measurements quoted in lanes.py)
        self.two_lanes      = two_lanes
        #graph=True replays the launches as one captured HIP graph (never with profiling)
        self.graph          = graph and not profiling
        self.static_argnums = tuple(static_argnums)
        self.profiling      = profiling
        self.fuse           = fuse
        #plan_only builds ops, buffers and launch parameters without touching a GPU; such an
        #interpreter cannot run
        #(device: a context other than the shared one of hip.Device.get(); it has its own streams, so programs on
        #different contexts, each driven by a thread of its own, run side by side on the GPU)
        self.mgr            = PlanOnlyDevice() if plan_only else (device if device is not None else hip.Device.get())
        self.workgroup_size = get_maximum_workgroup_size(self.mgr)
        self.bufferpool     = BufferPool(self.mgr, self.workgroup_size, reuse_buffers)
        self.sequence       = None
        #counts evaluations: a suspended stream sees from it whether something else has used the argument buffers
        self._evaluations   = 0
        self.analyze_closed_jaxpr(jaxpr)

    def analyze_closed_jaxpr(self, jaxpr):
        '''Starts the analysis of the top level jaxpr.
           Records operations into a sequence and creates required buffers.'''
        assert len(jaxpr.consts) == len(jaxpr.jaxpr.constvars)
        for constvar, constval in zip(jaxpr.jaxpr.constvars, jaxpr.consts):
            b = self.bufferpool.get_buffer(constvar)
            self.bufferpool.mark_buffer_as_constant(b, constvar, value=np.asarray(constval))

        for v in list(jaxpr.jaxpr.invars) + list(jaxpr.jaxpr.outvars):
            b = self.bufferpool.get_buffer(v)
            if b is None:
                continue
            #inputs and outputs own their storage: it is never handed to another variable
            self.bufferpool.mark_buffer_as_constant(b, v, None)

        self.input_buffers  = [self.bufferpool.get_buffer(v) for v in jaxpr.jaxpr.invars]
        self.all_ops        = ops.analyze_jaxpr(self.bufferpool, jaxpr.jaxpr)
        if self.fuse:
            self.all_ops    = fusion.fuse_ops(self.all_ops, self.bufferpool, jaxpr.jaxpr.outvars)
        self.output_buffers = [self.bufferpool.get_buffer(v) for v in jaxpr.jaxpr.outvars]
        #A result that is a view of an intermediate (a reshape of the last launch's output) shares that
        #intermediate's storage, which must stay untouched until the download: pinned to the end of the
        #program, whatever positions the passes above have given the launches.
        for b in self.output_buffers:
            if b is not None:
                b.accesses.append(np.inf)
        self.bufferpool.create_tensors()
        #lower every op now so that unsupported layouts fail at build time, not at run time
        self.launches = self._stream_unread_results([op.launch for op in self.all_ops])
        self.lane_plan = lanes.plan(self.all_ops, self.launches) if self.two_lanes else None
        self.early_parts = []

        if isinstance(self.mgr, PlanOnlyDevice):
            return
        self.sequence = self.mgr.sequence(profiling=self.profiling)
        self._input_slots = []
        #(elements, dtype) of a host array that can be handed to the device as it is
        self._input_specs = []
        for var in jaxpr.jaxpr.invars:
            shape, dtype = core.physical(var.aval)
            self._input_specs.append((int(np.prod(shape, dtype=np.int64)), dtype if dtype in (np.float32, np.int32, np.uint32) else None))
        for b in self.input_buffers:
            self._input_slots.append(self.sequence.record_upload(b.tensor, b.nbytes()) if b is not None else None)
        self._batch_tables = []
        for op, launch in zip(self.all_ops, self.launches):
            self.record_launch(self.sequence, launch, op)
        if self.lane_plan is not None and any(self.lane_plan.lane):
            for k, (lane, wait) in enumerate(zip(self.lane_plan.lane, self.lane_plan.wait)):
                if lane or wait:
                    self.sequence.set_launch_lane(k, lane, wait)
        #the first launch in parts that start while the rest of its (large) argument is still being uploaded
        self.early_parts = self._early_parts_of_first_launch()
        for part, slot, needed in self.early_parts:
            bufs = [((b.tensor if b is not None else None), off) for b, off in part.buffers]
            self.sequence.record_launch(part.kernel, part.grid, part.block, bufs, part.params, part.lds, early_part_of=(slot, needed))
        if self.graph:
            self.sequence.use_graph(True)
        self._output_slots = []
        self._output_sizes = []
        for b in self.output_buffers:
            if b is None:
                self._output_slots.append(None)
                self._output_sizes.append(None)
                continue
            self._output_slots.append(self.sequence.record_download(b.tensor, b.nbytes()))
            self._output_sizes.append(b.size)

    def _stream_unread_results(self, launches):
        '''Large results that no later launch of the program reads (they leave for the host, or simply stay) are stored
        past the caches by the kernels that can do that (kernels.with_streamed_result): they would only push out what the
        following launches could find there. Results that a later launch reads stay with the caches: the next launch often
        finds a good part of them in the 256 MB behind the L2s.'''
        touched_later = set()
        result = list(launches)
        for k in range(len(launches) - 1, -1, -1):
            launch = launches[k]
            members = launch.members or (launch,)
            if launch.streamable and not launch.members:
                out = launch.buffers[0][0]
                nbytes = out.size * 4 if out is not None else 0
                if (out is not None and out.tensor is not None and id(out.tensor) not in touched_later
                        and K.STREAM_RESULT_MIN_BYTES <= nbytes < 2**32):
                    result[k] = K.with_streamed_result(launch)
            for m in members:
                #(an array a later launch only writes - the next part of a concatenation - is not read by it; kernels that
                #add to what their result array holds do read it)
                touched_later |= {id(b.tensor) for i, (b, _) in enumerate(m.buffers) if b is not None and b.tensor is not None
                                  and (i not in m.written or m.kernel in K.ACCUMULATING_KERNELS)}
        return result

    #an argument from this size on is worth starting the first launch on while it is still arriving (the link moves
    #about 50 MB per millisecond; a part more costs a few microseconds of device time)
    EARLY_PARTS_MIN_BYTES = 16 << 20

    def _early_parts_of_first_launch(self):
        '''[(launch, upload slot, bytes of the argument the part needs)]: the program's first launch cut along the batch
        into parts that together compute what it computes, when it is a convolution or matrix product over a large
        argument whose images (rows) are computed independently by one kernel of the family in which a wave sums
        its contraction in one fixed order whatever the tiling (so every part's values are the whole launch's, bit for
        bit). The runtime issues a part as soon as the chunks of the argument it reads are on their way
        (vkj_seq_record_early_part); evaluations that do not upload that argument run the launch as it is.'''
        if (not self.all_ops or self.profiling or self.graph or (self.lane_plan is not None and any(self.lane_plan.lane))
                or self.all_ops[0].conv is None):
            return []
        out, lhs, rhs, geom, epilogue = self.all_ops[0].conv
        whole = self.launches[0]
        k = next((i for i, b in enumerate(self.input_buffers) if b is lhs), None)
        if k is None or self._input_slots[k] is None or lhs.nbytes() < self.EARLY_PARTS_MIN_BYTES:
            return []
        B = geom.batch
        nparts = 4 if B % 4 == 0 else 2 if B % 2 == 0 else 0
        plain = (whole.kernel.startswith('conv_gemm') and not any(tag in whole.kernel for tag in ('_mix', '_ks4')) and not whole.members)
        if (not nparts or not plain or geom.k_splits > 1 or lhs.size % B or out.size % B or geom.xs[0] != lhs.size // B
                or geom.os[0] != out.size // B or any(e.kind == 3 or e.op in (K.CONV_TAP, K.CONV_SOFTMAX) for e in epilogue)):
            return []
        parts = []
        for p in range(nparts):
            try:
                part = K.conv_gemm(out, lhs, rhs, geom._replace(batch=B // nparts), epilogue,
                                   lhs_offset=p * (lhs.size // nparts), out_offset=p * (out.size // nparts))
            except (ValueError, NotImplementedError):
                return []
            if part.kernel != whole.kernel:
                return []
            parts.append((part, self._input_slots[k], (p + 1) * (lhs.nbytes() // nparts)))
        return parts

    def record_launch(self, sequence, launch, op=None):
        '''Records one of this program's launches into `sequence` (its own, or another sequence on the same buffers:
        measurements replay single launches that way).'''
        if launch.members:
            #a batch of small launches reads its members' arguments from a table in HBM
            table = self.mgr.tensor(K.batch_table(launch, lambda b: b.tensor.device_ptr()))
            self._batch_tables.append(table)
            members = {id(b.tensor): b.tensor for m in launch.members for b, _ in m.buffers if b is not None}
            sequence.record_launch(launch.kernel, launch.grid, launch.block, [(table, 0)], launch.params, launch.lds,
                                   reached_through_tables=list(members.values()))
            return
        bufs = [((b.tensor if b is not None else None), off) for b, off in launch.buffers]
        for (b, _), (t, _) in zip(launch.buffers, bufs):
            assert b is None or t is not None, f'{op or launch.kernel}: buffer without storage'
        sequence.record_launch(launch.kernel, launch.grid, launch.block, bufs, launch.params, launch.lds)

    def _flatten_args(self, X, with_residency: bool = False, per_argument=None):
        '''`per_argument`: the leaves of every argument (static ones included) where the caller has them already.'''
        leaves, resident = [], []
        for i, x in enumerate(X if per_argument is None else per_argument):
            if i in self.static_argnums:
                continue
            these = x if per_argument is not None else [x] if type(x) is np.ndarray else tree_util.tree_leaves([x])
            leaves   += these
            named     = i in self.resident_argnums
            resident += [RESIDENT_CHECKED if named and _may_change_in_place(leaf) else RESIDENT if named or _is_immutable(leaf) else 0
                         for leaf in these]
        if len(self.input_buffers) != len(leaves):
            raise TypeError(f'Expected {len(self.input_buffers)} input arguments, received {len(leaves)}')
        return (leaves, resident) if with_residency else leaves

    def _convert_inputs(self, X, per_argument=None) -> tp.List[tp.Tuple]:
        '''(leaf number, transfer slot, the leaf, its device words, whether it is a resident one) for every argument
        leaf the program reads. The words of a leaf that is identified by its object alone are left out (None) and
        made when the leaf turns out to need an upload. Touches no state of the interpreter: it may run ahead of the
        evaluation it is for.'''
        X, resident = self._flatten_args(X, with_residency=True, per_argument=per_argument)
        if self.sequence is None:
            raise RuntimeError('this interpreter was built with plan_only=True and has no device to run on')
        return [(k, slot, x, None if resident[k] == RESIDENT else self._device_words(k, x), resident[k])
                for k, (slot, x) in enumerate(zip(self._input_slots, X)) if slot is not None]

    def _device_words(self, k: int, x) -> np.ndarray:
        #the common case without the general conversion: an array that already is what the device holds
        n, dtype = self._input_specs[k]
        if type(x) is np.ndarray and x.dtype == dtype and x.size == n and x.flags.c_contiguous:
            return x.reshape(-1).view(np.uint32)
        return _device_words_of_argument(x, self.jaxpr.jaxpr.invars[k].aval)

    def _select_uploads(self, converted) -> tp.List[tp.Optional[np.ndarray]]:
        '''One entry per transfer slot: the device words of every leaf that has to be copied. A resident leaf is
        copied when the object passed for it is not the one its buffer holds, and is noted as held from here on:
        to be called only when the evaluation that uploads these arguments follows at once.'''
        host = [None] * self.sequence.n_slots
        for k, slot, x, words, is_resident in converted:
            if is_resident:
                held = self._resident_leaves.get(k)
                mark = _fingerprint(x, words) if is_resident == RESIDENT_CHECKED else None
                if held is not None and held[0] is x and held[1] == mark:
                    continue                                    #already in HBM
                self._resident_leaves[k] = (x, mark)
            host[slot] = words if words is not None else self._device_words(k, x)
        return host

    def _host_inputs(self, X, per_argument=None) -> tp.List[tp.Optional[np.ndarray]]:
        return self._select_uploads(self._convert_inputs(X, per_argument))

    def _fresh_outputs(self, host) -> tp.List[tp.Optional[np.ndarray]]:
        #every call hands out fresh arrays: the runtime copies the results straight into them
        fresh = [np.empty(n, np.uint32) if n is not None else None for n in self._output_sizes]
        for slot, arr in zip(self._output_slots, fresh):
            if slot is not None:
                host[slot] = arr
        return fresh

    def _output_values(self, fresh) -> tp.Tuple:
        return tuple(None if b is None else view_or_convert_from_32bit(arr, b.dtype).reshape(b.shape)
                     for b, arr in zip(self.output_buffers, fresh))

    def evaluate(self, host, next_host_arrays=None):
        '''One evaluation of the recorded sequence: `host` holds the arrays to copy in and the fresh result arrays,
        slots left None keep what their buffers hold. Launches that share zero-initialised scratch memory (the
        counters of the sorted scatter-add) leave it zero again only when they run to the end: after an evaluation
        that failed, the zeros are written again before the error is passed on, so that a later evaluation does not
        start from whatever the failed one left.'''
        try:
            self.sequence.eval(host, flags=hip.EVAL_NULL_IS_RESIDENT, next_host_arrays=next_host_arrays)
        except BaseException:
            self._resident_leaves.clear()                       #nothing is known about what reached HBM
            for key, b in self.bufferpool.buffers.items():
                if isinstance(key, tuple) and key[:1] == ('zeroed',):
                    try:
                        b.tensor.upload(np.zeros(b.size, np.uint32))
                    except Exception:                            #a device that is gone reports the first error
                        pass
            raise
        finally:
            self._evaluations += 1

    def run_leaves(self, per_argument):
        '''`run` for a caller that has flattened the arguments already: one list of leaves per argument.'''
        host  = self._host_inputs(None, per_argument)
        fresh = self._fresh_outputs(host)
        self.evaluate(host)
        return self._output_values(fresh)

    def run(self, *X, return_all=False):
        '''Executes a previously recorded sequence with actual data'''
        host  = self._host_inputs(X)
        fresh = self._fresh_outputs(host)
        self.evaluate(host)
        output_values = self._output_values(fresh)
        if not return_all:
            return output_values
        all_arrays = [(var, buf.numpy() if buf is not None else None) for var, buf in self.bufferpool.buffers.items()]
        return output_values, dict(all_arrays)

    def run_stream(self, argument_tuples: tp.Iterable[tp.Tuple]):
        '''Runs the sequence on one tuple of arguments after the other and yields each result in
        turn. While the device works on one tuple, the next one is taken from the iterable, staged
        and uploaded, so that in the steady state a call costs the longer of the two instead of
        their sum (the reference copies, runs and reads back strictly in turn,
        vkjax/kompute_jaxpr_interpreter.py:72-81).'''
        end      = object()
        iterator = iter(argument_tuples)
        current  = next(iterator, end)
        if current is end:
            return
        in_place = False                                         #current's arguments were uploaded by the previous evaluation
        while True:
            if in_place and self._evaluations != stamp:
                in_place = False                                 #something else used the argument buffers in between
            host      = [None] * self.sequence.n_slots if in_place else self._host_inputs(tuple(current))
            following = next(iterator, end)
            next_host = self._host_inputs(tuple(following)) if following is not end else None
            fresh     = self._fresh_outputs(host)
            self.evaluate(host, next_host)
            stamp, in_place = self._evaluations, following is not end
            yield self._output_values(fresh)
            if following is end:
                return
            current = following

    def upload_inputs(self, *X):
        '''Copy arguments into their HBM buffers without running (for measurements with resident inputs).'''
        X = self._flatten_args(X)
        for b, x, var in zip(self.input_buffers, X, self.jaxpr.jaxpr.invars):
            if b is not None and b.size:
                b.tensor.upload(_device_words_of_argument(x, var.aval))

    def replay(self, iters: int = 1) -> float:
        '''Run only the kernels of the recorded sequence `iters` times on whatever the input
        buffers hold; returns the elapsed device time in milliseconds.'''
        return self.sequence.replay(iters)

    def read_outputs(self):
        return tuple(b.numpy() if b is not None else None for b in self.output_buffers)

    def get_profiling_info(self):
        timestamps = self.sequence.get_timestamps()
        deltas     = np.diff(timestamps)
        labels     = ['data2device'] + [op.equation for op in self.all_ops] + ['data2host']
        return list(zip(labels, deltas))


#kinds of resident leaves: identified by the object alone, or by the object and a fingerprint of its memory
RESIDENT, RESIDENT_CHECKED = 1, 2


def _is_immutable(leaf) -> bool:
    '''True for an argument leaf whose values cannot change while the caller holds it: a numpy array that is not
    writeable and does not look into a writeable one (or into anything but another array or a bytes object), or
    an array of jax.'''
    if type(leaf) is np.ndarray:
        while type(leaf) is np.ndarray:
            if leaf.flags.writeable:
                return False
            leaf = leaf.base
        return leaf is None or type(leaf) is bytes
    module = type(leaf).__module__
    return module.startswith('jaxlib') or module.startswith('jax.')


def _may_change_in_place(leaf) -> bool:
    return isinstance(leaf, np.ndarray) and not _is_immutable(leaf)


def _fingerprint(x: np.ndarray, words: np.ndarray):
    '''What a cheap look at a writeable array can tell about a change in place: its first and last 64 bytes (the
    object, and with it shape and element type, is compared by the caller).'''
    return (words[:16].tobytes(), words[-16:].tobytes())


def _device_words_of_argument(x, aval) -> np.ndarray:
    shape, dtype = core.physical(aval)
    if core.is_key_dtype(getattr(x, 'dtype', None)):
        #a typed key array of jax: its uint32 words are what the device holds
        import jax
        x = jax.random.key_data(x)
    words = to_device_words(np.asarray(x), dtype)
    if words.size != int(np.prod(shape, dtype=np.int64)):
        raise TypeError(f'argument of shape {np.shape(x)} does not match the traced shape {shape}')
    return words


def get_maximum_workgroup_size(mgr) -> int:
    devprops = mgr.get_device_properties()
    return min(devprops['max_work_group_invocations'], devprops['max_work_group_size'][0])
