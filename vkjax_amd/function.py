'''`wrap` / `Function`: trace a Python function once per argument signature and run it on the
device. Same behaviour as the reference (vkjax/function.py:7-47): the interpreter cache is
keyed by (shapes, numpy dtypes, tree structure) of the flattened arguments, outputs are
reshaped to the traced shapes and re-nested, `profiling=True` returns `(output, profiling_info)`.

Tracing uses `jax.make_jaxpr` when jax can be imported and the stand-in tracer of
`vkjax_amd.minijax` otherwise; a function written for one front-end must be traced with that one.
'''
import collections
import queue
import threading
import typing as tp

import numpy as np

from . import minijax
from .jaxpr_interpreter import JaxprInterpreter
from .minijax import core, tree_util


def _pick_frontend(frontend: tp.Optional[str]):
    if frontend in (None, 'auto'):
        try:
            import jax    # noqa: F401
            frontend = 'jax'
        except ImportError:
            frontend = 'minijax'
    if frontend == 'jax':
        import jax
        return jax.make_jaxpr, jax.tree_util
    if frontend == 'minijax':
        return minijax.make_jaxpr, tree_util
    raise ValueError(f'unknown frontend {frontend}')


class _Ahead:
    '''Iterates over `prepare(item) for item in iterable`, with the iterable and `prepare` running on
    a helper thread that stays up to two items ahead of the consumer. An exception raised there is
    raised again in the consumer; close() lets the helper go when the consumer stops early.'''

    def __init__(self, iterable, prepare, wake: tp.Optional[threading.Event] = None):
        self._iterable, self._prepare, self._wake = iterable, prepare, wake
        self._queue   = queue.Queue(maxsize=1)
        self._closed  = threading.Event()
        self._thread  = threading.Thread(target=self._work, name='vkjax-stream-ahead', daemon=True)
        self._thread.start()

    def _put(self, entry) -> bool:
        while not self._closed.is_set():
            try:
                self._queue.put(entry, timeout=0.05)
                return True
            except queue.Full:
                pass
        return False

    def _work(self):
        try:
            for item in self._iterable:
                if self._closed.is_set() or not self._put(('item', self._prepare(item))):
                    return
            self._put(('end', None))
        except BaseException as error:      # noqa: B902 - handed to the consumer
            self._put(('error', error))

    def __iter__(self):
        while True:
            kind, value = self._queue.get()
            if kind == 'end':
                return
            if kind == 'error':
                raise value
            yield value

    def close(self):
        self._closed.set()
        if self._wake is not None:
            self._wake.set()               #a helper waiting for the consumer must see the close


#Tracing (the stand-in tracer keeps its state in module globals) and the recording of a program happen one at a time,
#whichever thread asks
_TRACE_LOCK = threading.RLock()


class Function:
    def __init__(self, function: tp.Callable, static_argnums: tp.Tuple[int, ...] = (), profiling: bool = False,
                 *args, frontend: tp.Optional[str] = None, **kwargs):
        #what another Function over the same program on another device context is built from (stream(in_flight=...))
        self._made_from          = (function, tuple(static_argnums), args, dict(kwargs, frontend=frontend))
        self._in_flight_lanes: tp.List['Function'] = []
        make_jaxpr, self._tree   = _pick_frontend(frontend)
        self.jaxpr_function      = make_jaxpr(function, static_argnums, return_shape=True)
        self._jaxpr_interpreters = dict()
        self._output_shapes      = dict()
        self._profiling          = profiling
        self._static_argnums     = tuple(static_argnums)
        kwargs['profiling']      = profiling
        kwargs['static_argnums'] = static_argnums
        self._interpreter_args   = (args, kwargs)

    def __call__(self, *args: tp.Any, **kwargs: tp.Any) -> tp.Any:
        if self._tree is tree_util and not kwargs:
            #the arguments are flattened once, for the cache key and for the run
            leaves, structure = tree_util.tree_flatten(args)
            jaxpr_interpreter, output_shapes = self._get_or_create_jaxpr_interpreter(args, (leaves, structure))
            per_argument, at = [], 0
            for child in structure.children:
                per_argument.append(leaves[at:at + child.num_leaves])
                at += child.num_leaves
            output = jaxpr_interpreter.run_leaves(per_argument)
        else:
            jaxpr_interpreter, output_shapes = self._get_or_create_jaxpr_interpreter(args)
            output = jaxpr_interpreter.run(*args, **kwargs)
        output = self._restore_shapes(output, output_shapes)
        if not self._profiling:
            return output
        return output, jaxpr_interpreter.get_profiling_info()

    def stream(self, argument_tuples: tp.Iterable[tp.Tuple], in_flight: int = 1) -> tp.Iterator[tp.Any]:
        '''`(self(*args) for args in argument_tuples)` with the host work and the upload for each
        tuple overlapping the device work on the one before it: a helper thread takes the tuples
        from the iterable and flattens and converts their arguments while the calling thread waits
        for the device; the runtime stages and uploads them during the preceding evaluation.
        A tuple whose signature differs from its predecessor's is uploaded in its own turn.
        Arrays may be refilled by the caller as soon as the iterable is asked for the next tuple (their
        contents are copied when a tuple is taken), except those of `resident_argnums`.

        `in_flight` > 1: that many tuples are on the device at the same time. Each is evaluated by a lane of its own - a
        device context with its own streams, buffers and copy of the resident arguments, driven by its own thread -
        and the lanes take the tuples from the iterable in turn; results come back in the order of the tuples. The
        launches of one evaluation still run one after the other; what the GPU gains is that the start and the tail
        of one lane's launches are covered by the other lane's work (ResNet-50 at batch 64: two lanes finish a batch
        every 4.6 ms against 4.9 ms for one). The latency of a single result grows accordingly.

        No counterpart in the reference, whose calls copy, run and read back in turn
        (vkjax/kompute_jaxpr_interpreter.py:72-81).'''
        if self._profiling:
            raise ValueError('stream() does not collect profiling information; call the function instead')
        if int(in_flight) > 1:
            yield from self._stream_in_flight(argument_tuples, int(in_flight))
        else:
            yield from self._stream_one(argument_tuples)

    def _stream_in_flight(self, argument_tuples: tp.Iterable[tp.Tuple], lanes: int) -> tp.Iterator[tp.Any]:
        from . import hip
        function, static_argnums, args, kwargs = self._made_from
        while len(self._in_flight_lanes) < lanes:
            #(none of the lanes is this object: its context stays free for calls from the consumer's thread)
            device = hip.Device(hip.Device.get().index)
            self._in_flight_lanes.append(Function(function, static_argnums, False, *args, **dict(kwargs, device=device)))
        source      = iter(argument_tuples)
        source_lock = threading.Lock()
        holder      = [None]                               #the lane whose helper thread holds source_lock
        taken       = [0]                                  #tuples taken from the iterable so far
        orders      = [collections.deque() for _ in range(lanes)]      #per lane: the numbers of its tuples, in order
        stop        = threading.Event()
        #at most this many tuples between the iterable and the consumer, so that a lane that falls behind holds the
        #others back instead of letting their results pile up
        slots       = threading.Semaphore(4 * lanes)
        results     = queue.Queue(maxsize=2 * lanes)

        def release_source(k):
            if holder[0] == k:
                holder[0] = None
                source_lock.release()

        def share(k):
            '''Lane k's part of the iterable. Runs on the lane's helper thread; the lock is held from asking the iterable
            for a tuple until the lane has copied what the caller may refill (see _stream_one), so that the iterable is
            never asked for the next tuple before that.'''
            try:
                while not stop.is_set():
                    if not slots.acquire(timeout=0.05):
                        continue
                    source_lock.acquire()
                    holder[0] = k
                    if stop.is_set():
                        slots.release()
                        return
                    try:
                        item = next(source)
                    except StopIteration:
                        slots.release()
                        return
                    orders[k].append(taken[0])
                    taken[0] += 1
                    yield item
            finally:
                release_source(k)

        def put(entry) -> bool:
            while not stop.is_set():
                try:
                    results.put(entry, timeout=0.05)
                    return True
                except queue.Full:
                    pass
            return False

        def work(k):
            outputs = self._in_flight_lanes[k]._stream_one(share(k), taken=lambda: release_source(k))
            try:
                for output in outputs:
                    if not put(('result', orders[k].popleft(), output)):
                        break
            except BaseException as error:      # noqa: B902 - handed to the consumer
                put(('error', k, error))
            finally:
                outputs.close()
                put(('done', k, None))

        threads = [threading.Thread(target=work, args=(k,), name=f'vkjax-stream-lane-{k}', daemon=True) for k in range(lanes)]
        for t in threads:
            t.start()
        ready, number, done = {}, 0, 0
        try:
            while True:
                while number in ready:
                    output = ready.pop(number)
                    number += 1
                    slots.release()
                    yield output
                if done == lanes:
                    return
                kind, key, value = results.get()
                if kind == 'error':
                    raise value
                if kind == 'done':
                    done += 1
                else:
                    ready[key] = value
        finally:
            stop.set()
            for t in threads:
                t.join()

    def _stream_one(self, argument_tuples: tp.Iterable[tp.Tuple], taken: tp.Optional[tp.Callable[[], None]] = None) -> tp.Iterator[tp.Any]:
        '''stream() on this object's own device context. `taken`, if given, is called on the helper thread once a
        tuple's arrays have been copied as far as they have to be, i.e. when the iterable may be asked for the next.'''
        # Tracing and recording stay on the calling thread (a device context is used by one thread at
        # a time). When the helper meets a signature that has no interpreter yet, it hands the tuple
        # over as it is and prepares nothing further until the calling thread has dealt with it,
        # so that what each prepared tuple assumes to be resident in HBM holds when it runs.
        caught_up = threading.Event()
        caught_up.set()

        # A tuple is taken from the iterable up to four evaluations before its arguments are staged, and a
        # loader may refill the arrays it has handed out (one batch array, or a small ring of them) as soon as
        # it is asked for the next tuple. Argument leaves that would be passed on as views of the caller's
        # arrays are therefore copied when the tuple is taken, into one of RING arrays kept per leaf: at most
        # that many tuples are between the iterable and the end of their upload at any time (one being
        # prepared, one queued, the following one, the current one). Resident leaves are identified by the
        # object passed and are not copied: their contract is that the array stays as it is.
        RING = 4
        rings: tp.Dict[tp.Tuple[int, int], tp.List] = {}

        def owned(interpreter, converted):
            result = []
            for k, slot, x, words, is_resident in converted:
                if not is_resident and isinstance(x, np.ndarray) and np.may_share_memory(words, x):
                    ring = rings.setdefault((id(interpreter), k), [0, [None] * RING])
                    position = ring[0] % RING
                    ring[0] += 1
                    if ring[1][position] is None:
                        ring[1][position] = np.empty_like(words)
                    np.copyto(ring[1][position], words)
                    words = ring[1][position]
                result.append((k, slot, x, words, is_resident))
            return result

        def prepare(args):
            try:
                return prepare_taken(args)
            finally:
                if taken is not None:
                    taken()

        def prepare_taken(args):
            caught_up.wait()
            args      = tuple(args)                  #what __call__ sees as *args
            signature = self._signature(args)
            entry     = self._jaxpr_interpreters.get(signature)
            if entry is None:
                caught_up.clear()
                #traced and recorded by the calling thread, later: the arrays are copied now, as above
                resident = self._interpreter_args[1].get('resident_argnums', ())
                copy = lambda leaf: np.array(leaf) if isinstance(leaf, np.ndarray) else leaf
                args = tuple(a if i in resident or i in self._static_argnums else self._tree.tree_map(copy, a)
                             for i, a in enumerate(args))
                return [None, None, args]
            return [entry, self._output_shapes[signature], owned(entry, entry._convert_inputs(args))]

        def resolved(item):
            if item is not None and item[0] is None:
                interpreter, output_shapes = self._get_or_create_jaxpr_interpreter(item[2])
                item[:] = [interpreter, output_shapes, owned(interpreter, interpreter._convert_inputs(item[2]))]
                caught_up.set()
            return item

        ahead = _Ahead(argument_tuples, prepare, wake=caught_up)
        try:
            # The helper only converts arguments. Which of them have to be copied (resident ones that changed) is
            # settled here, immediately before the evaluation that copies them, so that what the interpreter notes as
            # held in HBM is true at every point where the consumer may stop or call the function in between.
            items   = iter(ahead)
            current = resolved(next(items, None))
            in_place = False                                     #current's arguments were uploaded by the previous evaluation
            while current is not None:
                interpreter, output_shapes, converted = current
                if in_place and interpreter._evaluations != stamp:
                    in_place = False                             #something else used the argument buffers in between
                host      = [None] * interpreter.sequence.n_slots if in_place else interpreter._select_uploads(converted)
                following = resolved(next(items, None))
                overlap   = following is not None and following[0] is interpreter
                next_host = interpreter._select_uploads(following[2]) if overlap else None
                fresh     = interpreter._fresh_outputs(host)
                interpreter.evaluate(host, next_host)
                stamp, in_place = interpreter._evaluations, overlap
                yield self._restore_shapes(interpreter._output_values(fresh), output_shapes)
                current = following
        finally:
            ahead.close()

    def _signature(self, args: tp.Tuple[tp.Any, ...], flattened=None):
        leaves, structure = flattened or self._tree.tree_flatten(args)
        array             = np.ndarray
        args_shape        = tuple(x.shape if type(x) is array else np.shape(x) for x in leaves)
        args_dtype        = tuple(x.dtype if type(x) is array else np.asarray(x).dtype if not hasattr(x, 'dtype') else np.dtype(x.dtype)
                                  for x in leaves)
        static_values     = tuple(repr(args[i]) for i in self._static_argnums if i < len(args))
        return (args_shape, args_dtype, structure, static_values)

    def _get_or_create_jaxpr_interpreter(self, args: tp.Tuple[tp.Any, ...], flattened=None):
        shape_structure = self._signature(args, flattened)
        if shape_structure not in self._jaxpr_interpreters:
            #new input shapes or structure, need to re-trace
            with _TRACE_LOCK:
                jaxpr, output_shapes = self.jaxpr_function(*args)
                iargs, ikwargs       = self._interpreter_args
                self._jaxpr_interpreters[shape_structure] = JaxprInterpreter(jaxpr, *iargs, **ikwargs)
                self._output_shapes[shape_structure]      = output_shapes
        return self._jaxpr_interpreters[shape_structure], self._output_shapes[shape_structure]

    def _restore_shapes(self, x, targetshapes):
        structure = self._tree.tree_structure(targetshapes)
        x         = self._tree.tree_unflatten(structure, x)
        #typed PRNG keys come back as their uint32 words, with the key's words as a trailing dimension
        def restore(a, shapestruct):
            a = np.asarray(a)
            return a if core.is_key_dtype(shapestruct.dtype) else a.reshape(shapestruct.shape)
        return self._tree.tree_map(restore, x, targetshapes)


def wrap(function: tp.Callable, *args, **kwargs) -> Function:
    '''`vkjax.wrap` (reference: vkjax/function.py:46-47): `wrap(f, static_argnums=(), profiling=False)(*args)` traces
    `f` for the arguments' signature and runs it on the device.

    Arguments are copied to the device on every call, as the reference does, with two exceptions that save the
    copy of weights and tables: leaves that cannot change while the caller holds them (numpy arrays with
    `flags.writeable == False`, jax arrays) are uploaded once and again only when another object is passed in their
    place; and `resident_argnums=(i, ...)` declares the same for every leaf of those arguments, writeable or not -
    an in-place change of such a writeable array is noticed only if it touches its first or last 64 bytes, so pass a
    new array for new values. Further keyword arguments: `frontend` ('jax', 'minijax', default:
    jax where importable), `fuse`, `reuse_buffers`, `graph`.'''
    return Function(function, *args, **kwargs)
