'''`wrap` / `Function`: trace a Python function once per argument signature and run it on the
device. Same behaviour as the reference (vkjax/function.py:7-47): the interpreter cache is
keyed by (shapes, numpy dtypes, tree structure) of the flattened arguments, outputs are
reshaped to the traced shapes and re-nested, `profiling=True` returns `(output, profiling_info)`.

Tracing uses `jax.make_jaxpr` when jax can be imported and the stand-in tracer of
`vkjax_amd.minijax` otherwise; a function written for one front-end must be traced with that one.
'''
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


class Function:
    def __init__(self, function: tp.Callable, static_argnums: tp.Tuple[int, ...] = (), profiling: bool = False,
                 *args, frontend: tp.Optional[str] = None, **kwargs):
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

    def stream(self, argument_tuples: tp.Iterable[tp.Tuple]) -> tp.Iterator[tp.Any]:
        '''`(self(*args) for args in argument_tuples)` with the host work and the upload for each
        tuple overlapping the device work on the one before it: a helper thread takes the tuples
        from the iterable and flattens and converts their arguments while the calling thread waits
        for the device; the runtime stages and uploads them during the preceding evaluation.
        A tuple whose signature differs from its predecessor's is uploaded in its own turn.
        Arrays may be refilled by the caller as soon as the iterable is asked for the next tuple (their
        contents are copied when a tuple is taken), except those of `resident_argnums`.
        No counterpart in the reference, whose calls copy, run and read back in turn
        (vkjax/kompute_jaxpr_interpreter.py:72-81).'''
        if self._profiling:
            raise ValueError('stream() does not collect profiling information; call the function instead')
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
