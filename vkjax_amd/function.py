'''`wrap` / `Function`: trace a Python function once per argument signature and run it on the
device. Same behaviour as the reference (vkjax/function.py:7-47): the interpreter cache is
keyed by (shapes, numpy dtypes, tree structure) of the flattened arguments, outputs are
reshaped to the traced shapes and re-nested, `profiling=True` returns `(output, profiling_info)`.

Tracing uses `jax.make_jaxpr` when jax can be imported and the stand-in tracer of
`vkjax_amd.minijax` otherwise; a function written for one front-end must be traced with that one.
'''
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
        jaxpr_interpreter, output_shapes = self._get_or_create_jaxpr_interpreter(args)
        output = jaxpr_interpreter.run(*args, **kwargs)
        output = self._restore_shapes(output, output_shapes)
        if not self._profiling:
            return output
        return output, jaxpr_interpreter.get_profiling_info()

    def _get_or_create_jaxpr_interpreter(self, args: tp.Tuple[tp.Any, ...]):
        leaves, structure = self._tree.tree_flatten(args)
        args_shape        = tuple(np.shape(x) for x in leaves)
        args_dtype        = tuple(np.asarray(x).dtype if not hasattr(x, 'dtype') else np.dtype(x.dtype) for x in leaves)
        static_values     = tuple(repr(args[i]) for i in self._static_argnums if i < len(args))
        shape_structure   = (args_shape, args_dtype, structure, static_values)
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
    return Function(function, *args, **kwargs)
