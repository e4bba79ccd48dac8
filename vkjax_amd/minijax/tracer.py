'''A small tracing front-end: the stand-in for `jax.make_jaxpr` on machines where
jax cannot be imported (reference call site: vkjax/function.py:9).

`make_jaxpr(f)(*args)` runs `f` on `Tracer` objects; every `lax` call appends one
equation to the innermost active `Trace`. Nothing is computed here.
'''
import typing as tp

import numpy as np

from . import core
from . import tree_util


class Trace:
    def __init__(self, parent: tp.Optional['Trace'] = None):
        self.parent    = parent
        self.eqns      = []
        self.constvars = []
        self.consts    = []
        self._const_ids: tp.Dict[int, core.Var] = {}

    def new_const(self, value: np.ndarray) -> core.Var:
        key = id(value)
        if key not in self._const_ids:
            value = np.asarray(value)
            aval  = core.ShapedArray(value.shape, core.canonicalize_dtype(value.dtype))
            var   = core.Var(None, '', aval)
            self._const_ids[key] = var
            self.constvars.append(var)
            self.consts.append(np.asarray(value, dtype=aval.dtype))
            #keep the object alive so its id stays unique for the life of the trace
            self._keepalive = getattr(self, '_keepalive', []) + [value]
        return self._const_ids[key]


_trace_stack: tp.List[Trace] = []


def current_trace() -> Trace:
    if not _trace_stack:
        raise RuntimeError('lax operations can only be used inside a function passed to '
                           'vkjax_amd.wrap / make_jaxpr')
    return _trace_stack[-1]


def _python_scalar_kind(x):
    if isinstance(x, (bool, np.bool_)):
        return 'bool'
    if isinstance(x, int):
        return 'int'
    if isinstance(x, float):
        return 'float'
    return None


_WEAK_DEFAULT = {'bool': np.dtype('bool'), 'int': np.dtype('int32'), 'float': np.dtype('float32')}
_CATEGORY     = {np.dtype('bool'): 0, np.dtype('int32'): 1, np.dtype('uint32'): 1, np.dtype('float32'): 2}
_KIND_CAT     = {'bool': 0, 'int': 1, 'float': 2}


def dtype_of(x) -> tp.Tuple[np.dtype, bool]:
    '''(canonical dtype, weak?) of a tracer, python scalar or array-like.'''
    if isinstance(x, Tracer):
        return x.aval.dtype, x.aval.weak_type
    kind = _python_scalar_kind(x)
    if kind is not None and not isinstance(x, np.generic):
        return _WEAK_DEFAULT[kind], True
    return core.canonicalize_dtype(np.asarray(x).dtype), False


def result_dtype(*xs) -> np.dtype:
    '''JAX-style promotion with x64 disabled over {bool, int32, uint32, float32};
    python scalars are weak: they only lift the category, never the width.'''
    strong = [d for d, w in map(dtype_of, xs) if not w]
    weak   = [d for d, w in map(dtype_of, xs) if w]

    def join(a, b):
        if a == b:
            return a
        ca, cb = _CATEGORY[a], _CATEGORY[b]
        if ca != cb:
            return a if ca > cb else b
        return np.dtype('int32')      #int32 with uint32

    if not strong:
        out = weak[0]
        for d in weak[1:]:
            out = join(out, d)
        return out
    out = strong[0]
    for d in strong[1:]:
        out = join(out, d)
    for d in weak:
        if _CATEGORY[d] > _CATEGORY[out]:
            out = d
    return out


class Tracer:
    __array_priority__ = 1000

    def __init__(self, trace: Trace, var: core.Var):
        self._trace = trace
        self._var   = var

    @property
    def aval(self) -> core.ShapedArray:
        return self._var.aval

    @property
    def shape(self):
        return self.aval.shape

    @property
    def dtype(self):
        return self.aval.dtype

    @property
    def ndim(self):
        return len(self.aval.shape)

    @property
    def size(self):
        return self.aval.size

    def __len__(self):
        if not self.shape:
            raise TypeError('len() of a scalar tracer')
        return self.shape[0]

    def __repr__(self):
        return f'Tracer<{self.aval}>'

    def __bool__(self):
        raise TypeError('the truth value of a traced array is not available at trace time')

    def __iter__(self):
        if not self.shape:
            raise TypeError('iteration over a scalar tracer')
        return (self[i] for i in range(self.shape[0]))

    #arithmetic is routed through the numpy-like layer, which applies dtype/rank promotion
    def _np(self):
        from . import numpy as mnp
        return mnp

    def __add__(self, o):      return self._np().add(self, o)
    def __radd__(self, o):     return self._np().add(o, self)
    def __sub__(self, o):      return self._np().subtract(self, o)
    def __rsub__(self, o):     return self._np().subtract(o, self)
    def __mul__(self, o):      return self._np().multiply(self, o)
    def __rmul__(self, o):     return self._np().multiply(o, self)
    def __truediv__(self, o):  return self._np().true_divide(self, o)
    def __rtruediv__(self, o): return self._np().true_divide(o, self)
    def __mod__(self, o):      return self._np().remainder(self, o)
    def __pow__(self, o):      return self._np().power(self, o)
    def __neg__(self):         return self._np().negative(self)
    def __abs__(self):         return self._np().abs(self)
    def __matmul__(self, o):   return self._np().matmul(self, o)
    def __rmatmul__(self, o):  return self._np().matmul(o, self)
    def __gt__(self, o):       return self._np().greater(self, o)
    def __ge__(self, o):       return self._np().greater_equal(self, o)
    def __lt__(self, o):       return self._np().less(self, o)
    def __le__(self, o):       return self._np().less_equal(self, o)
    def __eq__(self, o):       return self._np().equal(self, o)
    def __ne__(self, o):       return self._np().not_equal(self, o)
    def __or__(self, o):       return self._np().bitwise_or(self, o)
    def __ror__(self, o):      return self._np().bitwise_or(o, self)
    def __and__(self, o):      return self._np().bitwise_and(self, o)
    def __rand__(self, o):     return self._np().bitwise_and(o, self)
    def __lshift__(self, o):   return self._np().left_shift(self, o)
    def __rshift__(self, o):   return self._np().right_shift(self, o)
    __hash__ = object.__hash__

    def __getitem__(self, idx):
        return self._np().getitem(self, idx)

    @property
    def T(self):
        return self._np().transpose(self)

    @property
    def at(self):
        return self._np().IndexUpdateHelper(self)

    def reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        return self._np().reshape(self, shape)

    def astype(self, dtype):
        return self._np().astype(self, dtype)

    def ravel(self):
        return self._np().reshape(self, (-1,))

    def squeeze(self, axis=None):
        return self._np().squeeze(self, axis)

    def transpose(self, *axes):
        if len(axes) == 1 and isinstance(axes[0], (tuple, list)):
            axes = tuple(axes[0])
        return self._np().transpose(self, axes or None)

    def sum(self, axis=None, keepdims=False):    return self._np().sum(self, axis, keepdims=keepdims)
    def mean(self, axis=None, keepdims=False):   return self._np().mean(self, axis, keepdims=keepdims)
    def max(self, axis=None, keepdims=False):    return self._np().max(self, axis, keepdims=keepdims)
    def min(self, axis=None, keepdims=False):    return self._np().min(self, axis, keepdims=keepdims)
    def prod(self, axis=None, keepdims=False):   return self._np().prod(self, axis, keepdims=keepdims)
    def argmax(self, axis=None):                 return self._np().argmax(self, axis)
    def argmin(self, axis=None):                 return self._np().argmin(self, axis)


def to_invar(x, dtype: tp.Optional[np.dtype] = None) -> tp.Union[core.Var, core.Literal]:
    '''Turn an operand into something an equation can reference: a tracer's variable,
    a Literal for scalars, or a constant variable for arrays closed over by the function.'''
    trace = current_trace()
    if isinstance(x, Tracer):
        if x._trace is not trace:
            raise NotImplementedError('a traced value from an enclosing function cannot be used '
                                      'inside a nested jit; pass it as an argument instead')
        return x._var
    arr = np.asarray(x)
    if dtype is None:
        dtype = dtype_of(x)[0]
    if arr.ndim == 0:
        val = np.asarray(arr, dtype=dtype)[()]
        return core.Literal(val, core.ShapedArray((), dtype, weak_type=dtype_of(x)[1]))
    if arr.dtype != dtype:
        arr = arr.astype(dtype)
    return trace.new_const(arr if arr is not x else x)


def emit(name: str, operands: tp.Sequence, out_avals: tp.Sequence[core.ShapedArray],
         params: tp.Optional[dict] = None, multiple_results: bool = False):
    '''Append `outs = name[params] operands` to the current trace.'''
    trace   = current_trace()
    invars  = [to_invar(x) for x in operands]
    outvars = [core.Var(None, '', aval) for aval in out_avals]
    trace.eqns.append(core.JaxprEqn(invars, outvars, core.Primitive(name, multiple_results), dict(params or {})))
    outs = [Tracer(trace, v) for v in outvars]
    return outs if multiple_results else outs[0]


def _abstractify(x) -> core.ShapedArray:
    dtype, weak = dtype_of(x)
    return core.ShapedArray(np.shape(x), dtype, weak_type=weak)


def _trace_to_jaxpr(fun, in_avals: tp.Sequence[core.ShapedArray], in_tree, static: dict, nargs: int):
    '''Run `fun` on tracers. Returns (Jaxpr, consts, out_tree, out_avals).'''
    trace = Trace(_trace_stack[-1] if _trace_stack else None)
    _trace_stack.append(trace)
    try:
        invars  = [core.Var(None, '', aval) for aval in in_avals]
        tracers = [Tracer(trace, v) for v in invars]
        dyn     = iter(tree_util.tree_unflatten(in_tree, tracers))
        args    = [static[i] if i in static else next(dyn) for i in range(nargs)]
        out     = fun(*args)
        out_leaves, out_tree = tree_util.tree_flatten(out)
        outvars = []
        for leaf in out_leaves:
            if not isinstance(leaf, Tracer):
                #a constant output: materialise it through a (free) view of a literal/const
                from . import lax
                leaf = lax.convert_element_type(leaf, dtype_of(leaf)[0], force=True)
            outvars.append(leaf._var)
        jaxpr = core.Jaxpr(trace.constvars, invars, outvars, trace.eqns)
        return jaxpr, trace.consts, out_tree, [v.aval for v in outvars]
    finally:
        _trace_stack.pop()


def make_jaxpr(fun: tp.Callable, static_argnums: tp.Iterable[int] = (), return_shape: bool = False):
    '''Same calling convention as jax.make_jaxpr.'''
    static_argnums = tuple(static_argnums) if not isinstance(static_argnums, int) else (static_argnums,)

    def jaxpr_maker(*args):
        static  = {i: a for i, a in enumerate(args) if i in static_argnums}
        dynamic = tuple(a for i, a in enumerate(args) if i not in static_argnums)
        leaves, in_tree = tree_util.tree_flatten(dynamic)
        in_avals = [core.ShapedArray(a.shape, a.dtype) for a in map(_abstractify, leaves)]
        jaxpr, consts, out_tree, out_avals = _trace_to_jaxpr(fun, in_avals, in_tree, static, len(args))
        closed = core.ClosedJaxpr(jaxpr, consts)
        if not return_shape:
            return closed
        shapes = tree_util.tree_unflatten(out_tree, [core.ShapeDtypeStruct(a.shape, a.dtype) for a in out_avals])
        return closed, shapes

    return jaxpr_maker


def _call_nested(fun, primitive_name: str, jaxpr_param: str, extra_params: dict, closed: bool, args):
    '''Trace `fun` into an inner jaxpr and emit one call equation that carries it.
    Constants the inner function closes over become leading arguments of the call.'''
    leaves, in_tree = tree_util.tree_flatten(tuple(args))
    in_avals = [core.ShapedArray(a.shape, a.dtype) for a in map(_abstractify, leaves)]
    jaxpr, consts, out_tree, out_avals = _trace_to_jaxpr(fun, in_avals, in_tree, {}, len(args))
    inner = core.Jaxpr([], list(jaxpr.constvars) + list(jaxpr.invars), jaxpr.outvars, jaxpr.eqns)
    params = dict(extra_params)
    params[jaxpr_param] = core.ClosedJaxpr(inner, []) if closed else inner
    outs = emit(primitive_name, list(consts) + list(leaves), out_avals, params, multiple_results=True)
    return tree_util.tree_unflatten(out_tree, outs)


def jit(fun: tp.Callable):
    '''Inside a trace: emits `xla_call` with the function's own jaxpr (the form the
    reference inlines, vkjax/ops.py:218-244). Outside a trace it just returns `fun`'s tracing wrapper.'''
    def wrapped(*args):
        params = dict(device=None, backend=None, name=getattr(fun, '__name__', 'fn'), donated_invars=(False,) * 0)
        return _call_nested(fun, 'xla_call', 'call_jaxpr', params, closed=False, args=args)
    wrapped.__name__ = getattr(fun, '__name__', 'jit_fn')
    return wrapped


def custom_jvp(fun: tp.Callable):
    '''Emits `custom_jvp_call_jaxpr` (what jax.nn.relu looks like in a jaxpr of that era;
    reference: vkjax/ops.py:246-260). A derivative rule can be attached with `.defvjp(rule)`,
    `rule(cotangent, result, *arguments) -> cotangents of the arguments`; reverse-mode
    differentiation then uses it instead of differentiating the body (the entry `jvp_jaxpr_thunk`
    of the equation carries it; backends ignore that entry).'''
    def wrapped(*args):
        params = dict(num_consts=0, jvp_jaxpr_thunk=wrapped.vjp_rule)
        return _call_nested(fun, 'custom_jvp_call_jaxpr', 'fun_jaxpr', params, closed=True, args=args)
    wrapped.__name__ = getattr(fun, '__name__', 'custom_jvp_fn')
    wrapped.vjp_rule = None
    def defvjp(rule):
        wrapped.vjp_rule = rule
        return rule
    wrapped.defvjp = defvjp
    return wrapped
