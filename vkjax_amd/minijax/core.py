'''Minimal jaxpr data model.

The interpreter and the primitive dispatch only read a handful of attributes from a
traced program: `eqn.primitive.name`, `eqn.params`, `eqn.invars/outvars`,
`var.aval.shape/dtype`, `literal.val`, `jaxpr.invars/outvars/constvars/eqns`,
`closed.jaxpr/consts` (reference: vkjax/ops.py:52-65, vkjax/buffers.py:99-127,
vkjax/kompute_jaxpr_interpreter.py:27-63). The classes here carry exactly those
attribute names, so a program traced by real `jax.make_jaxpr` and one traced by the
stand-in tracer in this package drive the same dispatch code.
'''
import itertools
import typing as tp

import numpy as np


#dtypes that exist on the device (everything is 32 bits wide, reference: vkjax/buffers.py:68-77)
DEVICE_DTYPES = (np.dtype('bool'), np.dtype('int32'), np.dtype('uint32'), np.dtype('float32'))


def canonicalize_dtype(dtype) -> np.dtype:
    '''64-bit host types are narrowed the way JAX does with x64 disabled.'''
    dtype = np.dtype(dtype)
    if dtype == np.float64 or dtype == np.float16:
        return np.dtype('float32')
    if dtype in (np.dtype('int64'), np.dtype('int16'), np.dtype('int8')):
        return np.dtype('int32')
    if dtype in (np.dtype('uint64'), np.dtype('uint16'), np.dtype('uint8')):
        return np.dtype('uint32')
    if dtype not in DEVICE_DTYPES:
        raise NotImplementedError(f'{dtype} data types currently not supported')
    return dtype


class KeyTy:
    '''Element type of typed PRNG key arrays (jax prints it as `key<fry>`): one element is a
    whole threefry key, stored as `key_shape` trailing uint32 words. Newer jax versions route
    `jax.random` through the primitives random_wrap / random_bits / random_split / ... whose
    operands carry this type.'''
    name      = 'key<fry>'
    key_shape = (2,)
    impl_name = 'threefry2x32'

    def __eq__(self, other):
        return type(other).__name__ == 'KeyTy' and key_words_shape(other) == self.key_shape

    def __hash__(self):
        return hash(self.name)

    def __repr__(self):
        return self.name


key_fry = KeyTy()


def is_key_dtype(dtype) -> bool:
    '''True for KeyTy above and for jax's own key element type (matched by class name).'''
    return type(dtype).__name__ == 'KeyTy'


def key_words_shape(dtype) -> tp.Tuple[int, ...]:
    '''Trailing uint32 words of one key. Only the threefry implementation is supported.'''
    impl = getattr(dtype, '_impl', dtype)
    name = getattr(impl, 'name', None) if impl is not dtype else dtype.impl_name
    if name != 'threefry2x32':
        raise NotImplementedError(f'PRNG implementation {name}: only threefry2x32 keys are supported')
    return tuple(impl.key_shape)


def physical(aval) -> tp.Tuple[tp.Tuple[int, ...], np.dtype]:
    '''(shape, dtype) of the device array that holds a value of this abstract type.'''
    if is_key_dtype(aval.dtype):
        return tuple(aval.shape) + key_words_shape(aval.dtype), np.dtype('uint32')
    return tuple(aval.shape), canonicalize_dtype(aval.dtype)


class ShapedArray:
    __slots__ = ('shape', 'dtype', 'weak_type')

    def __init__(self, shape, dtype, weak_type=False):
        self.shape     = tuple(int(s) for s in shape)
        self.dtype     = dtype if is_key_dtype(dtype) else np.dtype(dtype)
        self.weak_type = bool(weak_type)

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=np.int64))

    def __eq__(self, other):
        return isinstance(other, ShapedArray) and self.shape == other.shape and self.dtype == other.dtype

    def __hash__(self):
        return hash((self.shape, self.dtype))

    def __repr__(self):
        short = {'float32': 'f32', 'int32': 'i32', 'uint32': 'u32', 'bool': 'bool'}.get(self.dtype.name, self.dtype.name)
        return f'{short}[{",".join(map(str, self.shape))}]'

    def str_short(self):
        return repr(self)


class ShapeDtypeStruct:
    '''What `make_jaxpr(..., return_shape=True)` hands back per output leaf.'''
    __slots__ = ('shape', 'dtype')

    def __init__(self, shape, dtype):
        self.shape = tuple(shape)
        self.dtype = dtype if is_key_dtype(dtype) else np.dtype(dtype)

    def __repr__(self):
        return f'ShapeDtypeStruct(shape={self.shape}, dtype={self.dtype.name})'


_var_counter = itertools.count()


class Var:
    '''A program variable. Hashable by identity, like jax.core.Var.'''
    __slots__ = ('count', 'suffix', 'aval')

    def __init__(self, count: tp.Optional[int], suffix: str, aval: ShapedArray):
        self.count  = next(_var_counter) if count is None else count
        self.suffix = suffix
        self.aval   = aval

    def __repr__(self):
        n, s = self.count, ''
        while True:
            s = chr(ord('a') + n % 26) + s
            n = n // 26 - 1
            if n < 0:
                break
        return s + self.suffix


class DropVar(Var):
    '''An output nobody reads; prints as `_` (the dispatch skips equations whose
    outputs are all dropped, reference: vkjax/ops.py:56-58).'''
    __slots__ = ()

    def __init__(self, aval):
        super().__init__(-1, '', aval)

    def __repr__(self):
        return '_'


class Literal:
    '''A scalar baked into an equation.'''
    __slots__ = ('val', 'aval', 'hash')

    def __init__(self, val, aval: ShapedArray):
        self.val  = val
        self.aval = aval
        #jax literals are unhashable but carry a .hash derived from the value, which the pool keys on,
        #so equal literals share one buffer (reference: vkjax/buffers.py:80-87)
        self.hash = hash((aval.dtype.str, np.asarray(val).tobytes()))

    def __repr__(self):
        return str(self.val)


class Primitive:
    __slots__ = ('name', 'multiple_results')

    def __init__(self, name: str, multiple_results: bool = False):
        self.name             = name
        self.multiple_results = multiple_results

    def __repr__(self):
        return self.name


class JaxprEqn(tp.NamedTuple):
    invars:    tp.List[tp.Union[Var, Literal]]
    outvars:   tp.List[Var]
    primitive: Primitive
    params:    tp.Dict[str, tp.Any]

    def __repr__(self):
        outs   = ' '.join(f'{v}:{v.aval}' for v in self.outvars)
        params = ''
        shown  = {k: v for k, v in self.params.items() if not isinstance(v, (Jaxpr, ClosedJaxpr))}
        if shown:
            params = '[' + ' '.join(f'{k}={v}' for k, v in shown.items()) + ']'
        return f'{outs} = {self.primitive.name}{params} ' + ' '.join(map(repr, self.invars))


class Jaxpr:
    __slots__ = ('constvars', 'invars', 'outvars', 'eqns')

    def __init__(self, constvars, invars, outvars, eqns):
        self.constvars = list(constvars)
        self.invars    = list(invars)
        self.outvars   = list(outvars)
        self.eqns      = list(eqns)

    def __repr__(self):
        head = '{ lambda ' + ' '.join(f'{v}:{v.aval}' for v in self.constvars) + ' ; ' \
             + ' '.join(f'{v}:{v.aval}' for v in self.invars) + ' .'
        body = '\n'.join('    ' + repr(e) for e in self.eqns)
        tail = '  in ( ' + ' '.join(map(repr, self.outvars)) + ' ) }'
        return f'{head}\n  let\n{body}\n{tail}'


class ClosedJaxpr:
    __slots__ = ('jaxpr', 'consts')

    def __init__(self, jaxpr: Jaxpr, consts):
        self.jaxpr  = jaxpr
        self.consts = list(consts)

    @property
    def literals(self):
        return self.consts

    def __repr__(self):
        return repr(self.jaxpr)


class GatherDimensionNumbers(tp.NamedTuple):
    offset_dims:          tp.Tuple[int, ...]
    collapsed_slice_dims: tp.Tuple[int, ...]
    start_index_map:      tp.Tuple[int, ...]


class ScatterDimensionNumbers(tp.NamedTuple):
    update_window_dims:           tp.Tuple[int, ...]
    inserted_window_dims:         tp.Tuple[int, ...]
    scatter_dims_to_operand_dims: tp.Tuple[int, ...]


class ConvDimensionNumbers(tp.NamedTuple):
    '''Each spec lists, for (batch|out-feature, feature|in-feature, spatial0, spatial1),
    which array dimension holds it.'''
    lhs_spec: tp.Tuple[int, ...]
    rhs_spec: tp.Tuple[int, ...]
    out_spec: tp.Tuple[int, ...]


def is_literal(v) -> bool:
    '''True for jax.core.Literal and for the Literal above (both carry `.val`).'''
    return hasattr(v, 'val')


def is_dropped(v) -> bool:
    return str(v) == '_'
