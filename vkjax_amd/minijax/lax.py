'''`lax`-level operations of the stand-in tracer: one function per primitive name the
dispatch accepts (reference: vkjax/ops.py:92-155 and the per-primitive functions
below it). Each function only checks shapes/dtypes, works out the result type and
records an equation; parameter names follow the jaxprs the reference consumed.
'''
import builtins
import typing as tp

import numpy as np

from . import core
from .core import GatherDimensionNumbers, ScatterDimensionNumbers, ConvDimensionNumbers
from .tracer import Tracer, emit, dtype_of, result_dtype, current_trace

_f32, _i32, _u32, _bool = map(np.dtype, ('float32', 'int32', 'uint32', 'bool'))


def _shape(x) -> tp.Tuple[int, ...]:
    return tuple(x.shape) if isinstance(x, Tracer) else tuple(np.shape(x))


def _aval(shape, dtype):
    return core.ShapedArray(shape, dtype)


def _as_dtype(x, dtype):
    '''Operand `x` expressed in `dtype`: scalars/arrays are converted on the host,
    traced values get a convert_element_type equation.'''
    dtype = np.dtype(dtype)
    if isinstance(x, Tracer):
        return x if x.dtype == dtype else convert_element_type(x, dtype)
    arr = np.asarray(x)
    return arr.astype(dtype) if arr.ndim else arr.astype(dtype)[()]


def broadcast_shapes(*shapes):
    shapes = [s for s in shapes if s != ()]
    if not shapes:
        return ()
    rank = builtins.max(len(s) for s in shapes)
    if builtins.any(len(s) != rank for s in shapes):
        raise TypeError(f'lax binary ops need equal ranks (or scalars), got {shapes}')
    out = []
    for dims in zip(*shapes):
        d = builtins.max(dims)
        if builtins.any(x != d and x != 1 for x in dims):
            raise TypeError(f'incompatible shapes for broadcasting: {shapes}')
        out.append(0 if 0 in dims else d)
    return tuple(out)


# ---------------------------------------------------------------- elementwise

def _binary(name, x, y, out_dtype=None, allowed=None):
    dtype = result_dtype(x, y)
    if allowed is not None and dtype not in allowed:
        raise TypeError(f'{name} does not accept {dtype}')
    x, y  = _as_dtype(x, dtype), _as_dtype(y, dtype)
    shape = broadcast_shapes(_shape(x), _shape(y))
    return emit(name, [x, y], [_aval(shape, out_dtype or dtype)])


def add(x, y): return _binary('add', x, y)
def sub(x, y): return _binary('sub', x, y)
def mul(x, y): return _binary('mul', x, y)
def div(x, y): return _binary('div', x, y)
def max(x, y): return _binary('max', x, y)
def min(x, y): return _binary('min', x, y)
def rem(x, y): return _binary('rem', x, y)
def pow(x, y): return _binary('pow', x, y, allowed=(_f32,))
def add_any(x, y): return _binary('add_any', x, y)
def nextafter(x, y): return _binary('nextafter', x, y, allowed=(_f32,))
def gt(x, y): return _binary('gt', x, y, out_dtype=_bool)
def ge(x, y): return _binary('ge', x, y, out_dtype=_bool)
def lt(x, y): return _binary('lt', x, y, out_dtype=_bool)
def le(x, y): return _binary('le', x, y, out_dtype=_bool)
def eq(x, y): return _binary('eq', x, y, out_dtype=_bool)
def ne(x, y): return _binary('ne', x, y, out_dtype=_bool)
def bitwise_or(x, y):  return _binary('or', x, y, allowed=(_i32, _u32, _bool))
def bitwise_and(x, y): return _binary('and', x, y, allowed=(_i32, _u32, _bool))
def bitwise_xor(x, y): return _binary('xor', x, y, allowed=(_i32, _u32, _bool))
def shift_left(x, y):  return _binary('shift_left', x, y, allowed=(_i32, _u32))
def shift_right_logical(x, y):    return _binary('shift_right_logical', x, y, allowed=(_i32, _u32))
def shift_right_arithmetic(x, y): return _binary('shift_right_arithmetic', x, y, allowed=(_i32, _u32))


def _unary_f32(name):
    def op(x):
        x = _as_dtype(x, _f32) if not isinstance(x, Tracer) else x
        if dtype_of(x)[0] != _f32:
            raise TypeError(f'{name} needs float32, got {dtype_of(x)[0]}')
        return emit(name, [x], [_aval(_shape(x), _f32)])
    op.__name__ = name
    return op


exp, log, rsqrt, erf, erf_inv = map(_unary_f32, ('exp', 'log', 'rsqrt', 'erf', 'erf_inv'))
cos, sin, tan, cosh, sinh, tanh = map(_unary_f32, ('cos', 'sin', 'tan', 'cosh', 'sinh', 'tanh'))
acos, asin, atan, acosh, asinh, atanh = map(_unary_f32, ('acos', 'asin', 'atan', 'acosh', 'asinh', 'atanh'))
ceil, floor = map(_unary_f32, ('ceil', 'floor'))
sqrt = _unary_f32('sqrt')
logistic, log1p, expm1, exp2, cbrt = map(_unary_f32, ('logistic', 'log1p', 'expm1', 'exp2', 'cbrt'))
def atan2(x, y): return _binary('atan2', x, y, allowed=(_f32,))


def is_finite(x):
    if dtype_of(x)[0] != _f32:
        raise TypeError('is_finite needs float32')
    return emit('is_finite', [x], [_aval(_shape(x), _bool)])


def round(x, rounding_method: int = 0):
    '''rounding_method 0: halves away from zero, 1: halves to even (jax.lax.RoundingMethod).'''
    if dtype_of(x)[0] != _f32:
        raise TypeError('round needs float32')
    return emit('round', [x], [_aval(_shape(x), _f32)], dict(rounding_method=int(rounding_method)))


def clamp(lo, x, hi):
    '''min(max(x, lo), hi); the bounds are scalars or have x's shape.'''
    dtype = dtype_of(x)[0]
    lo, hi = _as_dtype(lo, dtype), _as_dtype(hi, dtype)
    for b in (lo, hi):
        if _shape(b) not in ((), _shape(x)):
            raise TypeError('clamp bounds must be scalars or match the operand')
    return emit('clamp', [lo, x, hi], [_aval(_shape(x), dtype)])


def _unary_any(name):
    def op(x):
        return emit(name, [x], [_aval(_shape(x), dtype_of(x)[0])])
    op.__name__ = name
    return op


neg, abs, sign = map(_unary_any, ('neg', 'abs', 'sign'))
square = _unary_any('square')


def _unary_int(name, allowed):
    def op(x):
        if dtype_of(x)[0] not in allowed:
            raise TypeError(f'{name} does not accept {dtype_of(x)[0]}')
        return emit(name, [x], [_aval(_shape(x), dtype_of(x)[0])])
    op.__name__ = name
    return op


bitwise_not      = _unary_int('not', (_i32, _u32, _bool))
population_count = _unary_int('population_count', (_i32, _u32))
clz              = _unary_int('clz', (_i32, _u32))


def integer_pow(x, y: int):
    return emit('integer_pow', [x], [_aval(_shape(x), dtype_of(x)[0])], dict(y=int(y)))


def select(pred, on_true, on_false):
    dtype = result_dtype(on_true, on_false)
    on_true, on_false = _as_dtype(on_true, dtype), _as_dtype(on_false, dtype)
    if dtype_of(pred)[0] != _bool:
        raise TypeError('select predicate must be bool')
    shape = _shape(on_true)
    if not (_shape(pred) == shape == _shape(on_false)):
        raise TypeError(f'select needs equal shapes, got {_shape(pred)}, {shape}, {_shape(on_false)}')
    return emit('select', [pred, on_true, on_false], [_aval(shape, dtype)])


def convert_element_type(x, new_dtype, force=False):
    new_dtype = core.canonicalize_dtype(new_dtype)
    old_dtype = dtype_of(x)[0]
    if old_dtype == new_dtype and isinstance(x, Tracer) and not force:
        return x
    return emit('convert_element_type', [x], [_aval(_shape(x), new_dtype)],
                dict(new_dtype=new_dtype, weak_type=False))


def bitcast_convert_type(x, new_dtype):
    new_dtype = core.canonicalize_dtype(new_dtype)
    if new_dtype == _bool or dtype_of(x)[0] == _bool:
        raise TypeError('bitcast_convert_type does not apply to bool')
    return emit('bitcast_convert_type', [x], [_aval(_shape(x), new_dtype)], dict(new_dtype=new_dtype))


def stop_gradient(x):
    return emit('stop_gradient', [x], [_aval(_shape(x), dtype_of(x)[0])])


# ---------------------------------------------------------------- shape plumbing

def broadcast_in_dim(x, shape, broadcast_dimensions):
    shape = tuple(int(s) for s in shape)
    bdims = tuple(int(d) for d in broadcast_dimensions)
    xs    = _shape(x)
    if len(bdims) != len(xs):
        raise TypeError(f'broadcast_dimensions {bdims} must have one entry per operand dim {xs}')
    for i, d in enumerate(bdims):
        if xs[i] != 1 and xs[i] != shape[d]:
            raise TypeError(f'cannot broadcast {xs} to {shape} along {bdims}')
    return emit('broadcast_in_dim', [x], [_aval(shape, dtype_of(x)[0])],
                dict(shape=shape, broadcast_dimensions=bdims))


def broadcast(x, sizes):
    xs = _shape(x)
    return broadcast_in_dim(x, tuple(sizes) + xs, tuple(range(len(sizes), len(sizes) + len(xs))))


def reshape(x, new_sizes, dimensions=None):
    new_sizes = tuple(int(s) for s in new_sizes)
    if int(np.prod(new_sizes, dtype=np.int64)) != int(np.prod(_shape(x), dtype=np.int64)):
        raise TypeError(f'cannot reshape {_shape(x)} to {new_sizes}')
    return emit('reshape', [x], [_aval(new_sizes, dtype_of(x)[0])], dict(new_sizes=new_sizes, dimensions=dimensions))


def squeeze(x, dimensions):
    xs   = _shape(x)
    dims = tuple(d % len(xs) for d in dimensions)
    if builtins.any(xs[d] != 1 for d in dims):
        raise ValueError(f'cannot squeeze dims {dims} of {xs}')
    shape = tuple(s for i, s in enumerate(xs) if i not in dims)
    return emit('squeeze', [x], [_aval(shape, dtype_of(x)[0])], dict(dimensions=dims))


def expand_dims(x, dimensions):
    xs    = list(_shape(x))
    rank  = len(xs) + len(dimensions)
    dims  = sorted(d % rank for d in dimensions)
    for d in dims:
        xs.insert(d, 1)
    return reshape(x, xs)


def split(x, sizes, axis: int = 0):
    '''Pieces of `x` along `axis` with the given sizes (the `split` primitive of newer jax).'''
    xs    = _shape(x)
    axis  = axis % len(xs)
    sizes = tuple(int(n) for n in sizes)
    if builtins.sum(sizes) != xs[axis]:
        raise TypeError(f'split sizes {sizes} do not add up to {xs[axis]}')
    avals = [_aval(xs[:axis] + (n,) + xs[axis + 1:], dtype_of(x)[0]) for n in sizes]
    return emit('split', [x], avals, dict(sizes=sizes, axis=axis), multiple_results=True)


def iota(dtype, size: int):
    dtype = core.canonicalize_dtype(dtype)
    return emit('iota', [], [_aval((int(size),), dtype)], dict(dtype=dtype, shape=(int(size),), dimension=0))


def broadcasted_iota(dtype, shape, dimension: int):
    dtype = core.canonicalize_dtype(dtype)
    shape = tuple(int(s) for s in shape)
    return emit('iota', [], [_aval(shape, dtype)], dict(dtype=dtype, shape=shape, dimension=int(dimension)))


def concatenate(operands, dimension: int):
    operands = list(operands)
    dtype    = result_dtype(*operands)
    operands = [_as_dtype(o, dtype) for o in operands]
    shapes   = [_shape(o) for o in operands]
    rank     = len(shapes[0])
    dimension = dimension % rank
    for s in shapes:
        if len(s) != rank or builtins.any(a != b for i, (a, b) in enumerate(zip(s, shapes[0])) if i != dimension):
            raise TypeError(f'cannot concatenate {shapes} along {dimension}')
    out = list(shapes[0])
    out[dimension] = builtins.sum(s[dimension] for s in shapes)
    return emit('concatenate', operands, [_aval(out, dtype)], dict(dimension=dimension))


def slice(x, start_indices, limit_indices, strides=None):
    xs     = _shape(x)
    start  = tuple(int(s) for s in start_indices)
    limit  = tuple(int(s) for s in limit_indices)
    stride = tuple(int(s) for s in strides) if strides is not None else None
    if not (len(start) == len(limit) == len(xs)):
        raise TypeError('slice indices must have one entry per dimension')
    for s, l, n in zip(start, limit, xs):
        if not (0 <= s <= l <= n):
            raise TypeError(f'slice [{start}:{limit}] out of range for {xs}')
    st    = stride or (1,) * len(xs)
    shape = tuple((l - s + k - 1) // k for s, l, k in zip(start, limit, st))
    return emit('slice', [x], [_aval(shape, dtype_of(x)[0])],
                dict(start_indices=start, limit_indices=limit, strides=stride))


def transpose(x, permutation):
    perm = tuple(int(p) for p in permutation)
    xs   = _shape(x)
    if sorted(perm) != list(range(len(xs))):
        raise TypeError(f'bad permutation {perm} for rank {len(xs)}')
    return emit('transpose', [x], [_aval(tuple(xs[p] for p in perm), dtype_of(x)[0])], dict(permutation=perm))


def rev(x, dimensions):
    return emit('rev', [x], [_aval(_shape(x), dtype_of(x)[0])], dict(dimensions=tuple(int(d) for d in dimensions)))


# ---------------------------------------------------------------- contractions

def dot_general(lhs, rhs, dimension_numbers, precision=None):
    (lc, rc), (lb, rb) = dimension_numbers
    lc, rc, lb, rb = (tuple(int(i) for i in t) for t in (lc, rc, lb, rb))
    ls, rs = _shape(lhs), _shape(rhs)
    dtype  = result_dtype(lhs, rhs)
    lhs, rhs = _as_dtype(lhs, dtype), _as_dtype(rhs, dtype)
    if [ls[i] for i in lc] != [rs[i] for i in rc] or [ls[i] for i in lb] != [rs[i] for i in rb]:
        raise TypeError(f'dot_general: contracting/batch sizes differ for {ls} and {rs} with {dimension_numbers}')
    batch = tuple(ls[i] for i in lb)
    lfree = tuple(s for i, s in enumerate(ls) if i not in lc and i not in lb)
    rfree = tuple(s for i, s in enumerate(rs) if i not in rc and i not in rb)
    return emit('dot_general', [lhs, rhs], [_aval(batch + lfree + rfree, dtype)],
                dict(dimension_numbers=((lc, rc), (lb, rb)), precision=precision, preferred_element_type=None))


def _same_padding(in_size, window, stride):
    out   = -(-in_size // stride)
    total = builtins.max((out - 1) * stride + window - in_size, 0)
    return (total // 2, total - total // 2)


def padtype_to_pads(in_shape, window_shape, window_strides, padding: str):
    if padding.upper() == 'VALID':
        return [(0, 0)] * len(in_shape)
    if padding.upper() == 'SAME':
        return [_same_padding(n, k, s) for n, k, s in zip(in_shape, window_shape, window_strides)]
    raise ValueError(f'unknown padding {padding}')


def conv_general_dilated(lhs, rhs, window_strides, padding, lhs_dilation=None, rhs_dilation=None,
                         dimension_numbers=None, feature_group_count=1, batch_group_count=1, precision=None):
    ls, rs = _shape(lhs), _shape(rhs)
    nsp    = len(ls) - 2
    if dimension_numbers is None:
        dimension_numbers = ConvDimensionNumbers(tuple(range(nsp + 2)), tuple(range(nsp + 2)), tuple(range(nsp + 2)))
    elif not isinstance(dimension_numbers, ConvDimensionNumbers):
        if isinstance(dimension_numbers[0], str):
            dimension_numbers = conv_dimension_numbers(dimension_numbers)
        else:
            dimension_numbers = ConvDimensionNumbers(*(tuple(d) for d in dimension_numbers))
    dn     = dimension_numbers
    dtype  = result_dtype(lhs, rhs)
    lhs, rhs = _as_dtype(lhs, dtype), _as_dtype(rhs, dtype)
    lhs_dilation = tuple(lhs_dilation) if lhs_dilation is not None else (1,) * nsp
    rhs_dilation = tuple(rhs_dilation) if rhs_dilation is not None else (1,) * nsp
    strides      = tuple(int(s) for s in window_strides)
    in_sp   = [(ls[d] - 1) * ld + 1 if ls[d] > 0 else 0 for d, ld in zip(dn.lhs_spec[2:], lhs_dilation)]
    k_sp    = [(rs[d] - 1) * rd + 1 for d, rd in zip(dn.rhs_spec[2:], rhs_dilation)]
    if isinstance(padding, str):
        padding = padtype_to_pads(in_sp, k_sp, strides, padding)
    padding = tuple((int(lo), int(hi)) for lo, hi in padding)
    if ls[dn.lhs_spec[1]] != rs[dn.rhs_spec[1]] * feature_group_count:
        raise TypeError(f'conv: input features {ls[dn.lhs_spec[1]]} do not match the kernel\'s {rs[dn.rhs_spec[1]]}')
    out_sp  = [builtins.max((n + lo + hi - k) // s + 1, 0) for n, k, s, (lo, hi) in zip(in_sp, k_sp, strides, padding)]
    out     = [0] * (nsp + 2)
    out[dn.out_spec[0]] = ls[dn.lhs_spec[0]] // batch_group_count
    out[dn.out_spec[1]] = rs[dn.rhs_spec[0]]
    for d, n in zip(dn.out_spec[2:], out_sp):
        out[d] = n
    return emit('conv_general_dilated', [lhs, rhs], [_aval(out, dtype)],
                dict(window_strides=strides, padding=padding, lhs_dilation=lhs_dilation, rhs_dilation=rhs_dilation,
                     dimension_numbers=dn, feature_group_count=feature_group_count,
                     batch_group_count=batch_group_count, lhs_shape=ls, rhs_shape=rs, precision=precision))


def conv_dimension_numbers(spec: tp.Tuple[str, str, str]) -> ConvDimensionNumbers:
    '''("NHWC","HWIO","NHWC")-style strings to index tuples (batch/out, feature/in, spatial...).'''
    lhs, rhs, out = spec
    spatial = [c for c in rhs if c not in 'OI']
    def conv(s, lead):
        return tuple(s.index(c) for c in lead) + tuple(s.index(c) for c in
                     sorted((c for c in s if c not in lead), key=lambda c: s.index(c)))
    lhs_spec = conv(lhs, 'NC')
    out_spec = conv(out, 'NC')
    rhs_spec = (rhs.index('O'), rhs.index('I')) + tuple(rhs.index(c) for c in spatial)
    return ConvDimensionNumbers(lhs_spec, rhs_spec, out_spec)


# ---------------------------------------------------------------- reductions

def _reduce(name, x, axes, out_dtype=None, extra=None):
    xs   = _shape(x)
    axes = tuple(sorted(int(a) % builtins.max(len(xs), 1) for a in axes)) if len(xs) else ()
    shape = tuple(s for i, s in enumerate(xs) if i not in axes)
    params = dict(axes=axes)
    params.update(extra or {})
    return emit(name, [x], [_aval(shape, out_dtype or dtype_of(x)[0])], params)


def reduce_sum(x, axes):  return _reduce('reduce_sum', x, axes)
def reduce_max(x, axes):  return _reduce('reduce_max', x, axes)
def reduce_min(x, axes):  return _reduce('reduce_min', x, axes)
def reduce_prod(x, axes): return _reduce('reduce_prod', x, axes)


def reduce_or(x, axes):
    if dtype_of(x)[0] != _bool:
        raise TypeError('reduce_or takes booleans')
    return _reduce('reduce_or', x, axes)


def reduce_and(x, axes):
    if dtype_of(x)[0] != _bool:
        raise TypeError('reduce_and takes booleans')
    return _reduce('reduce_and', x, axes)


def argmax(x, axis: int, index_dtype=_i32):
    return _reduce('argmax', x, (axis,), core.canonicalize_dtype(index_dtype), dict(index_dtype=np.dtype(index_dtype)))


def argmin(x, axis: int, index_dtype=_i32):
    return _reduce('argmin', x, (axis,), core.canonicalize_dtype(index_dtype), dict(index_dtype=np.dtype(index_dtype)))


def reduce_window(x, init_value, computation, window_dimensions, window_strides, padding,
                  base_dilation=None, window_dilation=None):
    '''Only the monoids the device path has kernels for: `lax.max` with -inf and `lax.add` with 0.'''
    xs = _shape(x)
    wd = tuple(int(w) for w in window_dimensions)
    ws = tuple(int(s) for s in window_strides)
    if isinstance(padding, str):
        padding = padtype_to_pads(xs, wd, ws, padding)
    padding = tuple((int(lo), int(hi)) for lo, hi in padding)
    if computation is max and np.isneginf(init_value):
        name = 'reduce_window_max'
    elif computation is add and init_value == 0:
        name = 'reduce_window_sum'
    else:
        raise NotImplementedError('reduce_window supports (max, -inf) and (add, 0)')
    shape = tuple(builtins.max((n + lo + hi - w) // s + 1, 0) for n, w, s, (lo, hi) in zip(xs, wd, ws, padding))
    return emit(name, [x], [_aval(shape, dtype_of(x)[0])],
                dict(window_dimensions=wd, window_strides=ws, padding=padding,
                     base_dilation=tuple(base_dilation or (1,) * len(xs)),
                     window_dilation=tuple(window_dilation or (1,) * len(xs))))


def select_and_scatter_add(source, operand, select_prim, window_dimensions, window_strides, padding):
    '''The gradient of a max/min pooling as autodiff emits it (`select_prim` is `ge_p` or `le_p`).'''
    xs = _shape(operand)
    wd = tuple(int(w) for w in window_dimensions)
    ws = tuple(int(s) for s in window_strides)
    padding = tuple((int(lo), int(hi)) for lo, hi in padding)
    pooled  = tuple(builtins.max((n + lo + hi - w) // s + 1, 0) for n, w, s, (lo, hi) in zip(xs, wd, ws, padding))
    if _shape(source) != pooled:
        raise TypeError(f'select_and_scatter_add: source {_shape(source)} does not match the pooled shape {pooled}')
    if dtype_of(source)[0] != _f32 or dtype_of(operand)[0] != _f32:
        raise TypeError('select_and_scatter_add takes float32 operands')
    if getattr(select_prim, 'name', None) not in ('ge', 'le'):
        raise NotImplementedError('select_and_scatter_add selects with ge or le')
    return emit('select_and_scatter_add', [source, operand], [_aval(xs, _f32)],
                dict(select_prim=select_prim, window_dimensions=wd, window_strides=ws, padding=padding))


ge_p, le_p = core.Primitive('ge'), core.Primitive('le')


def pad(x, padding_value, padding_config):
    '''(low, high, interior) per dimension; negative low/high crop.'''
    dtype  = dtype_of(x)[0]
    config = tuple((int(lo), int(hi), int(it)) for lo, hi, it in padding_config)
    xs     = _shape(x)
    if len(config) != len(xs) or builtins.any(it < 0 for _, _, it in config):
        raise TypeError('pad needs one (low, high, interior >= 0) triple per dimension')
    shape  = tuple(builtins.max(n + builtins.max(n - 1, 0) * it + lo + hi, 0) for n, (lo, hi, it) in zip(xs, config))
    return emit('pad', [x, _as_dtype(padding_value, dtype)], [_aval(shape, dtype)], dict(padding_config=config))


# ---------------------------------------------------------------- indexing

def gather(operand, start_indices, dimension_numbers: GatherDimensionNumbers, slice_sizes,
           indices_are_sorted=False, unique_indices=False, mode=None, fill_value=None):
    dn   = GatherDimensionNumbers(*(tuple(int(i) for i in t) for t in dimension_numbers))
    ops  = _shape(operand)
    ids  = _shape(start_indices)
    ss   = tuple(int(s) for s in slice_sizes)
    if dtype_of(start_indices)[0] not in (_i32, _u32):
        raise TypeError('gather indices must be integers')
    if ids[-1] != len(dn.start_index_map):
        raise TypeError('last dim of start_indices must equal len(start_index_map)')
    offset_sizes = [s for i, s in enumerate(ss) if i not in dn.collapsed_slice_dims]
    if len(offset_sizes) != len(dn.offset_dims):
        raise TypeError('offset_dims do not match the non-collapsed slice dims')
    batch = list(ids[:-1])
    rank  = len(batch) + len(offset_sizes)
    out, bi, oi = [], iter(batch), iter(offset_sizes)
    for d in range(rank):
        out.append(next(oi) if d in dn.offset_dims else next(bi))
    for s, n in zip(ss, ops):
        if not 0 <= s <= n:
            raise TypeError(f'slice_sizes {ss} exceed operand shape {ops}')
    return emit('gather', [operand, start_indices], [_aval(out, dtype_of(operand)[0])],
                dict(dimension_numbers=dn, slice_sizes=ss, indices_are_sorted=indices_are_sorted,
                     unique_indices=unique_indices,
                     **({} if mode is None else dict(mode=mode, fill_value=fill_value))))


def scatter_add(operand, scatter_indices, updates, dimension_numbers: ScatterDimensionNumbers,
                indices_are_sorted=False, unique_indices=False, mode=None):
    dn = ScatterDimensionNumbers(*(tuple(int(i) for i in t) for t in dimension_numbers))
    dtype = result_dtype(operand, updates)
    operand, updates = _as_dtype(operand, dtype), _as_dtype(updates, dtype)
    if dtype_of(scatter_indices)[0] not in (_i32, _u32):
        raise TypeError('scatter indices must be integers')
    return emit('scatter-add', [operand, scatter_indices, updates], [_aval(_shape(operand), dtype)],
                dict(dimension_numbers=dn, indices_are_sorted=indices_are_sorted, unique_indices=unique_indices,
                     update_jaxpr=None, update_consts=(), **({} if mode is None else dict(mode=mode))))


# ---------------------------------------------------------------- rng

def threefry2x32(key0, key1, x0, x1):
    for v in (key0, key1, x0, x1):
        if dtype_of(v)[0] != _u32:
            raise TypeError('threefry2x32 takes uint32 operands')
    if _shape(key0) != _shape(key1) or _shape(x0) != _shape(x1):
        raise TypeError('threefry2x32: key halves / data halves must have equal shapes')
    shape = _shape(x0)
    return emit('threefry2x32', [key0, key1, x0, x1], [_aval(shape, _u32), _aval(shape, _u32)], multiple_results=True)



# typed keys: the primitives newer jax versions emit for jax.random (jax/_src/prng.py); a key
# array's element is a whole threefry key, see core.KeyTy

def _is_key(x) -> bool:
    return isinstance(x, Tracer) and core.is_key_dtype(x.dtype)


def random_seed(seeds, impl='fry'):
    if dtype_of(seeds)[0] not in (_i32, _u32):
        raise TypeError('random_seed takes integers')
    return emit('random_seed', [seeds], [_aval(_shape(seeds), core.key_fry)], dict(impl=impl))


def random_wrap(key_data, impl='fry'):
    if dtype_of(key_data)[0] != _u32 or _shape(key_data)[-1:] != core.key_fry.key_shape:
        raise TypeError('random_wrap takes uint32[..., 2]')
    return emit('random_wrap', [key_data], [_aval(_shape(key_data)[:-1], core.key_fry)], dict(impl=impl))


def random_unwrap(keys):
    if not _is_key(keys):
        raise TypeError('random_unwrap takes a key array')
    return emit('random_unwrap', [keys], [_aval(_shape(keys) + core.key_fry.key_shape, _u32)])


def random_bits(keys, bit_width: int, shape):
    if not _is_key(keys):
        raise TypeError('random_bits takes a key array')
    if bit_width != 32:
        raise NotImplementedError('random_bits: 32-bit words only (all device data is 32 bits wide)')
    shape = tuple(int(n) for n in shape)
    return emit('random_bits', [keys], [_aval(_shape(keys) + shape, _u32)], dict(bit_width=32, shape=shape))


def random_split(keys, shape):
    if not _is_key(keys):
        raise TypeError('random_split takes a key array')
    shape = tuple(int(n) for n in shape)
    return emit('random_split', [keys], [_aval(_shape(keys) + shape, core.key_fry)], dict(shape=shape))


def random_fold_in(keys, msgs):
    if not _is_key(keys) or dtype_of(msgs)[0] != _u32 or _shape(msgs) != _shape(keys):
        raise TypeError('random_fold_in takes a key array and uint32 data of the same shape')
    return emit('random_fold_in', [keys, msgs], [_aval(_shape(keys), core.key_fry)])
