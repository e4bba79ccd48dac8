'''The slice of the `jax.numpy` surface that the reference's tests and the benchmark
workloads use (reference: tests/test_basic_ops.py:15-160), expressed on the tracer's
`lax` layer. It adds numpy-style dtype and rank promotion on top of `lax`, and lowers
indexing to `gather` / `scatter-add` the way jax.numpy of that period did.
'''
import builtins
import typing as tp

import numpy as np

from . import core, lax
from .tracer import Tracer, dtype_of, result_dtype

float32, int32, uint32, bool_ = np.float32, np.int32, np.uint32, np.bool_
inf, pi, newaxis = np.inf, np.pi, None


def _shape(x):
    return tuple(x.shape) if isinstance(x, Tracer) else tuple(np.shape(x))


def asarray(x, dtype=None):
    if dtype is not None:
        return astype(x, dtype)
    return x


def astype(x, dtype):
    return lax.convert_element_type(x, dtype)


def _promote(*xs):
    '''Common dtype and common rank (leading 1s added by a free reshape); scalars are left alone.'''
    dtype = result_dtype(*xs)
    xs    = [lax._as_dtype(x, dtype) for x in xs]
    rank  = builtins.max(len(_shape(x)) for x in xs)
    out   = []
    for x in xs:
        s = _shape(x)
        if 0 < len(s) < rank:
            x = reshape(x, (1,) * (rank - len(s)) + s)
        out.append(x)
    return out


def _binop(f, floating=False):
    def op(x, y):
        x, y = _promote(x, y)
        if floating and dtype_of(x)[0] != np.float32:
            x, y = astype(x, np.float32), astype(y, np.float32)
        return f(x, y)
    return op


add, subtract, multiply   = _binop(lax.add), _binop(lax.sub), _binop(lax.mul)
true_divide               = _binop(lax.div, floating=True)
divide                    = true_divide
maximum, minimum          = _binop(lax.max), _binop(lax.min)
remainder                 = _binop(lax.rem)
greater, greater_equal    = _binop(lax.gt), _binop(lax.ge)
less, less_equal          = _binop(lax.lt), _binop(lax.le)
equal, not_equal          = _binop(lax.eq), _binop(lax.ne)
bitwise_or, bitwise_and   = _binop(lax.bitwise_or), _binop(lax.bitwise_and)
left_shift                = _binop(lax.shift_left)


def right_shift(x, y):
    x, y = _promote(x, y)
    return lax.shift_right_logical(x, y) if dtype_of(x)[0] == np.uint32 else lax.shift_right_arithmetic(x, y)


def power(x, y):
    if isinstance(y, int) and not isinstance(y, bool):
        return lax.integer_pow(x, y)
    x, y = _promote(x, y)
    return lax.pow(astype(x, np.float32), astype(y, np.float32))


def negative(x): return lax.neg(x)
def abs(x):      return lax.abs(x)
def exp(x):      return lax.exp(astype(x, np.float32))
def log(x):      return lax.log(astype(x, np.float32))
def sqrt(x):     return lax.sqrt(astype(x, np.float32))
def tanh(x):     return lax.tanh(astype(x, np.float32))


def reshape(x, newshape):
    if isinstance(newshape, int):
        newshape = (newshape,)
    newshape = list(newshape)
    size     = int(np.prod(_shape(x), dtype=np.int64))
    if -1 in newshape:
        known = int(np.prod([s for s in newshape if s != -1], dtype=np.int64))
        newshape[newshape.index(-1)] = size // builtins.max(known, 1)
    if not isinstance(x, Tracer):
        return np.reshape(x, newshape)
    return lax.reshape(x, tuple(newshape))


def squeeze(x, axis=None):
    s = _shape(x)
    if axis is None:
        axis = tuple(i for i, n in enumerate(s) if n == 1)
    elif isinstance(axis, int):
        axis = (axis,)
    return lax.squeeze(x, axis)


def expand_dims(x, axis):
    return lax.expand_dims(x, (axis,) if isinstance(axis, int) else tuple(axis))


def transpose(x, axes=None):
    rank = len(_shape(x))
    axes = tuple(reversed(range(rank))) if axes is None else tuple(a % rank for a in axes)
    return lax.transpose(x, axes)


def broadcast_to(x, shape):
    xs, shape = _shape(x), tuple(shape)
    if xs == shape:
        return x
    lead = len(shape) - len(xs)
    return lax.broadcast_in_dim(x, shape, tuple(range(lead, len(shape))))


def zeros(shape, dtype=np.float32):
    return np.zeros(shape, core.canonicalize_dtype(dtype))


def full(shape, fill_value, dtype=np.float32):
    return np.full(shape, fill_value, core.canonicalize_dtype(dtype))


def ones(shape, dtype=np.float32):
    return np.ones(shape, core.canonicalize_dtype(dtype))


def arange(n, dtype=np.int32):
    return lax.iota(dtype, n)


def where(pred, x, y):
    dtype = result_dtype(x, y)
    x, y  = lax._as_dtype(x, dtype), lax._as_dtype(y, dtype)
    shape = np.broadcast_shapes(_shape(pred), _shape(x), _shape(y))
    pred, x, y = (broadcast_to(v, shape) for v in (pred, x, y))
    if dtype_of(pred)[0] != np.bool_:
        pred = lax.ne(pred, 0)
    return lax.select(pred, x, y)


def concatenate(arrays, axis=0):
    arrays = list(arrays)
    return lax.concatenate(arrays, axis % len(_shape(arrays[0])))


def split(x, n: int, axis=0):
    s    = _shape(x)
    axis = axis % len(s)
    step = s[axis] // n
    outs = []
    for i in range(n):
        start = [0] * len(s); start[axis] = i * step
        limit = list(s);      limit[axis] = (i + 1) * step
        outs.append(lax.slice(x, start, limit))
    return outs


def dot(a, b):
    a, b = (lax._as_dtype(v, result_dtype(a, b)) for v in (a, b))
    sa, sb = _shape(a), _shape(b)
    if len(sa) == 0 or len(sb) == 0:
        return multiply(a, b)
    contract_b = 0 if len(sb) == 1 else len(sb) - 2
    return lax.dot_general(a, b, (((len(sa) - 1,), (contract_b,)), ((), ())))


matmul = dot


def _axes(x, axis):
    rank = len(_shape(x))
    if axis is None:
        return tuple(range(rank))
    if isinstance(axis, (int, np.integer)):
        axis = (int(axis),)
    return tuple(sorted(int(a) % builtins.max(rank, 1) for a in axis))


def _reduction(f):
    def op(x, axis=None, keepdims=False):
        axes = _axes(x, axis)
        if len(_shape(x)) == 0:
            axes = ()
        out  = f(x, axes)
        if keepdims:
            out = reshape(out, tuple(1 if i in axes else s for i, s in enumerate(_shape(x))))
        return out
    return op


sum, max, min, prod = map(_reduction, (lax.reduce_sum, lax.reduce_max, lax.reduce_min, lax.reduce_prod))
amax, amin = max, min


def mean(x, axis=None, keepdims=False):
    axes = _axes(x, axis)
    n    = int(np.prod([_shape(x)[a] for a in axes], dtype=np.int64))
    return true_divide(sum(astype(x, np.float32), axis, keepdims=keepdims), float(n))


def _arg_reduction(f):
    def op(x, axis=None):
        if axis is None:
            x, axis = reshape(x, (-1,)), 0
        return f(x, axis % len(_shape(x)), np.int32)
    return op


argmax, argmin = _arg_reduction(lax.argmax), _arg_reduction(lax.argmin)


# ---------------------------------------------------------------- indexing

def _normalize_index(idx, size: int):
    '''Wrap negative entries of a traced integer index (emits lt/add/select, as jax.numpy does).'''
    if isinstance(idx, Tracer):
        if idx.dtype == np.uint32:
            return idx
        return lax.select(lax.lt(idx, 0), lax.add(idx, size), idx)
    idx = np.asarray(idx)
    return np.where(idx < 0, idx + size, idx).astype(np.int32)


def getitem(x, index):
    if not isinstance(index, tuple):
        index = (index,)
    xs = _shape(x)
    if builtins.any(i is Ellipsis for i in index):
        pos   = [i is Ellipsis for i in index].index(True)
        nreal = builtins.sum(1 for i in index if i is not None and i is not Ellipsis)
        index = index[:pos] + (builtins.slice(None),) * (len(xs) - nreal) + index[pos + 1:]
    nreal = builtins.sum(1 for i in index if i is not None)
    index = index + (builtins.slice(None),) * (len(xs) - nreal)

    def is_array(i):
        return isinstance(i, Tracer) or (isinstance(i, (np.ndarray, list)) and np.ndim(i) > 0)

    if isinstance(x, Tracer) and core.is_key_dtype(x.dtype):
        #key arrays: static integers and unit-stride slices, as slice + squeeze (what newer jax traces)
        start, limit, dropped = [], [], []
        for ax, i in enumerate(index):
            if isinstance(i, (int, np.integer)):
                i = int(i) + (xs[ax] if i < 0 else 0)
                if not 0 <= i < xs[ax]:
                    raise IndexError(f'index {i} out of bounds for axis {ax} with size {xs[ax]}')
                start.append(i); limit.append(i + 1); dropped.append(ax)
            elif isinstance(i, builtins.slice) and i.step in (None, 1):
                s, l, _ = i.indices(xs[ax])
                start.append(s); limit.append(builtins.max(l, s))
            else:
                raise NotImplementedError('key arrays take integers and unit-stride slices as indices')
        return lax.squeeze(lax.slice(x, start, limit), dropped)

    arrays = [i for i in index if is_array(i)]
    if len(arrays) > 1 or (arrays and builtins.any(isinstance(i, (int, np.integer)) for i in index)):
        raise NotImplementedError('indexing with more than one array (or arrays mixed with ints)')

    #strided slices are taken first with lax.slice, leaving a unit-stride index
    if builtins.any(isinstance(i, builtins.slice) and i.step not in (None, 1) for i in index):
        start, limit, stride, rest, ax = [], [], [], [], 0
        for i in index:
            if i is None:
                rest.append(None); continue
            if isinstance(i, builtins.slice) and i.step not in (None, 1):
                s, l, k = i.indices(xs[ax])
                if k < 0:
                    raise NotImplementedError('negative slice steps')
                start.append(s); limit.append(builtins.max(l, s)); stride.append(k); rest.append(builtins.slice(None))
            else:
                start.append(0); limit.append(xs[ax]); stride.append(1); rest.append(i)
            ax += 1
        return getitem(lax.slice(x, start, limit, stride), tuple(rest))

    offset_dims, collapsed, start_map, slice_sizes, starts = [], [], [], [], []
    newaxes, out_ax, x_ax = [], 0, 0
    batch_shape, batch_pos = (), None
    for i in index:
        if i is None:
            newaxes.append(out_ax + len(newaxes)); continue
        n = xs[x_ax]
        if isinstance(i, (int, np.integer)):
            i = int(i) + (n if i < 0 else 0)
            if not 0 <= i < n:
                raise IndexError(f'index {i} out of bounds for axis {x_ax} with size {n}')
            collapsed.append(x_ax); start_map.append(x_ax); starts.append(i); slice_sizes.append(1)
        elif isinstance(i, builtins.slice):
            s, l, _ = i.indices(n)
            l = builtins.max(l, s)
            offset_dims.append(out_ax); out_ax += 1
            slice_sizes.append(l - s)
            if (s, l) != (0, n):
                start_map.append(x_ax); starts.append(s)
        else:
            arr = _normalize_index(i if isinstance(i, Tracer) else np.asarray(i), n)
            batch_shape, batch_pos = _shape(arr), out_ax
            out_ax += len(batch_shape)
            collapsed.append(x_ax); start_map.append(x_ax); starts.append(arr); slice_sizes.append(1)
        x_ax += 1

    if not start_map:
        out = x
    else:
        if arrays:
            cols = []
            for s in starts:
                if isinstance(s, int):
                    s = np.full(batch_shape, s, np.int32)
                cols.append(reshape(s, batch_shape + (1,)))
            indices = cols[0] if len(cols) == 1 else concatenate(cols, axis=-1)
        else:
            indices = np.asarray(starts, np.int32)
        dn  = core.GatherDimensionNumbers(tuple(offset_dims), tuple(collapsed), tuple(start_map))
        out = lax.gather(x, indices, dn, tuple(slice_sizes))
    if newaxes:
        out = lax.expand_dims(out, tuple(newaxes))
    return out


def take_along_axis(x, indices, axis=-1):
    xs, ids = _shape(x), _shape(indices)
    axis = axis % len(xs)
    if len(xs) != len(ids):
        raise ValueError('take_along_axis: indices must have the rank of the array')
    cols = []
    for d in range(len(xs)):
        if d == axis:
            col = _normalize_index(indices, xs[d])
        else:
            col = lax.broadcasted_iota(np.int32, ids, d)
        cols.append(reshape(col, ids + (1,)))
    gather_indices = concatenate(cols, axis=-1) if len(cols) > 1 else cols[0]
    dn = core.GatherDimensionNumbers((), tuple(range(len(xs))), tuple(range(len(xs))))
    return lax.gather(x, gather_indices, dn, (1,) * len(xs))


class IndexUpdateHelper:
    '''`x.at[idx].add(u)` for one integer-array index on the leading axis.'''
    def __init__(self, x):
        self.x = x

    def __getitem__(self, index):
        return _IndexUpdateRef(self.x, index)


class _IndexUpdateRef:
    def __init__(self, x, index):
        self.x, self.index = x, index

    def add(self, updates):
        return index_add(self.x, self.index, updates)


def index_add(x, idx, updates):
    """x with `updates` added at rows `idx` of the leading axis (`jax.ops.index_add(x, idx, y)` /
    `x.at[idx].add(y)`): one scatter-add whose windows are whole trailing slices."""
    if isinstance(idx, tuple):
        raise NotImplementedError('index_add with a tuple index')
    xs  = _shape(x)
    idx = _normalize_index(idx, xs[0])
    ids = _shape(idx)
    idx = reshape(idx, ids + (1,))
    updates = broadcast_to(lax._as_dtype(updates, dtype_of(x)[0]), ids + xs[1:])
    dn = core.ScatterDimensionNumbers(tuple(range(len(ids), len(ids) + len(xs) - 1)), (0,), (0,))
    return lax.scatter_add(x, idx, updates, dn)
