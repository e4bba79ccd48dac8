'''CPU oracle: a numpy restatement of every primitive on the device path.

TEST INFRASTRUCTURE ONLY. Nothing in the shipped package may import this module; it is
the checker that tests, the smoke run and the benchmark's CPU-baseline leg compare the
HIP path against.

Each function states the value the reference's ground truth (JAX's CPU backend, see
reference tests/test_basic_ops.py:346, tests/test_conv.py:100, tests/test_reduce_window.py:36)
produces for one primitive, and cites the reference kernel it corresponds to. Where a
reference shader departs from XLA semantics the XLA rule is followed and the departure is
named: out-of-window taps of a max-pool are -inf rather than 0
(vkjax/shaders/reduce_window_max_2d.comp:44-46), `select` picks instead of blending
(select.comp:12), gather start indices are clamped (gather.comp:75-86), a logical right
shift by >= 32 gives 0 (shift_right_logical.comp:12).

Arrays use the device's four 32-bit types (float32, int32, uint32, bool). Contractions and
sums accumulate in float64 and round once to float32, so the oracle is at least as accurate
as any fp32 evaluation order.

Pinning (tests/test_oracle_*.py): threefry2x32 against the Random123 known-answer vectors
and the published `jax.random.split(PRNGKey(0))` / `uniform(PRNGKey(0))` values; dot_general
against exact integer arithmetic and einsum; conv_general_dilated against a brute-force loop
written from vkjax/shaders/conv2d.comp:44-95, against torch.nn.functional.conv2d in float64,
and against the delta-kernel and 1x1 == GEMM special cases; reduce_window against brute force
and torch max_pool2d / avg_pool2d; gather / scatter-add against brute-force loops over the
XLA index rule and numpy fancy indexing / np.add.at; reductions and elementwise ops against
closed forms and hand-computed values; the key primitives of newer jax versions (random_bits,
random_split, ...) in the original counter layout against that same expansion and in the
partitionable layout against the values jax's documentation prints (tests/test_key_primitives.py).
Parity unpinned: the *jaxpr expansions* (which
primitives jax emits for jnp.dot, softmax, indexing, random.uniform) - they are produced by
jax, which is not importable here, and are restated from the reference's accepted-parameter
lists only.
'''
import math

import numpy as np

import builtins

f32, i32, u32 = np.float32, np.int32, np.uint32
builtins_max, builtins_min = builtins.max, builtins.min
_EW_ERR = dict(over='ignore', invalid='ignore', divide='ignore')


def _canon(x):
    x = np.asarray(x)
    if x.dtype == np.float64: return x.astype(f32)
    if x.dtype == np.int64:   return x.astype(i32)
    if x.dtype == np.uint64:  return x.astype(u32)
    return x


# ------------------------------------------------------------------ elementwise binary
# reference: vkjax/ops.py:73-114 and shaders add/sub/mul/div/max/min/gt/ge/lt/le/eq/ne/
# and/or/rem/pow/shift_*.comp (`result[i] = a[i] op b[i]`, implicit trailing broadcast)

def _bin(f):
    def op(a, b):
        a, b = _canon(a), _canon(b)
        with np.errstate(**_EW_ERR):
            return _canon(f(a, b))
    return op


add = _bin(np.add)
sub = _bin(np.subtract)
mul = _bin(np.multiply)
add_any = add
gt, ge, lt, le = _bin(np.greater), _bin(np.greater_equal), _bin(np.less), _bin(np.less_equal)
eq, ne = _bin(np.equal), _bin(np.not_equal)


def _maxmin(f):
    #lax.max/min propagate NaN; on bool they are or/and
    return _bin(lambda a, b: f(a, b))


max = _maxmin(np.maximum)
min = _maxmin(np.minimum)


@_bin
def div(a, b):
    if a.dtype.kind == 'f':
        return a / b
    #integer division truncates toward zero (C semantics), division by zero -> -1 like XLA
    q = np.where(b == 0, -1, np.trunc(a.astype(np.float64) / np.where(b == 0, 1, b)).astype(np.int64))
    return q.astype(a.dtype)


@_bin
def rem(a, b):
    if a.dtype.kind == 'f':
        return np.fmod(a, b)
    safe = np.where(b == 0, 1, b)
    r = np.fmod(a.astype(np.int64), safe.astype(np.int64))
    return np.where(b == 0, a, r).astype(a.dtype)


@_bin
def pow(a, b):
    return np.power(a.astype(np.float64), b.astype(np.float64)).astype(f32)


@_bin
def nextafter(a, b):
    return np.nextafter(a.astype(f32), b.astype(f32))


def _bitop(f):
    def op(a, b):
        a, b = _canon(a), _canon(b)
        return f(a, b)
    return op


globals()['or']  = _bitop(np.bitwise_or)
globals()['and'] = _bitop(np.bitwise_and)
xor = _bitop(np.bitwise_xor)
bit_or, bit_and = globals()['or'], globals()['and']


def shift_left(a, b):
    a, b = _canon(a), _canon(b)
    bu   = b.astype(np.int64) & 0xFFFFFFFF if b.dtype == u32 else b.astype(np.int64)
    out  = (a.astype(np.int64) & 0xFFFFFFFF) << np.clip(bu, 0, 32)
    out  = np.where((bu < 0) | (bu >= 32), 0, out) & 0xFFFFFFFF
    return out.astype(u32).view(a.dtype) if a.dtype != u32 else out.astype(u32)


def shift_right_logical(a, b):
    '''XLA: shifting by >= bit width gives 0 (pinned by reference tests/test_basic_ops.py:150-151,305:
    shift_right_logical(1, 32) == 0).'''
    a, b = _canon(a), _canon(b)
    a, b = np.broadcast_arrays(a, b)
    bu   = b.astype(np.int64) & 0xFFFFFFFF
    out  = (a.astype(np.int64) & 0xFFFFFFFF) >> np.minimum(bu, 32)
    out  = np.where(bu >= 32, 0, out)
    return out.astype(u32).view(a.dtype) if a.dtype != u32 else out.astype(u32)


def shift_right_arithmetic(a, b):
    '''Sign-propagating shift; a shift count >= 32 saturates to 31 (XLA).'''
    a, b = _canon(a), _canon(b)
    a, b = np.broadcast_arrays(a, b)
    bu   = np.minimum(b.astype(np.int64) & 0xFFFFFFFF, 31)
    if a.dtype == u32:
        #arithmetic shift reinterprets the bits as signed
        return (a.view(i32).astype(np.int64) >> bu).astype(i32).view(u32)
    return (a.astype(np.int64) >> bu).astype(i32)


# ------------------------------------------------------------------ elementwise unary
# reference: vkjax/ops.py:119-155, shaders exp/log/neg/abs/rsqrt/erf/erf_inv/unary_op.comp

def _un64(f):
    def op(x):
        x = _canon(x)
        with np.errstate(**_EW_ERR):
            return np.asarray(f(x.astype(np.float64))).astype(f32)
    return op


exp, log, sqrt = _un64(np.exp), _un64(np.log), _un64(np.sqrt)
rsqrt = _un64(lambda x: 1.0 / np.sqrt(x))
cos, sin, tan = _un64(np.cos), _un64(np.sin), _un64(np.tan)
cosh, sinh, tanh = _un64(np.cosh), _un64(np.sinh), _un64(np.tanh)
acos, asin, atan = _un64(np.arccos), _un64(np.arcsin), _un64(np.arctan)
acosh, asinh, atanh = _un64(np.arccosh), _un64(np.arcsinh), _un64(np.arctanh)
ceil, floor = _un64(np.ceil), _un64(np.floor)


logistic = _un64(lambda x: 1.0 / (1.0 + np.exp(-x)))
log1p, expm1, exp2, cbrt = _un64(np.log1p), _un64(np.expm1), _un64(np.exp2), _un64(np.cbrt)


def atan2(a, b):
    return np.arctan2(_canon(a).astype(np.float64), _canon(b).astype(np.float64)).astype(f32)


def is_finite(x):
    return np.isfinite(_canon(x))


def round(x, rounding_method=0, **_):
    '''rounding_method 0: halves away from zero; 1: halves to even (jax.lax.RoundingMethod).'''
    x = _canon(x).astype(np.float64)
    if int(getattr(rounding_method, 'value', rounding_method)) == 1:
        return np.rint(x).astype(f32)
    return (np.sign(x) * np.floor(np.abs(x) + 0.5)).astype(f32)


def square(x):
    return mul(x, x)


def clamp(lo, x, hi):
    return globals()['min'](globals()['max'](x, lo), hi)


def population_count(x):
    x = _canon(x)
    return np.array([bin(int(v) & 0xFFFFFFFF).count('1') for v in x.reshape(-1)], dtype=x.dtype).reshape(x.shape)


def clz(x):
    x = _canon(x)
    return np.array([32 - (int(v) & 0xFFFFFFFF).bit_length() for v in x.reshape(-1)], dtype=x.dtype).reshape(x.shape)


def _not(x):
    x = _canon(x)
    return ~x


globals()['not'] = _not


def erf(x):
    from scipy import special
    return special.erf(_canon(x).astype(np.float64)).astype(f32)


def erf_inv(x):
    from scipy import special
    return special.erfinv(_canon(x).astype(np.float64)).astype(f32)


def neg(x):
    x = _canon(x)
    return (-x.astype(np.int64)).astype(x.dtype) if x.dtype.kind in 'iu' else -x


def abs(x):
    x = _canon(x)
    return np.abs(x.astype(np.int64)).astype(x.dtype) if x.dtype.kind == 'i' else np.abs(x)


def sign(x):
    x = _canon(x)
    return np.sign(x).astype(x.dtype)


def integer_pow(x, y):
    '''x**y by repeated multiplication in the operand's own type (integers wrap);
    negative y is 1 / x**|y|. reference: vkjax/shaders/integer_pow.comp:14-28 (y >= 0 only).'''
    x = _canon(x)
    if x.dtype.kind == 'f':
        out = np.power(x.astype(np.float64), abs_int(y))
        return (1.0 / out if y < 0 else out).astype(f32)
    acc = np.ones_like(x, dtype=np.int64)
    for _ in range(y):
        acc = (acc * x.astype(np.int64))
        acc = ((acc + 2**31) % 2**32) - 2**31 if x.dtype == i32 else acc % 2**32
    return acc.astype(x.dtype)


def abs_int(y):
    return -y if y < 0 else y


def select(pred, on_true, on_false):
    '''A true pick, not the reference shader's arithmetic blend (select.comp:12), which
    turns inf/NaN in the unselected branch into NaN.'''
    return np.where(np.asarray(pred, bool), _canon(on_true), _canon(on_false))


def select_n(which, *cases):
    '''select_n of newer jax: case k where `which` is k; for a boolean `which`, case 1 where it is true.'''
    which = np.asarray(which)
    if which.dtype == np.bool_:
        assert len(cases) == 2
        return np.where(which, _canon(cases[1]), _canon(cases[0]))
    return np.choose(which, [_canon(c) for c in cases])


def copy(x, **_):
    return _canon(x).copy()


copy_p = copy


def optimization_barrier(*operands, **_):
    '''Identity on every operand (a scheduling fence for XLA, nothing to compute).'''
    return [_canon(x) for x in operands]


def convert_element_type(x, new_dtype, **_):
    '''float -> int truncates toward zero and saturates; NaN -> 0 (XLA). bool -> 0/1.
    reference: vkjax/shaders/convert_element_type.comp:9-12.'''
    x, new_dtype = _canon(x), np.dtype(new_dtype)
    if new_dtype == np.float64: new_dtype = np.dtype(f32)
    if new_dtype == np.int64:   new_dtype = np.dtype(i32)
    if new_dtype == np.bool_:
        return x != 0
    if x.dtype.kind == 'f' and new_dtype.kind in 'iu':
        info = np.iinfo(new_dtype)
        t = np.trunc(np.nan_to_num(x.astype(np.float64), nan=0.0, posinf=float(info.max), neginf=float(info.min)))
        return np.clip(t, info.min, info.max).astype(new_dtype)
    if x.dtype.kind in 'iu' and new_dtype.kind in 'iu':
        return x.astype(np.int64).astype(new_dtype) if x.dtype != new_dtype else x
    return x.astype(new_dtype)


def bitcast_convert_type(x, new_dtype, **_):
    return _canon(x).view(np.dtype(new_dtype))


def stop_gradient(x):
    return _canon(x)


# ------------------------------------------------------------------ shape plumbing

def broadcast_in_dim(x, shape, broadcast_dimensions, **_):
    '''reference: vkjax/ops.py:187-215, vkjax/shaders/broadcast_in_dim.comp:33-49.'''
    x = _canon(x)
    expanded = [1] * len(shape)
    for i, d in enumerate(broadcast_dimensions):
        expanded[d] = x.shape[i]
    return np.broadcast_to(x.reshape(expanded), shape).copy()


def reshape(x, new_sizes, dimensions=None, **_):
    assert dimensions is None
    return _canon(x).reshape(new_sizes)


def split(x, sizes, axis, **_):
    edges = np.cumsum([0] + [int(n) for n in sizes])
    return [np.take(x, np.arange(edges[i], edges[i + 1]), axis=axis) for i in range(len(sizes))]


def expand_dims(x, dimensions, **_):
    return np.expand_dims(x, tuple(dimensions))


def squeeze(x, dimensions, **_):
    return np.squeeze(_canon(x), axis=tuple(dimensions))


def iota(dtype, shape, dimension, **_):
    '''reference: vkjax/shaders/iota.comp:8-11 (dimension 0 of a 1-D result); the general
    form counts along `dimension` and is constant along the others.'''
    n   = shape[dimension]
    idx = np.arange(n).reshape([n if i == dimension else 1 for i in range(len(shape))])
    return np.broadcast_to(idx, shape).astype(dtype)


def concatenate(*xs, dimension, **_):
    return np.concatenate([_canon(x) for x in xs], axis=dimension)


def slice(x, start_indices, limit_indices, strides=None, **_):
    '''reference: vkjax/ops.py:534-547, vkjax/shaders/slice.comp:28-36.'''
    import builtins
    strides = strides or (1,) * len(start_indices)
    return _canon(x)[tuple(builtins.slice(s, l, k) for s, l, k in zip(start_indices, limit_indices, strides))].copy()


def transpose(x, permutation, **_):
    return np.transpose(_canon(x), permutation).copy()


def rev(x, dimensions, **_):
    return np.flip(_canon(x), axis=tuple(dimensions)).copy()


# ------------------------------------------------------------------ contractions

def dot_general(lhs, rhs, dimension_numbers, **_):
    '''reference: vkjax/ops.py:277-297, vkjax/shaders/dot_general.comp:10-34 (2-D, one
    contracting dim per side, no batch dims). Result dims: batch, lhs free, rhs free.'''
    (lc, rc), (lb, rb) = dimension_numbers
    lhs, rhs = _canon(lhs), _canon(rhs)
    is_float = lhs.dtype.kind == 'f'
    a = lhs.astype(np.float64) if is_float else lhs.astype(np.int64)
    b = rhs.astype(np.float64) if is_float else rhs.astype(np.int64)
    lfree = [i for i in range(a.ndim) if i not in lc and i not in lb]
    rfree = [i for i in range(b.ndim) if i not in rc and i not in rb]
    a = np.transpose(a, list(lb) + lfree + list(lc))
    b = np.transpose(b, list(rb) + list(rc) + rfree)
    bshape = a.shape[:len(lb)]
    fa, fb = a.shape[len(lb):len(lb) + len(lfree)], b.shape[len(rb) + len(rc):]
    k   = int(np.prod(a.shape[len(lb) + len(lfree):], dtype=np.int64))
    a2  = a.reshape(bshape + (-1, k)) if k else a.reshape(bshape + (int(np.prod(fa, dtype=np.int64)), 0))
    b2  = b.reshape(bshape + (k, -1)) if k else b.reshape(bshape + (0, int(np.prod(fb, dtype=np.int64))))
    out = np.matmul(a2, b2).reshape(bshape + tuple(fa) + tuple(fb))
    return out.astype(lhs.dtype)


def conv_general_dilated(lhs, rhs, window_strides, padding, lhs_dilation, rhs_dilation, dimension_numbers,
                         feature_group_count=1, batch_group_count=1, **_):
    '''2-D cross-correlation (no kernel flip) with strides, explicit low/high padding,
    input (lhs) and kernel (rhs) dilation, any dimension-number permutation, one group.
    out[b,o,y,x] = sum_{i0,i1,c} lhs_dilated_padded[b,c, y*s0 + i0*d0, x*s1 + i1*d1] * rhs[o,c,i0,i1]
    reference: vkjax/ops.py:463-487, vkjax/shaders/conv2d.comp:44-95.
    Evaluated tap by tap as float64 matrix products over the channel axis.'''
    assert feature_group_count == 1 and batch_group_count == 1
    lhs_spec, rhs_spec, out_spec = dimension_numbers
    x = np.transpose(_canon(lhs).astype(np.float64), [lhs_spec[0], lhs_spec[2], lhs_spec[3], lhs_spec[1]])   #N H W C
    w = np.transpose(_canon(rhs).astype(np.float64), [rhs_spec[2], rhs_spec[3], rhs_spec[1], rhs_spec[0]])   #H W I O
    n, h, wd, c = x.shape
    kh, kw, _, o = w.shape
    (ld0, ld1), (rd0, rd1) = lhs_dilation, rhs_dilation
    (s0, s1) = window_strides
    (p0lo, p0hi), (p1lo, p1hi) = padding
    hd, wdd = ((h - 1) * ld0 + 1 if h else 0), ((wd - 1) * ld1 + 1 if wd else 0)
    xd = np.zeros((n, hd, wdd, c))
    xd[:, ::ld0, ::ld1, :] = x
    #negative padding crops; a crop that reaches beyond the array's other end leaves nothing of it, but the
    #padded size is still m + lo + hi (element i of the padded axis is element i - lo of the array)
    def pad_or_crop(a, axis, lo, hi):
        m = a.shape[axis]
        size = builtins_max(m + lo + hi, 0)
        grown = np.zeros(a.shape[:axis] + (size,) + a.shape[axis + 1:])
        src_lo, dst_lo = builtins_max(-lo, 0), builtins_max(lo, 0)
        length = builtins_max(builtins_min(m - src_lo - builtins_max(-hi, 0), size - dst_lo), 0)
        src, dst = [np.s_[:]] * a.ndim, [np.s_[:]] * a.ndim
        src[axis], dst[axis] = np.s_[src_lo:src_lo + length], np.s_[dst_lo:dst_lo + length]
        grown[tuple(dst)] = a[tuple(src)]
        return grown
    xp = pad_or_crop(pad_or_crop(xd, 1, p0lo, p0hi), 2, p1lo, p1hi)
    keh, kew = (kh - 1) * rd0 + 1, (kw - 1) * rd1 + 1
    ho = (xp.shape[1] - keh) // s0 + 1 if xp.shape[1] >= keh else 0
    wo = (xp.shape[2] - kew) // s1 + 1 if xp.shape[2] >= kew else 0
    out = np.zeros((n, ho, wo, o))
    for i0 in range(kh):
        for i1 in range(kw):
            patch = xp[:, i0 * rd0: i0 * rd0 + (ho - 1) * s0 + 1: s0, i1 * rd1: i1 * rd1 + (wo - 1) * s1 + 1: s1, :]
            out  += patch @ w[i0, i1]
    inv = np.argsort([out_spec[0], out_spec[2], out_spec[3], out_spec[1]])
    return np.transpose(out, inv).astype(f32)


# ------------------------------------------------------------------ reductions
# reference: vkjax/ops.py:305-335, shaders reduce_{sum,max,min,prod}.comp, argmax/argmin.comp

def reduce_sum(x, axes, **_):
    x = _canon(x)
    if x.dtype.kind == 'f':
        return x.astype(np.float64).sum(axis=tuple(axes)).astype(f32)
    return x.astype(np.int64).sum(axis=tuple(axes)).astype(x.dtype)


def reduce_prod(x, axes, **_):
    x = _canon(x)
    if x.dtype.kind == 'f':
        return x.astype(np.float64).prod(axis=tuple(axes)).astype(f32)
    return x.astype(np.int64).prod(axis=tuple(axes)).astype(x.dtype)


def _extreme(dtype, largest: bool):
    '''XLA's init value of reduce_min (largest) / reduce_max: what a reduction over no elements returns.'''
    dtype = np.dtype(dtype)
    if dtype.kind == 'f':
        return dtype.type(np.inf if largest else -np.inf)
    if dtype.kind == 'b':
        return largest
    info = np.iinfo(dtype)
    return dtype.type(info.max if largest else info.min)


def reduce_max(x, axes, **_):
    x = _canon(x)
    return x.max(axis=tuple(axes), initial=_extreme(x.dtype, False)) if len(axes) else x


def reduce_min(x, axes, **_):
    x = _canon(x)
    return x.min(axis=tuple(axes), initial=_extreme(x.dtype, True)) if len(axes) else x


def reduce_or(x, axes, **_):
    return np.any(np.asarray(x, bool), axis=tuple(axes))


def reduce_and(x, axes, **_):
    return np.all(np.asarray(x, bool), axis=tuple(axes))


def _arg_reduce(x, axes, index_dtype, better):
    '''Index of the first best element along one axis; a NaN is better than any number and
    the first NaN wins (XLA). The reference shader (argmax.comp:50-52) uses a strict compare,
    which gives the same first-occurrence rule for ties and has no NaN rule.'''
    (axis,) = axes
    x   = np.moveaxis(_canon(x), axis, -1)
    out = np.zeros(x.shape[:-1], dtype=np.int64)
    best = x[..., 0].copy()
    for j in range(1, x.shape[-1]):
        v = x[..., j]
        upd = (better(v, best) | (np.isnan(v) & ~np.isnan(best))) if x.dtype.kind == 'f' else better(v, best)
        out  = np.where(upd, j, out)
        best = np.where(upd, v, best)
    return out.astype(np.dtype(index_dtype) if np.dtype(index_dtype) != np.int64 else i32)


def argmax(x, axes, index_dtype=i32, **_):
    return _arg_reduce(x, axes, index_dtype, np.greater)


def argmin(x, axes, index_dtype=i32, **_):
    return _arg_reduce(x, axes, index_dtype, np.less)


def _reduce_window(x, init, combine, window_dimensions, window_strides, padding, base_dilation=None,
                   window_dilation=None):
    x = _canon(x)
    n = x.ndim
    assert tuple(base_dilation or (1,) * n) == (1,) * n
    wdil = tuple(window_dilation or (1,) * n)
    xp = np.pad(x.astype(np.float64) if x.dtype.kind == 'f' else x.astype(np.int64),
                [(lo, hi) for lo, hi in padding], constant_values=init)
    out_shape = [(xp.shape[d] - (window_dimensions[d] - 1) * wdil[d] - 1) // window_strides[d] + 1 for d in range(n)]
    out = np.full(out_shape, init, dtype=xp.dtype)
    for tap in np.ndindex(*window_dimensions):
        sl = tuple(np.s_[t * wdil[d]: t * wdil[d] + (out_shape[d] - 1) * window_strides[d] + 1: window_strides[d]]
                   for d, t in enumerate(tap))
        out = combine(out, xp[sl])
    return out.astype(x.dtype)


def reduce_window_max(x, window_dimensions, window_strides, padding, **kw):
    '''Window maximum with -inf outside the array (XLA). The reference shader contributes
    0.0 for out-of-range taps (reduce_window_max_2d.comp:44-46), which differs whenever a
    border window holds only negative values; its own tests use positive inputs only.
    reference: vkjax/ops.py:505-524.'''
    x = _canon(x)
    init = -np.inf if x.dtype.kind == 'f' else np.iinfo(x.dtype).min
    return _reduce_window(x, init, np.maximum, window_dimensions, window_strides, padding, **kw)


def reduce_window_sum(x, window_dimensions, window_strides, padding, **kw):
    '''Window sum with 0 outside the array (average pooling divides it by the window size
    afterwards). No counterpart in the reference's primitive set.'''
    return _reduce_window(x, 0, np.add, window_dimensions, window_strides, padding, **kw)


def select_and_scatter_add(source, operand, select_prim, window_dimensions, window_strides, padding, **_):
    '''XLA select-and-scatter with addition (the gradient of a max/min pooling): every window of
    `operand` selects one of its elements, and the window's `source` value is added to the result
    at that position; the result has operand's shape and starts at 0. Selection follows XLA's
    evaluator: the window is scanned in row-major order over the positions inside the array
    (padding is never selected), the first one is taken, and a later one replaces it whenever
    select(selected, candidate) is false, with select = `ge` (max pooling) or `le` (min pooling);
    ties keep the earlier position. Windows are visited in row-major order, and sums follow it.'''
    name = getattr(select_prim, 'name', str(select_prim))
    keep = {'ge': lambda a, b: a >= b, 'le': lambda a, b: a <= b}[name]
    source, operand = _canon(source), _canon(operand)
    out = np.zeros(operand.shape, np.float64)
    for o in np.ndindex(*source.shape):
        selected = None
        for t in np.ndindex(*window_dimensions):
            pos = tuple(o[d] * window_strides[d] - padding[d][0] + t[d] for d in range(operand.ndim))
            if any(p < 0 or p >= operand.shape[d] for d, p in enumerate(pos)):
                continue
            if selected is None or not keep(operand[selected], operand[pos]):
                selected = pos
        if selected is not None:
            #float32 accumulation in visiting order, as a sequential scatter would do
            out[selected] = np.float32(np.float32(out[selected]) + source[o])
    return out.astype(f32)


def pad(x, padding_value, padding_config, **_):
    '''XLA pad: (low, high, interior) per dimension; negative low/high crop.'''
    x = _canon(x)
    value = np.asarray(padding_value, dtype=x.dtype).reshape(())
    for d, (lo, hi, interior) in enumerate(padding_config):
        n = x.shape[d]
        dilated = np.full(x.shape[:d] + (builtins_max(n + (n - 1) * interior, 0),) + x.shape[d + 1:], value, x.dtype)
        idx = [np.s_[:]] * x.ndim
        idx[d] = np.s_[::interior + 1]
        dilated[tuple(idx)] = x
        m = dilated.shape[d]
        grown = np.full(x.shape[:d] + (builtins_max(m + lo + hi, 0),) + x.shape[d + 1:], value, x.dtype)
        src_lo, dst_lo = builtins_max(-lo, 0), builtins_max(lo, 0)
        length = builtins_max(builtins_min(m - src_lo - builtins_max(-hi, 0), grown.shape[d] - dst_lo), 0)
        src, dst = [np.s_[:]] * x.ndim, [np.s_[:]] * x.ndim
        src[d], dst[d] = np.s_[src_lo:src_lo + length], np.s_[dst_lo:dst_lo + length]
        grown[tuple(dst)] = dilated[tuple(src)]
        x = grown
    return x


# ------------------------------------------------------------------ indexing

def _index_mode_name(mode) -> str:
    name = '' if mode is None else str(getattr(mode, 'name', mode)).upper().rsplit('.', 1)[-1]
    return {'FILL': 'FILL_OR_DROP', 'DROP': 'FILL_OR_DROP'}.get(name, name)      #the strings jax accepts for the enum


def gather(operand, start_indices, dimension_numbers, slice_sizes, mode=None, fill_value=None, **_):
    '''XLA gather. Output dims listed in offset_dims enumerate the positions inside a slice
    (slice dims that are not collapsed, in order); the remaining output dims are the batch
    dims of start_indices (all but its last). Each batch position holds one start vector,
    scattered into operand coordinates through start_index_map and clamped so the slice
    fits. With mode FILL_OR_DROP (newer jax versions) a slice that does not fit is not moved inside:
    its positions read as fill_value (default: NaN, the most negative signed integer, the largest
    unsigned one, True). reference: vkjax/ops.py:372-401, vkjax/shaders/gather.comp:62-103 (no clamping there).'''
    if _index_mode_name(mode) == 'FILL_OR_DROP':
        clamped = gather(operand, start_indices, dimension_numbers, slice_sizes)
        op, idx = _canon(operand), _canon(start_indices).astype(np.int64)
        outside = np.zeros(idx.shape[:-1], dtype=bool)
        for k, d in enumerate(dimension_numbers[2]):
            outside |= (idx[..., k] < 0) | (idx[..., k] > op.shape[d] - slice_sizes[d])
        if fill_value is None:
            kind = op.dtype.kind
            fill_value = np.nan if kind == 'f' else np.iinfo(op.dtype).min if kind == 'i' else np.iinfo(op.dtype).max if kind == 'u' else True
        #the batch dims of the result are those not listed in offset_dims, in order
        batch_dims = [d for d in range(clamped.ndim) if d not in dimension_numbers[0]]
        shape = [1] * clamped.ndim
        for d, n in zip(batch_dims, outside.shape):
            shape[d] = n
        return np.where(outside.reshape(shape), np.asarray(fill_value, op.dtype), clamped).astype(op.dtype)
    offset_dims, collapsed, start_index_map = dimension_numbers
    operand, idx = _canon(operand), _canon(start_indices).astype(np.int64)
    batch_shape  = idx.shape[:-1]
    kept         = [d for d in range(operand.ndim) if d not in collapsed]
    out_rank     = len(batch_shape) + len(kept)
    batch_dims   = [d for d in range(out_rank) if d not in offset_dims]
    #clamped start per batch position, per operand dim
    start = np.zeros(batch_shape + (operand.ndim,), dtype=np.int64)
    for k, d in enumerate(start_index_map):
        start[..., d] = np.clip(idx[..., k], 0, operand.shape[d] - slice_sizes[d])
    #index grids: batch dims then kept slice dims
    grids = np.meshgrid(*[np.arange(n) for n in batch_shape], *[np.arange(slice_sizes[d]) for d in kept],
                        indexing='ij', sparse=False) if (batch_shape or kept) else []
    bgrid, sgrid = grids[:len(batch_shape)], grids[len(batch_shape):]
    coords = []
    for d in range(operand.ndim):
        base = start[tuple(bgrid) + (d,)] if batch_shape else start[d]
        if kept and not batch_shape:
            base = np.broadcast_to(base, sgrid[0].shape)
        off  = sgrid[kept.index(d)] if d in kept else 0
        coords.append(base + off)
    vals = operand[tuple(coords)] if coords else operand
    #vals dims are (batch..., kept...) -> place them at batch_dims / offset_dims
    src_order = batch_dims + list(offset_dims)
    return np.transpose(vals, np.argsort(src_order)).copy() if vals.ndim else vals


def scatter_add(operand, scatter_indices, updates, dimension_numbers, mode=None, **_):
    '''XLA scatter with addition. update_window_dims are the dims of `updates` that run
    inside a window; the window spans the operand dims not in inserted_window_dims; the
    other update dims are the batch dims of scatter_indices. A window that does not fit
    entirely inside the operand is dropped; with mode CLIP (newer jax versions) it is moved inside
    instead. Float sums accumulate in float64.
    reference: vkjax/ops.py:404-433 (two fixed patterns), vkjax/shaders/scatter0.comp, scatter1.comp.'''
    uwd, iwd, sd2od = dimension_numbers
    operand, idx, updates = _canon(operand), _canon(scatter_indices).astype(np.int64), _canon(updates)
    if _index_mode_name(mode) == 'CLIP' and operand.size:
        sizes = [updates.shape[d] for d in uwd]
        window = iter(sizes)
        per_dim = [1 if d in iwd else next(window) for d in range(operand.ndim)]
        idx = idx.copy()
        for k, d in enumerate(sd2od):
            idx[..., k] = np.clip(idx[..., k], 0, operand.shape[d] - per_dim[d])
    acc = operand.astype(np.float64) if operand.dtype.kind == 'f' else operand.astype(np.int64)
    window_op_dims = [d for d in range(operand.ndim) if d not in iwd]
    scatter_dims   = [d for d in range(updates.ndim) if d not in uwd]
    batch_shape    = idx.shape[:-1]
    assert tuple(updates.shape[d] for d in scatter_dims) == tuple(batch_shape), (updates.shape, idx.shape)
    window_shape   = [updates.shape[d] for d in uwd]
    u = np.transpose(updates, scatter_dims + list(uwd)).reshape((-1,) + tuple(window_shape))
    flat_idx = idx.reshape(-1, idx.shape[-1])
    if tuple(iwd) == (0,) and tuple(sd2od) == (0,) and tuple(window_shape) == operand.shape[1:]:
        #whole rows addressed by one index each: the same sum, vectorised
        rows  = flat_idx[:, 0]
        valid = (rows >= 0) & (rows < operand.shape[0])
        np.add.at(acc, rows[valid], u[valid].astype(acc.dtype))
        return acc.astype(operand.dtype)
    wgrids = np.meshgrid(*[np.arange(n) for n in window_shape], indexing='ij') if window_shape else []
    for b in range(flat_idx.shape[0]):
        start = np.zeros(operand.ndim, dtype=np.int64)
        for k, d in enumerate(sd2od):
            start[d] = flat_idx[b, k]
        ok = all(0 <= start[d] and start[d] + (window_shape[window_op_dims.index(d)] if d in window_op_dims else 1)
                 <= operand.shape[d] for d in range(operand.ndim))
        if not ok:
            continue
        coords = tuple((start[d] + wgrids[window_op_dims.index(d)]) if d in window_op_dims else start[d]
                       for d in range(operand.ndim))
        np.add.at(acc, coords, u[b].astype(acc.dtype))
    return acc.astype(operand.dtype)


globals()['scatter-add'] = scatter_add


# ------------------------------------------------------------------ rng

_ROT = ((13, 15, 26, 6), (17, 29, 16, 24))


def threefry2x32(key0, key1, x0, x1):
    '''Threefry-2x32 with 20 rounds: rotation constants {13,15,26,6 | 17,29,16,24}, key
    schedule parity 0x1BD11BDA, five key injections with counters 1..5. A scalar key is
    shared by every lane. reference: vkjax/ops.py:550-560, vkjax/shaders/threefry2x32.comp:38-91.'''
    k0 = np.asarray(key0, dtype=np.uint64) & 0xFFFFFFFF
    k1 = np.asarray(key1, dtype=np.uint64) & 0xFFFFFFFF
    a  = np.asarray(x0, dtype=np.uint64) & 0xFFFFFFFF
    b  = np.asarray(x1, dtype=np.uint64) & 0xFFFFFFFF
    if k0.shape in ((), (1,)) and a.shape not in ((), (1,)):
        k0, k1 = k0.reshape(()), k1.reshape(())
    M  = np.uint64(0xFFFFFFFF)
    ks = (k0, k1, k0 ^ k1 ^ np.uint64(0x1BD11BDA))
    a, b = (a + ks[0]) & M, (b + ks[1]) & M
    for i in range(5):
        for r in _ROT[i % 2]:
            a = (a + b) & M
            b = ((b << np.uint64(r)) | (b >> np.uint64(32 - r))) & M
            b = b ^ a
        a = (a + ks[(i + 1) % 3]) & M
        b = (b + ks[(i + 2) % 3] + np.uint64(i + 1)) & M
    return a.astype(u32), b.astype(u32)


# Key primitives of newer jax versions (jax/_src/prng.py: threefry_seed, threefry_split,
# threefry_fold_in, threefry_random_bits). A key array is held as its uint32 words, shape
# (..., 2). Both counter layouts of jax are restated; which one applies is jax's configuration
# flag `jax_threefry_partitionable`, mirrored here by THREEFRY_PARTITIONABLE. Pins: the original
# layout against the published split(PRNGKey(0)) / uniform(PRNGKey(0)) values, the partitionable
# layout against the values jax's documentation prints for uniform(key(0)) = 0.947667 and
# uniform(split(key(0))[1]) = 0.00729382.
THREEFRY_PARTITIONABLE = False


def random_wrap(x, **_):
    return np.asarray(x, u32)


def random_unwrap(x, **_):
    return np.asarray(x, u32)


def random_clone(x, **_):
    return np.asarray(x, u32)


def random_seed(seeds, **_):
    seeds = _canon(seeds)
    low   = (seeds.astype(np.int64) & 0xFFFFFFFF).astype(u32)
    return np.stack([np.zeros_like(low), low], axis=-1)


def _threefry_2x32_flat(key, counts):
    '''jax's threefry_2x32: the flat counters are split into two halves (one zero appended when
    the count is odd), run through the block function, joined again and trimmed.'''
    n    = counts.size
    flat = np.concatenate([counts.reshape(-1), np.zeros(n % 2, u32)])
    a, b = threefry2x32(key[0], key[1], flat[:flat.size // 2], flat[flat.size // 2:])
    return np.concatenate([a, b])[:n].reshape(counts.shape)


def _single_key(keys):
    keys = np.asarray(keys, u32)
    if keys.shape != (2,):
        raise NotImplementedError('batched keys')
    return keys


def random_bits(keys, bit_width, shape, **_):
    assert bit_width == 32
    key = _single_key(keys)
    n   = int(np.prod(shape, dtype=np.int64))
    if THREEFRY_PARTITIONABLE:
        hi, lo = threefry2x32(key[0], key[1], np.zeros(n, u32), np.arange(n, dtype=u32))
        return (hi ^ lo).reshape(shape)
    return _threefry_2x32_flat(key, np.arange(n, dtype=u32)).reshape(shape)


def random_split(keys, shape, **_):
    key = _single_key(keys)
    num = int(np.prod(shape, dtype=np.int64))
    if THREEFRY_PARTITIONABLE:
        hi, lo = threefry2x32(key[0], key[1], np.zeros(num, u32), np.arange(num, dtype=u32))
        return np.stack([hi, lo], axis=-1).reshape(tuple(shape) + (2,))
    return _threefry_2x32_flat(key, np.arange(2 * num, dtype=u32)).reshape(tuple(shape) + (2,))


def random_fold_in(keys, msgs, **_):
    key = _single_key(keys)
    return _threefry_2x32_flat(key, np.array([0, np.asarray(msgs, u32).reshape(())], dtype=u32))
