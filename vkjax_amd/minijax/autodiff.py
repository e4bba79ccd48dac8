'''Reverse-mode differentiation for the stand-in tracer: `value_and_grad` / `grad`.

jax differentiates before a backend ever sees the program, so the jaxprs `vkjax.wrap` receives for a
training step already contain the backward pass, spelled with a small set of primitives: `add_any`,
transposed `dot_general`s, convolutions with lhs / rhs dilation and reversed kernels, `select_and_scatter_add`,
`pad`, `scatter-add`, broadcasts turned into `reduce_sum`s (the reference runs such programs in
tests/test_elegy_mlp.py:87-129 and tests/test_elegy_conv.py:51-94). This module produces programs of that
form without jax: the function is traced, its equations are replayed into the enclosing trace, and the
cotangents are propagated backwards with one rule per primitive. The rules are the textbook
vector-Jacobian products, written with the same primitives and operand conventions jax's own rules use
(e.g. the input gradient of a strided convolution is a convolution of the lhs-dilated cotangent with the
spatially reversed kernel).
'''
import typing as tp

import numpy as np

from . import core, lax, numpy as mnp, tree_util
from .tracer import Tracer, _abstractify, _trace_to_jaxpr, current_trace, dtype_of, emit

_f32 = np.dtype('float32')
_CALL_PARAMS = {'xla_call': 'call_jaxpr', 'core_call': 'call_jaxpr', 'closed_call': 'call_jaxpr', 'pjit': 'jaxpr',
                'jit': 'jaxpr', 'custom_jvp_call_jaxpr': 'fun_jaxpr', 'custom_jvp_call': 'call_jaxpr'}


def _shape(x):
    return tuple(x.shape) if isinstance(x, Tracer) else tuple(np.shape(x))


def _full(shape, value):
    '''A constant array as jax's rules make it: a broadcast of a scalar literal (no storage of its own).'''
    return lax.broadcast_in_dim(np.float32(value), tuple(shape), ()) if tuple(shape) else np.float32(value)


def _zeros_like(x):
    return _full(_shape(x), 0.0)


def _sum_to_shape(g, shape):
    '''Undo the implicit broadcast of a binary op: scalars were spread everywhere, size-1 dimensions along theirs.'''
    gs = _shape(g)
    if gs == tuple(shape):
        return g
    if tuple(shape) == ():
        return lax.reduce_sum(g, tuple(range(len(gs))))
    axes = tuple(d for d, (a, b) in enumerate(zip(gs, shape)) if a != b)
    return lax.reshape(lax.reduce_sum(g, axes), tuple(shape))


def _indicator(pred, yes, no, shape):
    return lax.select(pred, _full(shape, yes), _full(shape, no))


# ---------------------------------------------------------------- rules: (cotangent(s) of the result, operands, result, params) -> operand cotangents

RULES: tp.Dict[str, tp.Callable] = {}


def _rule(*names):
    def register(f):
        for n in names:
            RULES[n] = f
        return f
    return register


@_rule('add', 'add_any')
def _add(g, x, y, out):
    return (lambda: _sum_to_shape(g, _shape(x))), (lambda: _sum_to_shape(g, _shape(y)))


@_rule('sub')
def _sub(g, x, y, out):
    return (lambda: _sum_to_shape(g, _shape(x))), (lambda: _sum_to_shape(lax.neg(g), _shape(y)))


@_rule('mul')
def _mul(g, x, y, out):
    return (lambda: _sum_to_shape(lax.mul(g, y), _shape(x))), (lambda: _sum_to_shape(lax.mul(x, g), _shape(y)))


@_rule('div')
def _div(g, x, y, out):
    return ((lambda: _sum_to_shape(lax.div(g, y), _shape(x))),
            (lambda: _sum_to_shape(lax.mul(lax.mul(lax.neg(g), x), lax.integer_pow(y, -2)), _shape(y))))


@_rule('max', 'min')
def _maxmin(g, x, y, out):
    #each operand gets the cotangent where it equals the result, shared half and half where both do
    shape = _shape(out)
    def share(mine, other):
        e_mine, e_other = lax.eq(mnp.broadcast_to(mine, shape), out), lax.eq(mnp.broadcast_to(other, shape), out)
        part = lax.div(_indicator(e_mine, 1, 0, shape), _indicator(e_other, 2, 1, shape))
        return _sum_to_shape(lax.mul(g, part), _shape(mine))
    return (lambda: share(x, y)), (lambda: share(y, x))


@_rule('neg')
def _neg(g, x, out):
    return (lax.neg(g),)


@_rule('exp')
def _exp(g, x, out):
    return (lax.mul(g, out),)


@_rule('log')
def _log(g, x, out):
    return (lax.div(g, x),)


@_rule('sqrt')
def _sqrt(g, x, out):
    return (lax.mul(g, lax.div(np.float32(0.5), out)),)


@_rule('rsqrt')
def _rsqrt(g, x, out):
    return (lax.mul(g, lax.mul(np.float32(-0.5), lax.div(out, x))),)


@_rule('tanh')
def _tanh(g, x, out):
    return (lax.mul(lax.add(g, lax.mul(g, out)), lax.sub(np.float32(1.0), out)),)


@_rule('logistic')
def _logistic(g, x, out):
    return (lax.mul(g, lax.mul(out, lax.sub(np.float32(1.0), out))),)


@_rule('integer_pow')
def _integer_pow(g, x, out, y):
    if y == 0:
        return (None,)
    return (lax.mul(g, lax.mul(np.float32(y), lax.integer_pow(x, y - 1) if y != 1 else _full(_shape(x), 1.0))),)


@_rule('square')
def _square(g, x, out):
    return (lax.mul(g, lax.mul(np.float32(2.0), x)),)


@_rule('select')
def _select(g, pred, on_true, on_false, out):
    zeros = _zeros_like(g)
    return None, (lambda: lax.select(pred, g, zeros)), (lambda: lax.select(pred, zeros, g))


@_rule('convert_element_type')
def _convert(g, x, out, new_dtype, **_):
    return (g if dtype_of(x)[0] == _f32 else None,)


@_rule('stop_gradient')
def _stop_gradient(g, x, out):
    return (None,)


@_rule('reshape', 'squeeze', 'expand_dims')
def _reshape(g, x, out, **_):
    return (lax.reshape(g, _shape(x)),)


@_rule('transpose')
def _transpose(g, x, out, permutation):
    return (lax.transpose(g, tuple(int(i) for i in np.argsort(permutation))),)


@_rule('rev')
def _rev(g, x, out, dimensions):
    return (lax.rev(g, dimensions),)


@_rule('broadcast_in_dim')
def _broadcast_in_dim(g, x, out, shape, broadcast_dimensions):
    xs = _shape(x)
    summed = [d for d in range(len(shape)) if d not in broadcast_dimensions]
    summed += [d for i, d in enumerate(broadcast_dimensions) if xs[i] == 1 and shape[d] != 1]
    if summed:
        g = lax.reduce_sum(g, tuple(sorted(summed)))
    return (lax.reshape(g, xs),)


@_rule('reduce_sum')
def _reduce_sum(g, x, out, axes):
    xs = _shape(x)
    kept = tuple(d for d in range(len(xs)) if d not in axes)
    return (lax.broadcast_in_dim(g, xs, kept),)


@_rule('reduce_max', 'reduce_min')
def _reduce_chooser(g, x, out, axes):
    #the cotangent is shared equally between the positions that hold the extreme value
    xs = _shape(x)
    kept = tuple(d for d in range(len(xs)) if d not in axes)
    location = lax.convert_element_type(lax.eq(x, lax.broadcast_in_dim(out, xs, kept)), np.float32)
    counts   = lax.reduce_sum(location, axes)
    return (lax.div(lax.mul(lax.broadcast_in_dim(g, xs, kept), location), lax.broadcast_in_dim(counts, xs, kept)),)


def _remaining(rank, *groups):
    taken = set(int(d) for grp in groups for d in grp)
    return [d for d in range(rank) if d not in taken]


def _dot_operand_cotangent(g, other, dimension_numbers, operand_rank, operand_is_rhs):
    '''Cotangent of one operand of a batch-free dot_general: contract the result's cotangent with the other
    operand over the other operand's free dimensions, then put the dimensions back in the operand's order.'''
    (c_self, c_other), (b_self, b_other) = dimension_numbers
    if b_self or b_other:
        raise NotImplementedError('differentiation of dot_general with batch dimensions')
    self_kept  = _remaining(operand_rank, c_self)
    other_kept = _remaining(len(_shape(other)), c_other)
    #result dims: (lhs kept..., rhs kept...)
    if operand_is_rhs:
        g_other = list(range(len(other_kept)))                                   #the lhs's kept dims come first
    else:
        g_other = list(range(len(self_kept), len(self_kept) + len(other_kept)))
    product = lax.dot_general(g, other, ((tuple(g_other), tuple(other_kept)), ((), ())))
    #product dims: (self kept..., other's contracting dims in the order of the other operand's dims)
    contract_in_other_order = [c_self[i] for i in np.argsort(c_other)]
    order = np.argsort(self_kept + contract_in_other_order)
    if list(order) != list(range(len(order))):
        product = lax.transpose(product, tuple(int(i) for i in order))
    return product


@_rule('dot_general')
def _dot_general(g, x, y, out, dimension_numbers, **_):
    (cx, cy), (bx, by) = dimension_numbers
    swapped = ((cy, cx), (by, bx))
    return ((lambda: _dot_operand_cotangent(g, y, dimension_numbers, len(_shape(x)), False)),
            (lambda: _dot_operand_cotangent(g, x, swapped, len(_shape(y)), True)))


def _dilated(sizes, dilation):
    return [0 if s == 0 else 1 + d * (s - 1) for s, d in zip(sizes, dilation)]


@_rule('conv_general_dilated')
def _conv(g, lhs, rhs, out, window_strides, padding, lhs_dilation, rhs_dilation, dimension_numbers,
          feature_group_count, batch_group_count, **_):
    if feature_group_count != 1 or batch_group_count != 1:
        raise NotImplementedError('differentiation of grouped convolutions')
    dn = dimension_numbers
    lhs_sp = [_shape(lhs)[d] for d in dn.lhs_spec[2:]]
    rhs_sp = [_shape(rhs)[d] for d in dn.rhs_spec[2:]]
    out_sp = [_shape(g)[d] for d in dn.out_spec[2:]]
    lhs_dil, rhs_dil, out_dil = _dilated(lhs_sp, lhs_dilation), _dilated(rhs_sp, rhs_dilation), _dilated(out_sp, window_strides)
    swap = lambda spec: (spec[1], spec[0]) + tuple(spec[2:])
    #input: the cotangent, dilated by the strides, convolved with the spatially reversed kernel whose
    #feature dimensions trade places
    before = [k - lo - 1 for k, (lo, _) in zip(rhs_dil, padding)]
    after  = [l + k - 1 - o - b for l, k, o, b in zip(lhs_dil, rhs_dil, out_dil, before)]
    g_lhs = lambda: lax.conv_general_dilated(g, lax.rev(rhs, tuple(dn.rhs_spec[2:])), window_strides=tuple(lhs_dilation),
                                     padding=tuple(zip(before, after)), lhs_dilation=tuple(window_strides),
                                     rhs_dilation=tuple(rhs_dilation),
                                     dimension_numbers=core.ConvDimensionNumbers(dn.out_spec, swap(dn.rhs_spec), dn.lhs_spec))
    #kernel: the input convolved with the cotangent as the kernel, batch and feature dimensions trading places
    high = [o - l + (k - lo - 1) for o, l, k, (lo, _) in zip(out_dil, lhs_dil, rhs_dil, padding)]
    g_rhs = lambda: lax.conv_general_dilated(lhs, g, window_strides=tuple(rhs_dilation),
                                     padding=tuple((lo, hi) for (lo, _), hi in zip(padding, high)),
                                     lhs_dilation=tuple(lhs_dilation), rhs_dilation=tuple(window_strides),
                                     dimension_numbers=core.ConvDimensionNumbers(swap(dn.lhs_spec), swap(dn.out_spec), swap(dn.rhs_spec)))
    return g_lhs, g_rhs


@_rule('reduce_window_max')
def _reduce_window_max(g, x, out, window_dimensions, window_strides, padding, **_):
    return (lax.select_and_scatter_add(g, x, lax.ge_p, window_dimensions, window_strides, padding),)


@_rule('reduce_window_sum')
def _reduce_window_sum(g, x, out, window_dimensions, window_strides, padding, **_):
    xs, gs = _shape(x), _shape(g)
    out_dil = _dilated(gs, window_strides)
    before  = [w - lo - 1 for w, (lo, _) in zip(window_dimensions, padding)]
    after   = [n + w - 1 - o - b for n, w, o, b in zip(xs, window_dimensions, out_dil, before)]
    padded  = lax.pad(g, np.float32(0), [(b, a, s - 1) for b, a, s in zip(before, after, window_strides)])
    ones    = (1,) * len(xs)
    return (lax.reduce_window(padded, 0.0, lax.add, window_dimensions, ones, ((0, 0),) * len(xs)),)


@_rule('slice')
def _slice(g, x, out, start_indices, limit_indices, strides):
    xs = _shape(x)
    strides = strides or (1,) * len(xs)
    real_limits = [s + (n - 1) * k + 1 if n else s for s, n, k in zip(start_indices, _shape(g), strides)]
    return (lax.pad(g, np.float32(0), [(s, n - l, k - 1) for s, n, l, k in zip(start_indices, xs, real_limits, strides)]),)


@_rule('pad')
def _pad(g, x, value, out, padding_config):
    #crop the padding off again; the padding value's share is not needed by anything differentiated here
    negated = lax.pad(g, np.float32(0), [(-lo, -hi, 0) for lo, hi, _ in padding_config])
    xs = _shape(x)
    return lax.slice(negated, (0,) * len(xs), _shape(negated), tuple(it + 1 for _, _, it in padding_config)), None


@_rule('concatenate')
def _concatenate(g, *args, dimension):
    operands, cts, start = args[:-1], [], 0
    gs = _shape(g)
    for o in operands:
        n = _shape(o)[dimension]
        lo = [0] * len(gs); hi = list(gs)
        lo[dimension], hi[dimension] = start, start + n
        cts.append(lax.slice(g, lo, hi))
        start += n
    return tuple(cts)


@_rule('gather')
def _gather(g, operand, indices, out, dimension_numbers, slice_sizes, **_):
    dn = core.ScatterDimensionNumbers(update_window_dims=dimension_numbers.offset_dims,
                                      inserted_window_dims=dimension_numbers.collapsed_slice_dims,
                                      scatter_dims_to_operand_dims=dimension_numbers.start_index_map)
    return lax.scatter_add(_zeros_like(operand), indices, g, dn), None


_NOT_DIFFERENTIABLE = {'gt', 'ge', 'lt', 'le', 'eq', 'ne', 'argmax', 'argmin', 'iota', 'and', 'or', 'not', 'xor', 'sign', 'floor', 'ceil',
                       'round', 'is_finite', 'shift_left', 'shift_right_logical', 'shift_right_arithmetic', 'threefry2x32',
                       'random_bits', 'random_split', 'random_wrap', 'random_unwrap', 'random_fold_in', 'random_seed'}


# ---------------------------------------------------------------- driver

def _replay(jaxpr, consts, inputs, env, order):
    '''Emit the equations of `jaxpr` into the current trace (calls are inlined). `env` maps the jaxpr's
    variables to values of the current trace; `order` collects the equations with non-call primitives.'''
    def read(v):
        return v.val if core.is_literal(v) else env[v]
    for v, c in zip(jaxpr.constvars, consts):
        env[v] = c
    for v, x in zip(jaxpr.invars, inputs):
        env[v] = x
    for eqn in jaxpr.eqns:
        name = eqn.primitive.name
        if name in _CALL_PARAMS:
            inner = eqn.params[_CALL_PARAMS[name]]
            rule  = eqn.params.get('jvp_jaxpr_thunk') if name.startswith('custom_jvp') else None
            #a call with a derivative rule of its own is one unit for the backward pass: its body is replayed
            #for the values only
            outs  = _replay(getattr(inner, 'jaxpr', inner), getattr(inner, 'consts', []), [read(v) for v in eqn.invars], env,
                            order if not callable(rule) else [])
            if callable(rule):
                order.append(eqn)
        else:
            outs = emit(name, [read(v) for v in eqn.invars], [v.aval for v in eqn.outvars], eqn.params, eqn.primitive.multiple_results)
            outs = outs if eqn.primitive.multiple_results else [outs]
            order.append(eqn)
        for v, o in zip(eqn.outvars, outs):
            env[v] = o
    return [read(v) for v in jaxpr.outvars]


def value_and_grad(fun: tp.Callable, argnums: tp.Union[int, tp.Sequence[int]] = 0, has_aux: bool = False):
    '''`(value, gradient)` of a scalar-valued function with respect to the arguments `argnums` (pytrees of
    float32 arrays). Must be called while tracing (inside a function given to `make_jaxpr` / `wrap`);
    every traced value the function uses has to come in through its arguments.'''
    single = isinstance(argnums, int)
    wrt    = (argnums,) if single else tuple(argnums)

    def wrapped(*args):
        current_trace()
        leaves, in_tree = tree_util.tree_flatten(tuple(args))
        in_avals = [core.ShapedArray(a.shape, a.dtype) for a in map(_abstractify, leaves)]
        jaxpr, consts, out_tree, _ = _trace_to_jaxpr(fun, in_avals, in_tree, {}, len(args))
        env, order = {}, []
        outs   = _replay(jaxpr, consts, leaves, env, order)
        result = tree_util.tree_unflatten(out_tree, outs)
        value, aux = result if has_aux else (result, None)
        if _shape(value) != () or dtype_of(value)[0] != _f32:
            raise TypeError('value_and_grad needs a function that returns a float32 scalar')

        #positions of the differentiated leaves, and the values that depend on them (by identity: inlined
        #calls bind their own variables to the caller's values)
        counts  = [len(tree_util.tree_leaves([a])) for a in args]
        starts  = np.cumsum([0] + counts)
        wrt_pos = [p for i in wrt for p in range(starts[i], starts[i + 1])]
        value_of = lambda v: v.val if core.is_literal(v) else env[v]
        active  = {id(leaves[p]) for p in wrt_pos}
        for eqn in order:
            if any(id(value_of(v)) in active for v in eqn.invars):
                active.update(id(env[v]) for v in eqn.outvars)

        cts: tp.Dict[int, tp.Any] = {}
        def add_ct(target, g):
            cts[id(target)] = g if id(target) not in cts else lax.add_any(cts[id(target)], g)
        add_ct(value, np.float32(1.0))
        for eqn in reversed(order):
            outs_now = [env[v] for v in eqn.outvars]
            gs = [cts.get(id(o)) for o in outs_now]
            if all(g is None for g in gs) or not any(id(o) in active for o in outs_now):
                continue
            name = eqn.primitive.name
            if name in _NOT_DIFFERENTIABLE:
                continue
            operands = [value_of(v) for v in eqn.invars]
            if name in _CALL_PARAMS:
                #a custom derivative rule (single result): rule(cotangent, result, *arguments)
                in_cts = eqn.params['jvp_jaxpr_thunk'](_materialize(gs[0], outs_now[0]), outs_now[0], *operands)
            else:
                if name not in RULES:
                    raise NotImplementedError(f'no differentiation rule for {name}')
                g = gs if eqn.primitive.multiple_results else _materialize(gs[0], outs_now[0])
                out_arg = outs_now if eqn.primitive.multiple_results else outs_now[0]
                in_cts = RULES[name](g, *operands, out_arg, **eqn.params)
            for operand, ct in zip(operands, in_cts):
                #a rule may hand back a thunk so that nothing is emitted for an operand nobody differentiates
                if ct is not None and id(operand) in active:
                    add_ct(operand, ct() if callable(ct) else ct)
        grads = []
        for p in wrt_pos:
            g = cts.get(id(leaves[p]))
            grads.append(_materialize(g, leaves[p]) if g is not None else _zeros_like(leaves[p]))
        per_arg, k = [], 0
        for i in wrt:
            n = counts[i]
            per_arg.append(tree_util.tree_unflatten(tree_util.tree_structure([args[i]]), grads[k:k + n])[0])
            k += n
        gradient = per_arg[0] if single else tuple(per_arg)
        return ((value, aux), gradient) if has_aux else (value, gradient)
    return wrapped


def _materialize(g, like):
    '''A cotangent that is still the python/numpy seed becomes an array of the right shape.'''
    if isinstance(g, Tracer):
        return g
    return np.broadcast_to(np.asarray(g, np.float32), _shape(like)).copy() if _shape(like) != () else np.float32(g)


def grad(fun: tp.Callable, argnums: tp.Union[int, tp.Sequence[int]] = 0, has_aux: bool = False):
    def wrapped(*args):
        value, gradient = value_and_grad(fun, argnums, has_aux)(*args)
        return (gradient, value[1]) if has_aux else gradient
    return wrapped
