'''Primitive dispatch: jaxpr equation -> list of device ops.

Same contract as the reference's vkjax/ops.py: `analyze_jaxpr(bufferpool, jaxpr)` looks up one
module-level function per primitive name (`-` replaced by `_`), each taking
`(bufferpool, equation)` and returning a list of `Op`; unknown primitives raise
NotImplementedError(equation); equations whose outputs are all dropped are skipped
(reference: vkjax/ops.py:52-65). The accepted parameters follow the reference's functions and
are widened where the kernels allow it (any-rank transpose, iota along any dimension,
n-operand concatenate on any axis, general scatter-add, reduce_window_sum).

Instead of SPIR-V bytes an Op carries a launch descriptor for an ahead-of-time built gfx950
kernel. Element-wise work is expressed as an `EwChain` so that neighbouring element-wise ops
can later be merged into one launch; broadcasts, slices, transposes and reversals are read
through strides inside that kernel and never materialised on their own unless they are the
whole op.
'''
import typing as tp

import numpy as np

from . import kernels as K
from .buffers import Buffer, BufferPool
from .kernels import EW, EwChain, EwOperand, EwStep, Launch
from .minijax import core


class Op:
    '''One device launch. `buffers` lists the device arrays it touches in kernel-argument
    order (entries can be None), `shader` names the kernel, `equation` is the jaxpr equation it
    came from (or a label string for helper launches), as in the reference's Op tuple
    (vkjax/ops.py:28-41).'''
    __slots__ = ('equation', 'chain', '_launch', 'conv', 'index', 'meta')

    def __init__(self, equation, launch: tp.Optional[Launch] = None, chain: tp.Optional[EwChain] = None, conv=None, meta=None):
        self.equation = equation
        self.meta     = meta          #(kind, ...) structure of a plain launch that a fusion pass may want to recognise
        self.chain    = chain
        self._launch  = launch
        self.conv     = conv          #(out, lhs, rhs, geometry, epilogue list) for conv/dot ops, so a fusion pass can extend it
        self.index    = None          #position in the program (the pool's op counter when the op was created)

    @property
    def launch(self) -> Launch:
        if self._launch is None:
            if self.chain is not None:
                self._launch = K.lower_ew_chain(self.chain)
            else:
                out, lhs, rhs, geom, epilogue = self.conv
                self._launch = K.conv_gemm(out, lhs, rhs, geom, epilogue)
        return self._launch

    def invalidate(self):
        self._launch = None

    @property
    def buffers(self) -> tp.List[tp.Optional[Buffer]]:
        return [b for b, _ in self.launch.buffers]

    @property
    def shader(self) -> str:
        return self.launch.kernel

    @property
    def workgroup(self):
        return self.launch.grid

    def __repr__(self):
        return f'Op({self.shader}, {self.equation})'


def analyze_jaxpr(bufferpool: BufferPool, jaxpr) -> tp.List[Op]:
    '''Analyzes (possibly inner) jaxprs'''
    all_ops = []
    for eq in jaxpr.eqns:
        if all(core.is_dropped(v) for v in eq.outvars):
            continue
        if all(core.is_dropped(v) or 0 in core.physical(v.aval)[0] for v in eq.outvars):
            #nothing to compute: results without elements get their (token) storage and no launch
            for v in eq.outvars:
                if not core.is_dropped(v):
                    bufferpool.get_buffer(v)
            continue
        opname = eq.primitive.name.replace('-', '_')
        method = globals().get(opname, None)
        if method is None or not callable(method) or opname.startswith('_'):
            raise NotImplementedError(eq)
        if _reuse_equal_equation(bufferpool, eq):
            continue
        position   = bufferpool.op_counter
        method_ops = method(bufferpool, eq)
        for op in method_ops:
            if op.index is None:
                op.index = position
        all_ops += method_ops
    return all_ops


def _reuse_equal_equation(bufferpool: BufferPool, eq) -> bool:
    '''An element-wise or shape equation with the primitive, parameters and operands of an earlier one computes the same
    array: its result variable is bound to that equation's buffer and nothing is launched. (Tracing `x[i]` and
    `x.at[i].add(u)` normalises the same index array twice, three equations each time.) Results of the program keep
    their own storage and equation.'''
    from .buffers import hashable
    name = eq.primitive.name
    if not K.CHOICES.reuse_equal_equations or len(eq.outvars) != 1 or not (name in _BINARY or name in _UNARY or name in _REUSABLE_OTHERS):
        return False
    outvar = eq.outvars[0]
    if hashable(outvar) in bufferpool.buffers:
        return False                                       #a result of the program
    operands, cells = [], []
    for v in eq.invars:
        if core.is_literal(v):
            value = np.asarray(v.val)
            operands.append(('literal', str(value.dtype), value.shape, value.tobytes()))
        else:
            b = bufferpool.buffers.get(hashable(v))
            if b is None:
                return False
            operands.append((id(b._placeholder), str(b.dtype), b.shape))
            cells.append(b._placeholder)
    params = _params_without_jax_bookkeeping(eq.params)
    key = (name, repr(sorted(params.items())), tuple(operands), str(outvar.aval.dtype), tuple(outvar.aval.shape))
    seen = bufferpool.__dict__.setdefault('_equal_equations', {})
    #the entry keeps the operands' storage cells alive, so that the identities in the key cannot pass to other cells
    earlier = seen.get(key)
    if earlier is None or len(earlier[1]) != len(cells) or any(a is not b for a, b in zip(earlier[1], cells)):
        seen[key] = (outvar, cells)
        return False
    bufferpool.set_buffer(outvar, bufferpool.get_buffer(earlier[0]))
    return True


_REUSABLE_OTHERS = {'select', 'select_n', 'convert_element_type', 'integer_pow', 'square', 'reshape', 'broadcast_in_dim',
                    'squeeze', 'expand_dims'}


# ------------------------------------------------------------------ dtype helpers

_F, _I, _U, _B = 'f', 'i', 'u', 'b'


def _kind(dtype) -> str:
    dtype = np.dtype(dtype)
    if dtype == np.float32: return _F
    if dtype == np.int32:   return _I
    if dtype == np.uint32:  return _U
    if dtype == np.bool_:   return _B
    raise NotImplementedError(f'{dtype} data types currently not supported')


#primitive name -> {operand kind -> opcode name}
_BINARY = {
    'add': {_F: 'ADD_F', _I: 'ADD_I', _U: 'ADD_I'},
    'sub': {_F: 'SUB_F', _I: 'SUB_I', _U: 'SUB_I'},
    'mul': {_F: 'MUL_F', _I: 'MUL_I', _U: 'MUL_I', _B: 'AND_X'},
    'div': {_F: 'DIV_F', _I: 'DIV_I', _U: 'DIV_U'},
    'rem': {_F: 'REM_F', _I: 'REM_I', _U: 'REM_U'},
    'max': {_F: 'MAX_F', _I: 'MAX_I', _U: 'MAX_U', _B: 'OR_X'},
    'min': {_F: 'MIN_F', _I: 'MIN_I', _U: 'MIN_U', _B: 'AND_X'},
    'pow': {_F: 'POW_F'},
    'nextafter': {_F: 'NEXTAFTER_F'},
    'gt': {_F: 'GT_F', _I: 'GT_I', _U: 'GT_U', _B: 'GT_U'},
    'ge': {_F: 'GE_F', _I: 'GE_I', _U: 'GE_U', _B: 'GE_U'},
    'lt': {_F: 'LT_F', _I: 'LT_I', _U: 'LT_U', _B: 'LT_U'},
    'le': {_F: 'LE_F', _I: 'LE_I', _U: 'LE_U', _B: 'LE_U'},
    'eq': {_F: 'EQ_F', _I: 'EQ_X', _U: 'EQ_X', _B: 'EQ_X'},
    'ne': {_F: 'NE_F', _I: 'NE_X', _U: 'NE_X', _B: 'NE_X'},
    'and': {_I: 'AND_X', _U: 'AND_X', _B: 'AND_X'},
    'or':  {_I: 'OR_X', _U: 'OR_X', _B: 'OR_X'},
    'xor': {_I: 'XOR_X', _U: 'XOR_X', _B: 'XOR_X'},
    'shift_left':             {_I: 'SHL_X', _U: 'SHL_X'},
    'shift_right_logical':    {_I: 'SHR_L', _U: 'SHR_L'},
    'shift_right_arithmetic': {_I: 'SHR_A', _U: 'SHR_A'},
}
_BINARY['add_any'] = _BINARY['add']
_BINARY['atan2']   = {_F: 'ATAN2_F'}

_UNARY = {
    'exp': {_F: 'EXP_F'}, 'log': {_F: 'LOG_F'}, 'rsqrt': {_F: 'RSQRT_F'}, 'sqrt': {_F: 'SQRT_F'},
    'erf': {_F: 'ERF_F'}, 'erf_inv': {_F: 'ERFINV_F'},
    'neg': {_F: 'NEG_F', _I: 'NEG_I', _U: 'NEG_I'},
    'abs': {_F: 'ABS_F', _I: 'ABS_I', _U: 'NOP'},
    'sign': {_F: 'SIGN_F', _I: 'SIGN_I'},
    'cos': {_F: 'COS_F'}, 'sin': {_F: 'SIN_F'}, 'tan': {_F: 'TAN_F'},
    'cosh': {_F: 'COSH_F'}, 'sinh': {_F: 'SINH_F'}, 'tanh': {_F: 'TANH_F'},
    'acos': {_F: 'ACOS_F'}, 'asin': {_F: 'ASIN_F'}, 'atan': {_F: 'ATAN_F'},
    'acosh': {_F: 'ACOSH_F'}, 'asinh': {_F: 'ASINH_F'}, 'atanh': {_F: 'ATANH_F'},
    'ceil': {_F: 'CEIL_F'}, 'floor': {_F: 'FLOOR_F'},
    'logistic': {_F: 'LOGISTIC_F'}, 'log1p': {_F: 'LOG1P_F'}, 'expm1': {_F: 'EXPM1_F'}, 'exp2': {_F: 'EXP2_F'},
    'cbrt': {_F: 'CBRT_F'}, 'is_finite': {_F: 'ISFINITE_F'},
    'not': {_I: 'NOT_X', _U: 'NOT_X', _B: 'NOT_B'},
    'population_count': {_I: 'POPCNT_X', _U: 'POPCNT_X'}, 'clz': {_I: 'CLZ_X', _U: 'CLZ_X'},
}


def _opcode(table, name, dtype, equation):
    try:
        return EW[table[name][_kind(dtype)]]
    except KeyError:
        raise NotImplementedError(f'{name} on {np.dtype(dtype)}: {equation}')


def _params_without_jax_bookkeeping(params: dict) -> dict:
    #newer jax versions attach bookkeeping entries that do not change the computation
    return {k: v for k, v in params.items() if k not in ('accumulation_type', 'sharding')}


# ------------------------------------------------------------------ element-wise

def element_wise_binary_op(bufferpool: BufferPool, equation):
    assert _params_without_jax_bookkeeping(equation.params) == {}
    assert len(equation.invars) == 2
    assert len(equation.outvars) == 1
    outvar = equation.outvars[0]
    name   = equation.primitive.name
    inbufs = [bufferpool.get_buffer(v) for v in equation.invars]
    opcode = _opcode(_BINARY, name, inbufs[0].dtype, equation)
    #implicit trailing-aligned broadcast is read in place through zero strides
    #(the reference materialises it with an extra dispatch, vkjax/ops.py:84-86)
    operands = [K.broadcast_operand(b, outvar.aval.shape) for b in inbufs]
    outbuf   = bufferpool.get_buffer(outvar, increment_op_counter=True)
    chain    = EwChain(outbuf, outvar.aval.shape, operands[0], [EwStep(opcode, operands[1])])
    return [Op(equation, chain=chain)]


add = sub = mul = div = max = min = element_wise_binary_op
gt = ge = lt = le = eq = ne = element_wise_binary_op
add_any = pow = rem = nextafter = element_wise_binary_op
shift_left = shift_right_logical = shift_right_arithmetic = element_wise_binary_op
xor = atan2 = element_wise_binary_op
globals()['or']  = element_wise_binary_op
globals()['and'] = element_wise_binary_op


def element_wise_unary_op(bufferpool: BufferPool, equation):
    assert _params_without_jax_bookkeeping(equation.params) == {}
    assert len(equation.invars) == 1
    assert len(equation.outvars) == 1
    outvar, invar = equation.outvars[0], equation.invars[0]
    assert tuple(outvar.aval.shape) == tuple(invar.aval.shape)
    inbuf  = bufferpool.get_buffer(invar)
    opcode = _opcode(_UNARY, equation.primitive.name, inbuf.dtype, equation)
    outbuf = bufferpool.get_buffer(outvar, increment_op_counter=True)
    chain  = EwChain(outbuf, outvar.aval.shape, K.broadcast_operand(inbuf, outvar.aval.shape), [EwStep(opcode)])
    return [Op(equation, chain=chain)]


exp = log = neg = abs = rsqrt = sqrt = erf = erf_inv = sign = element_wise_unary_op
cos = sin = tan = cosh = sinh = tanh = element_wise_unary_op
acos = asin = atan = acosh = asinh = atanh = ceil = floor = element_wise_unary_op
#names newer jax versions emit (jax.nn.sigmoid -> logistic, jnp.logical_not -> not, ...)
logistic = log1p = expm1 = exp2 = cbrt = is_finite = population_count = clz = element_wise_unary_op
globals()['not'] = element_wise_unary_op


def square(bufferpool, equation):
    '''x * x in the operand's own type (newer jax traces jnp.square / x**2 as `square`).'''
    inbuf  = bufferpool.get_buffer(equation.invars[0])
    kind   = _kind(inbuf.dtype)
    if kind == _B:
        return noop(bufferpool, equation)
    outbuf  = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    operand = K.broadcast_operand(inbuf, outbuf.shape)
    return [Op(equation, chain=EwChain(outbuf, outbuf.shape, operand, [EwStep(EW['MUL_F' if kind == _F else 'MUL_I'], operand)]))]


def round(bufferpool, equation):
    '''rounding_method 0 (AWAY_FROM_ZERO) or 1 (TO_NEAREST_EVEN), given as an int or as jax's enum.'''
    method = equation.params.get('rounding_method', 0)
    method = int(getattr(method, 'value', method))
    if method not in (0, 1):
        raise NotImplementedError(equation)
    inbuf  = bufferpool.get_buffer(equation.invars[0])
    if _kind(inbuf.dtype) != _F:
        raise NotImplementedError(equation)
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    opcode = EW['ROUND_EVEN_F' if method else 'ROUND_AWAY_F']
    return [Op(equation, chain=EwChain(outbuf, outbuf.shape, K.broadcast_operand(inbuf, outbuf.shape), [EwStep(opcode)]))]


def clamp(bufferpool, equation):
    '''clamp(lo, x, hi) = min(max(x, lo), hi); scalar bounds are read in place.'''
    lo, x, hi = [bufferpool.get_buffer(v) for v in equation.invars]
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    shape  = outbuf.shape
    steps  = [EwStep(_opcode(_BINARY, 'max', x.dtype, equation), K.broadcast_operand(lo, shape)),
              EwStep(_opcode(_BINARY, 'min', x.dtype, equation), K.broadcast_operand(hi, shape))]
    return [Op(equation, chain=EwChain(outbuf, shape, K.broadcast_operand(x, shape), steps))]


def integer_pow(bufferpool, equation):
    inbuf  = bufferpool.get_buffer(equation.invars[0])
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    y      = int(equation.params['y'])
    if _kind(inbuf.dtype) == _F:
        op = EW['IPOW_F']
    else:
        if y < 0:
            raise NotImplementedError(f'negative integer power of integers: {equation}')
        op = EW['IPOW_I']
    chain = EwChain(outbuf, outbuf.shape, K.broadcast_operand(inbuf, outbuf.shape), [EwStep(op, imm=y)])
    return [Op(equation, chain=chain)]


def select(bufferpool, equation):
    '''3-operand select (pred, on_true, on_false), equal shapes (reference: vkjax/ops.py:338-347).'''
    shapes = [tuple(v.aval.shape) for v in equation.invars] + [tuple(equation.outvars[0].aval.shape)]
    assert all(s == shapes[0] for s in shapes)
    pred, on_true, on_false = [bufferpool.get_buffer(v) for v in equation.invars]
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    return [Op(equation, chain=_select_chain(outbuf, pred, on_true, on_false))]


def _select_chain(outbuf, pred, on_true, on_false):
    shape = outbuf.shape
    return EwChain(outbuf, shape, K.broadcast_operand(pred, shape),
                   [EwStep(EW['SEL_P'], K.broadcast_operand(on_true, shape)),
                    EwStep(EW['NOP'], K.broadcast_operand(on_false, shape))])


def select_n(bufferpool, equation):
    '''select_n(which, case0, case1) of newer jax: case1 where `which` is true.'''
    if len(equation.invars) != 3 or _kind(equation.invars[0].aval.dtype) != _B:
        raise NotImplementedError(equation)
    pred, on_false, on_true = [bufferpool.get_buffer(v) for v in equation.invars]
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    return [Op(equation, chain=_select_chain(outbuf, pred, on_true, on_false))]


_CONVERT = {
    (_F, _I): 'CVT_F2I', (_F, _U): 'CVT_F2U', (_I, _F): 'CVT_I2F', (_U, _F): 'CVT_U2F', (_B, _F): 'CVT_U2F',
    (_F, _B): 'CVT_F2B', (_I, _B): 'CVT_X2B', (_U, _B): 'CVT_X2B',
}


def convert_element_type(bufferpool, equation):
    invar, outvar = equation.invars[0], equation.outvars[0]
    src, dst = _kind(core.canonicalize_dtype(invar.aval.dtype)), _kind(core.canonicalize_dtype(outvar.aval.dtype))
    if (src, dst) not in _CONVERT:
        #same bits on the device (int <-> uint, bool -> int, same type): a view is enough
        return noop(bufferpool, equation)
    inbuf  = bufferpool.get_buffer(invar)
    outbuf = bufferpool.get_buffer(outvar, increment_op_counter=True)
    chain  = EwChain(outbuf, outbuf.shape, K.broadcast_operand(inbuf, outbuf.shape), [EwStep(EW[_CONVERT[(src, dst)]])])
    return [Op(equation, chain=chain)]


# ------------------------------------------------------------------ views and data movement

def noop(bufferpool, equation):
    '''No launch: the output is the input's storage seen with another dtype/shape.'''
    assert len(equation.invars) == len(equation.outvars) == 1
    inbuf  = bufferpool.get_buffer(equation.invars[0])
    outvar = equation.outvars[0]
    shape, dtype = core.physical(outvar.aval)
    outbuf = inbuf.view(dtype, shape)
    bufferpool.set_buffer(outvar, outbuf)
    return []


stop_gradient = squeeze = expand_dims = bitcast_convert_type = noop
copy = copy_p = noop


def optimization_barrier(bufferpool, equation):
    '''Identity on every operand (a scheduling fence for XLA): each result is its operand's storage.'''
    assert len(equation.invars) == len(equation.outvars)
    for invar, outvar in zip(equation.invars, equation.outvars):
        if not core.is_dropped(outvar):
            shape, dtype = core.physical(outvar.aval)
            bufferpool.set_buffer(outvar, bufferpool.get_buffer(invar).view(dtype, shape))
    return []
#a typed key array and its uint32 words are the same device array
random_wrap = random_unwrap = random_clone = noop


def reshape(bufferpool, equation):
    assert equation.params['dimensions'] is None
    assert len(equation.outvars) == 1
    assert len(equation.invars) >= 1
    invar, outvar = equation.invars[0], equation.outvars[0]
    assert core.canonicalize_dtype(invar.aval.dtype) == core.canonicalize_dtype(outvar.aval.dtype)
    buffer = bufferpool.get_buffer(invar)
    outbuf = buffer.view(buffer.dtype, outvar.aval.shape)
    bufferpool.set_buffer(outvar, outbuf)
    return []


def _copy_op(equation, outbuf: Buffer, operand: EwOperand):
    return Op(equation, chain=EwChain(outbuf, outbuf.shape, operand, []))


def broadcast_in_dim(bufferpool, equation):
    bdims = tuple(equation.params['broadcast_dimensions'])
    assert np.all(np.diff(bdims) > 0)
    invar, outvar = equation.invars[0], equation.outvars[0]
    inbuf = bufferpool.get_buffer(invar)
    if inbuf.size == int(np.prod(outvar.aval.shape, dtype=np.int64)):
        #same size, just the same storage with a new shape
        outbuf = inbuf.view(inbuf.dtype, outvar.aval.shape)
        bufferpool.set_buffer(outvar, outbuf)
        return []
    outbuf     = bufferpool.get_buffer(outvar, increment_op_counter=True)
    in_strides = K.row_major_strides(inbuf.shape)
    strides    = [0] * len(outbuf.shape)
    for i, d in enumerate(bdims):
        if inbuf.shape[i] != 1:
            if inbuf.shape[i] != outbuf.shape[d]:
                raise ValueError(f'Cannot broadcast from {inbuf.shape} to {outbuf.shape}')
            strides[d] = in_strides[i]
    return [_copy_op(equation, outbuf, EwOperand(inbuf, 0, tuple(strides)))]


def slice(bufferpool, equation):
    inbuf  = bufferpool.get_buffer(equation.invars[0])
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    n       = len(inbuf.shape)
    #a key array has its words as one more (whole) trailing dimension
    extra   = n - len(equation.params['start_indices'])
    start   = tuple(equation.params['start_indices']) + (0,) * extra
    strides = tuple(equation.params['strides'] or (1,) * (n - extra)) + (1,) * extra
    in_strides = K.row_major_strides(inbuf.shape)
    offset  = sum(int(s) * st for s, st in zip(start, in_strides))
    return [_copy_op(equation, outbuf, EwOperand(inbuf, offset, tuple(int(k) * st for k, st in zip(strides, in_strides))))]


def transpose(bufferpool, equation):
    perm   = tuple(equation.params['permutation'])
    inbuf  = bufferpool.get_buffer(equation.invars[0])
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    in_strides = K.row_major_strides(inbuf.shape)
    return [_copy_op(equation, outbuf, EwOperand(inbuf, 0, tuple(in_strides[p] for p in perm)))]


def rev(bufferpool, equation):
    inbuf  = bufferpool.get_buffer(equation.invars[0])
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    dims   = set(int(d) for d in equation.params['dimensions'])
    in_strides = K.row_major_strides(inbuf.shape)
    offset  = sum((inbuf.shape[d] - 1) * in_strides[d] for d in dims)
    strides = tuple(-st if d in dims else st for d, st in enumerate(in_strides))
    return [_copy_op(equation, outbuf, EwOperand(inbuf, offset, strides))]


def iota(bufferpool, equation):
    outvar = equation.outvars[0]
    dimension = int(equation.params['dimension'])
    assert 0 <= dimension < builtins_max(len(outvar.aval.shape), 1)
    outbuf = bufferpool.get_buffer(outvar, increment_op_counter=True)
    if _kind(outbuf.dtype) == _B:
        raise NotImplementedError(equation)
    return [Op(equation, launch=K.iota(outbuf, dimension), meta=('iota', outbuf, dimension))]


def concatenate(bufferpool, equation):
    outvar = equation.outvars[0]
    dim    = int(equation.params['dimension'])
    inbufs = [bufferpool.get_buffer(v) for v in equation.invars]
    for b in inbufs:
        assert b.shape[:dim] == tuple(outvar.aval.shape[:dim]) and b.shape[dim + 1:] == tuple(outvar.aval.shape[dim + 1:])
    outbuf = bufferpool.get_buffer(outvar, increment_op_counter=True)
    ops, offset = [], 0
    for b in inbufs:
        if b.size:
            ops.append(Op(equation, launch=K.concat_part(outbuf, b, dim, offset), meta=('concat_part', outbuf, b, dim, offset)))
        offset += b.shape[dim]
    return ops


def split(bufferpool, equation):
    '''split[sizes, axis] of newer jax: every piece is a strided copy out of the operand.'''
    axis   = int(equation.params['axis'])
    inbuf  = bufferpool.get_buffer(equation.invars[0])
    in_strides = K.row_major_strides(inbuf.shape)
    ops, start = [], 0
    for outvar, size in zip(equation.outvars, equation.params['sizes']):
        if not core.is_dropped(outvar) and int(size):
            outbuf = bufferpool.get_buffer(outvar)
            ops.append(_copy_op(equation, outbuf, EwOperand(inbuf, start * in_strides[axis], tuple(in_strides))))
        start += int(size)
    bufferpool.op_counter += 1
    return ops


# ------------------------------------------------------------------ nested calls (inlined)

def _inline_call(bufferpool, equation, jaxpr, consts=()):
    jaxpr = getattr(jaxpr, 'jaxpr', jaxpr)
    assert len(equation.invars) == len(jaxpr.invars)
    assert len(equation.outvars) == len(jaxpr.outvars)
    for constvar, value in zip(getattr(jaxpr, 'constvars', []), consts):
        b = bufferpool.get_buffer(constvar)
        bufferpool.mark_buffer_as_constant(b, constvar, value=value)
    for eq_var, jaxpr_var in zip(equation.invars, jaxpr.invars):
        if str(eq_var) == '*':
            continue
        #connect call parameters to the function-local variables
        bufferpool.set_buffer(jaxpr_var, bufferpool.get_buffer(eq_var))
    all_ops = analyze_jaxpr(bufferpool, jaxpr)
    for eq_var, jaxpr_var in zip(equation.outvars, jaxpr.outvars):
        if core.is_dropped(eq_var):
            continue
        if str(jaxpr_var) == '*':
            bufferpool.set_buffer(eq_var, None)
            continue
        #connect the function-local variables to the output variables
        bufferpool.set_buffer(eq_var, bufferpool.get_buffer(jaxpr_var))
    return all_ops


def xla_call(bufferpool, equation):
    assert equation.params.get('device') is None
    assert equation.params.get('backend') is None
    return _inline_call(bufferpool, equation, equation.params['call_jaxpr'])


core_call = closed_call = remat = xla_call


def pjit(bufferpool, equation):
    closed = equation.params['jaxpr']
    return _inline_call(bufferpool, equation, closed, getattr(closed, 'consts', ()))


jit = pjit      #the primitive's name in the newest jax versions


def custom_jvp_call_jaxpr(bufferpool, equation):
    closed = equation.params['fun_jaxpr']
    return _inline_call(bufferpool, equation, closed, getattr(closed, 'consts', ()))


def custom_jvp_call(bufferpool, equation):
    closed = equation.params['call_jaxpr']
    return _inline_call(bufferpool, equation, closed, getattr(closed, 'consts', ()))


def custom_vjp_call(bufferpool, equation):
    '''The forward function of a custom_vjp; jax versions name the parameter call_jaxpr or fun_jaxpr.'''
    closed = equation.params['call_jaxpr'] if 'call_jaxpr' in equation.params else equation.params['fun_jaxpr']
    return _inline_call(bufferpool, equation, closed, getattr(closed, 'consts', ()))


custom_vjp_call_jaxpr = custom_vjp_call


# ------------------------------------------------------------------ contractions

#contractions at least this long over the slowest dimension of both operands go to the kernel-gradient GEMM
WGRAD_MIN_PIXELS = 128


def _wgrad_ops(bufferpool, equation, outbuf, x, cot, wg: 'K.WgradGeometry'):
    '''X^T G over the pixels, split over the contraction; the slices are added by a column reduction.'''
    splits = K.choose_wgrad_splits(wg)
    if splits == 1:
        return [Op(equation, launch=K.wgrad_gemm(outbuf, x, cot, wg, 1))]
    position = bufferpool.op_counter
    bufferpool.op_counter -= 1                  #the temporary lives at the equation's own position
    partial = bufferpool.new_temporary(np.float32, (splits, wg.M * wg.N))
    bufferpool.op_counter = position
    launches = [K.wgrad_gemm(partial, x, cot, wg, splits)] + K.reduce(outbuf, partial, 1, splits, wg.M * wg.N, 'reduce_sum')
    return [Op(equation, launch=l) for l in launches]


def _product_ops(bufferpool, equation, outbuf, lhs, rhs, geom: 'K.ConvGeometry'):
    '''The implicit-GEMM launch of a convolution or matrix product; for a product with very few output tiles and a
    long contraction, a launch that sums slices of the contraction into a temporary and an element-wise launch that
    adds the slices in order (which later takes over the element-wise equations that follow).'''
    splits = K.conv_k_splits(lhs, rhs, geom)
    if splits <= 1:
        return [Op(equation, conv=(outbuf, lhs, rhs, geom, []))]
    position = bufferpool.op_counter
    bufferpool.op_counter -= 1                  #the temporary lives at the equation's own position
    partial = bufferpool.new_temporary(np.float32, (splits, outbuf.size))
    bufferpool.op_counter = position
    strides = K.row_major_strides(outbuf.shape)
    slices  = [K.EwOperand(partial, s * outbuf.size, strides) for s in range(splits)]
    total   = K.EwChain(outbuf, outbuf.shape, slices[0], [K.EwStep(K.EW['ADD_F'], o) for o in slices[1:]])
    return [Op(equation, conv=(partial, lhs, rhs, geom._replace(k_splits=splits), [])), Op(equation, chain=total)]


def dot_general(bufferpool, equation):
    '''2-D x 2-D, one contracting dimension per side, no batch dimensions, float32
    (reference: vkjax/ops.py:277-297). Lowered onto the implicit-GEMM kernel with a 1x1 window.'''
    assert equation.params.get('precision') is None
    (lc, rc), (lb, rb) = equation.params['dimension_numbers']
    assert (tuple(lb), tuple(rb)) == ((), ())
    assert tuple(lc) in [(0,), (1,)]
    assert tuple(rc) in [(0,), (1,)]
    assert len(equation.invars) == 2
    assert len(equation.outvars) == 1
    assert all(core.canonicalize_dtype(v.aval.dtype) == np.float32 for v in list(equation.invars) + list(equation.outvars))
    lhs, rhs = [bufferpool.get_buffer(v) for v in equation.invars]
    outbuf   = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    assert len(lhs.shape) == 2 and len(rhs.shape) == 2
    M, N = outbuf.shape
    Kc   = lhs.shape[lc[0]]
    lst, rst = K.row_major_strides(lhs.shape), K.row_major_strides(rhs.shape)
    if outbuf.size == 0:
        return []
    if Kc == 0:
        return [Op(equation, launch=K.fill(outbuf, 0))]            #an empty sum for every element
    if tuple(lc) == (0,) and tuple(rc) == (0,) and Kc >= WGRAD_MIN_PIXELS:
        #both operands contracted over their rows (a dense layer's weight gradient): read along the rows
        wg = K.WgradGeometry(images=1, Ho=Kc, Wo=1, H=Kc, W=1, C=M, KH=1, KW=1, N=N)
        return _wgrad_ops(bufferpool, equation, outbuf, lhs, rhs, wg)
    geom = K.ConvGeometry(batch=1, Ho=M, Wo=1, N=N, H=M, W=1, Cin=Kc, KH=1, KW=1,
                          xs=(0, lst[1 - lc[0]], 0, lst[lc[0]]),
                          ws=(rst[rc[0]] * Kc, rst[rc[0]] * Kc, rst[rc[0]], rst[1 - rc[0]]),
                          os=(M * N, N, N, 1))
    ops, rhs, geom, _ = _with_dense_kernel(bufferpool, equation, rhs, geom, lhs, outbuf)
    return ops + _product_ops(bufferpool, equation, outbuf, lhs, rhs, geom)


def conv_general_dilated(bufferpool, equation):
    '''2-D convolution, any ConvDimensionNumbers permutation, strides, low/high padding, lhs and
    rhs dilation, one feature group (reference: vkjax/ops.py:463-487).'''
    params = equation.params
    assert params.get('precision') is None
    assert params['batch_group_count'] == 1
    assert params['feature_group_count'] == 1
    outvar = equation.outvars[0]
    assert len(outvar.aval.shape) == 4      #2D conv
    assert all(core.canonicalize_dtype(v.aval.dtype) == np.float32 for v in list(equation.invars) + [outvar])
    lhs_spec, rhs_spec, out_spec = params['dimension_numbers']
    lhs, rhs = [bufferpool.get_buffer(v) for v in equation.invars]
    outbuf   = bufferpool.get_buffer(outvar, increment_op_counter=True)
    lst, rst, ost = (K.row_major_strides(b.shape) for b in (lhs, rhs, outbuf))
    pick = lambda seq, spec: tuple(seq[d] for d in spec)
    batch, Cin, H, W = pick(lhs.shape, lhs_spec)
    N, Cin_r, KH, KW = pick(rhs.shape, rhs_spec)
    _, _, Ho, Wo     = pick(outbuf.shape, out_spec)
    assert Cin == Cin_r
    xs = pick(lst, lhs_spec); ws = pick(rst, rhs_spec); os_ = pick(ost, out_spec)
    geom = K.ConvGeometry(batch=batch, Ho=Ho, Wo=Wo, N=N, H=H, W=W, Cin=Cin, KH=KH, KW=KW,
                          SH=params['window_strides'][0], SW=params['window_strides'][1],
                          PH=params['padding'][0][0], PW=params['padding'][1][0],
                          DH=params['rhs_dilation'][0], DW=params['rhs_dilation'][1],
                          LH=params['lhs_dilation'][0], LW=params['lhs_dilation'][1],
                          xs=(xs[0], xs[2], xs[3], xs[1]),
                          ws=(ws[2], ws[3], ws[1], ws[0]),
                          os=(os_[0], os_[2], os_[3], os_[1]))
    if outbuf.size == 0:
        return []
    if lhs.size == 0 or rhs.size == 0:
        return [Op(equation, launch=K.fill(outbuf, 0))]            #no input features, or an empty window: sums of nothing
    wg = _as_kernel_gradient(geom)
    if wg is not None:
        return _wgrad_ops(bufferpool, equation, outbuf, lhs, rhs, wg)
    if (geom.LH > 1 or geom.LW > 1) and geom.SH == geom.SW == 1 and geom.DH == geom.DW == 1:
        return _dilated_input_convolution(bufferpool, equation, outbuf, lhs, rhs, geom)
    ops, rhs, geom, _ = _with_dense_kernel(bufferpool, equation, rhs, geom, lhs, outbuf)
    return ops + _product_ops(bufferpool, equation, outbuf, lhs, rhs, geom)


def _with_dense_kernel(bufferpool, equation, rhs: Buffer, geom: 'K.ConvGeometry', lhs: Buffer, outbuf: Buffer, rhs_offset: int = 0):
    '''A kernel operand that is not laid out [ky, kx, in, out] with `out` contiguous (the swapped and reversed
    kernel of an input gradient, a transposed weight matrix, every other tap of a kernel) is copied into that
    layout first when it is no bigger than the activations: the GEMM kernel then reads it with 16-byte loads.
    Returns (ops, rhs, geometry, rhs offset).'''
    N, dense = geom.N, (geom.KW * geom.Cin * geom.N, geom.Cin * geom.N, geom.N, 1)
    if ((geom.ws == dense and rhs_offset % 4 == 0) or N % 4 != 0 or geom.M < 256 or geom.K * N > lhs.size + outbuf.size
            or builtins_min(geom.ws) < 0):
        return [], rhs, geom, rhs_offset
    position = bufferpool.op_counter
    bufferpool.op_counter -= 1                  #the copy lives at the equation's own position
    shape = (geom.KH, geom.KW, geom.Cin, N)
    copy  = bufferpool.new_temporary(np.float32, shape)
    bufferpool.op_counter = position
    op = Op(equation, chain=EwChain(copy, shape, EwOperand(rhs, rhs_offset, tuple(geom.ws)), []))
    return [op], copy, geom._replace(ws=dense), 0


def _dilated_input_convolution(bufferpool, equation, outbuf: Buffer, lhs: Buffer, rhs: Buffer, g: 'K.ConvGeometry'):
    '''A convolution over an lhs-dilated input (the input gradient of a strided convolution) touches a real
    input element only at every LH-th (LW-th) position, and which kernel taps meet real elements depends only
    on the output position modulo the dilation. So it is computed as LH * LW ordinary convolutions, one per
    residue class of output positions, each with the kernel taps of its class and writing every LH-th
    (LW-th) output position; classes that meet no tap are zero. The multiplications with the inserted zeros,
    (1 - 1 / (LH * LW)) of the total, are never issued.'''
    def classes(L, P, taps, out_size):
        result = []
        for a in range(builtins_min(L, out_size)):
            r0 = (P - a) % L
            n  = len(range(r0, taps, L))
            result.append((a, r0, n, (a + r0 - P) // L, -(-(out_size - a) // L)))     #class, first tap, taps, input shift, positions
        return result
    ops, launches = [], []
    rows, cols = classes(g.LH, g.PH, g.KH, g.Ho), classes(g.LW, g.PW, g.KW, g.Wo)
    if any(n == 0 for _, _, n, _, _ in rows + cols):
        ops.append(Op(equation, launch=K.fill(outbuf, 0)))
    for ah, rh, nh, ch, th in rows:
        for aw, rw, nw, cw, tw in cols:
            if nh == 0 or nw == 0:
                continue
            sub = g._replace(Ho=th, Wo=tw, KH=nh, KW=nw, PH=-ch, PW=-cw, LH=1, LW=1,
                             ws=(g.ws[0] * g.LH, g.ws[1] * g.LW, g.ws[2], g.ws[3]),
                             os=(g.os[0], g.os[1] * g.LH, g.os[2] * g.LW, g.os[3]))
            copies, kernel, sub, kernel_offset = _with_dense_kernel(bufferpool, equation, rhs, sub, lhs, outbuf,
                                                                    rh * g.ws[0] + rw * g.ws[1])
            ops += copies
            ops.append(Op(equation, launch=K.conv_gemm(outbuf, lhs, kernel, sub, rhs_offset=kernel_offset,
                                                       out_offset=ah * g.os[1] + aw * g.os[2])))
    return ops


def _as_kernel_gradient(g: 'K.ConvGeometry') -> tp.Optional['K.WgradGeometry']:
    '''The convolution autodiff emits for the kernel gradient of an NHWC / HWIO convolution: its "batch" is
    the forward input's (contiguous) feature dimension, its contraction runs over the forward batch and
    over the cotangent's pixels, which act as the window. Returns that convolution in forward terms, or
    None when the operands are laid out differently.'''
    images, C, N = g.Cin, g.batch, g.N
    x_dense   = g.xs == (1, g.W * C, C, g.H * g.W * C)
    cot_dense = g.ws == (g.KW * N, N, g.KH * g.KW * N, 1)
    out_dense = g.os == (N, g.Wo * C * N, C * N, 1)
    if not (x_dense and cot_dense and out_dense and g.LH == 1 and g.LW == 1 and images * g.KH * g.KW >= WGRAD_MIN_PIXELS):
        return None
    return K.WgradGeometry(images=images, Ho=g.KH, Wo=g.KW, H=g.H, W=g.W, C=C, KH=g.Ho, KW=g.Wo, N=N,
                           SH=g.DH, SW=g.DW, PH=g.PH, PW=g.PW, DH=g.SH, DW=g.SW)


# ------------------------------------------------------------------ reductions

def _reduction_identity_word(name: str, dtype, equation) -> int:
    kind = _kind(dtype)
    if name == 'reduce_sum':
        value = 0
    elif name == 'reduce_prod':
        value = 1
    elif name == 'reduce_max':
        value = {_F: -np.inf, _I: np.iinfo(np.int32).min, _U: 0, _B: 0}[kind]
    elif name == 'reduce_min':
        value = {_F: np.inf, _I: np.iinfo(np.int32).max, _U: np.iinfo(np.uint32).max, _B: 1}[kind]
    else:
        raise NotImplementedError(f'{name} over an empty range: {equation}')
    host = np.asarray(value, dtype=np.uint32 if kind == _B else dtype)
    return int(host.reshape(1).view(np.uint32)[0])


def reduce_op(bufferpool, equation):
    axes = tuple(int(a) for a in equation.params['axes'])
    if axes == ():
        return noop(bufferpool, equation)
    outvar, invar = equation.outvars[0], equation.invars[0]
    name   = equation.primitive.name
    inbuf  = bufferpool.get_buffer(invar)
    if name in ('reduce_or', 'reduce_and'):
        #jnp.any / jnp.all: on booleans (stored as 0 / 1) the maximum resp. minimum
        if _kind(inbuf.dtype) != _B:
            raise NotImplementedError(equation)
        name = 'reduce_max' if name == 'reduce_or' else 'reduce_min'
    outbuf = bufferpool.get_buffer(outvar, increment_op_counter=True)
    if _kind(inbuf.dtype) == _B and name not in ('reduce_max', 'reduce_min'):
        raise NotImplementedError(equation)
    if outbuf.size == 0:
        return []
    if inbuf.size == 0:
        #a reduction over no elements is the operation's identity (XLA's init value)
        return [Op(equation, launch=K.fill(outbuf, _reduction_identity_word(name, inbuf.dtype, equation)))]
    shape   = inbuf.shape
    strides = K.row_major_strides(shape)
    #merge neighbouring dims with the same role, drop size-1 dims
    groups = []
    for d, (s, st) in enumerate(zip(shape, strides)):
        if s == 1:
            continue
        red = d in axes
        if groups and groups[-1][0] == red:
            groups[-1] = (red, groups[-1][1] * s, st)
        else:
            groups.append((red, s, st))
    roles = [g[0] for g in groups]
    if not any(roles):
        #only size-1 dims are reduced: copy (argmax of a single element is index 0)
        if name in ('argmax', 'argmin'):
            return [Op(equation, launch=K.fill(outbuf, 0))]
        return [_copy_op(equation, outbuf, EwOperand(inbuf, 0, K.row_major_strides(outbuf.shape)))]
    if roles in ([True], [False, True], [True, False], [False, True, False]):
        outer = groups[0][1] if not roles[0] else 1
        inner = groups[-1][1] if not roles[-1] else 1
        R     = [g[1] for g in groups if g[0]][0]
        nsplit = K.plan_reduce_splits(outer, R, inner, name)
        partial = None
        if nsplit > 1:
            #scratch of this equation carries its position, like its operands
            bufferpool.op_counter -= 1
            partial = bufferpool.new_temporary(inbuf.dtype, (outer * nsplit * inner,))
            bufferpool.op_counter += 1
        ops = [Op(equation, launch=l) for l in K.reduce(outbuf, inbuf, outer, R, inner, name, partial, nsplit)]
        #the launch that reads the operand can take over the operand's element-wise producer (see fusion.py)
        ops[0].meta = ('reduce', outbuf, inbuf, outer, R, inner, name, partial, nsplit)
        return ops
    kept    = [(g[1], g[2]) for g in groups if not g[0]]
    reduced = [(g[1], g[2]) for g in groups if g[0]]
    return [Op(equation, launch=K.reduce_general(outbuf, inbuf, kept, reduced, name))]


reduce_max = reduce_min = reduce_sum = reduce_prod = argmin = argmax = reduce_or = reduce_and = reduce_op


def _reduce_window(bufferpool, equation, op_name):
    params = equation.params
    n = len(equation.outvars[0].aval.shape)
    if n > 4 or tuple(params.get('base_dilation') or (1,) * n) != (1,) * n:
        raise NotImplementedError(equation)
    inbuf  = bufferpool.get_buffer(equation.invars[0])
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    if _kind(inbuf.dtype) == _B:
        raise NotImplementedError(equation)
    if outbuf.size == 0:
        return []
    launch = K.pool(outbuf, inbuf, op_name, params['window_dimensions'], params['window_strides'],
                    [p[0] for p in params['padding']], tuple(params.get('window_dilation') or (1,) * n))
    return [Op(equation, launch=launch)]


def reduce_window_max(bufferpool, equation):
    '''Window maximum; positions outside the array count as -inf (reference: vkjax/ops.py:505-524,
    whose kernel used 0 there).'''
    return _reduce_window(bufferpool, equation, 'reduce_max')


def reduce_window_sum(bufferpool, equation):
    return _reduce_window(bufferpool, equation, 'reduce_sum')


# ------------------------------------------------------------------ indexing

def select_and_scatter_add(bufferpool, equation):
    '''Gradient of reduce_window_max / min as autodiff emits it: operands (source, operand),
    select_prim ge or le.'''
    params = equation.params
    select = getattr(params['select_prim'], 'name', str(params['select_prim']))
    if select not in ('ge', 'le'):
        raise NotImplementedError(equation)
    source, operand = [bufferpool.get_buffer(v) for v in equation.invars]
    if _kind(operand.dtype) != _F or _kind(source.dtype) != _F:
        raise NotImplementedError(equation)
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    if outbuf.size == 0:
        return []
    pad_low = [int(lo) for lo, _ in params['padding']]
    position = bufferpool.op_counter
    bufferpool.op_counter -= 1                  #the temporary lives at the equation's own position
    selected = bufferpool.new_temporary(np.uint32, source.shape)
    bufferpool.op_counter = position
    launches = K.select_scatter_add(outbuf, source, operand, selected, 'reduce_max' if select == 'ge' else 'reduce_min',
                                    params['window_dimensions'], params['window_strides'], pad_low)
    return [Op(equation, launch=l) for l in launches]


def pad(bufferpool, equation):
    inbuf, value = [bufferpool.get_buffer(v) for v in equation.invars]
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    if outbuf.size == 0:
        return []
    return [Op(equation, launch=K.pad(outbuf, inbuf, value, equation.params['padding_config']))]


def _index_mode(params) -> str:
    '''Name of the equation's GatherScatterMode ('CLIP', 'FILL_OR_DROP', 'PROMISE_IN_BOUNDS'), or '' when the
    front-end (old jax versions, the reference's era) has no such parameter.'''
    mode = params.get('mode')
    if mode is None:
        return ''
    name = str(getattr(mode, 'name', mode)).upper().rsplit('.', 1)[-1]
    return {'FILL': 'FILL_OR_DROP', 'DROP': 'FILL_OR_DROP'}.get(name, name)      #the strings jax accepts for the enum


def gather(bufferpool, equation):
    params = equation.params
    #start indices are clamped so that the slice stays inside the operand: that is XLA's gather, CLIP, and what
    #XLA makes of PROMISE_IN_BOUNDS; under FILL_OR_DROP a slice that does not fit reads as fill_value instead
    mode = _index_mode(params)
    if mode not in ('', 'CLIP', 'PROMISE_IN_BOUNDS', 'FILL_OR_DROP'):
        raise NotImplementedError(f'gather with mode={params["mode"]}: {equation}')
    dn     = params['dimension_numbers']
    offset_dims, collapsed, start_index_map = (tuple(dn.offset_dims), tuple(dn.collapsed_slice_dims), tuple(dn.start_index_map))
    slice_sizes = tuple(int(s) for s in params['slice_sizes'])
    operand, indices = [bufferpool.get_buffer(v) for v in equation.invars]
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    if outbuf.size == 0:
        return []
    if _kind(indices.dtype) not in (_I, _U):
        raise NotImplementedError(equation)
    fill = _gather_fill_word(operand.dtype, params.get('fill_value')) if mode == 'FILL_OR_DROP' else None
    op_rank, out_rank = len(operand.shape), len(outbuf.shape)
    n_batch = len(indices.shape) - 1
    #whole trailing slices addressed by one index on the leading axis: a row gather
    is_rows = (collapsed == (0,) and start_index_map == (0,) and indices.shape[-1] == 1 and slice_sizes[0] == 1
               and slice_sizes[1:] == tuple(operand.shape[1:])
               and offset_dims == tuple(range(n_batch, out_rank)))
    if is_rows:
        row_len = int(np.prod(operand.shape[1:], dtype=np.int64))
        n_idx   = int(np.prod(indices.shape[:-1], dtype=np.int64))
        known   = getattr(indices, 'constant_value', None)
        if n_idx == 1 and known is not None and operand.shape[0] > 0 and (fill is None or 0 <= int(np.asarray(known).reshape(-1)[0]) < operand.shape[0]):
            #one row whose number is known when the program is built (`keys[1]` of a split key, a static `x[3]`, which
            #old jax versions trace as a gather with a constant index): a copy of that row, which the consumer's
            #fusion can read in place. Clamped like any gather.
            row = builtins_min(builtins_max(int(np.asarray(known).reshape(-1)[0]), 0), operand.shape[0] - 1)
            return [_copy_op(equation, outbuf, EwOperand(operand, row * row_len, K.row_major_strides(outbuf.shape)))]
        return [Op(equation, launch=K.gather_rows(outbuf, operand, indices, n_idx, row_len, operand.shape[0], fill=fill))]
    return [Op(equation, launch=K.gather_general(outbuf, operand, indices, offset_dims, collapsed, start_index_map, slice_sizes, fill=fill))]


def _gather_fill_word(dtype, fill_value) -> int:
    '''The 32-bit pattern a FILL_OR_DROP gather returns for slices outside the operand: the equation's fill_value,
    or jax's default (NaN, the most negative signed integer, the largest unsigned one, True).'''
    dtype = np.dtype(dtype)
    if fill_value is None:
        fill_value = (np.nan if dtype.kind == 'f' else np.iinfo(dtype).min if dtype.kind == 'i'
                      else np.iinfo(dtype).max if dtype.kind == 'u' else True)
    if dtype.kind == 'b':
        return int(bool(fill_value))
    return int(np.asarray(fill_value, dtype).reshape(1).view(np.uint32)[0])


def scatter_add(bufferpool, equation):
    '''General XLA scatter-add (the reference implements two fixed patterns, vkjax/ops.py:404-433).
    The operand is copied to the output first, then updates are added with HBM atomics.'''
    #updates whose window does not fit into the operand are dropped: XLA's scatter, FILL_OR_DROP, and what holds
    #trivially under PROMISE_IN_BOUNDS; CLIP moves such windows inside instead
    if _index_mode(equation.params) not in ('', 'FILL_OR_DROP', 'PROMISE_IN_BOUNDS', 'CLIP'):
        raise NotImplementedError(f'scatter-add with mode={equation.params["mode"]}: {equation}')
    clip = _index_mode(equation.params) == 'CLIP'
    dn = equation.params['dimension_numbers']
    uwd, iwd, sd2od = tuple(dn.update_window_dims), tuple(dn.inserted_window_dims), tuple(dn.scatter_dims_to_operand_dims)
    operand, indices, updates = [bufferpool.get_buffer(v) for v in equation.invars]
    outbuf = bufferpool.get_buffer(equation.outvars[0])
    #scratch arrays of this equation must carry its position, like its inputs and outputs: the
    #position advances only after they have been created
    counter_before = bufferpool.op_counter
    bufferpool.op_counter += 1
    if _kind(operand.dtype) == _B or _kind(indices.dtype) not in (_I, _U):
        raise NotImplementedError(equation)
    if outbuf.size == 0:
        return []
    copy = _copy_op(equation, outbuf, EwOperand(operand, 0, K.row_major_strides(outbuf.shape)))
    if updates.size == 0:
        return [copy]
    n_batch = len(indices.shape) - 1
    is_rows = (iwd == (0,) and sd2od == (0,) and indices.shape[-1] == 1
               and uwd == tuple(range(n_batch, len(updates.shape)))
               and tuple(updates.shape[n_batch:]) == tuple(operand.shape[1:]))
    if is_rows:
        row_len = int(np.prod(operand.shape[1:], dtype=np.int64))
        n_idx   = int(np.prod(indices.shape[:-1], dtype=np.int64))
        n_rows  = operand.shape[0]
        #(up to 2**27 updates: the overflow table of the sorted form has at least two slots of eight bytes per update)
        if n_idx * row_len >= K.CHOICES.scatter_sort_threshold and n_idx <= 2**27 and n_rows < 2**31 - 1:
            #large: bucket the updates by row and sum each bucket (no atomics on the data, no copy of the operand)
            bufferpool.op_counter = counter_before
            count = bufferpool.zeroed_scratch(n_rows + 1, 'counters')      #every evaluation leaves the counters zero again
            count.accesses.append(counter_before)
            table = bufferpool.zeroed_scratch(2 * K.scatter_table_slots(n_idx), 'overflow')      #the overflow table: likewise
            table.accesses.append(counter_before)
            gathered = bufferpool.new_temporary(np.dtype('uint32'), (n_idx,))
            sorted_  = bufferpool.new_temporary(np.dtype('uint32'), (n_idx,))
            cap   = K.choose_scatter_bucket_cap(n_idx, n_rows, row_len)
            fixed = bufferpool.new_temporary(np.dtype('uint32'), (n_rows * cap,)) if cap else None
            uniform = _uniform_constant(operand)
            if uniform is not None:
                #a table that is a constant filled with one value (zeros, usually) is not read at all
                source = bufferpool.scalar_constant(uniform, operand.dtype)
                source.accesses.append(counter_before)
            else:
                source = operand
            bufferpool.op_counter = counter_before + 1
            launches = K.scatter_add_rows_sorted(outbuf, source, indices, updates, count, table, gathered, sorted_, n_idx, row_len, n_rows,
                                                 operand_is_scalar=uniform is not None, clip=clip, fixed=fixed, cap=cap)
            return [Op(equation, launch=l) for l in launches]
        ops = [copy, Op(equation, launch=K.scatter_add_rows(outbuf, indices, updates, n_idx, row_len, n_rows, clip=clip))]
        return ops
    return [copy, Op(equation, launch=K.scatter_add_general(outbuf, indices, updates, uwd, iwd, sd2od, clip=clip))]


def _uniform_constant(b):
    '''The value of a build-time constant whose elements are all the same, else None.'''
    value = getattr(b, 'constant_value', None)
    if value is None:
        return None
    value = np.asarray(value)
    if value.size == 0 or value.size != b.size:
        return None
    first = value.reshape(-1)[0]
    #bit-wise comparison: -0.0 is not 0.0 here, and a NaN-filled table is uniform
    return first if (value.reshape(-1).view(np.uint8).reshape(value.size, -1) == np.asarray(first).reshape(1).view(np.uint8)).all() else None


# ------------------------------------------------------------------ rng

def threefry2x32(bufferpool, equation):
    inbufs  = [bufferpool.get_buffer(v) for v in equation.invars]
    outbufs = [bufferpool.get_buffer(v) for v in equation.outvars]
    bufferpool.op_counter += 1
    assert inbufs[0].shape  == inbufs[1].shape
    assert inbufs[2].shape  == inbufs[3].shape
    assert outbufs[0].shape == outbufs[1].shape
    assert all(_kind(b.dtype) == _U for b in inbufs + outbufs)
    key_is_scalar = inbufs[0].shape in [(), (1,)]
    if not key_is_scalar:
        assert inbufs[0].shape == inbufs[2].shape
    if outbufs[0].size == 0:
        return []
    return [Op(equation, launch=K.threefry2x32(*outbufs, *inbufs, key_is_scalar=key_is_scalar),
               meta=('threefry', outbufs, inbufs, key_is_scalar))]


# Key primitives of newer jax versions (jax/_src/prng.py): jax.random.* is traced as
# random_wrap -> random_bits / random_split / random_fold_in -> random_unwrap and the backend expands
# them. Only the threefry implementation and single (unbatched) keys are supported. The counter
# layout follows jax's `jax_threefry_partitionable` setting:
#   original       bits = threefry_2x32(key, iota(n)) (halves layout, odd sizes padded with a zero counter)
#                  split = threefry_2x32(key, iota(2 num)).reshape(num, 2)
#   partitionable  the counter of element i is its 64-bit flat index (high word, low word);
#                  bits = y0 ^ y1, split = stack(y0, y1)

#None: follow jax's configuration where jax can be imported, otherwise the original layout
THREEFRY_PARTITIONABLE: tp.Optional[bool] = None


def threefry_partitionable() -> bool:
    if THREEFRY_PARTITIONABLE is not None:
        return bool(THREEFRY_PARTITIONABLE)
    try:
        import jax
        return bool(jax.config.jax_threefry_partitionable)
    except (ImportError, AttributeError):
        return False


def _single_key(bufferpool, equation) -> Buffer:
    keyvar = equation.invars[0]
    if tuple(keyvar.aval.shape) != ():
        raise NotImplementedError(f'batched keys are not supported: {equation}')
    core.key_words_shape(keyvar.aval.dtype)            #raises for implementations other than threefry
    return bufferpool.get_buffer(keyvar)


def _stream_op(equation, outbuf, layout, key, h, c0, c1, n):
    k0, k1 = (key, 0), (key, 1)
    return Op(equation, launch=K.threefry_stream(outbuf, k0, k1, h, c0, c1, [], layout=layout, n=n),
              meta=('random_stream', outbuf, layout, k0, k1, h, c0, c1, n))


def random_bits(bufferpool, equation):
    if int(equation.params['bit_width']) != 32:
        raise NotImplementedError(f'only 32-bit random words exist on the device: {equation}')
    key    = _single_key(bufferpool, equation)
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    n      = outbuf.size
    if n == 0:
        return []
    if n >= 2**32:
        raise NotImplementedError(equation)
    if threefry_partitionable():
        return [_stream_op(equation, outbuf, 'xor', key, n, 0, 0, n)]
    h = (n + 1) // 2
    return [_stream_op(equation, outbuf, 'halves', key, h, 0, h, n)]


def random_split(bufferpool, equation):
    key    = _single_key(bufferpool, equation)
    outbuf = bufferpool.get_buffer(equation.outvars[0], increment_op_counter=True)
    num    = outbuf.size // 2
    if num == 0:
        return []
    if threefry_partitionable():
        return [_stream_op(equation, outbuf, 'pairs', key, num, 0, 0, 2 * num)]
    return [_stream_op(equation, outbuf, 'halves', key, num, 0, num, 2 * num)]


def _inline_traced(bufferpool, equation, function, *example_arguments):
    '''Lowers an equation through its expansion into primitives that exist here.'''
    from . import minijax
    closed = minijax.make_jaxpr(function)(*example_arguments)
    return _inline_call(bufferpool, equation, closed, closed.consts)


def random_fold_in(bufferpool, equation):
    '''fold_in(key, data) = threefry_2x32(key, [0, data]) in both counter layouts.'''
    from .minijax import lax, numpy as mnp
    _single_key(bufferpool, equation)

    def expansion(key, data):
        k0 = lax.reshape(lax.slice(key, (0,), (1,)), ())
        k1 = lax.reshape(lax.slice(key, (1,), (2,)), ())
        y0, y1 = lax.threefry2x32(k0, k1, np.zeros((1,), np.uint32), mnp.reshape(data, (1,)))
        return mnp.concatenate([y0, y1])
    return _inline_traced(bufferpool, equation, expansion, np.zeros(2, np.uint32), np.uint32(0))


def random_seed(bufferpool, equation):
    '''Key words (seed >> 32, seed & 0xFFFFFFFF) of a 32-bit seed: (0, seed).'''
    from .minijax import lax, numpy as mnp
    core.key_words_shape(equation.outvars[0].aval.dtype)
    seedvar = equation.invars[0]
    shape   = tuple(seedvar.aval.shape)
    dtype   = core.canonicalize_dtype(seedvar.aval.dtype)
    if _kind(dtype) not in (_I, _U):
        raise NotImplementedError(equation)

    def expansion(seed):
        low = mnp.reshape(lax.convert_element_type(seed, np.uint32), shape + (1,))
        return mnp.concatenate([np.zeros(shape + (1,), np.uint32), low], axis=-1)
    return _inline_traced(bufferpool, equation, expansion, np.zeros(shape, dtype))


import builtins as _builtins
builtins_max = _builtins.max
builtins_min = _builtins.min
