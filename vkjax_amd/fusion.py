'''Peephole fusion over the op list of one program.

The reference issues one dispatch per jaxpr equation, plus one per implicit broadcast
(vkjax/kompute_jaxpr_interpreter.py:55-60, vkjax/ops.py:84-86), so a batch-norm + ReLU after a
convolution costs five full-size round trips through memory. Here two rewrites are applied
after the primitive dispatch and before storage is assigned:

  * chain + chain: an element-wise op whose input is the sole use of the previous element-wise
    op's full-size result continues that op's chain (one launch, intermediate never stored);
  * conv/dot + chain: add / sub / mul / div / max / min steps whose other operand is a scalar, a
    per-feature vector or a full-size tensor become the epilogue of the implicit-GEMM kernel and
    are applied to the accumulators before the only store.

Both keep the arithmetic and its order exactly as in the unfused program. A fused op sits at
the position of its last member, so the lifetimes of the earlier members' inputs are extended
to that position, and the skipped intermediates get no storage.
'''
import collections
import typing as tp

from . import kernels as K
from .kernels import EW, EwChain, EwOperand, EwStep


class FusedEquation(tuple):
    '''Label of a fused op: the equations it covers, in order.'''
    def __repr__(self):
        return ' ; '.join(str(getattr(e, 'primitive', e)) for e in self)


_EPILOGUE_OPS = {EW[n] for n in ('ADD_F', 'SUB_F', 'MUL_F', 'DIV_F', 'MAX_F', 'MIN_F')}
_SELECTS      = {EW['SEL_P'], EW['SEL_T'], EW['SEL_F']}


def _reads(op) -> tp.List:
    '''Buffers an op reads (for plain launches: every buffer it touches).'''
    if op.chain is not None:
        return [o.buffer for o in op.chain.operands() if o is not None]
    if op.conv is not None:
        out, lhs, rhs, geom, epilogue = op.conv
        return [lhs, rhs] + [e.operand for e in epilogue]
    return [b for b, _ in op.launch.buffers if b is not None]


def _out(op):
    if op.chain is not None:
        return op.chain.out
    if op.conv is not None:
        return op.conv[0]
    return None


def _is_full_contiguous(operand: EwOperand, shape) -> bool:
    return (operand.offset == 0 and tuple(operand.buffer.shape) == tuple(shape)
            and tuple(operand.strides) == K.row_major_strides(shape))


def _label(*ops):
    eqs = []
    for op in ops:
        eqs += list(op.equation) if isinstance(op.equation, FusedEquation) else [op.equation]
    return FusedEquation(eqs)


def _continuation_steps(chain: EwChain, producer_out) -> tp.Optional[tp.List[EwStep]]:
    '''The steps of `chain` re-expressed as a continuation of a chain that produced
    `producer_out`, or None if that value is not consumed as a plain full-size input exactly once.'''
    operands = chain.operands()
    hits = [k for k, o in enumerate(operands) if o is not None and o.buffer._placeholder is producer_out._placeholder]
    if len(hits) != 1:
        return None
    k = hits[0]
    if not _is_full_contiguous(operands[k], chain.shape):
        return None
    if k == 0:
        return list(chain.steps)
    if k == 1 and chain.steps[0].op not in _SELECTS and chain.steps[0].op != EW['NOP']:
        #acc = op(first, produced)  ->  acc = produced ; acc = op(first as operand on the other side, acc)
        s = chain.steps[0]
        return [EwStep(s.op, chain.first, not s.operand_left, s.imm)] + list(chain.steps[1:])
    return None


def _epilogue_steps(steps: tp.Sequence[EwStep], geom: K.ConvGeometry, out_shape) -> tp.Optional[tp.List[K.ConvEpilogueStep]]:
    result = []
    feature_dims = [d for d, s in enumerate(K.row_major_strides(out_shape)) if s == geom.os[3] and out_shape[d] == geom.N]
    for s in steps:
        if s.op not in _EPILOGUE_OPS or s.operand is None:
            return None
        o = s.operand
        if o.buffer.size == 1 and o.offset == 0:
            kind = 1
        elif _is_full_contiguous(o, out_shape):
            kind = 3
        elif (o.offset == 0 and o.buffer.size == geom.N and feature_dims
              and all((st == 1 if d == feature_dims[-1] else st == 0 or out_shape[d] == 1) for d, st in enumerate(o.strides))):
            kind = 2
        else:
            return None
        result.append(K.ConvEpilogueStep(s.op, kind, o.buffer, s.operand_left))
    return result


def fuse_ops(all_ops, bufferpool, outvars):
    from .ops import Op
    uses = collections.Counter()
    for op in all_ops:
        for b in _reads(op):
            uses[id(b._placeholder)] += 1
    for v in outvars:
        b = bufferpool.get_buffer(v)
        if b is not None:
            uses[id(b._placeholder)] += 2          #program outputs are never elided
            b.accesses.pop()                       #the lookup above is not a device access

    result: tp.List[tp.Optional[Op]] = []
    producer: tp.Dict[int, int] = {}               #placeholder id -> position in `result` of the op that wrote it

    def extend_lifetimes(op, index):
        for b in _reads(op):
            b.accesses.append(index)

    for op in all_ops:
        fused = None
        if op.chain is not None:
            for cand in [o for o in op.chain.operands()[:2] if o is not None]:
                pid = id(cand.buffer._placeholder)
                pos = producer.get(pid)
                if pos is None or uses[pid] != 1 or result[pos] is None:
                    continue
                prod = result[pos]
                steps = _continuation_steps(op.chain, _out(prod))
                if steps is None:
                    continue
                if prod.chain is not None:
                    if prod.chain.shape != op.chain.shape or 1 + len(prod.chain.steps) + len(steps) > K.EW_MAX_STEPS:
                        continue
                    chain = EwChain(op.chain.out, op.chain.shape, prod.chain.first, list(prod.chain.steps) + steps)
                    fused = Op(_label(prod, op), chain=chain)
                else:
                    out, lhs, rhs, geom, epilogue = prod.conv
                    if tuple(out.shape) != tuple(op.chain.shape) or len(epilogue) + len(steps) > K.CONV_MAX_EPI:
                        continue
                    extra = _epilogue_steps(steps, geom, op.chain.shape)
                    if extra is None:
                        continue
                    fused = Op(_label(prod, op), conv=(op.chain.out, lhs, rhs, geom, list(epilogue) + extra))
                fused.index = op.index
                extend_lifetimes(prod, op.index)
                _out(prod)._placeholder.elided = True
                result[pos] = None
                del producer[pid]
                break
        new = fused if fused is not None else op
        result.append(new)
        out = _out(new)
        if out is not None:
            producer[id(out._placeholder)] = len(result) - 1
    return [op for op in result if op is not None]
