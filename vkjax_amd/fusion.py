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
        reads = [lhs, rhs] + [e.operand for e in epilogue if e.operand is not None and e.op not in (K.CONV_TAP, K.CONV_SOFTMAX)]
        for e in epilogue:
            if e.derived is not None:
                reads += [e.derived.first] + [st[1] for st in e.derived.steps if st[1] is not None]
        return reads
    if op.meta is not None:
        if op.meta[0] == 'iota':
            return []
        if op.meta[0] == 'concat_part':
            return [op.meta[2]]
        if op.meta[0] == 'threefry':
            return list(op.meta[2])
        if op.meta[0] in ('random_stream', 'reduce'):
            return [b for b, _ in op.launch.buffers[1:] if b is not None]
        if op.meta[0] == 'softmax':
            return [op.meta[2]]
    return [b for b, _ in op.launch.buffers if b is not None]


def _out(op):
    if op.chain is not None:
        return op.chain.out
    if op.conv is not None:
        return op.conv[0]
    return None


def _walks_densely(strides, shape) -> bool:
    '''The strides are the row-major ones of `shape`; the stride of a dimension of size 1 is never used and may be anything.'''
    return len(strides) == len(shape) and all(n == 1 or s == r for s, r, n in zip(strides, K.row_major_strides(shape), shape))


def _through_copy(operand: EwOperand, copy: EwChain, shape) -> tp.Optional[EwOperand]:
    '''`operand` (of a chain over `shape`) reads the result of `copy`, a chain without steps, i.e. result[c] =
    source[offset + c . strides] over copy.shape. When every dimension the operand walks is one dimension of the
    copy's result (a transposition, a slice, a broadcast of it, or the whole of it), the operand that reads the
    copy's source directly is returned: the two index maps composed. None otherwise.'''
    src, cshape = copy.first, tuple(copy.shape)
    if operand.buffer.size != np_prod(cshape) or len(operand.strides) != len(shape):
        return None
    dense = K.row_major_strides(cshape)
    rest, start = operand.offset, []
    for e in range(len(cshape)):
        start.append(rest // dense[e])
        rest -= start[-1] * dense[e]
    if rest:
        return None
    strides, taken = [], set()
    for n, s in zip(shape, operand.strides):
        if n == 1 or s == 0:
            strides.append(0)
            continue
        dims = [e for e in range(len(cshape)) if cshape[e] > 1 and dense[e] == s and e not in taken]
        if len(dims) != 1 or start[dims[0]] + n > cshape[dims[0]]:
            return None
        taken.add(dims[0])
        strides.append(src.strides[dims[0]])
    return EwOperand(src.buffer, src.offset + sum(a * b for a, b in zip(start, src.strides)), tuple(strides))


def _is_full_contiguous(operand: EwOperand, shape) -> bool:
    return operand.offset == 0 and tuple(operand.buffer.shape) == tuple(shape) and _walks_densely(operand.strides, shape)


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
    last_reader: tp.Dict[int, int] = {}            #placeholder id -> position in `result` of the last op that read it

    def extend_lifetimes(op, index):
        for b in _reads(op):
            b.accesses.append(index)

    def fold_copies(op):
        '''An operand that is the full-size result of a pure copy (a broadcast, slice, transpose or reversal
        that was given a launch of its own) is read through that copy's strides instead; the copy goes away
        once nothing reads its result any more.'''
        chain, changed = op.chain, False
        first, steps = chain.first, list(chain.steps)
        for k, o in enumerate(chain.operands()):
            if o is None:
                continue
            pid = id(o.buffer._placeholder)
            pos = producer.get(pid)
            prod = result[pos] if pos is not None else None
            if prod is None or prod.chain is None or prod.chain.steps:
                continue
            source = _through_copy(o, prod.chain, chain.shape)
            if source is None:
                continue
            if k == 0:
                first = source
            else:
                steps[k - 1] = steps[k - 1]._replace(operand=source)
            changed = True
            uses[pid] -= 1
            uses[id(source.buffer._placeholder)] += 1
            source.buffer.accesses.append(op.index)
            if uses[pid] == 0:
                uses[id(source.buffer._placeholder)] -= 1
                _out(prod)._placeholder.elided = True
                result[pos] = None
                del producer[pid]
        if changed:
            new = Op(op.equation, chain=EwChain(chain.out, chain.shape, first, steps))
            new.index = op.index
            return new
        return op

    def conv_with_second_result(prod, op, pid):
        out, lhs, rhs, geom, epilogue = prod.conv
        #the merged launch stands where the chain stood: nothing in between may have read the convolution's result
        if last_reader.get(pid, -1) > producer[pid]:
            return None
        steps = _continuation_steps(op.chain, out)
        if steps is None or tuple(out.shape) != tuple(op.chain.shape) or op.chain.out.size != out.size:
            return None
        extra = _epilogue_steps(steps, geom, op.chain.shape)
        if extra is None or not K.conv_tap_supported(epilogue, extra) or K.conv_is_dense_rows(lhs, geom):
            return None
        tap = K.ConvEpilogueStep(K.CONV_TAP, 3, out)
        fused = Op(_label(prod, op), conv=(op.chain.out, lhs, rhs, geom, list(epilogue) + [tap] + extra))
        fused.index = op.index
        extend_lifetimes(prod, op.index)
        out.accesses.append(op.index)
        uses[pid] -= 1
        return fused

    for op in all_ops:
        fused = None
        if op.chain is not None:
            op = fold_copies(op)
            for cand in [o for o in op.chain.operands()[:2] if o is not None]:
                pid = id(cand.buffer._placeholder)
                pos = producer.get(pid)
                if pos is None or result[pos] is None:
                    continue
                prod = result[pos]
                if uses[pid] != 1:
                    #a convolution whose result something else reads as well can still take the chain over,
                    #by storing both: its result as it was, and the chain's
                    if prod.conv is not None and prod.conv[3].k_splits == 1 and _out(prod)._placeholder is cand.buffer._placeholder:
                        fused = conv_with_second_result(prod, op, pid)
                        if fused is not None:
                            result[pos] = None
                            break
                    continue
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
                    if geom.k_splits > 1 or tuple(out.shape) != tuple(op.chain.shape) or len(epilogue) + len(steps) > K.CONV_MAX_EPI:
                        continue
                    extra = _epilogue_steps(steps, geom, op.chain.shape)
                    if extra is None:
                        continue
                    if K.conv_is_dense_rows(lhs, geom) and not K.dense_rows_epilogue_supported(list(epilogue) + extra):
                        continue                                  #the chain stays a launch of its own
                    tap_at = [k for k, e in enumerate(epilogue) if e.op == K.CONV_TAP]
                    if tap_at and not K.conv_tap_supported(epilogue[:tap_at[0]], list(epilogue[tap_at[0] + 1:]) + extra):
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
        for b in _reads(new):
            last_reader[id(b._placeholder)] = len(result) - 1
        out = _out(new)
        if out is not None:
            producer[id(out._placeholder)] = len(result) - 1
        else:
            #a launch that is neither a chain nor a convolution may change its result buffer in place (scatter-add
            #accumulates into a copy of its operand): whoever produced that buffer before no longer describes what
            #it holds, so nothing behind this launch may be joined to that producer or read through it
            for b in _writes(new):
                producer.pop(id(b._placeholder), None)
    ops = fuse_random_streams([op for op in result if op is not None], bufferpool, outvars)
    ops = fuse_stream_chains(ops, bufferpool, outvars)
    ops = fuse_softmax(ops, bufferpool, outvars)
    ops = fuse_scale_relu_backward(ops, bufferpool, outvars)
    ops = fuse_reduce_prologues(ops, bufferpool, outvars)
    ops = fuse_reduce_scales(ops, bufferpool, outvars)
    ops = fuse_derived_epilogue_operands(ops, bufferpool, outvars)
    ops = fuse_index_wrap(ops, bufferpool, outvars)
    ops = fold_index_wrap(ops, bufferpool, outvars)
    ops = fuse_dense_softmax(ops, bufferpool, outvars)
    ops = remove_dead_ops(ops, bufferpool, outvars)
    return batch_small_chains(ops)


def fuse_softmax(ops, bufferpool, outvars):
    '''softmax over the last dimension as jax.nn.softmax spells it,

        m = reduce_max(x) ; e = exp(x - m) ; s = reduce_sum(e) ; y = e / s

    becomes one launch when m, e and s are used by nothing else. Same values, bit for bit: the fused kernel
    adds in the order of the row reduction it replaces.'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    pid  = lambda b: id(b._placeholder)
    removed, replacement = set(), {}

    def per_row(operand, shape):
        return (operand is not None and operand.offset == 0 and len(shape) >= 1
                and tuple(operand.strides) == K.row_major_strides(shape[:-1] + (1,))[:-1] + (0,))

    for i, R1 in enumerate(ops):
        if R1.meta is None or R1.meta[0] != 'reduce' or i + 3 >= len(ops):
            continue
        _, m, x, outer, rows, inner, name, _, nsplit = R1.meta
        C1, R2, C2 = ops[i + 1], ops[i + 2], ops[i + 3]
        if (name != 'reduce_max' or inner != 1 or nsplit != 1 or x.dtype != 'float32' or not 0 < rows < K.SOFTMAX_MAX_ROW
                or C1.chain is None or C2.chain is None or R2.meta is None or R2.meta[0] != 'reduce'):
            continue
        c1, c2 = C1.chain, C2.chain
        _, s, e, outer2, rows2, inner2, name2, _, nsplit2 = R2.meta
        flat = lambda shape: (int(np_prod(shape[:-1])), shape[-1]) if len(shape) else (1, 1)
        if (name2 != 'reduce_sum' or (outer2, rows2, inner2, nsplit2) != (outer, rows, 1, 1)
                or flat(c1.shape) != (outer, rows) or flat(c2.shape) != (outer, rows)
                or c1.first.buffer._placeholder is not x._placeholder or not _is_full_contiguous_any_shape(c1.first, c1.shape)
                or [st.op for st in c1.steps] != [EW['SUB_F'], EW['EXP_F']] or c1.steps[0].operand_left
                or c1.steps[0].operand.buffer._placeholder is not m._placeholder or not per_row(c1.steps[0].operand, c1.shape)
                or e._placeholder is not c1.out._placeholder
                or c2.first.buffer._placeholder is not c1.out._placeholder or not _is_full_contiguous_any_shape(c2.first, c2.shape)
                or [st.op for st in c2.steps] != [EW['DIV_F']] or c2.steps[0].operand_left
                or c2.steps[0].operand.buffer._placeholder is not s._placeholder or not per_row(c2.steps[0].operand, c2.shape)
                or uses[pid(m)] != 1 or uses[pid(c1.out)] != 2 or uses[pid(s)] != 1):
            continue
        members, last, arg_out = (R1, C1, R2, C2), C2, None
        #the arg-max over the same rows of the probabilities, right behind them: one more result of the same launch
        A = ops[i + 4] if i + 4 < len(ops) else None
        if (A is not None and A.meta is not None and A.meta[0] == 'reduce' and A.meta[6] == 'argmax' and A.meta[8] == 1
                and A.meta[2]._placeholder is c2.out._placeholder and tuple(A.meta[3:6]) == (outer, rows, 1) and A.meta[1].dtype == 'int32'):
            members, last, arg_out = (R1, C1, R2, C2, A), A, A.meta[1]
            removed.add(i + 3)
        fused = Op(_label(*members), launch=K.softmax_rows(c2.out, x, outer, rows, arg_out),
                   meta=('softmax', [c2.out] + ([arg_out] if arg_out is not None else []), x, outer, rows))
        fused.index = last.index
        x.accesses.append(last.index)
        if arg_out is not None:
            c2.out.accesses.append(last.index)
        for b in (m, c1.out, s):
            b._placeholder.elided = True
        removed |= {i, i + 1, i + 2}
        replacement[i + 3 + (arg_out is not None)] = fused
    return [replacement.get(i, op) for i, op in enumerate(ops) if i not in removed]


def fuse_index_wrap(ops, bufferpool, outvars):
    '''`select(x < 0, x + n, x)` on int32, the way tracing normalises an index that may count from the end, is two
    launches after chain fusion (x + n, and the comparison with the select, which needs x + n as a second full-size
    value). One opcode does it in one pass over x.'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    pid  = lambda b: id(b._placeholder)
    writer = {pid(op.chain.out): i for i, op in enumerate(ops) if op.chain is not None}
    same   = lambda a, b: a.buffer._placeholder is b.buffer._placeholder and a.offset == b.offset and tuple(a.strides) == tuple(b.strides)
    single = lambda o: o is not None and all(s == 0 for s in o.strides)
    removed, replacement = set(), {}
    for i, B in enumerate(ops):
        ch = B.chain
        if ch is None or [st.op for st in ch.steps] != [EW['LT_I'], EW['SEL_P'], EW['NOP']]:
            continue
        less, pick, carrier = ch.steps
        zero = getattr(less.operand.buffer, 'constant_value', None) if single(less.operand) else None
        if (less.operand_left or zero is None or np_prod(zero.shape) != 1 or int(zero.reshape(-1)[0]) != 0
                or not same(carrier.operand, ch.first) or not _is_full_contiguous_any_shape(pick.operand, ch.shape)):
            continue
        a = writer.get(pid(pick.operand.buffer))
        if a is None or a >= i or a in removed or uses[pid(pick.operand.buffer)] != 1:
            continue
        A = ops[a].chain
        if (tuple(A.shape) != tuple(ch.shape) or len(A.steps) != 1 or A.steps[0].op != EW['ADD_I'] or not single(A.steps[0].operand)
                or not same(A.first, ch.first) or A.out.dtype != ch.first.buffer.dtype):
            continue
        fused = Op(_label(ops[a], B), chain=EwChain(ch.out, ch.shape, ch.first, [EwStep(EW['WRAP_I'], A.steps[0].operand)]))
        fused.index = B.index
        A.steps[0].operand.buffer.accesses.append(B.index)
        pick.operand.buffer._placeholder.elided = True
        removed.add(a)
        replacement[i] = fused
    return [replacement.get(i, op) for i, op in enumerate(ops) if i not in removed]


def fold_index_wrap(ops, bufferpool, outvars):
    '''The normalised copy of an index array, `select(i < 0, i + n, i)` (one launch after fuse_index_wrap), is not made
    when everything that reads it is a row gather or a sorted row scatter-add: those kernels read the indices as they
    are and add n to the negative ones themselves.'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    pid  = lambda b: id(b._placeholder)
    removed, replacement = set(), {}
    for i, op in enumerate(ops):
        ch = op.chain
        if ch is None or len(ch.steps) != 1 or ch.steps[0].op != EW['WRAP_I'] or ch.steps[0].operand_left:
            continue
        o = ch.steps[0].operand
        amount = getattr(o.buffer, 'constant_value', None) if o is not None and all(st == 0 for st in o.strides) else None
        if (amount is None or np_prod(amount.shape) != 1 or not _is_full_contiguous_any_shape(ch.first, ch.shape)
                or str(ch.first.buffer.dtype) != 'int32' or str(ch.out.dtype) != 'int32'):
            continue
        readers = [j for j in range(len(ops)) if j != i and any(b._placeholder is ch.out._placeholder for b in _reads(ops[j]))]
        if not readers or len(readers) != uses[pid(ch.out)] or min(readers) < i:
            continue                                           #(also a result of the program: its uses count two more)
        ok = True
        for j in readers:
            r = replacement.get(j, ops[j])
            where = K.INDEX_WRAP_KERNELS.get(r.launch.kernel) if r.chain is None and r.conv is None else None
            places = [k for k, (b, _) in enumerate(r.launch.buffers) if b is not None and b._placeholder is ch.out._placeholder] if where else []
            ok = ok and where is not None and places == [where[0]]
        #the raw indices must still be what they were where the readers run
        last = max(readers)
        if not ok or any(w._placeholder is ch.first.buffer._placeholder for j in range(i + 1, last + 1) for w in _may_write(ops[j])):
            continue
        for j in readers:
            r = replacement.get(j, ops[j])
            launch = K.with_wrapped_index(r.launch, ch.first.buffer, ch.first.offset * 4, int(amount.reshape(-1)[0]))
            new = Op(_label(op, r), launch=launch, meta=r.meta)
            new.index = r.index
            ch.first.buffer.accesses.append(r.index)
            replacement[j] = new
        ch.out._placeholder.elided = True
        removed.add(i)
    return [replacement.get(i, op) for i, op in enumerate(ops) if i not in removed]


def fuse_dense_softmax(ops, bufferpool, outvars):
    '''A classifier's last layer: a product with at most 16 output features, read by nothing but the softmax launch
    right behind it, computes the softmax (and the arg-max that launch carries) on the row before it is stored
    (dense_rows_n16). The exponentials are added in the order of the separate launch: same values, bit for bit.'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    removed, replacement = set(), {}
    for i, (D, S) in enumerate(zip(ops, ops[1:])):
        if D.conv is None or S.meta is None or S.meta[0] != 'softmax':
            continue
        out, lhs, rhs, geom, epilogue = D.conv
        _, results, x, outer, rows = S.meta
        if (x._placeholder is not out._placeholder or uses[id(out._placeholder)] != 1 or (geom.M, geom.N) != (outer, rows)
                or any(e.op in (K.CONV_TAP, K.CONV_SOFTMAX) for e in epilogue)):
            continue
        steps = list(epilogue) + [K.ConvEpilogueStep(K.CONV_SOFTMAX, 0, results[1] if len(results) > 1 else None)]
        try:
            K.conv_gemm(results[0], lhs, rhs, geom, steps)
        except ValueError:
            continue                                   #another kernel serves this product
        fused = Op(_label(D, S), conv=(results[0], lhs, rhs, geom, steps))
        fused.index = S.index
        for b in _reads(D):
            b.accesses.append(S.index)
        out._placeholder.elided = True
        removed.add(i)
        replacement[i + 1] = fused
    return [replacement.get(i, op) for i, op in enumerate(ops) if i not in removed]


def np_prod(values) -> int:
    out = 1
    for v in values:
        out *= int(v)
    return out


def fuse_reduce_prologues(ops, bufferpool, outvars):
    '''A float column sum whose operand is, and is only, the result of `a * b` (b of the same shape or a
    vector over the columns) or of `-a` reads a (and b) itself and applies the step while loading: the
    pairs `multiply -> reduce_sum` and `negate -> reduce_sum` of a batch-norm backward pass lose a full-size
    array each. Values are unchanged (same products, same order of additions).'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    pid  = lambda b: id(b._placeholder)
    chain_writer = {pid(op.chain.out): i for i, op in enumerate(ops) if op.chain is not None}
    removed, replacement = set(), {}
    for i, R in enumerate(ops):
        if R.meta is None or R.meta[0] != 'reduce':
            continue
        _, out, inp, outer, rows, inner, name, partial, nsplit = R.meta
        w = chain_writer.get(pid(inp))
        if name != 'reduce_sum' or inner <= 1 or inp.dtype != 'float32' or w is None or w > i or w in removed or uses[pid(inp)] != 1:
            continue
        ch = ops[w].chain
        size = 1
        for d in ch.shape:
            size *= d
        if size != outer * rows * inner or len(ch.steps) != 1 or not _is_full_contiguous_any_shape(ch.first, ch.shape):
            continue
        step, prologue = ch.steps[0], None
        if step.op == EW['NEG_F'] and step.operand is None:
            prologue = ('neg', None)
        elif step.op == EW['MUL_F'] and step.operand is not None:
            o = step.operand
            if _is_full_contiguous_any_shape(o, ch.shape):
                prologue = ('mul', o.buffer)
            elif (o.offset == 0 and o.buffer.size == inner and ch.shape[-1] == inner
                  and tuple(o.strides) == (0,) * (len(ch.shape) - 1) + (1,)):
                prologue = ('mulv', o.buffer)
        if prologue is None:
            continue
        source = ch.first.buffer
        launch = K.reduce(out, source, outer, rows, inner, name, partial, nsplit, prologue=prologue)[0]
        fused  = Op(_label(ops[w], R), launch=launch, meta=None)
        fused.index = R.index
        for b in (source, prologue[1]):
            if b is not None:
                b.accesses.append(R.index)
        ch.out._placeholder.elided = True
        removed.add(w)
        replacement[i] = fused
    return [replacement.get(i, op) for i, op in enumerate(ops) if i not in removed]


def fuse_reduce_scales(ops, bufferpool, outvars):
    '''A float sum (one launch: not split into ranges) whose result is read once, by `sum / c` or `sum * c` with a
    single value c - a mean - stores the quotient / product itself: the element-wise launch behind it goes away. The
    division is the one the element-wise kernel would have made (same operands, same rounding).'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    pid  = lambda b: id(b._placeholder)
    removed, replacement = set(), {}
    for i, R in enumerate(ops):
        if R.meta is None or R.meta[0] != 'reduce' or i + 1 >= len(ops):
            continue
        _, out, inp, outer, rows, inner, name, partial, nsplit = R.meta
        if name != 'reduce_sum' or nsplit != 1 or inp.dtype != 'float32' or uses[pid(out)] != 1:
            continue
        #the reader: the next launch that reads the sum (nothing in between touches it, it has one use)
        C = next((j for j in range(i + 1, len(ops)) if any(b._placeholder is out._placeholder for b in _reads(ops[j]))), None)
        if C is None or ops[C].chain is None:
            continue
        #the sum is taken where its reader stood: its operand must still hold the same values there
        if any(w._placeholder is inp._placeholder for j in range(i + 1, C) for w in _may_write(ops[j])):
            continue
        ch = ops[C].chain
        if len(ch.steps) != 1 or ch.steps[0].operand is None:
            continue
        step = ch.steps[0]
        total, o = ch.first, step.operand
        if step.op == EW['MUL_F'] and o.buffer._placeholder is out._placeholder:
            total, o = o, ch.first                              #c * sum: the product is the same number
        elif step.op == EW['DIV_F'] and step.operand_left:
            continue                                            #c / sum
        kind = 'div' if step.op == EW['DIV_F'] else 'times' if step.op == EW['MUL_F'] else None
        if (kind is None or total.buffer._placeholder is not out._placeholder or not _is_full_contiguous_any_shape(total, ch.shape)
                or o.buffer.size != 1 or o.offset != 0 or ch.out.size != out.size):
            continue
        launch = K.reduce(ch.out, inp, outer, rows, inner, name, None, 1, post=(kind, o.buffer))[0]
        fused  = Op(_label(R, ops[C]), launch=launch, meta=None)
        fused.index = ops[C].index
        for b in (inp, o.buffer):
            b.accesses.append(ops[C].index)
        out._placeholder.elided = True
        removed.add(i)
        replacement[C] = fused
    return [replacement.get(i, op) for i, op in enumerate(ops) if i not in removed]


def fuse_scale_relu_backward(ops, bufferpool, outvars):
    '''The backward pass of a per-channel scale and shift followed by ReLU (a batch norm with fixed statistics
    and its activation), as reverse-mode differentiation emits it:

        m = select(ans > t, g, z) ; db = sum_rows(m) ; dx = m * k ; p = m * x ; dk = sum_rows(p)

    with m read by nothing else and p only by its sum, becomes ONE launch that reads ans, g and x once and
    writes dx and both column sums (their first stage, when the sums are split over row ranges). The sums are
    taken in the order of the reduce_cols launches they replace, so every value keeps its bits.'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    pid  = lambda b: id(b._placeholder)
    last_writer: tp.Dict[int, int] = {}
    for i, op in enumerate(ops):
        for b in _may_write(op):
            last_writer[pid(b)] = i
    readers: tp.Dict[int, tp.List[int]] = {}
    for i, op in enumerate(ops):
        for b in _reads(op):
            readers.setdefault(pid(b), []).append(i)
    single = lambda o: o is not None and o.offset == 0 and all(st == 0 for st in o.strides)
    removed, replacement = set(), {}

    def column_sum_of(i, buffer):
        '''(rows, inner, nsplit) when ops[i] is the float sum over the rows of `buffer` seen as [rows, inner].'''
        R = ops[i]
        if R.meta is None or R.meta[0] != 'reduce':
            return None
        _, out, inp, outer, rows, inner, name, partial, nsplit = R.meta
        if (name != 'reduce_sum' or outer != 1 or inner <= 1 or inp.dtype != 'float32' or inp._placeholder is not buffer._placeholder
                or rows * inner != buffer.size or not R.launch.kernel.startswith('reduce_cols_fsum_v')):
            return None
        return rows, inner, nsplit

    def select_chain(op):
        ch = op.chain
        return (ch is not None and [st.op for st in ch.steps] == [EW['GT_F'], EW['SEL_P'], EW['NOP']] and not ch.steps[0].operand_left
                and single(ch.steps[0].operand) and single(ch.steps[2].operand)
                and _is_full_contiguous_any_shape(ch.first, ch.shape) and _is_full_contiguous_any_shape(ch.steps[1].operand, ch.shape)
                and ch.out.dtype == 'float32' and ch.first.buffer.dtype == 'float32')

    chain_writer = {pid(op.chain.out): i for i, op in enumerate(ops) if op.chain is not None}
    for R1, first_sum in enumerate(ops):
        if first_sum.meta is None or first_sum.meta[0] != 'reduce':
            continue
        m = first_sum.meta[2]
        geometry = column_sum_of(R1, m)
        if geometry is None:
            continue
        rows, inner, nsplit = geometry
        C, P = None, None
        #several such backward passes can share one m (two branches of a residual block): each sum
        #goes with the first scaling and the first product that follow it
        for r in sorted(readers.get(pid(m), [])):
            other = ops[r].chain
            if r < R1 or other is None or [st.op for st in other.steps] != [EW['MUL_F']] or other.shape[-1] != inner or other.out.size != m.size:
                continue
            a, b = other.first, other.steps[0].operand
            if b is not None and a.buffer._placeholder is not m._placeholder:
                a, b = b, a
            if b is None or a.buffer._placeholder is not m._placeholder or not _is_full_contiguous_any_shape(a, other.shape):
                continue
            if _is_full_contiguous_any_shape(b, other.shape) and b.buffer.dtype == 'float32':
                P = P or (r, b.buffer)
            elif (b.offset == 0 and b.buffer.size == inner and b.buffer.dtype == 'float32'
                  and tuple(b.strides) == (0,) * (len(other.shape) - 1) + (1,)):
                C = C or (r, b.buffer)
        if C is None or P is None or C[0] == P[0]:
            continue
        p_out = ops[P[0]].chain.out
        R2 = [r for r in readers.get(pid(p_out), []) if column_sum_of(r, p_out) is not None]
        if uses[pid(p_out)] != 1 or len(R2) != 1 or column_sum_of(R2[0], p_out) != geometry:
            continue
        R2 = R2[0]
        if ops[R1].launch.kernel != ops[R2].launch.kernel or ops[R1].launch.params != ops[R2].launch.params:
            continue
        x, k = P[1], C[1]
        # with the select: where the select stood, if the three launches above are all that read its result
        M = chain_writer.get(pid(m))
        with_select = M is not None and M < min(R1, C[0], P[0]) and select_chain(ops[M]) and uses[pid(m)] == 3
        position = M if with_select else min(R1, C[0], P[0])
        involved = [R1, C[0], P[0], R2] + ([M] if with_select else [])
        if any(j in removed or j in replacement for j in involved):
            continue
        #everything the merged launch reads has to exist where the first of the launches it replaces stood
        sources = [x, k] + ([o.buffer for o in ops[M].chain.operands()] if with_select else [m])
        if any(last_writer.get(pid(b), -1) >= position for b in sources):
            continue
        dx, sum_m, sum_mx = ops[C[0]].chain.out, ops[R1].launch.buffers[0][0], ops[R2].launch.buffers[0][0]
        if with_select:
            ch = ops[M].chain
            launch = K.scale_relu_backward(ops[R1].launch, dx, sum_m, sum_mx, x, k, ch.steps[1].operand.buffer,
                                           select=(ch.first.buffer, ch.steps[0].operand.buffer, ch.steps[2].operand.buffer))
            m._placeholder.elided = True
        else:
            launch = K.scale_relu_backward(ops[R1].launch, dx, sum_m, sum_mx, x, k, m)
        fused = Op(_label(*[ops[j] for j in sorted(involved)]), launch=launch)
        fused.index = ops[position].index
        for b, _ in launch.buffers:
            if b is not None:
                b.accesses.append(fused.index)
        p_out._placeholder.elided = True
        removed |= set(involved) - {position}
        replacement[position] = fused
    return [replacement.get(i, op) for i, op in enumerate(ops) if i not in removed]


def _is_full_contiguous_any_shape(operand: EwOperand, shape) -> bool:
    '''The operand covers `shape` densely in row-major order (its buffer may carry another shape of the same size).'''
    size = 1
    for d in shape:
        size *= d
    return operand.offset == 0 and operand.buffer.size == size and _walks_densely(operand.strides, shape)


def fuse_stream_chains(ops, bufferpool, outvars):
    '''A launch that generates random words (random_bits lowered directly) followed by an
    element-wise chain over exactly those words whose operands are single values: the chain is
    applied by the generating kernel before its only store.'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    pid  = lambda b: id(b._placeholder)
    removed, replacement = set(), {}
    for si, S in enumerate(ops):
        if S.meta is None or S.meta[0] != 'random_stream':
            continue
        _, out, layout, key0, key1, h, c0, c1, n = S.meta
        if layout == 'pairs' or uses[pid(out)] != 1:
            continue
        for i in range(si + 1, len(ops)):
            op = ops[i]
            if not any(b._placeholder is out._placeholder for b in _reads(op)):
                continue
            ch = op.chain
            size = 1
            for d in (ch.shape if ch is not None else ()):
                size *= d
            if (ch is not None and ch.first.buffer._placeholder is out._placeholder and ch.first.offset == 0 and size == out.size
                    and tuple(ch.first.strides) == K.row_major_strides(ch.shape) and len(ch.steps) <= K.TF_MAX_STEPS
                    and all(st.op not in _SELECTS and st.op != EW['NOP'] and
                            (st.operand is None or (st.operand.buffer.size == 1 and st.operand.offset == 0)) for st in ch.steps)):
                fused = Op(_label(S, op), launch=K.threefry_stream(ch.out, key0, key1, h, c0, c1, list(ch.steps), layout=layout, n=n),
                           meta=('random_stream', ch.out, layout, key0, key1, h, c0, c1, n))
                fused.index = op.index
                for b in [key0[0], key1[0]] + [st.operand.buffer for st in ch.steps if st.operand is not None]:
                    b.accesses.append(fused.index)
                out._placeholder.elided = True
                removed.add(si)
                replacement[i] = fused
            break
    return [replacement.get(i, op) for i, op in enumerate(ops) if i not in removed]


def fuse_derived_epilogue_operands(ops, bufferpool, outvars):
    '''A per-feature operand of a convolution epilogue that is itself the result of a short chain over
    per-feature vectors and single values (the batch-norm scale gamma * rsqrt(var + eps)) is computed
    by the convolution kernel while it stages its epilogue operands; the chain's own launch and its
    result array go away. One such operand per convolution; the arithmetic is unchanged.'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    pid  = lambda b: id(b._placeholder)
    producer = {pid(op.chain.out): i for i, op in enumerate(ops) if op.chain is not None}
    allowed  = {EW[name] for name in K.CONV_DERIVED_OPS}
    unary    = {EW['NEG_F'], EW['RSQRT_F'], EW['SQRT_F']}
    removed  = set()
    result   = list(ops)
    for ci, op in enumerate(ops):
        if op.conv is None:
            continue
        out, lhs, rhs, geom, epilogue = op.conv
        N = geom.N
        if K.conv_is_dense_rows(lhs, geom):
            continue                                              #that kernel reads its epilogue operands as they are
        for ei, e in enumerate(epilogue):
            if e.kind != 2 or e.derived is not None or e.operand is None:
                continue
            pi = producer.get(pid(e.operand))
            if pi is None or pi >= ci or pi in removed or uses[pid(e.operand)] != 1:
                continue
            chain = ops[pi].chain
            n = 1
            for d in chain.shape:
                n *= d
            if n != N or not (1 <= len(chain.steps) <= K.CONV_MAX_DERIVED):
                continue

            def per_feature(o):
                '''(buffer) if the operand is one value or walks N contiguous values, else None'''
                if o.offset != 0:
                    return None
                if o.buffer.size == 1:
                    return o.buffer
                if o.buffer.size == N and tuple(o.strides) == K.row_major_strides(chain.shape):
                    return o.buffer
                return None
            first = per_feature(chain.first)
            steps = []
            for st in chain.steps:
                if st.op not in allowed or st.imm:
                    steps = None
                    break
                if st.op in unary:
                    if st.operand is not None:
                        steps = None
                        break
                    steps.append((st.op, None, False))
                else:
                    b = per_feature(st.operand) if st.operand is not None else None
                    if b is None:
                        steps = None
                        break
                    steps.append((st.op, b, bool(st.operand_left)))
            if first is None or steps is None:
                continue
            derived  = K.ConvDerivedOperand(first, tuple(steps))
            new_epi  = list(epilogue)
            new_epi[ei] = e._replace(operand=None, derived=derived)
            fused = Op(_label(ops[pi], op), conv=(out, lhs, rhs, geom, new_epi))
            fused.index = op.index
            for b in [first] + [st[1] for st in steps if st[1] is not None]:
                b.accesses.append(fused.index)
            e.operand._placeholder.elided = True
            removed.add(pi)
            result[ci] = fused
            break
    return [op for i, op in enumerate(result) if i not in removed]


def _writes(op) -> tp.List:
    if op.conv is not None:
        return [_out(op)] + [e.operand for e in op.conv[4] if e.op in (K.CONV_TAP, K.CONV_SOFTMAX) and e.operand is not None]
    if op.chain is not None:
        return [_out(op)]
    if op.meta is not None and op.meta[0] in ('iota', 'concat_part'):
        return [op.meta[1]]
    if op.meta is not None and op.meta[0] in ('threefry', 'softmax'):
        return list(op.meta[1])
    return [b for b, _ in op.launch.buffers[:1] if b is not None]      #kernels write their first argument


def remove_dead_ops(ops, bufferpool, outvars):
    '''Drops launches none of whose results is read by a later launch or returned (the unused half
    of a PRNG key split, for instance). The reference runs every equation; the values returned
    are the same.'''
    ops = list(ops)
    while True:
        uses = _use_counts(ops, bufferpool, outvars)
        #an accumulating kernel (scatter-add) also reads what it writes: such a use does not keep it alive
        dead = [i for i, op in enumerate(ops)
                if _writes(op) and all(uses[id(b._placeholder)] - sum(1 for r in _reads(op) if r._placeholder is b._placeholder) == 0
                                       for b in _writes(op))
                and not any(sum(1 for o in ops if any(w._placeholder is b._placeholder for w in _writes(o))) > 1 for b in _writes(op))]
        if not dead:
            return ops
        for i in dead:
            for b in _writes(ops[i]):
                b._placeholder.elided = True
        ops = [op for i, op in enumerate(ops) if i not in set(dead)]


def _use_counts(ops, bufferpool, outvars):
    uses = collections.Counter()
    for op in ops:
        for b in _reads(op):
            uses[id(b._placeholder)] += 1
    for v in outvars:
        b = bufferpool.get_buffer(v)
        if b is not None:
            uses[id(b._placeholder)] += 2
            b.accesses.pop()
    return uses


def fuse_random_streams(ops, bufferpool, outvars):
    '''Collapses the random-bits pipeline into one launch:

        c = iota(2h); a, b = threefry2x32(key, c[:h], c[h:]); bits = concatenate(a, b); out = chain(bits)

    where `chain` is an element-wise chain whose operands are single values (jax.random.uniform's
    shift / or / bitcast / sub / mul / add / max). The fused kernel generates the counters in
    registers and applies the chain before its only store, so of the iota, the two slices, the
    block function, the two concatenate copies and the chain only one write of the result remains.
    The arithmetic per element is unchanged.'''
    from .ops import Op
    uses = _use_counts(ops, bufferpool, outvars)
    pid  = lambda b: id(b._placeholder)
    writers = collections.defaultdict(list)          #placeholder id -> positions of the ops that write it
    for i, op in enumerate(ops):
        if op.chain is not None or op.conv is not None:
            writers[pid(_out(op))].append(i)
        elif op.meta is not None and op.meta[0] == 'iota':
            writers[pid(op.meta[1])].append(i)
        elif op.meta is not None and op.meta[0] == 'concat_part':
            writers[pid(op.meta[1])].append(i)
        elif op.meta is not None and op.meta[0] == 'threefry':
            for b in op.meta[1]:
                writers[pid(b)].append(i)
        else:
            for b, _ in op.launch.buffers[:1]:       #kernels write their first argument
                if b is not None:
                    writers[pid(b)].append(i)
    removed = set()
    replacement = {}
    for ti, T in enumerate(ops):
        if T.meta is None or T.meta[0] != 'threefry' or not T.meta[3]:
            continue
        (aa, ab), (key0, key1, x0, x1), _ = T.meta[1:]
        h = x0.size
        if aa.size != h or len(aa.shape) != 1:
            continue
        #counters: contiguous slices of one-dimensional uint32 iotas
        sources = []
        for xb in (x0, x1):
            w = writers.get(pid(xb), [])
            if len(w) != 1 or uses[pid(xb)] != 1:
                break
            C = ops[w[0]]
            if C.chain is None or C.chain.steps or len(C.chain.shape) != 1 or tuple(C.chain.first.strides) != (1,):
                break
            S  = C.chain.first.buffer
            ws = writers.get(pid(S), [])
            if len(ws) != 1 or ops[ws[0]].meta is None or ops[ws[0]].meta[0] != 'iota' or len(S.shape) != 1 or S.dtype != 'uint32':
                break
            sources.append((w[0], C.chain.first.offset, ws[0], S))
        if len(sources) != 2:
            continue
        #results: concatenated in order into one array
        if uses[pid(aa)] != 1 or uses[pid(ab)] != 1:
            continue
        cats = [i for i, op in enumerate(ops) if op.meta is not None and op.meta[0] == 'concat_part'
                and op.meta[2]._placeholder in (aa._placeholder, ab._placeholder)]
        if len(cats) != 2:
            continue
        m0, m1 = ops[cats[0]].meta, ops[cats[1]].meta
        if m0[2]._placeholder is not aa._placeholder:
            m0, m1 = m1, m0
        AC = m0[1]
        if (m0[2]._placeholder is not aa._placeholder or m1[2]._placeholder is not ab._placeholder or m1[1]._placeholder is not AC._placeholder
                or len(AC.shape) != 1 or AC.size != 2 * h or (m0[3], m0[4], m1[3], m1[4]) != (0, 0, 0, h)
                or sorted(writers[pid(AC)]) != sorted(cats)):
            continue
        #an element-wise chain on the bits whose operands are single values
        chain_pos = None
        if uses[pid(AC)] == 1:
            for i in range(max(cats) + 1, len(ops)):
                op = ops[i]
                if any(b._placeholder is AC._placeholder for b in _reads(op)):
                    ch = op.chain
                    n  = 1
                    for d in (ch.shape if ch is not None else ()):
                        n *= d
                    if (ch is not None and ch.first.buffer._placeholder is AC._placeholder and ch.first.offset == 0 and n == 2 * h
                            and tuple(ch.first.strides) == K.row_major_strides(ch.shape) and len(ch.steps) <= K.TF_MAX_STEPS
                            and all(st.op not in _SELECTS and st.op != EW['NOP'] and
                                    (st.operand is None or (st.operand.buffer.size == 1 and st.operand.offset == 0)) for st in ch.steps)):
                        chain_pos = i
                    break
        members = [sources[0][0], sources[1][0], ti] + cats + ([chain_pos] if chain_pos is not None else [])
        if removed & set(members):
            continue
        last  = max(members)
        out   = ops[chain_pos].chain.out if chain_pos is not None else AC
        steps = list(ops[chain_pos].chain.steps) if chain_pos is not None else []
        #a key word that is a one-element copy out of another array is read from there
        keys = []
        for kb in (key0, key1):
            w = writers.get(pid(kb), [])
            C = ops[w[0]] if len(w) == 1 else None
            if (C is not None and C.chain is not None and not C.chain.steps and kb.size == 1 and w[0] not in removed
                    and C.chain.first.buffer.dtype == kb.dtype):
                keys.append((C.chain.first.buffer, C.chain.first.offset))
                if uses[pid(kb)] == 1:
                    members.append(w[0])
                    kb._placeholder.elided = True
            else:
                keys.append((kb, 0))
        fused = Op(_label(*[ops[i] for i in sorted(members)]),
                   launch=K.threefry_stream(out, keys[0], keys[1], h, sources[0][1], sources[1][1], steps))
        fused.index = ops[last].index
        for b in [keys[0][0], keys[1][0]] + [st.operand.buffer for st in steps if st.operand is not None]:
            b.accesses.append(fused.index)
        for b in (x0, x1, aa, ab) + ((AC,) if chain_pos is not None else ()):
            b._placeholder.elided = True
        removed |= set(members)
        replacement[last] = fused
        #an iota nobody reads any more goes too
        for _, _, si, S in sources:
            uses[pid(S)] -= 1
            if uses[pid(S)] == 0 and si not in removed:
                removed.add(si)
                S._placeholder.elided = True
    return [replacement.get(i, op) for i, op in enumerate(ops) if i not in removed or i in replacement]


def _is_small(op) -> bool:
    '''An element-wise chain or a plain float column sum of a few workgroups, of a kind that has a batch kernel.'''
    if op.chain is None and not (op.conv is None and op.launch.kernel in K.REDUCE_BATCH_KERNELS):
        return False
    if op.launch.kernel in K.TRANSPOSE_BATCH_KERNELS:
        #a tiled copy that swaps two dimensions (a network's kernels, transposed for its backward pass): batched up to a
        #larger size, a launch of a few microseconds carries little more than its own latency
        return op.launch.grid[0] * op.launch.grid[1] * op.launch.grid[2] <= K.TRANSPOSE_BATCH_MAX_BLOCKS
    return op.launch.kernel in K.BATCH_KERNELS and op.launch.grid[0] <= K.BATCH_MAX_BLOCKS


def _small_reads(op) -> tp.List:
    return _reads(op) if op.chain is not None else [b for b, _ in op.launch.buffers[1:]]


def _small_out(op):
    return op.chain.out if op.chain is not None else op.launch.buffers[0][0]


def _may_write(op) -> tp.List:
    '''Buffers an op may change: its result where the op's structure is known, else everything it touches.'''
    if op.chain is not None or op.conv is not None or (op.meta is not None and op.meta[0] in ('iota', 'concat_part', 'threefry', 'reduce', 'softmax')):
        return _writes(op)
    return [b for b, _ in op.launch.buffers if b is not None]


def _touched(op) -> tp.List:
    if op.chain is not None or op.conv is not None:
        return _reads(op) + _writes(op)
    return [b for b, _ in op.launch.buffers if b is not None]


BATCH_MIN_GAIN = 4          #launches a program must save before its small chains are moved and batched


def batch_small_chains(ops):
    '''Programs with many little vectors (per-channel statistics, parameter updates of a training step)
    spend most of their launches on element-wise chains of a few workgroups, each paying a full launch
    latency. This pass

    1. moves every such chain that depends only on program inputs (or on chains moved before it) to the
       front, and every one whose result nothing but other moved chains reads to the end,
    2. sorts each run of consecutive small chains into dependency levels (read-after-write, write-after-read
       and write-after-write on the buffers) and turns every level's chains of one kernel variant into ONE
       launch of ew_chain_batch_* / reduce_cols_fsum_batch_*, and
    3. rebuilds the buffers' access positions from the final order, since storage is shared between
       buffers by those positions.

    Every chain computes what it computed before; only the order of independent launches changes.'''
    from .ops import Op
    pid = lambda b: id(b._placeholder)
    small = [_is_small(op) for op in ops]
    if sum(small) < BATCH_MIN_GAIN + 1:
        return ops

    # 1a. to the front
    written, touched, front = set(), set(), set()
    for i, op in enumerate(ops):
        if small[i] and not any(pid(b) in written for b in _small_reads(op)) and pid(_small_out(op)) not in touched:
            front.add(i)
            continue
        written |= {pid(b) for b in _may_write(op)}
        touched |= {pid(b) for b in _touched(op)}
    # 1b. to the end
    written, touched, back = set(), set(), set()
    for i in reversed(range(len(ops))):
        op = ops[i]
        if i not in front and small[i] and pid(_small_out(op)) not in touched and not any(pid(b) in written for b in _small_reads(op)):
            back.add(i)
            continue
        written |= {pid(b) for b in _may_write(op)}
        touched |= {pid(b) for b in _touched(op)}
    order = ([i for i in range(len(ops)) if i in front] + [i for i in range(len(ops)) if i not in front and i not in back]
             + [i for i in range(len(ops)) if i in back])
    moved = [ops[i] for i in order]

    # 2. runs of small chains -> levels -> batches
    result, saved, i = [], 0, 0
    while i < len(moved):
        if not _is_small(moved[i]):
            result.append(moved[i])
            i += 1
            continue
        j = i
        while j < len(moved) and j - i < 256 and _is_small(moved[j]):      #(levels are found pair by pair: bounded runs)
            j += 1
        run, level = moved[i:j], []
        for k, op in enumerate(run):
            reads, out = {pid(b) for b in _small_reads(op)}, pid(_small_out(op))
            lv = 0
            for q in range(k):
                q_reads, q_out = {pid(b) for b in _small_reads(run[q])}, pid(_small_out(run[q]))
                if q_out in reads or q_out == out or out in q_reads:
                    lv = max(lv, level[q] + 1)
            level.append(lv)
        for lv in range(max(level) + 1):
            by_kernel: tp.Dict[str, list] = {}
            for k, op in enumerate(run):
                if level[k] == lv:
                    by_kernel.setdefault(op.launch.kernel, []).append(op)
            for group in by_kernel.values():
                if len(group) == 1:
                    result.append(group[0])
                    continue
                batch = Op(_label(*group), launch=K.batch_launch([op.launch for op in group]))
                batch.index = min(op.index for op in group)
                result.append(batch)
                saved += len(group) - 1
        i = j
    if saved < BATCH_MIN_GAIN:
        return ops

    # 3. access positions of every buffer in the order the launches now have
    fresh: tp.Dict[int, tp.Tuple[list, list]] = {}
    for position, op in enumerate(result):
        launches = op.launch.members or (op.launch,)
        for launch in launches:
            for b, _ in launch.buffers:
                if b is not None:
                    fresh.setdefault(id(b.accesses), (b.accesses, []))[1].append(position)
        op.index = position
    for accesses, positions in fresh.values():
        accesses[:] = positions
    return result
