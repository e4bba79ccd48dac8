'''Launch descriptors for the gfx950 kernels.

Where the reference turned an op into SPIR-V by pasting shapes into GLSL text and compiling it
at run time (vkjax/shaders.py:16-42, vkjax/ops.py:36-41), the kernels here are built ahead of
time and take shapes and strides as kernel arguments. Each function below lays out the argument
block of one kernel (a struct of 32-bit fields that follows the pointer arguments, mirroring the
`struct ...Params` in vkjax_amd/csrc/kernels/*.hip) and picks grid, block and kernel variant.
'''
import contextlib
import os
import re
import typing as tp

import numpy as np

from .buffers import Buffer

_KDIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'csrc', 'kernels')


def _read_opcodes() -> tp.Dict[str, int]:
    text = open(os.path.join(_KDIR, 'ew_opcodes.h')).read()
    return {m.group(1): int(m.group(2)) for m in re.finditer(r'^EW_OP\((\w+),\s*(\d+)\)', text, re.M)}


EW = _read_opcodes()
EW_MAX_STEPS = 8
CONV_MAX_EPI = 6
BLOCK = 256


class _Choices:
    '''Which kernel variant a lowering picks where several would do. Every field has the value the heuristics work
    with; `overrides(...)` pins some of them for the duration of a `with` block, which is how tests reach every
    variant whatever the heuristics would choose, and how measurements compare variants.'''
    DEFAULTS = dict(
        ew_affine=None,                  #the straight-line affine kernel: None = where it pays, True = wherever it applies, False = never
        conv_tile=None,                  #name of the tile shape (CONV_TILES) instead of the estimate's choice
        conv_bk=None,                    #k step
        conv_chunk=None,                 #consecutive M tiles a lean block walks
        conv_blocks_per_cu=5,            #blocks of the lean 64 x 64 kernels a CU holds at once (94 registers); 0 = no evenly split grids
        conv_even_split_min_tiles=4.5,   #tiles per block from which an evenly split grid is used
        conv_general=False,              #never pick the lean kernel variant
        conv_b_general=False,            #element-wise loads of the kernel operand also where 16-byte loads would do
        conv_ksplit=None,                #the four-waves-per-tile kernel: always (where it applies) / never
        pool_gradient_2d=None,           #the 2-D kernels of a pooling gradient: None = where they apply, False = never, 'elements' = never the one for groups of 2 x 2 elements
        scatter_bucket_cap=None,         #slots per row in the sorted scatter-add's table of fixed-capacity buckets (0: no table)
        conv_dense_rows=None,            #the kernel for at most 16 output features: None = where it applies, False = never
        conv_mix=None,                   #mixed 64 x 64 / 32 x 32 tiling: None = by the heuristic, False = never, an int = that many M tiles stay 64 x 64
        conv_stem=None,                  #the patch kernel for few input features: False = never; None / True: where it applies; 64: its 64-position tiles only
        conv_k_splits=None,              #slices a contraction is cut into where that applies (None: by the heuristic, 1: never)
        conv_xcd_columns=0,              #four-waves-per-tile kernels: XCD columns over the tile grid (0: row-major ranges, None: least traffic)
        scatter_sort_threshold=1 << 18,  #update elements from which a row scatter-add sorts its updates instead of using atomics
        reuse_equal_equations=True,      #an equation that repeats an earlier one is bound to that one's buffer
    )

    def __init__(self):
        self.__dict__.update(self.DEFAULTS)


CHOICES = _Choices()


@contextlib.contextmanager
def overrides(**pinned):
    '''`with overrides(conv_tile='64x64', conv_bk=32): ...` - programs built inside the block use the given
    choices (fields of `_Choices.DEFAULTS`); the previous values return when the block is left.'''
    unknown = set(pinned) - set(_Choices.DEFAULTS)
    if unknown:
        raise TypeError(f'overrides: unknown choice(s) {sorted(unknown)}; known: {sorted(_Choices.DEFAULTS)}')
    saved = {name: getattr(CHOICES, name) for name in pinned}
    CHOICES.__dict__.update(pinned)
    try:
        yield CHOICES
    finally:
        CHOICES.__dict__.update(saved)


class Launch(tp.NamedTuple):
    kernel:  str
    grid:    tp.Tuple[int, int, int]
    block:   tp.Tuple[int, int, int]
    buffers: tp.List[tp.Tuple[tp.Optional[Buffer], int]]     #(buffer, byte offset) in argument order
    params:  bytes
    lds:     int = 0
    #algorithmic work of this launch, for roofline accounting
    bytes_moved: int = 0
    flops:       int = 0
    #a batch launch: the launches it evaluates, described to the kernel by a table in device memory
    #that is written when the launch is recorded (it holds device addresses)
    members: tp.Tuple['Launch', ...] = ()
    #the kernel stores its result (its first array) past the caches when bit 31 of its first parameter word is set
    #(see with_streamed_result)
    streamable: bool = False
    #which of `buffers` the kernel writes (positions); everything else it only reads
    written: tp.Tuple[int, ...] = (0,)


def _u32(*values) -> bytes:
    return np.asarray([int(v) & 0xFFFFFFFF for v in values], dtype=np.uint32).tobytes()


def _i32(*values) -> bytes:
    return np.asarray([int(v) for v in values], dtype=np.int32).tobytes()


def _pad(seq, n, fill=0):
    seq = list(seq)
    assert len(seq) <= n, (seq, n)
    return seq + [fill] * (n - len(seq))


def _cdiv(a, b):
    return -(-int(a) // int(b))


def row_major_strides(shape) -> tp.Tuple[int, ...]:
    strides, acc = [], 1
    for s in reversed(shape):
        strides.append(acc)
        acc *= int(s)
    return tuple(reversed(strides))


# --------------------------------------------------------------------------- element-wise chains

class EwOperand(tp.NamedTuple):
    '''An array read by an element-wise chain: element `coords` of the output reads
    buffer[offset + sum(coords * strides)] (strides in elements, one per output dim).'''
    buffer:  Buffer
    offset:  int
    strides: tp.Tuple[int, ...]


class EwStep(tp.NamedTuple):
    op:           int
    operand:      tp.Optional[EwOperand] = None
    operand_left: bool = False
    imm:          int = 0


class EwChain:
    '''out = step_n(... step_1(first) ...) over `shape`.'''
    def __init__(self, out: Buffer, shape, first: EwOperand, steps: tp.Sequence[EwStep]):
        self.out, self.shape, self.first, self.steps = out, tuple(int(s) for s in shape), first, list(steps)

    def operands(self) -> tp.List[tp.Optional[EwOperand]]:
        return [self.first] + [s.operand for s in self.steps]


def broadcast_operand(buf: Buffer, out_shape) -> EwOperand:
    '''Trailing-aligned numpy-style broadcast of `buf` to `out_shape` (reference: vkjax/ops.py:160-184).'''
    out_shape = tuple(out_shape)
    in_shape  = tuple(buf.shape)
    if len(in_shape) > len(out_shape):
        raise ValueError(f'Cannot broadcast from {in_shape} to {out_shape}')
    in_strides = row_major_strides(in_shape)
    strides    = [0] * len(out_shape)
    for i in range(1, len(in_shape) + 1):
        old, new = in_shape[-i], out_shape[-i]
        if old != new and old != 1:
            raise ValueError(f'Cannot broadcast from {in_shape} to {out_shape}')
        strides[-i] = in_strides[-i] if old == new and old != 1 else 0
    return EwOperand(buf, 0, tuple(strides))


def _collapse(shape, stride_sets):
    '''Drop size-1 dims and merge neighbours that every operand walks contiguously.'''
    dims    = [(s, [st[i] for st in stride_sets]) for i, s in enumerate(shape) if s != 1]
    if not dims:
        return [1], [[0] for _ in stride_sets]
    merged = [dims[0]]
    for size, strides in dims[1:]:
        psize, pstrides = merged[-1]
        if all(ps == s * size for ps, s in zip(pstrides, strides)):
            merged[-1] = (psize * size, strides)
        else:
            merged.append((size, strides))
    out_dims    = [m[0] for m in merged]
    out_strides = [[m[1][k] for m in merged] for k in range(len(stride_sets))]
    return out_dims, out_strides


def lower_ew_chain(chain: EwChain) -> Launch:
    operands = chain.operands()
    nsteps   = len(operands)
    if nsteps > EW_MAX_STEPS:
        raise ValueError(f'element-wise chain of {nsteps} steps exceeds the kernel limit of {EW_MAX_STEPS}')
    n = int(np.prod(chain.shape, dtype=np.int64))
    present = [o for o in operands if o is not None]
    #the output is walked contiguously; include its strides so that merging respects it
    out_strides = row_major_strides(chain.shape)
    dims, strides = _collapse(chain.shape, [out_strides] + [o.strides for o in present])
    if len(dims) > 4:
        raise NotImplementedError(f'element-wise access pattern with {len(dims)} irreducible dimensions: {chain.shape}')
    ndim    = len(dims)
    strides = strides[1:]
    transposed = _as_tiled_transpose(chain, dims, strides)
    if transposed is not None:
        return transposed
    affine = _as_affine_chain(chain, n, dims, strides)
    if affine is not None:
        return affine
    vec = 4
    if n % 4 or dims[-1] % 4:
        vec = 1
    for o, st in zip(present, strides):
        if st[-1] not in (0, 1):
            vec = 1
        elif st[-1] == 1 and (o.offset % 4 or any(s % 4 for s in st[:-1])):
            vec = 1
    magics = [_magic_division(d) for d in _pad(dims, 4, 1)]
    ops, flags, imms, stride_rows, buffers, extents, bases = [], [], [], [], [], [], []
    it = iter(strides)
    for k, o in enumerate(operands):
        step = chain.steps[k - 1] if k > 0 else None
        ops.append(step.op if step else 0)
        imms.append(step.imm if step else 0)
        flag = 2 if (step and step.operand_left) else 0
        if o is None:
            stride_rows.append([0, 0, 0, 0])
            buffers.append((None, 0))
            extents.append(0)
            bases.append(0)
        else:
            st = next(it)
            if o.buffer.size * 4 >= 2**32:
                raise NotImplementedError('element-wise operand of 4 GiB or more')
            extents.append(o.buffer.size * 4)
            bases.append(o.offset)
            flag |= 1 | (4 if st[-1] == 1 else 0)
            #simple addressing patterns the kernel resolves without multiplications
            if all(s == 0 for s in st):
                flag |= 3 << 4 | 64
            elif tuple(st) == row_major_strides(dims):
                flag |= 1 << 4
            elif st[-1] == 1 and all(s == 0 for s in st[:-1]):
                flag |= 2 << 4
                #a thread's vectors are BLOCK * vec elements apart: the same coordinate when the dimension's length divides that
                if (BLOCK * vec) % dims[-1] == 0:
                    flag |= 64
            stride_rows.append(_pad(st, 4))
            buffers.append((o.buffer, 0))
        flags.append(flag)
    while len(stride_rows) < EW_MAX_STEPS:
        stride_rows.append([0, 0, 0, 0])
        buffers.append((None, 0))
    params = (_u32(n, ndim, *_pad(dims, 4, 1), nsteps, *_pad(ops, EW_MAX_STEPS), *_pad(flags, EW_MAX_STEPS),
                   *_pad(imms, EW_MAX_STEPS))
              + _i32(*[s for row in stride_rows for s in row]) + _u32(*_pad(extents, EW_MAX_STEPS), *_pad(bases, EW_MAX_STEPS))
              + _u32(*[m for m, _ in magics], *[sh for _, sh in magics]))
    nbytes = 4 * n + sum(4 * min(n, o.buffer.size) for o in present)
    if n >= 2**31:
        raise NotImplementedError(f'element-wise op over {n} elements exceeds 32-bit indexing')
    slots = 2 if nsteps <= 2 else 4 if nsteps <= 4 else 6 if nsteps <= 6 else 8
    per_thread = {2: 1, 4: 2, 6: 2, 8: 1}[slots]               #vectors a thread works on (the kernel's U)
    return Launch(f'ew_chain_v{vec}_s{slots}', (_cdiv(_cdiv(n, vec), BLOCK * per_thread), 1, 1), (BLOCK, 1, 1),
                  [(chain.out, 0)] + buffers, params, bytes_moved=nbytes, streamable=vec == 4)


EW_AFFINE_BIG_ELEMENTS = 1 << 22
#Results from this size on that no later launch of the program reads are stored with the nontemporal hint: such an array
#only pushes out of the caches what could be reused, and the stores of a launch that reads and writes run faster past the
#L2 (relu on 64 M elements 92 -> 76 us, exp 96 -> 81 us). Results that the next launch reads are left to the caches.
STREAM_RESULT_MIN_BYTES = 64 << 20
STREAM_RESULT_BIT = 1 << 31
#kernels that add to what their result array already holds (their first array is read as well as written)
ACCUMULATING_KERNELS = ('scatter_add_rows', 'scatter_add_general')


def with_streamed_result(launch: Launch) -> Launch:
    '''`launch` with the flag set that makes its kernel store the result past the caches (bit 31 of the first
    parameter word, an element count below 2**31 in every kernel that is marked streamable).'''
    assert launch.streamable and not launch.members
    first = int(np.frombuffer(launch.params[:4], np.uint32)[0])
    assert first < STREAM_RESULT_BIT
    return launch._replace(params=_u32(first | STREAM_RESULT_BIT) + launch.params[4:])


def _as_affine_chain(chain: EwChain, n: int, dims, strides) -> tp.Optional[Launch]:
    '''ew_affine_v4 for float chains of the form ((first + s1 + s2 + s3) - vsub) * vmul + vadd + full, max(., floor)
    (every part optional, in this order; s and full arrays of the output's shape, v vectors over the fastest
    dimension, floor one value), for chains of more than four operands: a small launch is mostly the interpreter's
    latency, and on large arrays the interpreter's instructions cost a fifth of the bandwidth (batch norm + ReLU on
    51 M elements 4.5 TB/s, here 5.7). Shorter chains keep the general kernel, which is as fast for them and whose
    small launches are batched with their neighbours.'''
    operands = chain.operands()
    if (CHOICES.ew_affine is False or not chain.steps or any(o is None for o in operands) or n % 4 or dims[-1] % 4 or n * 4 >= 2**32 - 2**16
            or len(dims) > 2 or (CHOICES.ew_affine is None and len(operands) <= 4)
            or any(np.dtype(b.dtype) != np.float32 for b in [chain.out] + [o.buffer for o in operands])):
        return None
    dense = row_major_strides(dims)
    kind  = lambda st: ('full' if tuple(st) == dense else 'vec' if len(dims) == 2 and tuple(st) == (0, 1)
                        else 'one' if all(s == 0 for s in st) else None)
    kinds = [kind(st) for st in strides]
    if kinds[0] != 'full' or (len(dims) == 1 and 'vec' in kinds):
        return None
    steps, k = list(zip(chain.steps, operands[1:], kinds[1:])), 0
    sums, slot = [], {}
    while k < len(steps) and len(sums) < 3 and steps[k][0].op == EW['ADD_F'] and steps[k][2] == 'full':
        sums.append(steps[k][1]); k += 1
    template = ((0, EW['SUB_F'], 'vec', False), (1, EW['MUL_F'], 'vec', None), (2, EW['ADD_F'], 'vec', None),
                (3, EW['ADD_F'], 'full', None), (4, EW['MAX_F'], 'one', False))
    t = 0
    while k < len(steps):
        step, operand, what = steps[k]
        while t < len(template) and not (step.op == template[t][1] and what == template[t][2]
                                         and (template[t][3] is None or bool(step.operand_left) == template[t][3])):
            t += 1
        if t == len(template):
            return None
        slot[template[t][0]] = operand
        t += 1; k += 1
    if not sums and not slot:
        return None
    C = dims[-1] if len(dims) == 2 else 4
    if any(o.buffer.size != C for b, o in slot.items() if b in (0, 1, 2)):
        return None
    magic, shift = _magic_division(C // 4)
    at = lambda o: (o.buffer, o.offset * 4) if o is not None else (None, 0)
    buffers = ([(chain.out, 0), at(operands[0])] + [at(o) for o in _pad(sums, 3, None)]
               + [at(slot.get(b)) for b in range(5)])
    params  = _u32(n, C // 4, magic, shift, len(sums), sum(1 << b for b in slot))
    nbytes  = 4 * n + sum(4 * min(n, o.buffer.size) for o in operands)
    #(arrays of more than 16 MB: the variant that skips absent operands instead of loading through empty descriptors)
    kernel = 'ew_affine_big_v4' if n > EW_AFFINE_BIG_ELEMENTS else 'ew_affine_v4'
    return Launch(kernel, (_cdiv(n // 4, 2 * BLOCK), 1, 1), (BLOCK, 1, 1), buffers, params, bytes_moved=nbytes, streamable=True)


EW_BATCH_KERNELS     = ('ew_chain_v1_s2', 'ew_chain_v1_s4', 'ew_chain_v4_s2', 'ew_chain_v4_s4')
REDUCE_BATCH_KERNELS = ('reduce_cols_fsum_v1', 'reduce_cols_fsum_v4')
TRANSPOSE_BATCH_KERNELS = ('transpose_tiled_v4', 'transpose_tiled_v4_t128')
BATCH_KERNELS        = {**{k: k.replace('ew_chain_', 'ew_chain_batch_') for k in EW_BATCH_KERNELS},
                        **{k: k.replace('fsum_', 'fsum_batch_') for k in REDUCE_BATCH_KERNELS},
                        **{k: k.replace('tiled_', 'tiled_batch_') for k in TRANSPOSE_BATCH_KERNELS}}
EW_BATCH_ENTRY_BYTES        = 432
REDUCE_BATCH_ENTRY_BYTES    = 56
TRANSPOSE_BATCH_ENTRY_BYTES = 48
BATCH_MAX_BLOCKS         = 4096        #launches of more workgroups than this keep a launch of their own
REDUCE_NARROW_MAX_BLOCKS = 16          #column sums of at most this many workgroups trade block width for more blocks
TRANSPOSE_BATCH_MAX_BLOCKS = 1024      #... tiled transposes (the kernels of a network, for its backward pass) up to this many


def _blocks(launch: Launch) -> int:
    return launch.grid[0] * launch.grid[1] * launch.grid[2]


def batch_launch(members: tp.Sequence[Launch]) -> Launch:
    '''One launch for several small launches of the same kernel (element-wise chains or float column sums)
    that do not depend on one another.'''
    kernel = members[0].kernel
    assert kernel in BATCH_KERNELS and all(m.kernel == kernel and not m.members for m in members), [m.kernel for m in members]
    return Launch(BATCH_KERNELS[kernel], (sum(_blocks(m) for m in members), 1, 1), (BLOCK, 1, 1), [],
                  _u32(len(members)), bytes_moved=sum(m.bytes_moved for m in members), members=tuple(members))


def batch_table(launch: Launch, device_address: tp.Callable[[Buffer], int]) -> np.ndarray:
    '''The table of a batch launch as uint32 words, one entry per member: {first workgroup, 0 (tiled transposes: the
    x extent of the member's grid), the addresses of the member's arrays (0 = none), the member's parameter block
    (tiled transposes: then the y extent of its grid)}, padded to a multiple of 8 bytes.'''
    kind = launch.members[0].kernel
    is_chain, is_transpose = kind in EW_BATCH_KERNELS, kind in TRANSPOSE_BATCH_KERNELS
    entry_bytes, pointers = ((EW_BATCH_ENTRY_BYTES, 1 + EW_MAX_STEPS) if is_chain else
                             (TRANSPOSE_BATCH_ENTRY_BYTES, 2) if is_transpose else (REDUCE_BATCH_ENTRY_BYTES, 2))
    rows, first = [], 0
    for m in launch.members:
        assert len(m.buffers) == pointers, (m.kernel, len(m.buffers))
        addresses = [device_address(b) + off if b is not None else 0 for b, off in m.buffers]
        #(a transpose has a three-dimensional grid of its own: its x extent follows first_block, its y extent the parameters)
        row = (_u32(first, m.grid[0] if is_transpose else 0) + np.asarray(addresses, dtype=np.uint64).tobytes() + m.params
               + (_u32(m.grid[1]) if is_transpose else b''))
        rows.append(row + bytes(entry_bytes - len(row)))
        first += _blocks(m)
    table = b''.join(rows)
    assert len(table) == entry_bytes * len(launch.members)
    return np.frombuffer(table, dtype=np.uint32).copy()


TRANSPOSE_BIG_TILES = True


def _as_tiled_transpose(chain: EwChain, dims, strides) -> tp.Optional[Launch]:
    '''A pure copy whose collapsed form is out[b, i, j] = in[b * sb + j * sj + i] (the two fastest dimensions
    trade places) goes through the LDS-tiled kernel when both of them are at least 16 long.'''
    if chain.steps or len(dims) not in (2, 3):
        return None
    st = strides[0]
    B, I, J = ([1] + list(dims))[-3:]
    sb = st[0] if len(dims) == 3 else 0
    if st[-2] != 1 or st[-1] < I or I < 16 or J < 16 or B > 65535 or _cdiv(I, 64) > 65535:
        return None
    src = chain.first
    if src.buffer.size * 4 >= 2**32:
        return None
    n = B * I * J
    vec = all(v % 4 == 0 for v in (I, J, st[-1], sb, src.offset))
    if vec and I >= 128 and J >= 128 and I * J >= 1 << 16 and TRANSPOSE_BIG_TILES:
        return Launch('transpose_tiled_v4_t128', (_cdiv(J, 128), _cdiv(I, 128), B), (BLOCK, 1, 1), [(chain.out, 0), (src.buffer, src.offset * 4)],
                      _u32(B, I, J, sb, st[-1]), lds=0, bytes_moved=8 * n, streamable=True)
    return Launch('transpose_tiled_v4' if vec else 'transpose_tiled', (_cdiv(J, 64), _cdiv(I, 64), B), (BLOCK, 1, 1), [(chain.out, 0), (src.buffer, src.offset * 4)],
                  _u32(B, I, J, sb, st[-1]), bytes_moved=8 * n, streamable=bool(vec))


def iota(out: Buffer, dimension: int) -> Launch:
    n     = out.size
    inner = int(np.prod(out.shape[dimension + 1:], dtype=np.int64))
    size  = out.shape[dimension]
    vec   = 4 if n % 4 == 0 else 1
    return Launch(f'iota_nd_v{vec}', (_cdiv(_cdiv(n, vec), BLOCK), 1, 1), (BLOCK, 1, 1), [(out, 0)],
                  _u32(n, inner, size, int(out.dtype == np.float32)), bytes_moved=4 * n)


def fill(out: Buffer, word: int) -> Launch:
    n = out.size
    return Launch('fill_u32', (_cdiv(_cdiv(n, 4), BLOCK), 1, 1), (BLOCK, 1, 1), [(out, 0)], _u32(n, word), bytes_moved=4 * n)


def concat_part(out: Buffer, part: Buffer, dimension: int, offset_along_dim: int) -> Launch:
    inner      = int(np.prod(out.shape[dimension + 1:], dtype=np.int64))
    part_inner = part.shape[dimension] * inner
    out_inner  = out.shape[dimension] * inner
    n   = part.size
    vec = 4 if (part_inner % 4 == 0 and out_inner % 4 == 0 and (offset_along_dim * inner) % 4 == 0) else 1
    return Launch(f'concat_part_v{vec}', (_cdiv(_cdiv(n, vec), BLOCK), 1, 1), (BLOCK, 1, 1), [(out, 0), (part, 0)],
                  _u32(n, part_inner, out_inner, offset_along_dim * inner), bytes_moved=8 * n, streamable=vec == 4 and n < 2**31)


TF_MAX_STEPS = 8


_UNIFORM_CHAIN_OPS = [EW[name] for name in ('SHR_L', 'OR_X', 'SUB_F', 'MUL_F', 'ADD_F', 'MAX_F')]


def threefry_stream(out: Buffer, key0: tp.Tuple[Buffer, int], key1: tp.Tuple[Buffer, int], h: int, c0: int, c1: int,
                    steps: tp.Sequence[EwStep], layout: str = 'halves', n: tp.Optional[int] = None) -> Launch:
    '''Random words from counters generated in registers, the element-wise `steps` (operands: single
    values) applied before the only store. `h` blocks are run; the key words are given as
    (buffer, element offset). Layouts:
      halves  out[j], out[h + j] = steps(threefry2x32(key, c0 + j, c1 + j)); `n` (2h or 2h - 1) is the
              number of elements stored, and with n == 2h - 1 the last x1 counter is 0
      xor     out[j] = steps(y0 ^ y1) with y = threefry2x32(key, c0, c1 + j)
      pairs   out[2j], out[2j + 1] = threefry2x32(key, c0, c1 + j)  (no steps)'''
    if len(steps) > TF_MAX_STEPS:
        raise ValueError('too many steps')
    if layout == 'pairs' and steps:
        raise ValueError('the pairs layout takes no steps')
    n = 2 * h if n is None else n
    assert layout != 'halves' or n in (2 * h, 2 * h - 1)
    flags, buffers = [], []
    for s in steps:
        if s.operand is not None:
            assert s.operand.buffer.size == 1 and s.operand.offset == 0
        flags.append((1 if s.operand is not None else 0) | (2 if s.operand_left else 0))
        buffers.append((s.operand.buffer if s.operand is not None else None, 0))
    vec = 4 if h % 4 == 0 and (n == 2 * h if layout == 'halves' else layout == 'xor') else 1
    params = _u32(h, c0, c1, len(steps), *_pad([s.op for s in steps], TF_MAX_STEPS), *_pad(flags, TF_MAX_STEPS),
                  *_pad([s.imm for s in steps], TF_MAX_STEPS), n)
    kernel = {'halves': 'threefry2x32_stream', 'xor': 'threefry2x32_stream_xor', 'pairs': 'threefry2x32_stream_pairs'}[layout]
    #jax.random.uniform's chain has a kernel of its own with the steps compiled in
    if vec == 4 and [s.op for s in steps] == _UNIFORM_CHAIN_OPS and flags == [1, 1, 1, 1, 1, 3] and all(s.imm == 0 for s in steps):
        kernel += '_uniform'
    return Launch(f'{kernel}_v{vec}', (_cdiv(_cdiv(h, vec), BLOCK), 1, 1), (BLOCK, 1, 1),
                  [(out, 0), (key0[0], key0[1] * 4), (key1[0], key1[1] * 4)] + _pad(buffers, TF_MAX_STEPS, (None, 0)), params,
                  bytes_moved=4 * (h if layout == 'xor' else n))


# --------------------------------------------------------------------------- conv / dot

class ConvGeometry(tp.NamedTuple):
    '''Implicit-GEMM view of a convolution or matrix product (see csrc/kernels/conv_gemm.hip).'''
    batch: int; Ho: int; Wo: int; N: int
    H: int; W: int; Cin: int; KH: int; KW: int
    SH: int = 1; SW: int = 1; PH: int = 0; PW: int = 0; DH: int = 1; DW: int = 1; LH: int = 1; LW: int = 1
    xs: tp.Tuple[int, int, int, int] = (0, 0, 0, 1)      #lhs strides: batch, y, x, feature
    ws: tp.Tuple[int, int, int, int] = (0, 0, 0, 1)      #rhs strides: ky, kx, in feature, out feature
    os: tp.Tuple[int, int, int, int] = (0, 0, 0, 1)      #out strides: batch, y, x, feature
    #> 1: the contraction is cut into this many slices, each summed by blocks of its own into its own [M, N] matrix of
    #the result array (no epilogue); another launch adds the slices
    k_splits: int = 1

    @property
    def M(self): return self.batch * self.Ho * self.Wo
    @property
    def K(self): return self.KH * self.KW * self.Cin


class WgradGeometry(tp.NamedTuple):
    '''Kernel gradient of an NHWC / HWIO convolution in the forward convolution's own terms: X is
    [images, H, W, C], the output cotangent G is [images, Ho, Wo, N], the result [KH, KW, C, N]
    (see csrc/kernels/wgrad_gemm.hip). A product X^T G of row-major matrices is the 1x1 case.'''
    images: int; Ho: int; Wo: int; H: int; W: int; C: int; KH: int; KW: int; N: int
    SH: int = 1; SW: int = 1; PH: int = 0; PW: int = 0; DH: int = 1; DW: int = 1

    @property
    def pixels(self): return self.images * self.Ho * self.Wo
    @property
    def M(self): return self.KH * self.KW * self.C


def choose_wgrad_splits(g: WgradGeometry, compute_units: int = 256) -> int:
    '''Slices of the contraction: enough blocks to fill the chip several times over, at least four
    k steps of 32 pixels per slice.'''
    tiles = _cdiv(g.M, 64) * _cdiv(g.N, 64)
    want  = _cdiv(4 * compute_units, tiles)
    return max(1, min(want, g.pixels // 128, 1024))


def wgrad_gemm(out: Buffer, x: Buffer, cot: Buffer, g: WgradGeometry, splits: int) -> Launch:
    '''`out` holds `splits` partial results of M * N elements each (the result itself when splits == 1).'''
    for name, b in (('input', x), ('cotangent', cot)):
        if b.size * 4 >= 2**31:
            raise NotImplementedError(f'kernel gradient: {name} of {b.size * 4} bytes exceeds the 2 GiB the kernel addresses')
    assert x.size == g.images * g.H * g.W * g.C and cot.size == g.pixels * g.N and out.size == splits * g.M * g.N
    per_split = _cdiv(_cdiv(g.pixels, splits), 32) * 32
    assert per_split * splits >= g.pixels
    magics = [v for d in (g.Ho * g.Wo, g.Wo, g.C, g.KW) for v in _magic_division(d)]
    params = _i32(g.pixels, g.M, g.N, g.Ho, g.Wo, g.H, g.W, g.C, g.KW, g.SH, g.SW, g.PH, g.PW, g.DH, g.DW, per_split) \
           + _u32(*magics, x.size * 4, cot.size * 4)
    kernel = 'wgrad_gemm_64x64_' + ('a' if g.C % 4 == 0 else 's') + ('a' if g.N % 4 == 0 else 's')
    return Launch(kernel, (_cdiv(g.N, 64), _cdiv(g.M, 64), splits), (256, 1, 1), [(out, 0), (x, 0), (cot, 0)], params,
                  bytes_moved=4 * (x.size + cot.size + out.size), flops=2 * g.pixels * g.M * g.N)


class ConvDerivedOperand(tp.NamedTuple):
    '''A per-feature epilogue operand that the kernel computes instead of reading: `first` and the
    step operands are buffers of N values or of one value.'''
    first: Buffer
    steps: tp.Tuple[tp.Tuple[int, tp.Optional[Buffer], bool], ...]       #(opcode, operand or None, operand is the left argument)


class ConvEpilogueStep(tp.NamedTuple):
    op:           int
    kind:         int                    #1 scalar, 2 per-feature vector [N], 3 full tensor laid out like the output
    operand:      tp.Optional[Buffer]    #None when `derived` says how to compute it
    operand_left: bool = False
    derived:      tp.Optional[ConvDerivedOperand] = None


#A pseudo step: the value as it stands at this point of the epilogue is ALSO stored to `operand`, an array laid
#out like the result (the centred convolution result a backward pass needs besides the activation)
CONV_TAP = -1
#A pseudo step, the last of an epilogue: the rows of the result are replaced by their softmax before the store;
#`operand`, if not None, is an int32 array [M] that receives each row's arg-max. Only the kernel for products with at
#most 16 output features (dense_rows_n16) can do this.
CONV_SOFTMAX = -2


def conv_tap_supported(steps_before: tp.Sequence[ConvEpilogueStep], steps_after: tp.Sequence[ConvEpilogueStep]) -> bool:
    '''The kernel stores a second result before the first step of its straight-line epilogue, or after that
    epilogue's `acc - vector` step.'''
    real = list(steps_before) + list(steps_after)
    if any(e.op == CONV_TAP for e in real) or not real or len(real) > CONV_MAX_EPI - 1:
        return False
    slots = _epilogue_template_slots(real)
    return slots != 0 and (len(steps_before) == 0 or (len(steps_before) == 1 and bool(slots & 1)))


CONV_MAX_DERIVED = 3
CONV_DERIVED_OPS = ('ADD_F', 'SUB_F', 'MUL_F', 'DIV_F', 'MAX_F', 'MIN_F', 'NEG_F', 'RSQRT_F', 'SQRT_F')


#(tag, BM, BN, threads, resident blocks per CU, relative MFMA efficiency of the tile shape)
#(efficiencies are measured: TFLOP/s of each tile on large ResNet-50 layers relative to the best)
#(128 x 128 and 128 x 64 tiles of 2 x 2 waves reached 0.92 and 0.88 of the 64 x 64 tile's rate on large layers and were
#never the estimate's choice for any shape; they are no longer built)
CONV_TILES = (('64x64', 64, 64, 256, 4, 1.00), ('32x32', 32, 32, 64, 16, 0.80))
#k steps each tile shape is built with
CONV_TILE_BK = {'64x64': (32, 64), '32x32': (32, 64)}



def choose_conv_tile(M: int, N: int, compute_units: int = 256):
    '''Smallest estimated time: tiles are dealt out over the CUs, a tile costs BM*BN / efficiency,
    and a block of one wave can drive only one of a CU's four MFMA units.'''
    if CHOICES.conv_tile is not None:
        return next(t[:4] for t in CONV_TILES if t[0] == CHOICES.conv_tile)
    best, best_time = None, None
    for tag, bm, bn, nt, occupancy, eff in CONV_TILES:
        tiles   = _cdiv(M, bm) * _cdiv(N, bn)
        #with several resident blocks per CU the tail of the last round is shared out evenly
        per_cu  = tiles / compute_units if tiles >= compute_units * occupancy else _cdiv(tiles, compute_units)
        simd    = min(1.0, (nt / 256) * min(occupancy, per_cu))
        time    = per_cu * bm * bn / (eff * simd)
        if best_time is None or time < best_time:
            best, best_time = (tag, bm, bn, nt), time
    return best


def choose_conv_split(tiles_m: int, tiles_n: int, compute_units: int = 256) -> int:
    '''How many M tiles of a layer stay 64 x 64 tiles when the rest is computed as 32 x 32 tiles (0: no split).
    tiles / CUs = 3.06 means that some CUs work on four tiles while most have three; the whole rounds keep their
    64 x 64 tiles and the remainder is spread in quarter-size units. Measured on ResNet-50 layers: +15 % at 3.06 and
    1.53 tiles per CU, +7 % at 6.1, nothing at 12.25; not used when the last round is nearly full anyway.'''
    rounds = tiles_m * tiles_n / compute_units
    whole  = int(rounds)
    if whole < 1 or rounds >= 8 or rounds - whole == 0 or rounds - whole > 0.7:
        return 0
    return (whole * compute_units) // tiles_n


def choose_conv_chunk(tiles_m: int, tiles_n: int, compute_units: int = 256) -> int:
    '''M tiles one block works through. Longer chunks hide more start-up latency (only a block's
    first tile pays for the argument fetch and the first loads); enough blocks must remain to
    keep the CUs evenly loaded.'''
    chunk = 1
    while chunk < 8 and _cdiv(tiles_m, chunk * 2) * tiles_n >= 12 * compute_units:
        chunk *= 2
    return chunk


def choose_conv_xcd_columns(M: int, N: int, K: int, tiles_m: int, tiles_n: int) -> int:
    '''How the 8 XCDs (each with an L2 of its own; workgroup b runs on XCD b % 8) are laid over the tile grid of a
    four-waves-per-tile product: 0 = consecutive ranges of tiles in row-major order, else 1 + log2(xn) for 8 / xn rows of
    xn columns of XCDs. With xm x xn XCDs every L2 fetches M / xm rows of A and N / xn columns of B: xn * |A| + xm * |B|
    bytes over the chip. Row-major ranges are the default although they fetch the most: for the MLP's two wide products
    (256 x 784 x 512 and 256 x 512 x 512) the layout with the least traffic, 2 x 4, halves what the L2s fetch (FETCH_SIZE
    11.2 -> 5.4 MB per launch against 2.4 MB of operands) and the step takes 21.0 us instead of 20.4: these launches wait
    for round trips, not for bytes. `conv_xcd_columns=None` asks for the least traffic among the layouts that divide
    the tile grid.'''
    if (tiles_m * tiles_n) % 8:
        return 0
    if CHOICES.conv_xcd_columns is not None:
        xn = int(CHOICES.conv_xcd_columns)
        return xn.bit_length() if xn in (1, 2, 4, 8) and tiles_m % (8 // xn) == 0 and tiles_n % xn == 0 else 0
    best, best_bytes = 0, None
    for code, xn in ((1, 1), (2, 2), (3, 4), (4, 8)):
        xm = 8 // xn
        if tiles_m % xm or tiles_n % xn:
            continue
        nbytes = xn * M * K + xm * K * N
        if best_bytes is None or nbytes < best_bytes:
            best, best_bytes = code, nbytes
    return best


def choose_conv_m_blocks(tiles_m: int, tiles_n: int, compute_units: int = 256) -> int:
    '''0, or the number of blocks that share the M tiles of every N tile evenly: a grid of exactly as many blocks as
    the GPU holds at once (CHOICES.conv_blocks_per_cu per CU), each working through its tiles as one sequence of k steps, so
    that only its first tile pays for the argument fetch and the first loads. Worth it from about five tiles per
    block: with fewer, one tile more or less per block leaves CUs idle at the end (measured on ResNet-50 layers at
    batch 64: -4 to -5 % at 4.9 tiles per block, +1 to +8 % at 2.45).'''
    resident = int(CHOICES.conv_blocks_per_cu * compute_units)
    if resident < 1 or tiles_m * tiles_n < CHOICES.conv_even_split_min_tiles * resident:
        return 0
    return min(tiles_m, max(1, resident // tiles_n))


def choose_conv_bk(tag: str, g: 'ConvGeometry') -> int:
    '''The longer k step halves the barriers per MFMA. Measured on ResNet-50 layers it only pays
    for the 64x64 tile on long contractions, and only when whole k tiles stay inside one kernel
    tap (Cin % 64 == 0), which keeps the tap position in scalar registers.'''
    options = CONV_TILE_BK[tag]
    if CHOICES.conv_bk is not None and CHOICES.conv_bk in options:
        return CHOICES.conv_bk
    if tag == '64x64' and g.Cin % 64 == 0 and g.K >= 2048:
        return 64
    return 32


def _flatten_pointwise(g: ConvGeometry) -> ConvGeometry:
    '''A 1x1, stride-1, unpadded convolution over a dense feature-last array is a plain matrix
    product of the [M, Cin] pixel matrix: present it as one batch of M rows so the kernel skips
    the (batch, y, x) decode of every row.'''
    dense_in  = g.xs[3] == 1 and g.xs[1] == g.W * g.xs[2] and g.xs[0] == g.H * g.W * g.xs[2]
    dense_out = g.os == (g.Ho * g.Wo * g.N, g.Wo * g.N, g.N, 1)
    pointwise = (g.KH == g.KW == 1 and g.SH == g.SW == 1 and g.PH == g.PW == 0 and g.LH == g.LW == 1
                 and g.Ho == g.H and g.Wo == g.W)
    if not (pointwise and dense_in and dense_out) or (g.batch == 1 and g.Wo == 1):
        return g
    M = g.M
    return g._replace(batch=1, Ho=M, Wo=1, H=M, W=1, xs=(0, g.xs[2], 0, 1), os=(M * g.N, g.N, g.N, 1))


def _epilogue_template_slots(epilogue: tp.Sequence[ConvEpilogueStep]) -> int:
    '''Bit k set = step k of the kernel's straight-line epilogue (acc - vector, acc * vector,
    acc + vector, acc + full tensor, max(acc, scalar)) is present; 0 if the chain is not an
    ordered subset of those and has to go through the kernel's general step loop.'''
    template = ((EW['SUB_F'], 2, False), (EW['MUL_F'], 2, None), (EW['ADD_F'], 2, None),
                (EW['ADD_F'], 3, None), (EW['MAX_F'], 1, False))
    slots, k = 0, 0
    for e in epilogue:
        while k < len(template):
            op, kind, left = template[k]
            k += 1
            if e.op == op and e.kind == kind and (left is None or bool(e.operand_left) == left):
                slots |= 1 << (k - 1)
                break
        else:
            return 0
    return slots


def _magic_division(d: int) -> tp.Tuple[int, int]:
    '''(magic, shift) with n // d == (n * magic >> 32) >> shift for every 0 <= n < 2**31; magic 0 stands for d == 1.'''
    if d <= 1:
        return 0, 0
    l = (d - 1).bit_length()                  #ceil(log2(d))
    magic = -(-(1 << (31 + l)) // d)          #ceil(2**(31+l) / d) < 2**32
    return magic, l - 1


STEM_PATCH_FLOATS, STEM_PATCH_ROWS, STEM_VECTORS_PER_THREAD = 6272, 9, 6      #conv_gemm_stem_7x22's LDS patch
#conv_gemm_stem_7x22_m128: tiles of 128 output positions (up to three output rows), 512 threads
STEM128_PATCH_FLOATS, STEM128_PATCH_ROWS, STEM128_VECTORS_PER_THREAD = 7680, 11, 4


def _conv_stem_launch(out, lhs, rhs, g: 'ConvGeometry', epilogue, taps, compute_units, lhs_offset, rhs_offset, out_offset) -> tp.Optional[Launch]:
    '''conv_gemm_stem_7x22 where it applies: dense images with so few features that KW * Cin is 21 or 22 (7 x 7 x 3),
    seven kernel rows, a template epilogue; see the conditions listed at the kernel.'''
    #(offsets: whole images further on in both arrays - a launch over a part of the batch)
    if (CHOICES.conv_stem is False or CHOICES.conv_tile is not None or CHOICES.conv_general or rhs_offset or lhs_offset % 4 or out_offset % 4
            or (taps and (lhs_offset or out_offset))):
        return None
    M, N, K = g.M, g.N, g.K
    RL, WC = g.KW * g.Cin, g.W * g.Cin
    dense_in  = g.xs == (g.H * WC, WC, g.Cin, 1)
    dense_w   = g.ws == (g.KW * g.Cin * N, g.Cin * N, N, 1)
    dense_out = g.os == (g.Ho * g.Wo * N, g.Wo * N, N, 1)
    slots = _epilogue_template_slots(epilogue)
    left  = _cdiv(g.PW * g.Cin, 4) * 4
    right = max(0, (g.Wo - 1) * g.SW - g.PW + g.KW - g.W)          #pixels the last window reaches beyond the row
    pitch = _cdiv(left + (g.W + right) * g.Cin + 1, 4) * 4
    ok = (g.KH == 7 and RL in (21, 22) and dense_in and dense_w and dense_out and g.DH == g.DW == g.LH == g.LW == 1
          and g.PH >= 0 and g.PW >= 0 and WC % 4 == 0 and M % 64 == 0 and (g.Ho * g.Wo) % 64 == 0 and g.Wo >= 64 and N <= 64
          and (not epilogue or (slots != 0 and not slots & 8)) and g.KH + g.SH <= STEM_PATCH_ROWS
          and STEM_PATCH_ROWS * pitch <= STEM_PATCH_FLOATS and STEM_PATCH_ROWS * (WC // 4) <= 256 * STEM_VECTORS_PER_THREAD)
    if not ok:
        return None
    #a second result (the value before or after the first epilogue step) goes to the last operand slot, as in conv_gemm_body
    flags  = slots << 20 | ((taps[0][0] + 1) << 12 if taps else 0)
    params = (_i32(M, N, K, g.Ho, g.Wo, g.H, g.W, g.Cin, g.KH, g.KW, g.SH, g.SW, g.PH, g.PW, pitch, left)
              + _u32(flags, (lhs.size - lhs_offset) * 4, rhs.size * 4, (out.size - out_offset) * 4, *_magic_division(g.Ho * g.Wo), *_magic_division(g.Wo)))
    derived_ptrs, derived_desc = _conv_derived(epilogue, N)
    params += derived_desc
    operand_slots = _pad([(e.operand, 0) for e in epilogue], CONV_MAX_EPI, (None, 0))
    if taps:
        assert operand_slots[-1] == (None, 0)
        operand_slots[-1] = (taps[0][1], 0)
    buffers = [(out, out_offset * 4), (lhs, lhs_offset * 4), (rhs, 0)] + operand_slots + derived_ptrs
    nbytes  = 4 * (lhs.size + rhs.size + out.size) + sum(4 * e.operand.size for e in epilogue if e.operand is not None)
    nbytes += 4 * taps[0][1].size if taps else 0
    #twice the tile and twice the waves per block where the sizes allow it: the kernel and the patch take the same LDS,
    #so a CU holds 16 waves instead of 8
    if (CHOICES.conv_stem != 64 and M % 128 == 0 and (g.Ho * g.Wo) % 128 == 0 and g.KH + 2 * g.SH <= STEM128_PATCH_ROWS
            and STEM128_PATCH_ROWS * pitch <= STEM128_PATCH_FLOATS and STEM128_PATCH_ROWS * (WC // 4) <= 512 * STEM128_VECTORS_PER_THREAD):
        return Launch('conv_gemm_stem_7x22_m128', (min(M // 128, 2 * compute_units), 1, 1), (512, 1, 1), buffers, params,
                      bytes_moved=nbytes, flops=2 * M * N * K)
    return Launch('conv_gemm_stem_7x22', (min(M // 64, 2 * compute_units), 1, 1), (256, 1, 1), buffers, params,
                  bytes_moved=nbytes, flops=2 * M * N * K)


DENSE_ROWS_MAX_N = 16


def _dense_rows_shape(lhs: Buffer, g: 'ConvGeometry') -> bool:
    '''The operands of a product suit dense_rows_n16. `g` as the caller gave it: a matrix product, not a 1 x 1
    convolution over a feature map (those keep the kernels whose epilogue takes a residual operand).'''
    if (CHOICES.conv_dense_rows is False or CHOICES.conv_tile is not None or CHOICES.conv_bk is not None or CHOICES.conv_general
            or CHOICES.conv_ksplit is not None):
        return False
    M, N, K = g.M, g.N, g.K
    flat = (g.batch == 1 and g.Wo == 1 and g.KH == g.KW == 1 and g.SH == 1 and g.PH == g.PW == 0 and g.LH == 1 and g.H == g.Ho
            and g.xs[3] == 1 and g.xs[1] % 4 == 0 and g.xs[1] >= K)
    return (flat and 1 <= N <= DENSE_ROWS_MAX_N and K % 4 == 0 and K > 0 and tuple(g.ws[2:]) == (N, 1) and tuple(g.os[1:]) == (N, N, 1)
            and lhs.size * 4 < 2**31 and M * N * 4 < 2**31)


def conv_is_dense_rows(lhs: Buffer, g: 'ConvGeometry') -> bool:
    '''This product is computed by dense_rows_n16 whatever its epilogue: a fusion pass must not hand it an epilogue that
    kernel cannot apply (another kernel would add the products in another order than in the unfused program).'''
    return g.k_splits == 1 and _dense_rows_shape(lhs, g)


def dense_rows_epilogue_supported(epilogue: tp.Sequence[ConvEpilogueStep]) -> bool:
    real  = [e for e in epilogue if e.op != CONV_SOFTMAX]
    slots = _epilogue_template_slots(real)
    return (all(e.op != CONV_TAP and e.derived is None for e in real) and (not real or (slots != 0 and not slots & 8))
            and all(e.op != CONV_SOFTMAX for e in epilogue[:-1]))


def _dense_rows_launch(out, lhs, rhs, g: 'ConvGeometry', epilogue, taps, lhs_offset, rhs_offset, out_offset,
                       softmax: bool, arg_out: tp.Optional[Buffer]) -> tp.Optional[Launch]:
    '''dense_rows_n16 where it applies: a matrix product (or 1x1 convolution over a dense array) with at most 16 output
    features, a contraction that is a multiple of 4, dense operands, and an epilogue of per-feature and single-value
    template steps; see the kernel.'''
    if taps or lhs_offset or rhs_offset or out_offset or g.k_splits > 1:
        return None
    M, N, K = g.M, g.N, g.K
    slots = _epilogue_template_slots(epilogue)
    if not (_dense_rows_shape(lhs, g) and dense_rows_epilogue_supported(epilogue)):
        return None
    params  = _i32(M, N, K, g.xs[1]) + _u32(slots << 20 | int(softmax) << 29, lhs.size * 4, K * N * 4, M * N * 4)
    slots_p = _pad([(e.operand, 0) for e in epilogue], CONV_MAX_EPI, (None, 0))
    if softmax:
        slots_p[-1] = (arg_out, 0)
    nbytes  = (4 * (lhs.size + rhs.size + out.size) + sum(4 * e.operand.size for e in epilogue if e.operand is not None)
               + (4 * arg_out.size if arg_out is not None else 0))
    return Launch('dense_rows_n16', (_cdiv(M, 4), 1, 1), (256, 1, 1), [(out, 0), (lhs, 0), (rhs, 0)] + slots_p, params,
                  bytes_moved=nbytes, flops=2 * M * N * K)


def _conv_derived(epilogue, N):
    '''(pointer slots, descriptor words) of the one per-feature epilogue operand that the kernel computes itself.'''
    derived_ptrs, derived_desc = [(None, 0)] * (CONV_MAX_DERIVED + 1), _u32(*[0] * (3 + 2 * CONV_MAX_DERIVED))
    for i, e in enumerate(epilogue):
        if e.derived is not None:
            d = e.derived
            assert e.kind == 2 and len(d.steps) <= CONV_MAX_DERIVED and derived_desc == _u32(*[0] * (3 + 2 * CONV_MAX_DERIVED))
            arrays = [d.first] + [st[1] for st in d.steps]
            assert all(a is None or a.size in (1, N) for a in arrays)
            derived_ptrs = _pad([(a, 0) for a in arrays], CONV_MAX_DERIVED + 1, (None, 0))
            mask = sum(1 << k for k, a in enumerate(arrays) if a is not None and a.size == N and N != 1)
            derived_desc = _u32(i, len(d.steps), mask, *_pad([st[0] for st in d.steps], CONV_MAX_DERIVED),
                                *_pad([int(st[2]) for st in d.steps], CONV_MAX_DERIVED))
    return derived_ptrs, derived_desc


def _conv_fast_paths(lhs: Buffer, rhs: Buffer, g: ConvGeometry, lhs_offset: int = 0, rhs_offset: int = 0):
    '''(needs_masks, x_bias, a_fast, b_fast, c_contig) of a flattened geometry: which loaders and stores apply.'''
    N = g.N
    #some kernel tap of some output position falls outside the input (padding, or a window that overhangs)
    needs_masks = (g.PH > 0 or g.PW > 0 or (g.Ho - 1) * g.SH - g.PH + (g.KH - 1) * g.DH >= g.H
                   or (g.Wo - 1) * g.SW - g.PW + (g.KW - 1) * g.DW >= g.W)
    #the 16-byte A path keeps the validity of a row's taps in one 32-bit mask and addresses the
    #input from (PH, PW) positions before its start
    x_bias = (g.PH * g.xs[1] + g.PW * g.xs[2]) * 4
    #(negative padding, i.e. cropping, goes through the generic loader's coordinate checks)
    a_fast = (g.xs[3] == 1 and g.Cin % 4 == 0 and g.LH == 1 and g.LW == 1 and lhs_offset % 4 == 0 and g.PH >= 0 and g.PW >= 0
              and all(s % 4 == 0 and s >= 0 for s in g.xs[:3]) and (not needs_masks or g.KH * g.KW <= 32)
              and (lhs.size - lhs_offset) * 4 + x_bias <= 2**31)
    #16-byte loads of the kernel operand need a dense [ky, kx, in, out] array, not an output width that is a multiple of 4:
    #a buffer load of four words only has to start at a word (verified on gfx950 with integer-exact products of odd
    #widths); the words a vector reads beyond its row belong to columns >= N, which are never stored
    b_fast = (g.ws[3] == 1 and rhs_offset % 4 == 0 and not CHOICES.conv_b_general
              and g.ws[2] == N and g.ws[1] == g.Cin * N and g.ws[0] == g.KW * g.Cin * N)
    c_contig = g.os == (g.Ho * g.Wo * N, g.Wo * N, N, 1)
    return needs_masks, x_bias, a_fast, b_fast, c_contig


def _four_waves_per_tile(g: ConvGeometry, a_fast: bool, c_contig: bool, compute_units: int) -> bool:
    '''A product with so few 32 x 32 tiles that one wave per tile leaves most MFMA units idle: four waves per tile,
    each taking a quarter of every (128-long) k step.'''
    want = (CHOICES.conv_ksplit if CHOICES.conv_ksplit is not None else
            (_cdiv(g.M, 32) * _cdiv(g.N, 32) <= 2 * compute_units and g.K >= 256 and CHOICES.conv_tile is None and CHOICES.conv_bk is None))
    return bool(want) and a_fast and c_contig and (g.Cin % 64 == 0 or g.KH * g.KW == 1) and not CHOICES.conv_general




def conv_k_splits(lhs: Buffer, rhs: Buffer, g: ConvGeometry, compute_units: int = 256) -> int:
    '''Into how many slices the contraction of a product with very few tiles is cut (1: not at all). With 32 blocks on
    256 CUs, a layer whose kernel operand is megabytes long (the 3 x 3 layers of a network's last stages at batch 1)
    is bound by the rate at which those few CUs fetch it; slices spread the fetch over the chip. Every slice keeps at
    least four k steps, at most four slices (the launch that adds them is an element-wise chain with room for a
    following scale, shift and ReLU), and never more blocks than CUs.'''
    if _dense_rows_shape(lhs, g):
        return 1
    g = _flatten_pointwise(g)
    if g.K * g.N * 4 >= 2**31 or lhs.size * 4 >= 2**31 or g.M * g.N == 0:
        return 1
    _, _, a_fast, _, c_contig = _conv_fast_paths(lhs, rhs, g)
    if not _four_waves_per_tile(g, a_fast, c_contig, compute_units) or (g.Cin % 128 != 0 and g.KH * g.KW != 1):
        return 1
    tiles, ksteps = _cdiv(g.M, 32) * _cdiv(g.N, 32), _cdiv(g.K, 128)
    if CHOICES.conv_k_splits is not None:
        want = CHOICES.conv_k_splits
    else:
        want = min(4, compute_units // tiles, ksteps // 4)
    if want <= 1 or ksteps < 2:
        return 1
    per = _cdiv(ksteps, min(want, ksteps))
    return _cdiv(ksteps, per)


def conv_gemm(out: Buffer, lhs: Buffer, rhs: Buffer, g: ConvGeometry, epilogue: tp.Sequence[ConvEpilogueStep] = (),
              compute_units: int = 256, lhs_offset: int = 0, rhs_offset: int = 0, out_offset: int = 0) -> Launch:
    taps = [(i, e.operand) for i, e in enumerate(epilogue) if e.op == CONV_TAP]
    if taps:
        (tap_position, tap_buffer), = taps
        epilogue = [e for e in epilogue if e.op != CONV_TAP]
        if (not conv_tap_supported(epilogue[:tap_position], epilogue[tap_position:]) or out_offset or tap_buffer.size != out.size):
            raise ValueError('a second result at this point of the epilogue is not supported')
    softmax, arg_out = False, None
    if epilogue and epilogue[-1].op == CONV_SOFTMAX:
        softmax, arg_out = True, epilogue[-1].operand
        epilogue = list(epilogue[:-1])
        if len(epilogue) > CONV_MAX_EPI - 1 or (arg_out is not None and arg_out.size != g.M):
            raise ValueError('softmax epilogue: too many steps, or labels of another size')
    if any(e.op == CONV_SOFTMAX for e in epilogue):
        raise ValueError('softmax can only be the last step of an epilogue')
    if len(epilogue) > CONV_MAX_EPI:
        raise ValueError('too many epilogue steps')
    g_given, g = g, _flatten_pointwise(g)
    M, N, K = g.M, g.N, g.K
    for name, extent in (('lhs', lhs.size), ('rhs', rhs.size), ('out', out.size)):
        if extent * 4 >= 2**31:
            raise NotImplementedError(f'conv/dot {name} operand of {extent * 4} bytes exceeds the 2 GiB the kernel addresses')
    rows = _dense_rows_launch(out, lhs, rhs, g_given, epilogue, taps, lhs_offset, rhs_offset, out_offset, softmax, arg_out)
    if rows is not None:
        return rows
    if softmax:
        raise ValueError('softmax epilogue: only in the kernel for at most 16 output features')
    stem = _conv_stem_launch(out, lhs, rhs, g, epilogue, taps, compute_units, lhs_offset, rhs_offset, out_offset)
    if stem is not None:
        return stem
    tag, bm, bn, nt = choose_conv_tile(M, N, compute_units)
    bk = choose_conv_bk(tag, g)
    needs_masks, x_bias, a_fast, b_fast, c_contig = _conv_fast_paths(lhs, rhs, g, lhs_offset, rhs_offset)
    slots = _epilogue_template_slots(epilogue)
    #the lean kernel variant covers the common case only (see the kernel source)
    lean = (a_fast and b_fast and c_contig and (g.Cin % bk == 0 or g.KH * g.KW == 1)
            and (not epilogue or slots != 0) and not CHOICES.conv_general)
    #the output row number is the input row number (a matrix product, or a one-column image walked without stride,
    #padding or taps outside the input): the kernel then skips the row decode and the validity masks
    flat_rows = g.batch == 1 and g.Wo == 1 and g.SH == 1 and g.PH == 0 and g.PW == 0 and not needs_masks
    #a product with so few 32 x 32 tiles that one wave per tile leaves most MFMA units idle: four waves per
    #tile, each taking a quarter of every (128-long) k step
    ksplit = _four_waves_per_tile(g, a_fast, c_contig, compute_units) and (not epilogue or slots != 0)
    #(windows over 64 input features take a 64-long k step, with 16-byte loads of the kernel operand only)
    short_step = ksplit and g.Cin % 128 != 0 and g.KH * g.KW != 1
    if short_step and not b_fast:
        ksplit = False
    if ksplit:
        tag, bm, bn, nt, bk, lean = '32x32', 32, 32, 256, 64 if short_step else 128, True
    tiles_m, tiles_n = _cdiv(M, bm), _cdiv(N, bn)
    k_split_steps = 0
    if g.k_splits > 1:
        k_split_steps = _cdiv(_cdiv(K, 128), g.k_splits)
        if (not ksplit or short_step or epilogue or taps or out_offset or out.size != g.k_splits * M * N
                or _cdiv(_cdiv(K, 128), k_split_steps) != g.k_splits):
            raise ValueError('a sliced contraction needs the four-waves-per-tile kernel, no epilogue and one [M, N] matrix per non-empty slice')
    chunk = (CHOICES.conv_chunk or choose_conv_chunk(tiles_m, tiles_n, compute_units)) if lean and not ksplit else 1
    m_blocks = 0
    if lean and not ksplit and CHOICES.conv_chunk is None:
        m_blocks = choose_conv_m_blocks(tiles_m, tiles_n, compute_units)
        if m_blocks:
            chunk = 2                          #(a value other than 1 keeps the mixed tiling out; the kernel ignores it)
    #64 x 64 tiles that do not divide evenly among the CUs: as many M tiles as fill every CU equally stay 64 x 64, the
    #rows behind them are computed as 32 x 32 tiles with four waves per tile (a quarter of the work each)
    split_tiles_m = 0
    mixable = (lean and not ksplit and tag == '64x64' and chunk == 1 and b_fast and (g.Cin % 64 == 0 or g.KH * g.KW == 1) and K >= 256)
    if mixable and CHOICES.conv_mix is not None and CHOICES.conv_mix is not False:
        split_tiles_m = int(CHOICES.conv_mix)                      #tests: whatever the other pinned choices are
    elif mixable and CHOICES.conv_mix is None and CHOICES.conv_tile is None and CHOICES.conv_bk is None and CHOICES.conv_chunk is None:
        split_tiles_m = choose_conv_split(tiles_m, tiles_n, compute_units)
    if split_tiles_m >= tiles_m:
        split_tiles_m = 0
    kinds = [e.kind for e in epilogue]
    x_bytes = (lhs.size - lhs_offset) * 4
    w_bytes = K * N * 4 if b_fast else (rhs.size - rhs_offset) * 4
    first_full = kinds.index(3) + 1 if 3 in kinds else 0
    flags = (int(c_contig) | int(flat_rows) << 1 | int(needs_masks) << 2 | len(epilogue) << 8 | first_full << 16
             | slots << 20 | chunk << 25 | ((tap_position + 1) << 12 if taps else 0))
    if ksplit:
        flags |= choose_conv_xcd_columns(M, N, K, tiles_m, tiles_n) << 29
    descs = [0, 0]
    for i, e in enumerate(epilogue):
        assert e.op < 128 and 1 <= e.kind <= 3
        descs[i // 3] |= ((e.op * 2 + int(e.operand_left)) | e.kind << 8) << (10 * (i % 3))
    params = (_i32(M, N, K, g.Ho, g.Wo, g.H, g.W, g.Cin, g.KH, g.KW, g.SH, g.SW, g.PH, g.PW, g.DH, g.DW,
                   *g.xs[:3], tiles_m, tiles_n)
              #(rows beyond M are dropped by the descriptor's size: with slices, that of one slice's matrix)
              + _u32(flags, *descs, x_bytes, w_bytes, M * N * 4 if k_split_steps else (out.size - out_offset) * 4,
                     *_magic_division(g.Ho * g.Wo), *_magic_division(g.Wo))
              + _i32(g.LH, g.LW, g.xs[3], *g.ws, *g.os, split_tiles_m, k_split_steps, m_blocks, tiles_m // m_blocks if m_blocks else 0, tiles_m % m_blocks if m_blocks else 0))
    derived_ptrs, derived_desc = _conv_derived(epilogue, N)
    params += derived_desc
    buffers = [(out, out_offset * 4), (lhs, lhs_offset * 4), (rhs, rhs_offset * 4)]
    operand_slots = _pad([(e.operand, 0) for e in epilogue], CONV_MAX_EPI, (None, 0))
    if taps:
        assert operand_slots[-1] == (None, 0)
        operand_slots[-1] = (tap_buffer, 0)
    buffers += operand_slots + derived_ptrs
    kernel  = f'conv_gemm_{tag}x{bk}_' + (('ks4' if b_fast else 'ks4g') if ksplit else 'lean' if lean else ('f' if a_fast else 'g') + ('f' if b_fast else 'g'))
    nbytes  = 4 * (lhs.size + rhs.size + out.size) + sum(4 * e.operand.size for e in epilogue if e.operand is not None)
    nbytes += 4 * tap_buffer.size if taps else 0
    blocks = (m_blocks or _cdiv(tiles_m, chunk)) * tiles_n * max(1, g.k_splits)
    if split_tiles_m:
        kernel = f'conv_gemm_{tag}x{bk}_mix'
        blocks = split_tiles_m * tiles_n + _cdiv(M - split_tiles_m * 64, 32) * _cdiv(N, 32)
    return Launch(kernel, (blocks, 1, 1), (nt, 1, 1), buffers, params, bytes_moved=nbytes, flops=2 * M * N * K)


# --------------------------------------------------------------------------- reductions

RED = dict(reduce_sum=0, reduce_prod=1, reduce_max=2, reduce_min=3, argmax=4, argmin=5)
_RTYPE = {np.dtype('float32'): 0, np.dtype('int32'): 1, np.dtype('uint32'): 2, np.dtype('bool'): 2}


def _pow2_at_least(x: int) -> int:
    p = 1
    while p < x:
        p *= 2
    return p


def plan_reduce_splits(outer: int, R: int, inner: int, op: str, compute_units: int = 256) -> int:
    '''Into how many ranges R is cut so that outer x inner x splits fills the GPU (1 = a single launch).'''
    if op in ('argmax', 'argmin'):
        return 1                                   #index-returning reductions run unsplit
    if inner == 1:
        want  = 32 * compute_units                 #waves
        split = min(_cdiv(want, outer), R // 4096)         #at least 16 KB per wave
    else:
        tiles = _cdiv(inner, 256)
        #blocks: several per CU for arrays that stream from HBM for a while; one per CU for smaller ones, whose
        #second launch (it reduces the per-block results) would otherwise take as long as the first
        want  = (4 if outer * R * inner * 4 >= (128 << 20) else 1) * compute_units
        split = min(_cdiv(want, tiles * outer), R // 64)   #at least 64 rows per block
    return max(1, min(split, 65535))


def _reduce_launch(out: Buffer, inp: Buffer, outer: int, R: int, inner: int, op: str, nsplit: int, in_offset_ok=True,
                   prologue: tp.Optional[tp.Tuple[str, tp.Optional[Buffer]]] = None,
                   post: tp.Optional[tp.Tuple[str, Buffer]] = None) -> Launch:
    ty   = _RTYPE[inp.dtype]
    mode = {('reduce_sum', 0): 'fsum', ('reduce_max', 0): 'fmax', ('argmax', 0): 'fargmax', ('argmin', 0): 'fargmin'}.get((op, ty), 'any')
    r_chunk = _cdiv(_cdiv(R, nsplit), 4) * 4
    nsplit  = _cdiv(R, r_chunk)
    if post is not None:
        #('div' | 'times', one value): applied to every finished float sum of an unsplit reduction
        assert mode == 'fsum' and nsplit == 1 and prologue is None and post[0] in ('div', 'times') and post[1].size == 1
    if inner == 1:
        vec = 4 if R % 4 == 0 else 1
        params = _u32(outer, R, 1, RED[op], ty, r_chunk, nsplit, 0)
        if post is not None:
            return Launch(f'reduce_rows_fsum_{post[0]}_v{vec}', (_cdiv(outer * nsplit, 4), 1, 1), (BLOCK, 1, 1), [(out, 0), (inp, 0), (post[1], 0)],
                          params, bytes_moved=4 * (outer * R + outer * nsplit)), nsplit
        return Launch(f'reduce_rows_{mode}_v{vec}', (_cdiv(outer * nsplit, 4), 1, 1), (BLOCK, 1, 1), [(out, 0), (inp, 0)], params,
                      bytes_moved=4 * (outer * R + outer * nsplit)), nsplit
    vec = 4 if inner % 4 == 0 else 1
    TI  = min(64, _pow2_at_least(_cdiv(inner, vec)))
    #few blocks with many rows each (the second stage of a split sum): narrower blocks, more of them, more thread rows
    #walking the rows side by side
    #(up to the number of blocks below which small sums are batched with their neighbours into one launch)
    while TI > 8 and 2 * _cdiv(inner, TI * vec) * nsplit * outer <= REDUCE_NARROW_MAX_BLOCKS and _cdiv(R, nsplit) >= 128:
        TI //= 2
    params = _u32(outer, R, inner, RED[op], ty, r_chunk, nsplit, TI)
    blocks = _cdiv(inner, TI * vec) * nsplit * outer
    if blocks >= 2**31:
        raise NotImplementedError(f'reduction with {outer} outer rows and inner size {inner}')
    if prologue is not None:
        #the operand's element-wise producer applied while loading: ('mul', array of the same shape),
        #('mulv', vector over inner) or ('neg', None); float column sums only
        kind, second = prologue
        assert mode == 'fsum' and kind in ('mul', 'mulv', 'neg') and (second is None) == (kind == 'neg')
        assert second is None or second.size == (outer * R * inner if kind == 'mul' else inner)
        extra = 0 if second is None else second.size
        return Launch(f'reduce_cols_fsum_{kind}_v{vec}', (blocks, 1, 1), (BLOCK, 1, 1), [(out, 0), (inp, 0), (second, 0)], params,
                      bytes_moved=4 * (outer * R * inner + outer * nsplit * inner + extra)), nsplit
    if post is not None:
        return Launch(f'reduce_cols_fsum_{post[0]}_v{vec}', (blocks, 1, 1), (BLOCK, 1, 1), [(out, 0), (inp, 0), (post[1], 0)], params,
                      bytes_moved=4 * (outer * R * inner + outer * nsplit * inner)), nsplit
    return Launch(f'reduce_cols_{mode}_v{vec}', (blocks, 1, 1), (BLOCK, 1, 1), [(out, 0), (inp, 0)], params,
                  bytes_moved=4 * (outer * R * inner + outer * nsplit * inner)), nsplit


def reduce(out: Buffer, inp: Buffer, outer: int, R: int, inner: int, op: str,
           partial: tp.Optional[Buffer] = None, nsplit: int = 1, prologue=None, post=None) -> tp.List[Launch]:
    '''[outer, R, inner] -> [outer, inner]. With nsplit > 1, `partial` (outer * nsplit * inner words) receives
    the per-range results of a first launch and a second launch reduces them. `prologue`, `post`: see _reduce_launch.'''
    if nsplit <= 1:
        return [_reduce_launch(out, inp, outer, R, inner, op, 1, prologue=prologue, post=post)[0]]
    assert post is None
    first, nsplit = _reduce_launch(partial, inp, outer, R, inner, op, nsplit, prologue=prologue)
    if nsplit == 1:
        return [_reduce_launch(out, inp, outer, R, inner, op, 1, prologue=prologue)[0]]
    assert partial.size >= outer * nsplit * inner and partial.dtype == inp.dtype
    second = _reduce_launch(out, partial, outer, nsplit, inner, op, 1)[0]
    return [first, second]


def scale_relu_backward(column_sum: Launch, dx: Buffer, sum_m: Buffer, sum_mx: Buffer, x: Buffer, scale: Buffer, cotangent: Buffer,
                        select: tp.Optional[tp.Tuple[Buffer, Buffer, Buffer]] = None) -> Launch:
    '''dx = m * scale (scale a vector over the columns), and sum_m, sum_mx receive what `column_sum`, a reduce_cols
    launch over an array of that shape, would write for m and for m * x (same grid, same parameters, same order
    of additions). m is the cotangent itself, or with select = (ans, threshold, otherwise), two single values:
    ans > threshold ? cotangent : otherwise.'''
    assert column_sum.kernel in ('reduce_cols_fsum_v1', 'reduce_cols_fsum_v4'), column_sum.kernel
    n = cotangent.size
    assert dx.size == x.size == n
    ans, threshold, otherwise = select if select is not None else (None, None, None)
    assert select is None or (ans.size == n and threshold.size == otherwise.size == 1)
    name = 'scale_relu_backward_' if select is not None else 'scale_backward_'
    return Launch(name + column_sum.kernel[-2:], column_sum.grid, column_sum.block,
                  [(dx, 0), (sum_m, 0), (sum_mx, 0), (ans, 0), (threshold, 0), (cotangent, 0), (otherwise, 0), (x, 0), (scale, 0)],
                  column_sum.params, bytes_moved=4 * ((4 if select is not None else 3) * n + 2 * scale.size), written=(0, 1, 2))


SOFTMAX_MAX_ROW = 4096      #rows this short run unsplit in reduce_rows, whose summation order softmax_rows repeats


def softmax_rows(out: Buffer, inp: Buffer, outer: int, R: int, arg_out: tp.Optional[Buffer] = None) -> Launch:
    '''exp(x - max) / sum(exp(x - max)) over the rows of [outer, R]; see softmax_rows_body in reduce.hip.
    `arg_out`: also the arg-max of every result row (int32 [outer]).'''
    assert 0 < R < SOFTMAX_MAX_ROW and inp.size == out.size == outer * R and (arg_out is None or arg_out.size == outer)
    vec = 4 if R % 4 == 0 else 1
    return Launch(f'softmax_rows_v{vec}', (_cdiv(outer, 4), 1, 1), (BLOCK, 1, 1), [(out, 0), (inp, 0), (arg_out, 0)], _u32(outer, R),
                  bytes_moved=8 * outer * R + (4 * outer if arg_out is not None else 0), written=(0, 2))


def reduce_general(out: Buffer, inp: Buffer, kept, reduced, op: str) -> Launch:
    '''kept / reduced: lists of (size, stride) in row-major order of the output / of the reduce index.'''
    if len(kept) > 4 or len(reduced) > 4:
        raise NotImplementedError('reduction over more than 4 separate dimension groups')
    n_out = int(np.prod([k[0] for k in kept], dtype=np.int64))
    n_red = int(np.prod([r[0] for r in reduced], dtype=np.int64))
    params = _u32(n_out, n_red, RED[op], _RTYPE[inp.dtype], len(kept), len(reduced),
                  *_pad([k[0] for k in kept], 4, 1), *_pad([k[1] for k in kept], 4),
                  *_pad([r[0] for r in reduced], 4, 1), *_pad([r[1] for r in reduced], 4))
    return Launch('reduce_general', (_cdiv(n_out, 4), 1, 1), (BLOCK, 1, 1), [(out, 0), (inp, 0)], params,
                  bytes_moved=4 * (inp.size + out.size))


def _pool_divisions(dims) -> bytes:
    '''PoolParams.div_magic / div_shift for an array [batch, height, width, channels]: channels, width, height.'''
    pairs = [_magic_division(d) for d in (dims[3], dims[2], dims[1])]
    return _u32(*[m for m, _ in pairs], *[sh for _, sh in pairs])


def pool(out: Buffer, inp: Buffer, op: str, window, strides, pad_low, dilation) -> Launch:
    rank = len(inp.shape)
    if rank > 4:
        raise NotImplementedError('window reductions over more than 4 dimensions')
    lead     = 4 - rank
    in_dims  = [1] * lead + list(inp.shape)
    out_dims = [1] * lead + list(out.shape)
    window   = [1] * lead + list(window)
    strides  = [1] * lead + list(strides)
    dilation = [1] * lead + list(dilation)
    pad_low  = [0] * lead + list(pad_low)
    n   = out.size
    vec = 4 if (window[3] == 1 and strides[3] == 1 and pad_low[3] == 0 and in_dims[3] % 4 == 0
                and in_dims[3] == out_dims[3]) else 1
    params = (_u32(n, RED[op], _RTYPE[inp.dtype], *in_dims, *out_dims, *window, *strides, *dilation) + _i32(*pad_low)
              + _pool_divisions(out_dims))
    #[batch, y, x, channels] with a 3x3 or 2x2 window over y and x: the kernel that requests all taps at once
    if (vec == 4 and window[0] == 1 and strides[0] == 1 and pad_low[0] == 0 and in_dims[0] == out_dims[0]
            and (window[1], window[2]) in ((3, 3), (2, 2)) and inp.size * 4 < 2**31 and n * 4 < 2**32):
        return Launch(f'pool2d_{window[1]}x{window[2]}_v4', (_cdiv(_cdiv(n, 4), BLOCK), 1, 1), (BLOCK, 1, 1), [(out, 0), (inp, 0)], params,
                      bytes_moved=4 * (inp.size + out.size))
    return Launch(f'pool_v{vec}', (_cdiv(_cdiv(n, vec), BLOCK), 1, 1), (BLOCK, 1, 1), [(out, 0), (inp, 0)], params,
                  bytes_moved=4 * (inp.size + out.size))


def select_scatter_add(out: Buffer, source: Buffer, operand: Buffer, selected: Buffer, op: str, window, strides, pad_low) -> tp.List[Launch]:
    '''Gradient of a max (`op` = 'reduce_max': select with ge) or min pooling in two launches: the selected tap
    of every window into `selected` (uint32, source's shape), then the per-element sums; see reduce.hip.'''
    rank = len(operand.shape)
    if rank > 4:
        raise NotImplementedError('select_and_scatter_add over more than 4 dimensions')
    lead     = 4 - rank
    in_dims  = [1] * lead + list(operand.shape)
    out_dims = [1] * lead + list(source.shape)
    window   = [1] * lead + list(window)
    strides  = [1] * lead + list(strides)
    pad_low  = [0] * lead + list(pad_low)
    vec = 4 if (window[3] == 1 and strides[3] == 1 and pad_low[3] == 0 and in_dims[3] % 4 == 0
                and in_dims[3] == out_dims[3]) else 1
    if max(in_dims) >= 2**31 or any(abs(p) >= 2**30 for p in pad_low):
        raise NotImplementedError('select_and_scatter_add: dimension too large')
    assert tuple(selected.shape) == tuple(source.shape) and selected.dtype == np.uint32
    tail = _u32(RED[op], _RTYPE[operand.dtype], *in_dims, *out_dims, *window, *strides, 1, 1, 1, 1) + _i32(*pad_low)
    n_win, n = source.size, operand.size
    select, scatter = f'select_window_v{vec}', f'scatter_selected_v{vec}'
    #[batch, y, x, channels] floats with a 3x3 or 2x2 window over y and x: the kernels that request everything at once
    if (vec == 4 and window[0] == 1 and strides[0] == 1 and pad_low[0] == 0 and in_dims[0] == out_dims[0] and CHOICES.pool_gradient_2d is not False
            and (window[1], window[2]) in ((3, 3), (2, 2)) and operand.dtype == np.float32 and n * 4 < 2**31 and n_win * 4 < 2**31):
        #(an element lies in at most ceil(window / stride) windows per dimension; the variants are square in that count)
        most = max(_cdiv(window[1], strides[1]), _cdiv(window[2], strides[2]))
        select, scatter = f'select_window2d_{window[1]}x{window[2]}_v4', f'scatter_selected2d_{window[1]}x{window[2]}_n{most}x{most}_v4'
    first  = Launch(select, (_cdiv(_cdiv(n_win, vec), BLOCK), 1, 1), (BLOCK, 1, 1),
                    [(selected, 0), (operand, 0)], _u32(n_win) + tail + _pool_divisions(out_dims), bytes_moved=4 * (operand.size + source.size))
    second = Launch(scatter, (_cdiv(_cdiv(n, vec), BLOCK), 1, 1), (BLOCK, 1, 1),
                    [(out, 0), (source, 0), (selected, 0)], _u32(n) + tail + _pool_divisions(in_dims), bytes_moved=4 * (operand.size + 2 * source.size),
                    streamable=vec == 4 and n < 2**31)
    #3 x 3 windows at a stride of 2: a thread per group of 2 x 2 elements (by four channels), which shares its windows' loads
    if ('2d_3x3' in scatter and (strides[1], strides[2]) == (2, 2) and 0 <= pad_low[1] < 3 and 0 <= pad_low[2] < 3
            and CHOICES.pool_gradient_2d != 'elements'):
        groups = [((extent + pad - 1) >> 1) - (pad >> 1) + 1 for extent, pad in ((in_dims[1], pad_low[1]), (in_dims[2], pad_low[2]))]
        n_groups = in_dims[0] * groups[0] * groups[1] * in_dims[3]
        second = second._replace(kernel='scatter_selected2d_3x3_s2_v4', grid=(_cdiv(_cdiv(n_groups, 4), BLOCK), 1, 1),
                                 params=_u32(n_groups) + tail + _pool_divisions([in_dims[0], groups[0], groups[1], in_dims[3]]),
                                 streamable=n_groups < 2**31)
    return [first, second]


PAD_MAX_RANK = 6


def _merged_pad_dims(out_shape, in_shape, padding_config):
    '''(out extent, in extent, low, step) per dimension after folding every dimension the padding leaves alone into
    the one before it when that one has no interior padding: (w, c) -> w * C + c turns `low` into low * C.'''
    dims = [(int(o), int(i), int(c[0]), int(c[2]) + 1) for o, i, c in zip(out_shape, in_shape, padding_config)]
    merged: tp.List[tp.Tuple[int, int, int, int]] = []
    for o, i, low, step in reversed(dims):
        if merged:
            o2, i2, low2, step2 = merged[-1]
            if low2 == 0 and step2 == 1 and o2 == i2 and step == 1:
                merged[-1] = (o * o2, i * o2, low * o2, 1)
                continue
        merged.append((o, i, low, step))
    return merged[::-1]


def pad(out: Buffer, inp: Buffer, value: Buffer, padding_config) -> Launch:
    dims = _merged_pad_dims(out.shape, inp.shape, padding_config)
    if len(dims) > PAD_MAX_RANK:
        raise NotImplementedError('pad with rank > 6')
    if max(out.size, inp.size) >= 2**32 - 2**12 or any(abs(d[2]) >= 2**31 for d in dims):
        raise NotImplementedError('pad of arrays with 2^32 elements or more')
    #the dimensions fill the front of the tables (the kernel does not split its index for dimension 0) and the unused
    #ones behind them have extent 1; an empty operand keeps an extent of 0 no index can fall into
    dims = dims + [(1, 1, 0, 1)] * (PAD_MAX_RANK - len(dims))
    last = max((d for d in range(PAD_MAX_RANK) if dims[d][:3] != (1, 1, 0)), default=0)
    o, i, low, step = dims[last]
    vec = 4 if (step == 1 and low % 4 == 0 and o % 4 == 0 and i % 4 == 0) else 1
    params = _u32(out.size, *[d[0] for d in dims], *[d[1] for d in dims]) + _i32(*[d[2] for d in dims]) + _u32(*[d[3] for d in dims])
    return Launch(f'pad_nd_v{vec}', (_cdiv(_cdiv(out.size, vec), BLOCK), 1, 1), (BLOCK, 1, 1),
                  [(out, 0), (inp, 0), (value, 0)], params, bytes_moved=4 * (inp.size + out.size), streamable=vec == 4 and out.size < 2**31)


# --------------------------------------------------------------------------- gather / scatter / rng

IDX_MAX_RANK = 6


def gather_rows(out: Buffer, table: Buffer, idx: Buffer, n_idx: int, row_len: int, n_rows: int, idx_stride: int = 1,
                fill: tp.Optional[int] = None) -> Launch:
    '''`fill`: None clamps rows outside the table; a 32-bit pattern makes them read as that value instead.'''
    vec = 4 if row_len % 4 == 0 else 1
    total = n_idx * (row_len // vec)
    return Launch(f'gather_rows_v{vec}', (_cdiv(total, BLOCK), 1, 1), (BLOCK, 1, 1), [(out, 0), (table, 0), (idx, 0)],
                  _u32(n_idx, row_len, n_rows, idx_stride, int(fill is not None), fill or 0, 0), bytes_moved=4 * (2 * n_idx * row_len + n_idx),
                  streamable=vec == 4 and n_idx < 2**31)


def gather_general(out: Buffer, operand: Buffer, indices: Buffer, offset_dims, collapsed, start_index_map, slice_sizes,
                   fill: tp.Optional[int] = None) -> Launch:
    out_rank, op_rank = len(out.shape), len(operand.shape)
    if max(out_rank, op_rank, len(indices.shape)) > IDX_MAX_RANK:
        raise NotImplementedError('gather with rank > 6')
    batch_dims = list(indices.shape[:-1])
    params = _u32(out.size, out_rank, op_rank, indices.shape[-1],
                  *_pad(out.shape, IDX_MAX_RANK, 1), *_pad([int(d in offset_dims) for d in range(out_rank)], IDX_MAX_RANK),
                  *_pad(operand.shape, IDX_MAX_RANK, 1), *_pad(row_major_strides(operand.shape), IDX_MAX_RANK),
                  *_pad(slice_sizes, IDX_MAX_RANK, 1), *_pad([int(d in collapsed) for d in range(op_rank)], IDX_MAX_RANK),
                  *_pad(start_index_map, IDX_MAX_RANK), *_pad(batch_dims, IDX_MAX_RANK, 1), len(batch_dims),
                  int(fill is not None), fill or 0)
    return Launch('gather_general', (_cdiv(out.size, BLOCK), 1, 1), (BLOCK, 1, 1), [(out, 0), (operand, 0), (indices, 0)],
                  params, bytes_moved=4 * (2 * out.size + indices.size))


#kernels that can add a value to negative indices themselves: position of the index array among their arguments, and the
#byte offset of the `wrap` field in their parameter block
INDEX_WRAP_KERNELS = {'gather_rows_v1': (2, 24), 'gather_rows_v4': (2, 24), 'scatter_rows_rank': (3, 24)}


def with_wrapped_index(launch: Launch, raw: Buffer, raw_byte_offset: int, amount: int) -> Launch:
    '''`launch` reading the raw index array `raw` instead of its normalised copy, adding `amount` to negative indices itself.'''
    position, field = INDEX_WRAP_KERNELS[launch.kernel]
    assert launch.params[field:field + 4] == _u32(0)
    buffers = list(launch.buffers)
    buffers[position] = (raw, buffers[position][1] + raw_byte_offset)
    return launch._replace(buffers=buffers, params=launch.params[:field] + _u32(amount) + launch.params[field + 4:])


def scatter_add_rows(out: Buffer, idx: Buffer, updates: Buffer, n_idx: int, row_len: int, n_rows: int, idx_stride: int = 1,
                     clip: bool = False) -> Launch:
    '''`clip`: rows outside the table go to its first / last row instead of being dropped.'''
    total = n_idx * row_len
    return Launch('scatter_add_rows', (_cdiv(total, BLOCK), 1, 1), (BLOCK, 1, 1), [(out, 0), (idx, 0), (updates, 0)],
                  _u32(n_idx, row_len, n_rows, idx_stride, int(out.dtype == np.float32), int(clip)),
                  bytes_moved=4 * (total + n_idx + out.size))


def choose_scatter_bucket_cap(n_idx: int, n_rows: int, row_len: int) -> int:
    '''How many slots every table row gets in the sorted scatter-add's table of fixed-capacity buckets (0: none, every
    update goes through the overflow table): four times the average number of updates per row, as a power of two
    between 4 and 64 - with indices spread evenly a row with more than that is a rarity - as long as the slots take at
    most an eighth of the table's own size and eight words per update.'''
    if CHOICES.scatter_bucket_cap is not None:
        cap = int(CHOICES.scatter_bucket_cap)
        assert 0 <= cap <= 64
        return cap
    if n_rows == 0 or n_idx == 0:
        return 0
    cap = 4
    while cap < 64 and cap * n_rows < 4 * n_idx:
        cap *= 2
    while cap >= 4 and (cap * 8 > row_len or cap * n_rows > 8 * n_idx):
        cap //= 2
    return cap if cap >= 4 else 0


def scatter_table_slots(n_idx: int) -> int:
    '''Slots of the overflow table of a sorted scatter-add of n_idx updates: a power of two, at least 64 and at least
    twice the number of updates.'''
    return max(64, _pow2_at_least(2 * n_idx))


def scatter_add_rows_sorted(out: Buffer, operand: Buffer, idx: Buffer, updates: Buffer, count: Buffer, table: Buffer, gathered: Buffer,
                            sorted_: Buffer, n_idx: int, row_len: int, n_rows: int, operand_is_scalar: bool = False,
                            idx_stride: int = 1, clip: bool = False, fixed: tp.Optional[Buffer] = None, cap: int = 0) -> tp.List[Launch]:
    '''out = operand; out[idx[i], :] += updates[i, :] without atomics on the data: the first launch buckets the updates by
    row, then one wave per row sums its bucket. `count`: n_rows + 1 words, `table`: two words per slot of the overflow
    table (scatter_table_slots), both zero before and after; `fixed`: n_rows * cap words, the first `cap` updates of
    every row (cap = 0: no such table); `gathered`, `sorted_`: n_idx words each, room for the buckets of rows with
    more than cap updates. `operand` is the table, or one word when the table is a constant filled with a single
    value.'''
    slots = scatter_table_slots(n_idx)
    assert count.size == n_rows + 1 and table.size == 2 * slots and gathered.size == n_idx and sorted_.size == n_idx
    assert 0 <= cap <= 64 and (cap == 0 or (fixed is not None and fixed.size == n_rows * cap))
    if fixed is None:
        fixed = gathered                 #(never touched: no update's number within its row is below 0)
    params = _u32(n_idx, row_len, n_rows, idx_stride, int(operand_is_scalar), int(clip), 0, cap, slots - 1)
    vec    = 4 if row_len % 4 == 0 else 1
    kind   = 'f' if out.dtype == np.float32 else 'i'
    table_passes = 1 if operand_is_scalar else 2
    return [
        Launch('scatter_rows_rank', (_cdiv(n_idx, BLOCK), 1, 1), (BLOCK, 1, 1), [(count, 0), (fixed, 0), (table, 0), (idx, 0)], params,
               bytes_moved=8 * n_idx, written=(0, 1, 2)),
        Launch(f'scatter_rows_sum_{kind}_v{vec}', (_cdiv(n_rows, 4), 1, 1), (BLOCK, 1, 1),      #one wave per row
               [(out, 0), (operand, 0), (updates, 0), (count, 0), (fixed, 0), (table, 0), (gathered, 0), (sorted_, 0)], params,
               bytes_moved=4 * (n_idx * row_len + n_idx + n_rows + table_passes * n_rows * row_len), written=(0, 3, 5, 6, 7)),
    ]


def scatter_add_general(out: Buffer, indices: Buffer, updates: Buffer, update_window_dims, inserted_window_dims,
                        scatter_dims_to_operand_dims, clip: bool = False) -> Launch:
    upd_rank, op_rank = len(updates.shape), len(out.shape)
    if max(upd_rank, op_rank, len(indices.shape)) > IDX_MAX_RANK:
        raise NotImplementedError('scatter-add with rank > 6')
    window_dims = [updates.shape[d] for d in update_window_dims]
    it = iter(window_dims)
    window_sizes = [1 if d in inserted_window_dims else next(it) for d in range(op_rank)]
    batch_dims = list(indices.shape[:-1])
    params = _u32(updates.size, upd_rank, op_rank, indices.shape[-1], int(out.dtype == np.float32),
                  *_pad(updates.shape, IDX_MAX_RANK, 1), *_pad([int(d in update_window_dims) for d in range(upd_rank)], IDX_MAX_RANK),
                  *_pad(out.shape, IDX_MAX_RANK, 1), *_pad(row_major_strides(out.shape), IDX_MAX_RANK),
                  *_pad([int(d in inserted_window_dims) for d in range(op_rank)], IDX_MAX_RANK),
                  *_pad(window_sizes, IDX_MAX_RANK, 1), *_pad(scatter_dims_to_operand_dims, IDX_MAX_RANK),
                  *_pad(batch_dims, IDX_MAX_RANK, 1), int(clip))
    return Launch('scatter_add_general', (_cdiv(max(updates.size, 1), BLOCK), 1, 1), (BLOCK, 1, 1),
                  [(out, 0), (indices, 0), (updates, 0)], params, bytes_moved=4 * (updates.size + indices.size + out.size))


def threefry2x32(out0: Buffer, out1: Buffer, key0: Buffer, key1: Buffer, x0: Buffer, x1: Buffer, key_is_scalar: bool) -> Launch:
    n   = x0.size
    vec = 4 if n % 4 == 0 else 1
    return Launch(f'threefry2x32{"_k" if key_is_scalar else ""}_v{vec}', (_cdiv(_cdiv(n, vec), BLOCK), 1, 1), (BLOCK, 1, 1),
                  [(out0, 0), (out1, 0), (key0, 0), (key1, 0), (x0, 0), (x1, 0)], _u32(n, int(key_is_scalar)),
                  bytes_moved=16 * n, written=(0, 1))
