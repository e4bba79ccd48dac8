'''HBM buffer pool keyed by jaxpr variable.

Same role and the same liveness algorithm as the reference's BufferPool (vkjax/buffers.py:90-204):
every variable gets a `Buffer` (dtype, shape, list of op indices that touch it); buffers that
are views of each other share one tensor placeholder; after the whole program has been
analysed, `create_tensors` assigns device allocations largest-first and lets a buffer reuse
an allocation whose access interval does not overlap its own. Differences: allocations are
HBM buffers obtained through the C-ABI runtime (no padding to a workgroup multiple, kernels
guard their bounds), and constants are uploaded once at build time.

All device data is 32 bits wide, as in the reference (vkjax/buffers.py:54-77): bool is stored
as uint32 0/1, int64 is narrowed to int32, float64 to float32.
'''
import typing as tp

import numpy as np

from .minijax import core


class StorageCell:
    '''The device allocation that one or several buffers (views of one another) stand on. It is filled in when
    storage is assigned, after the whole program is known, so all views see the allocation at once.'''
    __slots__ = ('t', 'elided')

    def __init__(self, t=None):
        self.t = t
        #set when fusion keeps the value in registers: the variable never gets storage
        self.elided = False


TensorPlaceholder = StorageCell          #the reference's name for it (vkjax/buffers.py:13-15)


class PlannedTensor:
    '''Stand-in allocation used when a program is only planned (no device): it records the
    size an HBM buffer would have. It holds no data and cannot be executed on.'''
    def __init__(self, nbytes: int, initial_value: tp.Optional[np.ndarray] = None):
        self.nbytes        = int(nbytes)
        self.initial_value = initial_value
        self.handle        = None


class PlanOnlyDevice:
    '''Takes the place of hip.Device when only the plan (ops, liveness, launch parameters) is
    wanted, e.g. to inspect a program on a machine without a GPU. Running is impossible.'''
    index = None

    def tensor(self, array: np.ndarray) -> PlannedTensor:
        return PlannedTensor(max(array.nbytes, 4), array)

    def alloc(self, nbytes: int, packed: bool = False) -> PlannedTensor:
        return PlannedTensor(nbytes)

    def sequence(self, profiling=False):
        raise RuntimeError('this interpreter was built with plan_only=True and has no device to run on')

    def get_device_properties(self):
        return dict(device_name='plan-only', arch='gfx950', max_work_group_invocations=1024,
                    max_work_group_size=(1024, 1024, 64), compute_units=256, wavefront_size=64)


class Buffer:
    '''dtype, shape and liveness (`accesses`: positions of the ops that touch it) of one array in HBM. `tensor` is the
    device allocation of the storage cell the buffer stands on; views made by `view` share cell and access list, as in
    the reference (vkjax/buffers.py:17-51), where the sharing is done by intercepting attribute access.'''
    __slots__ = ('_cell', 'dtype', 'shape', 'accesses', 'constant_value')

    def __init__(self, tensor, dtype: np.dtype, shape: tp.Tuple[int, ...]):
        self._cell = tensor if isinstance(tensor, StorageCell) else StorageCell(tensor)
        self.dtype = np.dtype(dtype)
        self.shape = tuple(int(s) for s in shape)
        self.accesses: tp.List[float] = []
        self.constant_value = None

    @property
    def tensor(self):
        return self._cell.t

    @tensor.setter
    def tensor(self, allocation):
        self._cell.t = allocation

    @property
    def _placeholder(self) -> StorageCell:
        return self._cell

    @property
    def size(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64))

    def nbytes(self) -> int:
        if self.dtype.type not in {np.bool_, np.float32, np.int32, np.uint32}:
            raise NotImplementedError(self.dtype)
        #booleans are 32-bit on the device too
        return self.size * 4

    def view(self, new_dtype, new_shape) -> 'Buffer':
        '''Another dtype/shape on the same storage; shares the access list (reference: vkjax/buffers.py:48-51).'''
        other = Buffer(self._cell, new_dtype, new_shape)
        other.accesses = self.accesses
        return other

    def same_storage(self, other: 'Buffer') -> bool:
        return self._cell is other._cell

    def numpy(self) -> np.ndarray:
        '''Blocking read of the device contents as an array of this buffer's dtype and shape.'''
        t = self.tensor
        if self._placeholder.elided:
            return None
        if t is None or getattr(t, 'handle', None) is None:
            raise RuntimeError('buffer has no device storage')
        raw = t.download(self.nbytes()) if self.size else np.zeros(0, np.uint32)
        return view_or_convert_from_32bit(raw, self.dtype)[:self.size].reshape(self.shape)


def view_or_convert_from_32bit(x: np.ndarray, dtype) -> np.ndarray:
    dtype = np.dtype(dtype)
    if dtype == np.bool_:
        return x.view(np.uint32) != 0
    return x.view(dtype)


def to_device_words(x, dtype=None) -> np.ndarray:
    '''Flat uint32 image of an array as it is stored on the device
    (the counterpart of view_as_float32, reference: vkjax/buffers.py:68-77).'''
    x = np.asarray(x) if dtype is None else np.asarray(x, dtype=dtype)
    if x.dtype.type not in {np.bool_, np.float32, np.int32, np.int64, np.uint32, np.uint64, np.float64}:
        raise NotImplementedError(f'{x.dtype} data types currently not supported')
    if x.dtype == np.bool_:
        x = x.astype(np.uint32)
    elif x.dtype == np.float64:
        x = x.astype(np.float32)
    elif x.dtype == np.int64:
        x = x.astype(np.int32)
    elif x.dtype == np.uint64:
        x = x.astype(np.uint32)
    return np.ascontiguousarray(x).reshape(-1).view(np.uint32)


def hashable(var):
    '''Key of a variable in the pool; jax literals are unhashable but carry `.hash` (reference: vkjax/buffers.py:80-87).'''
    if core.is_literal(var):
        h = getattr(var, 'hash', None)
        if h is None:
            #literal classes without a value hash: equal scalars of one dtype still share one buffer
            h = hash(np.asarray(var.val).tobytes())
        #jax hashes the bare value, and hash(1) == hash(1.0): the dtype keeps an integer and a float literal apart
        return ('literal', str(var.aval.dtype), h)
    return var


def _is_unit(aval) -> bool:
    return type(aval).__name__ == 'AbstractUnit'


class BufferPool:
    def __init__(self, device, workgroup_size: int = 1, reuse_tensors: bool = True):
        self.device         = device
        self.workgroup_size = workgroup_size      #kept for interface parity; nothing is padded
        self.buffers: tp.Dict[tp.Any, tp.Optional[Buffer]] = dict()
        self.op_counter     = 0
        self.reuse_tensors  = reuse_tensors

    def get_buffer(self, var, increment_op_counter: bool = False) -> tp.Optional[Buffer]:
        varhash = hashable(var)
        if varhash not in self.buffers:
            if _is_unit(var.aval):
                return None
            shape, dtype = core.physical(var.aval)
            self.buffers[varhash] = Buffer(None, dtype, shape)
        b = self.buffers[varhash]
        if b is None:
            return None
        b.accesses.append(self.op_counter)
        if core.is_literal(var) and b.tensor is None:
            self.mark_buffer_as_constant(b, var, var.val)
        if increment_op_counter:
            self.op_counter += 1
        return b

    def new_temporary(self, dtype, shape) -> Buffer:
        '''A buffer that belongs to no jaxpr variable (scratch between two launches of one primitive).'''
        b = Buffer(None, dtype, shape)
        self.buffers[('tmp', len(self.buffers))] = b
        b.accesses.append(self.op_counter)
        return b

    def mark_buffer_as_constant(self, b: Buffer, var, value):
        if b.tensor is None:
            b.tensor = self._create_tensor(var, initial_value=value)
        if value is not None:
            b.constant_value = value          #known when the program is built: a lowering may look at it
        #the storage of a constant must never be handed to anything else
        b.accesses += [0, np.inf]

    def scalar_constant(self, value, dtype) -> Buffer:
        '''A one-element constant that belongs to no jaxpr variable; equal ones share storage.'''
        dtype = np.dtype(dtype)
        key   = ('scalar', str(dtype), np.asarray(value, dtype).tobytes())
        if key not in self.buffers:
            b = Buffer(self.device.tensor(to_device_words(np.asarray(value, dtype).reshape(1))), dtype, ())
            b.accesses += [0, np.inf]
            self.buffers[key] = b
        return self.buffers[key]

    def zeroed_scratch(self, n_words: int, use: str = '') -> Buffer:
        '''n_words of uint32 that hold zeros when the program is built and are never handed to anything else.
        Launches that use them leave them zero again, so launches of one size and use share one array.'''
        key = ('zeroed', int(n_words), use)
        if key not in self.buffers:
            b = Buffer(self.device.tensor(np.zeros(n_words, np.uint32)), np.dtype('uint32'), (n_words,))
            b.accesses += [0, np.inf]
            self.buffers[key] = b
        return self.buffers[key]

    def set_buffer(self, var, b: tp.Optional[Buffer]):
        if b is None:
            return
        self.buffers[hashable(var)] = b
        b.accesses.append(self.op_counter)

    def create_tensors(self):
        tensor_access_map: tp.Dict[tp.Any, tp.List[float]] = dict()
        keys    = list(self.buffers.keys())
        buffers = [self.buffers[k] for k in keys]
        order   = sorted((i for i, b in enumerate(buffers) if b is not None), key=lambda i: buffers[i].nbytes())
        #largest first: they are the easiest to reuse
        for i in reversed(order):
            b, v = buffers[i], keys[i]
            if b.tensor is not None or b._placeholder.elided:
                #constants, I/O, a view whose sibling already got storage, or a fused-away intermediate
                continue
            t = self._search_for_free_tensor(b, tensor_access_map) if self.reuse_tensors else None
            if t is None:
                t = self.device.alloc(max(b.nbytes(), 4))
                tensor_access_map[t] = list(b.accesses)
            b.tensor = t

    def _search_for_free_tensor(self, b: Buffer, tensor_access_map):
        lo, hi = min(b.accesses), max(b.accesses)
        for t, t_accesses in tensor_access_map.items():
            if t.nbytes < b.nbytes():
                continue
            if hi < min(t_accesses) or lo > max(t_accesses):
                tensor_access_map[t] = t_accesses + list(b.accesses)
                return t
        return None

    def _create_tensor(self, var, initial_value=None):
        shape, dtype = core.physical(var.aval)
        if core.is_literal(var):
            initial_value = var.val
        if initial_value is None:
            #an argument or result of the program: the small ones among them lie side by side in HBM, so that a call
            #sends a run of them with one transfer
            return self.device.alloc(max(int(np.prod(shape, dtype=np.int64)) * 4, 4), packed=True)
        initial_value = np.asarray(initial_value)
        assert initial_value.size == int(np.prod(shape, dtype=np.int64)), (initial_value.shape, shape)
        return self.device.tensor(to_device_words(initial_value, dtype))

    def unique_tensors(self) -> set:
        return set(b.tensor for b in self.buffers.values() if b is not None)

    def total_device_bytes(self) -> int:
        return sum(t.nbytes for t in self.unique_tensors() if t is not None)
