'''ctypes binding of the C-ABI device runtime (include/vkjax_hip.h, built to
vkjax_amd/lib/libvkjax_hip.so) and a thin object layer on top: Device, DeviceBuffer, Sequence.

This is what takes the place of `kp.Manager` / `kp.Tensor` / `kp.Sequence` in the reference
(vkjax/kompute_jaxpr_interpreter.py:19-63, vkjax/buffers.py:189-204). There is no fallback:
if the library or the code objects are missing, or no GPU is present, constructing a Device
raises.
'''
import ctypes as C
import os
import threading
import typing as tp

import numpy as np

_PKG    = os.path.dirname(os.path.abspath(__file__))
LIBDIR  = os.path.join(_PKG, 'lib')
LIBPATH = os.path.join(LIBDIR, 'libvkjax_hip.so')

KERNEL_MODULES = ('elementwise', 'conv_gemm', 'wgrad_gemm', 'reduce', 'index', 'threefry')

EVAL_SKIP_UPLOADS   = 1
EVAL_SKIP_DOWNLOADS = 2
EVAL_NULL_IS_RESIDENT = 4
STATIC_LANDING_BYTES  = 64 << 20       #VKJ_STATIC_LANDING_BYTES
NO_POINTER_SLOT       = 0xFFFFFFFF     #VKJ_NO_POINTER_SLOT


class Props(C.Structure):
    _fields_ = [('name', C.c_char * 256), ('arch', C.c_char * 64),
                ('compute_units', C.c_int32), ('wavefront_size', C.c_int32),
                ('max_threads_per_block', C.c_int32), ('max_block_dim_x', C.c_int32),
                ('lds_bytes_per_block', C.c_int32), ('clock_khz', C.c_int32),
                ('memory_clock_khz', C.c_int32), ('memory_bus_bits', C.c_int32),
                ('hbm_bytes', C.c_uint64)]


_H = C.c_uint64
_PROTOTYPES = {
    'vkj_last_error':          (C.c_char_p, []),
    'vkj_device_count':        (C.c_int, [C.POINTER(C.c_int)]),
    'vkj_ctx_create':          (C.c_int, [C.c_int, C.POINTER(_H)]),
    'vkj_ctx_destroy':         (C.c_int, [_H]),
    'vkj_device_props':        (C.c_int, [_H, C.POINTER(Props)]),
    'vkj_sync':                (C.c_int, [_H]),
    'vkj_module_load':         (C.c_int, [_H, C.c_void_p, C.c_size_t, C.POINTER(_H)]),
    'vkj_module_unload':       (C.c_int, [_H, _H]),
    'vkj_module_get_function': (C.c_int, [_H, _H, C.c_char_p, C.POINTER(_H)]),
    'vkj_buf_alloc':           (C.c_int, [_H, C.c_size_t, C.POINTER(_H)]),
    'vkj_buf_alloc_packed':    (C.c_int, [_H, C.c_size_t, C.POINTER(_H)]),
    'vkj_buf_free':            (C.c_int, [_H, _H]),
    'vkj_buf_size':            (C.c_int, [_H, _H, C.POINTER(C.c_size_t)]),
    'vkj_buf_device_ptr':      (C.c_int, [_H, _H, C.POINTER(C.c_uint64)]),
    'vkj_buf_memset':          (C.c_int, [_H, _H, C.c_size_t, C.c_int, C.c_size_t]),
    'vkj_buf_upload':          (C.c_int, [_H, _H, C.c_size_t, C.c_void_p, C.c_size_t]),
    'vkj_buf_download':        (C.c_int, [_H, _H, C.c_size_t, C.c_void_p, C.c_size_t]),
    'vkj_seq_create':          (C.c_int, [_H, C.c_int, C.POINTER(_H)]),
    'vkj_seq_destroy':         (C.c_int, [_H]),
    'vkj_seq_record_upload':   (C.c_int, [_H, _H, C.c_size_t, C.c_int, C.c_size_t]),
    'vkj_seq_set_launch_lane': (C.c_int, [_H, C.c_int, C.c_int, C.c_int]),
    'vkj_seq_record_early_part': (C.c_int, [_H, _H, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.c_uint32,
                                            C.c_void_p, C.c_size_t, C.POINTER(_H), C.POINTER(C.c_uint32),
                                            C.POINTER(C.c_uint64), C.c_int, C.c_int, C.c_size_t]),
    'vkj_seq_record_launch':   (C.c_int, [_H, _H, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.c_uint32,
                                          C.c_void_p, C.c_size_t, C.POINTER(_H), C.POINTER(C.c_uint32),
                                          C.POINTER(C.c_uint64), C.c_int]),
    'vkj_seq_record_download': (C.c_int, [_H, _H, C.c_size_t, C.c_int, C.c_size_t]),
    'vkj_seq_num_steps':       (C.c_int, [_H, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    'vkj_seq_eval':            (C.c_int, [_H, C.POINTER(C.c_void_p), C.c_int, C.c_uint32]),
    'vkj_seq_eval_next':       (C.c_int, [_H, C.POINTER(C.c_void_p), C.c_int, C.c_uint32, C.POINTER(C.c_void_p)]),
    'vkj_seq_eval_next_static': (C.c_int, [_H, C.POINTER(C.c_void_p), C.c_int, C.c_uint32, C.POINTER(C.c_void_p)]),
    'vkj_seq_replay':          (C.c_int, [_H, C.c_int, C.POINTER(C.c_float)]),
    'vkj_seq_use_graph':       (C.c_int, [_H, C.c_int]),
    'vkj_seq_timestamps':      (C.c_int, [_H, C.POINTER(C.c_float), C.c_int, C.POINTER(C.c_int)]),
}

_lib      = None
_lib_lock = threading.Lock()


def exported_symbols() -> tp.Tuple[str, ...]:
    return tuple(_PROTOTYPES)


def load_library() -> C.CDLL:
    '''Load libvkjax_hip.so and set the prototypes. Raises if it has not been built.'''
    global _lib
    with _lib_lock:
        if _lib is None:
            if not os.path.exists(LIBPATH):
                raise RuntimeError(f'{LIBPATH} is missing: build it with `python -m vkjax_amd.csrc.build`')
            lib = C.CDLL(LIBPATH)
            for name, (restype, argtypes) in _PROTOTYPES.items():
                fn = getattr(lib, name)          #AttributeError if the library does not export it
                fn.restype, fn.argtypes = restype, argtypes
            _lib = lib
    return _lib


class HipError(RuntimeError):
    pass


def _check(status: int, what: str):
    if status != 0:
        msg = load_library().vkj_last_error().decode('utf8', 'replace')
        raise HipError(f'{what} failed with status {status}: {msg}')


def device_count() -> int:
    n = C.c_int(0)
    status = load_library().vkj_device_count(C.byref(n))
    return n.value if status == 0 else 0


class DeviceBuffer:
    '''One HBM allocation (the counterpart of a kp.Tensor). Hashable by identity.'''
    def __init__(self, device: 'Device', nbytes: int, packed: bool = False):
        self.device = device
        self.nbytes = int(nbytes)
        h = _H(0)
        #(packed: a small array that is uploaded together with others, placed next to them: vkj_buf_alloc_packed)
        name = 'vkj_buf_alloc_packed' if packed else 'vkj_buf_alloc'
        _check(getattr(device.lib, name)(device.ctx, self.nbytes, C.byref(h)), f'{name}({nbytes})')
        self.handle = h.value

    def upload(self, array: np.ndarray, offset: int = 0):
        array = np.ascontiguousarray(array)
        _check(self.device.lib.vkj_buf_upload(self.device.ctx, self.handle, offset,
                                               array.ctypes.data_as(C.c_void_p), array.nbytes), 'vkj_buf_upload')

    def download(self, nbytes: tp.Optional[int] = None, offset: int = 0) -> np.ndarray:
        nbytes = self.nbytes - offset if nbytes is None else nbytes
        out = np.empty(nbytes // 4, dtype=np.uint32)
        _check(self.device.lib.vkj_buf_download(self.device.ctx, self.handle, offset,
                                                 out.ctypes.data_as(C.c_void_p), nbytes), 'vkj_buf_download')
        return out

    def memset(self, byte_value: int = 0):
        _check(self.device.lib.vkj_buf_memset(self.device.ctx, self.handle, 0, byte_value, self.nbytes), 'vkj_buf_memset')

    def device_ptr(self) -> int:
        p = C.c_uint64(0)
        _check(self.device.lib.vkj_buf_device_ptr(self.device.ctx, self.handle, C.byref(p)), 'vkj_buf_device_ptr')
        return p.value

    def free(self):
        if self.handle:
            _check(self.device.lib.vkj_buf_free(self.device.ctx, self.handle), 'vkj_buf_free')
            self.handle = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Device:
    '''A device context with the kernel code objects loaded (the counterpart of kp.Manager).'''
    _instances: tp.Dict[int, 'Device'] = {}
    _lock = threading.Lock()

    @classmethod
    def get(cls, index: tp.Optional[int] = None) -> 'Device':
        '''One shared context per device index. The index defaults to $VKJAX_DEVICE
        (reference: vkjax/kompute_jaxpr_interpreter.py:19).'''
        if index is None:
            index = int(os.environ.get('VKJAX_DEVICE', 0))
        with cls._lock:
            if index not in cls._instances:
                cls._instances[index] = Device(index)
            return cls._instances[index]

    def __init__(self, index: int = 0):
        self.lib   = load_library()
        self.index = index
        h = _H(0)
        _check(self.lib.vkj_ctx_create(index, C.byref(h)), f'vkj_ctx_create({index})')
        self.ctx = h.value
        self._functions: tp.Dict[str, int] = {}
        self._modules:   tp.Dict[str, int] = {}
        self._images = []
        for name in KERNEL_MODULES:
            path = os.path.join(LIBDIR, f'{name}.hsaco')
            if not os.path.exists(path):
                raise RuntimeError(f'{path} is missing: build it with `python -m vkjax_amd.csrc.build`')
            image = open(path, 'rb').read()
            buf   = C.create_string_buffer(image, len(image))
            m = _H(0)
            _check(self.lib.vkj_module_load(self.ctx, C.cast(buf, C.c_void_p), len(image), C.byref(m)),
                   f'vkj_module_load({name})')
            self._modules[name] = m.value
            self._images.append(buf)
        self._props = None

    def close(self):
        '''Unloads the code objects and destroys the context. Only for contexts made directly (the lanes of
        Function.stream(in_flight=...)): everything allocated or recorded on the context holds a reference to this
        object, so it is collected - and closed - after the last of them has gone. The shared contexts of get() live as
        long as the process.'''
        if getattr(self, 'ctx', 0):
            for module in self._modules.values():
                self.lib.vkj_module_unload(self.ctx, module)
            self._modules.clear()
            self._functions.clear()
            self.lib.vkj_ctx_destroy(self.ctx)
            self.ctx = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def props(self) -> Props:
        if self._props is None:
            p = Props()
            _check(self.lib.vkj_device_props(self.ctx, C.byref(p)), 'vkj_device_props')
            self._props = p
        return self._props

    def get_device_properties(self) -> dict:
        '''Same keys the reference reads from kp (vkjax/kompute_jaxpr_interpreter.py:100-102) plus the HIP ones.'''
        p = self.props
        return dict(device_name=p.name.decode(), arch=p.arch.decode(),
                    max_work_group_invocations=p.max_threads_per_block,
                    max_work_group_size=(p.max_block_dim_x, p.max_block_dim_x, 64),
                    compute_units=p.compute_units, wavefront_size=p.wavefront_size,
                    lds_bytes_per_block=p.lds_bytes_per_block, clock_khz=p.clock_khz,
                    memory_clock_khz=p.memory_clock_khz, memory_bus_bits=p.memory_bus_bits, hbm_bytes=p.hbm_bytes)

    def function(self, kernel_name: str) -> int:
        if kernel_name not in self._functions:
            last = None
            for mod in self._modules.values():
                f = _H(0)
                status = self.lib.vkj_module_get_function(self.ctx, mod, kernel_name.encode(), C.byref(f))
                if status == 0:
                    self._functions[kernel_name] = f.value
                    break
                last = status
            else:
                raise NotImplementedError(f'no kernel named {kernel_name} in the loaded code objects (status {last})')
        return self._functions[kernel_name]

    def alloc(self, nbytes: int, packed: bool = False) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes, packed)

    def tensor(self, array: np.ndarray) -> DeviceBuffer:
        '''Allocate and upload (blocking), like mgr.tensor + OpTensorSyncDevice (reference: vkjax/buffers.py:202-203).'''
        array = np.ascontiguousarray(array)
        buf = self.alloc(max(array.nbytes, 4))
        if array.nbytes:
            buf.upload(array)
        return buf

    def sync(self):
        _check(self.lib.vkj_sync(self.ctx), 'vkj_sync')

    def sequence(self, profiling: bool = False) -> 'Sequence':
        return Sequence(self, profiling)


class Sequence:
    '''A recorded list of uploads, launches and downloads replayed by one native call
    (the counterpart of kp.Sequence; reference: vkjax/kompute_jaxpr_interpreter.py:48-63,77).'''
    def __init__(self, device: Device, profiling: bool = False):
        self.device, self.profiling = device, profiling
        h = _H(0)
        _check(device.lib.vkj_seq_create(device.ctx, int(profiling), C.byref(h)), 'vkj_seq_create')
        self.handle  = h.value
        self.n_slots = 0
        self.n_launches = 0

    def _slot(self) -> int:
        self.n_slots += 1
        return self.n_slots - 1

    def record_upload(self, buf: DeviceBuffer, nbytes: int, offset: int = 0) -> int:
        slot = self._slot()
        _check(self.device.lib.vkj_seq_record_upload(self.handle, buf.handle, offset, slot, nbytes), 'vkj_seq_record_upload')
        return slot

    def record_download(self, buf: DeviceBuffer, nbytes: int, offset: int = 0) -> int:
        slot = self._slot()
        _check(self.device.lib.vkj_seq_record_download(self.handle, buf.handle, offset, slot, nbytes), 'vkj_seq_record_download')
        return slot

    def record_launch(self, kernel_name: str, grid, block, buffers: tp.Sequence[tp.Tuple[tp.Optional[DeviceBuffer], int]],
                      params: bytes, lds_bytes: int = 0, early_part_of: tp.Optional[tp.Tuple[int, int]] = None,
                      reached_through_tables: tp.Sequence[DeviceBuffer] = ()):
        '''`buffers` are (DeviceBuffer or None, byte offset) in kernel-argument order; they occupy
        the first 8*len(buffers) bytes of the argument block, `params` follows. `early_part_of` = (upload slot, bytes
        needed): the launch is not a step of the sequence but one part of the alternative form of its first launch
        (vkj_seq_record_early_part), issued while the rest of that slot's argument is still being uploaded.
        `reached_through_tables`: buffers the kernel reads or writes through addresses it finds in device memory (a batch
        launch's table) instead of its argument block; the runtime has to know them, for the order in which it sends
        arguments and issues launches and to keep them allocated.'''
        fn      = self.device.function(kernel_name)
        nptr    = len(buffers)
        kernarg = bytes(8 * nptr) + params
        present = [(8 * i, b, off) for i, (b, off) in enumerate(buffers) if b is not None]
        present += [(NO_POINTER_SLOT, b, 0) for b in reached_through_tables]
        n       = len(present)
        handles = (_H * max(n, 1))(*[b.handle for _, b, _ in present])
        argoffs = (C.c_uint32 * max(n, 1))(*[slot for slot, _, _ in present])
        byteoff = (C.c_uint64 * max(n, 1))(*[off for _, _, off in present])
        g = (C.c_uint32 * 3)(*[int(x) for x in grid])
        b = (C.c_uint32 * 3)(*[int(x) for x in block])
        if early_part_of is not None:
            slot, needed = early_part_of
            _check(self.device.lib.vkj_seq_record_early_part(self.handle, fn, g, b, lds_bytes, kernarg, len(kernarg),
                                                              handles, argoffs, byteoff, n, int(slot), int(needed)),
                   f'vkj_seq_record_early_part({kernel_name})')
            return
        _check(self.device.lib.vkj_seq_record_launch(self.handle, fn, g, b, lds_bytes, kernarg, len(kernarg),
                                                      handles, argoffs, byteoff, n), f'vkj_seq_record_launch({kernel_name})')
        self.n_launches += 1

    def set_launch_lane(self, launch: int, lane: int, wait_for_other_lane: bool):
        '''Launch number `launch` goes to lane 0 (the stream) or 1 (the side stream); with `wait_for_other_lane` its
        lane first waits for everything recorded before it on the other one.'''
        _check(self.device.lib.vkj_seq_set_launch_lane(self.handle, launch, lane, int(bool(wait_for_other_lane))), 'vkj_seq_set_launch_lane')

    def eval(self, host_arrays: tp.Sequence[tp.Optional[np.ndarray]], flags: int = 0,
             next_host_arrays: tp.Optional[tp.Sequence[tp.Optional[np.ndarray]]] = None, static_landing: bool = False):
        '''`next_host_arrays`: the arguments of the following evaluation (None per slot that stays as
        it is); they are uploaded while the device runs this one, and the following call passes None
        for them with EVAL_NULL_IS_RESIDENT. `static_landing`: through vkj_seq_eval_next_static, which
        allocates nothing and takes at most STATIC_LANDING_BYTES of following arguments.'''
        def pointers(arrays):
            ptrs = (C.c_void_p * max(len(arrays), 1))()
            for i, a in enumerate(arrays):
                ptrs[i] = a.ctypes.data if a is not None else None
            return ptrs
        ptrs = pointers(host_arrays)
        if next_host_arrays is None and not static_landing:
            _check(self.device.lib.vkj_seq_eval(self.handle, ptrs, len(host_arrays), flags), 'vkj_seq_eval')
            return
        if next_host_arrays is None:
            next_host_arrays = [None] * len(host_arrays)
        if len(next_host_arrays) != len(host_arrays):
            raise ValueError('next_host_arrays must have one entry per slot')
        name = 'vkj_seq_eval_next_static' if static_landing else 'vkj_seq_eval_next'
        _check(getattr(self.device.lib, name)(self.handle, ptrs, len(host_arrays), flags, pointers(next_host_arrays)), name)

    def replay(self, iters: int = 1) -> float:
        '''Launches only; returns elapsed device milliseconds for all iterations.'''
        ms = C.c_float(0)
        _check(self.device.lib.vkj_seq_replay(self.handle, iters, C.byref(ms)), 'vkj_seq_replay')
        return ms.value

    def use_graph(self, enable: bool = True):
        '''Issue the recorded launches as one captured HIP graph from the next eval / replay on.'''
        _check(self.device.lib.vkj_seq_use_graph(self.handle, int(bool(enable))), 'vkj_seq_use_graph')

    def get_timestamps(self) -> np.ndarray:
        n = C.c_int(0)
        _check(self.device.lib.vkj_seq_timestamps(self.handle, None, 0, C.byref(n)), 'vkj_seq_timestamps')
        out = np.zeros(n.value, dtype=np.float32)
        if n.value:
            _check(self.device.lib.vkj_seq_timestamps(self.handle, out.ctypes.data_as(C.POINTER(C.c_float)), n.value, C.byref(n)),
                   'vkj_seq_timestamps')
        return out

    def destroy(self):
        if self.handle:
            _check(self.device.lib.vkj_seq_destroy(self.handle), 'vkj_seq_destroy')
            self.handle = 0

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
