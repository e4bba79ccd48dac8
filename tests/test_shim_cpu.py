'''The C-ABI runtime's handle, lifetime and transfer logic on the CPU: vkjax_amd/csrc/shim.cpp is
compiled against a host-only stand-in of the HIP calls it makes (tests/fake_hip), so contexts,
modules, buffers and sequences can be created without a GPU. What is checked: objects that live
sequences refer to cannot be pulled from under them, stale handles are rejected, error paths
release what they had created, and an evaluation moves the bytes it should.'''
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from vkjax_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EINVAL, ESTATE = -1, -3


@pytest.fixture(scope='module')
def lib(tmp_path_factory):
    out  = str(tmp_path_factory.mktemp('fake_shim') / 'libvkjax_fake.so')
    csrc = os.path.join(ROOT, 'vkjax_amd', 'csrc')
    fake = os.path.join(ROOT, 'tests', 'fake_hip')
    subprocess.run(['g++', '-O1', '-g', '-fPIC', '-shared', '-pthread', '-std=c++17', f'-I{fake}', f'-I{csrc}',
                    f'-I{os.path.join(ROOT, "include")}', os.path.join(csrc, 'shim.cpp'), os.path.join(fake, 'fake_glue.cpp'), '-o', out],
                   check=True, capture_output=True, text=True)
    lib = C.CDLL(out)
    for name, (restype, argtypes) in hip._PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = restype, argtypes
    lib.fake_hip_live_objects.restype = C.c_long
    lib.fake_hip_launches.restype = C.c_long
    lib.fake_hip_creations.restype = C.c_long
    lib.fake_hip_copies.restype = C.c_long
    lib.fake_hip_copies_at_launch.restype = C.c_long
    lib.fake_hip_copies_at_launch.argtypes = [C.c_long]
    lib.fake_hip_on_synchronize.argtypes = [C.c_void_p]
    lib.fake_hip_fail_after.argtypes = [C.c_long]
    return lib


def H():
    return C.c_uint64(0)


class World:
    '''A context with one module (two kernels) in the stand-in runtime.'''
    def __init__(self, lib):
        self.lib = lib
        self.ctx, self.mod, self.fn = H(), H(), H()
        assert lib.vkj_ctx_create(0, C.byref(self.ctx)) == 0
        image = C.create_string_buffer(b'fake_add_one\nfake_nothing\n')
        assert lib.vkj_module_load(self.ctx, image, len(image), C.byref(self.mod)) == 0
        assert lib.vkj_module_get_function(self.ctx, self.mod, b'fake_add_one', C.byref(self.fn)) == 0

    def buf(self, nbytes):
        b = H()
        assert self.lib.vkj_buf_alloc(self.ctx, nbytes, C.byref(b)) == 0
        return b

    def add_one_sequence(self, n):
        '''upload slot 0 -> src; dst = src + 1; dst -> download slot 1'''
        lib = self.lib
        src, dst, seq = self.buf(4 * n), self.buf(4 * n), H()
        assert lib.vkj_seq_create(self.ctx, 0, C.byref(seq)) == 0
        assert lib.vkj_seq_record_upload(seq, src, 0, 0, 4 * n) == 0
        assert self.record_add_one(seq, dst, src, n) == 0
        assert lib.vkj_seq_record_download(seq, dst, 0, 1, 4 * n) == 0
        return seq, src, dst

    def record_add_one(self, seq, dst, src, n, fn=None):
        kernarg = bytes(16) + np.uint32(n).tobytes() + bytes(4)
        grid = (C.c_uint32 * 3)(1, 1, 1)
        bufs = (C.c_uint64 * 2)(dst.value, src.value)
        offs = (C.c_uint32 * 2)(0, 8)
        return self.lib.vkj_seq_record_launch(seq, fn or self.fn, grid, grid, 0, kernarg, len(kernarg), bufs, offs, None, 2)

    def eval(self, seq, x, nxt=None, flags=0, n=None):
        y = np.zeros(n or (x.size if x is not None else nxt.size), np.uint32)
        ptrs = (C.c_void_p * 2)(x.ctypes.data if x is not None else None, y.ctypes.data)
        if nxt is None:
            assert self.lib.vkj_seq_eval(seq, ptrs, 2, flags) == 0, self.lib.vkj_last_error()
        else:
            nptrs = (C.c_void_p * 2)(nxt.ctypes.data, None)
            assert self.lib.vkj_seq_eval_next(seq, ptrs, 2, flags, nptrs) == 0, self.lib.vkj_last_error()
        return y

    def close(self):
        assert self.lib.vkj_module_unload(self.ctx, self.mod) == 0
        assert self.lib.vkj_ctx_destroy(self.ctx) == 0


def test_eval_moves_the_bytes_and_everything_is_released(lib):
    before = lib.fake_hip_live_objects()
    w = World(lib)
    seq, src, dst = w.add_one_sequence(1000)
    x = np.arange(1000, dtype=np.uint32)
    assert np.array_equal(w.eval(seq, x), x + 1)
    #the following evaluation's arguments ride along; the next call passes NULL for the slot
    x2 = x * 3
    assert np.array_equal(w.eval(seq, x, nxt=x2), x + 1)
    assert np.array_equal(w.eval(seq, None, nxt=x, flags=hip.EVAL_NULL_IS_RESIDENT), x2 + 1)
    assert np.array_equal(w.eval(seq, None, flags=hip.EVAL_NULL_IS_RESIDENT, n=1000), x + 1)
    assert lib.vkj_seq_destroy(seq) == 0
    assert lib.vkj_buf_free(w.ctx, src) == 0 and lib.vkj_buf_free(w.ctx, dst) == 0
    w.close()
    assert lib.fake_hip_live_objects() == before


def test_many_arguments_are_staged_together(lib):
    '''From 8 MB of arguments on, all uploads of an evaluation are staged as one stream of 4 MB chunks by helper
    threads: many arrays of different sizes (some smaller than a chunk, one of several chunks, one empty slot
    passed as resident) have to arrive intact, in their own buffers.'''
    w = World(lib)
    sizes = [3, 1 << 20, 70001, (5 << 20) + 13, 1 << 18, 17]            #elements; 26 MB together
    seq = H()
    assert lib.vkj_seq_create(w.ctx, 0, C.byref(seq)) == 0
    bufs = [w.buf(4 * n) for n in sizes]
    for slot, (b, n) in enumerate(zip(bufs, sizes)):
        assert lib.vkj_seq_record_upload(seq, b, 0, slot, 4 * n) == 0
    for slot, (b, n) in enumerate(zip(bufs, sizes)):
        assert lib.vkj_seq_record_download(seq, b, 0, len(sizes) + slot, 4 * n) == 0
    rng = np.random.default_rng(3)
    for resident in (None, 2):
        xs = [rng.integers(0, 1 << 32, size=n, dtype=np.uint64).astype(np.uint32) for n in sizes]
        ys = [np.zeros(n, np.uint32) for n in sizes]
        ptrs = (C.c_void_p * (2 * len(sizes)))(*[None if k == resident else x.ctypes.data for k, x in enumerate(xs)], *[y.ctypes.data for y in ys])
        assert lib.vkj_seq_eval(seq, ptrs, 2 * len(sizes), hip.EVAL_NULL_IS_RESIDENT) == 0, lib.vkj_last_error()
        for k, (x, y) in enumerate(zip(xs, ys)):
            if k == resident:
                assert np.array_equal(y, previous[k]), k            #untouched: still what the first evaluation uploaded
            else:
                assert np.array_equal(y, x), k
        previous = xs
    assert lib.vkj_seq_destroy(seq) == 0
    w.close()


def test_module_unload_is_refused_while_a_sequence_uses_it(lib):
    w = World(lib)
    seq, src, dst = w.add_one_sequence(8)
    assert lib.vkj_module_unload(w.ctx, w.mod) == ESTATE
    assert b'live sequences' in lib.vkj_last_error()
    x = np.arange(8, dtype=np.uint32)
    assert np.array_equal(w.eval(seq, x), x + 1)                 #still whole
    assert lib.vkj_seq_destroy(seq) == 0
    assert lib.vkj_module_unload(w.ctx, w.mod) == 0
    #the module's functions went with it: recording one is a bad handle, not a use after free
    seq2 = H()
    assert lib.vkj_seq_create(w.ctx, 0, C.byref(seq2)) == 0
    assert w.record_add_one(seq2, dst, src, 8) == EINVAL
    f = H()
    assert lib.vkj_module_get_function(w.ctx, w.mod, b'fake_add_one', C.byref(f)) == EINVAL
    assert lib.vkj_seq_destroy(seq2) == 0
    for b in (src, dst):
        assert lib.vkj_buf_free(w.ctx, b) == 0
    assert lib.vkj_ctx_destroy(w.ctx) == 0


def test_buffer_freed_under_a_live_sequence_outlives_it(lib):
    before = lib.fake_hip_live_objects()
    w = World(lib)
    seq, src, dst = w.add_one_sequence(64)
    base = lib.fake_hip_live_objects()
    assert lib.vkj_buf_free(w.ctx, src) == 0                     #handle retired, memory kept
    assert lib.fake_hip_live_objects() == base
    n = C.c_size_t(0)
    assert lib.vkj_buf_size(w.ctx, src, C.byref(n)) == EINVAL    #stale handle
    assert lib.vkj_buf_free(w.ctx, src) == EINVAL
    x = np.arange(64, dtype=np.uint32)
    assert np.array_equal(w.eval(seq, x), x + 1)                 #the sequence still owns valid memory
    assert lib.vkj_seq_destroy(seq) == 0                         #... and releases it
    assert lib.fake_hip_live_objects() == base - 1 - 2           #src, and the two pinned staging buffers
    assert lib.vkj_buf_free(w.ctx, dst) == 0
    w.close()
    assert lib.fake_hip_live_objects() == before


def test_context_creation_releases_everything_when_a_step_fails(lib):
    before = lib.fake_hip_live_objects()
    made = 3 + 5 + 16                                            #three streams, five events, sixteen checkpoint events are created
    for successes in range(made):
        lib.fake_hip_fail_after(successes)
        ctx = H()
        assert lib.vkj_ctx_create(0, C.byref(ctx)) != 0
        assert b'injected' in lib.vkj_last_error()
        assert lib.fake_hip_live_objects() == before
    lib.fake_hip_fail_after(made)                                #nothing left to fail in creation
    ctx = H()
    assert lib.vkj_ctx_create(0, C.byref(ctx)) == 0
    lib.fake_hip_fail_after(-1)
    assert lib.vkj_ctx_destroy(ctx) == 0
    assert lib.fake_hip_live_objects() == before


def test_launches_follow_the_uploads(lib):
    '''An evaluation that brings large arguments sends them in the order in which the launches first read them,
    whatever the order they were recorded in, and issues each launch once everything it and the launches before it
    read has been handed to the copy engines - not after the last byte. The stand-in runs copies and kernels at once,
    so a launch issued too early would compute on bytes that are not there yet. Arguments that stay resident, small
    ones, and launches that read no argument at all are handled; nothing is created while evaluating.'''
    before = lib.fake_hip_live_objects()
    w = World(lib)
    n = 4 << 20                                                    #16 MB each: 16 chunks
    a, b, c, small = w.buf(4 * n), w.buf(4 * n), w.buf(4 * n), w.buf(4 * 16)
    ra, rb, rc, rs, free = w.buf(4 * n), w.buf(4 * n), w.buf(4 * n), w.buf(4 * 16), w.buf(4 * 16)
    seq = H()
    assert lib.vkj_seq_create(w.ctx, 0, C.byref(seq)) == 0
    #recorded in the reverse of the order of use
    assert lib.vkj_seq_record_upload(seq, c, 0, 2, 4 * n) == 0
    assert lib.vkj_seq_record_upload(seq, b, 0, 1, 4 * n) == 0
    assert lib.vkj_seq_record_upload(seq, small, 0, 3, 4 * 16) == 0
    assert lib.vkj_seq_record_upload(seq, a, 0, 0, 4 * n) == 0
    assert w.record_add_one(seq, free, free, 16) == 0              #reads no argument
    assert w.record_add_one(seq, ra, a, n) == 0
    assert w.record_add_one(seq, rb, b, n) == 0
    assert w.record_add_one(seq, rs, small, 16) == 0
    assert w.record_add_one(seq, rc, c, n) == 0
    for slot, buf, count in ((4, ra, n), (5, rb, n), (6, rc, n), (7, rs, 16)):
        assert lib.vkj_seq_record_download(seq, buf, 0, slot, 4 * count) == 0
    rng = np.random.default_rng(8)
    made = lib.fake_hip_creations()
    def run(resident=()):
        xs = [rng.integers(0, 1 << 30, size=n, dtype=np.uint32) for _ in range(3)] + [rng.integers(0, 1 << 30, size=16, dtype=np.uint32)]
        ys = [np.zeros(n, np.uint32) for _ in range(3)] + [np.zeros(16, np.uint32)]
        ptrs = (C.c_void_p * 8)(*[None if k in resident else x.ctypes.data for k, x in enumerate(xs)], *[y.ctypes.data for y in ys])
        copies, launches = lib.fake_hip_copies(), lib.fake_hip_launches()
        assert lib.vkj_seq_eval(seq, ptrs, 8, hip.EVAL_NULL_IS_RESIDENT if resident else 0) == 0, lib.vkj_last_error()
        assert lib.fake_hip_launches() - launches == 5
        return xs, ys, [lib.fake_hip_copies_at_launch(launches + k) - copies for k in range(5)]
    xs, ys, at = run()
    for k in (0, 1, 3):
        assert np.array_equal(ys[k], xs[k] + 1)
    assert np.array_equal(ys[2], xs[2] + 1)
    #the small one first (small arguments all go ahead, whoever reads them), then a (16 chunks), b, c. Launches go at
    #checkpoints: behind what the first launch reads, then after 2 MB, 4 MB, ... more (here: every array), and at the end
    assert at == [1, 17, 33, 33, 49], at
    held = xs
    #b stays where it is: a, the small one, c
    xs, ys, at = run(resident=(1,))
    assert np.array_equal(ys[0], xs[0] + 1) and np.array_equal(ys[1], held[1] + 1) and np.array_equal(ys[2], xs[2] + 1)
    assert np.array_equal(ys[3], xs[3] + 1)
    assert at == [1, 17, 17, 17, 33], at
    assert lib.fake_hip_creations() == made
    assert lib.vkj_seq_destroy(seq) == 0
    for buf in (a, b, c, small, ra, rb, rc, rs, free):
        assert lib.vkj_buf_free(w.ctx, buf) == 0
    w.close()
    assert lib.fake_hip_live_objects() == before


def test_packed_arrays_travel_in_one_transfer(lib):
    '''vkj_buf_alloc_packed places small arrays side by side in a slab, a sequence stages their uploads side by side
    too, and an evaluation that uploads neighbours sends them with one transfer; an array that stays resident splits
    the run; larger requests get allocations of their own; the slab's memory goes with its last array, also when that
    one was still recorded in a sequence when it was freed.'''
    before = lib.fake_hip_live_objects()
    w = World(lib)
    sizes = [25, 256, 65, 1000, 7, 300]                            #words; 100 B ... 4000 B
    n_big = 4 << 20
    small, made = [], lib.fake_hip_live_objects()
    for n in sizes:
        b = H()
        assert lib.vkj_buf_alloc_packed(w.ctx, 4 * n, C.byref(b)) == 0
        small.append(b)
    assert lib.fake_hip_live_objects() == made + 1                #ONE slab
    addresses = []
    for b in small:
        addr = C.c_uint64()
        assert lib.vkj_buf_device_ptr(w.ctx, b, C.byref(addr)) == 0
        addresses.append(addr.value)
    assert all((a - addresses[0]) % 256 == 0 for a in addresses)          #(the slab itself starts where hipMalloc puts it)
    assert [b - a for a, b in zip(addresses, addresses[1:])] == [-(-4 * n // 256) * 256 for n in sizes[:-1]]
    large = H()
    assert lib.vkj_buf_alloc_packed(w.ctx, 4 * n_big, C.byref(large)) == 0          #too large for a slab: on its own
    results = [w.buf(4 * n) for n in sizes] + [w.buf(4 * n_big)]
    seq, without_sequence = H(), lib.fake_hip_live_objects()
    assert lib.vkj_seq_create(w.ctx, 0, C.byref(seq)) == 0
    for k, (b, n) in enumerate(zip(small + [large], sizes + [n_big])):
        assert lib.vkj_seq_record_upload(seq, b, 0, k, 4 * n) == 0
        assert w.record_add_one(seq, results[k], b, n) == 0
    for k, n in enumerate(sizes + [n_big]):
        assert lib.vkj_seq_record_download(seq, results[k], 0, 7 + k, 4 * n) == 0
    rng = np.random.default_rng(12)
    def run(resident=()):
        xs = [rng.integers(0, 1 << 30, size=n, dtype=np.uint32) for n in sizes + [n_big]]
        ys = [np.zeros(n, np.uint32) for n in sizes + [n_big]]
        ptrs = (C.c_void_p * 14)(*[None if k in resident else x.ctypes.data for k, x in enumerate(xs)], *[y.ctypes.data for y in ys])
        copies = lib.fake_hip_copies()
        assert lib.vkj_seq_eval(seq, ptrs, 14, hip.EVAL_NULL_IS_RESIDENT if resident else 0) == 0, lib.vkj_last_error()
        return xs, ys, lib.fake_hip_copies() - copies
    xs, ys, copies = run()
    assert all(np.array_equal(y, x + 1) for x, y in zip(xs, ys))
    held = xs
    _, ys, downloads = run(resident=range(7))                      #nothing goes up: what the results cost to bring back
    assert all(np.array_equal(y, x + 1) for x, y in zip(held, ys))
    assert copies - downloads == 1 + 16                            #one run for the six small arrays, the large one's chunks
    xs, ys, copies = run(resident=(2,))
    assert all(np.array_equal(y, (held[k] if k == 2 else x) + 1) for k, (x, y) in enumerate(zip(xs, ys)))
    assert copies - downloads == 2 + 16                            #the arrays before and behind the one that stays
    #freed while the sequence still holds them: the slab stays until the sequence goes
    for b in small:
        assert lib.vkj_buf_free(w.ctx, b) == 0
    live = lib.fake_hip_live_objects()
    xs, ys, copies = run()
    assert all(np.array_equal(y, x + 1) for x, y in zip(xs, ys))
    assert lib.fake_hip_live_objects() == live                     #nothing has gone yet
    assert lib.vkj_seq_destroy(seq) == 0
    assert lib.fake_hip_live_objects() == without_sequence - 1     #everything the sequence had made, and the slab
    for b in [large] + results:
        assert lib.vkj_buf_free(w.ctx, b) == 0
    w.close()
    assert lib.fake_hip_live_objects() == before


def test_landing_allocation_failure_leaves_nothing_behind(lib):
    w = World(lib)
    seq, src, dst = w.add_one_sequence(16)
    x = np.arange(16, dtype=np.uint32)
    y = np.zeros(16, np.uint32)
    ptrs, nptrs = (C.c_void_p * 2)(x.ctypes.data, y.ctypes.data), (C.c_void_p * 2)(x.ctypes.data, None)
    base = lib.fake_hip_live_objects()
    lib.fake_hip_fail_after(1)                                   #landing buffer succeeds, its pinned staging does not
    assert lib.vkj_seq_eval_next(seq, ptrs, 2, 0, nptrs) != 0
    assert lib.fake_hip_live_objects() == base
    assert np.array_equal(w.eval(seq, x, nxt=x), x + 1)          #and the sequence still works
    assert lib.fake_hip_live_objects() == base + 2
    assert lib.vkj_seq_destroy(seq) == 0
    for b in (src, dst):
        assert lib.vkj_buf_free(w.ctx, b) == 0
    w.close()


def test_objects_of_another_context_and_bad_ranges_are_rejected(lib):
    w, w2 = World(lib), World(lib)
    seq, src, dst = w.add_one_sequence(4)
    other = w2.buf(16)
    assert lib.vkj_seq_record_upload(seq, other, 0, 2, 16) == EINVAL
    assert w.record_add_one(seq, other, src, 4) == EINVAL
    assert w.record_add_one(seq, dst, src, 4, fn=w2.fn) == EINVAL
    assert lib.vkj_seq_record_upload(seq, src, 8, 2, 16) == EINVAL       #range beyond the buffer
    assert lib.vkj_buf_free(w2.ctx, src) == EINVAL
    ptrs = (C.c_void_p * 2)(None, None)
    assert lib.vkj_seq_eval(seq, ptrs, 2, 0) == EINVAL                    #no host pointer for the upload
    assert lib.vkj_seq_destroy(seq) == 0
    for b in (src, dst):
        assert lib.vkj_buf_free(w.ctx, b) == 0
    assert lib.vkj_buf_free(w2.ctx, other) == 0
    w.close(); w2.close()


def test_static_entry_point_allocates_nothing_and_equals_the_allocating_one(lib):
    '''vkj_seq_eval_next_static (its host side; the stand-in build moves the landed bytes with a host copy): across
    its calls the stand-in runtime sees no allocation, pinned allocation, stream, event or graph being made, for
    small arguments and for ones that are staged in chunks by helper threads, and the results equal
    vkj_seq_eval_next's.'''
    w = World(lib)
    rng = np.random.default_rng(11)
    for n in (1000, 3 << 20):                                    #4 KB; 12 MB (three chunks)
        seq, src, dst = w.add_one_sequence(n)
        seq2, src2, dst2 = w.add_one_sequence(n)
        xs = [rng.integers(0, 1 << 32, size=n, dtype=np.uint64).astype(np.uint32) for _ in range(4)]
        want = [w.eval(seq2, xs[0], nxt=xs[1])] + [w.eval(seq2, None, nxt=x, flags=hip.EVAL_NULL_IS_RESIDENT, n=n) for x in xs[2:] + xs[:1]]
        made = lib.fake_hip_creations()
        got = []
        for k in range(4):
            y = np.zeros(n, np.uint32)
            ptrs  = (C.c_void_p * 2)(xs[0].ctypes.data if k == 0 else None, y.ctypes.data)
            nptrs = (C.c_void_p * 2)(xs[(k + 1) % 4].ctypes.data, None)
            assert lib.vkj_seq_eval_next_static(seq, ptrs, 2, hip.EVAL_NULL_IS_RESIDENT, nptrs) == 0, lib.vkj_last_error()
            got.append(y)
        assert lib.fake_hip_creations() == made
        for k, (a, b) in enumerate(zip(got, want)):
            assert np.array_equal(a, b) and np.array_equal(a, xs[k] + 1), (n, k)
        for q in (seq, seq2):
            assert lib.vkj_seq_destroy(q) == 0
        for b in (src, dst, src2, dst2):
            assert lib.vkj_buf_free(w.ctx, b) == 0
    w.close()


def test_static_entry_point_refuses_a_call_that_overlaps_another(lib):
    '''The static landing array is one per GPU: while a call is using it, a second call on that GPU (here: made from
    inside the first one's final synchronisation, from another context) is refused, and the first is unharmed.'''
    w, w2 = World(lib), World(lib)
    seq, src, dst = w.add_one_sequence(256)
    seq2, src2, dst2 = w2.add_one_sequence(256)
    x = np.arange(256, dtype=np.uint32)
    y, y2 = np.zeros(256, np.uint32), np.zeros(256, np.uint32)
    ptrs,  nptrs  = (C.c_void_p * 2)(x.ctypes.data, y.ctypes.data),  (C.c_void_p * 2)(x.ctypes.data, None)
    ptrs2, nptrs2 = (C.c_void_p * 2)(x.ctypes.data, y2.ctypes.data), (C.c_void_p * 2)(x.ctypes.data, None)
    seen = []

    @C.CFUNCTYPE(None)
    def reenter():
        seen.append(lib.vkj_seq_eval_next_static(seq2, ptrs2, 2, 0, nptrs2))
        seen.append(lib.vkj_last_error())
    lib.fake_hip_on_synchronize(C.cast(reenter, C.c_void_p))
    assert lib.vkj_seq_eval_next_static(seq, ptrs, 2, 0, nptrs) == 0, lib.vkj_last_error()
    assert seen[0] == ESTATE and b'busy' in seen[1], seen
    assert np.array_equal(y, x + 1) and not y2.any()
    assert lib.vkj_seq_eval_next_static(seq2, ptrs2, 2, 0, nptrs2) == 0      #free again once the first call has returned
    assert np.array_equal(y2, x + 1)
    for q in (seq, seq2):
        assert lib.vkj_seq_destroy(q) == 0
    for ww, bs in ((w, (src, dst)), (w2, (src2, dst2))):
        for b in bs:
            assert lib.vkj_buf_free(ww.ctx, b) == 0
        ww.close()


def test_static_entry_point_and_graphs(lib):
    '''A sequence that replays as a graph is refused until the graph exists (building it allocates) - but a graph is
    only ever built for more than one launch, so a single-launch sequence with graphs switched on is evaluated.'''
    w = World(lib)
    seq, src, dst = w.add_one_sequence(32)
    assert lib.vkj_seq_use_graph(seq, 1) == 0
    x = np.arange(32, dtype=np.uint32)
    y = np.zeros(32, np.uint32)
    ptrs = (C.c_void_p * 2)(x.ctypes.data, y.ctypes.data)
    assert lib.vkj_seq_eval_next_static(seq, ptrs, 2, 0, None) == 0, lib.vkj_last_error()
    assert np.array_equal(y, x + 1)
    assert w.record_add_one(seq, src, dst, 32) == 0              #a second launch: src = dst + 1
    assert lib.vkj_seq_eval_next_static(seq, ptrs, 2, 0, None) == ESTATE
    assert b'graph' in lib.vkj_last_error()
    assert lib.vkj_seq_eval(seq, ptrs, 2, 0) == 0                #builds it (the stand-in cannot: plain launches from now on)
    assert lib.vkj_seq_eval_next_static(seq, ptrs, 2, 0, None) == 0, lib.vkj_last_error()
    profiled = H()
    assert lib.vkj_seq_create(w.ctx, 1, C.byref(profiled)) == 0
    assert lib.vkj_seq_eval_next_static(profiled, None, 0, 0, None) == ESTATE
    for q in (seq, profiled):
        assert lib.vkj_seq_destroy(q) == 0
    for b in (src, dst):
        assert lib.vkj_buf_free(w.ctx, b) == 0
    w.close()


def test_launches_on_two_lanes(lib):
    '''vkj_seq_set_launch_lane: launches of lane 1 go to the side stream, waits make events at record time (none when
    evaluating), bad arguments are refused, and everything is released with the sequence.'''
    before = lib.fake_hip_live_objects()
    w = World(lib)
    n = 100
    a, b, c, seq = w.buf(4 * n), w.buf(4 * n), w.buf(4 * n), H()
    assert lib.vkj_seq_create(w.ctx, 0, C.byref(seq)) == 0
    assert lib.vkj_seq_record_upload(seq, a, 0, 0, 4 * n) == 0
    assert w.record_add_one(seq, b, a, n) == 0                   #b = a + 1
    assert w.record_add_one(seq, c, a, n) == 0                   #c = a + 1   (independent of the first: lane 1)
    assert w.record_add_one(seq, a, c, n) == 0                   #a = c + 1   (waits for lane 1, and for the first launch's read of a)
    assert lib.vkj_seq_record_download(seq, a, 0, 1, 4 * n) == 0
    assert lib.vkj_seq_set_launch_lane(seq, 1, 1, 0) == 0
    assert lib.vkj_seq_set_launch_lane(seq, 2, 0, 1) == 0
    assert lib.vkj_seq_set_launch_lane(seq, 3, 0, 0) == EINVAL    #no such launch
    assert lib.vkj_seq_set_launch_lane(seq, 0, 2, 0) == EINVAL    #no such lane
    made = lib.fake_hip_creations()
    x = np.arange(n, dtype=np.uint32)
    for _ in range(3):
        assert np.array_equal(w.eval(seq, x), x + 2)
    assert lib.fake_hip_creations() == made                      #fork, join and wait events exist since they were asked for
    assert lib.vkj_seq_set_launch_lane(seq, 2, 0, 0) == 0         #a wait that is taken back gives its event back
    assert lib.vkj_seq_set_launch_lane(seq, 1, 0, 0) == 0         #back on one lane
    assert np.array_equal(w.eval(seq, x), x + 2)
    assert lib.vkj_seq_destroy(seq) == 0
    for buf in (a, b, c):
        assert lib.vkj_buf_free(w.ctx, buf) == 0
    w.close()
    assert lib.fake_hip_live_objects() == before


def test_first_launch_in_parts_beside_the_upload(lib):
    '''vkj_seq_record_early_part: when an evaluation uploads the argument the parts read (in chunks, as the last of its
    uploads), each part is issued as soon as the chunks it needs have been handed over - the stand-in runs copies and
    kernels at once, so a part issued too early would compute on bytes that are not there yet - and the first launch
    itself is skipped; with the argument resident, or followed by another upload, the launch runs as recorded.
    Nothing is created while evaluating; bad arguments are refused; everything goes with the sequence.'''
    before = lib.fake_hip_live_objects()
    w = World(lib)
    n, nparts = 4 << 20, 4                                        #16 MB: uploads of 8 MB and more travel in chunks
    src, mid, dst, other, seq = w.buf(4 * n), w.buf(4 * n), w.buf(4 * n), w.buf(64), H()
    assert lib.vkj_seq_create(w.ctx, 0, C.byref(seq)) == 0
    grid = (C.c_uint32 * 3)(1, 1, 1)
    def part_args(p):
        kernarg = bytes(16) + np.uint32(n // nparts).tobytes() + bytes(4)
        bufs = (C.c_uint64 * 2)(mid.value, src.value)
        offs = (C.c_uint32 * 2)(0, 8)
        byte = (C.c_uint64 * 2)(p * 4 * n // nparts, p * 4 * n // nparts)
        return (seq, w.fn, grid, grid, 0, kernarg, len(kernarg), bufs, offs, byte, 2)
    assert lib.vkj_seq_record_upload(seq, src, 0, 0, 4 * n) == 0
    assert lib.vkj_seq_record_early_part(*part_args(0), 0, 4 * n // nparts) == ESTATE       #no launch to stand for yet
    assert w.record_add_one(seq, mid, src, n) == 0               #mid = src + 1: the launch the parts stand for
    assert w.record_add_one(seq, dst, mid, n) == 0               #dst = mid + 1
    assert lib.vkj_seq_record_download(seq, dst, 0, 1, 4 * n) == 0
    assert lib.vkj_seq_record_early_part(*part_args(0), 3, 4 * n // nparts) == EINVAL       #no upload in that slot
    assert lib.vkj_seq_record_early_part(*part_args(0), 0, 4 * n + 4) == EINVAL             #more than the argument has
    for p in range(nparts):
        assert lib.vkj_seq_record_early_part(*part_args(p), 0, (p + 1) * 4 * n // nparts) == 0, lib.vkj_last_error()
    assert lib.vkj_seq_record_early_part(*part_args(0), 0, 4 * n // nparts) == EINVAL       #parts come in ascending order
    made = lib.fake_hip_creations()
    rng = np.random.default_rng(3)
    for _ in range(2):
        x = rng.integers(0, 1 << 30, size=n, dtype=np.uint32)
        launches = lib.fake_hip_launches()
        assert np.array_equal(w.eval(seq, x), x + 2)
        assert lib.fake_hip_launches() - launches == nparts + 1   #the parts, then the second launch
    #the argument stays where it is: the launch as recorded
    launches = lib.fake_hip_launches()
    assert np.array_equal(w.eval(seq, None, flags=1, n=n), x + 2)            #VKJ_EVAL_NULL_IS_RESIDENT
    assert lib.fake_hip_launches() - launches == 2
    assert lib.fake_hip_creations() == made
    assert lib.vkj_seq_destroy(seq) == 0
    #another argument recorded behind it, which the launch does not read: sent behind it too, parts as before
    seq = H()
    assert lib.vkj_seq_create(w.ctx, 0, C.byref(seq)) == 0
    assert lib.vkj_seq_record_upload(seq, src, 0, 0, 4 * n) == 0
    assert lib.vkj_seq_record_upload(seq, other, 0, 2, 64) == 0
    assert w.record_add_one(seq, mid, src, n) == 0
    assert lib.vkj_seq_record_download(seq, mid, 0, 1, 4 * n) == 0
    for p in range(nparts):
        assert lib.vkj_seq_record_early_part(*part_args(p), 0, (p + 1) * 4 * n // nparts) == 0
    y, small = np.zeros(n, np.uint32), np.zeros(16, np.uint32)
    ptrs = (C.c_void_p * 3)(x.ctypes.data, y.ctypes.data, small.ctypes.data)
    launches = lib.fake_hip_launches()
    assert lib.vkj_seq_eval(seq, ptrs, 3, 0) == 0, lib.vkj_last_error()
    assert np.array_equal(y, x + 1) and lib.fake_hip_launches() - launches == nparts
    assert lib.vkj_seq_destroy(seq) == 0
    for b in (src, mid, dst, other):
        assert lib.vkj_buf_free(w.ctx, b) == 0
    w.close()
    assert lib.fake_hip_live_objects() == before
