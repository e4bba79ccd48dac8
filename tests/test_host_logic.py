'''Host-side behaviour that needs no GPU: the C ABI (library loads, exports every declared
symbol, fails cleanly without a device), the trace cache of Function, the buffer pool's
liveness reuse, the dispatch's error behaviour, and the kernel argument layouts.
The literal expectations come from the reference's own tests (tests/test_function.py:13-60,
tests/test_bufferpool.py:32-40,62-63).'''
import ctypes
import json
import os
import re
import subprocess

import numpy as np
import pytest

import vkjax_amd
from vkjax_amd import hip, kernels as K, minijax as mj, ops
from vkjax_amd.buffers import Buffer, BufferPool, PlanOnlyDevice, to_device_words, view_or_convert_from_32bit
from vkjax_amd.jaxpr_interpreter import JaxprInterpreter
from vkjax_amd.minijax import core

ROOT   = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = json.load(open(os.path.join(ROOT, 'tests', 'golden', 'known_answers.json')))['reference_test_literals']
jnp, lax = mj.numpy, mj.lax


# ------------------------------------------------------------------ C ABI

def test_library_exports_every_declared_symbol():
    header   = open(os.path.join(ROOT, 'include', 'vkjax_hip.h')).read()
    declared = set(re.findall(r'\b(vkj_\w+)\s*\(', header))
    assert len(declared) >= 25
    lib = hip.load_library()
    for name in declared:
        assert hasattr(lib, name), f'{name} declared in the header but not exported'
    assert declared == set(hip.exported_symbols())


def test_abi_fails_cleanly_on_bad_arguments():
    lib = hip.load_library()
    assert lib.vkj_ctx_destroy(0) == -1 and b'bad context handle' in lib.vkj_last_error()
    assert lib.vkj_sync(12345) != 0
    n = ctypes.c_int(-1)
    lib.vkj_device_count(ctypes.byref(n))
    assert n.value >= 0
    if n.value == 0:
        h = ctypes.c_uint64(0)
        assert lib.vkj_ctx_create(0, ctypes.byref(h)) == -4          #VKJ_ENODEV
        assert b'no HIP device' in lib.vkj_last_error()
        with pytest.raises(hip.HipError):
            hip.Device(0)


def test_code_objects_are_built_for_gfx950():
    for name in hip.KERNEL_MODULES:
        path = os.path.join(hip.LIBDIR, f'{name}.hsaco')
        assert os.path.exists(path), f'{path} missing: run python -m vkjax_amd.csrc.build'
        assert b'gfx950' in open(path, 'rb').read()


def test_kernel_argument_layouts_match_the_structs():
    '''sizeof of every kernel parameter struct, taken from the compiler, equals the length of
    the block the host packs.'''
    #the parameter structs and the #defines they use are lifted out of the kernel sources and
    #compiled on their own with the host compiler
    kdir  = os.path.join(ROOT, 'vkjax_amd', 'csrc', 'kernels')
    text  = ''.join(open(os.path.join(kdir, f)).read() for f in sorted(os.listdir(kdir)) if f.endswith('.hip'))
    defs  = re.findall(r'^#define\s+(?:EW_MAX_STEPS|CONV_MAX_EPI|CONV_MAX_DERIVED|IDX_MAX_RANK|TF_MAX_STEPS|PAD_MAX_RANK)\s+\d+\s*$', text, re.M)
    decls = re.findall(r'^struct\s+\w+\s*\{[^}]*\};', text, re.M)
    names = [re.match(r'struct\s+(\w+)', d).group(1) for d in decls]
    src   = '#include <cstdio>\n#include <cstdint>\n' + '\n'.join(defs) + '\n' + '\n'.join(decls) + '\nint main(){\n' \
          + ''.join(f'  printf("{n} %zu\\n", sizeof({n}));\n' for n in names) + '}\n'
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        open(os.path.join(tmp, 'sz.cpp'), 'w').write(src)
        exe = os.path.join(tmp, 'sz')
        subprocess.run(['g++', '-O0', '-w', os.path.join(tmp, 'sz.cpp'), '-o', exe], check=True, capture_output=True)
        sizes = dict(line.split() for line in subprocess.run([exe], check=True, capture_output=True, text=True).stdout.splitlines())
    sizes = {k: int(v) for k, v in sizes.items()}
    f32 = np.dtype('float32')
    b = lambda *shape: Buffer(None, f32, shape)
    i = lambda *shape: Buffer(None, np.dtype('int32'), shape)
    chain = K.EwChain(b(4, 8), (4, 8), K.broadcast_operand(b(4, 8), (4, 8)), [K.EwStep(K.EW['ADD_F'], K.broadcast_operand(b(8), (4, 8)))])
    geom  = K.ConvGeometry(batch=1, Ho=4, Wo=4, N=24, H=4, W=4, Cin=4, KH=1, KW=1, xs=(64, 16, 4, 1), ws=(96, 96, 24, 1), os=(384, 96, 24, 1))
    few   = K.ConvGeometry(batch=1, Ho=16, Wo=1, N=8, H=16, W=1, Cin=4, KH=1, KW=1, xs=(0, 4, 0, 1), ws=(32, 32, 8, 1), os=(128, 8, 8, 1))
    G, S = core.GatherDimensionNumbers, core.ScatterDimensionNumbers
    launches = {
        'EwParams': K.lower_ew_chain(chain), 'EwAffineParams': K.lower_ew_chain(K.EwChain(b(64, 8), (64, 8), K.broadcast_operand(b(64, 8), (64, 8)), [K.EwStep(K.EW[o], K.broadcast_operand(b(*sh), (64, 8))) for o, sh in (('ADD_F', (64, 8)), ('SUB_F', (8,)), ('MUL_F', (8,)), ('ADD_F', (8,)))])),
        'IotaParams': K.iota(i(8), 0), 'FillParams': K.fill(b(8), 0),
        'ConcatParams': K.concat_part(b(4, 8), b(4, 3), 1, 0), 'ConvParams': K.conv_gemm(b(1, 4, 4, 24), b(1, 4, 4, 4), b(1, 1, 4, 24), geom),
        'DenseRowsParams': K.conv_gemm(b(16, 8), b(16, 4), b(4, 8), few),
        'ConvStemParams': K.conv_gemm(b(1, 64, 64, 8), b(1, 128, 128, 3), b(7, 7, 3, 8),
                                      K.ConvGeometry(batch=1, Ho=64, Wo=64, N=8, H=128, W=128, Cin=3, KH=7, KW=7, SH=2, SW=2, PH=3, PW=3,
                                                     xs=(128 * 384, 384, 3, 1), ws=(168, 24, 8, 1), os=(64 * 512, 512, 8, 1))),
        'ReduceParams': K.reduce(b(4), b(4, 8), 4, 8, 1, 'reduce_sum')[0],
        'ReduceGeneralParams': K.reduce_general(b(4), b(4, 8), [(4, 8)], [(8, 1)], 'reduce_sum'),
        'PoolParams': K.pool(b(1, 2, 2, 4), b(1, 4, 4, 4), 'reduce_max', (1, 2, 2, 1), (1, 2, 2, 1), (0, 0, 0, 0), (1, 1, 1, 1)),
        'WgradParams': K.wgrad_gemm(b(2, 9 * 4 * 8), b(2, 8, 8, 4), b(2, 8, 8, 8),
                                    K.WgradGeometry(images=2, Ho=8, Wo=8, H=8, W=8, C=4, KH=3, KW=3, N=8, PH=1, PW=1), 2),
        'TransposeParams': K.lower_ew_chain(K.EwChain(b(40, 30), (40, 30), K.EwOperand(b(30, 40), 0, (1, 40)), [])),
        'PadParams': K.pad(b(6, 8), b(4, 8), b(), ((1, 1, 0), (0, 0, 0))),
        'GatherRowsParams': K.gather_rows(b(3, 8), b(4, 8), i(3, 1), 3, 8, 4),
        'GatherGeneralParams': K.gather_general(b(3, 8), b(4, 8), i(3, 1), (1,), (0,), (0,), (1, 8)),
        'ScatterRowsParams': K.scatter_add_rows(b(4, 8), i(3, 1), b(3, 8), 3, 8, 4),
        'ScatterSortParams': K.scatter_add_rows_sorted(b(4, 8), b(4, 8), i(3, 1), b(3, 8), *[Buffer(None, np.dtype('uint32'), (n,)) for n in (5, 128, 3, 3)],
                                                       3, 8, 4)[0],
        'ScatterGeneralParams': K.scatter_add_general(b(4, 8), i(3, 1), b(3, 8), (1,), (0,), (0,)),
        'ThreefryParams': K.threefry2x32(*[Buffer(None, np.dtype('uint32'), (8,)) for _ in range(6)], key_is_scalar=False),
        'ThreefryStreamParams': K.threefry_stream(Buffer(None, np.dtype('uint32'), (16,)), (Buffer(None, np.dtype('uint32'), (2,)), 0),
                                                  (Buffer(None, np.dtype('uint32'), (2,)), 1), 8, 0, 8, []),
    }
    #the convolution kernel takes two parameter structs, one after the other
    sizes['ConvParams'] += sizes['ConvDerived']
    sizes['ConvStemParams'] += sizes['ConvDerived']
    assert launches['EwAffineParams'].kernel == 'ew_affine_v4' and len(launches['EwAffineParams'].buffers) == 10
    assert launches['ConvStemParams'].kernel in ('conv_gemm_stem_7x22', 'conv_gemm_stem_7x22_m128') and launches['DenseRowsParams'].kernel == 'dense_rows_n16'
    assert len(launches['DenseRowsParams'].buffers) == 3 + K.CONV_MAX_EPI
    for struct, launch in launches.items():
        assert len(launch.params) == sizes[struct], (struct, len(launch.params), sizes[struct])
    assert sizes['ConvEpiPtrs'] == 8 * K.CONV_MAX_EPI and sizes['ThreefryStreamPtrs'] == 8 * K.TF_MAX_STEPS
    assert len(launches['ThreefryStreamParams'].buffers) == 3 + K.TF_MAX_STEPS
    assert sizes['ConvDerivedPtrs'] == 8 * (K.CONV_MAX_DERIVED + 1)
    assert len(launches['ConvParams'].buffers) == 3 + K.CONV_MAX_EPI + K.CONV_MAX_DERIVED + 1 and len(launches['EwParams'].buffers) == 1 + K.EW_MAX_STEPS


# ------------------------------------------------------------------ Function: trace cache

TRACED = []

def func0(x):
    TRACED.append(x)
    return x + 1


def test_function_retraces_only_on_new_shape_or_dtype():
    vk_func = vkjax_amd.Function(func0, frontend='minijax', plan_only=True)
    get = lambda *a: vk_func._get_or_create_jaxpr_interpreter(a)
    assert len(vk_func._jaxpr_interpreters) == 0
    TRACED.clear(); get(65)
    assert len(vk_func._jaxpr_interpreters) == 1 and isinstance(TRACED[-1], mj.Tracer)
    TRACED.clear(); get(77)
    assert len(vk_func._jaxpr_interpreters) == 1 and TRACED == []
    get(np.zeros([4, 4])); get(np.zeros([4, 4]))
    assert len(vk_func._jaxpr_interpreters) == 2
    get(np.zeros([4, 5]))
    assert len(vk_func._jaxpr_interpreters) == 3
    #dtype is part of the key, and is preserved in the traced output type
    x = np.arange(128).astype('uint32')
    (_, s0), (_, s1) = get(x), get(x.astype('float32'))
    assert len(vk_func._jaxpr_interpreters) == 5
    assert s0.dtype == np.uint32 and s1.dtype == np.float32


def test_static_argnums_are_not_device_arguments():
    def f(x, flag):
        return x * 2 if flag else x * 3
    vk = vkjax_amd.wrap(f, static_argnums=(1,), frontend='minijax', plan_only=True)
    interp, _ = vk._get_or_create_jaxpr_interpreter((np.ones(3), True))
    assert len(interp.input_buffers) == 1
    assert len(vk._jaxpr_interpreters) == 1
    vk._get_or_create_jaxpr_interpreter((np.ones(3), False))
    assert len(vk._jaxpr_interpreters) == 2


def test_wrong_argument_count_raises_typeerror():
    closed = mj.make_jaxpr(lambda x, y: x + y)(1.0, 2.0)
    interp = JaxprInterpreter(closed, plan_only=True)
    with pytest.raises(TypeError, match='Expected 2 input arguments, received 1'):
        interp.run(1.0)
    with pytest.raises(RuntimeError, match='plan_only'):
        interp.run(1.0, 2.0)


# ------------------------------------------------------------------ buffer pool

def test_bufferpool_lowlevel_reuse():
    pool = BufferPool(PlanOnlyDevice(), 1)
    aval = core.ShapedArray((10, 10), 'float32')
    v0, v1, v3 = core.Var(0, '', aval), core.Var(1, '', aval), core.Var(3, '', aval)
    pool.get_buffer(v0, increment_op_counter=True); assert pool.op_counter == 1
    pool.get_buffer(v1, increment_op_counter=True); assert pool.op_counter == 2
    pool.get_buffer(v0, increment_op_counter=True); assert pool.op_counter == 3
    pool.get_buffer(v3, increment_op_counter=True)
    assert [pool.buffers[v].accesses for v in (v0, v1, v3)] == GOLDEN['bufferpool_lowlevel_accesses']
    pool.create_tensors()
    assert len(pool.unique_tensors()) == GOLDEN['bufferpool_lowlevel_unique_tensors']


def test_bufferpool_highlevel_reuse():
    def func(a, b):
        c = a + 5
        d = c * b
        e = d - 2
        f = e ** 3
        g = f - 1
        h = g * 5
        return h
    closed = mj.make_jaxpr(func)(65, 5)
    pool = JaxprInterpreter(closed, reuse_buffers=True, fuse=False, plan_only=True).bufferpool
    assert len(pool.buffers) == 11
    assert len(pool.unique_tensors()) == GOLDEN['bufferpool_highlevel_unique_tensors']   #11 buffers overall, -3 re-used
    pool = JaxprInterpreter(closed, reuse_buffers=False, fuse=False, plan_only=True).bufferpool
    assert len(pool.unique_tensors()) == 11


def test_views_share_storage_and_32bit_canonicalisation():
    closed = mj.make_jaxpr(lambda x: lax.bitcast_convert_type((x + 1).reshape(2, 8), np.uint32))(np.zeros(16, np.float32))
    interp = JaxprInterpreter(closed, fuse=False, plan_only=True)
    assert [l.kernel for l in interp.launches] == ['ew_chain_v4_s2']      #reshape and bitcast are free
    words = to_device_words(np.array([True, False, True]))
    assert words.dtype == np.uint32 and words.tolist() == [1, 0, 1]
    assert view_or_convert_from_32bit(words, np.bool_).tolist() == [True, False, True]
    assert to_device_words(np.array([1.5], np.float64)).view(np.float32)[0] == 1.5
    assert to_device_words(np.array([-2], np.int64)).view(np.int32)[0] == -2
    with pytest.raises(NotImplementedError):
        to_device_words(np.array([1 + 2j]))


# ------------------------------------------------------------------ dispatch errors

def _eqn(name, invals, out_aval, **params):
    invars = [core.Var(None, '', core.ShapedArray(np.shape(v), np.asarray(v).dtype)) for v in invals]
    return core.JaxprEqn(invars, [core.Var(None, '', out_aval)], core.Primitive(name), params), invars


def test_unknown_primitive_and_bad_params():
    pool = BufferPool(PlanOnlyDevice())
    eq, invars = _eqn('cholesky', [np.zeros((2, 2), np.float32)], core.ShapedArray((2, 2), 'float32'))
    with pytest.raises(NotImplementedError):
        ops.analyze_jaxpr(pool, core.Jaxpr([], invars, eq.outvars, [eq]))
    eq, invars = _eqn('add', [np.zeros((2, 3), np.float32), np.zeros((4,), np.float32)], core.ShapedArray((2, 3), 'float32'))
    with pytest.raises(ValueError, match='Cannot broadcast'):
        ops.analyze_jaxpr(pool, core.Jaxpr([], invars, eq.outvars, [eq]))
    eq, invars = _eqn('exp', [np.zeros((2,), np.int32)], core.ShapedArray((2,), 'int32'))
    with pytest.raises(NotImplementedError):
        ops.analyze_jaxpr(pool, core.Jaxpr([], invars, eq.outvars, [eq]))
    eq, invars = _eqn('dot_general', [np.zeros((2, 3), np.float32), np.zeros((3, 2), np.float32)], core.ShapedArray((2, 2), 'float32'),
                      dimension_numbers=(((1,), (0,)), ((), ())), precision='HIGHEST')
    with pytest.raises(AssertionError):
        ops.analyze_jaxpr(pool, core.Jaxpr([], invars, eq.outvars, [eq]))
    with pytest.raises(NotImplementedError):
        core.canonicalize_dtype(np.complex64)


def test_dropped_outputs_are_skipped_and_calls_are_inlined():
    aval = core.ShapedArray((4,), 'float32')
    x = core.Var(None, '', aval)
    dropped = core.JaxprEqn([x], [core.DropVar(aval)], core.Primitive('exp'), {})
    kept    = core.JaxprEqn([x], [core.Var(None, '', aval)], core.Primitive('neg'), {})
    pool = BufferPool(PlanOnlyDevice())
    out = ops.analyze_jaxpr(pool, core.Jaxpr([], [x], kept.outvars, [dropped, kept]))
    assert len(out) == 1 and out[0].equation is kept
    closed = mj.make_jaxpr(lambda a, b: mj.jit(lambda u: u + u)(a) + mj.jit(lambda u, v: u + v)(b, 1.0))(5.0, 7.1)
    interp = JaxprInterpreter(closed, fuse=False, plan_only=True)
    assert [l.kernel for l in interp.launches] == ['ew_chain_v1_s2'] * 3


def test_opcode_table_and_tile_choice():
    assert K.EW['ADD_F'] == 1 and K.EW['SEL_P'] == 50 and len(set(K.EW.values())) == len(K.EW)
    tags = [t[0] for t in K.CONV_TILES]
    for m, n in [(200704, 256), (200704, 64), (3136, 512), (8, 16), (1, 1)]:
        tag, bm, bn, nt = K.choose_conv_tile(m, n)
        assert tag in tags and nt in (64, 256)
    assert K.choose_conv_tile(8, 16)[1] <= 64


def test_integer_and_float_literals_of_equal_hash_get_separate_buffers():
    '''jax literals carry hash(value), and hash(1) == hash(1.0): the pool must still keep them apart.'''
    from vkjax_amd.buffers import BufferPool, PlanOnlyDevice

    class JaxLikeLiteral:
        def __init__(self, val, dtype):
            self.val, self.aval, self.hash = val, core.ShapedArray((), dtype), hash(val)

    pool = BufferPool(PlanOnlyDevice())
    one_i, one_f, one_f_again = JaxLikeLiteral(1, np.int32), JaxLikeLiteral(1.0, np.float32), JaxLikeLiteral(1.0, np.float32)
    bi, bf, bf2 = pool.get_buffer(one_i), pool.get_buffer(one_f), pool.get_buffer(one_f_again)
    assert bi is not bf and bf is bf2
    assert bi.dtype == np.int32 and bf.dtype == np.float32
    assert bi.tensor.initial_value.view(np.int32)[0] == 1 and bf.tensor.initial_value.view(np.float32)[0] == 1.0


def test_ahead_iterator_keeps_order_passes_errors_on_and_lets_go():
    '''The helper-thread iterator behind Function.stream: results come in the order of the
    iterable, an exception raised by the iterable or by `prepare` reaches the consumer at the
    position where it happened, and close() releases a helper that is waiting for the consumer.'''
    import threading, time
    from vkjax_amd.function import _Ahead
    assert list(_Ahead(range(20), lambda i: i * i)) == [i * i for i in range(20)]
    assert list(_Ahead([], lambda i: i)) == []

    def failing(i):
        if i == 3:
            raise KeyError('three')
        return i
    got = []
    with pytest.raises(KeyError):
        for value in _Ahead(range(10), failing):
            got.append(value)
    assert got == [0, 1, 2]

    def endless():
        i = 0
        while True:
            yield i
            i += 1
    ahead = _Ahead(endless(), lambda i: i)
    it = iter(ahead)
    assert [next(it), next(it)] == [0, 1]
    ahead.close()
    ahead._thread.join(timeout=2.0)
    assert not ahead._thread.is_alive()

    # a helper parked on the consumer's event is released by close() too
    gate = threading.Event()
    def wait_for_consumer(i):
        gate.wait()
        return i
    parked = _Ahead(range(3), wait_for_consumer, wake=gate)
    time.sleep(0.05)
    parked.close()
    parked._thread.join(timeout=2.0)
    assert not parked._thread.is_alive()


def test_treedef_hash_and_equality():
    from vkjax_amd.minijax import tree_util
    a = tree_util.tree_structure(({'w': 1, 'b': [2, 3]}, None, (4,)))
    b = tree_util.tree_structure(({'b': [0, 0], 'w': 0}, None, (0,)))
    c = tree_util.tree_structure(({'b': (0, 0), 'w': 0}, None, (0,)))
    d = tree_util.tree_structure([{'b': [0, 0], 'w': 0}, None, (0,)])
    assert a == b and hash(a) == hash(b)
    assert a != c and a != d
    assert len({a, b, c, d}) == 3


def test_batch_of_one_fuses_like_any_other():
    '''Strides of dimensions of size 1 are never used; a leading batch dimension of 1 must not keep element-wise
    chains from joining each other or a convolution's epilogue.'''
    import vkjax_amd
    from vkjax_amd import workloads as W
    from vkjax_amd import kernels as K
    counts = []
    with K.overrides(conv_k_splits=1):         #(a sliced contraction would add a launch of its own)
        for batch in (1, 2):
            fn = vkjax_amd.wrap(W.resnet50, frontend='minijax', plan_only=True)
            interp, _ = fn._get_or_create_jaxpr_interpreter(tuple(W.resnet50_inputs(batch=batch, size=64, num_classes=40, width_scale=0.25)))
            counts.append(len(interp.launches))
    assert counts[0] == counts[1] == 57, counts


def test_long_contractions_of_few_tiles_are_sliced():
    '''A product with few 32 x 32 tiles and a long contraction is planned as a launch that sums up to four slices of
    the contraction into a temporary (one [M, N] matrix per slice, blocks = tiles x slices) followed by an element-wise
    launch that adds the slices in order and takes over the equations behind the product. Products with many tiles or
    short contractions are planned as before.'''
    import vkjax_amd
    from vkjax_amd import minijax as mj, kernels as K
    from vkjax_amd.jaxpr_interpreter import JaxprInterpreter
    def layer(x, w, b):
        return mj.nn.relu(mj.numpy.dot(x, w) + b)
    def plan(m, k, n, **kw):
        args = (np.zeros((m, k), np.float32), np.zeros((k, n), np.float32), np.zeros((n,), np.float32))
        return JaxprInterpreter(mj.make_jaxpr(layer)(*args), plan_only=True, **kw)
    interp = plan(49, 4608, 512)                                   #2 x 16 tiles, 36 k steps
    assert [l.kernel for l in interp.launches] == ['conv_gemm_32x32x128_ks4', 'ew_affine_v4']       #sum of four slices + bias, ReLU
    first, second = interp.launches
    assert first.grid == (32 * 4, 1, 1) and first.buffers[0][0].shape == (4, 49 * 512)
    assert np.frombuffer(first.params, np.int32)[-4 - 9] == 9      #k steps per slice: the fourth word from the end of ConvParams, which the 9 of ConvDerived follow
    assert second.buffers[0][0] is interp.output_buffers[0]
    assert len(plan(49, 4608, 512, fuse=False).launches) == 4      #slices, their sum, add, max
    assert [l.kernel for l in plan(49, 640, 512).launches] == ['conv_gemm_32x32x128_ks4']        #5 k steps: too short to slice
    assert [l.kernel for l in plan(49, 1024, 512).launches][0] == 'conv_gemm_32x32x128_ks4' and plan(49, 1024, 512).launches[0].grid == (64, 1, 1)
    assert len(plan(2048, 4608, 512).launches) == 1                #1024 tiles
    with K.overrides(conv_k_splits=3):
        forced = plan(40, 1000, 24)                                #8 k steps in 3 slices of 3, 3 and 2
    assert forced.launches[0].grid == (2 * 3, 1, 1) and forced.launches[0].buffers[0][0].shape == (3, 40 * 24)


def test_size_limits_are_reported_when_the_program_is_built():
    '''Kernels address an array through a 32-bit byte offset: an element-wise operand has to stay below 4 GiB and
    a convolution operand below 2 GiB. Larger ones are refused with NotImplementedError while the program is
    planned (nothing is allocated or launched); the largest allowed sizes plan.'''
    import vkjax_amd
    from vkjax_amd import minijax as mj
    def plan(f, *args):
        fn = vkjax_amd.wrap(f, frontend='minijax', plan_only=True)
        return fn._get_or_create_jaxpr_interpreter(args)[0]
    huge = lambda *shape: np.broadcast_to(np.float32(1), shape)            #no memory behind it
    interp = plan(lambda x: x * 2.0, huge((1 << 30) - 4))
    assert [l.kernel for l in interp.launches] == ['ew_chain_v4_s2'] and interp.launches[0].grid[0] == (1 << 20)
    with pytest.raises(NotImplementedError):
        plan(lambda x: x * 2.0, huge(1 << 30))
    with pytest.raises(NotImplementedError):
        plan(lambda x, w: mj.numpy.dot(x, w), huge(1 << 20, 512), huge(512, 8))       #2 GiB lhs
    interp = plan(lambda x, w: mj.numpy.dot(x, w), huge((1 << 20) - 64, 511), huge(511, 8))
    assert interp.launches[0].kernel.startswith('conv_gemm')


def test_softmax_plan_keeps_every_result_of_the_fused_launch():
    '''softmax over rows with the arg-max of the probabilities plans as ONE launch with three buffers (probabilities,
    input, labels), also when only the labels are returned: the launch is alive through its second result.'''
    from vkjax_amd import minijax as mj
    from vkjax_amd.jaxpr_interpreter import JaxprInterpreter
    def both(x):
        p = mj.nn.softmax(x, axis=-1)
        return p, mj.numpy.argmax(p, axis=1)
    def labels_only(x):
        return mj.numpy.argmax(mj.nn.softmax(x, axis=-1), axis=1)
    x = np.zeros((33, 64), np.float32)
    for f in (both, labels_only):
        interp = JaxprInterpreter(mj.make_jaxpr(f)(x), plan_only=True)
        assert [l.kernel for l in interp.launches] == ['softmax_rows_v4']
        buffers = [b for b, _ in interp.launches[0].buffers]
        assert len(buffers) == 3 and all(b is not None and b.tensor is not None for b in buffers)
        assert buffers[2] is interp.output_buffers[-1] and buffers[2].dtype == 'int32'
    #softmax alone: the labels argument is absent
    interp = JaxprInterpreter(mj.make_jaxpr(lambda v: mj.nn.softmax(v, axis=-1))(x), plan_only=True)
    assert [l.kernel for l in interp.launches] == ['softmax_rows_v4'] and interp.launches[0].buffers[2][0] is None


def test_repeated_equations_are_evaluated_once():
    '''An element-wise or shape equation with the primitive, parameters and operands of an earlier one is bound to that
    equation's buffer: indexing and scatter-add through the same index array normalise it once (two launches less),
    literals of different value or dtype are told apart, and results of the program keep equations of their own.'''
    import vkjax_amd
    from vkjax_amd import minijax as mj, ops, workloads as W
    from vkjax_amd.jaxpr_interpreter import JaxprInterpreter
    fn, make = W.WORKLOADS['gather_scatter']
    closed = mj.make_jaxpr(fn)(*make())
    kernels = lambda **kw: [l.kernel for l in JaxprInterpreter(closed, plan_only=True, **kw).launches]
    assert len(kernels()) == 3 and len(kernels(fuse=False)) == 6          #(fused: the gather and the scatter-add read the indices as they are and add n to the negative ones)
    from vkjax_amd import kernels as K
    with K.overrides(reuse_equal_equations=False):
        assert len(kernels()) == 3 and len(kernels(fuse=False)) == 9
    with pytest.raises(TypeError, match='unknown choice'):
        with K.overrides(no_such_choice=1):
            pass
    assert K.CHOICES.reuse_equal_equations is True
    def f(x):
        a = (x + 1.0) * (x + 1.0)          #x + 1 once
        b = (x + 2.0) * (x + np.float32(1.0))
        return a + b, x + 1.0              #the result x + 1 is an equation of its own
    x = np.zeros((8, 4), np.float32)
    interp = JaxprInterpreter(mj.make_jaxpr(f)(x), plan_only=True, fuse=False)
    names = [str(op.equation.primitive) for op in interp.all_ops]
    assert names.count('add') == 4 and names.count('mul') == 2, names          #x+1, x+2, a+b, the result x+1


def test_equal_equations_are_told_by_their_operands_storage_not_by_a_number():
    '''The table of earlier equations is keyed by the id() of the operands' storage cells. An id can pass to another
    object once its owner is gone, so an entry holds the cells themselves and a later equation is bound to the
    earlier one's result only if its operands' cells ARE those objects: an entry whose key matches but whose cells
    are other objects is replaced, not used.'''
    from vkjax_amd import minijax as mj, ops
    closed = mj.make_jaxpr(lambda x: ((x + 1.0) * (x + 1.0) * (x + 1.0)).sum())(np.zeros((8, 4), np.float32))
    jaxpr = closed.jaxpr
    adds = [eq for eq in jaxpr.eqns if eq.primitive.name == 'add']
    assert len(adds) == 3
    pool = BufferPool(PlanOnlyDevice())
    pool.get_buffer(jaxpr.invars[0])                                       #the argument has storage, as in a build
    assert ops._reuse_equal_equation(pool, adds[0]) is False               #noted
    (key, (outvar, cells)), = pool._equal_equations.items()
    assert len(cells) == 1 and key[2][0][0] == id(cells[0])
    assert ops._reuse_equal_equation(pool, adds[1]) is True                #same operand cell: bound to the first
    #the same key with a stranger in the cell's place, as after a recycled id
    class Cell:
        pass
    pool._equal_equations[key] = (outvar, [Cell()])
    assert ops._reuse_equal_equation(pool, adds[2]) is False
    assert pool._equal_equations[key][1][0] is cells[0]                    #the entry now describes the live operand


# ------------------------------------------------------------------ boundary details

def test_reference_module_path_resolves():
    '''The reference's own tests import the class as vkjax.kompute_jaxpr_interpreter.JaxprInterpreter
    (reference: tests/common.py:7, vkjax/function.py:1).'''
    import vkjax_amd as vkjax
    assert vkjax.kompute_jaxpr_interpreter.JaxprInterpreter is JaxprInterpreter
    from vkjax_amd.kompute_jaxpr_interpreter import JaxprInterpreter as by_import
    assert by_import is JaxprInterpreter


def test_no_temporary_shares_storage_with_a_program_output():
    '''A result that is a view of an intermediate keeps that intermediate's storage to the end of the
    program, also when launches were fused, moved or batched after the access positions were noted.'''
    from vkjax_amd import workloads as W

    def views_of_late_intermediates(x, idx, upd):
        a = jnp.tanh(x) * 2.0
        table = jnp.index_add(jnp.zeros((64, 8), np.float32), idx, upd)        #several launches for one equation
        b = (a + 1.0).reshape(16, 4)                                     #output = view of an intermediate
        c = jnp.sum(table, axis=0)
        d = (jnp.exp(a) - c.sum()).reshape(4, 16)
        return b, d, table.reshape(8, 64)

    rng  = np.random.default_rng(0)
    args = (rng.standard_normal((8, 8)).astype(np.float32), rng.integers(0, 64, (32,)).astype(np.int32),
            rng.standard_normal((32, 8)).astype(np.float32))
    programs = [(views_of_late_intermediates, args), (W.mlp_train_step, W.mlp_train_inputs(batch=8)),
                (W.convnet_train_step, W.convnet_train_inputs(batch=2))]
    for f, a in programs:
        for fuse in (True, False):
            closed = mj.make_jaxpr(f)(*a)
            interp = JaxprInterpreter(closed, fuse=fuse, plan_only=True)
            #storage of an output -> position of the first launch that touches it
            outputs = {id(b.tensor): min(b.accesses) for b in interp.output_buffers if b is not None}
            out_placeholders = {id(b._placeholder) for b in interp.output_buffers if b is not None}
            for key, b in interp.bufferpool.buffers.items():
                if b is None or b.tensor is None or id(b._placeholder) in out_placeholders or id(b.tensor) not in outputs:
                    continue
                #only something that is dead before the output is first written may have used its storage
                assert max(b.accesses) < outputs[id(b.tensor)], f'{f.__name__} fuse={fuse}: {key} shares storage with a live output'
            for b in interp.output_buffers:
                assert b is None or max(b.accesses) == np.inf


def test_index_modes():
    '''gather clamps and scatter-add drops by default (XLA); jax's other modes are planned with the matching kernel
    flag (a fill word for gather, clipping for scatter-add), and a mode nobody knows must not be ignored.'''
    x, idx, upd = np.zeros((8, 4), np.float32), np.zeros((3, 1), np.int32), np.zeros((3, 4), np.float32)
    dn = lax.GatherDimensionNumbers(offset_dims=(1,), collapsed_slice_dims=(0,), start_index_map=(0,))
    for mode, fill in (('clip', None), ('promise_in_bounds', None), (None, None), ('fill', 0x7FC00000), ('FILL_OR_DROP', 0x7FC00000)):
        closed = mj.make_jaxpr(lambda x, i: lax.gather(x, i, dn, (1, 4), mode=mode))(x, idx)
        (launch,) = JaxprInterpreter(closed, plan_only=True).launches
        assert np.frombuffer(launch.params, np.uint32)[-3:].tolist() == [int(fill is not None), fill or 0, 0], mode       #(fill flag, fill word, wrap)
    closed = mj.make_jaxpr(lambda x, i: lax.gather(x.astype(np.int32), i, dn, (1, 4), mode='fill', fill_value=-7))(x, idx)
    assert np.frombuffer(JaxprInterpreter(closed, plan_only=True).launches[-1].params, np.int32)[-3:].tolist() == [1, -7, 0]
    sd = lax.ScatterDimensionNumbers(update_window_dims=(1,), inserted_window_dims=(0,), scatter_dims_to_operand_dims=(0,))
    for mode, clip in (('clip', 1), ('drop', 0), (None, 0), ('promise_in_bounds', 0)):
        closed = mj.make_jaxpr(lambda x, i, u: lax.scatter_add(x, i, u, sd, mode=mode))(x, idx, upd)
        launch = JaxprInterpreter(closed, plan_only=True, fuse=False).launches[-1]
        assert launch.kernel == 'scatter_add_rows' and np.frombuffer(launch.params, np.uint32)[-1] == clip, mode
    for f, args in ((lambda x, i: lax.gather(x, i, dn, (1, 4), mode='one_hot'), (x, idx)),
                    (lambda x, i, u: lax.scatter_add(x, i, u, sd, mode='wrap'), (x, idx, upd))):
        with pytest.raises(NotImplementedError, match='mode'):
            JaxprInterpreter(mj.make_jaxpr(f)(*args), plan_only=True)


def test_evenly_split_conv_grids():
    '''Layers with at least 4.5 tiles per resident block get a grid of exactly 5 blocks per CU whose blocks share the
    M tiles of every N tile evenly; smaller ones keep one block per run of `chunk` tiles.'''
    from vkjax_amd import kernels as K
    assert K.choose_conv_m_blocks(784, 8) == 160            #ResNet-50 bs64, 28 x 28 x 512 outputs: 6272 tiles, 4.9 per block
    assert K.choose_conv_m_blocks(3136, 2) == 640
    assert K.choose_conv_m_blocks(3136, 1) == 0             #2.45 tiles per block: one more or less would unbalance the CUs
    assert K.choose_conv_m_blocks(10, 1) == 0
    assert K.choose_conv_m_blocks(100000, 1) == 1280 and K.choose_conv_m_blocks(4, 4000) == 1
    geom = K.ConvGeometry(batch=64, Ho=28, Wo=28, N=512, H=28, W=28, Cin=128, KH=1, KW=1, xs=(100352, 3584, 128, 1), ws=(65536, 65536, 512, 1), os=(401408, 14336, 512, 1))
    b = lambda *shape: Buffer(None, np.float32, shape)
    launch = K.conv_gemm(b(64, 28, 28, 512), b(64, 28, 28, 128), b(1, 1, 128, 512), geom)
    assert launch.kernel == 'conv_gemm_64x64x32_lean' and launch.grid[0] == 1280
    assert np.frombuffer(launch.params, np.int32)[-3 - 9:-9].tolist() == [160, 4, 144]   #blocks per N tile, tiles each, blocks with one more: the end of ConvParams, before the 9 of ConvDerived


def test_which_argument_leaves_count_as_immutable():
    '''Leaves that stay in HBM without being asked: only arrays nobody can write through.'''
    from vkjax_amd.jaxpr_interpreter import _is_immutable, _may_change_in_place
    a = np.arange(12, dtype=np.float32)
    assert not _is_immutable(a) and _may_change_in_place(a)
    view = a[2:8]
    view.flags.writeable = False
    assert not _is_immutable(view)                       #a window into a writeable array
    b = a.copy()
    b.flags.writeable = False
    assert _is_immutable(b) and _is_immutable(b[1:5]) and not _may_change_in_place(b)
    assert _is_immutable(np.frombuffer(b'\x00' * 16, np.float32))         #backed by a bytes object
    assert not _is_immutable(np.frombuffer(bytearray(16), np.float32))
    assert not _is_immutable(3.0) and not _is_immutable(np.float32(3.0)) and not _may_change_in_place(3.0)


def test_large_results_that_nothing_reads_again_are_stored_past_the_caches():
    '''Kernels that can store their result with the nontemporal hint are told to (bit 31 of their first parameter word)
    for results of 64 MB and more that no later launch of the program reads; a result that a later launch reads, a small
    one, and a kernel without that ability are left alone; a later launch that only writes the array (the second part
    of a concatenation) does not count as a reader.'''
    from vkjax_amd import kernels as K
    streamed = lambda interp: [(l.kernel, int(np.frombuffer(l.params[:4], np.uint32)[0]) >> 31) for l in interp.launches]
    big, small = np.zeros(1 << 24, np.float32), np.zeros(1 << 20, np.float32)
    plan = lambda f, *args: JaxprInterpreter(mj.make_jaxpr(f)(*args), plan_only=True)
    assert streamed(plan(lambda x: jnp.exp(x), big)) == [('ew_chain_v4_s2', 1)]
    assert streamed(plan(lambda x: jnp.exp(x), small)) == [('ew_chain_v4_s2', 0)]
    #the exponential is read by the sum: only a launch whose result leaves the program streams it
    assert streamed(plan(lambda x: jnp.sum(jnp.exp(x).reshape(4096, 4096), axis=0), big)) [0][1] == 0
    both = streamed(plan(lambda x: (jnp.exp(x), jnp.exp(x).reshape(4096, 4096).T), big))
    #(the result exp(x) keeps a launch of its own: streamed; the one the transposition reads is not; the transposed result is)
    assert [flag for _, flag in both] == [1, 0, 1] and both[2][0].startswith('transpose_tiled')
    assert streamed(plan(lambda x, y: lax.concatenate([x, y], 0), big, big)) == [('concat_part_v4', 1), ('concat_part_v4', 1)]
    for launch in plan(lambda x: jnp.exp(x), big).launches:
        assert launch.streamable and K.with_streamed_result(launch._replace(params=K._u32(launch.params and 5) + launch.params[4:])).params[:4] == K._u32(5 | 1 << 31)


def test_stream_in_flight_hands_out_results_in_order_whatever_the_lanes_do():
    '''Function.stream(in_flight=n) without a device: stand-in lanes that take their tuples at different speeds. Results
    come back in the order of the tuples; the iterable is never asked for a tuple while a lane has not finished copying
    the one before (the loader may refill its arrays); at most 4 n tuples are under way; an error raised by the
    iterable or by a lane reaches the consumer; a consumer that stops early leaves no thread behind.'''
    import threading, time
    import vkjax_amd

    class Lane:
        def __init__(self, delay, fail_at=None):
            self.delay, self.fail_at, self.taken_while_copying = delay, fail_at, 0
        def _stream_one(self, tuples, taken=None):
            for (value,) in tuples:
                state['copying'] += 1
                time.sleep(0.0005)                      #"copies" what the loader may refill
                state['overlapping_copies'] += state['copying'] > 1
                state['copying'] -= 1
                taken()
                if value == self.fail_at:
                    raise ValueError(f'lane failed at {value}')
                time.sleep(self.delay * (1 + value % 3))
                state['under_way'] = max(state['under_way'], state['taken'] - state['yielded'])
                yield value * 10

    def source(n, fail_at=None):
        for k in range(n):
            assert state['copying'] == 0, 'the iterable was asked for a tuple while a lane was still copying the one before'
            if k == fail_at:
                raise KeyError('no such batch')
            state['taken'] += 1
            yield (k,)

    def run(lanes, n, **kw):
        f = vkjax_amd.wrap(lambda x: x, frontend='minijax')
        f._in_flight_lanes = lanes
        return f.stream(source(n, **kw), in_flight=len(lanes))

    for delays in ((0.001, 0.004), (0.003, 0.0, 0.002)):
        state = dict(copying=0, overlapping_copies=0, under_way=0, taken=0, yielded=0)
        got = []
        for y in run([Lane(d) for d in delays], 40):
            got.append(y)
            state['yielded'] += 1
        assert got == [10 * k for k in range(40)]
        assert state['overlapping_copies'] == 0 and state['under_way'] <= 4 * len(delays) + 1, state
    lane_threads = lambda: [t for t in threading.enumerate() if t.name.startswith('vkjax-stream-lane')]
    assert not lane_threads()
    #errors: of the iterable, of a lane
    state = dict(copying=0, overlapping_copies=0, under_way=0, taken=0, yielded=0)
    with pytest.raises(KeyError, match='no such batch'):
        list(run([Lane(0.001), Lane(0.002)], 20, fail_at=7))
    assert not lane_threads()
    state = dict(copying=0, overlapping_copies=0, under_way=0, taken=0, yielded=0)
    with pytest.raises(ValueError, match='lane failed at 5'):
        list(run([Lane(0.001, fail_at=5), Lane(0.001, fail_at=5)], 20))
    assert not lane_threads()
    #a consumer that stops early
    state = dict(copying=0, overlapping_copies=0, under_way=0, taken=0, yielded=0)
    it = run([Lane(0.001), Lane(0.001)], 1000)
    assert [next(it) for _ in range(5)] == [0, 10, 20, 30, 40]
    it.close()
    assert not lane_threads() and state['taken'] < 40
