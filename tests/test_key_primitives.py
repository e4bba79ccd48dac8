'''The key primitives newer jax versions trace for jax.random (random_seed / random_wrap /
random_bits / random_split / random_fold_in / random_unwrap): oracle pins and launch plans on
the CPU, parity of the HIP path on the GPU. Both counter layouts of jax are covered.'''
import json
import os

import numpy as np
import pytest

from oracle import primitives as P
from oracle.eval_jaxpr import eval_closed_jaxpr
from tests.common import check_against_oracle
from vkjax_amd import minijax as mj, ops
from vkjax_amd.jaxpr_interpreter import JaxprInterpreter

lax, jnp, mrandom = mj.lax, mj.numpy, mj.random


@pytest.fixture(params=[False, True], ids=['original', 'partitionable'])
def layout(request):
    '''Sets the counter layout on the device path and in the oracle, and makes the stand-in tracer
    emit key primitives instead of expanding them.'''
    previous = ops.THREEFRY_PARTITIONABLE, P.THREEFRY_PARTITIONABLE, mrandom.key_primitives(True)
    ops.THREEFRY_PARTITIONABLE = P.THREEFRY_PARTITIONABLE = request.param
    yield request.param
    ops.THREEFRY_PARTITIONABLE, P.THREEFRY_PARTITIONABLE = previous[:2]
    mrandom.key_primitives(previous[2])


def uniform_of_raw_key(key):          return mrandom.uniform(key, (33, 65))
def uniform_scalar(key):              return mrandom.uniform(key, ())
def bits_odd(key):                    return mrandom.random_bits(key, (77,))
def bits_one(key):                    return mrandom.random_bits(key, (1,))
def split_then_uniform(key):
    k1, k2 = mrandom.split(key)
    return mrandom.uniform(k2, (128, 64), minval=-2.0, maxval=3.0), k1
def split_many(key):                  return mrandom.split(key, 7)
def fold_in_then_bits(key, step):     return mrandom.random_bits(mrandom.fold_in(key, step), (5, 3))
def typed_flow(seed):
    key = mrandom.key(seed)
    k1, k2 = mrandom.split(key)
    return mrandom.uniform(mrandom.fold_in(k1, 3), (16,)), mrandom.key_data(k2), mrandom.key_data(key)
def typed_key_array_slices(seed):
    keys = mrandom.split(mrandom.key(seed), 4)
    return mrandom.random_bits(keys[2], (6,)), mrandom.key_data(keys)

KEY = np.array([0x13198a2e, 0x03707344], np.uint32)
CASES = [
    (uniform_of_raw_key, [KEY]), (uniform_scalar, [KEY]), (bits_odd, [KEY]), (bits_one, [KEY]),
    (split_then_uniform, [KEY]), (split_many, [KEY]), (fold_in_then_bits, [KEY, np.uint32(77)]),
    (typed_flow, [np.int32(-5)]), (typed_key_array_slices, [np.int32(1234)]),
]


# ------------------------------------------------------------------ CPU: oracle pins and plans

def test_key_primitives_are_traced_not_expanded(layout):
    closed = mj.make_jaxpr(split_then_uniform)(KEY)
    names = [e.primitive.name for e in closed.jaxpr.eqns]
    assert 'random_bits' in names and 'random_split' in names and 'threefry2x32' not in names


def test_oracle_original_layout_equals_the_expanded_pipeline():
    '''The expansion jax's original layout performs while tracing (pinned against published jax
    values elsewhere) and the key primitives give the same words.'''
    P.THREEFRY_PARTITIONABLE = False
    for f, args in CASES[:7]:
        expanded = eval_closed_jaxpr(mj.make_jaxpr(f)(*args), *args)
        previous = mrandom.key_primitives(True)
        try:
            closed = mj.make_jaxpr(f)(*args)
        finally:
            mrandom.key_primitives(previous)
        assert any(e.primitive.name.startswith('random_') for e in closed.jaxpr.eqns)
        for a, b in zip(eval_closed_jaxpr(closed, *args), expanded):
            assert np.array_equal(a, b), f.__name__


def test_oracle_partitionable_layout_matches_documented_jax_values():
    '''jax's documentation (jax.random, with the partitionable layout that is its default) prints
    uniform(key(0)) = 0.947667 and, after `key, subkey = split(key)`, uniform(subkey) = 0.00729382.'''
    P.THREEFRY_PARTITIONABLE = True
    try:
        key0 = P.random_seed(np.int32(0))
        assert key0.tolist() == [0, 0]
        published = json.load(open(os.path.join(os.path.dirname(__file__), 'golden', 'known_answers.json')))['jax_random_partitionable_key0']
        bits = P.random_bits(key0, 32, ())
        assert np.float32((int(bits) >> 9) * 2.0**-23) == np.float32(published['uniform'])
        subkey = P.random_split(key0, (2,))[1]
        bits = P.random_bits(subkey, 32, ())
        assert abs(np.float32((int(bits) >> 9) * 2.0**-23) - np.float32(published['uniform_of_second_subkey'])) < 5e-9
        #closed form: element i of a draw is the xor of the block function's words on the counter (0, i)
        draw = P.random_bits(KEY, 32, (3, 5))
        for i in range(15):
            a, b = P.threefry2x32(KEY[0], KEY[1], np.zeros(1, np.uint32), np.array([i], np.uint32))
            assert draw.reshape(-1)[i] == a[0] ^ b[0]
    finally:
        P.THREEFRY_PARTITIONABLE = False


def test_fold_in_and_seed_closed_forms():
    assert P.random_seed(np.int32(-5)).tolist() == [0, 0xFFFFFFFB]
    a, b = P.threefry2x32(KEY[0], KEY[1], np.zeros(1, np.uint32), np.array([77], np.uint32))
    assert P.random_fold_in(KEY, np.uint32(77)).tolist() == [a[0], b[0]]


@pytest.mark.parametrize('f,args', CASES, ids=[c[0].__name__ for c in CASES])
def test_plans(layout, f, args):
    closed = mj.make_jaxpr(f)(*args)
    interp = JaxprInterpreter(closed, plan_only=True)
    kernels = [l.kernel for l in interp.launches]
    if f in (uniform_of_raw_key, uniform_scalar, bits_odd, bits_one):
        #one launch: the counters are generated in registers and the uniform chain is applied before the store
        assert len(kernels) == 1 and kernels[0].startswith('threefry2x32_stream_xor' if layout else 'threefry2x32_stream_v'), kernels
    if f is split_many:
        assert kernels == ['threefry2x32_stream_pairs_v1' if layout else 'threefry2x32_stream_v1']


def test_unsupported_forms_raise():
    def batched(key): return lax.random_bits(lax.random_split(lax.random_wrap(key), (3,)), 32, (4,))
    with pytest.raises(NotImplementedError):
        JaxprInterpreter(mj.make_jaxpr(batched)(KEY), plan_only=True)


# ------------------------------------------------------------------ GPU parity (bit-exact words)

@pytest.mark.gpu
@pytest.mark.parametrize('f,args', CASES, ids=[c[0].__name__ for c in CASES])
def test_hip_matches_oracle(layout, f, args):
    print(f'case: {f.__name__} partitionable={layout}', flush=True)
    for fuse in (True, False):
        check_against_oracle(f, args, exact=True, fuse=fuse)


@pytest.mark.gpu
def test_normal_draw_hip(layout):
    '''uniform -> erf_inv -> * sqrt(2) folded into the generating kernel; tolerance of element-wise float work.'''
    def draw(key): return mrandom.normal(key, (257, 129))
    print(f'case: normal draw partitionable={layout}', flush=True)
    y, ytrue, fn = check_against_oracle(draw, [KEY], rtol=1e-5, atol=1e-6)
    assert abs(float(y.mean())) < 0.02 and abs(float(y.std()) - 1.0) < 0.02
    interp = next(iter(fn._jaxpr_interpreters.values()))
    assert len(interp.launches) <= 2, [l.kernel for l in interp.launches]      #the generating kernel and, at most, the tail of the chain


@pytest.mark.gpu
def test_large_draw_both_layouts(layout):
    def draw(key): return mrandom.uniform(key, (1024, 1027))
    print(f'case: large draw partitionable={layout}', flush=True)
    y, ytrue, _ = check_against_oracle(draw, [KEY], exact=True)
    assert 0.0 <= y.min() and y.max() < 1.0 and abs(float(y.mean()) - 0.5) < 1e-3
