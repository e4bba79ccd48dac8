'''Reductions on the GPU against the numpy oracle: both kernels (contiguous rows, strided columns),
16-byte and 4-byte loads, reductions split into ranges with a second launch, index-returning
reductions with ties and NaNs. Integer-valued data keeps float sums exact, so every case is
compared bit for bit.'''
import numpy as np
import pytest

from vkjax_amd import minijax as mj
from tests.common import check_against_oracle

pytestmark = pytest.mark.gpu
jnp = mj.numpy
rng = np.random.RandomState(99)


def ints(shape, lo=-2, hi=3, dtype=np.float32):
    return rng.randint(lo, hi, size=shape).astype(dtype)


CASES = [
    #(shape, axes, expected kernel prefix, expected number of launches)
    ((3, 100003), (1,), 'reduce_rows', 2), ((2, 1 << 20), (1,), 'reduce_rows', 2), ((65, 1000), (1,), 'reduce_rows', 1),
    ((70000, 7), (1,), 'reduce_rows', 1), ((100000, 12), (0,), 'reduce_cols', 2), ((99999, 13), (0,), 'reduce_cols', 2),
    ((16, 5000, 24), (1,), 'reduce_cols', 2), ((1 << 22,), (0,), 'reduce_rows', 2), ((5, 7, 9, 64), (1, 2), 'reduce_cols', 1),
    ((64, 7, 7, 2048), (1, 2), 'reduce_cols', 1), ((300, 300), (0, 1), 'reduce_rows', 2),
]


@pytest.mark.parametrize('shape,axes,kernel,launches', CASES)
def test_sum_max_min_exact(shape, axes, kernel, launches):
    x = ints(shape)
    for name, f in (('sum', lambda x: jnp.sum(x, axis=axes)), ('max', lambda x: jnp.max(x, axis=axes)), ('min', lambda x: jnp.min(x, axis=axes))):
        print(f'{name} {shape} axes {axes}', flush=True)
        _, _, fn = check_against_oracle(f, [x], exact=True)
        kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
        assert all(k.startswith(kernel) for k in kernels) and len(kernels) == launches, kernels


def test_integer_and_product_reductions():
    check_against_oracle(lambda x: jnp.sum(x, axis=0), [ints((50000, 6), -1000, 1000, np.int32)], exact=True)
    check_against_oracle(lambda x: jnp.max(x, axis=1), [ints((9, 70001), -10**9, 10**9, np.int32)], exact=True)
    check_against_oracle(lambda x: jnp.min(x, axis=0), [rng.randint(0, 2**31, size=(40000, 3)).astype(np.uint32)], exact=True)
    x = np.ones((4, 30000), np.float32)
    x[:, ::1000] = 2.0                                      #products of powers of two are exact
    check_against_oracle(lambda x: jnp.prod(x, axis=1), [x], exact=True)


@pytest.mark.parametrize('shape,axis', [((7, 100001), 1), ((65536 + 3, 10), 1), ((50001, 9), 0), ((4, 3000, 8), 1)])
def test_argmax_argmin_ties_and_nans(shape, axis):
    x = ints(shape, -3, 4)                                   #many ties: the first occurrence must win
    check_against_oracle(lambda x: jnp.argmax(x, axis=axis), [x], exact=True)
    check_against_oracle(lambda x: jnp.argmin(x, axis=axis), [x], exact=True)
    x = rng.random_sample(shape).astype(np.float32)
    x[tuple(rng.randint(0, s, size=20) for s in shape)] = np.nan      #a NaN beats every number
    check_against_oracle(lambda x: jnp.argmax(x, axis=axis), [x], exact=True)
    check_against_oracle(lambda x: jnp.max(x, axis=axis), [x], exact=True)


@pytest.mark.parametrize('width', [1000, 1003, 64, 257])
def test_argmax_argmin_treat_signed_zeros_as_equal(width):
    '''-0.0 and +0.0 compare equal, so the first of them wins whatever its sign, also when the two sit in different
    lanes of the wave that reduces the row (numpy and XLA agree; widths divisible by 4 take the 16-byte kernel).'''
    x = np.full((6, width), -5.0, np.float32)
    x[0, 3], x[0, 200 % width] = -0.0, 0.0             #maximum: -0.0 first, +0.0 later in another lane
    x[1, 5], x[1, width - 1] = 0.0, -0.0
    x[2, 70 % width], x[2, 7] = -0.0, 0.0               #+0.0 first
    y = -x                                              #minimum: rows of +5 with zeros of either sign
    y[3:] = 0.0
    y[3, 1::2] = -0.0                                   #a whole row of zeros of alternating sign: index 0
    y[4, 0], y[5, :] = -0.0, -0.0
    x[3:] = y[3:]
    for a in (x, y):
        check_against_oracle(lambda a: jnp.argmax(a, axis=1), [a], exact=True)
        check_against_oracle(lambda a: jnp.argmin(a, axis=1), [a], exact=True)
        check_against_oracle(lambda a: jnp.argmax(a, axis=0), [a], exact=True)     #the column kernel
        check_against_oracle(lambda a: jnp.argmin(a, axis=0), [a], exact=True)
    #the arg-max that a softmax launch returns with its probabilities (all of them positive: same labels as numpy)
    check_against_oracle(lambda a: jnp.argmax(mj.nn.softmax(a, axis=-1), axis=-1), [x], exact=True)


def test_float_sum_within_tolerance():
    x = rng.random_sample((3, 1 << 21)).astype(np.float32)
    check_against_oracle(lambda x: jnp.sum(x, axis=1), [x], rtol=1e-5, atol=0)
    x = rng.random_sample((1 << 18, 24)).astype(np.float32)
    check_against_oracle(lambda x: jnp.sum(x, axis=0), [x], rtol=1e-5, atol=0)


def test_column_sums_take_over_their_operands_multiply_or_negate():
    '''sum(a * b), sum(a * per-column vector), sum(-a) over the leading dimensions: one launch family
    `reduce_cols_fsum_{mul,mulv,neg}` instead of an element-wise pass plus a reduction; same values as unfused.'''
    import vkjax_amd
    a, b, v = ints((6, 33, 17, 64)), ints((6, 33, 17, 64)), ints((64,))
    cases = [('mul', lambda a, b, v: jnp.sum(a * b, axis=(0, 1, 2))), ('mulv', lambda a, b, v: jnp.sum(a * v, axis=(0, 1, 2))),
             ('neg', lambda a, b, v: jnp.sum(-a, axis=(0, 1))), ('mul', lambda a, b, v: jnp.sum(a.reshape(-1, 64) * b.reshape(-1, 64), axis=0))]
    for kind, f in cases:
        print(f'prologue {kind}', flush=True)
        y, _, fn = check_against_oracle(f, [a, b, v], exact=True)
        kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
        assert kernels[0].startswith(f'reduce_cols_fsum_{kind}_v') and not any(k.startswith('ew_chain') for k in kernels), kernels
    #random floats: bit-identical to the unfused program
    x, y = rng.random_sample((5000, 96)).astype(np.float32), rng.random_sample((5000, 96)).astype(np.float32)
    f = lambda x, y: jnp.sum(x * y, axis=0)
    fused   = vkjax_amd.wrap(f, frontend='minijax')(x, y)
    unfused = vkjax_amd.wrap(f, frontend='minijax', fuse=False)(x, y)
    assert np.array_equal(fused, unfused)


@pytest.mark.parametrize('shape', [(256, 10), (64, 1000), (33, 7), (5, 64), (5, 65), (3, 4092), (2, 3, 50)])
def test_fused_softmax_equals_the_separate_launches(shape):
    '''jax.nn.softmax's reduce_max / subtract / exp / reduce_sum / divide as one launch: same bits as the five.'''
    import vkjax_amd
    x = (rng.random_sample(shape) * 12 - 6).astype(np.float32)
    f = lambda x: mj.nn.softmax(x, axis=-1)
    print(f'softmax {shape}', flush=True)
    y, _, fn = check_against_oracle(f, [x], rtol=1e-5, atol=1e-7)
    kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
    assert len(kernels) == 1 and kernels[0].startswith('softmax_rows'), kernels
    unfused = vkjax_amd.wrap(f, frontend='minijax', fuse=False)(x)
    assert np.array_equal(y, unfused)
    assert np.allclose(y.sum(axis=-1), 1.0, atol=1e-5)


def test_means_store_the_quotient_from_the_summing_launch():
    '''sum / c and sum * c with a single value c behind an unsplit float sum (a mean over rows, over columns, over
    the spatial positions of an activation) are one launch, reduce_{rows,cols}_fsum_{div,times}; the values are those
    of the two launches, bit for bit, and of the oracle within the tolerance of a float sum.'''
    import vkjax_amd
    x3 = rng.random_sample((6, 7, 7, 64)).astype(np.float32)
    x2 = rng.random_sample((300, 1000)).astype(np.float32)
    cases = [('global average', lambda x: jnp.mean(x, axis=(1, 2)), [x3], 'reduce_cols_fsum_div_v4'),
             ('mean over rows', lambda x: jnp.mean(x, axis=1), [x2], 'reduce_rows_fsum_div_v4'),
             ('mean over columns', lambda x: jnp.mean(x, axis=0), [x2[:64, :96]], 'reduce_cols_fsum_div_v4'),
             ('odd width', lambda x: jnp.mean(x, axis=1), [x2[:, :999].copy()], 'reduce_rows_fsum_div_v1'),
             ('sum times a value', lambda x, c: jnp.sum(x, axis=0) * c, [x2[:64, :96], np.float32(0.125)], 'reduce_cols_fsum_times_v4'),
             ('a value times the sum', lambda x, c: c * jnp.sum(x, axis=1), [x2, np.float32(3.0)], 'reduce_rows_fsum_times_v4'),
             ('sum divided by an argument', lambda x, c: jnp.sum(x, axis=1) / c, [x2, np.float32(7.0)], 'reduce_rows_fsum_div_v4')]
    for name, f, args, kernel in cases:
        print(f'case: {name}', flush=True)
        y, _, fn = check_against_oracle(f, args, rtol=1e-5, atol=0)
        kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
        assert kernels == [kernel], kernels
        unfused = vkjax_amd.wrap(f, frontend='minijax', fuse=False)
        assert np.array_equal(y, unfused(*args))
        assert len(list(unfused._jaxpr_interpreters.values())[0].launches) == 2
    #not taken over: a value divided by the sum, a sum that something else reads as well, a sum split into ranges
    for name, f, args, launches in [('c / sum', lambda x, c: c / jnp.sum(x, axis=1), [x2, np.float32(7.0)], 2),
                                    ('two readers', lambda x: (jnp.sum(x, axis=1) / 3.0, jnp.sum(x, axis=1) + 1.0), [x2], 3),
                                    ('split sum', lambda x: jnp.mean(x, axis=1), [rng.random_sample((2, 1 << 18)).astype(np.float32)], 3)]:
        print(f'case: {name}', flush=True)
        _, _, fn = check_against_oracle(f, args, rtol=1e-5, atol=0)
        assert len(list(fn._jaxpr_interpreters.values())[0].launches) == launches
