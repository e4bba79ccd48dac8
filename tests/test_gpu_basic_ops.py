'''Per-primitive parity of the HIP path against the CPU oracle, on the case list of the
reference's own test matrix (reference: tests/test_basic_ops.py:162-333; same functions, same
shapes, same tolerances), with seeded inputs. Runs on the GPU box only.'''
import numpy as np
import pytest

from vkjax_amd import minijax as mj
from tests.common import check_against_oracle

jnp, lax = mj.numpy, mj.lax
pytestmark = pytest.mark.gpu
rng = np.random.RandomState(1234)
random, randint, uniform = rng.random_sample, rng.randint, rng.uniform


def add0(x): return x + x
def add1(x): return x + 1.0
def add2(x, y): return x + y
def add3(x, y): return mj.jit(add0)(x) + mj.jit(add2)(y, x)
def add4(x, y): return mj.jit(add0)(x) + mj.jit(add2)(y, 1.0)
def add00(): return lax.add(5, 100)
def div0(x, y): return x / y
def sub0(x, y): return x - y
def mul0(x, y): return x * y
def reshape1(x): return (x + 1).reshape(4, -1)
def broadcast0(x): return lax.broadcast_in_dim(x, shape=(4,), broadcast_dimensions=())
def broadcast1(x): return lax.broadcast_in_dim(x + 1, shape=(4, 1, 1), broadcast_dimensions=(0,))
def broadcast2(x): return lax.broadcast_in_dim(x, shape=x.shape + (32,), broadcast_dimensions=tuple(np.arange(len(x.shape))))
def broadcast3(x): return lax.broadcast_in_dim(x, shape=(32,) + x.shape, broadcast_dimensions=(1,))
def dot0(x, y): return jnp.dot(x, y)
dot1_const = random([100, 32]).astype(np.float64)
def dot1(x): return jnp.dot(x, dot1_const)
def dot_general0(x, y): return lax.dot_general(x, y, (((0,), (0,)), ((), ())))
def dot_general1(x, y): return lax.dot_general(x, y, (((1,), (1,)), ((), ())))
def dot_general2(x, y): return lax.dot_general(x, y, (((0,), (1,)), ((), ())))
def reshape_dot(x, y): return x.reshape(-1, 4) @ y
def relu0(x): return mj.nn.relu(x)
def reduce_max0(x): return jnp.max(x, axis=0)
def reduce_min0(x): return jnp.min(x, axis=0)
def reduce_max1(x): return jnp.max(x, axis=1)
def reduce_max2(x): return jnp.max(x, axis=[1, 2, 5])
def reduce_sum0(x): return jnp.sum(x, axis=0)
def reduce_sum1(x): return jnp.sum(x, axis=1)
def reduce_sum2(x): return jnp.sum(x, axis=[0, 1, 2])
def no_reduce1(x): return jnp.sum(x + 1, axis=())
def reduce_prod0(x): return jnp.prod(x, axis=0)
def argmax0(x): return jnp.argmax(x, axis=0)
def argmin0(x): return jnp.argmin(x, axis=0)
def gt0(x, y): return x > y
def ge0(x, y): return x >= y
def lt0(x, y): return x < y
def le0(x, y): return x <= y
def eq0(x, y): return x == y
def eq1(x): return x == x.max(axis=-1)
def ne0(x, y): return x != y
def or0(x, y): return x | y
def and0(x, y): return x & y
def exp0(x): return jnp.exp(x)
def log0(x): return jnp.log(x)
def abs0(x): return jnp.abs(x)
def rsqrt0(x): return lax.rsqrt(x)
def iota0(): return jnp.arange(32)
def select0(x, y, z): return jnp.where(x, y, z)
def concatenate0(x, y): return jnp.concatenate([x, y], axis=-1)
def gather0(x): return x[:, :, 4:7, :]
def gather1a(x): return x[5, :]
def gather1b(x): return x[:, 5]
def gather_fn0(x, i):
    return lax.gather(x, i, mj.core.GatherDimensionNumbers(offset_dims=(), collapsed_slice_dims=(0, 1), start_index_map=(0, 1)),
                      slice_sizes=(1, 1))
def take_along_axis0(x, i): return jnp.take_along_axis(x, i, axis=-1)
#gradient of take_along_axis: a scatter-add of single elements into zeros (the reference's point form)
def take_along_axis0_g(x, i): return mj.grad(lambda *args: take_along_axis0(*args).ravel().mean())(x, i)
def gather_fn1(x, i):
    return lax.gather(x, i, mj.core.GatherDimensionNumbers(offset_dims=(0,), collapsed_slice_dims=(1,), start_index_map=(1,)),
                      slice_sizes=(len(x), 1))
def scatter_fn0(x, i, u):
    return lax.scatter_add(x, i, u, mj.core.ScatterDimensionNumbers(update_window_dims=(), inserted_window_dims=(0, 1),
                                                                    scatter_dims_to_operand_dims=(0, 1)))
def scatter_add_fn1(x, i, u):
    return lax.scatter_add(x, i, u, mj.core.ScatterDimensionNumbers(update_window_dims=(0,), inserted_window_dims=(1,),
                                                                    scatter_dims_to_operand_dims=(1,)))
def add_any0(x, y): return lax.add_any(x, y), np.float32(1)
def transpose0(x): return x.T
def rev0(x): return lax.rev(x, dimensions=[1, 2])
def integer_pow0(x): return x ** 2
def integer_pow1(x): return x ** 5
def pow0(x, y): return lax.pow(x, y)
def slice0(x): return lax.slice(x, [2], [33])
def slice1(x): return lax.slice(x, [55, 5], [101, 10])
def slice2(x): return lax.slice(x, [55, 5], [101, 10], [2, 3])
def squeeze0(x): return jnp.squeeze(x)
def threefry0a(): return lax.threefry2x32(*np.ones(4, 'uint32'))
def threefry0b(): return lax.threefry2x32(*np.ones([4, 10], 'uint32'))
def threefry1(x): return lax.threefry2x32(*x)
def convert_element_type0(x): return x.astype(np.int32)
def convert_element_type1(x): return x.astype(np.float32)
def bitcast_convert_type0(x): return lax.bitcast_convert_type(x, 'float32')
def shift_right_logical_1_32(): return lax.shift_right_logical(1, 32)


param_matrix = [
    (add0, 'add x+x scalar',            [5.0]),
    (add0, 'add x+x array1d',           [random(32)]),
    (add0, 'add x+x array3d',           [random((32, 32, 32))]),
    (add00, '5+100',                    []),
    (add1, 'add x+1 scalar',            [5.0]),
    (add1, 'add x+1 array3d',           [random((32, 32, 32))]),
    (add2, 'add x+y scalar-scalar',     [5.0, 7.0]),
    (add2, 'add x+y scalar-array3d',    [5.0, random((32, 32, 32))]),
    (add2, 'add x+y array3d-array3d',   [random((32, 32, 32)), random((32, 32, 32))]),
    (add2, 'broadcast_add [2,32]+[32]', [random((2, 32)), random((32))]),
    (add2, 'add x+y int',               [randint(65, size=(32, 32, 32)), randint(77, size=(32, 32, 32))]),
    (add3, 'add nested (x+x)+(y+x)',    [5.0, 7.1]),
    (add4, 'nested const (x+x)+(y+1)',  [5.0, 7.1]),
    (div0, 'div0 x/y',                  [random([2, 32, 32, 3]), 255.0]),
    (sub0, 'sub0 x-y',                  [random([2, 32, 32, 3]), 255.0]),
    (sub0, 'sub0 (2,10)-(2,1)',         [random([2, 10]), random([2, 1])]),
    (mul0, 'mul0 x*y',                  [random([2, 32, 32, 3]), 255.0]),
    (reshape1, 'reshape1',              [random([2, 32, 32])]),
    (broadcast0, 'broadcast scalar',    [random()]),
    (broadcast1, 'broadcast 1D->3D',    [random(4)]),
    (broadcast2, 'broadcast append',    [random(4)]),
    (broadcast3, '(128)->(32,128)',     [random(128)]),
    (dot0, 'dot0 x@y',                  [random([2, 100]), random([100, 32])]),
    (dot1, 'dot1 x@const',              [random([2, 100])]),
    (dot_general0, 'dot axes=(0,0)',    [random([100, 2]), random([100, 32])]),
    (dot_general1, 'dot axes=(1,1)',    [random([2, 100]), random([32, 100])]),
    (dot_general2, 'dot axes=(0,1)',    [random([100, 2]), random([32, 100])]),
    (reshape_dot, 'reshape_dot',        [random([2, 77, 102]), random([4, 4])]),
    (relu0, 'relu0',                    [random([32, 32, 32]) - 0.5]),
    (lax.max, 'max_float32',            [random([77, 99, 200]), random([77, 99, 200])]),
    (lax.min, 'min_float32',            [random([77, 99, 200]), random([77, 99, 200])]),
    (lax.max, 'max_int32',              [randint(-1000, 1000, [77, 99, 200]), randint(-1000, 1000, [77, 99, 200])]),
    (lax.min, 'min_int32',              [randint(-1000, 1000, [77, 99, 200]), randint(-1000, 1000, [77, 99, 200])]),
    (reduce_max0, 'max(axis=0)',        [random([32, 32])]),
    (reduce_min0, 'min(axis=0)',        [random([77, 99])]),
    (reduce_max1, 'max(axis=1)',        [random([32, 32]) - 1.0]),
    (reduce_max2, 'max(axis=125)',      [random([3, 33, 67, 99, 4, 7])]),
    (reduce_sum0, 'sum(axis=0) 2D',     [random([32, 32])]),
    (reduce_sum0, 'sum(axis=0) 1D',     [random([32])]),
    (reduce_sum1, 'sum(axis=1)',        [random([32, 32])]),
    (reduce_sum2, 'sum(axis=012)',      [random([65, 77, 22, 7])]),
    (no_reduce1, 'no_reduce1(axis=())', [random([32])]),
    (argmax0, 'argmax(axis=0)',         [random([99, 77])]),
    (argmin0, 'argmin(axis=0)',         [random([99, 77])]),
    (reduce_prod0, 'prod(axis=0)',      [random([32, 32]) + 0.5]),
    (gt0, 'gt0',                        [random([32, 32]), random([32, 32])]),
    (ge0, 'ge0',                        [random([32, 32]), random([32, 32])]),
    (ge0, 'ge0 float>=bool',            [random([32, 32]) + 0.5, random([32, 32]) > 0.5]),
    (ge0, 'ge0 bool>=float',            [random([32, 32]) > 0.5, random([32, 32]) + 0.5]),
    (lt0, 'lt0',                        [random([32, 32]), random([32, 32])]),
    (lt0, 'lt0 int[]<scalar',           [randint(999, size=[999]), 555]),
    (le0, 'le0',                        [random([77, 99]), random([77, 99])]),
    (eq0, 'eq0',                        [randint(0, 3, size=[32, 32]).astype(np.float32), randint(0, 3, size=[32, 32]).astype(np.float32)]),
    (eq1, 'eq1 x==x.max(-1)',           [random([32, 32])]),
    (ne0, 'x!=y',                       [random([77, 99]), random([77, 99])]),
    (or0, 'or0 x|y',                    [random([77, 32]).astype('float32').view('uint32'), random([77, 32]).astype('float32').view('uint32')]),
    (and0, 'and0 x&y',                  [random([77, 32]).astype('float32').view('uint32'), random([77, 32]).astype('float32').view('uint32')]),
    (exp0, 'exp(x)',                    [uniform(0, 5, size=[32, 32])]),
    (log0, 'log(x+100)',                [uniform(0, 5, size=[32, 32]) + 100]),
    (abs0, 'abs(x)',                    [random([32, 32, 32]) - 0.5]),
    (rsqrt0, 'rsqrt(x)',                [random([77, 40, 32]) * 10]),
    (iota0, 'iota0',                    []),
    (select0, 'select0',                [random([32, 32]) > 0.5, np.ones([32, 32]), np.zeros([32, 32])]),
    (concatenate0, 'concatenate0',      [random([32, 32, 32]), random([32, 32, 16])]),
    (gather0, 'gather0',                [random([40, 40, 40, 40])]),
    (gather1a, 'gather1a x[5,:]',       [random([8, 8])]),
    (gather1b, 'gather1b x[:,5]',       [random([8, 8])]),
    (gather_fn0, 'gather_fn0',          [random([32, 10]), np.c_[randint(0, 32, size=[32]), randint(0, 10, size=[32])].reshape(32, 1, 2)]),
    (scatter_fn0, 'scatter_fn0',        [random([32, 10]), np.c_[randint(0, 32, size=[32]), randint(0, 10, size=[32])].reshape(32, 1, 2),
                                         random([32]).reshape(32, 1)]),
    (take_along_axis0, 'take_along0',   [random([32, 10]), randint(0, 10, size=32)[:, np.newaxis]]),
    (take_along_axis0_g, 'take0_grad',  [random([32, 10]), randint(0, 10, size=32)[:, np.newaxis]]),
    (gather_fn1, 'gather_fn1',          [random([32, 10]), randint(0, 10, size=[1])]),
    (scatter_add_fn1, 'scatter_add1',   [random([32, 10]), randint(0, 10, size=[1]), random(32)]),
    (add_any0, 'add_any0',              [random([32, 32]), random([32, 32])]),
    (transpose0, 'random([N,N]).T',     [random([32, 32])]),
    (transpose0, 'random([N,M]).T',     [random([32, 65])]),
    (rev0, 'rev0 dims=1,2',             [random([33, 77, 88, 11])]),
    (integer_pow0, 'x**2',              [random([77, 9, 35])]),
    (integer_pow1, 'x**5',              [random([77, 9, 35]) * 2 - 1]),
    (integer_pow1, 'int**5',            [randint(-1000, 1000, size=[77, 9, 35])]),
    (pow0, 'x**scalar',                 [random([77, 9, 35]), random()]),
    (slice0, '1-D slice(x, [2],[33])',  [random([99])]),
    (slice1, '2-D slice no strides',    [random([199, 99])]),
    (slice2, '2-D slice + strides',     [random([199, 99])]),
    (squeeze0, '5-D squeeze',           [random([199, 99, 1, 1, 5])]),
    (threefry0a, 'all const size=1',    []),
    (threefry0b, 'all const size=n',    []),
    (threefry1, 'all zero size=1',      [np.zeros(4).astype('uint32')]),
    (threefry1, 'all ones size=1',      [np.ones(4).astype('uint32')]),
    (threefry1, 'all random size=1',    [randint(0, 10000000, size=4).astype('uint32')]),
    (threefry1, 'all random size=65',   [randint(0, 10000000, size=(4, 65)).astype('uint32')]),
    (threefry1, 'scalar_key_size=100',  [list(randint(0, 10000000, size=(2,)).astype('uint32'))
                                         + list(randint(0, 10000000, size=(2, 100)).astype('uint32'))]),
    (convert_element_type0, 'float2int', [random([77, 101]) * 65]),
    (convert_element_type1, 'int2float', [randint(77, 101, size=(99, 99))]),
    (convert_element_type1, 'bool2float', [random([77, 101]) > 0.5]),
    (bitcast_convert_type0, 'uint2float', [random([77, 101]).astype('float32').view('uint32')]),
    (lax.shift_left, 'x<<1',            [np.arange(-777, +777), 1]),
    (lax.shift_left, 'x<<y',            [np.arange(-777, +777), randint(0, 20, size=777 * 2)]),
    (lax.shift_right_logical, 'x>>1',   [np.arange(-777, +777), 1]),
    (shift_right_logical_1_32, '1>>32', []),
    (lax.shift_right_logical, 'uint>>9', [np.arange(-777, +777).astype('int32').view('uint32'), np.uint32(9)]),
    (lax.shift_right_arithmetic, 'x>>1', [np.arange(-777, +777), 1]),
    (lax.shift_right_arithmetic, 'uint32', [np.arange(-777, +777).astype('int32').view(np.uint32), np.uint32(1)]),
    (lax.erf, 'erf(x)',                 [random([111, 283]) * 10 - 5]),
    (lax.erf_inv, 'erf_inv(x)',         [random([111, 283]) * 2 - 1]),
    (lax.rem, 'rem(x,y)',               [randint(1000, 10000, size=[77, 99]), int(randint(1, 1000))]),
    (lax.nextafter, 'nextafter(X,inf)', [random([77, 101]) * 2 - 1, np.inf]),
    (lax.nextafter, 'nextafter(X,-inf)', [random([77, 101]) * 2 - 1, -np.inf]),
    (lax.nextafter, 'nextafter(X,0)',   [random([77, 101]) * 2 - 1, 0.0]),
    (lax.nextafter, 'nextafter(X,Y)',   [random([77, 101]) * 2 - 1, random([77, 101])]),
]

#names newer jax versions trace (jax.nn.sigmoid -> logistic, x**2 -> square, jnp.logical_not -> not, jnp.split -> split, ...)
def split0(x): return lax.split(x, (3, 0, 90, 6), axis=1)
def split1(x): return [p * 2.0 for p in lax.split(x + 1.0, (5, 2), axis=0)]
def clamp0(x): return lax.clamp(-0.25, x, 0.5)
def clamp1(lo, x, hi): return lax.clamp(lo, x, hi)
def round_even(x): return lax.round(x, 1)
_special = np.array([0.0, -0.0, 1.5, -2.5, np.inf, -np.inf, np.nan, 3e38, 1e-45] * 13, np.float32)
_halves  = np.concatenate([np.arange(-20, 20) + 0.5, random([500]) * 20 - 10, [0.0, -0.0, 2.5, 3.5, -2.5]]).astype(np.float32)

param_matrix += [
    (lax.logistic, 'logistic',          [random([77, 101]) * 20 - 10]),
    (lax.log1p, 'log1p',                [random([77, 101]) * 2 - 0.99]),
    (lax.log1p, 'log1p tiny',           [(random([77, 101]) * 2 - 1) * 1e-6]),
    (lax.expm1, 'expm1',                [random([77, 101]) * 4 - 2]),
    (lax.expm1, 'expm1 tiny',           [(random([77, 101]) * 2 - 1) * 1e-6]),
    (lax.exp2, 'exp2',                  [random([77, 101]) * 40 - 20]),
    (lax.cbrt, 'cbrt',                  [random([77, 101]) * 2000 - 1000]),
    (lax.atan2, 'atan2',                [random([77, 101]) * 2 - 1, random([77, 101]) * 2 - 1]),
    (lax.is_finite, 'is_finite',        [_special]),
    (lax.bitwise_not, 'not bool',       [random([77, 101]) > 0.5]),
    (lax.bitwise_not, 'not int',        [randint(-2**31, 2**31, size=[77, 101])]),
    (lax.sqrt, 'sqrt',                  [np.concatenate([random([500]) * 1e4, [0.0, 1.0, 4.0, np.inf, -1.0, 2.0 ** -140]]).astype(np.float32)]),
    (lax.bitwise_xor, 'xor int',        [randint(-2**31, 2**31, size=[77, 101]), randint(-2**31, 2**31, size=[77, 101])]),
    (lax.bitwise_xor, 'xor bool',       [random([77, 101]) > 0.5, random([77, 101]) > 0.3]),
    (lax.population_count, 'popcount',  [randint(0, 2**32, size=[77, 101], dtype=np.uint64).astype(np.uint32)]),
    (lax.clz, 'clz',                    [np.concatenate([[0, 1, 2**31, 2**32 - 1], 2**randint(0, 32, size=500) - 1]).astype(np.uint32)]),
    (lax.square, 'square float',        [random([77, 101]) * 20 - 10]),
    (lax.square, 'square int',          [randint(-100000, 100000, size=[77, 101])]),
    (lax.round, 'round away',           [_halves]),
    (round_even, 'round even',          [_halves]),
    (clamp0, 'clamp scalars',           [random([77, 101]) * 2 - 1]),
    (clamp1, 'clamp arrays',            [random([77, 101]) - 1, random([77, 101]) * 2 - 1, random([77, 101])]),
    (clamp0, 'clamp int',               [randint(-5, 5, size=[77, 101])]),
    (lambda x: lax.reduce_or(x, (1,)), 'any(axis=1)',    [random([77, 101]) > 0.99]),
    (lambda x: lax.reduce_and(x, (0, 2)), 'all(axis=0,2)', [random([7, 11, 13]) > 0.01]),
    (split0, 'split axis 1',            [random([7, 99, 5])]),
    (split1, 'split + chains',          [random([7, 33])]),
]

for fname in ['cos', 'sin', 'tan', 'cosh', 'sinh', 'tanh', 'acos', 'asin', 'atan', 'acosh', 'asinh', 'atanh',
              'ceil', 'floor', 'sign']:
    param_matrix += [(getattr(lax, fname), fname, [random([77, 101]) * 2 - 1])]

#(rtol, atol); everything else uses numpy.allclose defaults 1e-5 / 1e-8 (reference: tests/test_basic_ops.py:326-333)
TOLERANCES = {
    'erf(x)':        (1e-5, 1e-6),
    'erf_inv(x)':    (1e-5, 1e-5),
    'sum(axis=012)': (1e-4, 1e-8),
    'sin':           (1e-5, 1e-6),
    'sinh':          (1e-5, 1e-6),
    'tan':           (1e-5, 1e-6),
    'log1p tiny':    (1e-5, 1e-12),
    'expm1 tiny':    (1e-5, 1e-12),
    'expm1':         (1e-5, 1e-7),
    'atan2':         (1e-5, 1e-7),
    #dot: north-star tolerance for contractions
    'dot0 x@y': (1e-4, 1e-8), 'dot1 x@const': (1e-4, 1e-8), 'dot axes=(0,0)': (1e-4, 1e-8),
    'dot axes=(1,1)': (1e-4, 1e-8), 'dot axes=(0,1)': (1e-4, 1e-8), 'reshape_dot': (1e-4, 1e-8),
}


@pytest.mark.parametrize('f,desc,args', param_matrix, ids=[p[1] for p in param_matrix])
def test_matrix_hip_interpreter(f, desc, args):
    print(f'case: {getattr(f, "__name__", f)} | {desc}', flush=True)
    rtol, atol = TOLERANCES.get(desc, (1e-5, 1e-8))
    check_against_oracle(f, args, rtol=rtol, atol=atol)


def test_tiled_transposes():
    '''Copies that swap the two fastest dimensions go through the LDS-tiled kernel: ragged sizes, batches,
    NHWC <-> NCHW, a sliced source.'''
    cases = [(lambda x: lax.transpose(x, (1, 0)), [random([1000, 77])]),
             (lambda x: lax.transpose(x, (1, 0)), [random([64, 64])]),
             (lambda x: lax.transpose(x, (1, 0)), [random([68, 1004])]),
             (lambda x: lax.transpose(x[:, 8:48], (0, 2, 1)), [random([3, 36, 52])]),
             (lambda x: lax.transpose(x, (1, 0)), [randint(-9, 9, size=[129, 2050])]),
             (lambda x: lax.transpose(x, (0, 2, 1)), [random([5, 70, 33])]),
             (lambda x: lax.transpose(x, (0, 3, 1, 2)), [random([3, 17, 19, 24])]),
             (lambda x: lax.transpose(x, (0, 2, 3, 1)), [random([3, 24, 17, 19])]),
             (lambda x: lax.transpose(x[3:, 5:70], (1, 0)), [random([40, 100])]),
             (lambda x: lax.transpose(x, (1, 0)) * 2.0, [random([300, 200])]),
             #copies of copies are composed into one launch; a reversed leading dimension is a negative stride
             (lambda x: lax.transpose(lax.rev(x, (0, 1)), (0, 1, 3, 2)), [random([3, 3, 64, 128])]),
             (lambda x: lax.transpose(lax.rev(x, (0,)), (0, 2, 1)), [random([5, 33, 70])]),
             (lambda x: lax.transpose(lax.rev(x, (0, 1)), (0, 1, 3, 2)), [random([1, 1, 256, 64])]),
             (lambda x: lax.transpose(lax.transpose(x, (1, 0, 2)), (0, 2, 1)), [random([6, 5, 40])[:, :, 4:36]]),
             #128 x 128 tiles (both sides at least 128 long, multiples of four): ragged edges, a batch, a reversed batch
             (lambda x: lax.transpose(x, (1, 0)), [random([260, 516])]),
             (lambda x: lax.transpose(x, (0, 2, 1)), [random([3, 132, 512])]),
             (lambda x: lax.transpose(lax.rev(x, (0,)), (0, 2, 1)), [random([3, 128, 640])])]
    for k, (f, args) in enumerate(cases):
        print(f'case: tiled transpose {k}', flush=True)
        _, _, fn = check_against_oracle(f, args, exact=True)
        kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
        if k not in (9, 13):
            assert any(name.startswith('transpose_tiled') for name in kernels), kernels
        if k in (10, 11, 12, 13):
            assert len(kernels) == 1, kernels
        if k >= 14:
            assert kernels == ['transpose_tiled_v4_t128'], kernels


def test_point_and_column_scatter_add_forms():
    '''The two scatter-add forms of the reference (vkjax/ops.py:404-433): single elements `x[i0, i1] += u`
    (shaders/scatter0.comp:10-31; what the gradient of take_along_axis emits, tests/test_basic_ops.py:96,266) and a
    column `x[:, i0] += u` (shaders/scatter1.comp:10-23). Integer-valued operands make the sums exact whatever the
    order of the additions, so fused and unfused programs are compared bit for bit with the oracle, with repeated
    targets; random operands within the element-wise tolerance.'''
    rng = np.random.RandomState(5)
    ints = lambda *shape: rng.randint(-4, 5, size=shape).astype(np.float32)
    for rows, cols, n in ((32, 10, 32), (7, 3, 200), (300, 129, 64), (1, 1, 5)):
        points = np.c_[rng.randint(0, rows, size=[n]), rng.randint(0, cols, size=[n])].reshape(n, 1, 2)   #many targets repeat
        column = rng.randint(0, cols, size=[1])
        along  = rng.randint(0, cols, size=rows)[:, np.newaxis]
        for fuse in (True, False):
            print(f'case: scatter forms {rows}x{cols}, {n} points, fuse={fuse}', flush=True)
            check_against_oracle(scatter_fn0, [ints(rows, cols), points, ints(n, 1)], exact=True, fuse=fuse)
            check_against_oracle(scatter_add_fn1, [ints(rows, cols), column, ints(rows)], exact=True, fuse=fuse)
            #the scatter behind an element-wise step and in front of one, so that the fusion passes see it
            check_against_oracle(lambda x, i, u: scatter_fn0(x * 2.0, i, u + 1.0) - 3.0, [ints(rows, cols), points, ints(n, 1)], exact=True, fuse=fuse)
            check_against_oracle(lambda x, i, u: scatter_add_fn1(x * 2.0, i, u + 1.0) - 3.0, [ints(rows, cols), column, ints(rows)], exact=True, fuse=fuse)
            #the scattered array read by what follows (the result of an in-place accumulation is not its copy launch's)
            zeros = jnp.zeros((rows, cols), np.float32)
            check_against_oracle(lambda x, i, u: (scatter_fn0(x, i, u) * 2.0, -scatter_fn0(zeros, i, u), scatter_fn0(x, i, u).T + 1.0),
                                 [ints(rows, cols), points, ints(n, 1)], exact=True, fuse=fuse)
            check_against_oracle(lambda x, i, u: (scatter_add_fn1(x, i, u) * 2.0, jnp.sum(-scatter_add_fn1(zeros, i, u), axis=1)),
                                 [ints(rows, cols), column, ints(rows)], exact=True, fuse=fuse)
            rows_idx = rng.randint(-rows, rows, size=(n,)).astype(np.int32)
            check_against_oracle(lambda x, i, u: (jnp.index_add(x, i, u) * 2.0, -jnp.index_add(zeros, i, u)),
                                 [ints(rows, cols), rows_idx, ints(n, cols)], exact=True, fuse=fuse)
            #the gradient of take_along_axis with a cotangent of small integers instead of 1 / n
            g = lambda x, i: mj.grad(lambda x, i: (take_along_axis0(x, i) * 3.0).ravel().sum())(x, i)
            y, _, fn = check_against_oracle(g, [ints(rows, cols), along], exact=True, fuse=fuse)
            assert any(repr(op.equation).startswith('scatter-add') or 'scatter-add' in repr(op.equation)
                       for op in list(fn._jaxpr_interpreters.values())[0].all_ops)
            assert y.sum() == 3.0 * rows
            check_against_oracle(take_along_axis0_g, [random([rows, cols]), along], rtol=1e-5, atol=1e-8, fuse=fuse)
            check_against_oracle(scatter_fn0, [random([rows, cols]), points, random([n, 1])], rtol=1e-5, atol=1e-8, fuse=fuse)
            check_against_oracle(scatter_add_fn1, [random([rows, cols]), column, random([rows])], rtol=1e-5, atol=1e-8, fuse=fuse)


def test_nextafter_direction():
    '''reference: tests/test_basic_ops.py:367-382'''
    import vkjax_amd
    x = random([77, 101, 5]).astype(np.float32)
    vkfunc = vkjax_amd.wrap(lax.nextafter, frontend='minijax')
    assert np.all(vkfunc(x, np.inf) > x)
    assert np.all(x > vkfunc(x, -np.inf))
    assert np.all(np.sign(vkfunc(x, 0.0) - x) == np.sign(0 - x))
    x2 = random(x.shape).astype(np.float32)
    assert np.all(np.sign(vkfunc(x, x2) - x) == np.sign(x2 - x))


def test_max_pool_negative_border_and_select_with_inf():
    '''XLA semantics where the reference's shaders differ: padding of a max window is -inf, and
    select picks without touching the other branch.'''
    x = -1.0 - random([2, 5, 5, 3])
    def pool(x): return lax.reduce_window(x, -jnp.inf, lax.max, (1, 3, 3, 1), (1, 2, 2, 1), 'SAME')
    y, ytrue, _ = check_against_oracle(pool, [x], exact=True)
    assert np.all(y < 0)
    p = random([8, 8]) > 0.5
    a = np.where(random([8, 8]) > 0.5, np.inf, 1.0)
    b = np.where(random([8, 8]) > 0.5, np.nan, -2.0)
    check_against_oracle(select0, [p, a, b], exact=True)


def test_argmax_ties_and_nan():
    x = np.array([[1, 3, 3, 2], [np.nan, 5, np.nan, 1], [2, 2, 2, 2], [0, -1, 7, 7]], np.float32)
    def f(x): return jnp.argmax(x, axis=1), jnp.argmin(x, axis=1)
    (amax, amin), _, _ = check_against_oracle(f, [x], exact=True)
    assert amax.tolist() == [1, 0, 0, 2] and amin.tolist() == [0, 0, 0, 1]


def test_arrays_without_elements():
    '''Shapes with a dimension of size 0: results without elements cost no launch, a reduction or contraction over
    no elements gives the operation's identity (XLA's init values), and the rest of the program is untouched.'''
    import vkjax_amd
    f32 = lambda *shape: np.zeros(shape, np.float32)
    cases = [('add', lambda x, y: x + y, [f32(0, 5), f32(0, 5)], 0),
             ('sum over an empty axis', lambda x: jnp.sum(x, axis=0), [f32(0, 5)], 1),
             ('max over an empty axis', lambda x: lax.reduce_max(x, (1,)), [f32(3, 0)], 1),
             ('min over an empty axis', lambda x: lax.reduce_min(x, (1,)), [np.zeros((3, 0), np.int32)], 1),
             ('sum that stays empty', lambda x: jnp.sum(x, axis=1), [f32(0, 5)], 0),
             ('concatenate with an empty part', lambda x, y: lax.concatenate([x, y], 0), [f32(0, 5), np.ones((2, 5), np.float32)], 1),
             ('dot over an empty contraction', lambda x, y: jnp.dot(x, y) + 1.0, [f32(4, 0), f32(0, 3)], None),
             ('dot without rows', lambda x, y: jnp.dot(x, y), [f32(0, 8), np.ones((8, 3), np.float32)], 0),
             ('gather without indices', lambda t, i: t[i], [np.ones((6, 4), np.float32), np.zeros((0,), np.int32)], 0),
             ('transpose', lambda x: lax.transpose(x, (1, 0)), [f32(0, 7)], 0),
             ('empty and not', lambda x, y: (x * 2.0, y + 1.0), [f32(0), np.ones((3,), np.float32)], 1),
             ('convolution of an empty batch', lambda x, k: lax.conv_general_dilated(x, k, (1, 1), 'SAME', dimension_numbers=('NHWC', 'HWIO', 'NHWC')),
              [f32(0, 6, 6, 4), np.ones((3, 3, 4, 8), np.float32)], 0)]
    for name, f, args, launches in cases:
        print(f'case: {name}', flush=True)
        _, _, fn = check_against_oracle(f, args, exact=True)
        n = len(list(fn._jaxpr_interpreters.values())[0].launches)
        assert launches is None or n == launches, (name, n)
        check_against_oracle(f, args, exact=True, fuse=False)


def test_call_and_alias_primitives_of_newer_jax():
    '''The names and parameter layouts newer jax versions put into a jaxpr where the reference's era had xla_call /
    custom_jvp_call_jaxpr / select: pjit and jit (a closed jaxpr under `jaxpr`), closed_call / core_call / remat
    (`call_jaxpr`), custom_jvp_call (`call_jaxpr`), custom_vjp_call with either parameter name, copy, copy_p,
    optimization_barrier on several operands, select_n. The stand-in tracer does not produce them by itself, so the
    equations are emitted by hand, each around a body with a closed-over constant.'''
    from vkjax_amd.minijax import tracer, core
    bias = np.arange(12, dtype=np.float32).reshape(3, 4)
    body = lambda x, y: (lax.max(x * y + bias, 0.0), x - y)

    def nested(primitive, jaxpr_param, closed, **extra):
        return lambda x, y: tracer._call_nested(body, primitive, jaxpr_param, extra, closed=closed, args=(x, y))
    def aliases(x, y):
        a = tracer.emit('copy', [x], [core.ShapedArray(x.shape, x.dtype)])
        b = tracer.emit('copy_p', [y], [core.ShapedArray(y.shape, y.dtype)])
        a, b = tracer.emit('optimization_barrier', [a, b], [core.ShapedArray(x.shape, x.dtype)] * 2, multiple_results=True)
        pick = tracer.emit('select_n', [lax.gt(a, b), a, b], [core.ShapedArray(x.shape, x.dtype)])       #b where a > b
        wide = tracer.emit('expand_dims', [pick], [core.ShapedArray((1,) + tuple(x.shape) + (1,), x.dtype)], dict(dimensions=(0, 3)))
        return pick * 2.0, a + b, wide + 1.0
    cases = [('pjit', nested('pjit', 'jaxpr', True, name='body', donated_invars=(False, False), inline=False, keep_unused=False)),
             ('jit', nested('jit', 'jaxpr', True, name='body')),
             ('closed_call', nested('closed_call', 'call_jaxpr', True)),
             ('core_call', nested('core_call', 'call_jaxpr', False)),
             ('remat', nested('remat', 'call_jaxpr', False, prevent_cse=True, differentiated=False)),
             ('custom_jvp_call', nested('custom_jvp_call', 'call_jaxpr', True, num_consts=0, symbolic_zeros=False, jvp_jaxpr_fun=None)),
             ('custom_vjp_call', nested('custom_vjp_call', 'call_jaxpr', True, num_consts=0, bwd=None, fwd_jaxpr_thunk=None, out_trees=None, symbolic_zeros=False)),
             ('custom_vjp_call_jaxpr', nested('custom_vjp_call_jaxpr', 'fun_jaxpr', True, num_consts=0, bwd=None, fwd_jaxpr_thunk=None, out_trees=None)),
             ('copy, optimization_barrier, select_n', aliases)]
    x, y = random([3, 4]) - 0.5, random([3, 4]) - 0.5
    for name, f in cases:
        print(f'case: {name}', flush=True)
        check_against_oracle(f, [x, y], rtol=1e-6, atol=1e-7)
        check_against_oracle(f, [x, y], rtol=1e-6, atol=1e-7, fuse=False)
