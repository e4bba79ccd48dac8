'''conv_general_dilated parity against the CPU oracle on the reference's case list
(reference: tests/test_conv.py:66-85: NHWC/HWIO and NCHW/OIHW dimension numbers, 1x1/3x3/7x7,
VALID/SAME/uneven explicit padding, stride 2, rhs and lhs dilation), plus reduce_window
(reference: tests/test_reduce_window.py:18-21). Tolerance: rtol 1e-4 for contractions.'''
import numpy as np
import pytest

from vkjax_amd import minijax as mj
from tests.common import check_against_oracle

jnp, lax = mj.numpy, mj.lax
pytestmark = pytest.mark.gpu
rng = np.random.RandomState(4321)
random = rng.random_sample

NHWC = mj.core.ConvDimensionNumbers((0, 3, 1, 2), (3, 2, 0, 1), (0, 3, 1, 2))
NCHW = mj.core.ConvDimensionNumbers((0, 1, 2, 3), (0, 1, 2, 3), (0, 1, 2, 3))

kernel_1x1 = random([1, 1, 5, 33])

def conv0(x):     return lax.conv_general_dilated(x, kernel_1x1, (1, 1), 'VALID', dimension_numbers=NHWC)
def conv1(x, k):  return lax.conv_general_dilated(x, k, (1, 1), 'VALID', dimension_numbers=NHWC)
def conv1a(x, k): return lax.conv_general_dilated(x, k, (1, 1), 'VALID', dimension_numbers=NCHW)
def conv2(x, k):  return lax.conv_general_dilated(x, k, (1, 1), 'SAME', dimension_numbers=NHWC)
def conv3(x, k):  return lax.conv_general_dilated(x, k, (1, 1), [(2, 0), (0, 3)], dimension_numbers=NHWC)
def conv4(x, k):  return lax.conv_general_dilated(x, k, (2, 2), 'SAME', dimension_numbers=NHWC)
def conv5(x, k):  return lax.conv_general_dilated(x, k, (2, 2), 'VALID', rhs_dilation=(2, 2), dimension_numbers=NHWC)
def conv6a(x, k): return lax.conv_general_dilated(x, k, (1, 1), [(2, 2), (3, 3)], lhs_dilation=(2, 2), dimension_numbers=NHWC)
def conv6b(x, k): return lax.conv_general_dilated(x, k, (2, 2), [(0, 0), (0, 0)], lhs_dilation=(2, 2), dimension_numbers=NHWC)

param_matrix = [
    (conv0,  'conv0 1x1 const kernel no pad',               [random([11, 100, 100, 5])]),
    (conv1,  'conv1 1x1 var kernel no pad',                 [random([11, 100, 100, 33]), random([1, 1, 33, 11])]),
    (conv1,  'conv1 3x3 var kernel no pad',                 [random([40, 65, 33, 5]), random([3, 3, 5, 7])]),
    (conv1a, 'conv1a 3x3 convdims 0123',                    [random([40, 8, 65, 35]), random([39, 8, 3, 3])]),
    (conv2,  'conv2 1x1 var kernel +pad',                   [random([77, 17, 9, 12]), random([1, 1, 12, 11])]),
    (conv2,  'conv2 3x3 var kernel +pad',                   [random([23, 44, 19, 7]), random([3, 3, 7, 38])]),
    (conv2,  'conv2 7x7 var kernel +pad',                   [random([8, 12, 19, 3]), random([7, 7, 3, 4])]),
    (conv3,  'conv3 3x3 uneven pad',                        [random([15, 67, 42, 11]), random([3, 3, 11, 38])]),
    (conv4,  'conv4 1x1 window strides=2',                  [random([2, 67, 42, 3]), random([1, 1, 3, 2])]),
    (conv4,  'conv4 3x3 window strides=2',                  [random([15, 67, 42, 11]), random([3, 3, 11, 7])]),
    (conv5,  'conv5 3x3 window strides=2 + rhs_dilate=2',   [random([15, 67, 42, 11]), random([3, 3, 11, 7])]),
    (conv6a, 'conv6a 3x3 window strides=1 + lhs_dilate=2',  [random([15, 67, 42, 11]), random([3, 3, 11, 7])]),
    (conv6b, 'conv6b 3x3 window strides=2 + lhs_dilate=2',  [random([15, 67, 42, 11]), random([3, 3, 11, 7])]),
    #shapes that take the 16-byte-load paths and every tile size
    (conv2,  'fast 3x3 C64->64',              [random([8, 56, 56, 64]), random([3, 3, 64, 64])]),
    (conv1,  'fast 1x1 C64->256',            [random([16, 56, 56, 64]), random([1, 1, 64, 256])]),
    (conv4,  'fast 3x3 s2 C32->64',                         [random([4, 28, 28, 32]), random([3, 3, 32, 64])]),
    (conv4,  'fast 1x1 s2 C128->96 (N not tile multiple)',  [random([3, 14, 14, 128]), random([1, 1, 128, 96])]),
    (conv2,  'generic lhs, fast rhs 7x7 C3->64',            [random([2, 64, 64, 3]), random([7, 7, 3, 64])]),
]


@pytest.mark.parametrize('f,desc,args', param_matrix, ids=[p[1] for p in param_matrix])
def test_convmatrix(f, desc, args):
    print(f'case: {desc}', flush=True)
    check_against_oracle(f, args, rtol=1e-4, atol=1e-6)


def test_conv_integer_valued_is_exact():
    '''Small-integer inputs make every product and partial sum exact in fp32, so any accumulation
    order must give bit-identical results: catches indexing mistakes independently of rounding.'''
    x = rng.randint(-4, 5, size=[3, 20, 17, 16]).astype(np.float32)
    k = rng.randint(-3, 4, size=[3, 3, 16, 24]).astype(np.float32)
    check_against_oracle(conv2, [x, k], exact=True)
    check_against_oracle(conv4, [x, k], exact=True)


def test_dot_integer_valued_is_exact_all_layouts():
    a = rng.randint(-8, 9, size=[70, 132]).astype(np.float32)
    b = rng.randint(-8, 9, size=[132, 52]).astype(np.float32)
    check_against_oracle(lambda x, y: lax.dot_general(x, y, (((1,), (0,)), ((), ()))), [a, b], exact=True)
    check_against_oracle(lambda x, y: lax.dot_general(x, y, (((0,), (0,)), ((), ()))), [a.T.copy(), b], exact=True)
    check_against_oracle(lambda x, y: lax.dot_general(x, y, (((1,), (1,)), ((), ()))), [a, b.T.copy()], exact=True)
    check_against_oracle(lambda x, y: lax.dot_general(x, y, (((0,), (1,)), ((), ()))), [a.T.copy(), b.T.copy()], exact=True)


def test_dot_sizes():
    for m, k, n in [(256, 784, 512), (256, 512, 10), (64, 2048, 1000), (1, 1, 1), (129, 33, 65), (300, 64, 64)]:
        print(f'dot {m}x{k}x{n}', flush=True)
        a, b = random([m, k]) - 0.5, random([k, n]) - 0.5
        check_against_oracle(lambda x, y: jnp.dot(x, y), [a, b], rtol=1e-4, atol=1e-5)


def reduce_window_max0(x): return lax.reduce_window(x, -jnp.inf, lax.max, (1, 2, 2, 1), (1, 1, 1, 1), 'VALID')
def reduce_window_max1(x): return lax.reduce_window(x, -jnp.inf, lax.max, (1, 3, 3, 1), (1, 2, 2, 1), 'SAME')
def reduce_window_max2(x): return lax.reduce_window(x, -jnp.inf, lax.max, (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (0, 1), (0, 1), (0, 0)))
def reduce_window_sum0(x): return lax.reduce_window(x, 0.0, lax.add, (1, 2, 2, 1), (1, 2, 2, 1), 'VALID')
def reduce_window_sum1(x): return lax.reduce_window(x, 0.0, lax.add, (1, 3, 3, 1), (1, 2, 2, 1), 'SAME')
def reduce_window_odd(x):  return lax.reduce_window(x, -jnp.inf, lax.max, (1, 3, 2, 3), (1, 2, 1, 2), ((0, 0), (1, 1), (0, 1), (1, 0)))

pool_matrix = [
    (reduce_window_max0, '2x2 no-pad',        [random([11, 100, 111, 5])], True),
    (reduce_window_max1, '3x3 +pad',          [random([77, 10, 99, 17])], True),
    (reduce_window_max1, '3x3 +pad C64',      [random([4, 56, 56, 64]) - 0.5], True),
    (reduce_window_max1, '3x3 s2 odd sizes C8', [random([3, 15, 17, 8]) - 0.5], True),
    (reduce_window_max1, '3x3 s2 tiny C4',    [random([2, 3, 2, 4]) - 0.5], True),
    (reduce_window_max2, '3x3 s2 pad hi C12', [random([2, 14, 13, 12]) - 0.5], True),
    (reduce_window_sum1, 'sum 3x3 s2 SAME C8', [np.round(random([3, 15, 17, 8]) * 8)], True),
    (reduce_window_sum0, 'sum 2x2 s2',        [random([4, 28, 28, 32])], False),
    (reduce_window_sum1, 'sum 3x3 s2 SAME',   [random([3, 15, 17, 6])], False),
    (reduce_window_odd,  'window over C too', [random([3, 15, 17, 6]) - 0.5], True),
]


@pytest.mark.parametrize('f,desc,args,exact', pool_matrix, ids=[p[1] for p in pool_matrix])
def test_reduce_window_matrix(f, desc, args, exact):
    print(f'case: {desc}', flush=True)
    check_against_oracle(f, args, exact=exact, rtol=1e-5, atol=1e-6)


TILES = [('64x64', 32), ('64x64', 64), ('32x32', 32), ('32x32', 64)]


@pytest.mark.parametrize('tile,bk', TILES)
def test_every_tile_and_loader_variant(tile, bk):
    '''All 20 kernel instantiations: each tile shape and k step with 16-byte (f) or strided (g) loads on
    either operand, and the lean variant. The ff2 / ff3 cases have Cin % 64 == 0 (tap position kept in
    scalar registers) and a 1x1 unpadded kernel (rows addressed as a flat matrix): they qualify for the
    lean variant and run through both it and the general ff kernel.'''
    from vkjax_amd import kernels as K
    cases = {'ff': ([3, 20, 17, 16], [3, 3, 16, 24]), 'gg': ([2, 13, 11, 5], [3, 3, 5, 7]),
             'gf': ([2, 13, 11, 3], [3, 3, 3, 64]), 'fg': ([2, 13, 11, 8], [3, 3, 8, 10]),
             'ff2': ([2, 9, 11, 64], [3, 3, 64, 40]), 'ff3': ([2, 9, 11, 128], [1, 1, 128, 72])}
    for variant, (xs, ks) in cases.items():
        for general in (True, False):
            expected = variant[:2] if general or variant not in ('ff2', 'ff3') else 'lean'
            print(f'tile {tile} bk {bk} loaders {variant} -> {expected}', flush=True)
            x = rng.randint(-4, 5, size=xs).astype(np.float32)
            k = rng.randint(-3, 4, size=ks).astype(np.float32)
            #(a dense kernel operand takes 16-byte loads whatever its width)
            with K.overrides(conv_tile=tile, conv_bk=bk, conv_general=general, conv_b_general=variant[1] == 'g'):
                _, _, fn = check_against_oracle(conv2, [x, k], exact=True)
            kernel = list(fn._jaxpr_interpreters.values())[0].launches[0].kernel
            assert kernel == f'conv_gemm_{tile}x{bk}_{expected}', kernel


@pytest.mark.parametrize('tile,bk', TILES)
def test_lean_kernel_tile_chunks_with_epilogue(tile, bk):
    '''The lean variant walking 1, 2, 3 or 5 consecutive M tiles per block (the last block of a launch gets
    a shorter run), with and without padding taps, with a batch-norm + residual + ReLU epilogue, a
    bias + ReLU epilogue and none; integer-valued data, so every result is exact.'''
    from vkjax_amd import kernels as K
    from vkjax_amd import minijax as mj
    lax, nn = mj.lax, mj.nn
    dn = ('NHWC', 'HWIO', 'NHWC')

    def bn_res_relu(x, k, mean, scale, beta, res):
        y = lax.conv_general_dilated(x, k, (1, 1), 'SAME', dimension_numbers=dn)
        return nn.relu((y - mean) * scale + beta + res)

    def bias_relu(x, k, bias):
        return nn.relu(lax.conv_general_dilated(x, k, (2, 2), 'VALID', dimension_numbers=dn) + bias)

    with K.overrides(conv_tile=tile, conv_bk=bk):
        for chunk in (1, 2, 3, 5):
            for ksize, cin, cout in ((3, 64, 40), (1, 128, 72)):
                print(f'tile {tile} bk {bk} chunk {chunk} kernel {ksize}x{ksize} {cin}->{cout}', flush=True)
                x = rng.randint(-4, 5, size=[3, 13, 11, cin]).astype(np.float32)
                k = rng.randint(-3, 4, size=[ksize, ksize, cin, cout]).astype(np.float32)
                vec = lambda lo, hi: rng.randint(lo, hi, size=[cout]).astype(np.float32)
                res = rng.randint(-50, 50, size=[3, 13, 11, cout]).astype(np.float32)
                for f, args in ((bn_res_relu, [x, k, vec(-5, 5), vec(1, 4), vec(-9, 9), res]), (bias_relu, [x, k, vec(-9, 9)]),
                                (conv2, [x, k])):
                    with K.overrides(conv_chunk=chunk):
                        _, _, fn = check_against_oracle(f, args, exact=True)
                    launches = list(fn._jaxpr_interpreters.values())[0].launches
                    assert [l.kernel for l in launches] == [f'conv_gemm_{tile}x{bk}_lean'], [l.kernel for l in launches]
        # a grid of a fixed number of blocks that share the M tiles of every N tile evenly (here 1, 2, 3 or 5 blocks
        # per N tile: runs of unequal length, blocks with a single tile, one block with all of them)
        for per_n_tile in (1, 2, 3, 5):
            for ksize, cin, cout in ((3, 64, 40), (1, 128, 72)):
                tiles_n = -(-cout // int(tile.split('x')[1]))
                even = dict(conv_even_split_min_tiles=0.0, conv_blocks_per_cu=(per_n_tile * tiles_n + 0.5) / 256)
                print(f'tile {tile} bk {bk} {per_n_tile} blocks per N tile, kernel {ksize}x{ksize} {cin}->{cout}', flush=True)
                x = rng.randint(-4, 5, size=[3, 13, 11, cin]).astype(np.float32)
                k = rng.randint(-3, 4, size=[ksize, ksize, cin, cout]).astype(np.float32)
                vec = lambda lo, hi: rng.randint(lo, hi, size=[cout]).astype(np.float32)
                res = rng.randint(-50, 50, size=[3, 13, 11, cout]).astype(np.float32)
                for f, args in ((bn_res_relu, [x, k, vec(-5, 5), vec(1, 4), vec(-9, 9), res]), (bias_relu, [x, k, vec(-9, 9)])):
                    with K.overrides(**even):
                        _, _, fn = check_against_oracle(f, args, exact=True)
                    launches = list(fn._jaxpr_interpreters.values())[0].launches
                    assert [l.kernel for l in launches] == [f'conv_gemm_{tile}x{bk}_lean'], [l.kernel for l in launches]
                    tiles_m = -(-launches[0].buffers[0][0].size // cout // int(tile.split('x')[0]))
                    assert launches[0].grid[0] == min(per_n_tile, tiles_m) * tiles_n, (launches[0].grid, tiles_m, tiles_n)


def test_four_waves_per_tile_kernel():
    '''Products with few output tiles: four waves share a 32 x 32 tile, each taking a quarter of every 128-long
    k step. Dense layers with bias / ReLU, a contraction that is no multiple of 128, 1x1 and padded 3x3
    convolutions with a batch-norm + residual + ReLU epilogue; integer-valued data, so every result is exact.'''
    from vkjax_amd import kernels as K
    from vkjax_amd import minijax as mj
    lax, nn, jnp = mj.lax, mj.nn, mj.numpy
    dn = ('NHWC', 'HWIO', 'NHWC')
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)

    def dense(x, w, b): return nn.relu(jnp.dot(x, w) + b)
    def plain(x, w): return jnp.dot(x, w)
    def bn_res_relu(x, k, mean, scale, beta, res):
        y = lax.conv_general_dilated(x, k, (1, 1), 'SAME', dimension_numbers=dn)
        return nn.relu((y - mean) * scale + beta + res)

    cases = [(dense, [ints(-4, 5, 256, 784), ints(-3, 4, 784, 512), ints(-9, 9, 512)]),
             (dense, [ints(-4, 5, 70, 132), ints(-3, 4, 132, 36), ints(-9, 9, 36)]),
             (plain, [ints(-4, 5, 64, 2048), ints(-2, 3, 2048, 1000)]),
             (plain, [ints(-4, 5, 33, 256), ints(-2, 3, 256, 4)]),
             (dense, [ints(-4, 5, 256, 512), ints(-3, 4, 512, 10), ints(-9, 9, 10)]),
             (plain, [ints(-4, 5, 40, 388), ints(-2, 3, 388, 7)]),
             (bn_res_relu, [ints(-4, 5, 2, 9, 7, 128), ints(-3, 4, 1, 1, 128, 72), ints(-5, 5, 72), ints(1, 4, 72), ints(-9, 9, 72), ints(-50, 50, 2, 9, 7, 72)]),
             (bn_res_relu, [ints(-4, 5, 2, 9, 7, 256), ints(-3, 4, 3, 3, 256, 40), ints(-5, 5, 40), ints(1, 4, 40), ints(-9, 9, 40), ints(-50, 50, 2, 9, 7, 40)]),
             #windows over 64 and 192 features: the 64-long k step
             (bn_res_relu, [ints(-4, 5, 1, 14, 9, 64), ints(-3, 4, 3, 3, 64, 64), ints(-5, 5, 64), ints(1, 4, 64), ints(-9, 9, 64), ints(-50, 50, 1, 14, 9, 64)]),
             (bn_res_relu, [ints(-4, 5, 2, 5, 6, 192), ints(-3, 4, 3, 3, 192, 33), ints(-5, 5, 33), ints(1, 4, 33), ints(-9, 9, 33), ints(-50, 50, 2, 5, 6, 33)])]
    for f, args in cases:
        short = f is bn_res_relu and args[1].shape[0] == 3 and args[1].shape[2] % 128 != 0
        for b_general in (False, True):
            print(f'four waves per tile: {f.__name__} {[a.shape for a in args]} element-wise kernel loads {b_general}', flush=True)
            with K.overrides(conv_ksplit=True, conv_k_splits=1, conv_b_general=b_general):
                _, _, fn = check_against_oracle(f, args, exact=True)
            launches = list(fn._jaxpr_interpreters.values())[0].launches
            if short:                                     #(this variant exists with 16-byte loads of the kernel operand only)
                assert ([l.kernel for l in launches] == ['conv_gemm_32x32x64_ks4']) == (not b_general), [l.kernel for l in launches]
            else:
                assert [l.kernel for l in launches] == ['conv_gemm_32x32x128_ks4g' if b_general else 'conv_gemm_32x32x128_ks4'], [l.kernel for l in launches]


def test_xcd_layouts_of_the_four_waves_per_tile_kernel():
    '''The tile -> workgroup map of the four-waves-per-tile kernels with the XCDs laid over the tile grid as 8 x 1,
    4 x 2, 2 x 4 and 1 x 8 rectangles and as row-major ranges, plain and with a sliced contraction: every layout is
    a permutation of the tiles, so integer-valued products are exact under all of them.'''
    from vkjax_amd import kernels as K
    from vkjax_amd import minijax as mj
    nn, jnp = mj.nn, mj.numpy
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)
    def dense(x, w, b): return nn.relu(jnp.dot(x, w) + b)
    for m, k, n in ((256, 784, 512), (64, 1024, 256), (128, 300, 96), (32, 512, 256)):
        args = [ints(-4, 5, m, k), ints(-3, 4, k, n), ints(-9, 9, n)]
        for xn in (None, 0, 1, 2, 4, 8):
            for slices in (1, 2):
                print(f'xcd layout: {m}x{k}x{n}, {xn} columns, {slices} slice(s)', flush=True)
                with K.overrides(conv_ksplit=True, conv_k_splits=slices, conv_xcd_columns=xn):
                    _, _, fn = check_against_oracle(dense, args, exact=True)
                assert list(fn._jaxpr_interpreters.values())[0].launches[0].kernel == 'conv_gemm_32x32x128_ks4'


def test_sliced_contractions():
    '''Products with few tiles and a long contraction: blocks of their own sum slices of the contraction (2, 3, 4 and
    7 slices, also slices of unequal length and a last k step that is not full) into one matrix per slice, and an
    element-wise launch adds the slices and applies what follows the product. Dense layers, a 1x1 and padded 3x3
    convolutions whose later slices start at another kernel tap, with bias + ReLU, a batch-norm + residual + ReLU
    chain and nothing behind them; row counts that do not fill the last tile; both loaders of the kernel operand;
    integer-valued data, so every result is exact. The heuristic slices the layers it is meant for.'''
    from vkjax_amd import kernels as K
    from vkjax_amd import minijax as mj
    lax, nn, jnp = mj.lax, mj.nn, mj.numpy
    dn = ('NHWC', 'HWIO', 'NHWC')
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)

    def dense(x, w, b): return nn.relu(jnp.dot(x, w) + b)
    def plain(x, w): return jnp.dot(x, w)
    def bn_res_relu(x, k, mean, scale, beta, res):
        y = lax.conv_general_dilated(x, k, (1, 1), 'SAME', dimension_numbers=dn)
        return nn.relu((y - mean) * scale + beta + res)

    cases = [(dense, [ints(-4, 5, 49, 1024), ints(-3, 4, 1024, 96), ints(-9, 9, 96)]),
             (plain, [ints(-4, 5, 70, 900), ints(-2, 3, 900, 36)]),
             (plain, [ints(-4, 5, 33, 1300), ints(-2, 3, 1300, 7)]),
             (bn_res_relu, [ints(-4, 5, 1, 7, 7, 512), ints(-3, 4, 1, 1, 512, 72), ints(-5, 5, 72), ints(1, 4, 72), ints(-9, 9, 72), ints(-50, 50, 1, 7, 7, 72)]),
             (bn_res_relu, [ints(-4, 5, 1, 7, 7, 128), ints(-3, 4, 3, 3, 128, 40), ints(-5, 5, 40), ints(1, 4, 40), ints(-9, 9, 40), ints(-50, 50, 1, 7, 7, 40)]),
             (bn_res_relu, [ints(-4, 5, 2, 5, 6, 256), ints(-3, 4, 3, 3, 256, 33), ints(-5, 5, 33), ints(1, 4, 33), ints(-9, 9, 33), ints(-50, 50, 2, 5, 6, 33)])]
    for f, args in cases:
        for slices in (2, 3, 4, 7):
            for b_general in (False, True):
                print(f'sliced contraction: {f.__name__} {[a.shape for a in args]} {slices} slices, element-wise kernel loads {b_general}', flush=True)
                with K.overrides(conv_ksplit=True, conv_k_splits=slices, conv_b_general=b_general):
                    _, _, fn = check_against_oracle(f, args, exact=True)
                launches = list(fn._jaxpr_interpreters.values())[0].launches
                assert launches[0].kernel == ('conv_gemm_32x32x128_ks4g' if b_general else 'conv_gemm_32x32x128_ks4')
                assert launches[0].buffers[0][0].shape[0] > 1 and all(l.kernel.startswith(('ew_chain', 'ew_affine')) for l in launches[1:]), [l.kernel for l in launches]
    #by the heuristic: a 3x3 layer of a network's last stage on one image (32 tiles, 36 k steps), against float data
    x, k = rng.randn(1, 7, 7, 512).astype(np.float32), (rng.randn(3, 3, 512, 512) / 68).astype(np.float32)
    _, _, fn = check_against_oracle(lambda a, b: nn.relu(lax.conv_general_dilated(a, b, (1, 1), 'SAME', dimension_numbers=dn)), [x, k], rtol=1e-4, atol=1e-5)
    launches = list(fn._jaxpr_interpreters.values())[0].launches
    assert [l.kernel for l in launches][0] == 'conv_gemm_32x32x128_ks4' and launches[0].grid == (128, 1, 1) and len(launches) == 2


def test_mixed_tiling():
    '''Layers whose 64 x 64 tiles do not divide evenly among the CUs: the first M tiles as 64 x 64 tiles, the rows
    behind them as 32 x 32 tiles computed by four waves each, in one launch (conv_gemm_64x64x{32,64}_mix). Padded 3x3, strided and
    1x1 convolutions and a plain product, with a batch-norm + residual + ReLU epilogue, bias + ReLU and none; splits
    that leave one small tile row, several, a last tile that is not full in either direction; integer-valued data,
    so every result is exact.'''
    from vkjax_amd import kernels as K
    from vkjax_amd import minijax as mj
    lax, nn, jnp = mj.lax, mj.nn, mj.numpy
    dn = ('NHWC', 'HWIO', 'NHWC')
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)

    def bn_res_relu(stride):
        def f(x, k, mean, scale, beta, res):
            y = lax.conv_general_dilated(x, k, (stride, stride), 'SAME', dimension_numbers=dn)
            return nn.relu((y - mean) * scale + beta + res)
        return f
    def dense(x, w, b): return nn.relu(jnp.dot(x, w) + b)

    def conv_case(batch, h, w, ksize, cin, cout, stride=1):
        ho, wo = -(-h // stride), -(-w // stride)
        return (bn_res_relu(stride), [ints(-4, 5, batch, h, w, cin), ints(-3, 4, ksize, ksize, cin, cout), ints(-5, 5, cout), ints(1, 4, cout),
                                      ints(-9, 9, cout), ints(-50, 50, batch, ho, wo, cout)])
    cases = [conv_case(3, 13, 11, 3, 64, 72), conv_case(2, 14, 14, 3, 128, 256), conv_case(5, 7, 7, 1, 256, 100),
             conv_case(3, 14, 14, 3, 64, 64, stride=2), (conv2, [ints(-4, 5, 2, 20, 17, 64), ints(-3, 4, 3, 3, 64, 40)]),
             (dense, [ints(-4, 5, 300, 328), ints(-3, 4, 328, 136), ints(-9, 9, 136)])]
    for f, args in cases:
        for bk in (32, 64):
            for split in (1, 2, 5):
                print(f'mixed tiling: {f.__name__} {[a.shape for a in args]} bk {bk}, {split} M tiles of 64 rows', flush=True)
                with K.overrides(conv_tile='64x64', conv_bk=bk, conv_chunk=1, conv_ksplit=False, conv_mix=split):
                    _, _, fn = check_against_oracle(f, args, exact=True)
                launches = list(fn._jaxpr_interpreters.values())[0].launches
                m = launches[0].flops // (2 * int(np.prod(args[1].shape[:-1])) * args[1].shape[-1])
                expected = f'conv_gemm_64x64x{bk}_mix' if split * 64 < m else f'conv_gemm_64x64x{bk}_lean'
                assert [l.kernel for l in launches] == [expected], ([l.kernel for l in launches], m)


def test_stem_kernel_for_few_input_features():
    '''conv_gemm_stem_7x22 and its 512-thread form _m128: seven kernel rows whose KW * Cin values (21 or 22) are read from a
    patch of image rows in LDS. 7 x 7 on 3 features with stride 2 and padding 3 (the ResNet stem), stride 1, a 7 x 11 kernel on 2
    features, fewer than 64 output features, images that are not square, several tiles per block (more tiles than
    the grid has blocks), with a batch-norm + ReLU epilogue, bias + ReLU and none; integer-valued data, so every
    result is exact.'''
    from vkjax_amd import kernels as K
    from vkjax_amd import minijax as mj
    lax, nn = mj.lax, mj.nn
    dn = ('NHWC', 'HWIO', 'NHWC')
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)
    vec = lambda lo, hi, n: rng.randint(lo, hi, size=[n]).astype(np.float32)

    def conv(stride, padding):
        return lambda x, k: lax.conv_general_dilated(x, k, (stride, stride), padding, dimension_numbers=dn)
    def bn_relu(stride, padding):
        def f(x, k, mean, var, scale, beta):
            y = lax.conv_general_dilated(x, k, (stride, stride), padding, dimension_numbers=dn)
            return nn.relu((y - mean) * (scale * lax.rsqrt(var + 3.0)) + beta)       #var + 3 = 4: an exact rsqrt
        return f
    def bias_relu(stride, padding):
        return lambda x, k, b: nn.relu(lax.conv_general_dilated(x, k, (stride, stride), padding, dimension_numbers=dn) + b)

    def centred_and_activated(x, k, mean, scale, beta):           #a second result after the `- vector` step (what a training step keeps)
        y = lax.conv_general_dilated(x, k, (2, 2), ((3, 3), (3, 3)), dimension_numbers=dn) - mean
        return y, nn.relu(y * scale + beta)
    def raw_and_activated(x, k, scale, beta):                      #a second result before the first step
        y = lax.conv_general_dilated(x, k, (2, 2), ((3, 3), (3, 3)), dimension_numbers=dn)
        return y, nn.relu(y * scale + beta)

    p3 = ((3, 3), (3, 3))
    cases = [(centred_and_activated, [ints(-4, 5, 2, 128, 128, 3), ints(-3, 4, 7, 7, 3, 64), vec(-5, 5, 64), vec(1, 4, 64), vec(-9, 9, 64)]),
             (raw_and_activated, [ints(-4, 5, 3, 128, 192, 3), ints(-3, 4, 7, 7, 3, 48), vec(1, 4, 48), vec(-9, 9, 48)]),
             (bn_relu(2, p3), [ints(-4, 5, 2, 128, 128, 3), ints(-3, 4, 7, 7, 3, 64), vec(-5, 5, 64), np.ones(64, np.float32), vec(1, 4, 64) * 2, vec(-9, 9, 64)]),
             (conv(2, p3), [ints(-4, 5, 3, 20, 192, 3), ints(-3, 4, 7, 7, 3, 40)]),
             (bias_relu(1, p3), [ints(-4, 5, 1, 12, 64, 3), ints(-3, 4, 7, 7, 3, 64), vec(-9, 9, 64)]),
             (conv(2, ((3, 3), (5, 5))), [ints(-4, 5, 2, 16, 128, 2), ints(-3, 4, 7, 11, 2, 24)]),
             (conv(2, ((0, 2), (3, 4))), [ints(-4, 5, 1, 132, 128, 3), ints(-3, 4, 7, 7, 3, 64)]),
             (bn_relu(2, p3), [ints(-4, 5, 18, 128, 128, 3), ints(-3, 4, 7, 7, 3, 64), vec(-5, 5, 64), np.ones(64, np.float32), vec(1, 4, 64) * 2, vec(-9, 9, 64)])]
    seen = set()
    for f, args in cases:
        print(f'stem kernel: {[a.shape for a in args]}', flush=True)
        for fuse in (True, False):
            #tiles of 128 output positions (512 threads) where the sizes allow them, and the 64-position tiles everywhere
            for tile in (None, 64):
                with K.overrides(conv_stem=tile):
                    _, _, fn = check_against_oracle(f, args, exact=True, fuse=fuse)
                launches = list(fn._jaxpr_interpreters.values())[0].launches
                kernels = [l.kernel for l in launches if l.kernel.startswith('conv_gemm')]
                assert kernels in (['conv_gemm_stem_7x22'], ['conv_gemm_stem_7x22_m128']) and (tile is None or kernels == ['conv_gemm_stem_7x22']), kernels
                seen.add(kernels[0])
                if fuse and 'and_activated' in f.__name__:
                    assert len(launches) == 1, [l.kernel for l in launches]       #both results from the one launch
    assert seen == {'conv_gemm_stem_7x22', 'conv_gemm_stem_7x22_m128'}
    #a shape it does not take falls back to the general kernel
    _, _, fn = check_against_oracle(conv(2, p3), [ints(-4, 5, 2, 30, 26, 3), ints(-3, 4, 7, 7, 3, 64)], exact=True)
    assert [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches] == ['conv_gemm_64x64x32_gf']


def test_convolution_with_a_second_result():
    '''A convolution result that is returned (or read later) AND continued by an element-wise chain: one launch
    stores both, the value before the chain or after its `- vector` step and the chain's result. Integer-valued
    data, so both are exact; lean and general kernel variants, an output tile that is not full, and a chain of
    five steps with a residual operand.'''
    from vkjax_amd import minijax as mj
    lax, nn = mj.lax, mj.nn
    dn = ('NHWC', 'HWIO', 'NHWC')
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)

    def centred_and_activated(x, k, mean, scale, beta):
        y = lax.conv_general_dilated(x, k, (1, 1), 'SAME', dimension_numbers=dn) - mean
        return y, nn.relu(y * scale + beta)
    def raw_and_activated(x, k, scale, beta):
        y = lax.conv_general_dilated(x, k, (1, 1), 'SAME', dimension_numbers=dn)
        return y, nn.relu(y * scale + beta)
    def centred_residual(x, k, mean, scale, beta, res):
        y = lax.conv_general_dilated(x, k, (2, 2), 'SAME', dimension_numbers=dn) - mean
        return nn.relu(y * scale + beta + res), y

    cases = [(centred_and_activated, [ints(-4, 5, 2, 9, 7, 64), ints(-3, 4, 3, 3, 64, 128), ints(-5, 5, 128), ints(1, 4, 128), ints(-9, 9, 128)]),
             (centred_and_activated, [ints(-4, 5, 3, 6, 5, 12), ints(-3, 4, 1, 1, 12, 40), ints(-5, 5, 40), ints(1, 4, 40), ints(-9, 9, 40)]),
             (centred_and_activated, [ints(-4, 5, 1, 8, 8, 3), ints(-3, 4, 3, 3, 3, 8), ints(-5, 5, 8), ints(1, 4, 8), ints(-9, 9, 8)]),
             (raw_and_activated, [ints(-4, 5, 2, 9, 7, 64), ints(-3, 4, 1, 1, 64, 64), ints(1, 4, 64), ints(-9, 9, 64)]),
             (centred_residual, [ints(-4, 5, 2, 10, 8, 32), ints(-3, 4, 3, 3, 32, 64), ints(-5, 5, 64), ints(1, 4, 64), ints(-9, 9, 64),
                                 ints(-50, 50, 2, 5, 4, 64)])]
    for f, args in cases:
        print(f'second result: {f.__name__} {[a.shape for a in args]}', flush=True)
        _, _, fn = check_against_oracle(f, args, exact=True)
        launches = list(fn._jaxpr_interpreters.values())[0].launches
        assert len(launches) == 1 and launches[0].kernel.startswith('conv_gemm'), [l.kernel for l in launches]
        flags = int(np.frombuffer(launches[0].params, dtype=np.uint32)[21])
        assert (flags >> 12) & 15 in (1, 2), hex(flags)
        check_against_oracle(f, args, exact=True, fuse=False)


def test_single_image_with_a_one_column_result():
    '''Batch 1 and an output one column wide, with stride, padding or taps outside the input: the matrix-product
    shortcut of the 16-byte loader (output row = input row) must not be taken. Integer-valued, exact.'''
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)
    cases = [((1, 2, 2, 12), (3, 3, 12, 8), 2, ((0, 1), (0, 1))), ((1, 2, 2, 12), (3, 3, 12, 8), 1, ((0, 1), (0, 1))),
             ((1, 2, 2, 12), (3, 3, 12, 8), 2, ((1, 0), (1, 0))), ((1, 4, 2, 12), (3, 3, 12, 8), 2, ((0, 1), (0, 1))),
             ((1, 2, 2, 32), (3, 3, 32, 8), 2, ((0, 1), (0, 1))), ((1, 6, 1, 16), (3, 1, 16, 8), 2, ((0, 0), (0, 0))),
             ((1, 6, 1, 16), (3, 1, 16, 8), 1, ((0, 0), (0, 0))), ((1, 5, 3, 64), (3, 3, 64, 64), 1, ((1, 1), (0, 0)))]
    for xs, ks, stride, pad in cases:
        print(f'case: {xs} {ks} stride {stride} padding {pad}', flush=True)
        f = lambda x, k: lax.conv_general_dilated(x, k, (stride, stride), pad, dimension_numbers=NHWC)
        check_against_oracle(f, [ints(-3, 4, *xs), ints(-2, 3, *ks)], exact=True)


def test_gradient_of_a_strided_convolution_that_skips_the_whole_input():
    '''A stride that steps over the only input row: the input gradient is a convolution whose (negative) padding
    crops more than the cotangent holds. Every tap then lies outside, and the padded size still counts.'''
    from vkjax_amd import minijax as mj
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)
    x, k = ints(-3, 4, 2, 1, 5, 12), ints(-2, 3, 1, 2, 12, 16)
    conv = lambda x, k: lax.conv_general_dilated(x, k, (3, 1), ((2, 0), (2, 2)), rhs_dilation=(2, 1), dimension_numbers=NHWC)
    f = lambda x, k: mj.value_and_grad(lambda p: jnp.sum(conv(p[0], p[1]) * 2.0))((x, k))
    for fuse in (True, False):
        check_against_oracle(f, [x, k], exact=True, fuse=fuse)
