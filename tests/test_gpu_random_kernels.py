'''Seeded random geometry through the kernels whose applicability depends on the shape: the mixed 64 x 64 /
32 x 32 tiling (split point, k step and epilogue drawn at random), the stem kernel (kernel width x features of 21
or 22 in several factorisations, strides, paddings on all four sides, image sizes around its limits; shapes it does
not take fall back to the general kernel and are checked all the same) and the sorted scatter-add (table and index
sizes around the segment and block limits, crowded rows, indices outside the table), sliced contractions (number of
slices, 1x1 and 3x3 windows, k steps that are not full), the kernel for at most 16 output features, and the
straight-line kernel for sums of arrays followed by scale, shift, residual and ReLU. Integer-valued data: every
result equals the oracle's bit for bit.'''
import numpy as np
import pytest

from vkjax_amd import kernels as K, minijax as mj, ops
from tests.common import check_against_oracle

pytestmark = pytest.mark.gpu
lax, jnp, nn = mj.lax, mj.numpy, mj.nn
DN = ('NHWC', 'HWIO', 'NHWC')


def _mixed_tiling_case(rng, ints):
    b, h, w = int(rng.choice([1, 2, 3])), int(rng.randint(3, 20)), int(rng.randint(3, 20))
    ks, stride = int(rng.choice([1, 3])), int(rng.choice([1, 1, 2]))
    cin  = int(rng.choice([64, 68, 100, 128, 260])) if ks == 1 else int(rng.choice([64, 128, 192]))
    cout = int(rng.choice([8, 40, 64, 72, 130]))
    ho, wo = -(-h // stride), -(-w // stride)
    m = b * ho * wo
    if m < 70 or cin * ks * ks < 256:
        return None
    x, k = ints(-3, 4, b, h, w, cin), ints(-2, 3, ks, ks, cin, cout)
    conv = lambda x, k: lax.conv_general_dilated(x, k, (stride, stride), 'SAME', dimension_numbers=DN)
    epilogue = rng.randint(0, 3)
    if epilogue == 0:
        f, args = conv, [x, k]
    elif epilogue == 1:
        f, args = (lambda x, k, bias: nn.relu(conv(x, k) + bias)), [x, k, ints(-9, 9, cout)]
    else:
        f = lambda x, k, mean, scale, shift, res: nn.relu((conv(x, k) - mean) * scale + shift + res)
        args = [x, k, ints(-5, 5, cout), ints(1, 4, cout), ints(-9, 9, cout), ints(-50, 50, b, ho, wo, cout)]
    forced = dict(conv_tile='64x64', conv_bk=int(rng.choice([32, 64])), conv_chunk=1, conv_ksplit=False,
                  conv_mix=int(rng.randint(1, max(2, m // 64 + 1))))
    return f, args, forced, '_mix' if forced['conv_mix'] * 64 < m else '_lean'


def _stem_case(rng, ints):
    cin, kw = [(3, 7), (3, 7), (2, 11), (1, 21), (1, 22), (11, 2), (7, 3)][rng.randint(0, 7)]
    stride = int(rng.choice([1, 2, 2]))
    pw, ph = (int(rng.randint(0, kw)), int(rng.randint(0, kw))), (int(rng.randint(0, 5)), int(rng.randint(0, 5)))
    w = (int(rng.choice([64, 64, 96, 128])) - 1) * stride + kw - sum(pw) + int(rng.randint(0, stride))
    while w < 1 or (w * cin) % 4:
        w += 1
    wo = (w + sum(pw) - kw) // stride + 1
    ho = int(rng.choice([1, 2, 3, 5, 8]))
    while (ho * wo) % 64:
        ho += 1
    h = (ho - 1) * stride + 7 - sum(ph) + int(rng.randint(0, stride))
    if wo < 64 or h < 1:
        return None
    cout = int(rng.choice([8, 24, 40, 64]))
    x, k = ints(-3, 4, int(rng.choice([1, 2, 3])), h, w, cin), ints(-2, 3, 7, kw, cin, cout)
    f = lambda x, k, bias: nn.relu(lax.conv_general_dilated(x, k, (stride, stride), (ph, pw), dimension_numbers=DN) + bias)
    return f, [x, k, ints(-9, 9, cout)], {}, ''


def _scatter_case(rng, ints):
    rows, cols = int(rng.choice([1, 5, 64, 300, 1024, 1025, 5000, 70000])), int(rng.choice([1, 3, 4, 64, 256, 260]))
    n = int(rng.choice([1, 2, 17, 65, 256, 1000, 5000]))
    idx = rng.randint(-2, rows + 2, size=(n,)).astype(np.int32)
    if rng.randint(0, 2):
        idx[: n // 2] = idx[0]
    return (lambda t, i, u: jnp.index_add(t, i, u)), [ints(-9, 10, rows, cols), idx, ints(-3, 4, n, cols)], {}, 'scatter_rows_sum'


def _sliced_case(rng, ints):
    ks = int(rng.choice([1, 1, 3]))
    if ks == 1:
        m, kdim, n = int(rng.randint(1, 130)), int(rng.choice([256, 388, 512, 900, 1300, 2048])), int(rng.choice([17, 24, 40, 72, 96]))
        x, w = ints(-3, 4, m, kdim), ints(-2, 3, kdim, n)
        product, out_shape = (lambda x, w: jnp.dot(x, w)), (m, n)
    else:
        b, h, wd, cin, n = int(rng.choice([1, 2])), int(rng.randint(3, 9)), int(rng.randint(3, 9)), int(rng.choice([128, 256])), int(rng.choice([24, 40, 72]))
        x, w = ints(-3, 4, b, h, wd, cin), ints(-2, 3, 3, 3, cin, n)
        product, out_shape = (lambda x, w: lax.conv_general_dilated(x, w, (1, 1), 'SAME', dimension_numbers=DN)), (b, h, wd, n)
    epilogue = rng.randint(0, 3)
    if epilogue == 0:
        f, args = product, [x, w]
    elif epilogue == 1:
        f, args = (lambda x, w, bias: nn.relu(product(x, w) + bias)), [x, w, ints(-9, 9, n)]
    else:
        f = lambda x, w, mean, scale, shift, res: nn.relu((product(x, w) - mean) * scale + shift + res)
        args = [x, w, ints(-5, 5, n), ints(1, 4, n), ints(-9, 9, n), ints(-50, 50, *out_shape)]
    return f, args, dict(conv_ksplit=True, conv_k_splits=int(rng.randint(2, 6))), 'ks4'


def _few_features_case(rng, ints):
    m, kdim, n = int(rng.randint(1, 300)), 4 * int(rng.randint(1, 300)), int(rng.randint(1, 17))
    x, w = ints(-3, 4, m, kdim), ints(-2, 3, kdim, n)
    epilogue = rng.randint(0, 3)
    if epilogue == 0:
        return (lambda x, w: jnp.dot(x, w)), [x, w], {}, 'dense_rows_n16'
    if epilogue == 1 and n > 1:
        return (lambda x, w, bias: nn.relu(jnp.dot(x, w) + bias)), [x, w, ints(-9, 9, n)], {}, 'dense_rows_n16'
    if n > 1:
        return (lambda x, w, mean, scale, shift: (jnp.dot(x, w) - mean) * scale + shift), [x, w, ints(-5, 5, n), ints(1, 4, n), ints(-9, 9, n)], {}, 'dense_rows_n16'
    return None


def _affine_chain_case(rng, ints):
    shape = [(int(rng.randint(2, 70)), 4 * int(rng.randint(1, 40))), (2, int(rng.randint(1, 9)), int(rng.randint(1, 9)), 4 * int(rng.randint(1, 20)))][rng.randint(0, 2)]
    c, nsum = shape[-1], int(rng.randint(0, 4))
    parts = [int(rng.randint(0, 2)) for _ in range(5)]
    if nsum + sum(parts) == 0:
        return None
    arrays, vectors = [ints(-9, 10, *shape) for _ in range(5)], [ints(-5, 5, c), ints(-3, 4, c), ints(-9, 9, c)]
    def f(first, s1, s2, s3, full, vsub, vmul, vadd):
        v = first
        for a in (s1, s2, s3)[:nsum]:
            v = v + a
        if parts[0]: v = v - vsub
        if parts[1]: v = v * vmul
        if parts[2]: v = v + vadd
        if parts[3]: v = v + full
        if parts[4]: v = nn.relu(v)
        return v
    return f, arrays + vectors, dict(ew_affine=True), 'ew_affine_v4'


@pytest.mark.parametrize('seed', range(180))
def test_random_geometry(seed):
    cases = (_mixed_tiling_case, _stem_case, _scatter_case, _sliced_case, _few_features_case, _affine_chain_case)
    make  = cases[seed % 3 if seed < 90 else 3 + seed % 3]                   #(the first 90 seeds keep the cases they always had)
    #a draw that falls outside the kernel's range is drawn again (from the next stream of the seed), so that every seed runs a case
    for attempt in range(100):
        rng  = np.random.RandomState(777 + seed + 100000 * attempt)
        ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)
        case = make(rng, ints)
        if case is not None:
            break
    assert case is not None, 'a hundred draws outside the kernels\' range'
    f, args, forced, expected = case
    if seed < 90 and seed % 3 == 2:
        forced = dict(forced, scatter_sort_threshold=0)
    print(f'seed {seed} (draw {attempt}): {[a.shape for a in args]} {forced}', flush=True)
    with K.overrides(**forced):
        _, _, fn = check_against_oracle(f, args, exact=True)
    kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
    assert any(expected in k for k in kernels), kernels
