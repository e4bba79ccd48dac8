'''Pins the CPU oracle (oracle/primitives.py) to facts that do not come from the oracle itself:
published known-answer vectors, library routines, exact integer arithmetic, brute-force loops
written from the reference shaders' loop structure, and closed forms. CPU only.'''
import itertools
import json
import os

import numpy as np
import pytest
import torch

from oracle import primitives as P
from oracle.eval_jaxpr import eval_closed_jaxpr
from vkjax_amd import minijax as mj
from vkjax_amd.minijax import core

jnp, lax = mj.numpy, mj.lax
GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), 'golden', 'known_answers.json')))
rng = np.random.RandomState(7)


# ------------------------------------------------------------------ threefry / random

def test_threefry_random123_known_answers():
    for kat in GOLDEN['threefry2x32_kat']:
        k = [np.uint32(int(v, 16)) for v in kat['key']]
        c = [np.uint32(int(v, 16)) for v in kat['counter']]
        out = P.threefry2x32(k[0], k[1], np.array([c[0]], np.uint32), np.array([c[1]], np.uint32))
        assert [hex(int(out[0][0])), hex(int(out[1][0]))] == [hex(int(v, 16)) for v in kat['expected']]


def test_threefry_vector_equals_scalar_loop_and_scalar_key_broadcast():
    keys = rng.randint(0, 2**32, size=(2, 65), dtype=np.uint64).astype(np.uint32)
    data = rng.randint(0, 2**32, size=(2, 65), dtype=np.uint64).astype(np.uint32)
    a, b = P.threefry2x32(keys[0], keys[1], data[0], data[1])
    for i in range(65):
        ai, bi = P.threefry2x32(keys[0, i], keys[1, i], data[0, i:i + 1], data[1, i:i + 1])
        assert (ai[0], bi[0]) == (a[i], b[i])
    a, b = P.threefry2x32(keys[0, 0], keys[1, 0], data[0], data[1])
    a2, b2 = P.threefry2x32(np.full(65, keys[0, 0]), np.full(65, keys[1, 0]), data[0], data[1])
    assert np.array_equal(a, a2) and np.array_equal(b, b2)


def test_split_and_uniform_match_published_jax_values():
    key = mj.random.PRNGKey(0)
    assert key.tolist() == [0, 0]
    closed = mj.make_jaxpr(lambda k: mj.random.split(k))(key)
    (split,) = eval_closed_jaxpr(closed, key)
    assert split.tolist() == GOLDEN['jax_random_split_PRNGKey0']
    closed = mj.make_jaxpr(lambda k: (mj.random.random_bits(k, ()), mj.random.uniform(k, ())))(key)
    bits, u = eval_closed_jaxpr(closed, key)
    assert int(bits) == GOLDEN['jax_random_uniform_PRNGKey0']['bits']
    assert np.float32(u) == np.float32(GOLDEN['jax_random_uniform_PRNGKey0']['value'])
    #closed form of the bits -> float map
    assert np.float32(u) == np.float32((int(bits) >> 9) * 2.0 ** -23)


def test_normal_matches_published_jax_values():
    '''jax's documentation prints random.normal(PRNGKey(0), (1,)) = [-0.20584226] and the ten values of
    random.normal(PRNGKey(0), (10,)) in its quickstart; they pin the uniform -> erf_inv path end to end.'''
    key = mj.random.PRNGKey(0)
    for shape, name in (((1,), 'shape_1'), ((10,), 'shape_10')):
        closed = mj.make_jaxpr(lambda k: mj.random.normal(k, shape))(key)
        (x,) = eval_closed_jaxpr(closed, key)
        assert np.allclose(x, np.float32(GOLDEN['jax_random_normal_PRNGKey0'][name]), rtol=2e-6, atol=0)


def test_random_bits_odd_sizes_pad_and_trim():
    key = mj.random.PRNGKey(42)
    for n in (1, 2, 5, 6, 33):
        closed = mj.make_jaxpr(lambda k: mj.random.random_bits(k, (n,)))(key)
        (bits,) = eval_closed_jaxpr(closed, key)
        m = n + n % 2
        counts = np.arange(m, dtype=np.uint32)
        counts[n:] = 0
        a, b = P.threefry2x32(key[0], key[1], counts[:m // 2], counts[m // 2:])
        assert np.array_equal(bits, np.concatenate([a, b])[:n])


def test_randint_is_the_remainder_of_a_64_bit_draw():
    '''randint composes a key split, two draws and 32-bit remainder arithmetic that stands for
    (hi * 2**32 + lo) % span; with spans below 2**16 no product overflows, so the oracle's result must equal that
    remainder computed with Python's integers from the (pinned) draws of the two half keys. Bounds the wrong way
    round return minval.'''
    r = mj.random
    for seed, shape, lo, hi in ((0, (1,), 0, 9999), (17, (6, 5), -77, 1234), (5, (33,), 10, 11), (9, (4,), -3, 65000), (1, (3,), 8, 8), (2, (3,), 9, -9)):
        key = r.PRNGKey(seed)
        (got,) = eval_closed_jaxpr(mj.make_jaxpr(lambda k: r.randint(k, shape, lo, hi))(key), key)
        (keys,) = eval_closed_jaxpr(mj.make_jaxpr(lambda k: r.split(k))(key), key)
        (high,) = eval_closed_jaxpr(mj.make_jaxpr(lambda k: r.random_bits(k, shape))(keys[0]), keys[0])
        (low,)  = eval_closed_jaxpr(mj.make_jaxpr(lambda k: r.random_bits(k, shape))(keys[1]), keys[1])
        span = max(hi - lo, 1)
        want = [(int(h) * 2**32 + int(l)) % span + lo for h, l in zip(high.ravel(), low.ravel())]
        assert got.dtype == np.int32 and got.shape == shape and got.ravel().tolist() == want, (seed, shape, lo, hi)
        assert (got >= lo).all() and (got < max(hi, lo + 1)).all()


# ------------------------------------------------------------------ dot / conv

def test_dot_general_exact_integers_and_einsum_layouts():
    a = rng.randint(-9, 10, size=(13, 21)).astype(np.float32)
    b = rng.randint(-9, 10, size=(21, 17)).astype(np.float32)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(P.dot_general(a, b, (((1,), (0,)), ((), ()))), want)
    assert np.array_equal(P.dot_general(a.T, b, (((0,), (0,)), ((), ()))), want)
    assert np.array_equal(P.dot_general(a, b.T, (((1,), (1,)), ((), ()))), want)
    assert np.array_equal(P.dot_general(a.T, b.T, (((0,), (1,)), ((), ()))), want)
    x, y = rng.rand(4, 5, 6), rng.rand(4, 6, 7)
    got = P.dot_general(x, y, (((2,), (1,)), ((0,), (0,))))
    assert np.allclose(got, np.einsum('bik,bkj->bij', x, y), rtol=1e-6)


def conv_brute_force(lhs, rhs, strides, padding, lhs_dil, rhs_dil, dn):
    '''Loop nest of the reference shader (vkjax/shaders/conv2d.comp:44-95): for every output
    element walk the dilated kernel window and the input features; a tap contributes when its
    input coordinate lies inside the dilated input and on a multiple of the lhs dilation.'''
    ls, rs, os_ = dn
    B, C, H, W = (lhs.shape[d] for d in ls)
    O, _, KH, KW = (rhs.shape[d] for d in rs)
    Hd, Wd = (H - 1) * lhs_dil[0] + 1, (W - 1) * lhs_dil[1] + 1
    Ho = (Hd + padding[0][0] + padding[0][1] - ((KH - 1) * rhs_dil[0] + 1)) // strides[0] + 1
    Wo = (Wd + padding[1][0] + padding[1][1] - ((KW - 1) * rhs_dil[1] + 1)) // strides[1] + 1
    out_shape = [0] * 4
    for d, n in zip(os_, (B, O, Ho, Wo)):
        out_shape[d] = n
    out = np.zeros(out_shape, np.float64)
    for b, o, y, x in itertools.product(range(B), range(O), range(Ho), range(Wo)):
        acc = 0.0
        for i0, i1, c in itertools.product(range(KH), range(KW), range(C)):
            j0 = y * strides[0] + i0 * rhs_dil[0] - padding[0][0]
            j1 = x * strides[1] + i1 * rhs_dil[1] - padding[1][0]
            if j0 < 0 or j1 < 0 or j0 >= Hd or j1 >= Wd or j0 % lhs_dil[0] or j1 % lhs_dil[1]:
                continue
            li = [0] * 4; ri = [0] * 4
            for d, v in zip(ls, (b, c, j0 // lhs_dil[0], j1 // lhs_dil[1])): li[d] = v
            for d, v in zip(rs, (o, c, i0, i1)): ri[d] = v
            acc += float(lhs[tuple(li)]) * float(rhs[tuple(ri)])
        oi = [0] * 4
        for d, v in zip(os_, (b, o, y, x)): oi[d] = v
        out[tuple(oi)] = acc
    return out


NHWC = ((0, 3, 1, 2), (3, 2, 0, 1), (0, 3, 1, 2))
NCHW = ((0, 1, 2, 3), (0, 1, 2, 3), (0, 1, 2, 3))
CONV_CASES = [   #lhs, rhs, strides, padding, lhs_dilation, rhs_dilation, dims   (the variety of reference tests/test_conv.py:66-85)
    ((2, 6, 5, 3), (1, 1, 3, 4), (1, 1), ((0, 0), (0, 0)), (1, 1), (1, 1), NHWC),
    ((2, 7, 5, 2), (3, 3, 2, 3), (1, 1), ((0, 0), (0, 0)), (1, 1), (1, 1), NHWC),
    ((2, 3, 7, 6), (4, 3, 3, 3), (1, 1), ((0, 0), (0, 0)), (1, 1), (1, 1), NCHW),
    ((2, 6, 5, 2), (3, 3, 2, 3), (1, 1), ((1, 1), (1, 1)), (1, 1), (1, 1), NHWC),
    ((1, 8, 9, 1), (7, 7, 1, 2), (1, 1), ((3, 3), (3, 3)), (1, 1), (1, 1), NHWC),
    ((2, 7, 6, 2), (3, 3, 2, 2), (1, 1), ((2, 0), (0, 3)), (1, 1), (1, 1), NHWC),
    ((2, 7, 6, 2), (3, 3, 2, 2), (2, 2), ((0, 1), (0, 1)), (1, 1), (1, 1), NHWC),
    ((2, 9, 8, 2), (3, 3, 2, 2), (2, 2), ((0, 0), (0, 0)), (1, 1), (2, 2), NHWC),
    ((2, 5, 4, 2), (3, 3, 2, 2), (1, 1), ((2, 2), (3, 3)), (2, 2), (1, 1), NHWC),
    ((2, 5, 4, 2), (3, 3, 2, 2), (2, 2), ((0, 0), (0, 0)), (2, 2), (1, 1), NHWC),
]


@pytest.mark.parametrize('case', CONV_CASES, ids=[str(i) for i in range(len(CONV_CASES))])
def test_conv_matches_brute_force_and_torch(case):
    ls, rs, strides, padding, ldil, rdil, dn = case
    lhs, rhs = rng.rand(*ls), rng.rand(*rs)
    got = P.conv_general_dilated(lhs, rhs, strides, padding, ldil, rdil, dn)
    want = conv_brute_force(lhs, rhs, strides, padding, ldil, rdil, dn)
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    #independent library routine: torch conv2d in float64 on NCHW/OIHW, lhs dilation as zero insertion
    x = torch.from_numpy(np.transpose(lhs, [dn[0][0], dn[0][1], dn[0][2], dn[0][3]]).copy())
    w = torch.from_numpy(np.transpose(rhs, [dn[1][0], dn[1][1], dn[1][2], dn[1][3]]).copy())
    if ldil != (1, 1):
        xd = torch.zeros(x.shape[0], x.shape[1], (x.shape[2] - 1) * ldil[0] + 1, (x.shape[3] - 1) * ldil[1] + 1, dtype=x.dtype)
        xd[:, :, ::ldil[0], ::ldil[1]] = x
        x = xd
    x = torch.nn.functional.pad(x, (padding[1][0], padding[1][1], padding[0][0], padding[0][1]))
    y = torch.nn.functional.conv2d(x, w, stride=strides, dilation=rdil).numpy()
    inv = np.argsort([dn[2][0], dn[2][1], dn[2][2], dn[2][3]])
    assert np.allclose(got, np.transpose(y, inv), rtol=1e-6, atol=1e-6)


def test_conv_special_cases():
    x = rng.rand(2, 6, 7, 5)
    #1x1 stride 1 is a matrix product over the feature axis
    w = rng.rand(1, 1, 5, 3)
    got = P.conv_general_dilated(x, w, (1, 1), ((0, 0), (0, 0)), (1, 1), (1, 1), NHWC)
    assert np.allclose(got, (x.reshape(-1, 5) @ w.reshape(5, 3)).reshape(2, 6, 7, 3), rtol=1e-6)
    #a delta kernel with SAME padding shifts the image: tap (0, 2) reads x[y-1, x+1]
    d = np.zeros((3, 3, 5, 5)); d[0, 2] = np.eye(5)
    got = P.conv_general_dilated(x, d, (1, 1), ((1, 1), (1, 1)), (1, 1), (1, 1), NHWC)
    want = np.zeros_like(x); want[:, 1:, :-1] = x[:, :-1, 1:]
    assert np.array_equal(got, want.astype(np.float32))
    #integer-valued inputs: exact
    xi = rng.randint(-4, 5, size=(2, 6, 7, 5)).astype(np.float32)
    wi = rng.randint(-4, 5, size=(3, 3, 5, 4)).astype(np.float32)
    got = P.conv_general_dilated(xi, wi, (2, 2), ((0, 1), (1, 1)), (1, 1), (1, 1), NHWC)
    want = conv_brute_force(xi, wi, (2, 2), ((0, 1), (1, 1)), (1, 1), (1, 1), NHWC)
    assert np.array_equal(got, want.astype(np.float32))


# ------------------------------------------------------------------ window reductions

def test_reduce_window_against_brute_force_and_torch():
    x = rng.rand(2, 9, 10, 3) - 0.5
    for window, strides, padding in [((1, 2, 2, 1), (1, 1, 1, 1), ((0, 0),) * 4),
                                     ((1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (0, 1), (1, 1), (0, 0)))]:
        got_max = P.reduce_window_max(x, window, strides, padding)
        got_sum = P.reduce_window_sum(x, window, strides, padding)
        xt = torch.from_numpy(np.transpose(x, (0, 3, 1, 2)).copy())
        pads = (padding[2][0], padding[2][1], padding[1][0], padding[1][1])
        want_max = torch.nn.functional.max_pool2d(torch.nn.functional.pad(xt, pads, value=float('-inf')),
                                                  window[1:3], strides[1:3]).numpy()
        want_sum = torch.nn.functional.avg_pool2d(torch.nn.functional.pad(xt, pads, value=0.0), window[1:3], strides[1:3],
                                                  divisor_override=1).numpy()
        assert np.array_equal(got_max, np.transpose(want_max, (0, 2, 3, 1)).astype(np.float32))
        assert np.allclose(got_sum, np.transpose(want_sum, (0, 2, 3, 1)), rtol=1e-6, atol=1e-7)
    #all-negative input: a border window must not see a 0 from the padding
    neg = -1.0 - rng.rand(1, 4, 4, 1)
    out = P.reduce_window_max(neg, (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (0, 1), (0, 1), (0, 0)))
    assert np.all(out < 0)
    assert out[0, 1, 1, 0] == np.float32(neg[0, 2:4, 2:4, 0].max())


def test_same_padding_closed_form():
    for n, k, s in [(56, 3, 2), (112, 3, 2), (7, 3, 1), (224, 7, 2), (10, 2, 2), (99, 3, 2)]:
        lo, hi = lax._same_padding(n, k, s)
        out = -(-n // s)
        assert lo + hi == max((out - 1) * s + k - n, 0) and lo == (lo + hi) // 2
        assert (n + lo + hi - k) // s + 1 == out


# ------------------------------------------------------------------ gather / scatter

def test_gather_forms_against_numpy_indexing():
    x = rng.rand(6, 7, 8, 5).astype(np.float32)
    G = core.GatherDimensionNumbers
    assert np.array_equal(P.gather(x, np.array([4], np.int32), G((0, 1, 2, 3), (), (2,)), (6, 7, 3, 5)), x[:, :, 4:7, :])
    y = rng.rand(8, 8).astype(np.float32)
    assert np.array_equal(P.gather(y, np.array([5], np.int32), G((0,), (0,), (0,)), (1, 8)), y[5, :])
    assert np.array_equal(P.gather(y, np.array([5], np.int32), G((0,), (1,), (1,)), (8, 1)), y[:, 5])
    t = rng.rand(32, 10).astype(np.float32)
    i = np.c_[rng.randint(0, 32, 32), rng.randint(0, 10, 32)].reshape(32, 1, 2).astype(np.int32)
    assert np.array_equal(P.gather(t, i, G((), (0, 1), (0, 1)), (1, 1)), t[i[:, 0, 0], i[:, 0, 1]][:, None])
    idx = rng.randint(0, 32, size=(5, 3, 1)).astype(np.int32)
    assert np.array_equal(P.gather(t, idx, G((2,), (0,), (0,)), (1, 10)), t[idx[..., 0]])
    #start indices are clamped so that the slice fits
    assert np.array_equal(P.gather(y, np.array([99], np.int32), G((0,), (0,), (0,)), (1, 8)), y[7, :])
    assert np.array_equal(P.gather(y, np.array([-3], np.int32), G((0,), (0,), (0,)), (1, 8)), y[0, :])
    assert np.array_equal(P.gather(x, np.array([7], np.int32), G((0, 1, 2, 3), (), (2,)), (6, 7, 3, 5)), x[:, :, 5:8, :])


def test_scatter_add_forms_against_add_at():
    S = core.ScatterDimensionNumbers
    x = rng.rand(32, 10)
    i = np.c_[rng.randint(0, 32, 32), rng.randint(0, 10, 32)].reshape(32, 1, 2).astype(np.int32)
    u = rng.rand(32, 1)
    want = x.copy(); np.add.at(want, (i[:, 0, 0], i[:, 0, 1]), u[:, 0])
    assert np.allclose(P.scatter_add(x, i, u, S((), (0, 1), (0, 1))), want, rtol=1e-6)
    col, v = np.array([3], np.int32), rng.rand(32)
    want = x.copy(); want[:, 3] += v
    assert np.allclose(P.scatter_add(x, col, v, S((0,), (1,), (1,))), want, rtol=1e-6)
    rows = rng.randint(0, 32, size=(6, 4, 1)).astype(np.int32)
    upd  = rng.randint(-5, 6, size=(6, 4, 10)).astype(np.float32)
    want = np.zeros((32, 10)); np.add.at(want, rows[..., 0], upd)
    assert np.array_equal(P.scatter_add(np.zeros((32, 10), np.float32), rows, upd, S((2,), (0,), (0,))), want.astype(np.float32))
    #out-of-range windows are dropped
    bad = np.array([[40], [-1], [2]], np.int32)
    got = P.scatter_add(np.zeros((32, 10), np.float32), bad, np.ones((3, 10), np.float32), S((1,), (0,), (0,)))
    assert got.sum() == 10 and np.all(got[2] == 1)


# ------------------------------------------------------------------ reductions / element-wise

def test_gather_fill_and_scatter_clip_modes():
    '''The modes newer jax versions attach to indexing: a FILL_OR_DROP gather returns fill_value where the slice does
    not fit (instead of moving it inside), a CLIP scatter-add moves windows inside (instead of dropping them).
    Against plain numpy indexing.'''
    G, S = core.GatherDimensionNumbers, core.ScatterDimensionNumbers
    table = rng.random_sample((7, 5)).astype(np.float32)
    rows  = np.array([3, -1, 7, 0, 6, 100, -2**31], np.int64)
    inside = (rows >= 0) & (rows < 7)
    got = P.gather(table, rows[:, None].astype(np.int32), (G((1,), (0,), (0,))), (1, 5), mode='fill')
    assert np.array_equal(got[inside], table[rows[inside]]) and np.isnan(got[~inside]).all()
    got = P.gather(table.astype(np.int32) + 3, rows[:, None].astype(np.int32), (G((1,), (0,), (0,))), (1, 5), mode='FILL_OR_DROP')
    assert (got[~inside] == np.iinfo(np.int32).min).all() and np.array_equal(got[inside], (table.astype(np.int32) + 3)[rows[inside]])
    got = P.gather(table, rows[:, None].astype(np.int32), (G((1,), (0,), (0,))), (1, 5), mode='fill', fill_value=-2.5)
    assert (got[~inside] == -2.5).all()
    #windows of 2 x 3 at (r, c): they fit for r <= 5 and c <= 2
    starts = np.array([[0, 0], [5, 2], [6, 0], [2, 3], [-1, 1]], np.int32)
    got = P.gather(table, starts, G((1, 2), (), (0, 1)), (2, 3), mode='fill')
    for k, (r, c) in enumerate(starts):
        want = table[r:r + 2, c:c + 3] if 0 <= r <= 5 and 0 <= c <= 2 else np.full((2, 3), np.nan, np.float32)
        assert np.array_equal(got[k], want, equal_nan=True), k
    #the default mode moves the same windows inside
    assert np.array_equal(P.gather(table, starts, G((1, 2), (), (0, 1)), (2, 3))[2], table[5:7, 0:3])
    upd = rng.random_sample((7, 5)).astype(np.float32)
    want = table.astype(np.float64)
    np.add.at(want, np.clip(rows, 0, 6), upd)
    got = P.scatter_add(table, rows[:, None].astype(np.int32), upd, S((1,), (0,), (0,)), mode='clip')
    assert np.allclose(got, want, rtol=1e-6)
    dropped = table.astype(np.float64)
    np.add.at(dropped, rows[inside], upd[inside])
    assert np.allclose(P.scatter_add(table, rows[:, None].astype(np.int32), upd, S((1,), (0,), (0,))), dropped, rtol=1e-6)
    win = rng.random_sample((5, 2, 3)).astype(np.float32)
    want = table.astype(np.float64)
    for k, (r, c) in enumerate(starts):
        r, c = min(max(r, 0), 5), min(max(c, 0), 2)
        want[r:r + 2, c:c + 3] += win[k]
    assert np.allclose(P.scatter_add(table, starts, win, S((1, 2), (), (0, 1)), mode='clip'), want, rtol=1e-6)


def test_reductions_and_argmax_rules():
    x = rng.rand(5, 6, 7).astype(np.float32)
    assert np.allclose(P.reduce_sum(x, (0, 2)), x.astype(np.float64).sum(axis=(0, 2)), rtol=1e-6)
    assert np.array_equal(P.reduce_max(x, (1,)), x.max(axis=1))
    assert np.array_equal(P.reduce_min(x, (0, 1)), x.min(axis=(0, 1)))
    assert np.allclose(P.reduce_prod(x + 0.5, (2,)), (x + 0.5).astype(np.float64).prod(axis=2), rtol=1e-6)
    assert np.array_equal(P.argmax(x, (1,)), x.argmax(axis=1).astype(np.int32))
    assert np.array_equal(P.argmin(x, (2,)), x.argmin(axis=2).astype(np.int32))
    t = np.array([[1, 3, 3, 2], [np.nan, 5, np.nan, 1], [2, 2, 2, 2]], np.float32)
    assert P.argmax(t, (1,)).tolist() == [1, 0, 0]       #first of ties; first NaN wins
    assert P.argmin(t, (1,)).tolist() == [0, 0, 0]
    assert np.isnan(P.reduce_max(t, (1,))[1])
    z = np.array([[-1, -0.0, 0.0, -2], [-1, 0.0, -0.0, -2], [1, 0.0, -0.0, 2]], np.float32)
    assert P.argmax(z, (1,)).tolist() == [1, 1, 3]       #the two zeros are equal: the first of them wins, whatever its sign
    assert P.argmin(-z, (1,)).tolist() == [1, 1, 3]


def test_integer_and_shift_semantics():
    lit = GOLDEN['reference_test_literals']
    assert int(P.shift_right_logical(np.int32(1), np.int32(32))) == lit['shift_right_logical_1_32']
    a = np.arange(-777, 777).astype(np.int32)
    assert np.array_equal(P.shift_left(a, np.int32(1)), a * 2)
    assert np.array_equal(P.shift_right_arithmetic(a, np.int32(1)), a >> 1)
    assert np.array_equal(P.shift_right_logical(a, np.int32(1)), (a.view(np.uint32) >> 1).view(np.int32))
    assert np.array_equal(P.shift_right_logical(a.view(np.uint32), np.uint32(9)), a.view(np.uint32) >> 9)
    assert int(P.div(np.int32(-7), np.int32(2))) == -3 and int(P.rem(np.int32(-7), np.int32(2))) == -1
    assert np.array_equal(P.integer_pow(np.array([-3, 2, 1000], np.int32), 5), np.array([-243, 32, (1000**5 + 2**31) % 2**32 - 2**31], np.int32))
    assert np.array_equal(P.convert_element_type(np.array([1.9, -1.9, np.nan, 3e10], np.float32), np.int32),
                          np.array([1, -1, 0, 2**31 - 1], np.int32))
    assert np.array_equal(P.select(np.array([True, False]), np.array([np.inf, 1.0], np.float32), np.array([2.0, np.nan], np.float32)),
                          np.array([np.inf, np.nan], np.float32), equal_nan=True)
    assert np.array_equal(P.max(np.array([np.nan, 1.0], np.float32), np.array([0.0, np.nan], np.float32)),
                          np.array([np.nan, np.nan], np.float32), equal_nan=True)


def test_whole_program_identities():
    rng = np.random.RandomState(77)          #(a generator of its own: the values do not depend on which tests ran before)
    x = rng.rand(6, 10).astype(np.float32) * 4
    closed = mj.make_jaxpr(lambda v: mj.nn.softmax(v))(x)
    (p,) = eval_closed_jaxpr(closed, x)
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    assert np.allclose(p, e / e.sum(axis=1, keepdims=True), rtol=1e-6) and np.allclose(p.sum(axis=1), 1, atol=1e-6)
    c = 8
    args = [rng.rand(2, 3, 3, c).astype(np.float32)] + [rng.rand(c).astype(np.float32) + 0.5 for _ in range(4)]
    closed = mj.make_jaxpr(lambda v, s, b, m, var: mj.nn.batch_norm_inference(v, s, b, m, var))(*args)
    (y,) = eval_closed_jaxpr(closed, *args)
    v, s, b, m, var = [a.astype(np.float64) for a in args]
    assert np.allclose(y, (v - m) / np.sqrt(var + 1e-5) * s + b, rtol=1e-5, atol=1e-6)          #(float32 result; sums of terms of opposite sign come close to 0)
    closed = mj.make_jaxpr(lambda a, i: jnp.take_along_axis(a, i, axis=-1))(x, np.zeros((6, 1), np.int32))
    idx = rng.randint(0, 10, size=(6, 1)).astype(np.int32)
    (t,) = eval_closed_jaxpr(closed, x, idx)
    assert np.array_equal(t, np.take_along_axis(x, idx, axis=-1))


def test_reductions_over_no_elements_return_the_init_value():
    '''XLA reduces with an init value (lax.reduce_max: -inf / the smallest integer, reduce_min: +inf / the largest,
    reduce_sum: 0), which is what remains when the reduced range is empty.'''
    from oracle import primitives as P
    assert np.array_equal(P.reduce_max(np.zeros((3, 0), np.float32), (1,)), np.full(3, -np.inf, np.float32))
    assert np.array_equal(P.reduce_min(np.zeros((3, 0), np.float32), (1,)), np.full(3, np.inf, np.float32))
    assert np.array_equal(P.reduce_max(np.zeros((2, 0), np.int32), (1,)), np.full(2, -2**31, np.int32))
    assert np.array_equal(P.reduce_min(np.zeros((2, 0), np.int32), (1,)), np.full(2, 2**31 - 1, np.int32))
    assert np.array_equal(P.reduce_sum(np.zeros((0, 4), np.float32), (0,)), np.zeros(4, np.float32))
    #and nothing changes where there are elements
    x = np.array([[1.0, -3.0, np.nan], [2.0, 5.0, -1.0]], np.float32)
    assert np.array_equal(P.reduce_max(x, (1,)), np.array([np.nan, 5.0], np.float32), equal_nan=True)
    assert np.array_equal(P.reduce_min(x, (0,)), np.array([1.0, -3.0, np.nan], np.float32), equal_nan=True)


def test_convolution_with_a_crop_that_reaches_beyond_the_input():
    '''Negative padding larger than the input: the padded axis still has in + lo + hi positions, all of them
    outside the input. Brute force over the definition (element i of the padded axis is element i - lo).'''
    from oracle import primitives as P
    rng = np.random.default_rng(3)
    x, w = rng.standard_normal((2, 1, 5, 3)), rng.standard_normal((1, 2, 3, 4))
    padding = ((-2, 2), (1, 0))
    dn = ((0, 3, 1, 2), (3, 2, 0, 1), (0, 3, 1, 2))
    got = P.conv_general_dilated(x, w, (1, 1), padding, (1, 1), (1, 1), dn)
    Ho, Wo = 1 - 2 + 2 - 1 + 1, 5 + 1 + 0 - 2 + 1
    want = np.zeros((2, Ho, Wo, 4))
    for b in range(2):
        for ho in range(Ho):
            for wo in range(Wo):
                for ky in range(1):
                    for kx in range(2):
                        y, xx = ho + ky - padding[0][0], wo + kx - padding[1][0]
                        if 0 <= y < 1 and 0 <= xx < 5:
                            want[b, ho, wo] += x[b, y, xx] @ w[ky, kx]
    assert got.shape == want.shape and np.allclose(got, want, atol=1e-6)
    assert not np.any(got)                                  #every tap of every position lies outside the input
