'''Training-path programs: the primitives autodiff adds to a jaxpr (pad, select_and_scatter_add, convolutions
with lhs / rhs dilation, reversed kernels and permuted dimension numbers, transposed dot_generals, add_any) and
whole SGD steps, the way the reference runs them in tests/test_elegy_mlp.py:87-129 and
tests/test_elegy_conv.py:51-94. CPU part: the differentiation rules and the oracle against torch autograd
(an independent implementation); GPU part: the HIP path against the oracle on the same programs.'''
import numpy as np
import pytest

from oracle import primitives as P
from oracle.eval_jaxpr import eval_closed_jaxpr
from tests.common import check_against_oracle, assert_tree_close, oracle_outputs
from vkjax_amd import kernels as K, minijax as mj, workloads as W
from vkjax_amd.jaxpr_interpreter import JaxprInterpreter

lax, jnp, nn = mj.lax, mj.numpy, mj.nn
rng = np.random.RandomState(99)
random = lambda shape: rng.random_sample(shape).astype(np.float32)


def pad0(x): return lax.pad(x, 0.0, ((1, 2, 0), (0, 0, 0)))
def pad1(x): return lax.pad(x, -1.5, ((0, 0, 0), (2, 1, 1), (1, 0, 2), (0, 0, 0)))
def pad2(x): return lax.pad(x, 7.0, ((-1, 2, 0), (1, -2, 1), (0, 3, 0)))
def pad3(x, v): return lax.pad(x, v, ((0, 0, 3),))
def pad4(x): return lax.pad(x + 1, 0, ((2, 2, 1), (0, 1, 0)))
def pad5(x): return lax.pad(x, 0.5, ((0, 0, 0), (1, 2, 0), (3, 1, 0), (0, 0, 0)))             #untouched channels fold into the padded width
def pad6(x): return lax.pad(x, 0.0, ((0, 0, 0), (-1, 1, 0), (-2, -1, 0), (0, 0, 0), (0, 0, 0)))   #crops; two trailing dimensions fold
def pad7(x): return lax.pad(x, 2.0, ((1, 0, 0), (0, 0, 0), (0, 1, 1), (0, 0, 0), (2, 0, 0), (0, 0, 0)))   #six dimensions
def pad8(x): return lax.pad(x, 0.0, ((0, 0, 0), (0, 0, 0), (0, 0, 0)))                          #nothing to do: one dimension
def pad9(x): return lax.pad(x, 1.0, ((0, 0, 0), (0, 0, 1), (0, 0, 1), (0, 0, 0)))             #interior padding before untouched channels
def pool_grad(window, strides, padding, select=None):
    def f(g, x): return lax.select_and_scatter_add(g, x, select or lax.ge_p, window, strides, padding)
    return f

def _pooled(shape, window, strides, padding):
    return [(n + lo + hi - w) // s + 1 for n, w, s, (lo, hi) in zip(shape, window, strides, padding)]

_P = ((0, 0), (0, 1), (0, 1), (0, 0))
_SAME = ((0, 0), (1, 1), (1, 1), (0, 0))
_ties = np.round(random([2, 9, 9, 8]) * 3)          #many equal values: the first position of a window must win
pool_cases = [
    ('3x3 s2 pad hi C8',   (1, 3, 3, 1), (1, 2, 2, 1), _P,    random([2, 11, 12, 8]) - 0.5, None),
    ('3x3 s2 SAME C5',     (1, 3, 3, 1), (1, 2, 2, 1), _SAME, random([2, 9, 10, 5]) - 0.5, None),
    ('2x2 s2 C4',          (1, 2, 2, 1), (1, 2, 2, 1), ((0, 0),) * 4, random([3, 8, 6, 4]), None),
    ('3x3 s1 ties',        (1, 3, 3, 1), (1, 1, 1, 1), _SAME, _ties, None),
    ('min pooling',        (1, 2, 2, 1), (1, 1, 1, 1), ((0, 0),) * 4, random([2, 6, 7, 4]), lax.le_p),
    ('window over all dims', (2, 2, 1, 3), (1, 2, 1, 2), ((1, 0), (0, 0), (0, 0), (1, 1)), random([3, 6, 4, 7]), None),
    ('2-D array',          (3, 2), (2, 1), ((1, 1), (0, 1)), random([13, 9]), None),
]
pad_cases = [(pad0, [random([5, 8])]), (pad1, [random([2, 5, 6, 8])]), (pad2, [random([4, 7, 5])]),
             (pad3, [np.arange(9, dtype=np.int32), np.int32(-7)]), (pad4, [random([6, 12])]),
             (pad5, [random([2, 5, 6, 8])]), (pad6, [random([2, 6, 7, 3, 4])]), (pad7, [random([2, 3, 4, 2, 3, 4])]),
             (pad8, [random([3, 4, 5])]), (pad9, [random([2, 4, 5, 8])])]


def small_convnet_inputs():
    return W.convnet_train_inputs(batch=3, size=16, channels=(3, 8, 12), classes=5)


def tiny_resnet_inputs():
    return W.resnet50_train_inputs(batch=2, size=32, num_classes=10, width_scale=0.125)


def small_mlp_inputs():
    return W.mlp_train_inputs(batch=16, sizes=(40, 32, 24, 5))


# ------------------------------------------------------------------ CPU: pins of the oracle and of the differentiation rules

def test_select_and_scatter_add_oracle_equals_torch_max_pool_backward():
    torch = pytest.importorskip('torch')
    x = random([2, 9, 11, 3])
    xt = torch.tensor(x.transpose(0, 3, 1, 2), requires_grad=True)
    y = torch.nn.functional.max_pool2d(xt, 3, 2, padding=1)
    g = random(tuple(y.shape))
    y.backward(torch.tensor(g))
    mine = P.select_and_scatter_add(g.transpose(0, 2, 3, 1), x, lax.ge_p, (1, 3, 3, 1), (1, 2, 2, 1), _SAME)
    assert np.array_equal(mine, xt.grad.numpy().transpose(0, 2, 3, 1))
    #ties: the whole cotangent of a window goes to its first maximum
    flat = P.select_and_scatter_add(np.ones((1, 1), np.float32), np.zeros((2, 2), np.float32), lax.ge_p, (2, 2), (1, 1), ((0, 0), (0, 0)))
    assert flat.tolist() == [[1, 0], [0, 0]]


def test_pad_oracle_against_numpy_and_brute_force():
    x = random([3, 5, 4])
    assert np.array_equal(P.pad(x, 0.0, ((1, 2, 0), (3, 0, 0), (0, 1, 0))), np.pad(x, ((1, 2), (3, 0), (0, 1))))
    config = ((1, 2, 0), (0, 0, 1), (-1, 1, 2))
    shape = [n + (n - 1) * it + lo + hi for n, (lo, hi, it) in zip(x.shape, config)]
    brute = np.full(shape, 7.0, np.float32)
    for idx in np.ndindex(*x.shape):
        o = tuple(lo + i * (it + 1) for i, (lo, hi, it) in zip(idx, config))
        if all(0 <= p < s for p, s in zip(o, shape)):
            brute[o] = x[idx]
    assert np.array_equal(P.pad(x, 7.0, config), brute)


def _torch_convnet_grads(params, x, onehot):
    import torch
    F = torch.nn.functional
    T = lambda a: torch.tensor(a, dtype=torch.float64, requires_grad=True)
    tp, xt = {k: T(v) for k, v in params.items()}, T(x)
    y = F.conv2d(xt.permute(0, 3, 1, 2), tp['w1'].permute(3, 2, 0, 1), stride=2, padding=1)
    y = torch.relu(y * tp['scale'][None, :, None, None] + tp['shift'][None, :, None, None])
    y = F.max_pool2d(F.pad(y, (0, 1, 0, 1), value=-np.inf), 3, 2)
    y = torch.relu(F.conv2d(y, tp['w2'].permute(3, 2, 0, 1), padding=1))
    y = F.avg_pool2d(y, 2, 2).mean(dim=(2, 3))
    loss = F.cross_entropy(y @ tp['w3'] + tp['b3'], torch.tensor(onehot.argmax(1)))
    loss.backward()
    return float(loss), {k: v.grad.numpy() for k, v in tp.items()}, xt.grad.numpy()


def test_convnet_gradients_equal_torch_autograd():
    pytest.importorskip('torch')
    params, x, onehot = small_convnet_inputs()
    f = lambda p, x, o: mj.value_and_grad(W.convnet_loss, argnums=(0, 1))(p, x, o)
    closed = mj.make_jaxpr(f)(params, x, onehot)
    names = set(e.primitive.name for e in closed.jaxpr.eqns)
    assert {'select_and_scatter_add', 'pad', 'rev', 'add_any', 'conv_general_dilated'} <= names
    outs = eval_closed_jaxpr(closed, *mj.tree_leaves([params, x, onehot]))
    loss, grads, gx = _torch_convnet_grads(params, x, onehot)
    assert abs(float(outs[0]) - loss) < 1e-6
    for name, g in zip(sorted(params), outs[1:]):
        assert np.allclose(g, grads[name], rtol=1e-4, atol=1e-7), name
    assert np.allclose(outs[-1], gx, rtol=1e-4, atol=1e-7)


def test_conv_gradient_with_padding_beyond_kernel_equals_torch():
    '''Padding >= kernel size makes the input gradient a convolution with negative (cropping) padding.'''
    torch = pytest.importorskip('torch')
    F = torch.nn.functional
    x, w = random([2, 9, 8, 4]) - 0.5, random([3, 2, 4, 8]) - 0.5
    padding = ((3, 1), (2, 0))
    def loss(x, w):
        y = lax.conv_general_dilated(x, w, window_strides=(1, 1), padding=padding, dimension_numbers=W.NHWC)
        return jnp.sum(y * y) * 0.5
    closed = mj.make_jaxpr(lambda x, w: mj.grad(loss, argnums=(0, 1))(x, w))(x, w)
    assert any(e.primitive.name == 'conv_general_dilated' and min(min(p) for p in e.params['padding']) < 0 for e in closed.jaxpr.eqns)
    gx, gw = eval_closed_jaxpr(closed, x, w)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    y = F.conv2d(F.pad(xt.permute(0, 3, 1, 2), (2, 0, 3, 1)), wt.permute(3, 2, 0, 1))
    (y * y).sum().mul(0.5).backward()
    assert np.allclose(gx, xt.grad.numpy(), rtol=1e-4, atol=1e-6) and np.allclose(gw, wt.grad.numpy(), rtol=1e-4, atol=1e-6)


def test_mlp_gradients_equal_torch_autograd():
    torch = pytest.importorskip('torch')
    params, x, onehot = small_mlp_inputs()
    closed = mj.make_jaxpr(lambda p, x, o: mj.value_and_grad(W.mlp_loss)(p, x, o))(params, x, onehot)
    outs = eval_closed_jaxpr(closed, *mj.tree_leaves([params, x, onehot]))
    T = lambda a: torch.tensor(a, dtype=torch.float64, requires_grad=True)
    tp = {k: T(v) for k, v in params.items()}
    h = torch.relu(torch.tensor(x, dtype=torch.float64) @ tp['w1'] + tp['b1'])
    h = torch.relu(h @ tp['w2'] + tp['b2'])
    loss = torch.nn.functional.cross_entropy(h @ tp['w3'] + tp['b3'], torch.tensor(onehot.argmax(1)))
    loss.backward()
    assert abs(float(outs[0]) - float(loss)) < 1e-6
    for name, g in zip(sorted(params), outs[1:]):
        assert np.allclose(g, tp[name].grad.numpy(), rtol=1e-4, atol=1e-7), name


def test_gradient_rules_of_other_primitives_equal_torch_autograd():
    '''Rules not reached by the two networks: div, sqrt, rsqrt, logistic, integer_pow, reduce_max, transpose,
    slice, concatenate, gather, min, select.'''
    torch = pytest.importorskip('torch')
    def f(a, b, idx):
        t = lax.transpose(a, (1, 0))[1:4:2, :]                               #[2, 5]
        u = jnp.concatenate([t, lax.sqrt(b[:2] + 2.0)], axis=0)              #[4, 5]
        v = lax.logistic(u) / (1.5 + lax.integer_pow(u, 2)) + lax.rsqrt(u * u + 1.0)
        w = jnp.minimum(v, 0.9 * jnp.max(v, axis=1, keepdims=True))
        rows = b[idx]                                                        #gather [3, 5]
        s = lax.select(lax.gt(rows, 0.5), rows * rows, -rows)
        return jnp.sum(w * w) + jnp.sum(s) * 0.25
    a, b = random([5, 6]) + 0.1, random([4, 5])
    idx = np.array([3, 0, 3], np.int32)
    closed = mj.make_jaxpr(lambda a, b, i: mj.value_and_grad(f, argnums=(0, 1))(a, b, i))(a, b, idx)
    value, ga, gb = eval_closed_jaxpr(closed, a, b, idx)
    at, bt = (torch.tensor(v, dtype=torch.float64, requires_grad=True) for v in (a, b))
    t = at.T[1:4:2, :]
    u = torch.cat([t, torch.sqrt(bt[:2] + 2.0)], dim=0)
    v = torch.sigmoid(u) / (1.5 + u ** 2) + torch.rsqrt(u * u + 1.0)
    w = torch.minimum(v, 0.9 * v.amax(dim=1, keepdim=True))
    rows = bt[torch.tensor(idx, dtype=torch.long)]
    s = torch.where(rows > 0.5, rows * rows, -rows)
    total = (w * w).sum() + s.sum() * 0.25
    total.backward()
    assert abs(float(value) - float(total)) < 1e-5
    assert np.allclose(ga, at.grad.numpy(), rtol=1e-4, atol=1e-6) and np.allclose(gb, bt.grad.numpy(), rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize('name', ['mlp_train', 'convnet_train'])
def test_training_steps_plan_at_full_size(name):
    fn, make_inputs = W.WORKLOADS[name]
    interp = JaxprInterpreter(mj.make_jaxpr(fn)(*make_inputs()), plan_only=True)
    kernels = [l.kernel for l in interp.launches]
    assert any(k.startswith('conv_gemm') for k in kernels)
    if name == 'convnet_train':
        assert 'select_window2d_3x3_v4' in kernels and 'scatter_selected2d_3x3_s2_v4' in kernels and any(k.startswith('pad_nd') for k in kernels), kernels


@pytest.mark.parametrize('f,args', pad_cases, ids=[c[0].__name__ for c in pad_cases])
def test_pad_plans(f, args):
    JaxprInterpreter(mj.make_jaxpr(f)(*args), plan_only=True)


def test_pad_folds_untouched_dimensions():
    from vkjax_amd import kernels as K
    #NHWC with padded height and width: [N, H, W * C]; the vector kernel, because low * C is a multiple of 4
    assert K._merged_pad_dims((2, 8, 10, 8), (2, 5, 6, 8), ((0, 0, 0), (1, 2, 0), (3, 1, 0), (0, 0, 0))) == [(2, 2, 0, 1), (8, 5, 1, 1), (80, 48, 24, 1)]
    #interior padding keeps its dimension apart from the channels
    assert K._merged_pad_dims((2, 7, 8), (2, 4, 8), ((0, 0, 0), (0, 0, 1), (0, 0, 0))) == [(2, 2, 0, 1), (7, 4, 0, 2), (8, 8, 0, 1)]
    #nothing padded: one dimension
    assert K._merged_pad_dims((3, 4, 5), (3, 4, 5), ((0, 0, 0),) * 3) == [(60, 60, 0, 1)]
    #a crop in front of two untouched dimensions
    assert K._merged_pad_dims((3, 3, 4), (5, 3, 4), ((-1, -1, 0), (0, 0, 0), (0, 0, 0))) == [(36, 60, -12, 1)]


# ------------------------------------------------------------------ GPU parity

@pytest.mark.gpu
@pytest.mark.parametrize('f,args', pad_cases, ids=[c[0].__name__ for c in pad_cases])
def test_pad_hip(f, args):
    print(f'case: {f.__name__}', flush=True)
    check_against_oracle(f, args, exact=True)


@pytest.mark.gpu
@pytest.mark.parametrize('desc,window,strides,padding,x,select', pool_cases, ids=[c[0] for c in pool_cases])
def test_select_and_scatter_add_hip(desc, window, strides, padding, x, select):
    from vkjax_amd import kernels as K
    g = random(_pooled(x.shape, window, strides, padding)) + 0.25
    kernels = []
    #the kernels for [batch, y, x, channels] where they apply (with the one for groups of 2 x 2 elements under 3 x 3 windows at a
    #stride of 2, and without it), and the general ones
    for two_d in (None, False, 'elements'):
        print(f'case: {desc}, 2-D kernels {two_d}', flush=True)
        with K.overrides(pool_gradient_2d=two_d):
            _, _, fn = check_against_oracle(pool_grad(window, strides, padding, select), [g, x], exact=True)
        kernels.append([l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches if 'select' in l.kernel])
    assert all('2d' not in k for k in kernels[1])
    applies = len(window) == 4 and (window[0], window[3]) == (1, 1) and window[1:3] in ((3, 3), (2, 2)) and x.shape[3] % 4 == 0
    assert all('2d' in k for k in kernels[0]) == applies and bool(kernels[0]), (desc, kernels)
    assert all('2d' in k for k in kernels[2]) == applies and not any(k.endswith('_s2_v4') for k in kernels[2]), (desc, kernels)
    assert any(k.endswith('3x3_s2_v4') for k in kernels[0]) == (applies and window[1:3] == (3, 3) and strides[1:3] == (2, 2)), (desc, kernels)


@pytest.mark.gpu
def test_conv_gradient_forms_hip():
    '''Input and kernel gradients of strided, padded and dilated convolutions (the convolutions autodiff emits:
    lhs dilation, rhs dilation, reversed kernels, permuted dimension numbers, padding that can be negative).'''
    cases = [((2, 9, 10, 4), (3, 3, 4, 6), (2, 2), ((1, 1), (1, 1)), (1, 1)),
             ((2, 12, 11, 8), (3, 2, 8, 16), (1, 2), ((0, 2), (1, 0)), (2, 1)),
             ((1, 8, 8, 3), (1, 1, 3, 5), (2, 2), ((0, 0), (0, 0)), (1, 1)),
             ((2, 10, 9, 16), (3, 3, 16, 8), (3, 2), ((2, 1), (0, 1)), (1, 1)),
             ((2, 9, 8, 4), (3, 2, 4, 8), (1, 1), ((3, 1), (2, 0)), (1, 1))]        #padding >= kernel size: the input gradient crops
    for xs, ws, strides, padding, rhs_dilation in cases:
        print(f'case: conv gradients x{xs} w{ws} strides{strides} padding{padding} rhs_dilation{rhs_dilation}', flush=True)
        def loss(x, w):
            y = lax.conv_general_dilated(x, w, window_strides=strides, padding=padding, rhs_dilation=rhs_dilation, dimension_numbers=W.NHWC)
            return jnp.sum(y * y) * 0.5
        f = lambda x, w: mj.grad(loss, argnums=(0, 1))(x, w)
        check_against_oracle(f, [random(xs) - 0.5, random(ws) - 0.5], rtol=1e-4, atol=1e-5)


WGRAD_CASES = [   #x, kernel, strides, padding, rhs_dilation; the loader variant in the name
    ('aa', (4, 12, 12, 8), (3, 3, 8, 16), (1, 1), ((1, 1), (1, 1)), (1, 1)),
    ('aa strided', (3, 17, 15, 4), (3, 3, 4, 8), (2, 2), ((1, 1), (0, 1)), (1, 1)),
    ('sa stem', (2, 20, 20, 3), (7, 7, 3, 8), (2, 2), ((3, 3), (3, 3)), (1, 1)),
    ('as', (2, 10, 10, 8), (1, 1, 8, 10), (1, 1), ((0, 0), (0, 0)), (1, 1)),
    ('ss dilated', (2, 13, 11, 5), (2, 3, 5, 7), (1, 1), ((1, 1), (2, 2)), (2, 2)),
    ('aa wide', (2, 10, 10, 72), (3, 3, 72, 136), (1, 1), ((1, 1), (1, 1)), (1, 1)),
]


def _kernel_gradient_function(strides, padding, rhs_dilation):
    def loss(x, w):
        y = lax.conv_general_dilated(x, w, window_strides=strides, padding=padding, rhs_dilation=rhs_dilation, dimension_numbers=W.NHWC)
        return jnp.sum(y * y) * 0.5
    return lambda x, w: mj.grad(loss, argnums=1)(x, w)


@pytest.mark.parametrize('case', WGRAD_CASES, ids=[c[0] for c in WGRAD_CASES])
def test_kernel_gradients_take_the_wgrad_kernel(case):
    name, xs, ws, strides, padding, rhs_dilation = case
    closed = mj.make_jaxpr(_kernel_gradient_function(strides, padding, rhs_dilation))(random(xs), random(ws))
    kernels = [l.kernel for l in JaxprInterpreter(closed, plan_only=True).launches]
    assert f'wgrad_gemm_64x64_{name[:2]}' in kernels, kernels


def test_dense_layer_weight_gradient_takes_the_wgrad_kernel():
    closed = mj.make_jaxpr(lambda x, g: lax.dot_general(x, g, (((0,), (0,)), ((), ()))))(random([256, 40]), random([256, 10]))
    kernels = [l.kernel for l in JaxprInterpreter(closed, plan_only=True).launches]
    assert kernels[0] == 'wgrad_gemm_64x64_as' and (len(kernels) == 1 or kernels[1].startswith('reduce_cols')), kernels


@pytest.mark.gpu
@pytest.mark.parametrize('case', WGRAD_CASES, ids=[c[0] for c in WGRAD_CASES])
def test_kernel_gradient_hip(case):
    name, xs, ws, strides, padding, rhs_dilation = case
    print(f'case: kernel gradient {name} x{xs} w{ws}', flush=True)
    #integer-valued operands: every product and partial sum is exact, so the result does not depend on the split
    x = np.round(random(xs) * 8 - 4).astype(np.float32)
    w = np.round(random(ws) * 4 - 2).astype(np.float32)
    check_against_oracle(_kernel_gradient_function(strides, padding, rhs_dilation), [x, w], exact=True)
    #real-valued operands (their own seed: the data must not depend on which tests ran before). The gradients reach
    #+-12 as sums of some 10^5 products that cancel, so the absolute floor is 4e-6 of that range
    own = np.random.RandomState(len(name) + sum(xs) + sum(ws))
    xr, wr = (own.random_sample(shape).astype(np.float32) - 0.5 for shape in (xs, ws))
    check_against_oracle(_kernel_gradient_function(strides, padding, rhs_dilation), [xr, wr], rtol=1e-4, atol=5e-5)


@pytest.mark.gpu
def test_rows_contracted_dot_hip():
    for k, m, n in ((256, 40, 10), (1000, 65, 64), (4096, 128, 256), (130, 3, 5)):
        print(f'case: x^T g with {k} rows, {m} x {n}', flush=True)
        f = lambda x, g: lax.dot_general(x, g, (((0,), (0,)), ((), ())))
        x = np.round(random([k, m]) * 8 - 4).astype(np.float32)
        g = np.round(random([k, n]) * 8 - 4).astype(np.float32)
        check_against_oracle(f, [x, g], exact=True)
        check_against_oracle(f, [random([k, m]) - 0.5, random([k, n]) - 0.5], rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize('name,make_inputs', [('mlp_train', small_mlp_inputs), ('convnet_train', small_convnet_inputs),
                                              ('resnet50_train', tiny_resnet_inputs)])
def test_training_step_hip_matches_oracle(name, make_inputs):
    '''One SGD step: loss and every updated parameter against the oracle (reference tests/test_elegy_mlp.py:87-129
    compares exactly these after train_on_batch, rtol 1e-5 / atol 1e-6 there; contractions here use the tolerance
    of dot / conv).'''
    print(f'case: {name}', flush=True)
    fn, _ = W.WORKLOADS[name]
    #the 53-layer network accumulates the rounding differences of its contractions: the tolerance of its logits
    rtol, atol = (1e-3, 1e-5) if name == 'resnet50_train' else (1e-4, 1e-6)
    for fuse in (True, False):
        check_against_oracle(fn, make_inputs(), rtol=rtol, atol=atol, fuse=fuse)


@pytest.mark.gpu
@pytest.mark.parametrize('name,make_inputs,atol', [('mlp_train', small_mlp_inputs, 1e-6), ('convnet_train', small_convnet_inputs, 5e-5)])
def test_every_variable_of_a_training_step(name, make_inputs, atol):
    '''The reference's deep inspection of a training step (tests/common.py:67-81, tests/test_elegy_mlp.py:120-129,
    tests/test_elegy_conv.py:51-94): the program is built again without buffer reuse (and here without fusion, so
    that every equation keeps a launch and a buffer of its own), run with return_all=True, and EVERY variable of
    the jaxpr - not only the results - is compared with the evaluator's environment, at the reference's tolerances
    (numpy's default rtol 1e-5 with atol 1e-6 for the MLP, 5e-5 for the conv net).'''
    from vkjax_amd.minijax import tree_util
    fn, _  = W.WORKLOADS[name]
    args   = make_inputs()
    closed = mj.make_jaxpr(fn)(*args)
    interp = JaxprInterpreter(closed, reuse_buffers=False, fuse=False)
    outs, envpred = interp.run(*args, return_all=True)
    outs_true, envtrue = eval_closed_jaxpr(closed, *tree_util.tree_leaves(args), return_env=True)
    assert len(envtrue) >= len(closed.jaxpr.eqns) and len(outs) == len(outs_true)
    checked, worst = 0, (0.0, '')
    for var, vtrue in envtrue.items():
        if np.size(vtrue) == 0:
            continue
        vpred = envpred.get(var)
        assert vpred is not None, f'{var}: no buffer'
        assert np.shape(vpred) == np.shape(vtrue) and vpred.dtype == vtrue.dtype, (var, np.shape(vpred), np.shape(vtrue), vpred.dtype, vtrue.dtype)
        if vtrue.dtype.kind in 'iub':
            assert np.array_equal(vpred, vtrue), var
        else:
            err = float(np.max(np.abs(vpred.astype(np.float64) - vtrue) / (atol + 1e-5 * np.abs(vtrue))))
            worst = (err, str(var)) if err > worst[0] else worst
            assert err <= 1.0, f'{var} {np.shape(vtrue)}: |err| / (atol + rtol |y|) = {err:.3g}'
        checked += 1
    print(f'{name}: {checked} variables, worst |err| / (atol + rtol |y|) = {worst[0]:.3g} at {worst[1]}', flush=True)
    assert checked >= len(closed.jaxpr.eqns)


@pytest.mark.gpu
def test_repeated_training_steps_reduce_the_loss():
    import vkjax_amd
    params, x, onehot = small_mlp_inputs()
    step = vkjax_amd.wrap(lambda p, x, o: W.mlp_train_step(p, x, o, lr=0.2), frontend='minijax')
    losses = []
    for _ in range(10):
        loss, params = step(params, x, onehot)
        losses.append(float(loss))
    assert losses[-1] < 0.7 * losses[0], losses


def _scale_shift_relu_net(batch=6, size=10, channels=(8, 12, 12), seed=3):
    '''Three layers of 1x1 convolution -> per-channel scale and shift -> ReLU with a residual connection around
    the last one, and a squared-error loss: the shapes of a batch norm with fixed statistics in a residual block.'''
    rng = np.random.default_rng(seed)
    params = []
    cin = 4
    for c in channels:
        params.append({'w': (rng.standard_normal((1, 1, cin, c)) / np.sqrt(cin)).astype(np.float32),
                       'scale': (1 + 0.1 * rng.standard_normal(c)).astype(np.float32), 'bias': (0.1 * rng.standard_normal(c)).astype(np.float32),
                       'mean': (0.1 * rng.standard_normal(c)).astype(np.float32), 'var': (1 + 0.1 * rng.random(c)).astype(np.float32)})
        cin = c
    x = rng.standard_normal((batch, size, size, 4)).astype(np.float32)
    return params, x


def _scale_shift_relu_loss(trainable, fixed, x):
    h = x
    for k, (p, s) in enumerate(zip(trainable, fixed)):
        y = mj.lax.conv_general_dilated(h, p['w'], (1, 1), 'VALID', dimension_numbers=('NHWC', 'HWIO', 'NHWC'))
        y = (y - s['mean']) * (p['scale'] * mj.lax.rsqrt(s['var'] + 1e-5)) + p['bias']
        h = mj.nn.relu(y + h) if k == 2 else mj.nn.relu(y)
    return mj.numpy.sum(h * h)


def _scale_shift_relu_step(params, x):
    trainable = [{k: p[k] for k in ('w', 'scale', 'bias')} for p in params]
    fixed     = [{k: p[k] for k in ('mean', 'var')} for p in params]
    loss, grads = mj.value_and_grad(_scale_shift_relu_loss)(trainable, fixed, x)
    new = [{k: p[k] - np.float32(0.01) * g[k] for k in p} for p, g in zip(trainable, grads)]
    return loss, new


def test_convnet_step_keeps_its_batched_launches():
    '''The conv-net SGD step at its benchmark size: 39 launches, three of them batches of chains and column sums
    (the sums of the kernel gradients' slices and the parameter updates wait for the end of the step and share
    launches).'''
    from vkjax_amd.jaxpr_interpreter import JaxprInterpreter
    closed = mj.make_jaxpr(W.convnet_train_step)(*W.convnet_train_inputs())
    kernels = [l.kernel for l in JaxprInterpreter(closed, plan_only=True).launches]
    assert len(kernels) == 39 and sum('batch' in k for k in kernels) == 3, kernels


def test_scale_relu_backward_and_small_chain_batches_are_planned():
    import vkjax_amd
    f = vkjax_amd.wrap(_scale_shift_relu_step, frontend='minijax', plan_only=True)
    interp, _ = f._get_or_create_jaxpr_interpreter(_scale_shift_relu_net())
    kernels = [l.kernel for l in interp.launches]
    assert sum(k.startswith('scale_relu_backward') for k in kernels) == 2, kernels       #the two plain layers
    assert sum(k.startswith('scale_backward') for k in kernels) == 1, kernels            #the one whose cotangent the shortcut shares
    assert any(k.startswith('ew_chain_batch') for k in kernels), kernels
    assert any(k.startswith('reduce_cols_fsum_batch') for k in kernels), kernels        #the second stages of the column sums
    sums = next(l for l in interp.launches if l.kernel.startswith('reduce_cols_fsum_batch'))
    assert K.batch_table(sums, lambda b: 0x1000).nbytes == 56 * len(sums.members)
    plain = vkjax_amd.wrap(_scale_shift_relu_step, frontend='minijax', plan_only=True, fuse=False)
    unfused, _ = plain._get_or_create_jaxpr_interpreter(_scale_shift_relu_net())
    assert len(kernels) < len(unfused.launches) - 20
    #the table of a batch launch: one 432-byte entry per member, first workgroups ascending from 0
    batch = next(l for l in interp.launches if l.members and l.kernel.startswith('ew_chain_batch'))
    table = K.batch_table(batch, lambda b: 0x1000)
    assert table.nbytes == 432 * len(batch.members)
    firsts = table.reshape(len(batch.members), 108)[:, 0]
    assert firsts[0] == 0 and list(firsts) == list(np.cumsum([0] + [m.grid[0] for m in batch.members[:-1]]))
    assert batch.grid[0] == sum(m.grid[0] for m in batch.members)


@pytest.mark.gpu
def test_scale_relu_backward_and_small_chain_batches_keep_every_bit():
    '''The fused backward pass of scale/shift/ReLU adds in the order of the column sums it replaces, and batching
    small chains only changes which launch evaluates them: the step's results equal the unfused ones exactly,
    and both are within tolerance of the oracle. Second size: columns not a multiple of four (the v1 kernels).'''
    import vkjax_amd
    for kwargs in (dict(), dict(batch=3, size=7, channels=(6, 10, 10), seed=8)):
        args = _scale_shift_relu_net(**kwargs)
        fused   = vkjax_amd.wrap(_scale_shift_relu_step, frontend='minijax')(*args)
        unfused = vkjax_amd.wrap(_scale_shift_relu_step, frontend='minijax', fuse=False)(*args)
        assert_tree_close(fused, unfused, exact=True, what=f'fused against unfused {kwargs}')
        check_against_oracle(_scale_shift_relu_step, args, rtol=1e-4, atol=1e-5)


def _batch_stat_net_inputs(seed=0, batch=4, size=6, channels=((4, 8), (8, 8))):
    rng = np.random.default_rng(seed)
    params = [dict(w=(rng.standard_normal((3, 3, cin, cout)) / np.sqrt(9 * cin)).astype(np.float32),
                   scale=(1 + 0.1 * rng.standard_normal(cout)).astype(np.float32),
                   shift=(0.1 * rng.standard_normal(cout)).astype(np.float32)) for cin, cout in channels]
    return params, rng.standard_normal((batch, size, size, channels[0][0])).astype(np.float32)


def _batch_stat_net_loss(params, x):
    '''Convolution -> batch norm with the BATCH's own mean and variance -> ReLU, twice; mean of squares.'''
    h = x
    for p in params:
        y = mj.lax.conv_general_dilated(h, p['w'], (1, 1), 'SAME', dimension_numbers=('NHWC', 'HWIO', 'NHWC'))
        mean = mj.numpy.mean(y, axis=(0, 1, 2))
        var = mj.numpy.mean((y - mean) ** 2, axis=(0, 1, 2))
        h = mj.nn.relu((y - mean) * mj.lax.rsqrt(var + 1e-5) * p['scale'] + p['shift'])
    return mj.numpy.sum(h * h) / h.size


def _batch_stat_net_step(params, x):
    return mj.value_and_grad(_batch_stat_net_loss)(params, x)


def test_batch_norm_with_batch_statistics_equals_torch_autograd():
    '''The gradient flows through the batch mean and variance as well (reductions, rsqrt, broadcasts and their
    transposes); torch's batch_norm in training mode is the independent implementation.'''
    import torch
    params, x = _batch_stat_net_inputs()
    (loss, gradients), _ = oracle_outputs(_batch_stat_net_step, (params, x))
    grads = mj.tree_util.tree_leaves(gradients)
    tp = [{k: torch.tensor(v, requires_grad=True) for k, v in p.items()} for p in params]
    h = torch.tensor(x).permute(0, 3, 1, 2)
    for p in tp:
        y = torch.nn.functional.conv2d(h, p['w'].permute(3, 2, 0, 1), padding=1)
        h = torch.relu(torch.nn.functional.batch_norm(y, None, None, p['scale'], p['shift'], training=True, eps=1e-5))
    expected = (h * h).sum() / h.numel()
    expected.backward()
    assert np.allclose(loss, expected.detach().numpy(), rtol=1e-5)
    flat = [p[k].grad.numpy() for p in tp for k in sorted(p)]           #tree leaves come in sorted key order
    assert len(flat) == len(grads)
    for g, e in zip(grads, flat):
        assert np.allclose(g, e, rtol=1e-4, atol=1e-6), float(np.abs(g - e).max())


@pytest.mark.gpu
def test_batch_norm_with_batch_statistics_hip():
    for kwargs in (dict(), dict(seed=5, batch=8, size=12, channels=((4, 16), (16, 12)))):
        args = _batch_stat_net_inputs(**kwargs)
        for fuse in (True, False):
            check_against_oracle(_batch_stat_net_step, args, rtol=1e-4, atol=1e-5, fuse=fuse)
