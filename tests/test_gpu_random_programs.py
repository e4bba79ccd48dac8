'''Randomly generated programs of element-wise operations, broadcasts, slices, transposes, reshapes and
reductions, run fused and unfused on the GPU and compared bit for bit with the CPU oracle. Operands are small
integers held in float32, so every intermediate value is exact and no evaluation order can hide an error.
The generator is seeded: the programs are the same on every run.'''
import numpy as np
import pytest

from tests.common import check_against_oracle, oracle_outputs
from vkjax_amd import minijax as mj
from vkjax_amd.jaxpr_interpreter import JaxprInterpreter

lax, jnp = mj.lax, mj.numpy
N_PROGRAMS = 120


def make_program(seed):
    rng = np.random.RandomState(seed)
    rank = rng.randint(1, 5)
    shape = tuple(int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 33])) for _ in range(rank))
    n_inputs = rng.randint(1, 4)
    inputs = [rng.randint(-3, 4, size=shape).astype(np.float32) for _ in range(n_inputs)]
    #vectors that broadcast along the last dimension, as biases and batch-norm parameters do
    vectors = [rng.randint(-2, 3, size=shape[-1:]).astype(np.float32) for _ in range(2)]
    steps = []
    for _ in range(rng.randint(3, 12)):
        kind = rng.choice(['binary', 'binary', 'binary', 'unary', 'vector', 'scalar', 'select', 'transpose', 'slice', 'reshape', 'reduce', 'rev'])
        steps.append((kind, rng.randint(0, 1 << 30)))

    def program(*args):
        xs, vs = list(args[:n_inputs]), list(args[n_inputs:])
        values = list(xs)
        for kind, r in steps:
            pick = lambda k=0: values[(r >> (3 * k)) % len(values)]
            a = pick()
            if kind == 'binary':
                b = next((v for v in reversed(values) if v.shape == a.shape and v is not a), a)
                op = [lax.add, lax.sub, lax.max, lax.min, lax.mul][r % 5]
                out = op(a, b)
                if op is lax.mul:
                    out = lax.min(lax.max(out, -64.0), 64.0)          #keeps every later product exact
            elif kind == 'unary':
                out = [lax.neg, lax.abs, lax.sign, lambda v: lax.integer_pow(lax.min(lax.max(v, -8.0), 8.0), 2)][r % 4](a)
            elif kind == 'vector':
                if a.shape[-1:] != vs[0].shape:
                    continue
                out = [jnp.add, jnp.subtract, jnp.maximum][r % 3](a, vs[r % 2])
            elif kind == 'scalar':
                out = [lax.add, lax.mul, lax.max, lax.sub][r % 4](a, float(r % 5 - 2))
            elif kind == 'select':
                b = next((v for v in reversed(values) if v.shape == a.shape and v is not a), a)
                out = lax.select(lax.gt(a, b), a, lax.neg(b))
            elif kind == 'transpose':
                if a.ndim < 2:
                    continue
                perm = list(range(a.ndim))
                np.random.RandomState(r % 1000).shuffle(perm)
                out = lax.transpose(a, tuple(perm))
            elif kind == 'slice':
                start = [int((r >> k) % max(1, n // 2)) if n > 1 else 0 for k, n in enumerate(a.shape)]
                stride = [1 + (r >> (k + 5)) % 2 for k in range(a.ndim)]
                out = lax.slice(a, start, a.shape, stride)
                if 0 in out.shape:
                    continue
            elif kind == 'reshape':
                out = jnp.reshape(a, (-1,)) if r % 2 else jnp.reshape(a, (a.shape[0], -1)) if a.ndim > 1 else a
            elif kind == 'reduce':
                if a.ndim == 0:
                    continue
                axes = tuple(sorted(set(int(d) for d in np.random.RandomState(r % 1000).randint(0, a.ndim, size=1 + r % 2))))
                out = [jnp.sum, jnp.max, jnp.min][r % 3](a, axis=axes)
                out = lax.min(lax.max(out, -64.0), 64.0)
            else:
                out = lax.rev(a, (r % a.ndim,)) if a.ndim else a
            values.append(out)
        return tuple(values[n_inputs:][-3:]) if len(values) > n_inputs else (values[0] + 1.0,)
    return program, inputs + vectors


@pytest.mark.parametrize('seed', range(N_PROGRAMS))
def test_random_program_plans(seed):
    f, args = make_program(seed)
    _, closed = oracle_outputs(f, args)
    for fuse in (True, False):
        JaxprInterpreter(closed, plan_only=True, fuse=fuse)


@pytest.mark.gpu
@pytest.mark.parametrize('seed', range(N_PROGRAMS))
def test_random_program_hip(seed):
    f, args = make_program(seed)
    print(f'case: random program {seed}', flush=True)
    for fuse in (True, False):
        check_against_oracle(f, args, exact=True, fuse=fuse)


# ---------------------------------------------------------------------------------------------------------------
# Random small networks: convolutions followed by per-channel arithmetic, ReLU, residual additions and channel sums,
# with intermediate results that are read more than once, forward only or with reverse-mode gradients. These are
# the shapes the convolution epilogue, second-result, fused backward and batching passes look for; integer-valued
# data keeps every sum exact, so fused and unfused runs must agree with the oracle bit for bit.
N_NETWORKS = 60


def make_network(seed):
    rng = np.random.RandomState(5000 + seed)
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)
    batch, size, cin = int(rng.choice([1, 2, 3])), int(rng.choice([4, 5, 8])), int(rng.choice([4, 8]))
    x = ints(-3, 4, batch, size, size, cin)
    params, configs = [], []
    for _ in range(rng.randint(1, 3)):
        cout, k = int(rng.choice([4, 8, 12])), int(rng.choice([1, 3]))
        params.append(dict(w=ints(-2, 3, k, k, cin, cout), mean=ints(-2, 3, cout), scale=ints(1, 3, cout), shift=ints(-3, 4, cout)))
        configs.append((int(rng.choice([1, 1, 2])), int(rng.randint(0, 5))))
        cin = cout
    weights = ints(-2, 3, 1)[0]
    with_gradients = bool(seed % 2)

    def forward(params, x):
        h, extras = x, []
        for p, (stride, mode) in zip(params, configs):
            y = lax.conv_general_dilated(h, p['w'], (stride, stride), 'SAME', dimension_numbers=('NHWC', 'HWIO', 'NHWC'))
            if mode == 0:                                   #scale and shift with fixed statistics, ReLU
                z = mj.nn.relu((y - p['mean']) * p['scale'] + p['shift'])
            elif mode == 1:                                 #the centred result is read again AFTER the chain
                centred = y - p['mean']
                z = mj.nn.relu(centred * p['scale'] + p['shift'])
                extras.append(jnp.sum(centred, axis=(0, 1, 2)))
            elif mode == 2:                                 #the plain result is read BEFORE the chain that continues it
                total = jnp.sum(y, axis=(0, 1, 2))
                z = mj.nn.relu((y - lax.min(lax.max(total, -2.0), 2.0)) * p['scale'])
                extras.append(total)
            elif mode == 3:                                 #no activation
                z = y * p['scale'] + p['shift']
            else:                                           #residual connection where the shapes allow it
                z = (y - p['mean']) * p['scale']
                z = mj.nn.relu(z + h) if z.shape == h.shape else mj.nn.relu(z)
            h = lax.min(lax.max(z, -8.0), 8.0)
        return h, extras

    if not with_gradients:
        def program(params, x):
            h, extras = forward(params, x)
            return (h, *extras)
    else:
        def loss(params, x):
            h, extras = forward(params, x)
            return jnp.sum(h) * float(weights) + sum(jnp.sum(e) for e in extras)
        def program(params, x):
            return mj.value_and_grad(loss)(params, x)
    return program, (params, x)


@pytest.mark.parametrize('seed', range(N_NETWORKS))
def test_random_network_plans(seed):
    f, args = make_network(seed)
    _, closed = oracle_outputs(f, args)
    for fuse in (True, False):
        JaxprInterpreter(closed, plan_only=True, fuse=fuse)


@pytest.mark.gpu
@pytest.mark.parametrize('seed', range(N_NETWORKS))
def test_random_network_hip(seed):
    f, args = make_network(seed)
    print(f'case: random network {seed}', flush=True)
    for fuse in (True, False):
        check_against_oracle(f, args, exact=True, fuse=fuse)


# ---------------------------------------------------------------------------------------------------------------
# Random geometry of single primitives: convolutions (batch, image and kernel sizes from 1 up, strides, dilations,
# uneven padding) and their gradients, matrix products of odd sizes in all three layouts, pooling windows, row
# gathers and scatter-adds. Integer-valued data: exact results, fused and unfused.
N_GEOMETRIES = 160
dn = ('NHWC', 'HWIO', 'NHWC')


def make_geometry_case(seed):
    rng = np.random.RandomState(9000 + seed)
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)
    kind = ['conv', 'conv', 'conv', 'dot', 'pool', 'gather', 'scatter', 'convgrad'][seed % 8]
    if kind in ('conv', 'convgrad'):
        b, h, w = int(rng.choice([1, 1, 2, 3])), int(rng.randint(1, 10)), int(rng.randint(1, 10))
        cin, cout = int(rng.choice([1, 3, 4, 8, 12, 16, 32])), int(rng.choice([1, 4, 5, 8, 16, 64]))
        kh, kw = int(rng.choice([1, 2, 3])), int(rng.choice([1, 2, 3]))
        sh, sw = int(rng.choice([1, 1, 2, 3])), int(rng.choice([1, 1, 2]))
        dh, dw = int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2]))
        pad = ((int(rng.randint(0, 3)), int(rng.randint(0, 3))), (int(rng.randint(0, 3)), int(rng.randint(0, 3))))
        eh, ew = (kh - 1) * dh + 1, (kw - 1) * dw + 1
        if h + sum(pad[0]) < eh or w + sum(pad[1]) < ew:
            pad = ((eh, eh), (ew, ew))
        x, k = ints(-3, 4, b, h, w, cin), ints(-2, 3, kh, kw, cin, cout)
        #the second half of the seeds also draws an input dilation and other dimension numbers
        ld = [(1, 1), (1, 1), (2, 1), (2, 2), (3, 2)][rng.randint(0, 5)] if seed >= N_GEOMETRIES // 2 else (1, 1)
        layout = rng.randint(0, 3) if seed >= N_GEOMETRIES // 2 else 0
        dnums = [('NHWC', 'HWIO', 'NHWC'), ('NCHW', 'OIHW', 'NCHW'), ('NHWC', 'OIHW', 'NCHW')][layout]
        if layout == 1:
            x = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
        if layout in (1, 2):
            k = np.ascontiguousarray(k.transpose(3, 2, 0, 1))
        conv = lambda x, k: lax.conv_general_dilated(x, k, (sh, sw), pad, lhs_dilation=ld, rhs_dilation=(dh, dw), dimension_numbers=dnums)
        if kind == 'conv':
            return f'conv x{x.shape} k{k.shape} s{(sh, sw)} d{(dh, dw)} ld{ld} p{pad} {dnums}', conv, [x, k]
        return f'convgrad x{x.shape} k{k.shape} s{(sh, sw)} d{(dh, dw)} p{pad}', (lambda x, k: mj.value_and_grad(lambda p: jnp.sum(conv(p[0], p[1]) * 2.0))((x, k))), [x, k]
    if kind == 'dot':
        m, n, kk = int(rng.choice([1, 2, 7, 33, 64, 130])), int(rng.choice([1, 3, 4, 10, 64, 72])), int(rng.choice([1, 2, 5, 16, 127, 128, 260]))
        a, b = ints(-3, 4, m, kk), ints(-2, 3, kk, n)
        variant = rng.randint(0, 3)
        if variant == 0: return f'dot {m}x{kk}x{n}', (lambda a, b: jnp.dot(a, b)), [a, b]
        if variant == 1: return f'dot^T {m}x{kk}x{n}', (lambda a, b: jnp.dot(a, lax.transpose(b, (1, 0)))), [a, np.ascontiguousarray(b.T)]
        return f'dot T^ {m}x{kk}x{n}', (lambda a, b: jnp.dot(lax.transpose(a, (1, 0)), b)), [np.ascontiguousarray(a.T), b]
    if kind == 'pool':
        b, h, w, c = int(rng.choice([1, 2])), int(rng.randint(1, 12)), int(rng.randint(1, 12)), int(rng.choice([1, 3, 4, 8, 64]))
        wh, ww = int(rng.choice([1, 2, 3])), int(rng.choice([1, 2, 3]))
        sh, sw = int(rng.choice([1, 2, 3])), int(rng.choice([1, 2]))
        pad = ((0, 0), (int(rng.randint(0, 2)), int(rng.randint(0, 3))), (int(rng.randint(0, 2)), int(rng.randint(0, 3))), (0, 0))
        if h + sum(pad[1]) < wh or w + sum(pad[2]) < ww:
            pad = ((0, 0), (wh, wh), (ww, ww), (0, 0))
        x = ints(-9, 10, b, h, w, c)
        if rng.randint(0, 2):
            return f'maxpool x{x.shape} w{(wh, ww)} s{(sh, sw)} p{pad}', (lambda x: lax.reduce_window(x, -jnp.inf, lax.max, (1, wh, ww, 1), (1, sh, sw, 1), pad)), [x]
        return f'sumpool x{x.shape} w{(wh, ww)} s{(sh, sw)} p{pad}', (lambda x: lax.reduce_window(x, 0.0, lax.add, (1, wh, ww, 1), (1, sh, sw, 1), pad)), [x]
    rows, cols = int(rng.choice([1, 5, 64, 300])), int(rng.choice([1, 3, 4, 64, 256]))
    nidx = int(rng.choice([1, 2, 17, 256, 1000]))
    table, idx = ints(-9, 10, rows, cols), rng.randint(0, rows, size=(nidx,)).astype(np.int32)
    if kind == 'gather':
        return f'gather {rows}x{cols} <- {nidx}', (lambda t, i: t[i]), [table, idx]
    upd = ints(-3, 4, nidx, cols)
    return f'scatter-add {rows}x{cols} <- {nidx}', (lambda t, i, u: t.at[i].add(u)), [table, idx, upd]


@pytest.mark.parametrize('seed', range(N_GEOMETRIES))
def test_random_geometry_plans(seed):
    name, f, args = make_geometry_case(seed)
    _, closed = oracle_outputs(f, args)
    for fuse in (True, False):
        JaxprInterpreter(closed, plan_only=True, fuse=fuse)


@pytest.mark.gpu
@pytest.mark.parametrize('seed', range(N_GEOMETRIES))
def test_random_geometry_hip(seed):
    name, f, args = make_geometry_case(seed)
    print(f'case: random geometry {seed}: {name}', flush=True)
    for fuse in (True, False):
        check_against_oracle(f, args, exact=True, fuse=fuse)


# ---------------------------------------------------------------------------------------------------------------
# Random parameters of the remaining primitives: pad (negative and interior padding), concatenate (empty parts),
# argmax / argmin (NaNs, ties), products, broadcasts, indexing with negative and repeated indices, scatter-add along
# the first dimension, take_along_axis, iota, clamp / integer_pow, window reductions over any dimensions of
# rank-3 and rank-4 arrays. Integer-valued, exact, fused and unfused.
N_MISC = 120


def make_misc_case(seed):
    rng = np.random.RandomState(64000 + seed)
    ints = lambda lo, hi, *shape: rng.randint(lo, hi, size=shape).astype(np.float32)
    kind = ['pad', 'concat', 'argext', 'prod', 'bcast', 'index1', 'index2', 'scatter_dim', 'take_along', 'iota', 'clamp_pow', 'pool_general'][seed % 12]
    rank = rng.randint(1, 4)
    shape = tuple(int(rng.choice([1, 2, 3, 5, 8, 16, 33])) for _ in range(rank))
    x = ints(-4, 5, *shape)
    if kind == 'pad':
        cfg = tuple((int(rng.randint(-2, 4)), int(rng.randint(-2, 4)), int(rng.randint(0, 3))) for _ in shape)
        for d, (lo, hi, it) in enumerate(cfg):
            if shape[d] + (shape[d] - 1) * it + lo + hi < 0: cfg = tuple((0, 0, 0) for _ in shape)
        return f'pad {shape} {cfg}', (lambda x: lax.pad(x, 7.0, cfg)), [x]
    if kind == 'concat':
        axis = rng.randint(0, rank); parts = []
        for _ in range(rng.randint(1, 5)):
            s = list(shape); s[axis] = int(rng.choice([0, 1, 3, 4, 9])); parts.append(ints(-4, 5, *s))
        if sum(p.shape[axis] for p in parts) == 0: parts.append(x)
        return f'concat axis {axis} {[p.shape for p in parts]}', (lambda *ps: lax.concatenate(list(ps), axis)), parts
    if kind == 'argext':
        axis = rng.randint(0, rank)
        xs = x.copy()
        if rng.randint(0, 3) == 0: xs.flat[rng.randint(0, xs.size)] = np.nan
        fn = [jnp.argmax, jnp.argmin][rng.randint(0, 2)]
        return f'{fn.__name__} {shape} axis {axis}', (lambda x: fn(x, axis=axis)), [xs]
    if kind == 'prod':
        axis = rng.randint(0, rank)
        return f'prod {shape} axis {axis}', (lambda x: lax.reduce_prod(lax.min(lax.max(x, -2.0), 2.0), (axis,))), [x]
    if kind == 'bcast':
        new = (int(rng.choice([1, 2, 5])),) + shape + (int(rng.choice([1, 3, 4])),)
        return f'broadcast {shape} -> {new}', (lambda x: lax.broadcast_in_dim(x, new, tuple(range(1, rank + 1))) + 1.0), [x]
    if kind == 'index1':
        idx = rng.randint(-shape[0], shape[0], size=(int(rng.choice([1, 4, 17])),)).astype(np.int32)
        return f'x[idx] {shape} {idx.shape}', (lambda x, i: x[i]), [x, idx]
    if kind == 'index2':
        if rank < 2: return f'x[idx] {shape}', (lambda x, i: x[i]), [x, np.zeros((2,), np.int32)]
        idx = rng.randint(0, shape[1], size=(int(rng.choice([1, 3, 9])),)).astype(np.int32)
        return f'x[:, idx] {shape} {idx.shape}', (lambda x, i: x[:, i]), [x, idx]
    if kind == 'scatter_dim':
        idx = rng.randint(0, shape[0], size=(int(rng.choice([1, 5, 40])),)).astype(np.int32)
        upd = ints(-3, 4, idx.shape[0], *shape[1:])
        return f'x.at[idx].add {shape} {idx.shape}', (lambda x, i, u: x.at[i].add(u)), [x, idx, upd]
    if kind == 'take_along':
        axis = rng.randint(0, rank)
        ishape = list(shape); ishape[axis] = int(rng.choice([1, 2, 6]))
        idx = rng.randint(0, shape[axis], size=ishape).astype(np.int32)
        return f'take_along_axis {shape} axis {axis}', (lambda x, i: jnp.take_along_axis(x, i, axis=axis)), [x, idx]
    if kind == 'iota':
        n = int(rng.choice([1, 7, 64, 1000]))
        return f'iota {n}', (lambda x: lax.iota(np.int32, n) * 3 + x), [np.asarray(rng.randint(-5, 5), np.int32)]
    if kind == 'clamp_pow':
        p = int(rng.choice([0, 1, 2, 3, -1]))
        base = x if p >= 0 else np.where(x == 0, 1, x).astype(np.float32)
        return f'clamp+pow {shape} ^{p}', (lambda x: lax.integer_pow(lax.clamp(-3.0, x, 3.0), p) if p >= 0 else lax.clamp(-3.0, x, 3.0) * 2.0), [base]
    # pool_general: windows over arbitrary dims of a rank-3/4 array
    r = rng.randint(3, 5)
    shp = tuple(int(rng.choice([1, 2, 4, 6, 9])) for _ in range(r))
    win = tuple(int(rng.randint(1, min(3, s) + 1)) for s in shp)
    strd = tuple(int(rng.randint(1, 3)) for _ in shp)
    pads = tuple((int(rng.randint(0, 2)), int(rng.randint(0, 2))) for _ in shp)
    xx = ints(-9, 10, *shp)
    if rng.randint(0, 2):
        return f'window max {shp} {win} {strd} {pads}', (lambda x: lax.reduce_window(x, -jnp.inf, lax.max, win, strd, pads)), [xx]
    return f'window sum {shp} {win} {strd} {pads}', (lambda x: lax.reduce_window(x, 0.0, lax.add, win, strd, pads)), [xx]


@pytest.mark.parametrize('seed', range(N_MISC))
def test_random_misc_plans(seed):
    name, f, args = make_misc_case(seed)
    _, closed = oracle_outputs(f, args)
    for fuse in (True, False):
        JaxprInterpreter(closed, plan_only=True, fuse=fuse)


@pytest.mark.gpu
@pytest.mark.parametrize('seed', range(N_MISC))
def test_random_misc_hip(seed):
    name, f, args = make_misc_case(seed)
    print(f'case: random primitive {seed}: {name}', flush=True)
    for fuse in (True, False):
        check_against_oracle(f, args, exact=True, fuse=fuse)
