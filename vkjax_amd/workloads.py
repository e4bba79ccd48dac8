'''The five benchmark / parity workloads: the functions that get traced and their synthetic,
seeded inputs. Written against the stand-in tracer (`vkjax_amd.minijax`), they produce the
primitive sequences a jax front-end of the reference's era emits for the same models
(`jnp.dot + b`, relu under a custom-jvp call, softmax, NHWC convolutions with inference-mode
batch norm, `reduce_window` max pooling, threefry-based `random.uniform`, indexing gather and
`.at[].add` scatter).

Input recipe: numpy `default_rng(seed)`; "uniform" is `rng.random(shape, float32)`; He-normal is
`standard_normal * sqrt(2 / fan_in)`; all weights are generated on the host.
'''
import typing as tp

import numpy as np

from . import minijax as mj

jnp, lax, nn = mj.numpy, mj.lax, mj.nn

NHWC = mj.core.ConvDimensionNumbers((0, 3, 1, 2), (3, 2, 0, 1), (0, 3, 1, 2))


def he_normal(rng, shape, fan_in) -> np.ndarray:
    return (rng.standard_normal(shape, dtype=np.float32) * np.sqrt(2.0 / fan_in)).astype(np.float32)


# ------------------------------------------------------------------ 1: affine layer

def affine(x, W, b):
    return jnp.dot(x, W) + b


def affine_inputs(seed=1):
    rng = np.random.default_rng(seed)
    return [rng.random((8, 128), dtype=np.float32), rng.random((128, 16), dtype=np.float32), rng.random((16,), dtype=np.float32)]


# ------------------------------------------------------------------ 2: MLP

def mlp(params, x):
    h = nn.relu(jnp.dot(x, params['w1']) + params['b1'])
    h = nn.relu(jnp.dot(h, params['w2']) + params['b2'])
    logits = jnp.dot(h, params['w3']) + params['b3']
    probs  = nn.softmax(logits, axis=-1)
    return probs, jnp.argmax(probs, axis=1)


def mlp_inputs(seed=2, batch=256, sizes=(784, 512, 512, 10)):
    rng = np.random.default_rng(seed)
    x = rng.random((batch, sizes[0]), dtype=np.float32)
    params = {}
    for i in range(3):
        params[f'w{i + 1}'] = he_normal(rng, (sizes[i], sizes[i + 1]), sizes[i])
        params[f'b{i + 1}'] = np.zeros((sizes[i + 1],), np.float32)
    return [params, x]


# ------------------------------------------------------------------ 3: conv block

def conv_block(params, x):
    y = lax.conv_general_dilated(x, params['w'], window_strides=(1, 1), padding=((1, 1), (1, 1)), dimension_numbers=NHWC)
    y = nn.batch_norm_inference(y, params['scale'], params['shift'], params['mean'], params['var'])
    y = nn.relu(y)
    return lax.reduce_window(y, -jnp.inf, lax.max, (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (0, 1), (0, 1), (0, 0)))


def conv_block_inputs(seed=3, batch=32, size=56, channels=64):
    rng = np.random.default_rng(seed)
    x = rng.random((batch, size, size, channels), dtype=np.float32)
    params = dict(w=he_normal(rng, (3, 3, channels, channels), 9 * channels),
                  scale=rng.standard_normal(channels, dtype=np.float32), shift=rng.standard_normal(channels, dtype=np.float32),
                  mean=rng.standard_normal(channels, dtype=np.float32),
                  var=(0.5 + rng.random(channels, dtype=np.float32)).astype(np.float32))
    return [params, x]


# ------------------------------------------------------------------ 4: ResNet-50

RESNET50_STAGES = ((3, 64, 1), (4, 128, 2), (6, 256, 2), (3, 512, 2))      #(blocks, bottleneck width, stride of the first block)


def _same_pads(size, window, stride):
    out   = -(-size // stride)
    total = max((out - 1) * stride + window - size, 0)
    return (total // 2, total - total // 2)


def _conv_bn(p, x, stride=1, pads=None, relu=True):
    kh, kw = p['w'].shape[0], p['w'].shape[1]
    if pads is None:
        pads = (_same_pads(x.shape[1], kh, stride), _same_pads(x.shape[2], kw, stride))
    y = lax.conv_general_dilated(x, p['w'], window_strides=(stride, stride), padding=pads, dimension_numbers=NHWC)
    y = nn.batch_norm_inference(y, p['scale'], p['shift'], p['mean'], p['var'])
    return nn.relu(y) if relu else y


def resnet50(params, x):
    '''ResNet-50 forward, inference mode. Layer table: 7x7/2 stem (padding 3) + BN + ReLU,
    3x3/2 SAME max-pool, bottleneck stages (3, 4, 6, 3) with the stride on the 3x3 convolution
    and a strided 1x1 projection on the first block of each stage, global average pool, 1000-way
    dense layer. Returns (logits, argmax(logits)).'''
    y = _conv_bn(params['stem'], x, stride=2, pads=((3, 3), (3, 3)))
    y = lax.reduce_window(y, -jnp.inf, lax.max, (1, 3, 3, 1), (1, 2, 2, 1),
                          ((0, 0), _same_pads(y.shape[1], 3, 2), _same_pads(y.shape[2], 3, 2), (0, 0)))
    for s, (blocks, width, stride) in enumerate(RESNET50_STAGES):
        for b in range(blocks):
            p = params[f'stage{s}'][f'block{b}']
            st = stride if b == 0 else 1
            shortcut = _conv_bn(p['proj'], y, stride=st, relu=False) if 'proj' in p else y
            z = _conv_bn(p['conv1'], y)
            z = _conv_bn(p['conv2'], z, stride=st)
            z = _conv_bn(p['conv3'], z, relu=False)
            y = nn.relu(z + shortcut)
    y = jnp.mean(y, axis=(1, 2))
    logits = jnp.dot(y, params['fc']['w']) + params['fc']['b']
    return logits, jnp.argmax(logits, axis=1)


def _conv_bn_params(rng, kh, kw, cin, cout):
    return dict(w=he_normal(rng, (kh, kw, cin, cout), kh * kw * cin),
                scale=(0.5 + rng.random(cout, dtype=np.float32)).astype(np.float32),
                shift=(0.1 * rng.standard_normal(cout, dtype=np.float32)).astype(np.float32),
                mean=(0.1 * rng.standard_normal(cout, dtype=np.float32)).astype(np.float32),
                var=(0.5 + rng.random(cout, dtype=np.float32)).astype(np.float32))


def resnet50_params(seed=4, num_classes=1000, width_scale=1.0) -> dict:
    '''`width_scale` < 1 shrinks every channel count (test-sized variants of the same graph).'''
    rng = np.random.default_rng(seed)
    c = lambda n: max(4, int(n * width_scale) // 4 * 4)
    params = dict(stem=_conv_bn_params(rng, 7, 7, 3, c(64)))
    cin = c(64)
    for s, (blocks, width, stride) in enumerate(RESNET50_STAGES):
        stage = {}
        for b in range(blocks):
            w, cout = c(width), c(width * 4)
            block = dict(conv1=_conv_bn_params(rng, 1, 1, cin, w), conv2=_conv_bn_params(rng, 3, 3, w, w),
                         conv3=_conv_bn_params(rng, 1, 1, w, cout))
            if b == 0:
                block['proj'] = _conv_bn_params(rng, 1, 1, cin, cout)
            stage[f'block{b}'] = block
            cin = cout
        params[f'stage{s}'] = stage
    params['fc'] = dict(w=he_normal(rng, (cin, num_classes), cin), b=np.zeros((num_classes,), np.float32))
    return params


def resnet50_inputs(seed=4, batch=64, size=224, num_classes=1000, width_scale=1.0):
    params = resnet50_params(seed, num_classes, width_scale)
    rng = np.random.default_rng(seed + 1000)
    return [params, rng.random((batch, size, size, 3), dtype=np.float32)]


# ------------------------------------------------------------------ 5: RNG + gather / scatter-add

def rng_uniform(key, shape=(4096, 4096)):
    k1, k2 = mj.random.split(key)
    return mj.random.uniform(k2, shape)


def rng_inputs(seed=5):
    return [mj.random.PRNGKey(seed)]


def gather_scatter(table, idx, updates):
    rows = table[idx]
    return rows, jnp.index_add(jnp.zeros(table.shape, np.float32), idx, updates)


def gather_scatter_inputs(seed=5, rows=65536, cols=256, n0=8192, n1=32):
    rng = np.random.default_rng(seed)
    table   = rng.random((rows, cols), dtype=np.float32)
    idx     = rng.integers(0, rows, size=(n0, n1)).astype(np.int32)
    updates = rng.random((n0, n1, cols), dtype=np.float32)
    return [table, idx, updates]


# ------------------------------------------------------------------ training steps (forward, backward, SGD update)

def softmax_cross_entropy(logits, onehot):
    z    = logits - lax.stop_gradient(jnp.max(logits, axis=1, keepdims=True))
    logp = z - jnp.log(jnp.sum(jnp.exp(z), axis=1, keepdims=True))
    return -jnp.mean(jnp.sum(onehot * logp, axis=1))


def _sgd(params, grads, lr):
    return mj.tree_multimap(lambda p, g: p - np.float32(lr) * g, params, grads)


def mlp_loss(params, x, onehot):
    h = nn.relu(jnp.dot(x, params['w1']) + params['b1'])
    h = nn.relu(jnp.dot(h, params['w2']) + params['b2'])
    return softmax_cross_entropy(jnp.dot(h, params['w3']) + params['b3'], onehot)


def mlp_train_step(params, x, onehot, lr=0.05):
    '''One SGD step of the MLP on a batch: returns (loss, updated parameters). The backward pass is the
    program autodiff produces (transposed dot_generals, relu masks, bias gradients as reduce_sum).'''
    loss, grads = mj.value_and_grad(mlp_loss)(params, x, onehot)
    return loss, _sgd(params, grads, lr)


def mlp_train_inputs(seed=6, batch=256, sizes=(784, 512, 512, 10)):
    params, x = mlp_inputs(seed, batch, sizes)
    rng = np.random.default_rng(seed + 1000)
    onehot = np.eye(sizes[-1], dtype=np.float32)[rng.integers(0, sizes[-1], size=batch)]
    return [params, x, onehot]


def convnet_loss(params, x, onehot):
    '''A small convolutional classifier that exercises every gradient form of the path: strided 3x3 convolution,
    per-channel scale and shift, relu, 3x3/2 max pooling, 3x3 convolution, 2x2 average pooling, global mean, dense.'''
    y = lax.conv_general_dilated(x, params['w1'], window_strides=(2, 2), padding=((1, 1), (1, 1)), dimension_numbers=NHWC)
    y = nn.relu(y * params['scale'] + params['shift'])
    y = lax.reduce_window(y, -jnp.inf, lax.max, (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (0, 1), (0, 1), (0, 0)))
    y = nn.relu(lax.conv_general_dilated(y, params['w2'], window_strides=(1, 1), padding=((1, 1), (1, 1)), dimension_numbers=NHWC))
    y = lax.reduce_window(y, 0.0, lax.add, (1, 2, 2, 1), (1, 2, 2, 1), 'VALID') / 4.0
    y = jnp.mean(y, axis=(1, 2))
    return softmax_cross_entropy(jnp.dot(y, params['w3']) + params['b3'], onehot)


def convnet_train_step(params, x, onehot, lr=0.05):
    loss, grads = mj.value_and_grad(convnet_loss)(params, x, onehot)
    return loss, _sgd(params, grads, lr)


def convnet_train_inputs(seed=7, batch=64, size=64, channels=(3, 64, 128), classes=10):
    rng = np.random.default_rng(seed)
    c0, c1, c2 = channels
    params = dict(w1=he_normal(rng, (3, 3, c0, c1), 9 * c0), scale=(0.5 + rng.random(c1, dtype=np.float32)).astype(np.float32),
                  shift=(0.1 * rng.standard_normal(c1, dtype=np.float32)).astype(np.float32),
                  w2=he_normal(rng, (3, 3, c1, c2), 9 * c1), w3=he_normal(rng, (c2, classes), c2), b3=np.zeros((classes,), np.float32))
    x = rng.random((batch, size, size, c0), dtype=np.float32)
    onehot = np.eye(classes, dtype=np.float32)[rng.integers(0, classes, size=batch)]
    return [params, x, onehot]


_STATISTICS = ('mean', 'var')


def _split_statistics(params):
    '''(trainable arrays, batch-norm statistics) as two trees of the same nesting.'''
    if not isinstance(params, dict):
        return params, None
    trainable, fixed = {}, {}
    for k, v in params.items():
        if k in _STATISTICS:
            fixed[k] = v
        else:
            trainable[k], sub = _split_statistics(v)
            if sub:
                fixed[k] = sub
    return trainable, fixed


def _merge_statistics(trainable, fixed):
    if not isinstance(trainable, dict):
        return trainable
    merged = {k: _merge_statistics(v, (fixed or {}).get(k)) for k, v in trainable.items()}
    merged.update({k: v for k, v in (fixed or {}).items() if k not in merged})
    return merged


def resnet50_loss(trainable, statistics, x, onehot):
    logits, _ = resnet50(_merge_statistics(trainable, statistics), x)
    return softmax_cross_entropy(logits, onehot)


def resnet50_train_step(params, x, onehot, lr=0.01):
    '''One SGD step of ResNet-50 with frozen batch-norm statistics: gradients and updates for every
    convolution kernel, scale, shift and the dense layer; mean and variance stay as they are.
    Returns (loss, updated trainable arrays).'''
    trainable, statistics = _split_statistics(params)
    loss, grads = mj.value_and_grad(resnet50_loss)(trainable, statistics, x, onehot)
    return loss, _sgd(trainable, grads, lr)


def resnet50_train_inputs(seed=4, batch=64, size=224, num_classes=1000, width_scale=1.0):
    params, x = resnet50_inputs(seed, batch, size, num_classes, width_scale)
    rng = np.random.default_rng(seed + 2000)
    onehot = np.eye(num_classes, dtype=np.float32)[rng.integers(0, num_classes, size=batch)]
    return [params, x, onehot]


# ------------------------------------------------------------------ single primitives at sizes where memory bandwidth is the bound

def _uniform_words(n: int, seed: int) -> np.ndarray:
    return np.random.default_rng(seed).random(n, dtype=np.float32)


def _bn(c, seed=0):
    rng = np.random.default_rng(seed)
    return [(0.5 + rng.random(c, dtype=np.float32)).astype(np.float32), rng.standard_normal(c, dtype=np.float32),
            rng.standard_normal(c, dtype=np.float32), (0.5 + rng.random(c, dtype=np.float32)).astype(np.float32)]


_ACT  = (64, 56, 56, 256)          #a ResNet-50 activation of 51.4 M elements (205.5 MB)
_WIDE = (64, 112, 112, 64)         #the input of ResNet-50's max-pool
_N64M = 1 << 26

def _max_pool_gradient(x, g):
    '''The gradient that a 3 x 3 / 2 max pool hands back to its input for the cotangent g (select_and_scatter_add).'''
    import vkjax_amd.minijax as mj
    pooled = lambda v: lax.reduce_window(v, -jnp.inf, lax.max, (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (0, 1), (0, 1), (0, 0)))
    return mj.grad(lambda v, c: (pooled(v) * c).sum())(x, g)


#name -> (function, inputs, ALGORITHMIC bytes of one evaluation: every operand read once and every result written once)
PRIMITIVES: tp.Dict[str, tp.Tuple[tp.Callable, tp.Callable, tp.Callable]] = {
    'reduce_sum rows 65536x1000':   (lambda x: jnp.sum(x, axis=1), lambda: [_uniform_words(65536000, 1).reshape(65536, 1000)], lambda a: a[0].nbytes + 4 * 65536),
    'reduce_sum rows 4096x16384':   (lambda x: jnp.sum(x, axis=1), lambda: [_uniform_words(_N64M, 2).reshape(4096, 16384)], lambda a: a[0].nbytes + 4 * 4096),
    'reduce_sum columns 262144x256': (lambda x: jnp.sum(x, axis=0), lambda: [_uniform_words(_N64M, 3).reshape(262144, 256)], lambda a: a[0].nbytes + 4 * 256),
    'reduce_sum all 64M':           (lambda x: jnp.sum(x), lambda: [_uniform_words(_N64M, 4)], lambda a: a[0].nbytes + 4),
    'reduce_max rows 65536x1000':   (lambda x: jnp.max(x, axis=1), lambda: [_uniform_words(65536000, 5).reshape(65536, 1000)], lambda a: a[0].nbytes + 4 * 65536),
    'argmax rows 65536x1000':       (lambda x: jnp.argmax(x, axis=1), lambda: [_uniform_words(65536000, 6).reshape(65536, 1000)], lambda a: a[0].nbytes + 4 * 65536),
    'global average 64x7x7x2048':   (lambda x: jnp.mean(x, axis=(1, 2)), lambda: [_uniform_words(64 * 49 * 2048, 7).reshape(64, 7, 7, 2048)], lambda a: a[0].nbytes + 4 * 64 * 2048),
    'add 64M':                      (lambda x, y: x + y, lambda: [_uniform_words(_N64M, 8), _uniform_words(_N64M, 9)], lambda a: 3 * a[0].nbytes),
    'relu 64M':                     (lambda x: nn.relu(x - 0.5), lambda: [_uniform_words(_N64M, 10)], lambda a: 2 * a[0].nbytes),
    'exp 64M':                      (lambda x: jnp.exp(x), lambda: [_uniform_words(_N64M, 11)], lambda a: 2 * a[0].nbytes),
    'batch norm + relu 64x56x56x256': (lambda x, s, b, m, v: nn.relu(nn.batch_norm_inference(x, s, b, m, v)),
                                     lambda: [_uniform_words(int(np.prod(_ACT)), 12).reshape(_ACT)] + _bn(256), lambda a: 2 * a[0].nbytes + 4 * 4 * 256),
    'batch norm + residual + relu 64x56x56x256': (lambda x, r, s, b, m, v: nn.relu(nn.batch_norm_inference(x, s, b, m, v) + r),
                                     lambda: [_uniform_words(int(np.prod(_ACT)), 13).reshape(_ACT), _uniform_words(int(np.prod(_ACT)), 14).reshape(_ACT)] + _bn(256),
                                     lambda a: 3 * a[0].nbytes + 4 * 4 * 256),
    'max pool 3x3 s2 64x112x112x64': (lambda x: lax.reduce_window(x, -jnp.inf, lax.max, (1, 3, 3, 1), (1, 2, 2, 1), ((0, 0), (0, 1), (0, 1), (0, 0))),
                                     lambda: [_uniform_words(int(np.prod(_WIDE)), 15).reshape(_WIDE)], lambda a: a[0].nbytes + a[0].nbytes // 4),
    'sum pool 2x2 s2 64x112x112x64': (lambda x: lax.reduce_window(x, 0.0, lax.add, (1, 2, 2, 1), (1, 2, 2, 1), 'VALID'),
                                     lambda: [_uniform_words(int(np.prod(_WIDE)), 16).reshape(_WIDE)], lambda a: a[0].nbytes + a[0].nbytes // 4),
    'threefry2x32 8388608 lanes':   (lambda k0, k1, x0, x1: lax.threefry2x32(k0, k1, x0, x1),
                                     lambda: [np.uint32(0x13198a2e), np.uint32(0x03707344), np.arange(1 << 23, dtype=np.uint32), np.arange(1 << 23, 1 << 24, dtype=np.uint32)],
                                     lambda a: 4 * a[2].nbytes),
    'transpose 8192x8192':          (lambda x: lax.transpose(x, (1, 0)), lambda: [_uniform_words(_N64M, 17).reshape(8192, 8192)], lambda a: 2 * a[0].nbytes),
    'transpose NHWC to NCHW 64x56x56x256': (lambda x: lax.transpose(x, (0, 3, 1, 2)), lambda: [_uniform_words(int(np.prod(_ACT)), 18).reshape(_ACT)], lambda a: 2 * a[0].nbytes),
    'pad height and width 64x56x56x256': (lambda x: lax.pad(x, 0.0, ((0, 0, 0), (1, 1, 0), (1, 1, 0), (0, 0, 0))),
                                     lambda: [_uniform_words(int(np.prod(_ACT)), 19).reshape(_ACT)], lambda a: a[0].nbytes + 64 * 58 * 58 * 256 * 4),
    'iota 64M':                     (lambda x: lax.broadcasted_iota(np.float32, (1 << 13, 1 << 13), 1), lambda: [np.float32(0.0)], lambda a: 4 * _N64M),      #(the argument is not used: a program of one launch that only writes)
    'concatenate 2 x 32M':          (lambda x, y: lax.concatenate([x, y], 0), lambda: [_uniform_words(_N64M // 2, 20), _uniform_words(_N64M // 2, 21)],
                                     lambda a: 2 * (a[0].nbytes + a[1].nbytes)),
    'max pool gradient 3x3 s2 64x112x112x64': (_max_pool_gradient, lambda: [_uniform_words(int(np.prod(_WIDE)), 22).reshape(_WIDE),
                                                                            _uniform_words(int(np.prod(_WIDE)) // 4, 23).reshape(64, 56, 56, 64)],
                                     lambda a: 2 * a[0].nbytes + a[1].nbytes),
    'gather rows 262144x1KB of 65536': (lambda t, i: t[i], lambda: gather_scatter_inputs()[:2], lambda a: 2 * a[1].size * a[0].shape[1] * 4 + a[1].nbytes),
    'scatter-add rows 262144x1KB into 65536': (lambda i, u: jnp.index_add(jnp.zeros((65536, 256), np.float32), i, u), lambda: gather_scatter_inputs()[1:],
                                     lambda a: a[1].nbytes + a[0].nbytes + 65536 * 256 * 4),
    'uniform 4096x4096 from a key': (rng_uniform, rng_inputs, lambda a: 4096 * 4096 * 4),
}


WORKLOADS: tp.Dict[str, tp.Tuple[tp.Callable, tp.Callable]] = {
    'affine':         (affine, affine_inputs),
    'mlp':            (mlp, mlp_inputs),
    'conv_block':     (conv_block, conv_block_inputs),
    'resnet50':       (resnet50, resnet50_inputs),
    'rng_uniform':    (rng_uniform, rng_inputs),
    'gather_scatter': (gather_scatter, gather_scatter_inputs),
    'mlp_train':      (mlp_train_step, mlp_train_inputs),
    'convnet_train':  (convnet_train_step, convnet_train_inputs),
    'resnet50_train': (resnet50_train_step, resnet50_train_inputs),
}
