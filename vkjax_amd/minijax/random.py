'''Threefry-based random numbers with the counter layout of JAX's original
(non-partitionable) implementation: counters are `iota(n)`, the first half feeds
word 0 and the second half word 1 of the block function; odd sizes are padded with one
zero counter and trimmed. `split(key, n)` is `threefry(key, iota(2n)).reshape(n, 2)`.
(Primitive: reference vkjax/ops.py:550-560, vkjax/shaders/threefry2x32.comp.)

Newer jax versions do not expand these functions while tracing: they emit the key primitives
random_wrap / random_bits / random_split / random_fold_in / random_unwrap and leave the
expansion to the backend. `key_primitives(True)` makes this module trace that way, and typed
keys made by `key()` / `wrap_key_data()` always do.'''
import numpy as np

from . import lax, numpy as mnp
from .tracer import Tracer


def PRNGKey(seed: int) -> np.ndarray:
    seed = int(seed)
    return np.array([(seed >> 32) & 0xFFFFFFFF, seed & 0xFFFFFFFF], dtype=np.uint32)


def _key_halves(key):
    if not isinstance(key, Tracer):
        key = np.asarray(key, np.uint32)
        return key[0], key[1]
    k0 = lax.reshape(lax.slice(key, (0,), (1,)), ())
    k1 = lax.reshape(lax.slice(key, (1,), (2,)), ())
    return k0, k1


_EMIT_KEY_PRIMITIVES = False


def key_primitives(enable: bool) -> bool:
    '''Trace split / random_bits / fold_in as key primitives instead of expanding them. Returns the previous setting.'''
    global _EMIT_KEY_PRIMITIVES
    previous, _EMIT_KEY_PRIMITIVES = _EMIT_KEY_PRIMITIVES, bool(enable)
    return previous


def _is_typed(key) -> bool:
    return isinstance(key, Tracer) and lax.core.is_key_dtype(key.dtype)


def key(seed):
    '''A typed key from an integer seed (traced values only).'''
    return lax.random_seed(seed)


def wrap_key_data(data):
    return lax.random_wrap(data)


def key_data(keys):
    return lax.random_unwrap(keys) if _is_typed(keys) else keys


def fold_in(key, data):
    data = lax.convert_element_type(data, np.uint32) if isinstance(data, Tracer) else np.uint32(data)
    if _is_typed(key):
        return lax.random_fold_in(key, data)
    if _EMIT_KEY_PRIMITIVES:
        return lax.random_unwrap(lax.random_fold_in(lax.random_wrap(key), data))
    return threefry_2x32(key, mnp.concatenate([np.zeros((1,), np.uint32), mnp.reshape(data, (1,))]))


def threefry_2x32(key, count):
    '''Apply the block function to a flat uint32 counter array of any length.'''
    k0, k1 = _key_halves(key)
    n      = int(np.prod(count.shape))
    flat   = mnp.reshape(count, (-1,))
    odd    = n % 2
    if odd:
        flat = mnp.concatenate([flat, np.zeros((1,), np.uint32)])
    x0, x1 = mnp.split(flat, 2)
    y0, y1 = lax.threefry2x32(k0, k1, x0, x1)
    out    = mnp.concatenate([y0, y1])
    if odd:
        out = lax.slice(out, (0,), (n,))
    return mnp.reshape(out, count.shape)


def split(key, num: int = 2):
    if _is_typed(key):
        return lax.random_split(key, (num,))
    if _EMIT_KEY_PRIMITIVES:
        return lax.random_unwrap(lax.random_split(lax.random_wrap(key), (num,)))
    counts = lax.iota(np.uint32, num * 2)
    return mnp.reshape(threefry_2x32(key, counts), (num, 2))


def random_bits(key, shape):
    if _is_typed(key):
        return lax.random_bits(key, 32, tuple(shape))
    if _EMIT_KEY_PRIMITIVES:
        return lax.random_bits(lax.random_wrap(key), 32, tuple(shape))
    size = int(np.prod(shape, dtype=np.int64))
    bits = threefry_2x32(key, lax.iota(np.uint32, size))
    return mnp.reshape(bits, tuple(shape))


def uniform(key, shape=(), dtype=np.float32, minval=0.0, maxval=1.0):
    if np.dtype(dtype) != np.float32:
        raise NotImplementedError('uniform: float32 only')
    shape  = tuple(shape)
    bits   = random_bits(key, shape)
    #23 random mantissa bits under the exponent of 1.0 give a float in [1, 2)
    fbits  = lax.bitwise_or(lax.shift_right_logical(bits, np.uint32(32 - 23)), np.uint32(0x3F800000))
    floats = lax.sub(lax.bitcast_convert_type(fbits, np.float32), np.float32(1.0))
    scaled = lax.add(lax.mul(floats, np.float32(maxval - minval)), np.float32(minval))
    return lax.max(np.float32(minval), mnp.reshape(scaled, shape))


def normal(key, shape=(), dtype=np.float32):
    '''Standard normal samples the way jax.random.normal draws them: uniform on (-1, 1), then
    sqrt(2) * erf_inv.'''
    if np.dtype(dtype) != np.float32:
        raise NotImplementedError('normal: float32 only')
    lo = np.nextafter(np.float32(-1.0), np.float32(0.0))
    u  = uniform(key, shape, dtype, minval=lo, maxval=1.0)
    return lax.mul(np.float32(np.sqrt(2)), lax.erf_inv(u))


def randint(key, shape, minval, maxval, dtype=np.int32):
    '''Integers in [minval, maxval) the way jax.random.randint draws them (int32, Python-integer bounds): two
    32-bit draws from the halves of a split key stand for one 64-bit number, whose remainder by the span is
    taken in 32-bit arithmetic as ((hi % span) * (2**32 % span) + lo % span) % span.
    (The reference runs this composition in tests/test_random.py:45-60.)'''
    if np.dtype(dtype) != np.int32:
        raise NotImplementedError('randint: int32 only')
    minval, maxval = int(minval), int(maxval)
    info = np.iinfo(np.int32)
    maxval_out_of_range = maxval > info.max
    minval, maxval = max(info.min, min(info.max, minval)), max(info.min, min(info.max, maxval))
    shape = tuple(shape)
    keys  = split(key)
    k1    = mnp.reshape(lax.slice(keys, (0, 0), (1, 2)), (2,))
    k2    = mnp.reshape(lax.slice(keys, (1, 0), (2, 2)), (2,))
    higher_bits, lower_bits = random_bits(k1, shape), random_bits(k2, shape)
    span = maxval - minval if maxval > minval else 1
    if maxval_out_of_range and maxval > minval:
        span += 1
    span = np.uint32(span)
    multiplier = np.uint32(2 ** 16) % span
    multiplier = np.uint32((int(multiplier) * int(multiplier)) & 0xFFFFFFFF) % span
    offset = lax.add(lax.mul(lax.rem(higher_bits, span), multiplier), lax.rem(lower_bits, span))
    offset = lax.rem(offset, span)
    return lax.add(np.int32(minval), lax.convert_element_type(offset, np.int32))
