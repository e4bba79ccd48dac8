'''Neural-network helpers as they appear in traced programs (relu under a custom-jvp
call, softmax as max / sub / exp / sum / div), so that the device path sees the same
primitive sequences as with `jax.nn`.'''
import numpy as np

from . import lax, numpy as mnp
from .tracer import custom_jvp


@custom_jvp
def relu(x):
    return mnp.maximum(x, 0)


@relu.defvjp
def _relu_vjp(g, ans, x):
    #jax.nn.relu's own rule: the cotangent passes where x > 0 (no share at x == 0). The test is made on the
    #result (max(x, 0) > 0 exactly where x > 0), so the backward pass does not keep the pre-activation alive
    shape = tuple(g.shape)
    zeros = lax.broadcast_in_dim(np.float32(0), shape, ()) if shape else np.float32(0)
    return (lax.select(lax.gt(ans, zeros), g, zeros),)


def softmax(x, axis=-1):
    unnormalized = mnp.exp(x - lax.stop_gradient(mnp.max(x, axis, keepdims=True)))
    return unnormalized / mnp.sum(unnormalized, axis, keepdims=True)


def log_softmax(x, axis=-1):
    shifted = x - lax.stop_gradient(mnp.max(x, axis, keepdims=True))
    return shifted - mnp.log(mnp.sum(mnp.exp(shifted), axis, keepdims=True))


def batch_norm_inference(x, scale, shift, mean, var, eps=1e-5):
    '''Inference-mode batch norm over the trailing (channel) axis, written the way
    flax/haiku modules of the period lower it: the per-channel factor first, then three
    full-size broadcasting passes.'''
    inv = scale * lax.rsqrt(var + np.float32(eps))
    return (x - mean) * inv + shift
