'''Stand-in for the parts of jax that `vkjax.wrap` needs when jax itself cannot be
imported: a jaxpr data model, pytrees, and a tracing front-end (`make_jaxpr`, `jit`,
`lax`, a numpy-like layer, `nn`, `random`).'''
from . import core, tree_util, lax, nn, random
from . import numpy
from .tracer import make_jaxpr, jit, custom_jvp, Tracer
from .autodiff import grad, value_and_grad
from .tree_util import tree_flatten, tree_unflatten, tree_leaves, tree_structure, tree_map, tree_multimap
