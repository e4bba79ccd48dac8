'''Shared helpers of the parity tests: run a function through the device path and through the
CPU oracle on the same inputs and compare structure, shapes, dtypes and values, the way the
reference's tests compare vkjax against JAX's CPU backend (reference: tests/test_basic_ops.py:336-362).'''
import numpy as np

import vkjax_amd
from vkjax_amd import minijax as mj
from vkjax_amd.minijax import tree_util
from oracle.eval_jaxpr import eval_closed_jaxpr


def oracle_outputs(f, args, static_argnums=()):
    closed, shapes = mj.make_jaxpr(f, static_argnums, return_shape=True)(*args)
    leaves = tree_util.tree_leaves([a for i, a in enumerate(args) if i not in static_argnums])
    flat   = eval_closed_jaxpr(closed, *leaves)
    return tree_util.tree_unflatten(tree_util.tree_structure(shapes), flat), closed


def assert_tree_close(y, ytrue, rtol=1e-5, atol=1e-8, exact=False, what=''):
    assert tree_util.tree_structure(y) == tree_util.tree_structure(ytrue), what
    for a, b in zip(tree_util.tree_leaves(y), tree_util.tree_leaves(ytrue)):
        a, b = np.asarray(a), np.asarray(b)
        assert a.shape == b.shape, (what, a.shape, b.shape)
        assert a.dtype == b.dtype, (what, a.dtype, b.dtype)
        if exact or a.dtype.kind in 'iub':
            if not np.array_equal(a, b, equal_nan=a.dtype.kind == 'f'):
                bad = np.argwhere(~((a == b) | ((a != a) & (b != b)) if a.dtype.kind == 'f' else a != b))
                raise AssertionError(f'{what}: {len(bad)} of {a.size} elements differ, first at {bad[:3].tolist()}: '
                                     f'{a[tuple(bad[0])]!r} vs {b[tuple(bad[0])]!r}')
        else:
            if not np.allclose(a, b, rtol=rtol, atol=atol, equal_nan=True):
                err = np.abs(a.astype(np.float64) - b) / (atol + rtol * np.abs(b))
                i = np.unravel_index(np.nanargmax(err), err.shape) if err.ndim else ()
                raise AssertionError(f'{what}: max |err|/(atol+rtol|y|) = {np.nanmax(err):.3g} at {i}: {a[i]!r} vs {b[i]!r}')


def check_against_oracle(f, args, rtol=1e-5, atol=1e-8, exact=False, static_argnums=(), **wrap_kwargs):
    ytrue, closed = oracle_outputs(f, args, static_argnums)
    vkfunc = vkjax_amd.wrap(f, static_argnums=static_argnums, frontend='minijax', **wrap_kwargs)
    y = vkfunc(*args)
    assert_tree_close(y, ytrue, rtol, atol, exact, what=getattr(f, '__name__', 'f'))
    return y, ytrue, vkfunc
