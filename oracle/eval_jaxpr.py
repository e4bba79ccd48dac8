'''CPU oracle: evaluate a whole traced program with the numpy primitives.

TEST INFRASTRUCTURE ONLY (see primitives.py). This is the counterpart of the pure-JAX
evaluator the reference's tests compare every intermediate variable against
(reference: tests/common.py:12-51): it walks the equations in order, reads operands from
an environment, and writes results back; nested calls are evaluated recursively.
'''
import numpy as np

from . import primitives as P

_CALLS = {
    'xla_call':              lambda params: params['call_jaxpr'],
    'core_call':             lambda params: params['call_jaxpr'],
    'pjit':                  lambda params: params['jaxpr'],
    'jit':                   lambda params: params['jaxpr'],
    'closed_call':           lambda params: params['call_jaxpr'],
    'custom_jvp_call_jaxpr': lambda params: params['fun_jaxpr'],
    'custom_jvp_call':       lambda params: params['call_jaxpr'],
    'custom_vjp_call':       lambda params: params['call_jaxpr'] if 'call_jaxpr' in params else params['fun_jaxpr'],
    'custom_vjp_call_jaxpr': lambda params: params['call_jaxpr'] if 'call_jaxpr' in params else params['fun_jaxpr'],
    'remat':                 lambda params: params['call_jaxpr'],
}


def _physical(aval):
    '''A typed key array is held as its uint32 words: one more trailing dimension of 2.'''
    if type(aval.dtype).__name__ == 'KeyTy':
        return tuple(aval.shape) + (2,), np.dtype('uint32')
    return tuple(aval.shape), aval.dtype


def _canon_input(x, aval):
    shape, dtype = _physical(aval)
    return np.asarray(np.asarray(x), dtype=dtype).reshape(shape)


def eval_jaxpr(jaxpr, consts, *args, return_env=False):
    '''`jaxpr` is an open jaxpr (with .invars/.constvars/.eqns/.outvars), `consts` its
    constant values, `args` the flat argument leaves.'''
    env = {}

    def read(v):
        return np.asarray(v.val, dtype=v.aval.dtype) if hasattr(v, 'val') else env[v]

    assert len(args) == len(jaxpr.invars), (len(args), len(jaxpr.invars))
    for v, x in zip(jaxpr.invars, args):
        env[v] = _canon_input(x, v.aval)
    for v, x in zip(jaxpr.constvars, consts):
        env[v] = _canon_input(x, v.aval)

    for eqn in jaxpr.eqns:
        invals = [read(v) for v in eqn.invars]
        name   = eqn.primitive.name
        if name in _CALLS:
            inner = _CALLS[name](eqn.params)
            inner_consts = getattr(inner, 'consts', [])
            inner = getattr(inner, 'jaxpr', inner)
            outvals, inner_env = eval_jaxpr(inner, inner_consts, *invals, return_env=True)
            env.update(inner_env)
        else:
            fn = getattr(P, name.replace('-', '_'), None) or P.__dict__.get(name)
            if fn is None:
                raise NotImplementedError(f'oracle has no primitive {name}')
            params = {k: v for k, v in eqn.params.items()}
            if name in ('iota',):
                outvals = fn(**params)
            else:
                outvals = fn(*invals, **params)
            if not eqn.primitive.multiple_results:
                outvals = [outvals]
        for v, val in zip(eqn.outvars, outvals):
            val = np.asarray(val)
            shape, dtype = _physical(v.aval)
            assert val.shape == shape, (name, val.shape, shape)
            assert val.dtype == dtype, (name, val.dtype, dtype)
            env[v] = val

    outs = [read(v) for v in jaxpr.outvars]
    return (outs, env) if return_env else outs


def eval_closed_jaxpr(closed, *args, return_env=False):
    return eval_jaxpr(closed.jaxpr, closed.consts, *args, return_env=return_env)
