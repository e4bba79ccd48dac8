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
