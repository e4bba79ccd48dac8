'''The fp32 torch-CPU graphs that bench.py times as the CPU baseline (and compares the GPU results
with) against the numpy oracle of the traced programs, on small inputs: two independent
implementations of the same layers have to agree.'''
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench
from oracle.eval_jaxpr import eval_closed_jaxpr
from vkjax_amd import minijax as mj, workloads as W
from vkjax_amd.minijax import tree_util

CASES = [('affine', {}, 1e-5), ('mlp', dict(batch=16), 1e-4), ('conv_block', dict(batch=2, size=15, channels=8), 1e-4),
         ('resnet50', dict(batch=2, size=64, num_classes=32, width_scale=0.25), 1e-3),
         ('gather_scatter', dict(rows=50, cols=12, n0=9, n1=7), 1e-5)]


@pytest.mark.parametrize('workload,kwargs,rtol', CASES, ids=[c[0] for c in CASES])
def test_torch_graph_equals_oracle(workload, kwargs, rtol):
    fn, make_inputs = W.WORKLOADS[workload]
    inputs = make_inputs(**kwargs)
    run = bench.torch_cpu_graph(workload, inputs)
    got = run()
    expected = eval_closed_jaxpr(mj.make_jaxpr(fn)(*inputs), *tree_util.tree_leaves(inputs))
    assert len(got) == len(expected)
    for a, b in zip(got, expected):
        b = np.asarray(b)
        assert a.shape == b.shape
        if np.issubdtype(b.dtype, np.floating):
            assert np.allclose(a, b, rtol=rtol, atol=1e-5 * float(np.abs(b).max())), float(np.abs(a - b).max())
        else:
            assert np.array_equal(a, b)


def test_threefry_draw_has_no_torch_graph():
    assert bench.torch_cpu_graph('rng_uniform', W.rng_inputs()) is None


def test_check_outputs_flags_a_wrong_result():
    x = np.linspace(-1, 1, 50, dtype=np.float32).reshape(5, 10)
    assert bench.check_outputs([x, x.argmax(1)], [x.copy(), x.argmax(1)], 1e-4)['ok']
    y = x.copy(); y[2, 3] += 0.01
    assert not bench.check_outputs([y], [x], 1e-4)['ok']
