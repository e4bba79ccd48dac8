'''Every case of the GPU parity matrices, and the five benchmark workloads, traced, evaluated by
the oracle and planned (ops, buffers, launch parameters) without a device: the host half of the
path that the GPU tests then execute.'''
import numpy as np
import pytest

from tests import test_gpu_basic_ops, test_gpu_conv
from tests.common import oracle_outputs
from vkjax_amd import minijax as mj, workloads as W
from vkjax_amd.jaxpr_interpreter import JaxprInterpreter

CASES = [(f, d, a) for f, d, a in test_gpu_basic_ops.param_matrix] + [(f, d, a) for f, d, a in test_gpu_conv.param_matrix] \
      + [(f, d, a) for f, d, a, _ in test_gpu_conv.pool_matrix]


@pytest.mark.parametrize('f,desc,args', CASES, ids=[c[1] for c in CASES])
def test_case_traces_evaluates_and_plans(f, desc, args):
    ytrue, closed = oracle_outputs(f, args)
    for fuse in (False, True):
        interp = JaxprInterpreter(closed, fuse=fuse, plan_only=True)
        for launch in interp.launches:
            assert all(g >= 1 for g in launch.grid) and launch.block[0] in (64, 256, 512, 1024)
            assert launch.grid[1] <= 65535 and launch.grid[0] * launch.block[0] < 2**32
        for b in interp.output_buffers:
            assert b is None or b.tensor is not None


def test_workloads_plan_at_full_size():
    expected_flops = {'affine': 2 * 8 * 128 * 16, 'mlp': 342360064, 'conv_block': 7398752256, 'resnet50': 523153440768 + 262144000}
    for name, (fn, make_inputs) in W.WORKLOADS.items():
        closed = mj.make_jaxpr(fn)(*make_inputs())
        interp = JaxprInterpreter(closed, plan_only=True)
        flops  = sum(l.flops for l in interp.launches)
        if name in expected_flops:
            assert flops == expected_flops[name], (name, flops)
        n_conv = sum(l.kernel.startswith('conv_gemm') for l in interp.launches)
        if name == 'resnet50':
            assert n_conv == 54      #53 convolutions + the dense layer
