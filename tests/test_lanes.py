'''Launches on two lanes (vkjax_amd/lanes.py, vkj_seq_set_launch_lane): the plan orders every dependency between
launches - taken from the device allocations they touch, storage shared between buffers included - and a program
evaluated on two lanes gives the bits of the same program on one in-order stream. The reference has one in-order
sequence (vkjax/kompute_jaxpr_interpreter.py:55-60).'''
import numpy as np
import pytest

import vkjax_amd
from vkjax_amd import lanes, minijax as mj, workloads as W
from vkjax_amd.jaxpr_interpreter import JaxprInterpreter
from vkjax_amd.minijax import tree_util

from tests.test_training_path import small_convnet_inputs, small_mlp_inputs, tiny_resnet_inputs

SMALL = {'gather_scatter': lambda: W.gather_scatter_inputs(rows=4096, cols=64, n0=512, n1=16),
         'resnet50': lambda: W.resnet50_inputs(batch=2, size=64, num_classes=16, width_scale=0.25),
         'mlp': W.mlp_inputs, 'conv_block': lambda: W.conv_block_inputs(batch=2, size=20, channels=16),
         'rng_uniform': W.rng_inputs, 'mlp_train': small_mlp_inputs, 'convnet_train': small_convnet_inputs,
         'resnet50_train': tiny_resnet_inputs}


@pytest.mark.parametrize('name', sorted(SMALL) + ['gather_scatter at full size', 'resnet50 at batch 64'])
def test_plans_order_every_dependency(name):
    if name.endswith('full size'):
        fn, args = W.gather_scatter, W.gather_scatter_inputs()
    elif name.endswith('batch 64'):
        fn, args = W.resnet50, W.resnet50_inputs()
    else:
        fn, args = W.WORKLOADS[name][0], SMALL[name]()
    interp = JaxprInterpreter(mj.make_jaxpr(fn)(*args), plan_only=True, two_lanes=True)
    plan = interp.lane_plan
    lanes.check(plan)
    assert len(plan.lane) == len(interp.launches) and set(plan.lane) <= {0, 1}
    #a launch that nothing was moved away from keeps its place: with everything on one lane there are no waits
    assert any(plan.lane) or not any(plan.wait)
    if name == 'gather_scatter at full size':
        #the bucketing launch of the scatter-add depends on the indices only: it does not wait for the gather
        kernels = [l.kernel for l in interp.launches]
        rank = kernels.index('scatter_rows_rank')
        assert plan.lane[rank] == 1 and plan.lane[kernels.index('gather_rows_v4')] == 0
        assert kernels.index('gather_rows_v4') not in plan.depends_on[rank]
    if name == 'resnet50 at batch 64':
        assert sum(plan.lane) >= 4                           #the first block of every stage


def test_a_plan_that_misses_a_dependency_is_caught():
    plan = lanes.LanePlan(lane=[0, 1, 0], wait=[False, False, False], depends_on=[[], [0], [1]])
    with pytest.raises(AssertionError, match='may overtake'):
        lanes.check(plan)
    lanes.check(lanes.LanePlan(lane=[0, 1, 0], wait=[False, True, True], depends_on=[[], [0], [1]]))
    #a wait covers what was issued on the other lane BEFORE it: a later launch there is not covered
    with pytest.raises(AssertionError, match='may overtake'):
        lanes.check(lanes.LanePlan(lane=[0, 1, 0, 1, 0], wait=[False, False, True, False, False], depends_on=[[], [], [1], [], [3]]))


def test_default_is_one_lane():
    fn, args = W.gather_scatter, SMALL['gather_scatter']()
    assert JaxprInterpreter(mj.make_jaxpr(fn)(*args), plan_only=True).lane_plan is None


@pytest.mark.gpu
@pytest.mark.parametrize('name', sorted(SMALL))
def test_two_lanes_give_the_bits_of_one_stream(name):
    fn, args = W.WORKLOADS[name][0], SMALL[name]()
    if name == 'gather_scatter':
        args[2] = np.round(args[2] * 8)                      #(integer-valued updates: a small scatter-add adds atomically, in any order)
    print(f'case: {name}', flush=True)
    one = vkjax_amd.wrap(fn, frontend='minijax')
    two = vkjax_amd.wrap(fn, frontend='minijax', two_lanes=True)
    expected = tree_util.tree_leaves(one(*args))
    interp = two._get_or_create_jaxpr_interpreter(tuple(args))[0]
    for rep in range(3):                                      #the second lane is forked and joined anew by every evaluation
        got = tree_util.tree_leaves(two(*args))
        for a, b in zip(got, expected):
            assert np.array_equal(np.asarray(a), np.asarray(b), equal_nan=np.asarray(a).dtype.kind == 'f'), (name, rep)
    #replays (launches only, several in a row) join the lanes as well: same results afterwards
    interp.replay(3)
    for a, b in zip(interp.read_outputs(), expected):
        if a is not None:
            assert np.array_equal(np.asarray(a).reshape(-1), np.asarray(b).reshape(-1), equal_nan=True), name


@pytest.mark.gpu
def test_gather_beside_the_index_passes_at_full_size():
    table, idx, updates = W.gather_scatter_inputs()
    updates = np.round(updates * 8)
    two = vkjax_amd.wrap(W.gather_scatter, frontend='minijax', two_lanes=True)
    rows, acc = two(table, idx, updates)
    assert list(two._jaxpr_interpreters.values())[0].lane_plan.lane == [0, 1, 1]          #the gather beside both launches of the scatter-add
    assert np.array_equal(rows, table[idx])
    expected = np.zeros_like(table)
    np.add.at(expected, idx.reshape(-1), updates.reshape(-1, updates.shape[-1]))
    assert np.array_equal(acc, expected)
