'''vkj_seq_eval_next_static (the evaluation entry point that allocates nothing) against
vkj_seq_eval_next, through the C ABI: same program, same argument stream, results compared bit for
bit with each other and with numpy. Two runs in a row share the GPU's static landing array, the
second with a smaller input, so anything left over from the first would show. Arguments that do not
fit into the array are refused.'''
import ctypes as C

import numpy as np
import pytest

import vkjax_amd
from vkjax_amd import hip

pytestmark = pytest.mark.gpu


def _streamed(interp, batches, static_landing):
    '''Every batch through the interpreter's sequence, each one uploaded during the evaluation before it.'''
    seq, slot = interp.sequence, interp._input_slots[0]
    results = []
    for k, x in enumerate(batches):
        host = [None] * seq.n_slots
        if k == 0:
            host[slot] = x.reshape(-1).view(np.uint32)
        nxt = [None] * seq.n_slots
        if k + 1 < len(batches):
            nxt[slot] = batches[k + 1].reshape(-1).view(np.uint32)
        fresh = interp._fresh_outputs(host)
        seq.eval(host, flags=hip.EVAL_NULL_IS_RESIDENT, next_host_arrays=nxt if k + 1 < len(batches) else None,
                 static_landing=static_landing)
        results.append(interp._output_values(fresh)[0].copy())
    return results


def _program(x):
    return x * 3.0 + 1.0


def test_static_landing_matches_allocating_entry_point():
    rng = np.random.default_rng(7)
    for shape in ((3, 1000, 1001), (1200, 2048), (257,)):        #12 MB (odd size), 9.8 MB (chunked staging), then much smaller
        batches = [rng.standard_normal(shape).astype(np.float32) for _ in range(4)]
        a = vkjax_amd.wrap(_program, frontend='minijax')._get_or_create_jaxpr_interpreter((batches[0],))[0]
        b = vkjax_amd.wrap(_program, frontend='minijax')._get_or_create_jaxpr_interpreter((batches[0],))[0]
        expected = _streamed(a, batches, static_landing=False)
        got      = _streamed(b, batches, static_landing=True)
        for k, (g, e, x) in enumerate(zip(got, expected, batches)):
            assert np.array_equal(g.view(np.uint32), e.view(np.uint32)), (shape, k)
            assert np.array_equal(g, x * np.float32(3.0) + np.float32(1.0)), (shape, k)
        #the same sequence again: what the first stream left in the array and in the staging buffers does not matter
        again = _streamed(b, batches[::-1], static_landing=True)
        for k, (g, x) in enumerate(zip(again, batches[::-1])):
            assert np.array_equal(g, x * np.float32(3.0) + np.float32(1.0)), (shape, 'again', k)


def test_static_landing_refuses_what_does_not_fit():
    n = hip.STATIC_LANDING_BYTES // 4 + 64
    x = np.zeros(n, np.float32)
    interp = vkjax_amd.wrap(_program, frontend='minijax')._get_or_create_jaxpr_interpreter((x,))[0]
    seq, slot = interp.sequence, interp._input_slots[0]
    host = [None] * seq.n_slots
    host[slot] = x.view(np.uint32)
    fresh = interp._fresh_outputs(host)
    with pytest.raises(hip.HipError, match='static landing array holds'):
        seq.eval(host, next_host_arrays=list(host[:slot]) + [x.view(np.uint32)] + [None] * (seq.n_slots - slot - 1), static_landing=True)
    #the sequence is untouched by the refusal
    seq.eval(host, flags=0)
    assert np.array_equal(interp._output_values(fresh)[0], np.ones(n, np.float32))
    prof = vkjax_amd.wrap(_program, frontend='minijax', profiling=True)._get_or_create_jaxpr_interpreter((x[:16],))[0]
    h = [None] * prof.sequence.n_slots
    h[prof._input_slots[0]] = x[:16].view(np.uint32)
    prof._fresh_outputs(h)
    with pytest.raises(hip.HipError, match='timestamps'):
        prof.sequence.eval(h, next_host_arrays=[None] * len(h), static_landing=True)


def test_static_landing_with_graphs_switched_on():
    '''A program of one launch never becomes a graph, so it is evaluated although graphs are asked for; a program of
    several launches is refused until an ordinary evaluation has built its graph, and equals it afterwards.'''
    x = np.arange(4096, dtype=np.float32)
    one = vkjax_amd.wrap(_program, frontend='minijax', graph=True)._get_or_create_jaxpr_interpreter((x,))[0]
    assert len(one.launches) == 1
    got = _streamed(one, [x, x + 1, x + 2], static_landing=True)
    for k, g in enumerate(got):
        assert np.array_equal(g, (x + k) * np.float32(3.0) + np.float32(1.0)), k
    several = vkjax_amd.wrap(_program, frontend='minijax', graph=True, fuse=False)._get_or_create_jaxpr_interpreter((x,))[0]
    assert len(several.launches) == 2
    with pytest.raises(hip.HipError, match='graph has not been built'):
        _streamed(several, [x, x + 1], static_landing=True)
    expected = _streamed(several, [x, x + 1, x + 2], static_landing=False)
    got = _streamed(several, [x, x + 1, x + 2], static_landing=True)
    for g, e in zip(got, expected):
        assert np.array_equal(g.view(np.uint32), e.view(np.uint32))
