'''`vkModel` (reference: vkjax/elegy.py:6-35, exercised by tests/test_elegy_mlp.py:37-129): an elegy model whose
five jitted steps go through `wrap`. elegy (and jax) cannot be installed here, so the class is imported against
the stand-in package in tests/fake_elegy, which keeps elegy's step signatures and its jit_step protocol; the
module under test, vkjax_amd/elegy.py, is the real one. CPU part: what jit_step installs. GPU part: predict, a
test step and an SGD step through the wrapped members against the CPU oracle, as the reference compares its
vkModel with the plain elegy model.'''
import importlib
import os
import sys

import numpy as np
import pytest

from vkjax_amd import minijax as mj
from vkjax_amd.minijax import tree_util

jnp, nn = mj.numpy, mj.nn
FAKE = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'fake_elegy')


@pytest.fixture()
def vkelegy(monkeypatch):
    '''vkjax_amd.elegy imported with the stand-in `elegy` in sys.modules; both are gone again afterwards.'''
    monkeypatch.syspath_prepend(FAKE)
    for name in ('elegy', 'vkjax_amd.elegy'):
        monkeypatch.delitem(sys.modules, name, raising=False)
    module = importlib.import_module('vkjax_amd.elegy')
    yield module
    for name in ('elegy', 'vkjax_amd.elegy'):
        sys.modules.pop(name, None)


def mlp(params, image):
    '''Flatten, Linear, relu, Linear, relu, Linear (reference: tests/test_elegy_mlp.py:19-32)'''
    x = image.reshape(image.shape[0], -1)
    for k, (w, b) in enumerate(params):
        x = jnp.dot(x, w) + b
        if k + 1 < len(params):
            x = nn.relu(x)
    return x


def cross_entropy(y_true, logits):
    '''sparse categorical cross-entropy of integer labels, averaged (reference: tests/test_elegy_mlp.py:62-64)'''
    logp = nn.log_softmax(logits, axis=-1)
    return -jnp.take_along_axis(logp, y_true[:, np.newaxis], axis=-1).ravel().mean()


def make_states(rng, sizes=(2 * 8 * 8 * 3, 48, 32, 10)):
    layers = [((rng.standard_normal((a, b)) * np.sqrt(2.0 / a)).astype(np.float32), (rng.standard_normal(b) * 0.1).astype(np.float32))
              for a, b in zip(sizes[:-1], sizes[1:])]
    return {'params': layers}


def test_jit_step_installs_the_five_wrapped_steps(vkelegy):
    import vkjax_amd
    model = vkelegy.vkModel(mlp, cross_entropy)
    expected = {'call_summary_step_jit': (2, 3), 'call_pred_step_jit': (2, 3), 'call_test_step_jit': (5, 6),
                'call_train_step_jit': (5, 6), 'call_init_step_jit': ()}
    assert set(expected) <= model.jitted_members
    for name, static in expected.items():
        member = getattr(model, name)
        assert isinstance(member, vkjax_amd.Function), name
        assert member._static_argnums == static, (name, member._static_argnums)
    assert issubclass(vkelegy.vkModel, sys.modules['elegy'].Model)


def test_stand_in_train_step_equals_torch_autograd(vkelegy):
    '''The oracle's value of the stand-in model's SGD step (log-softmax, the gather of take_along_axis and its
    scatter-add gradient, three dense layers) against torch autograd, an independent implementation.'''
    import torch
    from oracle.eval_jaxpr import eval_closed_jaxpr
    rng = np.random.default_rng(3)
    x = rng.random((6, 2 * 8, 8, 3), dtype=np.float32)
    y = rng.integers(0, 10, size=6).astype(np.int32)
    states = make_states(rng)
    model = sys.modules['elegy'].Model(mlp, cross_entropy, learning_rate=0.25)
    closed = mj.make_jaxpr(model.call_train_step, (5, 6))(x, y, None, None, states, False, True)
    loss, *updated = eval_closed_jaxpr(closed, *tree_util.tree_leaves([x, y, states]))
    params = [(torch.tensor(w, dtype=torch.float64, requires_grad=True), torch.tensor(b, dtype=torch.float64, requires_grad=True))
              for w, b in states['params']]
    h = torch.tensor(x.reshape(6, -1), dtype=torch.float64)
    for k, (w, b) in enumerate(params):
        h = h @ w + b
        if k + 1 < len(params):
            h = torch.relu(h)
    tloss = torch.nn.functional.cross_entropy(h, torch.tensor(y).long())
    tloss.backward()
    assert np.allclose(loss, tloss.item(), rtol=1e-5)
    for got, p in zip(updated, [p for pair in params for p in pair]):
        assert np.allclose(got, (p - 0.25 * p.grad).detach().numpy(), rtol=1e-4, atol=1e-6)


@pytest.mark.gpu
def test_vkmodel_steps_match_the_oracle(vkelegy):
    from oracle.eval_jaxpr import eval_closed_jaxpr
    from tests.common import assert_tree_close
    elegy = sys.modules['elegy']
    rng = np.random.default_rng(21)
    x = rng.random((6, 2 * 8, 8, 3), dtype=np.float32)
    y = rng.integers(0, 10, size=6).astype(np.int32)
    states = make_states(rng)
    model, vkmodel = elegy.Model(mlp, cross_entropy), vkelegy.vkModel(mlp, cross_entropy)
    model.states = vkmodel.states = states
    vkmodel.initialized = True

    def oracle(step, static_argnums, *args):
        closed, shapes = mj.make_jaxpr(step, static_argnums, return_shape=True)(*args)
        leaves = tree_util.tree_leaves([a for i, a in enumerate(args) if i not in static_argnums])
        return tree_util.tree_unflatten(tree_util.tree_structure(shapes), eval_closed_jaxpr(closed, *leaves))

    #predict: call_pred_step_jit(x, states, False, False), as tests/test_elegy_mlp.py:44-58
    ypred, states_out = vkmodel.call_pred_step_jit(x, states, False, False)
    ytrue, _ = oracle(model.call_pred_step, (2, 3), x, states, False, False)
    assert_tree_close(ypred, ytrue, rtol=1e-4, atol=1e-6, what='call_pred_step_jit')
    assert_tree_close(states_out, states, exact=True, what='states pass through')
    assert np.allclose(vkmodel.predict(x), ytrue, rtol=1e-4, atol=1e-6)
    assert len(vkmodel.call_pred_step_jit._jaxpr_interpreters) == 1          #traced once, reused by predict()

    logs = vkmodel.test_on_batch(x, y)
    loss_true, _, _ = oracle(model.call_test_step, (5, 6), x, y, None, None, states, False, False)
    assert np.allclose(logs['loss'], loss_true, rtol=1e-4, atol=1e-6)

    #one SGD step: logs and every updated parameter (tests/test_elegy_mlp.py:110-118)
    logs_true, states_true = oracle(model.call_train_step, (5, 6), x, y, None, None, states, False, True)
    logs = vkmodel.train_on_batch(x, y)
    assert_tree_close(logs, logs_true, rtol=1e-4, atol=1e-6, what='train logs')
    assert_tree_close(vkmodel.states, states_true, rtol=1e-4, atol=1e-6, what='updated states')
    assert float(vkmodel.test_on_batch(x, y)['loss']) < float(loss_true)     #the step went downhill

    summary, _ = vkmodel.call_summary_step_jit(x, states, False, False)
    assert np.allclose(summary[0], np.sum(ytrue, dtype=np.float64), rtol=1e-4)
    y_init, _ = vkmodel.call_init_step_jit(x, states)
    assert np.allclose(y_init, ytrue, rtol=1e-4, atol=1e-6)
