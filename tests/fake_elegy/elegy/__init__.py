'''Stand-in for the `elegy` package, for tests only: just enough of `elegy.Model` for
vkjax_amd/elegy.py (the counterpart of the reference's vkjax/elegy.py:6-35) to be imported and
its five wrapped steps to be exercised where elegy itself (and jax) cannot be installed. It keeps
elegy 0.7's step signatures - `call_pred_step(x, states, initializing, training)`,
`call_test_step(x, y_true, sample_weight, class_weight, states, initializing, training)`, and so on
(reference: tests/test_elegy_mlp.py:44,127-128) - and its protocol: the constructor calls
`jit_step()`, which installs the `*_jit` members that `predict`, `test_on_batch` and
`train_on_batch` go through. A module is a function `(params, x) -> y`, a loss a function
`(y_true, y_pred) -> scalar`, the optimizer plain SGD; states are `{'params': tree}`.
Nothing in the package imports this.'''
from vkjax_amd import minijax as mj


class Model:
    def __init__(self, module, loss=None, learning_rate: float = 0.1):
        self.module, self.loss, self.learning_rate = module, loss, learning_rate
        self.states         = None
        self.initialized    = False
        self.jitted_members = set()
        self.jit_step()

    # ---- the five steps (pure functions of their arguments; the last two arguments are static) ----
    def call_pred_step(self, x, states, initializing, training):
        return self.module(states['params'], x), states

    def call_summary_step(self, x, states, initializing, training):
        y = self.module(states['params'], x)
        return [mj.numpy.sum(y)], states

    def _loss(self, params, x, y_true):
        return self.loss(y_true, self.module(params, x))

    def call_test_step(self, x, y_true, sample_weight, class_weight, states, initializing, training):
        loss = self._loss(states['params'], x, y_true)
        return loss, {'loss': loss}, states

    def call_train_step(self, x, y_true, sample_weight, class_weight, states, initializing, training):
        loss, grads = mj.value_and_grad(self._loss)(states['params'], x, y_true)
        params = mj.tree_util.tree_map(lambda p, g: p - self.learning_rate * g, states['params'], grads)
        return {'loss': loss}, {'params': params}

    def call_init_step(self, x, states):
        return self.module(states['params'], x), states

    def jit_step(self):
        #elegy installs jax.jit-ted members here; subclasses replace them
        for name in ('summary', 'pred', 'test', 'train', 'init'):
            setattr(self, f'call_{name}_step_jit', getattr(self, f'call_{name}_step'))
            self.jitted_members.add(f'call_{name}_step_jit')

    # ---- what a user calls ----
    def predict(self, x):
        y, self.states = self.call_pred_step_jit(x, self.states, False, False)
        return y

    def test_on_batch(self, x, y):
        loss, logs, self.states = self.call_test_step_jit(x, y, None, None, self.states, False, False)
        return logs

    def train_on_batch(self, x, y):
        logs, self.states = self.call_train_step_jit(x, y, None, None, self.states, False, True)
        return logs
