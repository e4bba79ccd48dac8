'''`vkModel`: an elegy model whose jitted steps run through `vkjax_amd.wrap` instead of
`jax.jit`, with the same static arguments as the reference (vkjax/elegy.py:6-35).
Importing this module needs `elegy` (and therefore jax); it is not imported by the package.'''
import elegy

from . import wrap


class vkModel(elegy.Model):
    def jit_step(self):
        self.call_summary_step_jit = wrap(self.call_summary_step, static_argnums=[2, 3])
        self.call_pred_step_jit    = wrap(self.call_pred_step,    static_argnums=[2, 3])
        self.call_test_step_jit    = wrap(self.call_test_step,    static_argnums=[5, 6])
        self.call_train_step_jit   = wrap(self.call_train_step,   static_argnums=[5, 6])
        self.call_init_step_jit    = wrap(self.call_init_step,    static_argnums=[])
        self.jitted_members |= {'call_summary_step_jit', 'call_pred_step_jit', 'call_test_step_jit',
                                'call_train_step_jit', 'call_init_step_jit'}
