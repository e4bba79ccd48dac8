'''The module path under which the reference keeps its interpreter
(vkjax/kompute_jaxpr_interpreter.py:14; imported that way by vkjax/function.py:1 and by the
reference's tests, tests/common.py:7): `vkjax.kompute_jaxpr_interpreter.JaxprInterpreter`
resolves here as it does there. The class itself lives in `jaxpr_interpreter`.'''
from .jaxpr_interpreter import JaxprInterpreter, get_maximum_workgroup_size

__all__ = ['JaxprInterpreter', 'get_maximum_workgroup_size']
