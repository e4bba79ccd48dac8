'''vkJAX jaxpr interpreter on AMD Instinct MI355X: `wrap(f)` traces a function into a jaxpr and
executes it through hand-written gfx950 kernels behind a C-ABI HIP runtime.'''
from .function import Function, wrap
from . import minijax
from . import kompute_jaxpr_interpreter
