from .compile import CompilationStats, CompiledFunction, compile
from .grad import grad, value_and_grad
from .jacobian import jacfwd, jacrev
from .jvp import jvp
from .vjp import vjp
from .vmap import vmap
