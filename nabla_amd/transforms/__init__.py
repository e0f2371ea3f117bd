from .compile import CompilationStats, CompiledFunction, compile
from .grad import grad, value_and_grad
from .jvp import jvp
from .vjp import vjp
