"""``vjp`` (nabla/transforms/vjp.py:28-94)."""
from __future__ import annotations

from typing import Any, Callable

from ..core import pytree
from ..core.backward import backward_on_trace
from ..core.tensor import Tensor
from ..core.tracing import trace


def vjp(fun: Callable, *primals: Any, has_aux: bool = False, create_graph: bool = True):
    """Returns ``(output, vjp_fn)``; ``vjp_fn(cotangent)`` gives one gradient per primal."""
    aux_box = []

    def wrapped(*a):
        out = fun(*a)
        if has_aux:
            out, aux = out
            aux_box.append(aux)
        return out

    from .grad import lift_to_vmap_level
    primals = lift_to_vmap_level(primals)  # (inside vmap: per-element gradients, see there)
    t = trace(wrapped, *primals)
    output = t.outputs

    def vjp_fn(cotangent: Any):
        cotangent = lift_to_vmap_level(cotangent)
        grads_map = backward_on_trace(t, cotangent, create_graph=create_graph)
        leaves = pytree.tree_leaves(primals)
        gl = [grads_map.get(x) if isinstance(x, Tensor) else None for x in leaves]
        return tuple(pytree.tree_unflatten(pytree.tree_structure(primals), gl))

    if has_aux:
        return output, vjp_fn, aux_box[0]
    return output, vjp_fn
