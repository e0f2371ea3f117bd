"""``jvp`` (nabla/transforms/jvp.py:41-125): trace the function, then push the tangents
forward through the trace (``core/forward.py``)."""
from __future__ import annotations

from typing import Any, Callable

from ..core import pytree
from ..core.forward import forward_on_trace
from ..core.tensor import Tensor
from ..core.tracing import trace


def jvp(fn: Callable, primals: tuple, tangents: tuple, *, has_aux: bool = False,
        create_graph: bool = True):
    """``(output, output_tangent)`` (plus ``aux`` with ``has_aux``) of ``fn`` at ``primals``
    along ``tangents``; outputs the tangents do not reach get zeros."""
    from ..ops.creation import zeros_like

    if not isinstance(primals, tuple):
        raise TypeError(f"primals must be a tuple, got {type(primals)}")
    if not isinstance(tangents, tuple):
        raise TypeError(f"tangents must be a tuple, got {type(tangents)}")
    if len(primals) != len(tangents):
        raise ValueError("primals and tangents must have the same length, "
                         f"got {len(primals)} and {len(tangents)}")
    aux_box = []

    def wrapped(*a):
        out = fn(*a)
        if has_aux:
            if not (isinstance(out, tuple) and len(out) == 2):
                raise ValueError("jvp: with has_aux=True the function must return (output, aux)")
            out, aux = out
            aux_box.append(aux)
        return out

    from ..core.tensor import BatchedTensor
    from .grad import lift_to_vmap_level
    # (inside vmap: primals and tangents carry the same hidden dimensions, see there)
    primals, tangents = lift_to_vmap_level(primals), lift_to_vmap_level(tangents)
    t = trace(wrapped, *primals)
    tmap = forward_on_trace(t, tangents, create_graph=create_graph)

    def tangent_of(x: Any) -> Any:
        if isinstance(x, Tensor):
            g = Tensor(impl=tmap[x._impl]) if x._impl in tmap else zeros_like(Tensor(impl=x._impl))
            return BatchedTensor(g, x._bd) if isinstance(x, BatchedTensor) else g
        return x

    out_tangents = pytree.tree_map(tangent_of, t.outputs)
    if has_aux:
        return t.outputs, out_tangents, aux_box[0]
    return t.outputs, out_tangents
