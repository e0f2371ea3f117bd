"""``grad`` / ``value_and_grad`` (nabla/transforms/grad.py:21-172)."""
from __future__ import annotations

from typing import Any, Callable

from ..core import pytree
from ..core.backward import backward_on_trace
from ..core.tensor import Tensor
from ..core.tracing import trace
from .utils import select_argnums


def lift_to_vmap_level(args):
    """Inside ``vmap``, a derivative is taken per element of the batch, also with respect to an
    argument that is the same for every element: such an argument is given the hidden
    dimensions of the running ``vmap`` calls (a broadcast view) before the function is traced,
    so that its gradient comes back with one slice per element instead of their sum."""
    from ..core.tensor import BatchedTensor
    from ..ops import batching

    level = batching.current_level()
    if not level:
        return args
    sizes = batching.level_sizes()

    def up(t):
        if isinstance(t, Tensor) and batching.batch_dims_of(t) < level:
            return BatchedTensor(batching.lift(t, level, sizes), level)
        return t

    return pytree.tree_map(up, args)


def _run(fun, argnums, create_graph, realize, args, kwargs, with_value: bool):
    from ..ops.creation import ones_like

    args = lift_to_vmap_level(args)
    t = trace(fun, *args, **kwargs)
    output = t.outputs
    if not isinstance(output, Tensor):
        raise TypeError(f"grad: output must be a Tensor, got {type(output)}")
    seed = ones_like(Tensor(impl=output._impl))  # (with the hidden dimensions, inside vmap)
    grads_map = backward_on_trace(t, seed, create_graph=create_graph)
    leaves = pytree.tree_leaves(args)
    grad_leaves = []
    for inp in leaves:
        g = grads_map.get(inp) if isinstance(inp, Tensor) else None
        if g is not None and not inp.dtype.is_float():
            g = None  # non-differentiable dtypes get no gradient (transforms/utils.py:19-37)
        grad_leaves.append(g)
    if realize and not create_graph:
        from .. import config
        from ..core.engine import GRAPH
        targets = [output] if with_value and not output.real else []
        targets += [g for g in grad_leaves if isinstance(g, Tensor) and not g.real]
        if targets and not config.TRACING:
            GRAPH.evaluate(*targets)
    struct = pytree.tree_unflatten(pytree.tree_structure(args), grad_leaves)
    return output, select_argnums(struct, argnums)


def grad(fun: Callable, argnums: int | tuple[int, ...] = 0, create_graph: bool = True,
         realize: bool = True) -> Callable:
    """Gradient of a scalar-valued ``fun`` w.r.t. the positional args ``argnums``.
    With the default ``create_graph=True`` the result stays lazy."""

    def wrapper(*args: Any, **kwargs: Any):
        return _run(fun, argnums, create_graph, realize, args, kwargs, False)[1]

    return wrapper


def value_and_grad(fun: Callable, argnums: int | tuple[int, ...] = 0, create_graph: bool = True,
                   realize: bool = True) -> Callable:
    """``(fun(*args), gradient)`` sharing one forward pass."""

    def wrapper(*args: Any, **kwargs: Any):
        return _run(fun, argnums, create_graph, realize, args, kwargs, True)

    return wrapper
