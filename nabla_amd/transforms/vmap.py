"""``vmap`` (nabla/transforms/vmap.py:291-362): map a function over one axis of its arguments.

Two ways to run the mapped function, with the same results:

* **batched** (the reference's way: hidden batch dimensions and a batching rule per op).  The
  mapped axis goes to the front, the function is called ONCE on ``BatchedTensor`` views that
  hide that axis, and every op call translates its axes and runs on the whole batch
  (nabla_amd/ops/batching.py).  The cost does not grow with the batch size: per-example
  gradients of a model are one forward and one backward pass over the batch.
* **element by element**: the function is traced once per batch element on slices of the
  arguments and the results are stacked, all inside one lazy graph.  Used when the function
  reaches an op that has no batching rule (scatters, gathers from a mapped table, convolutions
  with a mapped filter, the backward ops when called directly, custom kernels, optimizer and
  random ops) or when ``config.VMAP_BATCHED`` is off.

Composition (``grad`` of ``vmap``, ``vmap`` of ``grad``, nesting) is the reference's either way.

``in_axes`` / ``out_axes`` follow the reference (vmap.py:44-60, 63-150): an int or ``None`` for
every argument, a tuple / list with one entry per argument, and an entry may itself be a
container that matches the argument's structure (a scalar entry applies to every leaf).
"""
from __future__ import annotations

from typing import Any, Callable

from ..core.tensor import Tensor


def _broadcast_to_args(spec: Any, n: int) -> tuple:
    if isinstance(spec, (int, type(None))):
        return (spec,) * n
    if isinstance(spec, (list, tuple)):
        if len(spec) != n:
            raise ValueError(f"in_axes/out_axes length ({len(spec)}) != number of args ({n})")
        return tuple(spec)
    if isinstance(spec, dict):
        if n == 1:
            return (spec,)
        raise TypeError(f"Dict axis spec with {n} args — use tuple/list for multiple args")
    raise TypeError(f"Invalid axis spec type: {type(spec).__name__}")


def _walk(fn: Callable, tree: Any, spec: Any) -> Any:
    """Apply ``fn(leaf, axis)`` over ``tree`` with ``spec`` as a prefix of its structure."""
    if isinstance(tree, Tensor):
        if not isinstance(spec, (int, type(None))):
            raise TypeError(f"axis spec for a tensor must be int or None, got {type(spec).__name__}")
        return fn(tree, spec)
    if isinstance(tree, dict):
        sub = (lambda k: spec[k]) if isinstance(spec, dict) else (lambda k: spec)
        return {k: _walk(fn, v, sub(k)) for k, v in tree.items()}
    if isinstance(tree, (list, tuple)):
        if isinstance(spec, (list, tuple)):
            if len(spec) != len(tree):
                raise ValueError(f"axis spec length ({len(spec)}) != container length ({len(tree)})")
            items = [_walk(fn, v, s) for v, s in zip(tree, spec)]
        else:
            items = [_walk(fn, v, spec) for v in tree]
        return type(tree)(items) if not hasattr(tree, "_fields") else type(tree)(*items)
    return tree  # not a tensor: passed through to every call


def _batch_sizes(args: tuple, in_ax: tuple) -> list[int]:
    dims: list[int] = []

    def see(t: Tensor, ax):
        if ax is not None:
            nd = len(t.shape)
            if not -nd <= ax < nd:
                raise ValueError(f"vmap: axis {ax} out of range for a tensor of rank {nd}")
            dims.append(int(t.shape[ax]))
        return t

    for a, ax in zip(args, in_ax):
        _walk(see, a, ax)
    return dims


def vmap(func: Callable | None = None, in_axes: Any = 0, out_axes: Any = 0,
         axis_size: int | None = None, spmd_axis_name: str | None = None, mesh: Any = None) -> Callable:
    """Vectorise ``func`` over one axis of its arguments (usable as a decorator)."""
    if func is None:
        return lambda f: vmap(f, in_axes=in_axes, out_axes=out_axes, axis_size=axis_size,
                              spmd_axis_name=spmd_axis_name, mesh=mesh)
    if spmd_axis_name is not None or mesh is not None:
        raise NotImplementedError("vmap: sharding the mapped axis over a device mesh is not part of "
                                  "this one-GPU backend")

    def vectorized(*args: Any) -> Any:
        from .. import config
        from ..ops.batching import NoBatchRule
        from ..ops.view import moveaxis, stack

        if not args:
            raise ValueError("vmap requires at least one input argument.")
        in_ax = _broadcast_to_args(in_axes, len(args))
        dims = _batch_sizes(args, in_ax)
        if not dims:
            if axis_size is None:
                raise ValueError("All in_axes are None. Must specify axis_size.")
            size = int(axis_size)
        else:
            if any(d != dims[0] for d in dims):
                raise ValueError(f"Inconsistent batch dims: {dims}")
            size = dims[0]
            if axis_size is not None and int(axis_size) != size:
                raise ValueError(f"axis_size={axis_size} doesn't match inferred {size}")
        if config.VMAP_BATCHED and size > 0:
            try:
                return _run_batched(func, args, in_ax, out_axes, size)
            except NoBatchRule:
                pass  # an op of the function has no batching rule: map element by element

        # the mapped axis goes to the front once, then element i is a leading-index view
        fronted = tuple(_walk(lambda t, ax: t if ax is None else moveaxis(t, ax, 0), a, ax)
                        for a, ax in zip(args, in_ax))
        results = []
        for i in range(size):
            sliced = tuple(_walk(lambda t, ax: t if ax is None else t[i], a, ax)
                           for a, ax in zip(fronted, in_ax))
            results.append(func(*sliced))
        empty = size == 0
        if empty:
            # nothing to map over: one call on a stand-in element (zeros of an element's shape)
            # tells the structure and the element shapes of the result, which then comes back
            # with a mapped axis of length 0
            from ..ops.creation import zeros
            stand_in = tuple(_walk(lambda t, ax: t if ax is None else
                                   zeros(tuple(t.shape[1:]), dtype=t.dtype, device=t.device), a, ax)
                             for a, ax in zip(fronted, in_ax))
            results.append(func(*stand_in))

        first = results[0]
        is_single = not isinstance(first, (list, tuple))
        out_lists = [[r] if is_single else list(r) for r in results]
        out_ax = _broadcast_to_args(out_axes, len(out_lists[0]))

        def gather(k: int, spec: Any) -> Any:
            # walk the k-th output of every call in parallel, stacking tensor leaves
            def rec(nodes: list, sp: Any) -> Any:
                head = nodes[0]
                if isinstance(head, Tensor):
                    if sp is None:
                        return head
                    ax = sp if sp >= 0 else sp + len(head.shape) + 1
                    if empty:
                        from ..ops.creation import zeros
                        shape = list(head.shape)
                        shape.insert(ax, 0)
                        return zeros(tuple(shape), dtype=head.dtype, device=head.device)
                    return stack(nodes, axis=ax)
                if isinstance(head, dict):
                    return {key: rec([n[key] for n in nodes], sp[key] if isinstance(sp, dict) else sp)
                            for key in head}
                if isinstance(head, (list, tuple)):
                    subs = sp if isinstance(sp, (list, tuple)) else (sp,) * len(head)
                    items = [rec([n[j] for n in nodes], subs[j]) for j in range(len(head))]
                    return type(head)(items) if not hasattr(head, "_fields") else type(head)(*items)
                return head
            return rec([o[k] for o in out_lists], spec)

        stacked = [gather(k, ax) for k, ax in enumerate(out_ax)]
        return stacked[0] if is_single else type(first)(stacked)

    return vectorized


def _run_batched(func: Callable, args: tuple, in_ax: tuple, out_axes: Any, size: int) -> Any:
    """One call of ``func`` on views that hide the mapped axis (see the module docstring)."""
    from ..core.tensor import BatchedTensor
    from ..ops import batching
    from ..ops.view import broadcast_to, moveaxis, reshape

    outer = batching.current_level()
    level = outer + 1

    def hide(t: Tensor, ax):
        if ax is None:
            return t
        # the mapped axis becomes the last hidden dimension: behind those of the vmap calls
        # this one is nested in (which a tensor that does not come from them lacks: size 1)
        own = batching.batch_dims_of(t)
        front = moveaxis(t, ax, 0)  # (a logical move: hidden dimensions stay in front)
        phys = batching.plain(front)
        if own < outer:
            shape = tuple(phys.shape)
            phys = reshape(phys, shape[:own] + (1,) * (outer - own) + shape[own:])
        return BatchedTensor(phys, level)

    wrapped = tuple(_walk(hide, a, ax) for a, ax in zip(args, in_ax))
    batching.push_level(size)
    try:
        result = func(*wrapped)
    finally:
        batching.pop_level()

    is_single = not isinstance(result, (list, tuple))
    outs = [result] if is_single else list(result)
    out_ax = _broadcast_to_args(out_axes, len(outs))

    def show(t: Tensor, ax):
        own = batching.batch_dims_of(t)
        if own < level:
            # does not depend on the mapped arguments: the same for every element
            if ax is None:
                return t
            lshape = tuple(t.shape)
            rep = broadcast_to(reshape(t, (1,) + lshape), (size,) + lshape)
            return moveaxis(rep, 0, ax if ax >= 0 else ax + len(lshape) + 1)
        if ax is None:
            raise ValueError("vmap: out_axes is None for a result that depends on a mapped argument")
        phys = batching.plain(t)
        if phys.shape[outer] != size:  # a size-1 hidden dimension that was never broadcast
            shape = tuple(phys.shape)
            phys = broadcast_to(phys, shape[:outer] + (size,) + shape[outer + 1:])
        seen = BatchedTensor(phys, outer) if outer > 0 else phys
        nd = len(seen.shape)
        return moveaxis(seen, 0, ax if ax >= 0 else ax + nd)

    shown = [_walk(show, o, ax) for o, ax in zip(outs, out_ax)]
    return shown[0] if is_single else type(result)(shown)


__all__ = ["vmap"]
