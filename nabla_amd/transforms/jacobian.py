"""``jacrev`` and ``jacfwd`` (nabla/transforms/jacrev.py:27-115, jacfwd.py:32-119).

The reference walks the standard basis one direction at a time (jacrev.py:78-82 calls the
pullback once per output element, jacfwd.py:81-104 calls ``jvp`` once per input element) and
stacks the results.  ``jacrev`` here sends the whole basis through at once: it captures the
forward trace once (one ``vjp``) and maps its pullback over the identity with ``vmap``, so the
backward pass runs once on cotangents with a hidden axis of one direction per output element.
Where an op on the way has no batching rule ``vmap`` walks the directions one by one, which is the
reference's loop, and so does ``jacrev`` when it is itself called inside a ``vmap``.  ``jacfwd``
does the same with ``jvp``: the identity of an input as tangents with a hidden axis, one call per
input tensor.  Either way all rows are realised together in one plan.

The Jacobian of a function with one output tensor has shape ``(*out_shape, *in_shape)``;
several differentiated arguments give a tuple of Jacobians.  Several output tensors raise
``NotImplementedError`` with the reference's message (jacrev.py:191-194, jacfwd.py:189-192).
"""
from __future__ import annotations

from typing import Any, Callable

import numpy as np

from ..core import pytree
from ..core.tensor import Tensor
from .jvp import jvp
from .vjp import vjp


def resolve_argnums(argnums, n_args: int) -> tuple[int, ...]:
    """``None`` → every argument; negative indices count from the end
    (nabla/transforms/utils.py:52-67)."""
    if argnums is None:
        sel = tuple(range(n_args))
    elif isinstance(argnums, int):
        sel = (argnums,)
    else:
        sel = tuple(argnums)
    norm = tuple(a if a >= 0 else n_args + a for a in sel)
    for a in norm:
        if not 0 <= a < n_args:
            raise ValueError(f"argnum {a} out of bounds for {n_args} arguments")
    return norm


def _partial(fn: Callable, argnums, args: tuple):
    """The differentiated arguments and ``fn`` with the others held fixed
    (nabla/transforms/utils.py:112-127)."""
    norm = resolve_argnums(argnums, len(args))
    diff_args = tuple(args[i] for i in norm)

    def partial_func(*inner):
        full = list(args)
        for idx, a in zip(norm, inner):
            full[idx] = a
        return fn(*full)

    return diff_args, partial_func


def _tensor_leaves(tree: Any):
    return pytree.tree_flatten(tree, is_leaf=lambda x: isinstance(x, Tensor))


def _numel(t: Tensor) -> int:
    n = 1
    for d in t.shape:
        n *= int(d)
    return max(n, 1)


def _one_hot_like(t: Tensor, j: int | None) -> Tensor:
    """A tensor of ``t``'s shape and dtype that is one at flat position ``j`` (row-major) and
    zero elsewhere; all zeros for ``j = None`` (nabla/transforms/utils.py:130-156 builds the
    same vectors as rows of one host array)."""
    sh = tuple(int(d) for d in t.shape)
    a = np.zeros(max(int(np.prod(sh, dtype=np.int64)), 1), dtype=np.float32)
    if j is not None:
        a[j] = 1.0
    return Tensor.constant(a.reshape(sh), dtype=t.dtype)


def _identity_like(t: Tensor) -> Tensor:
    """The standard basis of ``t``'s space as one tensor ``(numel, *t.shape)``: slice ``j`` is the
    direction that selects element ``j`` (row-major)."""
    sh = tuple(int(d) for d in t.shape)
    n = max(int(np.prod(sh, dtype=np.int64)), 1)
    return Tensor.constant(np.eye(n, dtype=np.float32).reshape((n,) + sh), dtype=t.dtype)


def _basis(flat: list[Tensor]):
    """For every element of every tensor in ``flat``, the list of per-tensor directions that
    selects it."""
    sizes = [_numel(t) for t in flat]
    for k, n in enumerate(sizes):
        for j in range(n):
            yield [_one_hot_like(t, j if i == k else None) for i, t in enumerate(flat)]


_MULTI_OUT = ("{} with multiple output tensors is not yet supported. "
              "Wrap your function to return a single tensor.")


def jacrev(fn: Callable, argnums=None, has_aux: bool = False) -> Callable:
    """Jacobian by reverse mode: one pullback per output element."""
    from ..ops import batching
    from ..ops.view import reshape, stack
    from .vmap import vmap

    def jacrev_fn(*args: Any) -> Any:
        diff_args, partial_func = _partial(fn, argnums, args)
        if has_aux:
            output, pullback, aux = vjp(partial_func, *diff_args, has_aux=True)
        else:
            output, pullback = vjp(partial_func, *diff_args)
            aux = None
        flat_out, out_td = _tensor_leaves(output)
        if len(flat_out) != 1:
            raise NotImplementedError(_MULTI_OUT.format("jacrev"))
        flat_in, _ = _tensor_leaves(diff_args)
        if len(flat_in) != len(diff_args):
            raise NotImplementedError("jacrev: every differentiated argument must be one tensor")
        out_shape = tuple(int(d) for d in flat_out[0].shape)

        def pull(ct: Tensor):
            grads = pullback(pytree.tree_unflatten(out_td, [ct]))
            return tuple(_tensor_leaves(grads)[0])

        if batching.current_level() == 0:
            # the whole basis at once: cotangents with a hidden axis over a trace without one
            stacked = vmap(pull)(_identity_like(flat_out[0]))  # each (n_out, *in_shape)
        else:
            # inside a vmap the trace has hidden axes of its own, which a recorded op no longer
            # tells from the others: one replay per direction, as the reference does
            rows: list[list[Tensor]] = [[] for _ in flat_in]
            for direction in _basis(flat_out):
                for k, g in enumerate(pull(direction[0])):
                    rows[k].append(g)
            stacked = [r[0] if len(r) == 1 and not out_shape else stack(r, axis=0) for r in rows]
        jacs = []
        for j, x in zip(stacked, flat_in):
            in_shape = tuple(int(d) for d in x.shape)
            jacs.append(reshape(j, out_shape + in_shape))
        jac = jacs[0] if len(jacs) == 1 else tuple(jacs)
        return (jac, aux) if has_aux else jac

    return jacrev_fn


def jacfwd(fn: Callable, argnums=None, has_aux: bool = False) -> Callable:
    """Jacobian by forward mode: one ``jvp`` per input tensor over its whole basis (per input
    element where ``vmap`` cannot batch the function, inside a ``vmap``, or with ``has_aux``)."""
    from ..ops import batching
    from ..ops.creation import zeros_like
    from ..ops.view import permute, reshape, stack
    from .vmap import vmap

    def jacfwd_fn(*args: Any) -> Any:
        diff_args, partial_func = _partial(fn, argnums, args)
        flat_in, in_td = _tensor_leaves(diff_args)
        if len(flat_in) != len(diff_args):
            raise NotImplementedError("jacfwd: every differentiated argument must be one tensor")
        sizes = [_numel(t) for t in flat_in]

        aux = None
        out_shape: tuple[int, ...] = ()
        per_input: list[Tensor] = []  # for every input: (numel(input), *out_shape)
        if batching.current_level() == 0 and not has_aux:
            # one jvp per input tensor, its whole basis at once as tangents with a hidden axis
            for k, x in enumerate(flat_in):
                def push(tang: Tensor, k=k):
                    tangents = tuple(tang if i == k else zeros_like(t) for i, t in enumerate(flat_in))
                    _, tan = jvp(partial_func, tuple(diff_args), tangents)
                    t_flat, _ = _tensor_leaves(tan)
                    if len(t_flat) != 1:
                        raise NotImplementedError(_MULTI_OUT.format("jacfwd"))
                    return t_flat[0]

                col = vmap(push)(_identity_like(x))
                out_shape = tuple(int(d) for d in col.shape[1:])
                per_input.append(col)
        else:
            cols: list[Tensor] = []
            for direction in _basis(flat_in):
                tangents = pytree.tree_unflatten(in_td, direction)
                if not isinstance(tangents, tuple):
                    tangents = (tangents,)
                if has_aux:
                    out, tan, aux = jvp(partial_func, tuple(diff_args), tangents, has_aux=True)
                else:
                    out, tan = jvp(partial_func, tuple(diff_args), tangents)
                t_flat, _ = _tensor_leaves(tan)
                if len(t_flat) != 1:
                    raise NotImplementedError(_MULTI_OUT.format("jacfwd"))
                out_shape = tuple(int(d) for d in t_flat[0].shape)
                cols.append(t_flat[0])
            off = 0
            for n in sizes:
                chunk = cols[off:off + n]
                off += n
                per_input.append(stack(chunk, axis=0))

        jacs = []
        for x, j in zip(flat_in, per_input):
            in_shape = tuple(int(d) for d in x.shape)
            j = reshape(j, in_shape + out_shape)
            if in_shape and out_shape:
                ni, no = len(in_shape), len(out_shape)
                j = permute(j, tuple(range(ni, ni + no)) + tuple(range(ni)))
            jacs.append(j)
        jac = jacs[0] if len(jacs) == 1 else tuple(jacs)
        return (jac, aux) if has_aux else jac

    return jacfwd_fn


__all__ = ["jacrev", "jacfwd"]
