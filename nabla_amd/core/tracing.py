"""Trace data model: the op list that autodiff replays and the lowering walks.

Mirrors nabla/core/graph/tracing.py: ``OpNode`` (25-65), ``Trace`` with its DFS
topology (87-187) and ``trace(fn, *args)`` (383-414).  ``op_kwargs`` are the
ORIGINAL keyword arguments of the op call (nabla/ops/base.py:530-537).
"""
from __future__ import annotations

from typing import Any, Callable

from .pytree import PyTreeDef, tree_leaves
from .tensor import Tensor, TensorImpl


class OpNode:
    """One recorded op call: its output impls (siblings), the op, and its inputs."""

    __slots__ = ("_refs", "tree_def", "op", "op_args", "op_kwargs", "_op_hash")

    def __init__(self, _refs, tree_def: PyTreeDef | None, op, op_args, op_kwargs, _op_hash=None):
        if tree_def is not None and len(_refs) != tree_def.num_leaves:
            raise ValueError(
                f"OpNode: ref count {len(_refs)} doesn't match tree_def leaves {tree_def.num_leaves}"
            )
        self._refs = tuple(_refs)
        self.tree_def = tree_def
        self.op = op
        self.op_args = tuple(op_args)
        self.op_kwargs = op_kwargs
        self._op_hash = _op_hash

    def get_alive_outputs(self) -> list[TensorImpl | None]:
        return list(self._refs)

    @property
    def num_outputs(self) -> int:
        return len(self._refs)

    def __repr__(self) -> str:
        return f"OpNode(op={getattr(self.op, 'name', self.op)}, outputs={self.num_outputs})"


def _arg_impls(node: OpNode) -> list[TensorImpl]:
    out = []
    for a in node.op_args:
        if isinstance(a, TensorImpl):
            out.append(a)
        elif isinstance(a, Tensor):
            out.append(a._impl)
    return out


class Trace:
    """A captured computation subgraph: inputs, outputs, topologically sorted nodes."""

    def __init__(self, inputs: Any, outputs: Any) -> None:
        self.inputs = inputs
        self.outputs = outputs
        self._computed = False
        self.nodes: list[OpNode] = []
        self.gradient_leaves: list[TensorImpl] = []
        self._input_tensor_ids = {
            id(t._impl) for t in tree_leaves(inputs) if isinstance(t, Tensor)
        }

    def _compute_topology(self, stop_at_inputs: bool, collect_grad: bool) -> None:
        if self._computed:
            return
        visited: set[int] = set()
        nodes: list[OpNode] = []
        grad_leaves: list[TensorImpl] = []
        grad_seen: set[int] = set()

        def note_grad(impl: TensorImpl) -> None:
            if collect_grad and impl.requires_grad and id(impl) not in grad_seen:
                grad_seen.add(id(impl))
                grad_leaves.append(impl)

        roots = []
        for t in tree_leaves(self.outputs):
            if isinstance(t, Tensor):
                note_grad(t._impl)
                if t._impl.output_refs is not None:
                    roots.append(t._impl.output_refs)

        # iterative post-order DFS (graphs of several thousand nodes are normal)
        for root in roots:
            if id(root) in visited:
                continue
            stack: list[tuple[OpNode, int]] = [(root, 0)]
            on_stack = {id(root)}
            while stack:
                node, i = stack[-1]
                args = _arg_impls(node)
                advanced = False
                while i < len(args):
                    arg = args[i]
                    i += 1
                    note_grad(arg)
                    if stop_at_inputs and id(arg) in self._input_tensor_ids:
                        continue
                    child = arg.output_refs
                    if child is not None and id(child) not in visited and id(child) not in on_stack:
                        stack[-1] = (node, i)
                        stack.append((child, 0))
                        on_stack.add(id(child))
                        advanced = True
                        break
                if not advanced:
                    stack.pop()
                    on_stack.discard(id(node))
                    visited.add(id(node))
                    nodes.append(node)

        self.nodes = nodes
        if collect_grad:
            self.gradient_leaves = grad_leaves
        self._computed = True

    def compute(self) -> None:
        self._compute_topology(stop_at_inputs=True, collect_grad=False)

    def compute_for_backward(self) -> None:
        """Walk back to true leaves and collect ``requires_grad`` impls (tracing.py:179-187)."""
        self._compute_topology(stop_at_inputs=False, collect_grad=True)

    def __str__(self) -> str:
        if not self._computed:
            self.compute()
        lines = [f"Trace({len(self.nodes)} nodes)"]
        names: dict[int, str] = {}

        def nm(impl: TensorImpl) -> str:
            if id(impl) not in names:
                names[id(impl)] = f"%{len(names)}"
            return names[id(impl)]

        for n in self.nodes:
            ins = ", ".join(nm(a) for a in _arg_impls(n))
            outs = ", ".join(f"{nm(o)}:{o.dtype.name}{list(o.shape)}" for o in n._refs)
            kw = f" {n.op_kwargs}" if n.op_kwargs else ""
            lines.append(f"  {outs} = {n.op.name}({ins}){kw}")
        return "\n".join(lines)


def trace(fn: Callable[..., Any], *args: Any, **kwargs: Any) -> Trace:
    """Run ``fn`` with its tensor arguments marked traced and capture the graph."""
    inputs = [t for t in tree_leaves(args) + tree_leaves(kwargs) if isinstance(t, Tensor)]
    if not inputs:
        raise ValueError("trace: No input tensors found. Pass at least one Tensor.")
    saved = [(t, t.is_traced) for t in inputs]
    for t in inputs:
        t.is_traced = True
    try:
        outputs = fn(*args, **kwargs)
        tr = Trace(args, outputs)
        tr.compute()
        return tr
    finally:
        for t, flag in saved:
            t.is_traced = flag
