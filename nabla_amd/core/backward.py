"""Reverse-mode autodiff by trace replay.

Mirrors nabla/core/autograd/backward.py: ``_reduce_to_shape`` (31-54),
``_accumulate_cotangent`` (57-126), ``BackwardEngine`` (129-353),
``backward_on_trace`` (356-377) and the PyTorch-style ``backward`` (380-460).
Every VJP rule emits ordinary ops, so forward and backward end up in ONE lazy
graph that a later ``realize_all`` lowers as a whole.
"""
from __future__ import annotations

from typing import Any

from .pytree import tree_leaves
from .tensor import BatchedTensor, Tensor, TensorImpl
from .tracing import OpNode, Trace


def _reduce_to_shape(cot: Tensor, target_shape: tuple[int, ...]) -> Tensor:
    """Undo broadcasting: sum the cotangent down to the primal's shape."""
    from ..ops.reduction import reduce_sum

    cot_shape = tuple(cot.shape)
    if len(cot_shape) > len(target_shape):
        diff = len(cot_shape) - len(target_shape)
        cot = reduce_sum(cot, axis=list(range(diff)))
        cot_shape = tuple(cot.shape)
    axes = [i for i, (c, a) in enumerate(zip(cot_shape, target_shape)) if a == 1 and c > 1]
    if axes:
        cot = reduce_sum(cot, axis=axes, keepdims=True)
    return cot


def _accumulate_cotangent(cot_map: dict, target: TensorImpl, cot: Tensor) -> None:
    from ..ops.binary import add

    existing = cot_map.get(target)
    cot_map[target] = add(existing, cot) if existing is not None else cot


class BackwardEngine:
    """Backpropagation over a captured ``Trace``."""

    def __init__(self, trace: Trace, cotangents: Any, create_graph: bool = False):
        self.trace = trace
        self.create_graph = create_graph
        # value (by its impl) -> cotangent.  The cotangents are kept as the tensors they are: one
        # that comes from inside ``vmap`` (a whole basis of directions pulled back over a trace
        # made outside it) keeps its hidden dimensions through every VJP rule
        self.cotangent_map: dict[TensorImpl, Tensor] = {}
        outs = [t for t in tree_leaves(trace.outputs) if isinstance(t, Tensor)]
        cots = [c for c in tree_leaves(cotangents) if isinstance(c, Tensor)]
        if len(outs) != len(cots):
            raise ValueError(f"backward: {len(outs)} outputs but {len(cots)} cotangents")
        for o, c in zip(outs, cots):
            if tuple(o._impl.shape) == tuple(c._impl.shape):
                # the same storage shape (inside vmap: both with their hidden dimensions, and the
                # replay below runs on the stored tensors as they are)
                c = Tensor(impl=c._impl)
            elif isinstance(o, BatchedTensor) or tuple(o.shape) != tuple(c.shape):
                raise ValueError(f"cotangent shape {c.shape} does not match output shape {o.shape}")
            _accumulate_cotangent(self.cotangent_map, o._impl, c)

    def run(self) -> dict:
        for node in reversed(self.trace.nodes):
            self._process_node(node)
        return self._finalize()

    def _process_node(self, node: OpNode) -> None:
        op = node.op
        outs = node.get_alive_outputs()
        if not any(o is not None and o in self.cotangent_map for o in outs):
            return
        primals = [Tensor(impl=a) if isinstance(a, TensorImpl) else a for a in node.op_args]
        outputs = [Tensor(impl=o) if o is not None else None for o in outs]
        cots = []
        for o in outs:
            if o is None:
                cots.append(None)
            elif o in self.cotangent_map:
                cots.append(self.cotangent_map[o])
            else:
                from ..ops.creation import zeros_like
                cots.append(zeros_like(Tensor(impl=o)))
        # ops emitted by a VJP rule are part of the differentiable graph only
        # when a higher-order derivative is asked for
        flags = []
        if not self.create_graph:
            for t in primals + outputs + cots:
                if isinstance(t, Tensor):
                    flags.append((t._impl, t._impl.is_traced))
                    t._impl.is_traced = False
        try:
            in_cots = op.vjp_rule(primals, cots, outputs, node.op_kwargs or {})
        except Exception as e:
            raise RuntimeError(
                f"VJP rule failed for operation '{getattr(op, 'name', op)}': {e}"
            ) from e
        finally:
            for impl, f in flags:
                impl.is_traced = f
        for arg, c in zip(node.op_args, in_cots):
            if c is None or not isinstance(arg, TensorImpl):
                continue
            if not arg.dtype.is_float():
                continue
            c = _reduce_to_shape(c, arg.shape)
            _accumulate_cotangent(self.cotangent_map, arg, c)

    def _finalize(self) -> dict:
        from ..ops.creation import zeros_like
        grads: dict[Tensor, Tensor] = {}
        for inp in tree_leaves(self.trace.inputs):
            if not isinstance(inp, Tensor):
                continue
            c = self.cotangent_map.get(inp._impl)
            g = c if c is not None else zeros_like(Tensor(impl=inp._impl))
            # the gradient of a tensor seen from inside vmap hides the same dimensions
            if isinstance(inp, BatchedTensor) and not isinstance(g, BatchedTensor):
                g = BatchedTensor(g, inp._bd)
            grads[inp] = g
        return grads


def backward_on_trace(trace: Trace, cotangents: Any, *, create_graph: bool = False,
                      checkpoint_policy: str = "none") -> dict:
    """Pure-function backpropagation on a Trace; returns {input tensor: gradient}."""
    if not trace._computed:
        trace.compute()
    return BackwardEngine(trace, cotangents, create_graph=create_graph).run()


def backward(output: Tensor, gradient: Tensor | None = None, *, retain_graph: bool = False,
             create_graph: bool = False) -> None:
    """PyTorch-style: accumulate into ``.grad`` of every ``requires_grad`` leaf and
    realize all gradients as one batch (backward.py:380-460)."""
    from ..ops.binary import add
    from ..ops.creation import ones_like
    from .tensor import realize_all

    if gradient is None:
        if output.numel() != 1:
            raise RuntimeError("backward() without a gradient needs a scalar output")
        gradient = ones_like(output)
    tr = Trace((), output)
    tr.compute_for_backward()
    eng = BackwardEngine(tr, gradient, create_graph=create_graph)
    for node in reversed(tr.nodes):
        eng._process_node(node)
    new_grads = []
    for leaf in tr.gradient_leaves:
        g = eng.cotangent_map.get(leaf)
        if g is None:
            continue
        if leaf.cotangent is not None:
            g = add(Tensor(impl=leaf.cotangent), g)
        leaf.cotangent = g._impl
        new_grads.append(g)
    if new_grads:
        realize_all(*new_grads)
        for g in new_grads:
            g._impl.is_traced = False
            g._impl.output_refs = None
