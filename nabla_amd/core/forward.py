"""Forward-mode differentiation on a captured trace.

Mirrors nabla/core/autograd/forward.py: the trace of the function is walked in topological
order and every node pushes the tangents of its inputs to its outputs through the op's
``jvp_rule``.  Tangents are ordinary lazy tensors built from ordinary ops, so a JVP is
lowered, fused and cached like any other graph, and with ``create_graph=True`` it can be
differentiated again in either mode.

An op without a ``jvp_rule`` of its own falls back on its ``vjp_rule``: the input
cotangents J^T u are linear in the output cotangent u, so differentiating
``sum_i <(J^T u)_i, tangent_i>`` with respect to u gives J v.  That covers convolution,
pooling, gather, pad, concatenate and the fused attention op with the rules they already have.
"""
from __future__ import annotations

from typing import Any

from .pytree import tree_leaves
from .tensor import Tensor, TensorImpl
from .tracing import Trace


def _jvp_through_vjp(op, primals, tangents, outputs, kwargs) -> list:
    from ..ops.binary import add, mul
    from ..ops.creation import zeros_like
    from ..ops.reduction import reduce_sum
    from ..ops.unary import cast
    from .dtype import DType
    from .backward import backward_on_trace
    from .tracing import trace

    live = [i for i, t in enumerate(tangents) if t is not None]
    seeds = [zeros_like(o) for o in outputs]

    def paired(*us):
        ins = op.vjp_rule(primals, list(us), outputs, kwargs)
        total = None
        for i in live:
            if i >= len(ins) or ins[i] is None:
                continue
            term = reduce_sum(cast(mul(ins[i], tangents[i]), DType.float32))
            total = term if total is None else add(total, term)
        if total is None:
            raise NotImplementedError(f"'{op.name}' gives no cotangent for its differentiated inputs")
        return total

    t = trace(paired, *seeds)
    from ..ops.creation import ones_like
    grads = backward_on_trace(t, ones_like(t.outputs), create_graph=True)
    return [grads.get(s) if grads.get(s) is not None else zeros_like(s) for s in seeds]


def forward_on_trace(trace: Trace, tangents: Any, *, create_graph: bool = True) -> dict:
    """Push ``tangents`` (aligned with the trace's inputs) through the trace; returns
    {output TensorImpl: tangent TensorImpl} for every value a tangent reached."""
    from ..ops.base import Operation

    if not trace._computed:
        trace.compute()
    ins = [t for t in tree_leaves(trace.inputs) if isinstance(t, Tensor)]
    tans = tree_leaves(tangents)
    if len(ins) != len(tans):
        raise ValueError(f"jvp: {len(ins)} input tensors but {len(tans)} tangents")
    tmap: dict[TensorImpl, TensorImpl] = {}
    for x, t in zip(ins, tans):
        if t is None:
            continue
        if not isinstance(t, Tensor):
            raise TypeError(f"jvp: tangent of type {type(t)} for a tensor input")
        if tuple(t.shape) != tuple(x.shape):
            raise ValueError(f"tangent shape {tuple(t.shape)} does not match input shape {tuple(x.shape)}")
        if x.dtype.is_float():
            tmap[x._impl] = t._impl

    for node in trace.nodes:
        args = node.op_args
        if not any(isinstance(a, TensorImpl) and a in tmap for a in args):
            continue
        op = node.op
        primals = [Tensor(impl=a) if isinstance(a, TensorImpl) else a for a in args]
        tans_in = [Tensor(impl=tmap[a]) if isinstance(a, TensorImpl) and a in tmap else None for a in args]
        outs = [Tensor(impl=o) for o in node.get_alive_outputs()]
        kwargs = node.op_kwargs or {}
        flags = []
        if not create_graph:
            for t in primals + outs + tans_in:
                if isinstance(t, Tensor):
                    flags.append((t._impl, t._impl.is_traced))
                    t._impl.is_traced = False
        try:
            if type(op).jvp_rule is not Operation.jvp_rule:
                # rules written for dense tangents: an input the tangent did not reach is zero
                from ..ops.creation import zeros_like
                dense = [t if t is not None or not isinstance(p, Tensor) else zeros_like(p)
                         for p, t in zip(primals, tans_in)]
                out_tans = op.jvp_rule(primals, dense, outs, kwargs)
            else:
                out_tans = _jvp_through_vjp(op, primals, tans_in, outs, kwargs)
        except Exception as e:
            raise RuntimeError(f"JVP rule failed for operation '{getattr(op, 'name', op)}': {e}") from e
        finally:
            for impl, f in flags:
                impl.is_traced = f
        for o, t in zip(outs, out_tans):
            if t is not None and o.dtype.is_float():
                tmap[o._impl] = t._impl
    return tmap
