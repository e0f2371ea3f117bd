"""Softmax cross-entropy against integer class labels as one operation.

The reference computes ``-sum(one_hot(labels) * logsoftmax(logits)) / logits.shape[0]``
(nabla/nn/functional/losses.py:20-77): a one-hot tensor the size of the logits, a stored
log-softmax of the same size, and in the backward pass the VJP of logsoftmax over both.  The
same numbers come out of two row programs that never hold anything the size of the logits
but the logits themselves and their gradient:

    forward, per row:   lse = max + log(sum(exp(x - max)));  nll = lse - x[label]
    backward, per row:  dx  = (exp(x - lse) - [column == label]) * g_row

The label picks its logit by comparing a column index with the (broadcast) label inside the
kernel.  The op returns the per-row negative log-likelihood (fp32) and ``lse``; summing the
rows and dividing by ``logits.shape[0]`` stays with ordinary ops in the caller.
"""
from __future__ import annotations

from ..backend import ir
from ..core.dtype import DType
from ..core.tensor import Tensor
from .base import Operation

F32 = DType.float32


def _label_mask(labels: ir.Value, full_shape) -> ir.Value:
    """1.0 where the column index equals the row's label, else 0.0 (never stored)."""
    # (an integer column index against the integer label: an exact comparison in int32 registers)
    classes = ir.iota(full_shape[-1], labels.dtype, lead=full_shape[:-1])
    lab = ir.broadcast_to(ir.reshape(labels, tuple(labels.shape) + (1,)), full_shape)
    return ir.cast(ir.ew("eq", lab, classes), F32)


class SoftmaxCrossEntropyOp(Operation):
    """(logits [..., V], labels [...] integer) -> (nll [..., 1] fp32, lse [..., 1] fp32)."""

    multiple_results = True

    @property
    def name(self) -> str:
        return "softmax_cross_entropy"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        rows = tuple(x.shape[:-1]) + (1,)
        return [rows, rows], [F32, F32], [x.device] * 2

    def kernel(self, args, kwargs):
        x, labels = args
        xf = ir.cast(x, F32)
        last = x.rank - 1
        top = ir.reduce("max", xf, last)
        picked = ir.reduce("sum", ir.ew("mul", xf, _label_mask(labels, x.shape)), last)
        total = ir.reduce("sum", ir.ew("exp", ir.ew("sub", xf, ir.broadcast_to(top, x.shape))), last)
        lse = ir.ew("add", top, ir.ew("log", total))
        return [ir.ew("sub", lse, picked), lse]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        logits, labels = primals
        return [_xent_grad_op([logits, labels, outputs[1], cotangents[0]], {})[0], None]


class SoftmaxCrossEntropyGradOp(Operation):
    """(logits, labels, lse, g [..., 1]) -> d logits."""

    @property
    def name(self) -> str:
        return "softmax_cross_entropy_grad"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(x.shape)], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        x, labels, lse, g = args
        full = x.shape
        xf = ir.cast(ir.pin_after(x, g), F32)  # (all of this belongs to the backward kernel)
        prob = ir.ew("exp", ir.ew("sub", xf, ir.broadcast_to(lse, full)))
        diff = ir.ew("sub", prob, _label_mask(labels, full))
        return [ir.cast(ir.ew("mul", diff, ir.broadcast_to(ir.cast(g, F32), full)), x.dtype)]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # second order through ordinary ops: d logits = (softmax(x) - onehot) * g
        from ..transforms.vjp import vjp
        logits, labels, _, g = primals

        def same_with_primitives(x, g):
            from .unary import softmax
            return (softmax(x, axis=-1) - one_hot(labels, int(x.shape[-1]), x.dtype)) * g

        _, pull = vjp(same_with_primitives, logits, g)
        dx, dg = pull(cotangents[0])
        return [dx, None, None, dg]


_xent_op = SoftmaxCrossEntropyOp()
_xent_grad_op = SoftmaxCrossEntropyGradOp()


def one_hot(labels: Tensor, num_classes: int, dtype: DType | None = None) -> Tensor:
    """``labels[..., None] == arange(num_classes)``, cast to ``dtype`` when one is given."""
    from .comparison import equal
    from .creation import arange
    from .unary import cast
    from .view import unsqueeze
    hits = equal(unsqueeze(labels, -1), arange(0, num_classes, dtype=labels.dtype))
    return hits if dtype is None else cast(hits, dtype)


def softmax_cross_entropy_rows(logits: Tensor, labels: Tensor) -> Tensor:
    """Per-row negative log-likelihood ``[..., 1]`` (fp32) of integer ``labels`` under
    ``softmax(logits, axis=-1)``."""
    if tuple(labels.shape) != tuple(logits.shape[:-1]):
        raise ValueError(f"labels of shape {tuple(labels.shape)} do not index the rows of logits "
                         f"{tuple(logits.shape)}")
    return _xent_op([logits, labels], {})[0]
