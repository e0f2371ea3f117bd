"""Loss functions with the reference's signatures and values
(nabla/nn/functional/losses.py:15-77).

``cross_entropy_loss`` keeps the reference's normalisation -- the summed negative
log-likelihood is divided by ``logits.shape[0]`` alone, whatever the rank of the logits
(43-44) -- and its two target conventions: integer class ids (one rank below the logits) or a
dense distribution of the logits' shape.  Class ids along the last axis take the fused op of
``nabla_amd.ops.xent`` (no one-hot tensor, no stored log-softmax); everything else is spelled
with ordinary ops.
"""
from __future__ import annotations

from ...core.tensor import Tensor
from ...ops import xent as _xent
from ...ops.reduction import mean, reduce_sum
from ...ops.unary import cast, logsoftmax


def mse_loss(predictions: Tensor, targets: Tensor) -> Tensor:
    err = predictions - targets
    return mean(err * err)


def cross_entropy_loss(logits: Tensor, targets: Tensor, axis: int = -1) -> Tensor:
    rank = len(logits.shape)
    per_first_dim = 1.0 / float(int(logits.shape[0]))
    sparse = len(targets.shape) == rank - 1
    if sparse and axis % rank == rank - 1 and logits.dtype.is_float() and not targets.dtype.is_float():
        nll = _xent.softmax_cross_entropy_rows(logits, targets)
        return cast(reduce_sum(nll) * per_first_dim, logits.dtype)
    if len(targets.shape) < rank:
        targets = _one_hot(targets, num_classes=int(logits.shape[axis]), dtype=logits.dtype)
    return reduce_sum(targets * logsoftmax(logits, axis=axis)) * (-per_first_dim)


def _one_hot(indices: Tensor, num_classes: int, dtype=None) -> Tensor:
    return _xent.one_hot(indices, num_classes, dtype)
