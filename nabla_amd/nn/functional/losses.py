"""Losses (nabla/nn/functional/losses.py:15-77).  ``cross_entropy_loss`` divides
by ``logits.shape[0]`` only, as the reference does (43-44)."""
from __future__ import annotations

from ...core.tensor import Tensor
from ...ops.reduction import mean, reduce_sum
from ...ops.unary import logsoftmax


def mse_loss(predictions: Tensor, targets: Tensor) -> Tensor:
    diff = predictions - targets
    return mean(diff * diff)


def cross_entropy_loss(logits: Tensor, targets: Tensor, axis: int = -1) -> Tensor:
    log_probs = logsoftmax(logits, axis=axis)
    if len(targets.shape) < len(logits.shape):
        targets = _one_hot(targets, num_classes=int(logits.shape[axis]), dtype=logits.dtype)
    batch = int(logits.shape[0])
    return -reduce_sum(targets * log_probs) / float(batch)


def _one_hot(indices: Tensor, num_classes: int, dtype=None) -> Tensor:
    from ...ops.comparison import equal
    from ...ops.creation import arange
    from ...ops.unary import cast
    from ...ops.view import unsqueeze

    classes = arange(0, num_classes, dtype=indices.dtype)
    mask = equal(unsqueeze(indices, -1), classes)
    if dtype is not None:
        mask = cast(mask, dtype)
    return mask
