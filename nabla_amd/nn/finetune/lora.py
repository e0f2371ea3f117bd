"""LoRA adapters (nabla/nn/finetune/lora.py:16-127): an adapter is the plain dict
``{"A": (in, rank), "B": (rank, out)}`` and stands for the update ``(alpha / rank) * A @ B`` of a
frozen ``(in, out)`` weight.

``lora_linear`` is where this backend departs from the reference's arithmetic order.  The
reference forms the full ``(in, out)`` update and multiplies the activations with it, a second
full-size product forward and two more backward (``x^T dy`` and ``dy delta^T``).  With
``config.LORA_LOW_RANK_ORDER`` (the default) the activations go through the two thin factors
instead, ``((x @ A) @ B) * (alpha / rank)``: every adapter product is rank-sized in both
directions, and the result differs from the reference's by rounding only.  Switch the flag off
for the order as written there.
"""
from __future__ import annotations

from ... import config
from ...core.dtype import DType
from ...core.pytree import tree_map
from ...core.tensor import Tensor
from ...ops.creation import full, zeros
from ..functional.init import normal


def _factors(adapter: dict[str, Tensor]) -> tuple[Tensor, Tensor, float]:
    """(A, B, 1 / rank) of an adapter dict."""
    down, up = adapter["A"], adapter["B"]
    return down, up, 1.0 / float(int(down.shape[1]))


def init_lora_adapter(weight: Tensor, rank: int, init_std: float = 0.01,
                      dtype: DType | None = None) -> dict[str, Tensor]:
    """Fresh adapter for a 2-D ``weight``: Gaussian ``A``, zero ``B``, so that it starts as a no-op."""
    if len(weight.shape) != 2:
        raise ValueError("init_lora_adapter expects a 2D weight tensor")
    if rank <= 0:
        raise ValueError("rank must be > 0")
    fan_in, fan_out = (int(d) for d in weight.shape)
    kind = weight.dtype if dtype is None else dtype
    return {"A": normal((fan_in, rank), 0.0, init_std, dtype=kind),
            "B": zeros((rank, fan_out), dtype=kind, device=weight.device)}


def _scale_constant(value: float, like: Tensor) -> Tensor:
    """The scale as a constant of the graph (a lazy ``full``), not as a realized scalar: the
    planner can then read its value and fold it into the neighbouring product."""
    return full((), float(value), dtype=like.dtype, device=like.device)


def lora_delta(adapter: dict[str, Tensor], alpha: float = 1.0) -> Tensor:
    """The full-size update ``(alpha / rank) * A @ B``."""
    down, up, inv_rank = _factors(adapter)
    return (down @ up) * (alpha * inv_rank)


def lora_linear(x: Tensor, frozen_weight: Tensor, adapter: dict[str, Tensor],
                alpha: float = 1.0) -> Tensor:
    """``x @ (frozen_weight + delta)`` without ever adding the two weights."""
    base = x @ frozen_weight
    if not config.LORA_LOW_RANK_ORDER:
        return base + x @ lora_delta(adapter, alpha=alpha)
    down, up, inv_rank = _factors(adapter)
    # (the scale goes on the [tokens, rank] product, where the planner folds it into that
    # product's alpha, and the same happens to its two mirror images in the backward pass: no
    # kernel of its own anywhere)
    return base + ((x @ down) * _scale_constant(alpha * inv_rank, x)) @ up


def merge_lora_weight(frozen_weight: Tensor, adapter: dict[str, Tensor], alpha: float = 1.0) -> Tensor:
    return frozen_weight + lora_delta(adapter, alpha=alpha)


def unmerge_lora_weight(merged_weight: Tensor, adapter: dict[str, Tensor], alpha: float = 1.0) -> Tensor:
    return merged_weight - lora_delta(adapter, alpha=alpha)


def tree_lora_delta(adapters, alpha: float = 1.0, *, is_leaf=None):
    """Every adapter dict in a pytree replaced by its full-size update; other leaves untouched."""
    is_adapter = lambda node: isinstance(node, dict) and "A" in node and "B" in node
    stop = is_adapter if is_leaf is None else (lambda node: is_adapter(node) or is_leaf(node))
    return tree_map(lambda leaf: lora_delta(leaf, alpha=alpha) if is_adapter(leaf) else leaf,
                    adapters, is_leaf=stop)
