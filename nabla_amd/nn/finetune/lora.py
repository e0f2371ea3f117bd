"""LoRA helpers (nabla/nn/finetune/lora.py): init_lora_adapter 16-52,
lora_delta 55-69 = ``(A @ B) * (alpha / rank)``, lora_linear 72-79, merge / unmerge.

The reference writes ``lora_linear`` as ``x @ W + x @ delta``: a full ``[D, D]`` delta and
a second full GEMM forward, and two more full GEMMs in the backward pass (``x^T dy`` and
``dy delta^T``).  With ``config.LORA_LOW_RANK_ORDER`` (the default) the same function is
evaluated as ``x @ W + ((x @ A) @ B) * (alpha / rank)``: every adapter product is rank-sized
in both directions.  The two orders differ by rounding only; switch the flag off for the
order as written."""
from __future__ import annotations

from ... import config
from ...core.dtype import DType
from ...core.tensor import Tensor
from ...ops.creation import zeros
from ..functional.init import normal


def init_lora_adapter(weight: Tensor, rank: int, init_std: float = 0.01,
                      dtype: DType | None = None) -> dict[str, Tensor]:
    if len(weight.shape) != 2:
        raise ValueError("init_lora_adapter expects a 2D weight tensor")
    if rank <= 0:
        raise ValueError("rank must be > 0")
    in_features, out_features = int(weight.shape[0]), int(weight.shape[1])
    adapter_dtype = dtype or weight.dtype
    A = normal((in_features, rank), 0.0, init_std, dtype=adapter_dtype)
    B = zeros((rank, out_features), dtype=adapter_dtype, device=weight.device)
    return {"A": A, "B": B}


def lora_delta(adapter: dict[str, Tensor], alpha: float = 1.0) -> Tensor:
    A, B = adapter["A"], adapter["B"]
    rank = int(A.shape[1])
    return (A @ B) * (alpha / float(rank))


def lora_linear(x: Tensor, frozen_weight: Tensor, adapter: dict[str, Tensor],
                alpha: float = 1.0) -> Tensor:
    if config.LORA_LOW_RANK_ORDER:
        A, B = adapter["A"], adapter["B"]
        return (x @ frozen_weight) + ((x @ A) @ B) * (alpha / float(int(A.shape[1])))
    return (x @ frozen_weight) + (x @ lora_delta(adapter, alpha=alpha))


def merge_lora_weight(frozen_weight: Tensor, adapter: dict[str, Tensor], alpha: float = 1.0) -> Tensor:
    return frozen_weight + lora_delta(adapter, alpha=alpha)


def unmerge_lora_weight(merged_weight: Tensor, adapter: dict[str, Tensor], alpha: float = 1.0) -> Tensor:
    return merged_weight - lora_delta(adapter, alpha=alpha)
