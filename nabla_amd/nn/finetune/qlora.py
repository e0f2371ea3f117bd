"""QLoRA helpers (nabla/nn/finetune/qlora.py): ``quantize_nf4`` 41-75 (host side: blocks of
``block_size`` values scaled by their absolute maximum, nearest entry of the 16-level NF4
codebook 18-38 as a uint8 index, the flat tensor zero-padded to whole blocks),
``dequantize_nf4`` 77-98 (codebook gather, per-block scale, trim, reshape -- ordinary ops,
so it lowers to a gather plus one fused row program) and ``qlora_linear`` 101-113
(``x @ dequant(W) + x @ delta`` in ``compute_dtype``).  The adapter product follows
``config.LORA_LOW_RANK_ORDER`` like ``lora_linear``."""
from __future__ import annotations

from typing import Any

import numpy as np

from ... import config
from ...core.dtype import DType
from ...core.tensor import Tensor
from ...ops.unary import cast
from ...ops.view import gather, reshape, unsqueeze
from .lora import lora_delta

#: the sixteen NF4 levels as the reference tabulates them (four decimals)
NF4_CODEBOOK = np.array([-1.0, -0.6962, -0.5251, -0.3949, -0.2844, -0.1848, -0.0911, 0.0,
                         0.0796, 0.1609, 0.2461, 0.3379, 0.4407, 0.5626, 0.7230, 1.0],
                        dtype=np.float32)


def quantize_nf4(weight: Tensor, block_size: int = 64) -> dict[str, Any]:
    if len(weight.shape) != 2:
        raise ValueError("quantize_nf4 expects a 2D weight tensor")
    if block_size <= 0:
        raise ValueError("block_size must be > 0")
    w = weight.cast(DType.float32) if weight.dtype is not DType.float32 else weight
    flat = w.to_numpy().astype(np.float32).reshape(-1)
    numel = int(flat.size)
    pad = -numel % block_size
    if pad:
        flat = np.concatenate([flat, np.zeros(pad, np.float32)])
    blocks = flat.reshape(-1, block_size)
    scales = np.abs(blocks).max(axis=1, keepdims=True)
    scales[scales == 0] = 1.0
    normed = (blocks / scales).reshape(-1, 1)
    # nearest level; ties go to the lower index (argmin takes the first minimum)
    indices = np.abs(normed - NF4_CODEBOOK[None, :]).argmin(axis=1).astype(np.uint8)
    return {
        "indices": Tensor.from_dlpack(indices),
        "scales": Tensor.from_dlpack(scales.reshape(-1).astype(np.float32)),
        "original_shape": tuple(int(d) for d in weight.shape),
        "original_numel": numel,
        "padded_numel": int(flat.size),
        "block_size": int(block_size),
    }


def dequantize_nf4(qweight: dict[str, Any], *, dtype: DType = DType.float32) -> Tensor:
    block = int(qweight["block_size"])
    padded = int(qweight["padded_numel"])
    codebook = Tensor.from_dlpack(NF4_CODEBOOK).to(dtype)
    levels = gather(codebook, cast(qweight["indices"], DType.int32), axis=0)
    scaled = reshape(levels, (padded // block, block)) * unsqueeze(qweight["scales"].to(dtype), axis=1)
    flat = reshape(scaled, (padded,))
    return reshape(flat[:int(qweight["original_numel"])], tuple(qweight["original_shape"]))


def qlora_linear(x: Tensor, qweight: dict[str, Any], adapter: dict[str, Tensor], *,
                 alpha: float = 1.0, compute_dtype: DType = DType.float32) -> Tensor:
    w = dequantize_nf4(qweight, dtype=compute_dtype)
    xc = x.to(compute_dtype)
    if config.LORA_LOW_RANK_ORDER:
        A, B = adapter["A"].to(compute_dtype), adapter["B"].to(compute_dtype)
        return (xc @ w) + ((xc @ A) @ B) * (alpha / float(int(A.shape[1])))
    return (xc @ w) + (xc @ lora_delta(adapter, alpha=alpha).to(compute_dtype))
