"""QLoRA: NF4-coded frozen weights under a LoRA adapter (nabla/nn/finetune/qlora.py).

Format, as the reference defines it (41-75): the weight is flattened row-major and cut into
blocks of ``block_size`` values (the tail zero-padded); a block is stored as its absolute
maximum (``scales``, fp32, 1 for an all-zero block) and, per value, the index of the nearest of
the sixteen NF4 levels (18-38) after division by that maximum (``indices``, one uint8 each).
``quantize_nf4`` runs on the host, ``dequantize_nf4`` (77-98) and ``qlora_linear`` (101-113) on
the device.

``qlora_linear`` does not rebuild the dense weight where it can avoid it: with a bfloat16 or
float32 compute type and a weight whose width is a multiple of 8 the codes are the B operand of
the product itself -- the GEMM reads one byte per weight, looks the level up, applies the block
scale and feeds the matrix cores (``matmul_nf4``).  Other cases dequantise first with a gather
and one row program.
"""
from __future__ import annotations

from typing import Any

import numpy as np

from ... import config
from ...core.dtype import DType
from ...core.tensor import Tensor
from ...ops.unary import cast
from .lora import _scale_constant
from ...ops.view import gather, reshape, unsqueeze

#: the sixteen NF4 levels as the reference tabulates them (four decimals)
NF4_CODEBOOK = np.array([-1.0, -0.6962, -0.5251, -0.3949, -0.2844, -0.1848, -0.0911, 0.0,
                         0.0796, 0.1609, 0.2461, 0.3379, 0.4407, 0.5626, 0.7230, 1.0],
                        dtype=np.float32)


def _nearest_level(values: np.ndarray) -> np.ndarray:
    """Index of the closest codebook entry for every value in [-1, 1]; the lower index on a tie.
    The codebook is sorted, so only the two entries around a value can be closest."""
    hi = np.clip(np.searchsorted(NF4_CODEBOOK, values, side="left"), 1, NF4_CODEBOOK.size - 1)
    lo = hi - 1
    take_hi = np.abs(values - NF4_CODEBOOK[hi]) < np.abs(values - NF4_CODEBOOK[lo])
    return np.where(take_hi, hi, lo).astype(np.uint8)


def quantize_nf4(weight: Tensor, block_size: int = 64) -> dict[str, Any]:
    if len(weight.shape) != 2:
        raise ValueError("quantize_nf4 expects a 2D weight tensor")
    if block_size <= 0:
        raise ValueError("block_size must be > 0")
    host = weight.to(DType.float32).to_numpy().astype(np.float32, copy=False).ravel()
    count = int(host.size)
    n_blocks = -(-count // block_size)
    padded = np.zeros(n_blocks * block_size, np.float32)
    padded[:count] = host
    grid = padded.reshape(n_blocks, block_size)
    absmax = np.abs(grid).max(axis=1)
    absmax[absmax == 0.0] = 1.0
    codes = _nearest_level((grid / absmax[:, None]).ravel())
    return {
        "indices": Tensor.from_dlpack(codes),
        "scales": Tensor.from_dlpack(absmax.astype(np.float32)),
        "original_shape": tuple(int(d) for d in weight.shape),
        "original_numel": count,
        "padded_numel": int(padded.size),
        "block_size": int(block_size),
    }


def dequantize_nf4(qweight: dict[str, Any], *, dtype: DType = DType.float32) -> Tensor:
    """The dense weight in ``dtype``: level of every code times the scale of its block."""
    per_block = int(qweight["block_size"])
    n_blocks = int(qweight["padded_numel"]) // per_block
    table = Tensor.from_dlpack(NF4_CODEBOOK).to(dtype)
    levels = gather(table, cast(qweight["indices"], DType.int32), axis=0)
    by_block = reshape(levels, (n_blocks, per_block)) * unsqueeze(qweight["scales"].to(dtype), axis=1)
    dense = reshape(by_block, (n_blocks * per_block,))[:int(qweight["original_numel"])]
    return reshape(dense, tuple(qweight["original_shape"]))


def _fused_base_applies(x: Tensor, qweight: dict[str, Any], compute_dtype: DType) -> bool:
    shape = tuple(qweight["original_shape"])
    return (config.FUSED_NF4_MATMUL and compute_dtype in (DType.bfloat16, DType.float32) and
            shape[1] % 8 == 0 and int(qweight["block_size"]) % 8 == 0 and
            int(qweight["padded_numel"]) == shape[0] * shape[1] and len(x.shape) >= 2)


def qlora_linear(x: Tensor, qweight: dict[str, Any], adapter: dict[str, Tensor], *,
                 alpha: float = 1.0, compute_dtype: DType = DType.float32) -> Tensor:
    """``x @ W_nf4 + x @ delta`` in ``compute_dtype``; the adapter product follows
    ``config.LORA_LOW_RANK_ORDER`` like ``lora_linear``."""
    from .lora import lora_linear
    xc = x.to(compute_dtype)
    cast_adapter = {k: v.to(compute_dtype) for k, v in adapter.items()}
    if _fused_base_applies(xc, qweight, compute_dtype):
        from ...ops.quantized import matmul_nf4
        base = matmul_nf4(xc, qweight["indices"], qweight["scales"], tuple(qweight["original_shape"]),
                          int(qweight["block_size"]))
        down, up = cast_adapter["A"], cast_adapter["B"]
        scale = alpha / float(int(down.shape[1]))
        if config.LORA_LOW_RANK_ORDER:
            return base + ((xc @ down) * _scale_constant(scale, xc)) @ up
        return base + xc @ ((down @ up) * scale)
    return lora_linear(xc, dequantize_nf4(qweight, dtype=compute_dtype), cast_adapter, alpha=alpha)
