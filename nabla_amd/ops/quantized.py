"""Products with NF4-coded weights.

``dequantize_nf4`` followed by ``matmul`` (nabla/nn/finetune/qlora.py:77-113) builds the dense
weight first: a gather, a row program and a tensor of the weight's full size, every step.
``matmul_nf4`` is that pair as one op whose kernel takes the codes as the B operand of the
product (one byte per weight from memory, level lookup and block scale on the way into LDS).  The
coded weight is data, not a parameter: the VJP returns the input gradient only, which is the same
kernel on the transposed weight.
"""
from __future__ import annotations

from ..backend import ir
from ..core.dtype import DType
from ..core.tensor import Tensor
from .base import Operation


class MatmulNF4Op(Operation):
    """(x [..., K], codes uint8 [rows * cols], scales fp32 [rows * cols / block]) -> x @ W."""

    @property
    def name(self) -> str:
        return "matmul_nf4"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        rows, cols = kwargs["w_shape"]
        n = rows if kwargs["transpose"] else cols
        return [tuple(x.shape[:-1]) + (n,)], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        return [ir.matmul_nf4(args[0], args[1], args[2], kwargs["w_shape"], kwargs["block"],
                              kwargs["transpose"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        _, codes, scales = primals
        flipped = dict(kwargs, transpose=not kwargs["transpose"])
        return [_matmul_nf4_op([cotangents[0], codes, scales], flipped)[0], None, None]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        _, codes, scales = primals
        return [_matmul_nf4_op([tangents[0], codes, scales], dict(kwargs))[0]]


_matmul_nf4_op = MatmulNF4Op()


def matmul_nf4(x: Tensor, codes: Tensor, scales: Tensor, w_shape, block_size: int, *,
               transpose: bool = False) -> Tensor:
    """``x @ W`` (``x @ W^T`` with ``transpose``) for ``W`` of shape ``w_shape`` given as NF4 codes and
    block scales; ``x`` in bfloat16 or float32, the result in the same type."""
    rows, cols = (int(d) for d in w_shape)
    if codes.dtype is not DType.uint8 or scales.dtype is not DType.float32:
        raise TypeError(f"matmul_nf4 expects uint8 codes and float32 scales, got {codes.dtype}, {scales.dtype}")
    if x.dtype not in (DType.bfloat16, DType.float32):
        raise TypeError(f"matmul_nf4 computes in bfloat16 or float32, got {x.dtype}")
    if cols % 8 or int(block_size) % 8 or block_size <= 0:
        raise ValueError("matmul_nf4 needs a weight width and a block length that are multiples of 8")
    return _matmul_nf4_op([x, codes, scales], {"w_shape": (rows, cols), "block": int(block_size),
                                               "transpose": bool(transpose)})[0]
