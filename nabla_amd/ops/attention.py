"""Fused scaled-dot-product attention.

The reference builds attention from primitive ops -- matmul, mul by the scale, a
``where`` against a ``tril`` mask, softmax, matmul (nabla/nn/functional/layers.py:106-153)
-- and differentiates it through the VJP rules of those ops, which stores the S x S
scores and probabilities several times over.  Here the same function is one op with one
kernel forward and two backward; the probabilities are recomputed from the per-row
log-sum-exp the forward keeps.

``FusedAttentionOp`` takes heads-first tensors ``[B, H, S, hd]`` (what
``MultiHeadAttention`` passes, nabla/nn/modules/layers.py) and returns
``(output, lse, remainder)``: the third result is what rounding the output to bf16 cut off,
kept for the backward pass, whose row sums ``sum(d output * output)`` need more digits than
bf16 holds (a forward pass that nobody differentiates does not compute it).  ``fused_attention_applies`` says whether the kernels cover a call;
``scaled_dot_product_attention`` keeps the composition of primitive ops for every other
case.  Second-order derivatives go through primitive ops as well: the VJP rule of the
gradient op differentiates the matmul / softmax expression of the same gradients.
"""
from __future__ import annotations

import math

from .. import config
from ..backend import ir
from ..core.dtype import DType
from ..core.tensor import Tensor
from .base import Operation

_HEAD_SIZES = (64, 128)
_SEQ_MULTIPLE = 128


def fused_attention_applies(query: Tensor, key: Tensor, value: Tensor) -> bool:
    if not config.FUSED_ATTENTION:
        return False
    qs, ks, vs = tuple(query.shape), tuple(key.shape), tuple(value.shape)
    if len(qs) != 4 or qs != ks or qs != vs:
        return False
    if not (query.dtype is DType.bfloat16 and key.dtype is DType.bfloat16 and value.dtype is DType.bfloat16):
        return False
    b, h, s, hd = qs
    return hd in _HEAD_SIZES and s % _SEQ_MULTIPLE == 0 and s > 0 and b * h <= 65535


class FusedAttentionOp(Operation):
    multiple_results = True

    @property
    def name(self) -> str:
        return "fused_attention"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        q = args[0]
        shape = tuple(q.shape)
        return [shape, shape[:-1], shape], [q.dtype, DType.float32, q.dtype], [q.device] * 3

    def kernel(self, args, kwargs):
        return list(ir.attention(args[0], args[1], args[2], kwargs["scale"], kwargs["is_causal"]))

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        q, k, v = primals
        out, lse, out_lo = outputs
        return _fused_attention_grad_op([q, k, v, out, lse, out_lo, cotangents[0]], dict(kwargs))


class FusedAttentionGradOp(Operation):
    """(dq, dk, dv) from (q, k, v, output, lse, output's rounding remainder, d output)."""

    multiple_results = True

    @property
    def name(self) -> str:
        return "fused_attention_grad"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        q = args[0]
        shape = tuple(q.shape)
        return [shape] * 3, [q.dtype] * 3, [q.device] * 3

    def kernel(self, args, kwargs):
        return list(ir.attention_bwd(*args[:7], kwargs["scale"], kwargs["is_causal"]))

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # As a function of (q, k, v, d output) these gradients equal the ones the primitive ops
        # give (output and lse are themselves functions of q, k, v), so the second-order rule
        # differentiates that expression.
        from ..transforms.vjp import vjp
        q, k, v, _, _, _, g = primals
        scale, causal = kwargs["scale"], kwargs["is_causal"]
        _, pull = vjp(lambda q, k, v, g: tuple(_composite_vjp(q, k, v, g, scale, causal)), q, k, v, g)
        dq, dk, dv, dg = pull(tuple(cotangents))
        return [dq, dk, dv, None, None, None, dg]


def _composite_vjp(q, k, v, g, scale, causal):
    """(dq, dk, dv) out of differentiable primitive ops."""
    from .binary import matmul
    from .comparison import greater
    from .control_flow import where
    from .creation import full, ones, tril
    from .reduction import reduce_sum
    from .unary import softmax
    from .view import swap_axes

    scores = matmul(q, swap_axes(k, -2, -1)) * scale
    if causal:
        s = int(q.shape[-2])
        scores = where(greater(tril(ones((s, s), dtype=q.dtype)), 0.0), scores,
                       full((s, s), -1e9, dtype=q.dtype))
    p = softmax(scores, axis=-1)
    dv = matmul(swap_axes(p, -2, -1), g)
    dp = matmul(g, swap_axes(v, -2, -1))
    ds = p * (dp - reduce_sum(dp * p, axis=-1, keepdims=True)) * scale
    return [matmul(ds, k), matmul(swap_axes(ds, -2, -1), q), dv]


_fused_attention_op = FusedAttentionOp()
_fused_attention_grad_op = FusedAttentionGradOp()


def fused_attention(query: Tensor, key: Tensor, value: Tensor, *, is_causal: bool = False,
                    scale: float | None = None) -> Tensor:
    if not fused_attention_applies(query, key, value):
        raise ValueError(
            "fused_attention covers bfloat16 [B, H, S, hd] tensors of one shape with hd in "
            f"{_HEAD_SIZES} and S a multiple of {_SEQ_MULTIPLE}; got {tuple(query.shape)} "
            f"{query.dtype}, {tuple(key.shape)} {key.dtype}, {tuple(value.shape)} {value.dtype}")
    if scale is None:
        scale = 1.0 / math.sqrt(int(query.shape[-1]))
    return _fused_attention_op([query, key, value], {"scale": float(scale), "is_causal": bool(is_causal)})[0]
