"""Context-scoped flags (mirrors nabla/config.py:26-109).

``EAGER_MAX_GRAPH`` keeps its reference name: when set, every op call is
lowered immediately into the graph under construction instead of being
deferred; ``compile`` sets it while it traces.  ``VERIFY_EAGER_SHAPES`` checks
the lowering's shapes against ``compute_physical_shape``.
"""
from __future__ import annotations

import contextlib
import os
from contextvars import ContextVar


def _env_flag(name: str, default: bool = False) -> bool:
    return os.environ.get(name, "1" if default else "0") in {"1", "true", "TRUE", "True"}


_EAGER_MAX_GRAPH: ContextVar[bool] = ContextVar("EAGER_MAX_GRAPH", default=_env_flag("EAGER_MAX_GRAPH"))
_VERIFY_EAGER_SHAPES: ContextVar[bool] = ContextVar(
    "VERIFY_EAGER_SHAPES", default=_env_flag("VERIFY_EAGER_SHAPES")
)
_TRACING: ContextVar[bool] = ContextVar("TRACING", default=False)
# scaled_dot_product_attention as one fused op where its kernels apply (bf16, head size 64 or
# 128, no explicit mask or dropout); off: always the reference's composition of primitive ops
_FUSED_ATTENTION: ContextVar[bool] = ContextVar("FUSED_ATTENTION",
                                                default=_env_flag("NBK_FUSED_ATTENTION", True))

# lora_linear as x@W + ((x@A)@B)*s instead of the reference's x@W + x@((A@B)*s): the same
# function without the full-size delta and its two extra full GEMMs (three with the backward)
_LORA_LOW_RANK_ORDER: ContextVar[bool] = ContextVar("LORA_LOW_RANK_ORDER",
                                                    default=_env_flag("NBK_LORA_LOW_RANK_ORDER", True))

# gelu(x @ W + b) and its derivative as results of the product's own launch (computed from the
# fp32 accumulator; the pre-activation is never stored); off: a row program after the product.
# Off by default: the two transcendentals per element are vector-ALU work that a row program
# overlaps with its own memory traffic, while in the product's epilogue nothing runs beside
# them (measured on the transformer block: 1.40 ms against 1.36 ms per step with it on)
_FOLD_ACTIVATION: ContextVar[bool] = ContextVar("FOLD_ACTIVATION",
                                                default=_env_flag("NBK_FOLD_ACTIVATION", False))

# (x @ W) * c with c a constant of the graph as one product with alpha = c (how the low-rank
# adapters carry alpha / rank: no multiply kernel of its own in either direction)
_FOLD_SCALE: ContextVar[bool] = ContextVar("FOLD_SCALE", default=_env_flag("NBK_FOLD_SCALE", True))

# r + (x @ W) * alpha as one product whose epilogue reads r.  Off: measured on the LoRA decoder
# step, the epilogue's read of a full-size r (it starts when a tile's matrix work is over and
# nothing overlaps it) costs 33-41 us per 8192 x 2048 result where the separate sum kernel
# takes 17 us (29.5 -> 44.9 ms per decoder step with the fold on)
_FOLD_RESIDUAL: ContextVar[bool] = ContextVar("FOLD_RESIDUAL",
                                              default=_env_flag("NBK_FOLD_RESIDUAL", False))

# the same fold for products with a contraction of at most 16 only (a low-rank adapter's update
# on top of its base product): on: their kernel reads r for less than the sum kernel costs
_FOLD_THIN_RESIDUAL: ContextVar[bool] = ContextVar(
    "FOLD_THIN_RESIDUAL", default=_env_flag("NBK_FOLD_THIN_RESIDUAL", True))

# x @ W + u @ V with u @ V at most one K tile deep (a low-rank adapter's update folded onto its
# base product by the fold above) as ONE product with two operand pairs: the base result makes
# no trip through memory; off: the thin product reads the base result as its residual
_FOLD_THIN_PAIR: ContextVar[bool] = ContextVar(
    "FOLD_THIN_PAIR", default=_env_flag("NBK_FOLD_THIN_PAIR", True))

# relu(conv2d(x, w) + b) and relu(x @ W + b) as the epilogue of the convolution / product itself
# (`nbk_conv_desc.act`, `nbk_gemm_desc.act`); the relu's mask in the backward pass reads the
# result instead of the pre-activation; off: a row program after the producer
_FOLD_RELU: ContextVar[bool] = ContextVar("FOLD_RELU", default=_env_flag("NBK_FOLD_RELU", True))

# x1 @ W1 + x2 @ W2 (+ x3 @ W3), products that contribute to one value (the gradient of an
# activation that feeds several projections), as ONE product over all their contraction indices
# (`nbk_gemm_desc.term`); off: one product each and the kernel that adds them
_FOLD_PRODUCT_SUMS: ContextVar[bool] = ContextVar(
    "FOLD_PRODUCT_SUMS", default=_env_flag("NBK_FOLD_PRODUCT_SUMS", True))

# x^T dy1, x^T dy2, x^T dy3 (the weight gradients of projections that share their input), each
# split along K, as ONE batched launch that reads x once per cache; off: one launch each
_GROUP_SIBLING_PRODUCTS: ContextVar[bool] = ContextVar(
    "GROUP_SIBLING_PRODUCTS", default=_env_flag("NBK_GROUP_SIBLING_PRODUCTS", True))

# the column sums of dy (a bias gradient) as one more result of the weight-gradient product
# x^T dy that reads dy anyway; off: the reduction kernels read dy a second time
_FOLD_COLUMN_SUMS: ContextVar[bool] = ContextVar(
    "FOLD_COLUMN_SUMS", default=_env_flag("NBK_FOLD_COLUMN_SUMS", True))

# vmap runs the mapped function once on tensors with a hidden leading axis where every op it
# uses has a batching rule; off (or an op without a rule): one trace per element, stacked
_VMAP_BATCHED: ContextVar[bool] = ContextVar("VMAP_BATCHED", default=_env_flag("NBK_VMAP_BATCHED", True))

# the backward pass of the exact GELU computes GELU'(x) from the kept pre-activation, in the
# kernel that multiplies it with the cotangent; off: the forward kernel stores GELU'(x) as a
# second full-size result and the backward kernel reads it
_GELU_BACKWARD_FROM_INPUT: ContextVar[bool] = ContextVar(
    "GELU_BACKWARD_FROM_INPUT", default=_env_flag("NBK_GELU_BACKWARD_FROM_INPUT", True))

# x @ W for an NF4-coded W as one product that reads the codes (one byte per weight) and
# dequantises them on the way into LDS; off: dequantise into a dense weight first
_FUSED_NF4_MATMUL: ContextVar[bool] = ContextVar("FUSED_NF4_MATMUL",
                                                 default=_env_flag("NBK_FUSED_NF4_MATMUL", True))

# optimizer steps over pytrees as one launch per dtype (ops.optim); off: a group of tensor ops
# per leaf, as the reference writes them
_MULTI_TENSOR_OPTIMIZER: ContextVar[bool] = ContextVar(
    "MULTI_TENSOR_OPTIMIZER", default=_env_flag("NBK_MULTI_TENSOR_OPTIMIZER", True))

_FLAGS = {
    "EAGER_MAX_GRAPH": _EAGER_MAX_GRAPH,
    "VERIFY_EAGER_SHAPES": _VERIFY_EAGER_SHAPES,
    "TRACING": _TRACING,
    "FUSED_ATTENTION": _FUSED_ATTENTION,
    "LORA_LOW_RANK_ORDER": _LORA_LOW_RANK_ORDER,
    "FOLD_ACTIVATION": _FOLD_ACTIVATION,
    "FOLD_RESIDUAL": _FOLD_RESIDUAL,
    "FOLD_THIN_RESIDUAL": _FOLD_THIN_RESIDUAL,
    "FOLD_THIN_PAIR": _FOLD_THIN_PAIR,
    "FOLD_PRODUCT_SUMS": _FOLD_PRODUCT_SUMS,
    "FOLD_RELU": _FOLD_RELU,
    "FOLD_SCALE": _FOLD_SCALE,
    "FOLD_COLUMN_SUMS": _FOLD_COLUMN_SUMS,
    "GROUP_SIBLING_PRODUCTS": _GROUP_SIBLING_PRODUCTS,
    "VMAP_BATCHED": _VMAP_BATCHED,
    "GELU_BACKWARD_FROM_INPUT": _GELU_BACKWARD_FROM_INPUT,
    "FUSED_NF4_MATMUL": _FUSED_NF4_MATMUL,
    "MULTI_TENSOR_OPTIMIZER": _MULTI_TENSOR_OPTIMIZER,
}


def __getattr__(name: str):
    var = _FLAGS.get(name)
    if var is None:
        raise AttributeError(name)
    return var.get()


def set_flag(name: str, value: bool):
    return _FLAGS[name].set(bool(value))


def reset_flag(name: str, token) -> None:
    _FLAGS[name].reset(token)


@contextlib.contextmanager
def flag(name: str, value: bool):
    tok = set_flag(name, value)
    try:
        yield
    finally:
        reset_flag(name, tok)


def eager_mode(value: bool = True):
    return flag("EAGER_MAX_GRAPH", value)


def verify_eager_shapes(value: bool = True):
    return flag("VERIFY_EAGER_SHAPES", value)
