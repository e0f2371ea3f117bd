"""Layer normalisation over the last axis as one operation.

The reference writes ``layer_norm`` as nine tensor ops -- mean, subtract, square, mean, add
eps, rsqrt, multiply, scale, shift (nabla/nn/functional/layers.py:38-56) -- and its gradient
is whatever the VJP rules of those nine produce.  Here the forward is one op whose lowering
is one row program by construction (two reductions, fp32 throughout, one rounding on the way
out) and which also returns the row statistics (mean and reciprocal standard deviation, fp32,
one value per row); the backward is one op with the closed form

    xhat = (x - mean) * rstd          gy = g * weight
    dx   = rstd * (gy - mean_row(gy) - xhat * mean_row(gy * xhat))
    dweight = sum over rows of g * xhat        dbias = sum over rows of g

(biased variance and eps inside the rsqrt, as in the reference).  Other axes, or several, go
through the same arithmetic spelled with ordinary ops.
"""
from __future__ import annotations

from ..backend import ir
from ..core.dtype import DType
from ..core.tensor import Tensor
from .base import Operation

F32 = DType.float32


def _rows(v: ir.Value, full_shape) -> ir.Value:
    """A per-row value ``[..., 1]`` seen over the whole row."""
    return ir.broadcast_to(v, full_shape)


def _row_mean(v: ir.Value) -> ir.Value:
    return ir.ew("div", ir.reduce("sum", v, v.rank - 1), float(v.shape[-1]))


class LayerNormOp(Operation):
    """(x, [weight], [bias]) -> (y, mean, rstd); which of weight / bias are present is in kwargs."""

    multiple_results = True

    @property
    def name(self) -> str:
        return "layer_norm"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        stat = tuple(x.shape[:-1]) + (1,)
        return [tuple(x.shape), stat, stat], [x.dtype, F32, F32], [x.device] * 3

    def kernel(self, args, kwargs):
        x = args[0]
        rest = list(args[1:])
        w = rest.pop(0) if kwargs["has_weight"] else None
        b = rest.pop(0) if kwargs["has_bias"] else None
        xf = ir.cast(x, F32)
        mean = _row_mean(xf)
        centred = ir.ew("sub", xf, _rows(mean, x.shape))
        var = _row_mean(ir.ew("mul", centred, centred))
        rstd = ir.ew("rsqrt", ir.ew("add", var, float(kwargs["eps"])))
        y = ir.ew("mul", centred, _rows(rstd, x.shape))
        if w is not None:
            y = ir.ew("mul", y, ir.broadcast_to(w, x.shape))
        if b is not None:
            y = ir.ew("add", y, ir.broadcast_to(b, x.shape))
        return [ir.cast(y, x.dtype), mean, rstd]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .reduction import reduce_sum
        x = primals[0]
        w = primals[1] if kwargs["has_weight"] else None
        g = cotangents[0]
        _, mean, rstd = outputs
        args = [x, g, mean, rstd] + ([w] if w is not None else [])
        dx, gxhat = _layer_norm_grad_op(args, {"has_weight": w is not None, "eps": kwargs["eps"]})
        lead = list(range(len(x.shape) - 1))
        grads = [dx]
        if w is not None:
            grads.append(reduce_sum(gxhat, axis=lead) if lead else gxhat)
        if kwargs["has_bias"]:
            grads.append(reduce_sum(g, axis=lead) if lead else g)
        return grads


class LayerNormGradOp(Operation):
    """(x, g, mean, rstd, [weight]) -> (dx, g * xhat)."""

    multiple_results = True

    @property
    def name(self) -> str:
        return "layer_norm_grad"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(x.shape)] * 2, [x.dtype] * 2, [x.device] * 2

    def kernel(self, args, kwargs):
        x, g, mean, rstd = args[:4]
        w = args[4] if kwargs["has_weight"] else None
        full = x.shape
        gf = ir.cast(g, F32)
        xf = ir.cast(ir.pin_after(x, g), F32)  # (xhat is rebuilt here, not stored by the forward kernel)
        xhat = ir.ew("mul", ir.ew("sub", xf, _rows(mean, full)), _rows(rstd, full))
        gy = gf if w is None else ir.ew("mul", gf, ir.broadcast_to(w, full))
        gxhat = ir.ew("mul", gf, xhat)
        m1 = _row_mean(gy)
        m2 = _row_mean(ir.ew("mul", gy, xhat))
        inner = ir.ew("sub", ir.ew("sub", gy, _rows(m1, full)), ir.ew("mul", xhat, _rows(m2, full)))
        dx = ir.ew("mul", inner, _rows(rstd, full))
        return [ir.cast(dx, x.dtype), ir.cast(gxhat, x.dtype)]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # second order: differentiate the same two results written with ordinary ops (mean and
        # rstd are functions of x there, as they are in fact)
        from ..transforms.vjp import vjp
        x, g = primals[0], primals[1]
        w = primals[4] if kwargs["has_weight"] else None
        eps = kwargs["eps"]
        if w is None:
            _, pull = vjp(lambda x, g: _grad_pair_from_primitives(x, g, None, eps), x, g)
            dx, dg = pull(tuple(cotangents))
            return [dx, dg, None, None]
        _, pull = vjp(lambda x, g, w: _grad_pair_from_primitives(x, g, w, eps), x, g, w)
        dx, dg, dw = pull(tuple(cotangents))
        return [dx, dg, None, None, dw]


def _normalise(x: Tensor, axes, eps: float):
    """(xhat, rstd) over ``axes`` from differentiable primitives."""
    from .reduction import mean
    from .unary import rsqrt
    centred = x - mean(x, axis=axes, keepdims=True)
    rstd = rsqrt(mean(centred * centred, axis=axes, keepdims=True) + eps)
    return centred * rstd, rstd


def _grad_pair_from_primitives(x, g, w, eps):
    from .reduction import mean
    xhat, rstd = _normalise(x, -1, eps)
    gy = g if w is None else g * w
    dx = rstd * (gy - mean(gy, axis=-1, keepdims=True) - xhat * mean(gy * xhat, axis=-1, keepdims=True))
    return dx, g * xhat


_layer_norm_op = LayerNormOp()
_layer_norm_grad_op = LayerNormGradOp()


def layer_norm(x: Tensor, weight: Tensor | None = None, bias: Tensor | None = None,
               eps: float = 1e-5, axis=-1) -> Tensor:
    """``(x - mean) * rsqrt(var + eps) * weight + bias`` with the biased variance over ``axis``."""
    rank = len(x.shape)
    last_only = isinstance(axis, int) and axis % max(rank, 1) == rank - 1 and rank >= 1
    trailing = lambda t: t is None or (len(t.shape) == 1 and int(t.shape[0]) == int(x.shape[-1])
                                       and t.dtype is x.dtype)
    if last_only and x.dtype.is_float() and trailing(weight) and trailing(bias):
        args = [x] + [t for t in (weight, bias) if t is not None]
        kwargs = {"has_weight": weight is not None, "has_bias": bias is not None, "eps": float(eps)}
        return _layer_norm_op(args, kwargs)[0]
    out, _ = _normalise(x, axis, eps)
    if weight is not None:
        out = out * weight
    return out if bias is None else out + bias
