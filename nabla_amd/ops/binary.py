"""Binary arithmetic ops and matmul.

Mirrors nabla/ops/binary.py: AddOp 18-45, MulOp 48-79, SubOp 82-111, DivOp
114-156, MatmulOp 159-324 (1-D promotion and batch broadcast 234-287; VJP
303-314), PowOp.  VJP rules are written with the same ops as the reference so
the backward graph has the same meaning.
"""
from __future__ import annotations

from ..backend import ir
from ..core.dtype import promote
from ..core.tensor import Tensor
from .base import BinaryOperation, Operation, ensure_tensor


def _ew2(fn: str):
    def kernel(self, args, kwargs):
        a, b = args
        dt = promote(a.dtype, b.dtype)
        return [ir.ew(fn, ir.cast(a, dt), ir.cast(b, dt))]
    return kernel


class AddOp(BinaryOperation):
    @property
    def name(self) -> str:
        return "add"

    kernel = _ew2("add")

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return [cotangents[0], cotangents[0]]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [add(tangents[0], tangents[1])]


class MulOp(BinaryOperation):
    @property
    def name(self) -> str:
        return "mul"

    kernel = _ew2("mul")

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        x, y = primals
        g = cotangents[0]
        return [mul(g, y), mul(g, x)]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        x, y = primals
        return [add(mul(tangents[0], y), mul(x, tangents[1]))]


class SubOp(BinaryOperation):
    @property
    def name(self) -> str:
        return "sub"

    kernel = _ew2("sub")

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .unary import neg
        return [cotangents[0], neg(cotangents[0])]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [sub(tangents[0], tangents[1])]


class DivOp(BinaryOperation):
    @property
    def name(self) -> str:
        return "div"

    kernel = _ew2("div")

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # d(x/y)/dx = 1/y ; d(x/y)/dy = -x/y^2  (binary.py:136-146)
        from .unary import neg
        x, y = primals
        g = cotangents[0]
        return [div(g, y), neg(mul(g, div(x, mul(y, y))))]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        x, y = primals
        return [div(sub(mul(y, tangents[0]), mul(x, tangents[1])), mul(y, y))]


class PowOp(BinaryOperation):
    @property
    def name(self) -> str:
        return "pow"

    kernel = _ew2("pow")

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .unary import log
        x, y = primals
        g = cotangents[0]
        out = outputs[0]
        gx = mul(g, mul(y, pow(x, sub(y, 1.0))))
        gy = mul(g, mul(out, log(x)))
        return [gx, gy]


class MatmulOp(Operation):
    """Matrix product with 1-D promotion and numpy batch broadcasting."""

    @property
    def name(self) -> str:
        return "matmul"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x, y = args
        if x.shape[-1] != y.shape[-2]:
            raise ValueError(f"matmul: shapes {x.shape} and {y.shape} do not contract")
        shape = tuple(x.shape[:-1]) + (y.shape[-1],)
        return [shape], [promote(x.dtype, y.dtype)], [x.device]

    def kernel(self, args, kwargs):
        a, b = args
        dt = promote(a.dtype, b.dtype)
        return [ir.matmul(ir.cast(a, dt), ir.cast(b, dt))]

    def __call__(self, args, kwargs):
        from . import view as view_ops

        x = ensure_tensor(args[0])
        y = ensure_tensor(args[1])
        x1d, y1d = len(x.shape) == 1, len(y.shape) == 1
        if len(x.shape) == 0 or len(y.shape) == 0:
            raise ValueError("matmul: operands must have rank >= 1")
        if x1d:
            x = view_ops.unsqueeze(x, axis=0)
        if y1d:
            y = view_ops.unsqueeze(y, axis=-1)
        xb, yb = tuple(x.shape[:-2]), tuple(y.shape[:-2])
        if xb != yb:
            tb = self._broadcast_shapes(xb, yb)
            if xb != tb:
                x = view_ops.broadcast_to(x, tb + tuple(x.shape[-2:]))
            if yb != tb:
                y = view_ops.broadcast_to(y, tb + tuple(y.shape[-2:]))
        r = super().__call__([x, y], kwargs)[0]
        if x1d and y1d:
            r = view_ops.squeeze(view_ops.squeeze(r, axis=-1), axis=-1)
        elif x1d:
            r = view_ops.squeeze(r, axis=-2)
        elif y1d:
            r = view_ops.squeeze(r, axis=-1)
        return [r]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # dX = G @ W^T ; dW = X^T @ G  (binary.py:303-314)
        from .view import swap_axes
        x, y = primals
        g = cotangents[0]
        return [matmul(g, swap_axes(y, -2, -1)), matmul(swap_axes(x, -2, -1), g)]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        x, y = primals
        return [add(matmul(x, tangents[1]), matmul(tangents[0], y))]


_add_op, _mul_op, _sub_op, _div_op, _pow_op = AddOp(), MulOp(), SubOp(), DivOp(), PowOp()
_matmul_op = MatmulOp()


def add(x, y) -> Tensor:
    return _add_op([x, y], {})[0]


def mul(x, y) -> Tensor:
    return _mul_op([x, y], {})[0]


def sub(x, y) -> Tensor:
    return _sub_op([x, y], {})[0]


def div(x, y) -> Tensor:
    return _div_op([x, y], {})[0]


def pow(x, y) -> Tensor:  # noqa: A001
    return _pow_op([x, y], {})[0]


def matmul(x, y) -> Tensor:
    return _matmul_op([x, y], {})[0]
