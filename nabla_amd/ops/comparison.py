"""Comparisons and logical ops; results are bool (nabla/ops/comparison.py:27-130)."""
from __future__ import annotations

from ..backend import ir
from ..core.dtype import DType, promote
from ..core.tensor import Tensor
from .base import BinaryOperation, UnaryOperation


class _CompareOp(BinaryOperation):
    result_dtype = DType.bool
    _fn = ""
    _name = ""

    @property
    def name(self) -> str:
        return self._name

    def kernel(self, args, kwargs):
        a, b = args
        dt = promote(a.dtype, b.dtype)
        return [ir.ew(self._fn, ir.cast(a, dt), ir.cast(b, dt))]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return [None, None]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [None]


def _make(name: str, fn: str):
    cls = type(f"{name.title().replace('_', '')}Op", (_CompareOp,), {"_fn": fn, "_name": name})
    return cls()


_equal_op = _make("equal", "eq")
_not_equal_op = _make("not_equal", "ne")
_greater_op = _make("greater", "gt")
_greater_equal_op = _make("greater_equal", "ge")
_logical_and_op = _make("logical_and", "and")
_logical_or_op = _make("logical_or", "or")


class LogicalNotOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "logical_not"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(x.shape)], [DType.bool], [x.device]

    def kernel(self, args, kwargs):
        return [ir.ew("not", args[0])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return [None]


_logical_not_op = LogicalNotOp()


def equal(x, y) -> Tensor:
    return _equal_op([x, y], {})[0]


def not_equal(x, y) -> Tensor:
    return _not_equal_op([x, y], {})[0]


def greater(x, y) -> Tensor:
    return _greater_op([x, y], {})[0]


def greater_equal(x, y) -> Tensor:
    return _greater_equal_op([x, y], {})[0]


def less(x, y) -> Tensor:
    # less is greater with swapped operands (comparison.py:118-130)
    return _greater_op([y, x], {})[0]


def less_equal(x, y) -> Tensor:
    return _greater_equal_op([y, x], {})[0]


def logical_and(x, y) -> Tensor:
    return _logical_and_op([x, y], {})[0]


def logical_or(x, y) -> Tensor:
    return _logical_or_op([x, y], {})[0]


def logical_not(x) -> Tensor:
    return _logical_not_op([x], {})[0]
