"""Axis reductions.

Mirrors nabla/ops/reduction.py: ReduceSumOp 147-172, MeanOp 175-202,
ReduceMaxOp 205-245 (VJP gives the full cotangent to EVERY tied maximum,
219-230), _multi_axis_reduce 544-581 (one keepdims kernel per axis, descending,
then a separate squeeze / reshape), mean = sum / count 604-639, _ArgReduceOp
739-811 (int64 result).
"""
from __future__ import annotations

from ..backend import ir
from ..core.dtype import DType
from ..core.tensor import Tensor
from .base import ReduceOperation, ensure_tensor


class ReduceSumOp(ReduceOperation):
    @property
    def name(self) -> str:
        return "reduce_sum"

    def kernel(self, args, kwargs):
        return [ir.reduce("sum", args[0], kwargs.get("axis", 0))]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .view import broadcast_to
        return [broadcast_to(cotangents[0], primals[0].shape)]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [_reduce_sum_op([tangents[0]], dict(kwargs))[0]]


class _ReduceExtremeOp(ReduceOperation):
    _fn = "max"

    def kernel(self, args, kwargs):
        return [ir.reduce(self._fn, args[0], kwargs.get("axis", 0))]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .binary import mul
        from .comparison import equal
        from .view import broadcast_to
        x = primals[0]
        mask = equal(x, broadcast_to(outputs[0], x.shape))
        return [mul(broadcast_to(cotangents[0], x.shape), mask)]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        from .binary import mul
        from .comparison import equal
        from .view import broadcast_to
        x = primals[0]
        mask = equal(x, broadcast_to(outputs[0], x.shape))
        return [_reduce_sum_op([mul(tangents[0], mask)], dict(kwargs))[0]]


class ReduceMaxOp(_ReduceExtremeOp):
    _fn = "max"

    @property
    def name(self) -> str:
        return "reduce_max"


class ReduceMinOp(_ReduceExtremeOp):
    _fn = "min"

    @property
    def name(self) -> str:
        return "reduce_min"


class _ArgReduceOp(ReduceOperation):
    _fn = "max"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        shapes, _, devices = super().compute_physical_shape(args, kwargs, output_sharding)
        return shapes, [DType.int64], devices

    def kernel(self, args, kwargs):
        x = args[0]
        axis = kwargs.get("axis", -1)
        axis = axis + x.rank if axis < 0 else axis
        if axis == x.rank - 1:
            return [ir.argreduce(self._fn, x, axis)]
        # the kernel works along the last axis; other axes are permuted there and back
        perm = list(range(x.rank))
        perm[axis], perm[-1] = perm[-1], perm[axis]
        r = ir.argreduce(self._fn, ir.permute(x, perm), x.rank - 1)
        return [ir.permute(r, perm)]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return [None]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [None]


class ArgMaxOp(_ArgReduceOp):
    _fn = "max"

    @property
    def name(self) -> str:
        return "argmax"


class ArgMinOp(_ArgReduceOp):
    _fn = "min"

    @property
    def name(self) -> str:
        return "argmin"


_reduce_sum_op, _reduce_max_op, _reduce_min_op = ReduceSumOp(), ReduceMaxOp(), ReduceMinOp()
_argmax_op, _argmin_op = ArgMaxOp(), ArgMinOp()


def _multi_axis_reduce(op, x: Tensor, *, axis=None, keepdims: bool = False) -> Tensor:
    from .view import reshape, squeeze

    x = ensure_tensor(x)
    rank = len(x.shape)
    if axis is None:
        axis = tuple(range(rank))
    if isinstance(axis, (list, tuple)):
        axes = sorted({a if a >= 0 else rank + a for a in axis}, reverse=True)
        if not axes:
            return x
        res = x
        for ax in axes:
            res = op([res], {"axis": ax, "keepdims": True})[0]
        if not keepdims:
            out_shape = tuple(d for i, d in enumerate(x.shape) if i not in set(axes))
            res = reshape(res, out_shape)
        return res
    ax = axis if axis >= 0 else rank + axis
    res = op([x], {"axis": ax, "keepdims": True})[0]
    if not keepdims:
        res = squeeze(res, axis=ax)
    return res


def reduce_sum(x, *, axis=None, keepdims: bool = False) -> Tensor:
    return _multi_axis_reduce(_reduce_sum_op, x, axis=axis, keepdims=keepdims)


def reduce_max(x, *, axis=None, keepdims: bool = False) -> Tensor:
    return _multi_axis_reduce(_reduce_max_op, x, axis=axis, keepdims=keepdims)


def reduce_min(x, *, axis=None, keepdims: bool = False) -> Tensor:
    return _multi_axis_reduce(_reduce_min_op, x, axis=axis, keepdims=keepdims)


def mean(x, *, axis=None, keepdims: bool = False) -> Tensor:
    """``sum / count`` with ``count`` a Python int (reduction.py:623-639)."""
    x = ensure_tensor(x)
    s = reduce_sum(x, axis=axis, keepdims=keepdims)
    shape = x.shape
    if axis is None:
        count = 1
        for d in shape:
            count *= int(d)
    elif isinstance(axis, (list, tuple)):
        count = 1
        for a in axis:
            count *= int(shape[a])
    else:
        count = int(shape[axis])
    return s / count


def _argreduce(op, x, axis, keepdims):
    from .view import reshape, squeeze
    x = ensure_tensor(x)
    if axis is None:
        x = reshape(x, (-1,))
        axis = 0
    rank = len(x.shape)
    ax = axis if axis >= 0 else rank + axis
    r = op([x], {"axis": ax, "keepdims": True})[0]
    if not keepdims:
        r = squeeze(r, axis=ax)
    return r


def argmax(x, axis: int | None = -1, keepdims: bool = False) -> Tensor:
    return _argreduce(_argmax_op, x, axis, keepdims)


def argmin(x, axis: int | None = -1, keepdims: bool = False) -> Tensor:
    return _argreduce(_argmin_op, x, axis, keepdims)


sum = reduce_sum  # noqa: A001
max = reduce_max  # noqa: A001
min = reduce_min  # noqa: A001
