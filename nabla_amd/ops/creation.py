"""Creation ops (nabla/ops/creation.py): full / zeros / ones 50-93 and 353-426,
arange 96-149, tril / triu 225-274, constant 289-350, ``*_like`` 586-645.
Random ops are not provided: the reference draws them from MAX's RNG stream,
which cannot be reproduced; seeded host arrays are uploaded instead.
"""
from __future__ import annotations

import math
from typing import Any

from ..backend import ir
from ..core.context import Device, defaults
from ..core.dtype import DType
from ..core.tensor import Tensor
from .base import CreationOperation, UnaryOperation, ensure_tensor


class FullOp(CreationOperation):
    @property
    def name(self) -> str:
        return "full"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        return [tuple(kwargs["shape"])], [kwargs["dtype"]], [kwargs["device"]]

    def kernel(self, args, kwargs):
        return [ir.fill(kwargs["shape"], kwargs["dtype"], kwargs["value"])]


class ArangeOp(CreationOperation):
    @property
    def name(self) -> str:
        return "arange"

    @staticmethod
    def _count(start, stop, step) -> int:
        return max(0, int(math.ceil((stop - start) / step)))

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        n = self._count(kwargs["start"], kwargs["stop"], kwargs["step"])
        return [(n,)], [kwargs["dtype"]], [kwargs["device"]]

    def kernel(self, args, kwargs):
        n = self._count(kwargs["start"], kwargs["stop"], kwargs["step"])
        return [ir.iota(n, kwargs["dtype"], kwargs["start"], kwargs["step"])]


class _TriOp(UnaryOperation):
    _upper = False

    def kernel(self, args, kwargs):
        return [ir.tril(args[0], kwargs.get("k", 0), upper=self._upper)]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return [type(self)()([cotangents[0]], dict(kwargs))[0]]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [type(self)()([tangents[0]], dict(kwargs))[0]]


class TrilOp(_TriOp):
    @property
    def name(self) -> str:
        return "tril"


class TriuOp(_TriOp):
    _upper = True

    @property
    def name(self) -> str:
        return "triu"


_full_op, _arange_op, _tril_op, _triu_op = FullOp(), ArangeOp(), TrilOp(), TriuOp()


def _resolve(dtype, device):
    d_dtype, d_device = defaults()
    return dtype or d_dtype, device or d_device


def constant(value: Any, *, dtype: DType | None = None, device: Device | None = None) -> Tensor:
    return Tensor.constant(value, dtype=dtype, device=device)


def full(shape, value, *, dtype: DType | None = None, device: Device | None = None) -> Tensor:
    dtype, device = _resolve(dtype, device)
    if isinstance(shape, int):
        shape = (shape,)
    return _full_op([], {"shape": tuple(int(d) for d in shape), "value": float(value),
                         "dtype": dtype, "device": device})[0]


def zeros(shape, *, dtype=None, device=None) -> Tensor:
    return full(shape, 0.0, dtype=dtype, device=device)


def ones(shape, *, dtype=None, device=None) -> Tensor:
    return full(shape, 1.0, dtype=dtype, device=device)


def arange(start=0, stop=None, step=1, *, dtype=None, device=None) -> Tensor:
    if stop is None:
        start, stop = 0, start
    dtype, device = _resolve(dtype, device)
    if step == 0:
        raise ValueError("arange: step must not be zero")
    return _arange_op([], {"start": float(start), "stop": float(stop), "step": float(step),
                           "dtype": dtype, "device": device})[0]


def tril(x, k: int = 0) -> Tensor:
    return _tril_op([ensure_tensor(x)], {"k": int(k)})[0]


def triu(x, k: int = 0) -> Tensor:
    return _triu_op([ensure_tensor(x)], {"k": int(k)})[0]


def zeros_like(x: Tensor) -> Tensor:
    return full(x.shape, 0.0, dtype=x.dtype, device=x.device)


def ones_like(x: Tensor) -> Tensor:
    return full(x.shape, 1.0, dtype=x.dtype, device=x.device)


def full_like(x: Tensor, value) -> Tensor:
    return full(x.shape, value, dtype=x.dtype, device=x.device)
