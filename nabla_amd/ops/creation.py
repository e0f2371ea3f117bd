"""Creation ops (nabla/ops/creation.py): full / zeros / ones 50-93 and 353-426,
arange 96-149, tril / triu 225-274, constant 289-350, ``*_like`` 586-645.
``uniform`` / ``gaussian`` 152-183 and 462-511 draw from a device generator of this backend
(Philox4x32-10): the reference's numbers come from MAX's generator, whose stream is not part of
its sources, so values differ while distribution and reproducibility under a seed hold.
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


class RandomOp(CreationOperation):
    """A tensor drawn from the device generator (``uniform`` / ``gaussian`` at
    nabla/ops/creation.py:152-183).  Every evaluation draws anew: the generator's state lives on
    the device and moves on with every step that uses it."""

    draws_random = True  # (the engine keeps the result of the evaluation that draws it)

    def __init__(self, mode: str, public_name: str):
        self._mode, self._name = mode, public_name

    @property
    def name(self) -> str:
        return self._name

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        return [tuple(kwargs["shape"])], [kwargs["dtype"]], [kwargs["device"]]

    def kernel(self, args, kwargs):
        return [ir.random(kwargs["shape"], kwargs["dtype"], self._mode, kwargs["a"], kwargs["b"])]


_full_op, _arange_op, _tril_op, _triu_op = FullOp(), ArangeOp(), TrilOp(), TriuOp()
_uniform_op, _gaussian_op = RandomOp("uniform", "uniform"), RandomOp("normal", "gaussian")
_keep_mask_op = RandomOp("keep", "keep_mask")


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


def _shape_tuple(shape) -> tuple[int, ...]:
    return (int(shape),) if isinstance(shape, int) else tuple(int(d) for d in shape)


def uniform(shape=(), low: float = 0.0, high: float = 1.0, *, dtype=None, device=None) -> Tensor:
    """Samples of U[low, high) (creation.py:462-485)."""
    dtype, device = _resolve(dtype, device)
    return _uniform_op([], {"shape": _shape_tuple(shape), "a": float(low), "b": float(high),
                            "dtype": dtype, "device": device})[0]


def gaussian(shape=(), mean: float = 0.0, std: float = 1.0, *, dtype=None, device=None) -> Tensor:
    """Samples of N(mean, std^2) (creation.py:488-511)."""
    dtype, device = _resolve(dtype, device)
    return _gaussian_op([], {"shape": _shape_tuple(shape), "a": float(mean), "b": float(std),
                             "dtype": dtype, "device": device})[0]


normal = gaussian


def keep_mask(shape, p: float, *, dtype=None, device=None) -> Tensor:
    """``uniform(shape) > p`` as 1 / 0 in ``dtype`` (bool allowed) without the uniform tensor in
    between: the mask of dropout with rate ``p``."""
    dtype, device = _resolve(dtype, device)
    return _keep_mask_op([], {"shape": _shape_tuple(shape), "a": float(p), "b": 0.0,
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
