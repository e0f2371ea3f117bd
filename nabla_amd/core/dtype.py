"""Element types of the backend.

The reference takes ``max.dtype.DType`` straight from the Modular wheel
(nabla/__init__.py:21-22); this enum keeps the member names the reference's
user code spells (``DType.float32``, ``DType.bfloat16``, ``DType.int64``,
``DType.bool``) and adds the mappings to numpy / torch / the kernel ABI.
"""
from __future__ import annotations

import enum

import numpy as np
import torch


class DType(enum.Enum):
    float32 = "float32"
    bfloat16 = "bfloat16"
    float16 = "float16"
    int32 = "int32"
    int64 = "int64"
    uint8 = "uint8"
    bool = "bool"

    # -- classification ---------------------------------------------------
    def is_float(self) -> bool:
        return self in (DType.float32, DType.bfloat16, DType.float16)

    def is_integral(self) -> bool:
        return self in (DType.int32, DType.int64, DType.uint8)

    @property
    def size_in_bytes(self) -> int:
        return _SIZE[self]

    # -- conversions --------------------------------------------------------
    def to_torch(self) -> torch.dtype:
        return _TO_TORCH[self]

    def to_numpy(self):
        if self is DType.bfloat16:
            raise TypeError("numpy has no bfloat16; cast to float32 first")
        return _TO_NUMPY[self]

    @property
    def abi(self) -> int:
        """``nbk_dtype`` code of include/nbk.h."""
        return _ABI[self]

    @staticmethod
    def from_torch(dt: torch.dtype) -> "DType":
        try:
            return _FROM_TORCH[dt]
        except KeyError:
            raise TypeError(f"unsupported torch dtype {dt}") from None

    @staticmethod
    def from_numpy(dt) -> "DType":
        dt = np.dtype(dt)
        try:
            return _FROM_NUMPY[dt]
        except KeyError:
            raise TypeError(f"unsupported numpy dtype {dt}") from None

    def __repr__(self) -> str:
        return f"DType.{self.name}"


_SIZE = {
    DType.float32: 4, DType.bfloat16: 2, DType.float16: 2,
    DType.int32: 4, DType.int64: 8, DType.uint8: 1, DType.bool: 1,
}
_TO_TORCH = {
    DType.float32: torch.float32, DType.bfloat16: torch.bfloat16, DType.float16: torch.float16,
    DType.int32: torch.int32, DType.int64: torch.int64, DType.uint8: torch.uint8,
    DType.bool: torch.bool,
}
_FROM_TORCH = {v: k for k, v in _TO_TORCH.items()}
_TO_NUMPY = {
    DType.float32: np.float32, DType.float16: np.float16,
    DType.int32: np.int32, DType.int64: np.int64, DType.uint8: np.uint8, DType.bool: np.bool_,
}
_FROM_NUMPY = {np.dtype(v): k for k, v in _TO_NUMPY.items()}
_FROM_NUMPY[np.dtype(np.float64)] = DType.float32  # host doubles narrow to the default float
_ABI = {
    DType.float32: 0, DType.bfloat16: 1, DType.float16: 2,
    DType.int32: 3, DType.int64: 4, DType.uint8: 5, DType.bool: 5,  # one byte either way
}


def promote(a: DType, b: DType) -> DType:
    """Result type of a binary arithmetic op on ``a`` and ``b``."""
    if a is b:
        return a
    order = [DType.bool, DType.uint8, DType.int32, DType.int64, DType.float16, DType.bfloat16,
             DType.float32]
    if {a, b} == {DType.float16, DType.bfloat16}:
        return DType.float32
    return order[max(order.index(a), order.index(b))]
