"""Parameter initialisers (nabla/nn/functional/init.py).  The reference samples
from MAX's device RNG; here values come from a seeded numpy generator on the
host and are uploaded, so runs are reproducible but the streams differ."""
from __future__ import annotations

import math

import numpy as np

from ...core.dtype import DType
from ...core.tensor import Tensor

_RNG = np.random.default_rng(0)


def manual_seed(seed: int) -> None:
    global _RNG
    _RNG = np.random.default_rng(seed)


def _normal(shape, std: float, dtype: DType) -> Tensor:
    arr = (_RNG.standard_normal(tuple(shape)) * std).astype(np.float32)
    return Tensor.constant(arr, dtype=dtype)


def xavier_normal(shape, dtype: DType = DType.float32, gain: float = 1.0) -> Tensor:
    fan_in, fan_out = shape[0], shape[-1]
    return _normal(shape, gain * math.sqrt(2.0 / (fan_in + fan_out)), dtype)


def he_normal(shape, dtype: DType = DType.float32) -> Tensor:
    return _normal(shape, math.sqrt(2.0 / shape[0]), dtype)


def normal(shape, mean: float = 0.0, std: float = 1.0, dtype: DType = DType.float32) -> Tensor:
    arr = (_RNG.standard_normal(tuple(shape)) * std + mean).astype(np.float32)
    return Tensor.constant(arr, dtype=dtype)
