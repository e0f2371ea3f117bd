"""Small ops next to the hot path, each built from primitives the kernels already have:
``trunc`` / ``floor`` (nabla/ops/unary.py:405-432, 540-566: zero derivative), ``is_nan`` /
``is_inf`` (455-470), ``log1p`` (471-486), ``atanh``, ``logical_xor`` (comparison.py:258-262), ``outer``
(binary.py:575-600), ``flip`` (view/axes.py:844-854), ``split`` / ``chunk`` / ``unbind`` /
``minmax`` (multi_output.py:481-538).  They lower to the same row programs, views and index
kernels as their parts, so they add no kernels."""
from __future__ import annotations

import numpy as np

from ..backend import ir
from ..core.tensor import Tensor
from .base import UnaryOperation, ensure_tensor


class TruncOp(UnaryOperation):
    """Round toward zero; piecewise constant, so both derivative rules give zeros."""

    @property
    def name(self) -> str:
        return "trunc"

    def kernel(self, args, kwargs):
        return [ir.ew("trunc", args[0])]

    def _derivative(self, primal, output):
        from .creation import zeros_like
        return zeros_like(output)


_trunc_op = TruncOp()


def trunc(x) -> Tensor:
    x = ensure_tensor(x)
    return x if not x.dtype.is_float() else _trunc_op([x], {})[0]


def floor(x) -> Tensor:
    """Largest integer not above ``x``: ``trunc(x)``, less one where that lies above ``x``."""
    from .binary import sub
    from .comparison import greater
    from .unary import cast
    x = ensure_tensor(x)
    if not x.dtype.is_float():
        return x
    t = trunc(x)
    return sub(t, cast(greater(t, x), x.dtype))


def is_nan(x) -> Tensor:
    """True where ``x`` is not a number (the only value that differs from itself)."""
    from .comparison import not_equal
    x = ensure_tensor(x)
    return not_equal(x, x)


def is_inf(x) -> Tensor:
    from .comparison import equal
    from .unary import abs as abs_
    x = ensure_tensor(x)
    return equal(abs_(x), float("inf"))


def log1p(x) -> Tensor:
    """``log(1 + x)`` without losing small ``x``: with u = 1 + x as rounded, log(u) * x / (u - 1)
    corrects for the rounding of u, x itself is returned where u == 1 and u where it is infinite
    (the quotient would be inf / inf there).  The derivative that falls out of the parts equals the
    reference's 1 / (1 + x) up to that rounding."""
    from .binary import add, div, mul, sub
    from .comparison import equal
    from .control_flow import where
    from .unary import log
    from .comparison import logical_or
    from .creation import ones_like
    x = ensure_tensor(x)
    u = add(x, 1.0)
    d = sub(u, 1.0)
    one = equal(d, 0.0)
    big = is_inf(u)                                   # x = +inf: the answer is u itself
    ones = ones_like(x)
    safe = where(logical_or(one, big), ones, d)       # a divisor of 1 where the quotient is unused
    corrected = mul(log(where(big, ones, u)), div(where(big, ones, x), safe))
    return where(one, x, where(big, u, corrected))


def atanh(x) -> Tensor:
    """Inverse hyperbolic tangent as (log1p(x) - log1p(-x)) / 2, which keeps small arguments exact;
    the derivative of the parts is 1 / (1 - x^2), the reference's rule (unary.py, AtanhOp)."""
    from .binary import mul, sub
    from .unary import neg
    x = ensure_tensor(x)
    return mul(sub(log1p(x), log1p(neg(x))), 0.5)


def logical_xor(x, y) -> Tensor:
    from .comparison import not_equal
    from .unary import cast
    from ..core import DType
    x, y = ensure_tensor(x), ensure_tensor(y)
    return not_equal(cast(x, DType.bool), cast(y, DType.bool))


def outer(x, y) -> Tensor:
    """``x[..., :, None] * y[..., None, :]``: an (M, N) matrix for vectors (M,) and (N,)."""
    from .binary import mul
    from .view import unsqueeze
    x, y = ensure_tensor(x), ensure_tensor(y)
    if len(x.shape) < 1 or len(y.shape) < 1:
        raise ValueError(f"outer expects tensors of rank >= 1, got {tuple(x.shape)} and {tuple(y.shape)}")
    return mul(unsqueeze(x, -1), unsqueeze(y, -2))


def _axis(axis: int, rank: int) -> int:
    if not -rank <= axis < rank:
        raise ValueError(f"axis {axis} out of range for rank {rank}")
    return axis % rank


def flip(x, axis: int) -> Tensor:
    """Reverse ``x`` along ``axis``: a gather with descending indices (its gradient is the same
    gather of the cotangent, through scatter)."""
    from .view import gather
    x = ensure_tensor(x)
    a = _axis(axis, len(x.shape))
    n = int(x.shape[a])
    idx = Tensor.constant(np.arange(n - 1, -1, -1, dtype=np.int64))
    return gather(x, idx, axis=a)


def _pieces(x: Tensor, axis: int, sizes: list[int]) -> list[Tensor]:
    from .view import slice_tensor
    out, off = [], 0
    for s in sizes:
        start = [0] * len(x.shape)
        size = [int(d) for d in x.shape]
        start[axis], size[axis] = off, s
        out.append(slice_tensor(x, start, size))
        off += s
    return out


def split(x, num_splits: int, axis: int = 0) -> list:
    """``num_splits`` equal parts along ``axis`` (views; the size must divide evenly)."""
    x = ensure_tensor(x)
    a = _axis(axis, len(x.shape))
    n = int(x.shape[a])
    if num_splits <= 0 or n % num_splits:
        raise ValueError(f"split: axis size {n} is not divisible by num_splits={num_splits}")
    return _pieces(x, a, [n // num_splits] * num_splits)


def chunk(x, chunks: int, axis: int = 0) -> list:
    """Parts of ceil(n / chunks) along ``axis``; the last may be smaller."""
    x = ensure_tensor(x)
    a = _axis(axis, len(x.shape))
    n = int(x.shape[a])
    if chunks <= 0:
        raise ValueError(f"chunk: chunks must be > 0, got {chunks}")
    step = -(-n // chunks)
    sizes = [min(step, n - o) for o in range(0, n, step)] if n else []
    return _pieces(x, a, sizes)


def unbind(x, axis: int = 0) -> list:
    """The ``x.shape[axis]`` slices along ``axis``, with that axis removed."""
    from .view import squeeze
    x = ensure_tensor(x)
    a = _axis(axis, len(x.shape))
    return [squeeze(p, a) for p in _pieces(x, a, [1] * int(x.shape[a]))]


def minmax(x) -> dict:
    """``{'min': ..., 'max': ...}`` over all elements, both scalars."""
    from .reduction import reduce_max, reduce_min
    x = ensure_tensor(x)
    axes = list(range(len(x.shape)))
    if not axes:
        return {"min": x, "max": x}
    return {"min": reduce_min(x, axis=axes), "max": reduce_max(x, axis=axes)}


__all__ = ["atanh", "trunc", "floor", "is_nan", "is_inf", "log1p", "logical_xor", "outer", "flip", "split",
           "chunk", "unbind", "minmax"]
