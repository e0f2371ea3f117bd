"""Tensor facade and its implementation record.

Mirrors the data model of nabla/core/tensor/impl.py:42-119 (``TensorImpl``:
buffers, trace flags, cotangent, producer ``OpNode``) and the user-facing
surface of nabla/core/tensor/api.py (``realize`` 734-746, ``to_numpy`` /
``item`` / DLPack 957-1013, ``from_dlpack`` 441-469, generated operator
dunders 1405-1483, ``realize_all`` 1486-1521, ``backward`` 280-306).

A realized tensor owns one contiguous device allocation (a torch tensor used
purely as memory); an unrealized one is a promise that points at the
``OpNode`` that will produce it.
"""
from __future__ import annotations

import weakref
from typing import Any, Sequence

import numpy as np
import torch

from .context import Accelerator, Device, defaults
from .dtype import DType


class TensorImpl:
    __slots__ = (
        "_buffer",
        "shape",
        "dtype",
        "device",
        "is_traced",
        "requires_grad",
        "cotangent",
        "output_refs",
        "output_index",
        "__weakref__",
    )

    def __init__(self, shape, dtype: DType, device: Device | None = None, buffer=None,
                 is_traced: bool = False):
        self._buffer = buffer
        self.shape = tuple(int(d) for d in shape)
        self.dtype = dtype
        self.device = device if device is not None else Accelerator()
        self.is_traced = is_traced
        self.requires_grad = False
        self.cotangent = None
        self.output_refs = None  # OpNode
        self.output_index = 0

    @property
    def is_realized(self) -> bool:
        return self._buffer is not None

    @property
    def op(self):
        return self.output_refs.op if self.output_refs is not None else None

    @property
    def op_kwargs(self) -> dict:
        if self.output_refs is None:
            return {}
        return self.output_refs.op_kwargs or {}

    @property
    def parents(self):
        if self.output_refs is None:
            return []
        return [a for a in self.output_refs.op_args if isinstance(a, TensorImpl)]

    def __repr__(self) -> str:
        state = "real" if self.is_realized else "lazy"
        return f"TensorImpl(shape={self.shape}, dtype={self.dtype.name}, {state})"


def _storage_device() -> torch.device:
    from ..backend.executor import get_executor

    return get_executor().torch_device


# Scalars that appear in expressions such as ``x * 0.5`` become realized 0-d
# inputs (api.py:1300-1304); uploading one per op call would put a blocking
# host-to-device copy on every step, so they are cached by value.
_SCALAR_CACHE: dict[tuple, torch.Tensor] = {}


def _scalar_buffer(value, dtype: DType) -> torch.Tensor:
    dev = _storage_device()
    key = (repr(value), type(value).__name__, dtype, str(dev))
    buf = _SCALAR_CACHE.get(key)
    if buf is None:
        if len(_SCALAR_CACHE) > 4096:
            _SCALAR_CACHE.clear()
        buf = torch.tensor(value, dtype=dtype.to_torch()).to(dev)
        _SCALAR_CACHE[key] = buf
    return buf


class Tensor:
    """Multi-dimensional array with lazy evaluation and autograd hooks."""

    __slots__ = ("_impl", "__weakref__")
    __array_priority__ = 1000

    def __init__(self, data: Any = None, *, impl: TensorImpl | None = None, dtype: DType | None = None,
                 device: Device | None = None, is_traced: bool = False):
        if impl is not None:
            self._impl = impl
            return
        if data is None:
            raise TypeError("Tensor() needs data or impl")
        t = Tensor.constant(data, dtype=dtype, device=device)
        self._impl = t._impl
        self._impl.is_traced = is_traced

    # ---- construction -------------------------------------------------------
    @classmethod
    def _from_torch(cls, buf: torch.Tensor, device: Device | None = None) -> "Tensor":
        buf = buf.to(_storage_device())
        if not buf.is_contiguous():
            buf = buf.contiguous()
        impl = TensorImpl(tuple(buf.shape), DType.from_torch(buf.dtype), device, buffer=buf)
        return cls(impl=impl)

    @classmethod
    def from_dlpack(cls, array: Any) -> "Tensor":
        """Import any DLPack / numpy / torch array (api.py:441-469)."""
        if isinstance(array, Tensor):
            return array
        if isinstance(array, torch.Tensor):
            t = array.detach()
        elif isinstance(array, np.ndarray):
            arr = array
            if arr.dtype == np.float64:
                arr = arr.astype(np.float32)
            # ascontiguousarray promotes a 0-d array to one dimension; keep the caller's shape
            t = torch.from_numpy(np.ascontiguousarray(arr).reshape(arr.shape))
        elif hasattr(array, "__dlpack__"):
            t = torch.from_dlpack(array)
        else:
            t = torch.from_numpy(np.ascontiguousarray(np.asarray(array)))
        return cls._from_torch(t)

    @classmethod
    def constant(cls, value: Any, *, dtype: DType | None = None, device: Device | None = None) -> "Tensor":
        """A realized tensor holding ``value`` (creation.py:289-350)."""
        if isinstance(value, Tensor):
            return value
        d_dtype, d_device = defaults()
        device = device or d_device
        if isinstance(value, (bool, int, float)):
            if dtype is None:
                dtype = d_dtype if isinstance(value, float) else (
                    DType.bool if isinstance(value, bool) else d_dtype)
            buf = _scalar_buffer(value, dtype)
            return cls(impl=TensorImpl((), dtype, device, buffer=buf))
        if isinstance(value, torch.Tensor):
            t = value.detach()
        else:
            arr = np.asarray(value)
            if arr.dtype == np.float64:
                arr = arr.astype(np.float32)
            # ascontiguousarray promotes a 0-d array to one dimension; keep the caller's shape
            t = torch.from_numpy(np.ascontiguousarray(arr).reshape(arr.shape))
        if dtype is not None and t.dtype != dtype.to_torch():
            t = t.to(dtype.to_torch())
        return cls._from_torch(t, device)

    @classmethod
    def full(cls, shape, value, *, dtype=None, device=None):
        from ..ops.creation import full
        return full(shape, value, dtype=dtype, device=device)

    @classmethod
    def zeros(cls, shape, *, dtype=None, device=None):
        from ..ops.creation import zeros
        return zeros(shape, dtype=dtype, device=device)

    @classmethod
    def ones(cls, shape, *, dtype=None, device=None):
        from ..ops.creation import ones
        return ones(shape, dtype=dtype, device=device)

    @classmethod
    def arange(cls, start=0, stop=None, step=1, *, dtype=None, device=None):
        from ..ops.creation import arange
        return arange(start, stop, step, dtype=dtype, device=device)

    # ---- metadata -----------------------------------------------------------
    @property
    def shape(self) -> tuple[int, ...]:
        return self._impl.shape

    @property
    def dtype(self) -> DType:
        return self._impl.dtype

    @property
    def device(self) -> Device:
        return self._impl.device

    @property
    def rank(self) -> int:
        return len(self._impl.shape)

    ndim = rank

    def dim(self) -> int:
        return len(self._impl.shape)

    def size(self, dim: int | None = None):
        return self.shape if dim is None else self.shape[dim]

    def numel(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n

    @property
    def real(self) -> bool:
        return self._impl.is_realized

    is_realized = real

    @property
    def is_traced(self) -> bool:
        return self._impl.is_traced

    @is_traced.setter
    def is_traced(self, v: bool) -> None:
        self._impl.is_traced = bool(v)

    @property
    def requires_grad(self) -> bool:
        return self._impl.requires_grad

    @requires_grad.setter
    def requires_grad(self, v: bool) -> None:
        self._impl.requires_grad = bool(v)
        if v:
            self._impl.is_traced = True

    def requires_grad_(self, v: bool = True) -> "Tensor":
        self.requires_grad = v
        return self

    @property
    def is_leaf(self) -> bool:
        return self._impl.output_refs is None

    @property
    def op_kwargs(self) -> dict:
        return self._impl.op_kwargs

    @property
    def grad(self):
        c = self._impl.cotangent
        return Tensor(impl=c) if c is not None else None

    @grad.setter
    def grad(self, value) -> None:
        self._impl.cotangent = value._impl if value is not None else None

    def detach(self) -> "Tensor":
        """A realized copy of the value that shares storage and carries no history."""
        self.realize()
        impl = TensorImpl(self.shape, self.dtype, self.device, buffer=self._impl._buffer)
        return Tensor(impl=impl)

    def backward(self, gradient: "Tensor | None" = None, retain_graph: bool = False,
                 create_graph: bool = False) -> None:
        from .backward import backward as _backward
        _backward(self, gradient, retain_graph=retain_graph, create_graph=create_graph)

    # ---- evaluation ---------------------------------------------------------
    def realize(self) -> "Tensor":
        if not self.real:
            from .engine import GRAPH
            GRAPH.evaluate(self)
        return self

    @property
    def buffers(self) -> torch.Tensor:
        """The device allocation (realizes first)."""
        self.realize()
        return self._impl._buffer

    def to_torch(self) -> torch.Tensor:
        return self.buffers

    def to_numpy(self) -> np.ndarray:
        buf = self.buffers
        from ..backend.executor import get_executor
        get_executor().check_status()
        if buf.dtype == torch.bfloat16:
            buf = buf.float()
        return buf.detach().cpu().numpy()

    numpy = to_numpy

    def item(self):
        if self.numel() != 1:
            raise TypeError(f"item() needs a one-element tensor, shape is {self.shape}")
        return self.buffers.reshape(()).item()

    def __dlpack__(self, stream=None):
        return self.buffers.__dlpack__()

    def __dlpack_device__(self):
        return self.buffers.__dlpack_device__()

    def __array__(self, dtype=None, copy=None):
        a = self.to_numpy()
        return a.astype(dtype) if dtype is not None else a

    def __float__(self):
        return float(self.item())

    def __int__(self):
        return int(self.item())

    def __bool__(self):
        if self.numel() != 1:
            raise ValueError("truth value of a tensor with more than one element is ambiguous")
        return bool(self.item())

    def __len__(self) -> int:
        if not self.shape:
            raise TypeError("len() of a 0-d tensor")
        return self.shape[0]

    def __hash__(self) -> int:
        return id(self._impl)

    def __repr__(self) -> str:
        if self.real:
            return f"Tensor({self.to_numpy()!r}, dtype={self.dtype.name})"
        return f"Tensor(shape={self.shape}, dtype={self.dtype.name}, unrealized)"

    # ---- shape methods --------------------------------------------------------
    def reshape(self, *shape):
        from ..ops import view
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        return view.reshape(self, shape)

    view = reshape

    def squeeze(self, axis=None):
        from ..ops import view
        return view.squeeze(self, axis)

    def unsqueeze(self, axis: int):
        from ..ops import view
        return view.unsqueeze(self, axis)

    def swap_axes(self, a: int, b: int):
        from ..ops import view
        return view.swap_axes(self, a, b)

    transpose = swap_axes

    def permute(self, *order):
        from ..ops import view
        if len(order) == 1 and isinstance(order[0], (tuple, list)):
            order = tuple(order[0])
        return view.permute(self, order)

    def flatten(self, start_dim: int = 0, end_dim: int = -1):
        from ..ops import view
        return view.flatten(self, start_dim, end_dim)

    def broadcast_to(self, shape):
        from ..ops import view
        return view.broadcast_to(self, shape)

    def expand(self, *shape):
        return self.broadcast_to(shape)

    @property
    def T(self):
        return self.swap_axes(-2, -1)

    def cast(self, dtype: DType):
        from ..ops.unary import cast
        return cast(self, dtype)

    astype = cast

    def to(self, target):
        """``to(dtype)`` casts; ``to(device)`` is the identity on this single-device backend
        (api.py ``Tensor.to``)."""
        if isinstance(target, DType):
            return self if target is self.dtype else self.cast(target)
        return self

    def type_as(self, other: "Tensor"):
        return self.cast(other.dtype)

    def __getitem__(self, key):
        from ..ops.view import getitem
        return getitem(self, key)


class BatchedTensor(Tensor):
    """What a function sees of a mapped argument inside ``vmap``: the tensor with its first
    ``_bd`` (hidden) dimensions taken away.  The storage keeps them, in front; ``shape``,
    ``rank`` and the axis arguments of every op are those of one element, and each op call
    that meets such a tensor runs once on the whole batch with its axes shifted
    (nabla_amd/ops/batching.py).  Plays the part of the ``batch_dims`` counter of the
    reference's tensors (nabla/core/tensor/impl.py, nabla/ops/view/batch.py)."""

    __slots__ = ("_bd",)

    def __init__(self, physical: Tensor, batch_dims: int):
        Tensor.__init__(self, impl=physical._impl)
        self._bd = int(batch_dims)

    def physical(self) -> Tensor:
        """The same storage with the hidden dimensions in view."""
        return Tensor(impl=self._impl)

    @property
    def batch_shape(self) -> tuple[int, ...]:
        return tuple(self._impl.shape[:self._bd])

    @property
    def shape(self) -> tuple[int, ...]:
        return tuple(self._impl.shape[self._bd:])

    @property
    def rank(self) -> int:
        return len(self._impl.shape) - self._bd

    ndim = rank

    def dim(self) -> int:
        return len(self._impl.shape) - self._bd

    def __repr__(self) -> str:
        return (f"BatchedTensor(shape={self.shape}, batch={self.batch_shape}, "
                f"dtype={self.dtype.name})")


def _ensure_tensor(value: Any, like: Tensor) -> Tensor:
    if isinstance(value, Tensor):
        return value
    if isinstance(value, (bool, int, float)):
        dt = like.dtype
        if isinstance(value, float) and not dt.is_float():
            dt = defaults()[0]
        return Tensor.constant(value, dtype=dt, device=like.device)
    return Tensor.constant(value, device=like.device)


# ---- generated methods (api.py:1405-1483) -------------------------------------
def _bind() -> None:
    def binary(op_name: str, reverse: bool):
        def method(self, other):
            from .. import ops
            fn = getattr(ops, op_name)
            other_t = _ensure_tensor(other, self)
            return fn(other_t, self) if reverse else fn(self, other_t)
        return method

    for name, op_name, rev in [
        ("__add__", "add", False), ("__radd__", "add", True),
        ("__sub__", "sub", False), ("__rsub__", "sub", True),
        ("__mul__", "mul", False), ("__rmul__", "mul", True),
        ("__truediv__", "div", False), ("__rtruediv__", "div", True),
        ("__matmul__", "matmul", False), ("__rmatmul__", "matmul", True),
        ("__pow__", "pow", False), ("__rpow__", "pow", True),
    ]:
        setattr(Tensor, name, binary(op_name, rev))

    for name, op_name in {
        "__eq__": "equal", "__ne__": "not_equal", "__lt__": "less", "__le__": "less_equal",
        "__gt__": "greater", "__ge__": "greater_equal",
    }.items():
        setattr(Tensor, name, binary(op_name, False))

    def unary(op_name: str):
        def method(self):
            from .. import ops
            return getattr(ops, op_name)(self)
        return method

    for name in ["abs", "exp", "log", "relu", "sigmoid", "sqrt", "tanh", "erf", "rsqrt"]:
        setattr(Tensor, name, unary(name))
    setattr(Tensor, "__neg__", unary("neg"))
    setattr(Tensor, "__abs__", unary("abs"))

    def reduce(op_name: str):
        def method(self, axis=None, keepdims: bool = False):
            from .. import ops
            return getattr(ops, op_name)(self, axis=axis, keepdims=keepdims)
        return method

    for name, op_name in {"sum": "reduce_sum", "mean": "mean", "max": "reduce_max",
                          "min": "reduce_min"}.items():
        setattr(Tensor, name, reduce(op_name))

    def argreduce(op_name: str):
        def method(self, axis=None, keepdims: bool = False):
            from .. import ops
            return getattr(ops, op_name)(self, axis=axis, keepdims=keepdims)
        return method

    setattr(Tensor, "argmax", argreduce("argmax"))
    setattr(Tensor, "argmin", argreduce("argmin"))

    def axis_unary(op_name: str):
        def method(self, axis: int = -1):
            from .. import ops
            return getattr(ops, op_name)(self, axis=axis)
        return method

    setattr(Tensor, "softmax", axis_unary("softmax"))
    setattr(Tensor, "logsoftmax", axis_unary("logsoftmax"))

    def gelu(self, approximate: str = "none"):
        from .. import ops
        return ops.gelu(self, approximate=approximate)

    setattr(Tensor, "gelu", gelu)


_bind()


def realize_all(*tensors: Tensor) -> tuple[Tensor, ...]:
    """Evaluate several tensors as ONE graph (api.py:1486-1521)."""
    from .. import config
    from .engine import GRAPH

    if config.TRACING:
        return tensors
    pending = [t for t in tensors if isinstance(t, Tensor) and not t.real]
    if pending:
        GRAPH.evaluate(*pending)
    return tensors
