"""Operation base classes: the per-op plugin API.

Same class surface as nabla/ops/base.py: ``Operation`` (91-568) with ``name``,
``kernel(args, kwargs)`` (127-137), ``compute_physical_shape`` (397-409),
``vjp_rule`` / ``jvp_rule`` (454-470), ``adapt_kwargs``, ``execute`` (255-292)
and the ``__call__`` pipeline (294-395); ``BinaryOperation`` with explicit
numpy broadcasting (570-691), ``AxisOp`` (694-760), ``ReduceOperation``
(763-895), ``UnaryOperation`` with the ``_derivative`` shortcut (898-987),
``ShapeOp`` (990-1088) and ``CreationOperation`` (1091-1205).

Ops are stateless singletons invoked as ``op([tensors], {kwargs}) -> [tensors]``.
``kernel`` receives IR values (``nabla_amd.backend.ir.Value``) where the
reference passes MAX ``TensorValue``s and emits IR through the builder functions
of ``nabla_amd.backend.ir``.
"""
from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Any

from .. import config
from ..core.dtype import DType, promote
from ..core.pytree import PyTreeDef, _K_LEAF
from ..core.tensor import BatchedTensor, Tensor, TensorImpl
from ..core.tracing import OpNode

_LEAF_DEF = PyTreeDef(_K_LEAF, None, (), 1)

OpArgs = list
OpKwargs = dict
OpResult = list


def ensure_tensor(x: Any, like: Tensor | None = None) -> Tensor:
    """Wrap Python scalars / arrays as realized tensors (nabla/ops/utils.py:50-71)."""
    if isinstance(x, Tensor):
        return x
    if like is not None and isinstance(x, (bool, int, float)):
        from ..core.tensor import _ensure_tensor
        return _ensure_tensor(x, like)
    return Tensor.constant(x)


def _freeze_kwargs(kwargs: dict | None):
    if not kwargs:
        return ()
    from ..core.engine import _freeze
    return _freeze(kwargs)


class Operation(ABC):
    """Base class of every differentiable operation."""

    multiple_results: bool = False

    @property
    @abstractmethod
    def name(self) -> str: ...

    # -- lowering hook ------------------------------------------------------------
    def kernel(self, args: list, kwargs: dict) -> list:
        """Emit the IR for this op.  ``args`` are IR values, the result is a
        flat list of IR values (even for single-output ops)."""
        raise NotImplementedError(f"{type(self).__name__} must implement kernel")

    def compute_physical_shape(self, args: OpArgs, kwargs: OpKwargs, output_sharding=None):
        """``(shapes, dtypes, devices)`` of the outputs, one entry per output."""
        raise NotImplementedError(f"{type(self).__name__} must implement compute_physical_shape")

    def adapt_kwargs(self, args: OpArgs, kwargs: OpKwargs, batch_dims: int = 0) -> OpKwargs:
        return kwargs

    def execute(self, args: OpArgs, kwargs: OpKwargs):
        """Run this single op right away and return its realized outputs."""
        outs = self(args, kwargs)
        from ..core.tensor import realize_all
        realize_all(*outs)
        return outs

    # -- autodiff -------------------------------------------------------------------
    def vjp_rule(self, primals: list, cotangents: list, outputs: list, kwargs: dict) -> list:
        raise NotImplementedError(f"'{self.name}' does not implement vjp_rule")

    def jvp_rule(self, primals: list, tangents: list, outputs: list, kwargs: dict) -> list:
        raise NotImplementedError(f"'{self.name}' does not implement jvp_rule")

    # -- call pipeline ----------------------------------------------------------------
    def __call__(self, args: OpArgs, kwargs: OpKwargs) -> OpResult:
        kwargs = kwargs or {}
        for a in args:
            if type(a) is BatchedTensor:  # inside vmap: once for the whole batch, axes shifted
                from . import batching
                return batching.dispatch(self, args, kwargs)
        tensors = [a for a in args if isinstance(a, Tensor)]
        any_traced = False
        for t in tensors:
            if t._impl.is_traced:
                any_traced = True
                break
        adapted = self.adapt_kwargs(args, kwargs, 0)
        shapes, dtypes, devices = self.compute_physical_shape(args, adapted, None)
        outs = []
        impls = []
        for shape, dtype, device in zip(shapes, dtypes, devices):
            impl = TensorImpl(shape, dtype, device, is_traced=any_traced)
            impls.append(impl)
            outs.append(Tensor(impl=impl))
        self._setup_output_refs(outs, args, kwargs)
        if config.EAGER_MAX_GRAPH and not config.TRACING:
            from ..core.engine import GRAPH
            GRAPH.evaluate(*outs)
        return outs

    def _setup_output_refs(self, outputs: list, args: Any, logical_kwargs: dict | None,
                           op_hash=None) -> None:
        impls = [o._impl for o in outputs]
        stored = tuple(a._impl if isinstance(a, Tensor) else a for a in args)
        tree_def = _LEAF_DEF if len(impls) == 1 else PyTreeDef(list, None, (_LEAF_DEF,) * len(impls), len(impls))
        node = OpNode(tuple(impls), tree_def, self, stored, logical_kwargs or None,
                      _freeze_kwargs(logical_kwargs))
        for i, impl in enumerate(impls):
            impl.output_refs = node
            impl.output_index = i

    @staticmethod
    def _broadcast_shapes(s1, s2) -> tuple[int, ...]:
        s1, s2 = tuple(s1), tuple(s2)
        if len(s1) > len(s2):
            s2 = (1,) * (len(s1) - len(s2)) + s2
        elif len(s2) > len(s1):
            s1 = (1,) * (len(s2) - len(s1)) + s1
        out = []
        for d1, d2 in zip(s1, s2):
            if d1 == d2:
                out.append(d1)
            elif d1 == 1:
                out.append(d2)
            elif d2 == 1:
                out.append(d1)
            else:
                raise ValueError(f"Cannot broadcast shapes {s1} and {s2}")
        return tuple(out)

    def __repr__(self) -> str:
        return f"{type(self).__name__}(name={self.name!r})"


class BinaryOperation(Operation):
    """Elementwise binary op with numpy broadcasting made explicit before the
    op runs (base.py:639-652)."""

    #: comparison ops override this to produce bool
    result_dtype: DType | None = None

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x, y = args[0], args[1]
        dtype = self.result_dtype or promote(x.dtype, y.dtype)
        return [tuple(x.shape)], [dtype], [x.device]

    def __call__(self, args: OpArgs, kwargs: OpKwargs) -> OpResult:
        from . import view as view_ops

        x, y = args[0], args[1]
        if not isinstance(x, Tensor):
            x = ensure_tensor(x, y if isinstance(y, Tensor) else None)
        if not isinstance(y, Tensor):
            y = ensure_tensor(y, x)
        target = self._broadcast_shapes(x.shape, y.shape)
        if x.shape != target:
            x = view_ops.broadcast_to(x, target)
        if y.shape != target:
            y = view_ops.broadcast_to(y, target)
        return super().__call__([x, y], kwargs)


class AxisOp(Operation):
    """Ops that take ``axis`` keyword arguments (base.py:694-760)."""

    @staticmethod
    def _norm_axis(axis: int, rank: int) -> int:
        a = axis + rank if axis < 0 else axis
        if not 0 <= a < max(rank, 1):
            raise ValueError(f"axis {axis} out of range for rank {rank}")
        return a


class ReduceOperation(AxisOp):
    """Single-axis reduction; the kernel always keeps the reduced dim (size 1)
    and ``keepdims=False`` is a separate squeeze (reduction.py:559-581)."""

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        axis = self._norm_axis(kwargs.get("axis", -1), len(x.shape))
        shape = tuple(1 if i == axis else d for i, d in enumerate(x.shape))
        return [shape], [x.dtype], [x.device]


class UnaryOperation(Operation):
    """Elementwise unary op.  Subclasses may define ``_derivative(primal, output)``
    and inherit ``vjp = cotangent * derivative`` (base.py:914-949)."""

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(x.shape)], [x.dtype], [x.device]

    def _derivative(self, primal: Tensor, output: Tensor) -> Tensor:
        raise NotImplementedError(f"'{self.name}' defines neither _derivative nor vjp_rule")

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .binary import mul
        return [mul(cotangents[0], self._derivative(primals[0], outputs[0]))]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        from .binary import mul
        return [mul(tangents[0], self._derivative(primals[0], outputs[0]))]


class ShapeOp(Operation):
    """View / layout ops (base.py:990-1088)."""


class CreationOperation(Operation):
    """Ops without tensor inputs (base.py:1091-1205)."""

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return []
