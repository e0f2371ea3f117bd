"""``where`` (nabla/ops/control_flow.py:21-141).  cond / while_loop / scan need
region ops and are outside this backend's op set."""
from __future__ import annotations

from ..backend import ir
from ..core.dtype import DType, promote
from ..core.tensor import Tensor
from .base import Operation, ensure_tensor


class WhereOp(Operation):
    @property
    def name(self) -> str:
        return "where"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        c, x, y = args
        return [tuple(x.shape)], [promote(x.dtype, y.dtype)], [x.device]

    def kernel(self, args, kwargs):
        c, x, y = args
        dt = promote(x.dtype, y.dtype)
        return [ir.ew("where", c, ir.cast(x, dt), ir.cast(y, dt), dtype=dt)]

    def __call__(self, args, kwargs):
        from . import view as view_ops
        c, x, y = args
        tensors = [t for t in (x, y, c) if isinstance(t, Tensor)]
        like = tensors[0]
        x = ensure_tensor(x, like)
        y = ensure_tensor(y, x)
        c = ensure_tensor(c)
        target = self._broadcast_shapes(self._broadcast_shapes(c.shape, x.shape), y.shape)
        c, x, y = (view_ops.broadcast_to(t, target) for t in (c, x, y))
        return super().__call__([c, x, y], kwargs)

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # the condition is not differentiable (control_flow.py:122-131)
        from .creation import zeros_like
        c = primals[0]
        g = cotangents[0]
        z = zeros_like(g)
        return [None, where(c, g, z), where(c, z, g)]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [where(primals[0], tangents[1], tangents[2])]


_where_op = WhereOp()


def where(condition, x, y) -> Tensor:
    return _where_op([condition, x, y], {})[0]
