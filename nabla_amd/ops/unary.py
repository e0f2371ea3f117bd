"""Unary elementwise ops, softmax / logsoftmax and cast.

Mirrors nabla/ops/unary.py: ReluOp 20-54, sigmoid, tanh, ExpOp 97-110, NegOp
113-138, abs, _SoftmaxNativeOp 192-230, LogOp 233-250, SqrtOp 253-268, ErfOp
386-405, RsqrtOp 487-501, GeluOp 567-595 (exact erf form), _LogSoftmaxNativeOp
598-632, CastOp 660-697, public softmax / logsoftmax 820-871.
"""
from __future__ import annotations

import math

from ..backend import ir
from ..core.dtype import DType
from ..core.tensor import Tensor
from .base import AxisOp, Operation, UnaryOperation, ensure_tensor


def _ew1(fn: str):
    def kernel(self, args, kwargs):
        return [ir.ew(fn, args[0])]
    return kernel


class ReluOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "relu"

    kernel = _ew1("relu")

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # d relu / dx = (x > 0): zero at x == 0 (unary.py:31-42)
        from .comparison import greater
        from .control_flow import where
        from .creation import zeros_like
        # (the zero is a creation op, not a scalar leaf: the planner sees the comparison's constant
        # and can let it read relu's result where the pre-activation is not stored)
        mask = greater(primals[0], zeros_like(primals[0]))
        return [where(mask, cotangents[0], zeros_like(cotangents[0]))]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        from .binary import mul
        from .comparison import greater
        from .creation import zeros_like
        return [mul(tangents[0], greater(primals[0], zeros_like(primals[0])))]


class ExpOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "exp"

    kernel = _ew1("exp")

    def _derivative(self, primal, output):
        return output


class NegOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "neg"

    kernel = _ew1("neg")

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return [neg(cotangents[0])]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [neg(tangents[0])]


class AbsOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "abs"

    kernel = _ew1("abs")

    def _derivative(self, primal, output):
        from .binary import sub
        from .comparison import greater
        x = primal
        return sub(cast(greater(x, 0.0), x.dtype), cast(greater(neg(x), 0.0), x.dtype))


class LogOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "log"

    kernel = _ew1("log")

    def _derivative(self, primal, output):
        from .binary import div
        return div(1.0, primal)


class SqrtOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "sqrt"

    kernel = _ew1("sqrt")

    def _derivative(self, primal, output):
        from .binary import div, mul
        return div(0.5, output)


class RsqrtOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "rsqrt"

    kernel = _ew1("rsqrt")

    def _derivative(self, primal, output):
        # d x^(-1/2) = -0.5 * out^3
        from .binary import mul
        return mul(-0.5, mul(output, mul(output, output)))


class ErfOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "erf"

    kernel = _ew1("erf")

    def _derivative(self, primal, output):
        from .binary import mul
        x = primal
        return mul(2.0 / math.sqrt(math.pi), exp(neg(mul(x, x))))


class TanhOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "tanh"

    kernel = _ew1("tanh")

    def _derivative(self, primal, output):
        from .binary import mul, sub
        return sub(1.0, mul(output, output))


class SinOp(UnaryOperation):
    """unary.py (SinOp): derivative cos(x)."""

    @property
    def name(self) -> str:
        return "sin"

    kernel = _ew1("sin")

    def _derivative(self, primal, output):
        return cos(primal)


class CosOp(UnaryOperation):
    """unary.py (CosOp): derivative -sin(x)."""

    @property
    def name(self) -> str:
        return "cos"

    kernel = _ew1("cos")

    def _derivative(self, primal, output):
        return neg(sin(primal))


class SigmoidOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "sigmoid"

    kernel = _ew1("sigmoid")

    def _derivative(self, primal, output):
        from .binary import mul, sub
        return mul(output, sub(1.0, output))


class SiluOp(UnaryOperation):
    """``x * sigmoid(x)`` (unary.py:504-520); emitted as those two primitive ops, which the
    lowering fuses with their neighbours."""

    @property
    def name(self) -> str:
        return "silu"

    def kernel(self, args, kwargs):
        return [ir.ew("mul", args[0], ir.ew("sigmoid", args[0]))]

    def _derivative(self, primal, output):
        # sigmoid(x) + silu(x) * (1 - sigmoid(x))
        from .binary import add, mul, sub
        s = sigmoid(primal)
        return add(s, mul(output, sub(1.0, s)))


class GeluOp(UnaryOperation):
    """Exact GELU ``x * Phi(x)``; ``approximate="tanh"`` selects the tanh form."""

    @property
    def name(self) -> str:
        return "gelu"

    def kernel(self, args, kwargs):
        x = args[0]
        approx = kwargs.get("approximate", "none")
        if approx is True:
            approx = "tanh"
        elif approx is False:
            approx = "none"
        if approx == "none":
            return [ir.ew("gelu", x)]
        if approx != "tanh":
            raise ValueError(f"gelu: unknown approximation '{approx}'")
        c = math.sqrt(2.0 / math.pi)
        x3 = ir.ew("mul", ir.ew("mul", x, x), x)
        inner = ir.ew("mul", ir.ew("add", x, ir.ew("mul", x3, 0.044715)), c)
        return [ir.ew("mul", ir.ew("mul", x, 0.5), ir.ew("add", ir.ew("tanh", inner), 1.0))]

    def _derivative(self, primal, output):
        # GELU'(x) = cdf(x) + x * pdf(x)  (unary.py:583-595) as ONE elementwise function of x:
        # its erf and its density share one exponential, and a GELU of the same x in the same
        # kernel shares them too
        return _gelu_grad_op([primal], {})[0]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .. import config
        approx = kwargs.get("approximate", "none")
        if config.GELU_BACKWARD_FROM_INPUT and approx in ("none", False):
            return [_gelu_backward_op([primals[0], cotangents[0]], {})[0]]
        return super().vjp_rule(primals, cotangents, outputs, kwargs)


class GeluGradOp(UnaryOperation):
    """``Phi(x) + x * phi(x)``, the derivative of the exact GELU."""

    @property
    def name(self) -> str:
        return "gelu_grad"

    kernel = _ew1("dgelu")

    def _derivative(self, primal, output):
        # d/dx [Phi + x phi] = phi * (2 - x^2)
        from .binary import div, mul, sub
        x = primal
        pdf = div(exp(neg(div(mul(x, x), 2.0))), math.sqrt(2.0 * math.pi))
        return mul(pdf, sub(2.0, mul(x, x)))


class GeluBackwardOp(Operation):
    """(x, g) -> g * GELU'(x), with the derivative computed where the cotangent is: the forward
    kernel then writes the activation only, not a second tensor of the same size that holds the
    derivative until the backward pass (the pre-activation is kept instead, which exists
    anyway)."""

    @property
    def name(self) -> str:
        return "gelu_backward"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(x.shape)], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        x, g = args
        return [ir.ew("mul", g, ir.ew("dgelu", ir.pin_after(x, g)))]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .binary import mul
        x, g = primals
        d1 = _gelu_grad_op([x], {})[0]
        d2 = _gelu_grad_op._derivative(x, None)
        return [mul(cotangents[0], mul(g, d2)), mul(cotangents[0], d1)]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        from .binary import add, mul
        x, g = primals
        d1 = _gelu_grad_op([x], {})[0]
        d2 = _gelu_grad_op._derivative(x, None)
        return [add(mul(tangents[0], mul(g, d2)), mul(tangents[1], d1))]


def _softmax_ir(x, axis: int, log: bool):
    """max / sub / exp / sum (/ div | log, sub) along ``axis``; the planner fuses
    the chain into one row kernel."""
    r = x.rank
    axis = axis + r if axis < 0 else axis
    perm = None
    if axis != r - 1:
        perm = list(range(r))
        perm[axis], perm[-1] = perm[-1], perm[axis]
        x = ir.permute(x, perm)
    m = ir.reduce("max", x, -1)
    sh = ir.ew("sub", x, ir.broadcast_to(m, x.shape))
    e = ir.ew("exp", sh)
    s = ir.reduce("sum", e, -1)
    if log:
        out = ir.ew("sub", sh, ir.broadcast_to(ir.ew("log", s), x.shape))
    else:
        out = ir.ew("div", e, ir.broadcast_to(s, x.shape))
    if perm is not None:
        out = ir.permute(out, perm)
    return out


class _SoftmaxNativeOp(AxisOp, UnaryOperation):
    @property
    def name(self) -> str:
        return "softmax"

    def kernel(self, args, kwargs):
        return [_softmax_ir(args[0], kwargs.get("axis", -1), log=False)]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # s * (g - sum(g * s))  (unary.py:206-218)
        from .binary import mul, sub
        from .reduction import reduce_sum
        axis = kwargs.get("axis", -1)
        out, g = outputs[0], cotangents[0]
        s = reduce_sum(mul(g, out), axis=axis, keepdims=True)
        return [mul(out, sub(g, s))]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        from .binary import mul, sub
        from .reduction import reduce_sum
        axis = kwargs.get("axis", -1)
        out, t = outputs[0], tangents[0]
        s = reduce_sum(mul(t, out), axis=axis, keepdims=True)
        return [mul(out, sub(t, s))]


class _LogSoftmaxNativeOp(AxisOp, UnaryOperation):
    @property
    def name(self) -> str:
        return "logsoftmax"

    def kernel(self, args, kwargs):
        return [_softmax_ir(args[0], kwargs.get("axis", -1), log=True)]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # g - exp(out) * sum(g)  (unary.py:609-621)
        from .binary import mul, sub
        from .reduction import reduce_sum
        axis = kwargs.get("axis", -1)
        out, g = outputs[0], cotangents[0]
        return [sub(g, mul(exp(out), reduce_sum(g, axis=axis, keepdims=True)))]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        from .binary import mul, sub
        from .reduction import reduce_sum
        axis = kwargs.get("axis", -1)
        out, t = outputs[0], tangents[0]
        return [sub(t, reduce_sum(mul(exp(out), t), axis=axis, keepdims=True))]


class CastOp(UnaryOperation):
    @property
    def name(self) -> str:
        return "cast"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(x.shape)], [kwargs["dtype"]], [x.device]

    def kernel(self, args, kwargs):
        return [ir.cast(args[0], kwargs["dtype"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        x = primals[0]
        if not x.dtype.is_float():
            return [None]
        return [cast(cotangents[0], x.dtype)]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [cast(tangents[0], kwargs["dtype"])]


_relu_op, _exp_op, _neg_op, _abs_op = ReluOp(), ExpOp(), NegOp(), AbsOp()
_log_op, _sqrt_op, _rsqrt_op, _erf_op = LogOp(), SqrtOp(), RsqrtOp(), ErfOp()
_tanh_op, _sigmoid_op, _gelu_op, _cast_op = TanhOp(), SigmoidOp(), GeluOp(), CastOp()
_silu_op = SiluOp()
_gelu_grad_op = GeluGradOp()
_gelu_backward_op = GeluBackwardOp()
_softmax_native, _logsoftmax_native = _SoftmaxNativeOp(), _LogSoftmaxNativeOp()


def relu(x) -> Tensor:
    return _relu_op([ensure_tensor(x)], {})[0]


def exp(x) -> Tensor:
    return _exp_op([ensure_tensor(x)], {})[0]


def neg(x) -> Tensor:
    return _neg_op([ensure_tensor(x)], {})[0]


def abs(x) -> Tensor:  # noqa: A001
    return _abs_op([ensure_tensor(x)], {})[0]


def log(x) -> Tensor:
    return _log_op([ensure_tensor(x)], {})[0]


def sqrt(x) -> Tensor:
    return _sqrt_op([ensure_tensor(x)], {})[0]


def rsqrt(x) -> Tensor:
    return _rsqrt_op([ensure_tensor(x)], {})[0]


def erf(x) -> Tensor:
    return _erf_op([ensure_tensor(x)], {})[0]


_sin_op = SinOp()
_cos_op = CosOp()


def sin(x) -> Tensor:
    return _sin_op([ensure_tensor(x)], {})[0]


def cos(x) -> Tensor:
    return _cos_op([ensure_tensor(x)], {})[0]


def tanh(x) -> Tensor:
    return _tanh_op([ensure_tensor(x)], {})[0]


def sigmoid(x) -> Tensor:
    return _sigmoid_op([ensure_tensor(x)], {})[0]


def silu(x) -> Tensor:
    return _silu_op([ensure_tensor(x)], {})[0]


def gelu(x, approximate: str = "none") -> Tensor:
    kw = {} if approximate in ("none", False) else {"approximate": approximate}
    return _gelu_op([ensure_tensor(x)], kw)[0]


def cast(x, dtype: DType | None = None) -> Tensor:
    x = ensure_tensor(x)
    if dtype is None or dtype is x.dtype:
        return x
    return _cast_op([x], {"dtype": dtype})[0]


def softmax(x, axis: int = -1) -> Tensor:
    return _softmax_native([ensure_tensor(x)], {"axis": axis})[0]


def logsoftmax(x, axis: int = -1) -> Tensor:
    return _logsoftmax_native([ensure_tensor(x)], {"axis": axis})[0]
