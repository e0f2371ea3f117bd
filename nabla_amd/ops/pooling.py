"""max_pool2d and avg_pool2d over NHWC (nabla/ops/pooling.py:53-137, 140-211).

The reference unrolls pooling in Python -- one slice + reduce_max per output
pixel, then stack -- which makes a 32x32 feature map cost hundreds of graph
nodes.  Here it is one op with one kernel each way.  Semantics kept: windows
are clipped at the padded border (111-130), and the gradient follows the
reduce_max tie rule (reduction.py:219-230): every element equal to its
window's maximum receives that window's full cotangent.  avg_pool2d pads with
zeros first and divides every window by kh * kw, padding included (77-110).
"""
from __future__ import annotations

from ..backend import ir
from ..core.tensor import Tensor
from .base import Operation, ensure_tensor
from .convolution import _window


class MaxPool2DOp(Operation):
    @property
    def name(self) -> str:
        return "max_pool2d"

    @staticmethod
    def _out_shape(x_shape, kernel, stride, padding):
        n, h, w, c = x_shape
        ho = (h + padding[0] + padding[1] - kernel[0]) // stride[0] + 1
        wo = (w + padding[2] + padding[3] - kernel[1]) // stride[1] + 1
        if ho <= 0 or wo <= 0:
            raise ValueError(
                f"Non-positive pool2d output size H={ho}, W={wo}. Input={(h, w)}, "
                f"kernel={tuple(kernel)}, stride={tuple(stride)}, padding={tuple(padding)}."
            )
        return (n, ho, wo, c)

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return ([self._out_shape(x.shape, kwargs["kernel_size"], kwargs["stride"], kwargs["padding"])],
                [x.dtype], [x.device])

    def kernel(self, args, kwargs):
        return [ir.maxpool2d(args[0], kwargs["kernel_size"], kwargs["stride"], kwargs["padding"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return [_max_pool2d_grad_op([primals[0], outputs[0], cotangents[0]], dict(kwargs))[0]]

    def jvp_rule(self, primals, tangents, outputs, kwargs):
        return [_window_sum_at_maxima(primals[0], outputs[0], tangents[0], kwargs)]


class MaxPool2DGradOp(Operation):
    @property
    def name(self) -> str:
        return "max_pool2d_grad"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return [tuple(x.shape)], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        x, y, dy = args
        return [ir.maxpool2d_bwd(x, y, dy, kwargs["kernel_size"], kwargs["stride"],
                                 kwargs["padding"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # linear in dy, piecewise constant in x and y
        x, y, _ = primals
        return [None, None, _window_sum_at_maxima(x, y, cotangents[0], kwargs)]


def _window_sum_at_maxima(x: Tensor, y: Tensor, t: Tensor, kwargs) -> Tensor:
    """sum over each window of ``t`` where ``x`` equals the window maximum ``y``: the transpose
    of the max-pool gradient under its tie rule (and so the pool's JVP).  Written with
    reshapes for windows that tile the image (stride == kernel, no padding, extents divisible);
    other windows overlap or are clipped and have no such form here."""
    from .comparison import equal
    from .control_flow import where
    from .creation import zeros_like
    from .reduction import reduce_sum
    from .view import broadcast_to, reshape
    kh, kw = kwargs["kernel_size"]
    n, h, w, c = (int(d) for d in x.shape)
    if tuple(kwargs["stride"]) != (kh, kw) or any(kwargs["padding"]) or h % kh or w % kw:
        raise NotImplementedError(
            "forward mode / second order through max_pool2d needs windows that tile the image "
            "(stride == kernel_size, no padding, extents divisible by the kernel)")
    ho, wo = h // kh, w // kw
    six = (n, ho, kh, wo, kw, c)
    xr, tr = reshape(x, six), reshape(t, six)
    yr = broadcast_to(reshape(y, (n, ho, 1, wo, 1, c)), six)
    picked = where(equal(xr, yr), tr, zeros_like(tr))
    return reshape(reduce_sum(picked, axis=[2, 4], keepdims=True), (n, ho, wo, c))


class AvgPool2DOp(Operation):
    @property
    def name(self) -> str:
        return "avg_pool2d"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x = args[0]
        return ([MaxPool2DOp._out_shape(x.shape, kwargs["kernel_size"], kwargs["stride"],
                                        kwargs["padding"])], [x.dtype], [x.device])

    def kernel(self, args, kwargs):
        return [ir.avgpool2d(args[0], kwargs["kernel_size"], kwargs["stride"], kwargs["padding"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        return [_avg_pool2d_grad_op([cotangents[0]], dict(kwargs, x_shape=tuple(primals[0].shape)))[0]]


class AvgPool2DGradOp(Operation):
    """The transpose of avg_pool2d: cotangent [N,Ho,Wo,C] -> [N,H,W,C]."""

    @property
    def name(self) -> str:
        return "avg_pool2d_grad"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        return [tuple(kwargs["x_shape"])], [args[0].dtype], [args[0].device]

    def kernel(self, args, kwargs):
        return [ir.avgpool2d_bwd(args[0], kwargs["x_shape"], kwargs["kernel_size"], kwargs["stride"],
                                 kwargs["padding"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # linear: the transpose of the transpose is the pooling itself
        kw = {k: kwargs[k] for k in ("kernel_size", "stride", "padding")}
        return [_avg_pool2d_op([cotangents[0]], kw)[0]]


_max_pool2d_op = MaxPool2DOp()
_max_pool2d_grad_op = MaxPool2DGradOp()
_avg_pool2d_op = AvgPool2DOp()
_avg_pool2d_grad_op = AvgPool2DGradOp()


def _pool_args(x, kernel_size, stride, padding, dilation, what: str):
    """The window of a pooling call as per-side integers (a missing stride is the kernel size)."""
    x = ensure_tensor(x)
    if len(x.shape) != 4:
        raise ValueError(f"{what} expects an NHWC rank-4 tensor, got shape {tuple(x.shape)}")
    win = _window(kernel_size=kernel_size, stride=kernel_size if stride is None else stride,
                  padding=padding, dilation=dilation)
    if win["dilation"] != (1, 1):
        raise ValueError("pool2d currently supports only dilation=(1, 1)")
    return x, {"kernel_size": win["kernel_size"], "stride": win["stride"], "padding": win["padding"]}


def avg_pool2d(x, *, kernel_size, stride=None, padding=0, dilation=(1, 1)) -> Tensor:
    x, kw = _pool_args(x, kernel_size, stride, padding, dilation, "avg_pool2d")
    return _avg_pool2d_op([x], kw)[0]


def max_pool2d(x, *, kernel_size, stride=None, padding=0, dilation=(1, 1)) -> Tensor:
    x, kw = _pool_args(x, kernel_size, stride, padding, dilation, "max_pool2d")
    return _max_pool2d_op([x], kw)[0]
