"""2-D convolution, NHWC x HWIO (nabla/ops/convolution.py).

``Conv2DOp`` mirrors 220-416.  Its VJP has the meaning of 309-392 -- input
gradient = transposed convolution of the cotangent, cropped by the padding;
filter gradient = correlation of the padded input with the cotangent; bias
gradient = sum over N, H, W -- but emits the two dedicated gradient kernels
instead of the conv2d_transpose + pad + slice and permute + conv2d + permute
sequences.  Validation and its messages follow 602-696.
"""
from __future__ import annotations

from typing import Any

from ..backend import ir
from ..core.tensor import Tensor
from .base import Operation, ensure_tensor


# What each window argument may look like and which values it may hold.  One table drives the
# expansion to per-side integers and the range checks of both public functions; the wording of
# the errors is the reference's (convolution.py:602-696), which user code may match on.
_PADDING_FORMS = "padding must be int, (pad_h, pad_w), or (pad_top, pad_bottom, pad_left, pad_right)"
_WINDOW_ARGS = {
    # name: (entries after expansion, smallest allowed value)
    "stride": (2, 1),
    "dilation": (2, 1),
    "padding": (4, 0),
    "output_paddings": (2, 0),
    "kernel_size": (2, 1),
}


def _expand_window_arg(name: str, value) -> tuple[int, ...]:
    """An int or a short sequence -> one integer per side, checked against the argument's range."""
    width, lowest = _WINDOW_ARGS[name]
    seq = None
    if isinstance(value, int):
        seq = (value,) * width
    elif isinstance(value, (tuple, list)):
        if len(value) == width:
            seq = tuple(value)
        elif width == 4 and len(value) == 2:  # (pad_h, pad_w): both sides of an axis alike
            seq = (value[0], value[0], value[1], value[1])
    if seq is None:
        raise ValueError(_PADDING_FORMS if width == 4 else
                         f"{name} must be int or tuple/list of length 2, got {value}")
    out = tuple(int(v) for v in seq)
    if min(out) < lowest:
        bound = "> 0" if lowest == 1 else ">= 0"
        raise ValueError(f"{name} values must be {bound}, got {out}")
    return out


def _window(**given) -> dict[str, tuple[int, ...]]:
    """Expand every window argument first, then range-check in the order given (the order in
    which the reference reports a call that is wrong in two ways)."""
    shapes = {}
    for name, value in given.items():  # malformed arguments are reported before out-of-range ones
        width = _WINDOW_ARGS[name][0]
        ok = isinstance(value, int) or (isinstance(value, (tuple, list)) and
                                        (len(value) == width or (width == 4 and len(value) == 2)))
        if not ok:
            _expand_window_arg(name, value)  # raises with the form message
        shapes[name] = value
    return {name: _expand_window_arg(name, value) for name, value in shapes.items()}


def _check_bias(who: str, bias, c_out: int) -> None:
    if bias is None:
        return
    if len(bias.shape) != 1:
        raise ValueError(f"{who} bias must be rank-1 [C_out], got shape={tuple(bias.shape)}")
    if bias.shape[0] != c_out:
        raise ValueError(f"{who} bias size ({bias.shape[0]}) must match filter C_out ({c_out})")


def _rank4_operands(who: str, x, filter, bias):  # noqa: A002
    x, filter = ensure_tensor(x), ensure_tensor(filter)
    if len(x.shape) != 4 or len(filter.shape) != 4:
        raise ValueError(f"{who} expects rank-4 tensors, got x={tuple(x.shape)}, "
                         f"filter={tuple(filter.shape)}")
    return x, filter, (None if bias is None else ensure_tensor(bias))


def _out_hw(x_shape, w_shape, stride, padding) -> tuple[int, int]:
    ho = ir.conv_out_size(x_shape[1], w_shape[0], stride[0], padding[0], padding[1])
    wo = ir.conv_out_size(x_shape[2], w_shape[1], stride[1], padding[2], padding[3])
    if ho <= 0 or wo <= 0:
        raise ValueError(f"Non-positive conv2d output size H={ho}, W={wo}")
    return ho, wo


def _transpose_out_hw(x_shape, w_shape, stride, padding) -> tuple[int, int]:
    """Output size of the transposed convolution with dilation 1 and no output padding
    (convolution.py:140-160)."""
    pt, pb, pl, pr = padding
    ho = (x_shape[1] - 1) * stride[0] - pt - pb + w_shape[0]
    wo = (x_shape[2] - 1) * stride[1] - pl - pr + w_shape[1]
    if ho <= 0 or wo <= 0:
        raise ValueError(f"Non-positive conv2d_transpose output size H={ho}, W={wo}.")
    return ho, wo


class Conv2DOp(Operation):
    @property
    def name(self) -> str:
        return "conv2d"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x, w = args[0], args[1]
        ho, wo = _out_hw(x.shape, w.shape, kwargs["stride"], kwargs["padding"])
        return [(x.shape[0], ho, wo, w.shape[3])], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        x, w = args[0], args[1]
        bias = args[2] if len(args) > 2 else None
        return [ir.conv2d(x, w, bias, kwargs["stride"], kwargs["padding"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from .reduction import reduce_sum
        x, w = primals[0], primals[1]
        g = cotangents[0]
        kw = {"stride": kwargs["stride"], "padding": kwargs["padding"]}
        gx = _conv2d_dgrad_op([g, w], dict(kw, x_shape=tuple(x.shape)))[0]
        gw = _conv2d_wgrad_op([x, g], dict(kw, w_shape=tuple(w.shape)))[0]
        grads = [gx, gw]
        if len(primals) > 2:
            grads.append(reduce_sum(g, axis=[0, 1, 2]))
        return grads


class Conv2DInputGradOp(Operation):
    """dX of conv2d: ``dy`` [N,Ho,Wo,Cout] and ``w`` [R,S,Cin,Cout] -> [N,H,W,Cin]."""

    @property
    def name(self) -> str:
        return "conv2d_input_grad"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        return [tuple(kwargs["x_shape"])], [args[0].dtype], [args[0].device]

    def kernel(self, args, kwargs):
        return [ir.conv2d_dgrad(args[0], args[1], kwargs["x_shape"], kwargs["stride"],
                                kwargs["padding"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        # linear in both operands: d/d(dy) is a forward convolution, d/dw a filter gradient
        dy, w = primals
        g = cotangents[0]
        kw = {"stride": kwargs["stride"], "padding": kwargs["padding"]}
        g_dy = _conv2d_op([g, w], dict(kw))[0]
        g_w = _conv2d_wgrad_op([g, dy], dict(kw, w_shape=tuple(w.shape)))[0]
        return [g_dy, g_w]


class Conv2DFilterGradOp(Operation):
    """dW of conv2d: ``x`` [N,H,W,Cin] and ``dy`` [N,Ho,Wo,Cout] -> [R,S,Cin,Cout]."""

    @property
    def name(self) -> str:
        return "conv2d_filter_grad"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        return [tuple(kwargs["w_shape"])], [args[0].dtype], [args[0].device]

    def kernel(self, args, kwargs):
        return [ir.conv2d_wgrad(args[0], args[1], kwargs["w_shape"], kwargs["stride"],
                                kwargs["padding"])]

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        x, dy = primals
        g = cotangents[0]  # [R,S,Cin,Cout]
        kw = {"stride": kwargs["stride"], "padding": kwargs["padding"]}
        g_x = _conv2d_dgrad_op([dy, g], dict(kw, x_shape=tuple(x.shape)))[0]
        g_dy = _conv2d_op([x, g], dict(kw))[0]
        return [g_x, g_dy]



class Conv2DTransposeOp(Conv2DInputGradOp):
    """``conv2d_transpose`` (nabla/ops/convolution.py:424-566): ``x`` [N,H,W,Cin] and a filter
    [R,S,Cout,Cin] -> [N,Ho,Wo,Cout].  It is the input gradient of ``conv2d`` with the same
    filter read as HWIO, so it runs on the dgrad kernel and inherits its derivative rules
    (dX: a forward convolution of the cotangent; dW: a filter gradient)."""

    @property
    def name(self) -> str:
        return "conv2d_transpose"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        x, w = args[0], args[1]
        ho, wo = _transpose_out_hw(x.shape, w.shape, kwargs["stride"], kwargs["padding"])
        return [(x.shape[0], ho, wo, w.shape[2])], [x.dtype], [x.device]

    def kernel(self, args, kwargs):
        x, w = args[0], args[1]
        ho, wo = _transpose_out_hw(x.shape, w.shape, kwargs["stride"], kwargs["padding"])
        return [ir.conv2d_dgrad(x, w, (x.shape[0], ho, wo, w.shape[2]), kwargs["stride"],
                                kwargs["padding"])]


_conv2d_op = Conv2DOp()
_conv2d_transpose_op = Conv2DTransposeOp()
_conv2d_dgrad_op = Conv2DInputGradOp()
_conv2d_wgrad_op = Conv2DFilterGradOp()


def conv2d(x, filter, *, stride=(1, 1), dilation=(1, 1), padding=(0, 0, 0, 0), groups: int = 1,
           bias=None, input_layout: Any = None, filter_layout: Any = None) -> Tensor:  # noqa: A002
    x, filter, bias_t = _rank4_operands("conv2d", x, filter, bias)
    if input_layout is not None or filter_layout is not None:
        raise ValueError("conv2d currently supports only the default NHWC/RSCF layouts")
    win = _window(stride=stride, dilation=dilation, padding=padding)
    n_groups = int(groups)
    if n_groups <= 0:
        raise ValueError(f"groups must be > 0, got {n_groups}")
    if win["dilation"] != (1, 1):
        raise ValueError("conv2d currently supports only dilation=(1, 1)")
    if n_groups != 1:
        raise ValueError("conv2d grouped mode is not exposed")
    c_in, (_, _, c_in_w, c_out) = x.shape[-1], filter.shape
    if c_in != c_in_w * n_groups:
        raise ValueError(
            f"Input channels ({c_in}) must match filter channels*groups ({c_in_w * n_groups})")
    _check_bias("conv2d", bias_t, c_out)
    operands = [x, filter] + ([bias_t] if bias_t is not None else [])
    return _conv2d_op(operands, {"stride": win["stride"], "padding": win["padding"]})[0]


def conv2d_transpose(x, filter, *, stride=(1, 1), dilation=(1, 1), padding=(0, 0, 0, 0),  # noqa: A002
                     output_paddings=(0, 0), bias=None, input_layout: Any = None,
                     filter_layout: Any = None) -> Tensor:
    """Transposed 2-D convolution (convolution.py:699-787): ``x`` [N,H,W,Cin], ``filter``
    [R,S,Cout,Cin] (channels the other way round than ``conv2d``), optional ``bias`` [Cout].
    The same argument checks and messages as the reference; dilation and output padding other
    than the defaults are rejected, as there (762-763 for the output padding)."""
    x, filter, bias_t = _rank4_operands("conv2d_transpose", x, filter, bias)
    if input_layout is not None or filter_layout is not None:
        raise ValueError("conv2d_transpose currently supports only the default NHWC layouts")
    win = _window(stride=stride, dilation=dilation, padding=padding, output_paddings=output_paddings)
    if win["output_paddings"] != (0, 0):
        raise ValueError("conv2d_transpose currently supports only output_paddings=(0, 0)")
    if win["dilation"] != (1, 1):
        raise ValueError("conv2d_transpose currently supports only dilation=(1, 1)")
    c_in, (_, _, c_out, c_in_w) = x.shape[-1], filter.shape
    if c_in != c_in_w:
        raise ValueError(f"Input channels ({c_in}) must match filter input channels ({c_in_w})")
    _check_bias("conv2d_transpose", bias_t, c_out)
    y = _conv2d_transpose_op([x, filter], {"stride": win["stride"], "padding": win["padding"]})[0]
    return y if bias_t is None else y + bias_t
