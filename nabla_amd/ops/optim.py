"""Optimizer steps over a whole list of parameters as one operation.

The reference maps ``adamw_step`` / ``sgd_step`` over the leaves of the parameter pytree
(nabla/nn/optim/functional.py:14-39, 116-162; optimizer.py:242-305): a dozen tensor ops per leaf.
``adamw_multi`` and ``sgd_multi`` take the leaves as one argument list and lower to one launch
that streams every parameter, gradient and state tensor once.  The step counter of AdamW can be
a 0-d float32 tensor, so that the same plan serves every step.

Differentiating through an optimizer step (meta-gradients) goes back to the per-leaf arithmetic.
"""
from __future__ import annotations

from typing import Sequence

from ..backend import ir
from ..core.dtype import DType
from ..core.tensor import Tensor
from .base import Operation

UPDATE_DTYPES = (DType.float32, DType.bfloat16)


def _unpack(args, per: int, n: int):
    return [list(args[i * per:(i + 1) * per]) for i in range(n)]


class AdamWMultiOp(Operation):
    """(p_0, g_0, m_0, v_0, p_1, ..., [step]) -> (p'_0, m'_0, v'_0, p'_1, ...)."""

    multiple_results = True

    @property
    def name(self) -> str:
        return "adamw_multi"

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        groups = _unpack(args, 4, kwargs["n"])
        shapes = [tuple(g[0].shape) for g in groups for _ in range(3)]
        return shapes, [g[0].dtype for g in groups for _ in range(3)], [g[0].device for g in groups for _ in range(3)]

    def kernel(self, args, kwargs):
        n = kwargs["n"]
        groups = _unpack(args, 4, n)
        step = args[4 * n] if kwargs["step"] is None else kwargs["step"]
        hyper = {k: kwargs[k] for k in ("lr", "beta1", "beta2", "eps", "weight_decay", "bias_correction")}
        return ir.adamw_multi([g[0] for g in groups], [g[1] for g in groups], [g[2] for g in groups],
                              [g[3] for g in groups], step, **hyper)

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from ..nn.optim.functional import adamw_step
        from ..transforms.vjp import vjp
        n = kwargs["n"]
        step = primals[4 * n] if kwargs["step"] is None else kwargs["step"]
        hyper = {k: kwargs[k] for k in ("lr", "beta1", "beta2", "eps", "weight_decay", "bias_correction")}
        grads: list = []
        for i, (p, g, m, v) in enumerate(_unpack(primals, 4, n)):
            _, pull = vjp(lambda p, g, m, v: adamw_step(p, g, m, v, step, **hyper), p, g, m, v)
            grads += list(pull(tuple(cotangents[3 * i:3 * i + 3])))
        return grads + ([None] if kwargs["step"] is None else [])


class SGDMultiOp(Operation):
    """(p_0, g_0, [buf_0], p_1, ...) -> (p'_0, [buf'_0], p'_1, ...); buffers with momentum only."""

    multiple_results = True

    @property
    def name(self) -> str:
        return "sgd_multi"

    @staticmethod
    def _widths(kwargs):
        return (3, 2) if kwargs["momentum"] != 0.0 else (2, 1)

    def compute_physical_shape(self, args, kwargs, output_sharding=None):
        per_in, per_out = self._widths(kwargs)
        groups = _unpack(args, per_in, kwargs["n"])
        return ([tuple(g[0].shape) for g in groups for _ in range(per_out)],
                [g[0].dtype for g in groups for _ in range(per_out)],
                [g[0].device for g in groups for _ in range(per_out)])

    def kernel(self, args, kwargs):
        per_in, _ = self._widths(kwargs)
        groups = _unpack(args, per_in, kwargs["n"])
        bufs = [g[2] for g in groups] if per_in == 3 else None
        return ir.sgd_multi([g[0] for g in groups], [g[1] for g in groups], bufs, lr=kwargs["lr"],
                            momentum=kwargs["momentum"], weight_decay=kwargs["weight_decay"])

    def vjp_rule(self, primals, cotangents, outputs, kwargs):
        from ..nn.optim.functional import sgd_step
        from ..transforms.vjp import vjp
        per_in, per_out = self._widths(kwargs)
        hyper = {k: kwargs[k] for k in ("lr", "momentum", "weight_decay")}
        grads: list = []
        for i, group in enumerate(_unpack(primals, per_in, kwargs["n"])):
            if per_in == 3:
                _, pull = vjp(lambda p, g, b: sgd_step(p, g, b, **hyper), *group)
                grads += list(pull(tuple(cotangents[2 * i:2 * i + 2])))
            else:
                _, pull = vjp(lambda p, g: sgd_step(p, g, None, **hyper)[0], *group)
                grads += list(pull(cotangents[i]))
        return grads


_adamw_multi_op = AdamWMultiOp()
_sgd_multi_op = SGDMultiOp()


def _check_groups(who: str, groups: Sequence[Sequence[Tensor]]) -> None:
    dtype = groups[0][0].dtype
    if dtype not in UPDATE_DTYPES:
        raise TypeError(f"{who}: float32 or bfloat16 parameters, got {dtype}")
    for g in groups:
        for t in g:
            if t.dtype is not dtype or tuple(t.shape) != tuple(g[0].shape):
                raise ValueError(f"{who}: the tensors of one call share a dtype, and those of one "
                                 f"parameter a shape; got {tuple(t.shape)} {t.dtype} beside "
                                 f"{tuple(g[0].shape)} {dtype}")


def adamw_multi(params: Sequence[Tensor], grads: Sequence[Tensor], ms: Sequence[Tensor],
                vs: Sequence[Tensor], step, *, lr: float, beta1: float = 0.9, beta2: float = 0.999,
                eps: float = 1e-8, weight_decay: float = 0.0, bias_correction: bool = True):
    """One AdamW step (decoupled decay) for a list of parameters of one dtype: returns the lists
    ``(new_params, new_ms, new_vs)``.  ``step`` is the number of this step, from 1: a Python number
    or a tensor holding one value."""
    groups = [list(g) for g in zip(params, grads, ms, vs)]
    if not groups:
        return [], [], []
    _check_groups("adamw_multi", groups)
    kwargs = {"n": len(groups), "lr": float(lr), "beta1": float(beta1), "beta2": float(beta2),
              "eps": float(eps), "weight_decay": float(weight_decay),
              "bias_correction": bool(bias_correction), "step": None}
    args = [t for g in groups for t in g]
    if isinstance(step, Tensor):
        from .unary import cast
        from .view import reshape
        if step.dtype is not DType.float32:
            step = cast(step, DType.float32)
        args.append(step if tuple(step.shape) == () else reshape(step, ()))
    else:
        kwargs["step"] = float(step)
    out = _adamw_multi_op(args, kwargs)
    return out[0::3], out[1::3], out[2::3]


def sgd_multi(params: Sequence[Tensor], grads: Sequence[Tensor], bufs: Sequence[Tensor] | None = None,
              *, lr: float, momentum: float = 0.0, weight_decay: float = 0.0):
    """One SGD step for a list of parameters of one dtype: ``(new_params, new_bufs)``; the second
    is ``None`` without momentum."""
    with_mom = float(momentum) != 0.0
    if with_mom and bufs is None:
        raise ValueError("sgd_multi: momentum needs the momentum buffers")
    groups = [list(g) for g in (zip(params, grads, bufs) if with_mom else zip(params, grads))]
    if not groups:
        return [], ([] if with_mom else None)
    _check_groups("sgd_multi", groups)
    kwargs = {"n": len(groups), "lr": float(lr), "momentum": float(momentum),
              "weight_decay": float(weight_decay)}
    out = _sgd_multi_op([t for g in groups for t in g], kwargs)
    if with_mom:
        return out[0::2], out[1::2]
    return list(out), None
