"""Batching rules: how an op call that meets a ``BatchedTensor`` runs once on the whole batch.

The reference gives every tensor a ``batch_dims`` counter and lets each op translate its
logical axes to physical ones (nabla/ops/base.py:294-395 ``adapt_kwargs``,
nabla/ops/view/batch.py, nabla/transforms/vmap.py:153-288).  Here the same translation sits in
one place.  ``Operation.__call__`` hands a call over to :func:`dispatch` when one of its tensor
arguments is batched; the rule for the op's class

* brings every tensor argument to the same number of leading hidden dimensions (a tensor from
  an outer ``vmap`` level gets size-1 dimensions behind its own, an unmapped tensor in front
  of its shape) and broadcasts them to the batch sizes -- views, nothing is copied,
* shifts the axes that the keyword arguments name past the hidden dimensions (negative axes
  count from the end and stay as they are) and puts the batch sizes in front of shapes,
* runs the op on the plain tensors and wraps its results again.

An op without a rule raises :class:`NoBatchRule`; ``vmap`` then maps the function element by
element instead, which is always possible.  Backward passes never come through here: a VJP rule
replays on the plain tensors of the recorded ops, which form a valid program of their own.
"""
from __future__ import annotations

from contextvars import ContextVar
from typing import Any, Callable

from ..core.tensor import BatchedTensor, Tensor


class NoBatchRule(Exception):
    """The op has no batching rule (or not for this combination of arguments)."""


class Done:
    """What a rule returns when it has computed the batched result itself (plain tensors with the
    hidden dimensions in front), as a composition of ops that do have kernels for it."""

    def __init__(self, outs):
        self.outs = list(outs)


# sizes of the hidden dimensions of the vmap calls that are being traced, outermost first
# (per context: two threads that trace at the same time do not see each other's levels)
_LEVELS: ContextVar[tuple[int, ...]] = ContextVar("vmap_levels", default=())


def current_level() -> int:
    return len(_LEVELS.get())


def level_sizes() -> tuple[int, ...]:
    return _LEVELS.get()


def push_level(size: int) -> None:
    _LEVELS.set(_LEVELS.get() + (int(size),))


def pop_level() -> None:
    _LEVELS.set(_LEVELS.get()[:-1])


def plain(t: Tensor) -> Tensor:
    return t.physical() if isinstance(t, BatchedTensor) else t


def batch_dims_of(t: Any) -> int:
    return t._bd if isinstance(t, BatchedTensor) else 0


def lift(t: Tensor, bd: int, sizes: tuple[int, ...], logical_rank: int | None = None) -> Tensor:
    """``t`` as a plain tensor of shape ``sizes + (1,) * pad + t.shape``: hidden dimensions it
    does not have are size-1 dimensions broadcast to ``sizes``; ``logical_rank`` pads the
    element's own shape with leading 1s (numpy alignment of operands of different rank)."""
    from . import view

    own = batch_dims_of(t)
    phys = plain(t)
    lshape = tuple(phys.shape[own:])
    pad = 0 if logical_rank is None else logical_rank - len(lshape)
    if pad < 0:
        raise NoBatchRule("operand rank exceeds the result's")
    have = tuple(phys.shape[:own]) + (1,) * (bd - own)
    want_shape = have + (1,) * pad + lshape
    if tuple(phys.shape) != want_shape:
        phys = view.reshape(phys, want_shape)
    full = tuple(sizes) + (1,) * pad + lshape
    if want_shape != full:
        phys = view.broadcast_to(phys, full)
    return phys


def _shift(axis: int, bd: int) -> int:
    return axis if axis < 0 else axis + bd


# ------------------------------------------------------------------------------ rules
# rule(op, args, kwargs, bd, sizes) -> (plain args, physical kwargs[, post]); ``post`` turns the
# op's plain results into plain tensors with the hidden dimensions in front
def _rule_same_shape(op, args, kwargs, bd, sizes):
    """Elementwise ops whose operands already have one (logical) shape, reductions and other
    ops that name at most an ``axis``: lift everything, shift the axis."""
    out = [lift(a, bd, sizes) if isinstance(a, Tensor) else a for a in args]
    kw = dict(kwargs)
    if isinstance(kw.get("axis"), int):
        kw["axis"] = _shift(kw["axis"], bd)
    return out, kw


def _rule_broadcast_to(op, args, kwargs, bd, sizes):
    shape = tuple(kwargs["shape"])
    x = lift(args[0], bd, sizes, logical_rank=len(shape))
    return [x], dict(kwargs, shape=tuple(sizes) + shape)


def _rule_reshape(op, args, kwargs, bd, sizes):
    return [lift(args[0], bd, sizes)], dict(kwargs, shape=tuple(sizes) + tuple(kwargs["shape"]))


def _rule_permute(op, args, kwargs, bd, sizes):
    order = [int(o) for o in kwargs["order"]]
    rank = len(order)
    order = [o + rank if o < 0 else o for o in order]
    return [lift(args[0], bd, sizes)], dict(kwargs, order=tuple(range(bd)) + tuple(o + bd for o in order))


def _rule_slice(op, args, kwargs, bd, sizes):
    out = [lift(a, bd, sizes) if isinstance(a, Tensor) else a for a in args]
    return out, dict(kwargs, start=(0,) * bd + tuple(kwargs["start"]),
                     size=tuple(sizes) + tuple(kwargs["size"]))


def _rule_pad(op, args, kwargs, bd, sizes):
    pads = tuple((int(a), int(b)) for a, b in kwargs["paddings"])
    return [lift(args[0], bd, sizes)], dict(kwargs, paddings=((0, 0),) * bd + pads)


def _rule_layer_norm(op, args, kwargs, bd, sizes):
    # the statistics are per row either way; weight and bias are vectors over the last axis and
    # must be the same for every element of the batch
    if any(isinstance(a, BatchedTensor) for a in args[1:]):
        raise NoBatchRule("layer_norm with mapped weight or bias")
    return [lift(args[0], bd, sizes)] + list(args[1:]), dict(kwargs)


def _fold(t: Tensor, bd: int) -> Tensor:
    """The hidden dimensions and the first logical one as one dimension (ops whose kernels are
    written for a fixed rank with a leading batch: images, attention heads)."""
    from . import view
    shape = tuple(t.shape)
    n = 1
    for d in shape[:bd + 1]:
        n *= d
    return view.reshape(t, (n,) + shape[bd + 1:])


def _unfold(sizes: tuple[int, ...]):
    def post(outs):
        from . import view
        return [view.reshape(o, tuple(sizes) + (o.shape[0] // _prod(sizes),) + tuple(o.shape[1:]))
                for o in outs]
    return post


def _prod(dims) -> int:
    n = 1
    for d in dims:
        n *= d
    return n


def _rule_fold_leading(op, args, kwargs, bd, sizes):
    """Pooling windows and fused attention: every tensor argument has the element's leading batch
    axis; the hidden dimensions join it."""
    out = [_fold(lift(a, bd, sizes), bd) if isinstance(a, Tensor) else a for a in args]
    return out, dict(kwargs), _unfold(sizes)


def _rule_conv(op, args, kwargs, bd, sizes):
    if isinstance(args[1], BatchedTensor):
        return _conv_with_a_filter_per_element(args, kwargs, bd, sizes)
    # the images carry the batch; one filter for all of them.  A bias (third operand) is one
    # vector per output channel for every image
    if any(isinstance(a, BatchedTensor) for a in args[2:]):
        raise NoBatchRule("convolution with a mapped bias")
    return [_fold(lift(args[0], bd, sizes), bd), args[1]] + list(args[2:]), dict(kwargs), _unfold(sizes)


def _conv_with_a_filter_per_element(args, kwargs, bd, sizes):
    """conv2d where every element of the batch has a filter of its own (what per-example
    gradients with respect to a shared filter look like once the filter has been lifted to the
    batch): the kernels take one filter per launch, so the windows are laid out explicitly --
    pad, one shifted view of the images per filter tap, joined along the channel axis -- and
    the contraction over (tap, channel) is ONE batched matrix product whose batch is the hidden
    axis.  Every op of that composition has a kernel and a VJP rule for batched operands, so
    the launches do not grow with the batch, forward or backward.  Unit strides only (a strided
    window is not a view here): other strides leave it to the element-by-element map."""
    from . import binary, view
    x, w = args[0], args[1]
    (sh, sw), (pt, pb, pl, pr) = kwargs["stride"], kwargs["padding"]
    if (sh, sw) != (1, 1):
        raise NoBatchRule("convolution with a mapped filter and a stride")
    xl, wl = lift(x, bd, sizes), lift(w, bd, sizes)
    n, hh, ww, cin = xl.shape[bd:]
    r, s_, _, cout = wl.shape[bd:]
    ho, wo = hh + pt + pb - r + 1, ww + pl + pr - s_ + 1
    lead = tuple(sizes)
    if pt or pb or pl or pr:
        xl = view.pad(xl, [(0, 0)] * (bd + 1) + [(pt, pb), (pl, pr), (0, 0)])
    taps = []
    for i in range(r):
        for j in range(s_):
            start = (0,) * (bd + 1) + (i, j, 0)
            taps.append(view.slice_tensor(xl, start=start, size=lead + (n, ho, wo, cin)))
    cols = taps[0] if len(taps) == 1 else view.concatenate(taps, axis=-1)
    cols = view.reshape(cols, lead + (n * ho * wo, r * s_ * cin))
    y = binary.matmul(cols, view.reshape(wl, lead + (r * s_ * cin, cout)))
    y = view.reshape(y, lead + (n, ho, wo, cout))
    if len(args) > 2:
        b = lift(args[2], bd, sizes)                       # [*sizes, Cout]
        y = binary.add(y, view.reshape(b, lead + (1, 1, 1, cout)))
    return Done([y])


def _rule_gather(op, args, kwargs, bd, sizes):
    """Mapped indices into one table: the gathered axis is replaced by the indices' whole shape,
    hidden dimensions included, which then move to the front."""
    from . import view
    x, idx = args
    if isinstance(x, BatchedTensor):
        return _gather_from_a_table_per_element(x, idx, kwargs, bd, sizes)
    rank = len(x.shape)
    axis = int(kwargs.get("axis", 0))
    axis = axis + rank if axis < 0 else axis

    def post(outs):
        o = outs[0]
        order = list(range(axis, axis + bd)) + [i for i in range(len(o.shape)) if not axis <= i < axis + bd]
        return [view.permute(o, order) if axis else o]

    return [x, lift(idx, bd, sizes)], dict(kwargs, axis=axis), post


def _row_numbers(idx: Tensor, rows: int, bd: int, sizes) -> Tensor:
    """Indices into the rows of one table per batch element -> indices into all the tables laid
    end to end: ``idx + element * rows`` (negative indices wrap once first, as gather does), and
    whatever falls outside its own table goes to the first row past the last table, where the
    kernels' range check sees it."""
    from . import binary, comparison, control_flow, creation, view
    from ..core.dtype import DType
    il = lift(idx, bd, sizes)
    if il.dtype is not DType.int64:
        from .unary import cast
        il = cast(il, DType.int64)
    total = _prod(sizes)
    n = _prod(il.shape[bd:])
    il = view.reshape(il, (total, n))
    const = lambda v: creation.full((total, n), v, dtype=DType.int64)  # (int64 throughout: exact)
    wrapped = control_flow.where(comparison.less(il, const(0)), binary.add(il, const(rows)), il)
    first = view.broadcast_to(view.reshape(creation.arange(0, total * rows, rows, dtype=DType.int64),
                                           (total, 1)), (total, n))
    inside = comparison.logical_and(comparison.greater_equal(wrapped, const(0)),
                                    comparison.less(wrapped, const(rows)))
    outside = control_flow.where(inside, binary.add(wrapped, first), const(total * rows))
    return view.reshape(outside, (total * n,))


def _gather_from_a_table_per_element(x, idx, kwargs, bd, sizes):
    """gather where every element of the batch has a table of its own: the tables are laid end
    to end (a view) and the indices shifted to their own table, so one launch serves the batch.
    Along the first axis only (what an embedding does); other axes are mapped element by element."""
    from . import view
    xl = lift(x, bd, sizes)
    rank = len(xl.shape) - bd
    axis = int(kwargs.get("axis", 0))
    axis = axis + rank if axis < 0 else axis
    if axis != 0:
        raise NoBatchRule("gather from a mapped table along an inner axis")
    rows, rest = xl.shape[bd], tuple(xl.shape[bd + 1:])
    total = _prod(sizes)
    idx_shape = tuple(plain(idx).shape[batch_dims_of(idx):])
    flat_idx = _row_numbers(idx, rows, bd, sizes)
    out = view.gather(view.reshape(xl, (total * rows,) + rest), flat_idx, axis=0)
    return Done([view.reshape(out, tuple(sizes) + idx_shape + rest)])


def _rule_scatter(op, args, kwargs, bd, sizes):
    """scatter with mapped operands: as for a gather from a table per element, the tables are
    laid end to end and the indices shifted; rows of different elements never meet, and within
    one element the updates keep their order, so a row named twice still takes its last update."""
    from . import view
    x, idx, upd = args
    xl, ul = lift(x, bd, sizes), lift(upd, bd, sizes)
    rank = len(xl.shape) - bd
    axis = int(kwargs.get("axis", 0))
    axis = axis + rank if axis < 0 else axis
    if axis != 0:
        raise NoBatchRule("scatter along an inner axis with mapped operands")
    rows, rest = xl.shape[bd], tuple(xl.shape[bd + 1:])
    total = _prod(sizes)
    flat_idx = _row_numbers(idx, rows, bd, sizes)
    n = flat_idx.shape[0] // total
    out = view.scatter(view.reshape(xl, (total * rows,) + rest), flat_idx,
                       view.reshape(ul, (total * n,) + rest), axis=0)
    return Done([view.reshape(out, tuple(sizes) + (rows,) + rest)])


def _rules() -> list[tuple[type, Callable]]:
    from . import (attention, binary, control_flow, convolution, normalization, pooling, unary, view,
                   xent)
    from .base import BinaryOperation, ReduceOperation, UnaryOperation

    return [
        (view.GatherOp, _rule_gather),
        (view.ScatterOp, _rule_scatter),
        (convolution.Conv2DOp, _rule_conv),
        (pooling.MaxPool2DOp, _rule_fold_leading),
        (pooling.AvgPool2DOp, _rule_fold_leading),
        (attention.FusedAttentionOp, _rule_fold_leading),
        (xent.SoftmaxCrossEntropyOp, _rule_same_shape),
        (view.BroadcastToOp, _rule_broadcast_to),
        (view.ReshapeOp, _rule_reshape),
        (view.PermuteOp, _rule_permute),
        (view.SliceTensorOp, _rule_slice),
        (view.SliceUpdateOp, _rule_slice),
        (view.PadOp, _rule_pad),
        (view.ConcatenateOp, _rule_same_shape),
        (normalization.LayerNormOp, _rule_layer_norm),
        (binary.MatmulOp, _rule_same_shape),
        (control_flow.WhereOp, _rule_same_shape),
        (unary.GeluBackwardOp, _rule_same_shape),
        (BinaryOperation, _rule_same_shape),
        (ReduceOperation, _rule_same_shape),
        (UnaryOperation, _rule_same_shape),
    ]


_RULES: list[tuple[type, Callable]] | None = None


def _rule_for(op) -> Callable | None:
    global _RULES
    if _RULES is None:
        _RULES = _rules()
    for cls, rule in _RULES:
        if isinstance(op, cls):
            return rule
    return None


def dispatch(op, args: list, kwargs: dict) -> list:
    """Run ``op`` on arguments of which at least one is batched."""
    rule = _rule_for(op)
    if rule is None:
        raise NoBatchRule(f"op '{op.name}' has no batching rule")
    batched = [a for a in args if isinstance(a, BatchedTensor)]
    bd = max(a._bd for a in batched)
    sizes = [1] * bd
    for a in batched:
        for i, d in enumerate(a.batch_shape):
            if d != 1:
                if sizes[i] not in (1, d):
                    raise ValueError(f"vmap: mapped axes of sizes {sizes[i]} and {d} meet in '{op.name}'")
                sizes[i] = d
    got = rule(op, list(args), dict(kwargs or {}), bd, tuple(sizes))
    if isinstance(got, Done):  # the rule computed the result itself, out of other ops
        return [BatchedTensor(o, bd) for o in got.outs]
    outs = op(got[0], got[1])
    if len(got) > 2:
        outs = got[2](outs)
    return [BatchedTensor(o, bd) for o in outs]


__all__ = ["NoBatchRule", "dispatch", "lift", "plain", "batch_dims_of", "current_level", "level_sizes",
           "push_level", "pop_level"]
