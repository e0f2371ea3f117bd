"""Single-tensor and pytree optimizer updates.

Same functions, arguments and arithmetic as nabla/nn/optim/functional.py
(``sgd_step`` 14-39, ``sgd_update`` 42-113, ``adamw_step`` 116-162).  Every
update of one tensor is plain tensor arithmetic; over a pytree all leaves of one dtype go to
one launch (``ops.optim``) that reads param / grad / state once and writes each result once.
"""
from __future__ import annotations

import math
from typing import Any

from ... import config
from ...core import Tensor, is_tensor, realize_all, tree_flatten, tree_unflatten
from ...ops.creation import zeros_like
from ...ops.unary import exp, sqrt


def sgd_step(param: Tensor, grad: Tensor, momentum_buffer: Tensor | None = None, *, lr: float,
             weight_decay: float = 0.0, momentum: float = 0.0):
    """``(new_param, new_momentum_buffer)`` for one tensor (functional.py:14-39): L2 decay is
    added to the gradient, the first momentum step adopts the update as the buffer."""
    step_dir = grad
    if weight_decay != 0.0:
        step_dir = step_dir + param * weight_decay
    if momentum != 0.0:
        momentum_buffer = step_dir if momentum_buffer is None else momentum * momentum_buffer + step_dir
        step_dir = momentum_buffer
    return param - step_dir * lr, momentum_buffer


def adamw_step(param: Tensor, grad: Tensor, m: Tensor, v: Tensor, step, *, lr: float,
               beta1: float = 0.9, beta2: float = 0.999, eps: float = 1e-8,
               weight_decay: float = 0.0, bias_correction: bool = True):
    """``(new_param, m_t, v_t)`` for one tensor (functional.py:116-162).  ``step`` may be a
    0-d tensor (inside ``compile`` the counter is data): the bias corrections are then
    ``1 - exp(step * log(beta))``.  Decay is decoupled: added to the update, not the gradient."""
    m_t = m * beta1 + grad * (1.0 - beta1)
    v_t = v * beta2 + (grad * grad) * (1.0 - beta2)
    if not bias_correction:
        c1 = c2 = 1.0
    elif is_tensor(step):
        c1 = 1.0 - exp(step * math.log(beta1))
        c2 = 1.0 - exp(step * math.log(beta2))
    else:
        c1 = 1.0 - beta1 ** step
        c2 = 1.0 - beta2 ** step
    update = (m_t / c1) / (sqrt(v_t / c2) + eps)
    if weight_decay != 0.0:
        update = update + param * weight_decay
    return param - update * lr, m_t, v_t


# ---- pytree plumbing shared by the functional and the stateful forms ---------------------------
def _leaves_like(tree: Any, treedef_leaves: int) -> list:
    """Leaves of a state tree aligned with the parameter leaves (``None`` entries kept)."""
    if tree is None:
        return [None] * treedef_leaves
    leaves = tree_flatten(tree, is_leaf=lambda x: x is None)[0]
    if len(leaves) != treedef_leaves:
        raise ValueError(f"optimizer state has {len(leaves)} leaves for {treedef_leaves} parameters")
    return leaves


def map_update(fn, params: Any, grads: Any, *state_trees: Any):
    """Apply ``fn(p, g, *state) -> (new_p, *new_state)`` to every parameter leaf that has a
    tensor gradient; other leaves pass through.  Returns the new trees."""
    p_leaves, treedef = tree_flatten(params, is_leaf=lambda x: x is None)
    g_leaves = _leaves_like(grads, len(p_leaves))
    s_leaves = [_leaves_like(t, len(p_leaves)) for t in state_trees]
    outs = [[] for _ in range(1 + len(state_trees))]
    for i, (p, g) in enumerate(zip(p_leaves, g_leaves)):
        st = [s[i] for s in s_leaves]
        res = fn(p, g, *st) if is_tensor(p) and is_tensor(g) else (p, *st)
        for slot, r in zip(outs, res):
            slot.append(r)
    return tuple(tree_unflatten(treedef, o) for o in outs)


def _takes_list_kernel(p, g, state) -> bool:
    from ...ops.optim import UPDATE_DTYPES
    group = [p, g, *state]
    return (all(is_tensor(t) for t in group) and p.dtype in UPDATE_DTYPES and
            all(t.dtype is p.dtype and tuple(t.shape) == tuple(p.shape) for t in group) and
            all(int(d) > 0 for d in p.shape))


def list_update(per_leaf, per_list, params: Any, grads: Any, *state_trees: Any):
    """``map_update`` with one launch per dtype instead of one group of ops per leaf:
    ``per_list(ps, gs, *states) -> (new_ps, *new_states)`` takes all leaves of one dtype whose
    gradient and state tensors match the parameter in shape and type; whatever is left
    (mismatched types, missing state) goes through ``per_leaf`` as in ``map_update``."""
    if not config.MULTI_TENSOR_OPTIMIZER:
        return map_update(per_leaf, params, grads, *state_trees)
    p_leaves, treedef = tree_flatten(params, is_leaf=lambda x: x is None)
    g_leaves = _leaves_like(grads, len(p_leaves))
    s_leaves = [_leaves_like(t, len(p_leaves)) for t in state_trees]
    outs = [list(p_leaves)] + [list(s) for s in s_leaves]
    by_dtype: dict = {}
    for i, (p, g) in enumerate(zip(p_leaves, g_leaves)):
        st = [s[i] for s in s_leaves]
        if _takes_list_kernel(p, g, st):
            by_dtype.setdefault(p.dtype, []).append(i)
        elif is_tensor(p) and is_tensor(g):
            for slot, r in zip(outs, per_leaf(p, g, *st)):
                slot[i] = r
    for idx in by_dtype.values():
        res = per_list([p_leaves[i] for i in idx], [g_leaves[i] for i in idx],
                       *[[s[i] for i in idx] for s in s_leaves])
        for slot, new in zip(outs, res):
            if new is None:
                continue
            for i, t in zip(idx, new):
                slot[i] = t
    return tuple(tree_unflatten(treedef, o) for o in outs)


def unrealized(tree: Any) -> list:
    return [t for t in tree_flatten(tree, is_leaf=lambda x: x is None)[0] if is_tensor(t) and not t.real]


def sgd_over_trees(per_leaf, params: Any, grads: Any, bufs: Any, *, lr: float, momentum: float,
                   weight_decay: float):
    """``(new_params, new_bufs)``; without momentum the buffer tree comes back as it went in."""
    from ...ops.optim import sgd_multi
    if momentum != 0.0 and bufs is not None:
        return list_update(per_leaf, lambda ps, gs, bs: sgd_multi(
            ps, gs, bs, lr=lr, momentum=momentum, weight_decay=weight_decay), params, grads, bufs)
    if momentum != 0.0:
        return map_update(per_leaf, params, grads, bufs)
    new_params, = list_update(lambda p, g: (per_leaf(p, g, None)[0],),
                              lambda ps, gs: (sgd_multi(ps, gs, lr=lr, weight_decay=weight_decay)[0],),
                              params, grads)
    return new_params, bufs


def adamw_over_trees(per_leaf, params: Any, grads: Any, m: Any, v: Any, step, **hyper):
    """``(new_params, new_m, new_v)`` for one AdamW step; ``hyper`` as for ``adamw_step``."""
    from ...ops.optim import adamw_multi
    return list_update(per_leaf, lambda ps, gs, ms, vs: adamw_multi(ps, gs, ms, vs, step, **hyper),
                       params, grads, m, v)


def sgd_update(params: Any, grads: Any, state: dict | None = None, *, lr: float, momentum: float = 0.0,
               weight_decay: float = 0.0):
    """Functional SGD on pytrees (functional.py:42-113): returns ``(new_params, new_state)`` with
    ``state = {"momentum_buffers", "step"}``; a missing state starts from zero buffers."""
    from .optimizer import Optimizer

    if state is None:
        bufs = None
        if momentum != 0.0:
            p_leaves, treedef = tree_flatten(params, is_leaf=lambda x: x is None)
            bufs = tree_unflatten(treedef, [zeros_like(p) if is_tensor(p) else None for p in p_leaves])
        state = {"momentum_buffers": bufs, "step": 0}

    def one(p, g, buf):
        return sgd_step(p, g, buf, lr=lr, weight_decay=weight_decay, momentum=momentum)

    new_params, new_bufs = sgd_over_trees(one, params, grads, state["momentum_buffers"], lr=lr,
                                          momentum=momentum, weight_decay=weight_decay)
    if Optimizer._AUTO_REALIZE_UPDATED_PARAMS:
        todo = unrealized(new_params)
        if todo:
            realize_all(*todo)
    return new_params, {"momentum_buffers": new_bufs, "step": int(state["step"]) + 1}
