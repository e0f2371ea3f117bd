"""Stateful optimizers and the functional AdamW entry points.

Mirrors nabla/nn/optim/optimizer.py: ``Optimizer`` with its class-wide execution
policy (35-65), ``AdamW`` (68-160), ``SGD`` (163-232), ``adamw_init`` (235-239) and
``adamw_update`` (242-305).  ``step(grads)`` returns the new parameter tree; with
``grads=None`` the ``.grad`` attributes left by ``backward()`` are used.
"""
from __future__ import annotations

from typing import Any

from ... import config
from ...core import Tensor, is_tensor, realize_all, tree_flatten, tree_unflatten
from ...core.dtype import DType
from ...ops.creation import zeros_like
from .functional import adamw_over_trees, adamw_step, sgd_over_trees, sgd_step, unrealized


def _zeros_tree(params: Any):
    leaves, treedef = tree_flatten(params, is_leaf=lambda x: x is None)
    return tree_unflatten(treedef, [zeros_like(p) if is_tensor(p) else None for p in leaves])


def _grads_from_attributes(params: Any):
    leaves, treedef = tree_flatten(params, is_leaf=lambda x: x is None)
    return tree_unflatten(treedef, [p.grad if is_tensor(p) else None for p in leaves])


def _fresh_leaves(new_tree: Any, old_tree: Any):
    """Realized updated parameters become new graph leaves that keep the old
    ``requires_grad`` flag (optimizer.py:20-32): a step does not chain histories."""
    new_leaves, treedef = tree_flatten(new_tree, is_leaf=lambda x: x is None)
    old_leaves = tree_flatten(old_tree, is_leaf=lambda x: x is None)[0]
    out = []
    for n, o in zip(new_leaves, old_leaves):
        if is_tensor(n) and is_tensor(o) and n.real:
            n = n.detach()
            n.requires_grad_(bool(o.requires_grad))
        out.append(n)
    return tree_unflatten(treedef, out)


class Optimizer:
    """Base class; the two flags say whether ``step`` realizes what it returns."""

    _AUTO_REALIZE_UPDATED_PARAMS: bool = True
    _AUTO_REALIZE_UPDATED_STATE: bool = True

    def __init__(self, params: Any) -> None:
        self.params = params

    @classmethod
    def set_execution_policy(cls, *, auto_realize_updated_params: bool | None = None,
                             auto_realize_updated_state: bool | None = None) -> None:
        if auto_realize_updated_params is not None:
            Optimizer._AUTO_REALIZE_UPDATED_PARAMS = bool(auto_realize_updated_params)
        if auto_realize_updated_state is not None:
            Optimizer._AUTO_REALIZE_UPDATED_STATE = bool(auto_realize_updated_state)

    @classmethod
    def get_execution_policy(cls) -> dict[str, bool]:
        return {"auto_realize_updated_params": bool(Optimizer._AUTO_REALIZE_UPDATED_PARAMS),
                "auto_realize_updated_state": bool(Optimizer._AUTO_REALIZE_UPDATED_STATE)}

    def step(self, grads: Any = None) -> Any:
        raise NotImplementedError

    def _finish(self, old_params: Any, *state_trees: Any) -> Any:
        todo = []
        if self._AUTO_REALIZE_UPDATED_PARAMS:
            todo += unrealized(self.params)
        if self._AUTO_REALIZE_UPDATED_STATE:
            for t in state_trees:
                todo += unrealized(t)
        if todo:
            realize_all(*todo)
        self.params = _fresh_leaves(self.params, old_params)
        return self.params


class AdamW(Optimizer):
    """Adam with decoupled weight decay (Loshchilov & Hutter 2019)."""

    def __init__(self, params: Any, *, lr: float, betas: tuple[float, float] = (0.9, 0.999),
                 eps: float = 1e-8, weight_decay: float = 0.0) -> None:
        super().__init__(params)
        self.lr = float(lr)
        self.beta1, self.beta2 = float(betas[0]), float(betas[1])
        self.eps = float(eps)
        self.weight_decay = float(weight_decay)
        self.step_count = 0
        self.m = _zeros_tree(params)
        self.v = _zeros_tree(params)

    def step(self, grads: Any = None) -> Any:
        if grads is None:
            grads = _grads_from_attributes(self.params)
        old = self.params
        self.step_count += 1

        def one(p, g, m, v):
            if not (is_tensor(m) and is_tensor(v)):
                return p, m, v
            return adamw_step(p, g, m, v, self.step_count, lr=self.lr, beta1=self.beta1,
                              beta2=self.beta2, eps=self.eps, weight_decay=self.weight_decay)

        # (the counter goes in as data: one plan serves every step)
        step = Tensor.constant(float(self.step_count), dtype=DType.float32) \
            if config.MULTI_TENSOR_OPTIMIZER else self.step_count
        self.params, self.m, self.v = adamw_over_trees(
            one, self.params, grads, self.m, self.v, step, lr=self.lr, beta1=self.beta1,
            beta2=self.beta2, eps=self.eps, weight_decay=self.weight_decay)
        return self._finish(old, self.m, self.v)


class SGD(Optimizer):
    """Stochastic gradient descent with optional momentum and L2 decay."""

    def __init__(self, params: Any, *, lr: float, momentum: float = 0.0,
                 weight_decay: float = 0.0) -> None:
        super().__init__(params)
        self.lr = float(lr)
        self.momentum = float(momentum)
        self.weight_decay = float(weight_decay)
        self.step_count = 0
        self.momentum_buffers = _zeros_tree(params) if self.momentum != 0.0 else None

    def step(self, grads: Any = None) -> Any:
        if grads is None:
            grads = _grads_from_attributes(self.params)
        old = self.params
        self.step_count += 1

        def one(p, g, buf):
            return sgd_step(p, g, buf, lr=self.lr, weight_decay=self.weight_decay,
                            momentum=self.momentum)

        self.params, bufs = sgd_over_trees(one, self.params, grads, self.momentum_buffers, lr=self.lr,
                                           momentum=self.momentum, weight_decay=self.weight_decay)
        if self.momentum != 0.0:
            self.momentum_buffers = bufs
            return self._finish(old, self.momentum_buffers)
        return self._finish(old)


def adamw_init(params: Any) -> dict[str, Any]:
    """Zero moments and step 0 for a parameter pytree (optimizer.py:235-239)."""
    return {"m": _zeros_tree(params), "v": _zeros_tree(params), "step": 0}


def adamw_update(params: Any, grads: Any, state: dict[str, Any], *, lr: float,
                 weight_decay: float = 0.0, beta1: float = 0.9, beta2: float = 0.999,
                 eps: float = 1e-8, bias_correction: bool = True, realize: bool | None = None):
    """Functional AdamW on pytrees (optimizer.py:242-305): ``(new_params, new_state)``.  A tensor
    ``state["step"]`` stays a tensor (``step + 1.0``) so the update can live inside ``compile``."""
    prev = state["step"]
    step = prev + 1.0 if is_tensor(prev) else int(prev) + 1

    def one(p, g, m, v):
        if not (is_tensor(m) and is_tensor(v)):
            return p, m, v
        return adamw_step(p, g, m, v, step, lr=lr, beta1=beta1, beta2=beta2, eps=eps,
                          weight_decay=weight_decay, bias_correction=bias_correction)

    new_params, new_m, new_v = adamw_over_trees(
        one, params, grads, state["m"], state["v"], step, lr=lr, beta1=beta1, beta2=beta2, eps=eps,
        weight_decay=weight_decay, bias_correction=bias_correction)
    do_realize = Optimizer._AUTO_REALIZE_UPDATED_PARAMS if realize is None else bool(realize)
    if do_realize:
        todo = unrealized(new_params)
        if Optimizer._AUTO_REALIZE_UPDATED_STATE:
            todo += unrealized(new_m) + unrealized(new_v)
        if todo:
            realize_all(*todo)
    return new_params, {"m": new_m, "v": new_v, "step": step}
