"""Pytree utilities for argument handling in the transforms.

Same surface as nabla/core/common/pytree.py (tree_flatten / tree_unflatten /
tree_map / tree_leaves / tree_structure / register_pytree_node / PyTreeDef);
no arithmetic lives here.
"""
from __future__ import annotations

from typing import Any, Callable

_REGISTRY: dict[type, tuple[Callable, Callable]] = {}


def register_pytree_node(cls: type, flatten_fn: Callable, unflatten_fn: Callable) -> None:
    """``flatten_fn(obj) -> (children, aux)``; ``unflatten_fn(aux, children) -> obj``."""
    _REGISTRY[cls] = (flatten_fn, unflatten_fn)


class PyTreeDef:
    __slots__ = ("kind", "aux", "children", "num_leaves")

    def __init__(self, kind: Any, aux: Any, children: tuple, num_leaves: int):
        self.kind = kind
        self.aux = aux
        self.children = children
        self.num_leaves = num_leaves

    def _key(self):
        return (self.kind, self.aux, self.children)

    def __eq__(self, other):
        return isinstance(other, PyTreeDef) and self._key() == other._key()

    def __hash__(self):
        try:
            return hash(self._key())
        except TypeError:
            return hash((self.kind, repr(self.aux), self.children))

    def __repr__(self):
        if self.kind is _K_LEAF:
            return "*"
        return f"PyTreeDef({getattr(self.kind, '__name__', self.kind)}, {list(self.children)})"


_K_LEAF = "leaf"
_K_NONE = "none"
_LEAF_DEF = PyTreeDef(_K_LEAF, None, (), 1)


def is_tensor(x: Any) -> bool:
    from .tensor import Tensor

    return isinstance(x, Tensor)


def tree_flatten(tree: Any, is_leaf: Callable[[Any], bool] | None = None):
    leaves: list[Any] = []

    def go(node) -> PyTreeDef:
        if is_leaf is not None and is_leaf(node):
            leaves.append(node)
            return _LEAF_DEF
        if node is None:
            return PyTreeDef(_K_NONE, None, (), 0)
        t = type(node)
        if t in _REGISTRY:
            children, aux = _REGISTRY[t][0](node)
            defs = tuple(go(c) for c in children)
            return PyTreeDef(t, aux, defs, sum(d.num_leaves for d in defs))
        if t is list or t is tuple:
            defs = tuple(go(c) for c in node)
            return PyTreeDef(t, None, defs, sum(d.num_leaves for d in defs))
        if isinstance(node, tuple) and hasattr(node, "_fields"):  # namedtuple
            defs = tuple(go(c) for c in node)
            return PyTreeDef(t, None, defs, sum(d.num_leaves for d in defs))
        if t is dict:
            keys = tuple(sorted(node.keys(), key=repr))
            defs = tuple(go(node[k]) for k in keys)
            return PyTreeDef(dict, keys, defs, sum(d.num_leaves for d in defs))
        leaves.append(node)
        return _LEAF_DEF

    try:
        treedef = go(tree)
    finally:
        # the closure refers to itself: unless that is undone it lives, and `leaves` with it,
        # until the cycle collector runs (device memory of dropped tensors would wait for that)
        go = None
    return leaves, treedef


def tree_unflatten(treedef: PyTreeDef, leaves) -> Any:
    it = iter(leaves)

    def go(d: PyTreeDef):
        if d.kind is _K_LEAF:
            return next(it)
        if d.kind is _K_NONE:
            return None
        kids = [go(c) for c in d.children]
        if d.kind is list:
            return kids
        if d.kind is tuple:
            return tuple(kids)
        if d.kind is dict:
            return dict(zip(d.aux, kids))
        if d.kind in _REGISTRY:
            return _REGISTRY[d.kind][1](d.aux, kids)
        return d.kind(*kids)  # namedtuple

    try:
        return go(treedef)
    finally:
        go = None  # (self-referential closure holding `leaves`, as in tree_flatten)


def tree_leaves(tree: Any, is_leaf=None) -> list:
    return tree_flatten(tree, is_leaf)[0]


def tree_structure(tree: Any, is_leaf=None) -> PyTreeDef:
    return tree_flatten(tree, is_leaf)[1]


def tree_map(fn: Callable, tree: Any, *rest: Any, is_leaf=None) -> Any:
    leaves, treedef = tree_flatten(tree, is_leaf)
    others = [tree_flatten(r, is_leaf)[0] for r in rest]
    return tree_unflatten(treedef, [fn(*xs) for xs in zip(leaves, *others)])


def tensor_leaves(tree: Any) -> list:
    return [x for x in tree_leaves(tree) if is_tensor(x)]
