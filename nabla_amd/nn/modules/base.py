"""``Module``: the container layers are built from (interface of nabla/nn/modules/base.py:106-337).

A module is an ordinary object whose attributes happen to include tensors and other modules.
It keeps one record about them, ``_roles``: attribute name -> ``"parameter"`` (a tensor that
required a gradient when it was assigned), ``"buffer"`` (any other tensor) or ``"module"``.
Everything else is derived from that record and the attributes themselves: the ``_parameters``
/ ``_buffers`` / ``_modules`` views, the iterators, the state dict, and the pytree form that
lets a module pass through ``grad`` / ``compile`` / ``tree_map`` like a dict of its tensors
(children = the attributes that have a role, in assignment order; everything else, with the
roles and the training flag, is static structure).
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Any, Iterator

from ...core.pytree import is_tensor, register_pytree_node
from ...core.tensor import Tensor

PARAMETER, BUFFER, MODULE = "parameter", "buffer", "module"
_OWN_STATE = ("_roles", "_training")


def _role_of(value: Any) -> str | None:
    if isinstance(value, Module):
        return MODULE
    if is_tensor(value):
        return PARAMETER if value.requires_grad else BUFFER
    return None


def _flatten_module(module: "Module"):
    roles = module._roles
    names = tuple(roles)
    plain = tuple(sorted(((k, v) for k, v in vars(module).items()
                          if k not in roles and k not in _OWN_STATE), key=lambda kv: kv[0]))
    static = (type(module), names, tuple(roles[n] for n in names), plain, module._training)
    return [getattr(module, n) for n in names], static


def _unflatten_module(static, children) -> "Module":
    cls, names, kinds, plain, training = static
    module = object.__new__(cls)
    state = vars(module)
    state["_roles"] = dict(zip(names, kinds))  # roles travel with the structure, not the leaves
    state["_training"] = training
    state.update(zip(names, children))
    state.update(plain)
    return module


class Module:
    def __init_subclass__(cls, **kwargs: Any) -> None:
        super().__init_subclass__(**kwargs)
        register_pytree_node(cls, _flatten_module, _unflatten_module)

    def __init__(self) -> None:
        vars(self).update(_roles={}, _training=True)

    # ---- attribute bookkeeping ---------------------------------------------------------------
    def __setattr__(self, name: str, value: Any) -> None:
        if name in _OWN_STATE:
            vars(self)[name] = value
            return
        roles = self._roles
        roles.pop(name, None)  # a re-assigned attribute moves to the end, whatever it was before
        role = _role_of(value)
        if role is not None:
            roles[name] = role
        vars(self)[name] = value

    def __delattr__(self, name: str) -> None:
        self._roles.pop(name, None)
        object.__delattr__(self, name)

    def _having(self, role: str) -> "OrderedDict[str, Any]":
        return OrderedDict((n, getattr(self, n)) for n, r in self._roles.items() if r == role)

    @property
    def _parameters(self) -> "OrderedDict[str, Tensor]":
        return self._having(PARAMETER)

    @property
    def _buffers(self) -> "OrderedDict[str, Tensor]":
        return self._having(BUFFER)

    @property
    def _modules(self) -> "OrderedDict[str, Module]":
        return self._having(MODULE)

    def register_buffer(self, name: str, tensor: Tensor | None) -> None:
        setattr(self, name, tensor)

    # ---- calling -----------------------------------------------------------------------------
    def forward(self, *args: Any, **kwargs: Any) -> Any:
        raise NotImplementedError

    def __call__(self, *args: Any, **kwargs: Any) -> Any:
        return self.forward(*args, **kwargs)

    # ---- walking -----------------------------------------------------------------------------
    def _walk(self, role: str, prefix: str = "") -> Iterator[tuple[str, Any]]:
        """(dotted name, value) of every attribute with ``role``, this module's first, then its
        submodules' in assignment order."""
        for name, value in self._having(role).items():
            yield prefix + name, value
        for name, sub in self._having(MODULE).items():
            yield from sub._walk(role, f"{prefix}{name}.")

    def named_parameters(self, prefix: str = "") -> Iterator[tuple[str, Tensor]]:
        return self._walk(PARAMETER, prefix)

    def named_buffers(self, prefix: str = "") -> Iterator[tuple[str, Tensor]]:
        return self._walk(BUFFER, prefix)

    def parameters(self) -> Iterator[Tensor]:
        return (p for _, p in self.named_parameters())

    def buffers(self) -> Iterator[Tensor]:
        return (b for _, b in self.named_buffers())

    def modules(self) -> Iterator["Module"]:
        yield self
        for sub in self._having(MODULE).values():
            yield from sub.modules()

    # ---- modes and gradients -------------------------------------------------------------------
    def _set_training(self, flag: bool) -> "Module":
        for m in self.modules():
            vars(m)["_training"] = flag
        return self

    def train(self) -> "Module":
        return self._set_training(True)

    def eval(self) -> "Module":
        return self._set_training(False)

    def zero_grad(self) -> None:
        for p in self.parameters():
            p.grad = None

    # ---- state -------------------------------------------------------------------------------
    def state_dict(self) -> "OrderedDict[str, Tensor]":
        return OrderedDict([*self.named_parameters(), *self.named_buffers()])

    def load_state_dict(self, state_dict) -> None:
        """Assign every entry to the attribute its dotted name leads to; a tensor that replaces
        one keeps the old tensor's ``requires_grad`` (and with it the role)."""
        for dotted, value in state_dict.items():
            *path, leaf = dotted.split(".")
            owner = self
            for part in path:
                owner = getattr(owner, part)
            current = vars(owner).get(leaf)
            if is_tensor(current):
                value.requires_grad = current.requires_grad
            setattr(owner, leaf, value)

    # ---- display -----------------------------------------------------------------------------
    def extra_repr(self) -> str:
        return ""

    def __repr__(self) -> str:
        head = f"{type(self).__name__}({self.extra_repr()}"
        body = [f"  ({name}): {sub!r}" for name, sub in self._having(MODULE).items()]
        return "\n".join([head, *body]) + ")"
