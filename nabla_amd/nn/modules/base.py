"""``Module`` base class (nabla/nn/modules/base.py:106-337): parameters are
tensors with ``requires_grad`` assigned as attributes, submodules are tracked,
and every subclass is a pytree node (parameters, buffers, submodules are the
children) so modules pass through grad / compile unchanged."""
from __future__ import annotations

from collections import OrderedDict
from typing import Any, Iterator

from ...core.pytree import is_tensor, register_pytree_node
from ...core.tensor import Tensor, realize_all

_RESERVED = {"_parameters", "_buffers", "_modules", "_training"}


def _module_tree_flatten(module: "Module"):
    param_keys = tuple(module._parameters.keys())
    buffer_keys = tuple(module._buffers.keys())
    module_keys = tuple(module._modules.keys())
    children = ([module._parameters[k] for k in param_keys] +
                [module._buffers[k] for k in buffer_keys] +
                [module._modules[k] for k in module_keys])
    extras = []
    for key, value in module.__dict__.items():
        if key in _RESERVED or key in module._parameters or key in module._buffers \
                or key in module._modules:
            continue
        extras.append((key, value))
    aux = (type(module), param_keys, buffer_keys, module_keys,
           tuple(sorted(extras, key=lambda kv: kv[0])), bool(module._training))
    return children, aux


def _module_tree_unflatten(aux, children) -> "Module":
    cls, param_keys, buffer_keys, module_keys, extras, training = aux
    obj = object.__new__(cls)
    object.__setattr__(obj, "_parameters", OrderedDict())
    object.__setattr__(obj, "_buffers", OrderedDict())
    object.__setattr__(obj, "_modules", OrderedDict())
    object.__setattr__(obj, "_training", training)
    cursor = 0
    for keys, store in ((param_keys, obj._parameters), (buffer_keys, obj._buffers),
                        (module_keys, obj._modules)):
        for key in keys:
            value = children[cursor]
            cursor += 1
            store[key] = value
            object.__setattr__(obj, key, value)
    for key, value in extras:
        object.__setattr__(obj, key, value)
    return obj


class Module:
    def __init_subclass__(cls, **kwargs: Any) -> None:
        super().__init_subclass__(**kwargs)
        register_pytree_node(cls, _module_tree_flatten, _module_tree_unflatten)

    def __init__(self) -> None:
        object.__setattr__(self, "_parameters", OrderedDict())
        object.__setattr__(self, "_buffers", OrderedDict())
        object.__setattr__(self, "_modules", OrderedDict())
        object.__setattr__(self, "_training", True)

    def __setattr__(self, name: str, value: Any) -> None:
        if name in _RESERVED:
            object.__setattr__(self, name, value)
            return
        for store in (self._parameters, self._buffers, self._modules):
            store.pop(name, None)
        object.__setattr__(self, name, value)
        if isinstance(value, Module):
            self._modules[name] = value
        elif is_tensor(value):
            (self._parameters if value.requires_grad else self._buffers)[name] = value

    def register_buffer(self, name: str, tensor: Tensor | None) -> None:
        setattr(self, name, tensor)

    def forward(self, *args: Any, **kwargs: Any) -> Any:
        raise NotImplementedError

    def __call__(self, *args: Any, **kwargs: Any) -> Any:
        return self.forward(*args, **kwargs)

    def parameters(self) -> Iterator[Tensor]:
        for _, p in self.named_parameters():
            yield p

    def named_parameters(self, prefix: str = "") -> Iterator[tuple[str, Tensor]]:
        for name, p in self._parameters.items():
            yield (f"{prefix}{name}", p)
        for mname, m in self._modules.items():
            yield from m.named_parameters(prefix=f"{prefix}{mname}.")

    def buffers(self) -> Iterator[Tensor]:
        for _, b in self.named_buffers():
            yield b

    def named_buffers(self, prefix: str = "") -> Iterator[tuple[str, Tensor]]:
        for name, b in self._buffers.items():
            yield (f"{prefix}{name}", b)
        for mname, m in self._modules.items():
            yield from m.named_buffers(prefix=f"{prefix}{mname}.")

    def modules(self) -> Iterator["Module"]:
        yield self
        for m in self._modules.values():
            yield from m.modules()

    def train(self) -> "Module":
        for m in self.modules():
            object.__setattr__(m, "_training", True)
        return self

    def eval(self) -> "Module":
        for m in self.modules():
            object.__setattr__(m, "_training", False)
        return self

    def zero_grad(self) -> None:
        for p in self.parameters():
            p.grad = None

    def state_dict(self) -> "OrderedDict[str, Tensor]":
        out: "OrderedDict[str, Tensor]" = OrderedDict()
        for k, v in self.named_parameters():
            out[k] = v
        for k, v in self.named_buffers():
            out[k] = v
        return out

    def load_state_dict(self, state_dict) -> None:
        for name, value in state_dict.items():
            obj = self
            *path, leaf = name.split(".")
            for part in path:
                obj = obj._modules[part]
            if obj.__dict__.get(leaf) is not None and is_tensor(obj.__dict__[leaf]):
                value.requires_grad = obj.__dict__[leaf].requires_grad
            setattr(obj, leaf, value)

    def extra_repr(self) -> str:
        return ""

    def __repr__(self) -> str:
        lines = [f"{type(self).__name__}({self.extra_repr()}"]
        for name, m in self._modules.items():
            lines.append(f"  ({name}): {m!r}")
        return "\n".join(lines) + ")"
