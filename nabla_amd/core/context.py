"""Device / dtype defaults (mirrors nabla/core/common/context.py:45-139).

There is one kind of compute device here, the MI355X the process was started
on.  ``CPU()`` exists so that reference programs that name it keep running; a
tensor "on the CPU device" is simply a host tensor that is uploaded when it
first takes part in a computation.
"""
from __future__ import annotations

import contextlib
import os
from contextvars import ContextVar

from .dtype import DType


class Device:
    __slots__ = ("kind", "index")

    def __init__(self, kind: str, index: int = 0):
        self.kind = kind
        self.index = index

    def __eq__(self, other):
        return isinstance(other, Device) and (self.kind, self.index) == (other.kind, other.index)

    def __hash__(self):
        return hash((self.kind, self.index))

    def __repr__(self):
        return f"Device({self.kind}:{self.index})"


def CPU() -> Device:
    return Device("cpu", 0)


def Accelerator(index: int = 0) -> Device:
    return Device("gpu", index)


def _default_device_from_env() -> Device:
    # NABLA_DEFAULT_DEVICE keeps its reference meaning (context.py:74-90);
    # both settings compute on the GPU here.
    v = os.environ.get("NABLA_DEFAULT_DEVICE", "gpu").lower()
    return CPU() if v == "cpu" else Accelerator()


_DEFAULT_DEVICE: ContextVar[Device] = ContextVar("default_device", default=_default_device_from_env())
_DEFAULT_DTYPE: ContextVar[DType] = ContextVar("default_dtype", default=DType.float32)


def defaults() -> tuple[DType, Device]:
    return _DEFAULT_DTYPE.get(), _DEFAULT_DEVICE.get()


@contextlib.contextmanager
def default_device(device: Device):
    tok = _DEFAULT_DEVICE.set(device)
    try:
        yield
    finally:
        _DEFAULT_DEVICE.reset(tok)


@contextlib.contextmanager
def default_dtype(dtype: DType):
    tok = _DEFAULT_DTYPE.set(dtype)
    try:
        yield
    finally:
        _DEFAULT_DTYPE.reset(tok)


@contextlib.contextmanager
def defaults_like(t):
    t1 = _DEFAULT_DTYPE.set(t.dtype)
    t2 = _DEFAULT_DEVICE.set(t.device)
    try:
        yield
    finally:
        _DEFAULT_DEVICE.reset(t2)
        _DEFAULT_DTYPE.reset(t1)
