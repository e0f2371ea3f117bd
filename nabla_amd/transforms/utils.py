"""Helpers shared by grad / vjp (nabla/transforms/utils.py:19-100)."""
from __future__ import annotations

from typing import Any


def select_argnums(grads_struct: tuple, argnums):
    """Pick the gradient(s) for ``argnums`` out of the per-argument gradient tuple."""
    if isinstance(argnums, int):
        return grads_struct[argnums]
    return tuple(grads_struct[i] for i in argnums)
