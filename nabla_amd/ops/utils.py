"""``call_custom_kernel`` (nabla/ops/utils.py:765-824).

The reference loads a Mojo kernel library from ``kernel_path`` and emits
``ops.custom(name, device, values, out_types)``.  Here ``kernel_path`` names a
shared object (or a directory / ``.hip`` source next to which the built
``lib<name>.so`` lies) that exports ``int <func_name>(const nbk_tensor* in,
int n_in, nbk_tensor* out, int n_out, void* stream)``; the lowering records a
custom step that the kernel library resolves and calls.
"""
from __future__ import annotations

from pathlib import Path
from typing import Any, Union

from ..backend import ir


def _resolve_library(func_name: str, kernel_path) -> Path:
    paths = kernel_path if isinstance(kernel_path, list) else [kernel_path]
    tried = []
    for p in paths:
        p = Path(p).resolve()
        cands = [p] if p.suffix == ".so" else []
        if p.is_dir():
            cands += [p / f"lib{func_name}.so", p / f"{func_name}.so"] + sorted(p.glob("*.so"))
        elif p.suffix in (".hip", ".cpp", ".mojo"):
            cands += [p.with_suffix(".so"), p.parent / f"lib{p.stem}.so"]
        for c in cands:
            tried.append(str(c))
            if c.exists():
                return c
    raise FileNotFoundError(
        f"call_custom_kernel: no built kernel library for '{func_name}' (looked at {tried})"
    )


def call_custom_kernel(func_name: str, kernel_path: Union[str, Path, list], values: Any,
                       out_types: Any, device: Any = None, **kwargs: Any):
    """Invoke a custom HIP kernel by its exported name.

    ``values`` are IR values (what ``kernel()`` received); ``out_types`` are
    ``(shape, dtype)`` pairs or ``value.type``.  Returns IR value(s)."""
    lib_path = _resolve_library(func_name, kernel_path)
    values_list = [values] if isinstance(values, ir.Value) else list(values)
    unwrap = not isinstance(out_types, list)
    out_list = [out_types] if unwrap else list(out_types)
    results = ir.custom(func_name, str(lib_path), values_list, out_list)
    return results[0] if unwrap else results
