"""Comparison helpers for tests (nabla/core/testing.py:17-82, re-exported as
``nabla.testing``): ``batch_realize`` realizes every lazy tensor found in arbitrary pytrees in
one go, ``assert_allclose`` compares tensors, numpy / torch arrays, scalars and containers of
them leaf by leaf."""
from __future__ import annotations

from collections.abc import Mapping, Sequence
from typing import Any

import numpy as np

from .core import is_tensor, realize_all, tree_leaves


def batch_realize(*objs: Any) -> None:
    lazy = [leaf for obj in objs for leaf in tree_leaves(obj) if is_tensor(leaf) and not leaf.real]
    if lazy:
        realize_all(*lazy)


def _as_numpy(obj: Any) -> Any:
    if is_tensor(obj):
        a = obj
        if a.dtype.name == "bfloat16":
            a = a.cast(type(a.dtype).float32)
        return a.to_numpy()
    if hasattr(obj, "detach") and hasattr(obj, "cpu"):  # torch tensor
        t = obj.detach().cpu()
        return (t.float() if str(t.dtype) == "torch.bfloat16" else t).numpy()
    return obj


def assert_allclose(actual: Any, expected: Any, *, rtol: float = 1e-5, atol: float = 1e-8,
                    equal_nan: bool = False, err_msg: str = "") -> None:
    batch_realize(actual, expected)
    if isinstance(actual, Mapping) and isinstance(expected, Mapping):
        assert set(actual) == set(expected), f"key sets differ: {set(actual) ^ set(expected)}"
        for k in actual:
            assert_allclose(actual[k], expected[k], rtol=rtol, atol=atol, equal_nan=equal_nan,
                            err_msg=f"{err_msg}[{k!r}]")
        return
    if (isinstance(actual, Sequence) and isinstance(expected, Sequence)
            and not isinstance(actual, (str, bytes)) and not isinstance(expected, (str, bytes))):
        assert len(actual) == len(expected), f"lengths differ: {len(actual)} vs {len(expected)}"
        for i, (a, e) in enumerate(zip(actual, expected)):
            assert_allclose(a, e, rtol=rtol, atol=atol, equal_nan=equal_nan, err_msg=f"{err_msg}[{i}]")
        return
    np.testing.assert_allclose(np.asarray(_as_numpy(actual)), np.asarray(_as_numpy(expected)),
                               rtol=rtol, atol=atol, equal_nan=equal_nan, err_msg=err_msg)
