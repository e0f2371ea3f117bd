"""Fine-tuning checkpoints in the reference's on-disk format
(nabla/nn/finetune/checkpoint.py:19-170): a directory holding

* ``tensors.npz`` (``numpy.savez_compressed``): one array per tensor leaf, keyed by its path in
  the pytree -- ``lora`` for the adapter parameters, ``opt_m`` / ``opt_v`` for the AdamW
  moments; a dict level appends ``.key`` (keys visited in sorted order), a list or tuple level
  appends ``[i]``;
* ``meta.json``: ``step``, ``has_optimizer``, ``user_metadata`` and the sorted ``tensor_keys``.

Loading walks the caller's template trees, so only the keys the template names are read and
every restored tensor takes the template leaf's dtype.  bfloat16 leaves are stored as float32
(numpy has no bfloat16), which is lossless.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Any

import numpy as np

from ...core import Tensor, is_tensor
from ...core.dtype import DType

PathLike = str | Path


def _tensor_paths(tree: Any, prefix: str) -> list[tuple[str, Tensor]]:
    if is_tensor(tree):
        return [(prefix, tree)]
    out: list[tuple[str, Tensor]] = []
    if isinstance(tree, dict):
        for key in sorted(tree.keys(), key=str):
            out += _tensor_paths(tree[key], f"{prefix}.{key}" if prefix else str(key))
    elif isinstance(tree, (list, tuple)):
        for i, item in enumerate(tree):
            out += _tensor_paths(item, f"{prefix}[{i}]")
    return out


def _rebuild(tree: Any, prefix: str, arrays) -> Any:
    """A copy of ``tree`` whose tensor leaves are read from ``arrays`` under the same paths."""
    if is_tensor(tree):
        if prefix not in arrays:
            raise KeyError(f"Missing tensor key in checkpoint: {prefix}")
        return Tensor.from_dlpack(arrays[prefix]).to(tree.dtype)
    if isinstance(tree, dict):
        return {key: _rebuild(tree[key], f"{prefix}.{key}" if prefix else str(key), arrays)
                for key in tree}
    if isinstance(tree, (list, tuple)):
        items = [_rebuild(item, f"{prefix}[{i}]", arrays) for i, item in enumerate(tree)]
        return tuple(items) if isinstance(tree, tuple) else items
    return tree


def _to_array(t: Tensor) -> np.ndarray:
    return (t.cast(DType.float32) if t.dtype is DType.bfloat16 else t).to_numpy()


def save_finetune_checkpoint(path: PathLike, *, lora_params: Any,
                             optimizer_state: dict[str, Any] | None = None,
                             metadata: dict[str, Any] | None = None) -> None:
    out_dir = Path(path)
    out_dir.mkdir(parents=True, exist_ok=True)
    tensors = _tensor_paths(lora_params, "lora")
    step = None
    if optimizer_state is not None:
        step = int(optimizer_state.get("step", 0))
        for slot in ("m", "v"):
            if slot in optimizer_state:
                tensors += _tensor_paths(optimizer_state[slot], f"opt_{slot}")
    payload = {name: _to_array(t) for name, t in tensors}
    np.savez_compressed(out_dir / "tensors.npz", **payload)
    meta = {"step": step, "has_optimizer": optimizer_state is not None,
            "user_metadata": metadata or {}, "tensor_keys": sorted(payload)}
    with (out_dir / "meta.json").open("w", encoding="utf-8") as f:
        json.dump(meta, f, indent=2, sort_keys=True)


def load_finetune_checkpoint(path: PathLike, *, lora_template: Any,
                             optimizer_template: dict[str, Any] | None = None,
                             ) -> tuple[Any, dict[str, Any] | None, dict[str, Any]]:
    ckpt = Path(path)
    tensors_path, meta_path = ckpt / "tensors.npz", ckpt / "meta.json"
    if not tensors_path.exists():
        raise FileNotFoundError(f"Missing checkpoint tensor file: {tensors_path}")
    if not meta_path.exists():
        raise FileNotFoundError(f"Missing checkpoint metadata file: {meta_path}")
    with meta_path.open(encoding="utf-8") as f:
        meta = json.load(f)
    with np.load(tensors_path, allow_pickle=False) as arrays:
        lora = _rebuild(lora_template, "lora", arrays)
        opt = None
        if optimizer_template is not None and meta.get("has_optimizer", False):
            opt = {"step": int(meta.get("step") or 0)}
            for slot in ("m", "v"):
                opt[slot] = _rebuild(optimizer_template.get(slot), f"opt_{slot}", arrays)
    return lora, opt, meta
