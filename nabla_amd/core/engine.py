"""Graph engine: turns pending tensors into device buffers.

Takes the place of ``ComputeGraph.evaluate`` (nabla/core/graph/engine.py:289-733):
collect the op DAG under the targets (775-799), derive a structural cache key
(343-436), and on a miss lower the op list -- each ``op.kernel`` emits IR
(832-847) -- into a launch plan instead of compiling a MAX graph (656), then
run the plan on the leaf buffers (663) and store the results on the targets
(669-691).  Plans are cached by structure, never by value, so scalars and
weights can change freely between steps (nabla/ops/utils.py:165-197).
"""
from __future__ import annotations

import os
import time
from collections import OrderedDict
from contextvars import ContextVar
from typing import Any

from ..backend import ir
from ..backend.planner import plan_graph
from .tensor import Tensor, TensorImpl

_DEBUG = os.environ.get("NABLA_DEBUG", "0") in {"1", "true", "True"}
_DEBUG_CACHE = os.environ.get("NABLA_DEBUG_CACHE", "0") in {"1", "true", "True"}

_PLAN_CACHE: "OrderedDict[Any, Any]" = OrderedDict()
_PLAN_CACHE_MAX = 256
_STATS = {"hits": 0, "misses": 0, "lower_ms": 0.0}


def get_cache_stats() -> dict:
    """Hit / miss counters of the plan cache (engine.py:64-77)."""
    return dict(_STATS, size=len(_PLAN_CACHE))


def set_seed(seed: int) -> None:
    """Restart the device random generator (uniform, gaussian, dropout): after the same seed the
    same sequence of steps draws the same numbers."""
    from ..backend.executor import get_executor
    get_executor().seed(int(seed))


def clear_plan_cache() -> None:
    _PLAN_CACHE.clear()
    _STATS.update(hits=0, misses=0, lower_ms=0.0)


def _freeze(x: Any):
    """Hashable form of an op's kwargs."""
    if isinstance(x, dict):
        return tuple(sorted((k, _freeze(v)) for k, v in x.items()))
    if isinstance(x, (list, tuple)):
        return tuple(_freeze(v) for v in x)
    if isinstance(x, (TensorImpl, Tensor)):
        raise TypeError("tensors must be passed as op arguments, not keyword arguments")
    try:
        hash(x)
        return x
    except TypeError:
        return repr(x)


class ComputeGraph:
    """Evaluates lazily recorded ops.  One instance per context (engine.py:920-1012)."""

    def __init__(self) -> None:
        self.epoch = 0

    # ------------------------------------------------------------------ walk
    @staticmethod
    def _collect(targets: list[TensorImpl]):
        """Post-order list of OpNodes under ``targets`` stopping at realized
        tensors, and the realized leaves in first-visit order."""
        order = []
        leaves: list[TensorImpl] = []
        leaf_ids: dict[int, int] = {}
        scalar_bufs: dict[int, int] = {}
        seen: set[int] = set()

        def visit_leaf(impl: TensorImpl) -> None:
            if id(impl) in leaf_ids:
                return
            if not impl.shape:
                # 0-d constants come from a by-value cache and share their buffer: one graph
                # input per buffer (engine.py:185-258 dedups inputs by buffer identity), so
                # that ``x > 0.0`` written in twelve layers is one value, not twelve
                idx = scalar_bufs.get(id(impl._buffer))
                if idx is not None:
                    leaf_ids[id(impl)] = idx
                    return
                scalar_bufs[id(impl._buffer)] = len(leaves)
            leaf_ids[id(impl)] = len(leaves)
            leaves.append(impl)

        for t in targets:
            if t._buffer is not None:
                visit_leaf(t)
                continue
            root = t.output_refs
            if root is None:
                raise RuntimeError(f"Tensor {t} has no buffer and no producer: nothing to evaluate")
            if id(root) in seen:
                continue
            stack = [(root, 0)]
            seen.add(id(root))
            while stack:
                node, i = stack[-1]
                args = node.op_args
                pushed = False
                while i < len(args):
                    a = args[i]
                    i += 1
                    if not isinstance(a, TensorImpl):
                        continue
                    if a._buffer is not None:
                        visit_leaf(a)
                        continue
                    child = a.output_refs
                    if child is None:
                        raise RuntimeError(f"Tensor {a} has no graph values")
                    if id(child) not in seen:
                        seen.add(id(child))
                        stack[-1] = (node, i)
                        stack.append((child, 0))
                        pushed = True
                        break
                if not pushed:
                    stack.pop()
                    order.append(node)
        return order, leaves, leaf_ids

    @staticmethod
    def _structure_key(order, leaves, leaf_ids, targets):
        slot: dict[int, int] = {}
        parts = []
        for impl in leaves:
            parts.append(("L", impl.shape, impl.dtype))
        next_slot = len(leaves) + (1 << 40)
        for node in order:
            ins = []
            for a in node.op_args:
                if isinstance(a, TensorImpl):
                    if a._buffer is not None:
                        ins.append(leaf_ids[id(a)])
                    else:
                        ins.append(slot[id(a)])
                else:
                    ins.append(("c", _freeze(a)))
            kw = node._op_hash
            if kw is None:
                kw = _freeze(node.op_kwargs) if node.op_kwargs else ()
            parts.append((node.op.name, kw, tuple(ins), len(node._refs)))
            for o in node._refs:  # (numbered whether alive or not: the number says which result it is)
                if o is not None:
                    slot[id(o)] = next_slot
                next_slot += 1
        tk = tuple(leaf_ids[id(t)] if t._buffer is not None else slot[id(t)] for t in targets)
        return (tuple(parts), tk)

    # ------------------------------------------------------------------ lower
    @staticmethod
    def _lower(order, leaves, targets, leaf_ids):
        builder = ir.Builder()
        vals: dict[int, ir.Value] = {}
        with ir.building(builder):
            leaf_vals = [ir.input(impl.shape, impl.dtype) for impl in leaves]
            for key, idx in leaf_ids.items():
                vals[key] = leaf_vals[idx]
            for node in order:
                args = [vals[id(a)] if isinstance(a, TensorImpl) else a for a in node.op_args]
                try:
                    outs = node.op.kernel(args, node.op_kwargs or {})
                except Exception as e:
                    raise RuntimeError(
                        f"Graph building failed for operation '{node.op.name}': "
                        f"{type(e).__name__}: {e}"
                    ) from e
                if not isinstance(outs, (list, tuple)):
                    outs = [outs]
                if len(outs) != len(node._refs):
                    raise RuntimeError(
                        f"operation '{node.op.name}' produced {len(outs)} values for "
                        f"{len(node._refs)} outputs"
                    )
                for o, v in zip(node._refs, outs):
                    if o is None:
                        continue
                    if tuple(v.shape) != tuple(o.shape):
                        raise RuntimeError(
                            f"operation '{node.op.name}': kernel produced shape {v.shape}, "
                            f"compute_physical_shape promised {o.shape}"
                        )
                    if v.dtype is not o.dtype:
                        v = ir.cast(v, o.dtype)
                    vals[id(o)] = v
            out_vals = [vals[id(t)] for t in targets]
            plan = plan_graph(builder, out_vals)
        return plan

    # ------------------------------------------------------------------ evaluate
    def evaluate(self, tensor: Tensor, *extra: Tensor, return_model: bool = False):
        from ..backend.executor import get_executor

        tensors = [tensor, *extra]
        targets: list[TensorImpl] = []
        seen_t: set[int] = set()
        for t in tensors:
            impl = t._impl if isinstance(t, Tensor) else t
            if impl._buffer is None and id(impl) not in seen_t:
                seen_t.add(id(impl))
                targets.append(impl)
        if not targets:
            return None
        t0 = time.perf_counter()
        order, leaves, leaf_ids = self._collect(targets)
        # a random tensor is drawn once: whoever evaluates it first keeps it, so that a later
        # evaluation that reads it too (the backward pass of a dropout) sees the same numbers
        for node in order:
            if getattr(node.op, "draws_random", False):
                for o in node._refs:
                    if o is not None and o._buffer is None and id(o) not in seen_t:
                        seen_t.add(id(o))
                        targets.append(o)
        key = self._structure_key(order, leaves, leaf_ids, targets)
        ex = get_executor()
        bound = _PLAN_CACHE.get(key)
        if bound is None:
            _STATS["misses"] += 1
            t1 = time.perf_counter()
            plan = self._lower(order, leaves, targets, leaf_ids)
            bound = ex.bind(plan)
            _STATS["lower_ms"] += (time.perf_counter() - t1) * 1e3
            _PLAN_CACHE[key] = bound
            if len(_PLAN_CACHE) > _PLAN_CACHE_MAX:
                _PLAN_CACHE.popitem(last=False)
            if _DEBUG or _DEBUG_CACHE:
                print(f"[nabla_amd] plan cache MISS: {len(order)} ops -> {bound.plan.stats}")
        else:
            _STATS["hits"] += 1
            _PLAN_CACHE.move_to_end(key)
            if _DEBUG_CACHE:
                print(f"[nabla_amd] plan cache HIT ({len(order)} ops)")
        outs = bound.run([impl._buffer for impl in leaves])
        for impl, buf in zip(targets, outs):
            impl._buffer = buf
        self._cleanup(order, targets)
        self.epoch += 1
        if _DEBUG:
            print(f"[nabla_amd] evaluate: {len(order)} ops, {(time.perf_counter() - t0) * 1e3:.2f} ms host")
        return bound if return_model else None

    @staticmethod
    def _cleanup(order, targets) -> None:
        """Drop producer links of realized, untraced tensors so the recorded
        graph can be collected (engine.py:735-772)."""
        for impl in targets:
            if not impl.is_traced:
                impl.output_refs = None


_GRAPH_VAR: ContextVar[ComputeGraph | None] = ContextVar("nabla_amd_graph", default=None)


class _GraphProxy:
    """Context-local ComputeGraph (engine.py:920-1012)."""

    def _get(self) -> ComputeGraph:
        g = _GRAPH_VAR.get()
        if g is None:
            g = ComputeGraph()
            _GRAPH_VAR.set(g)
        return g

    def __getattr__(self, name: str):
        return getattr(self._get(), name)


GRAPH = _GraphProxy()
