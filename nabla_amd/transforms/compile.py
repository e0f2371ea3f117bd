"""``@compile``: signature-keyed cache of lowered steps.

Mirrors nabla/transforms/compile.py: ``CompilationStats`` (40-69), the cache key
of tensor signatures with ``$name`` symbols for dynamic dims + static values +
pytree structure (72-78, 207-268), ``CompiledFunction.__call__`` (172-205),
trace-and-compile on a miss (303-362, 387-484), cached replay through an input
plan of ``("arg", i) | ("captured", buffer)`` entries (508-555) and LRU
eviction (486-492).

A cached entry replays its launch plan without re-running the Python function.
Plans are specialised to concrete shapes, so an entry whose key holds symbolic
dims keeps one plan per concrete binding of those symbols; a new binding
re-traces inside the same entry and still counts as a hit of the signature,
which is what the reference's dynamic-dim tests observe.
"""
from __future__ import annotations

import time
from collections import OrderedDict
from dataclasses import dataclass, field
from typing import Any, Callable

from .. import config
from ..core.engine import GRAPH, ComputeGraph
from ..core.pytree import PyTreeDef, tree_flatten, tree_unflatten
from ..core.tensor import Tensor, TensorImpl


@dataclass
class CompilationStats:
    hits: int = 0
    misses: int = 0
    fallbacks: int = 0
    total_compile_time_ms: float = 0.0
    total_cached_exec_time_ms: float = 0.0
    cache_size: int = 0
    specializations: int = 0  # plans built for new bindings of symbolic dims

    @property
    def hit_rate(self) -> float:
        total = self.hits + self.misses + self.fallbacks
        return (self.hits / total * 100) if total > 0 else 0.0

    def __repr__(self) -> str:
        return (f"CompilationStats(hits={self.hits}, misses={self.misses}, "
                f"fallbacks={self.fallbacks}, hit_rate={self.hit_rate:.1f}%)")


@dataclass(frozen=True)
class _CacheKey:
    tensor_sigs: tuple
    static_vals: tuple
    treedef: PyTreeDef


@dataclass
class _Specialization:
    bound: Any                      # BoundPlan or None when nothing had to be computed
    input_plan: list                # ("arg", flat index) | ("captured", buffer)
    output_treedef: PyTreeDef
    output_slots: list              # per flat output: ("plan", i) | ("arg", flat idx) | ("static", v) | ("captured", buffer, shape, dtype)
    output_meta: list               # (shape, dtype) of plan outputs


@dataclass
class _CachedModel:
    specializations: dict = field(default_factory=dict)


class CompiledFunction:
    """A function whose lowered launch plan is cached by argument signature."""

    def __init__(self, fn: Callable, *, fullgraph: bool = False, max_cache_size: int = 64,
                 dynamic_dims: dict[int, dict[int, str]] | None = None):
        self.__wrapped__ = fn
        self.__name__ = getattr(fn, "__name__", repr(fn))
        self.__doc__ = fn.__doc__
        self.fullgraph = fullgraph
        self.max_cache_size = max_cache_size
        self.dynamic_dims = dynamic_dims or {}
        self._cache: "OrderedDict[_CacheKey, _CachedModel]" = OrderedDict()
        self._stats = CompilationStats()

    @property
    def stats(self) -> CompilationStats:
        self._stats.cache_size = len(self._cache)
        return self._stats

    def clear_cache(self) -> None:
        self._cache.clear()

    # ---- keys ---------------------------------------------------------------
    def _make_hashable_static(self, value: Any) -> Any:
        if isinstance(value, (str, bytes, int, float, bool, type(None))):
            return value
        if isinstance(value, (tuple, list)):
            return tuple(self._make_hashable_static(v) for v in value)
        if isinstance(value, dict):
            return tuple(sorted((self._make_hashable_static(k), self._make_hashable_static(v))
                                for k, v in value.items()))
        if isinstance(value, (set, frozenset)):
            return frozenset(self._make_hashable_static(v) for v in value)
        try:
            hash(value)
            return value
        except TypeError:
            return (type(value).__qualname__, repr(value))

    def _tensor_signature(self, t: Tensor, arg_idx: int):
        shape: list = list(t.shape)
        if arg_idx in self.dynamic_dims:
            for dim_idx, sym in self.dynamic_dims[arg_idx].items():
                if dim_idx < len(shape):
                    shape[dim_idx] = f"${sym}"
        return (tuple(shape), str(t.dtype), None)

    def _build_keys(self, flat: list):
        sigs, statics, concrete = [], [], []
        ti = 0
        for x in flat:
            if isinstance(x, Tensor):
                sigs.append(self._tensor_signature(x, ti))
                concrete.append(tuple(x.shape))
                ti += 1
            else:
                statics.append(self._make_hashable_static(x))
        return tuple(sigs), tuple(statics), tuple(concrete)

    # ---- call ---------------------------------------------------------------
    def __call__(self, *args: Any, **kwargs: Any):
        flat, treedef = tree_flatten((args, kwargs))
        pending = [x for x in flat if isinstance(x, Tensor) and not x.real]
        if pending:
            GRAPH.evaluate(*pending)
        sigs, statics, concrete = self._build_keys(flat)
        key = _CacheKey(sigs, statics, treedef)
        entry = self._cache.get(key)
        if entry is None:
            self._stats.misses += 1
            entry = _CachedModel()
            self._cache[key] = entry
            if len(self._cache) > self.max_cache_size:
                self._cache.popitem(last=False)
            t0 = time.perf_counter()
            spec = self._trace_and_compile(args, kwargs, flat)
            entry.specializations[concrete] = spec
            self._stats.total_compile_time_ms += (time.perf_counter() - t0) * 1e3
            return spec._first_result
        self._cache.move_to_end(key)
        self._stats.hits += 1
        spec = entry.specializations.get(concrete)
        if spec is None:
            self._stats.specializations += 1
            t0 = time.perf_counter()
            spec = self._trace_and_compile(args, kwargs, flat)
            entry.specializations[concrete] = spec
            self._stats.total_compile_time_ms += (time.perf_counter() - t0) * 1e3
            return spec._first_result
        t0 = time.perf_counter()
        out = self._execute_cached(spec, flat)
        self._stats.total_cached_exec_time_ms += (time.perf_counter() - t0) * 1e3
        return out

    # ---- miss ---------------------------------------------------------------
    def _trace_and_compile(self, args, kwargs, flat) -> _Specialization:
        arg_pos = {id(x._impl): i for i, x in enumerate(flat) if isinstance(x, Tensor)}
        tok = config.set_flag("TRACING", True)
        try:
            result = self.__wrapped__(*args, **kwargs)
        finally:
            config.reset_flag("TRACING", tok)
        out_flat, out_treedef = tree_flatten(result)
        targets: list[TensorImpl] = []
        target_idx: dict[int, int] = {}
        slots = []
        for o in out_flat:
            if isinstance(o, Tensor):
                impl = o._impl
                if impl._buffer is not None:
                    if id(impl) in arg_pos:
                        slots.append(("arg", arg_pos[id(impl)]))
                    else:
                        slots.append(("captured", impl._buffer, impl.shape, impl.dtype))
                else:
                    if id(impl) not in target_idx:
                        target_idx[id(impl)] = len(targets)
                        targets.append(impl)
                    slots.append(("plan", target_idx[id(impl)]))
            else:
                slots.append(("static", o))
        bound = None
        input_plan: list = []
        meta = [(t.shape, t.dtype) for t in targets]
        if targets:
            order, leaves, _ = ComputeGraph._collect(targets)
            for leaf in leaves:
                if id(leaf) in arg_pos:
                    input_plan.append(("arg", arg_pos[id(leaf)]))
                else:
                    input_plan.append(("captured", leaf._buffer))
            bound = GRAPH.evaluate(*[Tensor(impl=t) for t in targets], return_model=True)
        spec = _Specialization(bound, input_plan, out_treedef, slots, meta)
        spec._first_result = result  # type: ignore[attr-defined]
        return spec

    # ---- hit ----------------------------------------------------------------
    def _execute_cached(self, spec: _Specialization, flat: list):
        outs = []
        if spec.bound is not None:
            bufs = []
            for kind, v in spec.input_plan:
                bufs.append(flat[v]._impl._buffer if kind == "arg" else v)
            outs = spec.bound.run(bufs)
        leaves = []
        for slot in spec.output_slots:
            k = slot[0]
            if k == "plan":
                shape, dtype = spec.output_meta[slot[1]]
                leaves.append(Tensor(impl=TensorImpl(shape, dtype, buffer=outs[slot[1]])))
            elif k == "arg":
                leaves.append(flat[slot[1]])
            elif k == "captured":
                leaves.append(Tensor(impl=TensorImpl(slot[2], slot[3], buffer=slot[1])))
            else:
                leaves.append(slot[1])
        return tree_unflatten(spec.output_treedef, leaves)


def compile(fn: Callable | None = None, *, fullgraph: bool = False, max_cache_size: int = 64,  # noqa: A001
            dynamic_dims: dict[int, dict[int, str]] | None = None):
    """Compile a function for cached execution; usable as ``@compile`` or
    ``@compile(dynamic_dims={0: {0: "batch"}})``."""
    if fn is None:
        return lambda f: compile(f, fullgraph=fullgraph, max_cache_size=max_cache_size,
                                 dynamic_dims=dynamic_dims)
    return CompiledFunction(fn, fullgraph=fullgraph, max_cache_size=max_cache_size,
                            dynamic_dims=dynamic_dims)
