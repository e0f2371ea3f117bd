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


class CompilationStats:
    """Counters of one compiled function, under the reference's names (compile.py:40-69): calls
    answered from the cache (``hits``), signatures traced for the first time (``misses``), calls
    that ran uncompiled (``fallbacks``), the milliseconds spent tracing and lowering, and those
    spent in cached calls.  ``specializations`` counts plans built for a new binding of
    symbolic dims inside a known signature."""

    _COUNTERS = ("hits", "misses", "fallbacks", "specializations", "cache_size")
    _CLOCKS = ("total_compile_time_ms", "total_cached_exec_time_ms")

    def __init__(self) -> None:
        for name in self._COUNTERS:
            setattr(self, name, 0)
        for name in self._CLOCKS:
            setattr(self, name, 0.0)

    def clock(self, name: str):
        """Context manager that adds the time spent inside it to the clock ``name``."""
        return _Stopwatch(self, name)

    @property
    def calls(self) -> int:
        return self.hits + self.misses + self.fallbacks

    @property
    def hit_rate(self) -> float:
        """Share of calls answered from the cache, in percent."""
        return 100.0 * self.hits / self.calls if self.calls else 0.0

    def __repr__(self) -> str:
        return (f"CompilationStats(hits={self.hits}, misses={self.misses}, "
                f"fallbacks={self.fallbacks}, hit_rate={self.hit_rate:.1f}%)")


class _Stopwatch:
    __slots__ = ("stats", "name", "t0")

    def __init__(self, stats: CompilationStats, name: str):
        self.stats, self.name = stats, name

    def __enter__(self):
        self.t0 = time.perf_counter()
        return self

    def __exit__(self, *exc) -> None:
        spent = (time.perf_counter() - self.t0) * 1e3
        setattr(self.stats, self.name, getattr(self.stats, self.name) + spent)


def _static_key(value: Any) -> Any:
    """A hashable stand-in for a non-tensor argument, equal for equal arguments: containers are
    rebuilt from the stand-ins of their items (a dict as its sorted items, a set as a
    frozenset), hashable objects stand for themselves, anything else for its type and repr."""
    if isinstance(value, dict):
        return ("dict", tuple(sorted((_static_key(k), _static_key(v)) for k, v in value.items())))
    if isinstance(value, (set, frozenset)):
        return ("set", frozenset(_static_key(v) for v in value))
    if isinstance(value, (list, tuple)):
        return tuple(_static_key(v) for v in value)
    try:
        hash(value)
    except TypeError:
        return (type(value).__qualname__, repr(value))
    return value


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
                statics.append(_static_key(x))
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
        known = entry is not None
        if known:
            self._cache.move_to_end(key)
            self._stats.hits += 1
        else:
            self._stats.misses += 1
            entry = self._cache[key] = _CachedModel()
            if len(self._cache) > self.max_cache_size:
                self._cache.popitem(last=False)
        spec = entry.specializations.get(concrete)
        if spec is not None:
            with self._stats.clock("total_cached_exec_time_ms"):
                return self._execute_cached(spec, flat)
        if known:
            self._stats.specializations += 1
        with self._stats.clock("total_compile_time_ms"):
            spec = entry.specializations[concrete] = self._trace_and_compile(args, kwargs, flat)
        return spec._first_result

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
