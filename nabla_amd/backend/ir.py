"""Lowering IR: what ``Operation.kernel`` emits instead of MAX graph ops.

In the reference every ``kernel(args, kwargs)`` receives MAX ``TensorValue``s
and calls ``max.graph.ops.*`` (nabla/ops/base.py:127-137, engine.py:832-847).
Here it receives ``Value``s and calls the builder functions of this module;
the result is a small SSA graph that the planner turns into kernel launches.

Node kinds
    input                       a realized leaf buffer
    ew        fn, n inputs      elementwise, all tensor inputs have the output shape
    reduce    fn, axis          single axis, keepdims (reduction.py:147-245)
    reshape / broadcast / permute / slice      pure views
    fill / iota                 generators
    tril                        keep the lower triangle (creation.py:225-274)
    matmul, conv2d, conv2d_dgrad, conv2d_wgrad, maxpool2d, maxpool2d_bwd,
    gather, argreduce, pad, concat, slice_update, custom
"""
from __future__ import annotations

from contextvars import ContextVar
from typing import Any, Sequence

from ..core.dtype import DType, promote


class Value:
    __slots__ = ("shape", "dtype", "node", "index", "id")

    def __init__(self, shape, dtype: DType, node: "Node", index: int, vid: int):
        self.shape = tuple(int(d) for d in shape)
        self.dtype = dtype
        self.node = node
        self.index = index
        self.id = vid

    @property
    def rank(self) -> int:
        return len(self.shape)

    @property
    def type(self):
        """(shape, dtype) pair; what ``call_custom_kernel`` takes as an out_type."""
        return (self.shape, self.dtype)

    def numel(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n

    def __repr__(self) -> str:
        return f"%{self.id}:{self.dtype.name}{list(self.shape)}"


class Node:
    __slots__ = ("kind", "fn", "inputs", "attrs", "outputs", "pos")

    def __init__(self, kind: str, fn: str | None, inputs: Sequence[Value], attrs: dict, pos: int):
        self.kind = kind
        self.fn = fn
        self.inputs = list(inputs)
        self.attrs = attrs
        self.outputs: list[Value] = []
        self.pos = pos

    def __repr__(self) -> str:
        fn = f".{self.fn}" if self.fn else ""
        return f"{self.outputs} = {self.kind}{fn}({self.inputs}) {self.attrs or ''}"


class Builder:
    def __init__(self) -> None:
        self.nodes: list[Node] = []
        self.inputs: list[Value] = []
        self._n_values = 0
        self._cse: dict = {}

    def add(self, kind: str, inputs: Sequence[Value], outs: Sequence[tuple], fn: str | None = None,
            **attrs: Any) -> list[Value]:
        # common-subexpression elimination: the same pure op on the same values is
        # emitted once (a forward chain traced twice -- once for its value, once
        # under grad -- collapses to one)
        key = None
        if kind not in ("input", "custom"):
            try:
                key = (kind, fn, tuple(v.id for v in inputs),
                       tuple(sorted((k, _hashable(v)) for k, v in attrs.items())),
                       tuple((tuple(s), d) for s, d in outs))
                hit = self._cse.get(key)
                if hit is not None:
                    return hit.outputs
            except TypeError:
                key = None
        if kind in ("ew", "reduce", "argreduce", "matmul", "fill"):
            for _, dtype in outs:
                if dtype is DType.uint8:
                    # the kernels store one-byte results as 0 / 1 (bool); uint8 is for data that
                    # comes in from the host (quantised weights) and is cast before arithmetic
                    raise TypeError(f"'{fn or kind}' would produce uint8: cast uint8 data to "
                                    "int32 or a float type first")
        node = Node(kind, fn, inputs, attrs, len(self.nodes))
        for i, (shape, dtype) in enumerate(outs):
            node.outputs.append(Value(shape, dtype, node, i, self._n_values))
            self._n_values += 1
        self.nodes.append(node)
        if key is not None:
            self._cse[key] = node
        return node.outputs


def _hashable(v):
    if isinstance(v, Value):
        return ("%", v.id)
    if isinstance(v, (list, tuple)):
        return tuple(_hashable(x) for x in v)
    return v


_CURRENT: ContextVar[Builder | None] = ContextVar("nbk_ir_builder", default=None)


def current() -> Builder:
    b = _CURRENT.get()
    if b is None:
        raise RuntimeError("no lowering in progress: kernel() may only run inside evaluate()")
    return b


class building:
    """Context manager that makes ``builder`` the target of the functions below."""

    def __init__(self, builder: Builder):
        self.builder = builder

    def __enter__(self) -> Builder:
        self._tok = _CURRENT.set(self.builder)
        return self.builder

    def __exit__(self, *exc) -> None:
        _CURRENT.reset(self._tok)


def _numel(shape) -> int:
    n = 1
    for d in shape:
        n *= d
    return n


# ---- leaves ---------------------------------------------------------------------
def input(shape, dtype: DType) -> Value:  # noqa: A001 - mirrors graph "input"
    b = current()
    v = b.add("input", [], [(shape, dtype)])[0]
    b.inputs.append(v)
    return v


# ---- elementwise ------------------------------------------------------------------
UNARY_FNS = {"mov", "neg", "relu", "exp", "log", "sqrt", "rsqrt", "erf", "gelu", "dgelu", "tanh", "sigmoid", "sin", "cos",
             "abs", "not", "trunc", "nez"}
BINARY_FNS = {"add", "sub", "mul", "div", "max", "min", "gt", "ge", "eq", "ne", "lt", "le", "pow",
              "and", "or"}
TERNARY_FNS = {"where", "fma"}
BOOL_FNS = {"gt", "ge", "eq", "ne", "lt", "le", "and", "or", "not", "nez"}


def ew(fn: str, *xs: Value | float | int, dtype: DType | None = None) -> Value:
    """Elementwise ``fn``.  Tensor inputs must already share one shape (the
    reference makes broadcasts explicit before the op, base.py:645-652);
    Python numbers are immediates."""
    tensors = [x for x in xs if isinstance(x, Value)]
    if not tensors:
        raise ValueError(f"ew.{fn}: needs at least one tensor input")
    shape = tensors[0].shape
    for t in tensors[1:]:
        if t.shape != shape:
            raise ValueError(f"ew.{fn}: operand shapes differ: {[t.shape for t in tensors]}")
    arity = 1 if fn in UNARY_FNS else 2 if fn in BINARY_FNS else 3 if fn in TERNARY_FNS else 0
    if arity == 0:
        raise ValueError(f"ew: unknown function '{fn}'")
    if len(xs) != arity:
        raise ValueError(f"ew.{fn}: expected {arity} operands, got {len(xs)}")
    if dtype is None:
        if fn in BOOL_FNS:
            dtype = DType.bool
        elif fn == "where":
            vals = [x.dtype for x in xs[1:] if isinstance(x, Value)]
            dtype = vals[0] if len(vals) == 1 else promote(vals[0], vals[1]) if vals else DType.float32
        else:
            dtype = tensors[0].dtype
            for t in tensors[1:]:
                dtype = promote(dtype, t.dtype)
    # int64 values meet floats as floats: an int64 operand of a floating-point operation or of a
    # comparison with a float is converted first (its own exact step), so that whatever touches
    # int64 storage afterwards is either pure integer work or a plain float kernel
    if fn == "where" and isinstance(xs[0], Value) and xs[0].dtype is DType.int64:
        xs = (cast(xs[0], DType.bool),) + tuple(xs[1:])
        tensors = [x for x in xs if isinstance(x, Value)]
    floats = [t.dtype for t in tensors if t.dtype.is_float()]
    if fn not in ("mov", "trunc", "nez") and any(t.dtype is DType.int64 for t in tensors) and \
            (dtype.is_float() or (fn in BOOL_FNS and floats)):
        to = dtype if dtype.is_float() else floats[0]
        xs = tuple(cast(x, to) if isinstance(x, Value) and x.dtype is DType.int64 else x for x in xs)
        tensors = [x for x in xs if isinstance(x, Value)]
    operands = tuple(x if isinstance(x, Value) else float(x) for x in xs)
    return current().add("ew", tensors, [(shape, dtype)], fn=fn, operands=operands)[0]


def cast(x: Value, dtype: DType) -> Value:
    if x.dtype is dtype:
        return x
    if dtype is DType.bool:
        return ew("nez", x, dtype=dtype)
    if dtype.is_integral() and x.dtype.is_float():
        return ew("trunc", x, dtype=dtype)
    return ew("mov", x, dtype=dtype)


def pin_after(x: Value, dep: Value) -> Value:
    """``x`` unchanged, but to the planner an elementwise function of ``x`` and ``dep``: whatever is
    computed from the result cannot be scheduled before ``dep`` exists.  A backward op uses it on
    a forward value it re-reads, with its cotangent as ``dep``: without it the planner, which
    fuses a node into the group of its producers, would pull the cotangent-independent part of
    the backward arithmetic into the forward kernel and store full-size intermediates there."""
    d = dep if dep.shape == x.shape else broadcast_to(dep, x.shape)
    return current().add("ew", [x, d], [(x.shape, x.dtype)], fn="mov", operands=(x,))[0]


def tril(x: Value, k: int = 0, upper: bool = False) -> Value:
    """Zero everything above (below, if ``upper``) the k-th diagonal of the last two axes."""
    if x.rank < 2:
        raise ValueError("tril/triu needs rank >= 2")
    return current().add("tril", [x], [(x.shape, x.dtype)], k=int(k), upper=bool(upper))[0]


# ---- reductions ---------------------------------------------------------------------
def reduce(fn: str, x: Value, axis: int) -> Value:  # noqa: A001
    """Single-axis keepdims reduction; ``fn`` in {sum, max, min}."""
    if fn not in ("sum", "max", "min"):
        raise ValueError(f"reduce: unknown kind '{fn}'")
    if axis < 0:
        axis += x.rank
    if not 0 <= axis < x.rank:
        raise ValueError(f"reduce: axis {axis} out of range for rank {x.rank}")
    shape = x.shape[:axis] + (1,) + x.shape[axis + 1:]
    return current().add("reduce", [x], [(shape, x.dtype)], fn=fn, axis=axis)[0]


def argreduce(fn: str, x: Value, axis: int) -> Value:
    """Index (int64) of the first max / min along ``axis``, keepdims."""
    if axis < 0:
        axis += x.rank
    shape = x.shape[:axis] + (1,) + x.shape[axis + 1:]
    return current().add("argreduce", [x], [(shape, DType.int64)], fn=fn, axis=axis)[0]


# ---- views --------------------------------------------------------------------------
def reshape(x: Value, shape) -> Value:
    shape = tuple(int(d) for d in shape)
    if -1 in shape:
        known = _numel([d for d in shape if d != -1])
        shape = tuple(x.numel() // max(known, 1) if d == -1 else d for d in shape)
    if _numel(shape) != x.numel():
        raise ValueError(f"reshape: cannot view {x.shape} as {shape}")
    if shape == x.shape:
        return x
    return current().add("reshape", [x], [(shape, x.dtype)])[0]


def broadcast_to(x: Value, shape) -> Value:
    shape = tuple(int(d) for d in shape)
    if shape == x.shape:
        return x
    if len(shape) < x.rank:
        raise ValueError(f"broadcast_to: cannot broadcast {x.shape} to {shape}")
    for a, b in zip(x.shape[::-1], shape[::-1]):
        if a != b and a != 1:
            raise ValueError(f"broadcast_to: cannot broadcast {x.shape} to {shape}")
    return current().add("broadcast", [x], [(shape, x.dtype)])[0]


def permute(x: Value, perm) -> Value:
    perm = tuple(int(p) % max(x.rank, 1) for p in perm)
    if sorted(perm) != list(range(x.rank)):
        raise ValueError(f"permute: {perm} is not a permutation of rank {x.rank}")
    if perm == tuple(range(x.rank)):
        return x
    shape = tuple(x.shape[p] for p in perm)
    return current().add("permute", [x], [(shape, x.dtype)], perm=perm)[0]


def slice(x: Value, starts, stops, steps=None) -> Value:  # noqa: A001
    steps = tuple(steps) if steps is not None else (1,) * x.rank
    starts, stops = tuple(starts), tuple(stops)
    shape = []
    for d, a, b, s in zip(x.shape, starts, stops, steps):
        if s <= 0 or not (0 <= a <= b <= d):
            raise ValueError(f"slice: bad range [{a}:{b}:{s}] for extent {d}")
        shape.append((b - a + s - 1) // s)
    shape = tuple(shape)
    if shape == x.shape and all(s == 1 for s in steps):
        return x
    return current().add("slice", [x], [(shape, x.dtype)], starts=starts, steps=steps)[0]


# ---- generators -----------------------------------------------------------------------
def fill(shape, dtype: DType, value: float) -> Value:
    return current().add("fill", [], [(tuple(shape), dtype)], value=float(value))[0]


def iota(n: int, dtype: DType, start: float = 0.0, step: float = 1.0, lead=()) -> Value:
    """``start + step * j`` along an axis of ``n`` entries; with ``lead`` the same row repeated
    over leading dims ``lead`` (shape ``lead + (n,)``), which lets it sit inside the kernel of
    whatever reads it instead of being a tensor of its own."""
    shape = tuple(int(d) for d in lead) + (int(n),)
    return current().add("iota", [], [(shape, dtype)], start=float(start), step=float(step))[0]


# ---- contractions ---------------------------------------------------------------------
def matmul(a: Value, b: Value) -> Value:
    """``(..., M, K) @ (..., K, N)`` with identical leading dims (binary.py:197-287)."""
    if a.rank < 2 or b.rank < 2:
        raise ValueError("matmul: operands must have rank >= 2 (promote 1-D operands first)")
    if a.shape[-1] != b.shape[-2]:
        raise ValueError(f"matmul: contraction mismatch {a.shape} @ {b.shape}")
    if a.shape[:-2] != b.shape[:-2]:
        raise ValueError(f"matmul: batch dims differ {a.shape} vs {b.shape}")
    shape = a.shape[:-1] + (b.shape[-1],)
    return current().add("matmul", [a, b], [(shape, promote(a.dtype, b.dtype))])[0]


def matmul_nf4(x: Value, codes: Value, scales: Value, w_shape, block: int, transpose: bool) -> Value:
    """``x @ W`` (or ``x @ W^T``) for a weight of shape ``w_shape`` stored as NF4 codes (uint8, one per
    weight, row-major) and one fp32 scale per ``block`` consecutive codes."""
    rows, cols = (int(d) for d in w_shape)
    k, n = (cols, rows) if transpose else (rows, cols)
    if x.rank < 1 or x.shape[-1] != k:
        raise ValueError(f"matmul_nf4: contraction mismatch {x.shape} against a weight {tuple(w_shape)}"
                         f"{' transposed' if transpose else ''}")
    if codes.numel() != rows * cols or scales.numel() * int(block) != rows * cols:
        raise ValueError("matmul_nf4: codes / scales do not match the weight's shape and block length")
    return current().add("matmul_nf4", [x, codes, scales], [(x.shape[:-1] + (n,), x.dtype)],
                         w_shape=(rows, cols), block=int(block), transpose=bool(transpose))[0]


def conv_out_size(n: int, k: int, stride: int, pad_lo: int, pad_hi: int) -> int:
    return (n + pad_lo + pad_hi - k) // stride + 1


def conv2d(x: Value, w: Value, bias: Value | None, stride, padding) -> Value:
    """NHWC x HWIO correlation; padding = (top, bottom, left, right)."""
    n, h, wd, cin = x.shape
    r, s, cin2, cout = w.shape
    if cin != cin2:
        raise ValueError(f"conv2d: input channels {cin} vs filter {cin2}")
    ho = conv_out_size(h, r, stride[0], padding[0], padding[1])
    wo = conv_out_size(wd, s, stride[1], padding[2], padding[3])
    ins = [x, w] + ([bias] if bias is not None else [])
    return current().add("conv2d", ins, [((n, ho, wo, cout), x.dtype)], stride=tuple(stride),
                         padding=tuple(padding), has_bias=bias is not None)[0]


def conv2d_dgrad(dy: Value, w: Value, x_shape, stride, padding) -> Value:
    return current().add("conv2d_dgrad", [dy, w], [(tuple(x_shape), dy.dtype)], stride=tuple(stride),
                         padding=tuple(padding))[0]


def conv2d_wgrad(x: Value, dy: Value, w_shape, stride, padding) -> Value:
    return current().add("conv2d_wgrad", [x, dy], [(tuple(w_shape), x.dtype)], stride=tuple(stride),
                         padding=tuple(padding))[0]


def maxpool2d(x: Value, kernel, stride, padding) -> Value:
    n, h, w, c = x.shape
    ho = (h + padding[0] + padding[1] - kernel[0]) // stride[0] + 1
    wo = (w + padding[2] + padding[3] - kernel[1]) // stride[1] + 1
    return current().add("maxpool2d", [x], [((n, ho, wo, c), x.dtype)], kernel=tuple(kernel),
                         stride=tuple(stride), padding=tuple(padding))[0]


def maxpool2d_bwd(x: Value, y: Value, dy: Value, kernel, stride, padding) -> Value:
    return current().add("maxpool2d_bwd", [x, y, dy], [(x.shape, x.dtype)], kernel=tuple(kernel),
                         stride=tuple(stride), padding=tuple(padding))[0]


def avgpool2d(x: Value, kernel, stride, padding) -> Value:
    n, h, w, c = x.shape
    ho = (h + padding[0] + padding[1] - kernel[0]) // stride[0] + 1
    wo = (w + padding[2] + padding[3] - kernel[1]) // stride[1] + 1
    return current().add("avgpool2d", [x], [((n, ho, wo, c), x.dtype)], kernel=tuple(kernel),
                         stride=tuple(stride), padding=tuple(padding))[0]


def avgpool2d_bwd(dy: Value, x_shape, kernel, stride, padding) -> Value:
    return current().add("avgpool2d_bwd", [dy], [(tuple(x_shape), dy.dtype)], kernel=tuple(kernel),
                         stride=tuple(stride), padding=tuple(padding), x_shape=tuple(x_shape))[0]


# ---- indexing / movement ------------------------------------------------------------------
def gather(table: Value, idx: Value, axis: int) -> Value:
    if axis < 0:
        axis += table.rank
    shape = table.shape[:axis] + idx.shape + table.shape[axis + 1:]
    return current().add("gather", [table, idx], [(shape, table.dtype)], axis=axis)[0]


def scatter(x: Value, idx: Value, updates: Value, axis: int) -> Value:
    """Copy of ``x`` whose rows ``idx`` along ``axis`` are replaced by ``updates``."""
    if axis < 0:
        axis += x.rank
    want = x.shape[:axis] + idx.shape + x.shape[axis + 1:]
    if tuple(updates.shape) != tuple(want):
        raise ValueError(f"scatter: updates of shape {updates.shape}, expected {want}")
    return current().add("scatter", [x, idx, updates], [(x.shape, x.dtype)], axis=axis)[0]


def pad(x: Value, lo, hi, value: float = 0.0) -> Value:
    shape = tuple(d + a + b for d, a, b in zip(x.shape, lo, hi))
    if shape == x.shape:
        return x
    return current().add("pad", [x], [(shape, x.dtype)], lo=tuple(lo), hi=tuple(hi),
                         value=float(value))[0]


def concat(xs: Sequence[Value], axis: int) -> Value:
    xs = list(xs)
    if axis < 0:
        axis += xs[0].rank
    base = xs[0].shape
    total = 0
    dtype = xs[0].dtype
    for x in xs:
        if x.shape[:axis] != base[:axis] or x.shape[axis + 1:] != base[axis + 1:]:
            raise ValueError(f"concat: shapes differ off-axis: {[v.shape for v in xs]}")
        total += x.shape[axis]
        dtype = promote(dtype, x.dtype)
    shape = base[:axis] + (total,) + base[axis + 1:]
    if len(xs) == 1:
        return xs[0]
    return current().add("concat", xs, [(shape, dtype)], axis=axis)[0]


def slice_update(x: Value, update: Value, starts) -> Value:
    """Copy of ``x`` with the window at ``starts`` replaced by ``update``."""
    return current().add("slice_update", [x, update], [(x.shape, x.dtype)], starts=tuple(starts))[0]


def custom(name: str, library: str, inputs: Sequence[Value], out_types: Sequence[tuple]) -> list[Value]:
    return current().add("custom", list(inputs), [(tuple(s), d) for s, d in out_types], name=name,
                         library=str(library))


# ---- fused attention ----------------------------------------------------------------------
def attention(q: Value, k: Value, v: Value, scale: float, causal: bool) -> list[Value]:
    """[B, H, S, hd] heads -> (output [B, H, S, hd], log-sum-exp of the score rows [B, H, S],
    what rounding the output to its 16-bit type cut off [B, H, S, hd], for the backward pass)."""
    if not (q.shape == k.shape == v.shape) or q.rank != 4:
        raise ValueError(f"attention: q, k, v must share one [B, H, S, hd] shape, got "
                         f"{q.shape}, {k.shape}, {v.shape}")
    return current().add("attention", [q, k, v],
                         [(q.shape, q.dtype), (q.shape[:-1], DType.float32), (q.shape, q.dtype)],
                         scale=float(scale), causal=bool(causal))


def attention_bwd(q: Value, k: Value, v: Value, o: Value, lse: Value, o_lo: Value, dout: Value,
                  scale: float, causal: bool) -> list[Value]:
    """Gradients (dq, dk, dv) of ``attention`` from its inputs, its three outputs and d(output)."""
    return current().add("attention_bwd", [q, k, v, o, lse, o_lo, dout], [(q.shape, q.dtype)] * 3,
                         scale=float(scale), causal=bool(causal))


# ---- random tensors -------------------------------------------------------------------------
RANDOM_MODES = ("uniform", "normal", "keep")


def random(shape, dtype: DType, mode: str, a: float, b: float = 0.0) -> Value:  # noqa: A001
    """A tensor drawn from the device generator: ``uniform`` on [a, b), ``normal`` with mean a
    and deviation b, or ``keep``: 1 where a uniform [0, 1) draw exceeds ``a``, else 0 (the mask
    of dropout with rate a).  Every call is a stream of its own: two calls with equal
    arguments give different tensors, and one value read in two places is one tensor."""
    if mode not in RANDOM_MODES:
        raise ValueError(f"random: unknown mode '{mode}'")
    if not (dtype.is_float() or (mode == "keep" and dtype is DType.bool)):
        raise TypeError(f"random.{mode}: cannot draw {dtype}")
    shape = tuple(int(d) for d in shape)
    bld = current()
    stream = getattr(bld, "n_random", 0)
    bld.n_random = stream + 1
    return bld.add("random", [], [(shape, dtype)], mode=mode, a=float(a), b=float(b), stream=stream)[0]


# ---- optimizer updates over a list of parameters ---------------------------------------------
def _check_update_list(who: str, groups: Sequence[Sequence[Value]]) -> DType:
    first = groups[0][0]
    for vals in groups:
        for v in vals:
            if v.dtype is not first.dtype or v.shape != vals[0].shape:
                raise ValueError(f"{who}: every tensor of a parameter shares its shape, and all of "
                                 f"them one dtype; got {v.shape} {v.dtype} beside {vals[0].shape} "
                                 f"{first.dtype}")
    if first.dtype not in (DType.float32, DType.bfloat16):
        raise TypeError(f"{who}: float32 or bfloat16 parameters, got {first.dtype}")
    return first.dtype


def adamw_multi(params: Sequence[Value], grads: Sequence[Value], ms: Sequence[Value],
                vs: Sequence[Value], step: Value | float, *, lr: float, beta1: float, beta2: float,
                eps: float, weight_decay: float, bias_correction: bool) -> list[Value]:
    """One AdamW step for every parameter of the list: ``[p'_0, m'_0, v'_0, p'_1, ...]``.  ``step``
    (the number of this step, from 1) is a number or a 0-d float32 value."""
    groups = list(zip(params, grads, ms, vs))
    _check_update_list("adamw_multi", groups)
    inputs = [x for g in groups for x in g]
    attrs = dict(lr=float(lr), beta1=float(beta1), beta2=float(beta2), eps=float(eps),
                 weight_decay=float(weight_decay), bias_correction=bool(bias_correction),
                 n=len(groups), step=None)
    if isinstance(step, Value):
        if step.numel() != 1 or step.dtype is not DType.float32:
            raise TypeError(f"adamw_multi: the step counter is one float32 value, got {step}")
        inputs.append(step)
    else:
        attrs["step"] = float(step)
    outs = [(p.shape, p.dtype) for p in params for _ in range(3)]
    return current().add("adamw_multi", inputs, outs, **attrs)


def sgd_multi(params: Sequence[Value], grads: Sequence[Value], bufs: Sequence[Value] | None, *,
              lr: float, momentum: float, weight_decay: float) -> list[Value]:
    """One SGD step for every parameter of the list.  With momentum ``bufs`` holds the momentum
    buffers and the result is ``[p'_0, buf'_0, p'_1, ...]``; without, ``[p'_0, p'_1, ...]``."""
    with_mom = float(momentum) != 0.0
    if with_mom and bufs is None:
        raise ValueError("sgd_multi: momentum needs the momentum buffers")
    groups = list(zip(params, grads, bufs)) if with_mom else list(zip(params, grads))
    _check_update_list("sgd_multi", groups)
    inputs = [x for g in groups for x in g]
    outs = [(p.shape, p.dtype) for p in params for _ in range(2 if with_mom else 1)]
    return current().add("sgd_multi", inputs, outs, lr=float(lr), momentum=float(momentum),
                         weight_decay=float(weight_decay), n=len(groups))
