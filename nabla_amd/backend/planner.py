"""Lowering pass: IR graph -> launch plan.

This is the step that replaces "replay the trace into a MAX graph and let
``InferenceSession.load`` compile it" (nabla/core/graph/engine.py:575-663).

Passes
  1. dead-code elimination from the requested outputs;
  2. fusion: elementwise ops, last-axis reductions, tril masks and iotas that
     share an iteration domain ``lead x C`` are grouped into one row program
     each (softmax, layer_norm, cross-entropy and their backward graphs fuse
     this way without being pattern-matched); a node joins the group of one of
     its producers unless that would make the group graph cyclic;
  3. view folding: reshape / broadcast / permute / slice never run as kernels;
     they become offsets and strides of the consumers' operands.  A strided
     copy is inserted only where a consumer cannot take the view;
  4. code generation of row programs (phases, recomputation instead of
     spilling, register allocation, LDS staging of rows read in several phases);
  5. buffer assignment: intermediate buffers live in one arena with
     liveness-based offsets, outputs get allocations of their own.
"""
from __future__ import annotations

import heapq
import math
from dataclasses import dataclass, field
from typing import Any, Sequence

from ..core.dtype import DType
from . import ir, isa

FUSABLE = ("ew", "reduce", "tril", "iota")
#: values of these types live in row-program registers as int32, not as fp32
INT_REG_DTYPES = (DType.int32, DType.int64)
VIEW_KINDS = ("reshape", "broadcast", "permute", "slice")


def _wgrad_workspace_bytes(xs, ws, ys, n_cus: int = 256) -> int:
    """Scratch for the K-split partial sums of the filter gradient; the same rule as
    nbk_conv2d_wgrad_workspace() for a 256-CU device (the kernel falls back to an
    unsplit product if it is handed less than it wants)."""
    r, s_, cin, cout = ws
    m, k = r * s_ * cin, ys[0] * ys[1] * ys[2]
    tiles = ((m + 127) // 128) * ((cout + 127) // 128)
    want = max(1, min(2 * n_cus // tiles, max(k // 64, 1)))
    kps = ((k + want - 1) // want + 15) // 16 * 16
    splits = (k + kps - 1) // kps
    return 0 if splits <= 1 else splits * m * cout * 4


class FusionLimit(Exception):
    """A fused group does not fit the row-program limits; planning retries smaller."""


# --------------------------------------------------------------------------- data
def _as_stored(value: float, dtype: DType) -> float:
    """``value`` after one rounding to ``dtype`` (what a kernel reading the stored constant sees)."""
    import numpy as np
    if dtype is DType.bfloat16:
        bits = np.array([value], np.float32).view(np.uint32)
        if np.isfinite(value):
            bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & np.uint32(0xFFFF0000)
        return float(bits.astype(np.uint32).view(np.float32)[0])
    if dtype is DType.float16:
        return float(np.float16(value))
    if dtype is DType.float32:
        return float(np.float32(value))
    return value


def _numel(shape) -> int:
    n = 1
    for d in shape:
        n *= d
    return n


def contiguous_strides(shape) -> tuple[int, ...]:
    st = []
    acc = 1
    for d in reversed(shape):
        st.append(acc)
        acc *= max(d, 1)
    return tuple(reversed(st))


@dataclass
class Buf:
    id: int
    numel: int
    dtype: DType
    role: str  # 'input' | 'temp' | 'output'
    index: int = -1  # input / output position
    shape: tuple = ()
    offset: int = -1  # byte offset in the arena (temps)
    first: int = 1 << 60
    last: int = -1

    @property
    def nbytes(self) -> int:
        return max(self.numel, 1) * self.dtype.size_in_bytes


@dataclass(frozen=True)
class ViewRef:
    buf: int
    offset: int
    shape: tuple
    strides: tuple
    dtype: DType

    def is_contiguous(self) -> bool:
        exp = 1
        for d, s in zip(reversed(self.shape), reversed(self.strides)):
            if d == 1:
                continue
            if s != exp:
                return False
            exp *= d
        return True


@dataclass(frozen=True)
class Const:
    value: float
    shape: tuple
    dtype: DType


@dataclass
class OperandSpec:
    buf: int
    offset: int
    lead_strides: tuple
    col_stride: int
    dtype: DType
    vec_ok: bool
    stage_slot: int = -1
    is_output: bool = False


@dataclass
class Step:
    kind: str
    reads: list = field(default_factory=list)
    writes: list = field(default_factory=list)
    attrs: dict = field(default_factory=dict)


@dataclass
class Plan:
    bufs: list
    steps: list
    n_inputs: int
    outputs: list  # per plan output: (buf id, shape, dtype)
    arena_bytes: int = 0
    stats: dict = field(default_factory=dict)


# --------------------------------------------------------------------- view algebra
def _reshape_strides(old_shape, old_strides, new_shape):
    """Strides that view the same memory as ``new_shape``, or None (numpy's
    no-copy reshape rule)."""
    if _numel(old_shape) != _numel(new_shape):
        return None
    if _numel(new_shape) == 0:
        return contiguous_strides(new_shape)
    olds = [(d, s) for d, s in zip(old_shape, old_strides) if d != 1]
    new_strides = [0] * len(new_shape)
    oi = 0
    ni = 0
    n_old = len(olds)
    n_new = len(new_shape)
    while ni < n_new and new_shape[ni] == 1:
        ni += 1
    while oi < n_old and ni < n_new:
        # grow both sides until their element counts match
        np_ = new_shape[ni]
        op_ = olds[oi][0]
        oj, nj = oi + 1, ni + 1
        while np_ != op_:
            if np_ < op_:
                while nj < n_new and new_shape[nj] == 1:
                    nj += 1
                if nj >= n_new:
                    return None
                np_ *= new_shape[nj]
                nj += 1
            else:
                if oj >= n_old:
                    return None
                op_ *= olds[oj][0]
                oj += 1
        # old dims oi..oj must be mutually contiguous
        for k in range(oi, oj - 1):
            if olds[k][1] != olds[k + 1][1] * olds[k + 1][0]:
                return None
        st = olds[oj - 1][1]
        for k in range(nj - 1, ni - 1, -1):
            if new_shape[k] == 1:
                new_strides[k] = 0
                continue
            new_strides[k] = st
            st *= new_shape[k]
        oi, ni = oj, nj
        while ni < n_new and new_shape[ni] == 1:
            ni += 1
    if oi != n_old:
        return None
    return tuple(new_strides)


def _derive_view(node: ir.Node, base: ViewRef) -> ViewRef | None:
    """View of ``base`` after the view node; None if it needs a copy (reshape only)."""
    out = node.outputs[0]
    if node.kind == "broadcast":
        pad = len(out.shape) - len(base.shape)
        strides = [0] * pad + [0 if (d == 1 and o != 1) else s
                               for d, s, o in zip(base.shape, base.strides, out.shape[pad:])]
        return ViewRef(base.buf, base.offset, out.shape, tuple(strides), base.dtype)
    if node.kind == "permute":
        perm = node.attrs["perm"]
        return ViewRef(base.buf, base.offset, out.shape, tuple(base.strides[p] for p in perm),
                       base.dtype)
    if node.kind == "slice":
        off = base.offset + sum(a * s for a, s in zip(node.attrs["starts"], base.strides))
        strides = tuple(s * st for s, st in zip(base.strides, node.attrs["steps"]))
        return ViewRef(base.buf, off, out.shape, strides, base.dtype)
    if node.kind == "reshape":
        st = _reshape_strides(base.shape, base.strides, out.shape)
        if st is None:
            return None
        return ViewRef(base.buf, base.offset, out.shape, st, base.dtype)
    raise AssertionError(node.kind)


# ------------------------------------------------------------------------- grouping
class Unit:
    __slots__ = ("id", "nodes", "node_pos", "first_pos", "last_pos", "preds", "fused", "lead", "C",
                 "n_reduce", "ext", "hard", "alias")

    def __init__(self, uid: int, node: ir.Node, fused: bool):
        self.id = uid
        self.nodes = [node]
        self.node_pos = {node.pos}
        self.first_pos = node.pos
        self.last_pos = node.pos
        self.preds: set = set()
        self.fused = fused
        self.lead = None
        self.C = None
        self.n_reduce = 0
        self.ext: set = set()
        self.hard: set = set()   # preds that can never be merged into this unit
        self.alias = None        # set when this unit was merged into another

    def add(self, node: ir.Node) -> None:
        self.nodes.append(node)
        self.node_pos.add(node.pos)
        self.last_pos = max(self.last_pos, node.pos)


def _shape2(shape):
    return tuple(shape) if len(shape) > 0 else (1,)


class Planner:
    def __init__(self, builder: ir.Builder, outputs: Sequence[ir.Value], max_members: int = 28):
        self.b = builder
        self.outputs = list(outputs)
        self.max_members = max_members
        self.max_ext = 12
        self.bufs: list[Buf] = []
        self.steps: list[Step] = []
        self.loc: dict[int, Any] = {}  # value id -> ViewRef | Const
        self.unit_of: dict[int, Unit] = {}  # node pos -> unit
        self.alias_nodes: set[int] = set()  # broadcast nodes fused as row->full aliases
        from .. import config
        self.fold_column_sums = bool(config.FOLD_COLUMN_SUMS)
        self.group_siblings = bool(config.GROUP_SIBLING_PRODUCTS)
        self._sibling_groups: dict[int, list] = {}  # id(gemm step) -> members of its launch

    # ................................................................ liveness
    def _live_nodes(self) -> list[ir.Node]:
        live: set[int] = set()
        stack = [v.node for v in self.outputs]
        while stack:
            n = stack.pop()
            if n.pos in live:
                continue
            live.add(n.pos)
            for i in n.inputs:
                if i.node.pos not in live:
                    stack.append(i.node)
        return [n for n in self.b.nodes if n.pos in live]

    # ................................................................ helpers
    def _base(self, v: ir.Value) -> ir.Value:
        """Strip non-fused view nodes."""
        while v.node.kind in VIEW_KINDS and v.node.pos not in self.alias_nodes:
            v = v.node.inputs[0]
        return v

    @staticmethod
    def _find(u: "Unit | None") -> "Unit | None":
        while u is not None and u.alias is not None:
            u = u.alias
        return u

    def _unit(self, pos: int) -> "Unit | None":
        return self._find(self.unit_of.get(pos))

    def _producer_unit(self, v: ir.Value) -> "Unit | None":
        return self._unit(self._base(v).node.pos)

    def _is_member_value(self, v: ir.Value) -> bool:
        return v.node.kind in FUSABLE or v.node.pos in self.alias_nodes

    # ................................................................ int64
    _I32_OPEN = (-(2 ** 31) + 1, 2 ** 31 - 2)  # strictly inside the int32 range
    _COMPARISONS = ("eq", "ne", "gt", "ge", "lt", "le")

    def _inside_int32(self, x) -> bool:
        """Is ``x`` (an operand of an ew node) an index or constant made inside the kernel whose
        every value lies strictly inside the int32 range?"""
        lo, hi = self._I32_OPEN
        if not isinstance(x, ir.Value):
            return float(x) == int(x) and lo <= int(x) <= hi
        while x.node.kind in VIEW_KINDS:
            x = x.node.inputs[0]
        n = x.node
        if n.kind == "fill":
            v = n.attrs["value"]
            return v == int(v) and lo <= int(v) <= hi
        if n.kind == "iota":
            first = n.attrs["start"]
            last = first + n.attrs["step"] * max(x.shape[-1] - 1, 0)
            return lo <= min(first, last) and max(first, last) <= hi
        return False

    def _wants_int64_kernel(self, node: ir.Node) -> bool:
        """Does this fusable node have to run in the 64-bit integer kernel?  Row programs hold
        integers in 32-bit registers and read int64 storage saturated to the int32 range.
        That is exact for exactly one use of an int64 tensor: a comparison with an index or
        constant strictly inside the int32 range (labels against a class index, ids against a
        position), because saturation moves no value across such a bound.  Everything else
        that reads or makes int64 values -- arithmetic, selects, copies, casts, comparisons of
        two stored tensors -- is exact only in 64 bits."""
        i64 = DType.int64
        if node.kind == "iota":
            if node.outputs[0].dtype is i64 and not self._inside_int32(node.outputs[0]):
                raise NotImplementedError(
                    "an int64 index sequence that leaves the int32 range has no kernel; "
                    "build it on the host (Tensor.constant(numpy.arange(...)))")
            return False
        if node.kind == "tril":
            if node.outputs[0].dtype is i64:
                raise NotImplementedError("tril / triu of an int64 tensor: cast it to int32 or a "
                                          "floating-point type first")
            return False
        if node.kind != "ew":
            return False
        if node.outputs[0].dtype is not i64 and not any(i.dtype is i64 for i in node.inputs):
            return False
        xs = node.attrs["operands"]
        if node.fn in self._COMPARISONS and any(self._inside_int32(x) for x in xs):
            return False
        if node.fn not in isa.INT64_FNS:
            raise NotImplementedError(
                f"'{node.fn}' has no integer form: cast the int64 tensor to a floating-point type first")
        return True

    def _lower_int64_ew(self, n: ir.Node) -> None:
        """One launch of the 64-bit integer kernel for an elementwise node (operands as strided
        views of the result's shape, constants as immediates)."""
        out = n.outputs[0]
        ops = []
        for x in n.attrs["operands"]:
            if not isinstance(x, ir.Value):
                ops.append(int(x))
                continue
            ref = self._resolve(x)
            if isinstance(ref, Const):
                if ref.value != int(ref.value):
                    ref = self._materialize(ref)
                else:
                    ops.append(int(ref.value))
                    continue
            ops.append(ref)
        if all(isinstance(o, int) for o in ops):  # (a kernel needs one operand in memory)
            first = next(x for x in n.attrs["operands"] if isinstance(x, ir.Value))
            ops[list(n.attrs["operands"]).index(first)] = self._materialize(self._resolve(first))
        dst = self._alloc_value(out)
        self._emit(Step("ew64", [o.buf for o in ops if isinstance(o, ViewRef)], [dst.buf],
                        dict(fn=n.fn, operands=ops, dst=dst)))

    def _depends(self, u: Unit, g: Unit, skip: "Unit | None" = None) -> bool:
        """Does unit ``u`` (transitively) need ``g`` to have run?  Paths through
        ``skip`` are ignored (used when ``skip`` is about to be merged with g)."""
        if u is g:
            return True
        seen = {u.id}
        stack = [u]
        while stack:
            x = stack.pop()
            for p in x.preds:
                p = self._find(p)
                if p is g:
                    return True
                if p is skip or p.id in seen or p.last_pos < g.first_pos:
                    continue
                seen.add(p.id)
                stack.append(p)
        return False

    # ................................................................ fusion
    def _group(self, nodes: list[ir.Node]) -> list[Unit]:
        units: list[Unit] = []
        by_root: dict[int, list[Unit]] = {}  # external root value id -> fused units reading it

        def new_unit(node, fused) -> Unit:
            u = Unit(len(units), node, fused)
            units.append(u)
            self.unit_of[node.pos] = u
            return u

        def classify_inputs(node, g):
            """(soft preds, hard preds) of ``node`` seen from group ``g``; None if
            ``node`` cannot run inside ``g``.  A hard pred is read through a
            strided view or is not a row program, so it can never be merged in."""
            soft, hard = [], []
            for i in node.inputs:
                if self._is_member_value(i) and self._unit(i.node.pos) is g:
                    continue
                pu = self._producer_unit(i)
                if pu is None:
                    continue
                if pu is g:  # a strided view of a member: needs a trip through memory
                    return None
                if self._depends(pu, g):
                    return None
                (soft if (self._is_member_value(i) and pu.fused) else hard).append(pu)
            return soft, hard

        def dom_ok(g, kind, lead, last) -> bool:
            if g.lead != lead:
                return False
            if kind == "reduce":
                return (g.C is None or g.C == last) and g.n_reduce < 8
            return last == 1 or g.C is None or g.C == last

        def ext_ids(node, g):
            return {self._base(i).id for i in node.inputs
                    if not (self._is_member_value(i) and self._unit(i.node.pos) is g)}

        def join(g, node, kind, last, soft, hard):
            if kind == "reduce" or last != 1:
                g.C = last
            g.add(node)
            self.unit_of[node.pos] = g
            g.preds.update(soft)
            g.preds.update(hard)
            g.hard.update(hard)
            for e in ext_ids(node, g):
                if e not in g.ext:
                    g.ext.add(e)
                    by_root.setdefault(e, []).append(g)
            if kind == "reduce":
                g.n_reduce += 1

        def try_merge(g1: Unit, g2: Unit) -> bool:
            """Fold g2 into g1 when no third unit sits between them."""
            if g1 is g2 or not (g1.fused and g2.fused) or g1.lead != g2.lead:
                return False
            if g1.C is not None and g2.C is not None and g1.C != g2.C:
                return False
            if len(g1.nodes) + len(g2.nodes) > self.max_members or g1.n_reduce + g2.n_reduce > 8:
                return False
            if any(self._find(h) is g2 for h in g1.hard) or any(self._find(h) is g1 for h in g2.hard):
                return False
            if len(g1.ext | g2.ext) > self.max_ext + 4:
                return False
            for a, b in ((g1, g2), (g2, g1)):
                for p in a.preds:
                    p = self._find(p)
                    if p is b or p is a:
                        continue
                    if self._depends(p, b, skip=a):
                        return False
            g2.alias = g1
            for n in g2.nodes:
                g1.add(n)
            g1.first_pos = min(g1.first_pos, g2.first_pos)
            g1.preds = {self._find(p) for p in (g1.preds | g2.preds)} - {g1, g2}
            g1.hard = {self._find(p) for p in (g1.hard | g2.hard)} - {g1, g2}
            g1.ext |= g2.ext
            for e in g2.ext:
                by_root.setdefault(e, []).append(g1)
            g1.n_reduce += g2.n_reduce
            if g1.C is None:
                g1.C = g2.C
            return True

        for node in nodes:
            kind = node.kind
            if kind == "input" or kind == "fill":
                continue
            if kind in VIEW_KINDS:
                # row -> full broadcast of a fused value stays inside the group
                if kind == "broadcast":
                    src = node.inputs[0]
                    out = node.outputs[0]
                    g = self._unit(src.node.pos)
                    if (g is not None and g.fused and self._is_member_value(src) and
                            len(src.shape) == len(out.shape) and len(out.shape) >= 1 and
                            src.shape[:-1] == out.shape[:-1] and src.shape[-1] == 1 and
                            tuple(out.shape[:-1]) == g.lead and g.C in (None, out.shape[-1]) and
                            len(g.nodes) < self.max_members):
                        g.C = out.shape[-1]
                        g.add(node)
                        self.unit_of[node.pos] = g
                        self.alias_nodes.add(node.pos)
                continue
            # (integer reductions keep a 64-bit accumulator in a kernel of their own, and so does
            # elementwise work on int64 values: row-program registers are 32 bits wide)
            if kind not in FUSABLE or (kind == "reduce" and (
                    node.attrs["axis"] != node.inputs[0].rank - 1 or
                    node.inputs[0].dtype in INT_REG_DTYPES)) or self._wants_int64_kernel(node):
                u = new_unit(node, False)
                for i in node.inputs:
                    pu = self._producer_unit(i)
                    if pu is not None:
                        u.preds.add(pu)
                        u.hard.add(pu)
                continue

            # fusable node: find its domain
            out = node.outputs[0]
            dom_shape = _shape2(node.inputs[0].shape if kind == "reduce" else out.shape)
            lead, last = tuple(dom_shape[:-1]), dom_shape[-1]
            home = None
            if kind != "iota" and not (kind == "tril" and len(lead) == 0):
                cands: list[Unit] = []
                for i in node.inputs:
                    if self._is_member_value(i):
                        g = self._unit(i.node.pos)
                        if g is not None and g.fused and g not in cands:
                            cands.append(g)
                # groups that read one of the same external tensors over the same domain
                sib: list[Unit] = []
                dom_numel = _numel(dom_shape)
                for i in node.inputs:
                    # sharing a tensor pays only if it is read at full size: a broadcast scalar
                    # or bias in common would chain unrelated work into one oversized group
                    if self._base(i).numel() < dom_numel:
                        continue
                    for g in by_root.get(self._base(i).id, ()):
                        g = self._find(g)
                        if g.fused and g not in cands and g not in sib:
                            sib.append(g)
                cands.sort(key=lambda g: -g.last_pos)
                sib.sort(key=lambda g: -g.last_pos)
                for g in cands + sib[:4]:
                    if not dom_ok(g, kind, lead, last) or len(g.nodes) >= self.max_members:
                        continue
                    cl = classify_inputs(node, g)
                    if cl is None:
                        continue
                    if len(g.ext | ext_ids(node, g)) > self.max_ext:
                        continue
                    join(g, node, kind, last, *cl)
                    home = g
                    break
                if home is not None:
                    # producers that live in other groups: try to pull those groups in
                    for g2 in cands:
                        g2 = self._find(g2)
                        if g2 is not home and dom_ok(g2, "ew", lead, 1):
                            try_merge(home, g2)
            if home is None:
                g = new_unit(node, True)
                g.lead = lead
                g.C = last if (kind == "reduce" or last != 1) else None
                g.n_reduce = 1 if kind == "reduce" else 0
                for i in node.inputs:
                    pu = self._producer_unit(i)
                    if pu is not None and pu is not g:
                        g.preds.add(pu)
                        if not (self._is_member_value(i) and pu.fused):
                            g.hard.add(pu)
                    e = self._base(i).id
                    g.ext.add(e)
                    by_root.setdefault(e, []).append(g)
        live_units = [u for u in units if u.alias is None]
        for u in live_units:
            u.preds = {self._find(p) for p in u.preds} - {u}
        return live_units

    # ................................................................ ordering
    def _order(self, units: list[Unit]) -> list[Unit]:
        indeg = {u.id: 0 for u in units}
        succs: dict[int, list[Unit]] = {u.id: [] for u in units}
        for u in units:
            for p in u.preds:
                if p is u:
                    continue
                indeg[u.id] += 1
                succs[p.id].append(u)
        heap = [(u.first_pos, u.id) for u in units if indeg[u.id] == 0]
        heapq.heapify(heap)
        by_id = {u.id: u for u in units}
        out = []
        while heap:
            _, uid = heapq.heappop(heap)
            u = by_id[uid]
            out.append(u)
            for s in succs[uid]:
                indeg[s.id] -= 1
                if indeg[s.id] == 0:
                    heapq.heappush(heap, (s.first_pos, s.id))
        if len(out) != len(units):
            raise RuntimeError("lowering: fusion produced a cyclic group graph")
        return out

    # ................................................................ buffers
    def _new_buf(self, shape, dtype: DType, role: str = "temp", index: int = -1) -> Buf:
        b = Buf(len(self.bufs), _numel(shape), dtype, role, index, tuple(shape))
        self.bufs.append(b)
        return b

    def _emit(self, step: Step) -> None:
        if step.kind == "fill" and step.attrs["numel"] == 0:
            return
        if step.kind == "copy" and _numel(step.attrs["src"].shape) == 0:
            return
        idx = len(self.steps)
        for r in step.reads:
            b = self.bufs[r]
            b.last = max(b.last, idx)
            b.first = min(b.first, idx)
        for w in step.writes:
            b = self.bufs[w]
            b.first = min(b.first, idx)
            b.last = max(b.last, idx)
        self.steps.append(step)

    def _alloc_value(self, v: ir.Value) -> ViewRef:
        """Fresh contiguous storage for value ``v`` (an output allocation if it
        is a plan output that is not claimed yet)."""
        role, index = "temp", -1
        if v.id in self._out_pending:
            role, index = "output", self._out_pending.pop(v.id)
        b = self._new_buf(v.shape, v.dtype, role, index)
        ref = ViewRef(b.id, 0, v.shape, contiguous_strides(v.shape), v.dtype)
        self.loc[v.id] = ref
        if role == "output":
            self._out_done[index] = b.id
        return ref

    def _resolve(self, v: ir.Value):
        """Location (ViewRef | Const) of a value, folding view chains."""
        got = self.loc.get(v.id)
        if got is not None:
            return got
        n = v.node
        if n.kind == "fill":
            c = Const(n.attrs["value"], v.shape, v.dtype)
            self.loc[v.id] = c
            return c
        if n.kind in VIEW_KINDS:
            # (also a broadcast that lives inside a group as an alias of a row value: whoever
            # asks for its location reads it from outside the group, as a view of the stored row)
            base = self._resolve(n.inputs[0])
            if isinstance(base, Const):
                r = Const(base.value, v.shape, v.dtype)
            else:
                r = _derive_view(n, base)
                if r is None:  # reshape of a non-collapsible view
                    cont = self._materialize(base)
                    r = _derive_view(n, cont)
            self.loc[v.id] = r
            return r
        raise RuntimeError(f"lowering: value {v} used before it was produced ({n.kind})")

    def _materialize(self, src) -> ViewRef:
        """Contiguous copy of a view or constant in a fresh temp."""
        if isinstance(src, Const):
            b = self._new_buf(src.shape, src.dtype)
            self._emit(Step("fill", [], [b.id], dict(buf=b.id, numel=_numel(src.shape),
                                                      value=src.value, dtype=src.dtype)))
            return ViewRef(b.id, 0, src.shape, contiguous_strides(src.shape), src.dtype)
        if src.is_contiguous():
            return src
        # one copy per distinct view: a broadcast cotangent that feeds two products and a
        # reduction is materialised once (values are written once, so the copy stays valid)
        key = (src.buf, src.offset, tuple(src.shape), tuple(src.strides), src.dtype)
        hit = self._materialized.get(key)
        if hit is not None:
            return hit
        b = self._new_buf(src.shape, src.dtype)
        dst = ViewRef(b.id, 0, src.shape, contiguous_strides(src.shape), src.dtype)
        self._emit(Step("copy", [src.buf], [b.id], dict(src=src, dst=dst)))
        self._materialized[key] = dst
        return dst

    def _contig(self, v: ir.Value) -> ViewRef:
        return self._materialize(self._resolve(v))

    # ................................................................ build
    _REMAT_FNS = ("eq", "ne", "gt", "ge", "lt", "le", "mov", "not", "and", "or")

    def _rematerialize_masks(self) -> None:
        """A large tensor that is a cheap function of small ones (a one-hot: labels compared
        with an iota, cast to the compute type; a causal or padding mask) and has readers in
        several places is not worth a trip through memory: every reader after the first gets
        its own copy of the few nodes that make it, which then fuse into that reader's kernel.
        Cheap means: comparisons, logic and casts only, over broadcasts of values at least 64
        times smaller than the result."""
        nodes = self._live_nodes()
        users: dict[int, list[ir.Node]] = {}
        for n in nodes:
            for i in n.inputs:
                if not users.get(i.id) or users[i.id][-1] is not n:
                    users.setdefault(i.id, []).append(n)
        out_ids = {v.id for v in self.outputs}
        clones_before: dict[int, list[ir.Node]] = {}  # pos of a reader -> nodes to put before it
        for n in nodes:
            if not (n.kind == "ew" and n.fn in self._REMAT_FNS):
                continue
            v = n.outputs[0]
            readers = users.get(v.id, [])
            big = _numel(v.shape)
            if len(readers) < 2 or v.id in out_ids or big < (1 << 22):
                continue
            chain: list[ir.Node] = []
            ok, stack, seen = True, [n], set()
            while stack and ok:
                m = stack.pop()
                if m.pos in seen:
                    continue
                seen.add(m.pos)
                chain.append(m)
                if len(chain) > 8:
                    ok = False
                    break
                for i in m.inputs:
                    if _numel(i.shape) * 64 <= big:
                        continue  # a small leaf: read again by the copy
                    pn = i.node
                    if pn.kind in ("broadcast", "reshape", "iota") or (pn.kind == "ew" and pn.fn in self._REMAT_FNS):
                        stack.append(pn)
                    else:
                        ok = False
                        break
            if not ok:
                continue
            chain.sort(key=lambda m: m.pos)
            for reader in readers[1:]:
                if reader.pos in seen:
                    continue
                vmap: dict[int, ir.Value] = {}
                made = []
                for m in chain:
                    attrs = dict(m.attrs or {})
                    ins = [vmap.get(i.id, i) for i in m.inputs]
                    if "operands" in attrs:
                        attrs["operands"] = tuple(vmap.get(o.id, o) if isinstance(o, ir.Value) else o
                                                  for o in attrs["operands"])
                    c = ir.Node(m.kind, m.fn, ins, attrs, -1)
                    for k, o in enumerate(m.outputs):
                        nv = ir.Value(o.shape, o.dtype, c, k, self.b._n_values)
                        self.b._n_values += 1
                        c.outputs.append(nv)
                        vmap[o.id] = nv
                    made.append(c)
                reader.inputs = [vmap.get(i.id, i) if i.id == v.id else i for i in reader.inputs]
                if reader.attrs and "operands" in reader.attrs:
                    reader.attrs = dict(reader.attrs, operands=tuple(
                        vmap[v.id] if isinstance(o, ir.Value) and o.id == v.id else o
                        for o in reader.attrs["operands"]))
                clones_before.setdefault(id(reader), []).extend(made)
        if not clones_before:
            return
        out: list[ir.Node] = []
        for n in self.b.nodes:
            out.extend(clones_before.get(id(n), ()))
            out.append(n)
        for k, n in enumerate(out):
            n.pos = k
        self.b.nodes[:] = out

    def _fold_bias_into_matmul(self) -> None:
        """``x @ W + b`` with ``b`` a row vector broadcast over the leading axes: the add node
        itself turns into the matmul node with the bias as a third input
        (``attrs["bias_in"]``; it comes after everything the product reads, so program order
        stays a valid order) and the original product, now without readers, is dropped by the
        liveness pass.  The bias is added in the kernel's epilogue, before the result is
        rounded.  Only where the product has no other reader and is not split along K
        (partial products cannot carry an epilogue)."""
        nodes = self._live_nodes()
        n_users: dict[int, int] = {}
        for n in nodes:
            for i in n.inputs:
                n_users[i.id] = n_users.get(i.id, 0) + 1
        out_ids = {v.id for v in self.outputs}
        for n in nodes:
            if not (n.kind == "ew" and n.fn == "add" and len(n.inputs) == 2):
                continue
            out = n.outputs[0]
            for m, bb in ((n.inputs[0], n.inputs[1]), (n.inputs[1], n.inputs[0])):
                mm = m.node
                at = mm.attrs or {}
                if not (bb.node.kind == "broadcast" and mm.kind == "matmul" and
                        len(mm.outputs) == 1 and "bias_in" not in at and not at.get("act") and
                        n_users.get(m.id) == 1 and m.id not in out_ids and
                        self._epilogue_ok(mm, out)):
                    continue
                src = bb.node.inputs[0]
                N = m.shape[-1]
                if not (src.rank >= 1 and src.shape[-1] == N and _numel(src.shape) == N and
                        src.dtype is m.dtype):
                    continue
                n.kind, n.fn = "matmul", None
                n.inputs = list(mm.inputs) + [src]
                n.attrs = dict(at, bias_in=len(mm.inputs))
                break

    def _fold_sum_into_matmul(self, thin_only: bool = False) -> None:
        """``r + (x @ W) * alpha`` with ``r`` of the product's shape (a skip connection, the base
        product under a low-rank update, a gradient that two branches contribute to): the add
        node turns into the product, which reads ``r`` in its epilogue and adds it to the fp32
        accumulator before the one rounding of the result.  The scaled product and the sum
        never make their own trips through memory.  A chain of such sums folds link by link:
        the second product takes the first sum as its ``r``.

        ``thin_only``: only products with a contraction of at most 16 (the update of a low-rank
        adapter on top of its base product).  Their kernel is all memory traffic, many
        workgroups to a CU, and reads ``r`` for less than the separate sum kernel costs; the
        large products pay more for it than that kernel (one workgroup per CU, nothing runs
        beside its epilogue), so for them the fold stays behind ``config.FOLD_RESIDUAL``."""
        nodes = self._live_nodes()
        n_users: dict[int, int] = {}
        for n in nodes:
            for i in n.inputs:
                n_users[i.id] = n_users.get(i.id, 0) + 1
        out_ids = {v.id for v in self.outputs}

        def single_use(v: ir.Value) -> bool:
            return n_users.get(v.id) == 1 and v.id not in out_ids

        def constant_of(x):
            """The number an operand stands for: itself, or the fill behind a chain of views."""
            if not isinstance(x, ir.Value):
                return float(x)
            while x.node.kind in ("broadcast", "reshape"):
                x = x.node.inputs[0]
            if x.node.kind != "fill":
                return None
            # the unfused multiply would read the constant as stored: round it the same way
            return _as_stored(float(x.node.attrs["value"]), x.dtype)

        for n in nodes:
            if not (n.kind == "ew" and n.fn == "add" and len(n.inputs) == 2 and
                    all(isinstance(x, ir.Value) for x in n.attrs["operands"])):
                continue
            out = n.outputs[0]
            for m, r in ((n.inputs[1], n.inputs[0]), (n.inputs[0], n.inputs[1])):
                alpha, mm = 1.0, m.node
                if mm.kind == "ew" and mm.fn == "mul" and single_use(m):
                    # (x @ W) * c with c a number or a broadcast constant
                    xs = mm.attrs["operands"]
                    scaled = None
                    for x, other in ((xs[0], xs[1]), (xs[1], xs[0])):
                        if (isinstance(x, ir.Value) and x.node.kind == "matmul" and
                                x.dtype is m.dtype and x.shape == m.shape and
                                constant_of(other) is not None):
                            scaled = (x, constant_of(other))
                            break
                    if scaled is None:
                        continue
                    m, alpha = scaled
                    mm = m.node
                at = mm.attrs or {}
                if alpha != 1.0 and "bias_in" in at:
                    continue  # (the kernel scales the product only, not a bias folded earlier)
                # (and only on top of another product, the adapter's base: a sum with anything
                # else usually sits inside a fused row kernel already and would be cut out of it)
                if thin_only and not (mm.kind == "matmul" and mm.inputs[0].shape[-1] <= 16 and
                                      m.dtype is DType.bfloat16 and m.shape[-1] % 8 == 0 and
                                      r.node.kind == "matmul"):
                    continue
                if not (mm.kind == "matmul" and len(mm.outputs) == 1 and single_use(m) and
                        "res_in" not in at and not at.get("act") and
                        r.shape == out.shape and r.dtype is out.dtype and r.node.kind != "fill" and
                        self._epilogue_ok(mm, out)):
                    continue
                n.kind, n.fn = "matmul", None
                n.inputs = list(mm.inputs) + [r]
                n.attrs = dict(at, res_in=len(mm.inputs), alpha=alpha * at.get("alpha", 1.0))
                break

    def _fold_thin_pair_into_matmul(self) -> None:
        """``x @ W + u @ V`` with ``u @ V`` at most one K tile deep (the update of a low-rank
        adapter on top of its base product, already folded by `_fold_sum_into_matmul` into a
        thin product that reads the base product as its residual): the node turns into the base
        product with ``(u, V)`` as one more operand pair (``attrs["terms_in"]``: the index of the first of the
        pairs that follow the base product's own inputs), which the
        kernel multiplies as one more K tile into the same accumulator.  The base product no
        longer makes a trip through memory (one write and one read of the result saved, and
        the thin product's launch), and the sum is rounded once.  Only plain products on both
        sides (no activation, scale, second result; the base may carry a bias) of one bf16 dtype
        whose base has no other reader; the operands' layouts are checked when the node is lowered, and a pair the
        kernel cannot take runs as the two launches it replaced."""
        nodes = self._live_nodes()
        n_users: dict[int, int] = {}
        for n in nodes:
            for i in n.inputs:
                n_users[i.id] = n_users.get(i.id, 0) + 1
        out_ids = {v.id for v in self.outputs}
        def one_matrix(w: ir.Value) -> bool:
            """A 2-D right operand, or one broadcast over the batch axes of the left one."""
            while w.rank > 2:
                m = w.node
                if m.kind == "permute":  # (the transpose of the backward pass)
                    perm = tuple(m.attrs["perm"])
                    if perm[:-2] != tuple(range(w.rank - 2)):
                        return False
                    w = m.inputs[0]
                elif m.kind == "broadcast" and m.inputs[0].rank == 2 and \
                        tuple(m.inputs[0].shape) == tuple(w.shape[-2:]):
                    return True
                else:
                    return False
            return True

        for n in nodes:
            at = n.attrs or {}
            if not (n.kind == "matmul" and at.get("res_in") == 2 and len(n.inputs) == 3 and
                    len(n.outputs) == 1 and not at.get("act") and "bias_in" not in at and
                    at.get("alpha", 1.0) == 1.0):
                continue
            u, v, r = n.inputs
            base = r.node
            bat = base.attrs or {}
            k2 = u.shape[-1]
            if not (base.kind == "matmul" and len(base.outputs) == 1 and
                    len(base.inputs) == (3 if "bias_in" in bat else 2) and
                    not (set(bat) & {"res_in", "act", "terms_in"}) and
                    bat.get("alpha", 1.0) == 1.0 and
                    n_users.get(r.id) == 1 and r.id not in out_ids and
                    k2 <= 64 and k2 % 8 == 0 and one_matrix(v) and one_matrix(base.inputs[1]) and
                    base.inputs[0].shape[-1] % 64 == 0 and
                    u.shape[:-1] == base.inputs[0].shape[:-1] and
                    all(x.dtype is DType.bfloat16 for x in (u, v, r, *base.inputs, n.outputs[0]))):
                continue
            n.inputs = list(base.inputs) + [u, v]
            n.attrs = dict(bat, terms_in=len(base.inputs))

        # ``(X + u @ V) + x @ W``: contributions to one gradient arrive in the order of the
        # backward pass, and a thin product whose base product comes one link later in the chain
        # of sums was not folded above.  The base product takes the pair where it stands (``u``
        # and ``V`` exist before the thin product, which comes earlier) and the outer sum reads
        # ``X`` instead of the inner one; the thin product and the inner sum lose their readers.
        nodes = self._live_nodes()
        users: dict[int, list[ir.Node]] = {}
        for n in nodes:
            for i in n.inputs:
                users.setdefault(i.id, []).append(n)

        def only_reader(val: ir.Value):
            us = users.get(val.id, [])
            return us[0] if len(us) == 1 and val.id not in out_ids else None

        def plain_add(n: ir.Node) -> bool:
            return (n.kind == "ew" and n.fn == "add" and len(n.inputs) == 2 and
                    all(isinstance(x, ir.Value) for x in n.attrs["operands"]))

        for thin in nodes:
            tat = thin.attrs or {}
            if not (thin.kind == "matmul" and len(thin.inputs) == 2 and len(thin.outputs) == 1 and
                    not (set(tat) & {"res_in", "bias_in", "act", "terms_in"}) and
                    tat.get("alpha", 1.0) == 1.0):
                continue
            u, v = thin.inputs
            k2 = u.shape[-1]
            t_out = thin.outputs[0]
            if not (k2 <= 64 and k2 % 8 == 0 and one_matrix(v)):
                continue
            inner = only_reader(t_out)
            if inner is None or not plain_add(inner):
                continue
            x_val = inner.inputs[1] if inner.inputs[0].id == t_out.id else inner.inputs[0]
            outer = only_reader(inner.outputs[0])
            if outer is None or not plain_add(outer) or x_val.id == t_out.id:
                continue
            b_out = outer.inputs[1] if outer.inputs[0].id == inner.outputs[0].id else outer.inputs[0]
            base = b_out.node
            bat = base.attrs or {}
            if not (base.kind == "matmul" and base is not thin and len(base.outputs) == 1 and
                    len(base.inputs) == 2 and not (set(bat) & {"res_in", "bias_in", "act", "terms_in"}) and
                    bat.get("alpha", 1.0) == 1.0 and only_reader(b_out) is outer and
                    base.pos > thin.pos and base.inputs[0].shape[-1] % 64 == 0 and
                    one_matrix(base.inputs[1]) and u.shape[:-1] == base.inputs[0].shape[:-1] and
                    b_out.shape == t_out.shape == x_val.shape and
                    all(z.dtype is DType.bfloat16 for z in (u, v, t_out, b_out, x_val, *base.inputs,
                                                             inner.outputs[0], outer.outputs[0]))):
                continue
            base.inputs = list(base.inputs) + [u, v]
            base.attrs = dict(bat, terms_in=2)
            outer.inputs = [x_val, b_out]
            outer.attrs = dict(outer.attrs, operands=(x_val, b_out))
            users[b_out.id] = [outer]
            users[x_val.id] = [z for z in users.get(x_val.id, []) if z is not inner] + [outer]
            users[t_out.id] = []
            users[inner.outputs[0].id] = []

    def _fold_product_sums(self) -> None:
        """``x1 @ W1 + x2 @ W2 (+ x3 @ W3)``: a value that several products contribute to (the
        gradient of an activation that feeds the query, key and value projections:
        ``dq @ Wq^T + dk @ Wk^T + dv @ Wv^T``) is ONE product over the contraction indices of all
        pairs (`nbk_gemm_desc.term`): one launch with one prologue and one epilogue instead of
        three, one result instead of three results and the kernel that adds them.  Two shapes of
        the sum are folded, repeatedly: ``P + Q`` (the add node becomes the product) and
        ``(X + P) + Q`` with anything for ``X`` (contributions arrive in the order of the
        backward pass; the later product takes the earlier one's pairs where it stands and the
        outer sum reads ``X``).  Only plain bf16 products with one reader each, whose right
        operands are one matrix; at most three pairs a K tile or more deep and two shallower
        ones (what one launch takes; the kernel wants the deep pairs laid out alike, which
        holds for the projections of one activation and is checked by the library, which runs
        one launch per pair otherwise)."""
        out_ids = {v.id for v in self.outputs}

        def one_matrix(w: ir.Value) -> bool:
            while w.rank > 2:
                m = w.node
                if m.kind == "permute":
                    perm = tuple(m.attrs["perm"])
                    if perm[:-2] != tuple(range(w.rank - 2)):
                        return False
                    w = m.inputs[0]
                elif m.kind == "broadcast" and m.inputs[0].rank == 2 and \
                        tuple(m.inputs[0].shape) == tuple(w.shape[-2:]):
                    return True
                else:
                    return False
            return True

        def plain_add(n: ir.Node) -> bool:
            return (n.kind == "ew" and n.fn == "add" and len(n.inputs) == 2 and
                    all(isinstance(x, ir.Value) for x in n.attrs["operands"]))

        def pairs_of(mm: ir.Node):
            ins = mm.inputs
            return [(ins[0], ins[1])] + list(zip(ins[2::2], ins[3::2]))

        changed = True
        while changed:
            changed = False
            nodes = self._live_nodes()
            users: dict[int, list[ir.Node]] = {}
            for n in nodes:
                for i in n.inputs:
                    users.setdefault(i.id, []).append(n)

            def only_reader(val: ir.Value):
                us = users.get(val.id, [])
                return us[0] if len(us) == 1 and val.id not in out_ids else None

            def product(val: ir.Value, reader: ir.Node) -> bool:
                mm = val.node
                at = mm.attrs or {}
                if not (mm.kind == "matmul" and len(mm.outputs) == 1 and only_reader(val) is reader and
                        not (set(at) - {"terms_in", "alpha"}) and at.get("alpha", 1.0) == 1.0 and
                        at.get("terms_in", 2) == 2 and len(mm.inputs) % 2 == 0 and
                        val.dtype is DType.bfloat16):
                    return False
                for u, v in pairs_of(mm):
                    if not (u.dtype is DType.bfloat16 and v.dtype is DType.bfloat16 and one_matrix(v) and
                            u.shape[:-1] == mm.inputs[0].shape[:-1] and u.shape[-1] % 8 == 0):
                        return False
                return mm.inputs[0].shape[-1] % 64 == 0

            def fits(pairs) -> bool:
                deep = [u for u, _ in pairs if u.shape[-1] > 64]
                shallow = [u for u, _ in pairs if u.shape[-1] <= 64]
                return (1 <= len(deep) <= 3 and len(shallow) <= 2 and
                        all(u.shape[-1] % 64 == 0 for u in deep))

            def merged_inputs(first: ir.Node, second: ir.Node):
                """Pairs of both products, a deep one of the product that stays first."""
                pairs = pairs_of(first) + pairs_of(second)
                return [x for pair in pairs for x in pair] if fits(pairs) else None

            for n in nodes:
                if not plain_add(n):
                    continue
                x, y = n.inputs
                if x.shape != y.shape or x.shape != n.outputs[0].shape:
                    continue
                # P + Q: the add node becomes the product
                if product(x, n) and product(y, n) and x.node is not y.node:
                    ins = merged_inputs(x.node, y.node)
                    if ins is not None:
                        n.kind, n.fn = "matmul", None
                        n.inputs = ins
                        n.attrs = dict(terms_in=2)
                        changed = True
                        break
                # (X + P) + Q, either way round
                done = False
                for inner_v, q in ((x, y), (y, x)):
                    inner = inner_v.node
                    if not (plain_add(inner) and only_reader(inner_v) is n and product(q, n)):
                        continue
                    for p_v, other in ((inner.inputs[0], inner.inputs[1]), (inner.inputs[1], inner.inputs[0])):
                        if not (product(p_v, inner) and p_v.node is not q.node and
                                other.shape == n.outputs[0].shape and other.id != q.id):
                            continue
                        first, second = (q.node, p_v.node)       # the later one keeps its place
                        later = first if first.pos > second.pos else second
                        earlier = second if later is first else first
                        ins = merged_inputs(later, earlier)
                        if ins is None:
                            continue
                        later.inputs = ins
                        later.attrs = dict(terms_in=2)
                        keep = later.outputs[0]
                        n.inputs = [other, keep]
                        n.attrs = dict(n.attrs, operands=(other, keep))
                        changed = done = True
                        break
                    if done:
                        break
                if done:
                    break

    def _fold_scale_into_matmul(self) -> None:
        """``(x @ W) * c`` with ``c`` a number: the multiply node turns into the product with
        ``alpha = c`` (applied to the fp32 accumulator, also of K-split partial products, before
        the one rounding of the result).  The low-rank adapters put their ``alpha / rank`` on a
        [tokens, rank] product this way, and their backward pass on two more."""
        nodes = self._live_nodes()
        n_users: dict[int, int] = {}
        for n in nodes:
            for i in n.inputs:
                n_users[i.id] = n_users.get(i.id, 0) + 1
        out_ids = {v.id for v in self.outputs}

        def constant_of(x):
            if not isinstance(x, ir.Value):
                return float(x)
            while x.node.kind in ("broadcast", "reshape"):
                x = x.node.inputs[0]
            if x.node.kind != "fill":
                return None
            # the unfused multiply would read the constant as stored: round it the same way
            return _as_stored(float(x.node.attrs["value"]), x.dtype)

        for n in nodes:
            if not (n.kind == "ew" and n.fn == "mul" and len(n.attrs["operands"]) == 2):
                continue
            out = n.outputs[0]
            xs = n.attrs["operands"]
            for x, other in ((xs[0], xs[1]), (xs[1], xs[0])):
                if not (isinstance(x, ir.Value) and x.node.kind == "matmul"):
                    continue
                c = constant_of(other)
                mm, at = x.node, x.node.attrs or {}
                if (c is None or len(mm.outputs) != 1 or n_users.get(x.id) != 1 or x.id in out_ids or
                        x.dtype is not out.dtype or x.shape != out.shape or
                        out.dtype not in (DType.float32, DType.bfloat16) or
                        "bias_in" in at or "res_in" in at or at.get("act")):
                    continue
                n.kind, n.fn = "matmul", None
                n.inputs = list(mm.inputs)
                n.attrs = dict(at, alpha=c * at.get("alpha", 1.0))
                break

    def _fold_activation_into_matmul(self) -> None:
        """``gelu(x @ W + b)`` whose pre-activation has no reader but the activation and, in a
        training step, its derivative (``GeluOp``'s VJP multiplies the cotangent with
        ``dgelu`` of the same value): both become results of the product itself, computed in
        its epilogue from the fp32 accumulator, and the pre-activation never reaches memory.
        The node of the two that comes first in program order turns into the product (its
        inputs precede it, every reader of either result follows it)."""
        nodes = self._live_nodes()
        users: dict[int, list[ir.Node]] = {}
        for n in nodes:
            for i in n.inputs:
                if not any(u is n for u in users.get(i.id, ())):
                    users.setdefault(i.id, []).append(n)
        out_ids = {v.id for v in self.outputs}
        for mm in nodes:
            if (mm.kind != "matmul" or len(mm.outputs) != 1 or (mm.attrs or {}).get("act") or
                    "res_in" in (mm.attrs or {})):  # (the residual joins after the activation)
                continue
            h = mm.outputs[0]
            us = users.get(h.id, [])
            if h.id in out_ids or not us:
                continue
            act = [u for u in us if u.kind == "ew" and u.fn == "gelu"]
            der = [u for u in us if u.kind == "ew" and u.fn == "dgelu"]
            if len(act) != 1 or len(der) > 1 or len(us) != 1 + len(der):
                continue
            a_out = act[0].outputs[0]
            outs = [a_out] + [d.outputs[0] for d in der]
            if not self._epilogue_ok(mm, a_out) or any(
                    o.dtype is not a_out.dtype or o.shape != a_out.shape for o in outs):
                continue
            host = min(act + der, key=lambda n: n.pos)
            host.kind, host.fn = "matmul", None
            host.inputs = list(mm.inputs)
            host.attrs = dict(mm.attrs or {}, act="gelu")
            host.outputs = outs
            for k, v in enumerate(outs):
                v.node, v.index = host, k

    def _fold_relu_into_producer(self) -> None:
        """``relu(conv2d(x, w) + b)`` or ``relu(x @ W + b)`` whose pre-activation has no reader
        but the relu and, in a training step, the comparisons ``pre-activation > 0`` of the
        relu's VJP: the convolution / product applies the relu to its accumulator on the way
        out, and the comparisons read the result instead (max(h, 0) > 0 exactly where h > 0).
        The pre-activation never reaches memory and the relu's row kernel is gone."""
        nodes = self._live_nodes()
        users: dict[int, list[ir.Node]] = {}
        for n in nodes:
            for i in n.inputs:
                if not any(u is n for u in users.get(i.id, ())):
                    users.setdefault(i.id, []).append(n)
        out_ids = {v.id for v in self.outputs}
        for cv in nodes:
            at = cv.attrs or {}
            if cv.kind not in ("conv2d", "matmul") or len(cv.outputs) != 1 or at.get("act"):
                continue
            if cv.kind == "matmul" and ("res_in" in at or "terms_in" in at):
                continue  # (a residual joins after the activation)
            h = cv.outputs[0]
            us = users.get(h.id, [])
            if h.id in out_ids or not us:
                continue
            act = [u for u in us if u.kind == "ew" and u.fn == "relu"]
            def is_zero(x) -> bool:
                if not isinstance(x, ir.Value):
                    return float(x) == 0.0
                while x.node.kind in ("broadcast", "reshape"):
                    x = x.node.inputs[0]
                return x.node.kind == "fill" and float(x.node.attrs["value"]) == 0.0

            masks = [u for u in us if u.kind == "ew" and u.fn == "gt" and
                     len(u.attrs["operands"]) == 2 and u.attrs["operands"][0] is h and
                     is_zero(u.attrs["operands"][1])]
            if len(act) != 1 or len(us) != 1 + len(masks):
                continue
            y = act[0].outputs[0]
            if y.dtype is not h.dtype or y.shape != h.shape:
                continue
            if cv.kind == "matmul" and not self._epilogue_ok(cv, y):
                continue
            cv.attrs = dict(cv.attrs or {}, act="relu")
            cv.outputs = [y]
            y.node, y.index = cv, 0
            for m in masks:
                m.inputs = [y if i is h else i for i in m.inputs]
                m.attrs["operands"] = [y if o is h else o for o in m.attrs["operands"]]

    def _epilogue_ok(self, mm: ir.Node, out: ir.Value) -> bool:
        """The product ``mm`` may write ``out`` through its epilogue."""
        m = mm.outputs[0]
        if not (out.dtype is m.dtype and out.shape == m.shape and
                m.dtype in (DType.float32, DType.bfloat16)):
            return False
        a, b = mm.inputs[:2]
        dt = a.dtype if a.dtype is b.dtype else DType.float32
        # (batched x @ W is one product with all the rows)
        return self._split_k(_numel(m.shape[:-1]), m.shape[-1], a.shape[-1], dt) == 1

    def build(self) -> Plan:
        nodes = self._live_nodes()
        for i, v in enumerate(self.b.inputs):
            b = self._new_buf(v.shape, v.dtype, "input", i)
            self.loc[v.id] = ViewRef(b.id, 0, v.shape, contiguous_strides(v.shape), v.dtype)
        self.skip_nodes: set[int] = set()  # reductions folded into an earlier one
        self.n_split = 0                   # fusion groups cut in two at lowering time
        self._materialized: dict = {}
        self._deferred_reduces: list[list[Step]] = [[], []]  # first-stage / second-stage tasks
        self.users: dict[int, list[ir.Node]] = {}
        for n in nodes:
            for i in n.inputs:
                self.users.setdefault(i.id, []).append(n)
        units = self._group(nodes)
        order = self._order(units)

        # consumers outside the producing unit decide what must be stored
        self.need_store: set[int] = set()

        def stored_source(v: ir.Value) -> ir.Value:
            # a row value broadcast over its row inside a group (an alias node) and read from
            # outside that group is not worth a full-size store: the row value is stored and
            # the outside reader sees the broadcast as a view of it
            while v.node.pos in self.alias_nodes:
                v = v.node.inputs[0]
            return v

        for n in nodes:
            cu = self._unit(n.pos)
            for i in n.inputs:
                if n.kind in VIEW_KINDS and n.pos not in self.alias_nodes:
                    # a view forces its source into memory unless that is a view too
                    self.need_store.add(stored_source(i).id)
                    continue
                pu = self._unit(i.node.pos)
                if pu is None or pu is not cu or not cu.fused:
                    self.need_store.add(stored_source(i).id)
        # plan outputs: the first output that names a unit-produced value owns
        # that value's allocation; everything else is copied at the end
        self._out_pending: dict[int, int] = {}
        self._out_done: dict[int, int] = {}
        for oi, v in enumerate(self.outputs):
            self.need_store.add(v.id)
            if v.node.kind not in VIEW_KINDS + ("input", "fill") or v.node.pos in self.alias_nodes:
                if v.id not in self._out_pending:
                    self._out_pending[v.id] = oi

        for u in order:
            if u.fused:
                self._lower_group(u)
            else:
                self._lower_single(u.nodes[0])

        self._flush_reduces()
        outs = []
        for oi, v in enumerate(self.outputs):
            if oi in self._out_done:
                outs.append((self._out_done[oi], v.shape, v.dtype))
                continue
            src = self._resolve(v)
            if (isinstance(src, ViewRef) and src.offset == 0 and
                    tuple(src.strides) == tuple(contiguous_strides(v.shape)) and
                    self.bufs[src.buf].role == "temp" and
                    self.bufs[src.buf].numel == _numel(v.shape) and
                    self.bufs[src.buf].dtype is v.dtype):
                # the output is a reshape of a whole intermediate: that buffer becomes the
                # output allocation instead of being copied into one
                tb = self.bufs[src.buf]
                tb.role, tb.index = "output", oi
                outs.append((tb.id, v.shape, v.dtype))
                continue
            b = self._new_buf(v.shape, v.dtype, "output", oi)
            if isinstance(src, Const):
                self._emit(Step("fill", [], [b.id], dict(buf=b.id, numel=_numel(v.shape),
                                                          value=src.value, dtype=v.dtype)))
            else:
                dst = ViewRef(b.id, 0, v.shape, contiguous_strides(v.shape), v.dtype)
                self._emit(Step("copy", [src.buf], [b.id], dict(src=src, dst=dst)))
            outs.append((b.id, v.shape, v.dtype))
        if any(st.kind == "random" for st in self.steps):
            # the step drew random numbers: its last launch moves the generator on, so that
            # the next run (a replay of the recording included) draws new ones
            self._emit(Step("rng_advance", [], [], {}))
        arena = self._assign_arena()
        stats = {"steps": len(self.steps), "units": len(units),
                 "fused_groups": sum(1 for u in units if u.fused)}
        for s in self.steps:
            stats[s.kind] = stats.get(s.kind, 0) + 1
        if self.n_split:
            stats["split_groups"] = self.n_split
        return Plan(self.bufs, self.steps, len(self.b.inputs), outs, arena, stats)

    def _assign_arena(self) -> int:
        """First-fit offsets for temps whose live ranges overlap."""
        temps = [b for b in self.bufs if b.role == "temp" and b.last >= 0]
        temps.sort(key=lambda b: (b.first, -b.nbytes))
        placed: list[Buf] = []
        top = 0
        for b in temps:
            size = (b.nbytes + 255) & ~255
            busy = sorted((p.offset, p.offset + ((p.nbytes + 255) & ~255)) for p in placed
                          if not (p.last < b.first or p.first > b.last))
            off = 0
            for lo, hi in busy:
                if off + size <= lo:
                    break
                off = max(off, hi)
            b.offset = off
            top = max(top, off + size)
            placed.append(b)
        return top

    # ................................................................ singles
    def _lower_single(self, n: ir.Node) -> None:
        k = n.kind
        out = n.outputs[0]
        if k == "matmul":
            self._lower_matmul(n)
        elif k == "ew":
            self._lower_int64_ew(n)
        elif k == "reduce":
            self._lower_reduce_mid(n)
        elif k == "argreduce":
            x = n.inputs[0]
            axis = n.attrs["axis"]
            src = self._resolve(x)
            if axis != x.rank - 1:
                raise NotImplementedError("argmax/argmin lower only along the last axis; "
                                          "the op permutes other axes first")
            src = self._materialize(src)
            dst = self._alloc_value(out)
            self._emit(Step("argreduce", [src.buf], [dst.buf], dict(
                src=src, dst=dst, rows=_numel(x.shape[:-1]), C=x.shape[-1], fn=n.fn)))
        elif k == "gather":
            table, idx = n.inputs
            axis = n.attrs["axis"]
            t = self._contig(table)
            ix = self._contig(idx)
            dst = self._alloc_value(out)
            self._emit(Step("gather", [t.buf, ix.buf], [dst.buf], dict(
                table=t, idx=ix, dst=dst, outer=_numel(table.shape[:axis]),
                axis_len=table.shape[axis], n_idx=idx.numel(),
                inner=_numel(table.shape[axis + 1:]))))
        elif k == "scatter":
            x, idx, upd = n.inputs
            axis = n.attrs["axis"]
            src = self._resolve(x)
            ix = self._contig(idx)
            up = self._contig(upd)
            dst = self._alloc_value(out)
            if isinstance(src, Const):
                self._emit(Step("fill", [], [dst.buf], dict(buf=dst.buf, numel=out.numel(),
                                                             value=src.value, dtype=out.dtype)))
            else:
                self._copy_into(src, dst, [0] * out.rank, out.shape)
            wbuf = self._new_buf((x.shape[axis],), DType.int32, "temp", -1)
            self._emit(Step("scatter", [ix.buf, up.buf, dst.buf], [dst.buf, wbuf.id], dict(
                idx=ix, upd=up, dst=dst, winner=ViewRef(wbuf.id, 0, (x.shape[axis],), (1,), DType.int32),
                outer=_numel(x.shape[:axis]), axis_len=x.shape[axis], n_idx=idx.numel(),
                inner=_numel(x.shape[axis + 1:]))))
        elif k in ("conv2d", "conv2d_dgrad", "conv2d_wgrad"):
            ins = [self._contig(i) for i in n.inputs]
            dst = self._alloc_value(out)
            if k == "conv2d":
                xs, ws = n.inputs[0].shape, n.inputs[1].shape
                ys = out.shape
            elif k == "conv2d_dgrad":
                xs, ws, ys = out.shape, n.inputs[1].shape, n.inputs[0].shape
            else:
                xs, ws, ys = n.inputs[0].shape, out.shape, n.inputs[1].shape
            attrs = dict(ins=ins, dst=dst, x_shape=xs, w_shape=ws, y_shape=ys,
                         stride=n.attrs["stride"], padding=n.attrs["padding"],
                         has_bias=n.attrs.get("has_bias", False), act=n.attrs.get("act"))
            writes = [dst.buf]
            if k == "conv2d_wgrad":
                nbytes = _wgrad_workspace_bytes(xs, ws, ys)
                if nbytes:
                    wbuf = self._new_buf((nbytes // 4,), DType.float32, "temp", -1)
                    attrs["workspace"] = ViewRef(wbuf.id, 0, (nbytes // 4,), (1,), DType.float32)
                    attrs["workspace_bytes"] = nbytes
                    writes.append(wbuf.id)
            self._emit(Step(k, [i.buf for i in ins], writes, attrs))
        elif k == "matmul_nf4":
            x, codes, scales = (self._contig(i) for i in n.inputs)
            dst = self._alloc_value(out)
            kdim = n.inputs[0].shape[-1]
            self._emit(Step("gemm_nf4", [x.buf, codes.buf, scales.buf], [dst.buf], dict(
                x=x, codes=codes, scales=scales, dst=dst, M=_numel(n.inputs[0].shape[:-1]), K=kdim,
                N=out.shape[-1], w_shape=n.attrs["w_shape"], block=n.attrs["block"],
                transpose=n.attrs["transpose"])))
        elif k in ("attention", "attention_bwd"):
            self._lower_attention(n)
        elif k in ("maxpool2d", "maxpool2d_bwd", "avgpool2d", "avgpool2d_bwd"):
            ins = [self._contig(i) for i in n.inputs]
            dst = self._alloc_value(out)
            if k == "avgpool2d_bwd":
                xs, ys = out.shape, n.inputs[0].shape
            else:
                xs = n.inputs[0].shape
                ys = out.shape if k in ("maxpool2d", "avgpool2d") else n.inputs[1].shape
            self._emit(Step(k, [i.buf for i in ins], [dst.buf], dict(
                ins=ins, dst=dst, x_shape=xs, y_shape=ys, kernel=n.attrs["kernel"],
                stride=n.attrs["stride"], padding=n.attrs["padding"])))
        elif k == "pad":
            src = self._resolve(n.inputs[0])
            dst = self._alloc_value(out)
            self._emit(Step("fill", [], [dst.buf], dict(buf=dst.buf, numel=out.numel(),
                                                         value=n.attrs["value"], dtype=out.dtype)))
            self._copy_into(src, dst, n.attrs["lo"], n.inputs[0].shape)
        elif k == "concat":
            dst = self._alloc_value(out)
            axis = n.attrs["axis"]
            pos = 0
            for i in n.inputs:
                src = self._resolve(i)
                starts = [0] * out.rank
                starts[axis] = pos
                self._copy_into(src, dst, starts, i.shape)
                pos += i.shape[axis]
        elif k == "slice_update":
            x = self._resolve(n.inputs[0])
            upd = self._resolve(n.inputs[1])
            dst = self._alloc_value(out)
            self._copy_into(x, dst, [0] * out.rank, out.shape)
            self._copy_into(upd, dst, n.attrs["starts"], n.inputs[1].shape)
        elif k == "custom":
            ins = [self._contig(i) for i in n.inputs]
            dsts = [self._alloc_value(o) for o in n.outputs]
            self._emit(Step("custom", [i.buf for i in ins], [d.buf for d in dsts], dict(
                ins=ins, dsts=dsts, name=n.attrs["name"], library=n.attrs["library"])))
        elif k in ("adamw_multi", "sgd_multi"):
            self._lower_update_list(n)
        elif k == "random":
            dst = self._alloc_value(out)
            self._emit(Step("random", [], [dst.buf], dict(
                dst=dst, numel=out.numel(), mode=n.attrs["mode"], a=n.attrs["a"], b=n.attrs["b"],
                stream=n.attrs["stream"])))
        else:
            raise NotImplementedError(f"lowering: no rule for node kind '{k}'")

    def _lower_update_list(self, n: ir.Node) -> None:
        """An optimizer step over a list of parameters: one launch whose table holds, per
        parameter, where its tensors are read and where the results go."""
        count = n.attrs["n"]
        per_in = (len(n.inputs) - (1 if n.kind == "adamw_multi" and n.attrs["step"] is None else 0)) // count
        per_out = len(n.outputs) // count
        ins = [self._contig(i) for i in n.inputs]
        outs = [self._alloc_value(o) for o in n.outputs]
        entries = [dict(ins=ins[i * per_in:(i + 1) * per_in], outs=outs[i * per_out:(i + 1) * per_out],
                        numel=n.outputs[i * per_out].numel()) for i in range(count)]
        attrs = {key: val for key, val in n.attrs.items() if key != "n"}
        attrs["entries"] = entries
        attrs["dtype"] = n.outputs[0].dtype
        if n.kind == "adamw_multi" and n.attrs["step"] is None:
            attrs["step_ref"] = ins[-1]
        self._emit(Step(n.kind, [r.buf for r in ins], [r.buf for r in outs], attrs))

    def _copy_into(self, src, dst: ViewRef, starts, shape) -> None:
        off = dst.offset + sum(a * s for a, s in zip(starts, dst.strides))
        window = ViewRef(dst.buf, off, tuple(shape), dst.strides, dst.dtype)
        if isinstance(src, Const):
            src = self._materialize(src)
        self._emit(Step("copy", [src.buf], [dst.buf], dict(src=src, dst=window)))

    def _terminal(self, v: ir.Value) -> bool:
        """Nothing computes on ``v``: it only leaves the plan, possibly through views."""
        for u in self.users.get(v.id, ()):
            if u.kind not in VIEW_KINDS or not self._terminal(u.outputs[0]):
                return False
        return True

    def _emit_reduce(self, step: Step, stage: int, terminal: bool) -> None:
        """A reduction whose result only leaves the plan waits for the end of the plan, where all
        such reductions go out together (one launch per stage instead of one each)."""
        if terminal:
            self._deferred_reduces[stage].append(step)
        else:
            self._emit(step)

    def _fold_column_sums(self) -> None:
        """Deferred column sums whose matrix is the right operand of a product that was emitted
        with room for them (``colsum_key`` on both) become a result of that product's launch:
        the matrix is read once.  A product split along K leaves one row of partial sums per
        slice, which the second stage adds up as it would have the first stage's."""
        hosts = {}  # key -> (step, member of a joined launch)
        for idx, st in enumerate(self.steps):
            if st.kind != "gemm":
                continue
            keys = st.attrs.get("colsum_keys") or [st.attrs.get("colsum_key")]
            for member, key in enumerate(keys):
                if key is not None and key not in hosts:
                    hosts[key] = (idx, member)
        first, second = self._deferred_reduces
        for task in list(first):
            key = task.attrs.get("colsum_key")
            idx, member = hosts.pop(key, (None, 0)) if key is not None else (None, 0)
            if idx is None:
                continue
            host = self.steps[idx]
            batch, n = host.attrs["batch"], host.attrs["N"]
            ks = host.attrs["batch_inner"] if "colsum_keys" in host.attrs else batch
            stage2 = task.attrs.get("second")
            final = (stage2 or task).attrs["dst"]
            first.remove(task)
            if stage2 is not None:
                second.remove(stage2)
            if batch == 1:
                target = ViewRef(final.buf, final.offset, (1, n), (n, 1), final.dtype)
            else:
                # one row of partial sums per batch index of the launch; a joined launch writes
                # the rows of all its members, wanted or not
                target = host.attrs.get("colsum")
                if target is None:
                    tmp = self._new_buf((batch, n), DType.float32)
                    target = ViewRef(tmp.id, 0, (batch, n), (n, 1), DType.float32)
                rows = ViewRef(target.buf, member * ks * n, (ks, n), (n, 1), DType.float32)
                second.append(Step("reduce_mid", [target.buf], [final.buf], dict(
                    src=rows, dst=final, outer=1, red=ks, inner=n, fn="sum")))
            if host.attrs.get("colsum") is None:
                host.attrs["colsum"] = target
                host.writes.append(target.buf)
            b = self.bufs[target.buf]
            b.first, b.last = min(b.first, idx), max(b.last, idx)

    def _flush_reduces(self) -> None:
        if self.fold_column_sums:
            self._fold_column_sums()
        for tasks in self._deferred_reduces:
            if len(tasks) == 1:
                self._emit(tasks[0])
            elif tasks:
                self._emit(Step("reduce_batch", [r for t in tasks for r in t.reads],
                                [w for t in tasks for w in t.writes],
                                dict(tasks=[t.attrs for t in tasks])))
        self._deferred_reduces = [[], []]

    def _lower_reduce_mid(self, n: ir.Node) -> None:
        if n.pos in self.skip_nodes:
            return
        x = n.inputs[0]
        axis = n.attrs["axis"]
        out = n.outputs[0]
        kind = n.fn
        # A chain of keep-dims reductions over neighbouring axes (the un-broadcast of a bias
        # or norm-weight gradient walks the axes one at a time) is one reduction over the
        # merged axis: one pass over the input, fp32 accumulation throughout.
        lo = hi = axis
        # axis_of[i]: axis of x behind axis i of the value the chain has reached (None for a
        # size-1 axis that a reshape inserted)
        axis_of: list = list(range(x.rank))
        while True:
            users = self.users.get(out.id, ())
            if len(users) != 1 or out.id in self._out_pending:
                break
            m = users[0]
            via = None
            if m.kind == "reshape":
                # only size-1 axes may come and go
                keep = [(axis_of[i], d) for i, d in enumerate(out.shape) if d != 1]
                new_dims = [d for d in m.outputs[0].shape if d != 1]
                mu = self.users.get(m.outputs[0].id, ())
                if ([d for _, d in keep] != new_dims or len(mu) != 1 or
                        m.outputs[0].id in self._out_pending):
                    break
                via, m = m, mu[0]
            if (m.kind != "reduce" or m.fn != kind or m.pos in self.skip_nodes or
                    m.attrs["axis"] == m.inputs[0].rank - 1 or self._unit(m.pos) is None or
                    self._unit(m.pos).fused or m.outputs[0].dtype is not out.dtype):
                break
            cur_axes = axis_of
            if via is not None:
                it = iter(a for a, _ in keep)
                cur_axes = [next(it) if d != 1 else None for d in via.outputs[0].shape]
            a2 = cur_axes[m.attrs["axis"]]
            if a2 is None:
                break
            if a2 < lo and all(d == 1 for d in x.shape[a2 + 1:lo]):
                lo = a2
            elif a2 > hi and all(d == 1 for d in x.shape[hi + 1:a2]):
                hi = a2
            else:
                break
            self.skip_nodes.add(m.pos)
            if via is not None:
                self.skip_nodes.add(via.pos)
            axis_of = cur_axes
            out = m.outputs[0]
        src = self._contig(x)
        outer, red, inner = _numel(x.shape[:lo]), _numel(x.shape[lo:hi + 1]), _numel(x.shape[hi + 1:])
        # few output columns and a long axis: split the axis so the launch has
        # enough workgroups, then reduce the partials.  A workgroup covers 64 lanes x
        # one 16-byte vector of columns and wants about 64 rows (16 per wave).
        vec = 16 // x.dtype.size_in_bytes if inner % (16 // x.dtype.size_in_bytes) == 0 else 1
        blocks = outer * ((inner + 64 * vec - 1) // (64 * vec))
        split = 1
        if blocks < 256 and red >= 256 and x.dtype.is_float():  # (partials are fp32)
            want = min(256, red // 64, max(1, 1024 // max(blocks, 1)))
            for s in range(want, 1, -1):
                if red % s == 0 and outer * s <= 65535:
                    split = s
                    break
        terminal = self._terminal(out)
        # the column sums of a matrix that a product also reads as its row-contiguous right
        # operand (a bias gradient beside the weight gradient) can ride on that product
        fold = {}
        if (terminal and self.fold_column_sums and kind == "sum" and outer == 1 and
                x.dtype is DType.bfloat16 and out.dtype is DType.bfloat16):
            fold = dict(colsum_key=(src.buf, src.offset, red, inner))
        if split > 1:
            tmp = self._new_buf((outer, split, inner), DType.float32)
            tref = ViewRef(tmp.id, 0, (outer, split, inner),
                           contiguous_strides((outer, split, inner)), DType.float32)
            dst = self._alloc_value(out)
            second = Step("reduce_mid", [tmp.id], [dst.buf], dict(
                src=tref, dst=dst, outer=outer, red=split, inner=inner, fn=kind))
            if fold:
                fold["second"] = second
            self._emit_reduce(Step("reduce_mid", [src.buf], [tmp.id], dict(
                fold, src=src, dst=tref, outer=outer * split, red=red // split, inner=inner, fn=kind)),
                0, terminal)
            self._emit_reduce(second, 1, terminal)
            return
        dst = self._alloc_value(out)
        self._emit_reduce(Step("reduce_mid", [src.buf], [dst.buf], dict(
            fold, src=src, dst=dst, outer=outer, red=red, inner=inner, fn=kind)), 0, terminal)

    # ................................................................ matmul
    @staticmethod
    def _batch_groups(dims, strides):
        """Batch dims merged into as few (extent, stride) levels as their strides allow."""
        groups: list[tuple[int, int]] = []
        for d, s in zip(dims, strides):
            if d == 1:
                continue
            if groups and (groups[-1][1] == s * d or (groups[-1][1] == 0 and s == 0)):
                groups[-1] = (groups[-1][0] * d, s)
            else:
                groups.append((d, s))
        return groups

    @classmethod
    def _mat_operand(cls, ref: ViewRef):
        """(batch levels, row_stride, col_stride) if the view is a strided batch of
        matrices the GEMM can read directly (one unit stride, at most two batch
        levels), else None."""
        shape, st = ref.shape, ref.strides
        rs, cs = st[-2], st[-1]
        r, c = shape[-2], shape[-1]
        if r == 1:
            rs = c * cs if cs else 1
        if c == 1:
            cs = 1 if rs != 1 else (r * rs)
        if rs != 1 and cs != 1:
            return None
        if rs < 0 or cs < 0 or any(s < 0 for s in st[:-2]):
            return None
        groups = cls._batch_groups(shape[:-2], st[:-2])
        if len(groups) > 2:
            return None
        return (groups, rs, cs)

    def _matmul_out_layout(self, out: ir.Value):
        """Strides the product should be written with.  When its only reader is a permute
        that keeps the last axis (heads [B,H,S,hd] going back to [B,S,H,hd]), the GEMM
        writes that layout directly and the permute becomes a contiguous view."""
        strides = contiguous_strides(out.shape)
        if out.id in self._out_pending or out.rank < 3:
            return strides
        users = self.users.get(out.id, ())
        if len(users) != 1 or users[0].kind != "permute":
            return strides
        perm = users[0].attrs["perm"]
        if perm[-1] != out.rank - 1:
            return strides
        pst = contiguous_strides(tuple(out.shape[p] for p in perm))
        cand = [0] * out.rank
        for i, p in enumerate(perm):
            cand[p] = pst[i]
        if len(self._batch_groups(out.shape[:-2], cand[:-2])) > 2 or cand[-2] < out.shape[-1]:
            return strides
        return tuple(cand)

    def _lower_matmul(self, n: ir.Node) -> None:
        a, b = n.inputs[:2]
        out = n.outputs[0]
        epi: dict = {}
        at = n.attrs or {}
        if "bias_in" in at:
            epi["bias"] = self._contig(n.inputs[at["bias_in"]])
        if "res_in" in at:
            epi["residual"] = self._contig(n.inputs[at["res_in"]])
            epi["res_op"] = "add"
        if at.get("alpha", 1.0) != 1.0:
            epi["alpha"] = at["alpha"]
        if at.get("act"):
            epi["act"] = at["act"]
            if len(n.outputs) > 1:
                epi["aux_value"] = n.outputs[1]  # the activation's derivative, a second result
        ra, rb = self._resolve(a), self._resolve(b)
        if isinstance(ra, Const):
            ra = self._materialize(ra)
        if isinstance(rb, Const):
            rb = self._materialize(rb)
        pa = self._mat_operand(ra)
        if pa is None:
            ra = self._materialize(ra)
            pa = self._mat_operand(ra)
        pb = self._mat_operand(rb)
        if pb is None:
            rb = self._materialize(rb)
            pb = self._mat_operand(rb)
        M, K, N = a.shape[-2], a.shape[-1], b.shape[-1]
        batch = _numel(out.shape[:-2])
        if "terms_in" in at:
            # x[.., M, K] @ W + sum_i u_i[.., M, K_i] @ V_i with 2-D W and V_i: one unbatched
            # product over all rows, for which x and the u_i are read as whole row-major blocks
            # (copied if they are not)
            def rows_of(val, ref):
                if isinstance(ref, Const):
                    ref = self._materialize(ref)
                po = self._mat_operand(ref)
                whole = po is not None and (val.rank == 2 or (
                    len(po[0]) <= 1 and po[2] == 1 and
                    all(g == (_numel(val.shape[:-2]), val.shape[-2] * po[1]) for g in po[0])))
                if not whole:
                    ref = self._materialize(ref)
                    po = self._mat_operand(ref)
                return ref, po

            def one_matrix(val, ref):
                if isinstance(ref, Const):
                    ref = self._materialize(ref)
                if val.rank > 2:  # (broadcast over the batch axes: any one of the copies)
                    if any(st != 0 for d, st in zip(ref.shape[:-2], ref.strides[:-2]) if d > 1):
                        raise AssertionError("product with several operand pairs: a right operand is not one matrix")
                    ref = ViewRef(ref.buf, ref.offset, ref.shape[-2:], ref.strides[-2:], ref.dtype)
                po = self._mat_operand(ref)
                if po is None:
                    ref = self._materialize(ref)
                    po = self._mat_operand(ref)
                return ref, po

            ra, pa = rows_of(a, ra)
            rb, pb = one_matrix(b, rb)
            terms = []
            extra = n.inputs[at["terms_in"]:]
            for u, v in zip(extra[0::2], extra[1::2]):
                ru, pu = rows_of(u, self._resolve(u))
                rv, pv = one_matrix(v, self._resolve(v))
                terms.append(dict(a=ru, b=rv, K=u.shape[-1], a_rs=pu[1], a_cs=pu[2], b_rs=pv[1], b_cs=pv[2]))
            epi["terms"] = terms
            self._emit_plain_gemm(ra, rb, pa, pb, M * batch, N, K, out, epi)
            return
        # sum_b A[b] @ B[b] (the weight gradient x^T dy of a layer applied to a batch) is one
        # product over the contraction index (b, k) when both operands step through it with
        # one stride: no per-batch products to store and add up, fp32 accumulation throughout
        users = self.users.get(out.id, ())
        if (out.rank == 3 and batch > 1 and len(users) == 1 and out.id not in self._out_pending and
                users[0].kind == "reduce" and users[0].fn == "sum" and users[0].attrs["axis"] == 0 and
                users[0].pos not in self.skip_nodes and self._unit(users[0].pos) is not None and
                not self._unit(users[0].pos).fused and
                not (set(epi) - {"alpha"}) and  # a scale commutes with the sum; a bias, a residual
                                                # or an activation per batch element does not
                len(pa[0]) == 1 and len(pb[0]) == 1 and
                pa[0][0] == (batch, K * pa[2]) and pb[0][0] == (batch, K * pb[1])):
            red = users[0]
            self.skip_nodes.add(red.pos)
            self._emit_plain_gemm(ra, rb, pa, pb, M, N, K * batch, red.outputs[0], epi)
            return
        # (a second result or a residual is laid out like the product: both plain row-major then)
        c_strides = self._matmul_out_layout(out) if not ("aux_value" in epi or "residual" in epi) \
            else contiguous_strides(out.shape)
        gc = self._batch_groups(out.shape[:-2], c_strides[:-2])
        # one (outer, inner) split of the batch index has to serve A, B and C
        split = None
        for grp in (gc, pa[0], pb[0]):
            if len(grp) == 2:
                split = (grp[0][0], grp[1][0])
                break
        if split is not None:
            if len(pa[0]) == 2 and (pa[0][0][0], pa[0][1][0]) != split:
                ra = self._materialize(ra)
                pa = self._mat_operand(ra)
            if len(pb[0]) == 2 and (pb[0][0][0], pb[0][1][0]) != split:
                rb = self._materialize(rb)
                pb = self._mat_operand(rb)
            if len(gc) == 2 and (gc[0][0], gc[1][0]) != split:
                c_strides = contiguous_strides(out.shape)
                gc = self._batch_groups(out.shape[:-2], c_strides[:-2])
        inner = split[1] if split is not None else 1

        def levels(groups):
            if not groups:
                return 0, 0
            if len(groups) == 2:
                return groups[0][1], groups[1][1]
            s = groups[0][1]
            return (s * inner, s) if inner > 1 else (s, 0)

        a_bs, a_bs2 = levels(pa[0])
        b_bs, b_bs2 = levels(pb[0])
        c_bs, c_bs2 = levels(gc)
        # x[b, M, K] @ W[K, N] with contiguous x and result is one product with b * M rows:
        # the tiles of all batches then share W's panels in the order the GEMM walks them
        if (batch > 1 and inner == 1 and len(pa[0]) == 1 and all(st == 0 for _, st in pb[0]) and
                pa[2] == 1 and
                pa[0][0][1] == M * pa[1] and c_strides == contiguous_strides(out.shape)):
            M, batch = M * batch, 1
            a_bs = c_bs = 0
        if batch == 1 and c_strides == contiguous_strides(out.shape):
            self._emit_plain_gemm(ra, rb, pa, pb, M, N, K, out, epi)
            return
        if c_strides == contiguous_strides(out.shape):
            dst = self._alloc_value(out)
        else:
            buf = self._new_buf(out.shape, out.dtype, "temp", -1)
            dst = ViewRef(buf.id, 0, out.shape, c_strides, out.dtype)
            self.loc[out.id] = dst
        writes = [dst.buf]
        if "aux_value" in epi:
            epi["aux_dst"] = self._alloc_value(epi.pop("aux_value"))
            writes.append(epi["aux_dst"].buf)
        self._emit(Step("gemm", [ra.buf, rb.buf] + self._epi_bufs(epi), writes, dict(
            epi, a=ra, b=rb, dst=dst, M=M, N=N, K=K, batch=batch, batch_inner=inner,
            a_bs=a_bs, a_rs=pa[1], a_cs=pa[2], b_bs=b_bs, b_rs=pb[1], b_cs=pb[2],
            a_bs2=a_bs2, b_bs2=b_bs2, c_bs2=c_bs2,
            ldc=c_strides[-2] if out.rank >= 2 else N, c_bs=c_bs if batch > 1 else M * N,
            alpha=epi.get("alpha", 1.0))))

    @staticmethod
    def _split_k(M: int, N: int, K: int, dtype: DType, a_k_contiguous: bool = False,
                 rows_contiguous: bool = False) -> int:
        """Slices of the contraction axis for a product whose output has too few 128 x 128
        tiles to occupy the GPU while K is long (weight gradients: K = batch x sequence)."""
        if dtype is not DType.bfloat16:
            return 1
        if a_k_contiguous and N <= 32 and M >= 1024 and K % 64 == 0:
            return 1  # tall products with a few columns have a kernel that splits K by itself
        tiles = ((M + 127) // 128) * ((N + 127) // 128)
        if rows_contiguous and 128 <= tiles <= 256 and K >= 4096 and K % 128 == 0:
            # x^T dy with one workgroup per CU at most: every workgroup walks the same rows of
            # both operands at the same time, and on operands that come from memory (written
            # long before) the launch takes a third longer than on cached ones, whatever the
            # depth of its prefetch.  Two halves of K put two workgroups on a CU that read 40 MB
            # apart: 1024 x 4096 x 8192 113 -> 82 us, plus 10 us for the sum of the halves (four
            # slices: 67 us and 25)
            return 2
        ks = 1
        while tiles * ks < 512 and tiles < 128 and K % (ks * 2 * 64) == 0 and K // (ks * 2) >= 512:
            ks *= 2
        return ks

    @staticmethod
    def _colsum_key(ra: ViewRef, rb: ViewRef, pa, pb, M: int, N: int, K: int, ks: int, epi: dict):
        """What a deferred column sum must name to ride on this product (one launch, or ``ks``
        slices of K): the right operand is a whole row-major [K, N] bf16 matrix, the left one is
        row-contiguous too, and the launch is one that takes the 128 x 128 tile anyway (the
        kernel that carries the sums), with the alignment its direct loads ask for."""
        if epi or ra.dtype is not DType.bfloat16 or rb.dtype is not DType.bfloat16:
            return None
        if not (pa[1] == 1 and pa[2] != 1 and pb[2] == 1 and pb[1] == N):
            return None
        if M % 8 or N % 8 or M < 8 or N < 8 or K % (64 * ks) or K // ks <= 16:
            return None
        if pa[2] % 8 or pa[2] >= 1 << 22 or N >= 1 << 22 or ra.offset % 8 or rb.offset % 8:
            return None
        big = -(-M // 256) * -(-N // 256) * ks
        rounds = -(-big // 256)
        if big * 10 >= rounds * 256 * 6 and M >= 256 and N >= 256 and K // ks > 128:
            return None  # the 256 x 256 tile is the faster launch here
        return (rb.buf, rb.offset, K, N)

    def _emit_plain_gemm(self, ra: ViewRef, rb: ViewRef, pa, pb, M: int, N: int, K: int,
                         out: ir.Value, epi: dict | None = None) -> None:
        """One unbatched product into contiguous storage for ``out``; split along K into fp32
        partial products plus their sum when the output alone gives too few workgroups."""
        ks = self._split_k(M, N, K, ra.dtype if ra.dtype is rb.dtype else DType.float32,
                           a_k_contiguous=pa[2] == 1,
                           rows_contiguous=pa[1] == 1 and pa[2] != 1 and pb[2] == 1 and pb[1] != 1)
        dst = self._alloc_value(out)
        common = dict(a=ra, b=rb, M=M, N=N, a_rs=pa[1], a_cs=pa[2], b_rs=pb[1], b_cs=pb[2],
                      batch_inner=1, a_bs2=0, b_bs2=0, c_bs2=0, ldc=N, c_bs=M * N, alpha=1.0)
        epi = dict(epi or {})
        common["alpha"] = epi.get("alpha", 1.0)
        if ks > 1 and set(epi) - {"alpha"}:
            ks = 1  # (only a scale survives the split: it goes on the partial products)
        key = self._colsum_key(ra, rb, pa, pb, M, N, K, ks, epi) if self.fold_column_sums else None
        if key is not None:
            common["colsum_key"] = key
        if ks == 1:
            writes = [dst.buf]
            if "aux_value" in epi:
                epi["aux_dst"] = self._alloc_value(epi.pop("aux_value"))
                writes.append(epi["aux_dst"].buf)
            self._emit(Step("gemm", [ra.buf, rb.buf] + self._epi_bufs(epi), writes,
                            dict(common, **epi, dst=dst, K=K, batch=1, a_bs=0, b_bs=0)))
            return
        kc = K // ks
        terminal = self._terminal(out)
        if terminal and not epi and self.group_siblings and \
                self._join_sibling_product(ra, rb, common, kc, ks, key, dst):
            return
        tmp = self._new_buf((ks, M, N), DType.float32)
        tref = ViewRef(tmp.id, 0, (ks, M, N), contiguous_strides((ks, M, N)), DType.float32)
        step = Step("gemm", [ra.buf, rb.buf], [tmp.id], dict(
            common, dst=tref, K=kc, batch=ks, a_bs=kc * pa[2], b_bs=kc * pb[1]))
        self._emit(step)
        red = Step("reduce_mid", [tmp.id], [dst.buf], dict(
            src=tref, dst=dst, outer=1, red=ks, inner=M * N, fn="sum"))
        self._emit_reduce(red, 1, terminal)
        if terminal and not epi and common["alpha"] == 1.0:
            # (more may join: _join_sibling_product)
            self._sibling_groups[id(step)] = [dict(off=rb.offset, key=key, reduce=red)]

    def _join_sibling_product(self, ra: ViewRef, rb: ViewRef, common: dict, kc: int, ks: int, key,
                              dst: ViewRef) -> bool:
        """A K-split product A^T B' whose left operand, shape and slices are those of a product
        among the launches just emitted (nothing but products since), with B' in the same buffer
        as that one's right operand(s) and equally spaced with them, joins that launch as one
        more batch member: the batch index becomes (member, slice), the partial products of all
        members lie in one buffer, and the left operand is read once per cache for all of them
        (the weight gradients of the q, k and v projections: three launches -> one)."""
        M, N = common["M"], common["N"]
        for idx in range(len(self.steps) - 1, -1, -1):
            st = self.steps[idx]
            if st.kind != "gemm":
                return False
            members = self._sibling_groups.get(id(st))
            if members is None:
                continue
            h = st.attrs
            n = len(members)
            ks_h = h["batch_inner"] if n > 1 else h["batch"]
            hb = h["b"]
            same = (h["a"] == ra and h["M"] == M and h["N"] == N and h["K"] * ks_h == kc * ks and
                    all(h[f] == common[f] for f in ("a_rs", "a_cs", "b_rs", "b_cs", "ldc", "alpha")) and
                    hb.buf == rb.buf and hb.dtype is rb.dtype and
                    (members[0]["key"] is not None) == (key is not None))
            if not same:
                continue
            # members in the order of their addresses, equally spaced
            order = sorted(members + [dict(off=rb.offset, key=key, reduce=None)], key=lambda m: m["off"])
            spacing = order[1]["off"] - order[0]["off"]
            if spacing <= 0 or spacing % 8 or any(
                    order[j + 1]["off"] - order[j]["off"] != spacing for j in range(n)):
                continue
            # nothing emitted since may write what this member reads
            if any(w in (ra.buf, rb.buf) for later in self.steps[idx + 1:] for w in later.writes):
                return False
            # the launch has the tiles of all its members: fewer slices of K give it three
            # workgroups for two CUs, and fewer partial products go through memory (three
            # members of 64 tiles in the transformer block: 8, 4, 2 slices measured, two is best)
            tiles = -(-M // 128) * -(-N // 128) * (n + 1)
            k_all, ks_new = kc * ks, 2
            while tiles * ks_new < 384 and ks_new < ks:
                ks_new *= 2
            ks = ks_new if (ks_new < ks and k_all % (ks_new * 64) == 0) else ks
            kc = k_all // ks
            tmp = self.bufs[h["dst"].buf]
            tmp.numel = (n + 1) * ks * M * N
            tmp.shape = (n + 1, ks, M, N)
            h.pop("colsum_key", None)
            h.update(K=kc, batch_inner=ks, a_bs2=kc * common["a_cs"], b_bs2=kc * common["b_rs"],
                     c_bs2=M * N, a_bs=0, c_bs=ks * M * N)
            h.update(batch=(n + 1) * ks, b_bs=spacing,
                     b=ViewRef(hb.buf, order[0]["off"], hb.shape, hb.strides, hb.dtype),
                     dst=ViewRef(tmp.id, 0, ((n + 1) * ks, M, N),
                                 contiguous_strides(((n + 1) * ks, M, N)), DType.float32))
            if key is not None:
                h["colsum_keys"] = [m["key"] for m in order]
            for b in (self.bufs[ra.buf], self.bufs[rb.buf]):
                b.first, b.last = min(b.first, idx), max(b.last, idx)
            for j, m in enumerate(order):
                tref = ViewRef(tmp.id, j * ks * M * N, (ks, M, N), contiguous_strides((ks, M, N)),
                               DType.float32)
                if m["reduce"] is None:
                    m["reduce"] = Step("reduce_mid", [tmp.id], [dst.buf], dict(
                        src=tref, dst=dst, outer=1, red=ks, inner=M * N, fn="sum"))
                    self._emit_reduce(m["reduce"], 1, True)
                else:
                    m["reduce"].attrs.update(src=tref, red=ks)
            self._sibling_groups[id(st)] = order
            return True
        return False

    @staticmethod
    def _epi_bufs(epi: dict) -> list[int]:
        return [epi[k].buf for k in ("bias", "residual") if k in epi] + \
            [t[k].buf for t in epi.get("terms", ()) for k in ("a", "b")]

    # ................................................................ attention
    def _heads_operand(self, v: ir.Value) -> ViewRef:
        """A [B, H, S, hd] value where the attention kernels can read it: unit stride along hd
        and every other stride a non-negative multiple of 8 elements (16-byte rows); anything
        else is copied first."""
        ref = self._resolve(v)
        if isinstance(ref, Const):
            return self._materialize(ref)
        ok = ref.strides[-1] == 1 and ref.offset % 8 == 0
        for d, s in zip(ref.shape[:-1], ref.strides[:-1]):
            if d > 1 and (s <= 0 or s % 8):
                ok = False
        return ref if ok else self._materialize(ref)

    def _heads_layout(self, out: ir.Value):
        """Strides in which a [B, H, S, hd] result is written, or None for plain contiguous
        storage.  When it is read through one permute that keeps hd last (the transpose back to
        [B, S, H, hd]) it is written in that order, and the permute becomes a contiguous view."""
        strides = contiguous_strides(out.shape)
        users = self.users.get(out.id, ())
        perms = [u for u in users if u.kind == "permute"]
        # the attention kernels themselves read any layout, so the backward kernel reading the
        # forward result does not stand in the way
        if (out.id not in self._out_pending and len(perms) == 1 and
                perms[0].attrs["perm"][-1] == out.rank - 1 and
                all(u.kind in ("permute", "attention", "attention_bwd") for u in users)):
            perm = perms[0].attrs["perm"]
            pst = contiguous_strides(tuple(out.shape[p] for p in perm))
            cand = [0] * out.rank
            for i, p in enumerate(perm):
                cand[p] = pst[i]
            strides = tuple(cand)
        if strides == contiguous_strides(out.shape) or any(s % 8 for s in strides[:-1]):
            return None
        return strides

    def _heads_result(self, out: ir.Value) -> ViewRef:
        """Storage for a [B, H, S, hd] result (see ``_heads_layout``)."""
        strides = self._heads_layout(out)
        if strides is None:
            return self._alloc_value(out)
        buf = self._new_buf(out.shape, out.dtype, "temp", -1)
        dst = ViewRef(buf.id, 0, out.shape, strides, out.dtype)
        self.loc[out.id] = dst
        return dst

    def _heads_results_side_by_side(self, outs) -> list[ViewRef]:
        """Storage for dq, dk and dv.  Where all three are written in the transposed order they
        share one buffer, equally spaced: the weight gradients x^T dq, x^T dk, x^T dv of three
        projections of one input can then be one batched launch (``_join_sibling_product``)."""
        lay = [self._heads_layout(t) for t in outs]
        same = all(l is not None and l == lay[0] for l in lay) and \
            all(t.shape == outs[0].shape and t.dtype is outs[0].dtype for t in outs)
        n = _numel(outs[0].shape)
        if not (self.group_siblings and same and n % 8 == 0):
            return [self._heads_result(t) for t in outs]
        buf = self._new_buf((len(outs),) + tuple(outs[0].shape), outs[0].dtype, "temp", -1)
        refs = []
        for i, t in enumerate(outs):
            refs.append(ViewRef(buf.id, i * n, t.shape, lay[0], t.dtype))
            self.loc[t.id] = refs[-1]
        return refs

    def _lower_attention(self, n: ir.Node) -> None:
        B, H, S, hd = n.inputs[0].shape
        common = dict(B=B, H=H, S=S, hd=hd, scale=n.attrs["scale"], causal=n.attrs["causal"])
        if n.kind == "attention":
            q, k, v = (self._heads_operand(i) for i in n.inputs)
            o = self._heads_result(n.outputs[0])
            lse = self._alloc_value(n.outputs[1])
            # the rounding remainder of the output is only written where something reads it
            rest = n.outputs[2]
            o_lo = self._alloc_value(rest) if (self.users.get(rest.id) or rest.id in self._out_pending) else None
            self._emit(Step("attention", [q.buf, k.buf, v.buf],
                            [o.buf, lse.buf] + ([o_lo.buf] if o_lo is not None else []),
                            dict(common, q=q, k=k, v=v, o=o, lse=lse, o_lo=o_lo)))
            return
        q, k, v, o = (self._heads_operand(i) for i in n.inputs[:4])
        lse = self._contig(n.inputs[4])
        o_lo = self._heads_operand(n.inputs[5])
        dout = self._heads_operand(n.inputs[6])
        dq, dk, dv = self._heads_results_side_by_side(n.outputs)
        wbuf = self._new_buf((B * H * S,), DType.float32, "temp", -1)
        ws = ViewRef(wbuf.id, 0, (B * H * S,), (1,), DType.float32)
        self._emit(Step("attention_bwd", [q.buf, k.buf, v.buf, o.buf, lse.buf, o_lo.buf, dout.buf],
                        sorted({dq.buf, dk.buf, dv.buf}) + [wbuf.id],
                        dict(common, q=q, k=k, v=v, o=o, lse=lse, o_lo=o_lo, dout=dout, dq=dq, dk=dk, dv=dv,
                             workspace=ws, workspace_bytes=B * H * S * 4)))

    # ................................................................ groups
    def _lower_group(self, g: Unit) -> None:
        """One row program for the group; a group that exceeds a limit of the row-program
        format (operands, registers, instructions) is cut in two in program order, the values
        that cross the cut go through memory, and each half is lowered on its own."""
        snap = (len(self.bufs), dict(self.loc), dict(self._out_pending), dict(self._out_done),
                len(self.steps), dict(self._materialized))
        try:
            step = _RowCodegen(self, g).generate()
        except FusionLimit:
            if len(g.nodes) < 2:
                raise
            del self.bufs[snap[0]:]
            del self.steps[snap[4]:]
            self.loc, self._out_pending, self._out_done = snap[1], snap[2], snap[3]
            self._materialized = snap[5]
            self.n_split += 1
            nodes = sorted(g.nodes, key=lambda n: n.pos)
            cut = len(nodes) // 2
            first = {n.pos for n in nodes[:cut]}
            halves = []
            for part in (nodes[:cut], nodes[cut:]):
                keep = []
                for n in part:
                    if n.pos in self.alias_nodes and n.inputs[0].node.pos in first and n.pos not in first:
                        # a broadcast whose source stays on the other side: an ordinary view again
                        self.alias_nodes.discard(n.pos)
                        self.unit_of.pop(n.pos, None)
                        self.need_store.add(n.inputs[0].id)
                        continue
                    keep.append(n)
                if not keep:
                    continue
                u = Unit(-1, keep[0], True)
                for n in keep[1:]:
                    u.add(n)
                u.lead, u.C = g.lead, g.C
                u.n_reduce = sum(1 for n in keep if n.kind == "reduce")
                for n in keep:
                    self.unit_of[n.pos] = u
                halves.append(u)
            for n in nodes[cut:]:
                for i in n.inputs:
                    if i.node.pos in first:
                        self.need_store.add(i.id)
            for u in halves:
                self._lower_group(u)
            return
        self._emit(step)


# ------------------------------------------------------------------ row codegen
class _VReg:
    __slots__ = ("kind", "id", "t")

    def __init__(self, kind: str, vid: int, t: str = "f"):
        self.kind = kind  # 'v' vector | 's' scalar
        self.id = vid
        self.t = t        # what the 32 bits hold: 'f' fp32 (floats, bool, uint8) | 'i' int32


def _reg_type(dtype: DType) -> str:
    return "i" if dtype in INT_REG_DTYPES else "f"


class _RowCodegen:
    """Turns one fused group into a row program (see include/nbk.h for the ISA)."""

    def __init__(self, planner: Planner, g: Unit):
        self.p = planner
        self.g = g

    # --- domain ------------------------------------------------------------
    def _setup_domain(self):
        g = self.g
        lead, C = tuple(g.lead), g.C
        self.drop_last = False
        if C is None:
            # every member is a row scalar: iterate over the last leading dim instead
            if len(lead) >= 1:
                C = lead[-1]
                lead = lead[:-1]
                self.drop_last = True
            else:
                C = 1
        self.lead = lead
        self.C = C

    def _dom_strides(self, ref: ViewRef):
        """(lead strides, column stride) of an operand shaped like a member value."""
        shape, st = _shape2(ref.shape), ref.strides if ref.shape else (0,)
        if self.drop_last:
            shape, st = shape[:-1], st[:-1]
            if len(shape) == 0:
                return (), 0
        lead_st = tuple(0 if d == 1 else s for d, s in zip(shape[:-1], st[:-1]))
        col = 0 if shape[-1] == 1 else st[-1]
        return lead_st, col

    def _cls_of_shape(self, shape) -> str:
        shape = _shape2(shape)
        if self.drop_last:
            shape = shape[:-1] if len(shape) > 1 else shape
        return "F" if (shape[-1] == self.C and self.C != 1) or self.C == 1 else "R"

    # --- main ----------------------------------------------------------------
    def generate(self) -> Step:
        p, g = self.p, self.g
        self._setup_domain()
        members = sorted(g.nodes, key=lambda n: n.pos)
        member_pos = g.node_pos
        has_reduce = any(n.kind == "reduce" for n in members)
        has_tril = any(n.kind == "tril" for n in members)

        # classes and in-group test
        cls: dict[int, str] = {}
        for n in members:
            o = n.outputs[0]
            if n.kind == "reduce":
                cls[o.id] = "R"
            else:
                cls[o.id] = self._cls_of_shape(o.shape)

        def in_group(v: ir.Value) -> bool:
            return v.node.pos in member_pos and (v.node.kind in FUSABLE or v.node.pos in p.alias_nodes)

        # ---- operands ----------------------------------------------------------
        operands: list[OperandSpec] = []
        op_index: dict[tuple, int] = {}
        op_cls: list[str] = []

        def ext_operand(v: ir.Value):
            """('imm', value) or ('op', index, class) for an external input."""
            loc = p._resolve(v)
            if isinstance(loc, Const):
                return ("imm", float(loc.value), _reg_type(v.dtype))
            lead_st, col = self._dom_strides(loc)
            key = (loc.buf, loc.offset, lead_st, col)
            idx = op_index.get(key)
            if idx is None:
                idx = len(operands)
                op_index[key] = idx
                operands.append(OperandSpec(loc.buf, loc.offset, lead_st, col, loc.dtype, False))
                if all(s == 0 for s in lead_st) and col == 0:
                    op_cls.append("U")
                elif col == 0 and self.C != 1:
                    op_cls.append("R")
                else:
                    op_cls.append("F")
            return ("op", idx, op_cls[idx])

        # ---- phases ------------------------------------------------------------
        ph: dict[int, int] = {}      # value id -> phase it is computed in
        avail: dict[int, int] = {}   # row values: first phase whose prologue can read them
        for n in members:
            o = n.outputs[0]
            if n.kind == "reduce":
                x = n.inputs[0]
                pin = ph[x.id] if in_group(x) else 0
                ph[o.id] = pin
                avail[o.id] = pin + 1
                continue
            m = 0
            for i in n.inputs:
                if in_group(i):
                    m = max(m, avail[i.id] if cls[i.id] == "R" else ph[i.id])
            ph[o.id] = m
            if cls[o.id] == "R":
                avail[o.id] = m
        n_phase = max([0] + [avail.get(n.outputs[0].id, ph[n.outputs[0].id]) for n in members]) + 1

        need_store = p.need_store
        by_id = {n.outputs[0].id: n for n in members}

        # ---- instruction stream with virtual registers -----------------------------
        stream: list[list] = []  # [op, dst, a, b, c, aux]; registers are _VReg
        n_vregs = [0]
        imm_vals: list[float] = []

        def new_v(kind: str, t: str = "f") -> _VReg:
            n_vregs[0] += 1
            return _VReg(kind, n_vregs[0], t)

        sreg_of: dict[Any, _VReg] = {}   # row value id / ('op', idx) / ('imm', value) -> sreg
        out_operand: dict[int, int] = {}

        def store_operand(v: ir.Value) -> int:
            idx = out_operand.get(v.id)
            if idx is None:
                ref = p._alloc_value(v)
                lead_st, col = self._dom_strides(ref)
                idx = len(operands)
                operands.append(OperandSpec(ref.buf, ref.offset, lead_st, col, ref.dtype, False,
                                            is_output=True))
                op_cls.append("O")
                out_operand[v.id] = idx
            return idx

        def imm_index(val) -> int:
            """Slot of an immediate: a Python int is an integer register's (stored by its bits),
            a float an fp32 one."""
            for i, x in enumerate(imm_vals):
                if type(x) is not type(val):
                    continue
                if isinstance(val, int):
                    if x == val:
                        return i
                elif x == val or (x != x and val != val):
                    if math.copysign(1.0, x) == math.copysign(1.0, val) or x != x:
                        return i
            imm_vals.append(val)
            return len(imm_vals) - 1

        prologue: list[list] = []

        def scalar_for(key, emit, t: str = "f") -> _VReg:
            r = sreg_of.get(key)
            if r is None:
                r = new_v("s", t)
                sreg_of[key] = r
                emit(r)
            return r

        def scalar_imm(val: float, t: str = "f") -> _VReg:
            if t == "i" and val == val and abs(val) != math.inf and val == int(val):
                if not -2 ** 31 <= int(val) < 2 ** 31:
                    raise NotImplementedError(
                        f"the integer constant {int(val)} does not fit the 32-bit integer registers "
                        "of a fused kernel")
                return scalar_for(("imm", int(val), "i"), lambda r: prologue.append(
                    [isa.IMM, r, imm_index(int(val)), 0, 0, 0]), "i")
            return scalar_for(("imm", val), lambda r: prologue.append(
                [isa.IMM, r, imm_index(float(val)), 0, 0, 0]))

        def scalar_ext(idx: int) -> _VReg:
            return scalar_for(("op", idx), lambda r: prologue.append([isa.LDR, r, idx, 0, 0, 0]),
                              _reg_type(operands[idx].dtype))

        conv_v: dict = {}  # (register id, type) -> converted vector register, per phase

        def as_type(r: _VReg, t: str, body: list) -> _VReg:
            """``r`` as a register of type ``t``: itself, or its conversion (int32 <-> fp32, the
            float -> int direction toward zero).  A scalar converts once per row, in the
            prologue; a vector register in the body that asks."""
            if r.t == t:
                return r
            op = isa.EW["i2f" if t == "f" else "f2i"]
            if r.kind == "s":
                return scalar_for(("conv", r.id, t), lambda o: prologue.append([op, o, r, 0, 0, 0]), t)
            hit = conv_v.get((r.id, t))
            if hit is None:
                hit = new_v("v", t)
                body.append([op, hit, r, 0, 0, 0])
                conv_v[(r.id, t)] = hit
            return hit

        def truthy(r: _VReg, code: list, kind: str) -> _VReg:
            """A 0 / 1 float for the condition held in ``r``."""
            if r.t == "f":
                return r
            out = new_v(kind, "f")
            code.append([isa.EW["inez"], out, r, 0, 0, 0])
            return out

        def emit_ew(n: ir.Node, get, code: list, kind: str) -> _VReg:
            """Instructions for the elementwise node ``n`` into ``code``; ``get(x, t)`` gives the
            register of operand ``x`` (a Python number becomes an immediate of type ``t``).  Which
            form an operation takes follows the types: integer tensors compute in int32 where
            the operation has an integer form, everything else in fp32 with conversions at the
            edges."""
            fn = n.fn
            o = n.outputs[0]
            ot = _reg_type(o.dtype)
            xs = n.attrs["operands"]
            vals = [x for x in xs if isinstance(x, ir.Value)]

            def conv(r, t):
                if kind == "s" and r.kind != "s":
                    raise AssertionError("vector register in a row-scalar operation")
                return as_type(r, t, code)

            def out(name: str, regs, t: str) -> _VReg:
                r = new_v(kind, t)
                regs = list(regs) + [0] * (3 - len(regs))
                code.append([isa.EW[name], r, regs[0], regs[1], regs[2], 0])
                return r

            if fn in ("mov", "trunc", "nez"):
                src = get(xs[0], ot)
                if fn == "nez":
                    return out("inez" if src.t == "i" else "nez", [src], "f")
                if src.t == ot:
                    return out(fn if ot == "f" else "mov", [src], ot)
                return out("i2f" if ot == "f" else "f2i", [src], ot)
            if fn in ("gt", "ge", "eq", "ne", "lt", "le"):
                whole = all(v.dtype.is_integral() or v.dtype is DType.bool for v in vals) and \
                    all(isinstance(x, ir.Value) or float(x) == int(x) for x in xs)
                ct = "i" if whole and any(_reg_type(v.dtype) == "i" for v in vals) else "f"
                regs = [conv(get(x, ct), ct) for x in xs]
                return out(isa.INT_FORM[fn] if ct == "i" else fn, regs, "f")
            if fn in ("and", "or", "not"):
                return out(fn, [truthy(get(x, "f"), code, kind) for x in xs], "f")
            if fn == "where":
                cond = truthy(get(xs[0], "f"), code, kind)
                return out("where", [cond] + [conv(get(x, ot), ot) for x in xs[1:]], ot)
            if ot == "i" and fn in isa.INT_FORM and \
                    all(isinstance(x, ir.Value) or float(x) == int(x) for x in xs):
                return out(isa.INT_FORM[fn], [conv(get(x, "i"), "i") for x in xs], "i")
            r = out(fn, [conv(get(x, "f"), "f") for x in xs], "f")
            if ot == "i":  # an operation without an integer form (div, pow ...): fp32, then back
                r = out("f2i", [r], "i")
            return r

        def resolve_alias(v: ir.Value) -> ir.Value:
            while v.node.pos in p.alias_nodes and v.node.pos in member_pos:
                v = v.node.inputs[0]
            return v

        def tril_setup(n: ir.Node) -> _VReg:
            """Scalar register holding (matrix row index + k)."""
            key = ("tril", n.attrs["k"])
            r = sreg_of.get(key)
            if r is None:
                row = new_v("s")
                prologue.append([isa.LEADIDX, row, len(self.lead) - 1, 0, 0, 0])
                kreg = scalar_imm(float(n.attrs["k"]))
                r = new_v("s")
                prologue.append([isa.EW["add"], r, row, kreg, 0, 0])
                sreg_of[key] = r
            return r

        acc_slots: dict[int, int] = {}
        for phase in range(n_phase):
            prologue = []
            body: list[list] = []
            vreg_of: dict[Any, _VReg] = {}
            conv_v.clear()

            # 1. reductions finished by the previous body
            for n in members:
                if n.kind == "reduce" and avail[n.outputs[0].id] == phase:
                    r = new_v("s")
                    sreg_of[n.outputs[0].id] = r
                    prologue.append([isa.RED, r, acc_slots[n.outputs[0].id],
                                     isa.RED_KIND[n.fn], 0, 0])
            acc_slots_phase: dict[int, int] = {}

            # 2. sinks of this phase and the set of full values to (re)compute
            sinks: list[ir.Value] = []
            for n in members:
                o = n.outputs[0]
                if n.kind == "reduce":
                    if ph[o.id] == phase:
                        x = n.inputs[0]
                        if len(acc_slots_phase) >= isa.NACC:
                            raise FusionLimit("more than 4 reductions in one phase")
                        acc_slots_phase[o.id] = len(acc_slots_phase)
                        if in_group(x):
                            sinks.append(resolve_alias(x))
                elif cls[o.id] == "F" and ph[o.id] == phase and o.id in need_store:
                    sinks.append(o)
            needed: set[int] = set()
            stack = [s for s in sinks if in_group(s) and cls.get(s.id) == "F"]
            while stack:
                v = stack.pop()
                if v.id in needed:
                    continue
                needed.add(v.id)
                for i in v.node.inputs:
                    if in_group(i):
                        i2 = resolve_alias(i) if i.id not in need_store else i
                        if cls.get(i2.id) == "F" and in_group(i2):
                            stack.append(i2)

            # 3. row-scalar ops that become computable in this phase
            def scalar_operand(x, t: str = "f"):
                """Register of a row-class operand of a scalar op."""
                if not isinstance(x, ir.Value):
                    return scalar_imm(float(x), t)
                if in_group(x):
                    x2 = resolve_alias(x)
                    return sreg_of[x2.id]
                e = ext_operand(x)
                if e[0] == "imm":
                    return scalar_imm(e[1], e[2])
                return scalar_ext(e[1])

            for n in members:
                o = n.outputs[0]
                if n.kind in ("reduce",) or cls[o.id] != "R" or ph[o.id] != phase:
                    continue
                if n.pos in p.alias_nodes:
                    continue
                if n.kind != "ew":
                    raise FusionLimit(f"row-class node of kind {n.kind}")
                sreg_of[o.id] = emit_ew(n, scalar_operand, prologue, "s")
            # stores of row values that became available in this phase
            for n in members:
                o = n.outputs[0]
                if cls[o.id] == "R" and avail[o.id] == phase and o.id in need_store and \
                        n.pos not in p.alias_nodes:
                    prologue.append([isa.STR, store_operand(o), sreg_of[o.id], 0, 0, 0])

            # 4. body: full-class ops in topological order
            def vec_operand(x, t: str = "f"):
                if not isinstance(x, ir.Value):
                    return scalar_imm(float(x), t)
                if in_group(x):
                    x2 = resolve_alias(x) if x.id not in vreg_of else x
                    if cls.get(x2.id) == "R":
                        return sreg_of[x2.id]
                    return vreg_of[x2.id]
                e = ext_operand(x)
                if e[0] == "imm":
                    return scalar_imm(e[1], e[2])
                _, idx, c = e
                if c in ("U", "R"):
                    return scalar_ext(idx)
                key = ("op", idx)
                r = vreg_of.get(key)
                if r is None:
                    r = new_v("v", _reg_type(operands[idx].dtype))
                    vreg_of[key] = r
                    body.append([isa.LDG, r, idx, 0, 0, 0])
                return r

            for n in members:
                o = n.outputs[0]
                if n.kind == "reduce":
                    if ph[o.id] == phase:
                        x = n.inputs[0]
                        src = as_type(vec_operand(x), "f", body)  # (accumulators are fp32)
                        if src.kind == "s":  # reducing a row scalar broadcast: materialise it
                            t = new_v("v")
                            body.append([isa.EW["mov"], t, src, 0, 0, 0])
                            src = t
                        body.append([isa.ACC, acc_slots_phase[o.id], src, isa.RED_KIND[n.fn], 0, 0])
                    continue
                if o.id not in needed:
                    continue
                if n.pos in p.alias_nodes:
                    src = vec_operand(n.inputs[0])
                    r = new_v("v", src.t)
                    body.append([isa.EW["mov"], r, src, 0, 0, 0])
                elif n.kind == "ew":
                    r = emit_ew(n, vec_operand, body, "v")
                elif n.kind == "tril":
                    lim = tril_setup(n)
                    x = vec_operand(n.inputs[0])
                    zero = scalar_imm(0.0)  # (all bits clear: zero of either register type)
                    c = new_v("v")
                    body.append([isa.COLIDX, c, 0, 0, 0, 0])
                    m = new_v("v")
                    body.append([isa.EW["ge" if n.attrs["upper"] else "le"], m, c, lim, 0, 0])
                    r = new_v("v", x.t)
                    body.append([isa.EW["where"], r, m, x, zero, 0])
                elif n.kind == "iota":
                    start, step = n.attrs["start"], n.attrs["step"]
                    if _reg_type(o.dtype) == "i" and start == int(start) and step == int(step):
                        r = new_v("v", "i")
                        body.append([isa.COLIDX, r, 1, 0, 0, 0])  # the column as an int32
                        if step != 1:
                            t = new_v("v", "i")
                            body.append([isa.EW["imul"], t, r, scalar_imm(step, "i"), 0, 0])
                            r = t
                        if start != 0:
                            t = new_v("v", "i")
                            body.append([isa.EW["iadd"], t, r, scalar_imm(start, "i"), 0, 0])
                            r = t
                    else:
                        c = new_v("v")
                        body.append([isa.COLIDX, c, 0, 0, 0, 0])
                        r = new_v("v")
                        body.append([isa.EW["fma"], r, c, scalar_imm(n.attrs["step"]),
                                     scalar_imm(n.attrs["start"]), 0])
                        r = as_type(r, _reg_type(o.dtype), body)
                else:
                    raise AssertionError(n.kind)
                vreg_of[o.id] = r
                if o.id in need_store and ph[o.id] == phase:
                    body.append([isa.STG, store_operand(o), r, 0, 0, 0])

            for oid, slot in acc_slots_phase.items():
                prologue.append([isa.ACCINIT, slot, isa.RED_KIND[by_id[oid].fn], 0, 0, 0])
            acc_slots.update(acc_slots_phase)
            stream.extend(prologue)
            if body:
                stream.append([isa.BODY, 0, 0, 0, 0, len(body)])
                stream.extend(body)
        stream.append([isa.HALT, 0, 0, 0, 0, 0])

        ins = self._allocate(stream)
        if len(ins) > isa.MAX_INS:
            raise FusionLimit(f"{len(ins)} instructions")
        if len(operands) > isa.MAX_OPERANDS:
            raise FusionLimit(f"{len(operands)} operands")
        if len(imm_vals) > isa.MAX_IMM:
            raise FusionLimit(f"{len(imm_vals)} immediates")

        lead, C = self._finish_domain(operands, has_reduce, has_tril, stream, op_cls)
        # LDS staging of rows that are read in more than one phase
        n_stage = 0
        if has_reduce:
            loads: dict[int, int] = {}
            for i in ins:
                if i[0] == isa.LDG:
                    loads[i[2]] = loads.get(i[2], 0) + 1
            c_pad = (C + 3) & ~3
            for idx, cnt in sorted(loads.items()):
                if cnt >= 2 and n_stage < isa.MAX_STAGE and (n_stage + 1) * c_pad * 4 <= isa.STAGE_BYTES:
                    operands[idx].stage_slot = n_stage
                    n_stage += 1
        chunks = (C + 3) // 4
        # chunks a lane may own: long rows of few inputs keep up to 8 float4 per input in
        # registers (16 in all), which halves the workgroup and its barrier cost
        cpt_max = 8
        n_in = max(1, len({i[2] for i in ins if i[0] == isa.LDG}))
        while cpt_max > 1 and cpt_max * n_in > 16:
            cpt_max //= 2
        block = 64
        while block < isa.MAX_BLOCK and block * cpt_max < chunks:
            block *= 2
        reads = sorted({o.buf for o in operands if not o.is_output})
        writes = sorted({o.buf for o in operands if o.is_output})
        return Step("rowprog", reads, writes, dict(
            lead=lead, C=C, has_reduce=has_reduce, block=block, n_stage=n_stage,
            operands=operands, ins=ins, imm=imm_vals,
            members=[f"{n.kind}.{n.fn}" if n.fn else n.kind for n in members]))

    # --- domain collapse -----------------------------------------------------------
    def _finish_domain(self, operands, has_reduce, has_tril, stream, op_cls):
        lead = list(self.lead)
        C = self.C
        sts = [list(o.lead_strides) for o in operands]
        uses_leadidx = any(i[0] == isa.LEADIDX for i in stream)
        # drop unit leading dims, merge adjacent ones that every operand walks linearly
        k = 0
        while k < len(lead):
            if lead[k] == 1 and not (uses_leadidx and k == len(lead) - 1):
                del lead[k]
                for s in sts:
                    del s[k]
                continue
            k += 1
        if not uses_leadidx:
            k = 0
            while k + 1 < len(lead):
                if all(s[k] == s[k + 1] * lead[k + 1] for s in sts):
                    lead[k] = lead[k] * lead[k + 1]
                    del lead[k + 1]
                    for s in sts:
                        s[k] = s[k + 1]
                        del s[k + 1]
                    continue
                k += 1
        per_row = any(i[0] in (isa.LDR, isa.STR, isa.LEADIDX) for i in stream)
        row_ops = {i[2] for i in stream if i[0] == isa.LDR} | {i[1] for i in stream if i[0] == isa.STR}
        uniform_only = all(all(x == 0 for x in sts[j]) and operands[j].col_stride == 0
                           for j in row_ops)
        if not has_reduce and not has_tril and (not per_row or uniform_only):
            # pure elementwise: fold leading dims into the row while every
            # operand stays linear
            while lead:
                ok = all((o.col_stride == 1 and s[-1] == C) or
                         (o.col_stride == 0 and all(x == 0 for x in s))
                         for o, s in zip(operands, sts))
                if not ok:
                    break
                C *= lead[-1]
                lead.pop()
                for s in sts:
                    s.pop()
        if len(lead) > isa.MAX_LEAD:
            raise FusionLimit(f"{len(lead)} leading dims after collapse")
        for o, s in zip(operands, sts):
            o.lead_strides = tuple(s)
            o.vec_ok = bool(o.col_stride == 1 and o.offset % 4 == 0 and all(x % 4 == 0 for x in s))
        return tuple(lead), C

    # --- register allocation -------------------------------------------------------
    def _allocate(self, stream):
        """Map virtual registers to the 16 vector + 16 scalar physical ones.

        Vector registers live inside one body; scalar registers live across the
        program, and one that is read inside a body stays reserved until the
        body's last instruction (the body runs once per chunk)."""
        def regs_of(ins):
            op = ins[0]
            dst = None
            if op in (isa.IMM, isa.LDR, isa.LEADIDX, isa.RED, isa.LDG, isa.COLIDX) or op >= 16:
                dst = ins[1]
            srcs = [x for x in ins[2:5] if isinstance(x, _VReg)]
            return dst, srcs

        body_end: dict[int, int] = {}
        i = 0
        while i < len(stream):
            if stream[i][0] == isa.BODY:
                end = i + stream[i][5]
                for q in range(i + 1, end + 1):
                    body_end[q] = end
                i = end + 1
            else:
                i += 1
        last: dict[int, int] = {}
        reg_by_id: dict[int, _VReg] = {}
        for idx, ins in enumerate(stream):
            dst, srcs = regs_of(ins)
            for r in srcs + ([dst] if dst is not None else []):
                pos = body_end.get(idx, idx) if r.kind == "s" else idx
                last[r.id] = max(last.get(r.id, -1), pos)
                reg_by_id[r.id] = r
        free_at: dict[int, list[_VReg]] = {}
        for rid, pos in last.items():
            free_at.setdefault(pos, []).append(reg_by_id[rid])

        free_s = list(range(isa.NVEC + isa.NSCL - 1, isa.NVEC - 1, -1))
        free_v = list(range(isa.NVEC - 1, -1, -1))
        phys: dict[int, int] = {}
        out = []
        for idx, ins in enumerate(stream):
            if ins[0] == isa.BODY:
                free_v = list(range(isa.NVEC - 1, -1, -1))
            dst, srcs = regs_of(ins)
            enc = list(ins)
            for k in range(2, 5):
                if isinstance(enc[k], _VReg):
                    enc[k] = phys[enc[k].id]
            dying = free_at.get(idx, [])
            for r in dying:  # sources that die here may be reused by the destination
                if r.id in phys and (dst is None or r.id != dst.id):
                    (free_v if r.kind == "v" else free_s).append(phys[r.id])
            if dst is not None:
                pool = free_v if dst.kind == "v" else free_s
                if dst.id not in phys:
                    if not pool:
                        raise FusionLimit("out of registers")
                    phys[dst.id] = pool.pop()
                enc[1] = phys[dst.id]
                if any(r.id == dst.id for r in dying):
                    pool.append(phys[dst.id])
            out.append(tuple(int(x) for x in enc))
        return out


def _fold_empty(builder: ir.Builder) -> None:
    """Tensors without elements never reach a kernel.  A node whose results are all empty needs
    no work; a node that makes something out of nothing has a value that is known beforehand: a
    sum over an empty axis and a product with an empty contraction are zero (a maximum or minimum
    of nothing has no value and is an error, as in numpy).  Both kinds become constants here, so
    the passes and kernels behind see non-empty operands only."""
    for n in builder.nodes:
        if n.kind in ("input", "fill"):
            continue
        if all(_numel(o.shape) == 0 for o in n.outputs):
            value = 0.0
        elif any(_numel(i.shape) == 0 for i in n.inputs):
            if n.kind == "reduce" and n.fn != "sum":
                raise ValueError(f"{n.fn} over an axis of length 0 has no value "
                                 f"(input of shape {tuple(n.inputs[0].shape)})")
            if n.kind not in ("reduce", "matmul", "matmul_nf4", "concat", "pad", "slice_update",
                              "scatter"):
                raise NotImplementedError(f"'{n.kind}' with an empty operand and a non-empty result")
            if n.kind in ("concat", "pad", "slice_update", "scatter"):
                continue  # (copies of the empty pieces are skipped when they are lowered)
            value = 0.0
        else:
            continue
        n.kind, n.fn, n.inputs, n.attrs = "fill", None, [], {"value": value}


def plan_graph(builder: ir.Builder, outputs: Sequence[ir.Value]) -> Plan:
    """Plan with shrinking fusion limits until every group fits a row program."""
    last = None
    # graph rewrites happen once, before the attempts below share the builder
    _fold_empty(builder)
    pre = Planner(builder, outputs)
    pre._rematerialize_masks()
    from .. import config
    if config.FOLD_SCALE:
        pre._fold_scale_into_matmul()
    pre._fold_bias_into_matmul()
    if config.FOLD_RESIDUAL or config.FOLD_THIN_RESIDUAL:
        pre._fold_sum_into_matmul(thin_only=not config.FOLD_RESIDUAL)
        if config.FOLD_THIN_PAIR:
            pre._fold_thin_pair_into_matmul()
            if config.FOLD_PRODUCT_SUMS:
                pre._fold_product_sums()
        pre._fold_bias_into_matmul()  # (a bias on top of a sum that has just become a product)
    if config.FOLD_ACTIVATION:
        pre._fold_activation_into_matmul()
    if config.FOLD_RELU:
        pre._fold_relu_into_producer()
    outputs = pre.outputs
    for limit in (28, 16, 8, 4, 1):
        try:
            return Planner(builder, outputs, max_members=limit).build()
        except FusionLimit as e:  # retry with smaller groups
            last = e
    raise RuntimeError(f"lowering failed even without fusion: {last}")
