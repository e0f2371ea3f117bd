"""Ahead-of-time specialisation of row programs.

The interpreter in ``csrc/rowprog.hip`` runs any fused group, but it pays a
decode cost per instruction.  For the row programs that the lowering pass emits
for the five benchmark steps, this module turns the instruction stream into
straight-line HIP (same skeleton: persistent workgroups, 16-byte coalesced
chunks, LDS staging of rows that are read in several phases, wavefront-shuffle +
LDS-tree reductions) and writes them to ``csrc/rowprog_spec_gen*.hip`` together
with a lookup table keyed by a hash of the program.  ``nbk_rowprog_launch``
hashes the program it is given and uses the specialised kernel when one exists.

    python -m nabla_amd.backend.specialize          # regenerate the sources

Generation needs no GPU: the steps are traced with uninitialised host tensors
and planned; nothing is executed.
"""
from __future__ import annotations

import struct
from pathlib import Path

import torch

from . import isa
from .planner import Plan

CSRC = Path(__file__).resolve().parents[1] / "csrc"
N_FILES = 4  # generated sources are split so that they compile in parallel

_FNV_OFFSET = 0xCBF29CE484222325
_FNV_PRIME = 0x100000001B3


def cs_class(col_stride: int) -> int:
    return 0 if col_stride == 0 else 1 if col_stride == 1 else 2


def program_bytes(a: dict) -> bytes:
    """Canonical byte string of a row program; must match rp_program_hash() in
    csrc/rowprog.hip."""
    ops = a["operands"]
    out = struct.pack("<BBHBB", 1 if a["has_reduce"] else 0, len(ops), len(a["ins"]), len(a["imm"]),
                      a["n_stage"])
    for o in ops:
        out += struct.pack("<BBBb", o.dtype.abi, cs_class(o.col_stride), 1 if o.vec_ok else 0,
                           o.stage_slot)
    for i in a["ins"]:
        out += struct.pack("<BBBBBBH", i[0], i[1], i[2], i[3], i[4], 0, i[5])
    for v in a["imm"]:  # (an int is an integer register's immediate: its bits)
        out += struct.pack("<i", v) if isinstance(v, int) else struct.pack("<f", v)
    return out


def program_hash(a: dict) -> int:
    h = _FNV_OFFSET
    for b in program_bytes(a):
        h = ((h ^ b) * _FNV_PRIME) & 0xFFFFFFFFFFFFFFFF
    return h


# ------------------------------------------------------------------------ codegen
def _reg(r: int) -> str:
    return f"v{r}" if r < isa.NVEC else f"s{r}"


def _as_vec(r: int) -> str:
    return f"v{r}" if r < isa.NVEC else f"rp_splat(s{r})"


def _ew_vec(op: int, dst: int, a: int, b: int, c: int, lowp: bool = False) -> str:
    name = isa.EW_NAME[op]
    lp = ", true" if lowp else ""
    if name in isa.UNARY:
        return f"v{dst} = rp_un4<{op}{lp}>({_as_vec(a)});"
    if name in isa.BINARY:
        return f"v{dst} = rp_bin4<{op}{lp}>({_as_vec(a)}, {_as_vec(b)});"
    if name == "where":
        return f"v{dst} = rp_where4({_as_vec(a)}, {_as_vec(b)}, {_as_vec(c)});"
    return f"v{dst} = rp_fma4({_as_vec(a)}, {_as_vec(b)}, {_as_vec(c)});"


def _ew_scalar(op: int, dst: int, a: int, b: int, c: int, lowp: bool = False) -> str:
    name = isa.EW_NAME[op]
    lp = "_lowp" if lowp else ""
    if name in isa.UNARY:
        return f"s{dst} = rp_unary{lp}({op}, s{a});"
    if name in isa.BINARY:
        return f"s{dst} = rp_binary{lp}({op}, s{a}, s{b});"
    if name == "where":
        return f"s{dst} = rp_where(s{a}, s{b}, s{c});"
    return f"s{dst} = fmaf(s{a}, s{b}, s{c});"


MAX_RESIDENT_REGS = 16  # float4 registers a row-resident kernel may spend on inputs
PREFETCH_MAX_REGS = 8   # ... and on the next row's inputs when rows are software-pipelined


def full_inputs(a: dict) -> list[int]:
    """Operand indices that the bodies load with LDG."""
    return sorted({i[2] for i in a["ins"] if i[0] == isa.LDG})


def stage16_operand(a: dict) -> int | None:
    """The input whose row the LDS-staged generic form keeps: reduction programs over rows no
    register-resident form can hold, with a 16-bit, unit-stride input that at least two
    phases read.  (The row length a kernel meets at run time may differ from the one planned
    here; the launch checks it again.)"""
    if not a["has_reduce"] or a.get("n_stage", 0) or a["C"] % 4 or a["C"] * 2 > 64000:
        return None
    if (a["C"] + 3) // 4 <= 8 * 512:
        return None
    loads: dict[int, int] = {}
    for i in a["ins"]:
        if i[0] == isa.LDG:
            loads[i[2]] = loads.get(i[2], 0) + 1
    for k, n in sorted(loads.items()):
        o = a["operands"][k]
        if n >= 2 and o.dtype.abi in (1, 2) and o.vec_ok and o.col_stride == 1 and not o.is_output:
            return k
    return None


def generate_kernel(a: dict, name: str, cpt: int = 0, stage16: int | None = None) -> str:
    """HIP source of one specialised kernel for the row program ``a``.

    ``cpt`` = 0: generic form, chunk loops with a run-time trip count, rows that
    are read in several phases staged in LDS.  ``cpt`` > 0 (reduction programs
    only): every lane owns exactly ``cpt`` chunks of the row; all inputs are
    loaded once into registers with every load in flight together, the chunk
    loops are fully unrolled, and arithmetic repeated in a later phase is
    removed by the compiler's common-subexpression elimination."""
    ops = a["operands"]
    ins = a["ins"]
    block_mode = bool(a["has_reduce"])
    resident = cpt > 0
    assert not resident or block_mode
    inputs = full_inputs(a)
    # every stored tensor a 16-bit float: hardware transcendentals are accurate enough
    stored = {i[1] for i in ins if i[0] in (isa.STR, isa.STG)}
    lowp = bool(stored) and all(ops[k].dtype.abi in (1, 2) for k in stored)
    L: list[str] = []
    w = L.append
    if block_mode:
        # register-resident forms: cap registers so that two 512-lane workgroups (or
        # more smaller ones) share a CU and one loads while the other computes
        occ = ""
        if resident:
            # FULL: the row is exactly cpt chunks per lane, no lane or element is masked
            # STREAM: fp32 unit-stride operands are read and written with the non-temporal hint
            w("template <bool FULL, bool STREAM>")
        w(f"__global__ __launch_bounds__(512) {occ}void {name}(const nbk_rowprog P, int64_t rows) {{")
        w("  __shared__ float red_buf[64];")
        w("  int red_phase = 0; (void)red_phase;")
        w("  const int64_t C = P.C, c_pad = (C + 3) & ~(int64_t)3, n_chunks = c_pad >> 2;")
        w("  const bool writer = threadIdx.x == 0;")
        w("  (void)c_pad;")
    else:
        # FLAT: the launch has a single row (a flat array): no row arithmetic, every operand at offset 0
        w("template <bool FLAT>")
        w(f"__global__ __launch_bounds__(256) void {name}(const nbk_rowprog P, uint32_t cpr, "
          "uint64_t total_chunks) {")
        w("  const int64_t C = P.C;")
    w("  (void)C;")
    # operand descriptors with the specialised fields folded to constants
    for k, o in enumerate(ops):
        w(f"  nbk_operand o{k} = P.operand[{k}]; o{k}.dtype = {o.dtype.abi}; "
          f"o{k}.vec_ok = {1 if o.vec_ok else 0}; o{k}.stage_slot = {o.stage_slot};"
          + (f" o{k}.col_stride = {o.col_stride};" if o.col_stride in (0, 1) else ""))
    w("  const int64_t ld1 = P.lead_dim[1], ld2 = P.lead_dim[2], ld3 = P.lead_dim[3];")
    used_s = sorted({r for i in ins for r in (i[1], i[2], i[3], i[4]) if isa.NVEC <= r < 32})
    written = {i[1] for i in ins if i[0] in (isa.STR, isa.STG)}
    hoisted: dict[int, str] = {}
    for i in ins:
        # scalar operand reads do not depend on anything the row computes: issue them with
        # the row's first loads instead of between the phases, where their latency is exposed
        if i[0] == isa.LDR and i[2] not in written and i[2] not in hoisted:
            hoisted[i[2]] = f"ldr{i[2]}"
    decomp = ("rp_decompose_row((uint32_t)(ROW), P.n_lead, (uint32_t)ld1, (uint32_t)ld2, "
              "(uint32_t)ld3, LI);")
    if resident:
        # Software pipeline over the rows of a persistent workgroup: the loads of the next
        # row are issued before the current row is computed and stored, so a row's load
        # latency overlaps the previous row's arithmetic and never queues behind its stores.
        w(f"  int64_t colj[{cpt}]; int validj[{cpt}];")
        w("#pragma unroll")
        w(f"  for (int j = 0; j < {cpt}; ++j) {{")
        w("    const int64_t ch = threadIdx.x + (int64_t)j * blockDim.x;")
        w("    colj[j] = ch << 2;")
        w("    const int64_t left = C - colj[j];")
        w("    validj[j] = FULL ? 4 : (ch < n_chunks ? (left >= 4 ? 4 : (int)left) : 0);")
        w("  }")
        w("  uint32_t nlead[4];")
        w("  int64_t " + ", ".join(f"noff{k} = 0" for k in range(len(ops))) + ";")
        for k in hoisted:
            w(f"  float nldr{k} = 0.f;")
        for k in inputs:
            w(f"  float4 n{k}[{cpt}];")

        def fetch(row_expr: str, ind: str) -> None:
            w(ind + decomp.replace("ROW", row_expr).replace("LI", "nlead"))
            w(ind + "if (P.n_lead <= 1) {")
            for k in range(len(ops)):
                w(ind + f"  noff{k} = (int64_t)nlead[0] * o{k}.lead_stride[0];")
            w(ind + "} else {")
            for k in range(len(ops)):
                w(ind + f"  noff{k} = rp_row_offset(o{k}, nlead, 4);")
            w(ind + "}")
            for k in hoisted:
                w(ind + f"nldr{k} = rp_load1(o{k}.ptr, noff{k}, o{k}.dtype);")
            for k in inputs:
                full_load = f"rp_load4(o{k}, noff{k}, colj[j], 4)"
                if ops[k].dtype.abi == 0 and ops[k].vec_ok and ops[k].col_stride == 1:
                    full_load = (f"(STREAM ? rp_load4_stream((const float*)o{k}.ptr + noff{k} + colj[j]) : "
                                 f"{full_load})")
                w("#pragma unroll")
                w(ind + f"for (int j = 0; j < {cpt}; ++j) n{k}[j] = FULL ? {full_load} : "
                  f"(validj[j] > 0 ? rp_load4(o{k}, noff{k}, colj[j], validj[j]) : "
                  "make_float4(0.f, 0.f, 0.f, 0.f));")

        # the pipeline doubles the registers that hold inputs; past 8 float4 per lane that
        # costs more occupancy than the overlap returns
        prefetch = cpt * max(1, len(inputs)) <= PREFETCH_MAX_REGS
        if prefetch:
            fetch("blockIdx.x", "  ")
        w("  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {")
        if not prefetch:
            fetch("row", "    ")
        w("    uint32_t lead_idx[4] = {nlead[0], nlead[1], nlead[2], nlead[3]};")
        w("    (void)lead_idx;")
        for k in range(len(ops)):
            w(f"    const int64_t off{k} = noff{k};")
        for k in hoisted:
            w(f"    const float ldr{k} = nldr{k};")
        for k in inputs:
            w(f"    float4 r{k}[{cpt}];")
            w("#pragma unroll")
            w(f"    for (int j = 0; j < {cpt}; ++j) r{k}[j] = n{k}[j];")
        if prefetch:
            w("    if (row + gridDim.x < rows) {")
            fetch("row + gridDim.x", "      ")
            w("    }")
    elif block_mode:
        w("  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {")
        # the host rejects launches of 2^31 rows or more, so 32-bit division is exact
        w("    uint32_t lead_idx[4];")
        w("    " + decomp.replace("ROW", "row").replace("LI", "lead_idx"))
    else:
        # scalar operands that do not move with the row (constants such as 0.5 or 1/sqrt(2)) are
        # read once, not once per chunk
        for k in hoisted:
            w(f"  const bool uni{k} = (o{k}.lead_stride[0] | o{k}.lead_stride[1] | o{k}.lead_stride[2] | "
              f"o{k}.lead_stride[3]) == 0;")
            w(f"  const float pre{k} = uni{k} ? rp_load1(o{k}.ptr, 0, o{k}.dtype) : 0.f;")
        w("  const uint64_t stride = (uint64_t)gridDim.x * 256u;")
        w("  const bool small = total_chunks <= 0xffffffffull;  // 32-bit row arithmetic suffices")
        w("  for (uint64_t g = (uint64_t)blockIdx.x * 256u + threadIdx.x; g < total_chunks; g += stride) {")
        w("    uint32_t row, cc;")
        w("    if (FLAT) { row = 0; cc = (uint32_t)g; }")
        w("    else if (cpr == 1) { row = (uint32_t)g; cc = 0; }")
        w("    else if (total_chunks <= cpr) { row = 0; cc = (uint32_t)g; }")
        w("    else if (small) { row = (uint32_t)g / cpr; cc = (uint32_t)g - row * cpr; }")
        w("    else { row = (uint32_t)(g / cpr); cc = (uint32_t)(g - (uint64_t)row * cpr); }")
        w("    uint32_t lead_idx[4] = {0, 0, 0, 0};")
        w("    if (!FLAT && P.n_lead > 0) " + decomp.replace("ROW", "row").replace("LI", "lead_idx"))
        w("    const bool writer = cc == 0;")
        w("    const int64_t col = (int64_t)cc << 2;")
        w("    const int64_t left = C - col;")
        w("    const int valid = left >= 4 ? 4 : (int)left;")
    if not resident:
        if block_mode:
            for k in range(len(ops)):
                w(f"    const int64_t off{k} = rp_row_offset(o{k}, lead_idx, 4);")
            for k in hoisted:
                w(f"    const float ldr{k} = rp_load1(o{k}.ptr, off{k}, o{k}.dtype);")
        else:
            # per-lane rows: with at most one leading dim an offset is one multiply-add
            w("    int64_t " + ", ".join(f"off{k}" for k in range(len(ops))) + ";")
            w("    if (FLAT) {")
            w("      " + " ".join(f"off{k} = 0;" for k in range(len(ops))))
            w("    } else if (P.n_lead <= 1) {")
            for k in range(len(ops)):
                w(f"      off{k} = (int64_t)lead_idx[0] * o{k}.lead_stride[0];")
            w("    } else {")
            for k in range(len(ops)):
                w(f"      off{k} = rp_row_offset(o{k}, lead_idx, 4);")
            w("    }")
            for k in hoisted:
                w(f"    const float ldr{k} = uni{k} ? pre{k} : rp_load1(o{k}.ptr, off{k}, o{k}.dtype);")
        if block_mode and a["n_stage"] > 0:
            for k, o in enumerate(ops):
                if o.stage_slot >= 0:
                    w(f"    rp_stage_row(o{k}, off{k}, rp_stage_lds + {o.stage_slot} * c_pad, C, n_chunks);")
        if stage16 is not None:
            w(f"    rp_stage_row16(o{stage16}, off{stage16}, (uint2*)rp_stage_lds, n_chunks);")
    if used_s:
        w("    float " + ", ".join(f"s{r} = 0.f" for r in used_s) + ";")
    w("    float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;")
    w("    (void)acc0; (void)acc1; (void)acc2; (void)acc3; (void)writer;")

    pc = 0
    while pc < len(ins):
        op, dst, x, y, z, aux = ins[pc]
        if op == isa.HALT:
            break
        if op == isa.BODY:
            body = ins[pc + 1:pc + 1 + aux]
            ind = "      " if block_mode else "    "
            if resident:
                w("#pragma unroll")
                w(f"    for (int j = 0; j < {cpt}; ++j) {{")
                w("      const int64_t col = colj[j];")
                w("      const int valid = FULL ? 4 : validj[j];")
            elif block_mode:
                w("    for (int64_t ch = threadIdx.x; ch < n_chunks; ch += blockDim.x) {")
                w("      const int64_t col = ch << 2;")
                w("      const int64_t left = C - col;")
                w("      const int valid = left >= 4 ? 4 : (int)left;")
            else:
                w("    {")
            used_v = sorted({r for i in body for r in (i[1], i[2], i[3], i[4])
                             if r < isa.NVEC and i[0] not in (isa.STG,)} |
                            {i[2] for i in body if i[0] in (isa.STG, isa.ACC) and i[2] < isa.NVEC})
            if used_v:
                w(ind + "float4 " + ", ".join(f"v{r}" for r in used_v) + ";")
            for bop, bd, bx, by, bz, _ in body:
                if bop == isa.LDG:
                    o = ops[bx]
                    if resident:
                        w(ind + f"v{bd} = r{bx}[j];")
                    elif block_mode and o.stage_slot >= 0:
                        w(ind + f"v{bd} = *(const float4*)(rp_stage_lds + {o.stage_slot} * c_pad + col);")
                    elif stage16 is not None and bx == stage16:
                        w(ind + f"v{bd} = rp_staged16((const uint2*)rp_stage_lds, col, {o.dtype.abi});")
                    else:
                        w(ind + f"v{bd} = rp_load4(o{bx}, off{bx}, col, valid);")
                elif bop == isa.STG:
                    if resident:
                        od = ops[bd]
                        if od.dtype.abi == 0 and od.vec_ok and od.col_stride == 1:
                            w(ind + f"if (FULL && STREAM) rp_store4_stream((float*)o{bd}.ptr + off{bd} + col, "
                              f"{_as_vec(bx)}); else")
                        w(ind + f"if (FULL || valid > 0) rp_store4(o{bd}, off{bd}, col, valid, {_as_vec(bx)});")
                    else:
                        w(ind + f"rp_store4(o{bd}, off{bd}, col, valid, {_as_vec(bx)});")
                elif bop == isa.ACC:
                    w(ind + f"acc{bd} = rp_acc4(acc{bd}, {_as_vec(bx)}, {by}, valid);")
                elif bop == isa.COLIDX:
                    w(ind + f"v{bd} = rp_colidx4(col, {'true' if bx else 'false'});")
                else:
                    w(ind + _ew_vec(bop, bd, bx, by, bz, lowp))
            w("    }")
            pc += 1 + aux
            continue
        if op == isa.IMM:
            w(f"    s{dst} = P.imm[{x}];")
        elif op == isa.LDR:
            if x in hoisted:
                w(f"    s{dst} = {hoisted[x]};")
            else:
                w(f"    s{dst} = rp_load1(o{x}.ptr, off{x}, o{x}.dtype);")
        elif op == isa.STR:
            w(f"    if (writer) rp_store1(o{dst}.ptr, off{dst}, o{dst}.dtype, s{x});")
        elif op == isa.LEADIDX:
            w(f"    s{dst} = rp_ibits((int)lead_idx[{x}]);" if y else f"    s{dst} = (float)lead_idx[{x}];")
        elif op == isa.ACCINIT:
            w(f"    acc{dst} = rp_identity({x});")
        elif op == isa.RED:
            # consecutive reductions share one barrier
            group = [(dst, x, y)]
            while (len(group) < 4 and pc + len(group) < len(ins)
                   and ins[pc + len(group)][0] == isa.RED):
                g = ins[pc + len(group)]
                group.append((g[1], g[2], g[3]))
            n = len(group)
            w(f"    {{ float rv[{n}] = {{{', '.join(f'acc{g[1]}' for g in group)}}}; "
              f"const int rk[{n}] = {{{', '.join(str(g[2]) for g in group)}}}; "
              f"rp_block_reduce_n(rv, rk, {n}, red_buf, red_phase); "
              + " ".join(f"s{g[0]} = rv[{q}];" for q, g in enumerate(group)) + " }")
            pc += n
            continue
        else:
            w("    " + _ew_scalar(op, dst, x, y, z, lowp))
        pc += 1
    w("  }")
    w("}")
    return "\n".join(L)


def resident_variants(a: dict) -> list[int]:
    """Chunks-per-lane values for which a register-resident kernel is generated."""
    if not a["has_reduce"]:
        return []
    n_in = max(1, len(full_inputs(a)))
    return [c for c in (1, 2, 4, 8) if c * n_in <= MAX_RESIDENT_REGS]


_PRELUDE = '''// GENERATED by nabla_amd/backend/specialize.py -- do not edit.
// Straight-line versions of the row programs of the benchmark steps; the
// interpreter in rowprog.hip runs everything that is not listed here.
#include "rowprog_device.h"
#include "rowprog_spec.h"

extern __shared__ __align__(16) float rp_stage_lds[];
'''


def collect_programs() -> dict[int, dict]:
    """Plan the five benchmark steps at full size and return {hash: rowprog attrs}."""
    import nabla_amd as nb
    from nabla_amd import config
    from nabla_amd import workloads as W
    from nabla_amd.backend import executor
    from nabla_amd.core.engine import _PLAN_CACHE, clear_plan_cache

    class _PlanOnly:
        """Executor that plans but computes nothing (outputs stay uninitialised)."""

        name = "plan-only"
        torch_device = torch.device("cpu")

        def bind(self, plan: Plan):
            ex = self

            class _B:
                def __init__(self):
                    self.plan = plan

                def run(self, inputs, timer=None):
                    return [torch.empty(s, dtype=d.to_torch()) for _, s, d in plan.outputs]

            return _B()

        def current_stream(self):
            return 0

        def synchronize(self):
            pass

        def check_status(self):
            pass

    def leaves(shapes, dtype):
        if isinstance(shapes, dict):
            return {k: leaves(v, dtype) for k, v in shapes.items()}
        if isinstance(shapes, list):
            return [leaves(v, dtype) for v in shapes]
        return nb.Tensor._from_torch(torch.empty(shapes, dtype=dtype))

    prev = executor.set_executor(_PlanOnly())
    programs: dict[int, dict] = {}
    try:
        f32, bf16, i64 = torch.float32, torch.bfloat16, torch.int64
        jobs = []
        t = leaves(W.c1_shapes(), f32)
        jobs.append(lambda: W.c1_step(t))
        t2 = leaves(W.c2_shapes(), f32)
        jobs.append(lambda: W.c2_step(t2["x"], t2["y"]))
        t3 = leaves(W.c3_shapes(), bf16)
        jobs.append(lambda: W.c3_step(t3))
        s4 = W.c4_shapes()
        t4 = leaves({k: v for k, v in s4.items() if k != "labels"}, f32)
        t4["labels"] = nb.Tensor._from_torch(torch.zeros(s4["labels"], dtype=i64))
        jobs.append(lambda: W.c4_step(t4))
        s5 = W.c5_shapes(layers=2)
        t5 = leaves({k: v for k, v in s5.items() if k != "ids"}, bf16)
        t5["ids"] = nb.Tensor._from_torch(torch.zeros(s5["ids"], dtype=i64))
        jobs.append(lambda: W.c5_step(t5))

        def with_flags(job, **flags):
            """The same step under other evaluation orders (attention out of primitive ops,
            lora_linear as the reference writes it), so that those keep compiled kernels too."""
            def run():
                import contextlib
                with contextlib.ExitStack() as es:
                    for name, value in flags.items():
                        es.enter_context(config.flag(name, value))
                    res = job()
                    # (planned here: a flag of the planner is read when the step is realized)
                    nb.realize_all(*[x for x in nb.tree_leaves(res) if isinstance(x, nb.Tensor)])
                    return res
            return run

        # the loss over a batch too small for its label mask to be recomputed per reader (the
        # planner keeps one mask below 2^22 elements: the same program in another order)
        xs = nb.Tensor._from_torch(torch.empty((64, 32000), dtype=bf16))
        ls = nb.Tensor._from_torch(torch.zeros((64,), dtype=i64))

        def small_batch_loss():
            loss, g = nb.value_and_grad(lambda z: nb.nn.functional.cross_entropy_loss(z, ls))(xs)
            return [loss, g]

        jobs.append(small_batch_loss)
        jobs.append(with_flags(jobs[2], FUSED_ATTENTION=False))
        jobs.append(with_flags(jobs[4], FUSED_ATTENTION=False, LORA_LOW_RANK_ORDER=False))
        jobs.append(with_flags(jobs[4], FOLD_THIN_PAIR=False))
        jobs.append(with_flags(jobs[4], FOLD_PRODUCT_SUMS=False))
        jobs.append(with_flags(jobs[2], FOLD_PRODUCT_SUMS=False))
        jobs.append(with_flags(jobs[0], FOLD_RELU=False))
        jobs.append(with_flags(jobs[3], FOLD_RELU=False))
        for job in jobs:
            clear_plan_cache()
            res = job()
            flat = [x for x in nb.tree_leaves(res) if isinstance(x, nb.Tensor)]
            nb.realize_all(*flat)
            for bound in _PLAN_CACHE.values():
                for st in bound.plan.steps:
                    if st.kind == "rowprog":
                        programs.setdefault(program_hash(st.attrs), st.attrs)
    finally:
        executor.set_executor(prev)
    return programs


def write_sources(programs: dict[int, dict]) -> list[Path]:
    for old in CSRC.glob("rowprog_spec_gen*.hip"):
        old.unlink()
    items = sorted(programs.items())
    files = []
    for fi in range(N_FILES):
        chunk = items[fi::N_FILES]
        src = [_PRELUDE]
        for h, a in chunk:
            src.append(f"// members: {' '.join(a.get('members', []))}")
            src.append(generate_kernel(a, f"rp_spec_{h:016x}"))
            for c in resident_variants(a):
                src.append(generate_kernel(a, f"rp_spec_{h:016x}_c{c}", cpt=c))
            if stage16_operand(a) is not None:
                src.append(generate_kernel(a, f"rp_spec_{h:016x}_s16", stage16=stage16_operand(a)))
            src.append("")
        src.append(f"extern const rp_spec_entry rp_spec_table_{fi}[] = {{")
        for h, a in chunk:
            rv = resident_variants(a)
            flat = not a["has_reduce"]
            ks = [f"(const void*)rp_spec_{h:016x}" + ("<false>" if flat else "")]
            kf = ["nullptr"]
            kst = ["nullptr"]
            for c in (1, 2, 4, 8):
                ks.append(f"(const void*)rp_spec_{h:016x}_c{c}<false, false>" if c in rv else "nullptr")
                kf.append(f"(const void*)rp_spec_{h:016x}_c{c}<true, false>" if c in rv else "nullptr")
                kst.append(f"(const void*)rp_spec_{h:016x}_c{c}<true, true>" if c in rv else "nullptr")
            kflat = f"(const void*)rp_spec_{h:016x}<true>" if flat else "nullptr"
            k16 = f"(const void*)rp_spec_{h:016x}_s16" if stage16_operand(a) is not None else "nullptr"
            src.append(f"  {{0x{h:016x}ULL, {{{', '.join(ks)}}}, {{{', '.join(kf)}}}, "
                       f"{{{', '.join(kst)}}}, {kflat}, {k16}, {1 if a['has_reduce'] else 0}}},")
        src.append("  {0ULL, {nullptr, nullptr, nullptr, nullptr, nullptr}, "
                   "{nullptr, nullptr, nullptr, nullptr, nullptr}, "
                   "{nullptr, nullptr, nullptr, nullptr, nullptr}, nullptr, nullptr, 0}};")
        src.append(f"extern const int rp_spec_count_{fi} = {len(chunk)};")
        path = CSRC / f"rowprog_spec_gen{fi}.hip"
        path.write_text("\n".join(src) + "\n")
        files.append(path)
    return files


def main() -> None:
    programs = collect_programs()
    files = write_sources(programs)
    n_block = sum(1 for a in programs.values() if a["has_reduce"])
    print(f"specialised {len(programs)} row programs ({n_block} with reductions) into "
          f"{len(files)} files")


if __name__ == "__main__":
    main()
