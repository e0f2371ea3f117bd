"""The C-ABI library: it loads, exports every symbol that include/nbk.h declares,
and the ctypes mirrors of its structs have the layout the C compiler gives them.
No compute calls are made here (no GPU needed)."""
import ctypes as C
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "nbk.h"


def test_library_loads_and_exports_every_declared_symbol():
    from nabla_amd.backend import lib

    L = lib.load()
    hdr = HEADER.read_text()
    declared = set(re.findall(r"^\s*(?:int|int64_t|uint64_t|const char\*)\s+(nbk_[a-z0-9_]+)\s*\(", hdr, re.M))
    assert len(declared) >= 20
    for name in sorted(declared):
        assert hasattr(L, name), f"{name} is declared in nbk.h but not exported"
        assert name in lib.EXPORTS, f"{name} has no ctypes signature in lib.py"
    assert L.nbk_abi_version() == lib.ABI_VERSION
    m = re.search(r"#define NBK_ABI_VERSION (\d+)", hdr)
    assert int(m.group(1)) == lib.ABI_VERSION


def test_isa_numbers_match_header():
    from nabla_amd.backend import isa

    hdr = HEADER.read_text()
    enum = dict((k, int(v)) for k, v in re.findall(r"NBK_OP_([A-Z0-9]+)\s*=\s*(\d+)", hdr))
    for name, code in isa.STRUCT_NAMES.items():
        assert enum[name] == code, name
    for name, code in isa.EW.items():
        assert enum[name.upper()] == code, name
    lim = dict((k, int(v)) for k, v in re.findall(r"#define NBK_RP_([A-Z_]+) (\d+)", hdr))
    assert lim["MAX_OPERANDS"] == isa.MAX_OPERANDS and lim["MAX_INS"] == isa.MAX_INS
    assert lim["MAX_IMM"] == isa.MAX_IMM and lim["MAX_LEAD"] == isa.MAX_LEAD
    assert lim["NVEC"] == isa.NVEC and lim["NSCL"] == isa.NSCL and lim["NACC"] == isa.NACC


#: every struct of the header and its ctypes mirror
STRUCTS = {
    "nbk_operand": "Operand", "nbk_ins": "Ins", "nbk_rowprog": "RowProg", "nbk_gemm_desc": "GemmDesc",
    "nbk_gemm_nf4_desc": "GemmNf4Desc", "nbk_conv_desc": "ConvDesc", "nbk_pool_desc": "PoolDesc",
    "nbk_attn_desc": "AttnDesc", "nbk_attn_tensor": "AttnTensor", "nbk_reduce_task": "ReduceTask",
    "nbk_opt_tensor": "OptTensor", "nbk_adamw_desc": "AdamwDesc", "nbk_sgd_desc": "SgdDesc",
    "nbk_tensor": "TensorDesc", "nbk_gemm_term": "GemmTerm",
}


def test_struct_layouts_match_the_c_compiler(tmp_path):
    """Size of every struct and offset of every field, as gcc lays the header out, against the
    ctypes mirrors (a field named ``in`` in C is ``in_`` in Python)."""
    from nabla_amd.backend import lib

    hdr = HEADER.read_text()
    declared = set(re.findall(r"typedef struct (nbk_[a-z0-9_]+) \{", hdr))
    assert declared == set(STRUCTS), declared ^ set(STRUCTS)
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "nbk.h"', "int main(void) {"]
    for cname, pyname in STRUCTS.items():
        cls = getattr(lib, pyname)
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        for field, _ in cls._fields_:
            cfield = field[:-1] if field.endswith("_") else field
            lines.append(f'  printf("{cname}.{field} %zu\\n", offsetof({cname}, {cfield}));')
    lines += ["  return 0;", "}"]
    src = tmp_path / "sizes.c"
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", f"-I{ROOT / 'include'}", str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout
    got = dict((k, int(v)) for k, v in (line.split() for line in out.splitlines()))
    for cname, pyname in STRUCTS.items():
        cls = getattr(lib, pyname)
        assert got[cname] == C.sizeof(cls), (cname, got[cname], C.sizeof(cls))
        for field, _ in cls._fields_:
            assert got[f"{cname}.{field}"] == getattr(cls, field).offset, (cname, field)


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from nabla_amd.backend import lib

    monkeypatch.setattr(lib, "_lib", None)
    with pytest.raises(lib.NbkError, match="missing"):
        lib.load(tmp_path / "libnbk.so")


def test_no_gpu_means_no_executor():
    """Without a GPU the package must refuse to compute rather than fall back."""
    import torch
    from nabla_amd.backend import executor

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    prev = executor.set_executor(None)
    try:
        with pytest.raises(RuntimeError, match="no CPU execution path"):
            executor.get_executor()
    finally:
        executor.set_executor(prev)


def test_specialised_program_hash_matches_between_python_and_c(emulator):
    """The generator's hash and the library's hash must agree, or specialised
    kernels would silently never be used."""
    import numpy as np
    import nabla_amd as nb
    from nabla_amd.backend import lib, specialize
    from nabla_amd.backend.executor import BoundPlan
    from nabla_amd.core.engine import _PLAN_CACHE

    x = nb.Tensor.constant(np.ones((64, 8192), np.float32))
    y = nb.Tensor.constant(np.ones((64, 8192), np.float32))
    out, gx = nb.workloads.c2_step(x, y)
    nb.realize_all(out, gx)
    plan = list(_PLAN_CACHE.values())[-1].plan
    L = lib.load()

    class _FakeEx:
        lib = L
        torch_device = None

    progs = [s for s in plan.steps if s.kind == "rowprog"]
    assert progs
    for st in progs:
        assert L.nbk_rowprog_is_specialized(C.byref(_program_record(st.attrs))) == 1, \
            f"hash {specialize.program_hash(st.attrs):016x} not found in the library's table"


def test_generated_kernels_cover_every_row_program_of_the_benchmark_steps():
    """The five benchmark steps (and the other evaluation orders the generator plans) are planned
    as the generator plans them, and every row program that comes out must have its
    ahead-of-time kernel in the library: a planner change that alters a program without
    `python -m nabla_amd.backend.specialize` being run again would leave that program to the
    interpreter (correct, and ten times slower on the decoder's layer-norm backward)."""
    from nabla_amd.backend import lib, specialize
    programs = specialize.collect_programs()
    assert len(programs) >= 30
    L = lib.load()
    missing = [f"{h:016x} ({' '.join(a.get('members', []))[:60]})" for h, a in programs.items()
               if L.nbk_rowprog_is_specialized(C.byref(_program_record(a))) < 1]
    assert not missing, "row programs without a specialised kernel: " + "; ".join(missing)


def test_the_committed_traffic_counters_belong_to_the_kernel_the_stress_step_runs():
    """`bench.py` reports the HBM traffic of the stress step from `profiles/hbm_traffic_c2.json`,
    which names the kernel (by program hash) whose counters it holds.  A planner or op change
    that alters that row program must come with new counter runs, or the bench line would
    silently lose the figure."""
    import json
    from nabla_amd.backend import specialize
    with open(ROOT / "profiles" / "hbm_traffic_c2.json") as f:
        named = json.load(f)["kernel"]
    hashes = [f"{h:016x}" for h in specialize.collect_programs()]
    assert any(h in named for h in hashes), f"{named} is not a row program of the benchmark steps"


def _program_record(a):
    """The ctypes record of a planned row program, built as the executor builds it (operands at
    an aligned dummy address: nothing is launched)."""
    from nabla_amd.backend import lib
    rp = lib.RowProg()
    rp.n_lead = len(a["lead"])
    for i, d in enumerate(a["lead"]):
        rp.lead_dim[i] = d
    rp.C, rp.n_operands, rp.n_ins, rp.n_imm = a["C"], len(a["operands"]), len(a["ins"]), len(a["imm"])
    rp.has_reduce, rp.block, rp.n_stage = int(a["has_reduce"]), a["block"], a["n_stage"]
    for i, v in enumerate(a["imm"]):
        rp.imm[i] = v
    for i, o in enumerate(a["operands"]):
        od = rp.operand[i]
        od.ptr = 4096
        od.col_stride, od.dtype, od.vec_ok, od.stage_slot = o.col_stride, o.dtype.abi, int(o.vec_ok), o.stage_slot
        for j, s_ in enumerate(o.lead_strides):
            od.lead_stride[j] = s_
    for i, ins in enumerate(a["ins"]):
        d = rp.ins[i]
        d.op, d.dst, d.a, d.b, d.c, d.aux = ins
    return rp


def test_the_loss_program_over_long_bf16_rows_has_its_hand_scheduled_kernel(emulator, monkeypatch):
    """The hand-scheduled cross-entropy kernel is attached to its row program by the program's
    hash: if the planner ever emits that program differently, the library would quietly fall
    back to the generated kernel.  Planned here as the decoder plans it (bf16 logits in memory,
    int64 labels, mean over the rows) and asked of the library, without a launch."""
    import numpy as np
    import torch
    import nabla_amd as nb
    from nabla_amd.backend import lib
    from nabla_amd.core.engine import _PLAN_CACHE, clear_plan_cache
    monkeypatch.delenv("NBK_ROWPROG_HAND", raising=False)
    clear_plan_cache()
    rows, vocab = 8, 32000
    x = nb.Tensor.from_dlpack(torch.zeros(rows, vocab, dtype=torch.bfloat16))
    lab = nb.Tensor.constant(np.zeros((rows,), np.int64))
    loss, g = nb.value_and_grad(lambda z: nb.nn.functional.cross_entropy_loss(z, lab))(x)
    nb.realize_all(loss, g)
    plan = list(_PLAN_CACHE.values())[-1].plan
    long_rows = [s for s in plan.steps if s.kind == "rowprog" and s.attrs["C"] == vocab]
    assert len(long_rows) == 1, "loss and gradient are one row program"
    L = lib.load()
    rp = _program_record(long_rows[0].attrs)
    assert L.nbk_rowprog_is_specialized(C.byref(rp)) == 2
    rp.C = vocab + 4      # not whole 16-byte pieces: the generated kernels take it
    assert L.nbk_rowprog_is_specialized(C.byref(rp)) == 1
    clear_plan_cache()
