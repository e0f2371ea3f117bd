"""Plan execution on the GPU through libnbk.so.

``HipExecutor`` is the product path: it binds the plan's buffers to device
addresses (inputs and outputs are torch allocations used as plain memory,
intermediates live in one arena per plan) and issues every step as a call
into the C ABI of include/nbk.h on the current HIP stream.  It refuses to
work without the built library and a gfx950 device -- there is no CPU path
in this package.  The executor is replaceable (``set_executor``) only so that
host-side logic can be unit-tested against a reference interpreter of the
same launch records.
"""
from __future__ import annotations

import ctypes as C
import math
import os
from typing import Any, Sequence

import torch

from ..core.dtype import DType
from . import ir, isa, lib
from .planner import Plan, Step, ViewRef

_RED = {"sum": 0, "max": 1, "min": 2}


class BoundPlan:
    """A plan with its ctypes launch records prepared once.

    Only the addresses of plan inputs and outputs change from run to run; they
    are patched into the prepared records before launch."""

    def __init__(self, plan: Plan, ex: "HipExecutor"):
        self.plan = plan
        self.ex = ex
        self.arena = None
        if plan.arena_bytes > 0:
            self.arena = torch.empty(plan.arena_bytes, dtype=torch.uint8, device=ex.torch_device)
        self.base: list[int] = [0] * len(plan.bufs)
        if self.arena is not None:
            a0 = self.arena.data_ptr()
            for b in plan.bufs:
                if b.role == "temp" and b.offset >= 0:
                    self.base[b.id] = a0 + b.offset
        self.dynamic = [b.id for b in plan.bufs if b.role in ("input", "output")]
        self.calls: list[tuple] = []  # (fn, args tuple, patch list)
        self.has_gather = any(st.kind in ("gather", "scatter") for st in plan.steps)
        self._graphs: dict = {}  # pointer tuple -> recorded launch sequence (at most eight)
        self._seen: set = set()  # pointer tuples that have run once already
        self._graph_off = any(st.kind == "custom" for st in plan.steps)  # user kernels may not be capturable
        self._layout_outputs()
        self._prepare()

    # -- address helpers -------------------------------------------------------
    def _addr(self, ref: ViewRef) -> int:
        return self.base[ref.buf] + ref.offset * ref.dtype.size_in_bytes

    def _prepare(self) -> None:
        L = self.ex.lib
        plan = self.plan
        dyn = set(self.dynamic)
        for st in plan.steps:
            a = st.attrs
            k = st.kind
            patches: list = []  # (setter(addr_of_buf)) closures

            def ptr_field(obj, field, buf: int, byte_off: int):
                """Set obj.field = base[buf] + byte_off now, and again per run if dynamic."""
                setattr(obj, field, self.base[buf] + byte_off)
                if buf in dyn:
                    patches.append((obj, field, buf, byte_off))

            if k == "rowprog":
                rp = lib.RowProg()
                lead = a["lead"]
                rp.n_lead = len(lead)
                for i, d in enumerate(lead):
                    rp.lead_dim[i] = d
                rp.C = a["C"]
                rp.n_operands = len(a["operands"])
                rp.n_ins = len(a["ins"])
                rp.n_imm = len(a["imm"])
                rp.has_reduce = 1 if a["has_reduce"] else 0
                rp.block = a["block"]
                rp.n_stage = a["n_stage"]
                rp.reserved = 1 if self.ex.force_interpreter else 0
                imm_bits = C.cast(rp.imm, C.POINTER(C.c_int32))
                for i, v in enumerate(a["imm"]):
                    if isinstance(v, int):  # an integer register's immediate: its bit pattern
                        imm_bits[i] = v
                    else:
                        rp.imm[i] = v
                for i, o in enumerate(a["operands"]):
                    od = rp.operand[i]
                    for j, s in enumerate(o.lead_strides):
                        od.lead_stride[j] = s
                    od.col_stride = o.col_stride
                    od.dtype = o.dtype.abi
                    od.vec_ok = 1 if o.vec_ok else 0
                    od.stage_slot = o.stage_slot
                    ptr_field(od, "ptr", o.buf, o.offset * o.dtype.size_in_bytes)
                for i, ins in enumerate(a["ins"]):
                    d = rp.ins[i]
                    d.op, d.dst, d.a, d.b, d.c, d.aux = ins[0], ins[1], ins[2], ins[3], ins[4], ins[5]
                self.calls.append((L.nbk_rowprog_launch, [C.byref(rp)], patches, rp))
            elif k == "copy":
                src, dst = a["src"], a["dst"]
                rank = len(src.shape)
                shape = (C.c_int64 * max(rank, 1))(*src.shape)
                ss = (C.c_int64 * max(rank, 1))(*src.strides)
                ds = (C.c_int64 * max(rank, 1))(*dst.strides)
                holder = _Ptrs(2)
                ptr_field(holder, "p0", src.buf, src.offset * src.dtype.size_in_bytes)
                ptr_field(holder, "p1", dst.buf, dst.offset * dst.dtype.size_in_bytes)
                self.calls.append((L.nbk_copy_strided,
                                   [holder, ("p0", "p1"), src.dtype.abi, dst.dtype.abi, rank, shape,
                                    ss, ds], patches, None))
            elif k == "fill":
                holder = _Ptrs(1)
                ptr_field(holder, "p0", a["buf"], 0)
                self.calls.append((L.nbk_fill, [holder, ("p0",), a["dtype"].abi, a["numel"],
                                                float(a["value"])], patches, None))
            elif k == "reduce_mid":
                src, dst = a["src"], a["dst"]
                holder = _Ptrs(2)
                ptr_field(holder, "p0", src.buf, src.offset * src.dtype.size_in_bytes)
                ptr_field(holder, "p1", dst.buf, dst.offset * dst.dtype.size_in_bytes)
                self.calls.append((L.nbk_reduce_mid,
                                   [holder, ("p0", "p1"), src.dtype.abi, dst.dtype.abi, a["outer"],
                                    a["red"], a["inner"], _RED[a["fn"]]], patches, None))
            elif k == "reduce_batch":
                tasks = (lib.ReduceTask * len(a["tasks"]))()
                for t, ta in zip(tasks, a["tasks"]):
                    src, dst = ta["src"], ta["dst"]
                    ptr_field(t, "in_", src.buf, src.offset * src.dtype.size_in_bytes)
                    ptr_field(t, "out", dst.buf, dst.offset * dst.dtype.size_in_bytes)
                    t.outer, t.red, t.inner = ta["outer"], ta["red"], ta["inner"]
                    t.dtype_in, t.dtype_out, t.kind = src.dtype.abi, dst.dtype.abi, _RED[ta["fn"]]
                self.calls.append((L.nbk_reduce_mid_batch, [tasks, len(a["tasks"])], patches, tasks))
            elif k == "gemm":
                d = lib.GemmDesc()
                ra, rb, rc = a["a"], a["b"], a["dst"]
                ptr_field(d, "A", ra.buf, ra.offset * ra.dtype.size_in_bytes)
                ptr_field(d, "B", rb.buf, rb.offset * rb.dtype.size_in_bytes)
                ptr_field(d, "C", rc.buf, rc.offset * rc.dtype.size_in_bytes)
                d.bias = None
                d.residual = None
                if a.get("bias") is not None:
                    rbias = a["bias"]
                    if rbias.dtype is not rc.dtype:
                        raise TypeError(f"matmul bias is {rbias.dtype}, the result {rc.dtype}")
                    ptr_field(d, "bias", rbias.buf, rbias.offset * rbias.dtype.size_in_bytes)
                d.residual_op = 0
                if a.get("residual") is not None:
                    rres = a["residual"]
                    if rres.dtype is not rc.dtype:
                        raise TypeError(f"matmul residual is {rres.dtype}, the result {rc.dtype}")
                    ptr_field(d, "residual", rres.buf, rres.offset * rres.dtype.size_in_bytes)
                    d.residual_op = 1 if a["res_op"] == "mul" else 0
                d.M, d.N, d.K = a["M"], a["N"], a["K"]
                d.a_rs, d.a_cs, d.b_rs, d.b_cs = a["a_rs"], a["a_cs"], a["b_rs"], a["b_cs"]
                d.ldc = a["ldc"]
                d.batch, d.a_bs, d.b_bs, d.c_bs = a["batch"], a["a_bs"], a["b_bs"], a["c_bs"]
                d.batch_inner = a.get("batch_inner", 1)
                d.a_bs2, d.b_bs2, d.c_bs2 = a.get("a_bs2", 0), a.get("b_bs2", 0), a.get("c_bs2", 0)
                if ra.dtype is not rb.dtype:
                    raise TypeError(f"matmul operands differ in dtype: {ra.dtype} vs {rb.dtype}")
                d.dtype_ab = ra.dtype.abi
                d.dtype_c = rc.dtype.abi
                d.act = {None: 0, "relu": 1, "gelu": 2}[a.get("act")]
                d.C_aux, d.aux_op = None, 0
                if a.get("aux_dst") is not None:
                    raux = a["aux_dst"]
                    if raux.dtype is not rc.dtype:
                        raise TypeError(f"matmul second result is {raux.dtype}, the first {rc.dtype}")
                    ptr_field(d, "C_aux", raux.buf, raux.offset * raux.dtype.size_in_bytes)
                    d.aux_op = 1
                d.batch_reduce = 0
                d.alpha = a.get("alpha", 1.0)
                d.colsum = None
                if a.get("colsum") is not None:
                    rcs = a["colsum"]
                    if rcs.dtype is not rc.dtype:
                        raise TypeError(f"matmul column sums are {rcs.dtype}, the product {rc.dtype}")
                    ptr_field(d, "colsum", rcs.buf, rcs.offset * rcs.dtype.size_in_bytes)
                d.n_terms = 0
                for ti, term in enumerate(a.get("terms") or ()):
                    ta, tb = term["a"], term["b"]
                    if ta.dtype is not ra.dtype or tb.dtype is not ra.dtype:
                        raise TypeError(f"matmul term {ti} is {ta.dtype} / {tb.dtype}, the first pair {ra.dtype}")
                    t = d.term[ti]
                    ptr_field(t, "A", ta.buf, ta.offset * ta.dtype.size_in_bytes)
                    ptr_field(t, "B", tb.buf, tb.offset * tb.dtype.size_in_bytes)
                    t.K = term["K"]
                    t.a_rs, t.a_cs, t.b_rs, t.b_cs = term["a_rs"], term["a_cs"], term["b_rs"], term["b_cs"]
                    d.n_terms = ti + 1
                self.calls.append((L.nbk_gemm, [C.byref(d)], patches, d))
            elif k == "gemm_nf4":
                d = lib.GemmNf4Desc()
                rx, rcodes, rsc, rc = a["x"], a["codes"], a["scales"], a["dst"]
                if rcodes.dtype is not DType.uint8 or rsc.dtype is not DType.float32:
                    raise TypeError(f"matmul_nf4 wants uint8 codes and float32 scales, got {rcodes.dtype}, {rsc.dtype}")
                if rx.dtype is not rc.dtype or rx.dtype not in (DType.bfloat16, DType.float32):
                    raise TypeError(f"matmul_nf4 computes in bfloat16 or float32, got {rx.dtype} -> {rc.dtype}")
                ptr_field(d, "A", rx.buf, rx.offset * rx.dtype.size_in_bytes)
                ptr_field(d, "codes", rcodes.buf, rcodes.offset)
                ptr_field(d, "scales", rsc.buf, rsc.offset * 4)
                ptr_field(d, "C", rc.buf, rc.offset * rc.dtype.size_in_bytes)
                d.M = a["M"]
                d.w_rows, d.w_cols = a["w_shape"]
                d.lda, d.ldc = a["K"], a["N"]
                d.block = a["block"]
                d.transpose_w = 1 if a["transpose"] else 0
                d.dtype = rx.dtype.abi
                d.alpha = 1.0
                self.calls.append((L.nbk_gemm_nf4, [C.byref(d)], patches, d))
            elif k in ("conv2d", "conv2d_dgrad", "conv2d_wgrad"):
                d = lib.ConvDesc()
                xs, ws, ys = a["x_shape"], a["w_shape"], a["y_shape"]
                d.N, d.H, d.W, d.Cin = xs
                d.R, d.S, _, d.Cout = ws
                d.Ho, d.Wo = ys[1], ys[2]
                d.stride_h, d.stride_w = a["stride"]
                d.pad_t, d.pad_b, d.pad_l, d.pad_r = a["padding"]
                d.dtype = a["dst"].dtype.abi
                d.act = {None: 0, "relu": 1}[a.get("act")]
                n_ptr = 4 if k == "conv2d" else 3
                holder = _Ptrs(4)
                refs = list(a["ins"])
                if k == "conv2d" and not a["has_bias"]:
                    refs.append(None)
                refs.append(a["dst"])
                extra = []
                if k == "conv2d_wgrad":
                    ws = a.get("workspace")
                    refs.append(ws)
                    extra = [C.c_int64(a.get("workspace_bytes", 0) if ws is not None else 0)]
                    n_ptr = 4
                names = []
                for i, r in enumerate(refs):
                    nm = f"p{i}"
                    names.append(nm)
                    if r is None:
                        setattr(holder, nm, None)
                    else:
                        ptr_field(holder, nm, r.buf, r.offset * r.dtype.size_in_bytes)
                fn = {"conv2d": L.nbk_conv2d_fwd, "conv2d_dgrad": L.nbk_conv2d_dgrad,
                      "conv2d_wgrad": L.nbk_conv2d_wgrad}[k]
                self.calls.append((fn, [C.byref(d), holder, tuple(names[:n_ptr]), *extra], patches, d))
            elif k in ("maxpool2d", "maxpool2d_bwd", "avgpool2d", "avgpool2d_bwd"):
                d = lib.PoolDesc()
                xs, ys = a["x_shape"], a["y_shape"]
                d.N, d.H, d.W, d.C = xs
                d.Ho, d.Wo = ys[1], ys[2]
                d.kh, d.kw = a["kernel"]
                d.stride_h, d.stride_w = a["stride"]
                d.pad_t, d.pad_l = a["padding"][0], a["padding"][2]
                d.dtype = a["dst"].dtype.abi
                refs = list(a["ins"]) + [a["dst"]]
                holder = _Ptrs(4)
                names = []
                for i, r in enumerate(refs):
                    nm = f"p{i}"
                    names.append(nm)
                    ptr_field(holder, nm, r.buf, r.offset * r.dtype.size_in_bytes)
                fn = {"maxpool2d": L.nbk_maxpool2d_fwd, "maxpool2d_bwd": L.nbk_maxpool2d_bwd,
                      "avgpool2d": L.nbk_avgpool2d_fwd, "avgpool2d_bwd": L.nbk_avgpool2d_bwd}[k]
                self.calls.append((fn, [C.byref(d), holder, tuple(names)], patches, d))
            elif k in ("attention", "attention_bwd"):
                d = lib.AttnDesc()
                d.B, d.H, d.S, d.hd = a["B"], a["H"], a["S"], a["hd"]
                d.scale = a["scale"]
                d.causal = 1 if a["causal"] else 0
                d.dtype = a["q"].dtype.abi
                keep_alive = [d]

                def heads(ref):
                    """[B, H, S, hd] view -> (batch, sequence, head) strides."""
                    t = lib.AttnTensor()
                    sb, sh, ss, _ = ref.strides
                    t.sb, t.ss, t.sh = sb, ss, (sh if ref.shape[1] > 1 else a["hd"])
                    if ref.shape[0] == 1:
                        t.sb = 0
                    ptr_field(t, "ptr", ref.buf, ref.offset * ref.dtype.size_in_bytes)
                    keep_alive.append(t)
                    return C.byref(t)

                holder = _Ptrs(2)
                ptr_field(holder, "p0", a["lse"].buf, a["lse"].offset * 4)
                o_lo = heads(a["o_lo"]) if a.get("o_lo") is not None else None
                if k == "attention":
                    args = [_LATE, C.byref(d), heads(a["q"]), heads(a["k"]), heads(a["v"]), heads(a["o"]),
                            o_lo, _Late(holder, "p0")]
                    self.calls.append((L.nbk_attention_fwd, args, patches, keep_alive))
                else:
                    ws = a["workspace"]
                    ptr_field(holder, "p1", ws.buf, ws.offset * 4)
                    args = [_LATE, C.byref(d), heads(a["q"]), heads(a["k"]), heads(a["v"]), heads(a["o"]),
                            o_lo, _Late(holder, "p0"), heads(a["dout"]), heads(a["dq"]), heads(a["dk"]),
                            heads(a["dv"]), _Late(holder, "p1"), C.c_int64(a["workspace_bytes"])]
                    self.calls.append((L.nbk_attention_bwd, args, patches, keep_alive))
            elif k == "gather":
                t, ix, dst = a["table"], a["idx"], a["dst"]
                holder = _Ptrs(3)
                ptr_field(holder, "p0", t.buf, t.offset * t.dtype.size_in_bytes)
                ptr_field(holder, "p1", ix.buf, ix.offset * ix.dtype.size_in_bytes)
                ptr_field(holder, "p2", dst.buf, dst.offset * dst.dtype.size_in_bytes)
                self.calls.append((L.nbk_gather,
                                   [holder, ("p0", "p1", "p2"), t.dtype.abi, ix.dtype.abi, a["outer"],
                                    a["axis_len"], a["n_idx"], a["inner"],
                                    C.c_void_p(self.ex.status_flag.data_ptr())], patches, None))
            elif k == "scatter":
                ix, up, dst, wn = a["idx"], a["upd"], a["dst"], a["winner"]
                holder = _Ptrs(4)
                ptr_field(holder, "p0", ix.buf, ix.offset * ix.dtype.size_in_bytes)
                ptr_field(holder, "p1", up.buf, up.offset * up.dtype.size_in_bytes)
                ptr_field(holder, "p2", dst.buf, dst.offset * dst.dtype.size_in_bytes)
                ptr_field(holder, "p3", wn.buf, wn.offset * 4)
                self.calls.append((L.nbk_scatter,
                                   [_LATE, _Late(holder, "p0"), _Late(holder, "p1"), _Late(holder, "p2"),
                                    dst.dtype.abi, ix.dtype.abi, a["outer"], a["axis_len"], a["n_idx"],
                                    a["inner"], _Late(holder, "p3"),
                                    C.c_void_p(self.ex.status_flag.data_ptr())], patches, None))
            elif k == "argreduce":
                src, dst = a["src"], a["dst"]
                holder = _Ptrs(2)
                ptr_field(holder, "p0", src.buf, src.offset * src.dtype.size_in_bytes)
                ptr_field(holder, "p1", dst.buf, dst.offset * dst.dtype.size_in_bytes)
                self.calls.append((L.nbk_argmax_rows,
                                   [holder, ("p0", "p1"), src.dtype.abi, a["rows"], a["C"],
                                    1 if a["fn"] == "min" else 0], patches, None))
            elif k == "random":
                dst = a["dst"]
                holder = _Ptrs(1)
                ptr_field(holder, "p0", dst.buf, dst.offset * dst.dtype.size_in_bytes)
                self.calls.append((L.nbk_random,
                                   [holder, ("p0",), dst.dtype.abi, a["numel"],
                                    ir.RANDOM_MODES.index(a["mode"]), C.c_float(a["a"]), C.c_float(a["b"]),
                                    C.c_void_p(self.ex.rng_state.data_ptr()), C.c_uint32(a["stream"])],
                                   patches, None))
            elif k == "rng_advance":
                self.calls.append((L.nbk_rng_advance, [C.c_void_p(self.ex.rng_state.data_ptr())],
                                   patches, None))
            elif k in ("adamw_multi", "sgd_multi"):
                entries = a["entries"]
                table = (lib.OptTensor * len(entries))()
                in_fields = ("param", "grad", "m", "v")
                out_fields = ("param_out", "m_out", "v_out")
                for t, e in zip(table, entries):
                    for name, r in zip(in_fields, e["ins"]):
                        ptr_field(t, name, r.buf, r.offset * r.dtype.size_in_bytes)
                    for name, r in zip(out_fields, e["outs"]):
                        ptr_field(t, name, r.buf, r.offset * r.dtype.size_in_bytes)
                    t.numel = e["numel"]
                if k == "adamw_multi":
                    d = lib.AdamwDesc()
                    d.lr, d.beta1, d.beta2, d.eps = a["lr"], a["beta1"], a["beta2"], a["eps"]
                    d.weight_decay = a["weight_decay"]
                    d.bias_correction = 1 if a["bias_correction"] else 0
                    d.log_beta1 = math.log(a["beta1"]) if a["beta1"] > 0.0 else -math.inf
                    d.log_beta2 = math.log(a["beta2"]) if a["beta2"] > 0.0 else -math.inf
                    d.c1 = d.c2 = 1.0
                    d.step = None
                    if a["step"] is not None:
                        d.c1 = 1.0 - a["beta1"] ** a["step"]
                        d.c2 = 1.0 - a["beta2"] ** a["step"]
                    else:
                        r = a["step_ref"]
                        ptr_field(d, "step", r.buf, r.offset * 4)
                    fn = L.nbk_adamw_multi
                else:
                    d = lib.SgdDesc()
                    d.lr, d.momentum, d.weight_decay = a["lr"], a["momentum"], a["weight_decay"]
                    fn = L.nbk_sgd_multi
                d.dtype = a["dtype"].abi
                self.calls.append((fn, [C.byref(d), table, len(entries)], patches, (d, table)))
            elif k == "ew64":
                refs = a["operands"]
                ins = (lib.TensorDesc * len(refs))()
                imm = (C.c_int64 * len(refs))()
                out = lib.TensorDesc()
                dst = a["dst"]
                for t, r in list(zip(ins, refs)) + [(out, dst)]:
                    if isinstance(r, int):
                        continue  # (ptr stays NULL: the operand is the immediate)
                    t.dtype = r.dtype.abi
                    t.rank = len(r.shape)
                    for j, (d_, s_) in enumerate(zip(r.shape, r.strides)):
                        t.shape[j] = d_
                        t.stride[j] = s_
                    ptr_field(t, "ptr", r.buf, r.offset * r.dtype.size_in_bytes)
                for i, r in enumerate(refs):
                    if isinstance(r, int):
                        imm[i] = r
                        ins[i].rank = len(dst.shape)
                self.calls.append((L.nbk_ew_int64,
                                   [C.c_int32(isa.EW[a["fn"]]), ins, imm, len(refs), C.byref(out)],
                                   patches, (ins, imm, out)))
            elif k == "custom":
                ins = (lib.TensorDesc * max(len(a["ins"]), 1))()
                outs = (lib.TensorDesc * len(a["dsts"]))()
                for arr, refs in ((ins, a["ins"]), (outs, a["dsts"])):
                    for i, r in enumerate(refs):
                        t = arr[i]
                        t.dtype = r.dtype.abi
                        t.rank = len(r.shape)
                        for j, (d_, s_) in enumerate(zip(r.shape, r.strides)):
                            t.shape[j] = d_
                            t.stride[j] = s_
                        ptr_field(t, "ptr", r.buf, r.offset * r.dtype.size_in_bytes)
                self.calls.append((L.nbk_custom,
                                   [a["library"].encode(), a["name"].encode(), ins, len(a["ins"]),
                                    outs, len(a["dsts"])], patches, (ins, outs)))
            else:
                raise NotImplementedError(f"executor: unknown step kind '{k}'")

    def run(self, inputs: Sequence[torch.Tensor], timer=None) -> list[torch.Tensor]:
        """Launch every step on the current stream.  ``timer(step_index, kind)``,
        if given, is called before each launch and may return a callable to be
        invoked right after it (used to bracket kernels with HIP events)."""
        plan = self.plan
        ex = self.ex
        if len(inputs) != plan.n_inputs:
            raise ValueError(f"plan expects {plan.n_inputs} inputs, got {len(inputs)}")
        if timer is None:
            timer = ex.launch_timer
        keep = []
        large, small, small_dst = self._take_slabs()
        out_by_buf = {}
        for bid, (is_small, off, nbytes, shape, dtype) in self._out_layout.items():
            piece = (small if is_small else large)[off:off + nbytes]
            out_by_buf[bid] = piece.view(dtype.to_torch()).reshape(shape)
        outs: list[torch.Tensor] = [out_by_buf[bid] for bid, _, _ in plan.outputs]
        for b in plan.bufs:
            if b.role == "input":
                t = inputs[b.index]
                if t.device != ex.torch_device:
                    raise ValueError(f"input {b.index} lives on {t.device}, expected {ex.torch_device}")
                if not t.is_contiguous() or (t.data_ptr() % 16) != 0:
                    t = t.contiguous().clone()
                    keep.append(t)
                self.base[b.id] = t.data_ptr()
            elif b.role == "output":
                self.base[b.id] = out_by_buf[b.id].data_ptr()
        stream = C.c_void_p(ex.current_stream())
        base = self.base
        check = lib.check
        # Replay as a HIP graph: a step that runs again on the very buffers of an earlier
        # run (inputs unchanged, outputs in a slab of this plan that has come free again) is
        # recorded once and from then on costs one launch call instead of one per kernel.
        if ex.use_graphs and timer is None and not keep and len(self.calls) > 1 and not self._graph_off:
            key = tuple(base[b] for b in self.dynamic)
            g = self._graphs.get(key)
            if g is None and key in self._seen and len(self._graphs) < 8:
                g = self._record(key)
            if g is not None:
                check(ex.lib.nbk_graph_launch(g, stream))
                ex.graph_replays += 1
                if self.has_gather:
                    ex.status_dirty = True
                return self._finish(outs, small_dst)
            if len(self._seen) < 64:
                self._seen.add(key)
        self._issue(stream, timer)
        del keep
        if self.has_gather:
            ex.status_dirty = True
        return self._finish(outs, small_dst)

    # -- output storage ------------------------------------------------------------
    #: results up to this many bytes (losses, counters, small bias gradients) live apart from
    #: the large ones, so that a caller who keeps a loss keeps a few KB alive, not the step's
    #: gradients
    SMALL_OUTPUT_BYTES = 4096
    POOL_SLABS = 4

    def _layout_outputs(self) -> None:
        """Offsets of every distinct output buffer inside the step's two allocations."""
        self._out_layout: dict = {}
        totals = [0, 0]
        for bid, shape, dtype in self.plan.outputs:
            if bid in self._out_layout:
                continue
            n = 1
            for d in shape:
                n *= d
            nbytes = n * dtype.size_in_bytes
            is_small = nbytes <= self.SMALL_OUTPUT_BYTES
            self._out_layout[bid] = (is_small, totals[is_small], nbytes, tuple(shape), dtype)
            totals[is_small] += (max(nbytes, 1) + 255) & ~255
        self._out_bytes = (max(totals[0], 256), max(totals[1], 256))
        self._pools: tuple = ([], [])   # per class: [slab, use count when nobody holds a view]
        self._small_stage = None         # fixed small slab the kernels write once callers hoard
        self._runs = 0

    def _new_slab(self, nbytes: int):
        return torch.empty(nbytes, dtype=torch.uint8, device=self.ex.torch_device)

    @staticmethod
    def _use_count(slab) -> int:
        return torch._C._storage_Use_Count(slab.untyped_storage()._cdata)

    def _from_pool(self, cls: int):
        """A slab of this plan that no returned tensor (or anything made from one: views, DLPack
        exports) refers to any more, a new pooled one while the pool has room, else None.  The
        plan owns its slabs, so a step whose caller drops or overwrites the previous results
        runs on the same addresses again whatever the allocator does in between, which is what
        lets the step be replayed as a recorded graph."""
        pool = self._pools[cls]
        for slab, idle in pool:
            if self._use_count(slab) == idle:
                return slab
        if len(pool) < self.POOL_SLABS:
            slab = self._new_slab(self._out_bytes[cls])
            pool.append((slab, self._use_count(slab)))
            return slab
        return None

    def _take_slabs(self):
        """(large slab, small slab the kernels write, small slab the caller gets or None)."""
        self._runs += 1
        if self._runs == 1:
            # a plan that runs once (eager evaluation of a new expression) keeps nothing
            return self._new_slab(self._out_bytes[0]), self._new_slab(self._out_bytes[1]), None
        large = self._from_pool(0)
        if large is None:  # the caller holds the results of POOL_SLABS steps: plain allocations
            large = self._new_slab(self._out_bytes[0])
        if self._small_stage is None:
            small = self._from_pool(1)
            if small is not None:
                return large, small, None
            # the caller keeps the small results of many steps (a list of losses): from now on
            # the kernels write them to one fixed slab (same addresses every step, so the
            # recorded step stays valid) and each step hands out a copy
            self._small_stage = self._new_slab(self._out_bytes[1])
        return large, self._small_stage, True

    def _finish(self, outs, small_dst):
        if small_dst is None:
            return outs
        copy = self._small_stage.clone()  # ordered behind the step on the current stream
        done = {}
        for oi, (bid, _, _) in enumerate(self.plan.outputs):
            is_small, off, nbytes, shape, dtype = self._out_layout[bid]
            if is_small:
                if bid not in done:
                    done[bid] = copy[off:off + nbytes].view(dtype.to_torch()).reshape(shape)
                outs[oi] = done[bid]
        return outs

    def _record(self, key):
        """Capture the launch sequence (with the pointers now patched in) on the executor's
        side stream and return the executable graph, or None.  Any failure switches graphs off
        for this plan; nothing has executed either way."""
        ex = self.ex
        L = ex.lib
        side = ex.capture_stream()
        if side is None or L.nbk_graph_begin_capture(side) != 0:
            self._graph_off = True
            return None
        ok = True
        try:
            self._issue(side, None)
        except Exception:
            ok = False
        g = C.c_void_p()
        rc = L.nbk_graph_end_capture(side, C.byref(g))
        if not ok or rc != 0 or not g.value:
            self._graph_off = True
            return None
        self._graphs[key] = g
        return g

    def _issue(self, stream, timer) -> None:
        plan = self.plan
        base = self.base
        check = lib.check
        for si, (fn, args, patches, _keep) in enumerate(self.calls):
            after = timer(si, plan.steps[si].kind, stream) if timer is not None else None
            for obj, fieldname, buf, off in patches:
                setattr(obj, fieldname, base[buf] + off)
            if args[0] is _LATE:
                call_args = [C.c_void_p(getattr(x.h, x.n)) if type(x) is _Late else x for x in args[1:]]
            elif len(args) >= 2 and isinstance(args[0], _Ptrs):
                h = args[0]
                call_args = [C.c_void_p(getattr(h, n)) for n in args[1]] + list(args[2:])
            elif len(args) >= 3 and isinstance(args[1], _Ptrs):
                h = args[1]
                call_args = [args[0]] + [C.c_void_p(getattr(h, n)) for n in args[2]] + list(args[3:])
            else:
                call_args = args
            check(fn(*call_args, stream))
            if after is not None:
                after()


class _Ptrs:
    """Mutable holder for raw addresses that are patched per run."""

    __slots__ = ("p0", "p1", "p2", "p3")

    def __init__(self, n: int):
        self.p0 = self.p1 = self.p2 = self.p3 = None


class _Late:
    """An address argument read from its holder when the call is made."""

    __slots__ = ("h", "n")

    def __init__(self, holder: _Ptrs, name: str):
        self.h, self.n = holder, name


_LATE = "late"  # first element of an argument list that contains _Late entries


class HipExecutor:
    """Runs plans on one gfx950 GPU.  Construction fails without it."""

    name = "hip"

    def __init__(self, device: int = 0):
        self.lib = lib.load()
        if not torch.cuda.is_available():
            raise RuntimeError(
                "nabla_amd needs a ROCm GPU: torch.cuda.is_available() is False and the "
                "package has no CPU execution path"
            )
        lib.check(self.lib.nbk_init(device))
        self.torch_device = torch.device("cuda", device)
        self.status_flag = torch.zeros(1, dtype=torch.int32, device=self.torch_device)
        # generator state read by every random launch: [seed, steps drawn so far]
        self.rng_state = torch.zeros(2, dtype=torch.int64, device=self.torch_device)
        self.use_graphs = os.environ.get("NBK_GRAPHS", "1") != "0"  # replay repeated steps as HIP graphs
        self._capture_stream = None
        self.graph_replays = 0
        self.status_dirty = False        # a launched plan may have flagged a bad gather index
        self.force_interpreter = False   # plans bound while set never use specialised row kernels
        self.launch_timer = None         # callable(step index, kind, stream) -> callable | None: measurement hook; plans run as plain launches while set

    def current_stream(self) -> int:
        return torch.cuda.current_stream(self.torch_device).cuda_stream

    def seed(self, value: int) -> None:
        """Restart the random generator: the same seed gives the same numbers again."""
        v = int(value) & 0xFFFFFFFFFFFFFFFF
        self.rng_state.copy_(torch.tensor([v - (1 << 64) if v >= (1 << 63) else v, 0], dtype=torch.int64))

    def bind(self, plan: Plan) -> BoundPlan:
        return BoundPlan(plan, self)

    def capture_stream(self):
        """Side stream that graph recordings are made on (the default stream cannot record)."""
        if self._capture_stream is None:
            s = C.c_void_p()
            if self.lib.nbk_stream_create(C.byref(s)) != 0 or not s.value:
                return None
            self._capture_stream = s
        return self._capture_stream

    def synchronize(self) -> None:
        torch.cuda.current_stream(self.torch_device).synchronize()

    def check_status(self) -> None:
        """Raise if a kernel flagged a data-dependent error (out-of-range gather index)."""
        if not self.status_dirty:
            return
        self.status_dirty = False
        if int(self.status_flag.item()) != 0:
            self.status_flag.zero_()
            raise IndexError("gather: index out of range")


_EXECUTOR: Any = None


def get_executor():
    global _EXECUTOR
    if _EXECUTOR is None:
        _EXECUTOR = HipExecutor(0)
    return _EXECUTOR


def set_executor(ex) -> Any:
    """Install another executor (used by host-logic tests); returns the previous one."""
    global _EXECUTOR
    prev = _EXECUTOR
    _EXECUTOR = ex
    from ..core import engine
    engine.clear_plan_cache()
    from ..core import tensor as _t
    _t._SCALAR_CACHE.clear()
    return prev
