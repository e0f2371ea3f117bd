"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|c1|c2|c3|c4|c5]

Prints ONE JSON line.  With the default ``--workload all`` the line's headline (``value``,
``ms_per_step``, ``roofline``, ``cpu_baseline``) is the largest configuration, the 12-layer LoRA
fine-tuning step (c5: bf16, D2048, S2048, B4, V32000), and ``configs`` carries the same figures
for each of the five configurations, so that one line holds every clause of the metric: steps/s
per configuration, the MFMA fraction of the GEMM + attention kernels (c3, c5; convolutions for
c4) and the HBM fraction of the fused elementwise + reduction kernel (c2).

A step is one call of the public compiled function (``nb.compile(step)(*args)``: signature
hashing, pytree flattening, plan replay, result wrapping) with its inputs resident in HBM; K
calls are timed between device synchronisations after W warm-up calls.  The same plan called
one layer lower (``BoundPlan.run`` on prepared buffers) is timed beside it
(``plan_ms_per_step``).  Kernel durations for ``roofline`` come from HIP events recorded on the
launch stream around every launch of the dominant kind: inside the timed region when a step is
a single launch (c2), else from a second pass of plain launches, because the timed region
replays the step as one HIP graph, inside which events cannot be recorded (``kernel_timing``
says which).
"""
from __future__ import annotations

import argparse
import ctypes as C
import gc
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "train steps/sec fwd+bwd at 1 MI355X; GEMM % MFMA peak; fused-op % HBM BW"
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}
MFMA_KINDS = ("gemm", "attention", "attention_bwd", "conv2d", "conv2d_dgrad", "conv2d_wgrad")


class KernelTimer:
    """Brackets chosen plan steps with HIP events on the launch stream."""

    def __init__(self, lib, kinds):
        self.lib = lib
        self.kinds = set(kinds)
        self.pairs = []  # (step index, kind, start event, stop event)

    def __call__(self, si, kind, stream):
        if kind not in self.kinds:
            return None
        a, b = C.c_void_p(), C.c_void_p()
        self.lib.nbk_event_create(C.byref(a))
        self.lib.nbk_event_create(C.byref(b))
        self.lib.nbk_event_record(a, stream)
        self.pairs.append((si, kind, a, b))
        return lambda: self.lib.nbk_event_record(b, stream)

    def durations_ms(self):
        """{(step index, kind): mean duration in ms}"""
        acc = {}
        ms = C.c_float()
        for si, kind, a, b in self.pairs:
            self.lib.nbk_event_elapsed_ms(a, b, C.byref(ms))
            acc.setdefault((si, kind), []).append(ms.value)
            self.lib.nbk_event_destroy(a)
            self.lib.nbk_event_destroy(b)
        self.pairs = []
        return {k: sum(v) / len(v) for k, v in acc.items()}


def sync():
    import torch
    torch.cuda.synchronize()


# ------------------------------------------------------------------ host description
def host_info() -> dict:
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.startswith("model name"):
                    model = ln.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    blas = None
    try:
        from threadpoolctl import threadpool_info
        blas = max((p.get("num_threads", 1) for p in threadpool_info()
                    if p.get("user_api") == "blas"), default=None)
    except Exception:
        pass
    import torch
    return {"cpu_model": model, "os_cpu_count": os.cpu_count(), "numpy_blas_threads": blas,
            "torch_threads": torch.get_num_threads()}


def _cpu_entry(value, cores, sample, host):
    return dict(value=round(value, 5), unit="steps/s", cores=cores, kind="port", sample=sample,
                cpu_model=host["cpu_model"], blas_threads=host["numpy_blas_threads"],
                torch_threads=host["torch_threads"])


# ------------------------------------------------------------------ workloads
# The timed path uses the product only (nabla_amd.workloads: step programs and synthetic
# inputs).  The CPU oracle is imported inside the cpu_* functions and nowhere else.
def cpu_c1(host):
    from oracle import configs as oc
    inp = oc.c1_inputs()
    oc.c1_reference(**inp, dtype=np.float32)
    n, t0 = 0, time.perf_counter()
    while n < 20 or time.perf_counter() - t0 < 2.0:
        oc.c1_reference(**inp, dtype=np.float32)
        n += 1
    return _cpu_entry(n / (time.perf_counter() - t0), host["numpy_blas_threads"] or 1,
                      f"{n} full steps, numpy fp32 oracle (BLAS products, one core for the rest)", host)


def cpu_c2(host, rows=8192, cols=8192):
    # rows are independent, so a slice of them times like the whole step
    from oracle import configs as oc
    sample_rows = max(64, rows // 8)
    inp = oc.c2_inputs(sample_rows, cols, seed=0)
    oc.c2_reference(inp["x"][:64], inp["y"][:64], dtype=np.float32)
    reps, t0 = 0, time.perf_counter()
    while reps < 2 or (time.perf_counter() - t0 < 5.0 and reps < 40):
        oc.c2_reference(inp["x"], inp["y"], dtype=np.float32)
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return _cpu_entry(1.0 / (dt * rows / sample_rows), 1,
                      f"{sample_rows} of {rows} rows x {reps} passes, numpy fp32 oracle "
                      "(elementwise numpy: one core), scaled by rows", host)


def cpu_c3(host, batch=8):
    # batch elements are independent but for the mean and the parameter-gradient sums
    import torch
    from oracle import configs as oc
    from oracle import torch_steps as ts
    sample = 2
    t = oc.c3_inputs(sample, 1024, 1024, 4096, seed=0, bf16=True)
    ts.c3_step(oc.c3_inputs(1, 128, 1024, 4096, seed=0), 16, dtype=torch.float32)
    t0 = time.perf_counter()
    ts.c3_step(t, 16, dtype=torch.float32)
    dt = time.perf_counter() - t0
    return _cpu_entry(1.0 / (dt * batch / sample), host["torch_threads"],
                      f"{sample} of {batch} sequences, one full step, torch-CPU fp32 oracle "
                      "(oracle/torch_steps.py), scaled by batch", host)


def cpu_c4(host, batch=64):
    from oracle import configs as oc
    sample = 16
    small = oc.c4_inputs(batch=sample)
    oc.c4_reference(oc.c4_inputs(batch=1), dtype=np.float32)
    t0 = time.perf_counter()
    oc.c4_reference(small, dtype=np.float32)
    dt = time.perf_counter() - t0
    return _cpu_entry(1.0 / (dt * batch / sample), host["numpy_blas_threads"] or 1,
                      f"{sample} of {batch} images, one full step, numpy fp32 oracle "
                      "(BLAS products, one core for the rest), scaled by batch", host)


def cpu_c5(host, layers=12, batch=4):
    # one sequence (of four) through one and through two layers: the difference is a layer's
    # cost, the remainder the embedding, the final norm, the 32000-column head and the loss
    import torch
    from oracle import configs as oc
    from oracle import torch_steps as ts
    t = oc.c5_inputs(layers=2, batch=1, b_zero=False)
    one = dict(t, layers=t["layers"][:1], lora=t["lora"][:1])
    t0 = time.perf_counter()
    ts.c5_step(one, 16, dtype=torch.float32)
    t1 = time.perf_counter()
    ts.c5_step(t, 16, dtype=torch.float32)
    t2 = time.perf_counter()
    per_layer = max((t2 - t1) - (t1 - t0), 1e-9)
    rest = max((t1 - t0) - per_layer, 0.0)
    full = batch * (layers * per_layer + rest)
    return _cpu_entry(1.0 / full, host["torch_threads"],
                      f"1 of {batch} sequences through 1 and through 2 of {layers} layers, torch-CPU "
                      f"fp32 oracle (oracle/torch_steps.py; frozen-weight gradients skipped): "
                      f"{per_layer:.2f} s per layer, {rest:.2f} s embedding + head + loss, "
                      f"extrapolated to {layers} layers x {batch} sequences", host)


def workload_c1(nb):
    t = nb.workloads.synthetic_inputs("c1")
    return dict(name="c1 2-layer MLP fwd+grad fp32, x[128,784]", fn=nb.workloads.c1_step, args=(t,),
                dtype="f32", bound="mfma", algo=104.7e6, kinds=("gemm",), cpu=cpu_c1)


def workload_c2(nb, rows=8192, cols=8192):
    t = nb.workloads.synthetic_inputs("c2", rows=rows, cols=cols)
    algo_bytes = 3 * rows * cols * 4 + 2 * rows * 4
    return dict(name=f"c2 elementwise+reduction fwd+grad, x,y[{rows},{cols}] fp32",
                fn=nb.workloads.c2_step, args=(t["x"], t["y"]), dtype="f32", bound="hbm",
                algo=algo_bytes, kinds=("rowprog",), cpu=cpu_c2)


def workload_c3(nb, batch=8, seq=1024, d=1024, ff=4096):
    t = nb.workloads.synthetic_inputs("c3", batch=batch, seq=seq, d=d, ff=ff)
    T = batch * seq
    hd = d // 16
    qkvo = 4 * 2 * T * d * d
    mlp = 2 * 2 * T * d * ff
    attn_causal = 2 * 2 * batch * 16 * seq * seq * hd / 2
    flops = 3 * (qkvo + mlp + attn_causal)
    return dict(name=f"c3 pre-LN transformer block fwd+bwd bf16, B{batch} S{seq} D{d} FF{ff}",
                fn=lambda t: nb.workloads.c3_step(t, 16), args=(t,), dtype="bf16", bound="mfma",
                algo=flops, kinds=("gemm", "attention", "attention_bwd"), cpu=cpu_c3)


def workload_c4(nb):
    t = nb.workloads.synthetic_inputs("c4")
    return dict(name="c4 CNN step fp32, img[64,32,32,3]", fn=nb.workloads.c4_step, args=(t,),
                dtype="f32", bound="mfma", algo=58.4e9,
                kinds=("conv2d", "conv2d_dgrad", "conv2d_wgrad"), cpu=cpu_c4)


def workload_c5(nb, layers=12):
    t = nb.workloads.synthetic_inputs("c5", layers=layers)
    return dict(name=f"c5 LoRA step bf16, {layers} layers D2048 S2048 B4 V32000 r16 "
                     "(lora_linear in low-rank order)",
                fn=lambda t: nb.workloads.c5_step(t, 16), args=(t,), dtype="bf16", bound="mfma",
                algo=24.5e12 * layers / 12, kinds=("gemm", "attention", "attention_bwd"), cpu=cpu_c5)


WORKLOADS = {"c1": workload_c1, "c2": workload_c2, "c3": workload_c3, "c4": workload_c4,
             "c5": workload_c5}


def committed_traffic(workload: str, kernel_hashes: set):
    """HBM bytes per launch of the dominant kernel as the hardware counters saw them
    (FETCH_SIZE + WRITE_SIZE from two rocprofv3 --pmc runs of this command, each scaled by the
    same counter's reading for a plain copy of known size).  A process cannot read those
    counters for itself, so the figure comes from the committed summary of those runs, and
    only while the kernel timed here is still the kernel they profiled (its program hash is
    part of its name)."""
    path = os.path.join(ROOT, "profiles", f"hbm_traffic_{workload}.json")
    try:
        with open(path) as f:
            z = json.load(f)
    except (OSError, ValueError):
        return None, None
    if not any(h in z.get("kernel", "") for h in kernel_hashes):
        return None, f"profiles/hbm_traffic_{workload}.json is for {z.get('kernel')}, not the kernel timed here"
    return z.get("traffic_bytes_per_launch"), f"profiles/hbm_traffic_{workload}.json (rocprofv3 --pmc, kernel {z.get('kernel')})"


def result_digest(nb, out) -> dict:
    """What a step returned, condensed on the host: its first leaf's first element (the loss of
    the training steps), the sum of magnitudes over every leaf, and whether all are finite."""
    leaves, _ = nb.tree_flatten(out)
    head, total, finite = None, 0.0, True
    for leaf in leaves:
        if not isinstance(leaf, nb.Tensor):
            continue
        a = np.asarray(leaf.numpy(), dtype=np.float64)
        if head is None:
            head = float(a.reshape(-1)[0])
        finite = finite and bool(np.isfinite(a).all())
        total += float(np.abs(a).sum())
    return {"head": head, "abs_sum": total, "finite": finite}


def launch_flops(step) -> float:
    """Algorithmic flops of one MFMA launch of the plan (attention counted causal-aware)."""
    a, k = step.attrs, step.kind
    if k == "gemm":
        return 2.0 * a["M"] * a["N"] * a["K"] * max(a.get("batch", 1), 1)
    if k in ("attention", "attention_bwd"):
        f = 4.0 * a["B"] * a["H"] * a["S"] * a["S"] * a["hd"] * (0.5 if a["causal"] else 1.0)
        return f if k == "attention" else 2.5 * f
    if k.startswith("conv2d"):
        n, ho, wo, co = a["y_shape"]
        r, s, ci, _ = a["w_shape"]
        return 2.0 * n * ho * wo * co * r * s * ci
    return 0.0


def rowprog_bytes(step) -> float:
    """Algorithmic bytes of one row-program launch: every distinct operand read or written once
    (an operand that is broadcast along an axis counts the elements it has, not the ones it is
    read as)."""
    a = step.attrs
    total = 0.0
    for o in a["operands"]:
        n = a["C"] if o.col_stride != 0 else 1
        for d, st in zip(a["lead"], o.lead_strides):
            if st != 0:
                n *= d
        total += n * o.dtype.size_in_bytes
    return total


def launch_label(step) -> str:
    a, k = step.attrs, step.kind
    if k == "gemm":
        lay = ("n" if a["a_cs"] == 1 else "t") + ("n" if a["b_cs"] == 1 else "t")
        b = f" x{a['batch']}" if a.get("batch", 1) > 1 else ""
        return f"gemm {lay} {a['M']}x{a['N']}x{a['K']}{b}"
    if k in ("attention", "attention_bwd"):
        return f"{k} B{a['B']} H{a['H']} S{a['S']} hd{a['hd']}"
    if k.startswith("conv2d"):
        return f"{k} x{tuple(a['x_shape'])} w{tuple(a['w_shape'])}"
    return k


def measure(nb, L, ex, w, steps, warmup, with_cpu, host, calibrate_copy=False):
    import torch
    from nabla_amd.backend import lib as nbk_lib
    cf = nb.compile(w["fn"])
    args = w["args"]
    out = cf(*args)  # miss: trace, lower, bind
    first = result_digest(nb, out)  # (read now: the plan hands its result slabs out again)
    spec = next(iter(next(iter(cf._cache.values())).specializations.values()))
    plan = spec.bound.plan
    flat, _ = nb.tree_flatten((args, {}))
    inputs = [flat[v]._impl._buffer if kind == "arg" else v for kind, v in spec.input_plan]
    single = len(plan.steps) == 1

    if calibrate_copy:
        n = 64 * 1024 * 1024  # fp32 elements: 256 MiB read, 256 MiB written per launch
        src = torch.zeros(n, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        shape, st1 = (C.c_int64 * 1)(n), (C.c_int64 * 1)(1)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        for _ in range(3):
            nbk_lib.check(L.nbk_copy_strided(C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), 0, 0,
                                             1, shape, st1, st1, stream))
        sync()
        del src, dst

    for _ in range(warmup):
        out = cf(*args)
    sync()
    timer = KernelTimer(L, w["kinds"])
    replays0 = ex.graph_replays
    if single:
        ex.launch_timer = timer  # one launch per step: the events sit inside the timed region
    t0 = time.perf_counter()
    for _ in range(steps):
        out = cf(*args)
    sync()
    wall = time.perf_counter() - t0
    ex.launch_timer = None
    replays = ex.graph_replays - replays0
    if single:
        kernel_timing = "HIP events around the launch, inside the timed region"
        dur = timer.durations_ms()
    # the step that was timed (a graph replay for the multi-launch steps) still computes what the
    # first, plainly launched call computed
    last = result_digest(nb, out)
    del out
    if not (first["finite"] and last["finite"]):
        raise RuntimeError(f"{w['name']}: a result of the timed step is not finite: {first} / {last}")
    if abs(first["head"] - last["head"]) > 1e-6 * abs(first["head"]) + 1e-12 or \
            abs(first["abs_sum"] - last["abs_sum"]) > 1e-5 * abs(first["abs_sum"]) + 1e-12:
        raise RuntimeError(f"{w['name']}: the timed step's results differ from the first call's: "
                           f"{first} / {last}")
    # the same plan one layer below the public call
    for _ in range(min(warmup, 3)):
        spec.bound.run(inputs)
    sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        spec.bound.run(inputs)
    sync()
    wall_plan = time.perf_counter() - t0
    row_dur = {}
    if not single:
        n2 = min(steps, 20)
        if w["bound"] == "mfma":
            timer.kinds.add("rowprog")  # (reported beside the matrix kernels, not counted with them)
        for _ in range(n2):
            spec.bound.run(inputs, timer=timer)
        sync()
        dur = timer.durations_ms()
        if w["bound"] == "mfma":
            row_dur = {k: v for k, v in dur.items() if k[1] == "rowprog"}
            dur = {k: v for k, v in dur.items() if k[1] != "rowprog"}
        kernel_timing = (f"second pass of {n2} steps, plain launches bracketed by HIP events on the "
                         "launch stream (the timed region replays the step as one HIP graph, inside "
                         "which events cannot be recorded)")
    dom_ms = sum(dur.values())

    if w["bound"] == "hbm":
        achieved = w["algo"] / (dom_ms * 1e-3) / 1e9 if dom_ms else 0.0
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = w["algo"] / (dom_ms * 1e-3) / 1e12 if dom_ms else 0.0
        peak, unit = MFMA_PEAK_TFLOPS[w["dtype"]], "TFLOP/s"
    traffic, traffic_source = None, None
    if w["bound"] == "hbm":
        hashes = set()
        for call in spec.bound.calls:
            if call[0] is L.nbk_rowprog_launch:
                hashes.add(f"{L.nbk_rowprog_hash(C.byref(call[3])):016x}")
        traffic, traffic_source = committed_traffic(w["key"], hashes)
    roofline = {"bound": w["bound"], "achieved": round(achieved, 2), "peak": peak, "unit": unit,
                "frac": round(achieved / peak, 4), "traffic": traffic,
                "kernel": "+".join(k for k in w["kinds"] if k in plan.stats),
                "kernel_ms_per_step": round(dom_ms, 4), "launches_per_step": len(dur),
                "algorithmic_per_step": w["algo"], "kernel_timing": kernel_timing}
    if traffic_source:
        roofline["traffic_source"] = traffic_source
    if w["bound"] == "mfma":
        # per product shape: launches per step, mean duration, achieved rate from that shape's own
        # flop count (2 M N K; attention causal-aware)
        groups: dict = {}
        for (si, kind), ms in dur.items():
            st = plan.steps[si]
            g = groups.setdefault(launch_label(st), [0, 0.0, 0.0])
            g[0] += 1
            g[1] += ms
            g[2] += launch_flops(st)
        by = []
        for label, (n, ms, fl) in sorted(groups.items(), key=lambda kv: -kv[1][1]):
            tf = fl / (ms * 1e-3) / 1e12 if ms else 0.0
            by.append({"kernel": label, "launches": n, "avg_us": round(ms / n * 1e3, 2),
                       "tflops": round(tf, 1), "frac": round(tf / peak, 4)})
        roofline["by_kernel"] = by[:16]
        roofline["counted_flops_per_step"] = sum(g[2] for g in groups.values())
        if row_dur:
            # the fused elementwise / normalisation / loss kernels of the same step against the
            # HBM roofline: algorithmic bytes of each launch over its own duration
            rows = []
            for (si, _), ms in row_dur.items():
                st = plan.steps[si]
                rows.append((ms, rowprog_bytes(st), f"rows{tuple(st.attrs['lead'])} x {st.attrs['C']}, "
                             f"{len(st.attrs['operands'])} operands, {len(st.attrs['ins'])} instructions"))
            rows.sort(key=lambda r: -r[0])
            big = [r for r in rows if r[1] >= 32e6]  # launches that move at least 32 MB
            t_all, b_all = sum(r[0] for r in rows), sum(r[1] for r in rows)
            t_big, b_big = sum(r[0] for r in big), sum(r[1] for r in big)
            roofline["row_kernels"] = {
                "launches_per_step": len(rows), "ms_per_step": round(t_all, 4),
                "gb_per_s": round(b_all / (t_all * 1e-3) / 1e9, 1) if t_all else 0.0,
                "launches_over_32MB": len(big),
                "gb_per_s_over_32MB": round(b_big / (t_big * 1e-3) / 1e9, 1) if t_big else 0.0,
                "frac_of_hbm_peak_over_32MB": round(b_big / (t_big * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if t_big else 0.0,
                "slowest": [{"kernel": r[2], "us": round(r[0] * 1e3, 1), "gb_per_s": round(r[1] / (r[0] * 1e-3) / 1e9, 1)}
                            for r in rows[:6]]}
    res = {"self_check": {"first_result": first["head"], "same_after_timed_region": True, "finite": True},
           "workload": w["name"], "value": round(steps / wall, 3), "unit": "steps/s",
           "ms_per_step": round(wall / steps * 1e3, 4),
           "plan_ms_per_step": round(wall_plan / steps * 1e3, 4),
           "dtype": w["dtype"], "graph_replays_in_timed_region": replays,
           "plan": plan.stats, "roofline": roofline}
    if with_cpu:
        res["cpu_baseline"] = w["cpu"](host)
    return res


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all", choices=["all"] + sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a plain 256 MiB copy (nbk_copy_strided) three times before the "
                         "steps: the known-size kernel that hardware byte counters are scaled by")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        return 2

    import torch

    import nabla_amd as nb
    from nabla_amd.backend import lib as nbk_lib
    from nabla_amd.backend.executor import get_executor
    from nabla_amd.core import engine

    ex = get_executor()  # raises without libnbk.so or without a gfx950 GPU
    L = nbk_lib.load()
    host = host_info()
    names = sorted(WORKLOADS) if a.workload == "all" else [a.workload]
    results = {}
    for name in names:
        w = WORKLOADS[name](nb)
        w["key"] = name
        results[name] = measure(nb, L, ex, w, a.steps, a.warmup, not a.no_cpu, host,
                                calibrate_copy=a.calibrate_copy)
        del w
        engine.clear_plan_cache()
        gc.collect()
        torch.cuda.empty_cache()
    head = results[names[-1]]  # c5 (the largest configuration) when all five run
    # The one line stays small enough to be read whole from the end of a log: the headline
    # configuration with its three slowest product shapes, then one compact object per
    # configuration, last.  Everything else (every product shape, the slowest row kernels, plan
    # statistics, the CPU samples) goes to a side file.
    details = os.environ.get("NBK_BENCH_DETAILS", os.path.join(ROOT, "gpurun_out", "bench_details.json"))
    try:
        os.makedirs(os.path.dirname(details), exist_ok=True)
        with open(details, "w") as f:
            json.dump({"host": host, "configs": results}, f, indent=1)
    except OSError:
        details = None

    def brief_roofline(r: dict, shapes: int) -> dict:
        keep = {k: r[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel",
                                  "kernel_ms_per_step", "launches_per_step", "algorithmic_per_step")
                if k in r}
        if shapes and "by_kernel" in r:
            keep["by_kernel"] = r["by_kernel"][:shapes]
        if "row_kernels" in r:
            rk = r["row_kernels"]
            keep["row_kernels"] = {k: rk[k] for k in ("launches_per_step", "ms_per_step", "gb_per_s_over_32MB",
                                                     "frac_of_hbm_peak_over_32MB")}
        return keep

    def brief_config(v: dict) -> dict:
        r = v["roofline"]
        c = {"ms_per_step": v["ms_per_step"], "value": v["value"], "dtype": v["dtype"],
             "roofline": {"bound": r["bound"], "frac": r["frac"], "achieved": r["achieved"], "unit": r["unit"],
                          "kernel_ms_per_step": r["kernel_ms_per_step"], "traffic": r["traffic"]}}
        if "row_kernels" in r:
            c["row_kernels_frac_of_hbm_peak_over_32MB"] = r["row_kernels"]["frac_of_hbm_peak_over_32MB"]
        if "cpu_baseline" in v:
            c["cpu_baseline"] = {"value": v["cpu_baseline"]["value"], "cores": v["cpu_baseline"]["cores"]}
        return c

    line = {
        "metric": METRIC, "value": head["value"], "unit": "steps/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": head["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": head["workload"],
                   "step": "public compiled call: forward + gradients, inputs resident in HBM",
                   "plan_ms_per_step": head["plan_ms_per_step"], "launches_per_step": head["plan"]["steps"],
                   "graph_replays_in_timed_region": head["graph_replays_in_timed_region"],
                   "self_check": head["self_check"]},
        "roofline": brief_roofline(head["roofline"], 3), "cpu_baseline": head.get("cpu_baseline"),
        "host": {"cpu_model": host["cpu_model"], "os_cpu_count": host["os_cpu_count"]},
        "details_file": os.path.relpath(details, ROOT) if details else None,
    }
    line["roofline"]["kernel_timing"] = head["roofline"]["kernel_timing"]
    if len(names) > 1:
        line["configs"] = {k: brief_config(v) for k, v in results.items()}
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
