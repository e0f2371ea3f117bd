"""Benchmark of the hot path on one MI355X.

Default workload: the elementwise + reduction stress configuration
(x, y [8192, 8192] fp32; out = sum(exp(x*y - max(x*y)) * relu(x), axis=1) and
the gradient of sum(out) w.r.t. x), one compiled step per iteration with the
inputs already resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1|c2|c3|c4|c5]
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}


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
        out = {}
        ms = C.c_float()
        for si, kind, a, b in self.pairs:
            self.lib.nbk_event_elapsed_ms(a, b, C.byref(ms))
            out.setdefault((si, kind), []).append(ms.value)
            self.lib.nbk_event_destroy(a)
            self.lib.nbk_event_destroy(b)
        self.pairs = []
        return out


def sync():
    import torch
    torch.cuda.synchronize()


def compiled_plan(nb, fn, args):
    """Trace + lower ``fn`` once; returns (bound plan, input buffers, call that
    replays it).  The replay is what a cached ``@compile`` call executes."""
    cf = nb.compile(fn)
    out = cf(*args)
    spec = next(iter(next(iter(cf._cache.values())).specializations.values()))
    flat, _ = nb.tree_flatten((args, {}))

    def bufs():
        return [flat[v]._impl._buffer if kind == "arg" else v for kind, v in spec.input_plan]

    return cf, spec, bufs, out


# ------------------------------------------------------------------ workloads
# The timed path uses the product only (nabla_amd.workloads: step programs and synthetic
# inputs).  The CPU oracle is imported inside the cpu_baseline closures and nowhere else.
def workload_c2(nb, rows=8192, cols=8192):
    t = nb.workloads.synthetic_inputs("c2", rows=rows, cols=cols)
    algo_bytes = 3 * rows * cols * 4 + 2 * rows * 4
    return dict(name=f"c2 elementwise+reduction fwd+grad, x,y[{rows},{cols}] fp32",
                fn=nb.workloads.c2_step, args=(t["x"], t["y"]), dtype="f32", bound="hbm",
                algo=algo_bytes, dominant="rowprog", cpu=lambda: cpu_c2(rows, cols))


def cpu_c2(rows, cols):
    # rows are independent, so a slice of them times like the whole step; the slice is sized
    # for a run of about ten seconds (one untimed pass first: page faults, numpy warm-up)
    from oracle import configs as oc
    sample_rows = max(64, rows // 4)
    inp = oc.c2_inputs(sample_rows, cols, seed=0)
    oc.c2_reference(inp["x"][:64], inp["y"][:64], dtype=np.float32)
    reps, t0 = 0, time.perf_counter()
    while reps < 3 or (time.perf_counter() - t0 < 8.0 and reps < 40):
        oc.c2_reference(inp["x"], inp["y"], dtype=np.float32)
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return dict(value=round(1.0 / (dt * rows / sample_rows), 4), unit="steps/s", cores=1, kind="port",
                sample=f"{sample_rows} of {rows} rows x {reps} passes, numpy fp32 oracle, scaled by rows")


def workload_c1(nb):
    t = nb.workloads.synthetic_inputs("c1")

    def cpu():
        from oracle import configs as oc
        inp = oc.c1_inputs()
        t0 = time.perf_counter()
        n = 20
        for _ in range(n):
            oc.c1_reference(**inp, dtype=np.float32)
        return dict(value=n / (time.perf_counter() - t0), unit="steps/s", cores=os.cpu_count(),
                    kind="port", sample=f"{n} full steps, numpy fp32 oracle")

    return dict(name="c1 2-layer MLP fwd+grad fp32, x[128,784]", fn=nb.workloads.c1_step, args=(t,),
                dtype="f32", bound="mfma", algo=104.7e6, dominant="gemm", cpu=cpu)


def workload_c3(nb, batch=8, seq=1024, d=1024, ff=4096):
    t = nb.workloads.synthetic_inputs("c3", batch=batch, seq=seq, d=d, ff=ff)
    T = batch * seq
    hd = d // 16
    qkvo = 4 * 2 * T * d * d
    mlp = 2 * 2 * T * d * ff
    attn_causal = 2 * 2 * batch * 16 * seq * seq * hd / 2
    flops = 3 * (qkvo + mlp + attn_causal)

    def cpu():
        from oracle import configs as oc
        small = oc.c3_inputs(1, 128, d, ff, seed=0, bf16=True)
        t0 = time.perf_counter()
        oc.c3_reference(small, num_heads=16, dtype=np.float32)
        dt = time.perf_counter() - t0
        scale = T / 128.0
        return dict(value=1.0 / (dt * scale), unit="steps/s", cores=os.cpu_count(), kind="port",
                    sample="1 x 128 tokens of 8 x 1024, numpy fp32 oracle, scaled by tokens "
                           "(attention cost per token is under-counted)")

    return dict(name=f"c3 pre-LN transformer block fwd+bwd bf16, B{batch} S{seq} D{d} FF{ff}",
                fn=lambda t: nb.workloads.c3_step(t, 16), args=(t,), dtype="bf16", bound="mfma",
                algo=flops, dominant="gemm", cpu=cpu)


def workload_c4(nb):
    t = nb.workloads.synthetic_inputs("c4")

    def cpu():
        from oracle import configs as oc
        small = oc.c4_inputs(batch=4)
        t0 = time.perf_counter()
        oc.c4_reference(small, dtype=np.float32)
        dt = time.perf_counter() - t0
        return dict(value=1.0 / (dt * 16), unit="steps/s", cores=os.cpu_count(), kind="port",
                    sample="4 of 64 images, numpy fp32 oracle, scaled by batch")

    return dict(name="c4 CNN step fp32, img[64,32,32,3]", fn=nb.workloads.c4_step, args=(t,),
                dtype="f32", bound="mfma", algo=58.4e9, dominant="conv", cpu=cpu)


def workload_c5(nb, layers=12):
    t = nb.workloads.synthetic_inputs("c5", layers=layers)

    def cpu():
        return dict(value=None, unit="steps/s", cores=os.cpu_count(), kind="port",
                    sample="not run: one step is ~27 TFLOP on the host")

    return dict(name=f"c5 LoRA step bf16, {layers} layers D2048 S2048 B4 (lora_linear in low-rank order)",
                fn=lambda t: nb.workloads.c5_step(t, 16), args=(t,), dtype="bf16", bound="mfma",
                algo=24.5e12 * layers / 12, dominant="gemm", cpu=cpu)


WORKLOADS = {"c1": workload_c1, "c2": workload_c2, "c3": workload_c3, "c4": workload_c4,
             "c5": workload_c5}


def measured_traffic(workload: str):
    """HBM bytes per launch of the dominant kernel as the hardware counters saw them
    (FETCH_SIZE + WRITE_SIZE from two counter runs, scaled by the same counters' reading for
    a plain copy of known size).  Counters cannot be read from inside this process; the
    figure comes from the committed summary of those runs, None when there is none."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                        f"hbm_traffic_{workload}.json")
    try:
        with open(path) as f:
            return json.load(f).get("traffic_bytes_per_launch")
    except (OSError, ValueError):
        return None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a plain 256 MiB copy (nbk_copy_strided) three times before the "
                         "steps: the known-size kernel that hardware byte counters are scaled by")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        return 2

    import nabla_amd as nb
    from nabla_amd.backend import lib as nbk_lib
    from nabla_amd.backend.executor import get_executor

    ex = get_executor()  # raises without libnbk.so or without a gfx950 GPU
    L = nbk_lib.load()
    w = WORKLOADS[a.workload](nb)
    cf, spec, bufs, first = compiled_plan(nb, w["fn"], w["args"])
    plan = spec.bound.plan
    inputs = bufs()

    if a.calibrate_copy:
        import ctypes as C
        import torch
        n = 64 * 1024 * 1024  # fp32 elements: 256 MiB read, 256 MiB written per launch
        src = torch.zeros(n, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        shape = (C.c_int64 * 1)(n)
        st1 = (C.c_int64 * 1)(1)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        for _ in range(3):
            nbk_lib.check(L.nbk_copy_strided(C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), 0, 0,
                                             1, shape, st1, st1, stream))
        sync()
    for _ in range(a.warmup):
        spec.bound.run(inputs)
    sync()
    # (the fused attention kernels are MFMA work counted in the same algorithmic flops)
    dominant_kinds = {"rowprog": ["rowprog"], "gemm": ["gemm", "attention", "attention_bwd"],
                      "conv": ["conv2d", "conv2d_dgrad", "conv2d_wgrad"]}[w["dominant"]]
    timer = KernelTimer(L, dominant_kinds)
    if len(plan.steps) == 1:
        # one launch per step: the HIP events sit inside the timed region
        t0 = time.perf_counter()
        for _ in range(a.steps):
            spec.bound.run(inputs, timer=timer)
        sync()
        wall = time.perf_counter() - t0
    else:
        # several launches per step: the product path replays the repeated step as one HIP
        # graph, inside which no event can be recorded; the step rate is timed on that path
        # and the kernel durations for the roofline come from a second pass of plain launches
        # with events on the launch stream
        t0 = time.perf_counter()
        for _ in range(a.steps):
            spec.bound.run(inputs)
        sync()
        wall = time.perf_counter() - t0
        for _ in range(min(a.steps, 20)):
            spec.bound.run(inputs, timer=timer)
        sync()
    ms_per_step = wall / a.steps * 1e3
    dur = timer.durations_ms()
    per_step_total = {}
    for (si, kind), v in dur.items():
        per_step_total[(si, kind)] = sum(v) / len(v)
    dom_ms = sum(per_step_total.values())
    # the single longest launch of the dominant kind
    top = max(per_step_total.items(), key=lambda kv: kv[1]) if per_step_total else None

    if w["bound"] == "hbm":
        achieved = w["algo"] / (dom_ms * 1e-3) / 1e9 if dom_ms else 0.0
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = w["algo"] / (dom_ms * 1e-3) / 1e12 if dom_ms else 0.0
        peak, unit = MFMA_PEAK_TFLOPS[w["dtype"]], "TFLOP/s"
    roofline = {"bound": w["bound"], "achieved": round(achieved, 2), "peak": peak, "unit": unit,
                "frac": round(achieved / peak, 4), "traffic": measured_traffic(a.workload),
                "kernel": "+".join(k for k in dominant_kinds if k in plan.stats),
                "kernel_ms_per_step": round(dom_ms, 4),
                "launches_per_step": len(per_step_total)}
    cpu = None if a.no_cpu else w["cpu"]()
    line = {
        "metric": "train steps/sec fwd+bwd at 1 MI355X; GEMM % MFMA peak; fused-op % HBM BW",
        "value": round(a.steps / wall, 3), "unit": "steps/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": w["name"], "step": "compiled replay of forward + gradients",
                   "plan": plan.stats, "graph_replays": ex.graph_replays},
        "roofline": roofline, "cpu_baseline": cpu,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
