"""nbk_attention_bwd_static -- the attention backward pass for callers that cannot allocate --
through the C ABI against nbk_attention_bwd (the entry point that takes a caller workspace):
the same three gradients bit for bit, on two calls in a row, the second with a smaller input
(the built-in scratch still holds the first call's row sums then), and the size limit."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _desc(lib, t):
    a = lib.AttnTensor()
    a.ptr = t.data_ptr()
    a.sb, a.ss, a.sh = t.stride(0), t.stride(1), t.stride(2)
    return a


def _both_ways(lib, L, shape, causal, seed):
    B, S, H, hd = shape
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(seed)
    q, k, v, g = (torch.tensor(rng.standard_normal(shape), dtype=torch.bfloat16).cuda() for _ in range(4))
    o = torch.empty_like(q)
    lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")
    d = lib.AttnDesc()
    d.B, d.H, d.S, d.hd, d.scale, d.causal, d.dtype = B, H, S, hd, 1.0 / math.sqrt(hd), int(causal), 1
    o_lo = torch.empty_like(q)
    tq, tk, tv, to, tg, tol = (_desc(lib, t) for t in (q, k, v, o, g, o_lo))
    print(f"attention fwd {shape} causal={causal}", flush=True)
    lib.check(L.nbk_attention_fwd(C.byref(d), C.byref(tq), C.byref(tk), C.byref(tv), C.byref(to),
                                  C.byref(tol), C.c_void_p(lse.data_ptr()), st))
    want = [torch.full(shape, float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(3)]
    ws = torch.empty(L.nbk_attention_bwd_workspace(C.byref(d)), dtype=torch.uint8, device="cuda")
    print(f"nbk_attention_bwd {shape}", flush=True)
    lib.check(L.nbk_attention_bwd(C.byref(d), C.byref(tq), C.byref(tk), C.byref(tv), C.byref(to),
                                  C.byref(tol), C.c_void_p(lse.data_ptr()), C.byref(tg),
                                  *[C.byref(_desc(lib, t)) for t in want],
                                  C.c_void_p(ws.data_ptr()), ws.numel(), st))
    got = [torch.full(shape, float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(3)]
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    print(f"nbk_attention_bwd_static {shape}", flush=True)
    lib.check(L.nbk_attention_bwd_static(C.byref(d), C.byref(tq), C.byref(tk), C.byref(tv), C.byref(to),
                                         C.byref(tol), C.c_void_p(lse.data_ptr()), C.byref(tg),
                                         *[C.byref(_desc(lib, t)) for t in got], st))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    for name, a, b in zip(("dq", "dk", "dv"), got, want):
        assert torch.isfinite(b.float()).all(), name
        assert torch.equal(a, b), name
    return d, (tq, tk, tv, to, tg), lse, got


def test_attention_backward_without_allocation_matches_the_workspace_entry_point(hip):
    from nabla_amd.backend import lib
    L = lib.load()
    _both_ways(lib, L, (2, 512, 4, 128), True, 3)    # 4096 score rows
    _both_ways(lib, L, (1, 128, 2, 64), False, 4)    # then 256: the scratch holds stale rows beyond
    _both_ways(lib, L, (2, 256, 3, 64), True, 5)


def test_attention_backward_without_allocation_rejects_what_does_not_fit(hip):
    from nabla_amd.backend import lib
    L = lib.load()
    t = torch.zeros((1, 128, 1, 64), dtype=torch.bfloat16, device="cuda")
    lse = torch.zeros((1, 1, 128), dtype=torch.float32, device="cuda")
    a = _desc(lib, t)
    d = lib.AttnDesc()
    # B * H * S = 2^20 + 128 rows: one tile more than the built-in scratch holds.  Nothing is
    # launched: the check comes before any kernel, so the tensors need not be that large.
    d.B, d.H, d.S, d.hd, d.scale, d.causal, d.dtype = 8193, 1, 128, 64, 0.125, 1, 1
    with pytest.raises(ValueError, match="exceed"):
        lib.check(L.nbk_attention_bwd_static(C.byref(d), *([C.byref(a)] * 4), None, C.c_void_p(lse.data_ptr()),
                                             *([C.byref(a)] * 4), None))
