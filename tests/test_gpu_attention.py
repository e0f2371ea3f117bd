"""Fused attention kernels through the C ABI against float64 softmax attention on the CPU
(the composition of nabla/nn/functional/layers.py:106-153 and its autograd gradients)."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _reference(q, k, v, g, causal):
    """q, k, v, g: [B, S, H, hd] float64.  Returns o, lse ([B, H, S]), dq, dk, dv."""
    q, k, v = (t.clone().requires_grad_(True) for t in (q, k, v))
    S = q.shape[1]
    s = torch.einsum("bshd,bthd->bhst", q, k) / math.sqrt(q.shape[-1])
    if causal:
        s = s.masked_fill(~torch.ones(S, S, dtype=torch.bool).tril(), float("-inf"))
    o = torch.einsum("bhst,bthd->bshd", torch.softmax(s, -1), v)
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), g)
    return o.detach(), torch.logsumexp(s, -1).detach(), dq, dk, dv


def _close(got, want, what, tol=2e-2):
    """bf16 result against float64: half an ulp of the value plus ``tol`` of the tensor's scale."""
    got, want = got.double().cpu(), want.double()
    err = (got - want).abs() - 2.0 ** -8 * want.abs()
    assert torch.isfinite(got).all(), what
    assert err.max().item() <= tol * max(want.abs().max().item(), 1e-6), (what, err.max().item())


def _heads(t, lib, transposed_storage):
    """AttnTensor for a device tensor holding [B, S, H, hd] (or [B, H, S, hd] storage)."""
    a = lib.AttnTensor()
    a.ptr = t.data_ptr()
    if transposed_storage:
        B, H, S, hd = t.shape
        a.sb, a.sh, a.ss = H * S * hd, S * hd, hd
    else:
        B, S, H, hd = t.shape
        a.sb, a.ss, a.sh = S * H * hd, H * hd, hd
    return a


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("shape", [(1, 128, 1, 64), (2, 256, 3, 64), (1, 384, 2, 128), (2, 128, 2, 128),
                                   (1, 1024, 2, 64)])
def test_attention_forward_backward(hip, shape, causal):
    from nabla_amd.backend import lib
    B, S, H, hd = shape
    rng = np.random.default_rng(hash((shape, causal)) % 2 ** 31)
    q, k, v, g = (torch.tensor(rng.standard_normal(shape), dtype=torch.bfloat16) for _ in range(4))
    want = _reference(q.double(), k.double(), v.double(), g.double(), causal)
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    qd, kd, vd, gd = (t.cuda() for t in (q, k, v, g))
    o = torch.full(shape, float("nan"), dtype=torch.bfloat16, device="cuda")
    lse = torch.full((B, H, S), float("nan"), dtype=torch.float32, device="cuda")
    d = lib.AttnDesc()
    d.B, d.H, d.S, d.hd = B, H, S, hd
    d.scale = 1.0 / math.sqrt(hd)
    d.causal = int(causal)
    d.dtype = 1
    o_lo = torch.full(shape, float("nan"), dtype=torch.bfloat16, device="cuda")
    tq, tk, tv, to, tg, tol = (_heads(t, lib, False) for t in (qd, kd, vd, o, gd, o_lo))
    print(f"attention fwd {shape} causal={causal}", flush=True)
    lib.check(L.nbk_attention_fwd(C.byref(d), C.byref(tq), C.byref(tk), C.byref(tv), C.byref(to),
                                  C.byref(tol), C.c_void_p(lse.data_ptr()), st))
    torch.cuda.synchronize()
    _close(o, want[0], "o")
    # output plus its rounding remainder: what is left is the rounding of the probabilities
    # inside the kernel (bf16 operands of the second product), not that of the stored output
    both = o.double().cpu() + o_lo.double().cpu()
    assert (both - want[0]).abs().max().item() <= 3e-3 * want[0].abs().max().item() + 1e-6
    assert (lse.double().cpu() - want[1]).abs().max().item() < 2e-3
    # gradients land in heads-first storage ([B, H, S, hd]) to cover a second layout
    dq, dk, dv = (torch.full((B, H, S, hd), float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(3))
    tdq, tdk, tdv = (_heads(t, lib, True) for t in (dq, dk, dv))
    nbytes = L.nbk_attention_bwd_workspace(C.byref(d))
    assert nbytes == B * H * S * 4
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    print(f"attention bwd {shape} causal={causal}", flush=True)
    lib.check(L.nbk_attention_bwd(C.byref(d), C.byref(tq), C.byref(tk), C.byref(tv), C.byref(to),
                                  C.byref(tol), C.c_void_p(lse.data_ptr()), C.byref(tg), C.byref(tdq),
                                  C.byref(tdk), C.byref(tdv), C.c_void_p(ws.data_ptr()), nbytes, st))
    torch.cuda.synchronize()
    for got, w, name in ((dq, want[2], "dq"), (dk, want[3], "dk"), (dv, want[4], "dv")):
        _close(got.permute(0, 2, 1, 3), w, name)


@pytest.mark.parametrize("hd", [64, 128])
def test_attention_row_sums_keep_their_digits_when_values_share_a_large_part(hip, hd):
    """Values that all carry one large common vector (what a residual stream looks like after a
    few layers of diffuse attention): dP - delta then cancels most of dP, and delta = rowsum(dO * O)
    from bf16 O alone is several percent off in dQ and dK.  With the forward pass's rounding
    remainder the query and key gradients stay within 2e-2 of float64; without it they do not
    (which is what makes this a test of the remainder and not of the tolerance)."""
    from nabla_amd.backend import lib
    B, S, H = 1, 1024, 2
    shape = (B, S, H, hd)
    rng = np.random.default_rng(77 + hd)
    bf = lambda a: torch.tensor(a, dtype=torch.bfloat16)
    common = rng.standard_normal((1, 1, H, hd)) * 16.0
    q, k, g = (bf(rng.standard_normal(shape) * 0.3) for _ in range(3))
    v = bf(rng.standard_normal(shape) + common)
    want = _reference(q.double(), k.double(), v.double(), g.double(), True)
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    qd, kd, vd, gd = (t.cuda() for t in (q, k, v, g))
    o, o_lo = (torch.empty(shape, dtype=torch.bfloat16, device="cuda") for _ in range(2))
    lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")
    d = lib.AttnDesc()
    d.B, d.H, d.S, d.hd, d.scale, d.causal, d.dtype = B, H, S, hd, 1.0 / math.sqrt(hd), 1, 1
    tq, tk, tv, to, tg, tol = (_heads(t, lib, False) for t in (qd, kd, vd, o, gd, o_lo))
    print(f"attention fwd with remainder {shape}", flush=True)
    lib.check(L.nbk_attention_fwd(C.byref(d), C.byref(tq), C.byref(tk), C.byref(tv), C.byref(to),
                                  C.byref(tol), C.c_void_p(lse.data_ptr()), st))
    ws = torch.empty(L.nbk_attention_bwd_workspace(C.byref(d)), dtype=torch.uint8, device="cuda")
    err = {}
    for with_rest in (True, False):
        dq, dk, dv = (torch.empty(shape, dtype=torch.bfloat16, device="cuda") for _ in range(3))
        print(f"attention bwd {shape} remainder={with_rest}", flush=True)
        lib.check(L.nbk_attention_bwd(C.byref(d), C.byref(tq), C.byref(tk), C.byref(tv), C.byref(to),
                                      C.byref(tol) if with_rest else None, C.c_void_p(lse.data_ptr()),
                                      C.byref(tg), *[C.byref(_heads(t, lib, False)) for t in (dq, dk, dv)],
                                      C.c_void_p(ws.data_ptr()), ws.numel(), st))
        torch.cuda.synchronize()
        err[with_rest] = [((got.double().cpu() - w).abs().max() / w.abs().max()).item()
                          for got, w in zip((dq, dk, dv), want[2:])]
    assert max(err[True]) < 2e-2, err
    assert err[False][0] > 2.0 * err[True][0] and err[False][0] > 2e-2, err


def test_attention_rejects_what_the_kernels_do_not_cover(hip):
    from nabla_amd.backend import lib
    L = lib.load()
    t = torch.zeros((1, 128, 1, 64), dtype=torch.bfloat16, device="cuda")
    lse = torch.zeros((1, 1, 128), dtype=torch.float32, device="cuda")
    a = _heads(t, lib, False)
    for field, value, msg in (("hd", 32, "head size"), ("S", 100, "multiple of 128"), ("dtype", 0, "bf16")):
        d = lib.AttnDesc()
        d.B, d.H, d.S, d.hd, d.scale, d.causal, d.dtype = 1, 1, 128, 64, 0.125, 1, 1
        setattr(d, field, value)
        with pytest.raises(ValueError, match=msg):
            lib.check(L.nbk_attention_fwd(C.byref(d), C.byref(a), C.byref(a), C.byref(a), C.byref(a),
                                          None, C.c_void_p(lse.data_ptr()), None))
    d = lib.AttnDesc()
    d.B, d.H, d.S, d.hd, d.scale, d.causal, d.dtype = 1, 1, 128, 64, 0.125, 1, 1
    bad = _heads(t, lib, False)
    bad.ss = 60
    with pytest.raises(ValueError, match="strides"):
        lib.check(L.nbk_attention_fwd(C.byref(d), C.byref(bad), C.byref(a), C.byref(a), C.byref(a),
                                      None, C.c_void_p(lse.data_ptr()), None))
    with pytest.raises(ValueError, match="workspace"):
        lib.check(L.nbk_attention_bwd(C.byref(d), *([C.byref(a)] * 4), None, C.c_void_p(lse.data_ptr()),
                                      *([C.byref(a)] * 4), None, 0, None))


def test_attention_inside_the_transformer_block(hip):
    """The C3 block in bf16 goes through the fused kernels and agrees with the float64 oracle."""
    import nabla_amd as nb
    from oracle import configs as oc
    t = oc.c3_inputs(2, 256, 256, 512, seed=4, bf16=True)
    wl, wg = oc.c3_reference(t, num_heads=4)
    loss, grads = oc.c3_program(nb, oc.upload(nb, t, nb.DType.bfloat16), num_heads=4)
    nb.realize_all(loss, *grads.values())
    from nabla_amd.core.engine import _PLAN_CACHE
    st = list(_PLAN_CACHE.values())[-1].plan.stats
    assert st.get("attention") == 1 and st.get("attention_bwd") == 1 and st.get("copy", 0) == 0
    assert abs(loss.item() - wl) < 2e-2 * abs(wl)
    for k in oc.C3_PARAMS:
        got = grads[k].numpy().astype(np.float64)
        # (the key bias has a zero true gradient: measured on the scale of the query bias's)
        floor = np.abs(wg["bq"]).max() if k == "bk" else 0.0
        assert np.abs(got - wg[k]).max() <= 2e-2 * max(np.abs(wg[k]).max(), floor), k


def _run_fwd(lib, L, st, q, k, v, causal):
    """q, k, v: device bf16 [B, S, H, hd] (any strides with hd contiguous) -> o, lse."""
    B, S, H, hd = q.shape
    o = torch.empty((B, S, H, hd), dtype=torch.bfloat16, device="cuda")
    lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")
    d = lib.AttnDesc()
    d.B, d.H, d.S, d.hd, d.scale, d.causal, d.dtype = B, H, S, hd, 1.0 / math.sqrt(hd), int(causal), 1

    def desc(t):
        a = lib.AttnTensor()
        a.ptr = t.data_ptr()
        a.sb, a.ss, a.sh = t.stride(0), t.stride(1), t.stride(2)
        return a

    ts = [desc(t) for t in (q, k, v, o)]
    lib.check(L.nbk_attention_fwd(C.byref(d), *[C.byref(t) for t in ts], None, C.c_void_p(lse.data_ptr()), st))
    return o, lse, d, ts


@pytest.mark.parametrize("shape", [(8, 1024, 16, 64), (4, 2048, 16, 128)])
def test_attention_properties_at_full_size(hip, shape):
    """Size-independent facts at the benchmark shapes, where a float64 reference is too slow:
    probability rows sum to one (V = 1 gives O = 1 and dV = column sums of dO-weighted P),
    causality (later keys and values do not reach earlier queries), linearity in V, and the
    gradient identity sum(dQ * Q) = sum(dK * K) (scores are bilinear in Q and K)."""
    from nabla_amd.backend import lib
    B, S, H, hd = shape
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator(device="cuda").manual_seed(7)
    rnd = lambda: torch.randn(shape, generator=gen, device="cuda").to(torch.bfloat16)
    q, k, v, v2, g = rnd(), rnd(), rnd(), rnd(), rnd()
    print(f"attention properties {shape}", flush=True)
    ones = torch.ones_like(v)
    o1, lse, d, ts = _run_fwd(lib, L, st, q, k, ones, True)
    torch.cuda.synchronize()
    assert torch.isfinite(lse).all()
    assert (o1.float() - 1.0).abs().max().item() <= 2 ** -7          # rows of P sum to one
    o, _, _, _ = _run_fwd(lib, L, st, q, k, v, True)
    # causality: scramble the second half of K and V; the first half of the output must not move
    k_mod, v_mod = k.clone(), v.clone()
    k_mod[:, S // 2:] = rnd()[:, S // 2:]
    v_mod[:, S // 2:] = rnd()[:, S // 2:]
    o_mod, _, _, _ = _run_fwd(lib, L, st, q, k_mod, v_mod, True)
    torch.cuda.synchronize()
    assert torch.equal(o[:, :S // 2], o_mod[:, :S // 2])
    assert not torch.equal(o[:, S // 2:], o_mod[:, S // 2:])
    # linearity in V (same probabilities): O(v + v2) = O(v) + O(v2) up to bf16 rounding
    o2, _, _, _ = _run_fwd(lib, L, st, q, k, v2, True)
    o12, _, _, _ = _run_fwd(lib, L, st, q, k, (v.float() + v2.float()).to(torch.bfloat16), True)
    torch.cuda.synchronize()
    assert (o12.float() - (o.float() + o2.float())).abs().max().item() <= 0.06
    # backward: sum(dQ * Q) = sum(dK * K) per (batch, head); both equal sum(dS * S)
    dq, dk, dv = (torch.empty_like(q) for _ in range(3))

    def desc(t):
        a = lib.AttnTensor()
        a.ptr = t.data_ptr()
        a.sb, a.ss, a.sh = t.stride(0), t.stride(1), t.stride(2)
        return a

    o, lse, d, ts = _run_fwd(lib, L, st, q, k, v, True)
    ws = torch.empty(L.nbk_attention_bwd_workspace(C.byref(d)), dtype=torch.uint8, device="cuda")
    extra = [desc(t) for t in (g, dq, dk, dv)]
    lib.check(L.nbk_attention_bwd(C.byref(d), *[C.byref(t) for t in ts], None, C.c_void_p(lse.data_ptr()),
                                  *[C.byref(t) for t in extra], C.c_void_p(ws.data_ptr()), ws.numel(), st))
    torch.cuda.synchronize()
    a = (dq.float() * q.float()).sum(dim=(1, 3))
    b = (dk.float() * k.float()).sum(dim=(1, 3))
    scale = (dq.float().abs() * q.float().abs()).sum(dim=(1, 3))
    assert ((a - b).abs() <= 2e-2 * scale).all()
    # dV = P^T dO: with dO = 1 its sum over keys is the number of queries (rows of P sum to one)
    lib.check(L.nbk_attention_bwd(C.byref(d), *[C.byref(t) for t in ts], None, C.c_void_p(lse.data_ptr()),
                                  C.byref(desc(torch.ones_like(g))), *[C.byref(t) for t in extra[1:]],
                                  C.c_void_p(ws.data_ptr()), ws.numel(), st))
    torch.cuda.synchronize()
    total = dv.float().sum(dim=1)                                     # [B, H, hd]
    assert (total - S).abs().max().item() <= 2e-2 * S


def test_attention_strided_operands_from_different_buffers(hip):
    """q, k, v as slices of one packed [B, S, 3, H, hd] projection, the output written into a
    wider buffer: the strides the planner hands over inside multi-head attention."""
    from nabla_amd.backend import lib
    B, S, H, hd = 2, 256, 5, 64            # B * H = 10: not a multiple of the 8 XCDs
    rng = np.random.default_rng(9)
    packed = torch.tensor(rng.standard_normal((B, S, 3, H, hd)), dtype=torch.bfloat16)
    want = _reference(*(packed[:, :, i].double() for i in range(3)), torch.zeros(B, S, H, hd).double(), True)[0]
    pd = packed.cuda()
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    o, lse, _, _ = _run_fwd(lib, L, st, pd[:, :, 0], pd[:, :, 1], pd[:, :, 2], True)
    torch.cuda.synchronize()
    _close(o, want, "o from packed qkv")
