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
    tq, tk, tv, to, tg = (_heads(t, lib, False) for t in (qd, kd, vd, o, gd))
    print(f"attention fwd {shape} causal={causal}", flush=True)
    lib.check(L.nbk_attention_fwd(C.byref(d), C.byref(tq), C.byref(tk), C.byref(tv), C.byref(to),
                                  C.c_void_p(lse.data_ptr()), st))
    torch.cuda.synchronize()
    _close(o, want[0], "o")
    assert (lse.double().cpu() - want[1]).abs().max().item() < 2e-3
    # gradients land in heads-first storage ([B, H, S, hd]) to cover a second layout
    dq, dk, dv = (torch.full((B, H, S, hd), float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(3))
    tdq, tdk, tdv = (_heads(t, lib, True) for t in (dq, dk, dv))
    nbytes = L.nbk_attention_bwd_workspace(C.byref(d))
    assert nbytes == B * H * S * 4
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    print(f"attention bwd {shape} causal={causal}", flush=True)
    lib.check(L.nbk_attention_bwd(C.byref(d), C.byref(tq), C.byref(tk), C.byref(tv), C.byref(to),
                                  C.c_void_p(lse.data_ptr()), C.byref(tg), C.byref(tdq), C.byref(tdk),
                                  C.byref(tdv), C.c_void_p(ws.data_ptr()), nbytes, st))
    torch.cuda.synchronize()
    for got, w, name in ((dq, want[2], "dq"), (dk, want[3], "dk"), (dv, want[4], "dv")):
        _close(got.permute(0, 2, 1, 3), w, name)


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
                                          C.c_void_p(lse.data_ptr()), None))
    d = lib.AttnDesc()
    d.B, d.H, d.S, d.hd, d.scale, d.causal, d.dtype = 1, 1, 128, 64, 0.125, 1, 1
    bad = _heads(t, lib, False)
    bad.ss = 60
    with pytest.raises(ValueError, match="strides"):
        lib.check(L.nbk_attention_fwd(C.byref(d), C.byref(bad), C.byref(a), C.byref(a), C.byref(a),
                                      C.c_void_p(lse.data_ptr()), None))
    with pytest.raises(ValueError, match="workspace"):
        lib.check(L.nbk_attention_bwd(C.byref(d), *([C.byref(a)] * 4), C.c_void_p(lse.data_ptr()),
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
    scale = max(np.abs(g).max() for g in wg.values())
    for k in oc.C3_PARAMS:
        got = grads[k].numpy().astype(np.float64)
        assert np.abs(got - wg[k]).max() <= 3e-2 * max(np.abs(wg[k]).max(), 1e-2 * scale), k
