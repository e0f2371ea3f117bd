"""Optimizer steps over a list of parameters (nbk_adamw_multi / nbk_sgd_multi) through the C ABI,
against the formulas of nabla/nn/optim/functional.py:14-39 and 116-162 evaluated in float64 on
the same stored values.  fp32 results to 1e-5 of the tensor's largest value, bf16 results to
one rounding (2^-8 relative)."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

# one element; seven (a tail only); exactly one vector chunk of fp32 and of bf16; a chunk and a
# bit; many chunks with a ragged end
SIZES = [1, 7, 4096, 8192, 8193, 100003, 3 * 8192 + 5]


def _tensors(rng, n, tdt, misalign):
    """n groups (p, g, m, v) on the device; group `misalign` starts one element into its
    allocation, so none of its pointers is 16-byte aligned."""
    groups = []
    for i in range(n):
        size = SIZES[i % len(SIZES)] + (i // len(SIZES))
        off = 1 if i == misalign else 0

        def make(scale, positive=False):
            a = rng.standard_normal(size + off) * scale
            t = torch.tensor(np.abs(a) if positive else a, dtype=tdt).cuda()
            return t[off:]
        groups.append((make(0.5), make(1.0), make(0.1), make(0.01, positive=True)))
    return groups


def _table(lib, groups, outs):
    table = (lib.OptTensor * len(groups))()
    for t, (p, g, m, v), (po, mo, vo) in zip(table, groups, outs):
        t.param, t.grad, t.m, t.v = p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr()
        t.param_out = po.data_ptr()
        t.m_out = mo.data_ptr() if mo is not None else None
        t.v_out = vo.data_ptr() if vo is not None else None
        t.numel = p.numel()
    return table


def _close(got, want, dtype):
    got, want = got.double().cpu(), want.cpu()
    if dtype == "f32":
        scale = max(float(want.abs().max()), 1e-30)
        assert float((got - want).abs().max()) <= 1e-5 * scale
    else:  # one rounding to 8 mantissa bits (plus fp32 noise that can move a tie)
        err = (got - want).abs() - 2.0 ** -8 * want.abs()
        assert float(err.max()) <= 1e-6


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("counter", ["host", "device", "none"])
def test_adamw_multi_through_the_c_abi(hip, dtype, counter):
    from nabla_amd.backend import lib
    L = lib.load()
    rng = np.random.default_rng(40)
    tdt = torch.float32 if dtype == "f32" else torch.bfloat16
    n = 48 + 5  # more than one launch's table (NBK_OPT_MULTI_MAX entries)
    groups = _tensors(rng, n, tdt, misalign=3)
    in_place = counter == "device"
    if in_place:
        saved = [tuple(t.clone() for t in g) for g in groups]
        outs = [(p, m, v) for p, g, m, v in groups]
    else:
        saved = groups
        outs = [tuple(torch.full_like(p, float("nan")) for _ in range(3)) for p, *_ in groups]
    table = _table(lib, groups, outs)
    d = lib.AdamwDesc()
    lr, b1, b2, eps, wd, step = 1e-2, 0.9, 0.99, 1e-8, 0.03, 7
    d.lr, d.beta1, d.beta2, d.eps, d.weight_decay = lr, b1, b2, eps, wd
    d.log_beta1, d.log_beta2 = np.log(b1), np.log(b2)
    d.bias_correction = 0 if counter == "none" else 1
    d.c1, d.c2 = 1.0 - b1 ** step, 1.0 - b2 ** step
    d.step = None
    step_dev = torch.tensor([float(step)], dtype=torch.float32, device="cuda")
    if counter == "device":
        d.c1 = d.c2 = 0.0  # (not read when the counter is on the device)
        d.step = step_dev.data_ptr()
    d.dtype = 0 if dtype == "f32" else 1
    lib.check(L.nbk_adamw_multi(C.byref(d), table, n, C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    c1, c2 = (1.0, 1.0) if counter == "none" else (1.0 - b1 ** step, 1.0 - b2 ** step)
    for (p, g, m, v), (po, mo, vo) in zip(saved, outs):
        p, g, m, v = (t.double() for t in (p, g, m, v))
        m_t = m * b1 + g * (1 - b1)
        v_t = v * b2 + g * g * (1 - b2)
        want = p - lr * ((m_t / c1) / ((v_t / c2).sqrt() + eps) + wd * p)
        _close(mo, m_t, dtype)
        _close(vo, v_t, dtype)
        _close(po, want, dtype)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("momentum", [0.0, 0.9])
def test_sgd_multi_through_the_c_abi(hip, dtype, momentum):
    from nabla_amd.backend import lib
    L = lib.load()
    rng = np.random.default_rng(41)
    tdt = torch.float32 if dtype == "f32" else torch.bfloat16
    n = 9
    groups = _tensors(rng, n, tdt, misalign=5)
    outs = [(torch.full_like(p, float("nan")), torch.full_like(p, float("nan")) if momentum else None, None)
            for p, *_ in groups]
    table = _table(lib, groups, outs)
    d = lib.SgdDesc()
    d.lr, d.momentum, d.weight_decay = 0.05, momentum, 0.02
    d.dtype = 0 if dtype == "f32" else 1
    lib.check(L.nbk_sgd_multi(C.byref(d), table, n, C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    for (p, g, m, v), (po, mo, _) in zip(groups, outs):
        p, g, m = p.double(), g.double(), m.double()
        direction = g + 0.02 * p
        if momentum:
            direction = momentum * m + direction
            _close(mo, direction, dtype)
        _close(po, p - 0.05 * direction, dtype)


def test_update_list_rejects_bad_tables(hip):
    from nabla_amd.backend import lib
    L = lib.load()
    p = torch.zeros(16, device="cuda")
    table = _table(lib, [(p, p, p, p)], [(p, p, p)])
    d = lib.AdamwDesc()
    d.lr, d.beta1, d.beta2, d.eps, d.bias_correction, d.c1, d.c2 = 0.1, 0.9, 0.999, 1e-8, 1, 0.1, 0.001
    d.dtype = 3  # int32
    assert L.nbk_adamw_multi(C.byref(d), table, 1, None) != 0 and b"dtype" in L.nbk_last_error()
    d.dtype = 0
    table[0].numel = 0
    assert L.nbk_adamw_multi(C.byref(d), table, 1, None) != 0 and b"elements" in L.nbk_last_error()
    table[0].numel = 16
    table[0].v_out = None
    assert L.nbk_adamw_multi(C.byref(d), table, 1, None) != 0 and b"null" in L.nbk_last_error()
    d.c2 = 0.0
    table[0].v_out = p.data_ptr()
    assert L.nbk_adamw_multi(C.byref(d), table, 1, None) != 0 and b"bias" in L.nbk_last_error()
