"""GPU parity: the HIP path against the CPU oracle on the five benchmark
configurations (reduced sizes), full-size spot checks, the specialised row
kernels against the interpreter, data-movement / index kernels on awkward
shapes, user kernels, and ``compile`` on the device.

Tolerances: 1e-5 relative for fp32 work, 2e-2 for bf16, exact for integer results.  The
error of a tensor is max |got - want| over max |want| (one scale per tensor).
"""
import ctypes as C
from pathlib import Path

import numpy as np
import pytest
import torch

import nabla_amd as nb
from oracle import configs as oc

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5
BF16_TOL = 2e-2


def T(a, dtype=None):
    return nb.Tensor.constant(a, dtype=dtype)


def relerr(got, want, floor=0.0):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return np.abs(got - want).max() / max(np.abs(want).max(), floor, 1e-30)


# ---- C1 ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("batch,d_in,d_hidden,d_out", [(128, 784, 256, 10), (7, 33, 19, 3), (1, 8, 8, 1)])
def test_c1_mlp_step(hip, batch, d_in, d_hidden, d_out):
    t = oc.c1_inputs(batch, d_in, d_hidden, d_out, seed=4)
    t["b1"] = np.random.default_rng(1).uniform(-0.05, 0.05, t["b1"].shape).astype(np.float32)
    wl, wg = oc.c1_reference(**t)
    loss, grads = oc.c1_program(nb, oc.upload(nb, t))
    nb.realize_all(loss, *grads)
    assert abs(loss.item() - wl) <= F32_TOL * abs(wl) + 1e-9
    for g, w in zip(grads, wg):
        assert g.shape == w.shape
        assert relerr(g.numpy(), w) < F32_TOL


# ---- C2 ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("rows,cols", [(64, 512), (33, 1000), (5, 4108), (16, 8192), (3, 20000), (1, 1)])
def test_c2_chain_reduced(hip, rows, cols):
    t = oc.c2_inputs(rows, cols, seed=rows)
    wo, wg = oc.c2_reference(t["x"], t["y"])
    out, gx = oc.c2_program(nb, T(t["x"]), T(t["y"]))
    nb.realize_all(out, gx)
    assert relerr(out.numpy(), wo) < F32_TOL
    assert relerr(gx.numpy(), wg) < F32_TOL


def test_c2_full_size_rows_against_oracle(hip):
    """8192 x 8192 on the device; the oracle recomputes a sample of rows (rows are independent)."""
    t = oc.c2_inputs(8192, 8192, seed=0)
    out, gx = oc.c2_program(nb, T(t["x"]), T(t["y"]))
    nb.realize_all(out, gx)
    o, g = out.numpy(), gx.numpy()
    assert np.isfinite(o).all() and np.isfinite(g).all()
    rows = np.random.default_rng(0).choice(8192, 24, replace=False)
    rows = np.concatenate([rows, [0, 8191]])
    wo, wg = oc.c2_reference(t["x"][rows], t["y"][rows])
    assert relerr(o[rows], wo) < F32_TOL
    assert relerr(g[rows], wg) < F32_TOL
    # structure that holds for every row: the gradient vanishes exactly where relu(x) is flat
    # and p = x*y stays below the row maximum, and out >= 0
    assert (o >= 0).all()


def test_specialised_kernels_match_interpreter(hip):
    """The ahead-of-time row kernels and the interpreter run the same program:
    same operation order per element, so results agree to the last bit for the
    elementwise part and to reduction-order noise for sums."""
    from nabla_amd.backend import lib
    from nabla_amd.core import engine
    t = oc.c2_inputs(8192, 8192, seed=1)
    X, Y = T(t["x"]), T(t["y"])

    engine.clear_plan_cache()
    hip.force_interpreter = False
    out_s, gx_s = oc.c2_program(nb, X, Y)
    nb.realize_all(out_s, gx_s)
    L = lib.load()
    n_spec = 0
    for bound in engine._PLAN_CACHE.values():
        for call in bound.calls:
            if call[0] is L.nbk_rowprog_launch:
                n_spec += int(L.nbk_rowprog_is_specialized(C.byref(call[3])))
    assert n_spec >= 1, "the full-size C2 program must hit a specialised kernel"

    engine.clear_plan_cache()
    hip.force_interpreter = True
    try:
        out_i, gx_i = oc.c2_program(nb, X, Y)
        nb.realize_all(out_i, gx_i)
    finally:
        hip.force_interpreter = False
        engine.clear_plan_cache()
    np.testing.assert_allclose(out_s.numpy(), out_i.numpy(), rtol=2e-6, atol=0)
    np.testing.assert_allclose(gx_s.numpy(), gx_i.numpy(), rtol=2e-6, atol=1e-30)


def _row_program_kinds():
    """What nbk_rowprog_is_specialized says of every row program of the cached plans."""
    from nabla_amd.backend import lib
    from nabla_amd.core import engine
    L = lib.load()
    return [int(L.nbk_rowprog_is_specialized(C.byref(call[3])))
            for bound in engine._PLAN_CACHE.values() for call in bound.calls
            if call[0] is L.nbk_rowprog_launch]


def _hand_kernels_on():
    import os
    return os.environ.get("NBK_ROWPROG_HAND", "1") != "0" and os.environ.get("NBK_ROWPROG_INTERPRET", "0") != "1"


@pytest.mark.parametrize("rows,vocab", [(96, 32000), (700, 24000), (40, 20004), (33, 32768), (19, 16392),
                                        (300, 4104), (9, 32776), (64, 16384)])
def test_cross_entropy_over_long_rows(hip, rows, vocab):
    """Cross-entropy and its gradient over long bf16 rows against the interpreter and against
    float64.  Rows of whole 16-byte pieces, longer than the 16384 elements the planner stages in
    LDS as fp32 and up to 32768, take the hand-scheduled kernel (the row in registers: the
    benchmark's length, the longest and the shortest it takes, lengths whose last piece only some
    lanes hold); the others the generated kernels or the interpreter: the row staged in LDS, or
    re-read where its length is no multiple of 4."""
    from nabla_amd.backend import lib
    from nabla_amd.core import engine
    rng = np.random.default_rng(77)
    logits = (rng.standard_normal((rows, vocab)) * 3.0).astype(np.float32)
    labels = rng.integers(0, vocab, (rows,)).astype(np.int64)
    F = nb.nn.functional

    stored = torch.tensor(logits).to(torch.bfloat16).cuda()  # (logits that are bf16 in memory, as the decoder's)

    def run():
        x = nb.Tensor.from_dlpack(stored)
        lab = nb.Tensor.constant(labels)
        loss, g = nb.value_and_grad(lambda z: F.cross_entropy_loss(z, lab))(x)
        nb.realize_all(loss, g)
        return loss.item(), nb.cast(g, nb.DType.float32).numpy()

    engine.clear_plan_cache()
    loss_s, g_s = run()
    kinds = _row_program_kinds()
    assert max(kinds) >= 1, "the loss program of the decoder step must hit its specialised kernel"
    if _hand_kernels_on():
        assert (2 in kinds) == (vocab % 8 == 0 and 16384 < vocab <= 32768), kinds
    engine.clear_plan_cache()
    hip.force_interpreter = True
    try:
        loss_i, g_i = run()
    finally:
        hip.force_interpreter = False
        engine.clear_plan_cache()
    assert abs(loss_s - loss_i) <= 1e-5 * abs(loss_i)
    np.testing.assert_allclose(g_s, g_i, rtol=2e-2, atol=1e-8)
    x64 = torch.tensor(logits).to(torch.bfloat16).double().numpy()
    m = x64.max(1, keepdims=True)
    lse = m[:, 0] + np.log(np.exp(x64 - m).sum(1))
    want_loss = float((lse - x64[np.arange(rows), labels]).mean())
    p = np.exp(x64 - lse[:, None])
    p[np.arange(rows), labels] -= 1.0
    assert abs(loss_s - want_loss) <= 2.0 ** -8 * abs(want_loss)  # (the loss comes back in bf16)
    assert relerr(g_s, p / rows) <= BF16_TOL


def test_cross_entropy_over_rows_behind_two_leading_axes_and_a_row_pitch(hip):
    """The hand-scheduled kernel finds its rows through the program's leading strides: logits
    [batch, sequence, V] (two leading axes), and logits that are the first V columns of a wider
    buffer (a row pitch that is not the row length), against float64."""
    from nabla_amd.core import engine
    rng = np.random.default_rng(8)
    B, S, V, wide = 3, 7, 16392, 16392 + 40
    full = (rng.standard_normal((B, S, wide)) * 2.5).astype(np.float32)
    labels = rng.integers(0, V, (B, S)).astype(np.int64)
    stored = torch.tensor(full).to(torch.bfloat16).cuda()
    F = nb.nn.functional

    for sliced in (False, True):
        engine.clear_plan_cache()
        src = nb.Tensor.from_dlpack(stored if sliced else stored[:, :, :V].contiguous())
        lab = nb.Tensor.constant(labels)

        def loss_of(z):
            logits = nb.slice_tensor(z, [0, 0, 0], [B, S, V]) if sliced else z
            return F.cross_entropy_loss(logits, lab)

        loss, g = nb.value_and_grad(loss_of)(src)
        nb.realize_all(loss, g)
        if _hand_kernels_on():
            assert 2 in _row_program_kinds(), (sliced, _row_program_kinds())
        x64 = stored[:, :, :V].double().cpu().numpy().reshape(B * S, V)
        lse = torch.logsumexp(torch.tensor(x64), 1).numpy()
        want_loss = float((lse - x64[np.arange(B * S), labels.reshape(-1)]).sum() / B)
        p = np.exp(x64 - lse[:, None])
        p[np.arange(B * S), labels.reshape(-1)] -= 1.0
        got = nb.cast(g, nb.DType.float32).numpy()
        assert abs(loss.item() - want_loss) <= 2.0 ** -8 * abs(want_loss)
        assert relerr(got[:, :, :V].reshape(B * S, V), p / B) <= BF16_TOL
        if sliced:
            assert (got[:, :, V:] == 0).all()      # columns the loss never saw
    engine.clear_plan_cache()


def test_cross_entropy_rows_with_infinities_nans_and_labels_out_of_range(hip):
    """What the hand-scheduled cross-entropy kernel makes of rows the arithmetic breaks down on is
    what the interpreter makes of them: a row with +inf or NaN, or of nothing but -inf, is NaN in
    all of its gradient; -inf among finite logits has probability 0; a label outside [0, V)
    picks nothing (the row's gradient is its softmax)."""
    from nabla_amd.core import engine
    rows, vocab = 8, 16416
    rng = np.random.default_rng(5)
    logits = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    labels = rng.integers(0, vocab, (rows,)).astype(np.int64)
    labels[0], labels[1] = -1, vocab
    logits[2, 77] = np.inf
    logits[3, 16000] = np.nan
    logits[4, :] = -np.inf
    logits[5, 5:900] = -np.inf
    labels[5] = 3
    logits[6, labels[6]] = -np.inf          # the label's own logit: an infinite loss, finite gradient
    F = nb.nn.functional

    stored = torch.tensor(logits).to(torch.bfloat16).cuda()  # (logits that are bf16 in memory, as the decoder's)

    def run():
        x = nb.Tensor.from_dlpack(stored)
        lab = nb.Tensor.constant(labels)
        loss, g = nb.value_and_grad(lambda z: F.cross_entropy_loss(z, lab))(x)
        nb.realize_all(loss, g)
        return loss.item(), nb.cast(g, nb.DType.float32).numpy()

    engine.clear_plan_cache()
    loss_s, g_s = run()
    if _hand_kernels_on():
        assert 2 in _row_program_kinds()
    engine.clear_plan_cache()
    hip.force_interpreter = True
    try:
        loss_i, g_i = run()
    finally:
        hip.force_interpreter = False
        engine.clear_plan_cache()
    assert np.isnan(loss_s) and np.isnan(loss_i)
    assert np.array_equal(np.isnan(g_s), np.isnan(g_i))
    assert np.isnan(g_s[2]).all() and np.isnan(g_s[3]).all() and np.isnan(g_s[4]).all()
    fine = [0, 1, 5, 6, 7]
    np.testing.assert_allclose(g_s[fine], g_i[fine], rtol=2e-2, atol=1e-9)
    assert (g_s[5, 5:900] == 0).all()
    x64 = torch.tensor(logits[fine]).to(torch.bfloat16).double()
    p = torch.softmax(x64, 1).numpy()
    for i, r in enumerate(fine):
        if 0 <= labels[r] < vocab:
            p[i, labels[r]] -= 1.0
    assert relerr(g_s[fine], p / rows) <= BF16_TOL


# ---- C3 ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape,heads", [((2, 16, 32, 64), 4), ((2, 128, 256, 512), 4), ((1, 72, 64, 96), 2)])
def test_c3_block_fp32(hip, shape, heads):
    t = oc.c3_inputs(*shape, seed=0, bf16=False)
    wl, wg = oc.c3_reference(t, num_heads=heads)
    loss, grads = oc.c3_program(nb, oc.upload(nb, t), num_heads=heads)
    nb.realize_all(loss, *grads.values())
    assert abs(loss.item() - wl) < F32_TOL * abs(wl)
    for k in oc.C3_PARAMS:
        # bk's true gradient is zero (softmax is shift invariant): what comes back is the rounding
        # of sums that cancel, measured on the scale of bq's gradient (the same sums, uncancelled)
        floor = np.abs(wg["bq"]).max() if k == "bk" else 0.0
        assert relerr(grads[k].numpy(), wg[k], floor=floor) < F32_TOL, k


def test_c3_block_bf16(hip):
    t = oc.c3_inputs(2, 128, 256, 512, seed=1, bf16=True)
    wl, wg = oc.c3_reference(t, num_heads=4)
    loss, grads = oc.c3_program(nb, oc.upload(nb, t, dtype=nb.DType.bfloat16), num_heads=4)
    nb.realize_all(loss, *grads.values())
    assert loss.dtype == nb.DType.bfloat16
    assert abs(loss.item() - wl) < BF16_TOL * abs(wl)
    for k in oc.C3_PARAMS:
        assert grads[k].dtype == nb.DType.bfloat16
        floor = np.abs(wg["bq"]).max() if k == "bk" else 0.0  # (zero true gradient, see above)
        assert relerr(grads[k].numpy(), wg[k], floor=floor) < BF16_TOL, k


# ---- C4 ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("batch,hw,c", [(4, 8, (3, 8, 16, 32)), (3, 16, (3, 20, 24, 40)), (8, 32, (3, 64, 128, 256))])
def test_c4_cnn_step(hip, batch, hw, c):
    t = oc.c4_inputs(batch=batch, hw=hw, c=c, seed=2)
    wl, wg, wam, wlogits = oc.c4_reference(t)
    T4 = oc.upload(nb, t)
    loss, grads = oc.c4_program(nb, T4)
    logits = oc.c4_logits(nb, {k: T4[k] for k in oc.C4_PARAMS}, T4["img"])
    am = nb.argmax(logits, axis=-1)
    nb.realize_all(loss, am, logits, *grads.values())
    assert abs(loss.item() - wl) < F32_TOL * abs(wl)
    assert relerr(logits.numpy(), wlogits) < F32_TOL
    # the arg-max is an index and must be exact; the seeded inputs leave no two top logits
    # within fp32 noise of each other, so the oracle's index is the only right answer
    top2 = np.sort(wlogits, axis=-1)[:, -2:]
    assert ((top2[:, 1] - top2[:, 0]) > 1e-4 * np.abs(top2[:, 1])).all()
    np.testing.assert_array_equal(am.numpy(), wam)
    np.testing.assert_array_equal(am.numpy(), np.argmax(logits.numpy(), axis=-1))
    for k in oc.C4_PARAMS:
        assert relerr(grads[k].numpy(), wg[k]) < F32_TOL, k


# ---- C5 ------------------------------------------------------------------------------------------
def test_c5_lora_fp32(hip):
    t = oc.c5_inputs(layers=2, batch=2, seq=16, d_model=64, d_ff=128, vocab=97, rank=4, seed=0,
                     b_zero=False, bf16=False)
    wl, wg = oc.c5_reference(t, num_heads=4)
    loss, grads = oc.c5_program(nb, oc.upload(nb, t), num_heads=4)
    flat = [ad[k] for ad in grads for k in ("qA", "qB", "vA", "vB")]
    nb.realize_all(loss, *flat)
    assert abs(loss.item() - wl) < F32_TOL * abs(wl)
    for g, w in zip(flat, wg):
        assert relerr(g.numpy(), w) < F32_TOL


@pytest.mark.parametrize("seq,d_model,heads", [(64, 128, 4), (128, 256, 2), (256, 128, 2)])
def test_c5_lora_bf16(hip, seq, d_model, heads):
    """Head sizes 32 (attention as GEMM + softmax + GEMM), 128 and 64 (the fused kernels)."""
    t = oc.c5_inputs(layers=2, batch=2, seq=seq, d_model=d_model, d_ff=256, vocab=300, rank=8, seed=3,
                     b_zero=False, bf16=True)
    wl, wg = oc.c5_reference(t, num_heads=heads)
    loss, grads = oc.c5_program(nb, oc.upload(nb, t, dtype=nb.DType.bfloat16), num_heads=heads)
    flat = [ad[k] for ad in grads for k in ("qA", "qB", "vA", "vB")]
    nb.realize_all(loss, *flat)
    assert abs(loss.item() - wl) < BF16_TOL * abs(wl)
    for g, w in zip(flat, wg):
        assert relerr(g.numpy(), w) < BF16_TOL


# ---- movement, reductions and index kernels on awkward shapes ------------------------------------
@pytest.mark.parametrize("shape,perm", [((5, 7), (1, 0)), ((64, 96), (1, 0)), ((3, 33, 65), (2, 0, 1)),
                                        ((2, 4, 130, 64), (0, 2, 1, 3)), ((2, 3, 4, 5, 6), (4, 2, 0, 3, 1)),
                                        ((1, 1000), (1, 0))])
@pytest.mark.parametrize("dtype", ["f32", "bf16", "i32"])
def test_permute_copy_exact(hip, shape, perm, dtype):
    rng = np.random.default_rng(5)
    if dtype == "i32":
        a = rng.integers(-2 ** 31, 2 ** 31 - 1, shape).astype(np.int32)
        x = T(a)
    elif dtype == "bf16":
        a = oc.to_bf16_grid(rng.standard_normal(shape).astype(np.float32))
        x = T(a, dtype=nb.DType.bfloat16)
    else:
        a = rng.standard_normal(shape).astype(np.float32)
        x = T(a)
    # the trailing add forces a materialised copy in the permuted order
    y = nb.reshape(nb.permute(x, perm), (-1,))
    y.realize()
    np.testing.assert_array_equal(y.numpy(), np.transpose(a, perm).reshape(-1))


@pytest.mark.parametrize("shape,axis", [((4, 5, 6), 0), ((4, 5, 6), 1), ((2, 300, 7), 1), ((1000, 3), 0),
                                        ((8, 1, 16), 1), ((3, 4097), 1), ((70000,), 0), ((2, 3, 4, 5), 2)])
@pytest.mark.parametrize("kind", ["sum", "max", "min", "mean"])
def test_axis_reductions(hip, shape, axis, kind):
    rng = np.random.default_rng(6)
    a = rng.standard_normal(shape).astype(np.float32)
    fn = {"sum": nb.reduce_sum, "max": nb.reduce_max, "min": nb.reduce_min, "mean": nb.mean}[kind]
    want = {"sum": np.sum, "max": np.max, "min": np.min, "mean": np.mean}[kind](a.astype(np.float64), axis=axis)
    got = fn(T(a), axis=axis).numpy()
    assert got.shape == want.shape
    if kind in ("max", "min"):
        np.testing.assert_array_equal(got, want.astype(np.float32))
    else:
        absum = np.abs(a).astype(np.float64).sum(axis=axis) / (a.shape[axis] if kind == "mean" else 1)
        assert (np.abs(got - want) <= 1e-6 * absum + 1e-30).all()


def test_argmax_ties_and_nan(hip):
    a = np.zeros((6, 300), np.float32)
    a[0, [5, 9, 250]] = 3.0          # first maximum wins
    a[1, :] = -1.0                   # all equal -> 0
    a[2, 299] = 1.0
    a[3, 17] = np.inf
    a[4, [100, 200]] = [2.0, np.nan]  # NaN counts as the maximum, as in numpy/torch
    a[5, 0] = -np.inf
    got = nb.argmax(T(a), axis=-1).numpy()
    np.testing.assert_array_equal(got, torch.from_numpy(a).argmax(-1).numpy())
    got0 = nb.argmax(T(a), axis=0).numpy()
    np.testing.assert_array_equal(got0, torch.from_numpy(a).argmax(0).numpy())
    assert got.dtype == np.int64


def test_argmin_ties_nan_and_axes(hip):
    """argmin (nabla/ops/reduction.py:739-811, 880-896): int64, the first minimum on ties, a NaN
    counts as the minimum (numpy / torch convention), along the last, a middle and the leading
    axis, with and without keepdims, flattened for axis=None, f32 and bf16 -- exact."""
    a = np.ones((7, 300), np.float32)
    a[0, [5, 9, 250]] = -3.0          # first minimum wins
    a[1, :] = 2.0                     # all equal -> 0
    a[2, 299] = -1.0                  # last column
    a[3, 17] = -np.inf
    a[4, [100, 200]] = [-2.0, np.nan]  # NaN counts as the minimum
    a[5, 0] = np.inf
    a[6, [64, 128]] = [np.nan, np.nan]  # two NaNs in different lanes' strides: the first one
    want = torch.from_numpy(a).argmin(-1).numpy()
    np.testing.assert_array_equal(want, np.argmin(a, -1))
    got = nb.argmin(T(a), axis=-1).numpy()
    assert got.dtype == np.int64
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(nb.argmin(T(a), axis=0).numpy(), np.argmin(a, 0))
    np.testing.assert_array_equal(nb.argmin(T(a), axis=-1, keepdims=True).numpy(), want[:, None])
    rng = np.random.default_rng(21)
    b = rng.standard_normal((5, 33, 70)).astype(np.float32)
    for axis in (0, 1, 2, -2):
        np.testing.assert_array_equal(nb.argmin(T(b), axis=axis).numpy(), np.argmin(b, axis))
        np.testing.assert_array_equal(nb.argmax(T(b), axis=axis).numpy(), np.argmax(b, axis))
    np.testing.assert_array_equal(nb.argmin(T(b), axis=None).numpy(), np.argmin(b))
    # bf16 rounds many entries onto one value: ties resolve to the lowest index there too
    bb = torch.from_numpy(b).to(torch.bfloat16)
    got16 = nb.argmin(T(b).cast(nb.DType.bfloat16), axis=-1).numpy()
    np.testing.assert_array_equal(got16, bb.float().argmin(-1).numpy())
    # argmin(x) is argmax(-x) wherever no NaN is involved
    np.testing.assert_array_equal(nb.argmin(T(b), axis=1).numpy(), nb.argmax(-T(b), axis=1).numpy())


@pytest.mark.parametrize("dtype,tol", [("f32", F32_TOL), ("bf16", BF16_TOL)])
def test_sigmoid_value_and_gradient(hip, dtype, tol):
    """sigmoid (nabla/ops/unary.py SigmoidOp; derivative out * (1 - out)) against float64:
    values over the range where fp32 saturates either way, and the gradient under a random
    cotangent; sigmoid(x) + sigmoid(-x) = 1 as the invariant."""
    rng = np.random.default_rng(22)
    x = np.concatenate([rng.standard_normal(4000) * 3.0, np.linspace(-100.0, 100.0, 96)]).astype(np.float32)
    x = x.reshape(64, 64)
    w = rng.standard_normal(x.shape).astype(np.float32)
    dt = nb.DType.bfloat16 if dtype == "bf16" else nb.DType.float32
    if dtype == "bf16":
        x = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
        w = torch.from_numpy(w).to(torch.bfloat16).float().numpy()
    X, W = T(x).cast(dt), T(w).cast(dt)
    y = nb.sigmoid(X)
    g = nb.grad(lambda t: nb.reduce_sum(nb.sigmoid(t) * W))(X)
    s = nb.sigmoid(X) + nb.sigmoid(-X)
    nb.realize_all(y, g, s)
    x64 = x.astype(np.float64)
    want = np.where(x64 >= 0, 1.0 / (1.0 + np.exp(-np.abs(x64))), np.exp(-np.abs(x64)) / (1.0 + np.exp(-np.abs(x64))))
    tx = torch.tensor(x64, requires_grad=True)
    (torch.sigmoid(tx) * torch.tensor(w, dtype=torch.float64)).sum().backward()
    yn = y.cast(nb.DType.float32).numpy().astype(np.float64)
    gn = g.cast(nb.DType.float32).numpy().astype(np.float64)
    assert np.isfinite(yn).all() and np.isfinite(gn).all()
    assert relerr(yn, want) < tol
    assert relerr(gn, tx.grad.numpy()) < tol
    assert np.abs(s.cast(nb.DType.float32).numpy() - 1.0).max() < (2e-2 if dtype == "bf16" else 1e-6)
    if dtype == "f32":
        # elementwise, not only against the tensor's largest entry
        assert (np.abs(yn - want) <= 1e-6 * want + 1e-37).all()


def test_gather_rows_and_out_of_range(hip):
    rng = np.random.default_rng(7)
    table = rng.standard_normal((50, 24)).astype(np.float32)
    idx = rng.integers(0, 50, (3, 11)).astype(np.int64)
    got = nb.gather(T(table), T(idx), axis=0).numpy()
    np.testing.assert_array_equal(got, table[idx])
    idx32 = idx.astype(np.int32)
    np.testing.assert_array_equal(nb.gather(T(table), T(idx32), axis=0).numpy(), table[idx32])
    bad = idx.copy()
    bad[1, 2] = 50
    with pytest.raises(IndexError):
        nb.gather(T(table), T(bad), axis=0).numpy()
    # the flag is cleared by the failed call
    np.testing.assert_array_equal(nb.gather(T(table), T(idx), axis=0).numpy(), table[idx])


def test_integer_and_bool_elementwise_exact(hip):
    rng = np.random.default_rng(8)
    a = rng.integers(-1000, 1000, (17, 129)).astype(np.int32)
    b = rng.integers(-1000, 1000, (17, 129)).astype(np.int32)
    np.testing.assert_array_equal((T(a) + T(b)).numpy(), a + b)
    np.testing.assert_array_equal((T(a) * T(b)).numpy(), a * b)
    np.testing.assert_array_equal(nb.greater(T(a), T(b)).numpy(), a > b)
    np.testing.assert_array_equal(nb.where(nb.greater(T(a), T(b)), T(a), T(b)).numpy(), np.maximum(a, b))
    np.testing.assert_array_equal(nb.reduce_sum(T(a), axis=1).numpy(), a.sum(1))


def test_integers_above_2_pow_24_are_exact(hip):
    """The same cases as the emulator-backed host test, on the kernels."""
    from integer_cases import check_large_integers
    check_large_integers(nb)


def test_int64_beyond_the_int32_range_is_exact(hip):
    """Arithmetic, comparisons, selects and casts on int64 values outside the int32 range run in
    the 64-bit integer kernel; the label-against-class-index comparison stays fused and exact."""
    from integer_cases import check_int64_beyond_int32
    check_int64_beyond_int32(nb)


def test_tensors_without_elements_and_domain_edges(hip):
    from edge_cases import check_empty_tensors, check_log1p_and_atanh_at_the_edges
    check_empty_tensors(nb)
    check_log1p_and_atanh_at_the_edges(nb)


def test_slice_pad_concat_exact(hip):
    rng = np.random.default_rng(9)
    a = rng.standard_normal((6, 10, 12)).astype(np.float32)
    b = rng.standard_normal((6, 3, 12)).astype(np.float32)
    x, y = T(a), T(b)
    np.testing.assert_array_equal(x[1:5, ::1, 2:9].numpy(), a[1:5, :, 2:9])
    np.testing.assert_array_equal(nb.concatenate([x, y], axis=1).numpy(), np.concatenate([a, b], 1))
    g = nb.grad(lambda x: nb.reduce_sum(x[1:5, 2:4, 3:8] * 2.0))(x)
    want = np.zeros_like(a)
    want[1:5, 2:4, 3:8] = 2.0
    np.testing.assert_array_equal(g.numpy(), want)


@pytest.mark.parametrize("cfg", [
    dict(n=2, h=9, w=11, ci=3, co=5, k=3, stride=(1, 1), pad=(1, 1, 1, 1), dil=(1, 1)),
    dict(n=1, h=12, w=12, ci=4, co=6, k=3, stride=(2, 2), pad=(0, 1, 2, 0), dil=(1, 1)),
    dict(n=2, h=14, w=10, ci=2, co=4, k=3, stride=(1, 2), pad=(2, 2, 2, 2), dil=(1, 1)),
    dict(n=3, h=8, w=8, ci=16, co=8, k=1, stride=(1, 1), pad=(0, 0, 0, 0), dil=(1, 1)),
])
def test_conv2d_forward_and_grads(hip, cfg):
    from oracle import ops as O
    rng = np.random.default_rng(10)
    x = rng.standard_normal((cfg["n"], cfg["h"], cfg["w"], cfg["ci"])).astype(np.float32)
    w = rng.standard_normal((cfg["k"], cfg["k"], cfg["ci"], cfg["co"])).astype(np.float32)
    kw = dict(stride=cfg["stride"], padding=cfg["pad"])
    X, W = O.V(x.astype(np.float64)), O.V(w.astype(np.float64))
    out = O.conv2d(X, W, **kw)
    wgx, wgw = O.grad_of(O.reduce_sum(out * out), [X, W])
    f = lambda x, w: nb.reduce_sum(nb.conv2d(x, w, **kw) ** 2)
    got = nb.conv2d(T(x), T(w), **kw)
    gx, gw = nb.grad(f, argnums=(0, 1))(T(x), T(w))
    assert relerr(got.numpy(), out.a) < F32_TOL
    assert relerr(gx.numpy(), wgx) < F32_TOL
    assert relerr(gw.numpy(), wgw) < F32_TOL


@pytest.mark.parametrize("cfg", [
    dict(xs=(1, 4, 5, 2), ws=(3, 2, 6, 2), stride=(2, 1), pad=(1, 0, 1, 0)),     # the reference's vjp case
    dict(xs=(1, 4, 4, 2), ws=(3, 3, 5, 2), stride=(1, 1), pad=(1, 1, 1, 1)),     # ... and its jvp case
    dict(xs=(4, 16, 16, 64), ws=(4, 4, 32, 64), stride=(2, 2), pad=(1, 1, 1, 1)),  # a decoder upsampling layer
])
def test_conv2d_transpose_forward_and_grads(hip, cfg):
    """conv2d_transpose (the dgrad kernel behind a public op), its bias and all three gradients
    against the float64 oracle."""
    from oracle import ops as O
    rng = np.random.default_rng(12)
    x = rng.standard_normal(cfg["xs"]).astype(np.float32)
    w = (rng.standard_normal(cfg["ws"]) / np.sqrt(cfg["ws"][0] * cfg["ws"][1] * cfg["ws"][3])).astype(np.float32)
    b = rng.standard_normal(cfg["ws"][2]).astype(np.float32)
    kw = dict(stride=cfg["stride"], padding=cfg["pad"])
    X, W, B = (O.V(a.astype(np.float64)) for a in (x, w, b))
    out = O.conv2d_transpose(X, W, B, **kw)
    want = O.grad_of(O.reduce_sum(out * out), [X, W, B])
    f = lambda x, w, b: nb.reduce_sum(nb.conv2d_transpose(x, w, bias=b, **kw) ** 2)
    got = nb.conv2d_transpose(T(x), T(w), bias=T(b), **kw)
    assert tuple(got.shape) == out.a.shape
    assert relerr(got.numpy(), out.a) < F32_TOL
    for g, wg in zip(nb.grad(f, argnums=(0, 1, 2))(T(x), T(w), T(b)), want):
        assert relerr(g.numpy(), wg) < F32_TOL


# ---- user kernels ---------------------------------------------------------------------------------
class AddOneCustomOp(nb.ops.UnaryOperation):
    """Same shape as the reference's example op (tests/mojo/op.py:15-27)."""

    @property
    def name(self) -> str:
        return "my_kernel"

    def kernel(self, args, kwargs):
        kernel_dir = Path(__file__).parent / "custom_kernels"
        x = args[0]
        return [nb.ops.call_custom_kernel("my_kernel", kernel_dir, x, x.type)]


def test_custom_kernel_op(hip):
    a = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    y = AddOneCustomOp()([T(a)], {})[0]
    np.testing.assert_array_equal(y.numpy(), a + 1)
    # composes with built-in ops inside one graph
    z = nb.reduce_sum(AddOneCustomOp()([T(a) * 2.0], {})[0], axis=-1)
    np.testing.assert_array_equal(z.numpy(), (a * 2 + 1).sum(-1))


def test_custom_kernel_missing_library_is_an_error(hip):
    class Broken(AddOneCustomOp):
        def kernel(self, args, kwargs):
            return [nb.ops.call_custom_kernel("nope", Path(__file__).parent / "golden", args[0], args[0].type)]

    with pytest.raises(RuntimeError, match="no built kernel library"):
        Broken()([T(np.zeros(4, np.float32))], {})[0].numpy()


# ---- compile --------------------------------------------------------------------------------------
def test_compiled_train_step_on_device(hip):
    t = oc.c1_inputs(32, 48, 24, 5, seed=11)
    params = {k: T(t[k]) for k in ("W1", "b1", "W2", "b2")}
    x = T(t["x"])

    def step(params, x):
        def loss_fn(p):
            return nb.mean(nb.relu(x @ p["W1"] + p["b1"]) @ p["W2"] + p["b2"])
        loss, g = nb.value_and_grad(loss_fn)(params)
        return loss, {k: params[k] - 0.1 * g[k] for k in params}

    cstep = nb.compile(step)
    ref = {k: t[k].astype(np.float64) for k in params}
    p = params
    for _ in range(3):
        loss, p = cstep(p, x)
        wl, wg = oc.c1_reference(t["x"], *[ref[k].astype(np.float32) for k in ("W1", "b1", "W2", "b2")])
        assert abs(loss.item() - wl) <= F32_TOL * abs(wl) + 1e-8
        for k, g in zip(("W1", "b1", "W2", "b2"), wg):
            ref[k] = ref[k] - 0.1 * g
    assert cstep.stats.misses == 1 and cstep.stats.hits == 2
    for k in params:
        assert relerr(p[k].numpy(), ref[k]) < F32_TOL


def test_compiled_step_with_a_dynamic_batch_on_device(hip):
    """`compile(dynamic_dims={4: {0: "batch"}})` (nabla/transforms/compile.py:207-268, 508-555;
    the key counts the tensor leaves of the flattened arguments: four parameters, then x): one
    signature serves every batch size.  The MLP step is called with three batch sizes, back to
    the first, and repeatedly on one size (so that a replayed recording is among the calls);
    every loss and gradient is checked against the oracle at that size, and the statistics
    show a single miss."""
    from nabla_amd.core import engine
    t0 = oc.c1_inputs(8, 48, 24, 5, seed=12)
    t0["b1"] = np.random.default_rng(3).uniform(-0.05, 0.05, t0["b1"].shape).astype(np.float32)
    names = ("W1", "b1", "W2", "b2")
    params = {k: T(t0[k]) for k in names}

    @nb.compile(dynamic_dims={4: {0: "batch"}})
    def step(p, x):
        return nb.value_and_grad(lambda q: nb.mean(nb.relu(x @ q["W1"] + q["b1"]) @ q["W2"] + q["b2"]))(p)

    rng = np.random.default_rng(13)
    xs = {n: rng.uniform(-0.05, 0.05, (n, 48)).astype(np.float32) for n in (8, 37, 128, 1)}
    dev = {n: T(a) for n, a in xs.items()}
    plans_before = len(engine._PLAN_CACHE)
    calls = 0
    for n in (8, 37, 128, 8, 8, 8, 37, 1, 128, 37):
        loss, g = step(params, dev[n])
        calls += 1
        wl, wg = oc.c1_reference(xs[n], *[t0[k] for k in names])
        assert abs(loss.item() - wl) <= F32_TOL * abs(wl) + 1e-9, n
        for k, w in zip(names, wg):
            assert g[k].shape == w.shape
            assert relerr(g[k].numpy(), w) < F32_TOL, (n, k)
        del loss, g
    assert step.stats.misses == 1 and step.stats.hits == calls - 1, step.stats
    # one launch plan per batch size that was seen, not per call
    assert len(engine._PLAN_CACHE) - plans_before <= len(xs)


# ---- optimizer step (next row after the hot path: nn/optim) ---------------------------------------
@pytest.mark.parametrize("dtype,tol", [("f32", 2e-5), ("bf16", 2e-2)])
def test_adamw_and_sgd_steps_on_device(hip, dtype, tol):
    from nabla_amd.nn import optim
    rng = np.random.default_rng(21)
    shapes = {"w1": (256, 384), "b1": (1, 384), "w2": (384, 10)}
    p0 = {k: rng.standard_normal(s).astype(np.float32) * 0.1 for k, s in shapes.items()}
    dt = None if dtype == "f32" else nb.DType.bfloat16
    if dtype == "bf16":
        p0 = {k: oc.to_bf16_grid(v) for k, v in p0.items()}
    up = lambda tree: {k: T(v, dtype=dt) for k, v in tree.items()}
    tp = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in p0.items()}
    t_adam = torch.optim.AdamW(list(tp.values()), lr=1e-2, betas=(0.9, 0.99), weight_decay=0.02)
    adam = optim.AdamW(up(p0), lr=1e-2, betas=(0.9, 0.99), weight_decay=0.02)
    sp = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in p0.items()}
    t_sgd = torch.optim.SGD(list(sp.values()), lr=0.05, momentum=0.9, weight_decay=0.01)
    sgd = optim.SGD(up(p0), lr=0.05, momentum=0.9, weight_decay=0.01)
    for _ in range(3):
        g = {k: rng.standard_normal(s).astype(np.float32) for k, s in shapes.items()}
        if dtype == "bf16":
            g = {k: oc.to_bf16_grid(v) for k, v in g.items()}
        for k in shapes:
            tp[k].grad = torch.tensor(g[k], dtype=torch.float64)
            sp[k].grad = torch.tensor(g[k], dtype=torch.float64)
        t_adam.step()
        t_sgd.step()
        a_new = adam.step(up(g))
        s_new = sgd.step(up(g))
        if dtype == "f32":
            for k in shapes:
                assert relerr(a_new[k].numpy(), tp[k].detach().numpy()) < tol, k
                assert relerr(s_new[k].numpy(), sp[k].detach().numpy()) < tol, k
    # bf16 parameters accumulate one rounding per step: compare after the last step only
    for k in shapes:
        assert relerr(a_new[k].numpy(), tp[k].detach().numpy()) < tol * 3, k
        assert relerr(s_new[k].numpy(), sp[k].detach().numpy()) < tol * 3, k


# ---- replay of a repeated step as a HIP graph -----------------------------------------------------
def test_graph_replay_matches_eager_every_time(hip):
    """A compiled step called again on the same buffers is recorded once and replayed; every
    replay is checked against the oracle, with unrelated eager work and synchronisation between
    the replays, and a call on new buffers falls back to plain launches.  The plan owns the
    slabs its results live in, so the replay does not depend on what the allocator hands out:
    the caller just lets go of the previous results, as a training loop does."""
    if not hip.use_graphs:
        pytest.skip("graph replay is switched off (NBK_GRAPHS=0): nothing to replay")
    t = oc.c1_inputs(64, 96, 48, 10, seed=31)
    t["b1"] = np.random.default_rng(2).uniform(-0.05, 0.05, t["b1"].shape).astype(np.float32)
    wl, wg = oc.c1_reference(**t)
    dev = oc.upload(nb, t)
    step = nb.compile(lambda d: nb.workloads.c1_step(d))
    before = hip.graph_replays
    other = T(np.arange(12, dtype=np.float32))
    for it in range(7):
        loss, grads = step(dev)
        got = [loss.numpy()] + [g.numpy() for g in grads]
        assert abs(got[0] - wl) <= F32_TOL * abs(wl) + 1e-9, it
        for g, w in zip(got[1:], wg):
            assert relerr(g, w) < F32_TOL, it
        # unrelated work between replays (allocations of all sizes included)
        np.testing.assert_array_equal((other * 2.0 + float(it)).numpy(), np.arange(12) * 2.0 + it)
        junk = torch.empty((it + 1) << 20, dtype=torch.uint8, device="cuda")
        del junk
    assert hip.graph_replays - before >= 3, "the repeated step was not replayed as a graph"
    # new input buffers: pointers differ, the recording must not be used
    t2 = oc.c1_inputs(64, 96, 48, 10, seed=32)
    wl2, wg2 = oc.c1_reference(**t2)
    loss, grads = step(oc.upload(nb, t2))
    assert abs(loss.item() - wl2) <= F32_TOL * abs(wl2) + 1e-9
    for g, w in zip(grads, wg2):
        assert relerr(g.numpy(), w) < F32_TOL


def test_kept_losses_stay_valid_and_do_not_pin_the_gradients(hip):
    """A loop that keeps every loss tensor: each kept loss still reads its own step's value
    after later steps ran (no slab is written while something refers to it), the gradients of
    all those steps share a few recycled slabs instead of one allocation per kept loss, and
    the step is still replayed as a graph once the inputs repeat."""
    rng = np.random.default_rng(33)
    w = rng.standard_normal((256, 384)).astype(np.float32)
    W = T(w)

    @nb.compile
    def step(W, x):
        return nb.value_and_grad(lambda W: nb.mean(nb.tanh(x @ W) ** 2))(W)

    xs = [rng.standard_normal((32, 256)).astype(np.float32) for _ in range(9)]
    want = [float(np.mean(np.tanh(x.astype(np.float64) @ w.astype(np.float64)) ** 2)) for x in xs]
    kept, grad_ptrs = [], set()
    for x in xs:
        loss, g = step(W, T(x))
        kept.append(loss)
        grad_ptrs.add(g._impl._buffer.untyped_storage().data_ptr())
        del g
    for loss, wl in zip(kept, want):
        assert abs(loss.item() - wl) <= F32_TOL * abs(wl)
    assert len({l._impl._buffer.untyped_storage().data_ptr() for l in kept}) == len(kept)
    assert len(grad_ptrs) <= 3, "dropped gradients must be recycled although the losses are kept"
    # the same inputs again and again, still keeping the losses: replayed, values unchanged
    X = T(xs[0])
    before = hip.graph_replays
    for _ in range(6):
        loss, g = step(W, X)
        kept.append(loss)
        del g
    if hip.use_graphs:  # (NBK_GRAPHS=0: plain launches, the values are checked all the same)
        assert hip.graph_replays - before >= 3
    for loss in kept[-6:]:
        assert abs(loss.item() - want[0]) <= F32_TOL * abs(want[0])


# ---- avg_pool2d, silu -------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("kernel,stride,padding", [((2, 2), None, 0), ((3, 3), (2, 1), 1),
                                                   ((3, 2), (1, 2), (1, 0, 2, 1))])
def test_avg_pool2d_and_silu_on_device(hip, dtype, kernel, stride, padding):
    from oracle import ops as O
    rng = np.random.default_rng(31)
    x = rng.standard_normal((4, 17, 12, 24)).astype(np.float32)
    dt = nb.DType.float32 if dtype == "f32" else nb.DType.bfloat16
    if dtype == "bf16":
        import torch
        x = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    tol = 2e-5 if dtype == "f32" else 2e-2
    pad4 = (padding,) * 4 if isinstance(padding, int) else padding
    X = nb.Tensor.constant(x, dtype=dt)
    vx = O.V(x.astype(np.float64))
    want = O.avg_pool2d(O.silu(vx), kernel, stride, pad4)
    g = rng.standard_normal(want.a.shape).astype(np.float32)
    (wg,) = O.grad_of(O.reduce_sum(want * O.V(g.astype(np.float64))), [vx])

    def f(t):
        y = nb.avg_pool2d(nb.silu(t), kernel_size=kernel, stride=stride, padding=padding)
        return nb.reduce_sum(nb.cast(y, nb.DType.float32) * nb.Tensor.constant(g))

    y = nb.avg_pool2d(nb.silu(X), kernel_size=kernel, stride=stride, padding=padding)
    got = nb.cast(y, nb.DType.float32).numpy()
    assert np.abs(got - want.a).max() <= tol * max(np.abs(want.a).max(), 1.0)
    gx = nb.cast(nb.grad(f)(X), nb.DType.float32).numpy()
    assert np.abs(gx - wg).max() <= tol * max(np.abs(wg).max(), 1.0)


# ---- forward mode -----------------------------------------------------------------------------------
def test_jvp_on_device_against_oracle_central_differences(hip):
    """jvp of a small CNN + MLP head on the device: the tangent equals the float64 oracle's
    central difference along the same direction, and <J v, u> = <v, J^T u> against vjp."""
    from oracle import ops as O
    rng = np.random.default_rng(43)
    shapes = [(2, 8, 8, 3), (3, 3, 3, 8), (8,), (8, 5)]
    xs = [rng.standard_normal(s) for s in shapes]
    vs = [rng.standard_normal(s) for s in shapes]

    def fn(x, w, b, wl):
        h = nb.max_pool2d(nb.relu(nb.conv2d(x, w, padding=1, bias=b)), kernel_size=2)
        return nb.softmax(nb.mean(h, axis=(1, 2)) @ wl, axis=-1)

    def ofn(x, w, b, wl):
        h = O.max_pool2d(O.relu(O.conv2d(x, w, b, (1, 1), (1, 1, 1, 1))), (2, 2))
        return O.softmax(O.matmul(O.mean(h, axis=(1, 2)), wl), axis=-1)

    T = lambda a: nb.Tensor.constant(a.astype(np.float32))
    out, tan = nb.jvp(fn, tuple(T(x) for x in xs), tuple(T(v) for v in vs))
    eps = 1e-6
    p = ofn(*[O.V(x + eps * v) for x, v in zip(xs, vs)]).a
    m = ofn(*[O.V(x - eps * v) for x, v in zip(xs, vs)]).a
    want = (p - m) / (2 * eps)
    np.testing.assert_allclose(out.numpy(), ofn(*[O.V(x) for x in xs]).a, rtol=2e-5, atol=2e-6)
    assert np.abs(tan.numpy() - want).max() <= 2e-4 * max(np.abs(want).max(), 1e-3)
    u = rng.standard_normal(out.shape)
    _, pull = nb.vjp(fn, *[T(x) for x in xs])
    gs = pull(T(u))
    lhs = float((tan.numpy().astype(np.float64) * u).sum())
    rhs = sum(float((g.numpy().astype(np.float64) * v).sum()) for g, v in zip(gs, vs))
    assert abs(lhs - rhs) <= 2e-4 * max(abs(lhs), abs(rhs), 1e-3)


@pytest.mark.parametrize("jac", ["rev", "fwd"])
def test_jacobians_on_device_against_torch_cpu(hip, jac):
    """jacrev / jacfwd of softmax(gelu(x @ w)) on the device against torch's CPU Jacobian in
    float64, and the Hessian of sum(x^3) (forward over reverse) against diag(6x)."""
    rng = np.random.default_rng(47)
    x, w = rng.standard_normal((3, 5)), rng.standard_normal((5, 4))
    J = nb.jacrev if jac == "rev" else nb.jacfwd
    got = J(lambda a, b: nb.softmax(nb.gelu(nb.matmul(a, b)) * 0.7, axis=-1), argnums=(0, 1))(
        T(x.astype(np.float32)), T(w.astype(np.float32)))
    want = torch.autograd.functional.jacobian(
        lambda a, b: torch.softmax(torch.nn.functional.gelu(a @ b) * 0.7, dim=-1),
        (torch.tensor(x), torch.tensor(w)))
    for g, wnt in zip(got, want):
        assert g.numpy().shape == tuple(wnt.shape)
        assert relerr(g.numpy(), wnt.numpy()) <= 1e-5
    v = rng.standard_normal(6).astype(np.float32)
    h = J(nb.grad(lambda t: nb.reduce_sum(t * t * t)))(T(v)).numpy()
    assert relerr(h, np.diag(6.0 * v.astype(np.float64))) <= F32_TOL


def test_vmap_per_example_gradients_on_device(hip):
    """vmap(grad(loss)) over 16 examples of a small MLP loss on the device against the float64
    closed form, and grad(sum(vmap(loss))) against the sum of the per-example gradients."""
    rng = np.random.default_rng(49)
    W, X = rng.standard_normal((24, 8)), rng.standard_normal((16, 24))
    loss = lambda w, x: nb.reduce_sum(nb.tanh(x @ w) ** 2)
    got = nb.vmap(nb.grad(loss), in_axes=(None, 0))(T(W.astype(np.float32)), T(X.astype(np.float32)))
    th = np.tanh(X @ W)
    want = np.einsum("bi,bj->bij", X, 2 * th * (1 - th ** 2))
    assert got.numpy().shape == want.shape
    assert relerr(got.numpy(), want) <= F32_TOL
    total = nb.grad(lambda w: nb.reduce_sum(nb.vmap(loss, in_axes=(None, 0))(w, T(X.astype(np.float32)))))(
        T(W.astype(np.float32)))
    assert relerr(total.numpy(), want.sum(axis=0)) <= F32_TOL


def test_vmap_batched_per_example_gradients_of_a_block_on_device(hip):
    """Per-example gradients of a two-layer block with layer norm over 256 examples: vmap runs
    the function once on the batch (its launches do not grow with the batch), and the result is
    the float64 closed form per example, computed by looping in numpy."""
    from nabla_amd import config
    from nabla_amd.core import engine
    if not config.VMAP_BATCHED:
        pytest.skip("batched vmap is switched off (NBK_VMAP_BATCHED=0): the element-by-element map "
                    "is covered by test_vmap_per_example_gradients_on_device")
    rng = np.random.default_rng(50)
    n, s, d, h = 256, 8, 32, 64
    X, Y = rng.standard_normal((n, s, d)), rng.standard_normal((n, s, d))
    W1, W2 = rng.standard_normal((d, h)) / np.sqrt(d), rng.standard_normal((h, d)) / np.sqrt(h)
    F = nb.nn.functional
    calls = []

    def loss(p, x, y):
        calls.append(1)
        z = F.layer_norm(x, None, None)
        return nb.mean((nb.tanh(z @ p["w1"]) @ p["w2"] - y) ** 2.0)

    f32 = lambda a: T(a.astype(np.float32))
    engine.clear_plan_cache()
    g = nb.vmap(nb.grad(loss), in_axes=(None, 0, 0))({"w1": f32(W1), "w2": f32(W2)}, f32(X), f32(Y))
    got = {k: v.numpy() for k, v in g.items()}
    steps = sum(len(bp.plan.steps) for bp in engine._PLAN_CACHE.values())
    engine.clear_plan_cache()
    assert len(calls) == 1 and steps < 40
    mu, var = X.mean(-1, keepdims=True), X.var(-1, keepdims=True)
    Z = (X - mu) / np.sqrt(var + 1e-5)
    A = np.tanh(Z @ W1)
    R = 2.0 * (A @ W2 - Y) / (s * d)
    want2 = np.einsum("nsh,nsd->nhd", A, R)
    want1 = np.einsum("nsd,nsh->ndh", Z, (R @ W2.T) * (1.0 - A * A))
    assert got["w1"].shape == want1.shape and got["w2"].shape == want2.shape
    assert relerr(got["w2"], want2) <= 5e-5 and relerr(got["w1"], want1) <= 5e-5


def test_vmap_per_example_gradients_of_the_cnn_on_device(hip):
    """Per-example gradients of the CNN step (conv - relu - conv - relu - maxpool - conv - relu -
    mean - linear - cross-entropy) with respect to all eight shared parameters, as
    vmap(grad(loss), in_axes=(None, 0, 0)): the filters are lifted to the batch, so every
    convolution has a filter per element (windows laid out, one batched product), and the
    whole thing is one forward and one backward pass whose launches do not grow with the
    batch.  Values: the float64 oracle on each example alone."""
    from nabla_amd.core import engine
    F = nb.nn.functional
    names = oc.C4_PARAMS

    def one(params, img, label):
        logits = nb.workloads.c4_logits(params, nb.unsqueeze(img, 0))
        return F.cross_entropy_loss(logits, nb.unsqueeze(label, 0))

    steps = {}
    for n in (4, 12):
        t = oc.c4_inputs(batch=n, hw=8, c=(3, 8, 16, 24), classes=5, seed=40 + n)
        rng = np.random.default_rng(n)
        for k in ("c1b", "c2b", "c3b", "bl"):
            t[k] = (0.1 * rng.standard_normal(t[k].shape)).astype(np.float32)
        params = {k: T(t[k]) for k in names}
        engine.clear_plan_cache()
        calls = []

        def counted(p, img, label):
            calls.append(1)
            return nb.grad(one)(p, img, label)

        g = nb.vmap(counted, in_axes=(None, 0, 0))(params, T(t["img"]), T(t["labels"]))
        got = {k: g[k].numpy() for k in names}
        steps[n] = sum(len(bp.plan.steps) for bp in engine._PLAN_CACHE.values())
        engine.clear_plan_cache()
        assert len(calls) == 1, "the function was mapped element by element"
        for i in range(n):
            single = dict(t, img=t["img"][i:i + 1], labels=t["labels"][i:i + 1])
            _, wg, _, _ = oc.c4_reference(single)
            for k in names:
                assert got[k].shape == (n,) + wg[k].shape
                assert relerr(got[k][i], wg[k], floor=1e-6) < 5e-5, (n, i, k, relerr(got[k][i], wg[k]))
    assert steps[4] == steps[12], steps


def test_small_composite_ops_on_device(hip):
    """trunc / floor / is_nan / is_inf / flip exactly and log1p to fp32 rounding on the device
    (NaN and infinity must survive the kernels' compare instructions)."""
    x = np.array([-2.5, -2.0, -0.3, -0.0, 0.0, 0.7, 1.0, 1.5, 1e6 + 0.5, np.nan, np.inf, -np.inf] * 50, np.float32)
    fin = np.isfinite(x)
    np.testing.assert_array_equal(nb.trunc(T(x)).numpy()[fin], np.trunc(x)[fin])
    np.testing.assert_array_equal(nb.floor(T(x)).numpy()[fin], np.floor(x)[fin])
    np.testing.assert_array_equal(nb.is_nan(T(x)).numpy(), np.isnan(x))
    np.testing.assert_array_equal(nb.is_inf(T(x)).numpy(), np.isinf(x))
    y = np.array([0.0, 1e-12, -1e-12, 3e-8, -3e-8, 1e-4, -1e-4, 0.5, -0.5, 3.0, 100.0, -0.999] * 40, np.float32)
    got = nb.log1p(T(y)).numpy().astype(np.float64)
    np.testing.assert_allclose(got, np.log1p(y.astype(np.float64)), rtol=1e-6, atol=0)
    z = np.random.default_rng(5).standard_normal((7, 33, 5)).astype(np.float32)
    for ax in (0, 1, 2):
        np.testing.assert_array_equal(nb.flip(T(z), ax).numpy(), np.flip(z, ax))
    parts = nb.chunk(T(z), 4, axis=1)
    np.testing.assert_array_equal(parts[3].numpy(), z[:, 27:])
    # sin / cos: library routines in the row-program kernels, derivative through the trace
    a = np.random.default_rng(6).uniform(-8, 8, (33, 257)).astype(np.float32)
    np.testing.assert_allclose(nb.sin(T(a)).numpy(), np.sin(a.astype(np.float64)), rtol=0, atol=3e-7)
    np.testing.assert_allclose(nb.cos(T(a)).numpy(), np.cos(a.astype(np.float64)), rtol=0, atol=3e-7)
    g = nb.grad(lambda t: nb.reduce_sum(nb.sin(t) * nb.cos(t)))(T(a))
    np.testing.assert_allclose(g.numpy(), np.cos(2 * a.astype(np.float64)), rtol=0, atol=2e-6)


def test_gelu_bf16_over_its_whole_range(hip):
    """GELU of bf16 tensors takes a cheaper form in the kernels (the upper tail of the normal
    distribution as 2^polynomial instead of erf): every element within one bf16 step of the
    float64 value, from the far negative tail (where the result is all tail) to large arguments."""
    from scipy.special import ndtr
    a = oc.to_bf16_grid(np.concatenate([np.linspace(-12.0, 12.0, 1 << 16), [-30.0, 30.0, 0.0, -0.0, 1e-20, -1e-20]])
                        .astype(np.float32))
    got = nb.gelu(T(a, dtype=nb.DType.bfloat16))
    assert got.dtype == nb.DType.bfloat16
    got = got.numpy().astype(np.float64)
    want = a.astype(np.float64) * ndtr(a.astype(np.float64))
    assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + 1e-14)
    # and its gradient (the erf form, from the kept input) against the closed form
    g = nb.grad(lambda t: nb.reduce_sum(nb.cast(nb.gelu(t), nb.DType.float32)))(T(a[:4096], dtype=nb.DType.bfloat16))
    x = a[:4096].astype(np.float64)
    dwant = ndtr(x) + x * np.exp(-0.5 * x * x) / np.sqrt(2 * np.pi)
    assert np.all(np.abs(g.numpy().astype(np.float64) - dwant) <= 2.0 ** -7 * np.abs(dwant) + 1e-6)


# ---- scatter ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_scatter_on_device_is_exact_and_deterministic(hip, dtype):
    """Bit-exact against the oracle (numpy assignment), including rows named several times
    (the last update wins, whatever order the workgroups run in), negative indices, another
    axis, and the embedding-table gradient that is built on it."""
    from oracle import ops as O
    rng = np.random.default_rng(47)
    dt = nb.DType.float32 if dtype == "f32" else nb.DType.bfloat16
    rnd = lambda *s: torch.from_numpy(rng.standard_normal(s).astype(np.float32)).to(dt.to_torch()).float().numpy()
    x, upd = rnd(1000, 72), rnd(4096, 72)
    idx = rng.integers(-1000, 1000, size=4096).astype(np.int64)   # many duplicates, half negative
    T = lambda a: nb.Tensor.constant(a, dtype=dt)
    want = O.scatter(O.V(x), idx % 1000, O.V(upd)).a
    for _ in range(3):
        got = nb.scatter(T(x), nb.Tensor.constant(idx), T(upd))
        np.testing.assert_array_equal(nb.cast(got, nb.DType.float32).numpy(), want)
    x3, u3 = rnd(3, 17, 5), rnd(3, 2, 2, 5)
    i3 = np.array([[16, 0], [3, 16]], dtype=np.int32)
    got = nb.scatter(T(x3), nb.Tensor.constant(i3), T(u3), axis=1)
    np.testing.assert_array_equal(nb.cast(got, nb.DType.float32).numpy(), O.scatter(O.V(x3), i3, O.V(u3), axis=1).a)
    with pytest.raises(IndexError):
        nb.scatter(T(x), nb.Tensor.constant(np.array([1000], dtype=np.int64)), T(upd[:1])).numpy()
    if dtype == "f32":
        table, ids, w = rnd(500, 64), rng.integers(0, 500, size=(4, 33)).astype(np.int64), rnd(4, 33, 64)
        gt = nb.grad(lambda t: nb.reduce_sum(nb.nn.functional.embedding(nb.Tensor.constant(ids), t) * T(w)))(T(table))
        vt = O.V(table.astype(np.float64))
        (wt,) = O.grad_of(O.reduce_sum(O.gather(vt, ids) * O.V(w.astype(np.float64))), [vt])
        np.testing.assert_array_equal(gt.numpy(), wt.astype(np.float32))
