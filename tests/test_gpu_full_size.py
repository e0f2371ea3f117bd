"""GPU parity at the benchmark's own sizes: the transformer block (B8 S1024 D1024 H16, bf16), the
CNN step (batch 64, fp32) and the LoRA decoder at its real widths (D2048, 16 heads of 128, FF8192,
V32000, B4 S2048, bf16; one layer), so that the head-size-128 attention kernels, the 32000-column
cross-entropy kernels and the full-row / streaming instantiations of the row kernels that the
benchmark times are checked inside a training step.

Checker: the CPU oracle.  For the two bf16 steps it is ``oracle/torch_steps.py`` (the same
formulas on torch-CPU autograd, pinned against the numpy oracle in tests/test_oracle_pins.py),
because the numpy tape needs minutes at these sizes.

Error measure: max |got - want| over a tensor divided by max |want| over that tensor (one scale
per tensor; an element-wise ratio is meaningless for the many entries that are zero up to
rounding).  Tolerances: 1e-5 fp32, 2e-2 bf16, exact for indices.
"""
import numpy as np
import pytest
import torch

import nabla_amd as nb
from oracle import configs as oc
from oracle import torch_steps as ts

pytestmark = pytest.mark.gpu


def relerr(got, want, floor=0.0):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return np.abs(got - want).max() / max(np.abs(want).max(), floor, 1e-30)


def test_c3_transformer_block_at_benchmark_size(hip):
    t = oc.c3_inputs(8, 1024, 1024, 4096, seed=0, bf16=True)
    rng = np.random.default_rng(1)
    for k in oc.C3_PARAMS:  # biases and norm parameters off their trivial values
        if k[0] == "b" or k.startswith("ln"):
            t[k] = oc.to_bf16_grid(t[k] + 0.1 * rng.standard_normal(t[k].shape).astype(np.float32))
    loss, grads = oc.c3_program(nb, oc.upload(nb, t, dtype=nb.DType.bfloat16), num_heads=16)
    nb.realize_all(loss, *grads.values())
    got = {k: grads[k].numpy().astype(np.float64) for k in oc.C3_PARAMS}
    got_loss = loss.item()
    wl, wg = ts.c3_step(t, num_heads=16, dtype=torch.float64)
    assert abs(got_loss - wl) < 2e-2 * abs(wl)
    for k in oc.C3_PARAMS:
        assert got[k].shape == wg[k].shape
        # (bk's true gradient is zero -- softmax is shift invariant -- so it is measured on the
        # scale of bq's gradient, the same sums without the cancellation)
        floor = np.abs(wg["bq"]).max() if k == "bk" else 0.0
        assert relerr(got[k], wg[k], floor=floor) < 2e-2, (k, relerr(got[k], wg[k], floor=floor))


def test_c4_cnn_step_at_benchmark_size(hip):
    t = oc.c4_inputs(batch=64, seed=0)
    wl, wg, wam, wlogits = oc.c4_reference(t)
    # the seeded inputs have no two top logits closer than fp32 noise, so the index is decided
    top2 = np.sort(wlogits, axis=-1)[:, -2:]
    assert ((top2[:, 1] - top2[:, 0]) > 1e-4 * np.abs(top2[:, 1])).all()
    T4 = oc.upload(nb, t)
    loss, grads = oc.c4_program(nb, T4)
    logits = oc.c4_logits(nb, {k: T4[k] for k in oc.C4_PARAMS}, T4["img"])
    am = nb.argmax(logits, axis=-1)
    nb.realize_all(loss, am, logits, *grads.values())
    assert abs(loss.item() - wl) < 1e-5 * abs(wl)
    assert relerr(logits.numpy(), wlogits) < 1e-5
    assert am.numpy().dtype == np.int64
    np.testing.assert_array_equal(am.numpy(), wam)
    np.testing.assert_array_equal(am.numpy(), np.argmax(logits.numpy(), axis=-1))
    for k in oc.C4_PARAMS:
        g = grads[k].numpy().astype(np.float64)
        rms = np.sqrt(((g - wg[k]) ** 2).mean()) / np.abs(wg[k]).max()
        if k in ("k1", "c1b", "k2"):
            # Upstream of the 2 x 2 max-pooling in the backward pass.  Of the 2.1 million pooling
            # windows of this batch, two hold a pair of largest entries that agree to 8 and 3 units
            # in the last place of fp32 (oracle, fp64: 1.28906103 / 1.28906202); the fp32 product
            # that feeds the pool cannot order them, so the window's cotangent lands one pixel
            # beside where fp64 puts it.  That moves single elements of these three gradients by
            # one cotangent element (a few 1e-5 of the tensor's scale) whatever the kernels'
            # accuracy: the bound on the maximum is 1e-4, the bound on the root mean square, which
            # one moved element does not reach, stays 1e-5.  (At batch 8 no such window exists and
            # every gradient is within 1e-6: test_gpu_parity.py::test_c4_cnn_step.)
            assert relerr(g, wg[k]) < 1e-4 and rms < 1e-5, (k, relerr(g, wg[k]), rms)
        else:
            assert relerr(g, wg[k]) < 1e-5, (k, relerr(g, wg[k]))


def test_c5_lora_decoder_layer_at_benchmark_widths(hip):
    t = oc.c5_inputs(layers=1, batch=4, seq=2048, d_model=2048, d_ff=8192, vocab=32000, rank=16,
                     seed=0, b_zero=False, bf16=True)
    loss, grads = oc.c5_program(nb, oc.upload(nb, t, dtype=nb.DType.bfloat16), num_heads=16)
    flat = [ad[k] for ad in grads for k in ("qA", "qB", "vA", "vB")]
    nb.realize_all(loss, *flat)
    got = [g.numpy().astype(np.float64) for g in flat]
    got_loss = loss.item()
    del loss, grads, flat
    wl, wg = ts.c5_step(t, num_heads=16, dtype=torch.float32)
    assert abs(got_loss - wl) < 2e-2 * abs(wl)
    for name, g, w in zip(("qA", "qB", "vA", "vB"), got, wg):
        assert g.shape == w.shape and np.abs(w).max() > 0
        assert relerr(g, w) < 2e-2, (name, relerr(g, w))


def test_c5_lora_decoder_all_twelve_layers_at_benchmark_size(hip):
    """The step the benchmark times -- 12 layers, D2048, 16 heads of 128, FF8192, V32000, B4
    S2048, one plan of several hundred launches -- against the fp32 torch restatement.

    bf16: loss within 2e-2; each of the 48 adapter gradients within 2e-2 in the relative L2 norm
    (|got - want| over |want|, both as vectors) and within 2.5e-2 in the measure the other tests
    use (largest error over largest entry).  The second bound is the one exception to 2e-2 in
    this suite: 47 of the 48 tensors are inside 2e-2 in that measure too, the query-side
    adapter of layer 2 sits at 2.05e-2.  The query-side gradients pass through
    dS = P * (dP - delta), where a part common to all values cancels; what bf16 storage of q, k,
    v and dO leaves behind does not, and the same step with attention as the reference's
    composition of matmul / softmax / matmul in bf16 shows the same 1.3-1.9e-2 (L2) on these
    tensors.  (With delta taken from bf16 O alone, as before the forward kernel handed its
    rounding remainder on, they were at 2-4e-2.)

    fp32: the same plan in float32 -- every product, the unfused attention, the row programs
    at full width and depth -- within 2e-5 of the oracle on every gradient (measured 4-9e-6),
    which is what shows that nothing but rounding separates the bf16 numbers from the oracle.

    The oracle walks the four sequences one at a time (they only meet in the loss, a sum over
    sequences divided by their number), which keeps its activations at a quarter."""
    t = oc.c5_inputs(layers=12, batch=4, seq=2048, d_model=2048, d_ff=8192, vocab=32000, rank=16,
                     seed=0, b_zero=False, bf16=True)

    def device_step(dtype):
        loss, grads = oc.c5_program(nb, oc.upload(nb, t, dtype=dtype), num_heads=16)
        flat = [ad[k] for ad in grads for k in ("qA", "qB", "vA", "vB")]
        nb.realize_all(loss, *flat)
        got = [g.numpy().astype(np.float64) for g in flat]
        value = loss.item()
        del loss, grads, flat
        torch.cuda.empty_cache()
        return value, got

    loss16, got16 = device_step(nb.DType.bfloat16)
    loss32, got32 = device_step(nb.DType.float32)
    assert np.isfinite(loss16) and all(np.isfinite(g).all() for g in got16)
    batch = t["ids"].shape[0]
    wl, wg = 0.0, None
    for i in range(batch):
        one = dict(t, ids=t["ids"][i:i + 1])
        li, gi = ts.c5_step(one, num_heads=16, dtype=torch.float32)
        wl += li / batch
        wg = [g / batch for g in gi] if wg is None else [a + g / batch for a, g in zip(wg, gi)]
    names = [f"layer {i} {k}" for i in range(12) for k in ("qA", "qB", "vA", "vB")]
    l2 = lambda g, w: np.sqrt(((g - w) ** 2).sum() / (w ** 2).sum())
    assert abs(loss32 - wl) < 1e-5 * abs(wl), (loss32, wl)
    assert abs(loss16 - wl) < 2e-2 * abs(wl), (loss16, wl)
    worst = {"fp32": max(zip((relerr(g, w) for g, w in zip(got32, wg)), names)),
             "bf16 max": max(zip((relerr(g, w) for g, w in zip(got16, wg)), names)),
             "bf16 l2": max(zip((l2(g, w) for g, w in zip(got16, wg)), names))}
    print("worst errors:", worst, flush=True)
    inside = 0
    for name, g16, g32, w in zip(names, got16, got32, wg):
        assert g16.shape == w.shape and np.abs(w).max() > 0, name
        assert relerr(g32, w) < 2e-5, (name, "fp32", relerr(g32, w), worst)
        assert l2(g16, w) < 2e-2, (name, "bf16 l2", l2(g16, w), worst)
        assert relerr(g16, w) < 2.5e-2, (name, "bf16 max", relerr(g16, w), worst)
        inside += relerr(g16, w) < 2e-2
    assert inside >= 46, (inside, worst)
