"""Pins of the CPU oracle (oracle/ops.py): before it may judge the HIP path it is
itself checked against torch-CPU autograd in fp64, brute-force loops on tiny
inputs, and closed forms / invariants, chosen so that a dropped term, a wrong
sign or a transposed operand fails one of them."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as TF

from oracle import configs as oc
from oracle import ops as O

RNG = np.random.default_rng(7)


def _t(a):
    return torch.tensor(a, dtype=torch.float64, requires_grad=True)


def _close(a, b, tol=1e-10):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    assert a.shape == b.shape
    assert np.abs(a - b).max() <= tol * (1 + np.abs(b).max()), np.abs(a - b).max()


# ---- primitives vs torch autograd -----------------------------------------------
@pytest.mark.parametrize("name,ofn,tfn", [
    ("relu", O.relu, torch.relu), ("exp", O.exp, torch.exp), ("neg", O.neg, torch.neg),
    ("tanh", O.tanh, torch.tanh), ("erf", O.erf, torch.erf),
    ("gelu", O.gelu, lambda t: TF.gelu(t, approximate="none")),
    ("rsqrt", lambda v: O.rsqrt(v * v + 1.0), lambda t: torch.rsqrt(t * t + 1.0)),
    ("sqrt", lambda v: O.sqrt(v * v + 1.0), lambda t: torch.sqrt(t * t + 1.0)),
    ("log", lambda v: O.log(v * v + 1.0), lambda t: torch.log(t * t + 1.0)),
])
def test_unary_value_and_vjp(name, ofn, tfn):
    x = RNG.standard_normal((5, 7))
    v = O.V(x)
    out = ofn(v)
    w = RNG.standard_normal(out.a.shape)
    (g,) = O.grad_of(O.reduce_sum(out * w), [v])
    t = _t(x)
    to = tfn(t)
    (to * torch.tensor(w)).sum().backward()
    _close(out.a, to.detach().numpy())
    _close(g, t.grad.numpy())


def test_binary_broadcast_vjps():
    a, b = RNG.standard_normal((4, 1, 6)), RNG.standard_normal((3, 1)) + 3.0
    for ofn, tfn in ((O.add, torch.add), (O.sub, torch.sub), (O.mul, torch.mul), (O.div, torch.div)):
        va, vb = O.V(a), O.V(b)
        out = ofn(va, vb)
        w = RNG.standard_normal(out.a.shape)
        ga, gb = O.grad_of(O.reduce_sum(out * w), [va, vb])
        ta, tb = _t(a), _t(b)
        (tfn(ta, tb) * torch.tensor(w)).sum().backward()
        _close(out.a, tfn(ta, tb).detach().numpy())
        _close(ga, ta.grad.numpy())
        _close(gb, tb.grad.numpy())


def test_matmul_brute_force_and_vjp():
    a, b = RNG.standard_normal((2, 3, 4)), RNG.standard_normal((4, 5))
    brute = np.zeros((2, 3, 5))
    for n in range(2):
        for i in range(3):
            for j in range(5):
                for k in range(4):
                    brute[n, i, j] += a[n, i, k] * b[k, j]
    va, vb = O.V(a), O.V(b)
    out = O.matmul(va, vb)
    _close(out.a, brute)
    w = RNG.standard_normal(out.a.shape)
    ga, gb = O.grad_of(O.reduce_sum(out * w), [va, vb])
    ta, tb = _t(a), _t(b)
    ((ta @ tb) * torch.tensor(w)).sum().backward()
    _close(ga, ta.grad.numpy())
    _close(gb, tb.grad.numpy())  # includes the sum over the broadcast batch axis
    # a transposed operand must fail: the product is not symmetric
    assert np.abs(out.a - np.matmul(a, b[:, ::-1])).max() > 1e-3


def test_reductions_and_tie_rule():
    x = RNG.standard_normal((3, 4, 5))
    v = O.V(x)
    _close(O.reduce_sum(v, axis=(0, 2)).a, x.sum(axis=(0, 2)))
    _close(O.mean(v, axis=1, keepdims=True).a, x.mean(axis=1, keepdims=True))
    _close(O.reduce_max(v, axis=-1).a, x.max(axis=-1))
    (g,) = O.grad_of(O.reduce_sum(O.mean(v, axis=(1, 2))), [v])
    _close(g, np.full_like(x, 1.0 / 20))
    # ties: EVERY maximal element receives the full cotangent (reduction.py:219-230)
    t = np.array([[1.0, 3.0, 3.0, 2.0], [5.0, 5.0, 5.0, 0.0]])
    vt = O.V(t)
    (gt,) = O.grad_of(O.reduce_sum(O.reduce_max(vt, axis=1) * np.array([2.0, 7.0])), [vt])
    _close(gt, np.array([[0, 2, 2, 0], [7, 7, 7, 0]], dtype=float))
    assert np.array_equal(O.argmax(vt, axis=1), np.array([1, 0]))  # lowest index wins


def test_softmax_logsoftmax():
    x = RNG.standard_normal((4, 9)) * 3
    v = O.V(x)
    s = O.softmax(v, axis=-1)
    _close(s.a.sum(-1), np.ones(4))
    _close(O.logsoftmax(v).a, np.log(s.a))
    w = RNG.standard_normal((4, 9))
    for ofn, tfn in ((O.softmax, torch.softmax), (O.logsoftmax, torch.log_softmax)):
        (g,) = O.grad_of(O.reduce_sum(ofn(v, -1) * w), [v])
        t = _t(x)
        (tfn(t, -1) * torch.tensor(w)).sum().backward()
        _close(g, t.grad.numpy())
    # shift invariance of softmax
    _close(O.softmax(O.V(x + 100.0)).a, s.a)


def test_layer_norm_invariants_and_grads():
    x, w, b = RNG.standard_normal((6, 16)), RNG.standard_normal(16), RNG.standard_normal(16)
    y0 = O.layer_norm(O.V(x)).a
    _close(y0.mean(-1), np.zeros(6), 1e-12)
    assert np.abs(y0.var(-1) - 1.0).max() < 1e-4  # biased variance, eps 1e-5
    vx, vw, vb = O.V(x), O.V(w), O.V(b)
    out = O.layer_norm(vx, vw, vb)
    c = RNG.standard_normal(out.a.shape)
    gs = O.grad_of(O.reduce_sum(out * c), [vx, vw, vb])
    tx, tw, tb = _t(x), _t(w), _t(b)
    to = TF.layer_norm(tx, (16,), tw, tb, eps=1e-5)
    (to * torch.tensor(c)).sum().backward()
    _close(out.a, to.detach().numpy())
    for g, t in zip(gs, (tx, tw, tb)):
        _close(g, t.grad.numpy(), 1e-9)


def test_attention_matches_manual_torch_causal_and_not():
    q, k, v = (RNG.standard_normal((2, 3, 6, 4)) for _ in range(3))
    for causal in (False, True):
        vq, vk, vv = O.V(q), O.V(k), O.V(v)
        out = O.scaled_dot_product_attention(vq, vk, vv, is_causal=causal)
        tq, tk, tv = _t(q), _t(k), _t(v)
        sc = tq @ tk.transpose(-1, -2) / math.sqrt(4)
        if causal:
            sc = sc.masked_fill(~torch.tril(torch.ones(6, 6, dtype=torch.bool)), float("-inf"))
        to = torch.softmax(sc, -1) @ tv
        _close(out.a, to.detach().numpy())
        c = RNG.standard_normal(out.a.shape)
        gs = O.grad_of(O.reduce_sum(out * c), [vq, vk, vv])
        (to * torch.tensor(c)).sum().backward()
        for g, t in zip(gs, (tq, tk, tv)):
            _close(g, t.grad.numpy(), 1e-9)


def test_conv2d_brute_force_and_torch():
    x = RNG.standard_normal((2, 5, 6, 3))
    w = RNG.standard_normal((3, 2, 3, 4))
    bias = RNG.standard_normal(4)
    stride, pad = (2, 1), (1, 0, 2, 1)
    out = O.conv2d(O.V(x), O.V(w), O.V(bias), stride=stride, padding=pad)
    xp = np.pad(x, ((0, 0), (1, 0), (2, 1), (0, 0)))
    ho, wo = out.a.shape[1], out.a.shape[2]
    brute = np.zeros_like(out.a)
    for n in range(2):
        for i in range(ho):
            for j in range(wo):
                for co in range(4):
                    acc = bias[co]
                    for r in range(3):
                        for s in range(2):
                            for c in range(3):
                                acc += xp[n, i * 2 + r, j * 1 + s, c] * w[r, s, c, co]
                    brute[n, i, j, co] = acc
    _close(out.a, brute)
    vx, vw, vb = O.V(x), O.V(w), O.V(bias)
    o2 = O.conv2d(vx, vw, vb, stride=stride, padding=pad)
    c = RNG.standard_normal(o2.a.shape)
    gs = O.grad_of(O.reduce_sum(o2 * c), [vx, vw, vb])
    tx, tw, tb = _t(x), _t(w), _t(bias)
    to = TF.conv2d(TF.pad(tx.permute(0, 3, 1, 2), (2, 1, 1, 0)), tw.permute(3, 2, 0, 1), tb, stride=stride)
    (to.permute(0, 2, 3, 1) * torch.tensor(c)).sum().backward()
    for g, t in zip(gs, (tx, tw, tb)):
        _close(g, t.grad.numpy(), 1e-9)


def test_conv2d_transpose_brute_force_torch_and_adjoint():
    x = RNG.standard_normal((2, 4, 3, 5))
    w = RNG.standard_normal((3, 2, 4, 5))          # [R, S, Cout, Cin]
    bias = RNG.standard_normal(4)
    stride, pad = (2, 3), (1, 0, 2, 1)
    out = O.conv2d_transpose(O.V(x), O.V(w), O.V(bias), stride=stride, padding=pad)
    hf, wf = (4 - 1) * 2 + 3, (3 - 1) * 3 + 2
    assert out.a.shape == (2, hf - 1, wf - 3, 4)
    full = np.zeros((2, hf, wf, 4))
    for n in range(2):
        for i in range(4):
            for j in range(3):
                for r in range(3):
                    for s in range(2):
                        for co in range(4):
                            for ci in range(5):
                                full[n, i * 2 + r, j * 3 + s, co] += x[n, i, j, ci] * w[r, s, co, ci]
    _close(out.a, full[:, 1:hf, 2:wf - 1, :] + bias)
    # torch: weight [Cin, Cout, R, S]; no padding there, the crop is applied afterwards
    vx, vw, vb = O.V(x), O.V(w), O.V(bias)
    o2 = O.conv2d_transpose(vx, vw, vb, stride=stride, padding=pad)
    c = RNG.standard_normal(o2.a.shape)
    gs = O.grad_of(O.reduce_sum(o2 * c), [vx, vw, vb])
    tx, tw, tb = _t(x), _t(w), _t(bias)
    to = TF.conv_transpose2d(tx.permute(0, 3, 1, 2), tw.permute(3, 2, 0, 1), tb, stride=stride)
    to = to.permute(0, 2, 3, 1)[:, 1:hf, 2:wf - 1, :]
    _close(o2.a, to.detach().numpy(), 1e-12)
    (to * torch.tensor(c)).sum().backward()
    for g, t in zip(gs, (tx, tw, tb)):
        _close(g, t.grad.numpy(), 1e-9)
    # it is the adjoint of conv2d with the same filter read as HWIO: <convT(x), y> = <x, conv(y)>
    y = RNG.standard_normal(o2.a.shape)
    lhs = (O.conv2d_transpose(O.V(x), O.V(w), None, stride, pad).a * y).sum()
    rhs = (x * O.conv2d(O.V(y), O.V(w), None, stride, pad).a).sum()
    assert abs(lhs - rhs) <= 1e-10 * max(abs(lhs), 1.0)


def test_max_pool_window_clipping_and_ties():
    x = RNG.standard_normal((2, 5, 5, 3))
    out = O.max_pool2d(O.V(x), (3, 3), (2, 2), (1, 1, 1, 1))
    to = TF.max_pool2d(torch.tensor(x).permute(0, 3, 1, 2), 3, 2, 1).permute(0, 2, 3, 1)
    _close(out.a, to.numpy())
    t = np.zeros((1, 2, 2, 1))
    t[0, :, :, 0] = [[1.0, 1.0], [0.0, 1.0]]
    vt = O.V(t)
    (g,) = O.grad_of(O.reduce_sum(O.max_pool2d(vt, (2, 2)) * 5.0), [vt])
    _close(g[0, :, :, 0], np.array([[5.0, 5.0], [0.0, 5.0]]))  # all three tied maxima


def test_cross_entropy_divides_by_first_dim_only():
    logits = RNG.standard_normal((2, 3, 5))
    labels = RNG.integers(0, 5, (2, 3))
    v = O.V(logits)
    loss = O.cross_entropy_loss(v, labels)
    t = _t(logits)
    ref = TF.cross_entropy(t.reshape(-1, 5), torch.tensor(labels).reshape(-1), reduction="sum") / 2
    _close(loss.a, ref.detach().numpy())
    (g,) = O.grad_of(loss, [v])
    ref.backward()
    _close(g, t.grad.numpy())


def test_lora_linear_and_gather():
    x, w = RNG.standard_normal((3, 8)), RNG.standard_normal((8, 6))
    A, B = RNG.standard_normal((8, 2)), RNG.standard_normal((2, 6))
    vA, vB = O.V(A), O.V(B)
    out = O.lora_linear(O.V(x), O.V(w), vA, vB, alpha=4.0)
    _close(out.a, x @ w + x @ (A @ B) * 2.0)
    c = RNG.standard_normal(out.a.shape)
    gA, gB = O.grad_of(O.reduce_sum(out * c), [vA, vB])
    tA, tB = _t(A), _t(B)
    ((torch.tensor(x) @ torch.tensor(w) + torch.tensor(x) @ ((tA @ tB) * 2.0)) * torch.tensor(c)).sum().backward()
    _close(gA, tA.grad.numpy())
    _close(gB, tB.grad.numpy())
    table = RNG.standard_normal((7, 3))
    idx = np.array([[6, 0], [3, 3]])
    assert np.array_equal(O.gather(O.V(table), O.V(idx)).a, table[idx])


# ---- whole configurations vs torch autograd --------------------------------------
def test_config_c1_against_torch():
    inp = oc.c1_inputs(16, 24, 12, 5, seed=1)
    loss, grads = oc.c1_reference(**inp)
    ts = {k: _t(v) for k, v in inp.items()}
    tl = (torch.relu(ts["x"] @ ts["W1"] + ts["b1"]) @ ts["W2"] + ts["b2"]).mean()
    tl.backward()
    _close(loss, tl.item())
    for g, k in zip(grads, ("W1", "b1", "W2", "b2")):
        _close(g, ts[k].grad.numpy())


def test_config_c2_closed_form_gradient():
    inp = oc.c2_inputs(6, 40, seed=2)
    out, gx = oc.c2_reference(**inp)
    x, y = inp["x"].astype(np.float64), inp["y"].astype(np.float64)
    p = x * y
    m = p.max(1, keepdims=True)
    e = np.exp(p - m)
    r = np.maximum(x, 0)
    _close(out, (e * r).sum(1))
    # d/dx sum_j e_j r_j with the max treated through the tie rule
    closed = e * (x > 0) + y * (e * r - (p == m) * (e * r).sum(1, keepdims=True))
    _close(gx, closed)
    tx = _t(x)
    tp = tx * torch.tensor(y)
    (torch.exp(tp - tp.max(1, keepdim=True).values) * torch.relu(tx)).sum().backward()
    _close(gx, tx.grad.numpy())


def test_config_c3_against_torch_module_formulas():
    t = oc.c3_inputs(2, 8, 16, 32, seed=3, bf16=False)
    t = {k: v.astype(np.float64) + (0.1 * RNG.standard_normal(v.shape) if k.startswith("b") or k.startswith("ln") else 0)
         for k, v in t.items()}
    loss, grads = oc.c3_reference(t, num_heads=4)
    ts = {k: _t(v) for k, v in t.items()}

    def heads(z):
        return z.reshape(2, 8, 4, 4).transpose(1, 2)

    x = ts["x"]
    n1 = TF.layer_norm(x, (16,), ts["ln1_w"], ts["ln1_b"])
    q, k, v = (heads(n1 @ ts[w] + ts[b]) for w, b in (("wq", "bq"), ("wk", "bk"), ("wv", "bv")))
    a = TF.scaled_dot_product_attention(q, k, v, is_causal=True)
    x = x + a.transpose(1, 2).reshape(2, 8, 16) @ ts["wo"] + ts["bo"]
    n2 = TF.layer_norm(x, (16,), ts["ln2_w"], ts["ln2_b"])
    out = x + TF.gelu(n2 @ ts["w1"] + ts["b1"]) @ ts["w2"] + ts["b2"]
    tl = (out * out).mean()
    tl.backward()
    _close(loss, tl.item(), 1e-9)
    for k in oc.C3_PARAMS:
        _close(grads[k], ts[k].grad.numpy(), 1e-8)


def test_config_c4_against_torch():
    t = oc.c4_inputs(batch=3, hw=8, c=(3, 4, 6, 8), classes=5, seed=4)
    loss, grads, am, logits = oc.c4_reference(t)
    ts = {k: _t(v) for k, v in t.items() if k != "labels"}

    def conv(h, k, b):
        return TF.conv2d(h, ts[k].permute(3, 2, 0, 1), ts[b], padding=1)

    h = torch.relu(conv(ts["img"].permute(0, 3, 1, 2), "k1", "c1b"))
    h = TF.max_pool2d(torch.relu(conv(h, "k2", "c2b")), 2)
    h = torch.relu(conv(h, "k3", "c3b")).mean(dim=(2, 3))
    lg = h @ ts["wl"] + ts["bl"]
    tl = TF.cross_entropy(lg, torch.tensor(t["labels"]))
    tl.backward()
    _close(loss, tl.item(), 1e-9)
    _close(logits, lg.detach().numpy(), 1e-9)
    assert np.array_equal(am, lg.argmax(-1).numpy())
    for k in oc.C4_PARAMS:
        _close(grads[k], ts[k].grad.numpy(), 1e-8)


def test_config_c5_lora_grads_against_torch_and_zero_at_init():
    t = oc.c5_inputs(layers=2, batch=2, seq=6, d_model=16, d_ff=32, vocab=20, rank=2, seed=5,
                     b_zero=False, bf16=False)
    loss, grads = oc.c5_reference(t, num_heads=4, alpha=4.0)
    lora = [{k: _t(v) for k, v in ad.items()} for ad in t["lora"]]
    c = lambda a: torch.tensor(a, dtype=torch.float64)
    x = c(t["embed"])[torch.tensor(t["ids"])]
    heads = lambda z: z.reshape(2, 6, 4, 4).transpose(1, 2)
    for L, ad in zip(t["layers"], lora):
        n1 = TF.layer_norm(x, (16,), c(L["ln1_w"]), c(L["ln1_b"]))
        q = heads(n1 @ c(L["wq"]) + n1 @ ((ad["qA"] @ ad["qB"]) * 2.0) + c(L["bq"]))
        k = heads(n1 @ c(L["wk"]) + c(L["bk"]))
        v = heads(n1 @ c(L["wv"]) + n1 @ ((ad["vA"] @ ad["vB"]) * 2.0) + c(L["bv"]))
        a = TF.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + a.transpose(1, 2).reshape(2, 6, 16) @ c(L["wo"]) + c(L["bo"])
        n2 = TF.layer_norm(x, (16,), c(L["ln2_w"]), c(L["ln2_b"]))
        x = x + TF.gelu(n2 @ c(L["w1"]) + c(L["b1"])) @ c(L["w2"]) + c(L["b2"])
    x = TF.layer_norm(x, (16,), c(t["lnf_w"]), c(t["lnf_b"]))
    lg = x @ c(t["head"])
    tl = TF.cross_entropy(lg.reshape(-1, 20), torch.tensor(t["ids"]).reshape(-1), reduction="sum") / 2
    tl.backward()
    _close(loss, tl.item(), 1e-9)
    flat = [ad[k] for ad in lora for k in ("qA", "qB", "vA", "vB")]
    for g, tt in zip(grads, flat):
        _close(g, tt.grad.numpy(), 1e-8)
    # with B = 0 (the initialisation of the configuration) dA is exactly zero
    t0 = oc.c5_inputs(layers=1, batch=1, seq=4, d_model=8, d_ff=16, vocab=10, rank=2, seed=6,
                      b_zero=True, bf16=False)
    _, g0 = oc.c5_reference(t0, num_heads=2)
    assert np.all(g0[0] == 0) and np.all(g0[2] == 0) and np.abs(g0[1]).max() > 0


def test_nf4_quantisation_pins():
    """The NF4 restatement against what fixes it: nearest level by decision thresholds (the
    midpoints between levels -- a different formulation of the same rule), exact round trips
    for values that are level x scale, the all-zero block, padding, idempotence."""
    rng = np.random.default_rng(21)
    lv = O.NF4_LEVELS
    assert lv.size == 16 and np.all(np.diff(lv) > 0) and lv[0] == -1 and lv[-1] == 1 and lv[7] == 0
    w = rng.standard_normal((13, 10)).astype(np.float32)
    q = O.nf4_quantize(w, block_size=8)
    assert q["padded"] == 136 and q["numel"] == 130 and q["indices"].size == 136 and q["scales"].size == 17
    flat = np.pad(w.reshape(-1), (0, 6)).reshape(-1, 8)
    np.testing.assert_array_equal(q["scales"], np.abs(flat).max(1))
    mid = ((lv[1:].astype(np.float64) + lv[:-1]) / 2)
    normed = (flat / q["scales"][:, None]).reshape(-1)
    by_threshold = np.searchsorted(mid, normed.astype(np.float64), side="left")
    ties = np.isin(normed.astype(np.float64), mid)
    np.testing.assert_array_equal(q["indices"][~ties], by_threshold[~ties])
    # the block maximum is +-1 after scaling: first or last level
    peak = np.abs(flat).argmax(1)
    assert set(q["indices"].reshape(-1, 8)[np.arange(17), peak]) <= {0, 15}
    # values that are exactly level x scale come back exactly; requantising is a fixed point
    d = O.nf4_dequantize(q)
    assert d.shape == w.shape and d.dtype == np.float32
    q2 = O.nf4_quantize(d, block_size=8)
    np.testing.assert_array_equal(q2["indices"][:130], q["indices"][:130])
    np.testing.assert_array_equal(O.nf4_dequantize(q2), d)
    # all-zero block: scale 1, level 7 (0.0)
    z = O.nf4_quantize(np.zeros((2, 8), np.float32), block_size=8)
    assert np.all(z["scales"] == 1) and np.all(z["indices"] == 7) and np.all(O.nf4_dequantize(z) == 0)
    # lossy but bounded: the largest gap between neighbouring levels is 0.3038, so the error
    # is at most half of that times the block scale
    err = np.abs(d - w).reshape(-1)
    bound = 0.5 * np.diff(lv).max() * np.repeat(q["scales"], 8)[:130]
    assert np.all(err <= bound + 1e-6)


def test_avg_pool_and_silu_against_torch():
    """avg_pool2d is torch's with count_include_pad=True (symmetric padding), checked with
    overlapping windows, strides and padding; silu and both gradients against autograd."""
    import torch.nn.functional as F
    rng = np.random.default_rng(23)
    x = rng.standard_normal((2, 9, 8, 3))
    for kernel, stride, pad in (((2, 2), (2, 2), (0, 0)), ((3, 3), (2, 1), (1, 1)), ((3, 2), (1, 2), (1, 0))):
        xt = torch.tensor(x, requires_grad=True)
        yt = F.avg_pool2d(xt.permute(0, 3, 1, 2), kernel, stride, pad, count_include_pad=True).permute(0, 2, 3, 1)
        g = rng.standard_normal(tuple(yt.shape))
        yt.backward(torch.tensor(g))
        vx = O.V(x)
        y = O.avg_pool2d(vx, kernel, stride, (pad[0], pad[0], pad[1], pad[1]))
        np.testing.assert_allclose(y.a, yt.detach().numpy(), rtol=1e-12, atol=1e-12)
        (gx,) = O.grad_of(O.reduce_sum(y * O.V(g)), [vx])
        np.testing.assert_allclose(gx, xt.grad.numpy(), rtol=1e-12, atol=1e-12)
    # asymmetric padding (top 2, bottom 0): a window that lies wholly in the padding is 0
    y = O.avg_pool2d(O.V(np.ones((1, 2, 2, 1))), (2, 2), (2, 2), (2, 0, 0, 0))
    np.testing.assert_array_equal(y.a.reshape(-1), [0.0, 1.0])
    xt = torch.tensor(x, requires_grad=True)
    F.silu(xt).backward(torch.ones_like(xt))
    vx = O.V(x)
    s = O.silu(vx)
    np.testing.assert_allclose(s.a, F.silu(torch.tensor(x)).numpy(), rtol=1e-12)
    np.testing.assert_allclose(O.grad_of(O.reduce_sum(s), [vx])[0], xt.grad.numpy(), rtol=1e-12)


def test_scatter_and_gather_gradient_pins():
    """scatter is numpy's ``out[idx] = updates`` (last write wins on duplicates) and torch's
    index_copy for distinct indices; its VJP and the scatter-into-zeros VJP of gather are
    checked against the definitions."""
    rng = np.random.default_rng(25)
    x, upd = rng.standard_normal((6, 4)), rng.standard_normal((3, 4))
    idx = np.array([4, 0, 2])
    got = O.scatter(O.V(x), idx, O.V(upd), axis=0)
    want = x.copy(); want[idx] = upd
    np.testing.assert_array_equal(got.a, want)
    np.testing.assert_array_equal(got.a, torch.tensor(x).index_copy(0, torch.tensor(idx), torch.tensor(upd)).numpy())
    # along another axis, with a 2-d index
    x3, idx2 = rng.standard_normal((2, 5, 3)), np.array([[3, 1], [0, 4]])
    upd3 = rng.standard_normal((2, 2, 2, 3))
    want3 = x3.copy(); want3[:, idx2.reshape(-1), :] = upd3.reshape(2, 4, 3)
    np.testing.assert_array_equal(O.scatter(O.V(x3), idx2, O.V(upd3), axis=1).a, want3)
    # duplicates: the last update of a row wins
    dup = O.scatter(O.V(np.zeros((3, 2))), np.array([1, 1, 2, 1]), O.V(np.arange(8.0).reshape(4, 2)))
    np.testing.assert_array_equal(dup.a, [[0, 0], [6, 7], [4, 5]])
    # VJP: replaced rows of x get nothing, updates get the rows they were written to
    vx, vu = O.V(x), O.V(upd)
    g = rng.standard_normal((6, 4))
    gx, gu = O.grad_of(O.reduce_sum(O.scatter(vx, idx, vu) * O.V(g)), [vx, vu])
    wx = g.copy(); wx[idx] = 0
    np.testing.assert_array_equal(gx, wx)
    np.testing.assert_array_equal(gu, g[idx])
    # gather VJP = cotangent scattered into zeros (distinct indices: torch's index_select grad)
    tt = torch.tensor(x, requires_grad=True)
    gg = rng.standard_normal((3, 4))
    tt.index_select(0, torch.tensor(idx)).backward(torch.tensor(gg))
    vt = O.V(x)
    (gt,) = O.grad_of(O.reduce_sum(O.gather(vt, idx) * O.V(gg)), [vt])
    np.testing.assert_array_equal(gt, tt.grad.numpy())


# ---- casts, comparisons and the remaining view helpers ---------------------------------
def test_cast_values_truncation_and_vjp():
    """cast: float -> int truncates toward zero (numpy and torch agree), float -> narrower float
    rounds to nearest even, the VJP casts the cotangent back to the input type and an integer
    input receives no gradient."""
    x = np.array([-2.7, -0.5, 0.49, 1.5, 2.5, 1e6 + 0.75])
    got = O.cast(O.V(x), np.int64).a
    assert got.dtype == np.int64
    assert got.tolist() == [-2, 0, 0, 1, 2, 1000000]
    assert got.tolist() == torch.tensor(x).to(torch.int64).tolist()
    assert O.cast(O.V(x), np.int32).a.tolist() == torch.tensor(x).to(torch.int32).tolist()
    # fp64 -> fp32: nearest even; 1 + 2^-24 is a tie and goes to 1.0, 1 + 3 * 2^-24 to 1 + 2^-22
    ties = np.array([1.0 + 2.0 ** -24, 1.0 + 3.0 * 2.0 ** -24])
    assert O.cast(O.V(ties), np.float32).a.tolist() == [1.0, 1.0 + 2.0 ** -22]
    # bool -> float gives exact 0 / 1
    assert O.cast(O.V(np.array([True, False])), np.float64).a.tolist() == [1.0, 0.0]
    # gradient: a cast in the middle of a chain is the identity to the cotangent
    a = RNG.standard_normal((3, 4))
    v = O.V(a)
    w = RNG.standard_normal((3, 4))
    (g,) = O.grad_of(O.reduce_sum(O.cast(v * 3.0, np.float32) * w), [v])
    assert g.dtype == np.float64
    t = _t(a)
    ((t * 3.0).to(torch.float32) * torch.tensor(w, dtype=torch.float32)).sum().backward()
    _close(g, t.grad.numpy(), 1e-6)
    vi = O.V(np.arange(4))
    assert O.backward(O.reduce_sum(O.cast(vi, np.float64) * 2.0)).get(id(vi)) is None


def test_equal_is_exact_and_broadcasts():
    """equal: elementwise ==, bool result, numpy broadcasting, no gradient; the one-hot it
    builds in cross_entropy (labels against an iota) is the identity matrix's rows."""
    a = np.array([[0.0, -0.0, 1.0, np.nan]])
    b = np.array([[0.0], [1.0], [np.nan]])
    got = O.equal(O.V(a), O.V(b))
    assert got.a.dtype == np.bool_ and got.a.shape == (3, 4)
    assert got.a.tolist() == [[True, True, False, False], [False, False, True, False],
                              [False, False, False, False]]  # -0 == 0, NaN != NaN
    assert got.a.tolist() == torch.eq(torch.tensor(a), torch.tensor(b)).tolist()
    assert got.vjp is None and got.parents == ()
    labels = np.array([2, 0, 3, 3])
    onehot = O.equal(O.unsqueeze(O.V(labels), -1), O.V(np.arange(4))).a
    assert (onehot == np.eye(4, dtype=bool)[labels]).all()


def test_permute_against_element_loops_and_torch():
    """permute: out[i0, i1, i2] = x[...] with axis k of the result being axis order[k] of the
    input (an index loop on a tiny tensor), and the VJP is the inverse permutation -- a
    non-involutive order, so that using `order` where its inverse belongs fails."""
    x = RNG.standard_normal((2, 3, 4))
    order = (2, 0, 1)  # inverse is (1, 2, 0): not the same permutation
    v = O.V(x)
    out = O.permute(v, order)
    assert out.a.shape == (4, 2, 3)
    for i in range(4):
        for j in range(2):
            for k in range(3):
                assert out.a[i, j, k] == x[j, k, i]
    w = RNG.standard_normal(out.a.shape)
    (g,) = O.grad_of(O.reduce_sum(out * w), [v])
    t = _t(x)
    (t.permute(*order) * torch.tensor(w)).sum().backward()
    _close(g, t.grad.numpy())
    assert np.array_equal(g, np.transpose(w, (1, 2, 0)))
    # swap_axes is the two-axis case of the same thing
    _close(O.swap_axes(v, 0, 2).a, np.transpose(x, (2, 1, 0)))


def test_unsqueeze_shapes_and_vjp():
    x = RNG.standard_normal((3, 4))
    v = O.V(x)
    for axis, shape in ((0, (1, 3, 4)), (1, (3, 1, 4)), (-1, (3, 4, 1)), (2, (3, 4, 1))):
        out = O.unsqueeze(v, axis)
        assert out.a.shape == shape == tuple(torch.tensor(x).unsqueeze(axis).shape)
        assert np.array_equal(out.a.reshape(3, 4), x)
        w = RNG.standard_normal(shape)
        (g,) = O.grad_of(O.reduce_sum(out * w), [v])
        assert np.array_equal(g, w.reshape(3, 4))
    # a broadcast along the inserted axis sums back over it
    out = O.mul(O.unsqueeze(v, 1), O.V(np.ones((3, 5, 4))))
    (g,) = O.grad_of(O.reduce_sum(out), [v])
    _close(g, np.full((3, 4), 5.0))


def test_slice_tensor_window_and_zero_padded_vjp():
    """slice_tensor(x, start, size) is x[start : start + size] per axis (size, not stop), and
    its VJP puts the cotangent back into a zero tensor of the input's shape."""
    x = RNG.standard_normal((5, 6, 3))
    start, size = (1, 2, 0), (3, 2, 3)
    v = O.V(x)
    out = O.slice_tensor(v, start, size)
    assert out.a.shape == size
    for i in range(3):
        for j in range(2):
            for k in range(3):
                assert out.a[i, j, k] == x[1 + i, 2 + j, k]
    w = RNG.standard_normal(size)
    (g,) = O.grad_of(O.reduce_sum(out * w), [v])
    t = _t(x)
    (t[1:4, 2:4, :] * torch.tensor(w)).sum().backward()
    _close(g, t.grad.numpy())
    assert g[0].max() == 0.0 and g[4].min() == 0.0 and np.count_nonzero(g) == w.size
    # two overlapping windows of one tensor accumulate
    o2 = O.reduce_sum(O.slice_tensor(v, (0, 0, 0), (2, 6, 3))) + O.reduce_sum(O.slice_tensor(v, (1, 0, 0), (2, 6, 3)))
    (g2,) = O.grad_of(o2, [v])
    assert g2[0, 0, 0] == 1.0 and g2[1, 0, 0] == 2.0 and g2[2, 0, 0] == 1.0 and g2[3, 0, 0] == 0.0


def test_broadcast_to_values_and_summed_vjp():
    """broadcast_to: numpy's right-aligned rule on odd shapes (new leading axes and size-1
    axes stretched at once), and the VJP sums the cotangent over every axis that was added or
    stretched (view/shape.py:131-152) -- torch's `expand` is the independent check; summing
    over the wrong axes, or forgetting keepdims on a stretched axis, fails it."""
    x = RNG.standard_normal((3, 1, 5))
    shape = (2, 7, 3, 4, 5)
    v = O.V(x)
    out = O.broadcast_to(v, shape)
    assert out.a.shape == shape
    for a in range(2):
        for b in range(7):
            for j in range(4):
                assert np.array_equal(out.a[a, b, :, j, :], x[:, 0, :])
    w = RNG.standard_normal(shape)
    (g,) = O.grad_of(O.reduce_sum(out * w), [v])
    t = _t(x)
    (t.expand(*shape) * torch.tensor(w)).sum().backward()
    _close(g, t.grad.numpy())
    _close(g, w.sum(axis=(0, 1, 3)).reshape(3, 1, 5))
    # a 0-d value goes everywhere and collects everything
    s = O.V(np.array(1.5))
    o0 = O.broadcast_to(s, (3, 2))
    assert o0.a.shape == (3, 2) and (o0.a == 1.5).all()
    w0 = RNG.standard_normal((3, 2))
    (g0,) = O.grad_of(O.reduce_sum(o0 * w0), [s])
    assert g0.shape == () and abs(g0 - w0.sum()) < 1e-12


def test_pad_values_and_sliced_vjp():
    """pad: (before, after) per axis with a constant fill (view/shape.py:1313-1398), checked
    element by element and against torch's F.pad (whose argument order is last axis first);
    the VJP is the window of the cotangent that starts at `before` and has the input's size
    (1385-1390) -- unequal before/after widths, so that swapping them fails."""
    x = RNG.standard_normal((2, 3, 4))
    paddings = [(1, 0), (0, 2), (3, 1)]
    v = O.V(x)
    out = O.pad(v, paddings, value=-2.5)
    assert out.a.shape == (3, 5, 8)
    for i in range(3):
        for j in range(5):
            for k in range(8):
                inside = 1 <= i < 3 and j < 3 and 3 <= k < 7
                assert out.a[i, j, k] == (x[i - 1, j, k - 3] if inside else -2.5)
    t = _t(x)
    tp = TF.pad(t, (3, 1, 0, 2, 1, 0), value=-2.5)
    assert np.array_equal(out.a, tp.detach().numpy())
    w = RNG.standard_normal(out.a.shape)
    (g,) = O.grad_of(O.reduce_sum(out * w), [v])
    (tp * torch.tensor(w)).sum().backward()
    _close(g, t.grad.numpy())
    assert np.array_equal(g, w[1:3, 0:3, 3:7])
    # default fill is zero
    assert O.pad(v, [(0, 1), (0, 0), (0, 0)]).a[2].max() == 0.0


def test_concatenate_values_and_split_vjp():
    """concatenate: pieces of unequal length along a middle axis, in order (view/shape.py:821-980);
    the VJP hands each input its own slab of the cotangent -- checked against torch.cat and
    explicit slices, with three different lengths so that a wrong offset fails."""
    parts = [RNG.standard_normal((2, n, 3)) for n in (1, 4, 2)]
    vs = [O.V(p) for p in parts]
    out = O.concatenate(vs, axis=1)
    assert out.a.shape == (2, 7, 3)
    assert np.array_equal(out.a[:, 0:1], parts[0]) and np.array_equal(out.a[:, 1:5], parts[1]) \
        and np.array_equal(out.a[:, 5:7], parts[2])
    w = RNG.standard_normal(out.a.shape)
    gs = O.grad_of(O.reduce_sum(out * w), vs)
    ts = [_t(p) for p in parts]
    (torch.cat(ts, dim=1) * torch.tensor(w)).sum().backward()
    for g, t in zip(gs, ts):
        _close(g, t.grad.numpy())
    assert np.array_equal(gs[0], w[:, 0:1]) and np.array_equal(gs[1], w[:, 1:5]) and np.array_equal(gs[2], w[:, 5:7])
    # negative axis, and one tensor used twice accumulates both slabs
    o2 = O.concatenate([vs[0], vs[0]], axis=-1)
    assert o2.a.shape == (2, 1, 6)
    w2 = RNG.standard_normal(o2.a.shape)
    (g2,) = O.grad_of(O.reduce_sum(o2 * w2), [vs[0]])
    _close(g2, w2[..., :3] + w2[..., 3:])


def test_torch_steps_agree_with_the_numpy_oracle():
    """oracle/torch_steps.py (the full-size checker of the transformer and decoder steps) against
    oracle/configs.py in float64: loss and every gradient, non-trivial biases, norm weights and
    LoRA B factors so that no term is multiplied by zero or one."""
    from oracle import torch_steps as ts
    rng = np.random.default_rng(11)
    t = oc.c3_inputs(2, 12, 16, 40, seed=5, bf16=False)
    for k in oc.C3_PARAMS:
        if k[0] == "b" or k.startswith("ln"):
            t[k] = (t[k] + 0.3 * rng.standard_normal(t[k].shape)).astype(np.float32)
    wl, wg = oc.c3_reference(t, num_heads=4)
    gl, gg = ts.c3_step(t, num_heads=4)
    assert abs(gl - wl) <= 1e-12 * abs(wl)
    for k in oc.C3_PARAMS:
        _close(gg[k], wg[k], 1e-9)
    t5 = oc.c5_inputs(layers=2, batch=3, seq=10, d_model=24, d_ff=32, vocab=53, rank=4, seed=6,
                      b_zero=False, bf16=False)
    for L in t5["layers"]:
        for k in L:
            if k[0] == "b" or k.startswith("ln"):
                L[k] = (L[k] + 0.3 * rng.standard_normal(L[k].shape)).astype(np.float32)
    wl, wg = oc.c5_reference(t5, num_heads=4, alpha=8.0)
    gl, gg = ts.c5_step(t5, num_heads=4, alpha=8.0)
    assert abs(gl - wl) <= 1e-12 * abs(wl)
    assert len(gg) == len(wg) == 8
    for a, b in zip(gg, wg):
        assert np.abs(b).max() > 0
        _close(a, b, 1e-9)


def test_philox_known_answers():
    """Philox4x32 with 10 rounds against the known-answer vectors of the Random123 library
    (zeros, all ones, and the digits of pi as counter and key)."""
    from oracle.philox import philox4x32_10
    u = lambda *w: np.array(w, dtype=np.uint32)
    cases = [
        (u(0, 0, 0, 0), u(0, 0), u(0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
        (u(*[0xFFFFFFFF] * 4), u(0xFFFFFFFF, 0xFFFFFFFF), u(0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
        (u(0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), u(0xA4093822, 0x299F31D0),
         u(0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
    ]
    for ctr, key, want in cases:
        np.testing.assert_array_equal(philox4x32_10(ctr, key), want)
    # vectorised over a batch of counters, the same words come out
    ctrs = np.stack([c for c, _, _ in cases[:1]] * 3)
    np.testing.assert_array_equal(philox4x32_10(ctrs, cases[0][1][None, :]), np.stack([cases[0][2]] * 3))


def test_philox_streams_are_disjoint_and_uniform():
    """Streams, runs and seeds give different words; the unit floats fill [0, 1) evenly and the
    Box-Muller values have unit variance."""
    from oracle import philox
    base = philox.words(4096, 1, 0, 0)
    for other in (philox.words(4096, 2, 0, 0), philox.words(4096, 1, 1, 0), philox.words(4096, 1, 0, 1)):
        assert (base == other).mean() < 0.01
    u = philox.unit_floats(philox.words(1 << 18, 3, 0, 0))
    hist = np.histogram(u, bins=16, range=(0.0, 1.0))[0] / u.size
    assert np.abs(hist - 1.0 / 16).max() < 2e-3
    z = philox.normal(1 << 18, 0.0, 1.0, 3, 0, 0)
    assert abs(z.mean()) < 5e-3 and abs(z.std() - 1.0) < 5e-3
