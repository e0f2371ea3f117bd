"""Writes the golden vectors under tests/golden/ (run: python tests/golden/make_fixtures.py).

Inputs are seeded numpy arrays; expected outputs come from float64 torch autograd on formulas
written out here from the reference's definitions (file:line cited per block), independently
of ``oracle/`` and of the package under test, so that the same vectors pin both.  Nothing from
the reference is imported or executed.  Sizes are tiny: the whole set is a few hundred KB.
"""
from __future__ import annotations

import math
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
f64 = torch.float64


def tt(a, grad=False):
    return torch.tensor(np.asarray(a, dtype=np.float64), dtype=f64, requires_grad=grad)


def save(name, **arrays):
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    print(name, {k: v.shape for k, v in arrays.items()})


# ---------------------------------------------------------------- building blocks (torch fp64)
def layer_norm(x, w, b, eps=1e-5):
    # nabla/nn/functional/layers.py:38-56: biased variance, eps inside the rsqrt
    mu = x.mean(-1, keepdim=True)
    c = x - mu
    var = (c * c).mean(-1, keepdim=True)
    return c * torch.rsqrt(var + eps) * w + b


def gelu(x):
    # nabla/ops/unary.py:574-595: exact erf form
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def attention(q, k, v, causal):
    # nabla/nn/functional/layers.py:106-153: scale after the product, mask value -1e9
    s = (q @ k.transpose(-2, -1)) * (1.0 / math.sqrt(q.shape[-1]))
    if causal:
        m = torch.tril(torch.ones(q.shape[-2], k.shape[-2], dtype=f64)) > 0
        s = torch.where(m, s, torch.full_like(s, -1e9))
    return torch.softmax(s, -1) @ v


def block(x, p, heads, lora=None, alpha=16.0):
    # nabla/nn/modules/transformer.py:64-82 (pre-LN), attention.py:58-107, lora.py:55-79
    b, s, d = x.shape
    hd = d // heads
    split = lambda z: z.reshape(b, s, heads, hd).transpose(1, 2)
    h = layer_norm(x, p["ln1_w"], p["ln1_b"])

    def proj(name):
        y = h @ p["w" + name]
        if lora is not None and name + "A" in lora:
            A, B = lora[name + "A"], lora[name + "B"]
            y = y + h @ ((A @ B) * (alpha / A.shape[1]))
        return y + p["b" + name]

    a = attention(split(proj("q")), split(proj("k")), split(proj("v")), True)
    a = a.transpose(1, 2).reshape(b, s, d)
    x = x + a @ p["wo"] + p["bo"]
    h = layer_norm(x, p["ln2_w"], p["ln2_b"])
    return x + gelu(h @ p["w1"] + p["b1"]) @ p["w2"] + p["b2"]


def cross_entropy(logits, labels):
    # nabla/nn/functional/losses.py:20-44: -sum(onehot * logsoftmax) / logits.shape[0]
    lsm = torch.log_softmax(logits, -1)
    picked = torch.gather(lsm, -1, labels.unsqueeze(-1)).squeeze(-1)
    return -picked.sum() / logits.shape[0]


def conv_nhwc(x, w, bias, stride, pad):
    # nabla/ops/convolution.py:220-252: NHWC x HWIO, padding (top, bottom, left, right)
    pt, pb, pl, pr = pad
    xp = F.pad(x.permute(0, 3, 1, 2), (pl, pr, pt, pb))
    y = F.conv2d(xp, w.permute(3, 2, 0, 1), stride=stride).permute(0, 2, 3, 1)
    return y if bias is None else y + bias


# ---------------------------------------------------------------- configurations (reduced)
def fixture_c1():
    rng = np.random.default_rng(101)
    u = lambda *s: rng.uniform(-0.05, 0.05, s).astype(np.float32)
    t = {"x": u(8, 12), "W1": u(12, 6), "b1": u(1, 6), "W2": u(6, 3), "b2": u(1, 3)}
    p = {k: tt(t[k], True) for k in ("W1", "b1", "W2", "b2")}
    loss = (torch.relu(tt(t["x"]) @ p["W1"] + p["b1"]) @ p["W2"] + p["b2"]).mean()
    loss.backward()
    save("c1_mlp", **{"in_" + k: v for k, v in t.items()}, loss=np.float64(loss.item()),
         **{"g_" + k: p[k].grad.numpy() for k in p})


def fixture_c2():
    rng = np.random.default_rng(102)
    x = rng.standard_normal((6, 72)).astype(np.float32)
    y = rng.standard_normal((6, 72)).astype(np.float32)
    X = tt(x, True)
    prod = X * tt(y)
    out = (torch.exp(prod - prod.max(1, keepdim=True).values) * torch.relu(X)).sum(1)
    out.sum().backward()
    save("c2_stress", in_x=x, in_y=y, out=out.detach().numpy(), g_x=X.grad.numpy())


C3_KEYS = ["wq", "bq", "wk", "bk", "wv", "bv", "wo", "bo", "w1", "b1", "w2", "b2",
           "ln1_w", "ln1_b", "ln2_w", "ln2_b"]


def _block_params(rng, d, ff):
    n = lambda std, *s: (rng.standard_normal(s) * std).astype(np.float32)
    t = {k: n(0.2, d, d) for k in ("wq", "wk", "wv", "wo")}
    t["w1"], t["w2"] = n(0.2, d, ff), n(0.2, ff, d)
    for k, w in (("bq", d), ("bk", d), ("bv", d), ("bo", d), ("b1", ff), ("b2", d)):
        t[k] = n(0.1, 1, w)
    t["ln1_w"], t["ln2_w"] = 1.0 + n(0.1, d), 1.0 + n(0.1, d)
    t["ln1_b"], t["ln2_b"] = n(0.1, d), n(0.1, d)
    return t


def fixture_c3():
    rng = np.random.default_rng(103)
    d, ff, heads = 16, 32, 2
    t = _block_params(rng, d, ff)
    t["x"] = rng.standard_normal((2, 8, d)).astype(np.float32)
    p = {k: tt(t[k], True) for k in C3_KEYS}
    out = block(tt(t["x"]), p, heads)
    loss = (out * out).mean()
    loss.backward()
    save("c3_block", **{"in_" + k: v for k, v in t.items()}, heads=np.int64(heads),
         loss=np.float64(loss.item()), out=out.detach().numpy(),
         **{"g_" + k: p[k].grad.numpy() for k in C3_KEYS})


def fixture_c4():
    rng = np.random.default_rng(104)
    c = (3, 4, 6, 8)
    kaiming = lambda *s: (rng.standard_normal(s) * math.sqrt(2.0 / (s[0] * s[1] * s[2]))).astype(np.float32)
    t = {"img": rng.uniform(0, 1, (2, 8, 8, c[0])).astype(np.float32),
         "k1": kaiming(3, 3, c[0], c[1]), "k2": kaiming(3, 3, c[1], c[2]), "k3": kaiming(3, 3, c[2], c[3]),
         "c1b": (rng.standard_normal(c[1]) * 0.1).astype(np.float32),
         "c2b": (rng.standard_normal(c[2]) * 0.1).astype(np.float32),
         "c3b": (rng.standard_normal(c[3]) * 0.1).astype(np.float32),
         "wl": (rng.standard_normal((c[3], 5)) * 0.5).astype(np.float32),
         "bl": (rng.standard_normal((1, 5)) * 0.1).astype(np.float32),
         "labels": rng.integers(0, 5, (2,)).astype(np.int64)}
    keys = ["k1", "c1b", "k2", "c2b", "k3", "c3b", "wl", "bl"]
    p = {k: tt(t[k], True) for k in keys}
    pad = (1, 1, 1, 1)
    h = torch.relu(conv_nhwc(tt(t["img"]), p["k1"], p["c1b"], (1, 1), pad))
    h = torch.relu(conv_nhwc(h, p["k2"], p["c2b"], (1, 1), pad))
    h = F.max_pool2d(h.permute(0, 3, 1, 2), 2).permute(0, 2, 3, 1)
    h = torch.relu(conv_nhwc(h, p["k3"], p["c3b"], (1, 1), pad))
    logits = h.mean((1, 2)) @ p["wl"] + p["bl"]
    loss = cross_entropy(logits, torch.tensor(t["labels"]))
    loss.backward()
    save("c4_cnn", **{"in_" + k: v for k, v in t.items()}, loss=np.float64(loss.item()),
         logits=logits.detach().numpy(), argmax=logits.argmax(-1).numpy().astype(np.int64),
         **{"g_" + k: p[k].grad.numpy() for k in keys})


def fixture_c5():
    rng = np.random.default_rng(105)
    d, ff, heads, vocab, rank, layers = 16, 32, 2, 20, 2, 2
    n = lambda std, *s: (rng.standard_normal(s) * std).astype(np.float32)
    ids = rng.integers(0, vocab, (1, 8)).astype(np.int64)
    arrays = {"in_ids": ids, "in_embed": n(0.5, vocab, d), "in_head": n(0.3, d, vocab),
              "in_lnf_w": 1.0 + n(0.1, d), "in_lnf_b": n(0.1, d), "heads": np.int64(heads),
              "layers": np.int64(layers), "alpha": np.float64(4.0)}
    x = tt(arrays["in_embed"])[torch.tensor(ids)]
    lora_leaves = []
    for li in range(layers):
        t = _block_params(rng, d, ff)
        ad = {"qA": n(0.3, d, rank), "qB": n(0.3, rank, d), "vA": n(0.3, d, rank), "vB": n(0.3, rank, d)}
        for k, v in t.items():
            arrays[f"in_L{li}_{k}"] = v
        for k, v in ad.items():
            arrays[f"in_A{li}_{k}"] = v
        lt = {k: tt(v, True) for k, v in ad.items()}
        lora_leaves.append(lt)
        x = block(x, {k: tt(v) for k, v in t.items()}, heads, lora=lt, alpha=4.0)
    logits = layer_norm(x, tt(arrays["in_lnf_w"]), tt(arrays["in_lnf_b"])) @ tt(arrays["in_head"])
    loss = cross_entropy(logits, torch.tensor(ids))   # divides by the batch size (1), not by tokens
    loss.backward()
    arrays["loss"] = np.float64(loss.item())
    for li, lt in enumerate(lora_leaves):
        for k, v in lt.items():
            arrays[f"g_A{li}_{k}"] = v.grad.numpy()
    save("c5_lora", **arrays)


# ---------------------------------------------------------------- single kernels, awkward cases
def fixture_attention_bf16():
    """Causal attention on bfloat16 inputs (stored as their 16-bit patterns) with float64
    results (stored as float16: the comparison tolerance for bf16 kernels is 2e-2): output,
    log-sum-exp of the score rows and the three gradients for a given d(output).  This is the
    shape class the fused attention kernels take (head size 64, S a multiple of 128)."""
    rng = np.random.default_rng(6)
    shape = (1, 1, 128, 64)                                    # [B, H, S, hd]
    bits = {}
    vals = {}
    for name in ("q", "k", "v", "g"):
        t = torch.tensor(rng.standard_normal(shape), dtype=torch.float32).to(torch.bfloat16)
        bits[name] = t.view(torch.int16).numpy().view(np.uint16)
        vals[name] = t.to(f64)
    q, k, v = (vals[n].clone().requires_grad_(True) for n in ("q", "k", "v"))
    o = attention(q, k, v, causal=True)
    s = (q @ k.transpose(-2, -1)) / math.sqrt(shape[-1])
    s = s.masked_fill(~(torch.tril(torch.ones(shape[-2], shape[-2])) > 0), float("-inf"))
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), vals["g"])
    h = lambda t: t.detach().numpy().astype(np.float16)
    save("attention_bf16", **{"in_" + n + "_bf16_bits": b for n, b in bits.items()},
         o=h(o), lse=torch.logsumexp(s, -1).detach().numpy().astype(np.float32), dq=h(dq), dk=h(dk), dv=h(dv))


def fixture_kernels():
    rng = np.random.default_rng(106)
    # conv2d with stride (2, 1) and asymmetric padding (tests/unit test_convolution.py:51-195 shapes)
    x = rng.standard_normal((2, 7, 9, 3)).astype(np.float32)
    w = rng.standard_normal((3, 2, 3, 4)).astype(np.float32)
    X, W = tt(x, True), tt(w, True)
    y = conv_nhwc(X, W, None, (2, 1), (1, 0, 2, 1))
    (y * y).sum().backward()
    # max_pool2d 2x2 stride 2 on tie-free data, with the gradient of sum(y^2)
    pin = rng.permutation(2 * 6 * 6 * 3).reshape(2, 6, 6, 3).astype(np.float32)
    P = tt(pin, True)
    py = F.max_pool2d(P.permute(0, 3, 1, 2), 2).permute(0, 2, 3, 1)
    (py * py).sum().backward()
    # argmax with ties (lowest index wins) and gather of rows
    am = np.array([[1, 3, 3, 2], [5, 5, 5, 5], [0, -1, 7, 7], [-2, -2, -3, -2]], np.float32)
    table = rng.standard_normal((11, 5)).astype(np.float32)
    idx = rng.integers(0, 11, (2, 4)).astype(np.int64)
    # softmax / logsoftmax rows and layer_norm with their gradients
    s = rng.standard_normal((3, 10)).astype(np.float32)
    S = tt(s, True)
    sm = torch.softmax(S, -1)
    (sm * tt(np.arange(10))).sum().backward()
    lw, lb = rng.standard_normal(10).astype(np.float32), rng.standard_normal(10).astype(np.float32)
    S2, LW, LB = tt(s, True), tt(lw, True), tt(lb, True)
    ln = layer_norm(S2, LW, LB)
    (ln * ln * tt(np.arange(10) / 10.0)).sum().backward()
    save("kernels", conv_x=x, conv_w=w, conv_y=y.detach().numpy(), conv_gx=X.grad.numpy(),
         conv_gw=W.grad.numpy(), pool_x=pin, pool_y=py.detach().numpy(), pool_gx=P.grad.numpy(),
         argmax_x=am, argmax_y=np.array([1, 0, 2, 0], np.int64), gather_table=table, gather_idx=idx,
         gather_y=table[idx], sm_x=s, sm_y=sm.detach().numpy(), sm_gx=S.grad.numpy(),
         lsm_y=torch.log_softmax(tt(s), -1).numpy(), ln_w=lw, ln_b=lb, ln_y=ln.detach().numpy(),
         ln_gx=S2.grad.numpy(), ln_gw=LW.grad.numpy(), ln_gb=LB.grad.numpy())


if __name__ == "__main__":
    torch.manual_seed(0)
    fixture_c1()
    fixture_c2()
    fixture_c3()
    fixture_c4()
    fixture_c5()
    fixture_kernels()
    fixture_attention_bf16()
