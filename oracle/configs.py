"""TEST INFRASTRUCTURE -- the five benchmark configurations as (inputs, oracle
result, program) triples.

``*_inputs`` build the seeded synthetic inputs (numpy ``default_rng(seed)``,
generated on the host), ``*_reference`` evaluates the step with the fp64 oracle
of ``oracle.ops``, and ``*_program`` runs the same step of the package under
test (its ``workloads`` module; the package is passed in as ``nb`` so that
nothing here imports the product).  Sizes default to the full configuration and can be
reduced for parity tests.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from . import ops as O


def to_bf16_grid(a: np.ndarray) -> np.ndarray:
    """Round to the nearest bfloat16 value, returned as float32."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).float().numpy()


# ------------------------------------------------------------------ C1: MLP
def c1_inputs(batch=128, d_in=784, d_hidden=256, d_out=10, seed=0) -> dict:
    rng = np.random.default_rng(seed)
    u = lambda *s: rng.uniform(-0.05, 0.05, s).astype(np.float32)
    return {
        "x": u(batch, d_in), "W1": u(d_in, d_hidden), "b1": np.zeros((1, d_hidden), np.float32),
        "W2": u(d_hidden, d_out), "b2": np.zeros((1, d_out), np.float32),
    }


def c1_reference(x, W1, b1, W2, b2, dtype=np.float64):
    p = {k: O.V(v.astype(dtype)) for k, v in dict(W1=W1, b1=b1, W2=W2, b2=b2).items()}
    loss = O.mean(O.relu(O.V(x.astype(dtype)) @ p["W1"] + p["b1"]) @ p["W2"] + p["b2"])
    grads = O.grad_of(loss, [p["W1"], p["b1"], p["W2"], p["b2"]])
    return float(loss.a), grads


def c1_program(nb, t: dict):
    return nb.workloads.c1_step(t)


# ------------------------------------- C2: elementwise + reduction stress
def c2_inputs(rows=8192, cols=8192, seed=0) -> dict:
    rng = np.random.default_rng(seed)
    return {"x": rng.standard_normal((rows, cols), dtype=np.float32),
            "y": rng.standard_normal((rows, cols), dtype=np.float32)}


def c2_reference(x, y, dtype=np.float64):
    X, Y = O.V(x.astype(dtype)), O.V(y.astype(dtype))
    p = X * Y
    m = O.reduce_max(p, axis=1, keepdims=True)
    out = O.reduce_sum(O.exp(p - m) * O.relu(X), axis=1)
    (gx,) = O.grad_of(O.reduce_sum(out), [X])
    return out.a, gx


def c2_chain(nb, X, Y):
    return nb.workloads.c2_chain(X, Y)


def c2_program(nb, X, Y):
    """out and d(sum(out))/dx, both lazy."""
    return nb.workloads.c2_step(X, Y)


# ------------------------------------------------- C3: transformer block
C3_PARAMS = ["wq", "bq", "wk", "bk", "wv", "bv", "wo", "bo", "w1", "b1", "w2", "b2",
             "ln1_w", "ln1_b", "ln2_w", "ln2_b"]


def c3_inputs(batch=8, seq=1024, d_model=1024, d_ff=4096, seed=0, bf16=True) -> dict:
    rng = np.random.default_rng(seed)
    n = lambda std, *s: (rng.standard_normal(s) * std).astype(np.float32)
    t = {"x": n(1.0, batch, seq, d_model)}
    for k in ("wq", "wk", "wv", "wo"):
        t[k] = n(0.02, d_model, d_model)
    t["w1"] = n(0.02, d_model, d_ff)
    t["w2"] = n(0.02, d_ff, d_model)
    for k, d in (("bq", d_model), ("bk", d_model), ("bv", d_model), ("bo", d_model),
                 ("b1", d_ff), ("b2", d_model)):
        t[k] = np.zeros((1, d), np.float32)
    for k in ("ln1_w", "ln2_w"):
        t[k] = np.ones((d_model,), np.float32)
    for k in ("ln1_b", "ln2_b"):
        t[k] = np.zeros((d_model,), np.float32)
    if bf16:
        t = {k: to_bf16_grid(v) for k, v in t.items()}
    return t


def c3_reference(t: dict, num_heads=16, dtype=np.float64):
    p = {k: O.V(t[k].astype(dtype)) for k in C3_PARAMS}
    out = O.transformer_encoder_layer(O.V(t["x"].astype(dtype)), p, num_heads, is_causal=True)
    loss = O.mean(out * out)
    grads = O.grad_of(loss, [p[k] for k in C3_PARAMS])
    return float(loss.a), dict(zip(C3_PARAMS, grads))


def c3_block(nb, x, p: dict, num_heads: int):
    return nb.workloads.transformer_block(x, p, num_heads)


def c3_program(nb, t: dict, num_heads=16):
    return nb.workloads.c3_step(t, num_heads)


# -------------------------------------------------------------- C4: CNN step
C4_PARAMS = ["k1", "c1b", "k2", "c2b", "k3", "c3b", "wl", "bl"]


def c4_inputs(batch=64, hw=32, c=(3, 64, 128, 256), classes=10, seed=0) -> dict:
    rng = np.random.default_rng(seed)
    kaiming = lambda *s: (rng.standard_normal(s) * math.sqrt(2.0 / (s[0] * s[1] * s[2]))).astype(np.float32)
    t = {"img": rng.uniform(0, 1, (batch, hw, hw, c[0])).astype(np.float32)}
    t["k1"], t["k2"], t["k3"] = kaiming(3, 3, c[0], c[1]), kaiming(3, 3, c[1], c[2]), kaiming(3, 3, c[2], c[3])
    t["c1b"], t["c2b"], t["c3b"] = (np.zeros((n,), np.float32) for n in c[1:])
    t["wl"] = (rng.standard_normal((c[3], classes)) * math.sqrt(2.0 / c[3])).astype(np.float32)
    t["bl"] = np.zeros((1, classes), np.float32)
    t["labels"] = rng.integers(0, classes, (batch,)).astype(np.int64)
    return t


def c4_reference(t: dict, dtype=np.float64):
    p = {k: O.V(t[k].astype(dtype)) for k in C4_PARAMS}
    pad = (1, 1, 1, 1)
    h = O.relu(O.conv2d(O.V(t["img"].astype(dtype)), p["k1"], p["c1b"], padding=pad))
    h = O.relu(O.conv2d(h, p["k2"], p["c2b"], padding=pad))
    h = O.max_pool2d(h, (2, 2))
    h = O.relu(O.conv2d(h, p["k3"], p["c3b"], padding=pad))
    h = O.mean(h, axis=(1, 2))
    logits = O.linear(h, p["wl"], p["bl"])
    loss = O.cross_entropy_loss(logits, t["labels"])
    grads = O.grad_of(loss, [p[k] for k in C4_PARAMS])
    return float(loss.a), dict(zip(C4_PARAMS, grads)), O.argmax(logits, -1), logits.a


def c4_logits(nb, p: dict, img):
    return nb.workloads.c4_logits(p, img)


def c4_program(nb, t: dict):
    return nb.workloads.c4_step(t)


# ------------------------------------------------------ C5: LoRA decoder step
def c5_inputs(layers=12, batch=4, seq=2048, d_model=2048, d_ff=8192, vocab=32000, rank=16,
              seed=0, b_zero=True, bf16=True) -> dict:
    rng = np.random.default_rng(seed)
    n = lambda std, *s: (rng.standard_normal(s, dtype=np.float32) * np.float32(std))
    t = {"ids": rng.integers(0, vocab, (batch, seq)).astype(np.int64),
         "embed": n(0.02, vocab, d_model), "head": n(0.02, d_model, vocab),
         "lnf_w": np.ones((d_model,), np.float32), "lnf_b": np.zeros((d_model,), np.float32),
         "layers": [], "lora": []}
    for _ in range(layers):
        L = {k: n(0.02, d_model, d_model) for k in ("wq", "wk", "wv", "wo")}
        L["w1"], L["w2"] = n(0.02, d_model, d_ff), n(0.02, d_ff, d_model)
        for k, d in (("bq", d_model), ("bk", d_model), ("bv", d_model), ("bo", d_model),
                     ("b1", d_ff), ("b2", d_model)):
            L[k] = np.zeros((1, d), np.float32)
        L["ln1_w"], L["ln2_w"] = np.ones((d_model,), np.float32), np.ones((d_model,), np.float32)
        L["ln1_b"], L["ln2_b"] = np.zeros((d_model,), np.float32), np.zeros((d_model,), np.float32)
        t["layers"].append(L)
        ad = {}
        for proj in ("q", "v"):
            ad[proj + "A"] = n(0.02, d_model, rank)
            ad[proj + "B"] = np.zeros((rank, d_model), np.float32) if b_zero else n(0.02, rank, d_model)
        t["lora"].append(ad)
    if bf16:
        r = to_bf16_grid
        t["embed"], t["head"] = r(t["embed"]), r(t["head"])
        t["layers"] = [{k: r(v) for k, v in L.items()} for L in t["layers"]]
        t["lora"] = [{k: r(v) for k, v in a.items()} for a in t["lora"]]
    return t


def c5_reference(t: dict, num_heads=16, alpha=16.0, dtype=np.float64):
    conv = lambda a: O.V(a.astype(dtype))
    lora = [{k: conv(v) for k, v in a.items()} for a in t["lora"]]
    x = O.gather(conv(t["embed"]), O.V(t["ids"]), axis=0)
    b, s, d = x.a.shape
    hd = d // num_heads
    heads = lambda z: O.swap_axes(O.reshape(z, (b, s, num_heads, hd)), 1, 2)
    for L, ad in zip(t["layers"], lora):
        p = {k: conv(v) for k, v in L.items()}
        normed = O.layer_norm(x, p["ln1_w"], p["ln1_b"])
        q = heads(O.lora_linear(normed, p["wq"], ad["qA"], ad["qB"], alpha) + p["bq"])
        k = heads(O.linear(normed, p["wk"], p["bk"]))
        v = heads(O.lora_linear(normed, p["wv"], ad["vA"], ad["vB"], alpha) + p["bv"])
        a = O.scaled_dot_product_attention(q, k, v, is_causal=True)
        a = O.reshape(O.swap_axes(a, 1, 2), (b, s, d))
        x = x + O.linear(a, p["wo"], p["bo"])
        normed = O.layer_norm(x, p["ln2_w"], p["ln2_b"])
        x = x + O.linear(O.gelu(O.linear(normed, p["w1"], p["b1"])), p["w2"], p["b2"])
    x = O.layer_norm(x, conv(t["lnf_w"]), conv(t["lnf_b"]))
    logits = O.matmul(x, conv(t["head"]))
    loss = O.cross_entropy_loss(logits, t["ids"])
    flat = [ad[k] for ad in lora for k in ("qA", "qB", "vA", "vB")]
    grads = O.grad_of(loss, flat)
    return float(loss.a), grads


def c5_program(nb, t: dict, num_heads=16, alpha=16.0):
    """``t`` holds tensors of the package under test in the same nesting as c5_inputs."""
    return nb.workloads.c5_step(t, num_heads, alpha)


def upload(nb, tree, dtype=None):
    """numpy tree -> tensors of the package under test (float leaves cast to ``dtype``)."""
    if isinstance(tree, dict):
        return {k: upload(nb, v, dtype) for k, v in tree.items()}
    if isinstance(tree, list):
        return [upload(nb, v, dtype) for v in tree]
    if np.issubdtype(tree.dtype, np.floating):
        return nb.Tensor.constant(tree, dtype=dtype)
    return nb.Tensor.constant(tree)
