"""The five synthetic step programs the backend is measured on, written against
the public API exactly as a user of the reference would write them.

Each ``*_step`` takes tensors and returns lazy results (loss / outputs and
gradients); nothing here touches data or timing.  ``*_shapes`` describe the
leaf tensors of the full-size configuration.
"""
from __future__ import annotations

import nabla_amd as nb

F = nb.nn.functional

C3_PARAMS = ["wq", "bq", "wk", "bk", "wv", "bv", "wo", "bo", "w1", "b1", "w2", "b2",
             "ln1_w", "ln1_b", "ln2_w", "ln2_b"]
C4_PARAMS = ["k1", "c1b", "k2", "c2b", "k3", "c3b", "wl", "bl"]


# ---- C1: 2-layer MLP ------------------------------------------------------------
def c1_step(t: dict):
    def loss_fn(W1, b1, W2, b2, x):
        return nb.mean(nb.relu(x @ W1 + b1) @ W2 + b2)

    return nb.value_and_grad(loss_fn, argnums=(0, 1, 2, 3))(t["W1"], t["b1"], t["W2"], t["b2"], t["x"])


# ---- C2: elementwise + reduction stress ---------------------------------------------
def c2_chain(X, Y):
    p = X * Y
    m = nb.reduce_max(p, axis=1, keepdims=True)
    return nb.reduce_sum(nb.exp(p - m) * nb.relu(X), axis=1)


def c2_step(X, Y):
    """``out`` and the gradient of ``sum(out)`` w.r.t. ``x``."""
    out = c2_chain(X, Y)
    gx = nb.grad(lambda X, Y: nb.reduce_sum(c2_chain(X, Y)), argnums=0)(X, Y)
    return out, gx


# ---- C3: pre-LN transformer block -----------------------------------------------------
def transformer_block(x, p: dict, num_heads: int, lora=None, alpha: float = 16.0):
    """nn.TransformerEncoderLayer semantics (causal, dropout 0) on explicit
    parameter dicts; ``lora`` adds LoRA adapters on the Q and V projections."""
    b, s, d = x.shape
    hd = d // num_heads

    def heads(t):
        return nb.swap_axes(nb.reshape(t, (b, s, num_heads, hd)), 1, 2)

    normed = F.layer_norm(x, p["ln1_w"], p["ln1_b"])
    if lora is None:
        q = F.linear(normed, p["wq"], p["bq"])
        v = F.linear(normed, p["wv"], p["bv"])
    else:
        ll = nb.nn.finetune.lora_linear
        q = ll(normed, p["wq"], {"A": lora["qA"], "B": lora["qB"]}, alpha=alpha) + p["bq"]
        v = ll(normed, p["wv"], {"A": lora["vA"], "B": lora["vB"]}, alpha=alpha) + p["bv"]
    k = F.linear(normed, p["wk"], p["bk"])
    a = F.scaled_dot_product_attention(heads(q), heads(k), heads(v), is_causal=True)
    a = nb.reshape(nb.swap_axes(a, 1, 2), (b, s, d))
    x = x + F.linear(a, p["wo"], p["bo"])
    normed = F.layer_norm(x, p["ln2_w"], p["ln2_b"])
    ff = F.linear(nb.gelu(F.linear(normed, p["w1"], p["b1"])), p["w2"], p["b2"])
    return x + ff


def c3_step(t: dict, num_heads: int = 16):
    def loss_fn(params, x):
        out = transformer_block(x, params, num_heads)
        return nb.mean(out * out)

    return nb.value_and_grad(loss_fn, argnums=0)({k: t[k] for k in C3_PARAMS}, t["x"])


# ---- C4: CNN step ---------------------------------------------------------------------
def c4_logits(p: dict, img):
    h = nb.relu(nb.conv2d(img, p["k1"], padding=1, bias=p["c1b"]))
    h = nb.relu(nb.conv2d(h, p["k2"], padding=1, bias=p["c2b"]))
    h = nb.max_pool2d(h, kernel_size=2)
    h = nb.relu(nb.conv2d(h, p["k3"], padding=1, bias=p["c3b"]))
    h = nb.mean(h, axis=(1, 2))
    return F.linear(h, p["wl"], p["bl"])


def c4_step(t: dict):
    def loss_fn(params, img, labels):
        return F.cross_entropy_loss(c4_logits(params, img), labels)

    return nb.value_and_grad(loss_fn, argnums=0)({k: t[k] for k in C4_PARAMS}, t["img"], t["labels"])


# ---- C5: LoRA fine-tune step on a decoder stack ----------------------------------------
def c5_step(t: dict, num_heads: int = 16, alpha: float = 16.0):
    def loss_fn(lora, base, ids):
        x = F.embedding(ids, base["embed"])
        for L, ad in zip(base["layers"], lora):
            x = transformer_block(x, L, num_heads, lora=ad, alpha=alpha)
        x = F.layer_norm(x, base["lnf_w"], base["lnf_b"])
        return F.cross_entropy_loss(x @ base["head"], ids)

    base = {k: t[k] for k in ("embed", "head", "lnf_w", "lnf_b", "layers")}
    return nb.value_and_grad(loss_fn, argnums=0)(t["lora"], base, t["ids"])


# ---- leaf shapes of the full-size configurations ------------------------------------------
def _block_shapes(d: int, ff: int) -> dict:
    s = {k: (d, d) for k in ("wq", "wk", "wv", "wo")}
    s.update(w1=(d, ff), w2=(ff, d), b1=(1, ff), b2=(1, d))
    s.update({k: (1, d) for k in ("bq", "bk", "bv", "bo")})
    s.update({k: (d,) for k in ("ln1_w", "ln1_b", "ln2_w", "ln2_b")})
    return s


def c1_shapes():
    return {"x": (128, 784), "W1": (784, 256), "b1": (1, 256), "W2": (256, 10), "b2": (1, 10)}


def c2_shapes(rows=8192, cols=8192):
    return {"x": (rows, cols), "y": (rows, cols)}


def c3_shapes(batch=8, seq=1024, d=1024, ff=4096):
    return dict(_block_shapes(d, ff), x=(batch, seq, d))


def c4_shapes(batch=64, hw=32, c=(3, 64, 128, 256), classes=10):
    return {"img": (batch, hw, hw, c[0]), "k1": (3, 3, c[0], c[1]), "k2": (3, 3, c[1], c[2]),
            "k3": (3, 3, c[2], c[3]), "c1b": (c[1],), "c2b": (c[2],), "c3b": (c[3],),
            "wl": (c[3], classes), "bl": (1, classes), "labels": (batch,)}


def c5_shapes(layers=12, batch=4, seq=2048, d=2048, ff=8192, vocab=32000, rank=16):
    return {"ids": (batch, seq), "embed": (vocab, d), "head": (d, vocab), "lnf_w": (d,), "lnf_b": (d,),
            "layers": [_block_shapes(d, ff) for _ in range(layers)],
            "lora": [{"qA": (d, rank), "qB": (rank, d), "vA": (d, rank), "vB": (rank, d)}
                     for _ in range(layers)]}


# ---- synthetic inputs of the five configurations ---------------------------------------------
def synthetic_inputs(config: str, seed: int = 0, **size):
    """Seeded random leaf tensors for ``c1`` .. ``c5`` (sizes default to the full configuration;
    keyword arguments go to the matching ``*_shapes``).  Weights are small normals (uniform for
    the MLP, fan-in scaled for the CNN), biases zero, layer-norm weights one, LoRA ``B`` factors
    zero as at the start of fine-tuning; the transformer and LoRA configurations are bfloat16."""
    import math

    import numpy as np

    from .core.dtype import DType

    rng = np.random.default_rng(seed)
    shapes = {"c1": c1_shapes, "c2": c2_shapes, "c3": c3_shapes, "c4": c4_shapes, "c5": c5_shapes}[config](**size)
    float_dtype = DType.bfloat16 if config in ("c3", "c5") else DType.float32

    def leaf(name: str, shape):
        if name in ("ids", "labels"):
            hi = size.get("vocab", 32000) if name == "ids" else size.get("classes", 10)
            return nb.Tensor.constant(rng.integers(0, hi, shape).astype(np.int64))
        if name.startswith("b") or (name.endswith("b") and name[0] in "cl") or name in ("qB", "vB"):
            a = np.zeros(shape, np.float32)                      # biases, ln*_b, c*b, LoRA B
        elif name.startswith("ln") or name == "lnf_w":
            a = np.ones(shape, np.float32)                       # layer-norm weights
        elif config == "c1":
            a = rng.uniform(-0.05, 0.05, shape).astype(np.float32)
        elif name == "img":
            a = rng.uniform(0.0, 1.0, shape).astype(np.float32)
        elif config == "c4":
            a = (rng.standard_normal(shape) * math.sqrt(2.0 / math.prod(shape[:-1]))).astype(np.float32)
        elif name in ("x", "y"):
            a = rng.standard_normal(shape, dtype=np.float32)
        else:
            a = rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)
        return nb.Tensor.constant(a, dtype=float_dtype)

    def build(tree, name=""):
        if isinstance(tree, dict):
            return {k: build(v, k) for k, v in tree.items()}
        if isinstance(tree, list):
            return [build(v, name) for v in tree]
        return leaf(name, tree)

    return build(shapes)
