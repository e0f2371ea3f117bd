"""TEST INFRASTRUCTURE -- the transformer-block and LoRA-decoder steps on torch-CPU autograd.

``oracle.configs.c3_reference`` / ``c5_reference`` (numpy, one core for everything that is
not a matrix product) need minutes at the full benchmark sizes; the same two steps written
here on torch's CPU tensors run on all host cores and skip the products whose results nobody
asks for (gradients of frozen weights), which brings a full-size check down to seconds.  The
formulas are the reference's, restated (never imported):

  layer_norm   nabla/nn/functional/layers.py:38-56   biased variance, eps inside the rsqrt
  attention    nabla/nn/functional/layers.py:106-153 scale after the product, mask value -1e9
  gelu         nabla/ops/unary.py:567-595            exact erf form
  block        nabla/nn/modules/transformer.py:64-82 pre-LN; heads via reshape + swap_axes(1, 2)
               (modules/attention.py:58-107); Linear is x @ W + b with W (in, out)
  lora_linear  nabla/nn/finetune/lora.py:55-79       x @ W + x @ ((A @ B) * (alpha / rank))
  loss         nabla/nn/functional/losses.py:20-44   -sum(onehot * logsoftmax) / logits.shape[0]

Pinned by tests/test_oracle_pins.py::test_torch_steps_agree_with_the_numpy_oracle: in float64
both steps agree with ``oracle.configs`` (which is itself pinned against independent golden
vectors and closed forms) to 1e-9 on reduced sizes, loss and every gradient.
"""
from __future__ import annotations

import math

import numpy as np
import torch

C3_PARAMS = ["wq", "bq", "wk", "bk", "wv", "bv", "wo", "bo", "w1", "b1", "w2", "b2",
             "ln1_w", "ln1_b", "ln2_w", "ln2_b"]


def _layer_norm(x, w, b, eps=1e-5):
    mu = x.mean(-1, keepdim=True)
    c = x - mu
    var = (c * c).mean(-1, keepdim=True)
    return c * torch.rsqrt(var + eps) * w + b


def _gelu(x):
    return x * (0.5 * (1.0 + torch.erf(x * (1.0 / math.sqrt(2.0)))))


def _causal_attention(q, k, v):
    s = (q @ k.transpose(-2, -1)) * (1.0 / math.sqrt(q.shape[-1]))
    keep = torch.ones(q.shape[-2], k.shape[-2], dtype=torch.bool).tril()
    s = torch.where(keep, s, torch.full((), -1e9, dtype=s.dtype))
    return torch.softmax(s, -1) @ v


def _block(x, p, heads, lora=None, alpha=16.0):
    b, s, d = x.shape
    split = lambda z: z.reshape(b, s, heads, d // heads).transpose(1, 2)
    h = _layer_norm(x, p["ln1_w"], p["ln1_b"])

    def proj(name):
        y = h @ p["w" + name]
        if lora is not None and (name + "A") in lora:
            A, B = lora[name + "A"], lora[name + "B"]
            y = y + h @ ((A @ B) * (alpha / A.shape[1]))
        return y + p["b" + name]

    a = _causal_attention(split(proj("q")), split(proj("k")), split(proj("v")))
    x = x + a.transpose(1, 2).reshape(b, s, d) @ p["wo"] + p["bo"]
    h = _layer_norm(x, p["ln2_w"], p["ln2_b"])
    return x + _gelu(h @ p["w1"] + p["b1"]) @ p["w2"] + p["b2"]


def _cross_entropy(logits, labels):
    lsm = torch.log_softmax(logits, -1)
    return -torch.gather(lsm, -1, labels.unsqueeze(-1)).sum() / logits.shape[0]


def _leaf(a, dtype, grad=False):
    return torch.tensor(np.asarray(a), dtype=dtype).requires_grad_(grad)


def c3_step(t: dict, num_heads: int = 16, dtype=torch.float64):
    """loss = mean(block(x)^2) and its gradient w.r.t. the sixteen parameters, as
    (float, {name: float64 numpy array}); same inputs and result layout as
    ``oracle.configs.c3_reference``."""
    p = {k: _leaf(t[k], dtype, True) for k in C3_PARAMS}
    out = _block(_leaf(t["x"], dtype), p, num_heads)
    loss = (out * out).mean()
    grads = torch.autograd.grad(loss, [p[k] for k in C3_PARAMS])
    return float(loss.detach()), {k: g.double().numpy() for k, g in zip(C3_PARAMS, grads)}


def c5_step(t: dict, num_heads: int = 16, alpha: float = 16.0, dtype=torch.float64):
    """Cross-entropy of the LoRA decoder and its gradients w.r.t. the adapter factors only
    (qA, qB, vA, vB per layer, in that order), as ``oracle.configs.c5_reference`` returns them."""
    lora = [{k: _leaf(v, dtype, True) for k, v in ad.items()} for ad in t["lora"]]
    ids = torch.tensor(t["ids"])
    x = _leaf(t["embed"], dtype)[ids]
    for L, ad in zip(t["layers"], lora):
        x = _block(x, {k: _leaf(v, dtype) for k, v in L.items()}, num_heads, lora=ad, alpha=alpha)
    x = _layer_norm(x, _leaf(t["lnf_w"], dtype), _leaf(t["lnf_b"], dtype))
    loss = _cross_entropy(x @ _leaf(t["head"], dtype), ids)
    flat = [ad[k] for ad in lora for k in ("qA", "qB", "vA", "vB")]
    grads = torch.autograd.grad(loss, flat)
    return float(loss.detach()), [g.double().numpy() for g in grads]
