"""Layer modules (nabla/nn/modules): Linear stores its weight as (in, out) and
bias as (1, out) and computes ``x @ W + b`` (linear.py:30-54); LayerNorm;
Embedding; Dropout; Sequential; activations; MultiHeadAttention
(attention.py:58-107); pre-LN TransformerEncoderLayer (transformer.py:64-82)."""
from __future__ import annotations

from ...core.dtype import DType
from ...core.tensor import Tensor
from ...ops.creation import ones, zeros
from ...ops.view import reshape, swap_axes
from .. import functional as F
from .base import Module


class Linear(Module):
    def __init__(self, in_features: int, out_features: int, bias: bool = True, *,
                 dtype: DType = DType.float32) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        w = F.xavier_normal((in_features, out_features), dtype=dtype)
        w.requires_grad_(True)
        self.weight = w
        if bias:
            b = zeros((1, out_features), dtype=dtype).realize()
            b.requires_grad_(True)
            self.bias = b
        else:
            self.bias = None

    def forward(self, x: Tensor) -> Tensor:
        return F.linear(x, self.weight, self.bias)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None}")


class LayerNorm(Module):
    def __init__(self, normalized_shape: int, eps: float = 1e-5, elementwise_affine: bool = True, *,
                 dtype: DType = DType.float32) -> None:
        super().__init__()
        self.normalized_shape = int(normalized_shape)
        self.eps = float(eps)
        if elementwise_affine:
            w = ones((self.normalized_shape,), dtype=dtype).realize()
            w.requires_grad_(True)
            self.weight = w
            b = zeros((self.normalized_shape,), dtype=dtype).realize()
            b.requires_grad_(True)
            self.bias = b
        else:
            self.weight = None
            self.bias = None

    def forward(self, x: Tensor) -> Tensor:
        return F.layer_norm(x, self.weight, self.bias, eps=self.eps)


class Embedding(Module):
    def __init__(self, num_embeddings: int, embedding_dim: int, *, dtype: DType = DType.float32) -> None:
        super().__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        w = F.normal((num_embeddings, embedding_dim), dtype=dtype)
        w.requires_grad_(True)
        self.weight = w

    def forward(self, indices: Tensor) -> Tensor:
        return F.embedding(indices, self.weight)


class Dropout(Module):
    def __init__(self, p: float = 0.5) -> None:
        super().__init__()
        self.p = float(p)

    def forward(self, x: Tensor) -> Tensor:
        return F.dropout(x, self.p, training=self._training)


class ReLU(Module):
    def forward(self, x: Tensor) -> Tensor:
        return F.relu(x)


class GELU(Module):
    def forward(self, x: Tensor) -> Tensor:
        return F.gelu(x)


class Sequential(Module):
    def __init__(self, *layers: Module) -> None:
        super().__init__()
        for i, layer in enumerate(layers):
            setattr(self, str(i), layer)

    def forward(self, x):
        for m in self._modules.values():
            x = m(x)
        return x

    def __len__(self) -> int:
        return len(self._modules)

    def __getitem__(self, i: int) -> Module:
        return list(self._modules.values())[i]


class MultiHeadAttention(Module):
    def __init__(self, d_model: int, num_heads: int, dropout: float = 0.0, bias: bool = True, *,
                 dtype: DType = DType.float32) -> None:
        super().__init__()
        if d_model % num_heads != 0:
            raise ValueError(f"d_model ({d_model}) must be divisible by num_heads ({num_heads})")
        self.d_model = d_model
        self.num_heads = num_heads
        self.head_dim = d_model // num_heads
        self.dropout_p = float(dropout)
        self.q_proj = Linear(d_model, d_model, bias=bias, dtype=dtype)
        self.k_proj = Linear(d_model, d_model, bias=bias, dtype=dtype)
        self.v_proj = Linear(d_model, d_model, bias=bias, dtype=dtype)
        self.out_proj = Linear(d_model, d_model, bias=bias, dtype=dtype)

    def _reshape_to_heads(self, x: Tensor, batch: int, seq_len: int) -> Tensor:
        x = reshape(x, (batch, seq_len, self.num_heads, self.head_dim))
        return swap_axes(x, 1, 2)

    def forward(self, query: Tensor, key: Tensor, value: Tensor, attn_mask: Tensor | None = None,
                is_causal: bool = False) -> Tensor:
        batch, seq_q, seq_k = int(query.shape[0]), int(query.shape[1]), int(key.shape[1])
        q = self._reshape_to_heads(self.q_proj(query), batch, seq_q)
        k = self._reshape_to_heads(self.k_proj(key), batch, seq_k)
        v = self._reshape_to_heads(self.v_proj(value), batch, seq_k)
        out = F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, dropout_p=self.dropout_p,
                                             is_causal=is_causal, training=self._training)
        out = reshape(swap_axes(out, 1, 2), (batch, seq_q, self.d_model))
        return self.out_proj(out)


class TransformerEncoderLayer(Module):
    """Pre-LN block: ``x + MHA(LN1(x))`` then ``x + W2 gelu(W1 LN2(x))``."""

    def __init__(self, d_model: int, num_heads: int, dim_feedforward: int = 2048,
                 dropout: float = 0.1, *, dtype: DType = DType.float32) -> None:
        super().__init__()
        self.self_attn = MultiHeadAttention(d_model, num_heads, dropout=dropout, dtype=dtype)
        self.linear1 = Linear(d_model, dim_feedforward, dtype=dtype)
        self.linear2 = Linear(dim_feedforward, d_model, dtype=dtype)
        self.norm1 = LayerNorm(d_model, dtype=dtype)
        self.norm2 = LayerNorm(d_model, dtype=dtype)
        self.dropout1 = Dropout(dropout)
        self.dropout2 = Dropout(dropout)

    def forward(self, src: Tensor, src_mask: Tensor | None = None, is_causal: bool = False) -> Tensor:
        normed = self.norm1(src)
        attn_out = self.self_attn(normed, normed, normed, attn_mask=src_mask, is_causal=is_causal)
        src = src + self.dropout1(attn_out)
        normed = self.norm2(src)
        ff_out = self.linear2(F.gelu(self.linear1(normed)))
        return src + self.dropout2(ff_out)
