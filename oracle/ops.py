"""TEST INFRASTRUCTURE -- CPU oracle, not part of the product.

A numpy (fp64 by default) restatement of the reference's algorithm for the hot
path: each primitive op with the VJP rule the reference writes for it, and the
reverse replay of nabla/core/autograd/backward.py.  Only tests, the smoke entry
and the cpu_baseline leg of the benchmark may import this package.

Pinning (see tests/test_oracle_pins.py): every function here is checked
against torch-CPU autograd in fp64, against brute-force loops on tiny inputs
(matmul, conv2d, max_pool2d), and against closed forms (softmax rows sum to
one, layer_norm output has zero mean / unit variance, tie rule of reduce_max).
What those checks cannot see -- the bit-level rounding and accumulation order
of the MAX kernels the reference calls, its argmax tie-break, and the order in
which its backend applies scatter updates that name one row several times --
is parity unpinned; argmax adopts the lowest index (numpy / torch / jax agree)
and scatter the last update (numpy assignment).  The NF4 functions are pinned by
the decision thresholds between levels, exact round trips and the zero block.

The oracle is eager: a ``V`` carries a numpy value and, when gradients are
wanted, the closure that maps its cotangent to its parents' cotangents.
"""
from __future__ import annotations

import math
from typing import Callable, Sequence

import numpy as np
from scipy import special as _sp


class V:
    """Value with an optional reverse-mode rule (parents, vjp)."""

    __slots__ = ("a", "parents", "vjp", "name")

    def __init__(self, a, parents: Sequence["V"] = (), vjp: Callable | None = None, name: str = ""):
        self.a = np.asarray(a)
        self.parents = tuple(parents)
        self.vjp = vjp
        self.name = name

    @property
    def shape(self):
        return self.a.shape

    # operator sugar mirrors the reference's generated dunders (api.py:1405-1483)
    def __add__(self, o): return add(self, o)
    def __radd__(self, o): return add(o, self)
    def __sub__(self, o): return sub(self, o)
    def __rsub__(self, o): return sub(o, self)
    def __mul__(self, o): return mul(self, o)
    def __rmul__(self, o): return mul(o, self)
    def __truediv__(self, o): return div(self, o)
    def __rtruediv__(self, o): return div(o, self)
    def __matmul__(self, o): return matmul(self, o)
    def __neg__(self): return neg(self)


def _v(x, like: "V | None" = None) -> V:
    if isinstance(x, V):
        return x
    dt = like.a.dtype if like is not None and np.issubdtype(like.a.dtype, np.floating) else np.float64
    return V(np.asarray(x, dtype=dt))


def _reduce_to_shape(g: np.ndarray, shape) -> np.ndarray:
    """nabla/core/autograd/backward.py:31-54 -- undo broadcasting by summation."""
    shape = tuple(shape)
    if g.ndim > len(shape):
        g = g.sum(axis=tuple(range(g.ndim - len(shape))))
    axes = tuple(i for i, (c, a) in enumerate(zip(g.shape, shape)) if a == 1 and c > 1)
    if axes:
        g = g.sum(axis=axes, keepdims=True)
    return g.reshape(shape)


def backward(out: V, cotangent=None) -> dict:
    """Reverse replay (backward.py:129-353): topological order, per-op VJP,
    un-broadcast, accumulate by addition.  Returns {id(V): gradient}."""
    order, seen = [], set()
    stack = [(out, False)]
    while stack:
        v, done = stack.pop()
        if done:
            order.append(v)
            continue
        if id(v) in seen:
            continue
        seen.add(id(v))
        stack.append((v, True))
        for p in v.parents:
            if id(p) not in seen:
                stack.append((p, False))
    grads = {id(out): np.ones_like(out.a, dtype=np.float64) if cotangent is None else np.asarray(cotangent)}
    for v in reversed(order):
        g = grads.get(id(v))
        if g is None or v.vjp is None:
            continue
        for p, pg in zip(v.parents, v.vjp(g)):
            if pg is None or not np.issubdtype(p.a.dtype, np.floating):
                continue
            pg = _reduce_to_shape(np.asarray(pg), p.a.shape)
            grads[id(p)] = grads[id(p)] + pg if id(p) in grads else pg
    return grads


def grad_of(out: V, wrt: Sequence[V]) -> list[np.ndarray]:
    g = backward(out)
    return [g.get(id(w), np.zeros_like(w.a, dtype=np.float64)) for w in wrt]


# ------------------------------------------------------------------- binary
def _bcast(x, y):
    x = _v(x, y if isinstance(y, V) else None)
    y = _v(y, x)
    return x, y


def add(x, y) -> V:  # nabla/ops/binary.py:18-45
    x, y = _bcast(x, y)
    return V(x.a + y.a, (x, y), lambda g: (g, g))


def sub(x, y) -> V:  # binary.py:82-111
    x, y = _bcast(x, y)
    return V(x.a - y.a, (x, y), lambda g: (g, -g))


def mul(x, y) -> V:  # binary.py:48-79
    x, y = _bcast(x, y)
    return V(x.a * y.a, (x, y), lambda g: (g * y.a, g * x.a))


def div(x, y) -> V:  # binary.py:114-156: dx = g / y, dy = -(g * (x / (y*y)))
    x, y = _bcast(x, y)
    return V(x.a / y.a, (x, y), lambda g: (g / y.a, -(g * (x.a / (y.a * y.a)))))


def matmul(x, y) -> V:
    """binary.py:197-314: numpy batch broadcasting; dX = G @ swap(W), dW = swap(X) @ G."""
    x, y = _v(x), _v(y)
    out = np.matmul(x.a, y.a)

    def vjp(g):
        xa = x.a if x.a.ndim > 1 else x.a[None, :]
        ya = y.a if y.a.ndim > 1 else y.a[:, None]
        gg = g
        if x.a.ndim == 1:
            gg = np.expand_dims(gg, -2)
        if y.a.ndim == 1:
            gg = np.expand_dims(gg, -1)
        gx = np.matmul(gg, np.swapaxes(ya, -1, -2))
        gy = np.matmul(np.swapaxes(xa, -1, -2), gg)
        if x.a.ndim == 1:
            gx = gx.reshape(gx.shape[:-2] + (gx.shape[-1],))
        if y.a.ndim == 1:
            gy = gy.reshape(gy.shape[:-1])
        return gx, gy

    return V(out, (x, y), vjp)


# -------------------------------------------------------------------- unary
def neg(x) -> V:  # unary.py:113-138
    x = _v(x)
    return V(-x.a, (x,), lambda g: (-g,))


def relu(x) -> V:  # unary.py:20-54: derivative (x > 0), zero at x == 0
    x = _v(x)
    return V(np.maximum(x.a, 0), (x,), lambda g: (np.where(x.a > 0, g, 0.0),))


def exp(x) -> V:  # unary.py:97-110
    x = _v(x)
    out = np.exp(x.a)
    return V(out, (x,), lambda g: (g * out,))


def log(x) -> V:  # unary.py:233-250
    x = _v(x)
    return V(np.log(x.a), (x,), lambda g: (g / x.a,))


def sqrt(x) -> V:  # unary.py:253-268
    x = _v(x)
    out = np.sqrt(x.a)
    return V(out, (x,), lambda g: (g * 0.5 / out,))


def rsqrt(x) -> V:  # unary.py:487-501: derivative -0.5 * out^3
    x = _v(x)
    out = 1.0 / np.sqrt(x.a)
    return V(out, (x,), lambda g: (g * (-0.5 * out * out * out),))


def erf(x) -> V:  # unary.py:386-405: derivative 2/sqrt(pi) * exp(-x^2)
    x = _v(x)
    return V(_sp.erf(x.a), (x,), lambda g: (g * (2.0 / math.sqrt(math.pi)) * np.exp(-(x.a * x.a)),))


def tanh(x) -> V:
    x = _v(x)
    out = np.tanh(x.a)
    return V(out, (x,), lambda g: (g * (1.0 - out * out),))


def gelu(x) -> V:
    """unary.py:567-595: exact x * Phi(x); derivative cdf + x * pdf."""
    x = _v(x)
    cdf = 0.5 * (1.0 + _sp.erf(x.a / math.sqrt(2.0)))
    pdf = np.exp(-(x.a * x.a) / 2.0) / math.sqrt(2.0 * math.pi)
    return V(x.a * cdf, (x,), lambda g: (g * (cdf + x.a * pdf),))


def cast(x, dtype) -> V:  # unary.py:660-697: the VJP casts back
    x = _v(x)
    return V(x.a.astype(dtype), (x,), lambda g: (g.astype(x.a.dtype) if np.issubdtype(x.a.dtype, np.floating) else None,))


def softmax(x, axis: int = -1) -> V:  # unary.py:192-230: s * (g - sum(g * s))
    x = _v(x)
    e = np.exp(x.a - x.a.max(axis=axis, keepdims=True))
    s = e / e.sum(axis=axis, keepdims=True)
    return V(s, (x,), lambda g: (s * (g - (g * s).sum(axis=axis, keepdims=True)),))


def logsoftmax(x, axis: int = -1) -> V:  # unary.py:598-632: g - exp(out) * sum(g)
    x = _v(x)
    sh = x.a - x.a.max(axis=axis, keepdims=True)
    out = sh - np.log(np.exp(sh).sum(axis=axis, keepdims=True))
    return V(out, (x,), lambda g: (g - np.exp(out) * g.sum(axis=axis, keepdims=True),))


# ------------------------------------------------------ comparison / where
def greater(x, y) -> V:  # comparison.py:94-106 (bool, no gradient)
    x, y = _bcast(x, y)
    return V(x.a > y.a)


def equal(x, y) -> V:  # comparison.py:63-82
    x, y = _bcast(x, y)
    return V(x.a == y.a)


def where(c, x, y) -> V:  # control_flow.py:21-141: the condition gets no gradient
    c = _v(c)
    x, y = _bcast(x, y)
    cond = c.a.astype(bool)
    return V(np.where(cond, x.a, y.a), (x, y), lambda g: (np.where(cond, g, 0.0), np.where(cond, 0.0, g)))


# --------------------------------------------------------------- reductions
def _axes(axis, ndim):
    if axis is None:
        return tuple(range(ndim))
    if isinstance(axis, (list, tuple)):
        return tuple(a % ndim for a in axis)
    return (axis % ndim,)


def reduce_sum(x, axis=None, keepdims: bool = False) -> V:  # reduction.py:147-172, 544-581
    x = _v(x)
    ax = _axes(axis, x.a.ndim)
    out = x.a.sum(axis=ax, keepdims=keepdims)

    def vjp(g):
        gk = g if keepdims else np.expand_dims(g, ax) if ax else g
        return (np.broadcast_to(gk, x.a.shape),)

    return V(out, (x,), vjp)


def mean(x, axis=None, keepdims: bool = False) -> V:  # reduction.py:604-639: sum / count
    x = _v(x)
    ax = _axes(axis, x.a.ndim)
    count = 1
    for a in ax:
        count *= x.a.shape[a]
    return div(reduce_sum(x, axis=axis, keepdims=keepdims), float(count))


def reduce_max(x, axis=None, keepdims: bool = False) -> V:
    """reduction.py:205-245: every element equal to the maximum gets the FULL cotangent.
    Multi-axis reductions run one axis at a time, highest axis first (544-581)."""
    x = _v(x)
    ax = sorted(_axes(axis, x.a.ndim), reverse=True)
    cur = x
    for a in ax:
        cur = _reduce_max_1(cur, a)
    if not keepdims:
        kept = tuple(d for i, d in enumerate(x.a.shape) if i not in ax)
        cur = reshape(cur, kept)
    return cur


def _reduce_max_1(x: V, axis: int) -> V:
    m = x.a.max(axis=axis, keepdims=True)
    return V(m, (x,), lambda g: (np.broadcast_to(g, x.a.shape) * (x.a == m),))


def argmax(x, axis: int = -1) -> np.ndarray:  # reduction.py:739-811: int64, first maximum
    x = _v(x)
    return np.argmax(x.a, axis=axis).astype(np.int64)


# --------------------------------------------------------------------- views
def reshape(x, shape) -> V:  # view/shape.py:161-390
    x = _v(x)
    return V(x.a.reshape(shape), (x,), lambda g: (g.reshape(x.a.shape),))


def swap_axes(x, a: int, b: int) -> V:  # view/axes.py:43-441
    x = _v(x)
    return V(np.swapaxes(x.a, a, b), (x,), lambda g: (np.swapaxes(g, a, b),))


def permute(x, order) -> V:  # view/axes.py:762-868
    x = _v(x)
    inv = np.argsort(order)
    return V(np.transpose(x.a, order), (x,), lambda g: (np.transpose(g, inv),))


def broadcast_to(x, shape) -> V:  # view/shape.py:56-158
    x = _v(x)
    return V(np.broadcast_to(x.a, shape), (x,), lambda g: (g,))


def unsqueeze(x, axis: int) -> V:
    x = _v(x)
    return V(np.expand_dims(x.a, axis), (x,), lambda g: (g.reshape(x.a.shape),))


def slice_tensor(x, start, size) -> V:  # view/shape.py:586-818: VJP pads with zeros
    x = _v(x)
    sl = tuple(slice(s, s + n) for s, n in zip(start, size))

    def vjp(g):
        out = np.zeros(x.a.shape, dtype=g.dtype)
        out[sl] = g
        return (out,)

    return V(x.a[sl], (x,), vjp)


def pad(x, paddings, value: float = 0.0) -> V:  # view/shape.py:1313-1398
    x = _v(x)
    sl = tuple(slice(a, a + d) for (a, _), d in zip(paddings, x.a.shape))
    return V(np.pad(x.a, paddings, constant_values=value), (x,), lambda g: (g[sl],))


def concatenate(xs, axis: int = 0) -> V:  # view/shape.py:821-980
    xs = [_v(x) for x in xs]
    sizes = [x.a.shape[axis] for x in xs]

    def vjp(g):
        return tuple(np.split(g, np.cumsum(sizes)[:-1], axis=axis))

    return V(np.concatenate([x.a for x in xs], axis=axis), xs, vjp)


def scatter(x, idx, updates, axis: int = 0) -> V:
    """view/indexing.py:185-447, 483-504: ``out = x.copy(); out[idx] = updates`` along ``axis``.
    Duplicate indices: the reference leaves the order to its backend; here (and in the kernels)
    the last update wins, which is what numpy's assignment does (parity unpinned for
    duplicates: none of the reference's fixtures fixes that order)."""
    x, updates = _v(x), _v(updates)
    idx = (idx.a if isinstance(idx, V) else np.asarray(idx)).astype(np.int64)
    out = x.a.copy()
    sel = (slice(None),) * axis
    flat_idx = idx.reshape(-1)
    up = updates.a.reshape(x.a.shape[:axis] + (flat_idx.size,) + x.a.shape[axis + 1:])
    for j, i in enumerate(flat_idx):
        out[sel + (int(i),)] = up[sel + (j,)]

    def vjp(g):
        gx = g.copy()
        for i in flat_idx:
            gx[sel + (int(i),)] = 0
        gu = np.stack([g[sel + (int(i),)] for i in flat_idx], axis=axis).reshape(updates.a.shape)
        return (gx, gu)

    return V(out, (x, updates), vjp)


def gather(table, idx, axis: int = 0) -> V:  # view/indexing.py:100-182
    """take along ``axis``; the VJP scatters the cotangent into zeros (173-182), i.e. a row
    gathered several times receives the cotangent of its LAST occurrence, not their sum."""
    table = _v(table)
    idx = (idx.a if isinstance(idx, V) else np.asarray(idx)).astype(np.int64)
    y = np.take(table.a, idx, axis=axis)

    def vjp(g):
        return (scatter(V(np.zeros_like(table.a, dtype=g.dtype)), idx, V(g), axis).a,)

    return V(y, (table,), vjp)


def tril(x, k: int = 0) -> V:  # creation.py:225-274
    x = _v(x)
    return V(np.tril(x.a, k), (x,), lambda g: (np.tril(g, k),))


# --------------------------------------------------------------- convolution
def conv2d_forward(x: np.ndarray, w: np.ndarray, stride, padding) -> np.ndarray:
    """NHWC x HWIO correlation with zero padding (t, b, l, r); convolution.py:220-252.
    Formula of docs/dev/convolution_autodiff.md:5-20, vectorised over taps."""
    pt, pb, pl, pr = padding
    sh, sw = stride
    n, h, wd, cin = x.shape
    r, s, _, cout = w.shape
    xp = np.pad(x, ((0, 0), (pt, pb), (pl, pr), (0, 0)))
    ho = (h + pt + pb - r) // sh + 1
    wo = (wd + pl + pr - s) // sw + 1
    y = np.zeros((n, ho, wo, cout), dtype=np.result_type(x, w))
    for i in range(r):
        for j in range(s):
            patch = xp[:, i:i + (ho - 1) * sh + 1:sh, j:j + (wo - 1) * sw + 1:sw, :]
            y += patch @ w[i, j]
    return y


def conv2d(x, w, bias=None, stride=(1, 1), padding=(0, 0, 0, 0)) -> V:
    """convolution.py:220-392.  dX scatters each tap back (the transposed
    convolution cropped by the padding, 345-361); dW correlates the padded
    input with the cotangent (363-384); db sums the cotangent over N, H, W."""
    x, w = _v(x), _v(w)
    pt, pb, pl, pr = padding
    sh, sw = stride
    y = conv2d_forward(x.a, w.a, stride, padding)
    parents = [x, w]
    if bias is not None:
        bias = _v(bias)
        y = y + bias.a
        parents.append(bias)
    n, h, wd, cin = x.a.shape
    r, s, _, cout = w.a.shape
    ho, wo = y.shape[1], y.shape[2]

    def vjp(g):
        xp = np.pad(x.a, ((0, 0), (pt, pb), (pl, pr), (0, 0)))
        gxp = np.zeros_like(xp, dtype=g.dtype)
        gw = np.zeros_like(w.a, dtype=g.dtype)
        for i in range(r):
            for j in range(s):
                hs = slice(i, i + (ho - 1) * sh + 1, sh)
                ws = slice(j, j + (wo - 1) * sw + 1, sw)
                gxp[:, hs, ws, :] += g @ w.a[i, j].T
                gw[i, j] = np.tensordot(xp[:, hs, ws, :], g, axes=([0, 1, 2], [0, 1, 2]))
        gx = gxp[:, pt:pt + h, pl:pl + wd, :]
        out = [gx, gw]
        if bias is not None:
            out.append(g.sum(axis=(0, 1, 2)))
        return tuple(out)

    return V(y, parents, vjp)


def conv2d_transpose(x, w, bias=None, stride=(1, 1), padding=(0, 0, 0, 0)) -> V:
    """convolution.py:424-566, 699-787: transposed convolution of NHWC ``x`` [N,H,W,Cin] with
    a filter [R,S,Cout,Cin].  Every input pixel scatters ``x[n,i,j,:] @ w[r,s].T`` to output
    position (i*sh - pt + r, j*sw - pl + s); the output has (H-1)*sh - pt - pb + R rows
    (convolution.py:140-160 with dilation 1 and no output padding).  Gradients as in 522-566:
    dX is the forward convolution of the cotangent with the same filter, dW correlates the
    padded cotangent with x, db sums the cotangent over N, H, W."""
    x, w = _v(x), _v(w)
    pt, pb, pl, pr = padding
    sh, sw = stride
    n, h, wd, cin = x.a.shape
    r, s, cout, _ = w.a.shape
    hf, wf = (h - 1) * sh + r, (wd - 1) * sw + s          # size before the padding is cut off
    ho, wo = hf - pt - pb, wf - pl - pr
    if ho <= 0 or wo <= 0:
        raise ValueError(f"Non-positive conv2d_transpose output size H={ho}, W={wo}.")

    def taps():
        for i in range(r):
            for j in range(s):
                yield i, j, slice(i, i + (h - 1) * sh + 1, sh), slice(j, j + (wd - 1) * sw + 1, sw)

    full = np.zeros((n, hf, wf, cout), dtype=np.result_type(x.a, w.a))
    for i, j, hs, ws in taps():
        full[:, hs, ws, :] += x.a @ w.a[i, j].T
    y = full[:, pt:pt + ho, pl:pl + wo, :]
    parents = [x, w]
    if bias is not None:
        bias = _v(bias)
        y = y + bias.a
        parents.append(bias)

    def vjp(g):
        gp = np.pad(g, ((0, 0), (pt, pb), (pl, pr), (0, 0)))
        gx = np.zeros_like(x.a, dtype=g.dtype)
        gw = np.zeros_like(w.a, dtype=g.dtype)
        for i, j, hs, ws in taps():
            gx += gp[:, hs, ws, :] @ w.a[i, j]
            gw[i, j] = np.tensordot(gp[:, hs, ws, :], x.a, axes=([0, 1, 2], [0, 1, 2]))
        out = [gx, gw]
        if bias is not None:
            out.append(g.sum(axis=(0, 1, 2)))
        return tuple(out)

    return V(y, parents, vjp)


def max_pool2d(x, kernel, stride=None, padding=(0, 0, 0, 0)) -> V:
    """pooling.py:53-137: per output pixel, reduce_max over the window clipped to
    the image; the gradient follows reduce_max's tie rule per window."""
    x = _v(x)
    kh, kw = kernel
    sh, sw = stride if stride is not None else kernel
    pt, pb, pl, pr = padding
    n, h, w, c = x.a.shape
    ho = (h + pt + pb - kh) // sh + 1
    wo = (w + pl + pr - kw) // sw + 1
    y = np.full((n, ho, wo, c), -np.inf, dtype=x.a.dtype)
    wins = {}
    for i in range(ho):
        for j in range(wo):
            h0, h1 = max(0, i * sh - pt), min(h, i * sh - pt + kh)
            w0, w1 = max(0, j * sw - pl), min(w, j * sw - pl + kw)
            wins[(i, j)] = (h0, h1, w0, w1)
            if h0 < h1 and w0 < w1:
                y[:, i, j, :] = x.a[:, h0:h1, w0:w1, :].max(axis=(1, 2))

    def vjp(g):
        gx = np.zeros_like(x.a, dtype=g.dtype)
        for (i, j), (h0, h1, w0, w1) in wins.items():
            if h0 < h1 and w0 < w1:
                mask = x.a[:, h0:h1, w0:w1, :] == y[:, i:i + 1, j:j + 1, :]
                gx[:, h0:h1, w0:w1, :] += mask * g[:, i:i + 1, j:j + 1, :]
        return (gx,)

    return V(y, (x,), vjp)


# ------------------------------------------------------------ nn composites
def avg_pool2d(x, kernel, stride=None, padding=(0, 0, 0, 0)) -> V:
    """pooling.py:77-110, 140-173: the input is zero-padded first, then every window is summed
    and divided by kh * kw (the padding counts); the VJP of slice + sum + pad spreads
    g / (kh * kw) back over the window and drops what falls on the padding."""
    x = _v(x)
    kh, kw = kernel
    sh, sw = stride if stride is not None else kernel
    pt, pb, pl, pr = padding
    xp = np.pad(x.a, ((0, 0), (pt, pb), (pl, pr), (0, 0)))
    n, h, w, c = xp.shape
    ho, wo = (h - kh) // sh + 1, (w - kw) // sw + 1
    y = np.empty((n, ho, wo, c), dtype=x.a.dtype)
    for i in range(ho):
        for j in range(wo):
            y[:, i, j, :] = xp[:, i * sh:i * sh + kh, j * sw:j * sw + kw, :].sum(axis=(1, 2)) / (kh * kw)

    def vjp(g):
        gp = np.zeros(xp.shape, dtype=g.dtype)
        for i in range(ho):
            for j in range(wo):
                gp[:, i * sh:i * sh + kh, j * sw:j * sw + kw, :] += g[:, i:i + 1, j:j + 1, :] / (kh * kw)
        return (gp[:, pt:h - pb, pl:w - pr, :],)

    return V(y, (x,), vjp)


def silu(x) -> V:  # unary.py:504-520: x * sigmoid(x)
    x = _v(x)
    s = 1.0 / (1.0 + np.exp(-x.a))
    return V(x.a * s, (x,), lambda g: (g * (s + x.a * s * (1.0 - s)),))


def linear(x, w, b=None) -> V:  # nn/functional/layers.py:30-35
    out = matmul(x, w)
    return out + b if b is not None else out


def layer_norm(x, weight=None, bias=None, eps: float = 1e-5) -> V:
    """nn/functional/layers.py:38-56, op for op (biased variance)."""
    x = _v(x)
    mu = mean(x, axis=-1, keepdims=True)
    centered = x - mu
    var = mean(centered * centered, axis=-1, keepdims=True)
    out = centered * rsqrt(var + eps)
    if weight is not None:
        out = out * weight
    if bias is not None:
        out = out + bias
    return out


def scaled_dot_product_attention(q, k, v, is_causal: bool = False) -> V:
    """nn/functional/layers.py:106-153: scale after the product; causal mask is
    where(tril(ones) > 0, scores, -1e9)."""
    q, k, v = _v(q), _v(k), _v(v)
    scale = 1.0 / math.sqrt(q.a.shape[-1])
    scores = matmul(q, swap_axes(k, -2, -1)) * scale
    if is_causal:
        sq, sk = q.a.shape[-2], k.a.shape[-2]
        causal = tril(V(np.ones((sq, sk), dtype=q.a.dtype)))
        scores = where(greater(causal, 0.0), scores, V(np.full((sq, sk), -1e9, dtype=q.a.dtype)))
    return matmul(softmax(scores, axis=-1), v)


def multi_head_attention(x, p: dict, num_heads: int, is_causal: bool) -> V:
    """nn/modules/attention.py:58-107 with query = key = value = x."""
    b, s, d = x.a.shape
    hd = d // num_heads

    def heads(t):
        return swap_axes(reshape(t, (b, s, num_heads, hd)), 1, 2)

    q = heads(linear(x, p["wq"], p["bq"]))
    k = heads(linear(x, p["wk"], p["bk"]))
    v = heads(linear(x, p["wv"], p["bv"]))
    o = scaled_dot_product_attention(q, k, v, is_causal=is_causal)
    o = reshape(swap_axes(o, 1, 2), (b, s, d))
    return linear(o, p["wo"], p["bo"])


def transformer_encoder_layer(x, p: dict, num_heads: int, is_causal: bool = True) -> V:
    """nn/modules/transformer.py:64-82 (pre-LN, dropout 0)."""
    x = _v(x)
    normed = layer_norm(x, p["ln1_w"], p["ln1_b"])
    x = x + multi_head_attention(normed, p, num_heads, is_causal)
    normed = layer_norm(x, p["ln2_w"], p["ln2_b"])
    ff = linear(gelu(linear(normed, p["w1"], p["b1"])), p["w2"], p["b2"])
    return x + ff


def one_hot(idx: np.ndarray, num_classes: int, dtype) -> V:  # nn/functional/losses.py:52-77
    return V((np.expand_dims(idx, -1) == np.arange(num_classes)).astype(dtype))


def cross_entropy_loss(logits, targets: np.ndarray) -> V:
    """nn/functional/losses.py:20-44: -sum(onehot * logsoftmax) / logits.shape[0]."""
    logits = _v(logits)
    lp = logsoftmax(logits, axis=-1)
    oh = one_hot(np.asarray(targets), logits.a.shape[-1], logits.a.dtype)
    return neg(reduce_sum(oh * lp)) / float(logits.a.shape[0])


def lora_linear(x, w, A, B, alpha: float) -> V:
    """nn/finetune/lora.py:55-79: x @ W + x @ ((A @ B) * (alpha / rank))."""
    A = _v(A)
    scale = alpha / float(A.a.shape[1])
    return matmul(x, w) + matmul(x, matmul(A, B) * scale)


# ---- NF4 (nn/finetune/qlora.py) -------------------------------------------------------------
#: qlora.py:18-38
NF4_LEVELS = np.array([-1.0, -0.6962, -0.5251, -0.3949, -0.2844, -0.1848, -0.0911, 0.0,
                       0.0796, 0.1609, 0.2461, 0.3379, 0.4407, 0.5626, 0.7230, 1.0], dtype=np.float32)


def nf4_quantize(w: np.ndarray, block_size: int = 64) -> dict:
    """qlora.py:41-75 in fp32: flatten, zero-pad to whole blocks, scale every block by its
    absolute maximum (1 for an all-zero block), index of the nearest level (first on a tie)."""
    flat = np.asarray(w, dtype=np.float32).reshape(-1)
    numel = flat.size
    pad = (block_size - numel % block_size) % block_size
    flat = np.pad(flat, (0, pad))
    blocks = flat.reshape(-1, block_size)
    scales = np.max(np.abs(blocks), axis=-1, keepdims=True)
    scales[scales == 0] = 1.0
    normalized = blocks / scales
    indices = np.empty(normalized.size, dtype=np.uint8)
    for i, x in enumerate(normalized.reshape(-1)):
        indices[i] = int(np.argmin(np.abs(x - NF4_LEVELS)))
    return dict(indices=indices, scales=scales.reshape(-1).astype(np.float32), shape=tuple(np.shape(w)),
                numel=numel, padded=flat.size, block=block_size)


def nf4_dequantize(q: dict) -> np.ndarray:
    """qlora.py:77-98: level[index] * block scale, trimmed to the original element count."""
    levels = NF4_LEVELS[q["indices"].astype(np.int64)].reshape(-1, q["block"])
    flat = (levels * q["scales"][:, None]).reshape(-1)
    return flat[:q["numel"]].reshape(q["shape"])
