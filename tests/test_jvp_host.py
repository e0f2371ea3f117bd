"""Forward mode (``jvp``) on the host path.  The oracle has no forward mode, so the pins are
(a) central differences of the oracle's float64 forward functions along the tangent and
(b) the adjoint identity <J v, u> = <v, J^T u> against ``vjp``, whose rules are pinned
against the oracle's gradients elsewhere."""
import numpy as np
import pytest

import nabla_amd as nb
from oracle import ops as O

RNG = np.random.default_rng(41)
F = nb.nn.functional


def T(a, dtype=None):
    return nb.Tensor.constant(np.asarray(a, dtype=np.float32), dtype=dtype)


def central(f, xs, vs, eps=1e-6):
    """d/de f(x + e v) at e = 0 with the float64 oracle."""
    p = f(*[O.V(x + eps * v) for x, v in zip(xs, vs)])
    m = f(*[O.V(x - eps * v) for x, v in zip(xs, vs)])
    return (p.a - m.a) / (2 * eps)


def rand(*shape):
    return RNG.standard_normal(shape)


CASES = {
    "mlp_softmax": (lambda x, w, b: nb.softmax(nb.relu(x @ w + b) * 0.5, axis=-1),
                    lambda x, w, b: O.softmax(O.relu(O.matmul(x, w) + b) * 0.5, axis=-1),
                    [(5, 7), (7, 4), (4,)]),
    "layernorm_gelu": (lambda x, g, b: nb.gelu(F.layer_norm(x, g, b)),
                       lambda x, g, b: O.gelu(O.layer_norm(x, g, b)),
                       [(6, 16), (16,), (16,)]),
    "reductions_where": (lambda x, y: nb.reduce_sum(nb.where(nb.greater(x, y), x * y, nb.exp(y)), axis=0) /
                         nb.reduce_max(x * x, axis=0),
                         lambda x, y: O.reduce_sum(O.where(O.greater(x, y), x * y, O.exp(y)), axis=0) /
                         O.reduce_max(x * x, axis=0),
                         [(5, 6), (5, 6)]),
    "conv_pool": (lambda x, w, b: nb.avg_pool2d(nb.max_pool2d(nb.relu(nb.conv2d(x, w, padding=1, bias=b)),
                                                              kernel_size=2), kernel_size=2),
                  lambda x, w, b: O.avg_pool2d(O.max_pool2d(O.relu(O.conv2d(x, w, b, (1, 1), (1, 1, 1, 1))),
                                                            (2, 2)), (2, 2)),
                  [(2, 8, 8, 3), (3, 3, 3, 4), (4,)]),
    "views": (lambda x, y: nb.concatenate([nb.swap_axes(x, 0, 1)[1:3], nb.pad(y, paddings=[(1, 0), (0, 0)])], axis=0) * 2.0,
              lambda x, y: O.concatenate([O.slice_tensor(O.swap_axes(x, 0, 1), (1, 0), (2, 4)),
                                          O.pad(y, [(1, 0), (0, 0)])], axis=0) * 2.0,
              [(4, 5), (2, 4)]),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_jvp_against_central_differences_and_vjp(emulator, name):
    fn, ofn, shapes = CASES[name]
    xs = [rand(*s) for s in shapes]
    vs = [rand(*s) for s in shapes]
    out, tan = nb.jvp(fn, tuple(T(x) for x in xs), tuple(T(v) for v in vs))
    want = central(ofn, xs, vs)
    np.testing.assert_allclose(out.numpy(), ofn(*[O.V(x) for x in xs]).a, rtol=2e-5, atol=2e-6)
    assert np.abs(tan.numpy() - want).max() <= 2e-4 * max(np.abs(want).max(), 1.0), name
    # <J v, u> = <v, J^T u>
    u = rand(*out.shape)
    _, pull = nb.vjp(fn, *[T(x) for x in xs])
    gs = pull(T(u))
    lhs = float((tan.numpy().astype(np.float64) * u).sum())
    rhs = sum(float((g.numpy().astype(np.float64) * v).sum()) for g, v in zip(gs, vs))
    assert abs(lhs - rhs) <= 2e-4 * max(abs(lhs), abs(rhs), 1.0)


def test_jvp_embedding_and_partial_tangents(emulator):
    """Integer inputs carry no tangent; an output no tangent reaches gets zeros."""
    table, ids = rand(11, 6), RNG.integers(0, 11, size=(3, 4))
    v = rand(11, 6)
    tid = nb.Tensor.constant(ids.astype(np.int64))
    (emb, const), (temb, tconst) = nb.jvp(lambda t, i: (F.embedding(i, t) * 3.0, nb.cast(i, nb.DType.float32)),
                                          (T(table), tid), (T(v), nb.zeros_like(tid)))
    np.testing.assert_allclose(temb.numpy(), v[ids] * 3.0, rtol=1e-6)
    np.testing.assert_array_equal(tconst.numpy(), np.zeros(ids.shape, np.float32))


def test_jvp_of_grad_is_a_hessian_vector_product(emulator):
    x, v = rand(6), rand(6)
    f = lambda t: nb.reduce_sum(nb.exp(t) * t * t)
    _, hv = nb.jvp(nb.grad(f), (T(x),), (T(v),))
    # f = sum e^x x^2: f'' = e^x (x^2 + 4x + 2), diagonal
    want = np.exp(x) * (x * x + 4 * x + 2) * v
    np.testing.assert_allclose(hv.numpy(), want, rtol=2e-5, atol=1e-6)


def test_jvp_fused_attention_uses_the_vjp_fallback(emulator):
    import torch
    q, k, v_, tq = (torch.from_numpy(rand(1, 1, 128, 64).astype(np.float32)).to(torch.bfloat16).float().numpy()
                    for _ in range(4))
    bf = nb.DType.bfloat16
    fn = lambda a: nb.cast(F.scaled_dot_product_attention(a, T(k, bf), T(v_, bf), is_causal=True), nb.DType.float32)
    out, tan = nb.jvp(fn, (T(q, bf),), (T(tq, bf),))
    ofn = lambda a: O.scaled_dot_product_attention(a, O.V(k.astype(np.float64)), O.V(v_.astype(np.float64)), is_causal=True)
    want = central(ofn, [q.astype(np.float64)], [tq.astype(np.float64)])
    assert np.abs(tan.numpy() - want).max() <= 5e-2 * np.abs(want).max()


def test_jvp_argument_checks_and_aux(emulator):
    x = T(rand(3))
    with pytest.raises(TypeError, match="primals must be a tuple"):
        nb.jvp(lambda a: a, [x], (x,))
    with pytest.raises(TypeError, match="tangents must be a tuple"):
        nb.jvp(lambda a: a, (x,), [x])
    with pytest.raises(ValueError, match="same length"):
        nb.jvp(lambda a: a, (x,), (x, x))
    with pytest.raises(ValueError, match="tangent shape"):
        nb.jvp(lambda a: a * 2.0, (x,), (T(rand(4)),))
    out, tan, aux = nb.jvp(lambda a: (a * a, {"n": 3}), (x,), (nb.ones_like(x),), has_aux=True)
    assert aux == {"n": 3}
    np.testing.assert_allclose(tan.numpy(), 2 * x.numpy(), rtol=1e-6)
