"""``vmap`` on the host path against numpy: the argument conventions of the reference
(nabla/transforms/vmap.py:291-362; in_axes / out_axes per argument, None, containers, axis_size,
decorator form, nesting) and composition with grad / jacrev.  The expected values are numpy's
own batched results (einsum, broadcasting), which is what a vectorising map has to equal."""
import numpy as np
import pytest

import nabla_amd as nb

RNG = np.random.default_rng(61)


def T(a):
    return nb.Tensor.constant(np.asarray(a, dtype=np.float32))


def close(got, want, tol=1e-5):
    got = got.numpy()
    assert got.shape == np.asarray(want).shape, (got.shape, np.asarray(want).shape)
    np.testing.assert_allclose(got, want, rtol=tol, atol=tol)


def test_batched_matvec_and_axes(emulator):
    A, x = RNG.standard_normal((5, 3, 4)), RNG.standard_normal((5, 4))
    close(nb.vmap(lambda a, v: a @ v)(T(A), T(x)), np.einsum("bij,bj->bi", A, x))
    # unbatched matrix, batched vector
    close(nb.vmap(lambda a, v: a @ v, in_axes=(None, 0))(T(A[0]), T(x)), x @ A[0].T)
    # batch axis 1 on the input, axis 1 on the output
    At = np.moveaxis(A, 0, 1)                      # [3, 5, 4]
    got = nb.vmap(lambda a, v: a @ v, in_axes=(1, 0), out_axes=1)(T(At), T(x))
    close(got, np.einsum("bij,bj->ib", A, x))
    # negative axes
    got = nb.vmap(lambda a: nb.reduce_sum(a, axis=0), in_axes=-1, out_axes=-1)(T(A))
    close(got, A.sum(axis=0))


def test_multiple_outputs_containers_and_decorator(emulator):
    x, y = RNG.standard_normal((4, 3)), RNG.standard_normal((4, 3))

    @nb.vmap(in_axes=({"a": 0, "b": 0},), out_axes=(0, None))
    def f(d):
        return d["a"] * d["b"], nb.Tensor.constant(np.float32(2.0))

    prod, two = f({"a": T(x), "b": T(y)})
    close(prod, x * y)
    assert two.numpy().shape == () and float(two.numpy()) == 2.0
    s, d = nb.vmap(lambda a, b: [a + b, a - b], out_axes=[0, 1])(T(x), T(y))
    close(s, x + y)
    close(d, (x - y).T)


def test_nested_and_axis_size(emulator):
    x, y = RNG.standard_normal(3), RNG.standard_normal(4)
    outer = nb.vmap(nb.vmap(lambda a, b: a * b, in_axes=(None, 0)), in_axes=(0, None))
    close(outer(T(x), T(y)), np.outer(x, y))
    got = nb.vmap(lambda a: a * 2.0, in_axes=None, axis_size=3)(T(x))
    close(got, np.tile(2 * x, (3, 1)))


def test_per_example_gradients_and_jacobian(emulator):
    W, X = RNG.standard_normal((3, 2)), RNG.standard_normal((5, 3))
    loss = lambda w, x: nb.reduce_sum(nb.tanh(x @ w) ** 2)
    got = nb.vmap(nb.grad(loss), in_axes=(None, 0))(T(W), T(X))
    want = np.stack([np.outer(x, 2 * np.tanh(x @ W) * (1 - np.tanh(x @ W) ** 2)) for x in X])
    close(got, want, 1e-4)
    # grad of a vmapped function: d/dW sum_b loss(W, x_b) = sum of the per-example gradients
    total = nb.grad(lambda w: nb.reduce_sum(nb.vmap(loss, in_axes=(None, 0))(w, T(X))))(T(W))
    close(total, want.sum(axis=0), 1e-4)
    # batched Jacobian of an elementwise map: one diagonal per example
    J = nb.vmap(nb.jacrev(nb.exp))(T(X))
    close(J, np.stack([np.diag(np.exp(x)) for x in X]), 1e-4)


def test_errors(emulator):
    x, y = T(np.zeros((3, 2))), T(np.zeros((4, 2)))
    with pytest.raises(ValueError, match="Inconsistent batch dims"):
        nb.vmap(lambda a, b: a + b)(x, y)
    with pytest.raises(ValueError, match="Must specify axis_size"):
        nb.vmap(lambda a: a, in_axes=None)(x)
    with pytest.raises(ValueError, match="doesn't match inferred"):
        nb.vmap(lambda a: a, axis_size=5)(x)
    with pytest.raises(ValueError, match="number of args"):
        nb.vmap(lambda a, b: a, in_axes=(0,))(x, x)
    with pytest.raises(ValueError, match="at least one input"):
        nb.vmap(lambda: x)()
    with pytest.raises(NotImplementedError, match="mesh"):
        nb.vmap(lambda a: a, spmd_axis_name="dp")
