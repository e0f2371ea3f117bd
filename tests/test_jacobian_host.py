"""``jacrev`` / ``jacfwd`` on the host path.  The reference checks them against JAX
(tests/unit/test_jacobians.py:37-470), which is not installed here; the same functions and
shapes are pinned instead by closed forms (diag(2x), the Kronecker structure of x @ w) and
by ``torch.autograd.functional.jacobian`` on the CPU, plus rev/fwd agreement."""
import numpy as np
import pytest
import torch

import nabla_amd as nb

RNG = np.random.default_rng(7)


def T(a):
    return nb.Tensor.constant(np.asarray(a, dtype=np.float32))


def tj(f, *xs):
    j = torch.autograd.functional.jacobian(f, tuple(torch.tensor(x, dtype=torch.float64) for x in xs))
    return [a.numpy() for a in j]


def close(got, want):
    got = got.numpy()
    assert got.shape == want.shape, (got.shape, want.shape)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("jac", [nb.jacrev, nb.jacfwd], ids=["rev", "fwd"])
@pytest.mark.parametrize("shape", [(1,), (4,), (3, 4)])
def test_sum_of_squares(emulator, jac, shape):
    x = RNG.standard_normal(shape)
    close(jac(lambda t: nb.reduce_sum(t * t))(T(x)), 2 * x.astype(np.float32))


@pytest.mark.parametrize("jac", [nb.jacrev, nb.jacfwd], ids=["rev", "fwd"])
def test_vector_to_vector_is_diagonal(emulator, jac):
    x = RNG.standard_normal(3)
    close(jac(lambda t: t * t)(T(x)), np.diag(2 * x).astype(np.float32))
    close(jac(nb.exp)(T(x)), np.diag(np.exp(x)).astype(np.float32))


@pytest.mark.parametrize("jac", [nb.jacrev, nb.jacfwd], ids=["rev", "fwd"])
def test_matmul_jacobian(emulator, jac):
    x, w = RNG.standard_normal((4, 3)), RNG.standard_normal((3, 2))
    want = np.einsum("ik,lj->ijkl", np.eye(4), w)      # d(xw)[i,j] / dx[k,l] = [i == k] w[l,j]
    got = jac(lambda t: nb.matmul(t, T(w)))(T(x))
    close(got, want.astype(np.float32))
    np.testing.assert_allclose(got.numpy(), tj(lambda a: a @ torch.tensor(w), x)[0], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("jac", [nb.jacrev, nb.jacfwd], ids=["rev", "fwd"])
def test_composite_against_torch(emulator, jac):
    x, w = RNG.standard_normal((2, 3)), RNG.standard_normal((3, 3))
    f = lambda a, b: nb.softmax(nb.gelu(nb.matmul(a, b)) * 0.7, axis=-1)
    g = lambda a, b: torch.softmax(torch.nn.functional.gelu(a @ b) * 0.7, dim=-1)
    want = tj(g, x, w)
    got = jac(f, argnums=(0, 1))(T(x), T(w))
    assert isinstance(got, tuple) and len(got) == 2
    close(got[0], want[0].astype(np.float32))
    close(got[1], want[1].astype(np.float32))


@pytest.mark.parametrize("jac", [nb.jacrev, nb.jacfwd], ids=["rev", "fwd"])
def test_argnums(emulator, jac):
    x, y = RNG.standard_normal(4), RNG.standard_normal(4)
    f = lambda a, b: nb.reduce_sum(a * b)
    close(jac(f, argnums=0)(T(x), T(y)), y.astype(np.float32))
    close(jac(f, argnums=1)(T(x), T(y)), x.astype(np.float32))
    close(jac(f, argnums=-1)(T(x), T(y)), x.astype(np.float32))
    both = jac(f)(T(x), T(y))                            # None: every argument
    close(both[0], y.astype(np.float32))
    close(both[1], x.astype(np.float32))
    with pytest.raises(ValueError, match="out of bounds"):
        jac(f, argnums=2)(T(x), T(y))


@pytest.mark.parametrize("jac", [nb.jacrev, nb.jacfwd], ids=["rev", "fwd"])
def test_has_aux_and_multiple_outputs(emulator, jac):
    x = RNG.standard_normal(3)
    j, aux = jac(lambda t: (t * t, "kept"), has_aux=True)(T(x))
    assert aux == "kept"
    close(j, np.diag(2 * x).astype(np.float32))
    with pytest.raises(NotImplementedError, match="multiple output tensors"):
        jac(lambda t: (t * t, t + 1.0))(T(x))


def test_rev_and_fwd_agree_and_hessian(emulator):
    x = RNG.standard_normal((2, 3))
    f = lambda t: nb.reduce_sum(nb.exp(t) * t, axis=1)
    np.testing.assert_allclose(nb.jacrev(f)(T(x)).numpy(), nb.jacfwd(f)(T(x)).numpy(), rtol=1e-5, atol=1e-6)
    # forward over reverse: the Hessian of sum(x^3) is diag(6x)
    v = RNG.standard_normal(4)
    h = nb.jacfwd(nb.grad(lambda t: nb.reduce_sum(t * t * t)))(T(v))
    close(h, np.diag(6 * v).astype(np.float32))
