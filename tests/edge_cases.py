"""Edge cases shared by the host (emulator) and GPU tests: tensors without elements, log1p and
atanh at the ends of their domains."""
import numpy as np
import pytest


def check_empty_tensors(nb):
    T = nb.Tensor.constant
    e = np.zeros((0, 3), np.float32)
    assert (T(e) + 1).numpy().shape == (0, 3)
    assert nb.exp(T(e) * 2.0).numpy().shape == (0, 3)
    np.testing.assert_array_equal(nb.reduce_sum(T(e), axis=0).numpy(), np.zeros(3, np.float32))
    assert nb.reduce_sum(T(e), axis=1).numpy().shape == (0,)
    with pytest.raises(Exception, match="length 0"):
        nb.reduce_max(T(e), axis=0).numpy()
    assert (T(e) @ T(np.ones((3, 4), np.float32))).numpy().shape == (0, 4)
    np.testing.assert_array_equal((T(np.zeros((2, 0), np.float32)) @ T(np.ones((0, 4), np.float32))).numpy(),
                                  np.zeros((2, 4), np.float32))
    both = nb.concatenate([T(e), T(np.ones((2, 3), np.float32))], axis=0)
    np.testing.assert_array_equal(both.numpy(), np.ones((2, 3), np.float32))
    g = nb.grad(lambda x: nb.reduce_sum(x * x))(T(e))
    assert g.numpy().shape == (0, 3)
    # a compiled function with an empty argument and a non-empty one
    f = nb.compile(lambda a, b: (a * 2.0, nb.reduce_sum(a) + nb.reduce_sum(b)))
    a2, s = f(T(e), T(np.ones((2, 2), np.float32)))
    assert a2.numpy().shape == (0, 3) and float(s.numpy()) == 4.0
    # vmap over an axis of length 0 keeps the element shape
    out = nb.vmap(lambda r: (r * 2.0, nb.reduce_sum(r)))(T(e))
    assert out[0].numpy().shape == (0, 3) and out[1].numpy().shape == (0,)


def check_log1p_and_atanh_at_the_edges(nb):
    T = nb.Tensor.constant
    x = np.array([np.inf, 1.0, -1.0, 0.0, 1e-10, 3e38], np.float32)
    with np.errstate(all="ignore"):
        want = np.log1p(x.astype(np.float64))
    got = nb.log1p(T(x)).numpy()
    assert got[0] == np.inf and got[2] == -np.inf and got[3] == 0.0
    np.testing.assert_allclose(got[[1, 4, 5]], want[[1, 4, 5]], rtol=1e-6)
    a = nb.atanh(T(np.array([1.0, -1.0, 0.5, 0.0], np.float32))).numpy()
    assert a[0] == np.inf and a[1] == -np.inf and a[3] == 0.0
    np.testing.assert_allclose(a[2], np.arctanh(0.5), rtol=1e-6)
    # the gradient away from the edge is untouched by the edge handling
    g = nb.grad(lambda t: nb.reduce_sum(nb.log1p(t)))(T(np.array([0.5, 2.0, 1e-9], np.float32))).numpy()
    np.testing.assert_allclose(g, 1.0 / (1.0 + np.array([0.5, 2.0, 1e-9])), rtol=2e-6)
