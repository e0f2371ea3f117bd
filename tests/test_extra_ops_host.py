"""The small composite ops (``trunc``, ``floor``, ``is_nan``, ``is_inf``, ``log1p``,
``logical_xor``, ``outer``, ``flip``, ``split``, ``chunk``, ``unbind``, ``minmax``) against numpy on
the host path: integer-valued, boolean and view results exactly, ``log1p`` against numpy's
``log1p`` in float64 including arguments far below the fp32 epsilon, gradients in closed form."""
import numpy as np
import pytest

import nabla_amd as nb

RNG = np.random.default_rng(71)


def T(a, dtype=np.float32):
    return nb.Tensor.constant(np.asarray(a, dtype=dtype))


def test_trunc_floor_exact_and_zero_gradient(emulator):
    x = np.array([-2.5, -2.0, -0.3, -0.0, 0.0, 0.7, 1.0, 1.5, 1e6 + 0.5, -1e6 - 0.5], np.float32)
    np.testing.assert_array_equal(nb.trunc(T(x)).numpy(), np.trunc(x))
    np.testing.assert_array_equal(nb.floor(T(x)).numpy(), np.floor(x))
    g = nb.grad(lambda t: nb.reduce_sum(nb.floor(t) * t))(T(x))       # d/dx floor(x) x = floor(x)
    np.testing.assert_array_equal(g.numpy(), np.floor(x))
    i = np.arange(-3, 4, dtype=np.int32)
    np.testing.assert_array_equal(nb.floor(T(i, np.int32)).numpy(), i)


def test_nan_inf_xor(emulator):
    x = np.array([0.0, np.nan, np.inf, -np.inf, 1.0, -np.nan], np.float32)
    np.testing.assert_array_equal(nb.is_nan(T(x)).numpy(), np.isnan(x))
    np.testing.assert_array_equal(nb.is_inf(T(x)).numpy(), np.isinf(x))
    a, b = np.array([True, True, False, False]), np.array([True, False, True, False])
    np.testing.assert_array_equal(nb.logical_xor(T(a, bool), T(b, bool)).numpy(), a ^ b)


def test_log1p_small_and_large_arguments(emulator):
    x = np.array([0.0, 1e-12, -1e-12, 3e-8, -3e-8, 1e-4, -1e-4, 0.5, -0.5, 3.0, 100.0, -0.999], np.float32)
    got = nb.log1p(T(x)).numpy().astype(np.float64)
    want = np.log1p(x.astype(np.float64))
    np.testing.assert_allclose(got, want, rtol=3e-7, atol=0)
    g = nb.grad(lambda t: nb.reduce_sum(nb.log1p(t)))(T(x[5:])).numpy()
    np.testing.assert_allclose(g, 1.0 / (1.0 + x[5:].astype(np.float64)), rtol=2e-4)


def test_outer_flip(emulator):
    a, b = RNG.standard_normal(3), RNG.standard_normal(4)
    np.testing.assert_allclose(nb.outer(T(a), T(b)).numpy(), np.outer(a, b).astype(np.float32), rtol=1e-6)
    x = RNG.standard_normal((3, 4, 5)).astype(np.float32)
    for ax in (0, 1, -1):
        np.testing.assert_array_equal(nb.flip(T(x), ax).numpy(), np.flip(x, ax))
    w = RNG.standard_normal((3, 4, 5)).astype(np.float32)
    g = nb.grad(lambda t: nb.reduce_sum(nb.flip(t, 1) * T(w)))(T(x))
    np.testing.assert_array_equal(g.numpy(), np.flip(w, 1))
    with pytest.raises(ValueError, match="out of range"):
        nb.flip(T(x), 3)


def test_split_chunk_unbind_minmax(emulator):
    x = RNG.standard_normal((6, 5)).astype(np.float32)
    for got, want in zip(nb.split(T(x), 3, axis=0), np.split(x, 3, axis=0)):
        np.testing.assert_array_equal(got.numpy(), want)
    with pytest.raises(ValueError, match="not divisible"):
        nb.split(T(x), 4, axis=0)
    parts = nb.chunk(T(x), 2, axis=1)
    assert [tuple(p.shape) for p in parts] == [(6, 3), (6, 2)]
    np.testing.assert_array_equal(parts[1].numpy(), x[:, 3:])
    rows = nb.unbind(T(x), axis=1)
    assert len(rows) == 5 and tuple(rows[0].shape) == (6,)
    np.testing.assert_array_equal(rows[4].numpy(), x[:, 4])
    mm = nb.minmax(T(x))
    assert float(mm["min"].numpy()) == x.min() and float(mm["max"].numpy()) == x.max()
    # gradients flow back through the pieces into their places
    g = nb.grad(lambda t: nb.reduce_sum(nb.chunk(t, 2, axis=1)[1] * 2.0) + nb.reduce_sum(nb.unbind(t, 0)[2]))(T(x))
    want = np.zeros_like(x); want[:, 3:] += 2.0; want[2] += 1.0
    np.testing.assert_array_equal(g.numpy(), want)


def test_sin_cos_values_and_derivatives(emulator):
    x = RNG.uniform(-8, 8, (4, 37)).astype(np.float32)
    np.testing.assert_allclose(nb.sin(T(x)).numpy(), np.sin(x.astype(np.float64)), rtol=0, atol=2e-7)
    np.testing.assert_allclose(nb.cos(T(x)).numpy(), np.cos(x.astype(np.float64)), rtol=0, atol=2e-7)
    g = nb.grad(lambda t: nb.reduce_sum(nb.sin(t) * nb.cos(t)))(T(x))          # d/dx sin cos = cos 2x
    np.testing.assert_allclose(g.numpy(), np.cos(2 * x.astype(np.float64)), rtol=0, atol=1e-6)
    _, tan = nb.jvp(nb.cos, (T(x),), (T(np.ones_like(x)),))
    np.testing.assert_allclose(tan.numpy(), -np.sin(x.astype(np.float64)), rtol=0, atol=2e-7)
    # sinusoidal position table of the transformer examples: sin on even, cos on odd columns
    pos, d = np.arange(16)[:, None], np.arange(8)[None, :]
    ang = (pos / 10000 ** (2 * (d // 2) / 8)).astype(np.float32)
    table = nb.where(T((d % 2 == 0) * np.ones_like(ang), bool), nb.sin(T(ang)), nb.cos(T(ang)))
    want = np.where(d % 2 == 0, np.sin(ang.astype(np.float64)), np.cos(ang.astype(np.float64)))
    np.testing.assert_allclose(table.numpy(), want, rtol=0, atol=2e-7)


def test_atanh(emulator):
    x = np.array([0.0, 1e-10, -1e-10, 1e-4, -0.3, 0.5, 0.9, -0.99, 0.999], np.float32)
    got = nb.atanh(T(x)).numpy().astype(np.float64)
    np.testing.assert_allclose(got, np.arctanh(x.astype(np.float64)), rtol=1e-6, atol=0)
    g = nb.grad(lambda t: nb.reduce_sum(nb.atanh(t)))(T(x[3:])).numpy()
    np.testing.assert_allclose(g, 1.0 / (1.0 - x[3:].astype(np.float64) ** 2), rtol=3e-4)


def test_tensors_without_elements(emulator):
    from edge_cases import check_empty_tensors
    check_empty_tensors(nb)


def test_log1p_and_atanh_at_the_edges(emulator):
    from edge_cases import check_log1p_and_atanh_at_the_edges
    check_log1p_and_atanh_at_the_edges(nb)
