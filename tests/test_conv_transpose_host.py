"""``conv2d_transpose`` on the host path: the reference's own cases
(tests/unit/test_convolution.py:486-587: output shape, vjp and jvp at those shapes and strides)
checked against the float64 oracle (itself pinned by brute force and torch's
``conv_transpose2d``) instead of finite differences, plus the argument checks."""
import numpy as np
import pytest

import nabla_amd as nb
from oracle import ops as O

RNG = np.random.default_rng(53)


def T(a):
    return nb.Tensor.constant(np.asarray(a, dtype=np.float32))


def test_output_shape(emulator):
    y = nb.conv2d_transpose(T(RNG.standard_normal((2, 4, 5, 3))), T(RNG.standard_normal((3, 2, 7, 3))),
                            stride=(2, 1), dilation=(1, 1), padding=(1, 0, 2, 1), output_paddings=(0, 0))
    assert tuple(y.shape) == (2, (4 - 1) * 2 - 1 + 2 + 1, (5 - 1) - 3 + 1 + 1, 7)


@pytest.mark.parametrize("xs,ws,stride,padding,with_bias", [
    ((1, 4, 5, 2), (3, 2, 6, 2), (2, 1), (1, 0, 1, 0), False),
    ((1, 4, 4, 2), (3, 3, 5, 2), (1, 1), (1, 1, 1, 1), True),
    ((2, 3, 4, 3), (2, 2, 4, 3), (2, 2), 0, True),
    ((2, 5, 3, 4), (3, 1, 2, 4), (3, 2), (2, 1), False),
])
def test_forward_vjp_and_jvp_against_oracle(emulator, xs, ws, stride, padding, with_bias):
    x, w = RNG.standard_normal(xs), RNG.standard_normal(ws)
    b = RNG.standard_normal(ws[2]) if with_bias else None
    pad4 = (padding,) * 4 if isinstance(padding, int) else (
        (padding[0], padding[0], padding[1], padding[1]) if len(padding) == 2 else padding)

    def f(xt, wt, *bt):
        return nb.conv2d_transpose(xt, wt, stride=stride, padding=padding, bias=bt[0] if bt else None)

    prim = [T(x), T(w)] + ([T(b)] if with_bias else [])
    y, pull = nb.vjp(f, *prim)
    vs = [O.V(x), O.V(w)] + ([O.V(b)] if with_bias else [])
    oy = O.conv2d_transpose(vs[0], vs[1], vs[2] if with_bias else None, stride, pad4)
    np.testing.assert_allclose(y.numpy(), oy.a, rtol=2e-5, atol=2e-5)
    c = RNG.standard_normal(oy.a.shape)
    want = O.grad_of(O.reduce_sum(oy * c), vs)
    for g, wg in zip(pull(T(c)), want):
        np.testing.assert_allclose(g.numpy(), wg, rtol=2e-5, atol=2e-5)
    # forward mode: the map is bilinear in (x, w) and linear in the bias
    tx, tw = RNG.standard_normal(xs), RNG.standard_normal(ws)
    tans = [T(tx), T(tw)] + ([T(np.ones(ws[2]))] if with_bias else [])
    _, tan = nb.jvp(f, tuple(prim), tuple(tans))
    want_t = (O.conv2d_transpose(O.V(tx), O.V(w), None, stride, pad4).a
              + O.conv2d_transpose(O.V(x), O.V(tw), None, stride, pad4).a + (1.0 if with_bias else 0.0))
    np.testing.assert_allclose(tan.numpy(), want_t, rtol=2e-5, atol=2e-5)


def test_is_the_adjoint_of_conv2d(emulator):
    x, w = RNG.standard_normal((2, 3, 4, 5)), RNG.standard_normal((3, 3, 2, 5))
    y = RNG.standard_normal((2, 6, 8, 2))
    kw = dict(stride=(2, 2), padding=(1, 0, 1, 0))
    lhs = float((nb.conv2d_transpose(T(x), T(w), **kw).numpy().astype(np.float64) * y).sum())
    rhs = float((nb.conv2d(T(y), T(w), **kw).numpy().astype(np.float64) * x).sum())
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), 1.0)


def test_validation(emulator):
    x, w = T(np.zeros((1, 4, 4, 2))), T(np.zeros((3, 3, 5, 2)))
    with pytest.raises(ValueError, match="rank-4"):
        nb.conv2d_transpose(T(np.zeros((4, 4, 2))), w)
    with pytest.raises(ValueError, match="stride values must be > 0"):
        nb.conv2d_transpose(x, w, stride=(0, 1))
    with pytest.raises(ValueError, match="output_paddings"):
        nb.conv2d_transpose(x, w, output_paddings=(1, 0))
    with pytest.raises(ValueError, match="dilation"):
        nb.conv2d_transpose(x, w, dilation=(2, 1))
    with pytest.raises(ValueError, match="must match filter input channels"):
        nb.conv2d_transpose(x, T(np.zeros((3, 3, 5, 3))))
    with pytest.raises(ValueError, match="bias size"):
        nb.conv2d_transpose(x, w, bias=T(np.zeros(4)))
    with pytest.raises(ValueError, match="rank-1"):
        nb.conv2d_transpose(x, w, bias=T(np.zeros((1, 5))))
    with pytest.raises(ValueError, match="Non-positive"):
        nb.conv2d_transpose(T(np.zeros((1, 1, 1, 2))), T(np.zeros((1, 1, 5, 2))), padding=1).numpy()
