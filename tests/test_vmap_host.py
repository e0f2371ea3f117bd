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


# ---- the batched way: one call of the function, hidden batch dimension ----------------------
def _both_ways(fn, *args, **kw):
    """Result of ``vmap(fn, **kw)(*args)`` run batched and element by element, and how often each
    way called ``fn``."""
    from nabla_amd import config
    calls = []

    def counted(*a):
        calls.append(1)
        return fn(*a)

    out = {}
    for batched in (True, False):
        calls.clear()
        with config.flag("VMAP_BATCHED", batched):
            r = nb.vmap(counted, **kw)(*args)
        leaves = r if isinstance(r, (list, tuple)) else [r]
        out[batched] = ([t.numpy() for t in leaves], len(calls))
    return out


_X = RNG.standard_normal((6, 4, 5))
_Y = RNG.standard_normal((6, 5))
_CASES = {
    "rank mix": (lambda a, b: a * b + 1.0, (_X, _Y), {}),                      # [4,5] * [5]
    "unmapped higher rank": (lambda a, b: a + b, (_Y, _X), {"in_axes": (0, None)}),  # [5] + [6,4,5]
    "matvec both orders": (lambda a, v: (a @ v, v @ a.T), (_X, _Y), {}),
    "reductions": (lambda a: (nb.reduce_sum(a, axis=0), nb.reduce_max(a, axis=-1, keepdims=True),
                              nb.mean(a), nb.cast(nb.argmax(a, axis=1), nb.DType.float32)), (_X,), {}),
    "softmax and where": (lambda a: nb.where(nb.greater(a, 0.0), nb.softmax(a, axis=0), nb.exp(a)), (_X,), {}),
    "views": (lambda a: (a.T, a.reshape(5, 4), a[1:3, ::1], a[2], nb.unsqueeze(a, 1),
                         nb.flatten(a), nb.permute(a, (1, 0))), (_X,), {}),
    "pad concat stack": (lambda a, b: (nb.pad(a, [(1, 0), (0, 2)]), nb.concatenate([a, a * 2.0], axis=1),
                                       nb.stack([b, b + 1.0], axis=0)), (_X, _Y), {}),
    "layer norm": (lambda a: nb.nn.functional.layer_norm(a, T(np.linspace(0.5, 1.5, 5)), T(np.ones(5) * 0.1)),
                   (_X,), {}),
    "mapped axis in the middle, result axis last": (lambda a: nb.tanh(a) * 2.0, (_X,),
                                                    {"in_axes": 1, "out_axes": -1}),
    "constant result": (lambda a: (nb.ones((2,)), a), (_Y,), {"out_axes": (0, 0)}),
    "slice_update": (lambda a, b: nb.slice_update(a, nb.unsqueeze(b, 0), (1, 0), (1, 5)), (_X, _Y), {}),
    "tril": (lambda a: nb.tril(a @ a.T), (_X,), {}),
}


@pytest.mark.parametrize("name", sorted(_CASES))
def test_batched_way_calls_the_function_once_and_agrees(emulator, name):
    fn, arrays, kw = _CASES[name]
    got = _both_ways(fn, *[T(a) for a in arrays], **kw)
    (batched, n_b), (mapped, n_m) = got[True], got[False]
    assert n_b == 1 and n_m > 1  # (once against once per element of the mapped axis)
    assert len(batched) == len(mapped)
    for a, b in zip(batched, mapped):
        assert a.shape == b.shape
        np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-6)


def test_per_example_gradients_cost_one_pass(emulator):
    """vmap(grad(f)) with the parameters unmapped: one forward and one backward over the batch,
    the same launches for 4 and for 32 examples, results those of the element-wise map."""
    from nabla_amd import config
    from nabla_amd.core import engine
    W, B = RNG.standard_normal((5, 7)), RNG.standard_normal((7,))

    def loss(p, x, y):
        return nb.mean((nb.tanh(x @ p["w"] + p["b"]) - y) ** 2.0)

    steps = {}
    for n in (4, 32):
        X, Y = RNG.standard_normal((n, 3, 5)), RNG.standard_normal((n, 3, 7))
        res = {}
        for batched in (True, False):
            with config.flag("VMAP_BATCHED", batched):
                engine.clear_plan_cache()
                g = nb.vmap(nb.grad(loss), in_axes=(None, 0, 0))({"w": T(W), "b": T(B)}, T(X), T(Y))
                res[batched] = {k: v.numpy() for k, v in g.items()}
                if batched:
                    steps[n] = sum(len(bp.plan.steps) for bp in engine._PLAN_CACHE.values())
        engine.clear_plan_cache()
        assert res[True]["w"].shape == (n, 5, 7) and res[True]["b"].shape == (n, 7)
        for k in res[True]:
            np.testing.assert_allclose(res[True][k], res[False][k], rtol=1e-5, atol=1e-6)
        h = np.tanh(X @ W + B)
        dz = 2.0 * (h - Y) / 21.0 * (1.0 - h * h)
        np.testing.assert_allclose(res[True]["w"], np.einsum("nsi,nsj->nij", X, dz), rtol=1e-4, atol=1e-5)
    assert steps[4] == steps[32]


def test_nested_batched_maps_and_vjp_inside(emulator):
    A, Bm = RNG.standard_normal((4, 5)), RNG.standard_normal((3, 5))
    pair = nb.vmap(nb.vmap(lambda a, b: nb.reduce_sum(a * b), in_axes=(0, None)), in_axes=(None, 0))
    close(pair(T(A), T(Bm)), Bm @ A.T)
    # an inner map over a tensor that does not come from the outer one
    mixed = nb.vmap(lambda b: nb.vmap(lambda a: nb.reduce_sum(a * b))(T(A)))
    close(mixed(T(Bm)), Bm @ A.T)

    def pulled(x):
        out, back = nb.vjp(lambda v: nb.exp(v) * 2.0, x)
        return back(nb.ones_like(out))[0]

    close(nb.vmap(pulled)(T(A)), 2.0 * np.exp(A), 1e-4)


def test_ops_without_a_batching_rule_fall_back_to_the_map(emulator):
    """A gather along an inner axis of a table that is itself mapped has no batching rule: the
    function is tried once, then mapped element by element, with the right result either way."""
    tables, idx = RNG.standard_normal((3, 2, 7)), np.array([1, 6, 3, 3])
    calls = []

    def look_up(tab):
        calls.append(1)
        return nb.gather(tab, nb.Tensor.constant(idx.astype(np.int64)), axis=1) * 2.0

    got = nb.vmap(look_up)(T(tables))
    assert len(calls) == 1 + 3  # the batched attempt, then one call per element
    close(got, 2.0 * tables[:, :, idx])


def test_tables_and_filters_of_their_own_per_element(emulator):
    """Rules for operands that used to force the element-by-element map: a convolution whose
    filter (and bias) is mapped, a gather from a mapped table (mapped or shared indices, negative
    ones wrapping inside their own table), a scatter with mapped operands (a row named twice
    keeps its last update).  One call of the function each, values against numpy and against
    the element-by-element map, gradients included: per-example gradients with respect to a
    shared filter are one batched pass."""
    img, filt = RNG.standard_normal((3, 2, 6, 6, 4)), RNG.standard_normal((3, 3, 3, 4, 5))
    bias = RNG.standard_normal((3, 5))

    def check(fn, *args, **kw):
        got = _both_ways(fn, *args, **kw)
        (batched, n_b), (mapped, n_m) = got[True], got[False]
        assert n_b == 1 and n_m == 3, (n_b, n_m)
        for a, b in zip(batched, mapped):
            assert a.shape == b.shape
            np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-5)
        return batched

    check(lambda x, k, b: nb.conv2d(x, k, padding=(1, 1, 0, 2), bias=b), T(img), T(filt), T(bias))
    check(lambda k: nb.conv2d(T(img[0]), k), T(filt))

    def loss(k, b, x):
        return nb.reduce_sum(nb.relu(nb.conv2d(x, k, padding=(1, 1, 1, 1), bias=b)) ** 2.0)

    gk, gb = check(nb.grad(loss, argnums=(0, 1)), T(filt[0]), T(bias[0]), T(img), in_axes=(None, None, 0))
    assert gk.shape == (3, 3, 3, 4, 5) and gb.shape == (3, 5)
    # a strided convolution with a mapped filter still takes the element-by-element map
    got = _both_ways(lambda k: nb.conv2d(T(img[0]), k, stride=(2, 1)), T(filt))
    assert got[True][1] == 1 + 3
    np.testing.assert_allclose(got[True][0][0], got[False][0][0], rtol=1e-5, atol=1e-5)

    tables = RNG.standard_normal((3, 7, 2))
    idx = np.array([[1, 6, -1, 3], [0, 0, 2, 5], [6, -7, 3, 3]], dtype=np.int64)
    I = nb.Tensor.constant(idx)
    (got,) = check(lambda t, i: nb.gather(t, i, axis=0) * 2.0, T(tables), I)
    np.testing.assert_allclose(got, 2.0 * np.stack([tables[b][idx[b]] for b in range(3)]), rtol=1e-6)
    check(lambda t: nb.gather(t, nb.Tensor.constant(idx[0]), axis=0), T(tables))
    check(nb.grad(lambda t, i: nb.reduce_sum(nb.gather(t, i, axis=0) ** 2.0)), T(tables), I)
    upd = RNG.standard_normal((3, 4, 2))
    (got,) = check(lambda t, i, u: nb.scatter(t, i, u, axis=0), T(tables), I, T(upd))
    want = tables.astype(np.float32).copy()
    for b in range(3):
        for j in range(4):
            want[b, idx[b, j]] = upd[b, j]
    np.testing.assert_allclose(got, want, rtol=1e-6)
    # an index outside its own table is an error, not a row of the neighbouring table
    bad = idx.copy()
    bad[0, 0] = 7
    with pytest.raises(IndexError):
        nb.vmap(lambda t, i: nb.gather(t, i, axis=0))(T(tables), nb.Tensor.constant(bad)).numpy()


def test_window_index_and_fused_ops_join_the_hidden_axis(emulator):
    """Convolution and pooling (one filter, mapped images), gathers from one table with mapped
    indices, row-wise cross-entropy and the fused attention op run once on the batch: the hidden
    axis joins the op's own leading axis (or, for a gather, moves out of the middle)."""
    F = nb.nn.functional
    img, filt = RNG.standard_normal((3, 2, 8, 8, 4)), RNG.standard_normal((3, 3, 4, 5))
    table = RNG.standard_normal((7, 3))
    idx = nb.Tensor.constant(np.array([[1, 2], [6, 0], [3, 3]], dtype=np.int64))
    logits = RNG.standard_normal((3, 4, 9))
    labels = nb.Tensor.constant(RNG.integers(0, 9, (3, 4)).astype(np.int64))
    heads = nb.Tensor.constant(RNG.standard_normal((2, 1, 2, 128, 64)).astype(np.float32), dtype=nb.DType.bfloat16)
    cases = [
        (lambda x: nb.avg_pool2d(nb.max_pool2d(nb.relu(nb.conv2d(x, T(filt), padding=(1, 1, 1, 1))),
                                               kernel_size=2), kernel_size=2), (T(img),)),
        (lambda i: F.embedding(i, T(table)) * 2.0, (idx,)),
        (lambda i: nb.gather(T(table.T), i, axis=1), (idx,)),
        (lambda lg, lb: F.cross_entropy_loss(lg, lb), (T(logits), labels)),
        (lambda a: nb.cast(F.scaled_dot_product_attention(a, a, a, is_causal=True), nb.DType.float32), (heads,)),
    ]
    for fn, args in cases:
        got = _both_ways(fn, *args)
        (batched, n_b), (mapped, n_m) = got[True], got[False]
        assert n_b == 1 and n_m == args[0].shape[0]
        for a, b in zip(batched, mapped):
            assert a.shape == b.shape
            np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-6)


def test_convolution_with_a_bias_under_vmap(emulator):
    """conv2d(x, k, bias=b) mapped over images: the bias is the third operand of the op and has
    to survive the batching rule -- values against numpy's own sum (the no-bias result plus b),
    batched and element by element; a mapped bias has no rule and falls back to the element map,
    with the same values."""
    img, filt = RNG.standard_normal((3, 2, 6, 6, 4)), RNG.standard_normal((3, 3, 4, 5))
    bias = RNG.standard_normal((5,)) + 2.0
    f_nb = lambda x: nb.conv2d(x, T(filt), padding=(1, 1, 1, 1))
    f_b = lambda x: nb.conv2d(x, T(filt), padding=(1, 1, 1, 1), bias=T(bias))
    plain = _both_ways(f_nb, T(img))[True][0][0]
    got = _both_ways(f_b, T(img))
    (batched, n_b), (mapped, n_m) = got[True], got[False]
    assert n_b == 1 and n_m == 3
    np.testing.assert_allclose(batched[0], plain + bias, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(mapped[0], plain + bias, rtol=1e-5, atol=1e-5)
    # gradient with respect to the images through the biased convolution, per element
    g = _both_ways(nb.grad(lambda x: nb.reduce_sum(nb.relu(f_b(x)))), T(img))
    np.testing.assert_allclose(g[True][0][0], g[False][0][0], rtol=1e-5, atol=1e-5)
    # one bias per element of the batch
    biases = RNG.standard_normal((3, 5))
    got = _both_ways(lambda x, b: nb.conv2d(x, T(filt), padding=(1, 1, 1, 1), bias=b), T(img), T(biases))
    for way in (True, False):
        np.testing.assert_allclose(got[way][0][0], plain + biases[:, None, None, None, :], rtol=1e-5, atol=1e-5)


def test_forward_mode_inside_a_batched_map(emulator):
    X, V, W = RNG.standard_normal((5, 3)), RNG.standard_normal((5, 3)), RNG.standard_normal((3, 4))

    def pushed(x, v):
        return nb.jvp(lambda a: nb.tanh(a @ T(W)), (x,), (v,))

    out, tan = nb.vmap(pushed)(T(X), T(V))
    close(out, np.tanh(X @ W), 1e-5)
    close(tan, (1.0 - np.tanh(X @ W) ** 2) * (V @ W), 1e-5)


def test_jacobian_by_one_batched_pullback(emulator):
    """jacrev maps the pullback over the identity: the launches of a two-layer Jacobian do not
    grow with the number of outputs, and the result is the chain rule in numpy."""
    from nabla_amd import config
    from nabla_amd.core import engine
    W1, W2, x = RNG.standard_normal((5, 16)), RNG.standard_normal((16, 12)), RNG.standard_normal((5,))
    f = lambda v: nb.tanh(nb.tanh(v @ T(W1)) @ T(W2))
    h = np.tanh(x @ W1)
    y = np.tanh(h @ W2)
    want = ((1 - y ** 2)[:, None] * W2.T) @ ((1 - h ** 2)[:, None] * W1.T)
    steps = {}
    for batched in (True, False):
        with config.flag("VMAP_BATCHED", batched):
            engine.clear_plan_cache()
            J = nb.jacrev(f)(T(x))
            close(J, want, 1e-4)
            steps[batched] = sum(len(bp.plan.steps) for bp in engine._PLAN_CACHE.values())
    engine.clear_plan_cache()
    assert steps[True] * 3 < steps[False]
    H = nb.jacrev(nb.grad(lambda v: nb.reduce_sum(nb.tanh(v @ T(W1)) ** 2.0)))(T(x))
    t = np.tanh(x @ W1)
    d2 = 2.0 * ((1 - t ** 2) ** 2 - 2.0 * t * t * (1 - t ** 2))
    close(H, (W1 * d2) @ W1.T, 1e-4)


def test_forward_mode_jacobian_and_hessian_by_one_batched_pass(emulator):
    """jacfwd pushes the identity of its input through one jvp; forward over reverse gives the
    Hessian in one pass as well.  Launches against the per-direction loop, values against numpy."""
    from nabla_amd import config
    from nabla_amd.core import engine
    W1, W2, x = RNG.standard_normal((5, 16)), RNG.standard_normal((16, 12)), RNG.standard_normal((5,))
    f = lambda v: nb.tanh(nb.tanh(v @ T(W1)) @ T(W2))
    h = np.tanh(x @ W1)
    y = np.tanh(h @ W2)
    want = ((1 - y ** 2)[:, None] * W2.T) @ ((1 - h ** 2)[:, None] * W1.T)
    steps = {}
    for batched in (True, False):
        with config.flag("VMAP_BATCHED", batched):
            engine.clear_plan_cache()
            close(nb.jacfwd(f)(T(x)), want, 1e-4)
            steps[batched] = sum(len(bp.plan.steps) for bp in engine._PLAN_CACHE.values())
    engine.clear_plan_cache()
    assert steps[True] * 3 < steps[False]
    H = nb.jacfwd(nb.grad(lambda v: nb.reduce_sum(nb.tanh(v @ T(W1)) ** 2.0)))(T(x))
    t = np.tanh(x @ W1)
    d2 = 2.0 * ((1 - t ** 2) ** 2 - 2.0 * t * t * (1 - t ** 2))
    close(H, (W1 * d2) @ W1.T, 1e-4)
    # two differentiated arguments: one Jacobian each
    A, B = RNG.standard_normal((3, 4)), RNG.standard_normal((4,))
    ja, jb = nb.jacfwd(lambda a, b: nb.tanh(a @ b), argnums=(0, 1))(T(A), T(B))
    s = 1 - np.tanh(A @ B) ** 2
    want_a = np.zeros((3, 3, 4))
    for i in range(3):
        want_a[i, i] = s[i] * B
    close(ja, want_a, 1e-4)
    close(jb, s[:, None] * A, 1e-4)
