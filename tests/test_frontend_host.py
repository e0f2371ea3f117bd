"""Host logic (no GPU): tracing, autodiff replay, lowering / fusion / view
folding, plan cache and ``compile`` semantics, checked by running the produced
launch records on the numpy interpreter of oracle/emulator.py and comparing with
the CPU oracle.  The HIP path itself is covered by the ``gpu`` tests."""
import numpy as np
import pytest

import nabla_amd as nb
from oracle import configs as oc
from oracle import ops as O

RNG = np.random.default_rng(11)
F = nb.nn.functional


def T(a, dtype=None):
    return nb.Tensor.constant(a, dtype=dtype)


def last_plan():
    from nabla_amd.core.engine import _PLAN_CACHE
    return list(_PLAN_CACHE.values())[-1].plan


def relerr(a, b):
    return np.abs(np.asarray(a, np.float64) - b).max() / (np.abs(b).max() + 1e-30)


# ---- ops ---------------------------------------------------------------------------
def test_elementwise_broadcast_and_scalars(emulator):
    x = RNG.standard_normal((3, 1, 5)).astype(np.float32)
    y = RNG.standard_normal((4, 5)).astype(np.float32)
    z = (T(x) + T(y)) * 2.0 - 1.0 / (nb.exp(T(y)) + 1.0)
    ref = (x + y) * np.float32(2.0) - np.float32(1.0) / (np.exp(y) + np.float32(1.0))
    np.testing.assert_allclose(z.numpy(), ref, rtol=1e-6, atol=1e-6)
    assert z.shape == (3, 4, 5)
    # the arithmetic ops are single IEEE operations: bit-exact against numpy
    np.testing.assert_array_equal((T(x) * T(x) - T(x)).numpy(), x * x - x)


def test_comparisons_where_cast_are_exact(emulator):
    x = RNG.standard_normal((6, 7)).astype(np.float32)
    y = RNG.standard_normal((6, 7)).astype(np.float32)
    m = nb.greater(T(x), T(y))
    assert m.dtype is nb.DType.bool
    np.testing.assert_array_equal(m.numpy(), x > y)
    np.testing.assert_array_equal(nb.equal(T(x), T(x)).numpy(), np.ones_like(x, bool))
    np.testing.assert_array_equal(nb.where(m, T(x), T(y)).numpy(), np.where(x > y, x, y))
    np.testing.assert_array_equal(nb.cast(m, nb.DType.float32).numpy(), (x > y).astype(np.float32))
    np.testing.assert_array_equal(nb.less(T(x), 0.0).numpy(), x < 0)


def test_reductions_all_axes_and_keepdims(emulator):
    x = RNG.standard_normal((3, 4, 5)).astype(np.float32)
    for axis in (None, 0, 1, -1, (0, 2), (1, 2)):
        for keep in (False, True):
            np.testing.assert_allclose(nb.reduce_sum(T(x), axis=axis, keepdims=keep).numpy(),
                                       x.sum(axis=axis, keepdims=keep), rtol=1e-5, atol=1e-5)
            np.testing.assert_array_equal(nb.reduce_max(T(x), axis=axis, keepdims=keep).numpy(),
                                          x.max(axis=axis, keepdims=keep))
    np.testing.assert_allclose(nb.mean(T(x), axis=(0, 1)).numpy(), x.mean(axis=(0, 1)), rtol=1e-5)
    assert nb.argmax(T(x), axis=1).dtype is nb.DType.int64
    np.testing.assert_array_equal(nb.argmax(T(x), axis=1).numpy(), x.argmax(1))
    np.testing.assert_array_equal(nb.argmax(T(x), axis=-1, keepdims=True).numpy(),
                                  x.argmax(-1)[..., None])


def test_views_are_folded_not_copied(emulator):
    x = RNG.standard_normal((4, 6, 8)).astype(np.float32)
    y = nb.swap_axes(T(x), 0, 2)[1:5] * 1.0
    np.testing.assert_array_equal(y.numpy(), x.transpose(2, 1, 0)[1:5])
    stats = last_plan().stats
    assert stats.get("copy", 0) == 0, stats  # permute + slice became strides of one kernel
    z = nb.reshape(nb.permute(T(x), (1, 0, 2)), (6, 32))  # needs one materialisation
    np.testing.assert_array_equal(z.numpy(), x.transpose(1, 0, 2).reshape(6, 32))
    b = nb.broadcast_to(nb.unsqueeze(T(x[0, 0]), 0), (5, 8)) + 0.0
    np.testing.assert_array_equal(b.numpy(), np.broadcast_to(x[0, 0], (5, 8)))
    np.testing.assert_array_equal(nb.squeeze(nb.unsqueeze(T(x), 1), 1).numpy(), x)
    np.testing.assert_array_equal(nb.flatten(T(x), 1).numpy(), x.reshape(4, 48))
    np.testing.assert_array_equal(nb.moveaxis(T(x), 0, 2).numpy(), np.moveaxis(x, 0, 2))
    np.testing.assert_array_equal(nb.stack([T(x), T(x)], axis=1).numpy(), np.stack([x, x], 1))
    np.testing.assert_array_equal(
        nb.slice_update(T(x), T(np.zeros((2, 6, 3), np.float32)), (1, 0, 2), (2, 6, 3)).numpy(),
        np.concatenate([x[:, :, :2], np.where(np.isin(np.arange(4), [1, 2])[:, None, None],
                                               0, x[:, :, 2:5]), x[:, :, 5:]], 2))


def test_creation_ops(emulator):
    np.testing.assert_array_equal(nb.zeros((2, 3)).numpy(), np.zeros((2, 3), np.float32))
    np.testing.assert_array_equal(nb.full((4,), 2.5).numpy(), np.full(4, 2.5, np.float32))
    np.testing.assert_array_equal(nb.arange(0, 7, dtype=nb.DType.int64).numpy(), np.arange(7))
    np.testing.assert_array_equal(nb.arange(1, 4, 0.5).numpy(), np.arange(1, 4, 0.5, dtype=np.float32))
    x = RNG.standard_normal((2, 5, 5)).astype(np.float32)
    np.testing.assert_array_equal(nb.tril(T(x)).numpy(), np.tril(x))
    np.testing.assert_array_equal(nb.triu(T(x), 1).numpy(), np.triu(x, 1))
    np.testing.assert_array_equal(nb.ones_like(T(x)).numpy(), np.ones_like(x))


def test_matmul_promotion_rules(emulator):
    a = RNG.standard_normal((5, 4)).astype(np.float32)
    b = RNG.standard_normal((4, 3)).astype(np.float32)
    v = RNG.standard_normal((4,)).astype(np.float32)
    np.testing.assert_allclose((T(a) @ T(b)).numpy(), a @ b, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose((T(a) @ T(v)).numpy(), a @ v, rtol=1e-5, atol=1e-6)      # 1-D rhs
    np.testing.assert_allclose((T(v) @ T(b)).numpy(), v @ b, rtol=1e-5, atol=1e-6)      # 1-D lhs
    batched = RNG.standard_normal((2, 3, 5, 4)).astype(np.float32)
    np.testing.assert_allclose((T(batched) @ T(b)).numpy(), batched @ b, rtol=1e-5, atol=1e-6)  # batch broadcast
    with pytest.raises(ValueError):
        T(a) @ T(a)


# ---- autodiff -------------------------------------------------------------------------
def test_grad_value_and_grad_vjp_agree_with_oracle(emulator):
    x = RNG.standard_normal((4, 6)).astype(np.float32)
    w = RNG.standard_normal((6, 3)).astype(np.float32)

    def f(x, w):
        return nb.mean(nb.tanh(x @ w) * nb.sigmoid(x @ w))

    vx, vw = O.V(x.astype(np.float64)), O.V(w.astype(np.float64))
    h = O.matmul(vx, vw)
    ref_loss = O.mean(O.tanh(h) * (O.V(1.0) / (O.exp(O.neg(h)) + 1.0)))
    gx_ref, gw_ref = O.grad_of(ref_loss, [vx, vw])
    g = nb.grad(f, argnums=(0, 1))(T(x), T(w))
    assert relerr(g[0].numpy(), gx_ref) < 1e-5 and relerr(g[1].numpy(), gw_ref) < 1e-5
    val, g1 = nb.value_and_grad(f, argnums=1)(T(x), T(w))
    assert abs(val.item() - float(ref_loss.a)) < 1e-6
    assert relerr(g1.numpy(), gw_ref) < 1e-5
    out, pullback = nb.vjp(f, T(x), T(w))
    gx2, gw2 = pullback(nb.ones_like(out))
    assert relerr(gx2.numpy(), gx_ref) < 1e-5 and relerr(gw2.numpy(), gw_ref) < 1e-5


def test_grad_stays_lazy_and_unreached_inputs_get_zeros(emulator):
    x, y = T(np.ones((3,), np.float32)), T(np.ones((3,), np.float32))
    gx, gy = nb.grad(lambda a, b: nb.reduce_sum(a * 2.0), argnums=(0, 1))(x, y)
    assert not gx.real  # create_graph=True keeps results lazy (grad.py:23-25)
    np.testing.assert_array_equal(gx.numpy(), np.full(3, 2.0, np.float32))
    np.testing.assert_array_equal(gy.numpy(), np.zeros(3, np.float32))


def test_pytorch_style_backward_accumulates(emulator):
    w = T(RNG.standard_normal((4, 2)).astype(np.float32)).requires_grad_(True)
    x = T(RNG.standard_normal((3, 4)).astype(np.float32))
    loss = nb.mean((x @ w) * (x @ w))
    loss.backward()
    g1 = w.grad.numpy().copy()
    ref = 2 * x.numpy().T @ (x.numpy() @ w.numpy()) / 6
    np.testing.assert_allclose(g1, ref, rtol=1e-5, atol=1e-6)
    nb.mean((x @ w) * (x @ w)).backward()
    np.testing.assert_allclose(w.grad.numpy(), 2 * g1, rtol=1e-5, atol=1e-6)


def test_second_order_through_create_graph(emulator):
    x = T(np.array([0.3, -1.2, 2.0], np.float32))
    f = lambda t: nb.reduce_sum(t * t * t)
    gg = nb.grad(lambda t: nb.reduce_sum(nb.grad(f)(t)))(x)
    np.testing.assert_allclose(gg.numpy(), 6 * x.numpy(), rtol=1e-5)


def test_vjp_error_is_wrapped(emulator):
    class Broken(nb.UnaryOperation):
        @property
        def name(self):
            return "broken"

        def kernel(self, args, kwargs):
            from nabla_amd.backend import ir
            return [ir.ew("mov", args[0])]

    with pytest.raises(RuntimeError, match="VJP rule failed for operation 'broken'"):
        nb.grad(lambda t: nb.reduce_sum(Broken()([t], {})[0]))(T(np.ones(2, np.float32)))


# ---- fusion structure ---------------------------------------------------------------------
def test_layernorm_softmax_forward_is_one_kernel(emulator):
    x = RNG.standard_normal((8, 64)).astype(np.float32)
    w, b = np.ones(64, np.float32), np.zeros(64, np.float32)
    y = nb.softmax(F.layer_norm(T(x), T(w), T(b)), axis=-1)
    ref = O.softmax(O.layer_norm(O.V(x.astype(np.float64)), O.V(w), O.V(b))).a
    assert relerr(y.numpy(), ref) < 1e-5
    stats = last_plan().stats
    assert stats["rowprog"] == 1 and stats["steps"] == 1, stats


def test_bias_add_rides_in_the_matmul(emulator):
    """x @ W + b with a row-vector b: the add is folded into the product's epilogue; a product
    with a second reader keeps its add (the plain product is needed too)."""
    x = RNG.standard_normal((3, 16, 32)).astype(np.float32)
    W = RNG.standard_normal((32, 24)).astype(np.float32)
    b = RNG.standard_normal((1, 24)).astype(np.float32)
    y = T(x) @ T(W) + T(b)
    ref = x.astype(np.float64) @ W + b
    assert relerr(y.numpy(), ref) < 1e-5
    plan = last_plan()
    assert plan.stats == {"steps": 1, "units": 1, "fused_groups": 0, "gemm": 1}, plan.stats
    assert plan.steps[0].attrs.get("bias") is not None
    # two readers of the product
    X, Wt, bt = T(x), T(W), T(b)
    p = X @ Wt
    y2, z2 = p + bt, nb.relu(p)
    nb.realize_all(y2, z2)
    assert relerr(y2.numpy(), ref) < 1e-5
    assert relerr(z2.numpy(), np.maximum(x.astype(np.float64) @ W, 0)) < 1e-5
    plan = last_plan()
    assert all(s.attrs.get("bias") is None for s in plan.steps if s.kind == "gemm")
    # gradients flow through the folded form as before
    def loss(Wt, bt):
        return nb.reduce_sum(nb.relu(X @ Wt + bt))
    gW, gb = nb.grad(loss, argnums=(0, 1), realize=True)(Wt, bt)
    mask = ((x.astype(np.float64) @ W + b) > 0).astype(np.float64)
    assert relerr(gW.numpy(), np.einsum("bmk,bmn->kn", x.astype(np.float64), mask)) < 1e-5
    assert relerr(gb.numpy(), mask.sum(axis=(0, 1))[None, :]) < 1e-5


def test_forward_traced_twice_is_computed_once(emulator):
    x = T(RNG.standard_normal((16, 128)).astype(np.float32))
    y = T(RNG.standard_normal((16, 128)).astype(np.float32))
    out, gx = nb.workloads.c2_step(x, y)
    nb.realize_all(out, gx)
    plan = last_plan()
    progs = [s for s in plan.steps if s.kind == "rowprog"]
    assert len(progs) == 1, plan.stats
    n_exp = sum(1 for i in progs[0].attrs["members"] if i == "ew.exp")
    assert n_exp == 1  # common-subexpression elimination merged the two traces


def test_plan_cache_is_structural_not_by_value(emulator):
    from nabla_amd.core.engine import clear_plan_cache, get_cache_stats
    clear_plan_cache()
    for k in range(3):
        a = T(RNG.standard_normal((4, 4)).astype(np.float32))
        (nb.relu(a) * float(k + 1)).numpy()
    st = get_cache_stats()
    assert st["misses"] == 1 and st["hits"] == 2, st
    (nb.relu(T(np.ones((5, 4), np.float32))) * 2.0).numpy()  # another shape: new plan
    assert get_cache_stats()["misses"] == 2
    # x*x and x*y have different structure even with equal shapes
    a = T(np.full((4, 4), 3.0, np.float32))
    b = T(np.full((4, 4), 5.0, np.float32))
    np.testing.assert_array_equal((a * a).numpy(), np.full((4, 4), 9.0, np.float32))
    np.testing.assert_array_equal((a * b).numpy(), np.full((4, 4), 15.0, np.float32))


# ---- compile (behavioural spec: reference tests/unit/test_compile.py:18-77) --------------------
def test_compile_basic_hits_and_misses(emulator):
    @nb.compile
    def f(x):
        return x * 2.0 + 1.0

    x_np = np.array([1.0, 2.0, 3.0], dtype=np.float32)
    x = nb.Tensor.constant(x_np)
    np.testing.assert_allclose(f(x).to_numpy(), x_np * 2.0 + 1.0)
    assert f.stats.misses == 1 and f.stats.hits == 0
    np.testing.assert_allclose(f(x).to_numpy(), x_np * 2.0 + 1.0)
    assert f.stats.misses == 1 and f.stats.hits == 1
    np.testing.assert_allclose(f(T(x_np + 5)).to_numpy(), (x_np + 5) * 2.0 + 1.0)  # new values, same plan
    assert f.stats.hits == 2


def test_compile_dynamic_dims_reuse_signature(emulator):
    @nb.compile(dynamic_dims={0: {0: "batch"}})
    def f(x, w):
        return x @ w

    w_np = RNG.standard_normal((4, 3)).astype(np.float32)
    x1 = RNG.standard_normal((2, 4)).astype(np.float32)
    x2 = RNG.standard_normal((5, 4)).astype(np.float32)
    w = T(w_np)
    np.testing.assert_allclose(f(T(x1), w).to_numpy(), x1 @ w_np, atol=1e-5)
    assert f.stats.misses == 1
    f(T(x1), w)
    assert f.stats.hits == 1
    np.testing.assert_allclose(f(T(x2), w).to_numpy(), x2 @ w_np, atol=1e-5)
    assert f.stats.hits == 2 and f.stats.misses == 1  # a new batch size is not a new signature


def test_compile_train_step_with_pytrees_and_closures(emulator):
    scale = T(np.float32(0.5))

    @nb.compile
    def step(params, x):
        loss, g = nb.value_and_grad(lambda p, x: nb.mean((x @ p["w"] + p["b"]) ** 2.0) * scale)(params, x)
        return loss, {k: params[k] - g[k] * 0.1 for k in params}

    p = {"w": T(RNG.standard_normal((4, 2)).astype(np.float32)), "b": T(np.zeros((1, 2), np.float32))}
    x = T(RNG.standard_normal((8, 4)).astype(np.float32))
    l0, p1 = step(p, x)
    l1, p2 = step(p1, x)
    l2, _ = step(p2, x)
    assert step.stats.misses == 1 and step.stats.hits == 2
    assert l2.item() < l1.item() < l0.item()


# ---- nn modules ----------------------------------------------------------------------------
def test_modules_are_pytrees_and_track_parameters(emulator):
    nn = nb.nn
    nn.functional.manual_seed(0)
    layer = nn.TransformerEncoderLayer(16, 4, dim_feedforward=32, dropout=0.0)
    names = [n for n, _ in layer.named_parameters()]
    assert "self_attn.q_proj.weight" in names and "norm2.bias" in names and len(names) == 16
    leaves, treedef = nb.tree_flatten(layer)
    rebuilt = nb.tree_unflatten(treedef, leaves)
    x = T(RNG.standard_normal((2, 5, 16)).astype(np.float32))
    np.testing.assert_allclose(rebuilt(x, is_causal=True).numpy(), layer(x, is_causal=True).numpy())
    lin = nn.Linear(3, 2)
    assert lin.weight.shape == (3, 2) and lin.bias.shape == (1, 2)  # (in, out) and (1, out)
    sd = lin.state_dict()
    lin2 = nn.Linear(3, 2)
    lin2.load_state_dict(sd)
    np.testing.assert_array_equal(lin2.weight.numpy(), lin.weight.numpy())


def test_module_forward_matches_oracle_block(emulator):
    t = oc.c3_inputs(2, 8, 16, 32, seed=3, bf16=False)
    want, _ = oc.c3_reference(t, num_heads=4)
    nn = nb.nn
    layer = nn.TransformerEncoderLayer(16, 4, dim_feedforward=32, dropout=0.0)
    sd = {"self_attn.q_proj.weight": "wq", "self_attn.q_proj.bias": "bq", "self_attn.k_proj.weight": "wk",
          "self_attn.k_proj.bias": "bk", "self_attn.v_proj.weight": "wv", "self_attn.v_proj.bias": "bv",
          "self_attn.out_proj.weight": "wo", "self_attn.out_proj.bias": "bo", "linear1.weight": "w1",
          "linear1.bias": "b1", "linear2.weight": "w2", "linear2.bias": "b2", "norm1.weight": "ln1_w",
          "norm1.bias": "ln1_b", "norm2.weight": "ln2_w", "norm2.bias": "ln2_b"}
    layer.load_state_dict({k: T(t[v]) for k, v in sd.items()})
    out = layer(T(t["x"]), is_causal=True)
    assert abs(nb.mean(out * out).item() - want) < 1e-5 * abs(want)


# ---- whole configurations at reduced size -----------------------------------------------------
def test_configs_reduced_against_oracle(emulator):
    t = oc.c3_inputs(2, 16, 32, 64, seed=0, bf16=False)
    wl, wg = oc.c3_reference(t, num_heads=4)
    loss, grads = oc.c3_program(nb, oc.upload(nb, t), num_heads=4)
    nb.realize_all(loss, *grads.values())
    assert abs(loss.item() - wl) < 1e-5 * abs(wl)
    scale = max(np.abs(g).max() for g in wg.values())
    for k in oc.C3_PARAMS:
        assert np.abs(grads[k].numpy() - wg[k]).max() <= 2e-5 * max(np.abs(wg[k]).max(), 1e-3 * scale), k

    t = oc.c4_inputs(batch=4, hw=8, c=(3, 8, 16, 32), seed=0)
    wl, wg, wam, _ = oc.c4_reference(t)
    T4 = oc.upload(nb, t)
    loss, grads = oc.c4_program(nb, T4)
    am = nb.argmax(oc.c4_logits(nb, {k: T4[k] for k in oc.C4_PARAMS}, T4["img"]), axis=-1)
    nb.realize_all(loss, am, *grads.values())
    assert abs(loss.item() - wl) < 1e-5 * abs(wl)
    np.testing.assert_array_equal(am.numpy(), wam)
    for k in oc.C4_PARAMS:
        assert relerr(grads[k].numpy(), wg[k]) < 2e-5, k

    t = oc.c5_inputs(layers=2, batch=2, seq=8, d_model=32, d_ff=64, vocab=50, rank=4, seed=0,
                     b_zero=False, bf16=False)
    wl, wg = oc.c5_reference(t, num_heads=4)
    loss, grads = oc.c5_program(nb, oc.upload(nb, t), num_heads=4)
    flat = [ad[k] for ad in grads for k in ("qA", "qB", "vA", "vB")]
    nb.realize_all(loss, *flat)
    assert abs(loss.item() - wl) < 1e-5 * abs(wl)
    for g, w in zip(flat, wg):
        assert relerr(g.numpy(), w) < 2e-5


# ---- validation messages the reference tests match on --------------------------------------------
def test_conv_and_pool_validation(emulator):
    x = T(np.zeros((1, 4, 4, 2), np.float32))
    w = T(np.zeros((3, 3, 2, 2), np.float32))
    with pytest.raises(ValueError, match="stride values must be > 0"):
        nb.conv2d(x, w, stride=(0, 1))
    with pytest.raises(ValueError, match="dilation"):
        nb.conv2d(x, w, dilation=(2, 2))
    with pytest.raises(ValueError, match="grouped mode"):
        nb.conv2d(x, w, groups=2)
    with pytest.raises(ValueError, match="padding values must be >= 0"):
        nb.conv2d(x, w, padding=-1)
    with pytest.raises(ValueError, match="Input channels"):
        nb.conv2d(x, T(np.zeros((3, 3, 3, 2), np.float32)))
    with pytest.raises(ValueError, match="Non-positive pool2d output size"):
        nb.max_pool2d(x, kernel_size=9)
    with pytest.raises(ValueError, match="Cannot broadcast"):
        T(np.zeros((2, 3), np.float32)) + T(np.zeros((4,), np.float32))


def test_context_isolation_of_flags():
    """Flags are ContextVars: a change inside a copied context does not leak."""
    import contextvars
    from nabla_amd import config

    def inner():
        config.set_flag("EAGER_MAX_GRAPH", True)
        return config.EAGER_MAX_GRAPH

    assert contextvars.copy_context().run(inner) is True
    assert config.EAGER_MAX_GRAPH is False


def test_oversized_group_is_split_locally(emulator):
    """22 results of one shared input exceed the 20 operands of a row program: the planner
    cuts that group alone and everything else keeps its fusion."""
    from nabla_amd.core import engine
    rng = np.random.default_rng(5)
    x = rng.standard_normal((6, 40)).astype(np.float32)
    X = T(x)
    ys = [X * float(i + 1) for i in range(22)]
    z = nb.reduce_sum(nb.relu(X) * 2.0, axis=1)       # an unrelated group in the same graph
    engine.clear_plan_cache()
    nb.realize_all(z, *ys)
    plans = list(engine._PLAN_CACHE.values())
    assert len(plans) == 1
    stats = plans[0].plan.stats
    assert stats.get("split_groups", 0) >= 1 and 2 <= stats["rowprog"] <= 4, stats
    for i, y in enumerate(ys):
        np.testing.assert_array_equal(y.numpy(), x * np.float32(i + 1))
    np.testing.assert_allclose(z.numpy(), (np.maximum(x, 0) * 2).sum(1), rtol=1e-6)


# ---- fused attention -------------------------------------------------------------------------------
def _attn_inputs(b, h, s, hd, seed):
    rng = np.random.default_rng(seed)
    return [rng.standard_normal((b, h, s, hd)).astype(np.float32) for _ in range(4)]


def _bf16_round(a):
    import torch
    return torch.from_numpy(a).to(torch.bfloat16).float().numpy()


@pytest.mark.parametrize("causal", [True, False])
def test_fused_attention_op_matches_oracle_composition(emulator, causal):
    """bf16 heads of size 64 take the fused op; its value and its three gradients agree with the
    oracle's composition of primitive ops (float64 on the bf16-rounded inputs)."""
    q, k, v, g = (_bf16_round(a) for a in _attn_inputs(1, 2, 128, 64, seed=5))
    tq, tk, tv, tg = (T(a, dtype=nb.DType.bfloat16) for a in (q, k, v, g))

    def loss(tq, tk, tv):
        o = F.scaled_dot_product_attention(tq, tk, tv, is_causal=causal)
        return nb.reduce_sum(nb.cast(o * tg, nb.DType.float32))

    val, grads = nb.value_and_grad(loss, argnums=(0, 1, 2))(tq, tk, tv)
    nb.realize_all(val, *grads)
    kinds = last_plan().stats
    assert kinds.get("attention") == 1 and kinds.get("attention_bwd") == 1 and "gemm" not in kinds
    vq, vk, vv = (O.V(a.astype(np.float64)) for a in (q, k, v))
    want = O.scaled_dot_product_attention(vq, vk, vv, is_causal=causal)
    wl = O.reduce_sum(want * O.V(g.astype(np.float64)))
    wg = O.grad_of(wl, [vq, vk, vv])
    assert abs(val.item() - float(wl.a)) < 2e-2 * np.abs(want.a * g).sum()
    for got, w in zip(grads, wg):
        assert relerr(got.numpy().astype(np.float64), w) < 2e-2


def test_fused_attention_reads_and_writes_heads_in_place(emulator):
    """Inside multi-head attention the fused op reads q, k, v as strided views of the projections
    and writes the context in [B, S, H, hd] order: no head transpose is materialised."""
    t = oc.c3_inputs(1, 128, 128, 256, seed=2, bf16=True)
    wl, wg = oc.c3_reference(t, num_heads=2)
    loss, grads = oc.c3_program(nb, oc.upload(nb, t, nb.DType.bfloat16), num_heads=2)
    nb.realize_all(loss, *grads.values())
    st = last_plan().stats
    assert st.get("attention") == 1 and st.get("attention_bwd") == 1
    assert st.get("copy", 0) == 0, st
    assert abs(loss.item() - wl) < 2e-2 * abs(wl)
    scale = max(np.abs(g).max() for g in wg.values())
    for k in oc.C3_PARAMS:
        got = grads[k].numpy().astype(np.float64)
        assert np.abs(got - wg[k]).max() <= 3e-2 * max(np.abs(wg[k]).max(), 1e-2 * scale), k


def test_attention_falls_back_to_primitive_ops(emulator):
    """fp32, odd head sizes, explicit masks and second-order derivatives keep the composition."""
    q, k, v, _ = _attn_inputs(1, 2, 128, 64, seed=6)
    o = F.scaled_dot_product_attention(T(q), T(k), T(v), is_causal=True)
    o.realize()
    assert "attention" not in last_plan().stats
    with nb.config.flag("FUSED_ATTENTION", False):
        o = F.scaled_dot_product_attention(*(T(a, dtype=nb.DType.bfloat16) for a in (q, k, v)))
        o.realize()
        assert "attention" not in last_plan().stats
    with pytest.raises(ValueError, match="fused_attention covers"):
        nb.ops.attention.fused_attention(T(q), T(k), T(v))


def test_fused_attention_second_order_matches_primitive_ops(emulator):
    q, k, v, g = (_bf16_round(a) for a in _attn_inputs(1, 1, 128, 64, seed=8))
    w = _bf16_round(np.random.default_rng(9).standard_normal(q.shape).astype(np.float32))

    def second(fused):
        with nb.config.flag("FUSED_ATTENTION", fused):
            tq, tk, tv, tg, tw = (T(a, dtype=nb.DType.bfloat16) for a in (q, k, v, g, w))

            def inner(tq):
                return nb.reduce_sum(nb.cast(F.scaled_dot_product_attention(tq, tk, tv, is_causal=True) * tg,
                                             nb.DType.float32))

            def outer(tq):
                return nb.reduce_sum(nb.cast(nb.grad(inner)(tq) * tw, nb.DType.float32))

            return nb.grad(outer)(tq).numpy().astype(np.float64)

    a, b = second(True), second(False)
    assert np.isfinite(a).all() and np.abs(b).max() > 0
    assert relerr(a, b) < 5e-2


def test_weight_gradient_over_a_batch_is_one_product(emulator):
    """sum_b x[b]^T dy[b] contracts over (b, s) in a single GEMM: no per-batch products, no
    reduction afterwards."""
    x = RNG.standard_normal((3, 16, 8)).astype(np.float32)
    w = RNG.standard_normal((8, 5)).astype(np.float32)
    g = RNG.standard_normal((3, 16, 5)).astype(np.float32)
    gw = nb.grad(lambda w: nb.reduce_sum(nb.matmul(T(x), w) * T(g)), create_graph=False)(T(w))
    gw.realize()
    st = last_plan().stats
    assert "reduce_mid" not in st and st["gemm"] == 1, st
    np.testing.assert_allclose(gw.numpy(), np.einsum("bsd,bsn->dn", x, g), rtol=1e-5, atol=1e-5)


# ---- avg_pool2d, silu ------------------------------------------------------------------------------
@pytest.mark.parametrize("kernel,stride,padding", [((2, 2), None, 0), ((3, 3), (2, 1), 1), ((3, 2), (1, 2), (1, 0, 2, 1))])
def test_avg_pool2d_value_grad_and_second_order(emulator, kernel, stride, padding):
    x = RNG.standard_normal((2, 9, 8, 3)).astype(np.float32)
    pad4 = (padding,) * 4 if isinstance(padding, int) else padding
    y = nb.avg_pool2d(T(x), kernel_size=kernel, stride=stride, padding=padding)
    want = O.avg_pool2d(O.V(x.astype(np.float64)), kernel, stride, pad4)
    np.testing.assert_allclose(y.numpy(), want.a, rtol=1e-6, atol=1e-6)
    assert "avgpool2d" in last_plan().stats
    g = RNG.standard_normal(want.a.shape).astype(np.float32)
    vx = O.V(x.astype(np.float64))
    (wg,) = O.grad_of(O.reduce_sum(O.avg_pool2d(vx, kernel, stride, pad4) * O.V(g.astype(np.float64))), [vx])
    f = lambda t: nb.reduce_sum(nb.avg_pool2d(t, kernel_size=kernel, stride=stride, padding=padding) * T(g))
    np.testing.assert_allclose(nb.grad(f)(T(x)).numpy(), wg, rtol=1e-5, atol=1e-6)
    # the gradient does not depend on x (the op is linear): differentiating it again gives zeros
    gg = nb.grad(lambda t: nb.reduce_sum(nb.grad(f)(t) * nb.grad(f)(t)))(T(x))
    np.testing.assert_array_equal(gg.numpy(), np.zeros_like(x))


def test_avg_pool2d_validation(emulator):
    with pytest.raises(ValueError, match="rank-4"):
        nb.avg_pool2d(T(np.zeros((4, 4), np.float32)), kernel_size=2)
    with pytest.raises(ValueError, match="dilation"):
        nb.avg_pool2d(T(np.zeros((1, 4, 4, 1), np.float32)), kernel_size=2, dilation=2)
    with pytest.raises(ValueError, match="Non-positive"):
        nb.avg_pool2d(T(np.zeros((1, 2, 2, 1), np.float32)), kernel_size=3)


def test_silu_value_and_grad(emulator):
    x = RNG.standard_normal((5, 33)).astype(np.float32)
    vx = O.V(x.astype(np.float64))
    np.testing.assert_allclose(nb.silu(T(x)).numpy(), O.silu(vx).a, rtol=1e-6, atol=1e-6)
    (wg,) = O.grad_of(O.reduce_sum(O.silu(vx)), [vx])
    np.testing.assert_allclose(nb.grad(lambda t: nb.reduce_sum(nb.silu(t)))(T(x)).numpy(), wg, rtol=1e-5, atol=1e-6)


# ---- scatter / embedding-table gradient ----------------------------------------------------------------
def test_scatter_value_rules_and_embedding_table_gradient(emulator):
    x, upd = RNG.standard_normal((7, 5)).astype(np.float32), RNG.standard_normal((4, 5)).astype(np.float32)
    idx = np.array([5, 0, 3, 5], dtype=np.int64)  # row 5 twice: the later update wins
    I = nb.Tensor.constant(idx)
    got = nb.scatter(T(x), I, T(upd))
    np.testing.assert_array_equal(got.numpy(), O.scatter(O.V(x), idx, O.V(upd)).a)
    assert last_plan().stats.get("scatter") == 1
    x3 = RNG.standard_normal((2, 6, 3)).astype(np.float32)
    u3 = RNG.standard_normal((2, 2, 3)).astype(np.float32)
    i3 = np.array([-1, 2], dtype=np.int32)
    np.testing.assert_array_equal(nb.scatter(T(x3), nb.Tensor.constant(i3), T(u3), axis=1).numpy(),
                                  O.scatter(O.V(x3), i3 % 6, O.V(u3), axis=1).a)
    # gradients of scatter
    g = RNG.standard_normal((7, 5)).astype(np.float32)
    gx, gu = nb.grad(lambda a, b: nb.reduce_sum(nb.scatter(a, I, b) * T(g)), argnums=(0, 1))(T(x), T(upd))
    vx, vu = O.V(x.astype(np.float64)), O.V(upd.astype(np.float64))
    wx, wu = O.grad_of(O.reduce_sum(O.scatter(vx, idx, vu) * O.V(g.astype(np.float64))), [vx, vu])
    np.testing.assert_allclose(gx.numpy(), wx, rtol=1e-6)
    np.testing.assert_allclose(gu.numpy(), wu, rtol=1e-6)
    # the gradient of an embedding table: the cotangent scattered into zeros
    table = RNG.standard_normal((9, 4)).astype(np.float32)
    ids = np.array([[1, 7, 2], [0, 8, 3]], dtype=np.int64)
    w = RNG.standard_normal((2, 3, 4)).astype(np.float32)
    gt = nb.grad(lambda t: nb.reduce_sum(F.embedding(nb.Tensor.constant(ids), t) * T(w)))(T(table))
    vt = O.V(table.astype(np.float64))
    (wt,) = O.grad_of(O.reduce_sum(O.gather(vt, ids) * O.V(w.astype(np.float64))), [vt])
    np.testing.assert_allclose(gt.numpy(), wt, rtol=1e-6)
    with pytest.raises(Exception, match="updates of shape"):
        nb.scatter(T(x), I, T(upd[:2])).realize()


def test_gelu_of_a_linear_layer_is_folded_into_the_product(emulator):
    """gelu(x @ W + b) in a training step: the activation and its derivative are two results of
    the product's own launch (no row program reads the pre-activation), and loss and gradients
    still agree with the float64 oracle."""
    from nabla_amd import config
    from nabla_amd.core import engine
    from oracle import ops as O
    # (the fold keeps the derivative as the product's second result: the alternative to
    # recomputing it from the pre-activation in the backward kernel)
    with config.flag("FOLD_ACTIVATION", True), config.flag("GELU_BACKWARD_FROM_INPUT", False):
        try:
            _check_gelu_fold(engine, O)
        finally:
            engine.clear_plan_cache()


def _check_gelu_fold(engine, O):
    rng = np.random.default_rng(77)
    x, w, b = rng.standard_normal((6, 40)), rng.standard_normal((40, 24)) * 0.3, rng.standard_normal((1, 24))
    w2 = rng.standard_normal((24, 5))
    T = lambda a: nb.Tensor.constant(a.astype(np.float32))

    def loss_fn(w, b, w2):
        return nb.mean(nb.gelu(T(x) @ w + b) @ w2)

    engine.clear_plan_cache()
    loss, grads = nb.value_and_grad(loss_fn, argnums=(0, 1, 2))(T(w), T(b), T(w2))
    nb.realize_all(loss, *grads)
    plan = list(engine._PLAN_CACHE.values())[-1].plan
    fused = [st for st in plan.steps if st.kind == "gemm" and st.attrs.get("act") == "gelu"]
    assert len(fused) == 1 and fused[0].attrs.get("aux_dst") is not None and fused[0].attrs.get("bias") is not None
    assert not any("gelu" in m for st in plan.steps if st.kind == "rowprog" for m in st.attrs["members"])
    vw, vb, vw2 = O.V(w), O.V(b), O.V(w2)
    want = O.mean(O.matmul(O.gelu(O.matmul(O.V(x), vw) + vb), vw2))
    wg = O.grad_of(want, [vw, vb, vw2])
    assert abs(loss.item() - float(want.a)) <= 1e-5 * abs(float(want.a))
    for g, w_ in zip(grads, wg):
        assert np.abs(g.numpy() - w_).max() <= 1e-5 * np.abs(w_).max()
    # forward only: the activation alone, one result
    engine.clear_plan_cache()
    y = nb.gelu(T(x) @ T(w) + T(b))
    np.testing.assert_allclose(y.numpy(), O.gelu(O.matmul(O.V(x), O.V(w)) + O.V(b)).a, rtol=1e-5, atol=1e-6)
    plan = list(engine._PLAN_CACHE.values())[-1].plan
    assert [st.kind for st in plan.steps] == ["gemm"] and plan.steps[0].attrs.get("aux_dst") is None


def test_integers_above_2_pow_24_are_exact(emulator):
    """Integer tensors compute in integer registers: no value passes through fp32."""
    from integer_cases import check_large_integers
    check_large_integers(nb)


def test_int64_beyond_the_int32_range_is_exact(emulator):
    """Arithmetic, comparisons, selects and casts on int64 values outside the int32 range run in
    the 64-bit integer kernel; the label-against-class-index comparison stays fused and exact."""
    from integer_cases import check_int64_beyond_int32
    check_int64_beyond_int32(nb)


def test_sum_with_a_product_folds_into_its_epilogue_when_asked(emulator):
    """``r + x @ W + b`` becomes one product that reads ``r`` and ``b`` in its epilogue under
    ``FOLD_RESIDUAL`` (off by default: the epilogue read measured slower than the sum kernel);
    the numbers are the unfused ones up to the rounding points that disappear."""
    from nabla_amd import config
    from nabla_amd.core import engine
    rng = np.random.default_rng(12)
    x, w = rng.standard_normal((6, 40, 32)).astype(np.float32), rng.standard_normal((32, 24)).astype(np.float32)
    r, b = rng.standard_normal((6, 40, 24)).astype(np.float32), rng.standard_normal((1, 24)).astype(np.float32)
    want = r + x @ w + b

    def f():
        return T(r) + T(x) @ T(w) + T(b)

    plain = f().numpy()
    with config.flag("FOLD_RESIDUAL", True):
        engine.clear_plan_cache()
        folded = f().numpy()
        kinds = [[s.kind for s in bp.plan.steps] for bp in engine._PLAN_CACHE.values()]
    engine.clear_plan_cache()
    assert ["gemm"] in kinds, kinds
    np.testing.assert_allclose(plain, want, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(folded, want, rtol=1e-5, atol=1e-5)


def test_an_adapter_update_folds_into_the_sum_with_its_base_product(emulator):
    """``x @ W + h @ B`` with a contraction of at most 16 in the second product (a low-rank
    adapter's update) is two products and no sum kernel: the thin product's epilogue reads the
    base product.  A sum with anything that is not a product keeps its row kernel."""
    from nabla_amd import config
    from nabla_amd.core import engine
    rng = np.random.default_rng(31)
    x, w = rng.standard_normal((4, 16, 32)).astype(np.float32), rng.standard_normal((32, 24)).astype(np.float32)
    h, b = rng.standard_normal((4, 16, 8)).astype(np.float32), rng.standard_normal((8, 24)).astype(np.float32)
    r = rng.standard_normal((4, 16, 24)).astype(np.float32)
    bf = nb.DType.bfloat16

    def steps_of(f):
        engine.clear_plan_cache()
        out = f().numpy()
        steps = [s for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps]
        engine.clear_plan_cache()
        return out, steps

    got, steps = steps_of(lambda: nb.cast(T(x, dtype=bf) @ T(w, dtype=bf) + T(h, dtype=bf) @ T(b, dtype=bf),
                                          nb.DType.float32))
    assert sorted(s.kind for s in steps).count("gemm") == 2
    assert sum("residual" in s.attrs for s in steps if s.kind == "gemm") == 1, \
        [s.attrs for s in steps]
    want = _bf16_round(x) @ _bf16_round(w) + _bf16_round(h) @ _bf16_round(b)
    np.testing.assert_allclose(got, want, rtol=2e-2, atol=2e-2)
    with config.flag("FOLD_THIN_RESIDUAL", False):
        off, steps_off = steps_of(lambda: nb.cast(
            T(x, dtype=bf) @ T(w, dtype=bf) + T(h, dtype=bf) @ T(b, dtype=bf), nb.DType.float32))
    assert not any("residual" in s.attrs for s in steps_off if s.kind == "gemm")
    np.testing.assert_allclose(off, want, rtol=2e-2, atol=2e-2)
    _, steps_r = steps_of(lambda: nb.cast(T(r, dtype=bf) + T(h, dtype=bf) @ T(b, dtype=bf), nb.DType.float32))
    assert not any("residual" in s.attrs for s in steps_r if s.kind == "gemm")


def test_a_bias_gradient_rides_on_the_weight_gradient_product(emulator):
    """The column sums of dy (the cotangent's reduction to the bias' shape) become a result of
    the launch that computes x^T dy, whole or split along K; the numbers are those of the
    separate reduction, and ``FOLD_COLUMN_SUMS`` switches the fold off."""
    from nabla_amd import config
    from nabla_amd.core import engine
    rng = np.random.default_rng(3)
    bf = nb.DType.bfloat16
    for (B, S, D, N), split in (((2, 64, 32, 48), False), ((4, 256, 128, 128), True)):
        x, w = rng.standard_normal((B, S, D)).astype(np.float32), rng.standard_normal((D, N)).astype(np.float32) * 0.1
        b, g = rng.standard_normal((N,)).astype(np.float32), rng.standard_normal((B, S, N)).astype(np.float32)

        def loss(p):
            return nb.reduce_sum(nb.relu(T(x, dtype=bf) @ p["w"] + p["b"]) * T(g, dtype=bf))

        got = {}
        for on in (True, False):
            with config.flag("FOLD_COLUMN_SUMS", on):
                engine.clear_plan_cache()
                val, grads = nb.value_and_grad(loss)({"w": T(w, dtype=bf), "b": T(b, dtype=bf)})
                nb.realize_all(val, grads["w"], grads["b"])
                steps = [s for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps]
                hosts = [s for s in steps if s.kind == "gemm" and s.attrs.get("colsum") is not None]
                assert len(hosts) == (1 if on else 0)
                if on:
                    assert (hosts[0].attrs["batch"] > 1) == split
                got[on] = (nb.cast(grads["b"], nb.DType.float32).numpy(), nb.cast(grads["w"], nb.DType.float32).numpy())
        engine.clear_plan_cache()
        np.testing.assert_array_equal(got[True][1], got[False][1])
        np.testing.assert_allclose(got[True][0], got[False][0], rtol=2e-2, atol=2e-2)
        dy = _bf16_round(g) * (_bf16_round(x) @ _bf16_round(w * 1.0) + _bf16_round(b) > 0)
        np.testing.assert_allclose(got[True][0], dy.reshape(-1, N).sum(0), rtol=3e-2, atol=0.3)


def test_a_constant_scale_folds_into_the_product_it_multiplies(emulator):
    """``(x @ W) * c`` with ``c`` a constant of the graph is one product with ``alpha = c`` (the
    way the low-rank adapters carry ``alpha / rank``, forward and backward); a realized scalar
    tensor is a run-time value and keeps its own multiply."""
    from nabla_amd.core import engine
    from nabla_amd.nn.finetune import lora_linear
    rng = np.random.default_rng(21)
    x, w = rng.standard_normal((5, 24, 32)).astype(np.float32), rng.standard_normal((32, 16)).astype(np.float32)
    engine.clear_plan_cache()
    got = (T(x) @ T(w)) * nb.full((), 2.5)
    got.realize()
    steps = [s for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps]
    assert [s.kind for s in steps] == ["gemm"] and steps[0].attrs["alpha"] == 2.5
    np.testing.assert_allclose(got.numpy(), (x @ w) * 2.5, rtol=1e-5, atol=1e-5)
    engine.clear_plan_cache()
    kept = (T(x) @ T(w)) * 2.5
    kept.realize()
    assert sorted(s.kind for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps) == ["gemm", "rowprog"]
    np.testing.assert_allclose(kept.numpy(), (x @ w) * 2.5, rtol=1e-5, atol=1e-5)
    # an adapter with alpha / rank = 3: value and gradients against numpy, no multiply of its own
    a, b = rng.standard_normal((32, 4)).astype(np.float32) * 0.1, rng.standard_normal((4, 16)).astype(np.float32) * 0.1

    def loss(ad):
        return nb.reduce_sum(lora_linear(T(x), T(w), ad, alpha=12.0) * T(np.ones((5, 24, 16), np.float32)))

    engine.clear_plan_cache()
    val, grads = nb.value_and_grad(loss)({"A": T(a), "B": T(b)})
    nb.realize_all(val, grads["A"], grads["B"])
    kinds = [s.kind for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps]
    alphas = sorted(s.attrs.get("alpha", 1.0) for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps
                    if s.kind == "gemm")
    engine.clear_plan_cache()
    assert alphas.count(3.0) >= 2, (kinds, alphas)
    x2 = x.reshape(-1, 32)
    np.testing.assert_allclose(val.numpy(), (x2 @ w + 3.0 * (x2 @ a) @ b).sum(), rtol=1e-4)
    np.testing.assert_allclose(grads["B"].numpy(), 3.0 * (x2 @ a).T @ np.ones((120, 16), np.float32), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(grads["A"].numpy(), 3.0 * x2.T @ (np.ones((120, 16), np.float32) @ b.T), rtol=1e-4, atol=1e-4)


def test_adapter_updates_and_gradient_sums_are_one_product(emulator):
    """`x @ W + (x @ A) @ B` and its mirror image in the backward pass are ONE product with
    several operand pairs (`nbk_gemm_desc.term`), and so is a gradient that several products
    contribute to: in a two-layer decoder the four forward updates fold onto their base products,
    and the gradient of the second layer's normalised input,
    `dq Wq^T + (dq Bq^T) Aq^T + dk Wk^T + dv Wv^T + (dv Bv^T) Av^T`, is one launch with three deep
    and two shallow pairs.  No thin product is left that reads a base result, the gradients are
    those of the plans without the folds, and a rank that is no multiple of 8 keeps the thin
    products."""
    from nabla_amd import config
    from nabla_amd.core import engine

    def step(rank):
        engine.clear_plan_cache()
        t = oc.c5_inputs(layers=2, batch=2, seq=64, d_model=128, d_ff=256, vocab=300, rank=rank, seed=3,
                         b_zero=False, bf16=True)
        loss, grads = oc.c5_program(nb, oc.upload(nb, t, dtype=nb.DType.bfloat16), num_heads=4)
        flat = [ad[k] for ad in grads for k in ("qA", "qB", "vA", "vB")]
        nb.realize_all(loss, *flat)
        gemms = [s.attrs for s in list(engine._PLAN_CACHE.values())[-1].plan.steps if s.kind == "gemm"]
        return loss.item(), [g.numpy() for g in flat], gemms

    def same(got, want):
        assert abs(got[0] - want[0]) <= 2e-2 * abs(want[0])
        for a, b in zip(got[1], want[1]):
            assert np.abs(a - b).max() <= 2e-2 * np.abs(b).max()

    on = step(16)
    gemms = on[2]
    with_terms = [a for a in gemms if a.get("terms")]
    assert sorted(len(a["terms"]) for a in with_terms) == [1, 1, 1, 1, 4]
    assert all(a["batch"] == 1 and a["M"] == 128 and a["K"] == 128 for a in with_terms)
    big = [a for a in with_terms if len(a["terms"]) == 4][0]
    assert sorted(t["K"] for t in big["terms"]) == [16, 16, 128, 128]
    assert not [a for a in gemms if a["K"] <= 16 and a["N"] > 16]      # every update found its base
    with config.flag("FOLD_PRODUCT_SUMS", False):
        pairs_only = step(16)
    assert sorted(len(a["terms"]) for a in pairs_only[2] if a.get("terms")) == [1] * 6
    assert len(pairs_only[2]) == len(gemms) + 2
    same(on, pairs_only)
    with config.flag("FOLD_THIN_PAIR", False):
        off = step(16)
    assert not [a for a in off[2] if a.get("terms")]
    assert len(off[2]) == len(gemms) + 8
    same(on, off)
    assert not [a for a in step(4)[2] if a.get("terms") and any(t["K"] < 64 for t in a["terms"])]
    engine.clear_plan_cache()


def test_relu_after_a_convolution_is_its_epilogue(emulator):
    """`relu(conv2d(x, w) + b)`: the convolution applies the relu itself (`nbk_conv_desc.act`), the
    pre-activation is not stored, and the `pre-activation > 0` masks of the backward pass read the
    result.  Values and gradients as without the fold, and against torch in float64; a
    convolution whose pre-activation something else reads keeps its relu kernel."""
    import torch
    import torch.nn.functional as TF
    from nabla_amd import config
    from nabla_amd.core import engine
    rng = np.random.default_rng(41)
    x = rng.standard_normal((2, 9, 9, 4)).astype(np.float32)
    w1 = (rng.standard_normal((3, 3, 4, 8)) * 0.3).astype(np.float32)
    b1 = (rng.standard_normal((8,)) * 0.2).astype(np.float32)
    w2 = (rng.standard_normal((3, 3, 8, 6)) * 0.3).astype(np.float32)

    def loss_fn(w1, b1, w2, x):
        h = nb.relu(nb.conv2d(x, w1, padding=1, bias=b1))
        h = nb.relu(nb.conv2d(h, w2, stride=(2, 1), padding=(1, 0, 1, 1)))
        return nb.mean(h * h)

    def step():
        engine.clear_plan_cache()
        l, gs = nb.value_and_grad(loss_fn, argnums=(0, 1, 2, 3))(T(w1), T(b1), T(w2), T(x))
        nb.realize_all(l, *gs)
        steps = [s for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps]
        return l.item(), [g.numpy() for g in gs], steps

    on = step()
    convs = [s.attrs for s in on[2] if s.kind == "conv2d"]
    assert [a["act"] for a in convs] == ["relu", "relu"]
    with config.flag("FOLD_RELU", False):
        off = step()
    assert [s.attrs["act"] for s in off[2] if s.kind == "conv2d"] == [None, None]
    assert len(on[2]) < len(off[2])
    assert on[0] == off[0]
    for a, b in zip(on[1], off[1]):
        np.testing.assert_array_equal(a, b)
    tw1, tb1, tw2, tx = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (w1, b1, w2, x)]
    h = torch.relu(TF.conv2d(tx.permute(0, 3, 1, 2), tw1.permute(3, 2, 0, 1), tb1, padding=1))
    h = torch.relu(TF.conv2d(TF.pad(h, (1, 1, 1, 0)), tw2.permute(3, 2, 0, 1), stride=(2, 1)))
    tl = (h * h).mean()
    tl.backward()
    assert abs(on[0] - tl.item()) <= 1e-5 * abs(tl.item())
    for g, t in zip(on[1], (tw1, tb1, tw2, tx)):
        assert np.abs(g - t.grad.numpy()).max() <= 1e-5 * np.abs(t.grad.numpy()).max() + 1e-8
    # the pre-activation has another reader: no fold
    engine.clear_plan_cache()
    pre = nb.conv2d(T(x), T(w1), padding=1, bias=T(b1))
    both = nb.relu(pre) + pre * 0.5
    both.realize()
    steps = [s for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps]
    assert [s.attrs["act"] for s in steps if s.kind == "conv2d"] == [None]
    ref = TF.conv2d(torch.tensor(x).double().permute(0, 3, 1, 2), torch.tensor(w1).double().permute(3, 2, 0, 1),
                    torch.tensor(b1).double(), padding=1).permute(0, 2, 3, 1)
    np.testing.assert_allclose(both.numpy(), (torch.relu(ref) + 0.5 * ref).numpy(), rtol=1e-5, atol=1e-5)
    engine.clear_plan_cache()


def test_slices_of_the_contraction_axis():
    """How the planner splits K: products with fewer than 128 tiles of 128 x 128 and a long K
    until the launch has 512 workgroups; weight gradients x^T dy (both operands row-contiguous)
    with one workgroup per CU at most in two halves; nothing else, and fp32 never."""
    from nabla_amd.backend.planner import Planner
    bf16, f32 = nb.DType.bfloat16, nb.DType.float32
    split = Planner._split_k
    assert split(1024, 1024, 8192, bf16) == 8                    # 64 tiles
    assert split(1024, 1024, 8192, bf16, rows_contiguous=True) == 8
    assert split(2048, 16, 8192, bf16) == 16                     # 16 tiles, slices of 512
    assert split(1024, 4096, 8192, bf16) == 1                    # 256 tiles: whole ...
    assert split(1024, 4096, 8192, bf16, rows_contiguous=True) == 2   # ... but x^T dy in halves
    assert split(2048, 2048, 8192, bf16, rows_contiguous=True) == 2
    assert split(1024, 4096, 2048, bf16, rows_contiguous=True) == 1   # a short K stays whole
    assert split(2048, 4096, 8192, bf16, rows_contiguous=True) == 1   # 512 tiles: two per CU anyway
    assert split(8192, 16, 2048, bf16, a_k_contiguous=True) == 1      # the tall kernel splits K itself
    assert split(1024, 1024, 8192, f32) == 1


def test_weight_gradients_of_projections_that_share_their_input_are_one_launch(emulator):
    """x^T dq, x^T dk and x^T dv (the weight gradients of the q, k and v projections of a
    transformer block, each split along K = batch x sequence) are ONE batched launch: dq, dk and
    dv lie side by side in one buffer, the batch index of the launch is (projection, slice), and
    the three bias gradients are rows of its column sums.  Gradients as without the grouping."""
    from nabla_amd import config
    from nabla_amd.core import engine

    def step():
        engine.clear_plan_cache()
        t = oc.c3_inputs(2, 1024, 128, 256, seed=5, bf16=True)
        loss, grads = oc.c3_program(nb, oc.upload(nb, t, nb.DType.bfloat16), num_heads=2)
        nb.realize_all(loss, *grads.values())
        steps = list(engine._PLAN_CACHE.values())[-1].plan.steps
        return loss.item(), {k: g.numpy().astype(np.float64) for k, g in grads.items()}, steps, t

    on = step()
    wgrads = [s.attrs for s in on[2] if s.kind == "gemm" and s.attrs["a_rs"] == 1 and s.attrs["M"] == 128 and s.attrs["N"] == 128]
    joined = [a for a in wgrads if a.get("batch_inner", 1) > 1]
    assert len(joined) == 1 and len(wgrads) == 2, [(a["batch"], a.get("batch_inner")) for a in wgrads]
    a = joined[0]
    ks = a["batch_inner"]
    assert ks > 1 and a["batch"] == 3 * ks and a["a_bs"] == 0 and a["b_bs"] == 2 * 1024 * 128
    assert a["c_bs"] == ks * 128 * 128 and a["c_bs2"] == 128 * 128 and len(a["colsum_keys"]) == 3
    assert a["colsum"].shape == (3 * ks, 128)
    bwd = [s.attrs for s in on[2] if s.kind == "attention_bwd"][0]
    assert bwd["dq"].buf == bwd["dk"].buf == bwd["dv"].buf
    assert (bwd["dq"].offset, bwd["dk"].offset, bwd["dv"].offset) == (0, 2 * 1024 * 128, 2 * 2 * 1024 * 128)
    with config.flag("GROUP_SIBLING_PRODUCTS", False):
        off = step()
    assert not [s for s in off[2] if s.kind == "gemm" and s.attrs.get("batch_inner", 1) > 1 and s.attrs["a_bs"] == 0]
    assert len([s for s in off[2] if s.kind == "gemm"]) == len([s for s in on[2] if s.kind == "gemm"]) + 2
    want_loss, want = oc.c3_reference(on[3], num_heads=2)
    assert abs(on[0] - want_loss) <= 2e-2 * abs(want_loss)
    for k in on[1]:
        np.testing.assert_array_equal(on[1][k], off[1][k], err_msg=k)   # same sums in the same order
        scale = max(np.abs(want[k]).max(), np.abs(want["bq"]).max() if k == "bk" else 0.0)
        assert np.abs(on[1][k] - want[k]).max() <= 2e-2 * scale, k
    engine.clear_plan_cache()


def test_a_batch_summed_product_keeps_what_was_folded_onto_it(emulator):
    """sum_b A[b] @ B[b] becomes one product over (b, k).  A scale folded onto the batched product
    commutes with the sum and rides along as alpha; a bias or a residual added per batch element
    does not, so those products stay batched and are summed afterwards.  Values against numpy."""
    from nabla_amd import config
    from nabla_amd.core import engine
    rng = np.random.default_rng(31)
    xt = rng.standard_normal((3, 8, 16)).astype(np.float32)   # the weight-gradient form x^T @ dy
    a = np.ascontiguousarray(np.swapaxes(xt, 1, 2))
    b = rng.standard_normal((3, 8, 5)).astype(np.float32)
    bias = rng.standard_normal((1, 5)).astype(np.float32)
    res = rng.standard_normal((3, 16, 8)).astype(np.float32)
    w2 = rng.standard_normal((8, 5)).astype(np.float32)
    prod = np.einsum("bik,bkn->bin", a, b)
    A = lambda: nb.swap_axes(T(xt), 1, 2)
    engine.clear_plan_cache()
    got = nb.reduce_sum((A() @ T(b)) * nb.full((), 0.5), axis=0)
    got.realize()
    steps = [s for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps]
    assert [s.kind for s in steps] == ["gemm"] and steps[0].attrs["alpha"] == 0.5, [s.kind for s in steps]
    np.testing.assert_allclose(got.numpy(), 0.5 * prod.sum(0), rtol=1e-5, atol=1e-5)
    engine.clear_plan_cache()
    got = nb.reduce_sum(A() @ T(b) + T(bias), axis=0)
    np.testing.assert_allclose(got.numpy(), (prod + bias).sum(0), rtol=1e-5, atol=1e-5)
    for flag in ("FOLD_RESIDUAL", "FOLD_THIN_RESIDUAL"):
        with config.flag(flag, True):
            engine.clear_plan_cache()
            got = nb.reduce_sum((T(res) @ T(w2)) + A() @ T(b), axis=0)
            np.testing.assert_allclose(got.numpy(), (res @ w2 + prod).sum(0), rtol=1e-5, atol=1e-5)
    engine.clear_plan_cache()
    # a bf16 constant is folded as stored: bf16(0.3), not 0.3
    x16 = nb.Tensor.constant(a[0], dtype=nb.DType.bfloat16)
    w16 = nb.Tensor.constant(b[0], dtype=nb.DType.bfloat16)
    (x16 @ w16 * nb.full((), 0.3, dtype=nb.DType.bfloat16)).realize()
    alphas = [s.attrs.get("alpha") for bp in engine._PLAN_CACHE.values() for s in bp.plan.steps if s.kind == "gemm"]
    engine.clear_plan_cache()
    assert alphas == [0.30078125], alphas


def test_gelu_backward_recomputes_the_derivative_where_the_cotangent_is(emulator):
    """Two ways to get gelu's derivative to the backward pass -- recomputed from the pre-activation
    where the cotangent is (the default), or stored by the forward kernel -- agree with the
    float64 oracle, second order included."""
    from nabla_amd import config
    from nabla_amd.core import engine
    from oracle import ops as O
    rng = np.random.default_rng(78)
    x = rng.standard_normal((12, 40))

    def loss_fn(t):
        return nb.reduce_sum(nb.gelu(t * 1.5) * T(np.arange(40, dtype=np.float32)))

    vx = O.V(x)
    want = O.reduce_sum(O.gelu(vx * 1.5) * O.V(np.arange(40, dtype=np.float64)))
    (wg,) = O.grad_of(want, [vx])
    for flag in (True, False):
        with config.flag("GELU_BACKWARD_FROM_INPUT", flag):
            engine.clear_plan_cache()
            loss, g = nb.value_and_grad(loss_fn)(T(x.astype(np.float32)))
            nb.realize_all(loss, g)
            np.testing.assert_allclose(g.numpy(), wg, rtol=2e-5, atol=2e-6)
    engine.clear_plan_cache()
    # second order: d/dx sum(gelu'(x)) = sum gelu''(x), gelu''(x) = phi(x) (2 - x^2)
    h = nb.grad(lambda t: nb.reduce_sum(nb.grad(lambda u: nb.reduce_sum(nb.gelu(u)))(t)))(T(x.astype(np.float32)))
    pdf = np.exp(-0.5 * x * x) / np.sqrt(2 * np.pi)
    np.testing.assert_allclose(h.numpy(), pdf * (2 - x * x), rtol=2e-4, atol=2e-5)
