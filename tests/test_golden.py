"""Committed golden vectors (tests/golden/*.npz, written by tests/golden/make_fixtures.py from
float64 torch autograd) against (1) the CPU oracle, (2) the front end on the emulator and
(3) the HIP path.  The vectors are independent of both the oracle and the package."""
import os

import numpy as np
import pytest

import nabla_amd as nb
from oracle import configs as oc
from oracle import ops as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    z = np.load(os.path.join(GOLD, name + ".npz"))
    return {k: z[k] for k in z.files}


def rel(got, want, floor=0.0):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return np.abs(got - want).max() / max(np.abs(want).max(), floor, 1e-30)


def T(a):
    return nb.Tensor.constant(a)


def c5_tree(z):
    n = int(z["layers"])
    t = {"ids": z["in_ids"], "embed": z["in_embed"], "head": z["in_head"], "lnf_w": z["in_lnf_w"],
         "lnf_b": z["in_lnf_b"], "layers": [], "lora": []}
    for li in range(n):
        t["layers"].append({k[len(f"in_L{li}_"):]: v for k, v in z.items() if k.startswith(f"in_L{li}_")})
        t["lora"].append({k[len(f"in_A{li}_"):]: v for k, v in z.items() if k.startswith(f"in_A{li}_")})
    want = [z[f"g_A{li}_{k}"] for li in range(n) for k in ("qA", "qB", "vA", "vB")]
    return t, want


# ---- (1) the oracle ---------------------------------------------------------------------------------
def test_oracle_matches_golden():
    z = load("c1_mlp")
    loss, g = oc.c1_reference(z["in_x"], z["in_W1"], z["in_b1"], z["in_W2"], z["in_b2"])
    assert abs(loss - z["loss"]) < 1e-12
    for got, k in zip(g, ("W1", "b1", "W2", "b2")):
        assert rel(got, z["g_" + k]) < 1e-10
    z = load("c2_stress")
    out, gx = oc.c2_reference(z["in_x"], z["in_y"])
    assert rel(out, z["out"]) < 1e-12 and rel(gx, z["g_x"]) < 1e-12
    z = load("c3_block")
    t = {k[3:]: v for k, v in z.items() if k.startswith("in_")}
    loss, g = oc.c3_reference(t, num_heads=int(z["heads"]))
    assert abs(loss - z["loss"]) < 1e-10 * abs(z["loss"])
    scale = max(np.abs(z["g_" + k]).max() for k in oc.C3_PARAMS)
    for k in oc.C3_PARAMS:   # bk's gradient is zero in exact arithmetic: compare on the common scale
        assert rel(g[k], z["g_" + k], floor=1e-3 * scale) < 1e-9, k
    z = load("c4_cnn")
    t = {k[3:]: v for k, v in z.items() if k.startswith("in_")}
    loss, g, am, logits = oc.c4_reference(t)
    assert abs(loss - z["loss"]) < 1e-10 * abs(z["loss"])
    assert rel(logits, z["logits"]) < 1e-10
    np.testing.assert_array_equal(am, z["argmax"])
    for k in oc.C4_PARAMS:
        assert rel(g[k], z["g_" + k]) < 1e-9, k
    z = load("c5_lora")
    t, want = c5_tree(z)
    loss, g = oc.c5_reference(t, num_heads=int(z["heads"]), alpha=float(z["alpha"]))
    assert abs(loss - z["loss"]) < 1e-10 * abs(z["loss"])
    for got, w in zip(g, want):
        assert rel(got, w) < 1e-9
    z = load("kernels")
    X, W = O.V(z["conv_x"].astype(np.float64)), O.V(z["conv_w"].astype(np.float64))
    y = O.conv2d(X, W, stride=(2, 1), padding=(1, 0, 2, 1))
    gx, gw = O.grad_of(O.reduce_sum(y * y), [X, W])
    assert rel(y.a, z["conv_y"]) < 1e-12 and rel(gx, z["conv_gx"]) < 1e-12 and rel(gw, z["conv_gw"]) < 1e-12
    P = O.V(z["pool_x"].astype(np.float64))
    py = O.max_pool2d(P, (2, 2))
    (gp,) = O.grad_of(O.reduce_sum(py * py), [P])
    assert rel(py.a, z["pool_y"]) == 0 and rel(gp, z["pool_gx"]) == 0
    np.testing.assert_array_equal(O.argmax(O.V(z["argmax_x"].astype(np.float64)), -1), z["argmax_y"])


# ---- (2) / (3) the package, on the emulator and on the device ------------------------------------------
def run_package(tol):
    z = load("c1_mlp")
    loss, grads = nb.workloads.c1_step({k[3:]: T(v) for k, v in z.items() if k.startswith("in_")})
    assert abs(loss.item() - z["loss"]) <= tol * abs(z["loss"]) + 1e-9
    for g, k in zip(grads, ("W1", "b1", "W2", "b2")):
        assert rel(g.numpy(), z["g_" + k]) < tol, k
    z = load("c2_stress")
    out, gx = nb.workloads.c2_step(T(z["in_x"]), T(z["in_y"]))
    assert rel(out.numpy(), z["out"]) < tol and rel(gx.numpy(), z["g_x"]) < tol
    z = load("c3_block")
    t = {k[3:]: T(v) for k, v in z.items() if k.startswith("in_")}
    loss, grads = nb.workloads.c3_step(t, int(z["heads"]))
    assert abs(loss.item() - z["loss"]) < tol * abs(z["loss"])
    for k in oc.C3_PARAMS:
        # the key bias has no gradient (softmax ignores a shift of all its scores: the true value
        # is zero and what comes back is the rounding of sums that cancel), so it is measured on
        # the scale of the query bias's gradient, which is the same sum without the cancellation
        floor = np.abs(z["g_bq"]).max() if k == "bk" else 0.0
        assert rel(grads[k].numpy(), z["g_" + k], floor=floor) < tol, k
    z = load("c4_cnn")
    t = {k[3:]: T(v) for k, v in z.items() if k.startswith("in_")}
    loss, grads = nb.workloads.c4_step(t)
    logits = nb.workloads.c4_logits({k: t[k] for k in oc.C4_PARAMS}, t["img"])
    assert abs(loss.item() - z["loss"]) < tol * abs(z["loss"])
    assert rel(logits.numpy(), z["logits"]) < tol
    np.testing.assert_array_equal(nb.argmax(logits, axis=-1).numpy(), z["argmax"])
    for k in oc.C4_PARAMS:
        assert rel(grads[k].numpy(), z["g_" + k]) < tol, k
    z = load("c5_lora")
    tree, want = c5_tree(z)
    loss, grads = nb.workloads.c5_step(oc.upload(nb, tree), int(z["heads"]), float(z["alpha"]))
    flat = [ad[k] for ad in grads for k in ("qA", "qB", "vA", "vB")]
    assert abs(loss.item() - z["loss"]) < tol * abs(z["loss"])
    for g, w in zip(flat, want):
        assert rel(g.numpy(), w) < tol
    z = load("kernels")
    x, w = T(z["conv_x"]), T(z["conv_w"])
    kw = dict(stride=(2, 1), padding=(1, 0, 2, 1))
    y = nb.conv2d(x, w, **kw)
    gx, gw = nb.grad(lambda a, b: nb.reduce_sum(nb.conv2d(a, b, **kw) ** 2), argnums=(0, 1))(x, w)
    assert rel(y.numpy(), z["conv_y"]) < tol and rel(gx.numpy(), z["conv_gx"]) < tol
    assert rel(gw.numpy(), z["conv_gw"]) < tol
    p = T(z["pool_x"])
    py = nb.max_pool2d(p, kernel_size=(2, 2))
    gp = nb.grad(lambda a: nb.reduce_sum(nb.max_pool2d(a, kernel_size=(2, 2)) ** 2))(p)
    np.testing.assert_array_equal(py.numpy(), z["pool_y"])
    # the routing is exact (which element of each window receives the gradient); the value
    # 2 * y goes through the device's pow, which is not correctly rounded
    np.testing.assert_array_equal(gp.numpy() != 0, z["pool_gx"] != 0)
    assert rel(gp.numpy(), z["pool_gx"]) < tol
    np.testing.assert_array_equal(nb.argmax(T(z["argmax_x"]), axis=-1).numpy(), z["argmax_y"])
    np.testing.assert_array_equal(nb.gather(T(z["gather_table"]), T(z["gather_idx"]), axis=0).numpy(),
                                  z["gather_y"])
    s = T(z["sm_x"])
    assert rel(nb.softmax(s, axis=-1).numpy(), z["sm_y"]) < tol
    assert rel(nb.logsoftmax(s, axis=-1).numpy(), z["lsm_y"]) < tol
    ramp = T(np.arange(10, dtype=np.float32))
    gs = nb.grad(lambda a: nb.reduce_sum(nb.softmax(a, axis=-1) * ramp))(s)
    assert rel(gs.numpy(), z["sm_gx"]) < tol
    lw, lb, r10 = T(z["ln_w"]), T(z["ln_b"]), T((np.arange(10) / 10.0).astype(np.float32))
    F = nb.nn.functional
    assert rel(F.layer_norm(s, lw, lb).numpy(), z["ln_y"]) < tol
    g3 = nb.grad(lambda a, b, c: nb.reduce_sum(F.layer_norm(a, b, c) ** 2 * r10), argnums=(0, 1, 2))(s, lw, lb)
    for g, k in zip(g3, ("ln_gx", "ln_gw", "ln_gb")):
        assert rel(g.numpy(), z[k]) < tol, k


def test_frontend_on_emulator_matches_golden(emulator):
    run_package(1e-5)


@pytest.mark.gpu
def test_hip_matches_golden(hip):
    run_package(1e-5)


# ---- bf16 causal attention (the fused kernels' shape class) -------------------------------------------
def _attention_fixture():
    import torch
    z = load("attention_bf16")
    ins = {n: torch.from_numpy(z[f"in_{n}_bf16_bits"].view(np.int16)).view(torch.bfloat16) for n in "qkvg"}
    return z, ins


def test_oracle_attention_matches_golden():
    z, ins = _attention_fixture()
    q, k, v = (O.V(ins[n].double().numpy()) for n in "qkv")
    o = O.scaled_dot_product_attention(q, k, v, is_causal=True)
    dq, dk, dv = O.grad_of(O.reduce_sum(o * O.V(ins["g"].double().numpy())), [q, k, v])
    # the vectors are stored as float16: 2^-11 relative
    for got, name in ((o.a, "o"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert rel(got, z[name]) < 1e-3, name


def _package_attention(tol):
    z, ins = _attention_fixture()
    bf = nb.DType.bfloat16
    q, k, v, g = (nb.Tensor.from_dlpack(ins[n]) for n in "qkvg")
    assert q.dtype is bf

    def loss(q, k, v):
        o = nb.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
        return nb.reduce_sum(nb.cast(o * g, nb.DType.float32))

    o = nb.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    grads = nb.grad(loss, argnums=(0, 1, 2))(q, k, v)
    from nabla_amd.core.engine import _PLAN_CACHE
    nb.realize_all(o, *grads)
    assert any("attention_bwd" in b.plan.stats for b in _PLAN_CACHE.values())
    f32 = lambda t: nb.cast(t, nb.DType.float32).numpy()
    assert rel(f32(o), z["o"]) < tol
    for got, name in zip(grads, ("dq", "dk", "dv")):
        assert rel(f32(got), z[name]) < tol, name


def test_frontend_attention_on_emulator_matches_golden(emulator):
    _package_attention(2e-2)


@pytest.mark.gpu
def test_hip_attention_matches_golden(hip):
    _package_attention(2e-2)
