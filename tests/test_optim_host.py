"""Optimizers (nn/optim) on the emulator-backed host path, against torch.optim on the same
seeded inputs (fp64 in torch, fp32 here) and closed forms."""
import numpy as np
import pytest
import torch

import nabla_amd as nb
from nabla_amd.nn import optim


def T(a):
    return nb.Tensor.constant(np.asarray(a, dtype=np.float32))


def _params(rng):
    return {"w": rng.standard_normal((5, 7)).astype(np.float32),
            "b": rng.standard_normal((7,)).astype(np.float32),
            "nested": [rng.standard_normal((3,)).astype(np.float32)]}


def _torch_params(p):
    return [torch.tensor(p["w"], dtype=torch.float64, requires_grad=True),
            torch.tensor(p["b"], dtype=torch.float64, requires_grad=True),
            torch.tensor(p["nested"][0], dtype=torch.float64, requires_grad=True)]


def _flat(tree):
    return [tree["w"], tree["b"], tree["nested"][0]]


@pytest.mark.parametrize("momentum,wd", [(0.0, 0.0), (0.9, 0.0), (0.9, 0.01), (0.0, 0.1)])
def test_sgd_matches_torch(emulator, momentum, wd):
    rng = np.random.default_rng(0)
    p0 = _params(rng)
    tp = _torch_params(p0)
    topt = torch.optim.SGD(tp, lr=0.05, momentum=momentum, weight_decay=wd)
    opt = optim.SGD(nb.tree_map(T, p0), lr=0.05, momentum=momentum, weight_decay=wd)
    state = None
    fparams = nb.tree_map(T, p0)
    for step in range(4):
        g = nb.tree_map(lambda a: (rng.standard_normal(a.shape) * 0.3).astype(np.float32), p0)
        for t, gi in zip(tp, _flat(g)):
            t.grad = torch.tensor(gi, dtype=torch.float64)
        topt.step()
        new = opt.step(nb.tree_map(T, g))
        fparams, state = optim.sgd_update(fparams, nb.tree_map(T, g), state, lr=0.05,
                                          momentum=momentum, weight_decay=wd)
        for got, fgot, want in zip(_flat(new), _flat(fparams), tp):
            np.testing.assert_allclose(got.numpy(), want.detach().numpy(), rtol=2e-5, atol=1e-6)
            np.testing.assert_allclose(fgot.numpy(), want.detach().numpy(), rtol=2e-5, atol=1e-6)
    assert state["step"] == 4 and opt.step_count == 4


@pytest.mark.parametrize("wd", [0.0, 0.05])
def test_adamw_matches_torch(emulator, wd):
    rng = np.random.default_rng(1)
    p0 = _params(rng)
    tp = _torch_params(p0)
    topt = torch.optim.AdamW(tp, lr=1e-2, betas=(0.9, 0.99), eps=1e-8, weight_decay=wd)
    opt = optim.AdamW(nb.tree_map(T, p0), lr=1e-2, betas=(0.9, 0.99), eps=1e-8, weight_decay=wd)
    fparams, fstate = nb.tree_map(T, p0), optim.adamw_init(nb.tree_map(T, p0))
    for step in range(5):
        g = nb.tree_map(lambda a: (rng.standard_normal(a.shape) * 0.3).astype(np.float32), p0)
        for t, gi in zip(tp, _flat(g)):
            t.grad = torch.tensor(gi, dtype=torch.float64)
        topt.step()
        new = opt.step(nb.tree_map(T, g))
        fparams, fstate = optim.adamw_update(fparams, nb.tree_map(T, g), fstate, lr=1e-2,
                                             beta1=0.9, beta2=0.99, eps=1e-8, weight_decay=wd)
        for got, fgot, want in zip(_flat(new), _flat(fparams), tp):
            np.testing.assert_allclose(got.numpy(), want.detach().numpy(), rtol=1e-4, atol=2e-6)
            np.testing.assert_allclose(fgot.numpy(), want.detach().numpy(), rtol=1e-4, atol=2e-6)
    assert fstate["step"] == 5
    # moments are plain exponential averages
    assert all(t.real for t in _flat(opt.m)) and all(t.real for t in _flat(opt.v))


def test_adamw_step_with_tensor_counter_and_one_kernel_per_parameter(emulator):
    """Inside compile the step counter is a 0-d tensor; the bias correction then goes through
    exp(step * log(beta)) and must agree with the integer form.  The whole update of one
    parameter is at most two row programs (no other kernels)."""
    from nabla_amd.core import engine
    rng = np.random.default_rng(2)
    p, g = rng.standard_normal((6, 9)).astype(np.float32), rng.standard_normal((6, 9)).astype(np.float32)
    m, v = np.abs(rng.standard_normal((6, 9))).astype(np.float32) * 0.1, np.abs(rng.standard_normal((6, 9))).astype(np.float32) * 0.01
    engine.clear_plan_cache()
    a = optim.adamw_step(T(p), T(g), T(m), T(v), 3, lr=1e-2, weight_decay=0.01)
    nb.realize_all(*a)
    stats = [bp.plan.stats for bp in engine._PLAN_CACHE.values()]
    # nine scalar hyper-parameters travel as 0-d operands; with param, grad and both moments
    # that is more than one group may read, so the update is two programs, not one
    assert len(stats) == 1 and stats[0]["rowprog"] <= 2 and stats[0]["steps"] == stats[0]["rowprog"], stats
    engine.clear_plan_cache()
    b = optim.adamw_step(T(p), T(g), T(m), T(v), T(np.float32(3.0)), lr=1e-2, weight_decay=0.01)
    nb.realize_all(*b)
    stats = [bp.plan.stats for bp in engine._PLAN_CACHE.values()]
    # the two scalar bias corrections are tiny programs of their own
    assert len(stats) == 1 and stats[0]["rowprog"] <= 4 and stats[0]["steps"] == stats[0]["rowprog"], stats
    for x, y in zip(a, b):
        np.testing.assert_allclose(x.numpy(), y.numpy(), rtol=2e-5, atol=1e-7)
    # closed form of the first moments
    np.testing.assert_allclose(a[1].numpy(), 0.9 * m + 0.1 * g, rtol=1e-6)
    np.testing.assert_allclose(a[2].numpy(), 0.999 * v + 0.001 * g * g, rtol=1e-6, atol=1e-9)


def test_train_loop_with_backward_and_grad_attributes(emulator):
    """PyTorch-style: loss.backward() fills .grad, optimizer.step() with no arguments uses it,
    returned parameters are fresh leaves that still require grad."""
    rng = np.random.default_rng(3)
    x = T(rng.standard_normal((16, 4)))
    y = T(rng.standard_normal((16, 1)))
    w = T(rng.standard_normal((4, 1)) * 0.1)
    w.requires_grad_(True)
    opt = optim.SGD({"w": w}, lr=0.1)
    losses = []
    for _ in range(5):
        w = opt.params["w"]
        loss = nb.mean((x @ w - y) ** 2)
        loss.backward()
        losses.append(loss.item())
        opt.step()
        assert opt.params["w"].requires_grad and opt.params["w"].real
    assert losses[-1] < losses[0]


def test_execution_policy_flags(emulator):
    before = optim.Optimizer.get_execution_policy()
    try:
        optim.Optimizer.set_execution_policy(auto_realize_updated_params=False,
                                             auto_realize_updated_state=False)
        opt = optim.AdamW({"w": T(np.ones((2, 2)))}, lr=0.1)
        new = opt.step({"w": T(np.ones((2, 2)))})
        assert not new["w"].real and not opt.m["w"].real
        np.testing.assert_allclose(new["w"].numpy(), 1.0 - 0.1, rtol=1e-5)
    finally:
        optim.Optimizer.set_execution_policy(**before)


def test_a_pytree_step_is_one_launch_and_one_plan_for_every_step(emulator):
    """All leaves of one dtype go to one update launch; the AdamW counter travels as data, so the
    second step of the stateful optimizer finds the first step's plan."""
    from nabla_amd.core import engine
    rng = np.random.default_rng(5)
    p0 = _params(rng)
    opt = optim.AdamW(nb.tree_map(T, p0), lr=1e-2, weight_decay=0.01)
    opt.step(nb.tree_map(lambda a: T(rng.standard_normal(a.shape)), p0))  # (the zero moments are made here)
    engine.clear_plan_cache()
    for _ in range(3):
        opt.step(nb.tree_map(lambda a: T(rng.standard_normal(a.shape)), p0))
    plans = [bp.plan for bp in engine._PLAN_CACHE.values()]
    assert len(plans) == 1, [p.stats for p in plans]
    assert [s.kind for s in plans[0].steps] == ["adamw_multi"]
    assert len(plans[0].steps[0].attrs["entries"]) == 3

    sgd = optim.SGD(nb.tree_map(T, p0), lr=0.1, momentum=0.9)
    sgd.step(nb.tree_map(lambda a: T(rng.standard_normal(a.shape)), p0))
    engine.clear_plan_cache()
    for _ in range(2):
        sgd.step(nb.tree_map(lambda a: T(rng.standard_normal(a.shape)), p0))
    plans = [bp.plan for bp in engine._PLAN_CACHE.values()]
    assert len(plans) == 1 and [s.kind for s in plans[0].steps] == ["sgd_multi"]


def test_list_update_falls_back_per_leaf_and_matches_the_per_leaf_arithmetic(emulator):
    """Leaves the list kernel does not take (a gradient of another dtype) go through the per-leaf
    arithmetic in the same call; with the flag off everything does, and the numbers agree."""
    from nabla_amd import config
    rng = np.random.default_rng(6)
    p0 = _params(rng)
    g0 = nb.tree_map(lambda a: rng.standard_normal(a.shape).astype(np.float32), p0)

    def run():
        params, grads = nb.tree_map(T, p0), nb.tree_map(T, g0)
        grads["b"] = grads["b"].to(nb.DType.bfloat16)  # mismatched: per-leaf path
        state = optim.adamw_init(params)
        for _ in range(2):
            params, state = optim.adamw_update(params, grads, state, lr=1e-2, weight_decay=0.1)
        return [t.numpy() for t in _flat(params)] + [t.numpy() for t in _flat(state["v"])]

    fused = run()
    with config.flag("MULTI_TENSOR_OPTIMIZER", False):
        plain = run()
    for a, b in zip(fused, plain):
        np.testing.assert_allclose(a, b, rtol=2e-6, atol=1e-8)


def test_gradient_through_an_optimizer_step(emulator):
    """d/dp of sum(step(p)) through the list op equals that of the per-leaf arithmetic: for SGD
    with decay, 1 - lr * wd per element."""
    p = T(np.linspace(-1, 1, 12).reshape(3, 4))
    g = T(np.full((3, 4), 0.25))

    def f(p):
        new, _ = optim.sgd_update({"w": p}, {"w": g}, None, lr=0.1, weight_decay=0.5)
        return nb.reduce_sum(new["w"])

    dp = nb.grad(f)(p)
    np.testing.assert_allclose(dp.numpy(), np.full((3, 4), 1.0 - 0.1 * 0.5), rtol=1e-6)
