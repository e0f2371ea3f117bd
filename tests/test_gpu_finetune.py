"""QLoRA on the device: the NF4 dequantisation (uint8 -> int32 cast, 16-entry gather, block
scale) is exact against the oracle, qlora_linear agrees with the formula, a short training
loop reduces the loss, and a checkpoint written from device tensors reads back bit for bit."""
import numpy as np
import pytest

import nabla_amd as nb
from oracle import ops as O

pytestmark = pytest.mark.gpu
ft = nb.nn.finetune


def T(a, dtype=None):
    return nb.Tensor.constant(a, dtype=dtype)


@pytest.mark.parametrize("shape,block", [((16, 16), 8), ((13, 10), 64), ((2048, 512), 64), ((300, 7), 4)])
def test_dequantize_nf4_is_exact(hip, shape, block):
    w = np.random.default_rng(82).standard_normal(shape).astype(np.float32)
    qw = ft.quantize_nf4(T(w), block_size=block)
    want = O.nf4_quantize(w, block)
    np.testing.assert_array_equal(qw["indices"].to_numpy(), want["indices"])
    np.testing.assert_array_equal(qw["scales"].to_numpy(), want["scales"])
    np.testing.assert_array_equal(ft.dequantize_nf4(qw).to_numpy(), O.nf4_dequantize(want))
    got16 = ft.dequantize_nf4(qw, dtype=nb.DType.bfloat16)
    assert got16.dtype is nb.DType.bfloat16
    ref = O.nf4_dequantize(want)
    np.testing.assert_allclose(got16.cast(nb.DType.float32).to_numpy(), ref, rtol=2 ** -6, atol=1e-6)


@pytest.mark.parametrize("low_rank", [True, False])
def test_qlora_linear_and_training(hip, low_rank):
    rng = np.random.default_rng(2027)
    n, din, dout = 64, 12, 7
    x = rng.standard_normal((n, din)).astype(np.float32)
    w = rng.standard_normal((din, dout)).astype(np.float32)
    u, v = rng.standard_normal((din, 2)).astype(np.float32), rng.standard_normal((2, dout)).astype(np.float32)
    y = (x @ (w + 0.2 * (u @ v))).astype(np.float32)
    with nb.config.flag("LORA_LOW_RANK_ORDER", low_rank):
        qw = ft.quantize_nf4(T(w), block_size=8)
        adapter = ft.init_lora_adapter(T(w), rank=3, init_std=0.01)
        wd = O.nf4_dequantize(O.nf4_quantize(w, 8)).astype(np.float64)
        A, B = adapter["A"].to_numpy().astype(np.float64), adapter["B"].to_numpy().astype(np.float64)
        want = x @ wd + x @ ((A @ B) * (8.0 / 3))
        got = ft.qlora_linear(T(x), qw, adapter, alpha=8.0)
        np.testing.assert_allclose(got.to_numpy(), want, rtol=1e-5, atol=1e-5)
        opt = nb.nn.optim.adamw_init(adapter)

        def loss_fn(p):
            err = ft.qlora_linear(T(x), qw, p, alpha=8.0) - T(y)
            return nb.mean(err * err)

        initial = float(loss_fn(adapter).to_numpy())
        for _ in range(12):
            _, grads = nb.value_and_grad(loss_fn, realize=False)(adapter)
            adapter, opt = nb.nn.optim.adamw_update(adapter, grads, opt, lr=2e-2, weight_decay=0.0)
        assert float(loss_fn(adapter).to_numpy()) < initial


def test_checkpoint_roundtrip_from_device_tensors(hip, tmp_path):
    rng = np.random.default_rng(90)
    w = T(rng.standard_normal((10, 6)).astype(np.float32))
    adapter = ft.init_lora_adapter(w, rank=3, init_std=0.01)
    opt = nb.nn.optim.adamw_init(adapter)
    grads = {"A": T(rng.standard_normal((10, 3)).astype(np.float32)),
             "B": T(rng.standard_normal((3, 6)).astype(np.float32))}
    adapter, opt = nb.nn.optim.adamw_update(adapter, grads, opt, lr=1e-2)
    ft.save_finetune_checkpoint(tmp_path / "c", lora_params=adapter, optimizer_state=opt)
    template = ft.init_lora_adapter(w, rank=3)
    lora, lopt, meta = ft.load_finetune_checkpoint(tmp_path / "c", lora_template=template,
                                                   optimizer_template=nb.nn.optim.adamw_init(template))
    assert meta["has_optimizer"] and lopt["step"] == opt["step"]
    for k in ("A", "B"):
        np.testing.assert_array_equal(lora[k].to_numpy(), adapter[k].to_numpy())
        np.testing.assert_array_equal(lopt["m"][k].to_numpy(), opt["m"][k].to_numpy())


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("M,rows,cols,block", [(300, 256, 136, 8), (1024, 512, 512, 64), (65, 72, 40, 8)])
def test_gemm_on_nf4_codes_through_the_c_abi(hip, dtype, transpose, M, rows, cols, block):
    """nbk_gemm_nf4 against float64 x @ W (and x @ W^T) with W = level[code] * block scale from the
    oracle's dequantisation (rounded to bf16 once for the bf16 kernel, as the kernel does)."""
    import ctypes as C
    import torch
    from nabla_amd.backend import lib
    rng = np.random.default_rng(91)
    w = rng.standard_normal((rows, cols)).astype(np.float32)
    q = O.nf4_quantize(w, block)
    wd = torch.tensor(O.nf4_dequantize(q))
    K, N = (cols, rows) if transpose else (rows, cols)
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    x = torch.tensor(rng.standard_normal((M, K)).astype(np.float32) * 0.5).to(tdt)
    wk = wd.to(tdt).double()
    want = x.double() @ (wk.t() if transpose else wk)
    codes = torch.tensor(q["indices"]).cuda()
    scales = torch.tensor(q["scales"]).cuda()
    xd = x.cuda()
    out = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
    L = lib.load()
    d = lib.GemmNf4Desc()
    d.A, d.codes, d.scales, d.C = xd.data_ptr(), codes.data_ptr(), scales.data_ptr(), out.data_ptr()
    d.M, d.w_rows, d.w_cols, d.lda, d.ldc = M, rows, cols, K, N
    d.block, d.transpose_w, d.dtype, d.alpha = block, int(transpose), (1 if dtype == "bf16" else 0), 1.0
    print(f"gemm_nf4 M{M} W{rows}x{cols} block{block} {dtype} transpose={transpose}", flush=True)
    lib.check(L.nbk_gemm_nf4(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    rtol, atol = (2.0 ** -8, 2e-2) if dtype == "bf16" else (1e-5, 1e-5 * np.sqrt(K))
    err = (out.double().cpu() - want).abs() - rtol * want.abs()
    assert err.max().item() <= atol, err.max().item()
    d.block = 12
    with pytest.raises(ValueError, match="multiples of 8"):
        lib.check(L.nbk_gemm_nf4(C.byref(d), None))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_qlora_linear_on_the_codes_and_its_gradients(hip, dtype):
    """qlora_linear with a weight the fused product covers: one gemm_nf4 launch forward, the
    transposed one for the activations' gradient, values and gradients against the oracle."""
    from nabla_amd.core import engine
    rng = np.random.default_rng(2033)
    x = rng.standard_normal((4, 96, 256)).astype(np.float32) * 0.5
    w = rng.standard_normal((256, 128)).astype(np.float32) * 0.1
    dt = nb.DType.float32 if dtype == "f32" else nb.DType.bfloat16
    if dtype == "bf16":
        from oracle import configs as oc
        x = oc.to_bf16_grid(x)
    qw = ft.quantize_nf4(T(w), block_size=64)
    adapter = {"A": T(rng.standard_normal((256, 8)).astype(np.float32) * 0.05, dtype=dt),
               "B": T(rng.standard_normal((8, 128)).astype(np.float32) * 0.05, dtype=dt)}
    wd = O.nf4_dequantize(O.nf4_quantize(w, 64)).astype(np.float64)
    A, B = (adapter[k].to(nb.DType.float32).to_numpy().astype(np.float64) for k in "AB")

    def f(xt, p):
        return nb.reduce_sum(nb.cast(ft.qlora_linear(xt, qw, p, alpha=4.0, compute_dtype=dt), nb.DType.float32) ** 2)

    engine.clear_plan_cache()
    gx, gp = nb.grad(f, argnums=(0, 1))(T(x, dtype=dt), adapter)
    nb.realize_all(gx, gp["A"], gp["B"])
    steps = list(engine._PLAN_CACHE.values())[-1].plan.steps
    assert sorted(st.attrs["transpose"] for st in steps if st.kind == "gemm_nf4") == [False, True]
    vx, vA, vB = O.V(x.astype(np.float64)), O.V(A), O.V(B)
    out = O.matmul(vx, O.V(wd)) + O.matmul(vx, O.matmul(vA, vB) * 0.5)
    want = O.grad_of(O.reduce_sum(out * out), [vx, vA, vB])
    tol = 1e-5 if dtype == "f32" else 2e-2
    for g, wnt in zip((gx, gp["A"], gp["B"]), want):
        g = g.to(nb.DType.float32).to_numpy().astype(np.float64)
        assert np.abs(g - wnt).max() <= tol * np.abs(wnt).max()
