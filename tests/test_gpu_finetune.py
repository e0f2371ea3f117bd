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
