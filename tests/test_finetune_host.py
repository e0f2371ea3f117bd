"""QLoRA (NF4) and fine-tuning checkpoints on the host path: the cases of the reference's
tests/unit/nn/test_finetune_qlora.py and test_finetune_checkpoint.py, plus equality with the
oracle's restatement (indices and scales bit for bit, dequantised values exactly)."""
import json

import numpy as np
import pytest

import nabla_amd as nb
from oracle import ops as O

ft = nb.nn.finetune


def T(a, dtype=None):
    return nb.Tensor.constant(a, dtype=dtype)


@pytest.mark.parametrize("shape,block", [((8, 6), 8), ((12, 8), 8), ((16, 16), 8), ((13, 10), 64), ((5, 7), 4)])
def test_quantize_matches_oracle_bit_for_bit(emulator, shape, block):
    w = np.random.default_rng(80).standard_normal(shape).astype(np.float32)
    qw = ft.quantize_nf4(T(w), block_size=block)
    want = O.nf4_quantize(w, block)
    assert set(qw) == {"indices", "scales", "original_shape", "original_numel", "padded_numel", "block_size"}
    assert qw["original_shape"] == shape and qw["original_numel"] == w.size
    assert qw["padded_numel"] == want["padded"] and qw["block_size"] == block
    assert qw["indices"].dtype is nb.DType.uint8
    np.testing.assert_array_equal(qw["indices"].to_numpy(), want["indices"])
    np.testing.assert_array_equal(qw["scales"].to_numpy(), want["scales"])
    deq = ft.dequantize_nf4(qw)
    assert deq.shape == shape
    np.testing.assert_array_equal(deq.to_numpy(), O.nf4_dequantize(want))
    rel = np.abs(deq.to_numpy() - w).mean() / (np.abs(w).mean() + 1e-8)
    assert rel < 0.3


def test_quantize_validation(emulator):
    with pytest.raises(ValueError, match="2D weight"):
        ft.quantize_nf4(T(np.zeros((2, 3, 4), np.float32)))
    with pytest.raises(ValueError, match="block_size"):
        ft.quantize_nf4(T(np.zeros((2, 3), np.float32)), block_size=0)


def test_uint8_is_input_only(emulator):
    idx = nb.Tensor.from_dlpack(np.arange(6, dtype=np.uint8))
    assert idx.dtype is nb.DType.uint8
    np.testing.assert_array_equal(nb.cast(idx, nb.DType.int32).to_numpy(), np.arange(6, dtype=np.int32))
    with pytest.raises(Exception, match="uint8"):
        (idx + idx).realize()


@pytest.mark.parametrize("low_rank", [True, False])
def test_qlora_linear_forward_and_training(emulator, low_rank):
    rng = np.random.default_rng(2027)
    n, din, dout = 64, 12, 7
    x = rng.standard_normal((n, din)).astype(np.float32)
    w = rng.standard_normal((din, dout)).astype(np.float32)
    u, v = rng.standard_normal((din, 2)).astype(np.float32), rng.standard_normal((2, dout)).astype(np.float32)
    y = (x @ (w + 0.2 * (u @ v))).astype(np.float32)
    with nb.config.flag("LORA_LOW_RANK_ORDER", low_rank):
        qw = ft.quantize_nf4(T(w), block_size=8)
        adapter = ft.init_lora_adapter(T(w), rank=3, init_std=0.01)
        y1 = ft.qlora_linear(T(x), qw, adapter, alpha=8.0)
        y2 = ft.qlora_linear(T(x), qw, adapter, alpha=8.0)
        nb.testing.assert_allclose(y1, y2, rtol=1e-6, atol=1e-6)
        # against the formula on the oracle's dequantised weight
        wd = O.nf4_dequantize(O.nf4_quantize(w, 8)).astype(np.float64)
        A, B = adapter["A"].to_numpy().astype(np.float64), adapter["B"].to_numpy().astype(np.float64)
        want = x @ wd + x @ ((A @ B) * (8.0 / 3))
        np.testing.assert_allclose(y1.to_numpy(), want, rtol=2e-5, atol=2e-5)

        opt = nb.nn.optim.adamw_init(adapter)

        def loss_fn(p):
            err = ft.qlora_linear(T(x), qw, p, alpha=8.0) - T(y)
            return nb.mean(err * err)

        initial = float(loss_fn(adapter).to_numpy())
        for _ in range(12):
            _, grads = nb.value_and_grad(loss_fn, realize=False)(adapter)
            adapter, opt = nb.nn.optim.adamw_update(adapter, grads, opt, lr=2e-2, weight_decay=0.0)
        assert float(loss_fn(adapter).to_numpy()) < initial


def _adapter_and_state(seed):
    rng = np.random.default_rng(seed)
    w = T(rng.standard_normal((10, 6)).astype(np.float32))
    adapter = ft.init_lora_adapter(w, rank=3, init_std=0.01)
    opt = nb.nn.optim.adamw_init(adapter)
    grads = {"A": T(rng.standard_normal((10, 3)).astype(np.float32)),
             "B": T(rng.standard_normal((3, 6)).astype(np.float32))}
    adapter, opt = nb.nn.optim.adamw_update(adapter, grads, opt, lr=1e-2)
    return w, adapter, opt


def test_checkpoint_roundtrip_and_on_disk_format(emulator, tmp_path):
    w, adapter, opt = _adapter_and_state(90)
    ckpt = tmp_path / "ckpt"
    ft.save_finetune_checkpoint(ckpt, lora_params=adapter, optimizer_state=opt, metadata={"tag": "test"})
    # the format: key scheme of tensors.npz and the fields of meta.json
    with np.load(ckpt / "tensors.npz", allow_pickle=False) as z:
        assert sorted(z.files) == ["lora.A", "lora.B", "opt_m.A", "opt_m.B", "opt_v.A", "opt_v.B"]
        np.testing.assert_array_equal(z["lora.A"], adapter["A"].to_numpy())
        np.testing.assert_array_equal(z["opt_v.B"], opt["v"]["B"].to_numpy())
    meta = json.loads((ckpt / "meta.json").read_text())
    assert meta == {"step": int(opt["step"]), "has_optimizer": True, "user_metadata": {"tag": "test"},
                    "tensor_keys": ["lora.A", "lora.B", "opt_m.A", "opt_m.B", "opt_v.A", "opt_v.B"]}
    template = ft.init_lora_adapter(w, rank=3, init_std=0.01)
    lora, lopt, lmeta = ft.load_finetune_checkpoint(ckpt, lora_template=template,
                                                    optimizer_template=nb.nn.optim.adamw_init(template))
    for k in ("A", "B"):
        np.testing.assert_array_equal(lora[k].to_numpy(), adapter[k].to_numpy())
        np.testing.assert_array_equal(lopt["m"][k].to_numpy(), opt["m"][k].to_numpy())
        np.testing.assert_array_equal(lopt["v"][k].to_numpy(), opt["v"][k].to_numpy())
    assert lopt["step"] == opt["step"] and lmeta["user_metadata"]["tag"] == "test"


def test_checkpoint_nested_trees_without_optimizer_and_errors(emulator, tmp_path):
    rng = np.random.default_rng(91)
    tree = [{"qA": T(rng.standard_normal((4, 2)).astype(np.float32)),
             "vB": T(rng.standard_normal((2, 4)).astype(np.float32), dtype=nb.DType.bfloat16)},
            {"qA": T(rng.standard_normal((4, 2)).astype(np.float32)),
             "vB": T(rng.standard_normal((2, 4)).astype(np.float32), dtype=nb.DType.bfloat16)}]
    ckpt = tmp_path / "nested"
    ft.save_finetune_checkpoint(ckpt, lora_params=tree, metadata={"epoch": 1})
    with np.load(ckpt / "tensors.npz", allow_pickle=False) as z:
        assert sorted(z.files) == ["lora[0].qA", "lora[0].vB", "lora[1].qA", "lora[1].vB"]
    template = [{k: nb.zeros_like(v) for k, v in layer.items()} for layer in tree]
    lora, lopt, meta = ft.load_finetune_checkpoint(ckpt, lora_template=template)
    assert lopt is None and meta["user_metadata"]["epoch"] == 1 and meta["step"] is None
    for got, want in zip(lora, tree):
        assert got["vB"].dtype is nb.DType.bfloat16
        for k in want:
            np.testing.assert_array_equal(got[k].cast(nb.DType.float32).to_numpy(),
                                          want[k].cast(nb.DType.float32).to_numpy())
    with pytest.raises(FileNotFoundError):
        ft.load_finetune_checkpoint(tmp_path / "nonexistent", lora_template=template)
    with pytest.raises(KeyError, match="Missing tensor key"):
        ft.load_finetune_checkpoint(ckpt, lora_template=template + [dict(template[0])])


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_qlora_base_product_reads_the_codes(emulator, dtype):
    """A weight whose width is a multiple of 8: qlora_linear's base product is one launch on the
    NF4 codes (no dense weight in the plan), forward and, for the gradient with respect to the
    activations, the same kernel on the transposed weight; values against the oracle."""
    from nabla_amd.core import engine
    rng = np.random.default_rng(2031)
    n, din, dout = 24, 40, 16
    x = rng.standard_normal((2, n, din)).astype(np.float32)
    w = rng.standard_normal((din, dout)).astype(np.float32)
    dt = nb.DType.float32 if dtype == "f32" else nb.DType.bfloat16
    tol = 2e-5 if dtype == "f32" else 2e-2
    qw = ft.quantize_nf4(T(w), block_size=8)
    adapter = {"A": T(rng.standard_normal((din, 4)).astype(np.float32) * 0.1),
               "B": T(rng.standard_normal((4, dout)).astype(np.float32) * 0.1)}
    wd = O.nf4_dequantize(O.nf4_quantize(w, 8)).astype(np.float64)
    A, B = (adapter[k].to_numpy().astype(np.float64) for k in "AB")

    def f(xt, p):
        return nb.reduce_sum(ft.qlora_linear(xt, qw, p, alpha=2.0, compute_dtype=dt) ** 2)

    engine.clear_plan_cache()
    y = ft.qlora_linear(T(x), qw, adapter, alpha=2.0, compute_dtype=dt)
    want = x.astype(np.float64) @ wd + x.astype(np.float64) @ ((A @ B) * 0.5)
    got = y.to(nb.DType.float32).to_numpy()
    assert np.abs(got - want).max() <= tol * np.abs(want).max()
    kinds = [st.kind for st in list(engine._PLAN_CACHE.values())[-1].plan.steps]
    assert kinds.count("gemm_nf4") == 1 and "gather" not in kinds
    gx, gp = nb.grad(f, argnums=(0, 1))(T(x), adapter)
    nb.realize_all(gx, gp["A"], gp["B"])
    steps = list(engine._PLAN_CACHE.values())[-1].plan.steps
    assert sorted(st.attrs["transpose"] for st in steps if st.kind == "gemm_nf4") == [False, True]
    vx, vA, vB = O.V(x.astype(np.float64)), O.V(A), O.V(B)
    out = O.matmul(vx, O.V(wd)) + O.matmul(vx, O.matmul(vA, vB) * 0.5)
    wgx, wgA, wgB = O.grad_of(O.reduce_sum(out * out), [vx, vA, vB])
    for g, wnt in ((gx, wgx), (gp["A"], wgA), (gp["B"], wgB)):
        g = g.to(nb.DType.float32).to_numpy()
        assert np.abs(g - wnt).max() <= (tol if dtype == "f32" else 4e-2) * np.abs(wnt).max()
