"""Random tensors and dropout: shared by the emulator-backed host test and the GPU test.  The
expected numbers come from the numpy restatement of the generator (oracle/philox.py), which
the known-answer vectors of Philox4x32-10 pin."""
import numpy as np

from oracle import philox


def check_streams_match_the_generator(nb):
    """uniform / gaussian / keep mask element by element: the first tensor drawn after a seed is
    run 0, the next evaluation run 1; two tensors of one evaluation are streams 0 and 1."""
    nb.set_seed(1234)
    u = nb.uniform((37, 19), -2.0, 3.0)
    np.testing.assert_array_equal(u.numpy().ravel(), philox.uniform(37 * 19, -2.0, 3.0, 1234, 0, 0))
    g = nb.gaussian((1001,), 1.5, 0.5)
    np.testing.assert_allclose(g.numpy(), philox.normal(1001, 1.5, 0.5, 1234, 1, 0), rtol=2e-5, atol=2e-6)

    def two(_):
        return nb.uniform((8, 5)) , nb.uniform((8, 5))
    a, b = nb.compile(two)(nb.Tensor.constant(np.zeros(1, np.float32)))
    np.testing.assert_array_equal(a.numpy().ravel(), philox.uniform(40, 0.0, 1.0, 1234, 2, 0))
    np.testing.assert_array_equal(b.numpy().ravel(), philox.uniform(40, 0.0, 1.0, 1234, 2, 1))
    # bfloat16 output is the fp32 draw rounded once
    h = nb.uniform((64,), dtype=nb.DType.bfloat16)
    want = philox.uniform(64, 0.0, 1.0, 1234, 3, 0)
    np.testing.assert_allclose(h.to(nb.DType.float32).numpy(), want, rtol=2.0 ** -8)


def check_statistics(nb):
    nb.set_seed(99)
    u = nb.uniform((4096, 256)).numpy()
    assert 0.0 <= u.min() and u.max() < 1.0
    assert abs(u.mean() - 0.5) < 1e-3 and abs(u.var() - 1.0 / 12.0) < 1e-3
    # no visible dependence between neighbours or between the four words of a block
    flat = u.ravel()
    assert abs(np.corrcoef(flat[:-1], flat[1:])[0, 1]) < 5e-3
    assert abs(np.corrcoef(flat[0::4], flat[3::4])[0, 1]) < 5e-3
    z = nb.gaussian((4096, 256)).numpy()
    assert abs(z.mean()) < 3e-3 and abs(z.std() - 1.0) < 3e-3
    assert abs(np.mean(z ** 3)) < 1e-2 and abs(np.mean(z ** 4) - 3.0) < 3e-2


def check_dropout(nb):
    from nabla_amd.nn import functional as F
    nb.set_seed(5)
    x = nb.Tensor.constant(np.random.default_rng(0).standard_normal((300, 257)).astype(np.float32) + 3.0)
    p = 0.3
    # the backward pass multiplies by the mask the forward pass applied
    y, pull = nb.vjp(lambda t: F.dropout(t, p), x)
    gx = pull(nb.ones_like(y))
    gx = gx[0] if isinstance(gx, (tuple, list)) else gx
    y, gx, xh = y.numpy(), gx.numpy(), x.numpy()
    kept = y != 0
    np.testing.assert_array_equal(kept, philox.keep_mask(300 * 257, p, 5, 0, 0).reshape(300, 257))
    np.testing.assert_allclose(y[kept], xh[kept] / (1.0 - p), rtol=1e-6)
    np.testing.assert_allclose(gx, kept / np.float32(1.0 - p), rtol=1e-6)
    assert abs(kept.mean() - (1.0 - p)) < 5e-3
    # evaluation mode and the two ends of the range
    assert F.dropout(x, p, training=False) is x and F.dropout(x, 0.0) is x
    assert not F.dropout(x, 1.0).numpy().any()
    # a compiled step draws a new mask on every call, and the same ones again after the seed
    step = nb.compile(lambda t: F.dropout(t, 0.5))
    nb.set_seed(11)
    first = [step(x).numpy() for _ in range(3)]
    assert not np.array_equal(first[0] != 0, first[1] != 0) and not np.array_equal(first[1] != 0, first[2] != 0)
    nb.set_seed(11)
    again = [step(x).numpy() for _ in range(3)]
    for a, b in zip(first, again):
        np.testing.assert_array_equal(a, b)


def check_training_mode_encoder_layer(nb):
    """The encoder layer with its default arguments (dropout 0.1, training mode) runs forward and
    backward; in evaluation mode it is deterministic."""
    from nabla_amd.nn.modules import TransformerEncoderLayer
    rng = np.random.default_rng(3)
    layer = TransformerEncoderLayer(32, 4, 64)
    x = nb.Tensor.constant(rng.standard_normal((2, 8, 32)).astype(np.float32))
    nb.set_seed(1)
    a = layer(x).numpy()
    b = layer(x).numpy()
    assert np.isfinite(a).all() and not np.array_equal(a, b)

    def loss(t):
        return nb.mean(layer(t) ** 2)
    nb.set_seed(1)
    val, gx = nb.value_and_grad(loss)(x)
    assert np.isfinite(val.numpy()).all() and np.isfinite(gx.numpy()).all() and np.abs(gx.numpy()).max() > 0
    layer.eval()
    np.testing.assert_array_equal(layer(x).numpy(), layer(x).numpy())
