"""Integer tensors above 2^24 (where fp32 stops holding every integer) through the fused
elementwise kernels: shared by the emulator-backed host test and the GPU test.  Results must
equal numpy's bit for bit.  (Values stay inside the int32 range: fused kernels compute int64
tensors in 32-bit registers.)"""
import numpy as np


def check_large_integers(nb):
    T = nb.Tensor.constant
    rng = np.random.default_rng(123)
    big = 2 ** 24
    for dt in (np.int32, np.int64):
        a = rng.integers(big, 2 ** 30, (13, 67)).astype(dt)
        a[0, :4] = [big + 1, -(big + 1), 2 ** 30 + 5, -(2 ** 30) + 7]
        b = rng.integers(-5, 6, (13, 67)).astype(dt)
        A, B = T(a), T(b)
        np.testing.assert_array_equal((A + 0).numpy(), a)                     # 16777217 + 0 stays itself
        np.testing.assert_array_equal((A + B).numpy(), a + b)
        np.testing.assert_array_equal((A - B).numpy(), a - b)
        np.testing.assert_array_equal((B * 3 + A).numpy(), b * 3 + a)
        np.testing.assert_array_equal((-A).numpy(), -a)
        np.testing.assert_array_equal(nb.abs(-A).numpy(), np.abs(a))
        np.testing.assert_array_equal(nb.relu(A - 2 ** 29).numpy(), np.maximum(a - 2 ** 29, 0))
        # neighbours that fp32 cannot tell apart
        np.testing.assert_array_equal(nb.greater(A + 1, A).numpy(), np.ones(a.shape, bool))
        np.testing.assert_array_equal(nb.equal(A + 1, A).numpy(), np.zeros(a.shape, bool))
        np.testing.assert_array_equal(nb.equal(A + B, A).numpy(), b == 0)
        # where / select move the values untouched; constants above 2^24 too
        mask = T(b > 0)
        np.testing.assert_array_equal(nb.where(mask, A, B).numpy(), np.where(b > 0, a, b))
        got = nb.where(mask, A * 0 + 20000001, A).numpy()
        np.testing.assert_array_equal(got, np.where(b > 0, dt(20000001), a))
        # sums keep a 64-bit accumulator (int64 results beyond 2^31 are exact)
        np.testing.assert_array_equal(nb.reduce_sum(A, axis=1).numpy(), a.sum(1, dtype=dt))
        np.testing.assert_array_equal(nb.reduce_sum(A, axis=0).numpy(), a.sum(0, dtype=dt))
        np.testing.assert_array_equal(nb.reduce_max(A, axis=1).numpy(), a.max(1))
        np.testing.assert_array_equal(nb.reduce_min(A + B, axis=0).numpy(), (a + b).min(0))
        # casts at the edges
        np.testing.assert_array_equal(nb.cast(A, nb.DType.float32).numpy(), a.astype(np.float32))
        f = (a // 256 * 256).astype(np.float32) + np.float32(0.75)  # fractions are cut toward zero
        target = nb.DType.int64 if dt is np.int64 else nb.DType.int32
        np.testing.assert_array_equal(nb.cast(T(f), target).numpy(), np.trunc(f).astype(dt))
        np.testing.assert_array_equal(nb.cast(B, nb.DType.bool).numpy(), b != 0)
    # an index vector longer than 2^24 would be needed to see COLIDX lose exactness; the int
    # form is checked on a start beyond 2^24 instead
    r = nb.arange(big + 1, big + 1 + 40, dtype=nb.DType.int64) + T(np.zeros(40, np.int64))
    np.testing.assert_array_equal(r.numpy(), np.arange(big + 1, big + 41, dtype=np.int64))
