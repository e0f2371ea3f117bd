"""Integer tensors above 2^24 (where fp32 stops holding every integer) through the fused
elementwise kernels: shared by the emulator-backed host test and the GPU test.  Results must
equal numpy's bit for bit.  int64 tensors are also taken beyond 2^31 and 2^53: fused kernels
hold integers in 32-bit registers, so whatever computes on int64 values runs in the 64-bit
integer kernel, and the one use that stays fused (a comparison with an in-range index) must
not be fooled by values that only agree in their low 32 bits."""
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


def check_int64_beyond_int32(nb):
    """int64 arithmetic, comparisons, selects and casts on values outside the int32 range (and
    outside what a double holds exactly) equal numpy's int64 results bit for bit."""
    T = nb.Tensor.constant
    I64 = nb.DType.int64
    rng = np.random.default_rng(321)
    a = rng.integers(-2 ** 62, 2 ** 62, (9, 37)).astype(np.int64)
    a[0, :6] = [2 ** 31, 2 ** 40 + 5, -2 ** 33, 2 ** 53 + 1, -(2 ** 31) - 1, 2 ** 31 - 1]
    b = rng.integers(-2 ** 40, 2 ** 40, (9, 37)).astype(np.int64)
    b[0, :6] = [1, -7, 2 ** 33, -(2 ** 53), 0, 1]
    A, B = T(a), T(b)
    np.testing.assert_array_equal((A + 1).numpy(), a + 1)
    np.testing.assert_array_equal((A + B).numpy(), a + b)
    np.testing.assert_array_equal((A - B).numpy(), a - b)
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal((A * B).numpy(), a * b)          # wraps modulo 2^64, as numpy
        np.testing.assert_array_equal((B * 3 + A).numpy(), b * 3 + a)
    np.testing.assert_array_equal((-A).numpy(), -a)
    np.testing.assert_array_equal(nb.abs(A).numpy(), np.abs(a))
    np.testing.assert_array_equal(nb.relu(A).numpy(), np.maximum(a, 0))
    np.testing.assert_array_equal(nb.where(nb.greater(A, B), A, B).numpy(), np.maximum(a, b))
    # comparisons of two stored tensors whose low 32 bits agree
    c = a + 2 ** 32
    np.testing.assert_array_equal(nb.equal(A, T(c)).numpy(), np.zeros(a.shape, bool))
    np.testing.assert_array_equal(nb.greater(T(c), A).numpy(), c > a)
    np.testing.assert_array_equal(nb.greater(A + 1, A).numpy(), np.ones(a.shape, bool))
    np.testing.assert_array_equal(nb.equal(A + B, A).numpy(), b == 0)
    # selects and copies move all 64 bits
    mask = T(b > 0)
    np.testing.assert_array_equal(nb.where(mask, A, B).numpy(), np.where(b > 0, a, b))
    np.testing.assert_array_equal(nb.where(mask, A, A * 0 + 5000000000).numpy(), np.where(b > 0, a, 5000000000))
    # an int64 tensor as the condition
    with np.errstate(over="ignore"):
        high = b * 2 ** 32  # nothing in the low 32 bits
    np.testing.assert_array_equal(nb.where(T(high), A, B).numpy(), np.where(high != 0, a, b))
    # reductions
    np.testing.assert_array_equal(nb.reduce_sum(B, axis=1).numpy(), b.sum(1))
    np.testing.assert_array_equal(nb.reduce_max(A, axis=0).numpy(), a.max(0))
    np.testing.assert_array_equal(nb.reduce_min(A, axis=1).numpy(), a.min(1))
    np.testing.assert_array_equal(nb.argmax(A, axis=1).numpy(), a.argmax(1))
    np.testing.assert_array_equal(nb.argmin(A, axis=0).numpy(), a.argmin(0))
    # casts: to float (nearest), to int32 (low bits), to bool, from float (toward zero), from bool
    np.testing.assert_array_equal(nb.cast(A, nb.DType.float32).numpy(), a.astype(np.float32))
    np.testing.assert_array_equal(nb.cast(A, nb.DType.int32).numpy(), a.astype(np.int32))
    np.testing.assert_array_equal(nb.cast(T(high), nb.DType.bool).numpy(), high != 0)
    f = (rng.standard_normal((9, 37)) * 1e12).astype(np.float32)
    np.testing.assert_array_equal(nb.cast(T(f), I64).numpy(), np.trunc(f).astype(np.int64))
    np.testing.assert_array_equal(nb.cast(mask, I64).numpy(), (b > 0).astype(np.int64))
    # int64 meets float as float
    np.testing.assert_array_equal((A * T(np.float32(0.5))).numpy(), a.astype(np.float32) * np.float32(0.5))
    np.testing.assert_array_equal(nb.greater(B, T(np.zeros(b.shape, np.float32))).numpy(), b.astype(np.float32) > 0)
    # the fused use: labels against a class index.  A label that only matches a class in its
    # low 32 bits (2^32 + 3) selects nothing, as in the reference's one-hot comparison.
    labels = np.array([3, 2 ** 32 + 3, -1, 0, 6, 2 ** 31, -(2 ** 32) + 6], np.int64)
    classes = nb.arange(0, 7, dtype=I64)
    hits = nb.equal(nb.unsqueeze(T(labels), -1), classes).numpy()
    np.testing.assert_array_equal(hits, labels[:, None] == np.arange(7))
    logits = rng.standard_normal((7, 7)).astype(np.float32)
    picked = nb.reduce_sum(T(logits) * nb.cast(nb.equal(nb.unsqueeze(T(labels), -1), classes), nb.DType.float32), axis=1)
    want = np.where((labels >= 0) & (labels < 7), logits[np.arange(7), np.clip(labels, 0, 6)], 0.0)
    np.testing.assert_array_equal(picked.numpy(), want.astype(np.float32))
    np.testing.assert_array_equal(nb.greater(nb.unsqueeze(T(labels), -1), classes).numpy(), labels[:, None] > np.arange(7))
    np.testing.assert_array_equal(nb.less_equal(nb.unsqueeze(T(labels), -1), classes).numpy(), labels[:, None] <= np.arange(7))
