"""First GPU bring-up checks: every kernel family against torch-CPU fp64."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def T(a, dtype=None):
    import nabla_amd as nb
    return nb.Tensor.constant(a, dtype=dtype)


def test_elementwise_chain(hip):
    import nabla_amd as nb
    rng = np.random.default_rng(0)
    x = rng.standard_normal((37, 130)).astype(np.float32)
    y = rng.standard_normal((37, 130)).astype(np.float32)
    z = nb.relu(T(x) * T(y) + 1.0) - nb.exp(T(x) * 0.1)
    ref = np.maximum(x * y + 1, 0) - np.exp(x * np.float32(0.1))
    np.testing.assert_allclose(z.numpy(), ref, rtol=1e-6, atol=1e-6)


def test_row_reduce_and_grad(hip):
    import nabla_amd as nb
    rng = np.random.default_rng(1)
    for shape in [(8, 16), (33, 1000), (5, 4096 + 12)]:
        x = rng.standard_normal(shape).astype(np.float32)
        y = rng.standard_normal(shape).astype(np.float32)

        def f(X, Y):
            p = X * Y
            m = nb.reduce_max(p, axis=1, keepdims=True)
            return nb.reduce_sum(nb.exp(p - m) * nb.relu(X), axis=1)

        X, Y = T(x), T(y)
        out = f(X, Y)
        g = nb.grad(lambda X, Y: nb.reduce_sum(f(X, Y)), realize=True, create_graph=False)(X, Y)
        xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
        yt = torch.tensor(y, dtype=torch.float64)
        pt = xt * yt
        ot = (torch.exp(pt - pt.max(1, keepdim=True).values) * torch.relu(xt)).sum(1)
        ot.sum().backward()
        np.testing.assert_allclose(out.numpy(), ot.detach().numpy(), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(g.numpy(), xt.grad.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape", [(128, 128, 64), (200, 136, 72), (512, 384, 256), (64, 10, 256),
                                   (1024, 1024, 512),
                                   (5000, 4104, 192),    # 128 x 128 tiles, many, ragged edges
                                   (5000, 5128, 128),
                                   (4000, 2600, 192)])   # 256 x 256 tiles with ragged edges
def test_gemm(hip, dtype, layout, shape):
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(2)
    tdt = torch.float32 if dtype == "f32" else torch.bfloat16
    A = torch.tensor(rng.standard_normal((M, K)), dtype=tdt)
    B = torch.tensor(rng.standard_normal((K, N)), dtype=tdt)
    ref = (A.double() @ B.double()).numpy()
    a_dev = (A if layout[0] == "n" else A.t().contiguous()).cuda()
    b_dev = (B if layout[1] == "n" else B.t().contiguous()).cuda()
    c_dev = torch.empty((M, N), dtype=tdt, device="cuda")
    d = lib.GemmDesc()
    d.A, d.B, d.C = a_dev.data_ptr(), b_dev.data_ptr(), c_dev.data_ptr()
    d.M, d.N, d.K = M, N, K
    d.a_rs, d.a_cs = (K, 1) if layout[0] == "n" else (1, M)
    d.b_rs, d.b_cs = (N, 1) if layout[1] == "n" else (1, K)
    d.ldc = N
    d.batch, d.a_bs, d.b_bs, d.c_bs = 1, 0, 0, 0
    d.dtype_ab = d.dtype_c = 0 if dtype == "f32" else 1
    d.alpha = 1.0
    L = lib.load()
    lib.check(L.nbk_gemm(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = c_dev.double().cpu().numpy()
    # fp32: accumulation-order noise only; bf16: the result is rounded to 8 mantissa bits
    rtol, atol = (1e-5, 1e-5 * np.sqrt(K)) if dtype == "f32" else (2.0 ** -8, 2e-2)
    err = np.abs(got - ref) - rtol * np.abs(ref)
    assert err.max() <= atol, err.max()


@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape,k2,how", [
    ((512, 384, 256), 16, "same"),      # one more K tile of the launch (128 x 128 tiles)
    ((1024, 1024, 512), 8, "same"),     # 256 x 256 tiles; a single 16-byte piece per row of the pair
    ((4000, 2600, 192), 64, "same"),    # a whole tile deep, ragged edges
    ((1000, 520, 128), 24, "same"),
    ((512, 384, 256), 16, "bias"),      # the epilogue sees the sum of both products
    ((512, 384, 256), 12, "same"),      # K2 % 8 != 0: two launches give the sum
    ((512, 384, 256), 80, "same"),      # deeper than a tile: two launches
    ((512, 384, 256), 16, "other"),     # the pair laid out the other way round: two launches
    ((512, 384, 256), 16, "offset"),    # the pair not 16-byte aligned: two launches
    ((200, 136, 72), 16, "same"),       # K % 64 != 0: the guarded kernel, two launches
])
def test_gemm_with_a_second_operand_pair(hip, layout, shape, k2, how):
    """C = A @ B + A2 @ B2 (the update of a low-rank adapter inside its base product) through
    the C ABI against float64 of the same bf16 operands: where the pair meets the direct-to-LDS
    kernels' conditions it is one more K tile of the launch, elsewhere the library runs the two
    products one after the other, the second adding itself to the first."""
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(11)
    bf = torch.bfloat16
    A = torch.tensor(rng.standard_normal((M, K)), dtype=bf)
    B = torch.tensor(rng.standard_normal((K, N)), dtype=bf)
    A2 = torch.tensor(rng.standard_normal((M, k2)) * 3.0, dtype=bf)
    B2 = torch.tensor(rng.standard_normal((k2, N)) * 3.0, dtype=bf)
    bias = torch.tensor(rng.standard_normal((N,)) * 4.0, dtype=bf)
    first = (A.double() @ B.double()).numpy()
    ref = first + (A2.double() @ B2.double()).numpy()
    if how == "bias":
        ref = ref + bias.double().numpy()
    lay2 = layout if how != "other" else ("t" if layout[0] == "n" else "n") + ("t" if layout[1] == "n" else "n")

    def put(t, transposed, shift=0):
        t = t.t().contiguous() if transposed else t.contiguous()
        if not shift:
            return t.cuda(), 0
        flat = torch.zeros(t.numel() + 8, dtype=bf)
        flat[shift:shift + t.numel()] = t.reshape(-1)
        return flat.cuda(), shift * 2

    a_dev, _ = put(A, layout[0] == "t")
    b_dev, _ = put(B, layout[1] == "t")
    shift = 3 if how == "offset" else 0
    a2_dev, a2_off = put(A2, lay2[0] == "t", shift)
    b2_dev, b2_off = put(B2, lay2[1] == "t", shift)
    bias_dev = bias.cuda()
    c_dev = torch.full((M, N), float("nan"), dtype=bf, device="cuda")
    d = lib.GemmDesc()
    d.A, d.B, d.C = a_dev.data_ptr(), b_dev.data_ptr(), c_dev.data_ptr()
    d.M, d.N, d.K = M, N, K
    d.a_rs, d.a_cs = (K, 1) if layout[0] == "n" else (1, M)
    d.b_rs, d.b_cs = (N, 1) if layout[1] == "n" else (1, K)
    d.n_terms = 1
    t = d.term[0]
    t.A, t.B, t.K = a2_dev.data_ptr() + a2_off, b2_dev.data_ptr() + b2_off, k2
    t.a_rs, t.a_cs = (k2, 1) if lay2[0] == "n" else (1, M)
    t.b_rs, t.b_cs = (N, 1) if lay2[1] == "n" else (1, k2)
    d.ldc = N
    d.batch, d.a_bs, d.b_bs, d.c_bs = 1, 0, 0, 0
    d.dtype_ab = d.dtype_c = 1
    d.alpha = 1.0
    if how == "bias":
        d.bias = bias_dev.data_ptr()
    L = lib.load()
    lib.check(L.nbk_gemm(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = c_dev.double().cpu().numpy()
    # (two launches round the first product to bf16 before the second is added: one more
    # rounding, of a value that may be larger than the sum)
    err = np.abs(got - ref) - 2.0 ** -8 * (np.abs(ref) + np.abs(first))
    assert err.max() <= 2e-2, err.max()


@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape,ks,how", [
    ((512, 384, 256), (256, 128), "same"),            # two deep pairs behind A and B (128 x 128 tiles)
    ((1024, 1024, 512), (512, 512, 16, 8), "same"),   # 256 x 256 tiles; two deep, two shallow: all four terms
    ((4000, 2600, 192), (64, 24), "same"),            # ragged edges; a deep pair of one tile and a shallow one
    ((1024, 1024, 512), (512, 16), "bias"),
    ((512, 384, 256), (256, 128, 64), "same"),        # three deep pairs: the third runs as a launch of its own
    ((512, 384, 256), (256,), "pitch"),               # a deep pair with another row pitch: launch of its own
    ((512, 384, 256), (16, 16, 8), "same"),           # three shallow pairs: launches of their own
])
def test_gemm_with_several_operand_pairs(hip, layout, shape, ks, how):
    """C = A @ B + sum_i A_i @ B_i through the C ABI (a gradient that several products
    contribute to, with or without low-rank updates) against float64 of the same bf16 operands:
    up to two deep pairs laid out like A and B and two shallow ones run inside one launch, whatever
    else is asked for as one launch per pair that adds itself to the result so far."""
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(13)
    bf = torch.bfloat16

    def operands(k, pitch=0):
        A = torch.tensor(rng.standard_normal((M, k)), dtype=bf)
        B = torch.tensor(rng.standard_normal((k, N)), dtype=bf)
        if layout[0] == "n":
            a_dev = torch.zeros((M, k + pitch), dtype=bf)
            a_dev[:, :k] = A
            a_str = (k + pitch, 1)
        else:
            a_dev = torch.zeros((k, M + pitch), dtype=bf)
            a_dev[:, :M] = A.t()
            a_str = (1, M + pitch)
        if layout[1] == "n":
            b_dev = torch.zeros((k, N + pitch), dtype=bf)
            b_dev[:, :N] = B
            b_str = (N + pitch, 1)
        else:
            b_dev = torch.zeros((N, k + pitch), dtype=bf)
            b_dev[:, :k] = B.t()
            b_str = (1, k + pitch)
        return A, B, a_dev.cuda(), b_dev.cuda(), a_str, b_str

    main = operands(K)
    terms = [operands(k, 8 if how == "pitch" else 0) for k in ks]
    parts = [(main[0].double() @ main[1].double()).numpy()] + [(t[0].double() @ t[1].double()).numpy() for t in terms]
    ref = sum(parts)
    bias = torch.tensor(rng.standard_normal((N,)) * 4.0, dtype=bf)
    if how == "bias":
        ref = ref + bias.double().numpy()
    bias_dev = bias.cuda()
    c_dev = torch.full((M, N), float("nan"), dtype=bf, device="cuda")
    d = lib.GemmDesc()
    d.A, d.B, d.C = main[2].data_ptr(), main[3].data_ptr(), c_dev.data_ptr()
    d.M, d.N, d.K = M, N, K
    (d.a_rs, d.a_cs), (d.b_rs, d.b_cs) = main[4], main[5]
    d.ldc = N
    d.batch = 1
    d.dtype_ab = d.dtype_c = 1
    d.alpha = 1.0
    d.n_terms = len(terms)
    for i, (t, k) in enumerate(zip(terms, ks)):
        d.term[i].A, d.term[i].B, d.term[i].K = t[2].data_ptr(), t[3].data_ptr(), k
        (d.term[i].a_rs, d.term[i].a_cs), (d.term[i].b_rs, d.term[i].b_cs) = t[4], t[5]
    if how == "bias":
        d.bias = bias_dev.data_ptr()
    L = lib.load()
    lib.check(L.nbk_gemm(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = c_dev.double().cpu().numpy()
    # (launches of their own round the result so far to bf16 before they add to it)
    running = np.abs(np.cumsum(np.stack(parts), axis=0)).sum(axis=0)
    err = np.abs(got - ref) - 2.0 ** -8 * (np.abs(ref) + running)
    assert err.max() <= 2e-2, err.max()


def test_gemm_second_pair_errors(hip):
    """What the second operand pair does not go with is refused, not dropped."""
    from nabla_amd.backend import lib
    bf = torch.bfloat16
    x = torch.zeros((256, 256), dtype=bf, device="cuda")
    x32 = torch.zeros((256, 256), dtype=torch.float32, device="cuda")
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def desc(t=x, **kw):
        d = lib.GemmDesc()
        d.A = d.B = d.C = t.data_ptr()
        d.M = d.N = d.K = 256
        d.a_rs, d.a_cs, d.b_rs, d.b_cs, d.ldc = 256, 1, 256, 1, 256
        d.batch = 1
        d.dtype_ab = d.dtype_c = 1 if t is x else 0
        d.alpha = 1.0
        d.n_terms = 1
        d.term[0].A, d.term[0].B, d.term[0].K = x.data_ptr(), x.data_ptr(), 16
        d.term[0].a_rs, d.term[0].a_cs, d.term[0].b_rs, d.term[0].b_cs = 16, 1, 256, 1
        for k, v in kw.items():
            if k.startswith("t0_"):
                setattr(d.term[0], k[3:], v)
            else:
                setattr(d, k, v)
        return d

    assert L.nbk_gemm(C.byref(desc()), st) == 0
    for bad in (desc(t0_A=None), desc(batch=2), desc(t=x32), desc(t0_a_rs=16, t0_a_cs=2), desc(n_terms=5),
                desc(t0_K=12, act=1),               # two launches cannot carry an epilogue
                desc(colsum=x.data_ptr(), a_rs=1, a_cs=256)):
        assert L.nbk_gemm(C.byref(bad), st) != 0
        assert b"gemm" in L.nbk_last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape", [(384, 256, 2048), (1000, 520, 4096)])
def test_gemm_long_k_small_output(hip, layout, shape):
    """bf16 products with a long contraction and few 128 x 128 tiles (the shapes the planner
    would otherwise split along K), through the C ABI in one piece."""
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(5)
    A = torch.tensor(rng.standard_normal((M, K)), dtype=torch.bfloat16)
    B = torch.tensor(rng.standard_normal((K, N)), dtype=torch.bfloat16)
    ref = (A.double() @ B.double()).numpy()
    a_dev = (A if layout[0] == "n" else A.t().contiguous()).cuda()
    b_dev = (B if layout[1] == "n" else B.t().contiguous()).cuda()
    c_dev = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    d = lib.GemmDesc()
    d.A, d.B, d.C = a_dev.data_ptr(), b_dev.data_ptr(), c_dev.data_ptr()
    d.M, d.N, d.K = M, N, K
    d.a_rs, d.a_cs = (K, 1) if layout[0] == "n" else (1, M)
    d.b_rs, d.b_cs = (N, 1) if layout[1] == "n" else (1, K)
    d.ldc = N
    d.batch, d.a_bs, d.b_bs, d.c_bs = 1, 0, 0, 0
    d.dtype_ab = d.dtype_c = 1
    d.alpha = 1.0
    L = lib.load()
    lib.check(L.nbk_gemm(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = c_dev.double().cpu().numpy()
    err = np.abs(got - ref) - 2.0 ** -8 * np.abs(ref)
    assert err.max() <= 2e-2, err.max()


@pytest.mark.parametrize("shape,ks", [((1024, 1024, 2048), 1), ((256, 136, 512), 1), ((1024, 520, 4096), 4),
                                      ((8, 8, 64), 1), ((4096, 1024, 1024), 1)])
def test_gemm_column_sums(hip, shape, ks):
    """The weight gradient x^T dy with the column sums of dy (the bias gradient) as a second
    result of the same launch: whole, and split along K into fp32 partial products and partial
    sums.  The product must be what the launch without the sums gives, bit for bit; the sums
    are checked against fp64 with the rounding of their dtype and accumulation length."""
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(8)
    xt = torch.tensor(rng.standard_normal((K, M)), dtype=torch.bfloat16).cuda()   # x, read as x^T
    dy = torch.tensor(rng.standard_normal((K, N)) + 0.25, dtype=torch.bfloat16).cuda()
    odt = torch.bfloat16 if ks == 1 else torch.float32
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def run(with_sums):
        c = torch.full((ks, M, N), float("nan"), dtype=odt, device="cuda")
        cs = torch.full((ks, N), float("nan"), dtype=odt, device="cuda")
        d = lib.GemmDesc()
        d.A, d.B, d.C = xt.data_ptr(), dy.data_ptr(), c.data_ptr()
        d.M, d.N, d.K = M, N, K // ks
        d.a_rs, d.a_cs, d.b_rs, d.b_cs, d.ldc = 1, M, N, 1, N
        d.batch, d.a_bs, d.b_bs, d.c_bs, d.batch_inner = ks, (K // ks) * M, (K // ks) * N, M * N, 1
        d.dtype_ab, d.dtype_c, d.alpha = 1, (1 if ks == 1 else 0), 1.0
        d.colsum = cs.data_ptr() if with_sums else None
        lib.check(L.nbk_gemm(C.byref(d), st))
        torch.cuda.synchronize()
        return c, cs

    c0, _ = run(False)
    c1, cs = run(True)
    ref_c = (xt.double().t().cpu() @ dy.double().cpu()).numpy()
    got_c = c1.double().sum(0).cpu().numpy()
    assert (np.abs(got_c - ref_c) - 2.0 ** -8 * np.abs(ref_c)).max() <= 2e-2
    if K // ks > 16 and not (M >= 256 and N >= 256 and -(-M // 256) * -(-N // 256) * ks * 10 >= 256 * 6):
        # (the same kernel and tile with and without the sums: identical products)
        assert torch.equal(c0, c1)
    ref_s = dy.double().cpu().reshape(ks, K // ks, N).sum(1).numpy()
    got_s = cs.double().cpu().numpy()
    tol = 2.0 ** -8 * np.abs(ref_s) + 1e-4 * np.sqrt(K / ks)
    assert (np.abs(got_s - ref_s) <= tol).all(), np.abs(got_s - ref_s).max()


@pytest.mark.parametrize("shape,members,ks", [((1024, 1024, 2048), 3, 4), ((256, 136, 1024), 2, 2),
                                              ((128, 128, 512), 3, 1)])
def test_gemm_column_sums_over_two_batch_levels(hip, shape, members, ks):
    """x^T dy_m for several dy_m that lie equally spaced in one buffer, each split along K, as ONE
    launch: batch index (member, slice), the left operand shared (batch stride 0), partial
    products and partial column sums in (member, slice) order.  Every slice must be what the
    launch of that member alone gives, bit for bit."""
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(9)
    xt = torch.tensor(rng.standard_normal((K, M)), dtype=torch.bfloat16).cuda()
    gap = K * N + 64                                       # elements between members
    dys = torch.zeros(members * gap, dtype=torch.bfloat16, device="cuda")
    for m in range(members):
        dys[m * gap:m * gap + K * N] = torch.tensor(rng.standard_normal(K * N) + 0.25, dtype=torch.bfloat16).cuda()
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    kc = K // ks

    def run(first, count):
        c = torch.full((count * ks, M, N), float("nan"), dtype=torch.float32, device="cuda")
        cs = torch.full((count * ks, N), float("nan"), dtype=torch.float32, device="cuda")
        d = lib.GemmDesc()
        d.A, d.B, d.C = xt.data_ptr(), dys.data_ptr() + first * gap * 2, c.data_ptr()
        d.M, d.N, d.K = M, N, kc
        d.a_rs, d.a_cs, d.b_rs, d.b_cs, d.ldc = 1, M, N, 1, N
        d.batch, d.batch_inner = count * ks, ks
        d.a_bs, d.b_bs, d.c_bs = 0, gap, ks * M * N
        d.a_bs2, d.b_bs2, d.c_bs2 = kc * M, kc * N, M * N
        d.dtype_ab, d.dtype_c, d.alpha = 1, 0, 1.0
        d.colsum = cs.data_ptr()
        lib.check(L.nbk_gemm(C.byref(d), st))
        torch.cuda.synchronize()
        return c, cs

    c_all, cs_all = run(0, members)
    for m in range(members):
        c_one, cs_one = run(m, 1)
        assert torch.equal(c_all[m * ks:(m + 1) * ks], c_one), m
        assert torch.equal(cs_all[m * ks:(m + 1) * ks], cs_one), m
        dy = dys[m * gap:m * gap + K * N].reshape(K, N)
        ref_c = (xt.double().t().cpu() @ dy.double().cpu()).numpy()
        got_c = c_one.double().sum(0).cpu().numpy()
        assert np.abs(got_c - ref_c).max() <= 1e-3 * np.abs(ref_c).max()
        ref_s = dy.double().cpu().reshape(ks, kc, N).sum(1).numpy()
        assert np.abs(cs_one.double().cpu().numpy() - ref_s).max() <= 1e-4 * np.sqrt(kc)


def test_gemm_column_sums_refuses_what_the_kernel_does_not_cover(hip):
    from nabla_amd.backend import lib
    a = torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda")
    cs = torch.zeros((64,), dtype=torch.bfloat16, device="cuda")
    d = lib.GemmDesc()
    d.A, d.B, d.C, d.colsum = a.data_ptr(), a.data_ptr(), a.data_ptr(), cs.data_ptr()
    d.M = d.N = d.K = 64
    d.a_rs, d.a_cs, d.b_rs, d.b_cs, d.ldc = 64, 1, 64, 1, 64      # A K-contiguous: not covered
    d.batch, d.batch_inner, d.dtype_ab, d.dtype_c, d.alpha = 1, 1, 1, 1, 1.0
    L = lib.load()
    assert L.nbk_gemm(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)) != 0


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("act", [0, 1, 2])
@pytest.mark.parametrize("shape", [(256, 384, 128),      # 128 x 128 tiles
                                   (300, 200, 72),       # guarded kernel (K % 64 != 0)
                                   (640, 520, 2048),     # 128 x 128 tiles, long K
                                   (4096, 2560, 192)])   # 256 x 256 tiles
@pytest.mark.parametrize("res_op", [0, 1])
def test_gemm_epilogue(hip, dtype, act, shape, res_op):
    """act(alpha * A @ B + bias) (+ or x) residual, the fused way out of nbk_gemm."""
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(6)
    tdt = torch.float32 if dtype == "f32" else torch.bfloat16
    A = torch.tensor(rng.standard_normal((M, K)) / np.sqrt(K), dtype=tdt)
    B = torch.tensor(rng.standard_normal((N, K)), dtype=tdt)            # "nt": both K-contiguous
    bias = torch.tensor(rng.standard_normal((N,)), dtype=tdt)
    R = torch.tensor(rng.standard_normal((M, N)), dtype=tdt)
    alpha = 1.5
    z = alpha * (A.double() @ B.double().t()) + bias.double()
    z = z if act == 0 else (torch.relu(z) if act == 1 else torch.nn.functional.gelu(z))
    ref = (z * R.double() if res_op else z + R.double()).numpy()
    a_dev, b_dev, bias_dev, r_dev = A.cuda(), B.cuda(), bias.cuda(), R.cuda()
    c_dev = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
    d = lib.GemmDesc()
    d.A, d.B, d.C = a_dev.data_ptr(), b_dev.data_ptr(), c_dev.data_ptr()
    d.bias, d.residual = bias_dev.data_ptr(), r_dev.data_ptr()
    d.M, d.N, d.K = M, N, K
    d.a_rs, d.a_cs, d.b_rs, d.b_cs = K, 1, 1, K
    d.ldc = N
    d.batch, d.a_bs, d.b_bs, d.c_bs = 1, 0, 0, M * N
    d.dtype_ab = d.dtype_c = 0 if dtype == "f32" else 1
    d.act = act
    d.residual_op = res_op
    d.alpha = alpha
    L = lib.load()
    lib.check(L.nbk_gemm(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = c_dev.double().cpu().numpy()
    rtol, atol = (1e-5, 1e-5) if dtype == "f32" else (2.0 ** -8, 2e-2)
    err = np.abs(got - ref) - rtol * np.abs(ref)
    assert err.max() <= atol, err.max()


@pytest.mark.parametrize("b_layout", ["n", "t"])
@pytest.mark.parametrize("out", ["bf16", "f32"])
@pytest.mark.parametrize("shape", [(2048, 16, 2048), (1500, 8, 320), (1024, 32, 1024), (4100, 24, 256),
                                   (3000, 5, 192)])
def test_gemm_few_columns(hip, b_layout, out, shape):
    """bf16 products with at most 32 columns (the down-projection of a low-rank adapter and its
    transpose): rows of A straight into MFMA fragments, K split over the waves of a workgroup."""
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(13)
    A = torch.tensor(rng.standard_normal((M, K)) / np.sqrt(K), dtype=torch.bfloat16)
    B = torch.tensor(rng.standard_normal((K, N)), dtype=torch.bfloat16)
    odt = torch.bfloat16 if out == "bf16" else torch.float32
    alpha = 0.75
    ref = (alpha * (A.double() @ B.double())).numpy()
    a_dev = A.cuda()
    b_dev = (B if b_layout == "n" else B.t().contiguous()).cuda()
    c_dev = torch.full((M, N), float("nan"), dtype=odt, device="cuda")
    d = lib.GemmDesc()
    d.A, d.B, d.C = a_dev.data_ptr(), b_dev.data_ptr(), c_dev.data_ptr()
    d.M, d.N, d.K = M, N, K
    d.a_rs, d.a_cs = K, 1
    d.b_rs, d.b_cs = (N, 1) if b_layout == "n" else (1, K)
    d.ldc = N
    d.batch, d.a_bs, d.b_bs, d.c_bs = 1, 0, 0, 0
    d.dtype_ab, d.dtype_c = 1, (1 if out == "bf16" else 0)
    d.alpha = alpha
    L = lib.load()
    lib.check(L.nbk_gemm(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = c_dev.double().cpu().numpy()
    rtol, atol = (2.0 ** -8, 1e-4) if out == "bf16" else (1e-5, 1e-5)
    err = np.abs(got - ref) - rtol * np.abs(ref)
    assert err.max() <= atol, err.max()


@pytest.mark.parametrize("b_layout", ["n", "t"])
@pytest.mark.parametrize("out", ["bf16", "f32"])
@pytest.mark.parametrize("shape", [(4096, 512, 16), (3001, 1032, 16), (2048, 1024, 8), (1100, 2048, 13)])
def test_gemm_low_rank_product(hip, b_layout, out, shape):
    """bf16 products with a contraction of at most 16 (the up-projection of a low-rank
    adapter), with the scale and the residual the kernel adds on its way out."""
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(12)
    A = torch.tensor(rng.standard_normal((M, K)), dtype=torch.bfloat16)
    B = torch.tensor(rng.standard_normal((K, N)), dtype=torch.bfloat16)
    odt = torch.bfloat16 if out == "bf16" else torch.float32
    R = torch.tensor(rng.standard_normal((M, N)), dtype=odt)
    alpha = 0.375
    L = lib.load()
    for with_res in (False, True):
        ref = alpha * (A.double() @ B.double()) + (R.double() if with_res else 0.0)
        a_dev, r_dev = A.cuda(), R.cuda()
        b_dev = (B if b_layout == "n" else B.t().contiguous()).cuda()
        c_dev = torch.full((M, N), float("nan"), dtype=odt, device="cuda")
        d = lib.GemmDesc()
        d.A, d.B, d.C = a_dev.data_ptr(), b_dev.data_ptr(), c_dev.data_ptr()
        d.residual = r_dev.data_ptr() if with_res else None
        d.M, d.N, d.K = M, N, K
        d.a_rs, d.a_cs = K, 1
        d.b_rs, d.b_cs = (N, 1) if b_layout == "n" else (1, K)
        d.ldc = N
        d.batch, d.a_bs, d.b_bs, d.c_bs = 1, 0, 0, 0
        d.dtype_ab, d.dtype_c = 1, (1 if out == "bf16" else 0)
        d.alpha = alpha
        lib.check(L.nbk_gemm(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        got = c_dev.double().cpu().numpy()
        rtol, atol = (2.0 ** -8, 1e-5) if out == "bf16" else (1e-6, 1e-5)
        err = np.abs(got - ref.numpy()) - rtol * np.abs(ref.numpy())
        assert err.max() <= atol, (with_res, err.max())


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("shape", [(512, 512, 256), (300, 136, 72), (64, 40, 24), (1024, 256, 512)])
def test_gemm_activation_and_its_derivative_as_two_results(hip, dtype, shape):
    """C = gelu(A @ B + bias) and C_aux = gelu'(A @ B + bias) from one launch, against float64
    torch (exact erf form, nabla/ops/unary.py:567-595); every tile size and both dtypes."""
    from nabla_amd.backend import lib
    M, N, K = shape
    rng = np.random.default_rng(14)
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    A = torch.tensor(rng.standard_normal((M, K)) * 0.2, dtype=tdt)
    B = torch.tensor(rng.standard_normal((K, N)) * 0.2, dtype=tdt)
    bias = torch.tensor(rng.standard_normal((N,)), dtype=tdt)
    x = (A.double() @ B.double() + bias.double()).requires_grad_(True)
    y = torch.nn.functional.gelu(x)
    (dy,) = torch.autograd.grad(y.sum(), x)
    a_dev, b_dev, bias_dev = A.cuda(), B.cuda(), bias.cuda()
    c_dev = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
    c2_dev = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
    L = lib.load()
    d = lib.GemmDesc()
    d.A, d.B, d.C, d.bias = a_dev.data_ptr(), b_dev.data_ptr(), c_dev.data_ptr(), bias_dev.data_ptr()
    d.C_aux, d.aux_op, d.act = c2_dev.data_ptr(), 1, 2
    d.M, d.N, d.K = M, N, K
    d.a_rs, d.a_cs, d.b_rs, d.b_cs, d.ldc = K, 1, N, 1, N
    d.batch, d.a_bs, d.b_bs, d.c_bs = 1, 0, 0, 0
    d.dtype_ab = d.dtype_c = 1 if dtype == "bf16" else 0
    d.alpha = 1.0
    print(f"gemm gelu + derivative {shape} {dtype}", flush=True)
    lib.check(L.nbk_gemm(C.byref(d), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    rtol, atol = (2.0 ** -8, 2e-3) if dtype == "bf16" else (1e-5, 1e-5)
    for got, want in ((c_dev, y.detach()), (c2_dev, dy)):
        err = (got.double().cpu() - want).abs() - rtol * want.abs()
        assert err.max().item() <= atol, err.max().item()
    # the derivative without an activation, or together with a residual, is refused
    d.act = 0
    with pytest.raises(ValueError, match="derivative"):
        lib.check(L.nbk_gemm(C.byref(d), None))


def test_mlp_grads(hip):
    import nabla_amd as nb
    rng = np.random.default_rng(0)
    x = rng.uniform(-0.05, 0.05, (128, 784)).astype(np.float32)
    W1 = rng.uniform(-0.05, 0.05, (784, 256)).astype(np.float32)
    W2 = rng.uniform(-0.05, 0.05, (256, 10)).astype(np.float32)
    b1 = np.zeros((1, 256), np.float32)
    b2 = np.zeros((1, 10), np.float32)

    def loss_fn(W1, b1, W2, b2, x):
        return nb.mean(nb.relu(x @ W1 + b1) @ W2 + b2)

    args = [T(a) for a in (W1, b1, W2, b2, x)]
    loss, grads = nb.value_and_grad(loss_fn, argnums=(0, 1, 2, 3))(*args)
    nb.realize_all(loss, *grads)
    ta = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (W1, b1, W2, b2)]
    tl = (torch.relu(torch.tensor(x, dtype=torch.float64) @ ta[0] + ta[1]) @ ta[2] + ta[3]).mean()
    tl.backward()
    assert abs(loss.item() - tl.item()) <= 1e-5 * abs(tl.item()) + 1e-9
    for g, t in zip(grads, ta):
        ref = t.grad.numpy()
        assert np.abs(g.numpy() - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-9


def test_layernorm_softmax_grads(hip):
    import nabla_amd as nb
    F = nb.nn.functional
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 6, 256)).astype(np.float32)
    w = rng.standard_normal((256,)).astype(np.float32)
    b = rng.standard_normal((256,)).astype(np.float32)

    def loss_fn(x, w, b):
        y = F.layer_norm(x, w, b)
        return nb.mean(nb.softmax(y, axis=-1) * y)

    l, gs = nb.value_and_grad(loss_fn, argnums=(0, 1, 2))(T(x), T(w), T(b))
    nb.realize_all(l, *gs)
    tx, tw, tb = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (x, w, b)]
    ty = torch.nn.functional.layer_norm(tx, (256,), tw, tb)
    tl = (torch.softmax(ty, -1) * ty).mean()
    tl.backward()
    assert abs(l.item() - tl.item()) < 1e-5
    for g, t in zip(gs, (tx, tw, tb)):
        ref = t.grad.numpy()
        assert np.abs(g.numpy() - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-8


def test_conv_pool_grads(hip):
    import nabla_amd as nb
    rng = np.random.default_rng(4)
    x = rng.uniform(0, 1, (4, 12, 12, 3)).astype(np.float32)
    w1 = (rng.standard_normal((3, 3, 3, 8)) * 0.3).astype(np.float32)
    b1 = (rng.standard_normal((8,)) * 0.1).astype(np.float32)
    w2 = (rng.standard_normal((3, 3, 8, 16)) * 0.2).astype(np.float32)

    def loss_fn(w1, b1, w2, x):
        h = nb.relu(nb.conv2d(x, w1, stride=(1, 1), padding=1, bias=b1))
        h = nb.max_pool2d(h, kernel_size=2)
        h = nb.conv2d(h, w2, stride=(2, 1), padding=(1, 0, 2, 1))
        return nb.mean(h * h)

    l, gs = nb.value_and_grad(loss_fn, argnums=(0, 1, 2, 3))(T(w1), T(b1), T(w2), T(x))
    nb.realize_all(l, *gs)
    import torch.nn.functional as TF
    tw1, tb1, tw2, tx = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (w1, b1, w2, x)]
    h = TF.conv2d(tx.permute(0, 3, 1, 2), tw1.permute(3, 2, 0, 1), tb1, padding=1)
    h = TF.max_pool2d(torch.relu(h), 2)
    h = TF.conv2d(TF.pad(h, (2, 1, 1, 0)), tw2.permute(3, 2, 0, 1), stride=(2, 1))
    tl = (h * h).mean()
    tl.backward()
    assert abs(l.item() - tl.item()) <= 1e-5 * abs(tl.item())
    for g, t in zip(gs, (tw1, tb1, tw2, tx)):
        ref = t.grad.numpy()
        assert np.abs(g.numpy() - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-8


@pytest.mark.parametrize("shape,kernel,stride,pad", [((3, 12, 12, 16), (2, 2), (2, 2), (0, 0)),
                                                     ((2, 9, 11, 8), (3, 3), (2, 2), (1, 1)),
                                                     ((2, 8, 8, 12), (3, 2), (1, 1), (1, 0)),
                                                     ((2, 7, 7, 6), (2, 2), (2, 2), (0, 0))])
def test_max_pool_through_the_c_abi(hip, shape, kernel, stride, pad):
    """nbk_maxpool2d_fwd / _bwd against the oracle: channel counts that take the four-channel
    form (16-byte accesses) and one that does not, overlapping windows, clipped borders, and
    ties (values from a small set, so several elements of a window are its maximum and each
    takes the window's cotangent).  The four-channel form and the general form (the same tensors
    at addresses that are not 16-byte aligned) must agree bit for bit."""
    from nabla_amd.backend import lib
    from oracle import ops as O
    N, H, W, Cc = shape
    (kh, kw), (sh, sw), (pt, pl) = kernel, stride, pad
    rng = np.random.default_rng(21)
    x = rng.integers(-3, 4, shape).astype(np.float32) * 0.5
    vx = O.V(x)
    vy = O.max_pool2d(vx, kernel, stride, (pt, pt, pl, pl))
    Ho, Wo = vy.a.shape[1:3]
    g = rng.standard_normal(vy.a.shape).astype(np.float32)
    (want_gx,) = vy.vjp(g)
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    d = lib.PoolDesc()
    d.N, d.H, d.W, d.C, d.Ho, d.Wo = N, H, W, Cc, Ho, Wo
    d.kh, d.kw, d.stride_h, d.stride_w, d.pad_t, d.pad_l, d.dtype = kh, kw, sh, sw, pt, pl, 0
    results = []
    for shift in (0, 1):     # element offset of every tensor inside its allocation
        def dev(a):
            buf = torch.zeros(a.size + 4, dtype=torch.float32, device="cuda")
            buf[shift:shift + a.size] = torch.tensor(a.reshape(-1))
            return buf, buf[shift:shift + a.size]
        xb, xd = dev(x)
        yb, yd = dev(np.full(vy.a.shape, np.nan, np.float32))
        gb, gd = dev(g)
        dxb, dxd = dev(np.full(shape, np.nan, np.float32))
        lib.check(L.nbk_maxpool2d_fwd(C.byref(d), C.c_void_p(xd.data_ptr()), C.c_void_p(yd.data_ptr()), st))
        lib.check(L.nbk_maxpool2d_bwd(C.byref(d), C.c_void_p(xd.data_ptr()), C.c_void_p(yd.data_ptr()),
                                      C.c_void_p(gd.data_ptr()), C.c_void_p(dxd.data_ptr()), st))
        torch.cuda.synchronize()
        results.append((yd.cpu().numpy().reshape(vy.a.shape), dxd.cpu().numpy().reshape(shape)))
    for y, dx in results:
        np.testing.assert_array_equal(y, vy.a)
        np.testing.assert_allclose(dx, want_gx, rtol=1e-6, atol=1e-6)
    np.testing.assert_array_equal(results[0][1], results[1][1])


def test_gather_argmax_views(hip):
    import nabla_amd as nb
    rng = np.random.default_rng(5)
    table = rng.standard_normal((50, 24)).astype(np.float32)
    idx = rng.integers(0, 50, (3, 7)).astype(np.int64)
    out = nb.gather(T(table), T(idx), axis=0)
    assert np.array_equal(out.numpy(), table[idx])
    logits = rng.standard_normal((9, 33)).astype(np.float32)
    assert np.array_equal(nb.argmax(T(logits), axis=-1).numpy(), logits.argmax(-1))
    x = rng.standard_normal((4, 5, 6)).astype(np.float32)
    y = nb.permute(T(x), (2, 0, 1)) * 2.0
    np.testing.assert_array_equal(y.numpy(), x.transpose(2, 0, 1) * 2)
    z = nb.pad(T(x), [(1, 0), (0, 2), (1, 1)], value=-1.0)
    np.testing.assert_array_equal(z.numpy(), np.pad(x, [(1, 0), (0, 2), (1, 1)], constant_values=-1))
    c = nb.concatenate([T(x), T(x) + 1.0], axis=1)
    np.testing.assert_array_equal(c.numpy(), np.concatenate([x, x + 1], 1))


def test_gemm_two_batch_levels(hip):
    """Heads stay in place: A is [B,S,H,hd] read as a [B,H] batch of S x hd matrices and C is
    written in [B,S,H,hd] order, as the attention products of the transformer block do."""
    from nabla_amd.backend import lib
    Bn, S, H, hd = 2, 96, 3, 64
    rng = np.random.default_rng(11)
    q = torch.tensor(rng.standard_normal((Bn, S, H, hd)), dtype=torch.bfloat16)
    k = torch.tensor(rng.standard_normal((Bn, S, H, hd)), dtype=torch.bfloat16)
    p = torch.tensor(rng.standard_normal((Bn, H, S, S)), dtype=torch.bfloat16)
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    qd, kd, pd = q.cuda(), k.cuda(), p.cuda()
    # scores[b,h] = q[b,:,h,:] @ k[b,:,h,:]^T
    sc = torch.empty((Bn, H, S, S), dtype=torch.bfloat16, device="cuda")
    d = lib.GemmDesc()
    d.A, d.B, d.C = qd.data_ptr(), kd.data_ptr(), sc.data_ptr()
    d.M, d.N, d.K = S, S, hd
    d.a_rs, d.a_cs, d.b_rs, d.b_cs = H * hd, 1, 1, H * hd
    d.ldc = S
    d.batch, d.batch_inner = Bn * H, H
    d.a_bs, d.a_bs2 = S * H * hd, hd
    d.b_bs, d.b_bs2 = S * H * hd, hd
    d.c_bs, d.c_bs2 = H * S * S, S * S
    d.dtype_ab = d.dtype_c = 1
    d.alpha = 1.0
    lib.check(L.nbk_gemm(C.byref(d), st))
    # out[b,:,h,:] = p[b,h] @ k[b,:,h,:]  written with head stride hd, row stride H*hd
    out = torch.zeros((Bn, S, H, hd), dtype=torch.bfloat16, device="cuda")
    d2 = lib.GemmDesc()
    d2.A, d2.B, d2.C = pd.data_ptr(), kd.data_ptr(), out.data_ptr()
    d2.M, d2.N, d2.K = S, hd, S
    d2.a_rs, d2.a_cs, d2.b_rs, d2.b_cs = S, 1, H * hd, 1
    d2.ldc = H * hd
    d2.batch, d2.batch_inner = Bn * H, H
    d2.a_bs, d2.a_bs2 = H * S * S, S * S
    d2.b_bs, d2.b_bs2 = S * H * hd, hd
    d2.c_bs, d2.c_bs2 = S * H * hd, hd
    d2.dtype_ab = d2.dtype_c = 1
    d2.alpha = 1.0
    lib.check(L.nbk_gemm(C.byref(d2), st))
    torch.cuda.synchronize()
    ref_sc = torch.einsum("bshd,bthd->bhst", q.double(), k.double())
    ref_out = torch.einsum("bhst,bthd->bshd", p.double(), k.double())
    for got, ref in ((sc, ref_sc), (out, ref_out)):
        err = (got.double().cpu() - ref).abs() - 2.0 ** -8 * ref.abs()
        assert err.max().item() <= 2e-2


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("outer,red,inner", [(1, 8192, 1024), (3, 100, 40), (2, 77, 8), (1, 5, 1048576),
                                             (4, 300, 1), (1, 4096, 24)])
def test_reduce_mid_direct(hip, dtype, outer, red, inner):
    from nabla_amd.backend import lib
    rng = np.random.default_rng(12)
    tdt = torch.float32 if dtype == "f32" else torch.bfloat16
    x = torch.tensor(rng.standard_normal((outer, red, inner)), dtype=tdt)
    xd = x.cuda()
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    code = 0 if dtype == "f32" else 1
    for kind, fn in ((0, lambda t: t.sum(1)), (1, lambda t: t.max(1).values), (2, lambda t: t.min(1).values)):
        out = torch.empty((outer, inner), dtype=torch.float32, device="cuda")
        lib.check(L.nbk_reduce_mid(C.c_void_p(xd.data_ptr()), C.c_void_p(out.data_ptr()), code, 0,
                                   outer, red, inner, kind, st))
        torch.cuda.synchronize()
        ref = fn(x.double())
        if kind == 0:
            tol = 1e-6 * x.double().abs().sum(1) + 1e-30
            assert ((out.cpu().double() - ref).abs() <= tol).all()
        else:
            assert torch.equal(out.cpu().double(), ref)


@pytest.mark.parametrize("outer,red,inner", [(1, 2, 4194304), (3, 3, 65536 + 4 * 257), (1, 8, 65536), (2, 1, 70000),
                                             (1, 2, 65532)])
def test_reduce_mid_over_a_few_long_fp32_rows(hip, outer, red, inner):
    """The partial products of a GEMM split along K: a few fp32 rows of millions of elements
    (several pieces of the row per lane; rows shorter than 65536 take the general kernel).  Sums
    are exactly the fp32 sums in row order, with fp32 and with bf16 results; one launch for
    several such reductions gives the same bits."""
    from nabla_amd.backend import lib
    rng = np.random.default_rng(14)
    x = rng.standard_normal((outer, red, inner)).astype(np.float32)
    xd = torch.tensor(x).cuda()
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    acc = np.zeros((outer, inner), np.float32)
    for r in range(red):
        acc = acc + x[:, r]
    want = {0: acc, 1: x.max(1), 2: x.min(1)}
    tasks = (lib.ReduceTask * 6)()
    outs = []
    for i, (kind, dto) in enumerate([(0, 0), (0, 1), (1, 0), (1, 1), (2, 0), (2, 1)]):
        tdt = torch.float32 if dto == 0 else torch.bfloat16
        out = torch.full((outer, inner), float("nan"), dtype=tdt, device="cuda")
        lib.check(L.nbk_reduce_mid(C.c_void_p(xd.data_ptr()), C.c_void_p(out.data_ptr()), 0, dto,
                                   outer, red, inner, kind, st))
        torch.cuda.synchronize()
        ref = torch.tensor(want[kind]).to(tdt)
        assert torch.equal(out.cpu(), ref), (kind, dto)
        again = torch.full_like(out, float("nan"))
        t = tasks[i]
        t.in_, t.out = xd.data_ptr(), again.data_ptr()
        t.outer, t.red, t.inner = outer, red, inner
        t.dtype_in, t.dtype_out, t.kind = 0, dto, kind
        outs.append((out, again))
    lib.check(L.nbk_reduce_mid_batch(tasks, 6, st))
    torch.cuda.synchronize()
    for out, again in outs:
        assert torch.equal(out, again)


def test_reduce_mid_batch_matches_single_launches(hip):
    """One launch for many reductions: mixed dtypes, kinds, vector and element-wise shapes, more
    tasks than one launch holds; every result equals the single-task entry point's bit for bit."""
    from nabla_amd.backend import lib
    rng = np.random.default_rng(15)
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    specs = [(1, 128, 1024, "bf16", 0), (3, 64, 40, "f32", 1), (2, 77, 8, "bf16", 2), (1, 8, 4096, "f32", 0),
             (4, 300, 1, "f32", 0), (1, 515, 24, "bf16", 0)] * 5          # 30 tasks > 24 per launch
    tasks = (lib.ReduceTask * len(specs))()
    keep, want = [], []
    for t, (outer, red, inner, dt, kind) in zip(tasks, specs):
        tdt = torch.float32 if dt == "f32" else torch.bfloat16
        x = torch.tensor(rng.standard_normal((outer, red, inner)), dtype=tdt, device="cuda")
        out = torch.full((outer, inner), float("nan"), dtype=torch.float32, device="cuda")
        ref = torch.empty_like(out)
        code = 0 if dt == "f32" else 1
        lib.check(L.nbk_reduce_mid(C.c_void_p(x.data_ptr()), C.c_void_p(ref.data_ptr()), code, 0, outer, red,
                                   inner, kind, st))
        t.in_, t.out = x.data_ptr(), out.data_ptr()
        t.outer, t.red, t.inner = outer, red, inner
        t.dtype_in, t.dtype_out, t.kind = code, 0, kind
        keep.append((x, out))
        want.append(ref)
    lib.check(L.nbk_reduce_mid_batch(tasks, len(specs), st))
    torch.cuda.synchronize()
    for (x, out), ref in zip(keep, want):
        assert torch.equal(out, ref)
    with pytest.raises(ValueError, match="no tasks"):
        lib.check(L.nbk_reduce_mid_batch(tasks, 0, st))


@pytest.mark.parametrize("cin,cout,stride", [(16, 24, 1), (3, 8, 2), (32, 64, 1)])
def test_conv_forward_with_relu_through_the_c_abi(hip, cin, cout, stride):
    """`nbk_conv_desc.act = NBK_ACT_RELU`: max(conv(x, w) + bias, 0), bit for bit the relu of what
    the same launch without the activation stores, against torch in float64; the two gradient
    entry points refuse an activation."""
    import torch.nn.functional as F
    from nabla_amd.backend import lib
    rng = np.random.default_rng(17)
    N, H, W = 4, 11, 9
    x = torch.tensor(rng.standard_normal((N, H, W, cin)), dtype=torch.float32)
    w = torch.tensor(rng.standard_normal((3, 3, cin, cout)) * 0.3, dtype=torch.float32)
    b = torch.tensor(rng.standard_normal((cout,)), dtype=torch.float32)
    Ho, Wo = (H + 2 - 3) // stride + 1, (W + 2 - 3) // stride + 1
    d = lib.ConvDesc()
    d.N, d.H, d.W, d.Cin, d.R, d.S, d.Cout, d.Ho, d.Wo = N, H, W, cin, 3, 3, cout, Ho, Wo
    d.stride_h = d.stride_w = stride
    d.pad_t = d.pad_b = d.pad_l = d.pad_r = 1
    d.dtype = 0
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    xd, wd, bd = x.cuda(), w.cuda(), b.cuda()
    outs = []
    for act in (0, 1):
        d.act = act
        y = torch.full((N, Ho, Wo, cout), float("nan"), dtype=torch.float32, device="cuda")
        lib.check(L.nbk_conv2d_fwd(C.byref(d), C.c_void_p(xd.data_ptr()), C.c_void_p(wd.data_ptr()),
                                   C.c_void_p(bd.data_ptr()), C.c_void_p(y.data_ptr()), st))
        torch.cuda.synchronize()
        outs.append(y.cpu())
    assert torch.equal(outs[1], torch.relu(outs[0]))
    ref = F.conv2d(x.double().permute(0, 3, 1, 2), w.double().permute(3, 2, 0, 1), b.double(),
                   stride=stride, padding=1).permute(0, 2, 3, 1)
    assert (outs[1].double() - torch.relu(ref)).abs().max().item() <= 1e-5 * ref.abs().max().item()
    d.act = 1
    dx = torch.empty_like(xd)
    assert L.nbk_conv2d_dgrad(C.byref(d), C.c_void_p(outs[0].cuda().data_ptr()), C.c_void_p(wd.data_ptr()),
                              C.c_void_p(dx.data_ptr()), st) != 0
    d.act = 7
    y = torch.empty((N, Ho, Wo, cout), dtype=torch.float32, device="cuda")
    assert L.nbk_conv2d_fwd(C.byref(d), C.c_void_p(xd.data_ptr()), C.c_void_p(wd.data_ptr()),
                            C.c_void_p(bd.data_ptr()), C.c_void_p(y.data_ptr()), st) != 0


def test_conv_wgrad_workspace_and_fallback(hip):
    """The K-split filter gradient (with workspace) and the unsplit one (workspace NULL)
    agree to summation-order noise, and both match a float64 reference."""
    import torch.nn.functional as F
    from nabla_amd.backend import lib
    rng = np.random.default_rng(13)
    N, H, W, Cin, Cout = 8, 16, 16, 16, 24
    x = torch.tensor(rng.standard_normal((N, H, W, Cin)), dtype=torch.float32)
    dy = torch.tensor(rng.standard_normal((N, H, W, Cout)), dtype=torch.float32)
    d = lib.ConvDesc()
    d.N, d.H, d.W, d.Cin, d.R, d.S, d.Cout, d.Ho, d.Wo = N, H, W, Cin, 3, 3, Cout, H, W
    d.stride_h = d.stride_w = 1
    d.pad_t = d.pad_b = d.pad_l = d.pad_r = 1
    d.dtype = 0
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = L.nbk_conv2d_wgrad_workspace(C.byref(d))
    assert need > 0
    xd, dyd = x.cuda(), dy.cuda()
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    dw1 = torch.empty((3, 3, Cin, Cout), dtype=torch.float32, device="cuda")
    dw2 = torch.empty_like(dw1)
    lib.check(L.nbk_conv2d_wgrad(C.byref(d), C.c_void_p(xd.data_ptr()), C.c_void_p(dyd.data_ptr()),
                                 C.c_void_p(dw1.data_ptr()), C.c_void_p(ws.data_ptr()), need, st))
    lib.check(L.nbk_conv2d_wgrad(C.byref(d), C.c_void_p(xd.data_ptr()), C.c_void_p(dyd.data_ptr()),
                                 C.c_void_p(dw2.data_ptr()), None, 0, st))
    torch.cuda.synchronize()
    wt = torch.zeros((Cout, Cin, 3, 3), dtype=torch.float64, requires_grad=True)
    y = F.conv2d(x.double().permute(0, 3, 1, 2), wt, padding=1)
    (g,) = torch.autograd.grad(y, wt, dy.double().permute(0, 3, 1, 2))
    ref = g.permute(2, 3, 1, 0)
    scale = ref.abs().max().item()
    assert (dw1.cpu().double() - ref).abs().max().item() <= 1e-5 * scale
    assert (dw2.cpu().double() - ref).abs().max().item() <= 1e-5 * scale


def _tensor_desc(lib, t, shape=None, strides=None):
    d = lib.TensorDesc()
    d.ptr = t.data_ptr()
    d.dtype = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2, torch.int32: 3, torch.int64: 4,
               torch.bool: 5, torch.uint8: 5}[t.dtype]
    shape = tuple(t.shape) if shape is None else shape
    strides = tuple(t.stride()) if strides is None else strides
    d.rank = len(shape)
    for i, (n, st) in enumerate(zip(shape, strides)):
        d.shape[i], d.stride[i] = n, st
    return d


def test_int64_elementwise_kernel_through_the_c_abi(hip):
    """nbk_ew_int64: every operation on values beyond 2^31 and 2^53 against numpy's int64
    arithmetic (wrapping sums and products, division toward zero, powers modulo 2^64), operands
    of every integer type, broadcast through zero strides, a permuted operand, immediates, all
    four kinds of result, a rank-0 and an empty problem, and the argument errors."""
    from nabla_amd.backend import isa, lib
    L = lib.load()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(91)
    shape = (5, 7, 9)
    a = rng.integers(-2 ** 62, 2 ** 62, shape).astype(np.int64)
    a.reshape(-1)[:4] = [2 ** 31, -(2 ** 31) - 1, 2 ** 53 + 1, -(2 ** 63)]
    b = rng.integers(-2 ** 33, 2 ** 33, shape).astype(np.int64)
    b.reshape(-1)[:4] = [-1, 0, 3, -1]
    small = rng.integers(0, 6, shape).astype(np.int64)

    def run(fn, ins, out_dtype=torch.int64, imm=None, out_shape=shape):
        devs = [None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in ins]
        out = torch.empty(out_shape, dtype=out_dtype, device="cuda")
        descs = (lib.TensorDesc * len(ins))()
        for i, t in enumerate(devs):
            if t is None:
                descs[i].rank = len(out_shape)
                continue
            bshape = tuple(t.shape)
            strides = tuple(0 if n == 1 and m != 1 else s for n, m, s in zip(bshape, out_shape, t.stride()))
            descs[i] = _tensor_desc(lib, t, out_shape, strides)
        imms = (C.c_int64 * len(ins))(*([0] * len(ins)))
        for i, v in enumerate(imm or []):
            if v is not None:
                imms[i] = v
        od = _tensor_desc(lib, out)
        lib.check(L.nbk_ew_int64(isa.EW[fn], descs, imms, len(ins), C.byref(od), st))
        torch.cuda.synchronize()
        return out.cpu().numpy()

    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(run("add", [a, b]), a + b)
        np.testing.assert_array_equal(run("sub", [a, b]), a - b)
        np.testing.assert_array_equal(run("mul", [a, b]), a * b)
        np.testing.assert_array_equal(run("fma", [a, b, small]), a * b + small)
        np.testing.assert_array_equal(run("neg", [a]), -a)
        np.testing.assert_array_equal(run("abs", [a]), np.abs(a))
        want_pow = np.empty(shape, np.int64)
        for idx in np.ndindex(shape):
            v = pow(int(b[idx]), int(small[idx]), 2 ** 64)
            want_pow[idx] = v - 2 ** 64 if v >= 2 ** 63 else v
        np.testing.assert_array_equal(run("pow", [b, small]), want_pow)
    q = np.where(b == 0, 0, np.sign(a) * np.sign(b) * (np.abs(a.astype(object)) // np.maximum(np.abs(b.astype(object)), 1)))
    q = np.where((a == -(2 ** 63)) & (b == -1), -(2 ** 63), q).astype(np.int64)
    np.testing.assert_array_equal(run("div", [a, b]), q)
    np.testing.assert_array_equal(run("relu", [a]), np.maximum(a, 0))
    np.testing.assert_array_equal(run("max", [a, b]), np.maximum(a, b))
    np.testing.assert_array_equal(run("min", [a, b]), np.minimum(a, b))
    for fn, op in (("gt", np.greater), ("ge", np.greater_equal), ("eq", np.equal), ("ne", np.not_equal),
                   ("lt", np.less), ("le", np.less_equal)):
        np.testing.assert_array_equal(run(fn, [a, a + (small - 2) * 2 ** 32], torch.bool), op(a, a + (small - 2) * 2 ** 32))
    np.testing.assert_array_equal(run("where", [small > 2, a, b]), np.where(small > 2, a, b))
    np.testing.assert_array_equal(run("and", [small, b], torch.bool), (small != 0) & (b != 0))
    np.testing.assert_array_equal(run("not", [small * 2 ** 40], torch.bool), small == 0)
    # operand types: int32 and bool widen; a float is cut toward zero
    i32 = rng.integers(-2 ** 31, 2 ** 31, shape).astype(np.int32)
    np.testing.assert_array_equal(run("add", [a, i32]), a + i32)
    f = (rng.standard_normal(shape) * 1e15).astype(np.float32)
    np.testing.assert_array_equal(run("trunc", [f]), np.trunc(f).astype(np.int64))
    # results: int32 keeps the low bits, floats round to nearest
    np.testing.assert_array_equal(run("mov", [a], torch.int32), a.astype(np.int32))
    np.testing.assert_array_equal(run("mov", [a], torch.float32), a.astype(np.float32))
    # broadcast operands (zero strides), an immediate, a permuted view
    row = rng.integers(-2 ** 40, 2 ** 40, (1, 7, 1)).astype(np.int64)
    np.testing.assert_array_equal(run("add", [a, row]), a + row)
    np.testing.assert_array_equal(run("mul", [a, None], imm=[None, -3]), a * -3)
    at = torch.from_numpy(a).cuda()
    perm = at.permute(2, 0, 1)                                   # [9, 5, 7] view of [5, 7, 9] storage
    out = torch.empty((9, 5, 7), dtype=torch.int64, device="cuda")
    descs = (lib.TensorDesc * 2)()
    descs[0] = _tensor_desc(lib, perm, tuple(perm.shape), tuple(perm.stride()))
    descs[1].rank = 3
    imms = (C.c_int64 * 2)(0, 2 ** 40)
    lib.check(L.nbk_ew_int64(isa.EW["sub"], descs, imms, 2, C.byref(_tensor_desc(lib, out)), st))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), np.transpose(a, (2, 0, 1)) - 2 ** 40)
    # rank 0 and empty
    np.testing.assert_array_equal(run("add", [np.int64(2 ** 62), np.int64(2 ** 62)], out_shape=()), np.int64(-(2 ** 63)))
    assert run("add", [np.zeros((0, 3), np.int64), np.zeros((0, 3), np.int64)], out_shape=(0, 3)).shape == (0, 3)
    # errors: an operation without an integer form, a wrong operand count, a shape mismatch
    od = _tensor_desc(lib, out)
    with pytest.raises(ValueError, match="no 64-bit integer form"):
        lib.check(L.nbk_ew_int64(isa.EW["exp"], descs, imms, 1, C.byref(od), st))
    with pytest.raises(ValueError, match="takes 2 operands"):
        lib.check(L.nbk_ew_int64(isa.EW["add"], descs, imms, 1, C.byref(od), st))
    bad = _tensor_desc(lib, at)
    with pytest.raises(ValueError, match="differs from the result"):
        lib.check(L.nbk_ew_int64(isa.EW["neg"], (lib.TensorDesc * 1)(bad), imms, 1, C.byref(od), st))
