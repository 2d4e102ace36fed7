"""GPU parity: every entry point of the C ABI against the CPU oracle on the same seeded inputs, against the
fixtures written from the compiled reference, and — at the benchmark's full sizes, where the oracle cannot
finish — through sampled rows and size-independent properties.

Bars (from the benchmark contract): integer/index outputs bit-exact; FP32 GEMM-type outputs within
|d| <= 1e-5 * ||a_row||_2 * ||b_col||_2 per element; plain sums within the same bound read as a dot product with
a vector of ones; softmax/CE within 1e-6 absolute (exp/log of the device library vs glibc); copies, gathers,
col2im and max-pool backward bit-exact (same additions in the same order)."""
import ctypes
import os

import numpy as np
import pytest
import torch

import oraclelib as ol

pytestmark = pytest.mark.gpu

f32 = np.float32
G = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors.npz"))


@pytest.fixture(scope="module")
def api():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from origindl_amd import capi
    assert capi.is_available()
    print("\n[device]", capi.device_info(0), flush=True)
    return capi


@pytest.fixture(scope="module")
def o():
    return ol.oracle()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def gemm_bound(a, b):
    """1e-5 * ||a_row|| * ||b_col|| for C = a @ b (a [M,K], b [K,N])."""
    return 1e-5 * np.outer(np.linalg.norm(a.astype(np.float64), axis=1), np.linalg.norm(b.astype(np.float64), axis=0))


def assert_gemm_close(got, want, a, b, what):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bound = gemm_bound(a, b) + 1e-30
    worst = float((err / bound).max())
    assert worst <= 1.0, "%s: max |d| / (1e-5 |a_row||b_col|) = %.3f" % (what, worst)


# --------------------------------------------------------------------------------------------- GEMM
GEMM_SHAPES = [(128, 128, 128), (256, 384, 128), (64, 100, 10), (33, 47, 29), (512, 784, 1000), (512, 1000, 10),
               (1, 5, 1), (130, 16, 260), (4, 1000, 4), (257, 129, 131),
               # one dimension of at most 16 (the classifier layer's products), ragged against the tile edges
               (256, 3136, 10), (70, 65, 1), (300, 200, 4), (129, 64, 5), (67, 333, 9), (65, 129, 13), (128, 1000, 16),
               # about one workgroup per compute unit: the variants with a second wave set and operands fetched two
               # slabs ahead, ragged against the tile edges and with a last K slab that is not whole
               (2052, 1000, 2044), (1000, 1056, 1020)]


@pytest.mark.parametrize("m,k,n", GEMM_SHAPES)
def test_matmul_forward_backward_vs_oracle(api, o, m, k, n):
    print("\n[case] matmul fwd+bwd", m, k, n, flush=True)
    rng = np.random.default_rng(m * 7 + k * 3 + n)
    x, w, gy = (rng.standard_normal(s, dtype=f32) for s in ((m, k), (k, n), (m, n)))
    y = host(api.mat_mul(dev(x), dev(w)))
    gx, gw = (host(t) for t in api.mat_mul_backward(dev(x), dev(w), dev(gy)))
    # the full oracle is O(mnk) scalar work: sample rows for the largest shapes
    rows = np.arange(m) if m * k * n < 3e7 else np.sort(rng.choice(m, 24, replace=False))
    yo = np.empty((len(rows), n), f32)
    for i, r in enumerate(rows):
        o.orc_matmul_rows(x, w, yo[i:i + 1], int(r), int(r) + 1, n, k)
    assert_gemm_close(y[rows], yo, x[rows], w, "C")
    # gx rows are independent too: gx[r] = gy[r] . w^T
    wT = np.ascontiguousarray(w.T)
    gxo = np.empty((len(rows), k), f32)
    for i, r in enumerate(rows):
        o.orc_matmul_rows(gy, wT, gxo[i:i + 1], int(r), int(r) + 1, k, n)
    assert_gemm_close(gx[rows], gxo, gy[rows], wT, "dA")
    # gw[K,N] = x^T . gy: rows of gw are columns of x
    xT = np.ascontiguousarray(x.T)
    krows = np.arange(k) if m * k * n < 3e7 else np.sort(rng.choice(k, 24, replace=False))
    gwo = np.empty((len(krows), n), f32)
    for i, r in enumerate(krows):
        o.orc_matmul_rows(xT, gy, gwo[i:i + 1], int(r), int(r) + 1, n, m)
    assert_gemm_close(gw[krows], gwo, xT[krows], gy, "dB")


@pytest.mark.parametrize("m,k,n", [(512, 1000, 10), (511, 1001, 10), (3, 128, 16), (1, 4100, 1), (1030, 130, 7), (64, 2049, 3)])
def test_classifier_layer_products_on_the_vector_units(api, o, m, k, n):
    """Outputs of at most 16 columns over a K of 128 or more take gemm_skinny.hip: forward with bias and activation in
    one launch, both gradients in one launch, either gradient alone the same floats as both together."""
    print("\n[case] classifier products", m, k, n, flush=True)
    rng = np.random.default_rng(m + k + n)
    x, w, gy, b = (rng.standard_normal(s, dtype=f32) for s in ((m, k), (k, n), (m, n), (n,)))
    yo = np.empty((m, n), f32)
    o.orc_matmul(x, w, yo, m, n, k)
    assert_gemm_close(host(api.mat_mul(dev(x), dev(w))), yo, x, w, "C")
    dx, dw, db = dev(x), dev(w), dev(b)
    fused = torch.empty((m, n), device="cuda")
    plain = api.binary("add", api.mat_mul(dx, dw), dev(np.broadcast_to(b, (m, n)).copy()))
    for code, act in ((-1, None), (0, "relu"), (7, "silu")):
        api.lib().call("odl_hip_linear_act", dx.data_ptr(), dw.data_ptr(), db.data_ptr(), m, n, k, code, fused.data_ptr(), None, 0,
                       None)
        want = host(api.unary(act, plain)) if act else host(plain)
        assert np.array_equal(host(fused), want), act
    gx, gw = (host(t) for t in api.mat_mul_backward(dev(x), dev(w), dev(gy)))
    gxo, gwo = np.empty((m, k), f32), np.empty((k, n), f32)
    o.orc_matmul_backward(x, w, gy, gxo, gwo, m, k, n)
    assert_gemm_close(gx, gxo, gy, np.ascontiguousarray(w.T), "dA")
    assert_gemm_close(gw, gwo, np.ascontiguousarray(x.T), gy, "dB")
    gx1, none = api.mat_mul_backward(dev(x), dev(w), dev(gy), need_gw=False)
    assert none is None and np.array_equal(host(gx1), gx)
    none, gw1 = api.mat_mul_backward(dev(x), dev(w), dev(gy), need_gx=False)
    assert none is None and np.array_equal(host(gw1), gw)


@pytest.mark.parametrize("m,k,n", [(512, 784, 1000), (1024, 1024, 1024), (2048, 2048, 2048), (516, 780, 1004),
                                   (772, 1028, 520), (1000, 1000, 1000), (260, 516, 772), (2044, 2052, 1996)])
def test_matmul_backward_in_one_launch_equals_the_two_gradients_launched_alone(api, m, k, n):
    # Both gradients asked for together may run as one launch of two products (two workgroups per compute unit); asked
    # for one at a time they are launches of their own. The tile code is shared and K is walked in the same order, so the
    # results must agree bit for bit, whatever tile classes the two products fall into (64x64, 64x32, 128x128, ragged).
    print("\n[case] matmul backward pair", m, k, n, flush=True)
    import ctypes
    L = api.lib()
    g = torch.Generator(device="cuda").manual_seed(m + k + n)
    x, w, gy = (torch.randn(s, device="cuda", generator=g) for s in ((m, k), (k, n), (m, n)))
    nb = L.query("odl_hip_matmul_backward_workspace_bytes", m, k, n)
    ws = torch.empty(max(nb, 16) // 4, dtype=torch.int32, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    gx2, gw2, gx1, gw1 = (torch.full(s, float("nan"), device="cuda") for s in ((m, k), (k, n), (m, k), (k, n)))
    L.call("odl_hip_matmul_backward", P(x), P(w), P(gy), P(gx2), P(gw2), m, k, n, P(ws), nb, None)
    L.call("odl_hip_matmul_backward", P(x), P(w), P(gy), P(gx1), None, m, k, n, P(ws), nb, None)
    L.call("odl_hip_matmul_backward", P(x), P(w), P(gy), None, P(gw1), m, k, n, P(ws), nb, None)
    assert torch.equal(gx2, gx1) and torch.equal(gw2, gw1)
    want_gx, want_gw = gy.double() @ w.double().t(), x.double().t() @ gy.double()
    bx = 1e-5 * torch.outer(gy.double().norm(dim=1), w.double().norm(dim=1))
    bw = 1e-5 * torch.outer(x.double().norm(dim=0), gy.double().norm(dim=0))
    assert bool(((gx2.double() - want_gx).abs() <= bx).all()) and bool(((gw2.double() - want_gw).abs() <= bw).all())


@pytest.mark.parametrize("m,k,n", [
    (512, 1000, 10),     # the MLP's classifier layer: the three gradients in one launch, column sums one float a lane
    (256, 128, 10),      # the CNN's
    (300, 640, 16),      # sixteen classes: column sums in 16-byte pieces
    (64, 200, 12), (33, 130, 1), (17, 256, 3),
    (70000, 130, 16),    # more rows than the one-launch column sum takes: the sum as a launch of its own
    (512, 784, 1000),    # a wide layer: paired matrix gradients, then the column sum
    (5, 7, 3),
])
def test_linear_backward_equals_matmul_backward_and_sum_to(api, m, k, n):
    # Linear's backward as one library call: gx and gw must be the bits of odl_hip_matmul_backward, gb the bits of
    # Mat::sum_to of gy to the bias's shape — wherever the bias gradient rides in the classifier launch as well — and
    # every subset of the three must give the same values.
    print("\n[case] linear backward", m, k, n, flush=True)
    g = torch.Generator(device="cuda").manual_seed(m * 3 + k + n)
    x, w, gy = (torch.randn(s, device="cuda", generator=g) for s in ((m, k), (k, n), (m, n)))
    gx0, gw0 = api.mat_mul_backward(x, w, gy)
    gb0 = api.sum_to(gy, (1, n))
    gx, gw, gb = api.linear_backward(x, w, gy)
    assert torch.equal(gx, gx0) and torch.equal(gw, gw0) and torch.equal(gb, gb0)
    want = gy.double().sum(dim=0, keepdim=True)
    assert bool(((gb.double() - want).abs() <= 1e-5 * np.sqrt(m) * gy.double().norm(dim=0) + 1e-6).all())
    for need in ((True, False, True), (False, True, True), (False, False, True), (True, True, False)):
        got = api.linear_backward(x, w, gy, *need)
        for t, ref in zip(got, (gx0, gw0, gb0)):
            assert t is None or torch.equal(t, ref), need


def test_matmul_reference_unit_test_vectors(api):
    # tests/unit_test/operator/test_matmul.cpp:19-64, 119-143, 213-229
    x, w = dev(np.array([[1, 2], [3, 4]], f32)), dev(np.array([[5, 6], [7, 8]], f32))
    assert host(api.mat_mul(x, w)).ravel().tolist() == [19, 22, 43, 50]
    gx, gw = api.mat_mul_backward(x, w, dev(np.ones((2, 2), f32)))
    assert host(gx).ravel().tolist() == [11, 15, 11, 15] and host(gw).ravel().tolist() == [4, 4, 6, 6]
    a = dev(np.arange(1, 7, dtype=f32).reshape(2, 3))
    b = dev(np.arange(7, 13, dtype=f32).reshape(3, 2))
    assert host(api.mat_mul(a, b)).ravel().tolist() == [58, 64, 139, 154]
    assert (host(api.mat_mul(dev(np.ones((10, 10), f32)), dev(np.ones((10, 10), f32)))) == 10).all()
    with pytest.raises(api.OdlInvalidArgument):  # test_matmul.cpp:337-355
        api.mat_mul(dev(np.ones((2, 3), f32)), dev(np.ones((2, 3), f32)))


@pytest.mark.parametrize("size", [512, 1024, 2048])
def test_matmul_all_ones_gives_k(api, size):
    # tests/unit_test/operator/test_matmul.cpp:359-421 (device-only): ones(M,K) @ ones(K,N) == K exactly
    print("\n[case] ones", size, flush=True)
    a = torch.ones((size, size), device="cuda")
    assert bool((api.mat_mul(a, a) == float(size)).all())
    a = torch.ones((512, 1024), device="cuda")
    b = torch.ones((1024, 2048), device="cuda")
    assert bool((api.mat_mul(a, b) == 1024.0).all())
    assert api.mat_mul(torch.ones((1, 1000), device="cuda"), torch.ones((1000, 1), device="cuda")).item() == 1000.0


def test_matmul_batched(api, o):
    rng = np.random.default_rng(11)
    a, b = rng.standard_normal((3, 40, 50), dtype=f32), rng.standard_normal((3, 50, 60), dtype=f32)
    c = np.empty((3, 40, 60), f32)
    o.orc_matmul_batched(a, b, c, 3, 40, 60, 50, 1)
    got = host(api.mat_mul(dev(a), dev(b)))
    for i in range(3):
        assert_gemm_close(got[i], c[i], a[i], b[i], "bmm")
    o.orc_matmul_batched(a, b[0].copy(), c, 3, 40, 60, 50, 0)
    got = host(api.mat_mul(dev(a), dev(b[0].copy())))
    for i in range(3):
        assert_gemm_close(got[i], c[i], a[i], b[0], "3dx2d")


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_sgemm_all_layouts_split_k_and_bias(api, ta, tb):
    rng = np.random.default_rng(5 + 2 * ta + tb)
    M, N, K = 192, 136, 4096
    a = rng.standard_normal((K, M) if ta else (M, K), dtype=f32)
    b = rng.standard_normal((N, K) if tb else (K, N), dtype=f32)
    bias = rng.standard_normal(N, dtype=f32)
    A, B = (a.T if ta else a), (b.T if tb else b)
    want = A.astype(np.float64) @ B.astype(np.float64)
    for split in (1, 0, 7):
        got = host(api.sgemm(dev(a), dev(b), bool(ta), bool(tb), split_k=split))
        assert (np.abs(got - want) <= gemm_bound(A, B)).all(), (ta, tb, split)
    got = host(api.sgemm(dev(a), dev(b), bool(ta), bool(tb), bias=dev(bias), split_k=1))
    assert (np.abs(got - (want + bias)) <= gemm_bound(A, B) + 1e-6).all()
    got = host(api.sgemm(dev(a), dev(b), bool(ta), bool(tb), bias=dev(bias), split_k=5))
    assert (np.abs(got - (want + bias)) <= gemm_bound(A, B) + 1e-6).all()


@pytest.mark.parametrize("size", [1024, 2048, 4096, 8192])
def test_matmul_full_size_sampled_rows_and_linearity(api, o, size):
    # the square products of the benchmark, each size with its own tile shape and K walk: the oracle runs a seeded
    # sample of rows of C, dA and dB (rows are independent in its loop; three rows at 8192 keep it to seconds);
    # plus a size-independent property: (a1 + a2) @ b == a1 @ b + a2 @ b within the GEMM bound.
    print("\n[case] full size", size, flush=True)
    g = torch.Generator(device="cuda").manual_seed(1)
    a = torch.randn((size, size), device="cuda", generator=g)
    b = torch.randn((size, size), device="cuda", generator=g)
    gy = torch.randn((size, size), device="cuda", generator=g)
    c = api.mat_mul(a, b)
    gx, gw = api.mat_mul_backward(a, b, gy)
    rng = np.random.default_rng(2)
    rows = np.sort(rng.choice(size, 3 if size > 4096 else 6, replace=False))
    ah, bh, gyh = host(a), host(b), host(gy)
    ch, gxh, gwh = host(c), host(gx), host(gw)
    bT, aT = np.ascontiguousarray(bh.T), np.ascontiguousarray(ah.T)
    for r in rows:
        want = np.empty((1, size), f32)
        o.orc_matmul_rows(ah, bh, want, int(r), int(r) + 1, size, size)
        assert_gemm_close(ch[r:r + 1], want, ah[r:r + 1], bh, "C row %d" % r)
        o.orc_matmul_rows(gyh, bT, want, int(r), int(r) + 1, size, size)
        assert_gemm_close(gxh[r:r + 1], want, gyh[r:r + 1], bT, "dA row %d" % r)
        o.orc_matmul_rows(aT, gyh, want, int(r), int(r) + 1, size, size)
        assert_gemm_close(gwh[r:r + 1], want, aT[r:r + 1], gyh, "dB row %d" % r)
    a2 = torch.randn((size, size), device="cuda", generator=g)
    lhs = host(api.mat_mul(a + a2, b))
    rhs = ch + host(api.mat_mul(a2, b))
    bound = gemm_bound(np.abs(ah) + np.abs(host(a2)), bh)
    assert (np.abs(lhs - rhs) <= 3 * bound).all()


@pytest.mark.parametrize("m,k,n", [(2, 2, 2), (64, 64, 64), (200, 136, 520), (129, 17, 257), (512, 1000, 784), (1024, 1024, 1024),
                                   (1, 7, 1), (130, 1, 5)])
def test_matmul_float64_all_layouts_vs_the_double_oracle(api, o, m, k, n):
    """odl_hip_dgemm (FP64 matrix cores) against the double form of the reference's loops: every element within
    k * 2^-52 * sum |a||b| of it (a different but fixed summation order), integer-valued operands bit for bit, in all four
    layouts (NN; NT and TN are the two products of MatMul::backward; TT for completeness) and over ragged edges."""
    print("\n[case] matmul float64", m, k, n, flush=True)
    rng = np.random.default_rng(m * 7 + k + n)
    a, b = rng.standard_normal((m, k)), rng.standard_normal((k, n))
    want = np.empty((m, n), np.float64)
    o.orc_matmul_f64(a, b, want, m, n, k)
    bound = k * 2.0 ** -52 * (np.abs(a) @ np.abs(b)) + 1e-300
    for ta, tb in ((0, 0), (0, 1), (1, 0), (1, 1)):
        A = dev(np.ascontiguousarray(a.T) if ta else a)
        B = dev(np.ascontiguousarray(b.T) if tb else b)
        got = host(api.matmul_f64(A, B, bool(ta), bool(tb)))
        assert got.shape == (m, n) and (np.abs(got - want) <= bound).all(), (ta, tb)
    ai = rng.integers(-30, 30, (m, k)).astype(np.float64)
    bi = rng.integers(-30, 30, (k, n)).astype(np.float64)
    assert np.array_equal(host(api.matmul_f64(dev(ai), dev(bi))), ai @ bi)


def test_matmul_float64_batched_and_errors(api, o):
    rng = np.random.default_rng(5)
    a, b2, b3 = rng.standard_normal((3, 70, 33)), rng.standard_normal((33, 45)), rng.standard_normal((3, 33, 45))
    for b in (b2, b3):
        got = host(api.matmul_f64(dev(a), dev(b)))
        want = a @ b
        assert (np.abs(got - want) <= 33 * 2.0 ** -52 * (np.abs(a) @ np.abs(b))).all()
    with pytest.raises(api.OdlInvalidArgument):
        api.matmul_f64(dev(a[0]), dev(rng.standard_normal((34, 45))))
    with pytest.raises(api.OdlInvalidArgument):  # a leading dimension shorter than the row
        api.lib().call("odl_hip_dgemm", 0, 0, 4, 4, 4, 8, 2, 8, 4, 8, 4, 1, 0, 0, 0, None)
    # K = 0: an empty sum is 0
    z = host(api.matmul_f64(dev(np.zeros((5, 0))), dev(np.zeros((0, 6)))))
    assert z.shape == (5, 6) and (z == 0).all()


@pytest.mark.parametrize("N,C,H,W,OC,KH,KW,s,p", [
    (2, 3, 7, 6, 4, 3, 3, 1, 1), (3, 4, 9, 9, 5, 3, 3, 2, 1), (2, 2, 8, 5, 3, 2, 3, 1, 0), (1, 1, 3, 3, 2, 2, 2, 1, 0),
    (2, 5, 6, 6, 7, 1, 1, 1, 0), (2, 16, 14, 14, 24, 3, 3, 1, 1), (3, 1, 28, 28, 32, 3, 3, 1, 1),
    (9, 8, 24, 20, 130, 3, 3, 1, 1),   # 4320 output pixels: the filter gradient's reduction in two runs, the second shorter
    (2, 3, 64, 64, 16, 6, 6, 2, 2),    # 6x6 window, stride 2, padding 2
])
def test_conv_float64_vs_the_double_oracle(api, o, N, C, H, W, OC, KH, KW, s, p):
    """The convolution operators on float64 tensors (products on the FP64 matrix cores) against the double form of the
    reference's loops: im2col bit for bit in both layouts, col2im and every product within K * 2^-52 * sum |a||b| per
    element (a fixed but different summation order), integer data bit for bit."""
    print("\n[case] conv float64", N, C, H, W, OC, KH, KW, s, p, flush=True)
    rng = np.random.default_rng(N + 10 * C + OC)
    OH, OW = (H + 2 * p - KH) // s + 1, (W + 2 * p - KW) // s + 1
    M, K = N * OH * OW, C * KH * KW
    x, gy = rng.standard_normal((N, C, H, W)), rng.standard_normal((N, OC, OH, OW))
    w, b = rng.standard_normal((OC, C, KH, KW)) * np.sqrt(2.0 / K), rng.standard_normal((OC,))
    eps = 2.0 ** -52
    # im2col / col2im, both layouts
    for to_matrix, shape in ((1, (M, K)), (0, (N, C, KH, KW, OH, OW))):
        col = np.empty(shape)
        assert o.orc_im2col_f64(x, N, C, H, W, KH, KW, s, s, p, p, to_matrix, col) == 0
        assert np.array_equal(host(api.im2col_f64(dev(x), (KH, KW), s, p, bool(to_matrix))), col)
        img = np.empty_like(x)
        assert o.orc_col2im_f64(col, N, C, H, W, KH, KW, s, s, p, p, to_matrix, img) == 0
        assert np.array_equal(host(api.col2im_f64(dev(col), x.shape, (KH, KW), s, p, bool(to_matrix))), img)
    col = np.empty((M, K))
    o.orc_im2col_f64(x, N, C, H, W, KH, KW, s, s, p, p, 1, col)
    # forward with and without a bias
    y = np.empty((N, OC, OH, OW))
    assert o.orc_conv2d_f64(x, w, b, N, C, H, W, OC, KH, KW, s, s, p, p, y) == 0
    by = (K * eps * (np.abs(col) @ np.abs(w.reshape(OC, K)).T) + eps * np.abs(b)).reshape(N, OH, OW, OC).transpose(0, 3, 1, 2)
    assert (np.abs(host(api.conv2d_f64(dev(x), dev(w), dev(b), s, p)) - y) <= by + 1e-300).all()
    assert (np.abs(host(api.conv2d_f64(dev(x), dev(w), None, s, p)) - (y - b[None, :, None, None])) <= by + 4 * eps * np.abs(y)).all()
    # backward: gy's buffer read as [M, OC]
    gxo, gwo, gbo = np.empty_like(x), np.empty_like(w), np.empty_like(b)
    assert o.orc_conv2d_backward_f64(gy, x, w, N, C, H, W, OC, KH, KW, s, s, p, p, gxo, gwo, gbo) == 0
    gx, gw, gb = (host(t) for t in api.conv2d_backward_f64(dev(gy), dev(x), dev(w), True, s, p))
    gy2d = gy.reshape(M, OC)
    bgw = M * eps * (np.abs(gy2d).T @ np.abs(col)).reshape(w.shape)
    assert (np.abs(gw - gwo) <= bgw + 1e-300).all()
    bcol = OC * eps * (np.abs(gy2d) @ np.abs(w.reshape(OC, K)))
    bgx = np.empty_like(x)
    o.orc_col2im_f64(bcol, N, C, H, W, KH, KW, s, s, p, p, 1, bgx)
    assert (np.abs(gx - gxo) <= bgx + KH * KW * eps * np.abs(gxo) + 1e-300).all()
    assert (np.abs(gb - gbo) <= N * OH * OW * eps * np.abs(gy).sum((0, 2, 3))).all()
    gx2, gw2, gb2 = api.conv2d_backward_f64(dev(gy), dev(x), dev(w), False, s, p)
    assert gb2 is None and np.array_equal(host(gw2), gw) and np.array_equal(host(gx2), gx)
    # integers: every sum exact, whatever its order
    xi, wi = rng.integers(-8, 8, x.shape).astype(np.float64), rng.integers(-4, 4, w.shape).astype(np.float64)
    bi, gi = rng.integers(-4, 4, b.shape).astype(np.float64), rng.integers(-4, 4, gy.shape).astype(np.float64)
    assert o.orc_conv2d_f64(xi, wi, bi, N, C, H, W, OC, KH, KW, s, s, p, p, y) == 0
    assert np.array_equal(host(api.conv2d_f64(dev(xi), dev(wi), dev(bi), s, p)), y)
    assert o.orc_conv2d_backward_f64(gi, xi, wi, N, C, H, W, OC, KH, KW, s, s, p, p, gxo, gwo, gbo) == 0
    for got, want in zip(api.conv2d_backward_f64(dev(gi), dev(xi), dev(wi), True, s, p), (gxo, gwo, gbo)):
        assert np.array_equal(host(got), want)


def test_conv_float64_argument_errors(api):
    x, w = dev(np.zeros((1, 2, 4, 4))), dev(np.zeros((3, 2, 3, 3)))
    with pytest.raises(api.OdlInvalidArgument):  # the window does not fit
        api.conv2d_f64(dev(np.zeros((1, 2, 2, 2))), w)
    with pytest.raises(api.OdlInvalidArgument):  # a float32 operand
        api.conv2d_f64(x, dev(np.zeros((3, 2, 3, 3), f32)))
    with pytest.raises(api.OdlInvalidArgument):  # too small a workspace
        api.lib().call("odl_hip_conv2d_f64", x.data_ptr(), w.data_ptr(), None, 1, 2, 4, 4, 3, 3, 3, 1, 1, 0, 0, x.data_ptr(),
                       x.data_ptr(), 8, None)
    assert api.lib().query("odl_hip_conv2d_f64_workspace_bytes", 1, 2, 4, 4, 3, 3, 3, 1, 1, 0, 0) == 4 * 18 * 8 + (-4 * 18 * 8) % 256


def test_transpose(api, o):
    rng = np.random.default_rng(3)
    # tiles of 64x64: ragged edges on both sides, whole tiles read and written 16 bytes per lane, batches, single rows
    for shape in ((37, 53), (2, 3, 5), (128, 64), (1, 7), (3, 132, 68), (200, 260), (5, 64, 192), (130, 1), (257, 129),
                  (2, 4, 1000)):
        x = rng.standard_normal(shape, dtype=f32)
        want = np.empty(shape[:-2] + (shape[-1], shape[-2]), f32)
        o.orc_transpose(x, want, int(np.prod(shape[:-2])) if len(shape) > 2 else 1, shape[-2], shape[-1])
        assert np.array_equal(host(api.transpose(dev(x))), want)


# -------------------------------------------------------------------------------------- convolution
CONV_CASES = {"convA": ((1, 1), (1, 1)), "convB": ((2, 2), (1, 1)), "convC": ((1, 1), (0, 0)),
              "convD": ((2, 1), (0, 2)), "convE": ((1, 1), (0, 0))}


def conv_bounds(x, w, gy, s, p, o):
    """Per-element 1e-5 |a_row||b_col| bounds of the three conv GEMMs, built from the oracle's col matrix."""
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    OH, OW = gy.shape[2], gy.shape[3]
    M, K = N * OH * OW, C * KH * KW
    col = np.empty((M, K), f32)
    o.orc_im2col(x, N, C, H, W, KH, KW, s[0], s[1], p[0], p[1], 1, col)
    w2d = w.reshape(OC, K)
    gy2d = gy.reshape(M, OC)  # the reference's reinterpretation: same buffer, no permutation
    by = gemm_bound(col, w2d.T).reshape(N, OH, OW, OC).transpose(0, 3, 1, 2)
    bgw = gemm_bound(gy2d.T, col).reshape(w.shape)
    # gx sums up to KH*KW entries of gx_col: bound each by the largest gx_col bound of its row block
    bcol = gemm_bound(gy2d, w2d)
    bgx = np.empty((M, K), f32)
    bgx[:] = bcol
    gxb = np.empty_like(x)
    o.orc_col2im(np.ascontiguousarray(bgx), N, C, H, W, KH, KW, s[0], s[1], p[0], p[1], 1, gxb)
    return by, bgw, gxb


@pytest.mark.parametrize("name", sorted(CONV_CASES))
def test_conv_fixtures_from_the_compiled_reference(api, o, name):
    print("\n[case] conv fixture", name, flush=True)
    s, p = CONV_CASES[name]
    x, w, gy = G[f"{name}_x"], G[f"{name}_w"], G[f"{name}_gy"]
    b = G[f"{name}_b"] if f"{name}_b" in G else None
    by, bgw, bgx = conv_bounds(x, w, gy, s, p, o)
    y = host(api.conv2d(dev(x), dev(w), dev(b) if b is not None else None, s, p))
    assert (np.abs(y - G[f"{name}_y"]) <= by + 1e-6).all()
    gx, gw, gb = api.conv2d_backward(dev(gy), dev(x), dev(w), b is not None, s, p)
    assert (np.abs(host(gw) - G[f"{name}_gw"]) <= bgw + 1e-6).all()
    assert (np.abs(host(gx) - G[f"{name}_gx"]) <= bgx + 1e-6).all()
    if b is not None:
        n_terms = gy.size / gy.shape[1]
        assert (np.abs(host(gb) - G[f"{name}_gb"]) <= 1e-5 * np.sqrt(n_terms) *
                np.linalg.norm(gy.transpose(1, 0, 2, 3).reshape(gy.shape[1], -1), axis=1) + 1e-6).all()
    # data movement is exact
    KH, KW = w.shape[2], w.shape[3]
    assert np.array_equal(host(api.im2col(dev(x), (KH, KW), s, p, True)), G[f"{name}_col"])
    assert np.array_equal(host(api.im2col(dev(x), (KH, KW), s, p, False)), G[f"{name}_col6"])
    assert np.array_equal(host(api.col2im(dev(G[f"{name}_gcol"]), x.shape, (KH, KW), s, p, True)), G[f"{name}_im"])
    assert np.array_equal(host(api.col2im(dev(G[f"{name}_gcol6"]), x.shape, (KH, KW), s, p, False)), G[f"{name}_im6"])


def test_conv_reference_unit_test_vectors(api):
    # tests/unit_test/operator/test_conv2d.cpp:21-117, test_conv2d_transpose_output.cpp:54-94
    x9 = dev(np.arange(1, 10, dtype=f32).reshape(1, 1, 3, 3))
    ones = dev(np.ones((1, 1, 2, 2), f32))
    assert host(api.conv2d(x9, ones, None, 1, 0)).ravel().tolist() == [12, 16, 24, 28]
    assert host(api.conv2d(x9, ones, None, 2, 0)).ravel().tolist() == [12]
    x4 = dev(np.arange(1, 5, dtype=f32).reshape(1, 1, 2, 2))
    assert host(api.conv2d(x4, ones, dev(np.array([1], f32)), 1, 0)).ravel().tolist() == [11]
    assert tuple(api.conv2d(x4, ones, None, 1, 1).shape) == (1, 1, 3, 3)
    w2 = dev(np.array([1, 1, 1, 1, 2, 2, 2, 2], f32).reshape(2, 1, 2, 2))
    assert host(api.conv2d(x9, w2, None, 1, 0)).ravel().tolist() == [12, 16, 24, 28, 24, 32, 48, 56]
    # the reinterpretation vector recorded from the compiled reference
    gy = dev(np.arange(1, 9, dtype=f32).reshape(1, 2, 2, 2))
    w = dev(np.arange(1, 9, dtype=f32).reshape(2, 1, 2, 2))
    _, gw, _ = api.conv2d_backward(gy, x9, w, False, 1, 0)
    assert host(gw).ravel().tolist() == [62, 78, 110, 126, 74, 94, 134, 154]
    with pytest.raises(api.OdlInvalidArgument):
        api.conv2d(x4, dev(np.ones((1, 2, 2, 2), f32)), None, 1, 0)  # channel mismatch
    with pytest.raises(api.OdlInvalidArgument):
        api.conv2d(x4, dev(np.ones((1, 1, 3, 3), f32)), None, 1, 0)  # no valid output


# Shapes chosen to reach every code path of the conv entry points: gathered-operand (implicit GEMM) forward needs
# C*KH*KW % 4 == 0, weight-grad needs OC % 4 == 0, input-grad needs stride 1 and OC % 16 == 0; everything else
# takes the explicit im2col / col2im path. Kernel sizes 3 and 1 are compiled in, others (5, 2x3) are generic;
# OC <= 64 uses the 64-row tile, larger OC the 128-row tile.
CONV_SEEDED = [
    # N, C, H, W, OC, KH, KW, s, p
    (2, 16, 14, 14, 24, 3, 3, 1, 1),   # fwd + wgrad implicit, dgrad explicit
    (3, 8, 13, 13, 12, 3, 3, 2, 1),    # stride 2
    (2, 1, 28, 28, 32, 3, 3, 1, 1),    # one input channel: the direct (one thread per pixel) kernels, all three
    (3, 1, 28, 28, 64, 3, 3, 1, 1),    # the reference's MNIST stem, 64 filters: eight channel groups per gy row
    (2, 3, 17, 19, 16, 3, 3, 1, 1),    # three channels, W != H, two channel groups
    (2, 1, 20, 20, 8, 5, 5, 1, 2),     # 5x5 window, a single channel group
    (2, 1, 15, 15, 16, 3, 3, 2, 1),    # direct kernels at stride 2: the input gradient skips taps between outputs
    (2, 3, 12, 12, 32, 3, 3, 2, 0),    # stride 2 without padding, last row and column outside every window
    (2, 1, 9, 9, 48, 3, 3, 1, 1),      # 48 filters: direct forward and input gradient, weight gradient by GEMM
    (300, 1, 28, 28, 32, 3, 3, 1, 1),  # more pixels than one pass of the weight-gradient grid: several rows a thread
    (2, 16, 12, 10, 32, 3, 3, 1, 1),   # all three implicit, 64-row tiles, W != H
    (1, 32, 9, 9, 144, 3, 3, 1, 1),    # all three implicit, 128-row tiles with a ragged second tile
    (2, 8, 11, 11, 16, 1, 1, 1, 0),    # 1x1
    (2, 4, 12, 12, 16, 5, 5, 1, 2),    # generic kernel size
    (2, 6, 10, 9, 16, 2, 3, 1, 1),     # rectangular kernel, K = 36
    (2, 16, 15, 15, 20, 3, 3, 2, 0),   # stride 2 without padding
    (5, 64, 7, 7, 48, 3, 3, 1, 1),     # more pixels than one tile column, C = 64
    (2, 3, 64, 64, 16, 6, 6, 2, 2),    # the detector's stem: 6x6, stride 2, pad 2, three channels (a row a workgroup, MFMA)
    (3, 3, 37, 45, 16, 6, 6, 2, 2),    # the same over odd extents: a ragged last pixel tile, rows and columns past the image
    (2, 32, 40, 40, 64, 3, 3, 2, 1),   # its down-sampling convolutions
    (2, 16, 15, 13, 32, 3, 3, 2, 1),   # stride 2 over odd extents
    (3, 8, 14, 14, 16, 3, 3, 2, 0),    # stride 2 without padding
    (1, 4, 2, 2, 16, 3, 3, 2, 1),      # a 2x2 image under a 3x3 window at stride 2
    (5, 130, 12, 12, 48, 3, 3, 2, 1),  # stride 2, more input channels than two row tiles hold
    (2, 64, 20, 20, 128, 1, 1, 1, 0),  # its 1x1 bottleneck convolutions
    (3, 48, 9, 30, 33, 3, 3, 1, 1),    # LDS-patch forward with a ragged filter tile; three channel slabs
    (1, 16, 1, 1, 80, 3, 3, 1, 1),     # a single pixel: every tap row but the centre falls outside the image
    (2, 32, 3, 100, 16, 3, 3, 1, 1),   # the widest rows the LDS patch holds, two patch positions per thread
    (7, 16, 5, 6, 64, 3, 3, 1, 1),     # tiles that start and end in the middle of an image; 64 gradient channels
    (3, 16, 8, 8, 24, 3, 3, 1, 1),     # W a multiple of 4: the LDS patch is staged with 16-byte row loads
    (2, 48, 6, 28, 40, 3, 3, 1, 1),    # the same over three channel slabs and rows shared between tiles
    (3, 1, 12, 10, 16, 3, 3, 1, 1),    # one channel, 3x3/s1/p1: the one-pass backward, 16 filters, W != H
    (2, 1, 5, 7, 8, 3, 3, 1, 1),       # the same with 8 filters
    (1, 1, 1, 1, 32, 3, 3, 1, 1),      # a single pixel: only the centre tap meets it
    (700, 1, 6, 6, 32, 3, 3, 1, 1),    # more images than workgroups: several images a workgroup
    (130, 32, 14, 14, 64, 3, 3, 1, 1), # small images, few channels: the weight gradient with an image at a time in LDS
    (300, 16, 8, 6, 64, 3, 3, 1, 1),   # the same with more images than workgroups and W != H
    (128, 10, 6, 10, 96, 3, 3, 1, 1),  # the same with 90 gW columns: the last MFMA tile ragged, three row blocks
    (128, 12, 10, 10, 48, 3, 3, 1, 1), # image-resident forward: three filter tiles, the 27 steps of k in four uneven parts
    (140, 16, 12, 16, 32, 3, 3, 1, 1), # image-resident forward and input gradient with twelve full pixel tiles
    (3, 16, 8, 8, 40, 3, 3, 2, 1),     # stride 2 with channels in sixteens: several images per pixel tile, ragged filter tile
    (5, 32, 6, 28, 96, 3, 3, 2, 1),    # the same with 14-pixel output rows and two filter tiles
    (2, 48, 12, 52, 64, 3, 3, 2, 1),   # wide rows at stride 2
    (7, 16, 2, 2, 33, 3, 3, 2, 1),     # 2x2 images at stride 2: the top tap row always outside
    # more 3x3/s1/p1 layers with channels in groups of 32 and 64 or more filters: two filter tiles with a ragged second
    # one, three channel groups, rows wider than a pixel tile, a single pixel, tiles that cross image boundaries
    (3, 64, 10, 12, 128, 3, 3, 1, 1),
    (2, 32, 9, 70, 64, 3, 3, 1, 1),
    (4, 96, 6, 5, 192, 3, 3, 1, 1),
    (2, 32, 1, 1, 64, 3, 3, 1, 1),
    (5, 32, 7, 9, 68, 3, 3, 1, 1),
]


@pytest.mark.parametrize("N,C,H,W,OC,KH,KW,s,p", CONV_SEEDED)
def test_conv_vs_oracle_seeded(api, o, N, C, H, W, OC, KH, KW, s, p):
    print("\n[case] conv seeded", N, C, H, W, OC, KH, KW, s, p, flush=True)
    check_conv_case(api, o, N, C, H, W, OC, KH, KW, s, p)


@pytest.mark.parametrize("N,C,H,W,OC,KH,KW,s,p", [c for c in CONV_SEEDED if c[1] % 8 == 0])
def test_conv_tiled_forward_kernels_vs_oracle_seeded(api, o, N, C, H, W, OC, KH, KW, s, p):
    # Small layers whose channels come in groups of eight take the small-problem forward kernel (operands straight from
    # global memory, K shared between the waves of a workgroup); with it switched off the same shapes reach the tiled
    # forward kernels that larger layers use (implicit GEMM with and without K slices, the 1x1 product, im2col + GEMM).
    print("\n[case] conv seeded, tiled forward", N, C, H, W, OC, KH, KW, s, p, flush=True)
    api.lib().call("odl_hip_set_conv_direct", 0)
    try:
        check_conv_case(api, o, N, C, H, W, OC, KH, KW, s, p)
    finally:
        api.lib().call("odl_hip_set_conv_direct", 1)


@pytest.mark.parametrize("N,C,H,W,OC,KH,KW,s,p",
                         [c for c in CONV_SEEDED if c[5:] == (3, 3, 1, 1) and (c[1] % 16 == 0 or c[4] % 16 == 0)])
def test_conv_lds_patch_kernel_vs_oracle_seeded(api, o, N, C, H, W, OC, KH, KW, s, p):
    # The kernel that keeps the input patch in LDS takes 3x3/s1/p1 layers whose channel count is a multiple of 16
    # (forward: input channels; input gradient: filters) once they fill the chip; a threshold of 0 workgroups sends the
    # small seeded shapes through it as well.
    print("\n[case] conv seeded, LDS patch", N, C, H, W, OC, flush=True)
    api.lib().call("odl_hip_set_conv_patch_min_workgroups", 0)
    api.lib().call("odl_hip_set_conv_direct", 0)  # (the small-problem kernel would take these forwards first)
    try:
        check_conv_case(api, o, N, C, H, W, OC, KH, KW, s, p)
    finally:
        api.lib().call("odl_hip_set_conv_patch_min_workgroups", -1)
        api.lib().call("odl_hip_set_conv_direct", 1)


def check_conv_case(api, o, N, C, H, W, OC, KH, KW, s, p):
    rng = np.random.default_rng(N * 100 + C + OC)
    x = rng.standard_normal((N, C, H, W), dtype=f32)
    w = (rng.standard_normal((OC, C, KH, KW), dtype=f32) * f32(np.sqrt(2.0 / (C * KH * KW)))).astype(f32)
    b = rng.standard_normal(OC, dtype=f32)
    OH, OW = (H + 2 * p - KH) // s + 1, (W + 2 * p - KW) // s + 1
    gy = rng.standard_normal((N, OC, OH, OW), dtype=f32)
    yo, gxo, gwo, gbo = np.empty((N, OC, OH, OW), f32), np.empty_like(x), np.empty_like(w), np.empty_like(b)
    assert o.orc_conv2d(x, w, b, N, C, H, W, OC, KH, KW, s, s, p, p, yo) == 0
    assert o.orc_conv2d_backward(gy, x, w, N, C, H, W, OC, KH, KW, s, s, p, p, gxo, gwo, gbo) == 0
    by, bgw, bgx = conv_bounds(x, w, gy, (s, s), (p, p), o)
    assert (np.abs(host(api.conv2d(dev(x), dev(w), dev(b), s, p)) - yo) <= by + 1e-6).all()
    assert (np.abs(host(api.conv2d(dev(x), dev(w), None, s, p)) - (yo - b[None, :, None, None])) <= by + 2e-6).all()
    gx, gw, gb = api.conv2d_backward(dev(gy), dev(x), dev(w), True, s, p)
    assert (np.abs(host(gw) - gwo) <= bgw + 1e-6).all()
    assert (np.abs(host(gx) - gxo) <= bgx + 1e-6).all()
    # a sum of N*OH*OW terms per channel read as a dot product with ones: 1e-5 * |ones| * |gy_channel|
    gb_bound = 1e-5 * np.sqrt(N * OH * OW) * np.linalg.norm(gy.transpose(1, 0, 2, 3).reshape(OC, -1).astype(np.float64), axis=1)
    assert (np.abs(host(gb) - gbo) <= gb_bound + 1e-6).all()


@pytest.mark.parametrize("N,C", [(512, 10), (256, 10), (2048, 64), (7, 3), (1, 1), (100, 16), (33, 17), (1500, 33), (64, 48)])
def test_ce_loss_with_unit_gradient_in_one_launch_equals_the_two_calls(api, N, C):
    # the loss kernel that writes the gradient for an upstream gradient of 1 along: the loss is the float of the loss call
    # and the gradient the floats of the gradient call with gy = 1, bit for bit, for int32 and int64 labels
    print("\n[case] ce loss + unit gradient", N, C, flush=True)
    g = torch.Generator(device="cuda").manual_seed(N * 7 + C)
    x = torch.randn((N, C), device="cuda", generator=g) * 3.0
    for dt in (torch.int32, torch.int64):
        t = torch.randint(0, C, (N,), device="cuda", generator=g).to(dt)
        loss, bad, gx = api.softmax_cross_entropy_with_unit_grad(x, t)
        assert bad == 0
        want_loss = api.softmax_cross_entropy(x, t)
        assert np.float32(loss).tobytes() == np.float32(want_loss).tobytes()
        assert torch.equal(gx.view(torch.int32), api.softmax_cross_entropy_backward(x, t, 1.0).view(torch.int32))
    t_bad = torch.randint(0, C, (N,), device="cuda", generator=g).to(torch.int32)
    t_bad[N // 2] = C
    assert api.softmax_cross_entropy_with_unit_grad(x, t_bad)[1] == 1
    with pytest.raises(api.OdlInvalidArgument):
        api.softmax_cross_entropy_with_unit_grad(torch.zeros((4, 65), device="cuda"), torch.zeros(4, dtype=torch.int32, device="cuda"))


@pytest.mark.parametrize("N,C,H,W,OC,bias", [
    (256, 1, 28, 28, 32, True),   # the CNN's first layer under its pooling
    (3, 1, 12, 10, 16, False),
    (2, 3, 8, 6, 16, True),       # three input channels
    (5, 2, 2, 2, 48, True),       # one pooled pixel an image: every window cell meets the border
])
def test_conv_relu_pool_in_one_pass_equals_the_three_operators(api, N, C, H, W, OC, bias):
    # Conv2d + ReLU + MaxPool2d(2) of a first layer as one kernel: pooled values and window indices must be those of
    # conv2d_act(relu) followed by max_pool2d bit for bit, and the backward of the pooling and the ReLU taken from the
    # pooled tensor must give the floats of the one taken from the tensor that was pooled (zeros, negative zeros and the
    # signs of masked gradients included).
    print("\n[case] conv + relu + pool", N, C, H, W, OC, bias, flush=True)
    g = torch.Generator(device="cuda").manual_seed(N + C + H + OC)
    x = torch.randn((N, C, H, W), device="cuda", generator=g)
    w = torch.randn((OC, C, 3, 3), device="cuda", generator=g) * 0.3
    b = torch.randn((OC,), device="cuda", generator=g) if bias else None
    assert api.conv2d_relu_max_pool2d_ok(x.shape, w.shape)
    y = api.conv2d(x, w, b, 1, 1, activation="relu")
    want, want_idx = api.max_pool2d(y, 2, 2, 0)
    got, got_idx = api.conv2d_relu_max_pool2d(x, w, b)
    assert torch.equal(got, want) and torch.equal(got_idx, want_idx)
    assert torch.equal(api.conv2d_relu_max_pool2d(x, w, b, with_indices=False)[0], want)
    gy = torch.randn(want.shape, device="cuda", generator=g)
    gy.view(-1)[::7] = 0.0
    gy.view(-1)[3::11] = -0.0
    a = api.max_pool2d_backward_relu(gy, want_idx, y, 2, 2, 0)
    bq = api.max_pool2d_backward_relu_pooled(gy, got_idx, got, y.shape, 2, 2, 0)
    assert torch.equal(a.view(torch.int32), bq.view(torch.int32))  # the bit patterns: signed zeros count
    # the same with the indices kept as bytes (what the host layer's fused operator does): equal index values, equal floats
    got8, idx8 = api.conv2d_relu_max_pool2d(x, w, b, with_indices="bytes")
    assert torch.equal(got8, want) and torch.equal(idx8.to(torch.int64), want_idx)
    y8, i8 = api.max_pool2d_compact(y, 2, 2, 0)
    assert torch.equal(y8, want) and torch.equal(i8.to(torch.int64), want_idx)
    c8 = api.max_pool2d_backward_relu_pooled(gy, idx8, got8, y.shape, 2, 2, 0)
    assert torch.equal(a.view(torch.int32), c8.view(torch.int32))


@pytest.mark.parametrize("shape,k,st,p", [((3, 5, 9, 11), 3, 2, 1), ((2, 4, 12, 12), 3, 3, 0), ((2, 3, 10, 10), 5, 1, 2),
                                          ((1, 2, 7, 9), (2, 3), (2, 1), (0, 1))])
def test_max_pool_with_byte_indices_equals_the_eight_byte_ones(api, shape, k, st, p):
    g = torch.Generator(device="cuda").manual_seed(sum(shape))
    x = torch.randn(shape, device="cuda", generator=g)
    y, idx = api.max_pool2d(x, k, st, p)
    y8, idx8 = api.max_pool2d_compact(x, k, st, p)
    assert torch.equal(y, y8) and torch.equal(idx, idx8.to(torch.int64))


def test_conv_relu_pool_one_pass_is_offered_only_where_it_gives_the_same_bits(api):
    ok = api.conv2d_relu_max_pool2d_ok
    assert ok((4, 1, 28, 28), (32, 1, 3, 3))
    assert not ok((4, 1, 27, 28), (32, 1, 3, 3))            # an odd extent: the pooling drops a row
    assert not ok((4, 1, 28, 28), (24, 1, 3, 3))            # filters not in sixteens
    assert not ok((4, 32, 14, 14), (64, 32, 3, 3))          # many channels: the matrix kernels' layer
    assert not ok((4, 1, 28, 28), (32, 1, 3, 3), stride=2)
    assert not ok((4, 1, 28, 28), (32, 1, 3, 3), pool_kernel=3, pool_stride=3)
    assert not ok((4, 1, 28, 28), (32, 1, 5, 5), pad=2)
    x = torch.zeros((4, 32, 14, 14), device="cuda")
    w = torch.zeros((64, 32, 3, 3), device="cuda")
    with pytest.raises(api.OdlInvalidArgument):
        api.conv2d_relu_max_pool2d(x, w)
    with pytest.raises(api.OdlInvalidArgument):              # overlapping windows have no pooled-mask backward
        api.max_pool2d_backward_relu_pooled(torch.zeros((1, 1, 3, 3), device="cuda"),
                                            torch.zeros((1, 1, 3, 3), dtype=torch.int64, device="cuda"),
                                            torch.zeros((1, 1, 3, 3), device="cuda"), (1, 1, 7, 7), 3, 2, 0)


@pytest.mark.parametrize("N,C,H,W,OC", [
    (5, 1, 12, 10, 16),      # one input channel: the one-pass backward
    (130, 32, 14, 14, 64),   # small images, few channels: the image-resident weight gradient
    (3, 64, 8, 8, 64),       # the row-walking weight gradient with its side launch
    (2, 16, 12, 10, 32),     # the implicit products
])
def test_conv_backward_with_gradients_left_out(api, N, C, H, W, OC):
    # conv2d_backward writes only the gradients whose pointers are given (an operator whose input needs no gradient
    # passes none for gx; a layer without bias none for gb): every subset must give the values of the full call.
    # The kernels that compute several gradients in one pass skip the missing ones; the bias gradient alone takes
    # another kernel than beside the weight gradient, so it is compared to a few ulp of its sum.
    from origindl_amd import _lib
    rng = np.random.default_rng(N + C + OC)
    x, gy = rng.standard_normal((N, C, H, W), dtype=f32), rng.standard_normal((N, OC, H, W), dtype=f32)
    w = (rng.standard_normal((OC, C, 3, 3), dtype=f32) * f32(0.2)).astype(f32)
    dx, dgy, dw = dev(x), dev(gy), dev(w)
    L = _lib.lib()
    nb = L.query("odl_hip_conv2d_backward_workspace_bytes", N, C, H, W, OC, 3, 3, 1, 1, 1, 1)
    ws = torch.empty(max(nb, 16) // 4 + 4, dtype=torch.float32, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def run(want_gx, want_gw, want_gb):
        outs = [torch.full(shape, float("nan"), dtype=torch.float32, device="cuda") if want else None
                for shape, want in ((x.shape, want_gx), (w.shape, want_gw), ((OC,), want_gb))]
        ptr = [ctypes.c_void_p(t.data_ptr()) if t is not None else None for t in outs]
        print("[case] conv backward subset", N, C, H, W, OC, want_gx, want_gw, want_gb, flush=True)
        L.call("odl_hip_conv2d_backward", ctypes.c_void_p(dgy.data_ptr()), ctypes.c_void_p(dx.data_ptr()),
               ctypes.c_void_p(dw.data_ptr()), N, C, H, W, OC, 3, 3, 1, 1, 1, 1, ptr[0], ptr[1], ptr[2],
               ctypes.c_void_p(ws.data_ptr()), nb, st)
        return [host(t) if t is not None else None for t in outs]

    full = run(True, True, True)
    assert all(np.isfinite(t).all() for t in full)
    gb_tol = 1e-5 * np.sqrt(N * H * W) * np.linalg.norm(gy.transpose(1, 0, 2, 3).reshape(OC, -1).astype(np.float64), axis=1)
    for subset in ((True, False, False), (False, True, False), (False, False, True), (True, True, False),
                   (False, True, True), (True, False, True)):
        got = run(*subset)
        for name, g, f in zip(("gx", "gW", "gb"), got, full):
            if g is None:
                continue
            if name == "gb":
                assert (np.abs(g - f) <= gb_tol + 1e-6).all(), (subset, name)
            else:
                np.testing.assert_array_equal(g, f, err_msg="%s %s" % (subset, name))


@pytest.mark.parametrize("N,C,H,OC,s,p", [
    (32, 64, 56, 128, 1, 1),    # benchmark configuration C1
    (32, 128, 28, 256, 2, 1),   # benchmark configuration C2
    (256, 1, 28, 32, 1, 1),     # the CNN's first layer at its batch size: the direct kernels
    (256, 32, 14, 64, 1, 1),    # the CNN's second layer
])
def test_conv_full_size_properties(api, o, N, C, H, OC, s, p):
    # The benchmark's convolutions at full size. The oracle checks a sample of output pixels (each is one dot product of a
    # col row with a weight row); im2col/col2im adjointness and the bias-gradient identity hold at any size; the two
    # gradients are checked against float64 GEMMs over the reference's reinterpreted gy.
    print("\n[case] conv full size", N, C, H, OC, s, p, flush=True)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn((N, C, H, H), device="cuda", generator=g)
    w = torch.randn((OC, C, 3, 3), device="cuda", generator=g) * float(np.sqrt(2.0 / (C * 9)))
    b = torch.randn((OC,), device="cuda", generator=g)
    y = api.conv2d(x, w, b, s, p)
    OH = y.shape[2]
    gy = torch.randn(y.shape, device="cuda", generator=g)
    gx, gw, gb = api.conv2d_backward(gy, x, w, True, s, p)
    xh, wh, bh, yh = host(x), host(w), host(b), host(y)
    rng = np.random.default_rng(4)
    xp = np.pad(xh, ((0, 0), (0, 0), (p, p), (p, p)))
    for _ in range(40):
        n, oc, oh, ow = (int(rng.integers(0, d)) for d in (N, OC, OH, OH))
        win = xp[n, :, oh * s:oh * s + 3, ow * s:ow * s + 3].ravel()
        want = np.empty((1, 1), f32)
        o.orc_matmul(win.reshape(1, -1).copy(), wh[oc].reshape(-1, 1).copy(), want, 1, 1, win.size)
        want = f32(want[0, 0] + bh[oc])
        assert abs(yh[n, oc, oh, ow] - want) <= 1e-5 * np.linalg.norm(win) * np.linalg.norm(wh[oc]) + 1e-6
    # gb == gy.sum over (n, oh, ow)
    want_gb = host(gy).astype(np.float64).sum(axis=(0, 2, 3))
    np.testing.assert_allclose(host(gb), want_gb, atol=1e-5 * np.sqrt(N * OH * OH) * 80)
    # <im2col(x), c> == <x, col2im(c)>
    col = api.im2col(x, 3, s, p, True)
    c = torch.randn(col.shape, device="cuda", generator=g)
    lhs = float((col.double() * c.double()).sum())
    rhs = float((x.double() * api.col2im(c, x.shape, 3, s, p, True).double()).sum())
    assert abs(lhs - rhs) <= 1e-6 * float(col.double().norm() * c.double().norm())
    # gW and gx against float64 GEMMs on the reference's reinterpreted gy
    M, K = N * OH * OH, C * 9
    gy2d = gy.reshape(M, OC).double()
    want_gw = (gy2d.t() @ col.double()).reshape(w.shape)
    bnd = 1e-5 * torch.outer(gy2d.norm(dim=0), col.double().norm(dim=0)).reshape(w.shape)
    assert bool(((gw.double() - want_gw).abs() <= bnd).all())
    want_gx = api.col2im((gy2d @ w.reshape(OC, K).double()).float(), x.shape, 3, s, p, True)
    assert float((gx - want_gx).abs().max()) <= 9 * 1e-5 * float(gy2d.norm(dim=1).max() * w.reshape(OC, K).norm(dim=0).max())
    # The same two gradients against the oracle alone, on samples (nothing of the device's own output enters): three rows
    # gW[oc] = gy2d^T[oc, :] . col with col from the oracle's im2col and the reference's k-ascending sums
    # (conv2d.cpp:548-562), and twenty pixels of gx = col2im(gy2d . W2d) (conv2d.cpp:584-596), each from the nine col rows
    # that reach it, folded by the oracle's col2im on that image alone.
    gyh, gwh, gxh = host(gy), host(gw), host(gx)
    gy2dh, w2d = gyh.reshape(M, OC), np.ascontiguousarray(wh.reshape(OC, K))
    colh = np.empty((M, K), f32)
    assert o.orc_im2col(xh, N, C, H, H, 3, 3, s, s, p, p, 1, colh) == 0
    col_norm = np.linalg.norm(colh.astype(np.float64), axis=0)
    for oc in sorted({0, OC - 1, int(rng.integers(0, OC))}):
        row = np.ascontiguousarray(gy2dh[:, oc]).reshape(1, M)
        want = np.empty((1, K), f32)
        o.orc_matmul(row, colh, want, 1, K, M)
        bound = 1e-5 * np.linalg.norm(row.astype(np.float64)) * col_norm + 1e-7
        assert (np.abs(gwh[oc].reshape(-1) - want[0]) <= bound).all(), ("gW row", oc)
    del colh
    wcol_norm = np.linalg.norm(w2d.astype(np.float64), axis=0)
    for _ in range(20):
        n, c, h, wx = (int(rng.integers(0, d)) for d in (N, C, H, H))
        gcol = np.zeros((OH * OH, K), f32)
        bound = 1e-6
        for kh in range(3):
            for kw in range(3):
                hh, ww = h + p - kh, wx + p - kw
                if hh % s or ww % s or not (0 <= hh // s < OH and 0 <= ww // s < OH):
                    continue
                m = (hh // s) * OH + ww // s
                out = np.empty((1, K), f32)
                o.orc_matmul(np.ascontiguousarray(gy2dh[n * OH * OH + m]).reshape(1, OC), w2d, out, 1, K, OC)
                gcol[m] = out[0]
                bound += 1e-5 * np.linalg.norm(gy2dh[n * OH * OH + m].astype(np.float64)) * wcol_norm[(c * 3 + kh) * 3 + kw]
        img = np.empty((1, C, H, H), f32)
        assert o.orc_col2im(gcol, 1, C, H, H, 3, 3, s, s, p, p, 1, img) == 0
        assert abs(gxh[n, c, h, wx] - img[0, c, h, wx]) <= bound, ("gx pixel", n, c, h, wx)


# ------------------------------------------------------------------------------- reductions / broadcast
def sum_bound(v, axis_len):
    return 1e-5 * np.sqrt(axis_len) * np.linalg.norm(v.astype(np.float64)) + 1e-30


@pytest.mark.parametrize("shape,axis", [((512, 1000), 0), ((512, 10), 0), ((64, 33), 1), ((3, 4, 5), 1),
                                        ((8, 300, 7), 1), ((5000, 3), 0), ((2, 70000), 1), ((1, 9), 0)])
def test_sum_axis_vs_oracle(api, o, shape, axis):
    rng = np.random.default_rng(sum(shape) + axis)
    x = rng.standard_normal(shape, dtype=f32)
    outer, inner = int(np.prod(shape[:axis])), int(np.prod(shape[axis + 1:]))
    want = np.empty((outer, inner), f32)
    o.orc_sum_axis(x, outer, shape[axis], inner, want)
    got = host(api.sum(dev(x), axis)).reshape(outer, inner)
    xs = x.reshape(outer, shape[axis], inner)
    bound = 1e-5 * np.sqrt(shape[axis]) * np.linalg.norm(xs.astype(np.float64), axis=1)
    assert (np.abs(got - want) <= bound + 1e-30).all()
    kd = api.sum(dev(x), axis, keepdim=True)
    assert tuple(kd.shape) == tuple(1 if i == axis else s for i, s in enumerate(shape))
    # max over the same axis is exact
    wmax = np.empty((outer, inner), f32)
    o.orc_max_axis(x, outer, shape[axis], inner, wmax)
    assert np.array_equal(host(api.max(dev(x), axis)).reshape(outer, inner), wmax)


def test_sum_all_and_max_all(api, o):
    rng = np.random.default_rng(12)
    for n in (1, 7, 4096, 1_000_003):
        x = rng.standard_normal(n, dtype=f32)
        assert abs(host(api.sum(dev(x)))[0] - o.orc_sum_all(x, n)) <= 2 * sum_bound(x, n)
        assert host(api.max(dev(x)))[0] == o.orc_max_all(x, n)
    assert tuple(api.sum(dev(rng.standard_normal((3, 4), dtype=f32)), -1, keepdim=True).shape) == (1, 1)
    with pytest.raises(api.OdlInvalidArgument):
        api.sum(dev(np.ones((2, 2), f32)), 2)
    # src/mat/origin/cpu/math/max.cpp:25-40, 58-117 on the shapes that split the scan over workgroups: a long axis over
    # few columns (chunks merged with integer atomics), whole tensors of a million elements; infinities, NaNs that the
    # comparison skips, a NaN first element (the whole-tensor maximum then stays NaN), all-negative and all -inf data
    for outer, axis, inner in ((1, 5000, 300), (3, 700, 40), (2, 4096, 1028), (1, 100000, 7), (1, 70, 512), (5, 1001, 260)):
        x = (rng.standard_normal((outer, axis, inner), dtype=f32) - 2.0).astype(f32)
        x[0, axis // 2, 0] = np.inf
        x[0, 3, inner - 1] = np.nan
        x[outer - 1, :, 1] = -np.inf
        want = np.empty((outer, inner), f32)
        o.orc_max_axis(x, outer, axis, inner, want)
        assert np.array_equal(host(api.max(dev(x), 1)).reshape(outer, inner), want), (outer, axis, inner)
    for n, edit in ((300_001, None), (1 << 20, "nan_first"), (70_000, "neg_inf"), (1_000_000, "nan_inside")):
        x = (rng.standard_normal(n, dtype=f32) - 5.0).astype(f32)
        if edit == "nan_first":
            x[0] = np.nan
        elif edit == "neg_inf":
            x[:] = -np.inf
        elif edit == "nan_inside":
            x[12345] = np.nan
        got, want = host(api.max(dev(x)))[0], o.orc_max_all(x, n)
        assert got == want or (np.isnan(got) and np.isnan(want)), (n, edit)


def test_sum_to_fixtures_and_errors(api, o):
    for name in sorted(k[:-3] for k in G.files if k.startswith("sumto") and k.endswith("_rc")):
        x, ts, rc = G[f"{name}_x"], tuple(int(v) for v in G[f"{name}_t"]), int(G[f"{name}_rc"])
        if rc == -2:
            with pytest.raises(api.OdlRuntimeError):  # test_sum_to.cpp:53-60
                api.sum_to(dev(x), ts)
        elif rc != 0:
            with pytest.raises((api.OdlInvalidArgument, api.OdlRuntimeError)):
                api.sum_to(dev(x), ts)
        else:
            got = host(api.sum_to(dev(x), ts)).ravel()
            np.testing.assert_allclose(got, G[f"{name}_y"], atol=1e-5 * np.sqrt(x.size) * np.abs(x).max(), rtol=0)
    # tests/unit_test/operator/test_sum_to.cpp:179-191 and the left-alignment probe ({2,2} -> {2} = row sums)
    assert host(api.sum_to(dev(np.arange(1, 9, dtype=f32).reshape(2, 2, 2)), (2, 1))).ravel().tolist() == [10, 26]
    assert host(api.sum_to(dev(np.array([[1, 2], [3, 4]], f32)), (2,))).tolist() == [3, 7]
    assert host(api.sum_to(dev(np.array([[1, 2], [3, 4]], f32)), (1, 1))).ravel().tolist() == [10]
    # MLP bias gradients [512,1000] -> [1,1000] and [512,10] -> [1,10] against the oracle
    rng = np.random.default_rng(13)
    for shape, ts in (((512, 1000), (1, 1000)), ((512, 10), (1, 10)), ((3, 4, 5), (1, 4)), ((6, 5, 4, 3), (6, 1, 4))):
        x = rng.standard_normal(shape, dtype=f32)
        want = np.empty(int(np.prod(ts)), f32)
        assert o.orc_sum_to(x, ol.shape_arr(shape), len(shape), ol.shape_arr(ts), len(ts), want) == 0
        got = host(api.sum_to(dev(x), ts)).ravel()
        # each output is a dot product of `terms` inputs with ones: 1e-5 * sqrt(terms) * |those inputs|, the norms taken
        # by summing the squares over the same index sets
        terms, sq = x.size / want.size, np.empty_like(want)
        assert o.orc_sum_to((x * x).astype(f32), ol.shape_arr(shape), len(shape), ol.shape_arr(ts), len(ts), sq) == 0
        assert (np.abs(got - want) <= 1e-5 * np.sqrt(terms) * np.sqrt(sq) + 1e-30).all()
    same = rng.standard_normal((4, 5), dtype=f32)
    assert np.array_equal(host(api.sum_to(dev(same), (4, 5))), same)


def test_bias_grad_large_column_reduction(api):
    # scaled bias-gradient shape used for the HBM roofline: [16384, 4096] -> [1, 4096]
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((16384, 4096), device="cuda", generator=g)
    got = api.sum_to(x, (1, 4096)).double()
    want = x.double().sum(dim=0, keepdim=True)
    assert float((got - want).abs().max()) <= 1e-5 * float(np.sqrt(16384)) * float(x.double().norm(dim=0).max())
    gy = torch.randn((32, 128, 56, 56), device="cuda", generator=g)
    gb = api.sum_nchw_channels(gy).double()
    assert float((gb - gy.double().sum(dim=(0, 2, 3))).abs().max()) <= 1e-5 * float(np.sqrt(32 * 56 * 56)) * 400
    # short channels (one workgroup each, a single launch), a plane that is not a multiple of four, and one image
    for shape in ((32, 256, 14, 14), (5, 64, 7, 9), (1, 3, 5, 5), (3, 70, 33, 31)):
        gy = torch.randn(shape, device="cuda", generator=g)
        gb = api.sum_nchw_channels(gy).double()
        want = gy.double().sum(dim=(0, 2, 3))
        n = shape[0] * shape[2] * shape[3]
        assert float((gb - want).abs().max()) <= 1e-5 * float(np.sqrt(n)) * 40, shape


def test_broadcast_fixtures(api):
    for name in ("bcastA", "bcastB", "bcastC"):
        x, ds = G[f"{name}_x"], tuple(int(v) for v in G[f"{name}_d"])
        assert np.array_equal(host(api.broadcast_to(dev(x), ds)), G[f"{name}_y"])
        if int(G[f"{name}_rc"]) == 0:  # BroadcastTo::backward = left-aligned sum_to
            got = host(api.sum_to(dev(G[f"{name}_g"]), x.shape))
            np.testing.assert_allclose(got, G[f"{name}_gx"], atol=1e-5)
    x = np.arange(3, dtype=f32).reshape(3, 1)
    assert np.array_equal(host(api.broadcast_to(dev(x), (2, 3, 4))), np.broadcast_to(x, (2, 3, 4)))
    # src/mat/origin/cpu/math/broadcast.cpp (right-aligned, extent 1 repeats): rows, columns, scalars, repeated and copied
    # dimensions in turn, innermost extents that are and are not multiples of four
    rng = np.random.default_rng(5)
    for ss, ds in (((1, 4096), (33, 4096)), ((64, 1), (64, 100)), ((1,), (7, 12)), ((3, 1, 8), (5, 3, 6, 8)),
                   ((2, 1, 3, 1, 4), (2, 5, 3, 7, 4)), ((6, 10), (4, 6, 10)), ((5, 1, 1), (5, 4, 8)), ((1, 7), (9, 7)),
                   ((4, 1, 2), (4, 6, 2)), ((), (3, 4))):
        x = rng.standard_normal(ss, dtype=f32)
        assert np.array_equal(host(api.broadcast_to(dev(x), ds)), np.broadcast_to(x, ds)), (ss, ds)


# ------------------------------------------------------------------------------------ softmax / CE
def test_softmax_and_ce_vs_oracle(api, o):
    rng = np.random.default_rng(14)
    for N, C, is64 in ((512, 10, 1), (256, 10, 0), (7, 1000, 1), (1, 3, 0), (300, 65, 1), (33, 128, 0), (9, 400, 1),
                       (5, 2000, 0), (130, 256, 1), (67, 516, 0), (31, 1028, 1), (19, 2048, 0), (3, 2052, 1)):
        x = (rng.standard_normal((N, C), dtype=f32) * 3).astype(f32)
        t = rng.integers(0, C, size=N).astype(np.int64 if is64 else np.int32)
        p, gx, loss = np.empty_like(x), np.empty_like(x), np.zeros(1, f32)
        o.orc_softmax(x, N, C, 1, p)
        assert o.orc_softmax_ce_loss(x, t, is64, N, C, loss) == 0
        assert o.orc_softmax_ce_grad(x, t, is64, N, C, 1.0, gx) == 0
        # the denominator is a sum of C exponentials taken in another order than the reference's loop: about
        # sqrt(C) * 2^-24 relative (2.7e-6 at C = 2048), well inside the 1e-5 of the reference's strict tolerance
        np.testing.assert_allclose(host(api.softmax(dev(x))), p, atol=1e-6, rtol=4e-6)
        got_loss = api.softmax_cross_entropy(dev(x), dev(t))
        assert abs(got_loss - loss[0]) <= 1e-4 * abs(loss[0]) + 1e-6
        np.testing.assert_allclose(host(api.softmax_cross_entropy_backward(dev(x), dev(t), 1.0)), gx, atol=1e-6, rtol=0)
        sel, oh = np.empty(N, f32), np.empty((N, C), f32)
        o.orc_gather(p, t, is64, N, C, sel)
        o.orc_one_hot(t, is64, N, C, oh)
        assert np.array_equal(host(api.gather(dev(p), dev(t))), sel)  # integer indexing: bit-exact
        assert np.array_equal(host(api.one_hot(dev(t), C)), oh)
    # one_hot in 16-byte quads: labels at every position of a quad, out of range on both sides (gather.cpp:134 leaves the
    # row zero), 32- and 64-bit labels
    for C in (4, 8, 36):
        for dt in (np.int32, np.int64):
            t = np.concatenate([np.arange(-2, C + 3), rng.integers(0, C, 50)]).astype(dt)
            oh = np.empty((t.size, C), f32)
            o.orc_one_hot(t, int(dt is np.int64), t.size, C, oh)
            assert np.array_equal(host(api.one_hot(dev(t), C)), oh), (C, dt)
    x3 = rng.standard_normal((4, 6, 5), dtype=f32)
    p3 = np.empty_like(x3)
    o.orc_softmax(x3, 4, 6, 5, p3)
    np.testing.assert_allclose(host(api.softmax(dev(x3), 1)), p3, atol=1e-6, rtol=0)
    x4 = rng.standard_normal((3, 70, 9, 11), dtype=f32)  # a channel axis longer than the unrolled stretch of the scan
    p4 = np.empty_like(x4)
    o.orc_softmax(x4, 3, 70, 99, p4)
    np.testing.assert_allclose(host(api.softmax(dev(x4), 1)), p4, atol=1e-6, rtol=2e-6)


def test_ce_reference_unit_test_vectors_and_errors(api):
    # tests/unit_test/operator/test_softmax_cross_entropy.cpp:71-83, 131-161, 227-234
    loss = api.softmax_cross_entropy(dev(np.ones((1, 3), f32)), dev(np.array([1], np.int32)))
    assert abs(loss - np.log(3.0)) < 1e-6
    x = np.array([[1, 2, 3]], f32)
    gx = host(api.softmax_cross_entropy_backward(dev(x), dev(np.array([2], np.int32))))
    e = np.exp(x.astype(np.float64) - 3)
    np.testing.assert_allclose(gx, e / e.sum() - np.array([[0, 0, 1]]), atol=1e-6)
    with pytest.raises(api.OdlInvalidArgument):
        api.softmax_cross_entropy(dev(x), dev(np.array([3], np.int32)))
    with pytest.raises(api.OdlInvalidArgument):
        api.softmax_cross_entropy(dev(x), dev(np.array([0, 1], np.int32)))  # batch mismatch
    with pytest.raises(api.OdlInvalidArgument):
        api.gather(dev(G["oob_x"]), dev(G["oob_t"]))
    assert np.array_equal(host(api.one_hot(dev(G["oob_t"]), 3)), G["oob_onehot"])


def test_ce_fixtures(api):
    for name in ("ceA", "ceB", "ceC"):
        x, t = G[f"{name}_x"], G[f"{name}_t"]
        assert abs(api.softmax_cross_entropy(dev(x), dev(t)) - G[f"{name}_loss"][0]) <= 1e-4 * abs(G[f"{name}_loss"][0])
        np.testing.assert_allclose(host(api.softmax_cross_entropy_backward(dev(x), dev(t))), G[f"{name}_gx"], atol=1e-6)


def test_ce_grad_large_rows_sum_to_zero(api):
    # scaled shape used for the HBM roofline: [16384, 1000]; each row of softmax - one_hot sums to 0
    g = torch.Generator(device="cuda").manual_seed(6)
    x = torch.randn((16384, 1000), device="cuda", generator=g) * 2
    t = torch.randint(0, 1000, (16384,), device="cuda", generator=g)
    gx = api.softmax_cross_entropy_backward(x, t, 1.0)
    assert float(gx.double().sum(dim=1).abs().max()) < 1e-9 + 1e-6 / 16384 * 10
    want = (torch.softmax(x.double(), dim=1) - torch.nn.functional.one_hot(t, 1000)) / 16384
    assert float((gx.double() - want).abs().max()) < 1e-6 / 16384 * 20 + 1e-10


# ----------------------------------------------------------------------------------------- pooling
POOL_CASES = {"poolA": (2, 2, 2, 2, 0, 0), "poolB": (3, 3, 2, 2, 1, 1), "poolC": (5, 5, 1, 1, 2, 2),
              "poolD": (3, 2, 1, 2, 1, 0)}


@pytest.mark.parametrize("name", sorted(POOL_CASES))
def test_max_pool_fixtures_bit_exact(api, name):
    KH, KW, SH, SW, PH, PW = POOL_CASES[name]
    x = G[f"{name}_x"]
    y, idx = api.max_pool2d(dev(x), (KH, KW), (SH, SW), (PH, PW))
    assert np.array_equal(host(y), G[f"{name}_y"])
    assert np.array_equal(host(idx).view(np.uint64), G[f"{name}_idx"])
    gx = api.max_pool2d_backward(dev(G[f"{name}_gy"]), idx, x.shape, (KH, KW), (SH, SW), (PH, PW))
    assert np.array_equal(host(gx), G[f"{name}_gx"])


def test_max_pool_cnn_shapes_vs_oracle_bit_exact(api, o):
    # config 4's pools at reduced batch: [N,32,28,28] -> 14x14 and [N,64,14,14] -> 7x7, indices compared in full
    rng = np.random.default_rng(15)
    for N, C, H in ((8, 32, 28), (8, 64, 14)):
        x = np.maximum(rng.standard_normal((N, C, H, H), dtype=f32), 0)  # post-ReLU: many exact ties at 0
        y, idx = np.empty((N, C, H // 2, H // 2), f32), np.empty((N, C, H // 2, H // 2), np.uint64)
        assert o.orc_max_pool2d(x, N, C, H, H, 2, 2, 2, 2, 0, 0, y, idx) == 0
        gy = rng.standard_normal(y.shape, dtype=f32)
        gx = np.empty_like(x)
        assert o.orc_max_pool2d_backward(gy, idx, N, C, H, H, 2, 2, 2, 2, 0, 0, gx) == 0
        yd, idxd = api.max_pool2d(dev(x), 2, 2, 0)
        assert np.array_equal(host(yd), y) and np.array_equal(host(idxd).view(np.uint64), idx)
        assert np.array_equal(host(api.max_pool2d_backward(dev(gy), idxd, x.shape, 2, 2, 0)), gx)
    # windows that tile the image exactly take the output-side backward kernel (2x2/2 above, 3x3/3 here), everything
    # else the gather (an odd size whose last row and column no window covers; overlapping windows); gradients with
    # negative zeros keep their sign rules (0.f + -0.f = +0.f in both)
    for N, C, H, W, K, S in ((3, 5, 9, 12, 3, 3), (2, 4, 9, 9, 2, 2), (2, 3, 8, 8, 3, 2), (1, 2, 6, 6, 2, 2)):
        x = np.maximum(rng.standard_normal((N, C, H, W), dtype=f32), 0)
        OH, OW = (H - K) // S + 1, (W - K) // S + 1
        y, idx = np.empty((N, C, OH, OW), f32), np.empty((N, C, OH, OW), np.uint64)
        assert o.orc_max_pool2d(x, N, C, H, W, K, K, S, S, 0, 0, y, idx) == 0
        gy = rng.standard_normal(y.shape, dtype=f32)
        gy.ravel()[::7] = -0.0
        gx = np.empty_like(x)
        assert o.orc_max_pool2d_backward(gy, idx, N, C, H, W, K, K, S, S, 0, 0, gx) == 0
        yd, idxd = api.max_pool2d(dev(x), K, S, 0)
        got = host(api.max_pool2d_backward(dev(gy), idxd, x.shape, K, S, 0))
        assert np.array_equal(got, gx) and np.array_equal(np.signbit(got), np.signbit(gx)), (N, C, H, W, K, S)
    # tests/unit_test/operator/test_max_pool2d.cpp:20-45
    y, _ = api.max_pool2d(dev(np.arange(1, 17, dtype=f32).reshape(1, 1, 4, 4)), 2, 2, 0)
    assert host(y).ravel().tolist() == [6, 8, 14, 16]


def test_max_pool_overlapping_padded_windows_staged_in_lds_bit_exact(api, o):
    # max_pool2d.cpp:40-224 with padding cells counted as 0.0 and first maximum on strict >: the kernels that keep whole
    # planes in LDS, over the overlapping windows with compile-time sizes (3x3/2, 3x3/1, 5x5/1) and run-time ones (4x4/2,
    # 3x2 windows), one and several planes per workgroup with a ragged last workgroup; a padded 2x2/2, which does not
    # overlap, stays with the plain kernels
    rng = np.random.default_rng(151)
    for N, C, H, W, KH, KW, S, P in ((2, 3, 13, 9, 3, 3, 2, 1), (1, 5, 10, 10, 5, 5, 1, 2), (2, 2, 7, 8, 3, 3, 1, 1),
                                     (3, 2, 9, 10, 4, 4, 2, 1), (2, 3, 8, 7, 3, 2, 1, 1), (3, 1, 6, 6, 2, 2, 2, 1),
                                     (9, 251, 6, 7, 3, 3, 2, 1), (5, 500, 5, 5, 5, 5, 1, 2)):
        x = np.maximum(rng.standard_normal((N, C, H, W), dtype=f32), -0.2).astype(f32)  # ties at the clamp, some below the padding's 0
        OH, OW = (H + 2 * P - KH) // S + 1, (W + 2 * P - KW) // S + 1
        y, idx = np.empty((N, C, OH, OW), f32), np.empty((N, C, OH, OW), np.uint64)
        assert o.orc_max_pool2d(x, N, C, H, W, KH, KW, S, S, P, P, y, idx) == 0
        gy = rng.standard_normal(y.shape, dtype=f32)
        gx = np.empty_like(x)
        assert o.orc_max_pool2d_backward(gy, idx, N, C, H, W, KH, KW, S, S, P, P, gx) == 0
        yd, idxd = api.max_pool2d(dev(x), (KH, KW), S, P)
        assert np.array_equal(host(yd), y) and np.array_equal(host(idxd).view(np.uint64), idx), (N, C, H, W, KH, KW, S, P)
        got = host(api.max_pool2d_backward(dev(gy), idxd, x.shape, (KH, KW), S, P))
        assert np.array_equal(got, gx), (N, C, H, W, KH, KW, S, P)


# ----------------------------------------------------------------------------------------- metrics
def test_argmax_and_accuracy_bit_exact(api, o):
    rng = np.random.default_rng(16)
    y = rng.integers(0, 4, size=(1000, 10)).astype(f32)  # ties everywhere
    t = rng.integers(0, 10, size=1000).astype(np.int32)
    am = np.empty(1000, np.int64)
    o.orc_argmax_rows(y, 1000, 10, am)
    assert np.array_equal(host(api.argmax_rows(dev(y))), am)
    assert api.accuracy(dev(y), dev(t)) == o.orc_accuracy(y, t, 1000, 10)
    # wide rows take a wave per row: ties at every distance, a NaN at the head of a row (src/utils/metrics.cpp:42-53 never
    # finds anything greater than it: index 0), NaNs and infinities further in, widths around the multiples of 64
    for N, C in ((300, 32), (257, 63), (129, 64), (100, 65), (64, 1000), (5, 4097), (37, 256), (9, 1028), (3, 5000)):
        y = rng.integers(0, 3, size=(N, C)).astype(f32)
        y[rng.integers(0, N, N // 4), rng.integers(0, C, N // 4)] = np.nan
        y[rng.integers(0, N, N // 8), 0] = np.nan
        y[rng.integers(0, N, N // 8), rng.integers(0, C, N // 8)] = np.inf
        y[N - 1, :] = -np.inf
        t = rng.integers(0, C, size=N).astype(np.int32)
        am = np.empty(N, np.int64)
        o.orc_argmax_rows(y, N, C, am)
        assert np.array_equal(host(api.argmax_rows(dev(y))), am), (N, C)
        assert api.accuracy(dev(y), dev(t)) == o.orc_accuracy(y, t, N, C), (N, C)


# ------------------------------------------------------------------------------------- elementwise
def test_elementwise_vs_oracle_and_fixtures(api, o):
    a, b = G["ew_a"], G["ew_b"]
    for i, op in enumerate(("add", "sub", "mul", "div", "gt")):
        assert np.array_equal(host(api.binary(op, dev(a), dev(b))), G[f"ew_bin{i}"]), op
    for i, op in enumerate(("relu", "exp", "log", "neg", "square")):
        src = np.abs(a) + f32(0.1) if op == "log" else a
        got = host(api.unary(op, dev(src)))
        if op in ("exp", "log"):
            np.testing.assert_allclose(got, G[f"ew_un{i}"], rtol=2e-7, atol=1e-7)
        else:
            assert np.array_equal(got, G[f"ew_un{i}"]), op
    np.testing.assert_allclose(host(api.pow_scalar(dev(np.abs(a)), 0.5)), G["ew_pow05"], rtol=3e-7)
    rng = np.random.default_rng(17)
    big = rng.standard_normal(100003, dtype=f32)
    s = np.array([1.5], f32)
    want = np.empty_like(big)
    for i, op in enumerate(("add", "sub", "mul", "div", "gt")):
        o.orc_binary(i, big, big.size, s, 1, want)
        assert np.array_equal(host(api.binary(op, dev(big), dev(s))), want)
        o.orc_binary(i, s, 1, big, big.size, want)
        assert np.array_equal(host(api.binary(op, dev(s), dev(big))), want)
    with pytest.raises(api.OdlRuntimeError):
        api.binary("add", dev(big), dev(big[:5].copy()))
    acc = dev(big.copy())
    api.binary("add", acc, dev(big), out=acc)  # add_inplace: output aliases an input
    assert np.array_equal(host(acc), big + big)
    assert bool((api.fill((3, 5), 2.5) == 2.5).all())


def test_fused_optimizer_steps_match_the_op_by_op_sequence(api, o):
    """odl_hip_adam_step / odl_hip_sgd_step against (1) the same arithmetic issued as separate whole-tensor ops, the
    way the reference's optimizers issue it (src/optim/adam.cpp:52-113, sgd.cpp:18-75) — bit-identical — and
    (2) the oracle's elementwise ops on the CPU (powf of glibc vs the device: a few ulp on the denominator)."""
    rng = np.random.default_rng(23)
    n = 100003  # not a multiple of four: the scalar tail runs too
    p, g = rng.standard_normal(n, dtype=f32), rng.standard_normal(n, dtype=f32) * f32(0.1)
    m, v = rng.standard_normal(n, dtype=f32) * f32(0.05), np.abs(rng.standard_normal(n, dtype=f32)) * f32(0.01)
    b1, b2, eps, lr = f32(0.9), f32(0.999), f32(1e-8), f32(1e-3)
    for t in (1, 7):
        s1 = f32(1.0) / (f32(1.0) - f32(np.power(b1, f32(t))))
        s2 = f32(1.0) / (f32(1.0) - f32(np.power(b2, f32(t))))
        sc = lambda x: dev(np.array([x], f32))  # noqa: E731
        dp, dg, dm, dv = dev(p), dev(g), dev(m), dev(v)
        # separate ops
        m2 = api.binary("add", api.binary("mul", dm, sc(b1)), api.binary("mul", dg, sc(f32(1.0) - b1)))
        v2 = api.binary("add", api.binary("mul", dv, sc(b2)),
                        api.binary("mul", api.binary("mul", dg, dg), sc(f32(1.0) - b2)))
        den = api.binary("add", api.pow_scalar(api.binary("mul", v2, sc(s2)), 0.5), sc(eps))
        p2 = api.binary("sub", dp, api.binary("mul", api.binary("div", api.binary("mul", m2, sc(s1)), den), sc(lr)))
        # fused
        fm, fv = dev(m), dev(v)
        fp_ = api.adam_step(dp, dg, fm, fv, t, lr=lr, beta1=b1, beta2=b2, eps=eps)
        assert np.array_equal(host(fm), host(m2)) and np.array_equal(host(fv), host(v2))
        assert np.array_equal(host(fp_), host(p2))
        # CPU: the oracle's elementwise ops chained the same way
        def cpu(op, a, b):
            a, b = np.atleast_1d(np.asarray(a, f32)), np.atleast_1d(np.asarray(b, f32))
            out = np.empty(max(a.size, b.size), f32)
            assert o.orc_binary(op, a, a.size, b, b.size, out) == 0
            return out
        cm = cpu(0, cpu(2, m, b1), cpu(2, g, f32(1.0) - b1))
        cv = cpu(0, cpu(2, v, b2), cpu(2, cpu(2, g, g), f32(1.0) - b2))
        assert np.array_equal(host(fm), cm) and np.array_equal(host(fv), cv)
        cden = np.empty(n, f32)
        o.orc_pow_scalar(cpu(2, cv, s2), n, f32(0.5), cden)
        cp = cpu(1, p, cpu(2, cpu(3, cpu(2, cm, s1), cpu(0, cden, eps)), lr))
        np.testing.assert_allclose(host(fp_), cp, rtol=0, atol=1e-6)  # an ulp of p (|p| < 8) around a step of ~1e-3
    assert np.array_equal(host(api.sgd_step(dev(p), dev(g), 0.05)), p - g * f32(0.05))
    big = rng.standard_normal(4096, dtype=f32)
    dm0, dv0 = dev(np.zeros(4096, f32)), dev(np.zeros(4096, f32))
    out = host(api.adam_step(dev(big), dev(big), dm0, dv0, 1))
    # closed form at t = 1 from zero moments: m_hat = g and v_hat = g^2, so the step is lr * g / (|g| + eps)
    b64 = big.astype(np.float64)
    np.testing.assert_allclose(out, b64 - 1e-3 * b64 / (np.abs(b64) + 1e-8), rtol=0, atol=3e-7)


def test_multi_tensor_optimizer_steps_are_the_single_tensor_steps(api):
    """One launch over a list of parameters gives, tensor by tensor, the bits of the one-tensor entry points: sizes from
    one element to more than one workgroup's share, odd sizes (scalar tails), more tensors than one launch carries, and
    an empty tensor in the list."""
    import torch
    rng = np.random.default_rng(29)
    sizes = [1, 3, 10, 128, 1000, 1024, 1025, 784 * 100, 4097, 0, 7] + [33 + i for i in range(30)]
    p = [rng.standard_normal(n, dtype=f32) for n in sizes]
    g = [rng.standard_normal(n, dtype=f32) * f32(0.1) for n in sizes]
    m = [rng.standard_normal(n, dtype=f32) * f32(0.05) for n in sizes]
    v = [np.abs(rng.standard_normal(n, dtype=f32)) * f32(0.01) for n in sizes]
    ts = [1 + (i % 5) for i in range(len(sizes))]
    live = [i for i, n in enumerate(sizes) if n > 0]
    # Adam
    dm, dv = [dev(x) for x in m], [dev(x) for x in v]
    outs = api.adam_step_multi([dev(x) for x in p], [dev(x) for x in g], dm, dv, ts, lr=2e-3)
    for i in live:
        sm, sv = dev(m[i]), dev(v[i])
        want = api.adam_step(dev(p[i]), dev(g[i]), sm, sv, ts[i], lr=2e-3)
        assert np.array_equal(host(outs[i]), host(want)), sizes[i]
        assert np.array_equal(host(dm[i]), host(sm)) and np.array_equal(host(dv[i]), host(sv)), sizes[i]
    # the factors read from device memory for some entries, from the host arrays for the others
    fac = lambda t, b: f32(1.0) / (f32(1.0) - f32(np.power(f32(b), f32(t))))  # noqa: E731
    scales = [dev(np.array([fac(3, 0.9), fac(3, 0.999)], f32)) if i % 2 == 0 else None for i in range(len(sizes))]
    dm, dv = [dev(x) for x in m], [dev(x) for x in v]
    outs = api.adam_step_multi([dev(x) for x in p], [dev(x) for x in g], dm, dv, ts, device_scales=scales)
    for i in live[:12]:
        want = api.adam_step(dev(p[i]), dev(g[i]), dev(m[i]), dev(v[i]), 3 if i % 2 == 0 else ts[i])
        assert np.array_equal(host(outs[i]), host(want)), sizes[i]
    # unaligned operands: views one float into their buffers take the scalar path
    odd = [torch.empty(n + 1, dtype=torch.float32, device="cuda")[1:] for n in sizes]
    for t, x in zip(odd, p):
        t.copy_(torch.from_numpy(x))
    outs = api.sgd_step_multi(odd, [dev(x) for x in g], 0.05)
    for i in live:
        assert np.array_equal(host(outs[i]), p[i] - g[i] * f32(0.05)), sizes[i]
    outs = api.sgd_step_multi([dev(x) for x in p], [dev(x) for x in g], 0.05)
    for i in live:
        assert np.array_equal(host(outs[i]), host(api.sgd_step(dev(p[i]), dev(g[i]), 0.05))), sizes[i]
    # weight decay: grad += rate * param
    dg = [dev(x) for x in g]
    api.axpy_multi(1e-4, [dev(x) for x in p], dg)
    for i in live:
        assert np.array_equal(host(dg[i]), g[i] + f32(1e-4) * p[i]), sizes[i]
        assert np.array_equal(host(dg[i]), host(api.axpby(1.0, dev(g[i]), 1e-4, dev(p[i])))), sizes[i]
    # the hook and the step in one launch: the bits of the hook's launch followed by the step's, gradients included
    for unaligned in (False, True):
        def fresh(arrs):
            if not unaligned:
                return [dev(x) for x in arrs]
            views = [torch.empty(x.size + 1, dtype=torch.float32, device="cuda")[1:] for x in arrs]
            for t, x in zip(views, arrs):
                t.copy_(torch.from_numpy(x))
            return views
        dp, dg2, dm2, dv2 = fresh(p), fresh(g), fresh(m), fresh(v)
        api.axpy_multi(1e-4, dp, dg2)
        want = api.adam_step_multi(dp, dg2, dm2, dv2, ts, lr=2e-3)
        fp_, fg, fm, fv = fresh(p), fresh(g), fresh(m), fresh(v)
        got = api.adam_step_multi(fp_, fg, fm, fv, ts, lr=2e-3, weight_decay=1e-4)
        for i in live:
            assert np.array_equal(host(got[i]), host(want[i])), (sizes[i], unaligned)
            assert np.array_equal(host(fg[i]), host(dg2[i])) and np.array_equal(host(fm[i]), host(dm2[i])), sizes[i]
            assert np.array_equal(host(fv[i]), host(dv2[i])) and np.array_equal(host(fp_[i]), p[i]), sizes[i]
        dg2, fg = fresh(g), fresh(g)
        api.axpy_multi(1e-4, dp, dg2)
        want = api.sgd_step_multi(dp, dg2, 0.05)
        got = api.sgd_step_multi(fp_, fg, 0.05, weight_decay=1e-4)
        for i in live:
            assert np.array_equal(host(got[i]), host(want[i])) and np.array_equal(host(fg[i]), host(dg2[i])), sizes[i]
    with pytest.raises(api.OdlInvalidArgument):
        api.axpy_multi(0.5, [dev(p[3])], [dev(p[4])])
    # argument errors of the entry points themselves: a negative count, missing lists, a null tensor, a negative size
    import ctypes
    from origindl_amd import _lib
    L = _lib.lib()
    one = dev(p[4])
    ptrs, sizes = (ctypes.c_void_p * 1)(one.data_ptr()), (ctypes.c_int64 * 1)(one.numel())
    nulls, neg = (ctypes.c_void_p * 1)(None), (ctypes.c_int64 * 1)(-1)
    for args in ((-1, ctypes.c_float(1.0), ptrs, ptrs, sizes, None), (1, ctypes.c_float(1.0), None, ptrs, sizes, None),
                 (1, ctypes.c_float(1.0), nulls, ptrs, sizes, None), (1, ctypes.c_float(1.0), ptrs, ptrs, neg, None)):
        assert L.cdll.odl_hip_axpy_multi(*args) == _lib.ODL_ERR_INVALID_ARG, args[0]
    assert L.cdll.odl_hip_sgd_step_multi(1, ptrs, None, sizes, ctypes.c_float(0.1), ptrs, None) == _lib.ODL_ERR_INVALID_ARG
    assert L.cdll.odl_hip_adam_step_multi(1, ptrs, ptrs, ptrs, ptrs, sizes, ctypes.c_float(0.9), ctypes.c_float(0.999), None,
                                          None, None, ctypes.c_float(1e-8), ctypes.c_float(1e-3), ptrs,
                                          None) == _lib.ODL_ERR_INVALID_ARG  # no bias-correction factors at all
    assert L.cdll.odl_hip_axpy_multi(0, ctypes.c_float(1.0), None, None, None, None) == 0  # an empty list is a no-op


# ------------------------------------------------------------------ detector forward path (config 5's operators)
def test_sigmoid_silu_vs_oracle_and_fixtures(api, o):
    x = G["det_act_x"]
    for op, nm in ((6, "sigmoid"), (7, "silu")):
        np.testing.assert_allclose(host(api.unary(nm, dev(x))), G[f"det_{nm}"], rtol=3e-7, atol=1e-9)
    rng = np.random.default_rng(31)
    big = (rng.standard_normal(1 << 20, dtype=f32) * f32(5)).astype(f32)
    for op, nm in ((6, "sigmoid"), (7, "silu")):
        want = np.empty_like(big)
        o.orc_unary(op, big, big.size, want)
        np.testing.assert_allclose(host(api.unary(nm, dev(big))), want, rtol=3e-7, atol=1e-9)


def test_upsample_and_cat_bit_exact(api, o):
    xu = G["det_up_x"]
    assert np.array_equal(host(api.upsample(dev(xu), 2)), G["det_up22"])
    assert np.array_equal(host(api.upsample(dev(xu), (1, 3))), G["det_up13"])
    parts = [G[f"det_cat_in{i}"] for i in range(3)]
    assert np.array_equal(host(api.cat([dev(p) for p in parts], 1)), G["det_cat"])
    # the detector's own shapes: P5 -> P4 upsample and the concatenation that follows it
    rng = np.random.default_rng(32)
    a, b = rng.standard_normal((4, 128, 10, 10), dtype=f32), rng.standard_normal((4, 128, 20, 20), dtype=f32)
    up = host(api.upsample(dev(a), 2))
    want = np.empty((4, 128, 20, 20), f32)
    assert o.orc_upsample_nearest(a, 4, 128, 10, 10, 20, 20, 2, 2, want) == 0
    assert np.array_equal(up, want)
    cat = host(api.cat([dev(up), dev(b)], 1))
    assert np.array_equal(cat, np.concatenate([up, b], axis=1))
    # cpu/nn/upsample.cpp:62-63 (ih = oh / scale) over scales and row lengths that do and do not fill 16-byte quads
    for (N, C, H, W, sh, sw) in ((2, 3, 5, 6, 2, 2), (1, 2, 7, 4, 3, 1), (2, 2, 3, 4, 1, 3), (1, 1, 4, 3, 2, 4), (3, 1, 2, 5, 2, 2),
                                 (1, 4, 9, 2, 1, 2)):
        xs = rng.standard_normal((N, C, H, W), dtype=f32)
        want = np.empty((N, C, H * sh, W * sw), f32)
        assert o.orc_upsample_nearest(xs, N, C, H, W, H * sh, W * sw, sh, sw, want) == 0
        assert np.array_equal(host(api.upsample(dev(xs), (sh, sw))), want), (N, C, H, W, sh, sw)
    odd = [rng.standard_normal((3, c, 5), dtype=f32) for c in (3, 1, 7)]  # runs that are not multiples of four floats
    assert np.array_equal(host(api.cat([dev(p) for p in odd], 1)), np.concatenate(odd, axis=1))
    same = [rng.standard_normal((2, 4, 6), dtype=f32) for _ in range(3)]
    for dim in (0, 1, 2):
        assert np.array_equal(host(api.cat([dev(p) for p in same], dim)), np.concatenate(same, axis=dim)), dim
    with pytest.raises(api.OdlRuntimeError):
        api.cat([dev(odd[0]), dev(same[0])], 1)
    with pytest.raises(api.OdlInvalidArgument):  # an output row that would read past the input
        api.lib().call("odl_hip_upsample_nearest", None, 1, 1, 2, 2, 5, 4, 2, 2, None, None)


def test_compare_masks_activation_backward_split_and_upsample_backward(api):
    rng = np.random.default_rng(34)
    a = rng.integers(-3, 4, 100_003).astype(f32)
    b = rng.integers(-3, 4, 100_003).astype(f32)
    for nm, fn in (("gt", np.greater), ("eq", np.equal), ("ne", np.not_equal), ("lt", np.less), ("le", np.less_equal),
                   ("ge", np.greater_equal)):
        assert np.array_equal(host(api.binary(nm, dev(a), dev(b))), fn(a, b).astype(f32)), nm
        assert np.array_equal(host(api.binary(nm, dev(a), dev(np.array([1.0], f32)))), fn(a, f32(1)).astype(f32)), nm
    # activation gradients against the derivative in double precision: d sigmoid = y(1-y), d silu = s(1 + x(1-s))
    x = (rng.standard_normal(1 << 18) * 4).astype(f32)
    gy = rng.standard_normal(1 << 18).astype(f32)
    x64, g64 = x.astype(np.float64), gy.astype(np.float64)
    s64 = 1.0 / (1.0 + np.exp(-x64))
    y = host(api.unary("sigmoid", dev(x)))
    np.testing.assert_allclose(host(api.binary("sigmoid_backward", dev(gy), dev(y))), g64 * s64 * (1 - s64), rtol=2e-6,
                               atol=5e-7)  # 1 - y in single precision is off by up to an ulp of 1, times |gy| <= 5
    np.testing.assert_allclose(host(api.binary("silu_backward", dev(gy), dev(x))), g64 * s64 * (1 + x64 * (1 - s64)),
                               rtol=2e-6, atol=2e-7)
    # and against a centred difference of the forward kernel's own output at a few well-conditioned points
    pts = np.array([-2.0, -0.5, 0.25, 1.0, 3.0], f32)
    h = f32(1e-2)
    for nm in ("sigmoid", "silu"):
        hi, lo = host(api.unary(nm, dev(pts + h))), host(api.unary(nm, dev(pts - h)))
        arg = host(api.unary("sigmoid", dev(pts))) if nm == "sigmoid" else pts
        got = host(api.binary(nm + "_backward", dev(np.ones_like(pts)), dev(arg)))
        np.testing.assert_allclose(got, (hi.astype(np.float64) - lo) / (2 * float(h)), rtol=2e-3)
    # split undoes cat, along every axis and for ragged sizes
    t = rng.standard_normal((4, 11, 6), dtype=f32)
    for dim, sizes in ((0, [1, 3]), (1, [3, 1, 7]), (2, [2, 4])):
        pieces = api.split(dev(t), sizes, dim)
        want = np.split(t, np.cumsum(sizes)[:-1], axis=dim)
        assert all(np.array_equal(host(g), w) for g, w in zip(pieces, want)), dim
        assert np.array_equal(host(api.cat(pieces, dim)), t)
    with pytest.raises(api.OdlRuntimeError):
        api.split(dev(t), [3, 3], 1)
    # upsample backward sums each scale_h x scale_w block in row-major order (cpu/nn/upsample.cpp:100-130)
    g = rng.standard_normal((2, 5, 12, 18), dtype=f32)
    for sh, sw in ((2, 2), (3, 1), (1, 3)):
        H, W = 12 // sh, 18 // sw
        blocks = g.reshape(2, 5, H, sh, W, sw)
        want = np.zeros((2, 5, H, W), f32)
        for i in range(sh):
            for j in range(sw):
                want = want + blocks[:, :, :, i, :, j]
        assert np.array_equal(host(api.upsample_backward(dev(g), (2, 5, H, W), (sh, sw))), want), (sh, sw)
    ones = np.ones((1, 2, 8, 8), f32)  # the adjoint of a copy-to-4 is a sum of 4
    assert np.array_equal(host(api.upsample_backward(dev(ones), (1, 2, 4, 4), 2)), np.full((1, 2, 4, 4), 4, f32))


# ------------------------------------------------------------------ batch normalisation
BN_CASES = ("bnA", "bnB", "bnC", "bnD")


@pytest.mark.parametrize("name", BN_CASES)
def test_batch_norm_fixtures(api, name):
    # fixtures from the compiled reference: [N, C] and [N, C, H, W], training and evaluation, and the gradient.
    # Statistics are sums in a different (parallel) order than the reference's sequential loop: a few ulps of the mean
    # and variance, carried into y; everything downstream of given statistics is the same arithmetic.
    g = lambda k: G[f"{name}_{k}"]
    x, gamma, beta, rm, rv = (dev(g(k)) for k in ("x", "gamma", "beta", "rm", "rv"))
    for mode, training in (("train", True), ("eval", False)):
        y, mean, var, xn = api.batch_norm_forward(x, gamma, beta, rm, rv, training)
        tol = dict(rtol=2e-5, atol=2e-6) if training else dict(rtol=0, atol=0)
        for got, key in ((y, "y"), (mean, "mean"), (var, "var"), (xn, "xn")):
            np.testing.assert_allclose(host(got), g(f"{mode}_{key}"), err_msg=f"{mode} {key}", **tol)
        y_only = api.batch_norm_forward(x, gamma, beta, rm, rv, training, want_x_norm=False)[0]
        assert np.array_equal(host(y_only), host(y))
    gx, dg, db = api.batch_norm_backward(dev(g("gy")), gamma, dev(g("train_var")), dev(g("train_xn")))
    np.testing.assert_allclose(host(dg), g("dgamma"), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(host(db), g("dbeta"), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(host(gx), g("gx"), rtol=2e-5, atol=2e-5)


def test_batch_norm_vs_oracle_at_cnn_sizes(api, o):
    # the BatchNorm layers of the reference's conv_mnist example: [256, 32, 28, 28] and [256, 64, 14, 14]
    # (scaled down in N so that the scalar oracle stays quick), a plane that is not a multiple of four, and [N, C]
    rng = np.random.default_rng(41)
    for shape in ((32, 32, 28, 28), (32, 64, 14, 14), (5, 7, 5, 5), (512, 100)):
        N, C = shape[:2]
        P = int(np.prod(shape[2:])) if len(shape) == 4 else 1
        x = (rng.standard_normal(shape, dtype=f32) * f32(1.5) + f32(0.3)).astype(f32)
        gamma = (rng.random(C, dtype=f32) + f32(0.5)).astype(f32)
        beta = rng.standard_normal(C, dtype=f32)
        gy = rng.standard_normal(shape, dtype=f32)
        wy, wxn, wm, wv = np.empty(shape, f32), np.empty(shape, f32), np.empty(C, f32), np.empty(C, f32)
        zeros, ones = np.zeros(C, f32), np.ones(C, f32)
        assert o.orc_batch_norm_forward(x, gamma, beta, zeros, ones, 1, 1e-5, N, C, P, wy, wm, wv, wxn) == 0
        y, mean, var, xn = api.batch_norm_forward(dev(x), dev(gamma), dev(beta), dev(zeros), dev(ones), True)
        x64 = x.astype(np.float64).reshape(N, C, P)
        # against double precision: both sums are float sums over N*P terms, the parallel one the more accurate
        np.testing.assert_allclose(host(mean), x64.mean(axis=(0, 2)), rtol=0, atol=1e-6 * np.sqrt(N * P))
        np.testing.assert_allclose(host(var), x64.var(axis=(0, 2)), rtol=1e-6 * np.sqrt(N * P))
        np.testing.assert_allclose(host(mean), wm, rtol=0, atol=2e-6 * np.sqrt(N * P))
        np.testing.assert_allclose(host(var), wv, rtol=2e-6 * np.sqrt(N * P))
        np.testing.assert_allclose(host(y), wy, rtol=1e-4, atol=1e-4)
        # backward from the oracle's own saved statistics: the channel sums differ by summation order only
        wgx, wdg, wdb = np.empty(shape, f32), np.empty(C, f32), np.empty(C, f32)
        assert o.orc_batch_norm_backward(gy, gamma, wv, wxn, 1e-5, N, C, P, wgx, wdg, wdb) == 0
        gx, dg, db = api.batch_norm_backward(dev(gy), dev(gamma), dev(wv), dev(wxn))
        bound = 2e-6 * np.sqrt(N * P) * 4
        np.testing.assert_allclose(host(db), wdb, rtol=0, atol=bound * np.sqrt(N * P))
        np.testing.assert_allclose(host(dg), wdg, rtol=0, atol=bound * np.sqrt(N * P))
        np.testing.assert_allclose(host(gx), wgx, rtol=1e-4, atol=1e-5)
        # the backward that forms x_norm again from x and the statistics gives the same bits as the one reading the
        # saved x_norm of the same forward
        gx1, dg1, db1 = api.batch_norm_backward(dev(gy), dev(gamma), var, xn)
        gx2, dg2, db2 = api.batch_norm_backward_from_x(dev(gy), dev(x), dev(gamma), mean, var)
        assert all(np.array_equal(host(a), host(b)) for a, b in ((gx1, gx2), (dg1, dg2), (db1, db2))), shape
    # evaluation mode has no reduction: bit-exact against the oracle at any size
    x = rng.standard_normal((16, 64, 14, 14), dtype=f32)
    gamma, beta, rm = (rng.standard_normal(64, dtype=f32) for _ in range(3))
    rv = (rng.random(64, dtype=f32) + f32(0.1)).astype(f32)
    wy, wxn, wm, wv = np.empty_like(x), np.empty_like(x), np.empty(64, f32), np.empty(64, f32)
    assert o.orc_batch_norm_forward(x, gamma, beta, rm, rv, 0, 1e-5, 16, 64, 196, wy, wm, wv, wxn) == 0
    y, mean, var, xn = api.batch_norm_forward(dev(x), dev(gamma), dev(beta), dev(rm), dev(rv), False)
    assert np.array_equal(host(y), wy) and np.array_equal(host(xn), wxn)
    assert np.array_equal(host(mean), rm) and np.array_equal(host(var), rv)
    # the running-statistics update: momentum*running + (1 - momentum)*batch, products rounded first
    a, b = rng.standard_normal(1001, dtype=f32), rng.standard_normal(1001, dtype=f32)
    m = f32(0.1)
    assert np.array_equal(host(api.axpby(m, dev(a), f32(1.0) - m, dev(b))), m * a + (f32(1.0) - m) * b)
    with pytest.raises(api.OdlInvalidArgument):
        api.batch_norm_forward(dev(x), dev(gamma[:3].copy()), dev(beta), dev(rm), dev(rv), True)


@pytest.mark.parametrize("name", ["detA", "detB"])
def test_yolo_detect_fixtures(api, name):
    ag = G[f"{name}_anchor_grid"]
    b = dev(G["det_b"]) if name == "detA" else None
    got = host(api.yolo_detect_forward(dev(G["det_x"]), dev(G["det_w"]), b, dev(G["det_grid"]), dev(ag), 8.0, 3, 2))
    np.testing.assert_allclose(got, G[f"{name}_out"], rtol=2e-6, atol=1e-6)


def test_yolo_detect_at_detector_size_vs_oracle(api, o):
    # the P3 head of a width-0.25 YOLOv5: [4, 64, 40, 40] -> 3 anchors x 85
    rng = np.random.default_rng(33)
    N, C, H, W, A, NC = 4, 64, 40, 40, 3, 80
    CI = NC + 5
    x = rng.standard_normal((N, C, H, W), dtype=f32)
    w = (rng.standard_normal((A * CI, C, 1, 1), dtype=f32) * f32(0.2)).astype(f32)
    b = rng.standard_normal(A * CI, dtype=f32)
    gyy, gxx = np.meshgrid(np.arange(H), np.arange(W), indexing="ij")
    grid = np.broadcast_to(np.stack([gxx, gyy], -1).astype(f32) - f32(0.5), (1, A, H, W, 2)).copy()
    anchors = np.array([[10, 13], [16, 30], [33, 23]], f32)
    ag = np.broadcast_to(anchors.reshape(1, A, 1, 1, 2), (1, A, H, W, 2)).copy()
    want = np.empty((N, A * H * W, CI), f32)
    assert o.orc_yolo_detect_forward(x, w, b, grid, grid.size, ag, ag.size, H, W, N, C, H, W, 8.0, A, NC, want) == 0
    got = host(api.yolo_detect_forward(dev(x), dev(w), dev(b), dev(grid), dev(ag), 8.0, A, NC))
    # logits are sums of 64 products: the GEMM bound on the logit, carried through sigmoid (slope <= 1/4) and the box
    # transform (at most x2*stride, or x4*2s*anchor)
    np.testing.assert_allclose(got[..., 4:], want[..., 4:], rtol=0, atol=2e-6)
    np.testing.assert_allclose(got[..., :4], want[..., :4], rtol=2e-5, atol=2e-4)


@pytest.mark.parametrize("direct", [1, 0])
@pytest.mark.parametrize("N,C,H,OC,k,s,p", [
    (2, 16, 14, 24, 3, 1, 1),     # implicit forward, one pass
    (2, 1, 28, 32, 3, 1, 1),      # one input channel: the direct kernel
    (2, 5, 12, 24, 3, 1, 1),      # C*9 = 45, not a multiple of 4: explicit im2col + GEMM
    (64, 128, 14, 256, 3, 2, 1),  # strided, few tiles, long K: im2col + one product with the NCHW store in its epilogue
    (8, 128, 14, 256, 3, 2, 1),   # the same below a GFLOP: K slices summed by the reduction kernel
    (2, 64, 14, 128, 3, 1, 1),    # few tiles at stride 1: K slices summed by the reduction kernel
    (4, 64, 56, 128, 3, 1, 1),    # tile count just over a multiple of the CU count: tail pieces and their fix-up
    (2, 64, 20, 128, 1, 1, 0),    # 1x1
])
def test_conv_with_fused_activation_is_conv_then_activation(api, N, C, H, OC, k, s, p, direct):
    """direct = 1: the small shapes among these (channels in eights, under 1.6 GFLOP) go through the small-problem
    kernel; direct = 0: every shape takes the tiled kernel named beside it."""
    rng = np.random.default_rng(41)
    x = dev(rng.standard_normal((N, C, H, H), dtype=f32))
    w = dev((rng.standard_normal((OC, C, k, k), dtype=f32) * f32(np.sqrt(2.0 / (C * k * k)))).astype(f32))
    b = dev(rng.standard_normal(OC, dtype=f32))
    api.lib().call("odl_hip_set_conv_direct", direct)
    try:
        plain = api.conv2d(x, w, b, s, p)
        for act in ("silu", "relu"):
            assert np.array_equal(host(api.conv2d(x, w, b, s, p, activation=act)), host(api.unary(act, plain))), act
        with pytest.raises(api.OdlInvalidArgument):
            api.conv2d(x, w, b, s, p, activation="exp")
        # weights that do not change between calls: the filter copy made once gives the same bits as the per-call copy,
        # and shapes whose kernel reads the filter as it lies (with the tiled kernels: 1x1, few channels, the strided case
        # that goes through the col matrix) have no such copy
        small = C % 8 == 0 and 2 * N * ((H + 2 * p - k) // s + 1) ** 2 * C * k * k * OC <= 3 << 29
        packed = api.conv2d_pack_weights(x.shape, w, s, p)
        if direct and small:
            wp = np.zeros((-(-OC // 32) * 32, C, k * k), f32)
            wp[:OC] = host(w).reshape(OC, C, k * k)
            if k == 3 and p == 1:
                # 3x3 / padding 1: per (tile of 32 filters, channel pair, window row) a block [lane half][row][kw, one pad]
                want = np.zeros((wp.shape[0] // 32, C // 2, 3, 2, 32, 4), f32)
                want[..., :3] = wp.reshape(-1, 32, C // 2, 2, 3, 3).transpose(0, 2, 4, 3, 1, 5)
            else:
                # blocks of [lane half][row][4 channels] per (tile of 32 filters, tap, group of 8 channels)
                want = wp.reshape(-1, 32, C // 8, 2, 4, k * k).transpose(0, 5, 2, 3, 1, 4)
            assert packed is not None and packed.numel() == want.size
            assert np.array_equal(host(packed), want.reshape(-1))
        else:
            assert (packed is not None) == (k == 3 and C % 16 == 0 and not (s == 2 and N == 64))
            if packed is not None:
                assert np.array_equal(host(packed), host(w).reshape(OC, C, k * k).transpose(0, 2, 1).reshape(-1))
        for act in (None, "silu"):
            assert np.array_equal(host(api.conv2d(x, w, b, s, p, activation=act, packed=packed)),
                                  host(api.conv2d(x, w, b, s, p, activation=act))), act
    finally:
        api.lib().call("odl_hip_set_conv_direct", 1)


@pytest.mark.parametrize("N,C,H,W,OC,k,s,p", [
    (4, 64, 20, 20, 64, 1, 1, 0),     # K shared by four waves
    (4, 256, 10, 10, 128, 1, 1, 0),   # sixteen K shares
    (4, 32, 80, 80, 16, 1, 1, 0),     # half a filter tile, two pixel tiles a workgroup
    (2, 64, 40, 40, 255, 1, 1, 0),    # a detect head: the last filter tile one row short
    (4, 16, 160, 160, 32, 3, 2, 1),   # stride 2, two K shares of one channel group
    (4, 128, 10, 10, 128, 3, 1, 1),   # long K over few pixels
    (3, 24, 9, 13, 40, 3, 1, 1),      # three channel groups (no share divides them), ragged pixel and filter tiles
    (1, 8, 5, 5, 8, 3, 1, 1),         # a single pixel tile, a single group per tap
    (2, 16, 12, 12, 24, 5, 1, 2),     # 5x5: depth 4 over 25 taps x 2 groups
    (2, 32, 14, 10, 48, 3, 2, 0),     # stride 2 without padding
    (1, 1024, 4, 4, 64, 1, 1, 0),     # 128 channel groups: eight per share
    (2, 16, 7, 3, 32, 3, 1, 1),       # rows of three pixels: every window hangs over an edge or touches both
    (2, 8, 6, 9, 16, 3, 2, 1),        # stride 2 over an odd width: the last window hangs over the right edge
    (2, 8, 3, 2, 16, 3, 1, 1),        # rows of two pixels: the general kernel, not the three-floats-a-load one
    (1, 32, 1, 5, 16, 3, 1, 1),       # a single image row: the windows' outer rows lie in the padding
])
def test_conv_fused_into_channel_runs_equals_the_nodes_one_by_one(api, o, N, C, H, W, OC, k, s, p):
    """odl_hip_conv2d_fused with its input, output and residual each a run of channels of a wider tensor: the result
    must be, bit for bit, what the nodes give one after the other on tensors of their own — convolution (the same
    kernel, through odl_hip_conv2d), activation, add, and the copy into the concatenation — and must leave the rest of
    the wider output untouched. The convolution itself is held to the oracle by the seeded cases above."""
    print("\n[case] conv fused", N, C, H, W, OC, k, s, p, flush=True)
    rng = np.random.default_rng(C * 7 + OC)
    assert api.conv2d_fused_ok((N, C, H, W), (OC, C, k, k), s, p)
    OH, OW = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
    xbuf = dev(rng.standard_normal((N, C + 24, H, W), dtype=f32))
    rbuf = dev(rng.standard_normal((N, OC + 8, OH, OW), dtype=f32))
    ybuf0 = rng.standard_normal((N, OC + 40, OH, OW), dtype=f32)
    w = dev((rng.standard_normal((OC, C, k, k), dtype=f32) * f32(np.sqrt(2.0 / (C * k * k)))).astype(f32))
    b = dev(rng.standard_normal(OC, dtype=f32))
    xr, rr = xbuf[:, 16:16 + C], rbuf[:, 8:8 + OC]
    x, r = xr.contiguous(), rr.contiguous()
    packed = api.conv2d_pack_weights(x.shape, w, s, p)
    for act in (None, "silu", "relu"):
        for with_res in (False, True):
            for with_bias in (True, False):
                ybuf = dev(ybuf0)
                api.conv2d_fused(xr, w.shape, packed, b if with_bias else None, ybuf[:, 32:32 + OC], s, p, act,
                                 rr if with_res else None)
                step = api.conv2d(x, w, b if with_bias else None, s, p)
                if act:
                    step = api.unary(act, step)
                if with_res:
                    step = api.binary("add", r, step)
                want = ybuf0.copy()
                want[:, 32:32 + OC] = host(step)
                assert np.array_equal(host(ybuf), want), (act, with_res, with_bias)
    # dense operands (image strides 0) are the same call
    y = dev(np.zeros((N, OC, OH, OW), f32))
    api.conv2d_fused(x, w.shape, packed, b, y, s, p, "silu", r)
    assert np.array_equal(host(y), host(api.binary("add", r, api.unary("silu", api.conv2d(x, w, b, s, p)))))
    # against the oracle too, so that this test stands on its own
    yo = np.empty((N, OC, OH, OW), f32)
    assert o.orc_conv2d(host(x), host(w), host(b), N, C, H, W, OC, k, k, s, s, p, p, yo) == 0
    by, _, _ = conv_bounds(host(x), host(w), np.zeros((N, OC, OH, OW), f32), (s, s), (p, p), o)
    assert (np.abs(host(api.conv2d(x, w, b, s, p)) - yo) <= by + 1e-6).all()


def test_conv_fused_group_gives_each_member_the_floats_of_its_own_call(api):
    """The stage convolutions of a detect head as one launch: every member bit for bit what conv2d_fused gives it alone
    (K shares from 1 to 16, a last pixel tile that is ragged or lies wholly past the last pixel, inputs and outputs that
    are runs of wider tensors, a member without bias)."""
    rng = np.random.default_rng(77)
    for N, members, act in ((4, ((64, 40, 40, 255), (128, 20, 20, 255), (256, 10, 10, 255)), None),
                            (2, ((8, 7, 9, 33), (512, 3, 5, 64)), "silu"),
                            (1, ((16, 16, 16, 24), (32, 5, 5, 40), (64, 2, 2, 8), (128, 1, 1, 100)), "relu"),
                            (3, ((24, 11, 6, 70),), None)):
        xs, ws, pks, bs, ys, wants = [], [], [], [], [], []
        for i, (C, H, W, OC) in enumerate(members):
            xbuf = dev(rng.standard_normal((N, C + 8, H, W), dtype=f32))
            x = xbuf[:, 8:] if i % 2 == 0 else dev(host(xbuf)[:, 8:].copy())
            w = dev((rng.standard_normal((OC, C, 1, 1), dtype=f32) * f32(0.3)).astype(f32))
            b = dev(rng.standard_normal(OC, dtype=f32)) if i != 1 else None
            assert api.conv2d_fused_ok(x.shape, w.shape, 1, 0)
            pk = api.conv2d_pack_weights(x.shape, w, 1, 0)
            ybuf = dev(np.full((N, OC + 5, H, W), 3, f32))
            y = ybuf[:, 2:2 + OC] if i % 2 == 1 else dev(np.full((N, OC, H, W), 3, f32))
            alone = dev(np.zeros((N, OC, H, W), f32))
            api.conv2d_fused(x, w.shape, pk, b, alone, 1, 0, act)
            xs.append(x), ws.append(tuple(w.shape)), pks.append(pk), bs.append(b), ys.append((y, ybuf)), wants.append(host(alone))
        assert api.conv2d_fused_group_ok([x.shape for x in xs], ws)
        api.conv2d_fused_group(xs, ws, pks, bs, [y for y, _ in ys], act)
        for i, ((y, ybuf), want) in enumerate(zip(ys, wants)):
            assert np.array_equal(host(y), want), (N, members[i])
            if i % 2 == 1:
                assert np.all(host(ybuf)[:, :2] == 3) and np.all(host(ybuf)[:, 2 + want.shape[1]:] == 3)
    assert not api.conv2d_fused_group_ok([(2, 12, 8, 8)], [(16, 12, 1, 1)])                    # channels not a multiple of 8
    assert not api.conv2d_fused_group_ok([(2, 16, 8, 8)], [(16, 16, 3, 3)])                    # not a 1x1 window
    assert not api.conv2d_fused_group_ok([(2, 16, 8, 8), (3, 16, 8, 8)], [(16, 16, 1, 1)] * 2)  # batches differ
    x, y = dev(np.zeros((2, 12, 8, 8), f32)), dev(np.zeros((2, 16, 8, 8), f32))
    with pytest.raises(api.OdlInvalidArgument):
        api.conv2d_fused_group([x], [(16, 12, 1, 1)], [dev(np.zeros(16 * 12, f32))], [None], [y])


def test_detect_head_in_one_launch_equals_convolution_then_decoding(api):
    """Every stage of a detect head as one launch, the decoding in the convolutions' epilogues: the floats of
    conv2d_fused followed by yolo_decode for each stage (K shares from 1 to 16, ragged pixel tiles, an anchor grid
    coarser than the stage, inputs that are runs of wider tensors, a stage without bias, few and many classes)."""
    rng = np.random.default_rng(78)
    for N, A, NC, members in ((4, 3, 80, ((64, 40, 40), (128, 20, 20), (256, 10, 10))),
                              (2, 2, 1, ((8, 7, 9), (512, 3, 5))),
                              (1, 3, 6, ((16, 16, 16), (32, 6, 4), (64, 2, 2), (128, 1, 1))),
                              (3, 1, 0, ((24, 11, 6),))):
        CI = A * 0 + NC + 5
        OC = A * CI
        xs, pks, bs, grids, ags, strides, convs = [], [], [], [], [], [], []
        for i, (C, H, W) in enumerate(members):
            xbuf = dev(rng.standard_normal((N, C + 8, H, W), dtype=f32))
            x = xbuf[:, 8:] if i % 2 == 0 else dev(host(xbuf)[:, 8:].copy())
            w = dev((rng.standard_normal((OC, C, 1, 1), dtype=f32) * f32(0.3)).astype(f32))
            b = dev(rng.standard_normal(OC, dtype=f32)) if i != 1 else None
            pk = api.conv2d_pack_weights(x.shape, w, 1, 0)
            conv = dev(np.zeros((N, OC, H, W), f32))
            api.conv2d_fused(x, w.shape, pk, b, conv, 1, 0, None)
            gyy, gxx = np.meshgrid(np.arange(H), np.arange(W), indexing="ij")
            grids.append(dev(np.broadcast_to(np.stack([gxx, gyy], -1).astype(f32) - f32(0.5), (1, A, H, W, 2)).copy()))
            aH, aW = (H, W) if i != 2 else (max(H // 2, 1), max(W // 2, 1))  # (one stage with an anchor grid at half the size)
            ags.append(dev((rng.random((1, A, aH, aW, 2), dtype=f32) * f32(90) + f32(4)).astype(f32)))
            xs.append(x), pks.append(pk), bs.append(b), strides.append(float(8 << i)), convs.append(conv)
        assert api.yolo_detect_stages_ok([x.shape for x in xs], A, NC)
        rows = sum(A * x.shape[2] * x.shape[3] for x in xs)
        one, each = dev(np.full((N, rows + 9, CI), 7, f32)), dev(np.full((N, rows + 9, CI), 7, f32))
        api.yolo_detect_stages_forward(xs, pks, bs, grids, ags, strides, A, NC, one)
        r0 = 0
        for c, g, a, st in zip(convs, grids, ags, strides):
            r = A * c.shape[2] * c.shape[3]
            api.yolo_decode(c, g, a, st, A, NC, each[:, r0:r0 + r])
            r0 += r
        assert np.array_equal(host(one), host(each)), (N, A, NC, members)
    assert not api.yolo_detect_stages_ok([(2, 12, 8, 8)], 3, 80)                 # channels not a multiple of 8
    assert not api.yolo_detect_stages_ok([(2, 16, 8, 8), (3, 16, 4, 4)], 3, 80)  # batches differ
    with pytest.raises(api.OdlInvalidArgument):
        api.yolo_detect_stages_forward([dev(np.zeros((2, 12, 8, 8), f32))], [dev(np.zeros(16 * 255, f32))], [None],
                                       [dev(np.zeros((1, 3, 8, 8, 2), f32))], [dev(np.ones((1, 3, 8, 8, 2), f32))], [8.0], 3, 80,
                                       dev(np.zeros((2, 192, 85), f32)))


def test_conv_fused_refuses_what_it_does_not_cover(api):
    assert not api.conv2d_fused_ok((2, 3, 64, 64), (16, 3, 6, 6), 2, 2)        # three channels
    assert not api.conv2d_fused_ok((32, 64, 56, 56), (128, 64, 3, 3), 1, 1)    # 14.8 GFLOP: the tiled kernels' work
    x, y = dev(np.zeros((2, 12, 8, 8), f32)), dev(np.zeros((2, 16, 8, 8), f32))
    with pytest.raises(api.OdlInvalidArgument):
        api.conv2d_fused(x, (16, 12, 1, 1), dev(np.zeros(16 * 12, f32)), None, y, 1, 0)
    x = dev(np.zeros((2, 16, 8, 8), f32))
    w = dev(np.ones((16, 16, 1, 1), f32))
    packed = api.conv2d_pack_weights(x.shape, w, 1, 0)
    with pytest.raises(api.OdlInvalidArgument):  # an image stride shorter than the image
        api.lib().call("odl_hip_conv2d_fused", x.data_ptr(), 100, packed.data_ptr(), None, 2, 16, 8, 8, 16, 1, 1, 1, 1, 0, 0, -1,
                       None, 0, y.data_ptr(), 0, None)
    with pytest.raises(api.OdlInvalidArgument):
        api.conv2d_fused(x, w.shape, packed, None, y, 1, 0, "exp")


def test_detector_operators_on_channel_runs_are_the_dense_operators(api, o):
    """upsample, the SPPF chain of max pools, the image copy and the detect decoding, reading and writing runs of
    channels (rows, for the decoding) of wider tensors: bit-identical to the dense entry points."""
    rng = np.random.default_rng(77)
    # upsample: [4, 128, 10, 10] out of a 160-channel tensor into channels 64.. of a 256-channel one
    src = dev(rng.standard_normal((4, 160, 10, 10), dtype=f32))
    dst0 = rng.standard_normal((4, 256, 20, 20), dtype=f32)
    dst = dev(dst0)
    api.upsample_view(src[:, 32:160], dst[:, 64:192], 2)
    want = dst0.copy()
    want[:, 64:192] = host(api.upsample(src[:, 32:160].contiguous(), 2))
    assert np.array_equal(host(dst), want)
    for (N, C, H, W, sh, sw) in ((2, 3, 5, 6, 2, 2), (1, 2, 7, 4, 3, 1), (3, 1, 2, 5, 2, 4)):
        xs = dev(rng.standard_normal((N, C, H, W), dtype=f32))
        ys = dev(np.zeros((N, C + 2, H * sh, W * sw), f32))
        api.upsample_view(xs, ys[:, 1:1 + C], (sh, sw))
        assert np.array_equal(host(ys)[:, 1:1 + C], host(api.upsample(xs, (sh, sw)))), (N, C, H, W, sh, sw)
    # SPPF: x = channels 0..128 of the 512-channel concatenation itself, three 5x5 pools into channels 128..512
    for (N, C, H, W, K, count) in ((4, 128, 10, 10, 5, 3), (2, 5, 7, 9, 3, 2), (1, 3, 20, 20, 9, 1), (2, 4, 1, 1, 5, 3)):
        buf0 = rng.standard_normal((N, (count + 1) * C, H, W), dtype=f32)
        buf = dev(buf0)
        api.max_pool2d_chain(buf[:, :C], K, count, buf[:, C:])
        want, cur = buf0.copy(), dev(np.ascontiguousarray(buf0[:, :C]))
        for j in range(count):
            cur, _ = api.max_pool2d(cur, K, 1, K // 2, with_indices=False)
            want[:, (j + 1) * C:(j + 2) * C] = host(cur)
        assert np.array_equal(host(buf), want), (N, C, H, W, K, count)
    with pytest.raises(api.OdlInvalidArgument):
        api.max_pool2d_chain(dev(np.zeros((1, 1, 8, 8), f32)), 4, 1, dev(np.zeros((1, 1, 8, 8), f32)))  # even window
    with pytest.raises(api.OdlInvalidArgument):
        api.max_pool2d_chain(dev(np.zeros((1, 1, 100, 100), f32)), 3, 1, dev(np.zeros((1, 1, 100, 100), f32)))  # plane too large
    # image copy in both directions, runs that are and are not multiples of four floats
    for (N, C, H, W) in ((4, 64, 20, 20), (3, 5, 3, 7)):
        a0 = rng.standard_normal((N, C + 3, H, W), dtype=f32)
        a, d = dev(a0), dev(np.zeros((N, C + 9, H, W), f32))
        api.copy_images(a[:, 2:2 + C], d[:, 4:4 + C])
        want = np.zeros((N, C + 9, H, W), f32)
        want[:, 4:4 + C] = a0[:, 2:2 + C]
        assert np.array_equal(host(d), want)
        back = dev(np.zeros((N, C, H, W), f32))
        api.copy_images(d[:, 4:4 + C], back)
        assert np.array_equal(host(back), a0[:, 2:2 + C])
    # detect: decoding into the stage's rows of the concatenated output = the dense call's decoding
    N, C, H, W, A, NC = 4, 64, 20, 20, 3, 80
    CI = NC + 5
    x = dev(rng.standard_normal((N, C, H, W), dtype=f32))
    w = dev((rng.standard_normal((A * CI, C, 1, 1), dtype=f32) * f32(0.2)).astype(f32))
    b = dev(rng.standard_normal(A * CI, dtype=f32))
    gyy, gxx = np.meshgrid(np.arange(H), np.arange(W), indexing="ij")
    grid = dev(np.broadcast_to(np.stack([gxx, gyy], -1).astype(f32) - f32(0.5), (1, A, H, W, 2)).copy())
    ag = dev(np.broadcast_to(np.array([[10, 13], [16, 30], [33, 23]], f32).reshape(1, A, 1, 1, 2), (1, A, H, W, 2)).copy())
    dense = host(api.yolo_detect_forward(x, w, b, grid, ag, 16.0, A, NC))
    out0 = rng.standard_normal((N, 500 + A * H * W + 70, CI), dtype=f32)
    out = dev(out0)
    api.yolo_decode(api.conv2d(x, w, b, 1, 0), grid, ag, 16.0, A, NC, out[:, 500:500 + A * H * W])
    want = out0.copy()
    want[:, 500:500 + A * H * W] = dense
    assert np.array_equal(host(out), want)
    # the stages of a head decoded in one launch = one call a stage (a stage with a ragged last pixel tile among them)
    convs, grids, ags, wants = [], [], [], []
    strides = (8.0, 16.0, 32.0)
    for (H, W) in ((20, 20), (10, 13), (5, 5)):
        convs.append(dev(rng.standard_normal((N, A * CI, H, W), dtype=f32) * f32(3)))
        gyy, gxx = np.meshgrid(np.arange(H), np.arange(W), indexing="ij")
        grids.append(dev(np.broadcast_to(np.stack([gxx, gyy], -1).astype(f32) - f32(0.5), (1, A, H, W, 2)).copy()))
        ags.append(dev((rng.random((1, A, H, W, 2), dtype=f32) * f32(90) + f32(4)).astype(f32)))
    rows = sum(A * c.shape[2] * c.shape[3] for c in convs)
    one, each = dev(np.full((N, rows + 9, CI), 7, f32)), dev(np.full((N, rows + 9, CI), 7, f32))
    api.yolo_decode_stages(convs, grids, ags, strides, A, NC, one)
    r0 = 0
    for c, g, a, st in zip(convs, grids, ags, strides):
        r = A * c.shape[2] * c.shape[3]
        api.yolo_decode(c, g, a, st, A, NC, each[:, r0:r0 + r])
        r0 += r
    assert np.array_equal(host(one), host(each))
    assert np.all(host(one)[:, rows:] == 7)
    with pytest.raises(api.OdlInvalidArgument):
        api.yolo_decode_stages(convs, grids[:2], ags, strides, A, NC, one)


# ------------------------------------------------------------------ element types besides float32
DT = {"f32": (0, np.float32), "f64": (1, np.float64), "i8": (2, np.int8), "i32": (3, np.int32), "i64": (4, np.int64),
      "u8": (5, np.uint8)}


def _typed_values(rng, np_t, n, positive=False):
    if np_t in (np.float32, np.float64):
        v = rng.standard_normal(n) * 40
        return (np.abs(v) if positive else v).astype(np_t)
    hi = {np.int8: 100, np.uint8: 200}.get(np_t, 100000)
    lo = 0 if (positive or np_t is np.uint8) else -hi
    return rng.integers(lo, hi, size=n).astype(np_t)


def test_convert_between_all_element_types_is_a_static_cast(api):
    # src/mat/origin/cuda/type_conversion.cu: dst[i] = static_cast<Dst>(src[i]); numpy's astype is the same conversion
    # wherever C++ defines it (values inside the destination's range; float -> integer truncates towards zero)
    L = api.lib()
    rng = np.random.default_rng(51)
    n = 100_003
    for sname, (scode, s_t) in DT.items():
        for dname, (dcode, d_t) in DT.items():
            small = d_t in (np.int8, np.uint8) or s_t in (np.int8, np.uint8)
            src = _typed_values(rng, s_t, n, positive=(d_t is np.uint8))
            if small:
                src = (src % 100).astype(s_t) if s_t not in (np.float32, np.float64) else np.clip(src, 0 if d_t is np.uint8 else -100, 100).astype(s_t)
            d_src = dev(src)
            d_dst = torch.empty(n, dtype=getattr(torch, np.dtype(d_t).name), device="cuda")
            L.call("odl_hip_convert", d_src.data_ptr(), scode, d_dst.data_ptr(), dcode, n, None)
            assert np.array_equal(host(d_dst), src.astype(d_t)), (sname, dname)
    assert [L.query("odl_hip_dtype_size", c) for c in range(7)] == [4, 8, 1, 4, 8, 1, 0]
    with pytest.raises(api.OdlInvalidArgument):
        L.call("odl_hip_convert", d_src.data_ptr(), 9, d_dst.data_ptr(), 0, 4, None)


@pytest.mark.parametrize("name", ["f32", "f64", "i8", "i32", "i64", "u8"])
def test_max_broadcast_sum_to_cat_split_in_every_element_type(api, name):
    """Mat::max, broadcast_to, sum_to, cat and split dispatch over the element type in the reference
    (src/mat/origin/cuda/math/{max,broadcast_to,sum_to}.cu, shape/{cat,split}.cu). Checked against numpy: max and the
    copies bit for bit, sums of integers bit for bit (they wrap in the type's width), sums of doubles within n * 2^-52."""
    L = api.lib()
    code, t = DT[name]
    tt = getattr(torch, np.dtype(t).name)
    rng = np.random.default_rng(77 + code)
    is_float = t in (np.float32, np.float64)

    def shape_arr(shape):
        return (ctypes.c_int64 * max(len(shape), 1))(*shape)

    # ---- max over an axis of [outer, axis, inner] and over the whole tensor
    for outer, axis, inner in ((1, 300, 1), (4, 37, 5), (3, 1, 7), (2, 513, 64)):
        x = _typed_values(rng, t, outer * axis * inner).reshape(outer, axis, inner)
        if is_float and axis > 1:
            x[0, axis // 2, 0] = np.nan  # never wins: `m < v` is false for it
        out = torch.empty((outer, inner), dtype=tt, device="cuda")
        dx = dev(x)
        L.call("odl_hip_max_axis_dtype", code, dx.data_ptr(), outer, axis, inner, out.data_ptr(), None)
        want = np.fmax.reduce(x, axis=1) if is_float else x.max(axis=1)
        assert np.array_equal(host(out), want.astype(t)), (name, outer, axis, inner)
        one = torch.empty(1, dtype=tt, device="cuda")
        L.call("odl_hip_max_all_dtype", code, dx.data_ptr(), x.size, one.data_ptr(), None)
        assert host(one)[0] == (np.nanmax(x) if is_float else x.max())
    # ---- broadcast_to (right-aligned)
    for src, dst in (((1, 5), (7, 5)), ((3, 1), (3, 9)), ((4,), (2, 3, 4)), ((2, 1, 3), (2, 5, 3)), ((1,), (6,))):
        x = _typed_values(rng, t, int(np.prod(src))).reshape(src)
        out = torch.empty(dst, dtype=tt, device="cuda")
        dx = dev(x)
        L.call("odl_hip_broadcast_to_dtype", code, dx.data_ptr(), shape_arr(src), len(src), shape_arr(dst), len(dst),
               out.data_ptr(), None)
        assert np.array_equal(host(out), np.broadcast_to(x, dst)), (name, src, dst)
    with pytest.raises(api.OdlInvalidArgument):
        L.call("odl_hip_broadcast_to_dtype", code, dx.data_ptr(), shape_arr((3,)), 1, shape_arr((4,)), 1, out.data_ptr(), None)
    # ---- sum_to (left-aligned): reduced where the target has a 1, trailing source dimensions summed away
    for src, dst, axes in (((4, 5), (1, 5), (0,)), ((4, 5), (4, 1), (1,)), ((3, 4, 5), (3,), (1, 2)), ((2, 3, 4), (1, 3, 1), (0, 2)),
                           ((6, 7), (6, 7), ())):
        x = _typed_values(rng, t, int(np.prod(src))).reshape(src)
        nb = L.query("odl_hip_sum_to_dtype_workspace_bytes", code, shape_arr(src), len(src), shape_arr(dst), len(dst))
        ws = torch.empty(max(nb, 4), dtype=torch.uint8, device="cuda")
        out = torch.empty(dst, dtype=tt, device="cuda")
        dx = dev(x)
        L.call("odl_hip_sum_to_dtype", code, dx.data_ptr(), shape_arr(src), len(src), shape_arr(dst), len(dst), out.data_ptr(),
               ws.data_ptr(), nb, None)
        with np.errstate(over="ignore"):
            want = x.sum(axis=axes, dtype=t).reshape(dst) if axes else x
        if is_float:
            terms = x.size // max(int(np.prod(dst)), 1)
            bound = terms * np.finfo(t).eps * np.abs(x).sum(axis=axes).reshape(dst) if axes else 0
            assert (np.abs(host(out) - want) <= bound).all(), (name, src, dst)
        else:
            assert np.array_equal(host(out), want), (name, src, dst)
    with pytest.raises(api.OdlRuntimeError):  # a larger target (sum_to.cpp:24-28)
        L.call("odl_hip_sum_to_dtype", code, dx.data_ptr(), shape_arr((2, 2)), 2, shape_arr((3, 3)), 2, out.data_ptr(), None, 0, None)
    # ---- cat along each dimension, and split (one piece at a time) back
    for shapes, dim in ((((2, 3, 5), (2, 4, 5), (2, 1, 5)), 1), (((3, 4), (2, 4)), 0), (((2, 3, 2), (2, 3, 7)), 2), (((5,), (3,), (9,)), 0)):
        xs = [_typed_values(rng, t, int(np.prod(sh))).reshape(sh) for sh in shapes]
        want = np.concatenate(xs, axis=dim)
        outer = int(np.prod(want.shape[:dim])) if dim else 1
        inner = int(np.prod(want.shape[dim + 1:])) if dim + 1 < want.ndim else 1
        dxs = [dev(x) for x in xs]
        ptrs = (ctypes.c_void_p * len(xs))(*[d.data_ptr() for d in dxs])
        sizes = (ctypes.c_int64 * len(xs))(*[sh[dim] for sh in shapes])
        out = torch.empty(want.shape, dtype=tt, device="cuda")
        L.call("odl_hip_cat_dtype", code, ptrs, sizes, len(xs), outer, inner, out.data_ptr(), None)
        assert np.array_equal(host(out), want), (name, shapes, dim)
        off = 0
        for x in xs:
            piece = torch.empty(x.shape, dtype=tt, device="cuda")
            L.call("odl_hip_slice_axis_dtype", code, out.data_ptr(), outer, want.shape[dim], inner, off, x.shape[dim],
                   piece.data_ptr(), None)
            assert np.array_equal(host(piece), x)
            off += x.shape[dim]


@pytest.mark.parametrize("name", ["f32", "f64", "i8", "i32", "i64", "u8"])
def test_gather_and_upsample_in_every_element_type(api, name):
    """Mat::gather, upsample and upsample_backward dispatch over the element type in the reference
    (src/mat/origin/cuda/nn/gather.cu:189, upsample.cu:176, 224): copies bit for bit; the backward sums in the type."""
    L = api.lib()
    code, t = DT[name]
    tt = getattr(torch, np.dtype(t).name)
    rng = np.random.default_rng(91 + code)
    N, C = 37, 11
    x = _typed_values(rng, t, N * C).reshape(N, C)
    for is64, it in ((0, np.int32), (1, np.int64)):
        idx = rng.integers(0, C, N).astype(it)
        out = torch.empty(N, dtype=tt, device="cuda")
        dx, di = dev(x), dev(idx)
        L.call("odl_hip_gather_dtype", code, dx.data_ptr(), di.data_ptr(), is64, N, C, out.data_ptr(), None)
        assert np.array_equal(host(out), x[np.arange(N), idx])
        bad = idx.copy()
        bad[5] = C
        dbad = dev(bad)
        with pytest.raises(api.OdlInvalidArgument):
            L.call("odl_hip_gather_dtype", code, dx.data_ptr(), dbad.data_ptr(), is64, N, C, out.data_ptr(), None)
    for (n, c, h, w, sh, sw) in ((2, 3, 4, 5, 2, 2), (1, 2, 3, 3, 3, 1), (2, 1, 5, 4, 1, 2)):
        img = _typed_values(rng, t, n * c * h * w).reshape(n, c, h, w)
        up = torch.empty((n, c, h * sh, w * sw), dtype=tt, device="cuda")
        dimg = dev(img)
        L.call("odl_hip_upsample_nearest_dtype", code, dimg.data_ptr(), n, c, h, w, h * sh, w * sw, sh, sw, up.data_ptr(), None)
        assert np.array_equal(host(up), img.repeat(sh, axis=2).repeat(sw, axis=3))
        gy = _typed_values(rng, t, n * c * h * sh * w * sw).reshape(n, c, h * sh, w * sw)
        gx = torch.empty((n, c, h, w), dtype=tt, device="cuda")
        dgy = dev(gy)
        L.call("odl_hip_upsample_nearest_backward_dtype", code, dgy.data_ptr(), n, c, h, w, h * sh, w * sw, sh, sw, gx.data_ptr(), None)
        with np.errstate(over="ignore"):
            want = gy.reshape(n, c, h, sh, w, sw).sum(axis=(3, 5), dtype=t)
        if t in (np.float32, np.float64):
            np.testing.assert_allclose(host(gx), want, rtol=8 * np.finfo(t).eps, atol=8 * np.finfo(t).eps * np.abs(gy).max() * sh * sw)
        else:
            assert np.array_equal(host(gx), want)


@pytest.mark.parametrize("name", ["f64", "i8", "i32", "i64", "u8"])
def test_elementwise_fill_and_sum_in_every_element_type(api, name):
    L = api.lib()
    code, t = DT[name]
    tt = getattr(torch, np.dtype(t).name)
    rng = np.random.default_rng(52 + code)
    n = 70_001
    a, b = _typed_values(rng, t, n), _typed_values(rng, t, n)
    b[b == 0] = 3
    is_float = t is np.float64

    def run_binary(op, x, y):
        out = torch.empty(max(x.size, y.size), dtype=tt, device="cuda")
        dx, dy = dev(x), dev(y)  # both kept alive until the call has been made
        L.call("odl_hip_binary_dtype", op, code, dx.data_ptr(), x.size, dy.data_ptr(), y.size, out.data_ptr(), None)
        return host(out)

    with np.errstate(over="ignore"):
        wide = np.float64 if is_float else np.int64
        quotient = a / b if is_float else np.trunc(a.astype(np.float64) / b.astype(np.float64)).astype(np.int64).astype(t)
        want = [a + b, a - b, a * b, quotient] + [f(a, b).astype(t) for f in (np.greater, np.equal, np.not_equal, np.less,
                                                                              np.less_equal, np.greater_equal)]
        for op, w in enumerate(want):
            assert np.array_equal(run_binary(op, a, b), w.astype(t)), (name, op)  # integer arithmetic wraps in numpy too
        one = np.array([3], t)
        assert np.array_equal(run_binary(0, a, one), (a + one).astype(t))
        assert np.array_equal(run_binary(1, one, a), (one - a).astype(t))
        # unary: relu, negate, square everywhere
        da = dev(a)
        for op, w in ((0, np.maximum(a, 0)), (3, (0 - a.astype(wide)).astype(t) if not is_float else -a),
                      (4, (a.astype(wide) * a.astype(wide)).astype(t) if not is_float else a * a)):
            out = torch.empty(n, dtype=tt, device="cuda")
            L.call("odl_hip_unary_dtype", op, code, da.data_ptr(), n, out.data_ptr(), None)
            assert np.array_equal(host(out), w.astype(t)), (name, "unary", op)
    out = torch.empty(n, dtype=tt, device="cuda")
    if is_float:
        pos = np.abs(a) + 0.5
        for op, f in ((1, lambda v: np.exp(v / 40)), (2, np.log), (5, np.sqrt)):
            src = a / 40 if op == 1 else pos
            dsrc = dev(src)
            L.call("odl_hip_unary_dtype", op, code, dsrc.data_ptr(), n, out.data_ptr(), None)
            np.testing.assert_allclose(host(out), np.exp(src) if op == 1 else f(src), rtol=1e-14)
        dpos = dev(pos)
        L.call("odl_hip_pow_scalar_dtype", code, dpos.data_ptr(), n, 2.5, out.data_ptr(), None)
        np.testing.assert_allclose(host(out), pos ** 2.5, rtol=1e-14)
    else:
        for op in (1, 2, 5, 6, 7):  # the reference throws for integer inputs (tests/unit_test/operator/test_log.cpp:210-225)
            with pytest.raises(api.OdlInvalidArgument):
                L.call("odl_hip_unary_dtype", op, code, da.data_ptr(), n, out.data_ptr(), None)
        with pytest.raises(api.OdlInvalidArgument):
            L.call("odl_hip_pow_scalar_dtype", code, da.data_ptr(), n, 2.0, out.data_ptr(), None)
    # fill
    v = np.array([7], t)
    L.call("odl_hip_fill_dtype", out.data_ptr(), code, n, v.ctypes.data, None)
    assert (host(out) == v[0]).all()
    # sums: [outer, axis, inner] in both layouts and the whole tensor (which passes through a float, as the reference's)
    for outer, axis, inner in ((1, n, 1), (3, 1000, 1), (4, 300, 50), (1, 5000, 3), (2, 7, 1), (1, 4096 * 64, 1),
                               (70000, 8, 1)):  # more rows than a grid's second dimension holds
        x = _typed_values(rng, t, outer * axis * inner).reshape(outer, axis, inner)
        nb = L.query("odl_hip_sum_axis_dtype_workspace_bytes", code, outer, axis, inner)
        ws = torch.empty(max(nb, 8), dtype=torch.uint8, device="cuda")
        res = torch.empty(outer * inner, dtype=tt, device="cuda")
        dx = dev(x)
        for through_float in (0, 1):
            L.call("odl_hip_sum_axis_dtype", code, dx.data_ptr(), outer, axis, inner, through_float, res.data_ptr(),
                   ws.data_ptr(), nb, None)
            if is_float:
                w = x.sum(axis=1).reshape(-1)
                w = w.astype(np.float32).astype(t) if through_float else w
                np.testing.assert_allclose(host(res), w, rtol=1e-6 if through_float else 1e-12, atol=1e-9)
            else:
                w = x.astype(np.int64).sum(axis=1).reshape(-1).astype(t)  # the wrapped sum in the type's own width
                w = w.astype(np.float32).astype(t) if through_float else w
                assert np.array_equal(host(res), w), (name, outer, axis, inner, through_float)


def test_permute_is_numpy_transpose_in_every_element_width(api):
    # src/mat/origin/cpu/shape/permute.cpp:22-110: output dimension d is input dimension dims[d]
    import ctypes
    L = api.lib()
    rng = np.random.default_rng(61)
    for name, shape, perm in (("f32", (4, 3, 5, 7), (0, 2, 3, 1)), ("f32", (2, 3, 85, 6, 5), (0, 1, 3, 4, 2)),
                              ("f64", (6, 5), (1, 0)), ("u8", (3, 4, 5), (2, 0, 1)), ("i64", (7,), (0,)),
                              ("i32", (2, 1, 3, 1, 4), (4, 3, 2, 1, 0)), ("f32", (3, 2, 85, 12, 20), (0, 1, 3, 4, 2)),
                              ("f32", (130, 70), (1, 0)), ("f32", (64, 128), (1, 0)), ("u8", (5, 67, 130), (0, 2, 1)),
                              ("i64", (3, 65, 66), (0, 2, 1)), ("f64", (2, 3, 4, 5), (0, 1, 2, 3)),
                              ("i32", (6, 1, 9), (2, 1, 0)), ("f32", (4, 5, 6, 7), (2, 3, 0, 1))):
        code, t = DT[name]
        x = _typed_values(rng, t, int(np.prod(shape))).reshape(shape)
        dx = dev(x)
        out = torch.empty(tuple(shape[p] for p in perm), dtype=getattr(torch, np.dtype(t).name), device="cuda")
        sh, pm = (ctypes.c_int64 * len(shape))(*shape), (ctypes.c_int * len(perm))(*perm)
        L.call("odl_hip_permute", dx.data_ptr(), code, sh, len(shape), pm, out.data_ptr(), None)
        assert np.array_equal(host(out), np.transpose(x, perm)), (name, shape, perm)
    sh, pm = (ctypes.c_int64 * 2)(3, 4), (ctypes.c_int * 2)(0, 0)
    with pytest.raises(api.OdlInvalidArgument):
        L.call("odl_hip_permute", dx.data_ptr(), 0, sh, 2, pm, out.data_ptr(), None)


def test_linear_with_the_activation_in_the_epilogue_equals_linear_then_relu(api):
    # src/nn/layers/linear.cpp:80-106 followed by src/operators/activation/relu.cpp: the fused entry must give the bits
    # of the two run in turn, for the single-pass, K-sliced and tail-split schedules of the product
    L = api.lib()
    rng = np.random.default_rng(77)
    for M, K, N in ((512, 784, 1000), (64, 100, 10), (300, 1024, 1024), (1536, 640, 2304), (33, 17, 5)):
        x, w = dev(rng.standard_normal((M, K), dtype=np.float32)), dev(rng.standard_normal((K, N), dtype=np.float32))
        b = dev(rng.standard_normal((N,), dtype=np.float32))
        nb = L.query("odl_hip_sgemm_workspace_bytes", 0, 0, M, N, K, 0)
        ws = torch.empty(max(nb, 16), dtype=torch.uint8, device="cuda")
        plain, fused = torch.empty((M, N), device="cuda"), torch.empty((M, N), device="cuda")
        L.call("odl_hip_sgemm", 0, 0, M, N, K, x.data_ptr(), K, w.data_ptr(), N, plain.data_ptr(), N, b.data_ptr(), 0,
               ws.data_ptr(), nb, None)
        for act, f in ((-1, lambda v: v), (0, lambda v: np.maximum(v, np.float32(0)))):
            L.call("odl_hip_linear_act", x.data_ptr(), w.data_ptr(), b.data_ptr(), M, N, K, act, fused.data_ptr(),
                   ws.data_ptr(), nb, None)
            assert np.array_equal(host(fused), f(host(plain))), (M, K, N, act)
    with pytest.raises(api.OdlInvalidArgument):
        L.call("odl_hip_linear_act", x.data_ptr(), w.data_ptr(), b.data_ptr(), M, N, K, 3, fused.data_ptr(), ws.data_ptr(),
               nb, None)


@pytest.mark.parametrize("M,N,K", [(64, 64, 256), (200, 136, 520), (512, 1000, 784), (1024, 1024, 1024), (260, 2052, 4100),
                                   (1536, 1536, 512), (2304, 2304, 512), (2560, 3072, 256)])
def test_the_straight_to_lds_gemm_in_all_four_layouts_over_ragged_edges(api, M, N, K):
    # The variant whose operands go from global memory straight into LDS (64x32, 64x64 and 128x128 tiles, K in slices or
    # whole, 324 tiles whose last 68 are cut into K pieces, 480 tiles at two workgroups per compute unit):
    # ragged edges in M, N and K (zero-filled by the loads), the four operand layouts of
    # src/mat/origin/cpu/math/matmul.cpp:113-218 and src/operators/math/mat_mul.cpp:123-182, bias in the epilogue.
    L = api.lib()
    rng = np.random.default_rng(M + N + K)
    a, b = rng.standard_normal((M, K), dtype=np.float32), rng.standard_normal((K, N), dtype=np.float32)
    bias = rng.standard_normal((N,), dtype=np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    bound = gemm_bound(a, b)
    for ta in (0, 1):
        for tb in (0, 1):
            da, db = dev(a.T if ta else a), dev(b.T if tb else b)
            c = torch.full((M, N), float("nan"), device="cuda")
            nb = L.query("odl_hip_sgemm_workspace_bytes", ta, tb, M, N, K, 0)
            ws = torch.empty(max(nb, 16), dtype=torch.uint8, device="cuda")
            L.call("odl_hip_sgemm", ta, tb, M, N, K, da.data_ptr(), da.shape[1], db.data_ptr(), db.shape[1], c.data_ptr(), N,
                   None, 0, ws.data_ptr(), nb, None)
            got = host(c).astype(np.float64)
            assert (np.abs(got - want) <= bound).all(), (ta, tb, np.abs(got - want).max())
            L.call("odl_hip_sgemm", ta, tb, M, N, K, da.data_ptr(), da.shape[1], db.data_ptr(), db.shape[1], c.data_ptr(), N,
                   dev(bias).data_ptr(), 0, ws.data_ptr(), nb, None)
            assert np.array_equal(host(c), (got.astype(np.float32) + bias)), (ta, tb, "bias")


def test_float64_batch_norm_matches_float64_numpy(api):
    # src/mat/origin/cuda/normalization/batch_norm.cu:497-560 and its backward: the float32 algorithm on doubles
    # (two-pass statistics, biased variance); checked against numpy in float64, [N,C] and [N,C,H,W], both forms of backward
    import ctypes
    L = api.lib()
    rng = np.random.default_rng(5)
    for N, C, P in ((6, 5, 1), (4, 3, 35), (2, 2, 1)):
        x = rng.standard_normal((N, C, P)) * 2 + 1
        gamma, beta = rng.standard_normal(C) + 1.5, rng.standard_normal(C)
        rm, rv = rng.standard_normal(C), rng.random(C) + 0.5
        gy = rng.standard_normal((N, C, P))
        eps = 1e-5
        d = {k: dev(v) for k, v in dict(x=x, gamma=gamma, beta=beta, rm=rm, rv=rv, gy=gy).items()}
        y, xn = torch.empty_like(d["x"]), torch.empty_like(d["x"])
        mean, var = torch.empty(C, dtype=torch.float64, device="cuda"), torch.empty(C, dtype=torch.float64, device="cuda")
        for training in (1, 0):
            L.call("odl_hip_batch_norm_forward_f64", d["x"].data_ptr(), d["gamma"].data_ptr(), d["beta"].data_ptr(),
                   d["rm"].data_ptr(), d["rv"].data_ptr(), training, ctypes.c_double(eps), N, C, P, y.data_ptr(),
                   mean.data_ptr(), var.data_ptr(), xn.data_ptr(), None)
            m = x.mean(axis=(0, 2)) if training else rm
            v = ((x - m[None, :, None]) ** 2).mean(axis=(0, 2)) if training else rv
            want_xn = (x - m[None, :, None]) / np.sqrt(v + eps)[None, :, None]
            np.testing.assert_allclose(host(mean), m, rtol=1e-13, atol=1e-14)
            np.testing.assert_allclose(host(var), v, rtol=1e-12, atol=1e-14)
            np.testing.assert_allclose(host(xn), want_xn, rtol=1e-11, atol=1e-12)
            np.testing.assert_allclose(host(y), gamma[None, :, None] * want_xn + beta[None, :, None], rtol=1e-11, atol=1e-12)
        # backward with the batch statistics of the training forward
        m = x.mean(axis=(0, 2))
        v = ((x - m[None, :, None]) ** 2).mean(axis=(0, 2))
        sd = np.sqrt(v + eps)
        want_xn = (x - m[None, :, None]) / sd[None, :, None]
        dm, dv = dev(m), dev(v)
        dxn = dev(want_xn)
        gx = torch.empty_like(d["x"])
        dgamma, dbeta = torch.empty(C, dtype=torch.float64, device="cuda"), torch.empty(C, dtype=torch.float64, device="cuda")
        want_dgamma, want_dbeta = (gy * want_xn).sum(axis=(0, 2)), gy.sum(axis=(0, 2))
        cnt = N * P
        want_gx = (gamma / sd)[None, :, None] * (gy - (want_dbeta / cnt)[None, :, None] - want_xn * (want_dgamma / cnt)[None, :, None])
        for from_x, src in ((0, dxn), (1, d["x"])):
            L.call("odl_hip_batch_norm_backward_f64", d["gy"].data_ptr(), src.data_ptr(), from_x, d["gamma"].data_ptr(),
                   dm.data_ptr(), dv.data_ptr(), ctypes.c_double(eps), N, C, P, gx.data_ptr(), dgamma.data_ptr(),
                   dbeta.data_ptr(), None)
            np.testing.assert_allclose(host(dgamma), want_dgamma, rtol=1e-11, atol=1e-12)
            np.testing.assert_allclose(host(dbeta), want_dbeta, rtol=1e-11, atol=1e-12)
            np.testing.assert_allclose(host(gx), want_gx, rtol=1e-10, atol=1e-11)


@pytest.mark.parametrize("N,C,H,W,S", [(3, 16, 23, 13, 1), (2, 8, 2, 4, 1), (1, 24, 57, 56, 1), (5, 32, 14, 14, 1),
                                       (2, 64, 9, 37, 1), (3, 16, 28, 28, 2), (2, 8, 27, 13, 2), (1, 24, 112, 111, 2),
                                       (4, 128, 28, 28, 2), (2, 8, 4, 4, 2), (1, 16, 31, 6, 2)])
def test_col2im_3x3_streaming_rows_is_bit_identical_to_the_scatter_loop(api, o, N, C, H, W, S):
    # src/mat/origin/cpu/conv/conv2d.cpp:320-349 adds a pixel's taps in ascending (kh, kw); the kernel that walks down a band
    # of position rows with four of them in LDS must give the same float at stride 1 and 2: bands that do not divide the
    # rows, one-band images, odd and even heights and widths, rows of 2 to 56 positions, one to sixteen 8-channel chunks
    rng = np.random.default_rng(N * 1000 + C * 10 + H + W + S)
    OH, OW = (H + 2 - 3) // S + 1, (W + 2 - 3) // S + 1
    col = rng.standard_normal((N * OH * OW, C * 9), dtype=f32)
    want = np.empty((N, C, H, W), f32)
    o.orc_col2im(col, N, C, H, W, 3, 3, S, S, 1, 1, 1, want)
    got = host(api.col2im(dev(col), (N, C, H, W), 3, S, 1, True))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("N,C,H,W,S", [(3, 16, 23, 13, 1), (2, 8, 2, 4, 1), (1, 24, 57, 56, 1), (5, 32, 14, 14, 1), (2, 64, 9, 37, 1),
                                       (3, 16, 28, 28, 2), (2, 8, 27, 13, 2), (1, 24, 112, 111, 2), (2, 8, 4, 4, 2),
                                       (1, 16, 31, 6, 2), (1, 8, 1, 1, 1), (1, 8, 3, 200, 1), (2, 8, 130, 5, 2)])
def test_im2col_3x3_matrix_layout_is_bit_identical_to_the_gather_loop(api, o, N, C, H, W, S):
    # src/mat/origin/cpu/conv/conv2d.cpp:39-207 copies x[n, c, oh*S-1+kh, ow*S-1+kw] (zero outside the image) to
    # col[(n, oh, ow)][(c, kh, kw)]; the tiled kernel must give the same matrix at stride 1 and 2: pixel tiles that cross
    # image rows and images, one-row and one-pixel images, very wide and very tall images, odd and even sizes
    rng = np.random.default_rng(N * 1000 + C * 10 + H + W + S)
    x = rng.standard_normal((N, C, H, W), dtype=f32)
    OH, OW = (H + 2 - 3) // S + 1, (W + 2 - 3) // S + 1
    want = np.empty((N * OH * OW, C * 9), f32)
    o.orc_im2col(x, N, C, H, W, 3, 3, S, S, 1, 1, 1, want)
    got = host(api.im2col(dev(x), 3, S, 1, True))
    assert np.array_equal(got, want)


def test_max_pool_backward_with_the_relu_mask_folded_in_equals_the_two_steps(api):
    # src/operators/pooling/max_pool2d.cpp:60-86 then src/operators/activation/relu.cpp:23-29 (gy * (x > 0 ? 1 : 0)): the
    # fused entry must give the bits of the two calls in turn, signed zeros included — windows that tile the image exactly
    # (one masked write per cell) and windows that do not (the two steps behind one call)
    import ctypes
    L = api.lib()
    rng = np.random.default_rng(171)
    for N, C, H, W, K, S, P in ((3, 5, 8, 12, 2, 2, 0), (2, 4, 9, 9, 3, 3, 0), (2, 3, 9, 10, 3, 2, 1), (1, 2, 7, 7, 2, 2, 0),
                                (4, 16, 28, 28, 2, 2, 0)):
        x = np.maximum(rng.standard_normal((N, C, H, W), dtype=f32), 0)  # a ReLU output: zeros where the mask is 0
        xd = dev(x)
        y, idx = api.max_pool2d(xd, K, S, P)
        gy = rng.standard_normal(tuple(y.shape), dtype=f32)
        gy.ravel()[::5] = -0.0
        gyd = dev(gy)
        gx_pool = api.max_pool2d_backward(gyd, idx, x.shape, K, S, P)
        want = host(gx_pool) * (x > 0).astype(f32)  # the product, so that -g * 0 keeps its sign
        got = torch.empty_like(xd)
        L.call("odl_hip_max_pool2d_backward_relu", gyd.data_ptr(), idx.data_ptr(), xd.data_ptr(), N, C, H, W, K, K, S, S, P, P,
               got.data_ptr(), None)
        g = host(got)
        assert np.array_equal(g, want) and np.array_equal(np.signbit(g), np.signbit(want)), (N, C, H, W, K, S, P)
@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(64, 32, 14, 14), (5, 7, 3, 3), (33, 19), (256, 64, 14, 14)])
@pytest.mark.parametrize("training", [True, False])
def test_batch_norm_with_the_relu_folded_in_equals_the_two_steps(api, shape, training):
    """relu(batch_norm(x)) in one call, and its backward from the gradient of the ReLU's output, give the bits of
    batch_norm_forward, relu, relu's backward (gy * (y > 0), relu.cpp:45-52) and batch_norm_backward run in turn:
    the mask is the one expression gamma * x_norm + beta > 0 either way, and the channel sums add the same products
    in the same order."""
    rng = np.random.default_rng(hash(shape) % 1000 + training)
    C = shape[1]
    x = rng.standard_normal(shape, dtype=f32)
    gy = rng.standard_normal(shape, dtype=f32)
    gamma = rng.standard_normal(C, dtype=f32)  # both signs: a negative scale flips which side of the mean survives
    beta = (rng.standard_normal(C, dtype=f32) * f32(0.5)).astype(f32)
    rm = rng.standard_normal(C, dtype=f32)
    rv = (rng.random(C, dtype=f32) + f32(0.1)).astype(f32)
    y0, mean0, var0, _ = api.batch_norm_forward(dev(x), dev(gamma), dev(beta), dev(rm), dev(rv), training,
                                                want_x_norm=False)
    want_y = api.unary("relu", y0)
    y, mean, var = api.batch_norm_relu_forward(dev(x), dev(gamma), dev(beta), dev(rm), dev(rv), training)
    assert np.array_equal(host(y), host(want_y))
    assert np.array_equal(host(mean), host(mean0)) and np.array_equal(host(var), host(var0))
    assert 0.2 < float((host(y) > 0).mean()) < 0.8  # the mask is neither empty nor full
    masked = api.binary("relu_backward", dev(gy), y0)
    want = api.batch_norm_backward_from_x(masked, dev(x), dev(gamma), mean0, var0)
    got = api.batch_norm_relu_backward_from_x(dev(gy), dev(x), dev(gamma), dev(beta), mean, var)
    for a, b, name in zip(got, want, ("gx", "dgamma", "dbeta")):
        assert np.array_equal(host(a), host(b)), name
    with pytest.raises(api.OdlInvalidArgument):
        api.batch_norm_relu_backward_from_x(dev(gy), dev(x), dev(gamma), dev(beta[:1].copy()), mean, var)


