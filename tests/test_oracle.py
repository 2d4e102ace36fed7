"""Pins the CPU oracle (oracle/oracle.c) three ways, without a GPU:
  1. the known-answer vectors the reference's own unit tests hold (cited per test),
  2. fixtures written from the compiled reference CPU backend (tests/golden/ref_vectors.npz), bit for bit,
     and — where oracle/_ref was built — the compiled reference itself on fresh seeded inputs,
  3. independent mathematics: float64 numpy closed forms, direct 7-loop convolution, adjointness of
     im2col/col2im, brute-force pooling.
A plausible slip in the oracle (dropped term, wrong sign/index, transposed operand) fails at least one."""
import os

import numpy as np
import pytest

import oraclelib as ol

f32 = np.float32
G = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors.npz"))
o = ol.oracle()
needs_ref = pytest.mark.skipif(not ol.have_ref(), reason="compiled reference (oracle/_ref) not built here")


def conv_out(i, k, s, p):
    return (i + 2 * p - k) // s + 1


def run_conv2d(x, w, b, s, p):
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    y = np.empty((N, OC, conv_out(H, KH, s[0], p[0]), conv_out(W, KW, s[1], p[1])), f32)
    assert o.orc_conv2d(x, w, b, N, C, H, W, OC, KH, KW, s[0], s[1], p[0], p[1], y) == 0
    return y


def run_conv2d_backward(gy, x, w, s, p, bias=True):
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    gx, gw, gb = np.empty_like(x), np.empty_like(w), np.empty((OC,), f32)
    assert o.orc_conv2d_backward(gy, x, w, N, C, H, W, OC, KH, KW, s[0], s[1], p[0], p[1], gx, gw,
                                 gb if bias else None) == 0
    return gx, gw, gb


# ------------------------------------------------------------------ 1. reference unit-test vectors
def test_matmul_reference_vectors():
    # tests/unit_test/operator/test_matmul.cpp:19-64
    for a, b, exp, (m, k, n) in [
        ([1, 2, 3, 4], [5, 6, 7, 8], [19, 22, 43, 50], (2, 2, 2)),
        ([1, 2], [3, 4], [11], (1, 2, 1)),
        ([1, 2, 3, 4, 5, 6], [7, 8, 9, 10, 11, 12], [58, 64, 139, 154], (2, 3, 2)),
    ]:
        c = np.empty((m, n), f32)
        o.orc_matmul(np.array(a, f32), np.array(b, f32), c, m, n, k)
        assert c.ravel().tolist() == exp
    # test_matmul.cpp:119-143: gy = ones -> gx = [[11,15],[11,15]], gw = [[4,4],[6,6]]
    x, w, gy = np.array([1, 2, 3, 4], f32), np.array([5, 6, 7, 8], f32), np.ones(4, f32)
    gx, gw = np.empty(4, f32), np.empty(4, f32)
    o.orc_matmul_backward(x, w, gy, gx, gw, 2, 2, 2)
    assert gx.tolist() == [11, 15, 11, 15] and gw.tolist() == [4, 4, 6, 6]
    # test_matmul.cpp:359-421: all-ones operands give K everywhere
    a, b, c = np.ones((5, 1000), f32), np.ones((1000, 3), f32), np.empty((5, 3), f32)
    o.orc_matmul(a, b, c, 5, 3, 1000)
    assert (c == 1000).all()
    # the float64 form of the same loops: the unit-test vectors above in double, integer-valued operands (every partial
    # sum exact, so any order gives the same bits as numpy's), and random operands against numpy's own double product
    for a, b, exp, (m, k, n) in [([1, 2, 3, 4], [5, 6, 7, 8], [19, 22, 43, 50], (2, 2, 2)),
                                 ([1, 2, 3, 4, 5, 6], [7, 8, 9, 10, 11, 12], [58, 64, 139, 154], (2, 3, 2))]:
        c = np.empty((m, n), np.float64)
        o.orc_matmul_f64(np.array(a, np.float64), np.array(b, np.float64), c, m, n, k)
        assert c.ravel().tolist() == exp
    rng = np.random.default_rng(8)
    ai, bi = rng.integers(-50, 50, (23, 41)).astype(np.float64), rng.integers(-50, 50, (41, 17)).astype(np.float64)
    c = np.empty((23, 17), np.float64)
    o.orc_matmul_f64(ai, bi, c, 23, 17, 41)
    assert np.array_equal(c, ai @ bi)
    ar, br = rng.standard_normal((23, 41)), rng.standard_normal((41, 17))
    o.orc_matmul_f64(ar, br, c, 23, 17, 41)
    bound = 1e-15 * 41 * (np.abs(ar) @ np.abs(br))
    assert (np.abs(c - ar @ br) <= bound).all()
    # a transposed operand or a dropped term would show: against the float32 oracle on float32-exact inputs
    c32 = np.empty((23, 17), f32)
    o.orc_matmul(ai.astype(f32), bi.astype(f32), c32, 23, 17, 41)
    o.orc_matmul_f64(ai, bi, c, 23, 17, 41)
    assert np.array_equal(c32.astype(np.float64), c)


def _im2col_np(x, KH, KW, SH, SW, PH, PW):
    """col[(n,oh,ow)][(c,kh,kw)] built from slices of the padded image (an independent restatement, any float type)"""
    N, C, H, W = x.shape
    OH, OW = (H + 2 * PH - KH) // SH + 1, (W + 2 * PW - KW) // SW + 1
    xp = np.pad(x, ((0, 0), (0, 0), (PH, PH), (PW, PW)))
    col = np.empty((N, OH, OW, C, KH, KW), x.dtype)
    for kh in range(KH):
        for kw in range(KW):
            col[:, :, :, :, kh, kw] = xp[:, :, kh:kh + SH * OH:SH, kw:kw + SW * OW:SW].transpose(0, 2, 3, 1)
    return col.reshape(N * OH * OW, C * KH * KW)


def _col2im_np(col, shape, KH, KW, SH, SW, PH, PW):
    N, C, H, W = shape
    OH, OW = (H + 2 * PH - KH) // SH + 1, (W + 2 * PW - KW) // SW + 1
    c6 = col.reshape(N, OH, OW, C, KH, KW)
    xp = np.zeros((N, C, H + 2 * PH, W + 2 * PW), col.dtype)
    for kh in range(KH):
        for kw in range(KW):
            xp[:, :, kh:kh + SH * OH:SH, kw:kw + SW * OW:SW] += c6[:, :, :, :, kh, kw].transpose(0, 3, 1, 2)
    return xp[:, :, PH:PH + H, PW:PW + W]


def test_conv2d_f64_restatement_is_pinned():
    # The convolution over doubles. The compiled reference cannot pin it: its CPU im2col copies a float buffer into
    # the double result (conv2d.cpp:87, 159), so a double convolution on the CPU returns garbage; the device code
    # dispatches over the element type (cuda/conv/conv2d.cu:412-664) and is what the doubles here restate. Pinned by
    # the reference's own known answers with integer data, by the float32 restatement (itself equal to the compiled
    # reference bit for bit) on data both types hold exactly, and by the mathematics: a direct convolution, and the
    # backward products written out with numpy on gy's buffer read as [N*OH*OW, OC].
    rng = np.random.default_rng(20261125)
    for (N, C, H, W, OC, KH, KW, SH, SW, PH, PW) in ((2, 3, 7, 6, 4, 3, 3, 1, 1, 1, 1), (3, 4, 9, 9, 5, 3, 3, 2, 2, 1, 1),
                                                    (2, 2, 8, 5, 3, 2, 3, 2, 1, 0, 2)):
        OH, OW = (H + 2 * PH - KH) // SH + 1, (W + 2 * PW - KW) // SW + 1
        x, gy = rng.standard_normal((N, C, H, W)), rng.standard_normal((N, OC, OH, OW))
        w, b = rng.standard_normal((OC, C, KH, KW)), rng.standard_normal((OC,))
        y, gx, gw, gb = np.empty((N, OC, OH, OW)), np.empty_like(x), np.empty_like(w), np.empty_like(b)
        assert o.orc_conv2d_f64(x, w, b, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, y) == 0
        assert o.orc_conv2d_backward_f64(gy, x, w, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, gx, gw, gb) == 0
        col = _im2col_np(x, KH, KW, SH, SW, PH, PW)
        want_y = (col @ w.reshape(OC, -1).T + b).reshape(N, OH, OW, OC).transpose(0, 3, 1, 2)
        gy2d = gy.reshape(N * OH * OW, OC)  # the buffer as it lies
        want_gw = (gy2d.T @ col).reshape(w.shape)
        want_gx = _col2im_np(gy2d @ w.reshape(OC, -1), x.shape, KH, KW, SH, SW, PH, PW)
        for got, want in ((y, want_y), (gw, want_gw), (gx, want_gx), (gb, gy.sum((0, 2, 3)))):
            assert np.abs(got - want).max() <= 1e-13 * (1 + np.abs(want).max())
        got_col, got_img = np.empty_like(col), np.empty_like(x)
        assert o.orc_im2col_f64(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, got_col) == 0 and np.array_equal(got_col, col)
        assert o.orc_col2im_f64(col, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, got_img) == 0
        assert np.abs(got_img - _col2im_np(col, x.shape, KH, KW, SH, SW, PH, PW)).max() <= 1e-13
    # test_conv2d.cpp:21-48 and the reinterpreted filter gradient quoted below, in doubles
    x9, ones = np.arange(1.0, 10.0).reshape(1, 1, 3, 3), np.ones((1, 1, 2, 2))
    y4 = np.empty((1, 1, 2, 2))
    assert o.orc_conv2d_f64(x9, ones, None, 1, 1, 3, 3, 1, 2, 2, 1, 1, 0, 0, y4) == 0
    assert y4.ravel().tolist() == [12, 16, 24, 28]
    gy8, w8 = np.arange(1.0, 9.0).reshape(1, 2, 2, 2), np.arange(1.0, 9.0).reshape(2, 1, 2, 2)
    gx9, gw8 = np.empty_like(x9), np.empty_like(w8)
    assert o.orc_conv2d_backward_f64(gy8, x9, w8, 1, 1, 3, 3, 2, 2, 2, 1, 1, 0, 0, gx9, gw8, None) == 0
    assert gw8.ravel().tolist() == [62, 78, 110, 126, 74, 94, 134, 154]
    # integers both element types hold exactly: the two restatements agree to the last bit
    xi = rng.integers(-8, 8, (2, 3, 6, 5)).astype(np.float64)
    wi = rng.integers(-4, 4, (4, 3, 3, 2)).astype(np.float64)
    bi = rng.integers(-4, 4, (4,)).astype(np.float64)
    OH, OW = (6 + 2 - 3) // 2 + 1, (5 + 0 - 2) // 1 + 1  # 3x2 window, stride 2x1, padding 1x0
    gi = rng.integers(-4, 4, (2, 4, OH, OW)).astype(np.float64)
    y64, y32 = np.empty((2, 4, OH, OW)), np.empty((2, 4, OH, OW), f32)
    assert o.orc_conv2d_f64(xi, wi, bi, 2, 3, 6, 5, 4, 3, 2, 2, 1, 1, 0, y64) == 0
    assert o.orc_conv2d(xi.astype(f32), wi.astype(f32), bi.astype(f32), 2, 3, 6, 5, 4, 3, 2, 2, 1, 1, 0, y32) == 0
    assert np.array_equal(y64, y32.astype(np.float64))
    g64 = [np.empty_like(xi), np.empty_like(wi), np.empty_like(bi)]
    g32 = [np.empty(xi.shape, f32), np.empty(wi.shape, f32), np.empty(bi.shape, f32)]
    assert o.orc_conv2d_backward_f64(gi, xi, wi, 2, 3, 6, 5, 4, 3, 2, 2, 1, 1, 0, *g64) == 0
    assert o.orc_conv2d_backward(gi.astype(f32), xi.astype(f32), wi.astype(f32), 2, 3, 6, 5, 4, 3, 2, 2, 1, 1, 0, *g32) == 0
    for a64, a32 in zip(g64, g32):
        assert np.array_equal(a64, a32.astype(np.float64))


def test_conv2d_reference_vectors():
    x9 = np.arange(1, 10, dtype=f32).reshape(1, 1, 3, 3)
    ones = np.ones((1, 1, 2, 2), f32)
    # tests/unit_test/operator/test_conv2d.cpp:21-48, 50-70, 93-117, 218-236
    assert run_conv2d(x9, ones, None, (1, 1), (0, 0)).ravel().tolist() == [12, 16, 24, 28]
    assert run_conv2d(x9, ones, None, (2, 2), (0, 0)).ravel().tolist() == [12]
    x4 = np.arange(1, 5, dtype=f32).reshape(1, 1, 2, 2)
    assert run_conv2d(x4, ones, np.array([1], f32), (1, 1), (0, 0)).ravel().tolist() == [11]
    assert run_conv2d(np.ones((1, 1, 1, 1), f32), np.ones((1, 1, 1, 1), f32), None, (1, 1), (0, 0)).item() == 1
    # test_conv2d_transpose_output.cpp:54-94: NCHW ordering of two output channels
    w2 = np.array([1, 1, 1, 1, 2, 2, 2, 2], f32).reshape(2, 1, 2, 2)
    assert run_conv2d(x9, w2, None, (1, 1), (0, 0)).ravel().tolist() == [12, 16, 24, 28, 24, 32, 48, 56]


def test_conv2d_backward_reinterpretation_vector():
    # Recorded from the compiled reference for x=1..9 [1,1,3,3], W [2,1,2,2], gy=1..8 [1,2,2,2]:
    # the reference's gW is 62 78 110 126 74 94 134 154 (gy's NCHW buffer read as [N*OH*OW, OC]);
    # the mathematical gradient would be 37 47 67 77 85 111 163 189.
    x = np.arange(1, 10, dtype=f32).reshape(1, 1, 3, 3)
    gy = np.arange(1, 9, dtype=f32).reshape(1, 2, 2, 2)
    w = np.arange(1, 9, dtype=f32).reshape(2, 1, 2, 2)
    gx, gw, _ = run_conv2d_backward(gy, x, w, (1, 1), (0, 0), bias=False)
    assert gw.ravel().tolist() == [62, 78, 110, 126, 74, 94, 134, 154]
    assert np.array_equal(gw, G["convC_gw"]) and np.array_equal(gx, G["convC_gx"])


def test_sum_to_reference_vectors():
    # tests/unit_test/operator/test_sum_to.cpp: [2,2]->[1,1]=10; [2,3]->[2,1]=[6,15]; [2,2,2]->[2,1]=[10,26] (179-191)
    def st(x, ss, ts):
        dst = np.zeros(max(int(np.prod(ts)), 1), f32)
        rc = o.orc_sum_to(np.array(x, f32), ol.shape_arr(ss), len(ss), ol.shape_arr(ts), len(ts), dst)
        return rc, dst.tolist()

    assert st([1, 2, 3, 4], (2, 2), (1, 1)) == (0, [10])
    assert st([1, 2, 3, 4, 5, 6], (2, 3), (2, 1)) == (0, [6, 15])
    assert st(list(range(1, 9)), (2, 2, 2), (2, 1)) == (0, [10, 26])
    assert st(list(range(1, 9)), (2, 2, 2), (1, 1, 1)) == (0, [36])
    # test_sum_to.cpp:53-60: a larger target throws runtime_error
    assert st([1, 2], (2,), (2, 2))[0] == ol.ctypes.c_int(-2).value
    # a probe of the compiled reference: x{2} broadcast to {2,2}, gy=[[1,2],[3,4]] -> x.grad=[3,7]
    assert st([1, 2, 3, 4], (2, 2), (2,)) == (0, [3, 7])


def test_softmax_ce_reference_vectors():
    # tests/unit_test/operator/test_softmax_cross_entropy.cpp:71-83: uniform logits -> log 3
    loss = np.zeros(1, f32)
    assert o.orc_softmax_ce_loss(np.ones((1, 3), f32), np.array([1], np.int32), 0, 1, 3, loss) == 0
    assert abs(loss[0] - np.log(3.0)) < 1e-6
    # 131-161: gx = softmax(x) - one_hot for N = 1
    x = np.array([[1, 2, 3]], f32)
    gx = np.empty_like(x)
    assert o.orc_softmax_ce_grad(x, np.array([2], np.int32), 0, 1, 3, 1.0, gx) == 0
    e = np.exp(x.astype(np.float64) - 3)
    np.testing.assert_allclose(gx, e / e.sum() - np.array([[0, 0, 1]]), atol=1e-6)
    # 227-234: an out-of-range label throws
    assert o.orc_softmax_ce_loss(x, np.array([3], np.int32), 0, 1, 3, loss) == -1


def test_max_pool_reference_vectors():
    # tests/unit_test/operator/test_max_pool2d.cpp:20-45
    x = np.arange(1, 17, dtype=f32).reshape(1, 1, 4, 4)
    y, idx = np.empty((1, 1, 2, 2), f32), np.empty((1, 1, 2, 2), np.uint64)
    assert o.orc_max_pool2d(x, 1, 1, 4, 4, 2, 2, 2, 2, 0, 0, y, idx) == 0
    assert y.ravel().tolist() == [6, 8, 14, 16] and idx.ravel().tolist() == [3, 3, 3, 3]
    # 127-149: the gradient lands on the maximum only
    x = np.array([1, 2, 3, 4], f32)
    y, idx, gx = np.empty(1, f32), np.empty(1, np.uint64), np.empty(4, f32)
    o.orc_max_pool2d(x, 1, 1, 2, 2, 2, 2, 2, 2, 0, 0, y, idx)
    o.orc_max_pool2d_backward(np.ones(1, f32), idx, 1, 1, 2, 2, 2, 2, 2, 2, 0, 0, gx)
    assert gx.tolist() == [0, 0, 0, 1]


# ---------------------------------------------------- 2. fixtures from the compiled reference, bit for bit
CONV_CASES = {"convA": ((1, 1), (1, 1)), "convB": ((2, 2), (1, 1)), "convC": ((1, 1), (0, 0)),
              "convD": ((2, 1), (0, 2)), "convE": ((1, 1), (0, 0))}


@pytest.mark.parametrize("name", sorted(CONV_CASES))
def test_conv_fixtures_bit_exact(name):
    s, p = CONV_CASES[name]
    x, w, gy = G[f"{name}_x"], G[f"{name}_w"], G[f"{name}_gy"]
    b = G[f"{name}_b"] if f"{name}_b" in G else None
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    assert np.array_equal(run_conv2d(x, w, b, s, p), G[f"{name}_y"])
    gx, gw, gb = run_conv2d_backward(gy, x, w, s, p, bias=b is not None)
    assert np.array_equal(gx, G[f"{name}_gx"]) and np.array_equal(gw, G[f"{name}_gw"])
    if b is not None:
        assert np.array_equal(gb, G[f"{name}_gb"])
    for tm, ck, gk, ik in ((1, "col", "gcol", "im"), (0, "col6", "gcol6", "im6")):
        col = np.empty_like(G[f"{name}_{ck}"])
        assert o.orc_im2col(x, N, C, H, W, KH, KW, s[0], s[1], p[0], p[1], tm, col) == 0
        assert np.array_equal(col, G[f"{name}_{ck}"])
        im = np.empty_like(x)
        assert o.orc_col2im(G[f"{name}_{gk}"], N, C, H, W, KH, KW, s[0], s[1], p[0], p[1], tm, im) == 0
        assert np.array_equal(im, G[f"{name}_{ik}"])


POOL_CASES = {"poolA": (2, 2, 2, 2, 0, 0), "poolB": (3, 3, 2, 2, 1, 1), "poolC": (5, 5, 1, 1, 2, 2),
              "poolD": (3, 2, 1, 2, 1, 0)}


@pytest.mark.parametrize("name", sorted(POOL_CASES))
def test_pool_fixtures_bit_exact(name):
    KH, KW, SH, SW, PH, PW = POOL_CASES[name]
    x = G[f"{name}_x"]
    N, C, H, W = x.shape
    y, idx = np.empty_like(G[f"{name}_y"]), np.empty_like(G[f"{name}_idx"])
    assert o.orc_max_pool2d(x, N, C, H, W, KH, KW, SH, SW, PH, PW, y, idx) == 0
    assert np.array_equal(y, G[f"{name}_y"]) and np.array_equal(idx, G[f"{name}_idx"])
    gx = np.empty_like(x)
    assert o.orc_max_pool2d_backward(G[f"{name}_gy"], idx, N, C, H, W, KH, KW, SH, SW, PH, PW, gx) == 0
    assert np.array_equal(gx, G[f"{name}_gx"])


def test_reduction_fixtures_bit_exact():
    for name in [k[:-3] for k in G.files if k.startswith("sumto") and k.endswith("_rc")]:
        x, ts, rc = G[f"{name}_x"], G[f"{name}_t"], int(G[f"{name}_rc"])
        dst = np.zeros_like(G[f"{name}_y"])
        got = o.orc_sum_to(x, ol.shape_arr(x.shape), x.ndim, ts, len(ts), dst)
        assert got == rc, name
        if rc == 0:
            assert np.array_equal(dst, G[f"{name}_y"]), name
    for name in ("bcastA", "bcastB", "bcastC"):
        x, ds, g = G[f"{name}_x"], G[f"{name}_d"], G[f"{name}_g"]
        y = np.empty_like(G[f"{name}_y"])
        o.orc_broadcast_to(x, ol.shape_arr(x.shape), x.ndim, ds, len(ds), y)
        assert np.array_equal(y, G[f"{name}_y"])
        gx = np.zeros_like(G[f"{name}_gx"])
        rc = o.orc_sum_to(g, ds, len(ds), ol.shape_arr(x.shape), x.ndim, gx)  # BroadcastTo::backward
        assert rc == int(G[f"{name}_rc"])
        if rc == 0:
            assert np.array_equal(gx, G[f"{name}_gx"])
    for name in ("sumA", "sumB", "sumC", "sumD"):
        x, axis = G[f"{name}_x"], int(G[f"{name}_axis"])
        y, mx = np.empty_like(G[f"{name}_y"]), np.empty_like(G[f"{name}_max"])
        if axis < 0:
            y[0], mx[0] = o.orc_sum_all(x, x.size), o.orc_max_all(x, x.size)
        else:
            outer, inner = int(np.prod(x.shape[:axis])), int(np.prod(x.shape[axis + 1:]))
            o.orc_sum_axis(x, outer, x.shape[axis], inner, y)
            o.orc_max_axis(x, outer, x.shape[axis], inner, mx)
        assert np.array_equal(y, G[f"{name}_y"]) and np.array_equal(mx, G[f"{name}_max"])


def test_ce_fixtures_bit_exact():
    for name, is64 in (("ceA", 0), ("ceB", 1), ("ceC", 1)):
        x, t = G[f"{name}_x"], G[f"{name}_t"]
        N, C = x.shape
        loss, gx, p = np.zeros(1, f32), np.empty_like(x), np.empty_like(x)
        sel, oh = np.empty(N, f32), np.empty((N, C), f32)
        assert o.orc_softmax_ce_loss(x, t, is64, N, C, loss) == 0
        assert o.orc_softmax_ce_grad(x, t, is64, N, C, 1.0, gx) == 0
        o.orc_softmax(x, N, C, 1, p)
        assert o.orc_gather(p, t, is64, N, C, sel) == 0 and o.orc_one_hot(t, is64, N, C, oh) == 0
        for got, key in ((loss, "loss"), (gx, "gx"), (p, "p"), (sel, "sel"), (oh, "oh")):
            assert np.array_equal(got, G[f"{name}_{key}"]), (name, key)
    t, x = G["oob_t"], G["oob_x"]
    sel, oh, loss = np.zeros(4, f32), np.empty((4, 3), f32), np.zeros(1, f32)
    assert o.orc_gather(x, t, 0, 4, 3, sel) == int(G["oob_gather_rc"]) == -1
    assert o.orc_one_hot(t, 0, 4, 3, oh) == int(G["oob_onehot_rc"]) == 0
    assert np.array_equal(oh, G["oob_onehot"])
    assert o.orc_softmax_ce_loss(x, t, 0, 4, 3, loss) == int(G["oob_ce_rc"]) == -1


def test_elementwise_fixtures_bit_exact():
    a, b = G["ew_a"], G["ew_b"]
    for op in range(5):
        out = np.empty_like(a)
        assert o.orc_binary(op, a, a.size, b, b.size, out) == 0
        assert np.array_equal(out, G[f"ew_bin{op}"]), op
    for op in range(5):
        src = np.abs(a) + f32(0.1) if op == 2 else a
        out = np.empty_like(a)
        o.orc_unary(op, src, a.size, out)
        assert np.array_equal(out, G[f"ew_un{op}"]), op
    out = np.empty_like(a)
    o.orc_pow_scalar(np.abs(a), a.size, 0.5, out)
    assert np.array_equal(out, G["ew_pow05"])
    assert o.orc_binary(0, a, a.size, b[:5].copy(), 5, out) == -2  # "complex broadcasting" runtime_error


def _mlp_oracle(steps):
    x, t = G["mlp_x"], G["mlp_t"]
    N, D = x.shape
    p = [G[f"mlp_{k}"].copy() for k in ("W1", "b1", "W2", "b2")]
    Hd, C = p[0].shape[1], p[2].shape[1]
    m = [np.zeros_like(a) for a in p]
    v = [np.zeros_like(a) for a in p]
    g = [np.empty_like(a) for a in p]
    loss, logits = np.zeros(1, f32), np.empty((N, C), f32)
    for s in range(1, steps + 1):
        rc = o.orc_mlp_train_step(x, t, 1, N, D, Hd, C, *p, m[0], v[0], m[1], v[1], m[2], v[2], m[3], v[3], s,
                                  1e-3, 0.9, 0.999, 1e-8, 1e-4, loss, *g, logits)
        assert rc == 0
    return p, g, loss, logits


@pytest.mark.parametrize("steps", [1, 2])
def test_mlp_train_step_fixture_bit_exact(steps):
    p, g, loss, logits = _mlp_oracle(steps)
    for a, k in zip(p, ("W1", "b1", "W2", "b2")):
        assert np.array_equal(a, G[f"mlp{steps}_{k}"]), k
    for a, k in zip(g, ("gW1", "gb1", "gW2", "gb2")):
        assert np.array_equal(a, G[f"mlp{steps}_{k}"]), k
    assert np.array_equal(loss, G[f"mlp{steps}_loss"]) and np.array_equal(logits, G[f"mlp{steps}_logits"])


def test_cnn_train_step_fixture_bit_exact():
    names = ("Wc1", "bc1", "Wc2", "bc2", "Wl1", "bl1", "Wl2", "bl2")
    x, t = G["cnn_x"], G["cnn_t"]
    p = [G[f"cnn_{k}"].copy() for k in names]
    N, _, S, _ = x.shape
    C1, C2, Hd, Cc = p[0].shape[0], p[2].shape[0], p[4].shape[1], p[6].shape[1]
    g = [np.empty_like(a) for a in p]
    loss, logits = np.zeros(1, f32), np.empty((N, Cc), f32)
    idx1 = np.empty((N, C1, S // 2, S // 2), np.uint64)
    idx2 = np.empty((N, C2, S // 4, S // 4), np.uint64)
    assert o.orc_cnn_train_step(x, t, 0, N, S, C1, C2, Hd, Cc, *p, 0.01, loss, idx1, idx2, *g, logits) == 0
    for a, ga, k in zip(p, g, names):
        assert np.array_equal(ga, G[f"cnn1_g{k}"]), k
        assert np.array_equal(a, G[f"cnn1_{k}"]), k
    assert np.array_equal(loss, G["cnn1_loss"]) and np.array_equal(logits, G["cnn1_logits"])


@needs_ref
def test_against_compiled_reference_fresh_inputs():
    r = ol.ref()
    rng = np.random.default_rng(7)
    # GEMM fwd+bwd incl. the MLP's skinny shapes at reduced M
    for m, k, n in ((33, 47, 29), (64, 784, 100), (64, 100, 10), (1, 5, 1)):
        x, w, gy = (rng.standard_normal(s, dtype=f32) for s in ((m, k), (k, n), (m, n)))
        y, gx, gw = np.empty((m, n), f32), np.empty((m, k), f32), np.empty((k, n), f32)
        assert r.odl_ref_matmul_fwd_bwd(x, w, gy, y, gx, gw, m, k, n) == 0
        y2, gx2, gw2 = np.empty_like(y), np.empty_like(gx), np.empty_like(gw)
        o.orc_matmul(x, w, y2, m, n, k)
        o.orc_matmul_backward(x, w, gy, gx2, gw2, m, k, n)
        assert np.array_equal(y, y2) and np.array_equal(gx, gx2) and np.array_equal(gw, gw2)
    # batched
    a, b = rng.standard_normal((3, 4, 5), dtype=f32), rng.standard_normal((3, 5, 6), dtype=f32)
    c, c2 = np.empty((3, 4, 6), f32), np.empty((3, 4, 6), f32)
    assert r.odl_ref_matmul_batched(a, b, c, 3, 4, 6, 5, 1) == 0
    o.orc_matmul_batched(a, b, c2, 3, 4, 6, 5, 1)
    assert np.array_equal(c, c2)
    assert r.odl_ref_matmul_batched(a, b[0].copy(), c, 3, 4, 6, 5, 0) == 0
    o.orc_matmul_batched(a, b[0].copy(), c2, 3, 4, 6, 5, 0)
    assert np.array_equal(c, c2)
    # transpose of a 3-D tensor's last two dims
    t3, d, d2 = rng.standard_normal((2, 3, 5), dtype=f32), np.empty((2, 5, 3), f32), np.empty((2, 5, 3), f32)
    assert r.odl_ref_transpose(t3, d, ol.shape_arr(t3.shape), 3) == 0
    o.orc_transpose(t3, d2, 2, 3, 5)
    assert np.array_equal(d, d2)
    # a conv case of config C2's geometry (stride 2, pad 1) at reduced channel counts
    N, C, H, W, OC = 2, 6, 12, 12, 8
    x, w = rng.standard_normal((N, C, H, W), dtype=f32), rng.standard_normal((OC, C, 3, 3), dtype=f32)
    b, gy = rng.standard_normal(OC, dtype=f32), rng.standard_normal((N, OC, 6, 6), dtype=f32)
    gx, gw, gb = np.empty_like(x), np.empty_like(w), np.empty_like(b)
    assert r.odl_ref_conv2d_backward(gy, x, w, b, N, C, H, W, OC, 3, 3, 2, 2, 1, 1, gx, gw, gb) == 0
    gx2, gw2, gb2 = run_conv2d_backward(gy, x, w, (2, 2), (1, 1))
    assert np.array_equal(gx, gx2) and np.array_equal(gw, gw2) and np.array_equal(gb, gb2)
    # accuracy / argmax with ties
    y = rng.integers(0, 3, size=(50, 6)).astype(f32)
    t = rng.integers(0, 6, size=50).astype(np.int32)
    acc = np.zeros(1, f32)
    assert r.odl_ref_accuracy(y, t, 50, 6, acc) == 0
    assert acc[0] == o.orc_accuracy(y, t, 50, 6)


def test_argmax_rows_is_the_first_maximum():
    # src/utils/metrics.cpp:40-53: the scan starts at column 0 and moves on strict > only, so among equal maxima the
    # first wins — which is numpy's argmax; accuracy is then the mean of (argmax == label) in float
    o = ol.oracle()
    rng = np.random.default_rng(77)
    y = rng.integers(0, 3, size=(400, 7)).astype(f32)  # three distinct values in seven columns: ties in every row
    y[::5, 0] = 2  # maximum in the first column
    y[1::5, :] = -1.5  # a whole row of equal values
    y[2::5, 6] = 9  # maximum in the last column only
    am = np.full(400, -1, np.int64)
    o.orc_argmax_rows(y, 400, 7, am)
    assert np.array_equal(am, np.argmax(y, axis=1))
    assert (am[1::5] == 0).all() and (am[2::5] == 6).all()
    t = rng.integers(0, 7, size=400).astype(np.int32)
    assert o.orc_accuracy(y, t, 400, 7) == f32((np.argmax(y, axis=1) == t).sum()) / f32(400)
    one = np.array([[3.0]], f32)
    o.orc_argmax_rows(one, 1, 1, am)
    assert am[0] == 0


BN_CASES = {"bnA": (6, 5, 0, 0), "bnB": (3, 4, 5, 6), "bnC": (1, 2, 3, 3), "bnD": (4, 3, 2, 2)}


def bn_forward(x, gamma, beta, rm, rv, training, eps=1e-5, want_xn=True):
    N, C = x.shape[:2]
    P = int(np.prod(x.shape[2:])) if x.ndim == 4 else 1
    y, xn = np.empty_like(x), np.empty_like(x)
    mean, var = np.empty(C, f32), np.empty(C, f32)
    assert o.orc_batch_norm_forward(x, gamma, beta, rm, rv, training, eps, N, C, P, y, mean, var,
                                    xn if want_xn else None) == 0
    return y, mean, var, xn


def bn_backward(gy, gamma, var, xn, eps=1e-5):
    N, C = gy.shape[:2]
    P = int(np.prod(gy.shape[2:])) if gy.ndim == 4 else 1
    gx, dg, db = np.empty_like(gy), np.empty(C, f32), np.empty(C, f32)
    assert o.orc_batch_norm_backward(gy, gamma, var, xn, eps, N, C, P, gx, dg, db) == 0
    return gx, dg, db


@pytest.mark.parametrize("name", list(BN_CASES))
def test_batch_norm_fixtures_bit_exact(name):
    # written from the compiled reference (Mat::batch_norm_forward / batch_norm / batch_norm_backward and the layers)
    g = lambda k: G[f"{name}_{k}"]
    x, gamma, beta, rm, rv = g("x"), g("gamma"), g("beta"), g("rm"), g("rv")
    for mode, training in (("train", 1), ("eval", 0)):
        y, mean, var, xn = bn_forward(x, gamma, beta, rm, rv, training)
        for got, key in ((y, "y"), (mean, "mean"), (var, "var"), (xn, "xn")):
            assert np.array_equal(got, g(f"{mode}_{key}")), (mode, key)
        assert np.array_equal(bn_forward(x, gamma, beta, rm, rv, training, want_xn=False)[0], y)
    gx, dg, db = bn_backward(g("gy"), gamma, g("train_var"), g("train_xn"))
    assert np.array_equal(gx, g("gx")) and np.array_equal(dg, g("dgamma")) and np.array_equal(db, g("dbeta"))
    # the layers: three training forwards of x*(1 + 0.25*step) from running mean 0 / variance 1, each folding the batch
    # statistics in as running = 0.1*running + 0.9*batch (batch_norm2d.cpp:77-80), then an evaluation forward of x
    C = x.shape[1]
    ones, zeros = np.ones(C, f32), np.zeros(C, f32)
    rmean, rvar = zeros.copy(), ones.copy()
    for step in range(3):
        xs = (x * f32(1.0 + 0.25 * step)).astype(f32)
        y, mean, var, _ = bn_forward(xs, ones, zeros, rmean, rvar, 1)
        rmean = f32(0.1) * rmean + (f32(1.0) - f32(0.1)) * mean
        rvar = f32(0.1) * rvar + (f32(1.0) - f32(0.1)) * var
    assert np.array_equal(y, g("layer_ytrain"))
    assert np.array_equal(bn_forward(x, ones, zeros, rmean, rvar, 0)[0], g("layer_yeval"))


@needs_ref
def test_batch_norm_against_compiled_reference_fresh_inputs():
    r = ol.ref()
    rng = np.random.default_rng(17)
    for N, C, H, W in ((7, 3, 0, 0), (2, 5, 4, 7), (5, 1, 1, 1), (3, 6, 9, 9)):
        xs = (N, C) if H == 0 else (N, C, H, W)
        x = rng.standard_normal(xs, dtype=f32)
        gamma, beta, rm = (rng.standard_normal(C, dtype=f32) for _ in range(3))
        rv = (rng.random(C, dtype=f32) + f32(0.1)).astype(f32)
        gy = rng.standard_normal(xs, dtype=f32)
        for training in (1, 0):
            y, xn, mean, var = np.empty(xs, f32), np.empty(xs, f32), np.empty(C, f32), np.empty(C, f32)
            assert r.odl_ref_batch_norm_forward(x, gamma, beta, rm, rv, training, 1e-3, N, C, H, W, y, mean, var, xn) == 0
            y2, mean2, var2, xn2 = bn_forward(x, gamma, beta, rm, rv, training, eps=1e-3)
            assert all(np.array_equal(a, b) for a, b in ((y, y2), (mean, mean2), (var, var2), (xn, xn2)))
        gx, dg, db = np.empty(xs, f32), np.empty(C, f32), np.empty(C, f32)
        assert r.odl_ref_batch_norm_backward(gy, x, gamma, mean2, var2, xn2, 1e-3, N, C, H, W, gx, dg, db) == 0
        gx2, dg2, db2 = bn_backward(gy, gamma, var2, xn2, eps=1e-3)
        assert np.array_equal(gx, gx2) and np.array_equal(dg, dg2) and np.array_equal(db, db2)

# ------------------------------------------------------------------------ 3. independent mathematics
def test_batch_norm_against_float64_and_finite_differences():
    rng = np.random.default_rng(18)
    x = (rng.standard_normal((8, 3, 5, 7)) * 3 + 1).astype(f32)
    gamma, beta = rng.standard_normal(3).astype(f32), rng.standard_normal(3).astype(f32)
    y, mean, var, xn = bn_forward(x, gamma, beta, np.zeros(3, f32), np.ones(3, f32), 1)
    x64 = x.astype(np.float64)
    np.testing.assert_allclose(mean, x64.mean(axis=(0, 2, 3)), rtol=1e-5)
    np.testing.assert_allclose(var, x64.var(axis=(0, 2, 3)), rtol=1e-5)  # the biased (population) variance
    # normalised activations have zero mean and (almost) unit variance per channel whatever the input's scale
    assert np.abs(xn.astype(np.float64).mean(axis=(0, 2, 3))).max() < 1e-6
    np.testing.assert_allclose(xn.astype(np.float64).var(axis=(0, 2, 3)), var / (var + 1e-5), rtol=1e-5)
    np.testing.assert_allclose(y, gamma[None, :, None, None] * xn + beta[None, :, None, None], rtol=1e-6, atol=1e-6)

    def loss64(xv, gv, bv, r):
        m, v = xv.mean(axis=(0, 2, 3), keepdims=True), xv.var(axis=(0, 2, 3), keepdims=True)
        return float((((xv - m) / np.sqrt(v + 1e-5) * gv[None, :, None, None] + bv[None, :, None, None]) * r).sum())

    r = rng.standard_normal(x.shape)
    gx, dg, db = bn_backward(r.astype(f32), gamma, var, xn)
    g64, b64 = gamma.astype(np.float64), beta.astype(np.float64)
    h = 1e-4
    for idx in [(0, 0, 0, 0), (3, 1, 2, 5), (7, 2, 4, 6)]:  # the statistics depend on x: the full Jacobian is checked
        xp, xm = x64.copy(), x64.copy()
        xp[idx] += h
        xm[idx] -= h
        fd = (loss64(xp, g64, b64, r) - loss64(xm, g64, b64, r)) / (2 * h)
        assert abs(gx[idx] - fd) <= 2e-3 * max(1.0, abs(fd)), (idx, gx[idx], fd)
    for c in range(3):
        gp, gm = g64.copy(), g64.copy()
        gp[c] += h
        gm[c] -= h
        assert abs(dg[c] - (loss64(x64, gp, b64, r) - loss64(x64, gm, b64, r)) / (2 * h)) <= 1e-3 * max(1.0, abs(dg[c]))
        np.testing.assert_allclose(db[c], r[:, c].sum(), rtol=1e-4, atol=1e-4)
    # evaluation mode is a per-channel affine map of x with the running statistics
    rm, rv = rng.standard_normal(3).astype(f32), (rng.random(3) + 0.5).astype(f32)
    ye = bn_forward(x, gamma, beta, rm, rv, 0)[0]
    want = (x64 - rm[None, :, None, None]) / np.sqrt(rv[None, :, None, None].astype(np.float64) + 1e-5)
    np.testing.assert_allclose(ye, want * g64[None, :, None, None] + b64[None, :, None, None], rtol=1e-5, atol=1e-5)



def test_matmul_against_float64():
    rng = np.random.default_rng(1)
    a, b = rng.standard_normal((37, 211), dtype=f32), rng.standard_normal((211, 19), dtype=f32)
    c = np.empty((37, 19), f32)
    o.orc_matmul(a, b, c, 37, 19, 211)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    bound = 1e-5 * np.outer(np.linalg.norm(a, axis=1), np.linalg.norm(b, axis=0))
    assert (np.abs(c - ref) <= bound).all()
    rows = np.empty((5, 19), f32)
    o.orc_matmul_rows(a, b, rows, 10, 15, 19, 211)
    assert np.array_equal(rows, c[10:15])
    gy = rng.standard_normal((37, 19), dtype=f32)
    gx, gw = np.empty_like(a), np.empty_like(b)
    o.orc_matmul_backward(a, b, gy, gx, gw, 37, 211, 19)
    np.testing.assert_allclose(gx, gy.astype(np.float64) @ b.T.astype(np.float64), rtol=0, atol=2e-5 * 19)
    np.testing.assert_allclose(gw, a.T.astype(np.float64) @ gy.astype(np.float64), rtol=0, atol=2e-5 * 37)


def direct_conv(x, w, b, s, p):
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (p[0], p[0]), (p[1], p[1])))
    OH, OW = conv_out(H, KH, s[0], p[0]), conv_out(W, KW, s[1], p[1])
    y = np.zeros((N, OC, OH, OW))
    for oh in range(OH):
        for ow in range(OW):
            win = xp[:, :, oh * s[0]:oh * s[0] + KH, ow * s[1]:ow * s[1] + KW]
            y[:, :, oh, ow] = np.einsum("nckl,ockl->no", win, w.astype(np.float64))
    return y + (0 if b is None else b.astype(np.float64)[None, :, None, None])


@pytest.mark.parametrize("s,p,k", [((1, 1), (1, 1), (3, 3)), ((2, 2), (1, 1), (3, 3)), ((2, 1), (0, 2), (2, 3))])
def test_conv_forward_against_direct_convolution(s, p, k):
    rng = np.random.default_rng(3)
    x, w = rng.standard_normal((2, 3, 9, 8), dtype=f32), rng.standard_normal((4, 3) + k, dtype=f32)
    b = rng.standard_normal(4, dtype=f32)
    np.testing.assert_allclose(run_conv2d(x, w, b, s, p), direct_conv(x, w, b, s, p), atol=1e-4)


def test_conv_backward_is_the_true_gradient_when_the_view_is_harmless():
    # With OC == 1 the [N,OC,OH,OW] -> [N*OH*OW, OC] view is the identity permutation, so the reference's
    # gW/gx are the mathematical gradients; check them against the adjoint of the direct convolution.
    rng = np.random.default_rng(4)
    x, w = rng.standard_normal((2, 3, 7, 7), dtype=f32), rng.standard_normal((1, 3, 3, 3), dtype=f32)
    s, p = (2, 2), (1, 1)
    y = direct_conv(x, w, None, s, p)
    gy = rng.standard_normal(y.shape).astype(f32)
    gx, gw, gb = run_conv2d_backward(gy, x, w, s, p)
    eps = 1e-3
    for _ in range(6):  # <gy, conv(x + eps*e_i)> - <gy, conv(x)> = eps * gx_i  (conv is linear in x and in w)
        i = tuple(rng.integers(0, d) for d in x.shape)
        xe = x.astype(np.float64).copy()
        xe[i] += eps
        assert abs(((direct_conv(xe, w, None, s, p) - y) * gy).sum() / eps - gx[i]) < 1e-3
        j = tuple(rng.integers(0, d) for d in w.shape)
        we = w.astype(np.float64).copy()
        we[j] += eps
        assert abs(((direct_conv(x, we, None, s, p) - y) * gy).sum() / eps - gw[j]) < 1e-3
    np.testing.assert_allclose(gb, gy.astype(np.float64).sum(axis=(0, 2, 3)), atol=1e-4)


@pytest.mark.parametrize("to_matrix", [0, 1])
def test_im2col_col2im_are_adjoint(to_matrix):
    rng = np.random.default_rng(5)
    N, C, H, W, KH, KW, SH, SW, PH, PW = 2, 3, 7, 6, 3, 2, 2, 1, 1, 1
    OH, OW = conv_out(H, KH, SH, PH), conv_out(W, KW, SW, PW)
    x = rng.standard_normal((N, C, H, W), dtype=f32)
    c = rng.standard_normal((N * OH * OW, C * KH * KW) if to_matrix else (N, C, KH, KW, OH, OW), dtype=f32)
    col, im = np.empty_like(c), np.empty_like(x)
    assert o.orc_im2col(x, N, C, H, W, KH, KW, SH, SW, PH, PW, to_matrix, col) == 0
    assert o.orc_col2im(c, N, C, H, W, KH, KW, SH, SW, PH, PW, to_matrix, im) == 0
    assert abs((col.astype(np.float64) * c).sum() - (x.astype(np.float64) * im).sum()) < 1e-3
    # the two layouts hold the same numbers, permuted
    if to_matrix:
        col6 = np.empty((N, C, KH, KW, OH, OW), f32)
        o.orc_im2col(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 0, col6)
        assert np.array_equal(col.reshape(N, OH, OW, C, KH, KW).transpose(0, 3, 4, 5, 1, 2), col6)


def test_sum_to_is_left_aligned_numpy_sum():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((3, 4, 5), dtype=f32)
    for ts, axes in (((1, 4, 5), (0,)), ((3, 1, 5), (1,)), ((3, 4, 1), (2,)), ((3, 1), (1, 2)), ((1, 4), (0, 2))):
        dst = np.empty(int(np.prod(ts)), f32)
        assert o.orc_sum_to(x, ol.shape_arr(x.shape), 3, ol.shape_arr(ts), len(ts), dst) == 0
        np.testing.assert_allclose(dst, x.astype(np.float64).sum(axis=axes).ravel(), atol=1e-5)


def test_softmax_rows_and_loss_closed_forms():
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((9, 13), dtype=f32) * 4).astype(f32)
    p = np.empty_like(x)
    o.orc_softmax(x, 9, 13, 1, p)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, atol=1e-6)
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    np.testing.assert_allclose(p, e / e.sum(axis=1, keepdims=True), atol=1e-6)
    t = rng.integers(0, 13, size=9).astype(np.int64)
    loss, gx = np.zeros(1, f32), np.empty_like(x)
    o.orc_softmax_ce_loss(x, t, 1, 9, 13, loss)
    sm = e / e.sum(axis=1, keepdims=True)
    assert abs(loss[0] + np.log(sm[np.arange(9), t] + 1e-8).mean()) < 1e-5
    o.orc_softmax_ce_grad(x, t, 1, 9, 13, 2.0, gx)
    oh = np.eye(13)[t]
    np.testing.assert_allclose(gx, (sm - oh) * (2.0 / 9), atol=1e-6)
    assert abs(gx.sum()) < 1e-5  # rows of softmax - one_hot sum to zero
    # softmax along a middle axis (outer, axis, inner)
    x3 = rng.standard_normal((2, 5, 3), dtype=f32)
    p3 = np.empty_like(x3)
    o.orc_softmax(x3, 2, 5, 3, p3)
    e3 = np.exp(x3.astype(np.float64) - x3.max(axis=1, keepdims=True))
    np.testing.assert_allclose(p3, e3 / e3.sum(axis=1, keepdims=True), atol=1e-6)


def test_max_pool_brute_force_with_ties_and_padding():
    rng = np.random.default_rng(9)
    N, C, H, W, K, S, P = 2, 2, 6, 6, 3, 2, 1
    x = rng.integers(-2, 2, size=(N, C, H, W)).astype(f32)
    OH = conv_out(H, K, S, P)
    y, idx = np.empty((N, C, OH, OH), f32), np.empty((N, C, OH, OH), np.uint64)
    assert o.orc_max_pool2d(x, N, C, H, W, K, K, S, S, P, P, y, idx) == 0
    xp = np.pad(x, ((0, 0), (0, 0), (P, P), (P, P)))  # zero padding, not -inf
    for n in range(N):
        for c in range(C):
            for oh in range(OH):
                for ow in range(OH):
                    win = xp[n, c, oh * S:oh * S + K, ow * S:ow * S + K].ravel()
                    assert y[n, c, oh, ow] == win.max()
                    assert idx[n, c, oh, ow] == int(np.argmax(win))  # numpy argmax = first maximum
    gy = rng.standard_normal(y.shape, dtype=f32)
    gx = np.empty_like(x)
    o.orc_max_pool2d_backward(gy, idx, N, C, H, W, K, K, S, S, P, P, gx)
    # gradient mass is conserved except where the maximum was a padding cell
    exp = np.zeros_like(xp, dtype=np.float64)
    for n in range(N):
        for c in range(C):
            for oh in range(OH):
                for ow in range(OH):
                    kh, kw = divmod(int(idx[n, c, oh, ow]), K)
                    exp[n, c, oh * S + kh, ow * S + kw] += gy[n, c, oh, ow]
    np.testing.assert_allclose(gx, exp[:, :, P:-P, P:-P], atol=1e-6)


def test_broadcast_is_right_aligned():
    x = np.array([1, 2], f32)
    y = np.empty((2, 2), f32)
    o.orc_broadcast_to(x, ol.shape_arr((2,)), 1, ol.shape_arr((2, 2)), 2, y)
    assert np.array_equal(y, np.broadcast_to(x, (2, 2)))
    x = np.arange(3, dtype=f32).reshape(3, 1)
    y = np.empty((2, 3, 4), f32)
    o.orc_broadcast_to(x, ol.shape_arr((3, 1)), 2, ol.shape_arr((2, 3, 4)), 3, y)
    assert np.array_equal(y, np.broadcast_to(x, (2, 3, 4)))


def test_adam_step_closed_form():
    # one Adam step from zero moments: m_hat = g, v_hat = g^2, update = lr * g / (|g| + eps) (+ weight decay in g)
    p, g_, loss, _ = _mlp_oracle(1)
    W2, gW2 = G["mlp_W2"].astype(np.float64), g_[2].astype(np.float64)
    g = gW2 + 1e-4 * W2
    np.testing.assert_allclose(p[2], W2 - 1e-3 * g / (np.abs(g) + 1e-8), atol=2e-7)


# ------------------------------------------------------------------ detector forward path (config 5's operators)
def _detect_inputs(name):
    aH, aW = G[f"{name}_anchor_grid"].shape[2:4]
    return (G["det_x"], G["det_w"], G["det_b"] if name == "detA" else None, G["det_grid"], G[f"{name}_anchor_grid"],
            int(aH), int(aW))


def test_detector_ops_fixtures_bit_exact():
    o = ol.oracle()
    x = G["det_act_x"]
    for op, nm in ((6, "sigmoid"), (7, "silu")):
        got = np.empty_like(x)
        o.orc_unary(op, x, x.size, got)
        assert np.array_equal(got, G[f"det_{nm}"]), nm
    xu = G["det_up_x"]
    for nm, (sh, sw) in (("up22", (2, 2)), ("up13", (1, 3))):
        got = np.empty((2, 3, 4 * sh, 5 * sw), f32)
        assert o.orc_upsample_nearest(xu, 2, 3, 4, 5, 4 * sh, 5 * sw, sh, sw, got) == 0
        assert np.array_equal(got, G[f"det_{nm}"]), nm
    parts = [G[f"det_cat_in{i}"] for i in range(3)]
    got = np.empty((3, 8, 7), f32)
    assert o.orc_cat(ol.ptr_arr(parts), np.asarray([2, 5, 1], np.int64), 3, 3, 7, got) == 0
    assert np.array_equal(got, G["det_cat"])
    for name in ("detA", "detB"):
        xd, wd, bd, grid, ag, aH, aW = _detect_inputs(name)
        got = np.empty_like(G[f"{name}_out"])
        assert o.orc_yolo_detect_forward(xd, wd, bd, grid, grid.size, ag, ag.size, aH, aW, 2, 6, 4, 5, 8.0, 3, 2, got) == 0
        assert np.array_equal(got, G[f"{name}_out"]), name


def test_detector_ops_against_plain_numpy():
    """The same operators written independently: float64 formulas, np.repeat, np.concatenate, an einsum for the 1x1
    convolution followed by the published YOLOv5 decoding (xy = (2s + grid) * stride, wh = (2s)^2 * anchor)."""
    o = ol.oracle()
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(1000, dtype=f32) * f32(4)).astype(f32)
    sg, si = np.empty_like(x), np.empty_like(x)
    o.orc_unary(6, x, x.size, sg)
    o.orc_unary(7, x, x.size, si)
    x64 = x.astype(np.float64)
    np.testing.assert_allclose(sg, 1 / (1 + np.exp(-x64)), rtol=3e-7)
    np.testing.assert_allclose(si, x64 / (1 + np.exp(-x64)), rtol=3e-7, atol=1e-30)
    xu = rng.standard_normal((2, 3, 5, 4), dtype=f32)
    up = np.empty((2, 3, 15, 8), f32)
    assert o.orc_upsample_nearest(xu, 2, 3, 5, 4, 15, 8, 3, 2, up) == 0
    assert np.array_equal(up, np.repeat(np.repeat(xu, 3, axis=2), 2, axis=3))
    assert o.orc_upsample_nearest(xu, 2, 3, 5, 4, 16, 8, 3, 2, np.empty((2, 3, 16, 8), f32)) == -1  # row 15 -> input row 5
    parts = [rng.standard_normal((2, c, 3, 4), dtype=f32) for c in (4, 1, 6)]
    cat = np.empty((2, 11, 3, 4), f32)
    assert o.orc_cat(ol.ptr_arr(parts), np.asarray([4, 1, 6], np.int64), 3, 2, 12, cat) == 0
    assert np.array_equal(cat, np.concatenate(parts, axis=1))
    N, C, H, W, A, NC = 2, 5, 3, 4, 3, 4
    CI = NC + 5
    xd = rng.standard_normal((N, C, H, W), dtype=f32)
    wd = rng.standard_normal((A * CI, C, 1, 1), dtype=f32)
    bd = rng.standard_normal(A * CI, dtype=f32)
    gyy, gxx = np.meshgrid(np.arange(H), np.arange(W), indexing="ij")
    grid = np.broadcast_to(np.stack([gxx, gyy], -1).astype(f32) - f32(0.5), (1, A, H, W, 2)).copy()
    anchors = (rng.random((A, 2), dtype=f32) * f32(20) + f32(2)).astype(f32)
    ag = np.broadcast_to(anchors.reshape(1, A, 1, 1, 2), (1, A, H, W, 2)).copy()
    got = np.empty((N, A * H * W, CI), f32)
    assert o.orc_yolo_detect_forward(xd, wd, bd, grid, grid.size, ag, ag.size, H, W, N, C, H, W, 16.0, A, NC, got) == 0
    conv = np.einsum("nchw,oc->nohw", xd.astype(np.float64), wd[:, :, 0, 0].astype(np.float64)) + bd[None, :, None, None]
    s = 1 / (1 + np.exp(-conv.reshape(N, A, CI, H, W).transpose(0, 1, 3, 4, 2)))
    want = s.copy()
    want[..., 0:2] = (s[..., 0:2] * 2 + grid) * 16.0
    want[..., 2:4] = (s[..., 2:4] * 2) ** 2 * ag
    np.testing.assert_allclose(got, want.reshape(N, A * H * W, CI), rtol=2e-5, atol=2e-6)
