"""The C++ host layer (origindl_amd/host: Mat / Tensor / Operator / nn / optim over the C ABI) driven through
tests/api_driver.cpp — the very driver source that, compiled against the reference, produced the fixtures.
Same calls, two backends: here they run on the gfx950 backend and are compared with the reference's outputs
(tests/golden/ref_vectors.npz) and with the CPU oracle.

Bars: indices and data movement bit-exact; GEMM/conv outputs within 1e-5*|a_row|*|b_col|; training-step loss within
1e-4 relative (the benchmark contract), gradients and updated parameters within the GEMM bound of their products."""
import os

import numpy as np
import pytest

import oraclelib as ol

pytestmark = pytest.mark.gpu

f32 = np.float32
G = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors.npz"))


@pytest.fixture(scope="module")
def h():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return ol.host_driver()


@pytest.fixture(scope="module")
def o():
    return ol.oracle()


def test_tensor_level_matmul_forward_backward(h, o):
    # tests/unit_test/operator/test_matmul.cpp:119-143 through Tensor::backward()
    x, w, gy = np.array([1, 2, 3, 4], f32), np.array([5, 6, 7, 8], f32), np.ones(4, f32)
    y, gx, gw = np.empty(4, f32), np.empty(4, f32), np.empty(4, f32)
    assert h.odl_host_matmul_fwd_bwd(x, w, gy, y, gx, gw, 2, 2, 2) == 0
    assert y.tolist() == [19, 22, 43, 50] and gx.tolist() == [11, 15, 11, 15] and gw.tolist() == [4, 4, 6, 6]
    rng = np.random.default_rng(0)
    for m, k, n in ((64, 784, 100), (33, 47, 29), (128, 256, 128)):
        x, w, gy = (rng.standard_normal(s, dtype=f32) for s in ((m, k), (k, n), (m, n)))
        y, gx, gw = np.empty((m, n), f32), np.empty((m, k), f32), np.empty((k, n), f32)
        assert h.odl_host_matmul_fwd_bwd(x, w, gy, y, gx, gw, m, k, n) == 0
        yo, gxo, gwo = np.empty_like(y), np.empty_like(gx), np.empty_like(gw)
        o.orc_matmul(x, w, yo, m, n, k)
        o.orc_matmul_backward(x, w, gy, gxo, gwo, m, k, n)
        nrm = np.linalg.norm
        assert (np.abs(y - yo) <= 1e-5 * np.outer(nrm(x, axis=1), nrm(w, axis=0))).all()
        assert (np.abs(gx - gxo) <= 1e-5 * np.outer(nrm(gy, axis=1), nrm(w, axis=1))).all()
        assert (np.abs(gw - gwo) <= 1e-5 * np.outer(nrm(x, axis=0), nrm(gy, axis=0))).all()


CONV_CASES = {"convA": ((1, 1), (1, 1)), "convB": ((2, 2), (1, 1)), "convC": ((1, 1), (0, 0)),
              "convD": ((2, 1), (0, 2)), "convE": ((1, 1), (0, 0))}


@pytest.mark.parametrize("name", sorted(CONV_CASES))
def test_conv_operator_matches_reference_fixtures(h, name):
    s, p = CONV_CASES[name]
    x, w, gy = G[f"{name}_x"], G[f"{name}_w"], G[f"{name}_gy"]
    b = G[f"{name}_b"] if f"{name}_b" in G else None
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    y = np.empty_like(G[f"{name}_y"])
    assert h.odl_host_conv2d(x, w, b, N, C, H, W, OC, KH, KW, s[0], s[1], p[0], p[1], y) == 0
    np.testing.assert_allclose(y, G[f"{name}_y"], atol=2e-5 * np.abs(G[f"{name}_y"]).max(), rtol=0)
    gx, gw, gb = np.empty_like(x), np.empty_like(w), np.empty((OC,), f32)
    assert h.odl_host_conv2d_backward(gy, x, w, b, N, C, H, W, OC, KH, KW, s[0], s[1], p[0], p[1], gx, gw,
                                      gb if b is not None else None) == 0
    np.testing.assert_allclose(gx, G[f"{name}_gx"], atol=2e-5 * max(np.abs(G[f"{name}_gx"]).max(), 1), rtol=0)
    np.testing.assert_allclose(gw, G[f"{name}_gw"], atol=2e-5 * max(np.abs(G[f"{name}_gw"]).max(), 1), rtol=0)
    if b is not None:
        np.testing.assert_allclose(gb, G[f"{name}_gb"], atol=2e-5 * max(np.abs(G[f"{name}_gb"]).max(), 1), rtol=0)
    col = np.empty_like(G[f"{name}_col"])
    assert h.odl_host_im2col(x, N, C, H, W, KH, KW, s[0], s[1], p[0], p[1], 1, col) == 0
    assert np.array_equal(col, G[f"{name}_col"])
    im = np.empty_like(x)
    g6 = G[f"{name}_gcol6"]
    assert h.odl_host_col2im(g6, ol.shape_arr(g6.shape), 6, N, C, H, W, KH, KW, s[0], s[1], p[0], p[1], 0, im) == 0
    assert np.array_equal(im, G[f"{name}_im6"])


POOL_CASES = {"poolA": (2, 2, 2, 2, 0, 0), "poolB": (3, 3, 2, 2, 1, 1), "poolC": (5, 5, 1, 1, 2, 2),
              "poolD": (3, 2, 1, 2, 1, 0)}


@pytest.mark.parametrize("name", sorted(POOL_CASES))
def test_max_pool_through_the_mat_interface_bit_exact(h, name):
    KH, KW, SH, SW, PH, PW = POOL_CASES[name]
    x = G[f"{name}_x"]
    N, C, H, W = x.shape
    y, idx = np.empty_like(G[f"{name}_y"]), np.empty_like(G[f"{name}_idx"])
    assert h.odl_host_max_pool2d(x, N, C, H, W, KH, KW, SH, SW, PH, PW, y, idx) == 0  # std::vector<size_t> round trip
    assert np.array_equal(y, G[f"{name}_y"]) and np.array_equal(idx, G[f"{name}_idx"])
    gx = np.empty_like(x)
    assert h.odl_host_max_pool2d_backward(G[f"{name}_gy"], idx, N, C, H, W, KH, KW, SH, SW, PH, PW, gx) == 0
    assert np.array_equal(gx, G[f"{name}_gx"])


def test_sum_to_broadcast_and_error_codes(h):
    for name in sorted(k[:-3] for k in G.files if k.startswith("sumto") and k.endswith("_rc")):
        x, ts, rc = G[f"{name}_x"], G[f"{name}_t"], int(G[f"{name}_rc"])
        dst = np.zeros_like(G[f"{name}_y"])
        got = h.odl_host_sum_to(x, ol.shape_arr(x.shape), x.ndim, ts, len(ts), dst)
        assert (got == 0) == (rc == 0), name  # same calls succeed / throw as in the reference
        if rc == -2:
            assert got == -2, name            # runtime_error for a larger target (test_sum_to.cpp:53-60)
        if rc == 0:
            np.testing.assert_allclose(dst, G[f"{name}_y"], atol=1e-5, rtol=1e-6)
    for name in ("bcastA", "bcastB", "bcastC"):
        x, ds, g = G[f"{name}_x"], G[f"{name}_d"], G[f"{name}_g"]
        y = np.empty_like(G[f"{name}_y"])
        assert h.odl_host_broadcast_to(x, ol.shape_arr(x.shape), x.ndim, ds, len(ds), y) == 0
        assert np.array_equal(y, G[f"{name}_y"])
        gx = np.zeros_like(G[f"{name}_gx"])
        rc = h.odl_host_broadcast_to_backward(x, ol.shape_arr(x.shape), x.ndim, ds, len(ds), g, gx)
        assert (rc == 0) == (int(G[f"{name}_rc"]) == 0)
        if rc == 0:
            np.testing.assert_allclose(gx, G[f"{name}_gx"], atol=1e-5)
    for name in ("sumA", "sumB", "sumC", "sumD"):
        x, axis = G[f"{name}_x"], int(G[f"{name}_axis"])
        y, mx = np.empty_like(G[f"{name}_y"]), np.empty_like(G[f"{name}_max"])
        assert h.odl_host_sum(x, ol.shape_arr(x.shape), x.ndim, axis, 0, y) == 0
        assert h.odl_host_max(x, ol.shape_arr(x.shape), x.ndim, axis, mx) == 0
        np.testing.assert_allclose(y, G[f"{name}_y"], atol=1e-5 * np.sqrt(x.size) * 4, rtol=0)
        assert np.array_equal(mx, G[f"{name}_max"])


def test_softmax_ce_operator_and_label_errors(h):
    for name, is64 in (("ceA", 0), ("ceB", 1), ("ceC", 1)):
        x, t = G[f"{name}_x"], G[f"{name}_t"]
        N, C = x.shape
        loss, gx, p = np.zeros(1, f32), np.empty_like(x), np.empty_like(x)
        assert h.odl_host_softmax_ce(x, t, is64, N, C, loss, gx) == 0
        assert abs(loss[0] - G[f"{name}_loss"][0]) <= 1e-4 * abs(G[f"{name}_loss"][0])
        np.testing.assert_allclose(gx, G[f"{name}_gx"], atol=1e-6)
        assert h.odl_host_softmax(x, ol.shape_arr(x.shape), 2, -1, p) == 0
        np.testing.assert_allclose(p, G[f"{name}_p"], atol=1e-6)
        sel, oh = np.empty(N, f32), np.empty((N, C), f32)
        assert h.odl_host_gather(G[f"{name}_p"], t, is64, N, C, sel) == 0 and np.array_equal(sel, G[f"{name}_sel"])
        assert h.odl_host_one_hot(t, is64, N, C, oh) == 0 and np.array_equal(oh, G[f"{name}_oh"])
    t, x = G["oob_t"], G["oob_x"]
    sel, oh, loss = np.zeros(4, f32), np.empty((4, 3), f32), np.zeros(1, f32)
    assert h.odl_host_gather(x, t, 0, 4, 3, sel) == int(G["oob_gather_rc"]) == -1
    assert h.odl_host_one_hot(t, 0, 4, 3, oh) == 0 and np.array_equal(oh, G["oob_onehot"])
    assert h.odl_host_softmax_ce(x, t, 0, 4, 3, loss, None) == int(G["oob_ce_rc"]) == -1


def test_elementwise_operators_and_accuracy(h, o):
    a, b = G["ew_a"], G["ew_b"]
    sa = ol.shape_arr(a.shape)
    for op in range(5):
        out = np.empty_like(a)
        assert h.odl_host_binary(op, a, sa, 1, b, sa, 1, out) == 0
        assert np.array_equal(out, G[f"ew_bin{op}"]), op
    for op, tol in ((0, 0), (1, 2e-7), (2, 2e-7), (3, 0), (4, 0)):
        src = np.abs(a) + f32(0.1) if op == 2 else a
        out = np.empty_like(a)
        assert h.odl_host_unary(op, src, a.size, out) == 0
        np.testing.assert_allclose(out, G[f"ew_un{op}"], rtol=tol, atol=tol / 2)
    out = np.empty_like(a)
    assert h.odl_host_pow_scalar(np.abs(a), a.size, 0.5, out) == 0
    np.testing.assert_allclose(out, G["ew_pow05"], rtol=3e-7)
    assert h.odl_host_binary(0, a, sa, 1, b[:5].copy(), ol.shape_arr((5,)), 1, out) == -2  # "complex broadcasting"
    rng = np.random.default_rng(1)
    y = rng.integers(0, 4, size=(200, 10)).astype(f32)
    t = rng.integers(0, 10, size=200).astype(np.int32)
    acc = np.zeros(1, f32)
    assert h.odl_host_accuracy(y, t, 200, 10, acc) == 0
    assert acc[0] == o.orc_accuracy(y, t, 200, 10)


def gemm_tol(*mats):
    """a loose absolute tolerance for quantities produced by a chain of products of the given matrices"""
    t = 1.0
    for m in mats:
        t *= np.sqrt((m.astype(np.float64) ** 2).sum() / max(m.shape[0], 1))
    return 2e-5 * max(t, 1e-3)


@pytest.mark.parametrize("steps", [1, 2])
def test_mlp_training_step_matches_the_reference(h, steps):
    # Sequential(Linear, ReLU, Linear) + softmax CE + WeightDecay(1e-4) + Adam(1e-3): the reference's outputs for
    # the same seeded inputs are in the fixtures (written through the same driver source).
    x, t = G["mlp_x"], G["mlp_t"]
    N, D = x.shape
    p = [G[f"mlp_{k}"].copy() for k in ("W1", "b1", "W2", "b2")]
    Hd, C = p[0].shape[1], p[2].shape[1]
    g = [np.empty_like(a) for a in p]
    loss, logits = np.zeros(1, f32), np.empty((N, C), f32)
    assert h.odl_host_mlp_train(x, t, 1, N, D, Hd, C, *p, steps, 1e-3, 0.9, 0.999, 1e-8, 1e-4, loss, *g, logits) == 0
    ref_loss = G[f"mlp{steps}_loss"][0]
    assert abs(loss[0] - ref_loss) <= 1e-4 * abs(ref_loss)
    np.testing.assert_allclose(logits, G[f"mlp{steps}_logits"], atol=1e-5)
    for a, k in zip(g, ("gW1", "gb1", "gW2", "gb2")):
        np.testing.assert_allclose(a, G[f"mlp{steps}_{k}"], atol=2e-6, rtol=1e-4)
    for a, k in zip(p, ("W1", "b1", "W2", "b2")):
        # Adam's first steps move every weight by ~lr regardless of the gradient's size, so where a gradient is
        # ~1e-8 a 1-ulp difference flips the sign of the update: compare within 2*lr there, tightly elsewhere
        ref, gref = G[f"mlp{steps}_{k}"], np.abs(G[f"mlp1_g{k}"])
        tight = gref > 1e-5
        np.testing.assert_allclose(a[tight], ref[tight], atol=2e-5 * steps)
        assert np.abs(a - ref).max() <= 2.1e-3 * steps


@pytest.mark.parametrize("wd", [1e-4, 0.0])
def test_recorded_training_step_replays_bit_for_bit(h, wd):
    """The MLP step (forward, softmax-CE, backward, weight-decay hook, Adam) recorded once into a graph and replayed
    must leave exactly what the same number of ordinary steps leaves: same kernels, same arithmetic, the loss and the
    upstream gradient read from device memory instead of passing through the host, Adam's bias-correction factors
    rewritten before every replay. Ordinary work runs between the replays (the driver queues an unrelated kernel and
    reads its result back), so a replay that depended on leftover state would show."""
    x, t = G["mlp_x"], G["mlp_t"]
    N, D = x.shape
    p0 = [G[f"mlp_{k}"] for k in ("W1", "b1", "W2", "b2")]
    Hd, C = p0[0].shape[1], p0[2].shape[1]
    for steps in (2, 5):
        res = {}
        for name in ("odl_host_mlp_train", "odl_host_mlp_train_graph"):
            p = [a.copy() for a in p0]
            g = [np.empty_like(a) for a in p]
            loss, logits = np.zeros(1, f32), np.empty((N, C), f32)
            assert getattr(h, name)(x, t, 1, N, D, Hd, C, *p, steps, 1e-3, 0.9, 0.999, 1e-8, wd, loss, *g, logits) == 0
            res[name] = (loss, logits, p, g)
        (le, ye, pe, ge), (lg, yg, pg, gg) = res["odl_host_mlp_train"], res["odl_host_mlp_train_graph"]
        assert le[0] == lg[0] and np.array_equal(ye, yg), steps
        for a, b in zip(pe, pg):
            assert np.array_equal(a, b), steps
        if wd == 0.0:  # with the hook the two drivers report the gradients at different moments
            for a, b in zip(ge, gg):
                assert np.array_equal(a, b), steps


def test_upload_into_recycled_memory_waits_for_the_kernels_still_reading_it(h):
    """On a created stream (which the null stream does not wait for), five 2048^3 products of an all-ones matrix are
    queued, the matrix is dropped and a host array of its size uploaded straight away — the pool serves the upload from
    the block the products are still reading. The copy must queue behind them: every product element is still 2048
    and the uploaded tensor arrived whole."""
    wrong = np.full(2, -1, np.int64)
    assert h.odl_host_upload_ordering(2048, 5, wrong) == 0
    assert wrong.tolist() == [0, 0]


def test_a_failed_capture_leaves_the_thread_usable_and_replays_report_bad_labels(h):
    """An exception in the middle of a capture (here: a host-to-device copy, which a recorded step may not contain) unwinds
    past the Graph object; its destructor gives the capture up. Afterwards ordinary steps run, a fresh capture records and
    replays bit for bit, a Graph that did not begin a capture cannot end it, and after a replay on labels with an
    out-of-range entry the loss's flag word says so (the ordinary call would have thrown)."""
    rng = np.random.default_rng(44)
    N, D, C = 64, 32, 10
    x = rng.standard_normal((N, D), dtype=f32)
    t = rng.integers(0, C, size=N).astype(np.int32)
    stage, flags = np.zeros(1, np.int32), np.full(2, -1, np.int32)
    assert h.odl_host_graph_abort_recovery(x, t, N, D, C, stage, flags) == 0
    assert stage[0] == 5, stage[0]
    assert flags.tolist() == [1, 0]


def test_a_layer_paired_with_its_relu_gives_the_bits_of_the_two_modules_run_in_turn(h):
    """Sequential runs Linear+ReLU, Conv2d+ReLU(+MaxPool2d) and BatchNorm2d+ReLU as one operator each (activation in
    the epilogue, backward masked with the output or, for the normalisation, with the mask formed again). The network's output and every gradient — parameters and input — must equal, bit for bit, what
    the modules give when called one after the other (src/nn/sequential.cpp, src/operators/activation/relu.cpp)."""
    diffs = np.full(2, -1, np.int64)
    assert h.odl_host_paired_layers_match_separate_modules(64, diffs) == 0
    assert diffs.tolist() == [0, 0], diffs


def test_deferred_fills_behave_like_fills_at_creation(h):
    """zeros / ones / full queue their kernel at the first use of the buffer. Seen from outside nothing may change:
    a copy to the host sees the values, a buffer made before a capture is filled before it (not on every replay),
    zeros += zeros stays zeros, -0.0 += zeros becomes +0.0 (src/mat/origin/cpu/math/add.cpp adds every element), and a
    constant operand takes part in backward."""
    out = np.full(5, -1.0)
    assert h.odl_host_pending_fill_semantics(4096, out) == 0
    assert out.tolist() == [4096.0, 3.0, 0.0, 0.0, 2.5], out


def test_reference_example_network_with_batch_norm_trains_and_replays(h):
    """The network of the reference's tests/example/mnist/conv_mnist.cpp (two conv + BatchNorm + ReLU + pool blocks,
    two Linear layers, Adam + WeightDecay) at batch 16: eight ordinary steps, and two ordinary steps followed by six
    replays of a recorded step, must end with the same training loss and the same evaluation-mode loss (which depends
    on the running statistics every step folded in) bit for bit; and training must reduce the loss."""
    ms, eager, replayed = np.zeros(1, f32), np.zeros(3, f32), np.zeros(3, f32)
    assert h.odl_host_cnn_bn_bench(16, 6, 2, 0, ms, eager) == 0
    assert h.odl_host_cnn_bn_bench(16, 4, 2, 2, ms, replayed) == 0
    assert eager[1] < eager[0] and np.isfinite(eager).all()
    assert np.array_equal(eager, replayed), (eager, replayed)


def test_cnn_training_step_matches_the_reference(h):
    names = ("Wc1", "bc1", "Wc2", "bc2", "Wl1", "bl1", "Wl2", "bl2")
    x, t = G["cnn_x"], G["cnn_t"]
    p = [G[f"cnn_{k}"].copy() for k in names]
    N, _, S, _ = x.shape
    C1, C2, Hd, Cc = p[0].shape[0], p[2].shape[0], p[4].shape[1], p[6].shape[1]
    g = [np.empty_like(a) for a in p]
    loss, logits = np.zeros(1, f32), np.empty((N, Cc), f32)
    assert h.odl_host_cnn_train(x, t, 0, N, S, C1, C2, Hd, Cc, *p, 0.01, loss, *g, logits) == 0
    assert abs(loss[0] - G["cnn1_loss"][0]) <= 1e-4 * abs(G["cnn1_loss"][0])
    np.testing.assert_allclose(logits, G["cnn1_logits"], atol=1e-5)
    for a, ga, k in zip(p, g, names):
        np.testing.assert_allclose(ga, G[f"cnn1_g{k}"], atol=5e-6, rtol=1e-4, err_msg=k)
        np.testing.assert_allclose(a, G[f"cnn1_{k}"], atol=1e-6, rtol=1e-5, err_msg=k)  # SGD: p - 0.01 * g


def test_mlp_step_at_benchmark_size_against_the_oracle(h, o):
    # config 1: x[512,784] uniform, Linear 784->1000 + ReLU, Linear 1000->10, softmax CE, weight decay 1e-4, Adam 1e-3
    rng = np.random.default_rng(5)
    N, D, Hd, C = 512, 784, 1000, 10
    x = rng.random((N, D), dtype=f32)
    t = rng.integers(0, C, size=N).astype(np.int64)
    W1 = ((rng.random((D, Hd), dtype=f32) * 2 - 1) * f32(np.sqrt(6.0 / D))).astype(f32)
    W2 = ((rng.random((Hd, C), dtype=f32) * 2 - 1) * f32(np.sqrt(6.0 / Hd))).astype(f32)
    b1, b2 = np.zeros((1, Hd), f32), np.zeros((1, C), f32)
    po = [a.copy() for a in (W1, b1, W2, b2)]
    mo, vo = [np.zeros_like(a) for a in po], [np.zeros_like(a) for a in po]
    go = [np.empty_like(a) for a in po]
    loss_o, logits_o = np.zeros(1, f32), np.empty((N, C), f32)
    assert o.orc_mlp_train_step(x, t, 1, N, D, Hd, C, *po, mo[0], vo[0], mo[1], vo[1], mo[2], vo[2], mo[3], vo[3], 1,
                                1e-3, 0.9, 0.999, 1e-8, 1e-4, loss_o, *go, logits_o) == 0
    ph = [a.copy() for a in (W1, b1, W2, b2)]
    gh = [np.empty_like(a) for a in ph]
    loss_h, logits_h = np.zeros(1, f32), np.empty((N, C), f32)
    assert h.odl_host_mlp_train(x, t, 1, N, D, Hd, C, *ph, 1, 1e-3, 0.9, 0.999, 1e-8, 1e-4, loss_h, *gh, logits_h) == 0
    assert abs(loss_h[0] - loss_o[0]) <= 1e-4 * abs(loss_o[0])
    np.testing.assert_allclose(logits_h, logits_o, atol=2e-4)
    for a, b in zip(gh, go):
        np.testing.assert_allclose(a, b, atol=2e-6, rtol=2e-3)


def test_cnn_step_at_reduced_batch_against_the_oracle(h, o):
    # config 4's network (conv 1->32, pool, conv 32->64, pool, 3136->128->10) at batch 8, SGD
    rng = np.random.default_rng(6)
    N, S, C1, C2, Hd, Cc = 8, 28, 32, 64, 128, 10
    Fd = C2 * (S // 4) ** 2
    x = rng.random((N, 1, S, S), dtype=f32)
    t = rng.integers(0, Cc, size=N).astype(np.int32)
    shapes = ((C1, 1, 3, 3), (C1,), (C2, C1, 3, 3), (C2,), (Fd, Hd), (1, Hd), (Hd, Cc), (1, Cc))
    fans = (9, 0, 9 * C1, 0, Fd, 0, Hd, 0)
    params = [(rng.standard_normal(s, dtype=f32) * f32(np.sqrt(2.0 / f) if f else 0.05)).astype(f32)
              for s, f in zip(shapes, fans)]
    po = [a.copy() for a in params]
    go = [np.empty_like(a) for a in po]
    loss_o, logits_o = np.zeros(1, f32), np.empty((N, Cc), f32)
    idx1 = np.empty((N, C1, S // 2, S // 2), np.uint64)
    idx2 = np.empty((N, C2, S // 4, S // 4), np.uint64)
    assert o.orc_cnn_train_step(x, t, 0, N, S, C1, C2, Hd, Cc, *po, 0.01, loss_o, idx1, idx2, *go, logits_o) == 0
    ph = [a.copy() for a in params]
    gh = [np.empty_like(a) for a in ph]
    loss_h, logits_h = np.zeros(1, f32), np.empty((N, Cc), f32)
    assert h.odl_host_cnn_train(x, t, 0, N, S, C1, C2, Hd, Cc, *ph, 0.01, loss_h, *gh, logits_h) == 0
    assert abs(loss_h[0] - loss_o[0]) <= 1e-4 * abs(loss_o[0])
    np.testing.assert_allclose(logits_h, logits_o, atol=5e-4)
    for a, b, s in zip(gh, go, shapes):
        np.testing.assert_allclose(a, b, atol=2e-5 * max(np.abs(b).max(), 1.0), rtol=0, err_msg=str(s))
    for a, b in zip(ph, po):
        np.testing.assert_allclose(a, b, atol=1e-6 + 0.01 * 2e-5 * 10, rtol=0)


def test_cnn_step_at_batch_256_against_the_oracle_with_pool_indices_in_full(h, o):
    """The CNN training configuration at its real batch of 256: the whole step (forward, loss, backward, SGD) against
    the oracle's step, and both pools' uint64 argmax indices compared in full.

    The indices are compared twice. (1) On identical inputs, bit for bit: the oracle's own post-ReLU activations
    ([256,32,28,28] and [256,64,14,14], full of exact ties at 0) go through the device pool, whose values and indices
    must equal the oracle's for every one of the 1 605 632 + 802 816 windows
    (src/mat/origin/cpu/pooling/max_pool2d.cpp:110-139: first maximum under strict >). (2) End to end: the device's own
    conv -> ReLU -> pool chain against the oracle's chain. There the pool inputs differ in the last bits (two GEMM
    summation orders), so an index may differ only where the window's two candidates are closer than the convolution's
    own bound; every differing window is checked for that and they must be rare."""
    import torch
    from origindl_amd import capi
    rng = np.random.default_rng(6)
    N, S, C1, C2, Hd, Cc = 256, 28, 32, 64, 128, 10
    Fd = C2 * (S // 4) ** 2
    x = rng.random((N, 1, S, S), dtype=f32)
    t = rng.integers(0, Cc, size=N).astype(np.int32)
    shapes = ((C1, 1, 3, 3), (C1,), (C2, C1, 3, 3), (C2,), (Fd, Hd), (1, Hd), (Hd, Cc), (1, Cc))
    fans = (9, 0, 9 * C1, 0, Fd, 0, Hd, 0)
    params = [(rng.standard_normal(s, dtype=f32) * f32(np.sqrt(2.0 / f) if f else 0.05)).astype(f32)
              for s, f in zip(shapes, fans)]
    po = [a.copy() for a in params]
    go = [np.empty_like(a) for a in po]
    loss_o, logits_o = np.zeros(1, f32), np.empty((N, Cc), f32)
    idx1 = np.empty((N, C1, S // 2, S // 2), np.uint64)
    idx2 = np.empty((N, C2, S // 4, S // 4), np.uint64)
    print("\n[case] cnn step batch 256: oracle", flush=True)
    assert o.orc_cnn_train_step(x, t, 0, N, S, C1, C2, Hd, Cc, *po, 0.01, loss_o, idx1, idx2, *go, logits_o) == 0
    print("[case] cnn step batch 256: device", flush=True)
    ph = [a.copy() for a in params]
    gh = [np.empty_like(a) for a in ph]
    loss_h, logits_h = np.zeros(1, f32), np.empty((N, Cc), f32)
    assert h.odl_host_cnn_train(x, t, 0, N, S, C1, C2, Hd, Cc, *ph, 0.01, loss_h, *gh, logits_h) == 0
    assert abs(loss_h[0] - loss_o[0]) <= 1e-4 * abs(loss_o[0])
    np.testing.assert_allclose(logits_h, logits_o, atol=5e-4)
    for a, b, s in zip(gh, go, shapes):
        np.testing.assert_allclose(a, b, atol=2e-5 * max(np.abs(b).max(), 1.0), rtol=0, err_msg=str(s))
    for a, b in zip(ph, po):
        np.testing.assert_allclose(a, b, atol=1e-6 + 0.01 * 2e-5 * 10, rtol=0)

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    def oracle_layer(inp, w, b, C, H, OC):
        a = np.empty((N, OC, H, H), f32)
        assert o.orc_conv2d(inp, w, b, N, C, H, H, OC, 3, 3, 1, 1, 1, 1, a) == 0
        o.orc_unary(0, a, a.size, a)  # ReLU in place
        y, idx = np.empty((N, OC, H // 2, H // 2), f32), np.empty((N, OC, H // 2, H // 2), np.uint64)
        assert o.orc_max_pool2d(a, N, OC, H, H, 2, 2, 2, 2, 0, 0, y, idx) == 0
        return a, y, idx

    def near_tie_only(act_dev, idx_dev, idx_ref, act_ref, slack):
        """every window whose index differs holds, in the device's own activation, two candidates within `slack`"""
        bad = np.argwhere(idx_dev != idx_ref)
        for n, c, i, j in bad:
            cand = lambda a, k: a[n, c, 2 * i + int(k) // 2, 2 * j + int(k) % 2]  # noqa: E731
            kd, kr = idx_dev[n, c, i, j], idx_ref[n, c, i, j]
            assert abs(cand(act_dev, kd) - cand(act_dev, kr)) <= slack and abs(cand(act_ref, kd) - cand(act_ref, kr)) <= slack
        return len(bad)

    inp_o, inp_d = x, dev(x)
    for li, (w, b, C, H, OC, idx_step) in enumerate(((params[0], params[1], 1, S, C1, idx1),
                                                     (params[2], params[3], C1, S // 2, C2, idx2))):
        print("[case] cnn step batch 256: pool", li + 1, flush=True)
        a_o, y_o, idx_o = oracle_layer(inp_o, w, b, C, H, OC)
        assert np.array_equal(idx_o, idx_step)  # the layer-by-layer oracle is the oracle's training step
        # (1) identical inputs: values and all indices bit-exact
        y_d, idx_d = capi.max_pool2d(dev(a_o), 2, 2, 0)
        assert np.array_equal(y_d.cpu().numpy(), y_o)
        assert np.array_equal(idx_d.cpu().numpy().view(np.uint64), idx_o)
        # (2) the device's own chain
        a_d = capi.unary("relu", capi.conv2d(inp_d, dev(w), dev(b), 1, 1))
        p_d, idx_own = capi.max_pool2d(a_d, 2, 2, 0)
        slack = 1e-5 * float(np.sqrt(9 * C)) * float(np.abs(inp_o).max()) * float(np.linalg.norm(w.reshape(OC, -1), axis=1).max())
        differing = near_tie_only(a_d.cpu().numpy(), idx_own.cpu().numpy().view(np.uint64), idx_o, a_o, slack)
        print("[case] windows whose argmax differs end to end: %d of %d" % (differing, idx_o.size), flush=True)
        assert differing <= idx_o.size * 1e-4
        inp_o, inp_d = y_o, p_d


def test_reference_example_nn_linear_runs_unchanged_on_the_gpu():
    """oracle/_ref/example_nn_linear_hip is the reference's tests/example/linear_regression/nn_linear.cpp compiled,
    unmodified, against origindl_amd/host/include and linked to the gfx950 backend (make -C oracle ref-examples; built
    only where the reference checkout exists). It fits y = 2x + 5 on the device with nn::Linear + SGD; the reference's
    own integration test accepts |w-2| < 0.1 and |b-5| < 0.1 (tests/unit_test/autograd/test_linear_regression.cpp:47-101)."""
    import re
    import subprocess
    exe = ol.ref_binary("example_nn_linear_hip")  # raises when the build recorded the binary and it is gone
    if exe is None:
        pytest.skip("the example binary is built only where the reference checkout is present")
    out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert out.returncode == 0, out.stdout[-2000:]
    assert "Use Device: cuda:0" in out.stdout
    last = [l for l in out.stdout.splitlines() if l.startswith("iter199")][-1]
    m = re.search(r"loss = ([-0-9.e]+), w = ([-0-9.e]+), b = ([-0-9.e]+)", last)
    loss, w, b = (float(v) for v in m.groups())
    assert abs(w - 2.0) < 0.1 and abs(b - 5.0) < 0.1 and loss < 0.05, last


def test_detector_ops_through_the_mat_interface(h):
    """sigmoid / silu / upsample / cat / yolo_detect_forward called on Mat objects exactly as the reference driver
    called them to write the fixtures."""
    x = G["det_act_x"]
    for op, nm in ((6, "sigmoid"), (7, "silu")):
        got = np.empty_like(x)
        assert h.odl_host_activation(op, x, x.size, got) == 0
        np.testing.assert_allclose(got, G[f"det_{nm}"], rtol=3e-7, atol=1e-9)
    xu = G["det_up_x"]
    for nm, (sh, sw) in (("up22", (2, 2)), ("up13", (1, 3))):
        got = np.empty((2, 3, 4 * sh, 5 * sw), f32)
        assert h.odl_host_upsample(xu, 2, 3, 4, 5, 4 * sh, 5 * sw, sh, sw, got) == 0
        assert np.array_equal(got, G[f"det_{nm}"])
    assert h.odl_host_upsample(xu, 2, 3, 4, 5, 9, 10, 2, 2, np.empty((2, 3, 9, 10), f32)) == -1  # row 8 -> input row 4
    parts = [G[f"det_cat_in{i}"] for i in range(3)]
    got = np.empty((3, 8, 7), f32)
    assert h.odl_host_cat(ol.ptr_arr(parts), np.asarray([2, 5, 1], np.int64), 3, 3, 7, got) == 0
    assert np.array_equal(got, G["det_cat"])
    for name in ("detA", "detB"):
        ag = G[f"{name}_anchor_grid"]
        got = np.empty_like(G[f"{name}_out"])
        assert h.odl_host_yolo_detect(G["det_x"], G["det_w"], G["det_b"] if name == "detA" else None, G["det_grid"], ag,
                                      ag.shape[2], ag.shape[3], 2, 6, 4, 5, 8.0, 3, 2, got) == 0
        np.testing.assert_allclose(got, G[f"{name}_out"], rtol=2e-6, atol=1e-6)


BN_CASES = {"bnA": (6, 5, 0, 0), "bnB": (3, 4, 5, 6), "bnC": (1, 2, 3, 3), "bnD": (4, 3, 2, 2)}


@pytest.mark.parametrize("name", list(BN_CASES))
def test_batch_norm_through_mat_operator_and_layers(h, o, name):
    """Mat::batch_norm_forward / batch_norm / batch_norm_backward, and nn::BatchNorm1d / BatchNorm2d, called exactly as
    the reference driver called them to write the fixtures. The layer's backward has no reference fixture — the
    reference's operator throws there — so it is checked against the oracle's backward applied to the same forward."""
    N, C, H, W = BN_CASES[name]
    g = lambda k: G[f"{name}_{k}"]
    x, gamma, beta, rm, rv = g("x"), g("gamma"), g("beta"), g("rm"), g("rv")
    for mode, training in (("train", 1), ("eval", 0)):
        y, xn, mean, var = np.empty_like(x), np.empty_like(x), np.empty(C, f32), np.empty(C, f32)
        assert h.odl_host_batch_norm_forward(x, gamma, beta, rm, rv, training, 1e-5, N, C, H, W, y, mean, var, xn) == 0
        tol = dict(rtol=2e-5, atol=2e-6) if training else dict(rtol=0, atol=0)
        for got, key in ((y, "y"), (mean, "mean"), (var, "var"), (xn, "xn")):
            np.testing.assert_allclose(got, g(f"{mode}_{key}"), err_msg=f"{mode} {key}", **tol)
        y_only = np.empty_like(x)
        assert h.odl_host_batch_norm_forward(x, gamma, beta, rm, rv, training, 1e-5, N, C, H, W, y_only, None, None,
                                             None) == 0
        assert np.array_equal(y_only, y)
    gx, dg, db = np.empty_like(x), np.empty(C, f32), np.empty(C, f32)
    assert h.odl_host_batch_norm_backward(g("gy"), x, gamma, g("train_mean"), g("train_var"), g("train_xn"), 1e-5, N, C,
                                          H, W, gx, dg, db) == 0
    np.testing.assert_allclose(dg, g("dgamma"), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(db, g("dbeta"), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(gx, g("gx"), rtol=2e-5, atol=2e-5)
    # the layers: three training forwards (running statistics folded in on the device), an evaluation forward
    yt, ye, grads = np.empty_like(x), np.empty_like(x), np.empty(x.size + 2 * C, f32)
    assert h.odl_host_batch_norm_layer(x, N, C, H, W, 3, 1e-5, 0.1, 0.25, 1, yt, ye, grads) == 0
    np.testing.assert_allclose(yt, g("layer_ytrain"), rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(ye, g("layer_yeval"), rtol=2e-5, atol=2e-6)
    # backward of sum(y*y) through the last training forward (x scaled by 1.5, gamma 1, beta 0): gy = 2y
    xs = (x * f32(1.5)).astype(f32)
    P = max(H * W, 1)
    wy, wxn, wm, wv = np.empty_like(x), np.empty_like(x), np.empty(C, f32), np.empty(C, f32)
    ones, zeros = np.ones(C, f32), np.zeros(C, f32)
    assert o.orc_batch_norm_forward(xs, ones, zeros, zeros, ones, 1, 1e-5, N, C, P, wy, wm, wv, wxn) == 0
    wgx, wdg, wdb = np.empty_like(x), np.empty(C, f32), np.empty(C, f32)
    assert o.orc_batch_norm_backward((wy * f32(2)).astype(f32), ones, wv, wxn, 1e-5, N, C, P, wgx, wdg, wdb) == 0
    # the gradient of a normalised tensor's sum of squares is a difference of nearly equal terms (the exact input
    # gradient is 2*eps/(var+eps)*... , close to zero): absolute tolerances at the scale of the terms (|2y| ~ 4)
    np.testing.assert_allclose(grads[:x.size].reshape(x.shape), wgx, rtol=0, atol=2e-5)
    np.testing.assert_allclose(grads[x.size:x.size + C], wdg, rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(grads[x.size + C:], wdb, rtol=0, atol=1e-4)


def test_batch_norm_layer_rejects_wrong_inputs(h):
    x = np.ones((2, 3, 4, 4), f32)
    buf = np.empty(200, f32)
    # a [N, C] layer fed channel count 48 vs 3 features is caught by shape, as is a CPU tensor by the device check
    hc = ol.host_driver(cpu=True)
    assert hc.odl_hostcpu_batch_norm_forward(x, np.ones(3, f32), np.ones(3, f32), np.ones(3, f32), np.ones(3, f32), 1,
                                             1e-5, 2, 3, 4, 4, buf, buf, buf, buf) == -2


def _run_pnnx(drv, prefix, param, binp, x, out_shape, reps=1, entry="pnnx_forward"):
    out = np.empty(out_shape, f32)
    oshape, nd, ms = np.zeros(8, np.int64), np.zeros(1, np.int32), np.zeros(1, f32)
    N, C, H, W = x.shape
    rc = getattr(drv, prefix + entry)(param.encode(), binp.encode(), x, N, C, H, W, reps, out, out.size, oshape, nd, ms)
    return rc, out, tuple(oshape[:nd[0]]), float(ms[0])


def test_yolov5n_pnnx_forward_matches_the_reference(h, tmp_path):
    """A YOLOv5n-architecture model in PNNX's file format (synthetic weights written by tests/pnnx_synth.py from a
    seed) run by this repository's graph runner on the GPU, against the output the reference's own PNNX runner
    produced for the same files on the CPU (fixture y5n64_out). Roughly sixty convolutions deep: every logit is a
    chain of fp32 GEMMs whose summation order differs, so the bar is the GEMM bound carried through the network —
    measured deviation is 5e-7 relative to |value| + 1; 1e-5 is asserted."""
    import pnnx_synth
    param, binp, shp = pnnx_synth.write(str(tmp_path / "y5n"), seed=3, batch=1, size=64, num_classes=80)
    rc, out, oshape, _ = _run_pnnx(h, "odl_host_", param, binp, G["y5n64_x"], shp)
    assert rc == 0 and oshape == tuple(shp) == (1, 252, 85)
    want = G["y5n64_out"]
    err = np.abs(out - want) / (np.abs(want) + 1.0)
    print("\n[yolov5n 64x64] max scaled deviation %.3g" % err.max(), flush=True)
    assert err.max() < 1e-5
    # a second forward on the same graph object reuses the uploaded weights and gives the same answer
    rc, out2, _, _ = _run_pnnx(h, "odl_host_", param, binp, G["y5n64_x"], shp, reps=3)
    assert rc == 0 and np.array_equal(out, out2)


def test_yolov5n_pnnx_forward_at_the_benchmark_size_matches_the_reference(h, tmp_path):
    """The detector benchmark configuration itself — batch 4 at 320x320 — against the reference's PNNX runner: the fixture
    ref_y5n320.npz (tests/golden/make_golden.py) holds every 16th of the 6300 output rows of each image, all three
    detection scales among them. Same bar as at 64x64."""
    import pnnx_synth
    sys_path_golden = os.path.join(os.path.dirname(__file__), "golden")
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(sys_path_golden, "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    F = np.load(os.path.join(sys_path_golden, "ref_y5n320.npz"))
    x = mg.y5n320_input()
    assert float(x.astype(np.float64).sum()) == float(F["x_sum"])  # the seeded input is the one the fixture was made from
    param, binp, shp = pnnx_synth.write(str(tmp_path / "y5n"), seed=mg.Y5N320_SEED, batch=4, size=320, num_classes=80)
    assert tuple(shp) == tuple(int(v) for v in F["out_shape"]) == (4, 6300, 85)
    print("\n[case] yolov5n 4x3x320x320", flush=True)
    rc, out, oshape, _ = _run_pnnx(h, "odl_host_", param, binp, x, shp)
    assert rc == 0 and oshape == (4, 6300, 85)
    got, want = out[:, ::int(F["row_step"]), :], F["rows"]
    assert got.shape == want.shape
    err = np.abs(got - want) / (np.abs(want) + 1.0)
    print("[yolov5n 320x320, batch 4] max scaled deviation %.3g over %d values" % (err.max(), want.size), flush=True)
    assert err.max() < 1e-5
    assert np.isfinite(out).all()


def test_float64_matmul_and_its_gradients_through_the_tensor_api(h):
    """F::mat_mul on float64 tensors, forward and backward through the autograd graph (MatMul::backward,
    src/operators/math/mat_mul.cpp:123-182), on the FP64 matrix cores against the compiled reference on the CPU (where it
    was built) and against numpy: within k * 2^-52 * sum |a||b| per element."""
    rng = np.random.default_rng(12)
    for (m, k, n) in ((5, 7, 3), (130, 257, 96), (64, 512, 200)):
        x, w, gy = rng.standard_normal((m, k)), rng.standard_normal((k, n)), rng.standard_normal((m, n))
        y, gx, gw = np.empty((m, n)), np.empty((m, k)), np.empty((k, n))
        assert h.odl_host_matmul_f64_fwd_bwd(x, w, gy, y, gx, gw, m, k, n) == 0
        eps = 2.0 ** -52
        assert (np.abs(y - x @ w) <= k * eps * (np.abs(x) @ np.abs(w))).all()
        assert (np.abs(gx - gy @ w.T) <= n * eps * (np.abs(gy) @ np.abs(w.T))).all()
        assert (np.abs(gw - x.T @ gy) <= m * eps * (np.abs(x.T) @ np.abs(gy))).all()
        if ol.have_ref():
            r = ol.ref()
            yr, gxr, gwr = np.empty((m, n)), np.empty((m, k)), np.empty((k, n))
            assert r.odl_ref_matmul_f64_fwd_bwd(x, w, gy, yr, gxr, gwr, m, k, n) == 0
            assert (np.abs(y - yr) <= k * eps * (np.abs(x) @ np.abs(w))).all()
            assert (np.abs(gx - gxr) <= n * eps * (np.abs(gy) @ np.abs(w.T))).all()
            assert (np.abs(gw - gwr) <= m * eps * (np.abs(x.T) @ np.abs(gy))).all()


def test_float64_conv2d_and_its_gradients_through_the_tensor_api(h):
    """F::conv2d on float64 tensors, forward and backward through the autograd graph (Conv2dOp, conv2d.cpp:404-599 in
    doubles; the reference's device code dispatches over the element type, cuda/conv/conv2d.cu:412-664) against the double
    oracle. (The compiled reference is no witness here: its CPU im2col returns garbage for doubles.)"""
    o = ol.oracle()
    rng = np.random.default_rng(21)
    eps = 2.0 ** -52
    for (N, C, H, W, OC, KH, KW, s, p) in ((2, 3, 7, 6, 4, 3, 3, 1, 1), (3, 4, 9, 9, 5, 3, 3, 2, 1), (4, 8, 16, 16, 12, 3, 3, 1, 1)):
        OH, OW = (H + 2 * p - KH) // s + 1, (W + 2 * p - KW) // s + 1
        x, gy = rng.standard_normal((N, C, H, W)), rng.standard_normal((N, OC, OH, OW))
        w, b = rng.standard_normal((OC, C, KH, KW)), rng.standard_normal((OC,))
        y, gx, gw, gb = np.empty((N, OC, OH, OW)), np.empty_like(x), np.empty_like(w), np.empty_like(b)
        assert h.odl_host_conv2d_f64_fwd_bwd(gy, x, w, b, N, C, H, W, OC, KH, KW, s, s, p, p, y, gx, gw, gb) == 0
        yo, gxo, gwo, gbo = np.empty_like(y), np.empty_like(x), np.empty_like(w), np.empty_like(b)
        assert o.orc_conv2d_f64(x, w, b, N, C, H, W, OC, KH, KW, s, s, p, p, yo) == 0
        assert o.orc_conv2d_backward_f64(gy, x, w, N, C, H, W, OC, KH, KW, s, s, p, p, gxo, gwo, gbo) == 0
        terms = N * OH * OW * C * KH * KW  # a loose common bound: every output is a sum of at most this many products
        for got, want in ((y, yo), (gx, gxo), (gw, gwo), (gb, gbo)):
            assert np.abs(got - want).max() <= terms * eps * (1 + np.abs(want).max()), (N, C, H, W)
        assert np.isfinite(y).all() and np.isfinite(gx).all() and np.isfinite(gw).all()


def test_float64_softmax_through_the_tensor_api(h):
    """F::softmax on float64 tensors, forward and backward: the reference composes it out of max, broadcast_to, subtract,
    exp, sum and divide (src/operators/activation/softmax.cpp:34-129), each of which dispatches over the element type on
    its device (src/mat/origin/cuda/math/{max,broadcast_to,sum}.cu). Against numpy in doubles, and against the compiled
    reference on the CPU where it was built."""
    rng = np.random.default_rng(33)
    for shape, axis in (((5, 7), 1), ((4, 3, 6), 1), ((2, 3, 4, 5), -1), ((300, 1000), 1), ((6, 2), 0)):
        x, gy = rng.standard_normal(shape) * 3, rng.standard_normal(shape)
        y, gx = np.empty(shape), np.empty(shape)
        sh = np.asarray(shape, np.int64)
        assert h.odl_host_softmax_f64_fwd_bwd(x, gy, sh, len(shape), axis, y, gx) == 0
        e = np.exp(x - x.max(axis=axis, keepdims=True))
        want = e / e.sum(axis=axis, keepdims=True)
        want_gx = want * (gy - (gy * want).sum(axis=axis, keepdims=True))
        n = shape[axis]
        assert np.abs(y - want).max() <= 4 * n * 2.0 ** -52
        assert np.abs(gx - want_gx).max() <= 16 * n * 2.0 ** -52 * (1 + np.abs(gy).max())
        if ol.have_ref():
            yr, gxr = np.empty(shape), np.empty(shape)
            assert ol.ref().odl_ref_softmax_f64_fwd_bwd(x, gy, sh, len(shape), axis, yr, gxr) == 0
            assert np.abs(y - yr).max() <= 4 * n * 2.0 ** -52 and np.abs(gx - gxr).max() <= 16 * n * 2.0 ** -52 * (1 + np.abs(gy).max())


def test_pnnx_runner_with_nodes_folded_together_gives_the_floats_of_running_them_one_by_one(h, tmp_path):
    """The runner folds a residual add into the convolution before it, lets producers write straight into a
    concatenation's output, runs SPPF's three pools as one launch and the detect head (three convolutions that decode
    their own sums into their rows of the final tensor) as one launch. With all of that switched off every node runs on its own, as in the reference's runner
    (src/pnnx/pnnx_graph.cpp:286-528); the convolutions are the same kernels either way, so the outputs must agree bit
    for bit — at 64x64 (one image, planes down to 2x2) and at the benchmark's 4 x 320x320. The recorded forward holds
    53 launches folded against 92 plain."""
    import pnnx_synth
    for batch, size, seed in ((1, 64, 3), (4, 320, 0)):
        param, binp, shp = pnnx_synth.write(str(tmp_path / ("y5n%d" % size)), seed=seed, batch=batch, size=size, num_classes=80)
        x = np.random.default_rng(size).random((batch, 3, size, size), dtype=f32)
        nodes = {}
        outs = {}
        try:
            for fusion in (1, 0):
                assert h.odl_host_pnnx_set_fusion(fusion) == 0
                rc, outs[fusion], _, _ = _run_pnnx(h, "odl_host_", param, binp, x, shp, reps=2)
                assert rc == 0
                rc, replayed, _, _ = _run_pnnx(h, "odl_host_", param, binp, x, shp, reps=2, entry="pnnx_forward_graph")
                assert rc == 0 and np.array_equal(replayed, outs[fusion])
                n = np.zeros(1, np.int64)
                assert h.odl_host_pnnx_last_graph_nodes(n) == 0
                nodes[fusion] = int(n[0])
        finally:
            h.odl_host_pnnx_set_fusion(1)
        print("\n[yolov5n %dx%d] launches per forward: %d folded, %d node by node" % (size, size, nodes[1], nodes[0]), flush=True)
        assert np.array_equal(outs[1], outs[0])
        assert np.isfinite(outs[1]).all()
        assert nodes[1] <= 70 and nodes[0] >= 85


def test_pnnx_runner_head_too_large_for_one_launch_runs_stage_by_stage_with_the_same_floats(h, tmp_path):
    """At 8 x 640x640 the first detect stage's convolution (51200 pixels, 64 -> 255 channels: 1.67 GFLOP) is past what
    the small-problem kernel takes, so the head is not one launch: its stages run one after the other and one launch
    decodes the three. Every node on its own (fusion off) runs the same convolution kernels: same floats."""
    import pnnx_synth
    param, binp, shp = pnnx_synth.write(str(tmp_path / "y5n640"), seed=5, batch=8, size=640, num_classes=80)
    x = np.random.default_rng(640).random((8, 3, 640, 640), dtype=f32)
    outs = {}
    try:
        for fusion in (1, 0):
            assert h.odl_host_pnnx_set_fusion(fusion) == 0
            rc, outs[fusion], _, _ = _run_pnnx(h, "odl_host_", param, binp, x, shp, reps=1)
            assert rc == 0
    finally:
        h.odl_host_pnnx_set_fusion(1)
    assert outs[1].shape == (8, 25200, 85) and np.isfinite(outs[1]).all()
    assert np.array_equal(outs[1], outs[0])


def test_pnnx_runner_rejects_bad_files(h, tmp_path):
    import pnnx_synth
    param, binp, shp = pnnx_synth.write(str(tmp_path / "y5n"), seed=1, batch=1, size=32, num_classes=3)
    x = np.zeros((1, 3, 32, 32), f32)
    bad = tmp_path / "bad.param"
    bad.write_text("1234\n1 1\n")
    assert _run_pnnx(h, "odl_host_", str(bad), binp, x, shp)[0] == -2          # wrong magic -> runtime_error
    assert _run_pnnx(h, "odl_host_", str(tmp_path / "nope.param"), binp, x, shp)[0] == -2
    text = open(param).read().replace("nn.SiLU model.1.act", "nn.GELU model.1.act")
    bad.write_text(text)
    assert _run_pnnx(h, "odl_host_", str(bad), binp, x, shp)[0] == -2          # unsupported operator type
    trunc = tmp_path / "trunc.bin"
    trunc.write_bytes(open(binp, "rb").read()[:4000])
    assert _run_pnnx(h, "odl_host_", param, str(trunc), x, shp)[0] == -2
    assert _run_pnnx(h, "odl_host_", param, binp, x, shp)[0] == 0


def test_recorded_detector_forward_replays_bit_for_bit(h, tmp_path):
    """The YOLOv5n-architecture forward recorded into a graph: every replay reads the input tensor in place, and the
    last one (on the fixture's input) must give exactly the ordinary forward's output."""
    import pnnx_synth
    param, binp, shp = pnnx_synth.write(str(tmp_path / "y5n"), seed=3, batch=1, size=64, num_classes=80)
    x = G["y5n64_x"]
    rc, eager, _, _ = _run_pnnx(h, "odl_host_", param, binp, x, shp, reps=2)
    assert rc == 0
    rc, replayed, _, ms = _run_pnnx(h, "odl_host_", param, binp, x, shp, reps=4, entry="pnnx_forward_graph")
    assert rc == 0 and ms > 0
    assert np.array_equal(replayed, eager)
    np.testing.assert_allclose(replayed, G["y5n64_out"], rtol=1e-4, atol=1e-4)


def test_the_references_own_operator_unit_tests_pass_on_this_backend():
    """oracle/_ref/reference_operator_tests_hip is 32 of the reference's GoogleTest operator suites
    (tests/unit_test/operator/test_{matmul,matmul_3d,conv2d,max_pool2d,softmax,softmax_cross_entropy,sum,sum_to,
    broadcast_to,transpose,reshape,flatten,pow,add,sub,mul,div,neg,exp,log,square,relu,sigmoid,silu,cat,upsample,
    compare,batch_norm,split,linear,leaky_relu,type_promotion}.cpp), eight suites of the callers of those operators
    (tests/unit_test/nn/test_{batch_norm,mlp,conv2d_layer}.cpp, optim/test_{adam,weight_decay}.cpp,
    autograd/test_linear_regression.cpp, core/test_no_grad.cpp, utils/test_accuracy.cpp) and the six suites of the
    Tensor class itself (tests/unit_test/tensor/test_{create_tensor,multi_type_tensor,tensor_attributes,tensor_index,
    tensor_operations,tensor_options}.cpp) compiled UNMODIFIED, from where they lie, against this repository's host layer
    and linked to the gfx950 backend (make -C oracle ref-unit-tests; built only where the reference checkout exists).
    The parametrised suites are instantiated per device; the instances labelled CUDA — the device this backend answers
    to — run here, and so do the three Tensor suites that are not parametrised (they hold data on the host and on the
    device but compute nothing). The cases over the other element types (type promotion, int and double inputs, sums in
    all six types, the float64 batch norm) run too: conversion, elementwise arithmetic, pow and sums exist on the device
    for every type, batch norm for both floating-point types. No case is left out by name."""
    import re
    import subprocess
    exe = ol.ref_binary("reference_operator_tests_hip")  # raises when the build recorded the binary and it is gone
    if exe is None:
        pytest.skip("the unit-test binary is built only where the reference checkout is present")
    out = subprocess.run([exe, "--gtest_filter=*CUDA*:TensorCreateTest.*:MultiTypeTensorTest.*:TensorOptionsTest.*",
                          "--gtest_brief=1"],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    tail = out.stdout[-3000:]
    print("\n" + "\n".join(tail.splitlines()[-4:]), flush=True)
    assert out.returncode == 0, tail
    ran = int(re.search(r"\[==========\] (\d+) tests from (\d+) test suites ran", out.stdout).group(1))
    passed = int(re.search(r"\[  PASSED  \] (\d+) tests", out.stdout).group(1))
    assert ran >= 613 and passed >= ran - 4, tail  # four cases skip themselves (a second device, or raw CUDA calls)
