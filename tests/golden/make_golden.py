"""Writes tests/golden/ref_vectors.npz: inputs and outputs of the *compiled reference CPU backend*
(oracle/_ref/libodl_ref.so, built from the reference sources by `make -C oracle ref`) for the behaviours
that none of the reference's own unit tests pin numerically: conv2d_backward (incl. the gy reinterpretation),
im2col/col2im in both layouts, max-pool indices with ties and zero padding, left-aligned sum_to,
softmax-CE with int32/int64 labels, and reduced-size MLP (Adam + weight decay, 2 steps) and CNN (SGD) training
steps. Run in the build container only (the reference is not available elsewhere):

    make -C oracle ref && python tests/golden/make_golden.py

The fixtures are data (inputs + expected outputs); tests compare the plain-C oracle against them bit for bit.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oraclelib as ol  # noqa: E402

f32 = np.float32


def conv_cases():
    # name: N C H W OC KH KW SH SW PH PW bias
    return {
        "convA": (2, 3, 7, 6, 4, 3, 3, 1, 1, 1, 1, 1),
        "convB": (3, 4, 9, 9, 5, 3, 3, 2, 2, 1, 1, 1),
        "convC": (1, 1, 3, 3, 2, 2, 2, 1, 1, 0, 0, 0),
        "convD": (2, 2, 8, 5, 3, 2, 3, 2, 1, 0, 2, 1),
        "convE": (2, 5, 6, 6, 7, 1, 1, 1, 1, 0, 0, 1),
    }


def main():
    r = ol.ref()
    rng = np.random.default_rng(20240611)
    out = {}

    # --- convolution forward/backward, im2col/col2im ------------------------------------------------
    for name, (N, C, H, W, OC, KH, KW, SH, SW, PH, PW, bias) in conv_cases().items():
        OH, OW = (H + 2 * PH - KH) // SH + 1, (W + 2 * PW - KW) // SW + 1
        if name == "convC":  # the integer-valued case whose reference gW is quoted in the survey
            x = np.arange(1, 10, dtype=f32).reshape(1, 1, 3, 3)
            gy = np.arange(1, 9, dtype=f32).reshape(1, 2, 2, 2)
            w = np.arange(1, 9, dtype=f32).reshape(2, 1, 2, 2)
        else:
            x = rng.standard_normal((N, C, H, W), dtype=f32)
            gy = rng.standard_normal((N, OC, OH, OW), dtype=f32)
            w = (rng.standard_normal((OC, C, KH, KW), dtype=f32) * f32(np.sqrt(2.0 / (C * KH * KW)))).astype(f32)
        b = rng.standard_normal((OC,), dtype=f32) if bias else None
        y = np.empty((N, OC, OH, OW), f32)
        gx, gw, gb = np.empty_like(x), np.empty_like(w), np.empty((OC,), f32)
        col = np.empty((N * OH * OW, C * KH * KW), f32)
        col6 = np.empty((N, C, KH, KW, OH, OW), f32)
        assert r.odl_ref_conv2d(x, w, b, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, y) == 0
        assert r.odl_ref_conv2d_backward(gy, x, w, b, N, C, H, W, OC, KH, KW, SH, SW, PH, PW, gx, gw,
                                         gb if bias else None) == 0
        assert r.odl_ref_im2col(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, col) == 0
        assert r.odl_ref_im2col(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 0, col6) == 0
        gcol = rng.standard_normal(col.shape, dtype=f32)
        gcol6 = rng.standard_normal(col6.shape, dtype=f32)
        im, im6 = np.empty_like(x), np.empty_like(x)
        assert r.odl_ref_col2im(gcol, ol.shape_arr(gcol.shape), 2, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, im) == 0
        assert r.odl_ref_col2im(gcol6, ol.shape_arr(gcol6.shape), 6, N, C, H, W, KH, KW, SH, SW, PH, PW, 0, im6) == 0
        out.update({f"{name}_x": x, f"{name}_w": w, f"{name}_gy": gy, f"{name}_y": y, f"{name}_gx": gx,
                    f"{name}_gw": gw, f"{name}_col": col, f"{name}_col6": col6, f"{name}_gcol": gcol,
                    f"{name}_gcol6": gcol6, f"{name}_im": im, f"{name}_im6": im6})
        if bias:
            out[f"{name}_b"] = b
            out[f"{name}_gb"] = gb

    # --- max pool: ties, negatives with zero padding, overlapping windows ----------------------------
    pool_cases = {
        "poolA": (2, 3, 6, 6, 2, 2, 2, 2, 0, 0),
        "poolB": (1, 2, 7, 7, 3, 3, 2, 2, 1, 1),
        "poolC": (2, 2, 5, 5, 5, 5, 1, 1, 2, 2),
        "poolD": (1, 3, 6, 5, 3, 2, 1, 2, 1, 0),
    }
    for name, (N, C, H, W, KH, KW, SH, SW, PH, PW) in pool_cases.items():
        OH, OW = (H + 2 * PH - KH) // SH + 1, (W + 2 * PW - KW) // SW + 1
        # few distinct values -> many ties; mostly negative -> zero padding wins at the borders
        x = (rng.integers(-3, 2, size=(N, C, H, W)).astype(f32)) * f32(0.5)
        y = np.empty((N, C, OH, OW), f32)
        idx = np.empty((N, C, OH, OW), np.uint64)
        gy = rng.standard_normal(y.shape, dtype=f32)
        gx = np.empty_like(x)
        assert r.odl_ref_max_pool2d(x, N, C, H, W, KH, KW, SH, SW, PH, PW, y, idx) == 0
        assert r.odl_ref_max_pool2d_backward(gy, idx, N, C, H, W, KH, KW, SH, SW, PH, PW, gx) == 0
        out.update({f"{name}_x": x, f"{name}_y": y, f"{name}_idx": idx, f"{name}_gy": gy, f"{name}_gx": gx})

    # --- sum / sum_to / broadcast backward -------------------------------------------------------------
    sumto_cases = {
        "sumtoA": ((4, 5), (1, 5)),
        "sumtoB": ((4, 5), (4, 1)),
        "sumtoC": ((2, 3, 4), (2, 1)),      # left-aligned: dims 1 (->1) and surplus dim 2 are reduced
        "sumtoD": ((2, 3, 4), (1, 3, 1)),
        "sumtoE": ((3, 2), (2,)),           # not left-alignable by value: surplus dim reduced, [3] != [2] -> throws
        "sumtoF": ((2, 2), (2,)),           # {2,2}->{2}: reduces dim 1 (row sums)
        "sumtoG": ((6, 7), ()),             # to a 0-dim scalar
        "sumtoH": ((2, 3), (2, 3, 4)),      # larger target -> runtime_error
    }
    for name, (ss, ts) in sumto_cases.items():
        x = rng.standard_normal(ss, dtype=f32)
        te = int(np.prod(ts)) if len(ts) else 1
        dst = np.zeros((max(te, 1),), f32)
        rc = r.odl_ref_sum_to(x, ol.shape_arr(ss), len(ss), ol.shape_arr(ts), len(ts), dst)
        out.update({f"{name}_x": x, f"{name}_t": ol.shape_arr(ts), f"{name}_rc": np.int32(rc), f"{name}_y": dst})
    # broadcast_to (right-aligned) forward + its (left-aligned) backward
    for name, (ss, ds) in {"bcastA": ((1, 5), (4, 5)), "bcastB": ((2,), (2, 2)), "bcastC": ((3, 1), (3, 4))}.items():
        x = rng.standard_normal(ss, dtype=f32)
        g = rng.standard_normal(ds, dtype=f32)
        y = np.empty(ds, f32)
        gxb = np.empty(ss, f32)
        assert r.odl_ref_broadcast_to(x, ol.shape_arr(ss), len(ss), ol.shape_arr(ds), len(ds), y) == 0
        rc = r.odl_ref_broadcast_to_backward(x, ol.shape_arr(ss), len(ss), ol.shape_arr(ds), len(ds), g, gxb)
        out.update({f"{name}_x": x, f"{name}_d": ol.shape_arr(ds), f"{name}_g": g, f"{name}_y": y,
                    f"{name}_rc": np.int32(rc), f"{name}_gx": gxb})
    for name, (shape, axis, keep) in {"sumA": ((5, 7), 0, 0), "sumB": ((5, 7), 1, 1), "sumC": ((3, 4, 5), 1, 0),
                                      "sumD": ((300, 17), -1, 0)}.items():
        x = rng.standard_normal(shape, dtype=f32)
        oshape = [d for i, d in enumerate(shape) if i != axis] if axis >= 0 else [1]
        dst = np.empty((int(np.prod(oshape)),), f32)
        assert r.odl_ref_sum(x, ol.shape_arr(shape), len(shape), axis, keep, dst) == 0
        mx = np.empty_like(dst)
        assert r.odl_ref_max(x, ol.shape_arr(shape), len(shape), axis, mx) == 0
        out.update({f"{name}_x": x, f"{name}_axis": np.int32(axis), f"{name}_y": dst, f"{name}_max": mx})

    # --- softmax / CE ---------------------------------------------------------------------------------------
    for name, (N, C, is64) in {"ceA": (8, 10, 0), "ceB": (5, 3, 1), "ceC": (1, 7, 1)}.items():
        x = (rng.standard_normal((N, C), dtype=f32) * f32(3)).astype(f32)
        t = rng.integers(0, C, size=(N,)).astype(np.int64 if is64 else np.int32)
        loss = np.zeros((1,), f32)
        gx = np.empty_like(x)
        p = np.empty_like(x)
        assert r.odl_ref_softmax_ce(x, t, is64, N, C, loss, gx) == 0
        assert r.odl_ref_softmax(x, ol.shape_arr(x.shape), 2, -1, p) == 0
        sel = np.empty((N,), f32)
        oh = np.empty((N, C), f32)
        assert r.odl_ref_gather(p, t, is64, N, C, sel) == 0
        assert r.odl_ref_one_hot(t, is64, N, C, oh) == 0
        out.update({f"{name}_x": x, f"{name}_t": t, f"{name}_loss": loss, f"{name}_gx": gx, f"{name}_p": p,
                    f"{name}_sel": sel, f"{name}_oh": oh})
    # out-of-range labels: gather throws invalid_argument, one_hot skips silently
    tb = np.array([0, 5, -1, 2], np.int32)
    xb = rng.standard_normal((4, 3), dtype=f32)
    sel = np.zeros((4,), f32)
    oh = np.empty((4, 3), f32)
    out["oob_t"] = tb
    out["oob_x"] = xb
    out["oob_gather_rc"] = np.int32(r.odl_ref_gather(xb, tb, 0, 4, 3, sel))
    out["oob_onehot_rc"] = np.int32(r.odl_ref_one_hot(tb, 0, 4, 3, oh))
    out["oob_onehot"] = oh
    lossb = np.zeros((1,), f32)
    out["oob_ce_rc"] = np.int32(r.odl_ref_softmax_ce(xb, tb, 0, 4, 3, lossb, None))

    # --- training steps at reduced size ---------------------------------------------------------------------
    N, D, Hd, C = 16, 20, 12, 5
    x = rng.random((N, D), dtype=f32)
    t = rng.integers(0, C, size=(N,)).astype(np.int64)
    W1 = ((rng.random((D, Hd), dtype=f32) * 2 - 1) * f32(np.sqrt(6.0 / D))).astype(f32)
    b1 = (rng.standard_normal((1, Hd), dtype=f32) * f32(0.1)).astype(f32)
    W2 = ((rng.random((Hd, C), dtype=f32) * 2 - 1) * f32(np.sqrt(6.0 / Hd))).astype(f32)
    b2 = (rng.standard_normal((1, C), dtype=f32) * f32(0.1)).astype(f32)
    out.update({"mlp_x": x, "mlp_t": t, "mlp_W1": W1, "mlp_b1": b1, "mlp_W2": W2, "mlp_b2": b2})
    for steps in (1, 2):
        p = [a.copy() for a in (W1, b1, W2, b2)]
        loss = np.zeros((1,), f32)
        g = [np.empty_like(a) for a in p]
        logits = np.empty((N, C), f32)
        assert r.odl_ref_mlp_train(x, t, 1, N, D, Hd, C, *p, steps, 1e-3, 0.9, 0.999, 1e-8, 1e-4, loss, *g, logits) == 0
        for nm, a in zip(("W1", "b1", "W2", "b2"), p):
            out[f"mlp{steps}_{nm}"] = a
        for nm, a in zip(("gW1", "gb1", "gW2", "gb2"), g):
            out[f"mlp{steps}_{nm}"] = a
        out[f"mlp{steps}_loss"] = loss
        out[f"mlp{steps}_logits"] = logits

    N, S, C1, C2, Hd, Cc = 4, 8, 3, 4, 6, 5
    Fd = C2 * (S // 4) ** 2
    x = rng.random((N, 1, S, S), dtype=f32)
    t = rng.integers(0, Cc, size=(N,)).astype(np.int32)
    params = [
        (rng.standard_normal((C1, 1, 3, 3), dtype=f32) * f32(np.sqrt(2.0 / 9))).astype(f32),
        (rng.standard_normal((C1,), dtype=f32) * f32(0.1)).astype(f32),
        (rng.standard_normal((C2, C1, 3, 3), dtype=f32) * f32(np.sqrt(2.0 / (9 * C1)))).astype(f32),
        (rng.standard_normal((C2,), dtype=f32) * f32(0.1)).astype(f32),
        (rng.standard_normal((Fd, Hd), dtype=f32) * f32(np.sqrt(1.0 / Fd))).astype(f32),
        (rng.standard_normal((1, Hd), dtype=f32) * f32(0.1)).astype(f32),
        (rng.standard_normal((Hd, Cc), dtype=f32) * f32(np.sqrt(1.0 / Hd))).astype(f32),
        (rng.standard_normal((1, Cc), dtype=f32) * f32(0.1)).astype(f32),
    ]
    names = ("Wc1", "bc1", "Wc2", "bc2", "Wl1", "bl1", "Wl2", "bl2")
    out.update({"cnn_x": x, "cnn_t": t})
    for nm, a in zip(names, params):
        out[f"cnn_{nm}"] = a
    p = [a.copy() for a in params]
    g = [np.empty_like(a) for a in p]
    loss = np.zeros((1,), f32)
    logits = np.empty((N, Cc), f32)
    assert r.odl_ref_cnn_train(x, t, 0, N, S, C1, C2, Hd, Cc, *p, 0.01, loss, *g, logits) == 0
    for nm, a, ga in zip(names, p, g):
        out[f"cnn1_{nm}"] = a
        out[f"cnn1_g{nm}"] = ga
    out["cnn1_loss"] = loss
    out["cnn1_logits"] = logits

    # --- elementwise, pow ---------------------------------------------------------------------------------
    a = (rng.standard_normal((257,), dtype=f32) * f32(2)).astype(f32)
    b = (rng.standard_normal((257,), dtype=f32) + f32(3)).astype(f32)
    out["ew_a"], out["ew_b"] = a, b
    for op in range(5):
        o = np.empty_like(a)
        assert r.odl_ref_binary(op, a, ol.shape_arr(a.shape), 1, b, ol.shape_arr(b.shape), 1, o) == 0
        out[f"ew_bin{op}"] = o
    for op in range(5):
        src = np.abs(a) + f32(0.1) if op == 2 else a
        o = np.empty_like(a)
        assert r.odl_ref_unary(op, src, a.size, o) == 0
        out[f"ew_un{op}"] = o
    o = np.empty_like(a)
    assert r.odl_ref_pow_scalar(np.abs(a), a.size, 0.5, o) == 0
    out["ew_pow05"] = o

    # --- detector forward path: sigmoid / silu, nearest upsample, cat, yolo detect head ----------------------
    rd = np.random.default_rng(20240902)
    xa = (rd.standard_normal((301,), dtype=f32) * f32(3)).astype(f32)
    out["det_act_x"] = xa
    for op, nm in ((6, "sigmoid"), (7, "silu")):
        o = np.empty_like(xa)
        assert r.odl_ref_activation(op, xa, xa.size, o) == 0
        out[f"det_{nm}"] = o
    xu = rd.standard_normal((2, 3, 4, 5), dtype=f32)
    for nm, (sh, sw) in (("up22", (2, 2)), ("up13", (1, 3))):
        o = np.empty((2, 3, 4 * sh, 5 * sw), f32)
        assert r.odl_ref_upsample(xu, 2, 3, 4, 5, 4 * sh, 5 * sw, sh, sw, o) == 0
        out[f"det_{nm}"] = o
    out["det_up_x"] = xu
    parts = [rd.standard_normal((3, c, 7), dtype=f32) for c in (2, 5, 1)]
    o = np.empty((3, 8, 7), f32)
    keep = ol.ptr_arr(parts)
    assert r.odl_ref_cat(keep, np.asarray([2, 5, 1], np.int64), 3, 3, 7, o) == 0
    for i, pt in enumerate(parts):
        out[f"det_cat_in{i}"] = pt
    out["det_cat"] = o
    # detect head: N=2, C=6, H=4, W=5, anchors=3, classes=2 (CI=7); the anchor grid is coarser than the map (2x5)
    N, C, H, W, A, NC = 2, 6, 4, 5, 3, 2
    CI = NC + 5
    xd = rd.standard_normal((N, C, H, W), dtype=f32)
    wd = (rd.standard_normal((A * CI, C, 1, 1), dtype=f32) * f32(0.5)).astype(f32)
    bd = rd.standard_normal((A * CI,), dtype=f32)
    gy_, gx_ = np.meshgrid(np.arange(H, dtype=f32), np.arange(W, dtype=f32), indexing="ij")
    grid = np.broadcast_to(np.stack([gx_, gy_], -1) - f32(0.5), (1, A, H, W, 2)).astype(f32).copy()
    for nm, (aH, aW) in (("detA", (H, W)), ("detB", (2, 5))):
        anchors = (rd.random((A, 2), dtype=f32) * f32(30) + f32(4)).astype(f32)
        ag = np.broadcast_to(anchors.reshape(1, A, 1, 1, 2), (1, A, aH, aW, 2)).astype(f32).copy()
        ag += (rd.random(ag.shape, dtype=f32) * f32(0.25)).astype(f32)  # make every cell distinguishable
        o = np.empty((N, A * H * W, CI), f32)
        assert r.odl_ref_yolo_detect(xd, wd, bd if nm == "detA" else None, grid, ag, aH, aW, N, C, H, W, 8.0, A, NC, o) == 0
        out[f"{nm}_anchor_grid"], out[f"{nm}_out"] = ag, o
    out["det_x"], out["det_w"], out["det_b"], out["det_grid"] = xd, wd, bd, grid

    # --- a whole YOLOv5n-architecture forward through the reference's PNNX runner (synthetic weights, 64x64 input) --
    import tempfile
    import pnnx_synth
    with tempfile.TemporaryDirectory() as tmp:
        param, binp, shp = pnnx_synth.write(os.path.join(tmp, "y5n"), seed=3, batch=1, size=64, num_classes=80)
        xin = np.random.default_rng(7).random((1, 3, 64, 64), dtype=f32)
        o = np.empty(shp, f32)
        oshape, nd, ms = np.zeros(8, np.int64), np.zeros(1, np.int32), np.zeros(1, f32)
        assert r.odl_ref_pnnx_forward(param.encode(), binp.encode(), xin, 1, 3, 64, 64, 1, o, o.size, oshape, nd, ms) == 0
        assert tuple(oshape[:nd[0]]) == tuple(shp)
    out["y5n64_x"], out["y5n64_out"] = xin, o

    # --- batch normalisation: Mat-level forward (training and evaluation) and backward in both layouts, and the
    # layers (running statistics over three training forwards, gradients through autograd, an evaluation forward) ---
    rb = np.random.default_rng(11)
    for nm, (N, C, H, W) in {"bnA": (6, 5, 0, 0), "bnB": (3, 4, 5, 6), "bnC": (1, 2, 3, 3), "bnD": (4, 3, 2, 2)}.items():
        P = max(H * W, 1)
        xs = (N, C) if H == 0 else (N, C, H, W)
        x = (rb.standard_normal(xs, dtype=f32) * f32(2) + f32(0.5)).astype(f32)
        gamma = (rb.random(C, dtype=f32) + f32(0.5)).astype(f32)
        beta = rb.standard_normal(C, dtype=f32)
        rm = rb.standard_normal(C, dtype=f32)
        rv = (rb.random(C, dtype=f32) + f32(0.25)).astype(f32)
        gy = rb.standard_normal(xs, dtype=f32)
        out[f"{nm}_x"], out[f"{nm}_gamma"], out[f"{nm}_beta"], out[f"{nm}_rm"], out[f"{nm}_rv"], out[f"{nm}_gy"] = \
            x, gamma, beta, rm, rv, gy
        for mode, training in (("train", 1), ("eval", 0)):
            y, xn = np.empty(xs, f32), np.empty(xs, f32)
            mean, var = np.empty(C, f32), np.empty(C, f32)
            assert r.odl_ref_batch_norm_forward(x, gamma, beta, rm, rv, training, 1e-5, N, C, H, W, y, mean, var, xn) == 0
            out[f"{nm}_{mode}_y"], out[f"{nm}_{mode}_mean"], out[f"{nm}_{mode}_var"], out[f"{nm}_{mode}_xn"] = y, mean, var, xn
            y_only = np.empty(xs, f32)
            assert r.odl_ref_batch_norm_forward(x, gamma, beta, rm, rv, training, 1e-5, N, C, H, W, y_only, None, None,
                                                None) == 0
            assert np.array_equal(y_only, y)
            if training:
                gx, dg, db = np.empty(xs, f32), np.empty(C, f32), np.empty(C, f32)
                assert r.odl_ref_batch_norm_backward(gy, x, gamma, mean, var, xn, 1e-5, N, C, H, W, gx, dg, db) == 0
                out[f"{nm}_gx"], out[f"{nm}_dgamma"], out[f"{nm}_dbeta"] = gx, dg, db
        # the reference's operator cannot run backward in training mode (it moves its saved statistics away,
        # operators/normalization/batch_norm.cpp:78-83), so the layer fixture holds the two forwards only
        yt, ye = np.empty(xs, f32), np.empty(xs, f32)
        assert r.odl_ref_batch_norm_layer(x, N, C, H, W, 3, 1e-5, 0.1, 0.25, 0, yt, ye, None) == 0
        assert r.odl_ref_batch_norm_layer(x, N, C, H, W, 3, 1e-5, 0.1, 0.25, 1, yt.copy(), ye.copy(),
                                          np.empty(x.size + 2 * C, f32)) == -2
        out[f"{nm}_layer_ytrain"], out[f"{nm}_layer_yeval"] = yt, ye

    # --- a model file written by the reference itself (.odl, src/io/model_io.cpp:116-168): an MLP({4, 8, 2}) ---
    mlp_params = np.random.default_rng(13).standard_normal(58).astype(f32)
    assert r.odl_ref_save_mlp(mlp_params, os.path.join(HERE, "ref_mlp.odl").encode()) == 0
    out["io_mlp_params"] = mlp_params
    xio = np.random.default_rng(14).standard_normal((3, 4)).astype(f32)
    back, yio = np.empty(58, f32), np.empty((3, 2), f32)
    assert r.odl_ref_load_mlp(os.path.join(HERE, "ref_mlp.odl").encode(), 1, xio, back, yio) == 0
    assert np.array_equal(back, mlp_params)
    out["io_mlp_x"], out["io_mlp_y"] = xio, yio

    path = os.path.join(HERE, "ref_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")
    detector_at_benchmark_size(r)


Y5N320_SEED, Y5N320_INPUT_SEED, Y5N320_ROW_STEP = 3, 8, 16


def y5n320_input():
    """The [4,3,320,320] uniform[0,1) input of the detector benchmark configuration, from a fixed seed (the test
    regenerates it instead of storing 4.9 MB; the fixture keeps its float64 sum as a guard)."""
    return np.random.default_rng(Y5N320_INPUT_SEED).random((4, 3, 320, 320), dtype=f32)


def detector_at_benchmark_size(r):
    """tests/golden/ref_y5n320.npz: the YOLOv5n-architecture forward at the benchmark's own size, [4,3,320,320], through
    the reference's PNNX runner (about a minute on one core here). The output is [4, 6300, 85]; every 16th of the 6300
    rows of each image is kept (394 rows an image: all three detection scales are sampled, 0.5 MB)."""
    import tempfile
    import pnnx_synth
    with tempfile.TemporaryDirectory() as tmp:
        param, binp, shp = pnnx_synth.write(os.path.join(tmp, "y5n"), seed=Y5N320_SEED, batch=4, size=320, num_classes=80)
        xin = y5n320_input()
        o = np.empty(shp, f32)
        oshape, nd, ms = np.zeros(8, np.int64), np.zeros(1, np.int32), np.zeros(1, f32)
        assert r.odl_ref_pnnx_forward(param.encode(), binp.encode(), xin, 4, 3, 320, 320, 1, o, o.size, oshape, nd, ms) == 0
        assert tuple(oshape[:nd[0]]) == tuple(shp) == (4, 6300, 85)
    path = os.path.join(HERE, "ref_y5n320.npz")
    np.savez_compressed(path, rows=np.ascontiguousarray(o[:, ::Y5N320_ROW_STEP, :]), row_step=np.int64(Y5N320_ROW_STEP),
                        x_sum=np.float64(xin.astype(np.float64).sum()), out_shape=np.asarray(shp, np.int64))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    if "--detector-only" in sys.argv:
        detector_at_benchmark_size(ol.ref())
    else:
        main()
