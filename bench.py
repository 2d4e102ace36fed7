"""Benchmark of the hot path on one MI355X.

Default workload (the one the headline metric is quoted on): standalone matmul forward + backward, fp32,
M = N = K = 4096 — one step = C = A.B, dA = dC.B^T, dB = A^T.dC = 6*M*N*K FLOP — on synthetic N(0,1) operands
already resident in HBM. Prints ONE JSON line: value = TFLOP/s of the whole step, plus
  roofline      the MFMA GEMM kernel: 2*M*N*K FLOP per launch / average launch duration measured with events on the
                launch stream over the timed region, against the 157.3 TFLOP/s FP32 matrix peak;
  cpu_baseline  the reference's own CPU backend (oracle/_ref, when its build travelled with the tree) or the plain-C
                port of it (oracle/), timed on this box's host cores on a bounded row slice of the same three products;
  extras        the other hot-path kernels at the benchmark's shapes (conv C1/C2 fwd+bwd, im2col/col2im, bias-gradient
                and softmax-CE-gradient streams) with their own roofline fractions, and MLP train-step GEMM time.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--size 4096] [--no-extras] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def time_region(torch, fn, steps, warmup):
    """ms per call of fn, timed with events on the current stream (the stream the kernels are launched on)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def time_region_auto(torch, fn, target_ms=40.0, warmup=3):
    """ms per call for the short kernels of `extras`: a probe of ten calls sizes the timed run to about `target_ms` of
    device time (at least 10, at most 4000 calls), so that a kernel of a few microseconds is timed over thousands of
    back-to-back launches and not over the clock ramp of the first ten."""
    probe = time_region(torch, fn, 10, warmup)
    n = int(min(4000, max(10, target_ms / max(probe, 1e-4))))
    return time_region(torch, fn, n, 2)


def cpu_baseline_gemm(size, budget_s=18.0):
    """Reference CPU algorithm on a row slice of each of the three products; rows are independent in its loop
    (src/mat/origin/cpu/math/matmul.cpp:27-41), so time scales linearly with the number of rows."""
    import numpy as np
    import oraclelib as ol
    rng = np.random.default_rng(0)
    a = rng.standard_normal((size, size), dtype=np.float32)
    b = rng.standard_normal((size, size), dtype=np.float32)
    use_ref = ol.have_ref()

    def run(rows):
        out = np.empty((rows, size), np.float32)
        sl = np.ascontiguousarray(a[:rows])
        t0 = time.perf_counter()
        for _ in range(3):  # C rows, dA rows, dB rows: three products of identical shape on a slice
            if use_ref:
                assert ol.ref().odl_ref_matmul(sl, b, out, rows, size, size) == 0
            else:
                ol.oracle().orc_matmul(sl, b, out, rows, size, size)
        return time.perf_counter() - t0

    probe_rows = 2
    t_probe = run(probe_rows)
    rows = int(max(2, min(size, probe_rows * budget_s / max(t_probe, 1e-6))))
    t = run(rows)
    flop = 3 * 2.0 * rows * size * size
    return {
        "value": flop / t / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "reference" if use_ref else "port",
        "sample": "%d of %d rows of each of C, dA, dB (%.1f s; full step extrapolates to %.0f s)"
                  % (rows, size, t, t * size / rows),
    }


def extras(torch, capi, steps, warmup):
    """The other hot kernels at the benchmark's shapes. Outputs and workspaces are allocated once and every timed
    call is one direct C-ABI call with prebuilt arguments, so that microsecond-scale kernels are not timed through
    Python allocation and argument checking."""
    import ctypes
    from origindl_amd import _lib
    out = {}
    g = torch.Generator(device="cuda").manual_seed(0)
    L = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    keep = []  # tensors behind the raw pointers

    def rnd(*shape):
        return torch.randn(shape, device="cuda", generator=g)

    def ptr(t):
        keep.append(t)
        return ctypes.c_void_p(t.data_ptr())

    def empty(*shape):
        return torch.empty(shape, dtype=torch.float32, device="cuda")

    def ws(nbytes):
        nbytes = int(nbytes)
        if nbytes == 0:
            return None, 0
        t = torch.empty((nbytes + 3) // 4, dtype=torch.int32, device="cuda")
        return ptr(t), nbytes

    def direct(name, *args):
        fn = getattr(L.cdll, name)
        L.check(fn(*args))  # argument errors surface here, once
        return lambda: fn(*args)

    # conv2d forward + weight-grad + input-grad at the benchmark's convolution configurations C1 and C2
    for name, (N, C, H, OC, s, p) in {"conv_c1": (32, 64, 56, 128, 1, 1), "conv_c2": (32, 128, 28, 256, 2, 1)}.items():
        x, w, b = rnd(N, C, H, H), rnd(OC, C, 3, 3) * (2.0 / (C * 9)) ** 0.5, rnd(OC)
        OH = (H + 2 * p - 3) // s + 1
        gy = rnd(N, OC, OH, OH)
        M, K = N * OH * OH, C * 9
        geom = (N, C, H, H, OC, 3, 3, s, s, p, p)
        y, gx, gw, gb = empty(N, OC, OH, OH), empty(N, C, H, H), empty(OC, C, 3, 3), empty(OC)
        wf, nf = ws(L.query("odl_hip_conv2d_workspace_bytes", *geom))
        wb, nbb = ws(L.query("odl_hip_conv2d_backward_workspace_bytes", *geom))
        fwd = direct("odl_hip_conv2d", ptr(x), ptr(w), ptr(b), *geom, ptr(y), wf, nf, stream)
        bwd = direct("odl_hip_conv2d_backward", ptr(gy), ptr(x), ptr(w), *geom, ptr(gx), ptr(gw), ptr(gb), wb, nbb,
                     stream)
        ms_f = time_region_auto(torch, fwd)
        ms_b = time_region_auto(torch, bwd)
        flop = 6.0 * M * K * OC
        tf = flop / (ms_f + ms_b) / 1e9
        out[name] = {"fwd_ms": ms_f, "bwd_ms": ms_b, "tflops": tf, "frac_mfma_peak": tf / PEAK_FP32_MFMA_TFLOPS,
                     "flop": flop}
        col, img = empty(M, K), empty(N, C, H, H)
        ig = (N, C, H, H, 3, 3, s, s, p, p, 1)
        ms_i = time_region_auto(torch, direct("odl_hip_im2col", ptr(x), *ig, ptr(col), stream))
        ms_c = time_region_auto(torch, direct("odl_hip_col2im", ptr(col), *ig, ptr(img), stream))
        nbytes = 4.0 * (x.numel() + M * K)
        out[name + "_im2col"] = {"ms": ms_i, "gbs": nbytes / ms_i / 1e6, "frac_hbm": nbytes / ms_i / 1e6 / PEAK_HBM_GBS}
        out[name + "_col2im"] = {"ms": ms_c, "gbs": nbytes / ms_c / 1e6, "frac_hbm": nbytes / ms_c / 1e6 / PEAK_HBM_GBS}
        wr, nr = ws(L.query("odl_hip_sum_nchw_channels_workspace_bytes", N, OC, OH * OH))
        ms_gb = time_region_auto(torch, direct("odl_hip_sum_nchw_channels", ptr(gy), N, OC, OH * OH, ptr(gb), wr, nr, stream))
        nb = 4.0 * (gy.numel() + OC)
        out[name + "_bias_grad"] = {"ms": ms_gb, "gbs": nb / ms_gb / 1e6, "frac_hbm": nb / ms_gb / 1e6 / PEAK_HBM_GBS}
        del x, w, b, gy, col, img, y, gx, gw
        keep.clear()
    # The first layer of the CNN (config 4): one input channel, 32 filters — direct kernels, HBM bound. Algorithmic
    # bytes: forward reads x and writes y; backward reads gy and x once and writes gx and gW.
    N, C, H, OC = 256, 1, 28, 32
    x, w, b, gy = rnd(N, C, H, H), rnd(OC, C, 3, 3) / 3.0, rnd(OC), rnd(N, OC, H, H)
    geom = (N, C, H, H, OC, 3, 3, 1, 1, 1, 1)
    y, gx, gw, gb = empty(N, OC, H, H), empty(N, C, H, H), empty(OC, C, 3, 3), empty(OC)
    wf, nf = ws(L.query("odl_hip_conv2d_workspace_bytes", *geom))
    wb, nbb = ws(L.query("odl_hip_conv2d_backward_workspace_bytes", *geom))
    fwd = direct("odl_hip_conv2d", ptr(x), ptr(w), ptr(b), *geom, ptr(y), wf, nf, stream)
    bwd = direct("odl_hip_conv2d_backward", ptr(gy), ptr(x), ptr(w), *geom, ptr(gx), ptr(gw), None, wb, nbb, stream)
    ms_f, ms_b = time_region_auto(torch, fwd), time_region_auto(torch, bwd)
    nb_f, nb_b = 4.0 * (x.numel() + y.numel()), 4.0 * (gy.numel() + 2 * x.numel() + gw.numel())
    out["conv_first_layer_256x1x28x28_to_32"] = {
        "fwd_ms": ms_f, "bwd_ms": ms_b, "fwd_gbs": nb_f / ms_f / 1e6, "bwd_gbs": nb_b / ms_b / 1e6,
        "fwd_frac_hbm": nb_f / ms_f / 1e6 / PEAK_HBM_GBS, "bwd_frac_hbm": nb_b / ms_b / 1e6 / PEAK_HBM_GBS}
    # its 2x2 max-pool: forward reads x, writes y and the uint64 indices; backward reads gy and the indices, writes gx
    OHp = H // 2
    yp, idx = empty(N, OC, OHp, OHp), torch.empty((N, OC, OHp, OHp), dtype=torch.int64, device="cuda")
    gyp, gxp = rnd(N, OC, OHp, OHp), empty(N, OC, H, H)
    pg = (N, OC, H, H, 2, 2, 2, 2, 0, 0)
    pf = direct("odl_hip_max_pool2d", ptr(y), *pg, ptr(yp), ptr(idx), stream)
    pb = direct("odl_hip_max_pool2d_backward", ptr(gyp), ptr(idx), *pg, ptr(gxp), stream)
    ms_pf, ms_pb = time_region_auto(torch, pf), time_region_auto(torch, pb)
    nb_p = 4.0 * y.numel() + 12.0 * yp.numel()
    out["max_pool_2x2_256x32x28x28"] = {
        "fwd_ms": ms_pf, "bwd_ms": ms_pb, "fwd_gbs": nb_p / ms_pf / 1e6, "bwd_gbs": nb_p / ms_pb / 1e6,
        "fwd_frac_hbm": nb_p / ms_pf / 1e6 / PEAK_HBM_GBS, "bwd_frac_hbm": nb_p / ms_pb / 1e6 / PEAK_HBM_GBS}
    del x, w, b, gy, y, gx, gw, yp, idx, gyp, gxp
    keep.clear()
    # gradient reductions: the MLP's own shapes (launch-bound) and scaled shapes that can saturate HBM
    for name, shape in (("bias_grad_512x1000", (512, 1000)), ("bias_grad_16384x4096_scaled", (16384, 4096))):
        x, o = rnd(*shape), empty(1, shape[1])
        ss, ts = (ctypes.c_int64 * 2)(*shape), (ctypes.c_int64 * 2)(1, shape[1])
        wr, nr = ws(L.query("odl_hip_sum_to_workspace_bytes", ss, 2, ts, 2))
        ms = time_region_auto(torch, direct("odl_hip_sum_to", ptr(x), ss, 2, ts, 2, ptr(o), wr, nr, stream))
        nb = 4.0 * (x.numel() + shape[1])
        out[name] = {"ms": ms, "gbs": nb / ms / 1e6, "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS}
    for name, (N, C) in (("softmax_ce_grad_512x10", (512, 10)), ("softmax_ce_grad_16384x1000_scaled", (16384, 1000))):
        x, gx = rnd(N, C), empty(N, C)
        t = torch.randint(0, C, (N,), device="cuda", generator=g)
        ms = time_region_auto(torch, direct("odl_hip_softmax_ce_grad", ptr(x), ptr(t), 1, N, C, ctypes.c_float(1.0), ptr(gx),
                                            stream))
        nb = 8.0 * N * C + 8.0 * N
        out[name] = {"ms": ms, "gbs": nb / ms / 1e6, "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS}
    # batch normalisation at the shape of the first BatchNorm2d of the reference's conv_mnist example, batch 256.
    # Algorithmic bytes: forward reads x and writes y and x_norm; backward reads gy and x_norm and writes gx (the
    # statistics passes re-read what the first pass brought in; 51 MB fits the 256 MB last-level cache).
    N, C, P = 256, 64, 28 * 28
    x, gam, bet = rnd(N, C, P), rnd(C), rnd(C)
    rmean, rvar = torch.zeros(C, device="cuda"), torch.ones(C, device="cuda")
    y, xn, gx, gyb = empty(N, C, P), empty(N, C, P), empty(N, C, P), rnd(N, C, P)
    mean, var, dg, dbt = empty(C), empty(C), empty(C), empty(C)
    wbn, nbn = ws(L.query("odl_hip_batch_norm_workspace_bytes", N, C, P))
    f = direct("odl_hip_batch_norm_forward", ptr(x), ptr(gam), ptr(bet), ptr(rmean), ptr(rvar), 1, ctypes.c_float(1e-5),
               N, C, P, ptr(y), ptr(mean), ptr(var), ptr(xn), wbn, nbn, stream)
    b = direct("odl_hip_batch_norm_backward", ptr(gyb), ptr(gam), ptr(var), ptr(xn), ctypes.c_float(1e-5), N, C, P,
               ptr(gx), ptr(dg), ptr(dbt), wbn, nbn, stream)
    ms_f, ms_b = time_region_auto(torch, f), time_region_auto(torch, b)
    nb = 12.0 * N * C * P
    out["batch_norm_256x64x28x28"] = {"fwd_ms": ms_f, "bwd_ms": ms_b, "fwd_gbs": nb / ms_f / 1e6,
                                      "bwd_gbs": nb / ms_b / 1e6, "fwd_frac_hbm": nb / ms_f / 1e6 / PEAK_HBM_GBS,
                                      "bwd_frac_hbm": nb / ms_b / 1e6 / PEAK_HBM_GBS}
    del x, y, xn, gx, gyb
    keep.clear()
    # The streaming operators of the path at sizes that can saturate HBM (the MLP's and CNN's own shapes are a few
    # microseconds of launch latency each). Algorithmic bytes: every input read once, every output written once.
    def hbm_row(name, fn, nbytes):
        ms = time_region_auto(torch, fn)
        out[name] = {"ms": ms, "gbs": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS}

    R, Cc = 16384, 4096
    big, big2, res = rnd(R, Cc), rnd(R, Cc), empty(R, Cc)
    nbig = 4.0 * R * Cc
    hbm_row("transpose_16384x4096", direct("odl_hip_transpose", ptr(big), ptr(res), 1, R, Cc, stream), 2 * nbig)
    shp, perm = (ctypes.c_int64 * 5)(32, 3, 85, 80, 80), (ctypes.c_int * 5)(0, 1, 3, 4, 2)
    npm = 4.0 * 32 * 3 * 85 * 80 * 80
    hbm_row("permute_detect_head_32x3x85x80x80", direct("odl_hip_permute", ptr(big), 0, shp, 5, perm, ptr(res), stream), 2 * npm)
    hbm_row("relu_64Mi", direct("odl_hip_unary", 0, ptr(big), R * Cc, ptr(res), stream), 2 * nbig)
    hbm_row("add_64Mi", direct("odl_hip_binary", 0, ptr(big), R * Cc, ptr(big2), R * Cc, ptr(res), stream), 3 * nbig)
    row = rnd(1, Cc)
    ss, ts = (ctypes.c_int64 * 2)(1, Cc), (ctypes.c_int64 * 2)(R, Cc)
    hbm_row("broadcast_to_1x4096_to_16384x4096", direct("odl_hip_broadcast_to", ptr(row), ss, 2, ts, 2, ptr(res), stream),
            nbig + 4.0 * Cc)
    rs = empty(R)
    wr, nr = ws(L.query("odl_hip_sum_axis_workspace_bytes", R, Cc, 1))
    hbm_row("row_sums_16384x4096", direct("odl_hip_sum_axis", ptr(big), R, Cc, 1, ptr(rs), wr, nr, stream), nbig + 4.0 * R)
    sm_in, sm_out = rnd(R, 1000), empty(R, 1000)
    hbm_row("softmax_16384x1000", direct("odl_hip_softmax", ptr(sm_in), R, 1000, 1, ptr(sm_out), stream), 8.0 * R * 1000)
    am = torch.empty((R,), dtype=torch.int64, device="cuda")
    hbm_row("argmax_rows_16384x1000", direct("odl_hip_argmax_rows", ptr(sm_in), R, 1000, ptr(am), stream), 4.0 * R * 1000 + 8.0 * R)
    tot = empty(1)
    wr, nr = ws(L.query("odl_hip_sum_all_workspace_bytes", R * Cc))
    hbm_row("sum_all_64Mi", direct("odl_hip_sum_all", ptr(big), R * Cc, ptr(tot), wr, nr, stream), nbig)
    cm = empty(Cc)
    hbm_row("max_over_rows_16384x4096", direct("odl_hip_max_axis", ptr(big), 1, R, Cc, ptr(cm), stream), nbig + 4.0 * Cc)
    hbm_row("max_along_rows_16384x4096", direct("odl_hip_max_axis", ptr(big), R, Cc, 1, ptr(rs), stream), nbig + 4.0 * R)
    # the detector's shape operators at batch 32: 2x nearest upsample of a P4 map, the concatenation that follows it,
    # SiLU over a P3 map, and the float32 -> float64 conversion of the same map
    up_in, up_out = rnd(32, 128, 40, 40), empty(32, 128, 80, 80)
    hbm_row("upsample2x_32x128x40x40", direct("odl_hip_upsample_nearest", ptr(up_in), 32, 128, 40, 40, 80, 80, 2, 2, ptr(up_out),
                                              stream), 4.0 * (up_in.numel() + up_out.numel()))
    cat_b, cat_out = rnd(32, 64, 80, 80), empty(32, 192, 80, 80)
    ins = (ctypes.c_void_p * 2)(up_out.data_ptr(), cat_b.data_ptr())
    szs = (ctypes.c_int64 * 2)(128, 64)
    keep.extend([ins, szs])
    hbm_row("cat_channels_128+64_at_32x80x80", direct("odl_hip_cat", ins, szs, 2, 32, 6400, ptr(cat_out), stream),
            8.0 * cat_out.numel())
    hbm_row("silu_32x192x80x80", direct("odl_hip_unary", 7, ptr(cat_out), cat_out.numel(), ptr(cat_out), stream), 8.0 * cat_out.numel())
    f64 = torch.empty(cat_b.shape, dtype=torch.float64, device="cuda")
    hbm_row("convert_f32_to_f64_13Mi", direct("odl_hip_convert", ptr(cat_b), 0, ptr(f64), 1, cat_b.numel(), stream),
            12.0 * cat_b.numel())
    del up_in, up_out, cat_b, cat_out, f64
    pm_, gm_, mm_, vm_ = rnd(R * 1024), rnd(R * 1024), torch.zeros(R * 1024, device="cuda"), torch.zeros(R * 1024, device="cuda")
    f32c = ctypes.c_float
    hbm_row("adam_step_16Mi", direct("odl_hip_adam_step", ptr(pm_), ptr(gm_), ptr(mm_), ptr(vm_), R * 1024, f32c(0.9), f32c(0.999),
                                     f32c(10.0), f32c(1000.0), f32c(1e-8), f32c(1e-3), ptr(pm_), stream), 7 * 4.0 * R * 1024)
    del big, big2, res, row, rs, sm_in, sm_out, am, pm_, gm_, mm_, vm_
    keep.clear()
    # config 2's other shapes: forward + both gradient GEMMs, 6*M*N*K FLOP per step
    for (M, K, N) in ((1024, 1024, 1024), (2048, 2048, 2048), (8192, 8192, 8192), (512, 784, 1000), (512, 1000, 10)):
        a, b, dc = rnd(M, K), rnd(K, N), rnd(M, N)
        c, da, db = empty(M, N), empty(M, K), empty(K, N)
        wsz = max(L.query("odl_hip_matmul_backward_workspace_bytes", M, K, N),
                  L.query("odl_hip_matmul_workspace_bytes", 1, M, N, K, 0))
        wp, nw = ws(wsz)
        fwd = direct("odl_hip_matmul", ptr(a), ptr(b), ptr(c), 1, M, N, K, 0, wp, nw, stream)
        bwd = direct("odl_hip_matmul_backward", ptr(a), ptr(b), ptr(dc), ptr(da), ptr(db), M, K, N, wp, nw, stream)
        def both():
            fwd()
            bwd()

        ms = time_region(torch, both, 3, 1) if M >= 8192 else time_region_auto(torch, both)
        flop = 6.0 * M * N * K
        tf = flop / ms / 1e9
        out["gemm_fwd_bwd_%dx%dx%d" % (M, K, N)] = {"ms": ms, "tflops": tf, "frac_mfma_peak": tf / PEAK_FP32_MFMA_TFLOPS,
                                                      "flop": flop}
        del a, b, dc, c, da, db
        keep.clear()
    # the same three products on float64 tensors (FP64 matrix cores, 78.6 TFLOP/s): C = A.B, dA = dC.B^T, dB = A^T.dC
    for S in (2048, 4096):
        a, b, dc = (torch.randn((S, S), device="cuda", dtype=torch.float64, generator=g) for _ in range(3))
        c, da, db = (torch.empty((S, S), device="cuda", dtype=torch.float64) for _ in range(3))
        calls = [direct("odl_hip_dgemm", 0, 0, S, S, S, ptr(a), S, ptr(b), S, ptr(c), S, 1, 0, 0, 0, stream),
                 direct("odl_hip_dgemm", 0, 1, S, S, S, ptr(dc), S, ptr(b), S, ptr(da), S, 1, 0, 0, 0, stream),
                 direct("odl_hip_dgemm", 1, 0, S, S, S, ptr(a), S, ptr(dc), S, ptr(db), S, 1, 0, 0, 0, stream)]

        def all_three():
            for f in calls:
                f()

        ms = time_region_auto(torch, all_three)
        flop = 6.0 * S * S * S
        out["gemm_f64_fwd_bwd_%d" % S] = {"ms": ms, "tflops": flop / ms / 1e9, "frac_fp64_mfma_peak": flop / ms / 1e9 / 78.6,
                                            "flop": flop}
        del a, b, dc, c, da, db
        keep.clear()
    # the MLP's six GEMMs (config 1): 512x784x1000 and 512x1000x10, forward + backward
    x1, w1, g1 = rnd(512, 784), rnd(784, 1000), rnd(512, 1000)
    x2, w2, g2 = rnd(512, 1000), rnd(1000, 10), rnd(512, 10)

    def mlp_gemms():
        capi.mat_mul(x1, w1)
        capi.mat_mul(x2, w2)
        capi.mat_mul_backward(x2, w2, g2)
        capi.mat_mul_backward(x1, w1, g1)

    ms = time_region_auto(torch, mlp_gemms)
    flop = 6.0 * 512 * (784 * 1000 + 1000 * 10)
    out["mlp_gemms_fwd_bwd"] = {"ms": ms, "tflops": flop / ms / 1e9, "flop": flop}
    return out


def train_steps(steps, warmup, with_cpu):
    """Configs 1 and 4 as whole training steps through the C++ host layer (Tensor/Operator/nn/optim over the C ABI):
    forward, softmax-CE loss (read back each step, as the reference's loop does), backward, optimizer step, on
    tensors resident in HBM. The same driver source compiled against the reference gives the CPU time beside it."""
    import numpy as np
    import oraclelib as ol
    out = {}
    if not os.path.exists(ol.HOST_DRIVER_SO):
        return {"error": "host layer not built"}
    h = ol.host_driver()
    # loss = [loss of the first step from the initial parameters, loss of the last step]: the first is the number to
    # compare between the ordinary run, the replayed run and the CPU reference (they take different numbers of steps)
    ms, loss = np.zeros(1, np.float32), np.zeros(2, np.float32)
    rc = h.odl_host_mlp_bench(512, 784, 1000, 10, steps, warmup, ms, loss)
    out["mlp_512x784x1000x10_adam"] = {"rc": rc, "ms_per_step": float(ms[0]), "loss_step_1": float(loss[0]),
                                       "gemm_flop_per_step": 6.0 * 512 * (784 * 1000 + 1000 * 10)}
    # the same step with the network as one nn::MLP object, the way the reference's own training loop builds it
    rc = h.odl_host_mlp_model_bench(512, 784, 1000, 10, steps, warmup, 0, ms, loss)
    out["mlp_512x784x1000x10_adam"].update({"nn_MLP_object_rc": rc, "nn_MLP_object_ms_per_step": float(ms[0]),
                                            "nn_MLP_object_loss_step_1": float(loss[0])})
    rc = h.odl_host_cnn_bench(256, steps, warmup, ms, loss)
    out["cnn_b256_sgd"] = {"rc": rc, "ms_per_step": float(ms[0]), "loss_step_1": float(loss[0])}
    # the same steps recorded once into a HIP graph and replayed (one submission per step instead of ~50 launches);
    # the loss is still read back after every step
    rc = h.odl_host_mlp_bench_graph(512, 784, 1000, 10, steps, warmup, 1, ms, loss)
    out["mlp_512x784x1000x10_adam"].update({"graph_replay_rc": rc, "graph_replay_ms_per_step": float(ms[0]),
                                            "graph_replay_loss_step_1": float(loss[0])})
    rc = h.odl_host_cnn_bench_graph(256, steps, warmup, 1, ms, loss)
    out["cnn_b256_sgd"].update({"graph_replay_rc": rc, "graph_replay_ms_per_step": float(ms[0]),
                                "graph_replay_loss_step_1": float(loss[0])})
    # the network of the reference's own conv_mnist example (with its BatchNorm layers, Adam + WeightDecay), batch 256;
    # device only: the reference's BatchNorm operator cannot run backward
    losses = np.zeros(3, np.float32)
    rc = h.odl_host_cnn_bn_bench(256, steps, warmup, 0, ms, losses)
    out["cnn_batchnorm_b256_adam"] = {"rc": rc, "ms_per_step": float(ms[0]), "loss_before": float(losses[0]),
                                      "loss_last_step": float(losses[1]), "loss_eval_mode": float(losses[2])}
    rc = h.odl_host_cnn_bn_bench(256, steps, warmup, 1, ms, losses)
    out["cnn_batchnorm_b256_adam"].update({"graph_replay_rc": rc, "graph_replay_ms_per_step": float(ms[0])})
    # the same two steps run by the REFERENCE's own Tensor / Operator / nn / optim object code over binding/ (its
    # op-by-op graph: no fused layers, no recorded step; built only where the reference checkout was present)
    if os.path.exists(ol.BIND_DRIVER_SO):
        bd = ol.binding_driver()
        rc = bd.odl_bind_mlp_bench(512, 784, 1000, 10, steps, warmup, ms, loss)
        out["mlp_512x784x1000x10_adam"].update({"reference_classes_over_binding_rc": rc,
                                                "reference_classes_over_binding_ms_per_step": float(ms[0]),
                                                "reference_classes_over_binding_loss_step_1": float(loss[0])})
        rc = bd.odl_bind_cnn_bench(256, steps, warmup, ms, loss)
        out["cnn_b256_sgd"].update({"reference_classes_over_binding_rc": rc,
                                    "reference_classes_over_binding_ms_per_step": float(ms[0]),
                                    "reference_classes_over_binding_loss_step_1": float(loss[0])})
    out["yolov5n_forward_4x3x320x320"] = yolo_forward(h, ol.ref() if with_cpu and ol.have_ref() else None, steps)
    if with_cpu and ol.have_ref():
        r = ol.ref()
        rc = r.odl_ref_mlp_bench(512, 784, 1000, 10, 1, 0, ms, loss)
        out["mlp_512x784x1000x10_adam"]["cpu_reference_ms_per_step"] = float(ms[0])
        out["mlp_512x784x1000x10_adam"]["cpu_reference_loss_step_1"] = float(loss[0])
        rc = r.odl_ref_cnn_bench(4, 1, 0, ms, loss)
        out["cnn_b256_sgd"]["cpu_reference_ms_per_step_extrapolated_from_batch_4"] = float(ms[0]) * 64.0
        out["cnn_b256_sgd"]["cpu_reference_loss_step_1_at_batch_4"] = float(loss[0])
    return out


def yolo_forward(h, ref, reps):
    """Config 5: a YOLOv5n-architecture model (depth 0.33, width 0.25, random weights from a seed, written in PNNX's
    file format by tests/pnnx_synth.py) run forward on [4,3,320,320] by the host layer's PNNX graph runner; the
    reference's own runner on one CPU core beside it, at batch 1 (its time scales with the batch)."""
    import tempfile
    import numpy as np
    import pnnx_synth
    res = {}
    with tempfile.TemporaryDirectory() as tmp:
        def run(drv, name, batch, n):
            param, binp, shp = pnnx_synth.write(os.path.join(tmp, "y5n_b%d" % batch), seed=0, batch=batch, size=320)
            x = np.random.default_rng(0).random((batch, 3, 320, 320), dtype=np.float32)
            o = np.empty(shp, np.float32)
            oshape, nd, ms = np.zeros(8, np.int64), np.zeros(1, np.int32), np.zeros(1, np.float32)
            t0 = time.perf_counter()
            rc = getattr(drv, name)(param.encode(), binp.encode(), x, batch, 3, 320, 320, n, o, o.size, oshape, nd, ms)
            return rc, float(ms[0]), time.perf_counter() - t0, o
        n = max(10, reps) + 1
        rc, ms, _, o = run(h, "odl_host_pnnx_forward", 4, n)
        gflop = pnnx_synth.flops(4, 320) / 1e9
        res.update({"rc": rc, "ms_per_forward": ms, "conv_gflop": gflop, "tflops": gflop / ms if ms > 0 else None,
                    "output_shape": list(o.shape), "output_mean": float(o.mean())})
        # the same forward recorded into a graph and replayed, and how many launches it holds
        nodes = np.zeros(1, np.int64)
        rc, ms_g, _, og = run(h, "odl_host_pnnx_forward_graph", 4, n)
        h.odl_host_pnnx_last_graph_nodes(nodes)
        res.update({"graph_replay_rc": rc, "graph_replay_ms_per_forward": ms_g, "launches_per_forward": int(nodes[0]),
                    "graph_replay_equals_eager": bool(np.array_equal(o, og))})
        # every node on its own, as the reference's runner goes through the graph (no add / concatenation / pool chain
        # folded into its producer): same kernels for the convolutions, same floats
        h.odl_host_pnnx_set_fusion(0)
        try:
            rc, ms_p, _, op = run(h, "odl_host_pnnx_forward", 4, n)
            rc2, _, _, _ = run(h, "odl_host_pnnx_forward_graph", 4, 2)
            h.odl_host_pnnx_last_graph_nodes(nodes)
        finally:
            h.odl_host_pnnx_set_fusion(1)
        res.update({"node_by_node_rc": rc, "node_by_node_ms_per_forward": ms_p, "node_by_node_launches_per_forward": int(nodes[0]),
                    "node_by_node_equals_folded": bool(np.array_equal(o, op))})
        if ref is not None:
            rc, _, wall, _ = run(ref, "odl_ref_pnnx_forward", 1, 1)
            res["cpu_reference_ms_per_forward_batch_1"] = wall * 1e3
            res["cpu_reference_ms_per_forward_extrapolated_to_batch_4"] = wall * 4e3
    return res


# HBM-side bytes of one 4096^3 GEMM launch, a recorded constant (counters cannot be read from inside this process):
# FETCH_SIZE (scaled 2.000x by the calibration copy) 738.0 MiB on average over the NN / NT / TN variants
# (713 / 763 / 737; between 510 and 880 from run to run) + WRITE_SIZE (1.000x) 64.0 MiB, from the two `rocprofv3 --pmc`
# runs of `--pmc-probe` summarised in profiles/hot_kernels_hbm_traffic.md.
GEMM_4096_TRAFFIC_BYTES = int((738.0 + 64.0) * 1024 * 1024)


def pmc_probe(torch, capi, gemm_step):
    """A short, fixed launch sequence for counter runs (`rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`):
    first a plain elementwise copy-like kernel of known traffic (negate of 64 Mi floats: 256 MiB read, 256 MiB
    written) that calibrates the counters, then each hot kernel a few times."""
    g = torch.Generator(device="cuda").manual_seed(0)
    cal = torch.randn((64 * 1024 * 1024,), device="cuda", generator=g)
    for _ in range(3):
        capi.unary("neg", cal)
    for _ in range(3):
        gemm_step()
    x = torch.randn((32, 64, 56, 56), device="cuda", generator=g)
    w = torch.randn((128, 64, 3, 3), device="cuda", generator=g) * 0.06
    b = torch.randn((128,), device="cuda", generator=g)
    gy = torch.randn((32, 128, 56, 56), device="cuda", generator=g)
    for _ in range(2):
        capi.conv2d(x, w, b, 1, 1)
        capi.conv2d_backward(gy, x, w, True, 1, 1)
    for _ in range(2):
        col = capi.im2col(x, 3, 1, 1, True)
        capi.col2im(col, x.shape, 3, 1, 1, True)
    del col
    big = torch.randn((16384, 4096), device="cuda", generator=g)
    logits = torch.randn((16384, 1000), device="cuda", generator=g)
    t = torch.randint(0, 1000, (16384,), device="cuda", generator=g)
    for _ in range(3):
        capi.sum_to(big, (1, 4096))
        capi.softmax_cross_entropy_backward(logits, t, 1.0)
    torch.cuda.synchronize()
    print("pmc probe done")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--size", type=int, default=4096)
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--train-probe", action="store_true",
                    help="only the MLP/CNN training steps through the C++ host layer (for rocprofv3 --kernel-trace)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="few launches of each hot kernel plus a plain copy of known size, for rocprofv3 --pmc runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; nothing here uses a second one (no collectives, no sharding). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    if args.train_probe:
        print(json.dumps(train_steps(args.steps, args.warmup, False)))
        return

    import torch
    from origindl_amd import capi  # raises if libodl_hip.so is missing: there is no fallback

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)
    S = args.size
    g = torch.Generator(device="cuda").manual_seed(1)
    a = torch.randn((S, S), device="cuda", generator=g)
    b = torch.randn((S, S), device="cuda", generator=g)
    dc = torch.randn((S, S), device="cuda", generator=g)
    # outputs and the (possibly empty) workspace are allocated once: the timed region is kernels only
    c, da, db = torch.empty_like(a), torch.empty_like(a), torch.empty_like(a)
    import ctypes
    lib = capi.lib()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ws_bytes = max(lib.query("odl_hip_matmul_backward_workspace_bytes", S, S, S),
                   lib.query("odl_hip_matmul_workspace_bytes", 1, S, S, S, 0))
    ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.int32, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731

    def step():
        lib.call("odl_hip_matmul", p(a), p(b), p(c), 1, S, S, S, 0, p(ws), ws_bytes, st)
        lib.call("odl_hip_matmul_backward", p(a), p(b), p(dc), p(da), p(db), S, S, S, p(ws), ws_bytes, st)

    if args.pmc_probe:
        pmc_probe(torch, capi, step)
        return

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ev_ms = e0.elapsed_time(e1) / args.steps
    ms = max(wall_ms, ev_ms)
    flop_step = 6.0 * S * S * S
    value = flop_step / ms / 1e9

    # the dominant kernel: three launches of the MFMA GEMM per step (NN, NT, TN), each 2*S^3 FLOP
    launch_ms = ev_ms / 3.0
    achieved = 2.0 * S * S * S / launch_ms / 1e9
    line = {
        "metric": "fwd+bwd TFLOP/s (GEMM %d^3) fp32 at 1 GPU" % S,
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic N(0,1) operands, seeded, resident in HBM",
        "config": {"workload": "matmul fwd+bwd: C=A.B, dA=dC.B^T, dB=A^T.dC, M=N=K=%d" % S, "flop_per_step": flop_step},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_FP32_MFMA_TFLOPS,
                     "traffic": GEMM_4096_TRAFFIC_BYTES if S == 4096 else None,
                     "traffic_source": ("recorded constant: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py "
                                        "--pmc-probe`, profiles/hot_kernels_hbm_traffic.md" if S == 4096 else None),
                     "kernel": "sgemm_dma_kernel<128,128,16,TA,TB,2> (NN, NT, TN)", "launch_ms": launch_ms},
        "device": capi.device_info(0),
    }
    if not args.no_extras:
        line["extras"] = extras(torch, capi, max(3, args.steps // 2), max(2, args.warmup // 2))
        line["extras"]["train_steps"] = train_steps(max(5, args.steps // 2), 3, not args.no_cpu)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_gemm(S)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
