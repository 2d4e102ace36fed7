"""CPU-side checks of the boundary: the header parses, the built library exports every declared symbol,
argument validation that needs no GPU behaves, and compute entry points refuse to run without a device."""
import ctypes
import os

import pytest

from origindl_amd import _lib


def test_header_declares_the_expected_surface():
    protos = _lib.parse_header()
    for name in ("odl_hip_sgemm", "odl_hip_matmul", "odl_hip_matmul_backward", "odl_hip_im2col", "odl_hip_col2im",
                 "odl_hip_conv2d", "odl_hip_conv2d_backward", "odl_hip_sum_axis", "odl_hip_sum_all", "odl_hip_sum_to",
                 "odl_hip_sum_nchw_channels", "odl_hip_broadcast_to", "odl_hip_max_axis", "odl_hip_softmax",
                 "odl_hip_gather", "odl_hip_one_hot", "odl_hip_softmax_ce_loss", "odl_hip_softmax_ce_grad",
                 "odl_hip_max_pool2d", "odl_hip_max_pool2d_backward", "odl_hip_argmax_rows", "odl_hip_accuracy",
                 "odl_hip_binary", "odl_hip_unary", "odl_hip_pow_scalar", "odl_hip_fill", "odl_hip_malloc",
                 "odl_hip_free", "odl_hip_memcpy_h2d", "odl_hip_memcpy_d2h", "odl_hip_device_count",
                 "odl_hip_last_error"):
        assert name in protos, name
    ret, args = protos["odl_hip_sgemm"]
    assert ret is ctypes.c_int and len(args) == 16


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m origindl_amd.build"
    cdll = ctypes.CDLL(_lib.LIB_PATH)
    for name in _lib.parse_header():
        assert hasattr(cdll, name), "%s declared in include/odl_hip.h but not exported" % name


def test_workspace_queries_need_no_gpu():
    l = _lib.lib()
    # conv C1 of the benchmark runs as implicit GEMM: no col matrix (231 MB); only the weights re-ordered to
    # [OC][tap][C] and the K pieces of its last 16 tiles
    wp = 128 * 64 * 9 * 4
    assert l.query("odl_hip_conv2d_workspace_bytes", 32, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1) == wp + 16 * 12 * 128 * 128 * 4
    # a tile count that is a multiple of the CU count needs no K pieces
    assert l.query("odl_hip_conv2d_workspace_bytes", 32, 64, 32, 32, 128, 3, 3, 1, 1, 1, 1) == wp
    # a 1x1 window's weights are in tap order as they are
    assert l.query("odl_hip_conv2d_workspace_bytes", 64, 128, 32, 32, 256, 1, 1, 1, 1, 0, 0) == 0
    # a small problem (up to 1.6 GFLOP, channels in eights) goes to the kernel that reads its operands straight from
    # global memory: the workspace holds the filter copy in that kernel's order, whole tiles of 32 filters
    assert l.query("odl_hip_conv2d_workspace_bytes", 32, 64, 32, 32, 128, 1, 1, 1, 1, 0, 0) == 128 * 64 * 4
    assert l.query("odl_hip_conv2d_workspace_bytes", 4, 64, 40, 40, 255, 1, 1, 1, 1, 0, 0) == 256 * 64 * 4
    # (a 3x3 / padding 1 window's three rows are padded to four floats each in that copy; other windows are not)
    assert l.query("odl_hip_conv2d_packed_weights_bytes", 4, 128, 10, 10, 128, 3, 3, 1, 1, 1, 1) == 128 * 128 * 12 * 4
    assert l.query("odl_hip_conv2d_packed_weights_bytes", 4, 128, 10, 10, 128, 3, 3, 1, 1, 0, 0) == 128 * 128 * 9 * 4
    assert l.query("odl_hip_conv2d_fused_ok", 4, 128, 10, 10, 128, 3, 3, 1, 1, 1, 1) == 1
    assert l.query("odl_hip_conv2d_fused_ok", 4, 3, 320, 320, 16, 6, 6, 2, 2, 2, 2) == 0
    assert l.query("odl_hip_conv2d_fused_ok", 32, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1) == 0
    # one input channel under a 3x3 window: the direct kernel, no matrix and no workspace
    assert l.query("odl_hip_conv2d_workspace_bytes", 256, 1, 28, 28, 32, 3, 3, 1, 1, 1, 1) == 0
    # its backward: the weight-gradient partials (one [32][9] block per workgroup) and the reordered filter
    assert 0 < l.query("odl_hip_conv2d_backward_workspace_bytes", 256, 1, 28, 28, 32, 3, 3, 1, 1, 1, 1) < 2 * 1024 * 1024
    # C*KH*KW = 45 is not a multiple of 4: explicit im2col path, workspace = the col matrix [N*OH*OW, 45]
    assert l.query("odl_hip_conv2d_workspace_bytes", 16, 5, 28, 28, 32, 3, 3, 1, 1, 1, 1) == 16 * 28 * 28 * 45 * 4
    assert l.query("odl_hip_conv2d_backward_workspace_bytes", 32, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1) < 100352 * 576 * 4
    assert l.query("odl_hip_conv2d_workspace_bytes", 1, 1, 2, 2, 1, 3, 3, 1, 1, 0, 0) == 0  # no valid output
    # 3x3/s1/p1 over 32 input channels with enough pixels to fill the chip: the LDS-patch kernel's re-ordered filter
    # copy (9*C*OC floats, rows padded to the 64-row tile) bounds the forward's need from below; a batch too small
    # for it (fewer than 256 workgroups) asks for less
    assert l.query("odl_hip_conv2d_workspace_bytes", 256, 32, 14, 14, 64, 3, 3, 1, 1, 1, 1) >= 9 * 32 * 64 * 4
    assert l.query("odl_hip_conv2d_workspace_bytes", 256, 32, 14, 14, 64, 3, 3, 1, 1, 1, 1) < 256 * 196 * 288 * 4
    assert (l.query("odl_hip_conv2d_backward_workspace_bytes", 256, 32, 14, 14, 64, 3, 3, 1, 1, 1, 1) >=
            9 * 64 * 32 * 4)
    assert l.query("odl_hip_sum_axis_workspace_bytes", 4096, 10, 1) == 0
    assert l.query("odl_hip_sum_axis_workspace_bytes", 1, 16384, 4096) > 0
    src = (ctypes.c_int64 * 2)(512, 1000)
    dst = (ctypes.c_int64 * 2)(1, 1000)
    assert l.query("odl_hip_sum_to_workspace_bytes", src, 2, dst, 2) >= 0


def test_compute_refuses_to_run_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    l = _lib.lib()
    rc = l.cdll.odl_hip_fill(None, 4, ctypes.c_float(1.0), None)
    assert rc == _lib.ODL_ERR_RUNTIME and "HIP device" in l.last_error()
    with pytest.raises(_lib.OdlRuntimeError):
        l.call("odl_hip_sgemm", 0, 0, 4, 4, 4, None, 4, None, 4, None, 4, None, 0, None, 0, None)


def test_host_layer_refuses_cpu_compute():
    """The C++ host layer has no CPU compute path: with tensors left on the CPU every operator call throws
    runtime_error (the API driver reports -2), while creation / transfer of CPU tensors still works."""
    import numpy as np
    import oraclelib as ol
    if not os.path.exists(ol.HOST_CPU_DRIVER_SO):
        pytest.skip("host layer not built")
    h = ol.host_driver(cpu=True)
    assert h.odl_hostcpu_ping() == 1
    a, b, c = np.ones((2, 3), np.float32), np.ones((3, 2), np.float32), np.zeros((2, 2), np.float32)
    assert h.odl_hostcpu_matmul(a, b, c, 2, 2, 3) == -2
    assert h.odl_hostcpu_unary(0, a, 6, np.zeros_like(a)) == -2
    loss = np.zeros(1, np.float32)
    assert h.odl_hostcpu_softmax_ce(a, np.zeros(2, np.int32), 0, 2, 3, loss, None) == -2
    assert (c == 0).all()
