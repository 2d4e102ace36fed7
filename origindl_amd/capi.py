"""Thin convenience layer over the C ABI (include/odl_hip.h) for tests, the smoke check and the benchmark.

torch is used for exactly two things: device memory (tensors own the buffers whose raw pointers go through the
C ABI) and the stream the kernels are launched on. No torch operator computes anything here, and nothing
falls back to torch or to the CPU: every function below is one call into libodl_hip.so.

Names and argument meaning follow the reference's Mat interface (include/origin/mat/mat.h) and operators
(src/operators/**): mat_mul, mat_mul_backward, im2col, col2im, conv2d, conv2d_backward, sum, sum_to,
broadcast_to, max, softmax, gather, one_hot, softmax_cross_entropy(+_backward), max_pool2d(+_backward),
accuracy, and the elementwise set. Errors surface as OdlInvalidArgument / OdlRuntimeError, the counterparts of
the reference's std::invalid_argument / std::runtime_error."""
import builtins as _builtins
import ctypes

import numpy as np
import torch

from ._lib import OdlInvalidArgument, OdlRuntimeError, lib  # noqa: F401

_f32 = torch.float32


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _chk(t, name="tensor", dtype=_f32):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous() and t.dtype == dtype):
        raise OdlInvalidArgument("%s must be a contiguous %s device tensor" % (name, dtype))
    return t


def _empty(shape, dtype=_f32):
    return torch.empty(tuple(int(s) for s in shape), dtype=dtype, device="cuda")


def _ws(nbytes):
    nbytes = int(nbytes)
    if nbytes == 0:
        return None, 0
    buf = torch.empty((nbytes + 3) // 4, dtype=torch.int32, device="cuda")
    return buf, nbytes


def _shape_arr(shape):
    arr = (ctypes.c_int64 * _builtins.max(len(shape), 1))(*[int(s) for s in shape])
    return arr


def _labels(t):
    if t.dtype == torch.int64:
        return _chk(t, "labels", torch.int64), 1
    if t.dtype == torch.int32:
        return _chk(t, "labels", torch.int32), 0
    raise OdlInvalidArgument("indices must be int32 or int64, but got %s" % t.dtype)


def conv_outsize(i, k, s, p):
    return (i + 2 * p - k) // s + 1


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else (int(v[0]), int(v[1]))


# ------------------------------------------------------------------------------------------ runtime
def device_count():
    n = ctypes.c_int(0)
    lib().call("odl_hip_device_count", ctypes.byref(n))
    return n.value


def is_available():
    return device_count() > 0


def device_info(device=0):
    buf = ctypes.create_string_buffer(256)
    lib().call("odl_hip_device_info", device, buf, 256)
    return buf.value.decode()


def synchronize():
    lib().call("odl_hip_synchronize")


# --------------------------------------------------------------------------------------------- GEMM
def sgemm(a, b, trans_a=False, trans_b=False, bias=None, split_k=0, out=None):
    """C = op(A) . op(B) (+ bias per column)."""
    _chk(a, "A"), _chk(b, "B")
    M, K = (a.shape[1], a.shape[0]) if trans_a else (a.shape[0], a.shape[1])
    K2, N = (b.shape[1], b.shape[0]) if trans_b else (b.shape[0], b.shape[1])
    if K != K2:
        raise OdlInvalidArgument("Matrix dimensions must be compatible for multiplication: K=%d vs %d" % (K, K2))
    c = out if out is not None else _empty((M, N))
    need = lib().query("odl_hip_sgemm_workspace_bytes", int(trans_a), int(trans_b), M, N, K, split_k)
    ws, nb = _ws(need)
    lib().call("odl_hip_sgemm", int(trans_a), int(trans_b), M, N, K, _p(a), a.shape[1], _p(b), b.shape[1], _p(c), N,
               _p(bias), split_k, _p(ws), nb, _stream())
    return c


def mat_mul(a, b):
    """Mat::matmul: 2-D x 2-D, 3-D x 2-D, 3-D x 3-D (src/mat/origin/cpu/math/matmul.cpp:113-218)."""
    _chk(a, "a"), _chk(b, "b")
    if a.dim() < 2 or b.dim() < 2:
        raise OdlInvalidArgument("Matrix multiplication requires at least 2D tensors")
    if a.dim() == 2 and b.dim() == 2:
        batch, M, K, bb = 1, a.shape[0], a.shape[1], 0
        oshape = (M, b.shape[1])
    elif a.dim() == 3 and b.dim() == 2:
        batch, M, K, bb = a.shape[0], a.shape[1], a.shape[2], 0
        oshape = (batch, M, b.shape[1])
    elif a.dim() == 3 and b.dim() == 3:
        if a.shape[0] != b.shape[0]:
            raise OdlInvalidArgument("Matrix dimensions must be compatible: batch %d vs %d" % (a.shape[0], b.shape[0]))
        batch, M, K, bb = a.shape[0], a.shape[1], a.shape[2], 1
        oshape = (batch, M, b.shape[2])
    else:
        raise OdlInvalidArgument("Matrix multiplication requires compatible dimensions")
    if b.shape[-2] != K:
        raise OdlInvalidArgument("Matrix dimensions must be compatible for multiplication: %s x %s"
                                 % (tuple(a.shape), tuple(b.shape)))
    N = b.shape[-1]
    c = _empty(oshape)
    ws, nb = _ws(lib().query("odl_hip_matmul_workspace_bytes", batch, M, N, K, bb))
    lib().call("odl_hip_matmul", _p(a), _p(b), _p(c), batch, M, N, K, bb, _p(ws), nb, _stream())
    return c


def mat_mul_backward(x, w, gy, need_gx=True, need_gw=True):
    """MatMul::backward (src/operators/math/mat_mul.cpp:123-182) -> (gx, gw)."""
    _chk(x, "x"), _chk(w, "w"), _chk(gy, "gy")
    M, K = x.shape
    N = w.shape[1]
    gx = _empty((M, K)) if need_gx else None
    gw = _empty((K, N)) if need_gw else None
    ws, nb = _ws(lib().query("odl_hip_matmul_backward_workspace_bytes", M, K, N))
    lib().call("odl_hip_matmul_backward", _p(x), _p(w), _p(gy), _p(gx), _p(gw), M, K, N, _p(ws), nb, _stream())
    return gx, gw


def linear_backward(x, w, gy, need_gx=True, need_gw=True, need_gb=True):
    """Backward of Linear::forward for 2-D inputs (src/nn/layers/linear.cpp:88-104) -> (gx, gw, gb[1, N])."""
    _chk(x, "x"), _chk(w, "w"), _chk(gy, "gy")
    M, K = x.shape
    N = w.shape[1]
    gx = _empty((M, K)) if need_gx else None
    gw = _empty((K, N)) if need_gw else None
    gb = _empty((1, N)) if need_gb else None
    ws, nb = _ws(lib().query("odl_hip_linear_backward_workspace_bytes", M, K, N))
    lib().call("odl_hip_linear_backward", _p(x), _p(w), _p(gy), _p(gx), _p(gw), _p(gb), M, K, N, _p(ws), nb, _stream())
    return gx, gw, gb


def transpose(x):
    _chk(x, "x")
    if x.dim() < 2:
        return x.clone()
    rows, cols = x.shape[-2], x.shape[-1]
    outer = int(np.prod(x.shape[:-2])) if x.dim() > 2 else 1
    out = _empty(tuple(x.shape[:-2]) + (cols, rows))
    lib().call("odl_hip_transpose", _p(x), _p(out), outer, rows, cols, _stream())
    return out


# ------------------------------------------------------------------------------------------- conv
def im2col(img, kernel_size, stride, pad, to_matrix=True):
    _chk(img, "img")
    if img.dim() != 4:
        raise OdlInvalidArgument("im2col: input must be 4D (N, C, H, W)")
    (KH, KW), (SH, SW), (PH, PW) = _pair(kernel_size), _pair(stride), _pair(pad)
    N, C, H, W = img.shape
    OH, OW = conv_outsize(H, KH, SH, PH), conv_outsize(W, KW, SW, PW)
    shape = (N * OH * OW, C * KH * KW) if to_matrix else (N, C, KH, KW, OH, OW)
    col = _empty([_builtins.max(s, 0) for s in shape])
    lib().call("odl_hip_im2col", _p(img), N, C, H, W, KH, KW, SH, SW, PH, PW, int(to_matrix), _p(col), _stream())
    return col


def col2im(col, input_shape, kernel_size, stride, pad, to_matrix=True):
    _chk(col, "col")
    if len(input_shape) != 4:
        raise OdlInvalidArgument("col2im: input_shape must be 4D (N, C, H, W)")
    (KH, KW), (SH, SW), (PH, PW) = _pair(kernel_size), _pair(stride), _pair(pad)
    N, C, H, W = [int(s) for s in input_shape]
    OH, OW = conv_outsize(H, KH, SH, PH), conv_outsize(W, KW, SW, PW)
    want = (N * OH * OW, C * KH * KW) if to_matrix else (N, C, KH, KW, OH, OW)
    if tuple(col.shape) != want:
        raise OdlInvalidArgument("col2im: invalid col shape %s for input_shape %s" % (tuple(col.shape), (N, C, H, W)))
    img = _empty((N, C, H, W))
    lib().call("odl_hip_col2im", _p(col), N, C, H, W, KH, KW, SH, SW, PH, PW, int(to_matrix), _p(img), _stream())
    return img


def matmul_f64(a, b, trans_a=False, trans_b=False):
    """Mat::matmul on float64 tensors: 2-D x 2-D, 3-D x 2-D or 3-D x 3-D (src/mat/origin/cpu/math/matmul.cpp:113-218);
    trans_a / trans_b read a 2-D operand as its transpose (the two products of MatMul::backward)."""
    _chk(a, "a", torch.float64), _chk(b, "b", torch.float64)
    batch, sa, sb = 1, 0, 0
    if a.dim() == 3:
        batch, sa = a.shape[0], a.shape[1] * a.shape[2]
        sb = b.shape[1] * b.shape[2] if b.dim() == 3 else 0
    ar, ac = a.shape[-2], a.shape[-1]
    br, bc = b.shape[-2], b.shape[-1]
    M, K = (ac, ar) if trans_a else (ar, ac)
    Kb, N = (bc, br) if trans_b else (br, bc)
    if K != Kb:
        raise OdlInvalidArgument("matmul: inner dimensions differ (%d and %d)" % (K, Kb))
    c = _empty(((batch, M, N) if a.dim() == 3 else (M, N)), torch.float64)
    lib().call("odl_hip_dgemm", int(trans_a), int(trans_b), M, N, K, _p(a), ac, _p(b), bc, _p(c), N, batch, sa, sb, M * N, _stream())
    return c


def conv2d_pack_weights(x_shape, w, stride=1, pad=0):
    """The filter copy, in the order the forward kernel for inputs of x_shape reads it, for weights that stay the same
    from call to call; None when that kernel reads the filter as it lies. Pass it to conv2d(packed=...)."""
    _chk(w, "W")
    N, C, H, W = (int(d) for d in x_shape)
    OC, _, KH, KW = w.shape
    (SH, SW), (PH, PW) = _pair(stride), _pair(pad)
    nbytes = lib().query("odl_hip_conv2d_packed_weights_bytes", N, C, H, W, OC, KH, KW, SH, SW, PH, PW)
    if nbytes == 0:
        return None
    packed = _empty((nbytes // 4,))  # rounded up to whole tiles of output channels for some kernels
    lib().call("odl_hip_conv2d_pack_weights", _p(w), N, C, H, W, OC, KH, KW, SH, SW, PH, PW, _p(packed), _stream())
    return packed


def conv2d(x, w, b=None, stride=1, pad=0, activation=None, packed=None):
    """Mat::conv2d (src/mat/origin/cpu/conv/conv2d.cpp:404-512); activation "relu" / "silu" runs in the epilogue."""
    _chk(x, "x"), _chk(w, "W")
    if x.dim() != 4:
        raise OdlInvalidArgument("conv2d: x must be 4D (N, C, H, W)")
    if w.dim() != 4:
        raise OdlInvalidArgument("conv2d: W must be 4D (OC, C, KH, KW)")
    N, C, H, W = x.shape
    OC, Cw, KH, KW = w.shape
    if C != Cw:
        raise OdlInvalidArgument("conv2d: channel mismatch - x has %d channels, but W expects %d" % (C, Cw))
    if b is not None and (b.dim() != 1 or b.shape[0] != OC):
        raise OdlInvalidArgument("conv2d: b must be 1D with size %d" % OC)
    (SH, SW), (PH, PW) = _pair(stride), _pair(pad)
    OH, OW = conv_outsize(H, KH, SH, PH), conv_outsize(W, KW, SW, PW)
    y = _empty((N, OC, _builtins.max(OH, 0), _builtins.max(OW, 0)))
    ws, nb = _ws(lib().query("odl_hip_conv2d_workspace_bytes", N, C, H, W, OC, KH, KW, SH, SW, PH, PW))
    act = -1 if activation is None else _UN[activation]
    lib().call("odl_hip_conv2d_act_packed", _p(x), _p(w), _p(packed), _p(b), N, C, H, W, OC, KH, KW, SH, SW, PH, PW, act,
               _p(y), _p(ws), nb, _stream())
    return y


def conv2d_backward(gy, x, w, has_bias=True, stride=1, pad=0):
    """Mat::conv2d_backward (conv2d.cpp:514-599) -> (gx, gW, gb or None)."""
    _chk(gy, "gy"), _chk(x, "x"), _chk(w, "W")
    if gy.dim() != 4 or x.dim() != 4 or w.dim() != 4:
        raise OdlInvalidArgument("conv2d_backward: gy, x and W must be 4D")
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    (SH, SW), (PH, PW) = _pair(stride), _pair(pad)
    gx, gw = _empty(x.shape), _empty(w.shape)
    gb = _empty((OC,)) if has_bias else None
    ws, nb = _ws(lib().query("odl_hip_conv2d_backward_workspace_bytes", N, C, H, W, OC, KH, KW, SH, SW, PH, PW))
    lib().call("odl_hip_conv2d_backward", _p(gy), _p(x), _p(w), N, C, H, W, OC, KH, KW, SH, SW, PH, PW, _p(gx), _p(gw),
               _p(gb), _p(ws), nb, _stream())
    return gx, gw, gb


# ---- the same operators on float64 tensors (src/mat/origin/cuda/conv/conv2d.cu:412-664 dispatches over the element type)
_f64 = torch.float64


def im2col_f64(img, kernel_size, stride, pad, to_matrix=True):
    _chk(img, "img", _f64)
    if img.dim() != 4:
        raise OdlInvalidArgument("im2col: input must be 4D (N, C, H, W)")
    (KH, KW), (SH, SW), (PH, PW) = _pair(kernel_size), _pair(stride), _pair(pad)
    N, C, H, W = img.shape
    OH, OW = conv_outsize(H, KH, SH, PH), conv_outsize(W, KW, SW, PW)
    shape = (N * OH * OW, C * KH * KW) if to_matrix else (N, C, KH, KW, OH, OW)
    col = _empty([_builtins.max(s, 0) for s in shape], _f64)
    lib().call("odl_hip_im2col_f64", _p(img), N, C, H, W, KH, KW, SH, SW, PH, PW, int(to_matrix), _p(col), _stream())
    return col


def col2im_f64(col, input_shape, kernel_size, stride, pad, to_matrix=True):
    _chk(col, "col", _f64)
    (KH, KW), (SH, SW), (PH, PW) = _pair(kernel_size), _pair(stride), _pair(pad)
    N, C, H, W = [int(s) for s in input_shape]
    OH, OW = conv_outsize(H, KH, SH, PH), conv_outsize(W, KW, SW, PW)
    want = (N * OH * OW, C * KH * KW) if to_matrix else (N, C, KH, KW, OH, OW)
    if tuple(col.shape) != want:
        raise OdlInvalidArgument("col2im: invalid col shape %s for input_shape %s" % (tuple(col.shape), (N, C, H, W)))
    img = _empty((N, C, H, W), _f64)
    lib().call("odl_hip_col2im_f64", _p(col), N, C, H, W, KH, KW, SH, SW, PH, PW, int(to_matrix), _p(img), _stream())
    return img


def conv2d_f64(x, w, b=None, stride=1, pad=0):
    """Mat::conv2d (conv2d.cpp:404-512) on float64 tensors."""
    _chk(x, "x", _f64), _chk(w, "W", _f64)
    if b is not None:
        _chk(b, "b", _f64)
    if x.dim() != 4 or w.dim() != 4 or x.shape[1] != w.shape[1]:
        raise OdlInvalidArgument("conv2d: x must be (N, C, H, W) and W (OC, C, KH, KW) with the same C")
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    (SH, SW), (PH, PW) = _pair(stride), _pair(pad)
    OH, OW = conv_outsize(H, KH, SH, PH), conv_outsize(W, KW, SW, PW)
    if OH <= 0 or OW <= 0:
        raise OdlInvalidArgument("conv2d: the window does not fit the padded image")
    y = _empty((N, OC, OH, OW), _f64)
    ws, nb = _ws(lib().query("odl_hip_conv2d_f64_workspace_bytes", N, C, H, W, OC, KH, KW, SH, SW, PH, PW))
    lib().call("odl_hip_conv2d_f64", _p(x), _p(w), _p(b), N, C, H, W, OC, KH, KW, SH, SW, PH, PW, _p(y), _p(ws), nb, _stream())
    return y


def conv2d_backward_f64(gy, x, w, has_bias=True, stride=1, pad=0):
    """Mat::conv2d_backward (conv2d.cpp:514-599) on float64 tensors -> (gx, gW, gb or None)."""
    _chk(gy, "gy", _f64), _chk(x, "x", _f64), _chk(w, "W", _f64)
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    (SH, SW), (PH, PW) = _pair(stride), _pair(pad)
    gx, gw = _empty(x.shape, _f64), _empty(w.shape, _f64)
    gb = _empty((OC,), _f64) if has_bias else None
    ws, nb = _ws(lib().query("odl_hip_conv2d_backward_f64_workspace_bytes", N, C, H, W, OC, KH, KW, SH, SW, PH, PW))
    lib().call("odl_hip_conv2d_backward_f64", _p(gy), _p(x), _p(w), N, C, H, W, OC, KH, KW, SH, SW, PH, PW, _p(gx), _p(gw),
               _p(gb), _p(ws), nb, _stream())
    return gx, gw, gb


# ------------------------------------------------------------------------------- reductions / broadcast
def _split_axis(shape, axis):
    outer = int(np.prod(shape[:axis])) if axis > 0 else 1
    inner = int(np.prod(shape[axis + 1:])) if axis + 1 < len(shape) else 1
    return outer, int(shape[axis]), inner


def sum(x, axis=-1, keepdim=False):  # noqa: A001 - the reference's name
    """Mat::sum (src/mat/origin/cpu/math/sum.cpp:15-90): axis -1 sums everything into shape {1}."""
    _chk(x, "x")
    if axis == -1:
        out = _empty([1] * x.dim() if keepdim else (1,))
        ws, nb = _ws(lib().query("odl_hip_sum_all_workspace_bytes", x.numel()))
        lib().call("odl_hip_sum_all", _p(x), x.numel(), _p(out), _p(ws), nb, _stream())
        return out
    if axis < 0 or axis >= x.dim():
        raise OdlInvalidArgument("Invalid axis %d for sum operation. Tensor has %d dimensions" % (axis, x.dim()))
    outer, ax, inner = _split_axis(x.shape, axis)
    oshape = [1 if i == axis else s for i, s in enumerate(x.shape)] if keepdim else \
        [s for i, s in enumerate(x.shape) if i != axis]
    out = _empty(oshape)
    ws, nb = _ws(lib().query("odl_hip_sum_axis_workspace_bytes", outer, ax, inner))
    lib().call("odl_hip_sum_axis", _p(x), outer, ax, inner, _p(out), _p(ws), nb, _stream())
    return out


def max(x, axis=-1):  # noqa: A001
    """Mat::max (src/mat/origin/cpu/math/max.cpp:20-121)."""
    _chk(x, "x")
    if axis == -1:
        out = _empty((1,))
        lib().call("odl_hip_max_all", _p(x), x.numel(), _p(out), _stream())
        return out
    if axis < 0 or axis >= x.dim():
        raise OdlInvalidArgument("Invalid axis %d for max operation. Tensor has %d dimensions" % (axis, x.dim()))
    outer, ax, inner = _split_axis(x.shape, axis)
    out = _empty([s for i, s in enumerate(x.shape) if i != axis])
    lib().call("odl_hip_max_axis", _p(x), outer, ax, inner, _p(out), _stream())
    return out


def sum_to(x, shape):
    """Mat::sum_to (src/mat/origin/cpu/math/sum_to.cpp:11-76), left-aligned."""
    _chk(x, "x")
    shape = tuple(int(s) for s in shape)
    ss, ts = _shape_arr(x.shape), _shape_arr(shape)
    out = _empty(shape)
    ws, nb = _ws(lib().query("odl_hip_sum_to_workspace_bytes", ss, x.dim(), ts, len(shape)))
    lib().call("odl_hip_sum_to", _p(x), ss, x.dim(), ts, len(shape), _p(out), _p(ws), nb, _stream())
    return out


def sum_nchw_channels(gy):
    _chk(gy, "gy")
    N, OC = gy.shape[0], gy.shape[1]
    P = int(np.prod(gy.shape[2:]))
    out = _empty((OC,))
    ws, nb = _ws(lib().query("odl_hip_sum_nchw_channels_workspace_bytes", N, OC, P))
    lib().call("odl_hip_sum_nchw_channels", _p(gy), N, OC, P, _p(out), _p(ws), nb, _stream())
    return out


def broadcast_to(x, shape):
    _chk(x, "x")
    shape = tuple(int(s) for s in shape)
    out = _empty(shape)
    lib().call("odl_hip_broadcast_to", _p(x), _shape_arr(x.shape), x.dim(), _shape_arr(shape), len(shape), _p(out),
               _stream())
    return out


# --------------------------------------------------------------------------------- softmax / CE
def softmax(x, axis=-1):
    _chk(x, "x")
    if axis < 0:
        axis += x.dim()
    if axis < 0 or axis >= x.dim():
        raise OdlInvalidArgument("Invalid axis for softmax. Tensor has %d dimensions" % x.dim())
    outer, ax, inner = _split_axis(x.shape, axis)
    y = _empty(x.shape)
    lib().call("odl_hip_softmax", _p(x), outer, ax, inner, _p(y), _stream())
    return y


def gather(x, idx):
    _chk(x, "input")
    idx, is64 = _labels(idx)
    if x.dim() != 2:
        raise OdlInvalidArgument("gather: input must be 2D (N, C)")
    if idx.dim() != 1:
        raise OdlInvalidArgument("gather: indices must be 1D (N,)")
    if x.shape[0] != idx.shape[0]:
        raise OdlInvalidArgument("gather: batch size mismatch")
    out = _empty((x.shape[0],))
    lib().call("odl_hip_gather", _p(x), _p(idx), is64, x.shape[0], x.shape[1], _p(out), _stream())
    return out


def one_hot(idx, num_classes):
    idx, is64 = _labels(idx)
    if idx.dim() != 1:
        raise OdlInvalidArgument("one_hot: indices must be 1D (N,)")
    if num_classes <= 0:
        raise OdlInvalidArgument("one_hot: num_classes must be positive, but got %d" % num_classes)
    out = _empty((idx.shape[0], num_classes))
    lib().call("odl_hip_one_hot", _p(idx), is64, idx.shape[0], num_classes, _p(out), _stream())
    return out


def _ce_check(x, t):
    _chk(x, "x")
    t, is64 = _labels(t)
    if x.dim() != 2:
        raise OdlInvalidArgument("SoftmaxCrossEntropy expects x to be 2D (N, C)")
    if t.dim() != 1:
        raise OdlInvalidArgument("SoftmaxCrossEntropy expects target to be 1D (N,)")
    if x.shape[0] != t.shape[0]:
        raise OdlInvalidArgument("SoftmaxCrossEntropy: batch size mismatch")
    return t, is64


def softmax_cross_entropy(x, t):
    """SoftmaxCrossEntropy::forward -> python float (the reference reads the sum back to the host too)."""
    t, is64 = _ce_check(x, t)
    N, C = x.shape
    ws, nb = _ws(lib().query("odl_hip_softmax_ce_loss_workspace_bytes", N))
    loss = ctypes.c_float(0)
    lib().call("odl_hip_softmax_ce_loss", _p(x), _p(t), is64, N, C, ctypes.byref(loss), _p(ws), nb, _stream())
    return loss.value


def softmax_cross_entropy_backward(x, t, gy=1.0):
    t, is64 = _ce_check(x, t)
    N, C = x.shape
    gx = _empty(x.shape)
    lib().call("odl_hip_softmax_ce_grad", _p(x), _p(t), is64, N, C, ctypes.c_float(gy), _p(gx), _stream())
    return gx


def softmax_cross_entropy_with_unit_grad(x, t):
    """Loss and the gradient for an upstream gradient of 1 in one launch (odl_hip_softmax_ce_loss_grad_device)
    -> (loss as a python float, bad-label flag, gx); raises where the library has no such kernel."""
    t, is64 = _ce_check(x, t)
    N, C = x.shape
    if lib().query("odl_hip_softmax_ce_loss_grad_ok", N, C) != 1:
        raise OdlInvalidArgument("softmax_cross_entropy: no one-launch loss and gradient for this batch")
    ws, nb = _ws(lib().query("odl_hip_softmax_ce_loss_workspace_bytes", N))
    out2 = torch.zeros(2, dtype=torch.float32, device="cuda")
    gx = _empty(x.shape)
    lib().call("odl_hip_softmax_ce_loss_grad_device", _p(x), _p(t), is64, N, C, _p(out2), None, _p(gx), _p(ws), nb, _stream())
    words = out2.cpu()
    return float(words[0]), int(words.view(torch.int32)[1]), gx


# ----------------------------------------------------------------------------------------- pooling
def max_pool2d(x, kernel_size, stride, pad, with_indices=True):
    _chk(x, "x")
    if x.dim() != 4:
        raise OdlInvalidArgument("max_pool2d: x must be 4D (N, C, H, W)")
    (KH, KW), (SH, SW), (PH, PW) = _pair(kernel_size), _pair(stride), _pair(pad)
    N, C, H, W = x.shape
    OH, OW = conv_outsize(H, KH, SH, PH), conv_outsize(W, KW, SW, PW)
    y = _empty((N, C, _builtins.max(OH, 0), _builtins.max(OW, 0)))
    idx = torch.empty(y.shape, dtype=torch.int64, device="cuda") if with_indices else None  # uint64 bit pattern
    lib().call("odl_hip_max_pool2d", _p(x), N, C, H, W, KH, KW, SH, SW, PH, PW, _p(y), _p(idx), _stream())
    return y, idx


def conv2d_relu_max_pool2d_ok(x_shape, w_shape, stride=1, pad=1, pool_kernel=2, pool_stride=2, pool_pad=0):
    """Whether Conv2d + ReLU + MaxPool2d of these shapes run as one pass (odl_hip_conv2d_relu_max_pool2d_ok)."""
    N, C, H, W = [int(v) for v in x_shape]
    OC, _, KH, KW = [int(v) for v in w_shape]
    (SH, SW), (PH, PW) = _pair(stride), _pair(pad)
    (PKH, PKW), (PSH, PSW), (PPH, PPW) = _pair(pool_kernel), _pair(pool_stride), _pair(pool_pad)
    return lib().query("odl_hip_conv2d_relu_max_pool2d_ok", N, C, H, W, OC, KH, KW, SH, SW, PH, PW, PKH, PKW, PSH, PSW, PPH,
                       PPW) == 1


def conv2d_relu_max_pool2d(x, w, b=None, stride=1, pad=1, pool_kernel=2, pool_stride=2, pool_pad=0, with_indices=True):
    """max_pool2d(relu(conv2d(x, w, b))) in one pass -> (pooled, indices); raises where there is no such kernel."""
    _chk(x, "x"), _chk(w, "W")
    if b is not None:
        _chk(b, "b")
    N, C, H, W = x.shape
    OC, _, KH, KW = w.shape
    (SH, SW), (PH, PW) = _pair(stride), _pair(pad)
    (PKH, PKW), (PSH, PSW), (PPH, PPW) = _pair(pool_kernel), _pair(pool_stride), _pair(pool_pad)
    y = _empty((N, OC, H // 2, W // 2))
    if with_indices == "bytes":
        idx = torch.empty(y.shape, dtype=torch.uint8, device="cuda")
        lib().call("odl_hip_conv2d_relu_max_pool2d_compact", _p(x), _p(w), _p(b), N, C, H, W, OC, KH, KW, SH, SW, PH, PW, PKH,
                   PKW, PSH, PSW, PPH, PPW, _p(y), _p(idx), _stream())
        return y, idx
    idx = torch.empty(y.shape, dtype=torch.int64, device="cuda") if with_indices else None  # uint64 bit pattern
    lib().call("odl_hip_conv2d_relu_max_pool2d", _p(x), _p(w), _p(b), N, C, H, W, OC, KH, KW, SH, SW, PH, PW, PKH, PKW, PSH, PSW,
               PPH, PPW, _p(y), _p(idx), _stream())
    return y, idx


def max_pool2d_compact(x, kernel_size, stride, pad):
    """max_pool2d with the window-local indices as bytes (odl_hip_max_pool2d_compact) -> (y, idx uint8)."""
    _chk(x, "x")
    (KH, KW), (SH, SW), (PH, PW) = _pair(kernel_size), _pair(stride), _pair(pad)
    N, C, H, W = x.shape
    OH, OW = conv_outsize(H, KH, SH, PH), conv_outsize(W, KW, SW, PW)
    y = _empty((N, C, _builtins.max(OH, 0), _builtins.max(OW, 0)))
    idx = torch.empty(y.shape, dtype=torch.uint8, device="cuda")
    lib().call("odl_hip_max_pool2d_compact", _p(x), N, C, H, W, KH, KW, SH, SW, PH, PW, _p(y), _p(idx), _stream())
    return y, idx


def max_pool2d_backward_relu(gy, idx, x, kernel_size, stride, pad):
    """MaxPool2d::backward then ReLU::backward, x the tensor that was pooled (odl_hip_max_pool2d_backward_relu)."""
    _chk(gy, "gy"), _chk(x, "x")
    (KH, KW), (SH, SW), (PH, PW) = _pair(kernel_size), _pair(stride), _pair(pad)
    N, C, H, W = x.shape
    gx = _empty((N, C, H, W))
    lib().call("odl_hip_max_pool2d_backward_relu", _p(gy), _p(idx), _p(x), N, C, H, W, KH, KW, SH, SW, PH, PW, _p(gx), _stream())
    return gx


def max_pool2d_backward_relu_pooled(gy, idx, y, input_shape, kernel_size, stride, pad):
    """The same from the pooled tensor y (odl_hip_max_pool2d_backward_relu_pooled)."""
    _chk(gy, "gy"), _chk(y, "y")
    (KH, KW), (SH, SW), (PH, PW) = _pair(kernel_size), _pair(stride), _pair(pad)
    N, C, H, W = [int(v) for v in input_shape]
    gx = _empty((N, C, H, W))
    name = "odl_hip_max_pool2d_backward_relu_pooled_compact" if idx.dtype == torch.uint8 else "odl_hip_max_pool2d_backward_relu_pooled"
    lib().call(name, _p(gy), _p(idx), _p(y), N, C, H, W, KH, KW, SH, SW, PH, PW, _p(gx), _stream())
    return gx


def max_pool2d_backward(gy, idx, input_shape, kernel_size, stride, pad):
    _chk(gy, "gy")
    if gy.dim() != 4:
        raise OdlInvalidArgument("max_pool2d_backward: gy must be 4D (N, C, OH, OW)")
    if idx is None or idx.numel() != gy.numel():
        raise OdlInvalidArgument("max_pool2d_backward: indices size mismatch")
    (KH, KW), (SH, SW), (PH, PW) = _pair(kernel_size), _pair(stride), _pair(pad)
    N, C, H, W = [int(s) for s in input_shape]
    gx = _empty((N, C, H, W))
    lib().call("odl_hip_max_pool2d_backward", _p(gy), _p(idx), N, C, H, W, KH, KW, SH, SW, PH, PW, _p(gx), _stream())
    return gx


# ----------------------------------------------------------------------------------------- metrics
def argmax_rows(y):
    _chk(y, "y")
    out = torch.empty((y.shape[0],), dtype=torch.int64, device="cuda")
    lib().call("odl_hip_argmax_rows", _p(y), y.shape[0], y.shape[1], _p(out), _stream())
    return out


def accuracy(y, t):
    _chk(y, "y"), _chk(t, "target", torch.int32)
    if y.dim() != 2 or t.dim() != 1 or y.shape[0] != t.shape[0]:
        raise OdlInvalidArgument("accuracy expects y (N, C) and target (N,)")
    ws, nb = _ws(lib().query("odl_hip_accuracy_workspace_bytes", y.shape[0]))
    acc = ctypes.c_float(0)
    lib().call("odl_hip_accuracy", _p(y), _p(t), y.shape[0], y.shape[1], ctypes.byref(acc), _p(ws), nb, _stream())
    return acc.value


# -------------------------------------------------------------------------------------- elementwise
_BIN = {"add": 0, "sub": 1, "mul": 2, "div": 3, "gt": 4, "eq": 5, "ne": 6, "lt": 7, "le": 8, "ge": 9,
        "sigmoid_backward": 10, "silu_backward": 11, "relu_backward": 12}
_UN = {"relu": 0, "exp": 1, "log": 2, "neg": 3, "square": 4, "sqrt": 5, "sigmoid": 6, "silu": 7}


def binary(op, a, b, out=None):
    _chk(a, "a"), _chk(b, "b")
    big = a if a.numel() >= b.numel() else b
    out = out if out is not None else _empty(big.shape)
    lib().call("odl_hip_binary", _BIN[op], _p(a), a.numel(), _p(b), b.numel(), _p(out), _stream())
    return out


def unary(op, a):
    _chk(a, "a")
    out = _empty(a.shape)
    lib().call("odl_hip_unary", _UN[op], _p(a), a.numel(), _p(out), _stream())
    return out


def pow_scalar(a, e):
    _chk(a, "a")
    out = _empty(a.shape)
    lib().call("odl_hip_pow_scalar", _p(a), a.numel(), ctypes.c_float(e), _p(out), _stream())
    return out


def upsample(x, scale):
    """Mat::upsample, nearest (src/mat/origin/cpu/nn/upsample.cpp:22-75): output is (H*scale_h, W*scale_w)."""
    _chk(x, "x")
    if x.dim() != 4:
        raise OdlInvalidArgument("Upsample: input must be 4D (N, C, H, W)")
    sh, sw = _pair(scale)
    N, C, H, W = x.shape
    y = _empty((N, C, H * sh, W * sw))
    lib().call("odl_hip_upsample_nearest", _p(x), N, C, H, W, H * sh, W * sw, sh, sw, _p(y), _stream())
    return y


def upsample_backward(gy, x_shape, scale):
    """Mat::upsample_backward (src/mat/origin/cpu/nn/upsample.cpp:80-135)."""
    _chk(gy, "gy")
    sh, sw = _pair(scale)
    N, C, H, W = (int(v) for v in x_shape)
    gx = _empty((N, C, H, W))
    lib().call("odl_hip_upsample_nearest_backward", _p(gy), N, C, H, W, gy.shape[2], gy.shape[3], sh, sw, _p(gx),
               _stream())
    return gx


def split(x, sizes, dim):
    """Mat::split (the backward of cat): pieces of the given sizes along dim."""
    _chk(x, "x")
    outer, ax, inner = _split_axis(x.shape, dim)
    if _builtins.sum(sizes) != ax:
        raise OdlRuntimeError("split: sizes sum to %d, but dimension %d has %d elements" % (_builtins.sum(sizes), dim, ax))
    out, off = [], 0
    for sz in sizes:
        shape = list(x.shape)
        shape[dim] = sz
        piece = _empty(shape)
        lib().call("odl_hip_slice_axis", _p(x), outer, ax, inner, off, sz, _p(piece), _stream())
        out.append(piece)
        off += sz
    return out


def cat(xs, dim=0):
    """Mat::cat (src/mat/origin/cpu/shape/cat.cpp:20-140)."""
    if len(xs) < 1:
        raise OdlRuntimeError("cat: requires at least 1 input")
    for x in xs:
        _chk(x, "input")
        if x.dim() != xs[0].dim():
            raise OdlRuntimeError("cat: all inputs must have same number of dimensions")
        for d in range(x.dim()):
            if d != dim and x.shape[d] != xs[0].shape[d]:
                raise OdlRuntimeError("cat: dimension %d mismatch: %d vs %d" % (d, x.shape[d], xs[0].shape[d]))
    shape = list(xs[0].shape)
    shape[dim] = _builtins.sum(int(x.shape[dim]) for x in xs)
    outer, _, inner = _split_axis(shape, dim)
    out = _empty(shape)
    ptrs = (ctypes.c_void_p * len(xs))(*[x.data_ptr() for x in xs])
    sizes = (ctypes.c_int64 * len(xs))(*[int(x.shape[dim]) for x in xs])
    lib().call("odl_hip_cat", ptrs, sizes, len(xs), outer, inner, _p(out), _stream())
    return out


def yolo_detect_forward(x, conv_w, conv_b, grid, anchor_grid, stride, num_anchors, num_classes):
    """Mat::yolo_detect_forward (src/mat/origin/cpu/custom/yolo_detect.cpp:28-166) -> [N, A*H*W, classes+5]."""
    for name, t in (("x", x), ("conv_weight", conv_w), ("grid", grid), ("anchor_grid", anchor_grid)):
        _chk(t, name)
    if x.dim() != 4:
        raise OdlInvalidArgument("yolo_detect_forward: input must be 4D (N, C, H, W)")
    N, C, H, W = x.shape
    aH = anchor_grid.shape[2] if anchor_grid.dim() >= 3 else H
    aW = anchor_grid.shape[3] if anchor_grid.dim() >= 4 else W
    out = _empty((N, H * W * num_anchors, num_classes + 5))
    ws, nb = _ws(lib().query("odl_hip_yolo_detect_workspace_bytes", N, C, H, W, num_anchors, num_classes))
    lib().call("odl_hip_yolo_detect_forward", _p(x), _p(conv_w), _p(conv_b), _p(grid), grid.numel(), _p(anchor_grid),
               anchor_grid.numel(), aH, aW, N, C, H, W, float(stride), num_anchors, num_classes, _p(out), _p(ws), nb,
               _stream())
    return out


# ------------------------------------------------------------------ runs of channels inside wider NCHW tensors
def _run(t, name):
    """A 4-D float32 device tensor that is dense, or a run of channels of one (`buf[:, c0:c1]`): -> its image stride."""
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == _f32 and t.dim() == 4):
        raise OdlInvalidArgument("%s must be a 4D float32 device tensor (or a run of channels of one)" % name)
    N, C, H, W = t.shape
    s = t.stride()
    if (s[1], s[2], s[3]) != (H * W, W, 1) or (N > 1 and s[0] < C * H * W):
        raise OdlInvalidArgument("%s must be NCHW with only the images spaced apart, got strides %s" % (name, tuple(s)))
    return int(s[0]) if N > 1 else C * H * W


def conv2d_fused_ok(x_shape, w_shape, stride=1, pad=0):
    N, C, H, W = (int(d) for d in x_shape)
    (SH, SW), (PH, PW) = _pair(stride), _pair(pad)
    return lib().query("odl_hip_conv2d_fused_ok", N, C, H, W, int(w_shape[0]), int(w_shape[2]), int(w_shape[3]), SH, SW, PH, PW) == 1


def conv2d_fused(x, w_shape, packed, b, y, stride=1, pad=0, activation=None, residual=None):
    """y = residual + act(conv(x, W) + b) where x, y and residual may each be a run of channels of a wider tensor
    (a torch view `buf[:, c0:c1]`); packed = conv2d_pack_weights(x.shape, W, ...). The nodes nn.Conv2d, nn.SiLU,
    pnnx.Expression add and the copy of torch.cat of the reference's graph runner (src/pnnx/pnnx_graph.cpp:286-528)."""
    xs, ys = _run(x, "x"), _run(y, "y")
    rs = _run(residual, "residual") if residual is not None else 0
    N, C, H, W = x.shape
    OC, _, KH, KW = (int(d) for d in w_shape)
    (SH, SW), (PH, PW) = _pair(stride), _pair(pad)
    OH, OW = conv_outsize(H, KH, SH, PH), conv_outsize(W, KW, SW, PW)
    if tuple(y.shape) != (N, OC, OH, OW) or (residual is not None and tuple(residual.shape) != tuple(y.shape)):
        raise OdlInvalidArgument("conv2d_fused: y (and residual) must be [%d, %d, %d, %d]" % (N, OC, OH, OW))
    act = -1 if activation is None else _UN[activation]
    lib().call("odl_hip_conv2d_fused", _p(x), xs, _p(packed), _p(b), N, C, H, W, OC, KH, KW, SH, SW, PH, PW, act,
               _p(residual), rs, _p(y), ys, _stream())
    return y


def conv2d_fused_group_ok(x_shapes, w_shapes):
    S = len(x_shapes)
    if not (1 <= S <= 4) or len(w_shapes) != S:
        return False
    if any(len(w) != 4 or int(w[2]) != 1 or int(w[3]) != 1 or int(w[1]) != int(x[1]) or int(x[0]) != int(x_shapes[0][0])
           for x, w in zip(x_shapes, w_shapes)):
        return False
    i64 = lambda vs: (ctypes.c_int64 * S)(*[int(v) for v in vs])
    return lib().query("odl_hip_conv2d_fused_group_ok", S, int(x_shapes[0][0]), i64(x[1] for x in x_shapes), i64(x[2] for x in x_shapes),
                       i64(x[3] for x in x_shapes), i64(w[0] for w in w_shapes)) == 1


def conv2d_fused_group(xs, w_shapes, packeds, bs, ys, activation=None):
    """One to four 1x1 convolutions (stride 1, no padding) of independent inputs as one launch: member i is
    conv2d_fused(xs[i], w_shapes[i], packeds[i], bs[i], ys[i], 1, 0, activation), bit for bit. The stage convolutions of
    the reference's YoloDetect node (src/pnnx/pnnx_graph.cpp:286-528)."""
    S = len(xs)
    if not (1 <= S <= 4) or len(w_shapes) != S or len(packeds) != S or len(bs) != S or len(ys) != S:
        raise OdlInvalidArgument("conv2d_fused_group: 1 to 4 members with a filter shape, a filter copy, a bias (or None) and an output each")
    xst, yst = [_run(x, "x") for x in xs], [_run(y, "y") for y in ys]
    N = int(xs[0].shape[0])
    for x, w, y in zip(xs, w_shapes, ys):
        if tuple(y.shape) != (N, int(w[0]), x.shape[2], x.shape[3]) or x.shape[0] != N or int(w[1]) != x.shape[1] or tuple(w[2:]) != (1, 1):
            raise OdlInvalidArgument("conv2d_fused_group: a member's x, filter shape and y do not belong together")
    act = -1 if activation is None else _UN[activation]
    ptr = lambda ts: (ctypes.c_void_p * S)(*[None if t is None else t.data_ptr() for t in ts])
    i64 = lambda vs: (ctypes.c_int64 * S)(*[int(v) for v in vs])
    lib().call("odl_hip_conv2d_fused_group", S, ptr(xs), i64(xst), ptr(packeds), ptr(bs), N, i64(x.shape[1] for x in xs),
               i64(x.shape[2] for x in xs), i64(x.shape[3] for x in xs), i64(w[0] for w in w_shapes), act, ptr(ys), i64(yst), _stream())
    return ys


def upsample_view(x, y, scale):
    sh, sw = _pair(scale)
    xs, ys = _run(x, "x"), _run(y, "y")
    N, C, H, W = x.shape
    lib().call("odl_hip_upsample_nearest_view", _p(x), xs, N, C, H, W, y.shape[2], y.shape[3], sh, sw, _p(y), ys, _stream())
    return y


def max_pool2d_chain(x, K, count, y):
    """y[:, (j-1)*C : j*C] = the K x K / stride 1 / padding K/2 max pool applied j times to x, j = 1..count."""
    xs, ys = _run(x, "x"), _run(y, "y")
    N, C, H, W = x.shape
    if tuple(y.shape) != (N, count * C, H, W):
        raise OdlInvalidArgument("max_pool2d_chain: y must hold %d stages of x's shape" % count)
    lib().call("odl_hip_max_pool2d_chain", _p(x), xs, N, C, H, W, K, count, _p(y), ys, _stream())
    return y


def copy_images(src, dst):
    ss, ds = _run(src, "src"), _run(dst, "dst")
    if tuple(src.shape) != tuple(dst.shape):
        raise OdlInvalidArgument("copy_images: shapes differ")
    N, C, H, W = src.shape
    lib().call("odl_hip_copy_images", _p(src), ss, _p(dst), ds, N, C * H * W, _stream())
    return dst


def yolo_decode(conv, grid, anchor_grid, stride, num_anchors, num_classes, out_rows):
    """The decoding half of yolo_detect_forward: conv[N, A*(classes+5), H, W] -> out_rows, the stage's rows
    `out[:, r0 : r0 + A*H*W, :]` of the tensor that concatenates the stages."""
    _chk(conv, "conv"), _chk(grid, "grid"), _chk(anchor_grid, "anchor_grid")
    N, _, H, W = conv.shape
    CI = num_classes + 5
    if tuple(out_rows.shape) != (N, num_anchors * H * W, CI) or out_rows.stride()[1:] != (CI, 1):
        raise OdlInvalidArgument("yolo_decode: out_rows must be [%d, %d, %d] rows of a dense tensor" % (N, num_anchors * H * W, CI))
    aH = anchor_grid.shape[2] if anchor_grid.dim() >= 3 else H
    aW = anchor_grid.shape[3] if anchor_grid.dim() >= 4 else W
    lib().call("odl_hip_yolo_decode", _p(conv), _p(grid), grid.numel(), _p(anchor_grid), anchor_grid.numel(), aH, aW, N, H, W,
               float(stride), num_anchors, num_classes, _p(out_rows), int(out_rows.stride()[0]) if N > 1 else 0, _stream())
    return out_rows


def yolo_decode_stages(convs, grids, anchor_grids, strides, num_anchors, num_classes, out):
    """yolo_decode for every stage of a head in one launch: stage s fills the rows of out[N, rows, classes+5] that follow
    those of stage s - 1, from row 0 (the concatenation the reference's YoloDetect node makes,
    src/pnnx/pnnx_graph.cpp:286-528)."""
    S = len(convs)
    if not (1 <= S <= 4) or len(grids) != S or len(anchor_grids) != S or len(strides) != S:
        raise OdlInvalidArgument("yolo_decode_stages: 1 to 4 stages with a grid, an anchor grid and a stride each")
    _chk(out, "out")
    CI = num_classes + 5
    N = out.shape[0]
    outs, row0, aHs, aWs = [], 0, [], []
    for c, g, a in zip(convs, grids, anchor_grids):
        _chk(c, "conv"), _chk(g, "grid"), _chk(a, "anchor_grid")
        if c.dim() != 4 or c.shape[0] != N or c.shape[1] != num_anchors * CI:
            raise OdlInvalidArgument("yolo_decode_stages: a stage's convolution must be [%d, %d, H, W]" % (N, num_anchors * CI))
        H, W = int(c.shape[2]), int(c.shape[3])
        aHs.append(int(a.shape[2]) if a.dim() >= 3 else H), aWs.append(int(a.shape[3]) if a.dim() >= 4 else W)
        outs.append(out.data_ptr() + row0 * CI * 4)
        row0 += num_anchors * H * W
    if out.dim() != 3 or out.shape[2] != CI or row0 > out.shape[1]:
        raise OdlInvalidArgument("yolo_decode_stages: out must be [%d, >= %d, %d]" % (N, row0, CI))
    ptr = lambda ts: (ctypes.c_void_p * S)(*[t.data_ptr() for t in ts])
    i64 = lambda vs: (ctypes.c_int64 * S)(*[int(v) for v in vs])
    lib().call("odl_hip_yolo_decode_stages", S, ptr(convs), ptr(grids), i64(g.numel() for g in grids), ptr(anchor_grids),
               i64(a.numel() for a in anchor_grids), i64(aHs), i64(aWs), N, i64(c.shape[2] for c in convs),
               i64(c.shape[3] for c in convs), (ctypes.c_float * S)(*[float(v) for v in strides]), num_anchors, num_classes,
               (ctypes.c_void_p * S)(*outs), int(out.shape[1]) * CI, _stream())
    return out


def yolo_detect_stages_ok(x_shapes, num_anchors, num_classes):
    S = len(x_shapes)
    if not (1 <= S <= 4) or any(len(x) != 4 or int(x[0]) != int(x_shapes[0][0]) for x in x_shapes):
        return False
    i64 = lambda vs: (ctypes.c_int64 * S)(*[int(v) for v in vs])
    return lib().query("odl_hip_yolo_detect_stages_ok", S, int(x_shapes[0][0]), i64(x[1] for x in x_shapes), i64(x[2] for x in x_shapes),
                       i64(x[3] for x in x_shapes), num_anchors, num_classes) == 1


def yolo_detect_stages_forward(xs, packeds, bs, grids, anchor_grids, strides, num_anchors, num_classes, out):
    """Mat::yolo_detect_forward (src/mat/origin/cpu/custom/yolo_detect.cpp:28-166) for every stage of a head in one
    launch, stage s written behind stage s - 1 into out[N, rows, classes+5]: conv2d_fused then yolo_decode, bit for bit."""
    S = len(xs)
    if not (1 <= S <= 4) or any(len(v) != S for v in (packeds, bs, grids, anchor_grids, strides)):
        raise OdlInvalidArgument("yolo_detect_stages_forward: 1 to 4 stages with a filter copy, a bias (or None), a grid, an anchor grid and a stride each")
    _chk(out, "out")
    CI = num_classes + 5
    N = int(out.shape[0])
    xst = [_run(x, "x") for x in xs]
    outs, row0, aHs, aWs = [], 0, [], []
    for x, a in zip(xs, anchor_grids):
        if x.shape[0] != N:
            raise OdlInvalidArgument("yolo_detect_stages_forward: a stage's batch differs from the output's")
        H, W = int(x.shape[2]), int(x.shape[3])
        aHs.append(int(a.shape[2]) if a.dim() >= 3 else H), aWs.append(int(a.shape[3]) if a.dim() >= 4 else W)
        outs.append(out.data_ptr() + row0 * CI * 4)
        row0 += num_anchors * H * W
    if out.dim() != 3 or out.shape[2] != CI or row0 > out.shape[1]:
        raise OdlInvalidArgument("yolo_detect_stages_forward: out must be [%d, >= %d, %d]" % (N, row0, CI))
    ptr = lambda ts: (ctypes.c_void_p * S)(*[None if t is None else t.data_ptr() for t in ts])
    i64 = lambda vs: (ctypes.c_int64 * S)(*[int(v) for v in vs])
    lib().call("odl_hip_yolo_detect_stages_forward", S, ptr(xs), i64(xst), ptr(packeds), ptr(bs), ptr(grids),
               i64(g.numel() for g in grids), ptr(anchor_grids), i64(a.numel() for a in anchor_grids), i64(aHs), i64(aWs), N,
               i64(x.shape[1] for x in xs), i64(x.shape[2] for x in xs), i64(x.shape[3] for x in xs),
               (ctypes.c_float * S)(*[float(v) for v in strides]), num_anchors, num_classes, (ctypes.c_void_p * S)(*outs),
               int(out.shape[1]) * CI, _stream())
    return out


def _bn_dims(x, who):
    if x.dim() not in (2, 4):
        raise OdlInvalidArgument("%s: x must have 2 or 4 dimensions, but got shape %s" % (who, tuple(x.shape)))
    return x.shape[0], x.shape[1], (x.shape[2] * x.shape[3] if x.dim() == 4 else 1)


def batch_norm_forward(x, gamma, beta, running_mean, running_var, training, eps=1e-5, want_x_norm=True):
    """Mat::batch_norm_forward (src/mat/origin/cpu/normalization/batch_norm.cpp:31-258) -> (y, mean, var, x_norm);
    want_x_norm=False is the y-only Mat::batch_norm (x_norm is None)."""
    for name, t in (("x", x), ("gamma", gamma), ("beta", beta), ("running_mean", running_mean),
                    ("running_var", running_var)):
        _chk(t, name)
    N, C, P = _bn_dims(x, "batch_norm")
    for name, t in (("gamma", gamma), ("beta", beta), ("running_mean", running_mean), ("running_var", running_var)):
        if tuple(t.shape) != (C,):
            raise OdlInvalidArgument("batch_norm: gamma, beta, running_mean, running_var must have shape (%d)" % C)
    y, mean, var = _empty(x.shape), _empty((C,)), _empty((C,))
    xn = _empty(x.shape) if want_x_norm else None
    ws, nb = _ws(lib().query("odl_hip_batch_norm_workspace_bytes", N, C, P) if training else 0)
    lib().call("odl_hip_batch_norm_forward", _p(x), _p(gamma), _p(beta), _p(running_mean), _p(running_var),
               1 if training else 0, float(eps), N, C, P, _p(y), _p(mean), _p(var), _p(xn), _p(ws), nb, _stream())
    return y, mean, var, xn


def batch_norm_backward(gy, gamma, saved_var, saved_x_norm, eps=1e-5):
    """Mat::batch_norm_backward (batch_norm.cpp:279-418) -> (gx, dgamma, dbeta)."""
    for name, t in (("gy", gy), ("gamma", gamma), ("saved_var", saved_var), ("saved_x_norm", saved_x_norm)):
        _chk(t, name)
    N, C, P = _bn_dims(gy, "batch_norm_backward")
    if saved_x_norm.shape != gy.shape or tuple(gamma.shape) != (C,) or tuple(saved_var.shape) != (C,):
        raise OdlInvalidArgument("batch_norm_backward: shape mismatch")
    gx, dg, db = _empty(gy.shape), _empty((C,)), _empty((C,))
    ws, nb = _ws(lib().query("odl_hip_batch_norm_workspace_bytes", N, C, P))
    lib().call("odl_hip_batch_norm_backward", _p(gy), _p(gamma), _p(saved_var), _p(saved_x_norm), float(eps), N, C, P,
               _p(gx), _p(dg), _p(db), _p(ws), nb, _stream())
    return gx, dg, db


def batch_norm_backward_from_x(gy, x, gamma, saved_mean, saved_var, eps=1e-5):
    """The same gradients from x and the saved statistics (x_norm formed again in the kernel) -> (gx, dgamma, dbeta)."""
    for name, t in (("gy", gy), ("x", x), ("gamma", gamma), ("saved_mean", saved_mean), ("saved_var", saved_var)):
        _chk(t, name)
    N, C, P = _bn_dims(gy, "batch_norm_backward")
    if x.shape != gy.shape or any(tuple(t.shape) != (C,) for t in (gamma, saved_mean, saved_var)):
        raise OdlInvalidArgument("batch_norm_backward: shape mismatch")
    gx, dg, db = _empty(gy.shape), _empty((C,)), _empty((C,))
    ws, nb = _ws(lib().query("odl_hip_batch_norm_workspace_bytes", N, C, P))
    lib().call("odl_hip_batch_norm_backward_from_x", _p(gy), _p(x), _p(gamma), _p(saved_mean), _p(saved_var), float(eps),
               N, C, P, _p(gx), _p(dg), _p(db), _p(ws), nb, _stream())
    return gx, dg, db


def batch_norm_relu_forward(x, gamma, beta, running_mean, running_var, training, eps=1e-5):
    """relu(batch_norm(x)) written once (the BatchNorm2d + ReLU pair of tests/example/mnist/conv_mnist.cpp)
    -> (y, mean, var)."""
    for name, t in (("x", x), ("gamma", gamma), ("beta", beta), ("running_mean", running_mean),
                    ("running_var", running_var)):
        _chk(t, name)
    N, C, P = _bn_dims(x, "batch_norm")
    for t in (gamma, beta, running_mean, running_var):
        if tuple(t.shape) != (C,):
            raise OdlInvalidArgument("batch_norm: gamma, beta, running_mean, running_var must have shape (%d)" % C)
    y, mean, var = _empty(x.shape), _empty((C,)), _empty((C,))
    ws, nb = _ws(lib().query("odl_hip_batch_norm_workspace_bytes", N, C, P) if training else 0)
    lib().call("odl_hip_batch_norm_relu_forward", _p(x), _p(gamma), _p(beta), _p(running_mean), _p(running_var),
               1 if training else 0, float(eps), N, C, P, _p(y), _p(mean), _p(var), _p(ws), nb, _stream())
    return y, mean, var


def batch_norm_relu_backward_from_x(gy, x, gamma, beta, saved_mean, saved_var, eps=1e-5):
    """Backward of the pair: gy is the gradient of the ReLU's output; the mask is formed again from x and the saved
    statistics -> (gx, dgamma, dbeta)."""
    for name, t in (("gy", gy), ("x", x), ("gamma", gamma), ("beta", beta), ("saved_mean", saved_mean),
                    ("saved_var", saved_var)):
        _chk(t, name)
    N, C, P = _bn_dims(gy, "batch_norm_backward")
    if x.shape != gy.shape or any(tuple(t.shape) != (C,) for t in (gamma, beta, saved_mean, saved_var)):
        raise OdlInvalidArgument("batch_norm_backward: shape mismatch")
    gx, dg, db = _empty(gy.shape), _empty((C,)), _empty((C,))
    ws, nb = _ws(lib().query("odl_hip_batch_norm_workspace_bytes", N, C, P))
    lib().call("odl_hip_batch_norm_relu_backward_from_x", _p(gy), _p(x), _p(gamma), _p(beta), _p(saved_mean),
               _p(saved_var), float(eps), N, C, P, _p(gx), _p(dg), _p(db), _p(ws), nb, _stream())
    return gx, dg, db


def axpby(a, x, b, y):
    """a*x + b*y with each product rounded first: the running-statistics update of the BatchNorm layers
    (src/nn/layers/batch_norm2d.cpp:77-80)."""
    _chk(x, "x"), _chk(y, "y")
    if x.shape != y.shape:
        raise OdlInvalidArgument("axpby: shape mismatch")
    out = _empty(x.shape)
    lib().call("odl_hip_axpby", float(a), _p(x), float(b), _p(y), x.numel(), _p(out), _stream())
    return out


def adam_step(p, g, m, v, t, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8):
    """One fused Adam step (src/optim/adam.cpp:52-113): returns the new parameter, updates m and v in place.
    The bias-correction scales are computed in float32 on the host exactly as the reference computes them."""
    for name, x in (("p", p), ("g", g), ("m", m), ("v", v)):
        _chk(x, name)
    f = np.float32
    b1p, b2p = f(np.power(f(beta1), f(t))), f(np.power(f(beta2), f(t)))
    s1, s2 = f(1.0) / (f(1.0) - b1p), f(1.0) / (f(1.0) - b2p)
    out = _empty(p.shape)
    lib().call("odl_hip_adam_step", _p(p), _p(g), _p(m), _p(v), p.numel(), float(f(beta1)), float(f(beta2)), float(s1),
               float(s2), float(f(eps)), float(f(lr)), _p(out), _stream())
    return out


def sgd_step(p, g, lr):
    """p - g*lr in one launch (src/optim/sgd.cpp:18-75 without momentum or weight decay)."""
    _chk(p, "p"), _chk(g, "g")
    out = _empty(p.shape)
    lib().call("odl_hip_sgd_step", _p(p), _p(g), p.numel(), float(np.float32(lr)), _p(out), _stream())
    return out


def _ptr_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() if t is not None else None for t in tensors])


def _size_array(tensors):
    return (ctypes.c_int64 * len(tensors))(*[t.numel() for t in tensors])


def adam_step_multi(ps, gs, ms, vs, ts, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, device_scales=None, weight_decay=0.0):
    """One launch over a list of parameters (Optimizer::step, src/optim/optimizer.cpp:19-53, walks them one by one):
    entry i gets what adam_step gives at step count ts[i]. Returns the new parameters; ms and vs are updated in place.
    device_scales: optional list whose non-None entries are device tensors of two floats used instead of ts[i].
    weight_decay != 0: gs[i] += weight_decay * ps[i] first, in place and in the same launch (the WeightDecay hook)."""
    for group in (ps, gs, ms, vs):
        for x in group:
            _chk(x, "adam_step_multi operand")
    f = np.float32
    s1 = [f(1.0) / (f(1.0) - f(np.power(f(beta1), f(t)))) for t in ts]
    s2 = [f(1.0) / (f(1.0) - f(np.power(f(beta2), f(t)))) for t in ts]
    outs = [_empty(p.shape) for p in ps]
    n = len(ps)
    if weight_decay != 0.0:
        lib().call("odl_hip_adam_step_multi_decay", n, _ptr_array(ps), _ptr_array(gs), _ptr_array(ms), _ptr_array(vs),
                   _size_array(ps), float(f(weight_decay)), float(f(beta1)), float(f(beta2)), (ctypes.c_float * n)(*s1),
                   (ctypes.c_float * n)(*s2), _ptr_array(device_scales) if device_scales is not None else None,
                   float(f(eps)), float(f(lr)), _ptr_array(outs), _stream())
        return outs
    lib().call("odl_hip_adam_step_multi", n, _ptr_array(ps), _ptr_array(gs), _ptr_array(ms), _ptr_array(vs),
               _size_array(ps), float(f(beta1)), float(f(beta2)), (ctypes.c_float * n)(*s1), (ctypes.c_float * n)(*s2),
               _ptr_array(device_scales) if device_scales is not None else None, float(f(eps)), float(f(lr)),
               _ptr_array(outs), _stream())
    return outs


def sgd_step_multi(ps, gs, lr, weight_decay=0.0):
    """p - g*lr for every pair of the lists in one launch (weight_decay != 0: g += weight_decay * p first, in place)."""
    for group in (ps, gs):
        for x in group:
            _chk(x, "sgd_step_multi operand")
    outs = [_empty(p.shape) for p in ps]
    if weight_decay != 0.0:
        lib().call("odl_hip_sgd_step_multi_decay", len(ps), _ptr_array(ps), _ptr_array(gs), _size_array(ps),
                   float(np.float32(weight_decay)), float(np.float32(lr)), _ptr_array(outs), _stream())
        return outs
    lib().call("odl_hip_sgd_step_multi", len(ps), _ptr_array(ps), _ptr_array(gs), _size_array(ps), float(np.float32(lr)),
               _ptr_array(outs), _stream())
    return outs


def axpy_multi(alpha, xs, ys):
    """ys[i] += alpha * xs[i] in place, one launch (the WeightDecay hook over all parameters)."""
    for group in (xs, ys):
        for x in group:
            _chk(x, "axpy_multi operand")
    for x, y in zip(xs, ys):
        if x.shape != y.shape:
            raise OdlInvalidArgument("axpy_multi: shape mismatch")
    lib().call("odl_hip_axpy_multi", len(xs), float(np.float32(alpha)), _ptr_array(xs), _ptr_array(ys), _size_array(xs),
               _stream())


def fill(shape, value):
    out = _empty(shape)
    lib().call("odl_hip_fill", _p(out), out.numel(), ctypes.c_float(value), _stream())
    return out
