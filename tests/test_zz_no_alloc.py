"""The entry point that allocates nothing: odl_hip_sum_axis_noalloc keeps its partial sums in an array that is part of
the library's device image instead of a caller's workspace. Same kernels, same plan, same order of additions as
odl_hip_sum_axis, so the two must agree bit for bit — on two calls in a row, the second smaller than the first (the
array keeps the first call's partials), and whatever ran before in the process."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _entry():
    from origindl_amd import _lib
    L = _lib.lib()
    return L


def _both(L, x, outer, axis, inner):
    from origindl_amd import capi
    ref = torch.empty(outer * inner, dtype=torch.float32, device="cuda")
    nb = L.query("odl_hip_sum_axis_workspace_bytes", outer, axis, inner)
    ws = torch.empty(max(nb, 1), dtype=torch.uint8, device="cuda")
    L.call("odl_hip_sum_axis", x.data_ptr(), outer, axis, inner, ref.data_ptr(), ws.data_ptr() if nb else None, nb,
           capi._stream())
    got = torch.full((outer * inner,), float("nan"), dtype=torch.float32, device="cuda")
    L.call("odl_hip_sum_axis_noalloc", x.data_ptr(), outer, axis, inner, got.data_ptr(), capi._stream())
    torch.cuda.synchronize()
    return got.cpu().numpy(), ref.cpu().numpy(), nb


def test_sum_axis_without_allocation_matches_the_workspace_entry_point():
    assert torch.cuda.is_available(), "this test needs the MI355X"
    L = _entry()
    limit = L.query("odl_hip_sum_axis_noalloc_max_bytes")
    assert limit == 8 << 20
    g = torch.Generator(device="cuda").manual_seed(11)
    # two calls in a row on column sums whose partials go through the scratch array: the bias gradient of the scaled
    # benchmark shape (the whole 8 MiB), then a smaller one ([4096, 1000] -> [1000], a part of the same array); after them
    # shapes that need no partial sums at all (one launch), a middle axis, one long row cut in pieces, an empty axis
    shapes = [(1, 16384, 4096), (1, 4096, 1000),
              (1, 512, 1000), (1, 512, 10), (3, 700, 36), (1, 300000, 1), (2, 3000, 512),
              (8, 300, 7), (5000, 3, 1), (2, 0, 5), (1, 40000, 64)]
    used_scratch = 0
    for outer, axis, inner in shapes:
        print("\n[case] sum_axis_noalloc", outer, axis, inner, flush=True)
        x = torch.randn((outer, max(axis, 1), inner), device="cuda", generator=g)[:, :axis, :].contiguous()
        got, ref, nb = _both(L, x, outer, axis, inner)
        used_scratch += nb > 0
        assert nb <= limit
        assert np.array_equal(got, ref), (outer, axis, inner)
        want = x.double().sum(dim=1).reshape(-1).cpu().numpy()
        bound = 1e-5 * np.sqrt(max(axis, 1)) * x.double().norm(dim=1).reshape(-1).cpu().numpy() + 1e-30
        assert (np.abs(got - want) <= bound).all(), (outer, axis, inner)
    assert used_scratch >= 4
    # larger than the array: refused with a message, nothing launched
    outer, axis, inner = 1, 16384, 5120  # 410 slices of 5120 columns: a few KB over the array
    assert L.query("odl_hip_sum_axis_workspace_bytes", outer, axis, inner) > limit
    x = torch.zeros((4,), device="cuda")
    rc = L.cdll.odl_hip_sum_axis_noalloc(ctypes.c_void_p(x.data_ptr()), outer, axis, inner, ctypes.c_void_p(x.data_ptr()), None)
    from origindl_amd import _lib
    assert rc == _lib.ODL_ERR_INVALID_ARG
    assert b"built-in scratch" in L.cdll.odl_hip_last_error()
    assert L.cdll.odl_hip_sum_axis_noalloc(None, -1, 2, 2, None, None) == _lib.ODL_ERR_INVALID_ARG
