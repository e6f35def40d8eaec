"""The entry point that allocates nothing (tpk_three_nn_static_f32), called through the C ABI and
compared bit for bit with tpk_three_nn_f32 on the same inputs: two calls in a row, the second on a
smaller problem (the library's fixed scratch array still holds the first call's contents)."""
import ctypes
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "torch-points-kernels_amd", "torch_points_kernels", "libtpk_hip.so")


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _three_nn_both_ways(lib, dev, b, n, m, seed, clustered=False):
    g = torch.Generator().manual_seed(seed)
    unknown = torch.rand(b, n, 3, generator=g).to(dev)
    known = torch.rand(b, m, 3, generator=g)
    if clustered:
        # uneven density: the grid in LDS gives such clouds up, and the search over curve-ordered cells, whose
        # ordered copies and boxes fill the scratch array, answers them
        centres = torch.rand(b, 4, 3, generator=g)
        known = centres[:, torch.randint(0, 4, (m,), generator=g)] + 0.002 * torch.randn(b, m, 3, generator=g)
    known = known.contiguous().to(dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # the existing entry point, with a workspace the caller allocates
    ws_bytes = lib.tpk_three_nn_workspace_bytes(b, n, m)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    want_d = torch.full((b, n, 3), -7.0, device=dev)
    want_i = torch.full((b, n, 3), -7, dtype=torch.int32, device=dev)
    st = lib.tpk_three_nn_f32(b, n, m, _ptr(unknown), _ptr(known), _ptr(want_d), _ptr(want_i),
                              _ptr(ws) if ws_bytes else None, ctypes.c_size_t(ws_bytes), stream)
    assert st == 0
    # the entry point without allocation: outputs are the caller's, everything else is the library's
    got_d = torch.full((b, n, 3), -9.0, device=dev)
    got_i = torch.full((b, n, 3), -9, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    st = lib.tpk_three_nn_static_f32(b, n, m, _ptr(unknown), _ptr(known), _ptr(got_d), _ptr(got_i), stream)
    assert st == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    np.testing.assert_array_equal(got_i.cpu().numpy(), want_i.cpu().numpy())
    np.testing.assert_array_equal(got_d.cpu().numpy(), want_d.cpu().numpy())
    return ws_bytes


def test_three_nn_without_allocation(dev):
    lib = ctypes.CDLL(LIB)
    lib.tpk_three_nn_workspace_bytes.restype = ctypes.c_size_t
    lib.tpk_three_nn_static_scratch_bytes.restype = ctypes.c_size_t
    capacity = lib.tpk_three_nn_static_scratch_bytes()
    assert capacity == 8 << 20
    # first a problem that fills most of the array, then a smaller one that reuses its front part
    used = _three_nn_both_ways(lib, dev, 16, 16384, 4096, seed=21)
    assert 0 < used <= capacity
    used = _three_nn_both_ways(lib, dev, 16, 16384, 4096, seed=24, clustered=True)
    assert 0 < used <= capacity
    used = _three_nn_both_ways(lib, dev, 3, 1500, 700, seed=22)
    assert 0 < used <= capacity
    # a shape that takes no workspace (all pairs): also served, also without allocation
    assert _three_nn_both_ways(lib, dev, 2, 100, 50, seed=23) == 0
    # beyond the array: refused with its own status before anything is launched
    b, n, m = 32, 16384, 16384
    assert lib.tpk_three_nn_workspace_bytes(b, n, m) > capacity
    out_d = torch.full((4,), -3.0, device=dev)
    st = lib.tpk_three_nn_static_f32(b, n, m, _ptr(out_d), _ptr(out_d), _ptr(out_d), _ptr(out_d), None)
    assert st == -4
    lib.tpk_status_string.restype = ctypes.c_char_p
    assert b"scratch" in lib.tpk_status_string(st)
    torch.cuda.synchronize()
    assert (out_d == -3.0).all()
