"""The allocation-free entry point axc_conv2d_minmax_static against axc_conv2d_minmax, both through the C ABI:
same bits, on two calls in a row, the second with a smaller input (the static workspace keeps what the first
call left in it)."""
import ctypes

import numpy as np
import pytest
import torch

import refimpl

pytestmark = pytest.mark.gpu

MM = (-1.0, 1.0, -0.5, 0.5)


def _both(pkg, lib, table, xs, fs, strides, padding, seed):
    from tf_approximate_amd import ops
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=seed)
    dev = torch.device("cuda:0")
    xd, fd = torch.from_numpy(x).to(dev), torch.from_numpy(f).to(dev)
    desc = ops.make_desc(xs, fs, [1, strides[0], strides[1], 1], padding)
    dims = ops.conv2d_geometry(desc)
    shape = (dims.batch, int(dims.out_rows), int(dims.out_cols), dims.out_depth)
    nbytes = ctypes.c_size_t()
    assert lib.axc_conv2d_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)) == 0
    ws = torch.empty(max(nbytes.value, 256), dtype=torch.uint8, device=dev)
    want = torch.full(shape, float("nan"), dtype=torch.float32, device=dev)
    got = torch.full(shape, float("nan"), dtype=torch.float32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    rc = lib.axc_conv2d_minmax(table.handle, ctypes.byref(desc), xd.data_ptr(), fd.data_ptr(), *MM, want.data_ptr(),
                               ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, lib.axc_last_error()
    rc = lib.axc_conv2d_minmax_static(table.handle, ctypes.byref(desc), xd.data_ptr(), fd.data_ptr(), *MM,
                                      got.data_ptr(), stream)
    assert rc == 0, lib.axc_last_error()
    torch.cuda.synchronize()
    return want.cpu().numpy(), got.cpu().numpy(), (x, f)


def test_static_workspace_entry_point_matches_on_two_calls(pkg, oracle):
    from tf_approximate_amd import _lib, ops
    lib = _lib.load()
    table_host = pkg.synth.table_random(5)
    table = ops.TruthTable(table_host)
    limit = ctypes.c_size_t()
    assert lib.axc_conv2d_static_workspace_limit(ctypes.byref(limit)) == 0 and limit.value == 32 << 20
    # first call: a K-split layer (int32 partial sums in the workspace too); second: smaller, other geometry
    cases = [((4, 14, 14, 256), (3, 3, 256, 64), (1, 1), "SAME", 11),
             ((2, 9, 11, 12), (3, 3, 12, 20), (2, 1), "VALID", 12)]
    for xs, fs, strides, padding, seed in cases:
        want, got, (x, f) = _both(pkg, lib, table, xs, fs, strides, padding, seed)
        assert not np.isnan(want).any() and not np.isnan(got).any()
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), "static-workspace call differs"
    # the smaller case once more against the oracle: the existing entry point's bar
    rc, y_ref, _ = oracle.conv2d(table_host, x, f, *MM, strides=cases[1][2], padding=cases[1][3])
    assert rc == 0 and refimpl.linf_rel(got, y_ref) <= 1e-5


def test_static_workspace_calls_allocate_nothing(pkg):
    """Free device memory as the runtime reports it is the same before and after calls of the static entry point
    (after one warm-up call, which may load the kernels' code), with per-kernel profiling off and on."""
    from tf_approximate_amd import _lib, ops
    lib = _lib.load()
    table = ops.TruthTable(pkg.synth.table_random(6))
    xs, fs = (4, 14, 14, 256), (3, 3, 256, 64)     # K split: the widest use of the workspace
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=21)
    dev = torch.device("cuda:0")
    xd, fd = torch.from_numpy(x).to(dev), torch.from_numpy(f).to(dev)
    desc = ops.make_desc(xs, fs, [1, 1, 1, 1], "SAME")
    out = torch.empty((4, 14, 14, 64), dtype=torch.float32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

    def call():
        rc = lib.axc_conv2d_minmax_static(table.handle, ctypes.byref(desc), xd.data_ptr(), fd.data_ptr(), *MM,
                                          out.data_ptr(), stream)
        assert rc == 0, lib.axc_last_error()

    call()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(dev)
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before, "the static entry point changed free device memory by %d bytes" % (
        free_before - free_after)


def test_static_workspace_refuses_layers_beyond_its_limit(pkg):
    from tf_approximate_amd import _lib, ops
    lib = _lib.load()
    table = ops.TruthTable(pkg.synth.table_exact())
    xs, fs = (64, 112, 112, 64), (1, 1, 64, 64)          # 51 MB of activation codes alone
    desc = ops.make_desc(xs, fs, [1, 1, 1, 1], "SAME")
    nbytes = ctypes.c_size_t()
    assert lib.axc_conv2d_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)) == 0
    assert nbytes.value > 32 << 20
    # refused before any pointer is touched
    rc = lib.axc_conv2d_minmax_static(table.handle, ctypes.byref(desc), None, None, *MM, None, None)
    assert rc == _lib.INVALID_ARGUMENT
    assert b"static workspace" in lib.axc_last_error()
