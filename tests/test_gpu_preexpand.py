"""The dense kernel that reads pre-expanded rows (lutgemm_px_kernel.hip) against the oracle.

The planner only picks it for layers with many output pixels, so the small cases here force it through
axc_set_preexpand(1); every case also checks, from the library's own kernel timers, that this kernel is the one that
ran.  Shapes cover one and many fills, odd and even fill counts (the two ways a tile hands LDS buffer 0 to the next
tile), several tiles per workgroup, ragged row tiles, column counts that are not multiples of 16 or of 4, strides,
dilation, padding taps, K cut over tiles, the layer entry point and the codes entry point."""
import ctypes

import numpy as np
import pytest
import torch

import gpu_util
import refimpl

pytestmark = pytest.mark.gpu

MM = (-1.0, 1.0, -0.5, 0.5)

CASES = [
    # input, filter, strides, dilations, padding
    ((2, 9, 9, 8), (1, 1, 8, 16), (1, 1), (1, 1), "SAME"),        # one fill
    ((2, 9, 9, 8), (3, 3, 8, 16), (1, 1), (1, 1), "SAME"),        # nine fills (odd), padding taps
    ((1, 12, 11, 16), (3, 3, 16, 24), (1, 1), (1, 1), "SAME"),    # 18 fills (even), two column tiles
    ((3, 17, 13, 16), (3, 3, 16, 30), (2, 2), (1, 1), "VALID"),   # columns not a multiple of four: untransposed store
    ((2, 20, 20, 24), (5, 5, 24, 7), (1, 1), (1, 1), "SAME"),     # fewer than 16 columns
    ((2, 21, 19, 6), (3, 3, 6, 20), (1, 2), (2, 2), "SAME"),      # 6 channels in two quads, dilation, mixed strides
    ((1, 40, 40, 32), (1, 1, 32, 100), (1, 1), (1, 1), "SAME"),   # seven column tiles: two blocks of the tile order
    ((70, 9, 9, 8), (3, 3, 8, 24), (2, 2), (1, 1), "VALID"),      # many small images
    ((9, 60, 60, 8), (1, 1, 8, 160), (1, 1), (1, 1), "SAME"),     # 8 row tiles x 10 column tiles
]


def _ran_px(ops):
    prof = ops.profile_read()
    return "lutgemm_px" in prof and "lutgemm_expand" not in prof


@pytest.fixture()
def forced(pkg):
    from tf_approximate_amd import ops
    ops.set_preexpand(1)
    ops.profile_enable(True)
    ops.profile_reset()
    yield ops
    ops.profile_enable(False)
    ops.set_preexpand(0)


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_preexpanded_rows_vs_oracle(pkg, oracle, forced, case):
    xs, fs, strides, dil, padding = case
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=len(str(case)))
    table = pkg.synth.table_random(9) if xs[0] % 2 else pkg.synth.table_asymmetric()
    y, acc = gpu_util.run_op(pkg, table, x, f, MM, strides, padding, dil)
    assert _ran_px(forced), case
    rc, y_ref, acc_ref = oracle.conv2d_fast(table, x, f, *MM, strides=strides, padding=padding, dilations=dil, threads=8)
    assert rc == 0
    assert np.array_equal(acc, acc_ref), case
    assert refimpl.linf_rel(y, y_ref) <= 1e-5, case


SPLIT_CASES = [
    # few output pixels under a long K: the planner cuts K over tiles, each tile a whole number of pre-expanded fills
    ((2, 8, 8, 64), (3, 3, 64, 32), (1, 1), "SAME"),
    ((1, 14, 14, 256), (1, 1, 256, 64), (1, 1), "SAME"),
    ((4, 7, 7, 128), (3, 3, 128, 48), (1, 1), "VALID"),
    ((3, 9, 9, 40), (5, 5, 40, 20), (2, 2), "SAME"),          # 10 channel quads: a split starts inside a tap
]


@pytest.mark.parametrize("case", SPLIT_CASES, ids=[str(i) for i in range(len(SPLIT_CASES))])
def test_preexpanded_rows_with_k_split_vs_oracle(pkg, oracle, forced, case):
    xs, fs, strides, padding = case
    plan = forced.conv2d_tile_plan(xs, fs, (1, strides[0], strides[1], 1), padding)
    assert plan["k_splits"] > 1, plan
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=len(str(case)))
    table = pkg.synth.table_random(17)
    y, acc = gpu_util.run_op(pkg, table, x, f, MM, strides, padding)
    prof = forced.profile_read()
    assert _ran_px(forced) and "splitk_epilogue" in prof, (case, sorted(prof))
    rc, y_ref, acc_ref = oracle.conv2d_fast(table, x, f, *MM, strides=strides, padding=padding, threads=8)
    assert rc == 0
    assert np.array_equal(acc, acc_ref), case
    assert refimpl.linf_rel(y, y_ref) <= 1e-5, case


def test_many_tiles_per_workgroup_match_the_other_kernel(pkg, forced):
    """1x1 32 -> 192 on 8 x 112 x 112: 25 row tiles x 12 column tiles, more than one tile per workgroup, one fill each
    (every tile's fill is fetched by the tile before it).  Compared bit for bit with the kernel that expands inside
    every tile, which the full-size tests pin against the oracle."""
    xs, fs = (8, 112, 112, 32), (1, 1, 32, 192)
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=4)
    table = pkg.synth.table_random(3)
    y, acc = gpu_util.run_op(pkg, table, x, f, MM)
    assert _ran_px(forced)
    forced.set_preexpand(-1)
    forced.profile_reset()
    y0, acc0 = gpu_util.run_op(pkg, table, x, f, MM)
    assert not _ran_px(forced)
    assert np.array_equal(acc, acc0)
    assert np.array_equal(y.view(np.uint32), y0.view(np.uint32))


def test_layer_entry_point_on_preexpanded_rows(pkg, oracle, forced):
    """Per-batch min/max, fake quantization, bias and ReLU around the pre-expanded kernel."""
    rng = np.random.default_rng(77)
    xs, fs = (2, 18, 18, 16), (3, 3, 16, 40)
    x = rng.uniform(-2.0, 1.0, size=xs).astype(np.float32)
    w = (rng.standard_normal(fs) * 0.3).astype(np.float32)
    bias = rng.uniform(-1, 1, size=fs[3]).astype(np.float32)
    table = pkg.synth.table_noisy(5)
    dev = gpu_util.dev()
    layer = pkg.FakeApproxConv2D((1, 1), table, "SAME", activation="relu")
    y = layer(torch.from_numpy(x).to(dev), torch.from_numpy(w).to(dev), torch.from_numpy(bias).to(dev)).cpu().numpy()
    assert _ran_px(forced)
    r = (float(x.min()), float(x.max()), float(w.min()), float(w.max()))
    fq = pkg.fake_quant.fake_quant_with_min_max_vars
    rc, y_ref, _ = oracle.conv2d_fast(table, fq(x, r[0], r[1]), fq(w, r[2], r[3]), *r, strides=(1, 1), padding="SAME")
    assert rc == 0
    y_ref = np.maximum((y_ref + bias).astype(np.float32), 0.0)
    assert refimpl.linf_rel(y, y_ref) <= 1e-5


def test_codes_and_tf1_entry_points_on_preexpanded_rows(pkg, oracle, forced):
    """uint8 codes in, int32 sums out (axc_conv2d_codes_acc_i32), and the tf1 integer op with its own padding origin."""
    from tf_approximate_amd import ops
    rng = np.random.default_rng(8)
    table_np = pkg.synth.table_random(21)
    table = pkg.TruthTable(table_np)
    for xs, fs, strides, padding, zp in [((1, 13, 13, 32), (3, 3, 32, 64), (2, 2), "SAME", 0),
                                         ((3, 6, 6, 16), (1, 1, 16, 48), (1, 1), "VALID", 255),
                                         ((2, 11, 9, 16), (1, 1, 16, 20), (2, 3), "SAME", 9)]:
        qa = rng.integers(0, 256, xs).astype(np.uint8)
        qb = rng.integers(0, 256, fs).astype(np.uint8)
        forced.profile_reset()
        acc = ops.conv2d_codes_acc_i32(table, torch.from_numpy(qa).to(gpu_util.dev()),
                                       torch.from_numpy(qb).to(gpu_util.dev()), zp,
                                       (1, strides[0], strides[1], 1), padding).cpu().numpy()
        assert _ran_px(forced), (xs, fs)
        patches = refimpl.gather_patches(qa, zp, fs[0], fs[1], strides, padding, (1, 1))
        n, oh, ow = patches.shape[:3]
        want = oracle.lut_gemm_codes(table_np, patches.reshape(n * oh * ow, -1), qb.reshape(-1, fs[3]))
        assert np.array_equal(acc.reshape(n * oh * ow, fs[3]), want)
    xs, fs, stride, padding, mm = (2, 7, 7, 256), (3, 3, 256, 16), 1, "SAME", (-1.0, 1.0, -0.5, 0.5)
    x = rng.integers(0, 256, size=xs).astype(np.uint8)
    f = rng.integers(0, 256, size=fs).astype(np.uint8)
    forced.profile_reset()
    out, _, _ = ops.ax_conv2d(torch.from_numpy(x).to(gpu_util.dev()), torch.from_numpy(f).to(gpu_util.dev()), *mm,
                              [1, stride, stride, 1], padding, table)
    assert _ran_px(forced)
    off_in = ops.float_to_quantized_unclamped_quint8(0.0, mm[0], mm[1])
    off_f = ops.float_to_quantized_unclamped_quint8(0.0, mm[2], mm[3])
    assert np.array_equal(out.cpu().numpy(), oracle.axconv2d_tf1(table_np, x, f, off_in, off_f, stride, padding))


def test_workspace_without_room_for_the_rows_still_serves(pkg, forced):
    """The workspace query counts the pre-expanded rows; the allocation-free entry point has 32 MiB and runs a layer
    whose rows alone take 128 MiB without them - same bits."""
    from tf_approximate_amd import _lib, ops
    lib = _lib.load()
    xs, fs = (16, 28, 28, 256), (1, 1, 256, 1024)
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=21)
    dev = gpu_util.dev()
    xd, fd = torch.from_numpy(x).to(dev), torch.from_numpy(f).to(dev)
    table = ops.TruthTable(pkg.synth.table_random(1))
    desc = ops.make_desc(xs, fs, [1, 1, 1, 1], "SAME")
    nbytes = ctypes.c_size_t()
    assert lib.axc_conv2d_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)) == 0
    assert nbytes.value > 128 << 20
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
    shape = (xs[0], xs[1], xs[2], fs[3])
    want = torch.full(shape, float("nan"), dtype=torch.float32, device=dev)
    got = torch.full(shape, float("nan"), dtype=torch.float32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    assert lib.axc_conv2d_minmax(table.handle, ctypes.byref(desc), xd.data_ptr(), fd.data_ptr(), *MM, want.data_ptr(),
                                 ws.data_ptr(), ws.numel(), stream) == 0, lib.axc_last_error()
    torch.cuda.synchronize()
    assert _ran_px(forced)
    forced.profile_reset()
    assert lib.axc_conv2d_minmax_static(table.handle, ctypes.byref(desc), xd.data_ptr(), fd.data_ptr(), *MM,
                                        got.data_ptr(), stream) == 0, lib.axc_last_error()
    torch.cuda.synchronize()
    assert not _ran_px(forced)
    assert np.array_equal(want.cpu().numpy().view(np.uint32), got.cpu().numpy().view(np.uint32))


def test_planner_picks_preexpanded_rows_for_many_pixels_only(pkg):
    """Without forcing: the north-star layer runs out of pre-expanded rows, a 14 x 14 layer of the same filter does not."""
    from tf_approximate_amd import ops
    table = pkg.synth.table_random(2)
    dev = gpu_util.dev()
    ops.set_preexpand(0)
    ops.profile_enable(True)
    try:
        for xs, expect in (((64, 56, 56, 64), True), ((4, 14, 14, 64), False)):
            x = torch.zeros(xs, dtype=torch.float32, device=dev)
            f = torch.zeros((3, 3, 64, 64), dtype=torch.float32, device=dev)
            op = pkg.ApproxConv2DWithMinMaxVars([1, 1, 1, 1], 8, table, "SAME")
            ops.profile_reset()
            op(x, f, *MM)
            torch.cuda.synchronize()
            assert _ran_px(ops) == expect, xs
    finally:
        ops.profile_enable(False)


def test_rows_are_built_by_the_pre_pass_launches(pkg, oracle):
    """The pre-expanded rows depend on the filter and the table only, so they are built by further workgroups of a
    launch that is there anyway: the patch-sum launch (float inputs with a multiple of four channels: bands, flat
    pixel list, few pixels of many channels, workgroups of 512 and of 1024), else the filter pre-pass launch (the flat
    layout of a 3-channel input, whose patch-sum kernel carries no filter work, with and without the quad of padding
    that makes its quad count even; integer-code inputs).  The library's kernel timers then show no launch of
    px_expand_rows_kernel; every case is checked against the oracle."""
    from tf_approximate_amd import ops
    table = pkg.synth.table_noisy(21)
    ops.set_preexpand(1)
    ops.profile_enable(True)
    try:
        for xs, fs, strides, carrier in (((3, 20, 20, 16), (3, 3, 16, 24), (1, 1), "patch_sums"),
                                         ((2, 30, 30, 64), (1, 1, 64, 40), (1, 1), "patch_sums"),     # flat pixel list
                                         ((2, 14, 14, 512), (1, 1, 512, 16), (1, 1), "patch_sums"),   # few pixels, many channels
                                         ((4, 300, 300, 8), (3, 3, 8, 16), (1, 1), "patch_sums"),     # bands of 900 pixels:
                                                                                                        # workgroups of 1024
                                         ((2, 40, 40, 3), (7, 7, 3, 16), (2, 2), "filter_pack"),      # 6 quads per filter row
                                         ((2, 40, 40, 3), (3, 3, 3, 16), (1, 1), "filter_pack")):     # 3 quads and one of padding
            x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=sum(xs))
            op = pkg.ApproxConv2DWithMinMaxVars([1, strides[0], strides[1], 1], 8, table, "SAME")
            xd, fd = torch.from_numpy(x).to(gpu_util.dev()), torch.from_numpy(f).to(gpu_util.dev())
            ops.profile_reset()
            y = op(xd, fd, *MM).cpu().numpy()
            prof = ops.profile_read()
            assert "lutgemm_px" in prof and "lutgemm_expand" not in prof, (xs, prof)
            assert "px_expand_rows" not in prof and ("filter_pack" in prof) == (carrier == "filter_pack"), (xs, prof)
            rc, y_ref, _ = oracle.conv2d_fast(table, x, f, *MM, strides=strides, padding="SAME")
            assert rc == 0
            assert refimpl.linf_rel(y, y_ref) <= 1e-5
        # the codes entry point: no patch sums, the rows ride in the filter pre-pass launch
        xs, fs = (3, 20, 20, 16), (3, 3, 16, 24)
        rng = np.random.default_rng(4)
        qa = rng.integers(0, 256, xs).astype(np.uint8)
        qb = rng.integers(0, 256, fs).astype(np.uint8)
        ops.profile_reset()
        acc = ops.conv2d_codes_acc_i32(pkg.TruthTable(table), torch.from_numpy(qa).to(gpu_util.dev()),
                                       torch.from_numpy(qb).to(gpu_util.dev()), 3, (1, 1, 1, 1), "SAME").cpu().numpy()
        prof = ops.profile_read()
        assert "lutgemm_px" in prof and "filter_pack" in prof and "px_expand_rows" not in prof, prof
        patches = refimpl.gather_patches(qa, 3, 3, 3, (1, 1), "SAME", (1, 1))
        n, oh, ow = patches.shape[:3]
        want = oracle.lut_gemm_codes(table, patches.reshape(n * oh * ow, -1), qb.reshape(-1, fs[3]))
        assert np.array_equal(acc.reshape(n * oh * ow, fs[3]), want)
    finally:
        ops.profile_enable(False)
        ops.set_preexpand(0)
