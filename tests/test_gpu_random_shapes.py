"""Seeded random layer shapes against the oracle: ragged channel / column counts, strides, dilations, both
paddings, tiny and K-heavy layers, so that every tile-plan branch (column-tile widths, K splits, the ragged tail of
the tile order, partial wavefront-rows) and every pre-pass variant meets odd sizes."""
import numpy as np
import pytest

import gpu_util
import refimpl

pytestmark = pytest.mark.gpu


def _random_case(rng):
    kh, kw = (int(v) for v in rng.choice([1, 1, 2, 3, 3, 5], size=2))
    sh, sw = (int(v) for v in rng.choice([1, 1, 2, 3], size=2))
    dh, dw = (int(v) for v in rng.choice([1, 1, 1, 2], size=2))
    c = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 31, 32, 64, 100, 256]))
    co = int(rng.choice([1, 2, 3, 4, 7, 8, 15, 16, 17, 30, 32, 33, 48, 64, 65, 100]))
    n = int(rng.integers(1, 4))
    h = int(rng.integers((kh - 1) * dh + 1, 24))
    w = int(rng.integers((kw - 1) * dw + 1, 24))
    if c >= 100:   # keep the oracle quick
        h, w = min(h, 10), min(w, 10)
    padding = str(rng.choice(["SAME", "VALID"]))
    lo = float(rng.choice([-1.0, 0.0, -3.0]))
    mm = (lo, lo + float(rng.choice([1.0, 2.5])), -0.5, 0.25)
    return (n, h, w, c), (kh, kw, c, co), (sh, sw), (dh, dw), padding, mm


@pytest.mark.parametrize("seed", range(48))
def test_random_layer_vs_oracle(pkg, oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    xs, fs, strides, dil, padding, mm = _random_case(rng)
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, mm, seed=seed)
    table = pkg.synth.table_random(seed) if seed % 2 else pkg.synth.table_asymmetric()
    y, acc = gpu_util.run_op(pkg, table, x, f, mm, strides, padding, dil)
    rc, y_ref, acc_ref = oracle.conv2d_fast(table, x, f, *mm, strides=strides, padding=padding, dilations=dil)
    assert rc == 0
    assert acc.shape == acc_ref.shape, (xs, fs, strides, dil, padding)
    assert np.array_equal(acc, acc_ref), (xs, fs, strides, dil, padding)
    assert refimpl.linf_rel(y, y_ref) <= 1e-5, (xs, fs, strides, dil, padding)


@pytest.mark.parametrize("seed", range(12))
def test_random_layer_entry_point_vs_composition(pkg, oracle, seed):
    """The same for the layer entry point (off-grid inputs: the fused fake quantization has real work to do)."""
    import torch
    rng = np.random.default_rng(2000 + seed)
    xs, fs, strides, dil, padding, mm = _random_case(rng)
    x = rng.uniform(mm[0], mm[1], size=xs).astype(np.float32)
    w = (rng.standard_normal(fs) * 0.3).astype(np.float32)
    bias = rng.uniform(-1, 1, size=fs[3]).astype(np.float32)
    table = pkg.synth.table_noisy(seed)
    dev = gpu_util.dev()
    layer = pkg.FakeApproxConv2D(strides, table, padding, dilation_rate=dil, activation="relu" if seed % 2 else None)
    y = layer(torch.from_numpy(x).to(dev), torch.from_numpy(w).to(dev), torch.from_numpy(bias).to(dev)).cpu().numpy()
    r = (float(x.min()), float(x.max()), float(w.min()), float(w.max()))
    fq = pkg.fake_quant.fake_quant_with_min_max_vars
    rc, y_ref, _ = oracle.conv2d_fast(table, fq(x, r[0], r[1]), fq(w, r[2], r[3]), *r, strides=strides, padding=padding,
                                      dilations=dil)
    assert rc == 0
    y_ref = (y_ref + bias).astype(np.float32)
    if seed % 2:
        y_ref = np.maximum(y_ref, 0.0)
    assert refimpl.linf_rel(y, y_ref) <= 1e-5, (xs, fs, strides, dil, padding)


EXTREMES = [
    ((2, 7, 7, 512), (1, 1, 512, 4096), (1, 1), (1, 1), "SAME"),    # 256 column tiles
    ((1, 5, 5, 3600), (3, 3, 3600, 8), (1, 1), (1, 1), "VALID"),    # K = 32400, just below the int32 bound
    ((1, 300, 3, 4), (3, 3, 4, 16), (1, 1), (1, 1), "SAME"),        # tall and narrow
    ((1, 3, 1000, 4), (1, 7, 4, 16), (1, 2), (1, 1), "SAME"),       # flat and wide, strided along the row
    ((3, 64, 64, 1), (5, 5, 1, 1), (1, 1), (2, 2), "SAME"),         # one channel in, one column out, dilated
    ((1, 1, 1, 1), (1, 1, 1, 1), (1, 1), (1, 1), "VALID"),          # a single product
    ((70, 9, 9, 8), (3, 3, 8, 24), (2, 2), (1, 1), "VALID"),        # many small images
]


@pytest.mark.parametrize("case", EXTREMES, ids=[str(i) for i in range(len(EXTREMES))])
def test_extreme_shapes_vs_oracle(pkg, oracle, case):
    xs, fs, strides, dil, padding = case
    mm = (-1.0, 1.0, -0.5, 0.5)
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, mm, seed=7)
    table = pkg.synth.table_random(9)
    y, acc = gpu_util.run_op(pkg, table, x, f, mm, strides, padding, dil)
    rc, y_ref, acc_ref = oracle.conv2d_fast(table, x, f, *mm, strides=strides, padding=padding, dilations=dil,
                                            threads=8)
    assert rc == 0
    assert np.array_equal(acc, acc_ref), case
    assert refimpl.linf_rel(y, y_ref) <= 1e-5, case


WIDE_ROWS = [
    # rows of many channels: the patch sums hold only a column segment of every band in LDS (whole rows would leave
    # one workgroup per CU, or not fit at all); inputs off the quantization grid, so the order of the sums counts
    ((30, 20, 41, 256), (3, 3, 256, 8), (1, 1), (1, 1), "SAME"),     # odd width, padding on both sides
    ((48, 21, 40, 256), (3, 3, 256, 8), (2, 2), (1, 1), "SAME"),     # stride 2: padding after only
    ((40, 17, 50, 192), (3, 5, 192, 8), (1, 3), (1, 2), "SAME"),     # stride 3 and dilation 2 along the row
    ((6, 19, 37, 320), (5, 3, 320, 8), (2, 1), (2, 1), "VALID"),     # no padding, dilated and strided rows
    ((3, 12, 30, 512), (3, 3, 512, 16), (1, 1), (1, 1), "SAME"),     # three rows do not fit LDS: long chains
    ((2, 9, 26, 1024), (3, 3, 1024, 8), (1, 1), (1, 1), "SAME"),     # ... nor does one row twice
]


@pytest.mark.parametrize("case", WIDE_ROWS, ids=[str(i) for i in range(len(WIDE_ROWS))])
def test_wide_rows_of_many_channels_vs_oracle(pkg, oracle, case):
    xs, fs, strides, dil, padding = case
    mm = (-1.0, 1.0, -0.5, 0.5)
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, mm, seed=len(str(case)))
    x = (x + np.float32(0.0013)).astype(np.float32)
    table = pkg.synth.table_random(3)
    y, acc = gpu_util.run_op(pkg, table, x, f, mm, strides, padding, dil)
    rc, y_ref, acc_ref = oracle.conv2d_fast(table, x, f, *mm, strides=strides, padding=padding, dilations=dil,
                                            threads=8)
    assert rc == 0
    assert np.array_equal(acc, acc_ref), case
    assert np.array_equal(y, y_ref), case     # the same sums in the same order: no tolerance needed


@pytest.mark.parametrize("columns", [32, 64])
def test_wider_column_tiles_vs_oracle(pkg, oracle, columns):
    """The tile planner has so far always chosen 16-column tiles; the 32- and 64-column variants of the kernel
    (other accumulator shapes, rotated activation dwords, the untransposed store path for 64) are pinned here by
    forcing the width through axc_set_tile_columns."""
    pkg.ops.set_tile_columns(columns)
    try:
        _wider_tile_cases(pkg, oracle, columns)
    finally:
        pkg.ops.set_tile_columns(0)


def _wider_tile_cases(pkg, oracle, columns):
    mm = (-1.0, 1.0, -0.5, 0.5)
    cases = [((2, 24, 24, 16), (3, 3, 16, 64), (1, 1), (1, 1), "SAME"),
             ((1, 17, 19, 8), (1, 1, 8, 48), (2, 2), (1, 1), "SAME"),
             ((2, 15, 15, 12), (5, 5, 12, 100), (1, 1), (1, 1), "VALID"),
             ((4, 40, 40, 64), (3, 3, 64, 64), (1, 1), (1, 1), "SAME"),
             ((1, 30, 30, 4), (3, 3, 4, 70), (2, 2), (1, 1), "SAME"),
             ((3, 9, 9, 5), (3, 3, 5, 33), (1, 1), (2, 2), "SAME"),
             ((8, 56, 56, 64), (1, 1, 64, 256), (1, 1), (1, 1), "SAME")]
    for xs, fs, strides, dil, padding in cases:
        plan = pkg.ops.conv2d_tile_plan(xs, fs, [1, strides[0], strides[1], 1], padding)
        assert plan["columns_per_tile"] == columns
        x, f, _, _ = refimpl.grid_case(pkg, xs, fs, mm, seed=3)
        table = pkg.synth.table_random(9)
        y, acc = gpu_util.run_op(pkg, table, x, f, mm, strides, padding, dil)
        rc, y_ref, acc_ref = oracle.conv2d_fast(table, x, f, *mm, strides=strides, padding=padding, dilations=dil,
                                                threads=8)
        assert rc == 0
        assert np.array_equal(acc, acc_ref), (columns, xs, fs)
        assert refimpl.linf_rel(y, y_ref) <= 1e-5, (columns, xs, fs)


def _sweep_case(seed):
    """Case `seed` of the wider sweep: the random layer above, sometimes with larger images and batches (several
    tiles, K splits, partial tiles), every fifth case depthwise, every second input off the quantization grid."""
    rng = np.random.default_rng(50000 + seed)
    xs, fs, strides, dil, padding, mm = _random_case(rng)
    if seed % 3 == 0 and fs[2] <= 32:
        xs = (int(rng.integers(1, 6)), int(rng.integers(max(20, (fs[0] - 1) * dil[0] + 1), 70)),
              int(rng.integers(max(20, (fs[1] - 1) * dil[1] + 1), 70)), xs[3])
    dw = seed % 5 == 4
    if dw:
        fs = (fs[0], fs[1], fs[2], 1)
        if seed % 2:
            fs, dil, strides = (3, 3, fs[2], 1), (1, 1), (int(rng.choice([1, 2])),) * 2
        if xs[1] < (fs[0] - 1) * dil[0] + 1 or xs[2] < (fs[1] - 1) * dil[1] + 1:
            return None
    return xs, fs, strides, dil, padding, mm, dw


@pytest.mark.parametrize("block", range(5))
def test_random_sweep_slice_vs_oracle(pkg, oracle, block):
    """150 fixed-seed cases of the sweep (30 per test), dense and depthwise, whole outputs against the oracle."""
    for seed in range(block * 30, block * 30 + 30):
        case = _sweep_case(seed)
        if case is None:
            continue
        xs, fs, strides, dil, padding, mm, dw = case
        print("sweep case", seed, xs, fs, strides, dil, padding, "depthwise" if dw else "dense", flush=True)
        x, f, _, _ = refimpl.grid_case(pkg, xs, fs, mm, seed=seed)
        if seed % 2:
            x = (x + np.float32(0.0013)).astype(np.float32)
        table = pkg.synth.table_random(seed)
        y, acc = gpu_util.run_op(pkg, table, x, f, mm, strides, padding, dil, depthwise=dw)
        if dw:
            rc, y_ref, acc_ref = oracle.depthwise_conv2d(table, x, f, *mm, strides=strides, padding=padding,
                                                          dilations=dil)
        else:
            rc, y_ref, acc_ref = oracle.conv2d_fast(table, x, f, *mm, strides=strides, padding=padding,
                                                    dilations=dil, threads=16)
        assert rc == 0 and acc.shape == acc_ref.shape, (seed, case)
        assert np.array_equal(acc, acc_ref), (seed, case)
        assert refimpl.linf_rel(y, y_ref) <= 1e-5, (seed, case)
