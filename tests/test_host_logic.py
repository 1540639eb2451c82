"""CPU-side checks of the product's host code: the C-ABI library loads and exports every symbol the
header declares, and its geometry / quantization-parameter / argument-checking logic agrees with the
oracle and with the reference's error behaviour.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib(pkg):
    from tf_approximate_amd import _lib
    return _lib.load()


@pytest.fixture(scope="module")
def ops(pkg):
    from tf_approximate_amd import ops
    return ops


def test_library_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "axconv.h")).read()
    declared = set(re.findall(r"\b(axc_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 20
    for name in sorted(declared):
        assert hasattr(lib, name), name
    from tf_approximate_amd import _lib
    assert declared == {n for n, _, _ in _lib.SYMBOLS}


def test_status_strings(lib):
    assert lib.axc_status_string(0) == b"OK"
    assert lib.axc_status_string(1) == b"INVALID_ARGUMENT"
    assert lib.axc_status_string(2) == b"UNIMPLEMENTED"
    assert lib.axc_status_string(3) == b"RUNTIME_ERROR"


@pytest.mark.parametrize("mm", [(-1.0, 1.0, -0.3, 0.3), (0.0, 1.0, -0.5, 0.5), (0.0, 6.0, -0.017, 0.093),
                                (-2.5, 0.0, 0.0, 0.0), (0.0, 0.0, -1.0, 2.0)])
def test_quant_props_bit_equal_to_oracle(ops, oracle, mm):
    a = ops.quant_props(*mm)
    b = oracle.quant_props(*mm)
    pairs = [(a.input_scale, b.in_scale), (a.input_inv_scale, b.in_inv_scale), (a.input_offset, b.in_offset),
             (a.filter_scale, b.f_scale), (a.filter_inv_scale, b.f_inv_scale), (a.filter_offset, b.f_offset),
             (a.s1xs2, b.s1xs2), (a.m1, b.m1), (a.m2, b.m2), (a.m1xm2, b.m1xm2)]
    for x, y in pairs:
        assert np.float32(x).tobytes() == np.float32(y).tobytes()
    zc = oracle.quantize(np.zeros(1, np.float32), b.in_offset, b.in_inv_scale)[0]
    assert a.input_zero_code == zc


def test_geometry_matches_oracle(ops, oracle):
    rng = np.random.default_rng(0)
    for _ in range(300):
        h, w = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        kh, kw = int(rng.integers(1, 9)), int(rng.integers(1, 9))
        s = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        d = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        padding = "SAME" if rng.integers(0, 2) else "VALID"
        rc, g = oracle.geometry((2, h, w, 3), (kh, kw, 3, 5), s, padding, d)
        desc = ops.make_desc((2, h, w, 3), (kh, kw, 3, 5), (1, s[0], s[1], 1), padding, (), "NHWC", (1, d[0], d[1], 1))
        if rc != 0:
            with pytest.raises(ops.InvalidArgumentError):
                ops.conv2d_geometry(desc)
            continue
        dims = ops.conv2d_geometry(desc)
        assert (dims.out_rows, dims.out_cols) == (g.out_rows, g.out_cols)
        assert (dims.pad_rows_before, dims.pad_cols_before) == (g.pad_rows_before, g.pad_cols_before)
        assert (dims.pad_rows_after, dims.pad_cols_after) == (g.pad_rows_after, g.pad_cols_after)


def test_nchw_strides_are_read_in_format_order(ops):
    desc = ops.make_desc((2, 3, 10, 12), (3, 3, 3, 5), (1, 1, 2, 2), "SAME", (), "NCHW", (1, 1, 1, 1))
    dims = ops.conv2d_geometry(desc)
    assert (dims.batch, dims.in_depth, dims.input_rows, dims.input_cols) == (2, 3, 10, 12)
    assert (dims.out_rows, dims.out_cols) == (5, 6)


def _ws(lib, desc, depthwise=False):
    n = ctypes.c_size_t()
    fn = lib.axc_depthwise_conv2d_workspace_bytes if depthwise else lib.axc_conv2d_workspace_bytes
    return fn(ctypes.byref(desc), ctypes.byref(n)), n.value


def test_attr_errors_mirror_the_reference(ops, lib):
    """Messages of InitApproxConv2DParameters / the launchers (tf2/src/approx_nn_conv_ops.cpp:120,162,224,231,287-303)."""
    ok = dict(input_shape=(1, 8, 8, 4), filter_shape=(3, 3, 4, 8), strides=(1, 1, 1, 1), padding="SAME")

    def geom(**kw):
        a = dict(ok)
        a.update(kw)
        return ops.conv2d_geometry(ops.make_desc(**a))

    with pytest.raises(ops.InvalidArgumentError, match="strides in the batch and depth"):
        geom(strides=(2, 1, 1, 1))
    with pytest.raises(ops.InvalidArgumentError, match="strides in the batch and depth"):
        geom(strides=(1, 1, 1, 2))
    with pytest.raises(ops.InvalidArgumentError, match="strides should be larger than 0"):
        geom(strides=(1, 0, 1, 1))
    with pytest.raises(ops.InvalidArgumentError, match="dilations in the batch and depth"):
        geom(dilations=(1, 1, 1, 2))
    with pytest.raises(ops.InvalidArgumentError, match="Dilated rates should be larger than 0"):
        geom(dilations=(1, 0, 1, 1))
    with pytest.raises(ops.InvalidArgumentError, match="4 dimensions"):
        geom(strides=(1, 1))
    with pytest.raises(ops.InvalidArgumentError, match="must be 4-dimensional"):
        geom(input_shape=(8, 8, 4))
    with pytest.raises(ops.InvalidArgumentError, match="evenly divisible"):
        geom(filter_shape=(3, 3, 3, 8))
    with pytest.raises(ops.InvalidArgumentError, match="Invalid data format"):
        geom(data_format="NHCW")

    def ws(**kw):
        a = dict(ok)
        a.update(kw)
        rc, _ = _ws(lib, ops.make_desc(**a))
        return rc, lib.axc_last_error().decode()

    rc, msg = ws(padding="EXPLICIT", explicit_paddings=(0, 0, 1, 1, 1, 1, 0, 0))
    assert rc == 2 and msg == "Explicit padding is not implemented."
    rc, msg = ws(filter_shape=(3, 3, 2, 8))
    assert rc == 2 and "grouped convolutions" in msg
    rc, msg = ws(input_shape=(1, 4, 8, 8), data_format="NCHW")
    assert rc == 2 and "only supports NHWC" in msg
    rc, msg = ws(num_bits=4)
    assert rc == 1 and "num_bits" in msg
    rc, msg = ws(input_shape=(1, 200, 200, 64), filter_shape=(30, 30, 64, 8), padding="VALID")
    assert rc == 1 and "patch length" in msg            # int32 accumulator bound, K >= 32768
    rc, msg = ws(input_shape=(1, 2100, 2100, 1), filter_shape=(2049, 2049, 1, 1), padding="VALID")
    assert rc == 1 and msg == "ApproxConv2DOp: Patch too large for buffer"


def test_tile_plans_fit_the_kernels(ops, lib):
    """What the planner hands the LUT-GEMM kernels, over many layers and all pinned modes (the query needs no GPU:
    without one it plans for 256 CUs).  A tile holds at most 8 wavefronts x 2 * 64 / columns pixel slots of 64 pixels,
    the row tiles cover the pixels without an empty one, every K split has fills, and pre-expanded rows only come with
    16-column tiles, channel quads in pairs and splits of whole pairs of fills; plan code 2 (the kernel without barriers
    between fills) only with tiles of 16 to 63 wavefront-rows."""
    shapes = []
    for n, hw in [(1, 1), (1, 7), (2, 8), (4, 14), (64, 14), (64, 28), (16, 56), (64, 56), (128, 32), (128, 8), (3, 33)]:
        for c, co in [(3, 16), (8, 16), (16, 16), (64, 64), (40, 20), (256, 1024), (512, 128), (128, 130), (2048, 512)]:
            for k in (1, 3):
                if n * hw * hw * max(c, co) <= 64 * 56 * 56 * 1024 and k * k * c < 32768:
                    shapes.append(((n, hw, hw, c), (k, k, c, co)))
    seen_px = seen_free = seen_split = seen_px_split = 0
    try:
        for columns, mode in [(0, 0), (0, 1), (0, -1), (16, 1), (32, 0), (64, 0)]:
            assert lib.axc_set_tile_columns(columns) == 0 and lib.axc_set_preexpand(mode) == 0
            for xs, fs in shapes:
                pl = ops.conv2d_tile_plan(xs, fs)
                nt, rows, ks = pl["columns_per_tile"], pl["rows_per_tile"], pl["k_splits"]
                m = xs[0] * xs[1] * xs[2]
                what = (columns, mode, xs, fs, pl)
                assert nt in (16, 32, 64) and (columns == 0 or nt == columns), what
                assert rows % 64 == 0 and 0 < rows // 64 <= 8 * 2 * (64 // nt), what
                assert (pl["row_tiles"] - 1) * rows < m <= pl["row_tiles"] * rows, what
                assert pl["column_tiles"] == -(-fs[3] // nt), what
                tiles = pl["row_tiles"] * pl["column_tiles"] * ks
                assert 1 <= pl["workgroups"] <= tiles, what
                fps = pl["fills_per_split"]
                if xs[3] % 4 == 0:   # (other channel counts may use the flat layout, which counts quads per filter row)
                    fills = fs[0] * fs[1] * (xs[3] // 4) * (nt // 16)
                    assert 1 <= ks <= 16 and (ks - 1) * fps < fills <= ks * fps, what
                if pl["preexpanded_rows"]:
                    assert mode >= 0 and nt == 16 and fps % 2 == 0 and (xs[3] % 4 or (xs[3] // 4) % 2 == 0), what
                    assert pl["column_tiles"] * (fps * ks // 2) * 65536 <= (2 << 30) + ks * 65536, what
                elif mode == 1 and nt == 16 and xs[3] % 8 == 0:
                    assert pl["column_tiles"] * fs[0] * fs[1] * (xs[3] // 8) * 65536 > 2 << 30, what
                if pl["preexpanded_rows"] == 2:
                    # the kernel without barriers keeps its counters in the pixel slot a 64th wavefront-row would
                    # use, and is only picked for tiles of two wavefront-rows per wavefront and 16 fills or more
                    assert 16 <= rows // 64 <= 63 and fps // 2 >= (16 if fs[0] * fs[1] > 1 else 32), what
                assert pl["preexpanded_rows"] in (0, 1, 2), what
                seen_px += bool(pl["preexpanded_rows"])
                seen_free += pl["preexpanded_rows"] == 2
                seen_split += ks > 1
                seen_px_split += bool(pl["preexpanded_rows"]) and ks > 1
    finally:
        assert lib.axc_set_tile_columns(0) == 0 and lib.axc_set_preexpand(0) == 0
    assert seen_px > 50 and seen_split > 50 and seen_px_split > 5 and seen_free > 5


def test_workspace_sizes(ops, lib):
    desc = ops.make_desc((64, 56, 56, 64), (3, 3, 64, 64), (1, 1, 1, 1), "SAME")
    rc, n = _ws(lib, desc)
    assert rc == 0
    xq = 64 * 56 * 56 * 64            # one byte per activation
    psum = 64 * 56 * 56 * 4
    rows = 4 * (9 * 16 // 2) * 65536  # pre-expanded rows: 4 column tiles x 72 fills (pairs of channel quads) x 64 KiB
    assert xq + psum + rows < n < xq + psum + rows + (1 << 20)
    assert lib.axc_set_preexpand(-1) == 0
    rc, n = _ws(lib, desc)
    assert lib.axc_set_preexpand(0) == 0
    assert rc == 0 and xq + psum < n < xq + psum + (1 << 20)
    assert lib.axc_set_preexpand(2) == 1
    rc, n0 = _ws(lib, ops.make_desc((0, 56, 56, 64), (3, 3, 64, 64), (1, 1, 1, 1), "SAME"))
    assert rc == 0 and n0 == 0        # empty output: nothing to do (approx_nn_conv_ops.cpp:449)
    rc, nd = _ws(lib, ops.make_desc((2, 8, 8, 6), (3, 3, 6, 1), (1, 1, 1, 1), "SAME"), depthwise=True)
    assert rc == 0 and nd >= 9 * 6 + 6 * 4
    rc, _ = _ws(lib, ops.make_desc((2, 8, 8, 6), (3, 3, 6, 2), (1, 1, 1, 1), "SAME"), depthwise=True)
    assert rc == 1


def test_table_file_errors_need_no_gpu(lib, tmp_path):
    """Short read / missing file -> InvalidArgument with the reference's text (approx_ops_types.h:213)."""
    p = tmp_path / "short.bin"
    p.write_bytes(b"\x01" * 4096)
    h = ctypes.c_void_p()
    assert lib.axc_table_create_from_file(str(p).encode(), 8, ctypes.byref(h)) == 1
    assert lib.axc_last_error() == b"ApproxTF: Couldn't read the lookup table!"
    assert lib.axc_table_create_from_file(str(tmp_path / "none.bin").encode(), 8, ctypes.byref(h)) == 1
    assert lib.axc_table_create_from_file(b"", 7, ctypes.byref(h)) == 1
    assert b"num_bits" in lib.axc_last_error()


def test_synthetic_tables(pkg):
    s = pkg.synth
    assert s.table_exact()[3 * 256 + 5] == 15
    for t in (s.table_noisy(7), s.table_truncated(2), s.table_truncated(4), s.table_uniform_error(11),
              s.table_random(13), s.table_asymmetric()):
        assert t.dtype == np.uint16 and t.shape == (65536,)
    assert np.array_equal(s.table_noisy(7), s.table_noisy(7))
    t4 = s.table_truncated(4).reshape(256, 256).astype(np.int64)
    ab = np.arange(256)[:, None] * np.arange(256)[None, :]
    assert np.array_equal(t4, ab - ab % 16)
    assert s.table_asymmetric().reshape(256, 256)[0].min() > 0


def test_missing_library_fails_loudly(pkg, monkeypatch):
    from tf_approximate_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libaxconv_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()


def test_table_file_tool_round_trip_and_reference_format(pkg, golden_dir, tmp_path):
    """tables.py writes the reference's file format: its exact table is byte-identical to the reference's
    mul8u_1JFF.bin (the exact multiplier), and a written table reads back unchanged."""
    import subprocess
    import sys
    from tf_approximate_amd import tables
    out = tmp_path / "exact.bin"
    tool = os.path.join(os.path.dirname(golden_dir), "..", "tf-approximate_amd", "tables.py")
    r = subprocess.run([sys.executable, tool, "exact", str(out)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    with open(out, "rb") as a, open(os.path.join(golden_dir, "tables", "mul8u_1JFF.bin"), "rb") as b:
        assert a.read() == b.read()
    t = pkg.synth.table_noisy(3)
    tables.write_table(tmp_path / "n.bin", t)
    assert np.array_equal(tables.read_table(tmp_path / "n.bin"), np.asarray(t).reshape(-1))
    stats = tables.error_stats(tables.read_table(out))
    assert stats["wrong_entries"] == 0 and stats["symmetric"]
    with pytest.raises(ValueError):
        tables.write_table(tmp_path / "bad.bin", np.zeros(10))


def test_table_from_a_c_model(pkg, golden_dir, tmp_path):
    """tables.py cmodel: a multiplier written in C is tabulated in the reference's order (input code outer).  An exact
    model reproduces the reference's exact table byte for byte; an asymmetric model (drops the low bits of the
    FILTER operand only) pins which argument is which."""
    import subprocess
    import sys
    from tf_approximate_amd import tables
    src = tmp_path / "models.c"
    src.write_text("#include <stdint.h>\n"
                   "uint64_t mul_exact(uint64_t a, uint64_t b) { return a * b; }\n"
                   "uint16_t mul_drop(uint8_t a, uint8_t b) { return (uint16_t)(a * (b & 0xf0)); }\n")
    exact = tables.table_from_c_model(str(src), "mul_exact")
    assert exact.astype("<u2").tobytes() == open(os.path.join(golden_dir, "tables", "mul8u_1JFF.bin"), "rb").read()
    drop = tables.table_from_c_model(str(src), "mul_drop", proto="u8").reshape(256, 256)
    a = np.arange(256)[:, None]
    b = np.arange(256)[None, :]
    assert np.array_equal(drop, a * (b & 0xf0))
    tool = os.path.join(os.path.dirname(golden_dir), "..", "tf-approximate_amd", "tables.py")
    out = tmp_path / "drop.bin"
    r = subprocess.run([sys.executable, tool, "cmodel", str(src), "mul_drop", str(out), "u8"], stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    assert np.array_equal(tables.read_table(out).reshape(256, 256), drop)
    with pytest.raises(RuntimeError, match="compiling"):
        tables.table_from_c_model(str(src), "no_such_function")
    with pytest.raises(ValueError):
        tables.table_from_c_model(str(src), "mul exact")


def test_table_tuning_matches_argmin_with_the_tie_rule(ops, oracle, pkg):
    """axc_table_tune_weights against an independent numpy arg-min (first smallest column, own column wins ties)
    and against the oracle's restatement of the reference loop."""
    i = np.arange(256, dtype=np.int64)[:, None]
    for table in (pkg.synth.table_noisy(7), pkg.synth.table_truncated(4), pkg.synth.table_random(3),
                  pkg.synth.table_exact()):
        t = np.asarray(table, np.uint16).reshape(256, 256).astype(np.int64)
        want = np.empty((256, 256), np.uint16)
        for w in range(256):
            err = np.abs(i * w - t).sum(axis=0)             # per candidate column
            best = int(np.argmin(err))
            if err[w] == err[best]:
                best = w
            want[:, w] = t[:, best]
        got = ops.tune_table(table).reshape(256, 256)
        assert np.array_equal(got, want)
        assert np.array_equal(got.reshape(-1), oracle.table_tune_weights(table))
    # a tie the own column must win: columns 5 and 9 both exact for weight 9
    t = pkg.synth.table_exact().reshape(256, 256).copy()
    t[:, 5] = t[:, 9]
    assert np.array_equal(ops.tune_table(t).reshape(256, 256)[:, 9], t[:, 9])
    t2 = pkg.synth.table_exact().reshape(256, 256).copy()
    t2[:, 9] = 0                                            # weight 9's own column is bad, 5 holds its products
    t2[:, 5] = np.arange(256) * 9
    assert np.array_equal(ops.tune_table(t2).reshape(256, 256)[:, 9], t2[:, 5])


def test_tf1_zero_point_and_output_range_closed_forms(ops):
    """FloatToQuantizedUnclamped<quint8>(0, min, max) and QuantizationRangeForMultiplication<quint8, quint8, qint32>
    (tf1/axqconv/quantization_utils.h:49-64,114-140) on cases the formula fixes by hand."""
    zp = ops.float_to_quantized_unclamped_quint8
    assert zp(0.0, 0.0, 1.0) == 0 and zp(0.0, 0.0, 6.0) == 0           # min = 0: code 0
    assert zp(0.0, -1.0, 1.0) == 128                                    # -1 * 127.5 = -127.5 rounds away from zero
    assert zp(0.0, -0.5, 1.5) == 64                                     # -0.5 * 127.5 = -63.75
    assert zp(0.0, -3.0, 0.0) == 255                                    # -3 * 85 = -255
    assert zp(0.0, 1.0, 3.0) == -128                                    # unclamped: 0 lies below the range, 1 * 127.5
    assert zp(0.0, 2.0, 2.0) == 0                                       # empty range: lowest code
    # exhaustive on a grid against exact rational arithmetic
    from fractions import Fraction
    rng = np.random.default_rng(4)
    for _ in range(200):
        lo, hi = sorted(np.float32(rng.uniform(-8, 8, size=2)))
        if lo == hi:
            continue
        width = Fraction(float(np.float32(hi - lo)))                    # the reference subtracts in float
        scale = Fraction(256) / (width * Fraction(256, 255))
        v = Fraction(float(lo)) * scale
        if abs(v - round(v)) == Fraction(1, 2) or abs((abs(v) % 1) - Fraction(1, 2)) < Fraction(1, 10 ** 6):
            continue                                                    # stay away from what double rounding decides
        want = -int(abs(v) + Fraction(1, 2)) * (1 if v >= 0 else -1)
        assert zp(0.0, float(lo), float(hi)) == want
    lo, hi = ops.quantization_range_for_multiplication(0.0, 255.0, 0.0, 255.0)
    assert lo == -2147483648.0 and hi == 2147483648.0                   # one level = 1.0; int32 max rounds up in float
    lo, hi = ops.quantization_range_for_multiplication(-1.0, 1.0, 0.0, 510.0)
    level = np.float32(np.float32(2.0) / np.float32(255.0)) * np.float32(2.0)
    assert np.float32(lo) == np.float32(level * np.float32(-2147483648.0)) and np.float32(hi) == -np.float32(lo)
    assert ops.quantization_range_for_multiplication(1.0, 1.0, 0.0, 1.0) == (0.0, 0.0)
