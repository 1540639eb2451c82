"""Pins the oracle's convolution path (reference: tf2/src/approx_nn_conv_kernels.cpp:167-308,
approx_nn_conv_ops.cpp:70-206,311-404) against independent statements: an index-gather numpy
implementation, integer matmul / library conv for the exact table, the reference's own direct-loop
form, and closed-form identities."""
import os

import numpy as np
import pytest

import refimpl

MM = (-1.0, 1.0, -0.5, 0.5)

CASES = [
    # x_shape, f_shape, strides, padding, dilations
    ((1, 8, 8, 4), (3, 3, 4, 6), (1, 1), "SAME", (1, 1)),
    ((2, 9, 7, 3), (3, 3, 3, 5), (1, 1), "VALID", (1, 1)),
    ((2, 11, 10, 5), (3, 2, 5, 7), (2, 2), "SAME", (1, 1)),
    ((1, 12, 13, 2), (3, 3, 2, 4), (1, 2), "SAME", (2, 2)),
    ((1, 12, 13, 2), (3, 3, 2, 4), (1, 1), "VALID", (2, 1)),
    ((3, 6, 6, 8), (1, 1, 8, 9), (1, 1), "SAME", (1, 1)),      # 1x1 path (GEMMCombined)
    ((2, 6, 6, 8), (1, 1, 8, 9), (2, 2), "VALID", (1, 1)),     # 1x1 but strided: generic path
    ((4, 5, 4, 3), (5, 4, 3, 6), (1, 1), "VALID", (1, 1)),     # filter == image path (GEMMCombined)
    ((1, 10, 10, 1), (8, 8, 1, 1), (1, 1), "SAME", (1, 1)),    # even filter: asymmetric SAME padding
]


def _qparams(oracle, mm):
    qp = oracle.quant_props(*mm)
    return (qp.in_offset, qp.in_scale, qp.f_offset, qp.f_scale)


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
@pytest.mark.parametrize("tname", ["random", "asymmetric"])
def test_oracle_vs_numpy_gather(oracle, pkg, case, tname):
    xs, fs, strides, padding, dil = case
    table = pkg.synth.table_random(3) if tname == "random" else pkg.synth.table_asymmetric()
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=hash(str(case)) % 1000)
    rc, y, acc = oracle.conv2d(table, x, f, *MM, strides=strides, padding=padding, dilations=dil)
    assert rc == 0
    acc_np, y_np = refimpl.lut_conv_numpy(table, x, f, _qparams(oracle, MM), strides, padding, dil)
    assert acc.shape == acc_np.shape
    assert np.array_equal(acc.astype(np.int64), acc_np)
    assert refimpl.linf_rel(y, y_np) < 2e-6


@pytest.mark.parametrize("case", CASES[:5], ids=[str(i) for i in range(5)])
def test_exact_table_is_integer_convolution(oracle, pkg, case):
    """With T[a][b] = a*b the sums are a plain convolution of the codes, zero-point padded."""
    xs, fs, strides, padding, dil = case
    x, f, qa, qb = refimpl.grid_case(pkg, xs, fs, MM, seed=5)
    rc, y, acc = oracle.conv2d(pkg.synth.table_exact(), x, f, *MM, strides=strides, padding=padding, dilations=dil)
    assert rc == 0
    zp = oracle.quantize(np.zeros(1, np.float32), oracle.quant_props(*MM).in_offset,
                         oracle.quant_props(*MM).in_inv_scale)[0]
    # convolve (qa - zp) with qb by the library, then add zp * sum(qb): padding contributes zp * qb
    lib = refimpl.torch_conv2d_f64(qa.astype(np.float64) - float(zp), qb.astype(np.float64), strides, padding, dil)
    lib = lib + float(zp) * qb.astype(np.float64).reshape(-1, fs[3]).sum(axis=0)
    assert np.array_equal(acc.astype(np.float64), lib)


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_exact_table_equals_library_conv_of_fake_quantized(oracle, pkg, case):
    """The reference's own acceptance test: exact table vs conv2d on the fake-quantized tensors,
    max-normalized Linf ~ 1e-7 (tf2/test/test_table_approx_conv_2d.py:46-63, tf2/README.md:30-31)."""
    xs, fs, strides, padding, dil = case
    rng = np.random.default_rng(11)
    x = pkg.fake_quant.fake_quant_with_min_max_vars(rng.uniform(-1, 1, xs).astype(np.float32), MM[0], MM[1])
    f = pkg.fake_quant.fake_quant_with_min_max_vars(rng.uniform(-0.5, 0.5, fs).astype(np.float32), MM[2], MM[3])
    rc, y, _ = oracle.conv2d(pkg.synth.table_exact(), x, f, *MM, strides=strides, padding=padding, dilations=dil)
    assert rc == 0
    ref = refimpl.torch_conv2d_f64(x, f, strides, padding, dil)
    assert refimpl.linf_rel(y, ref) < 2e-6


def test_reference_test_recipe(oracle, pkg):
    """rand[1,64,64,1] * rand[8,8,1,1], min/max 0/1, stride 1, SAME -- the reference test at reduced image size."""
    rng = np.random.default_rng(0)
    x = pkg.fake_quant.fake_quant_with_min_max_vars(rng.random((1, 64, 64, 1), dtype=np.float32), 0.0, 1.0)
    f = pkg.fake_quant.fake_quant_with_min_max_vars(rng.random((8, 8, 1, 1), dtype=np.float32), 0.0, 1.0)
    rc, y, _ = oracle.conv2d(pkg.synth.table_exact(), x, f, 0.0, 1.0, 0.0, 1.0)
    assert rc == 0
    assert refimpl.linf_rel(y, refimpl.torch_conv2d_f64(x, f)) < 1e-6


# SAME padding with an odd total (even filters, strides that leave one spare row): the im2col form takes
# pad_before = total / 2 from the windowed-output-size rule, the direct form its own origin
# ((O - 1) * s + K - I) / 2 (approx_nn_conv_ops_ref.cpp:242-251); the two must pick the same origin.
ODD_TOTAL_CASES = [
    ((1, 10, 10, 1), (8, 8, 1, 1), (1, 1), "SAME", (1, 1)),    # total 7: before 3, after 4
    ((2, 9, 11, 3), (4, 2, 3, 5), (2, 3), "SAME", (1, 1)),     # rows: total 3; cols: total 0 (11 = 3*3 + 2)
    ((1, 7, 6, 2), (2, 2, 2, 3), (1, 1), "SAME", (1, 1)),      # total 1: before 0, after 1
    ((1, 8, 8, 2), (4, 4, 2, 3), (2, 2), "SAME", (1, 1)),      # total 2 with an even filter
    ((1, 5, 5, 1), (2, 3, 1, 2), (2, 2), "SAME", (1, 1)),      # rows total 1, cols total 2
]


@pytest.mark.parametrize("case", [c for c in CASES if c[4] == (1, 1)][:6] + ODD_TOTAL_CASES)
def test_im2col_form_equals_direct_form(oracle, pkg, case):
    """The reference's two statements of the formula (im2col+GEMM vs the direct 7-deep loop) agree."""
    xs, fs, strides, padding, _ = case
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=2)
    table = pkg.synth.table_noisy(7)
    rc, y, _ = oracle.conv2d(table, x, f, *MM, strides=strides, padding=padding)
    rc2, yd = oracle.conv2d_direct(table, x, f, *MM, strides=strides, padding=padding)
    assert rc == 0 and rc2 == 0
    assert refimpl.linf_rel(y, yd) < 1e-6


def test_fast_form_equals_reference_order_form(oracle, pkg):
    for case in CASES:
        xs, fs, strides, padding, dil = case
        x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=4)
        table = pkg.synth.table_random(9)
        rc, y, acc = oracle.conv2d(table, x, f, *MM, strides=strides, padding=padding, dilations=dil)
        rc2, yf, accf = oracle.conv2d_fast(table, x, f, *MM, strides=strides, padding=padding, dilations=dil, threads=2)
        assert rc == 0 and rc2 == 0
        assert np.array_equal(acc, accf)
        assert refimpl.linf_rel(yf, y) < 1e-6


def test_padding_taps_are_looked_up_not_skipped(oracle, pkg):
    """Input range [0, max] gives zero point 0; with T[0][b] != 0 a skipped tap changes the sum."""
    table = pkg.synth.table_asymmetric()          # T[0][b] = 7b + 5
    mm = (0.0, 1.0, -0.5, 0.5)
    x, f, qa, qb = refimpl.grid_case(pkg, (1, 5, 5, 2), (3, 3, 2, 3), mm, seed=8)
    rc, _, acc = oracle.conv2d(table, x, f, *mm)
    assert rc == 0
    t = table.reshape(256, 256).astype(np.int64)
    # corner pixel (0,0): 5 of 9 taps are outside the image
    expect = 0
    for kh in range(3):
        for kw in range(3):
            for c in range(2):
                ih, iw = kh - 1, kw - 1
                a = qa[0, ih, iw, c] if (0 <= ih < 5 and 0 <= iw < 5) else 0
                expect += t[a, qb[kh, kw, c, 1]]
    assert acc[0, 0, 0, 1] == expect
    skipped = expect - sum(t[0, qb[kh, kw, c, 1]] for kh in range(3) for kw in range(3) for c in range(2)
                           if not (0 <= kh - 1 < 5 and 0 <= kw - 1 < 5))
    assert skipped != expect


def test_table_difference_identity(oracle, pkg):
    """out_T - out_exact = s1*s2 * sum(T[qa,qb] - qa*qb): here T = exact + 1, so acc grows by K everywhere."""
    x, f, _, _ = refimpl.grid_case(pkg, (1, 7, 7, 3), (3, 3, 3, 4), MM, seed=1)
    exact = pkg.synth.table_exact()
    plus1 = (exact.astype(np.int64) + 1).clip(0, 65535).astype(np.uint16)
    _, _, acc0 = oracle.conv2d(exact, x, f, *MM)
    _, _, acc1 = oracle.conv2d(plus1, x, f, *MM)
    assert np.array_equal(acc1 - acc0, np.full(acc0.shape, 27, np.int32))


def test_chunk_boundary_and_fp32_accumulator(oracle, pkg):
    """M*K above the reference's 4 Mi-element im2col buffer: the op runs in two chunks
    (approx_nn_conv_ops.cpp:118-202).  Also: the reference-order fp32 accumulator equals the integer sum
    whenever that sum is below 2^24."""
    xs, fs = (1, 96, 96, 64), (3, 3, 64, 2)              # K = 576 -> 7281 patches per chunk, M = 9216
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=6, codes="halfnormal")
    table = pkg.synth.table_exact()
    rc, y, acc = oracle.conv2d(table, x, f, *MM)
    rc2, yf, accf = oracle.conv2d_fast(table, x, f, *MM, threads=4)
    assert rc == 0 and rc2 == 0
    assert np.array_equal(acc, accf)
    assert acc.max() < (1 << 24)
    assert refimpl.linf_rel(y, yf) < 1e-6
    # The reference sums the 576 raw patch values sequentially in fp32 and multiplies by the filter offset:
    # with a large input mean (half-normal codes on [-1, 1]) that rounding dominates, ~1e-4 of the output.
    ref = refimpl.torch_conv2d_f64(x, f)
    assert refimpl.linf_rel(y, ref) < 2e-3


def test_depthwise_is_dense_per_channel(oracle, pkg):
    mm = (-1.0, 1.0, -0.5, 0.5)
    x, f, _, _ = refimpl.grid_case(pkg, (2, 9, 8, 5), (3, 3, 5, 1), mm, seed=12)
    table = pkg.synth.table_truncated(4)
    rc, y, acc = oracle.depthwise_conv2d(table, x, f, *mm, strides=(2, 2))
    assert rc == 0 and y.shape == (2, 5, 4, 5)
    for c in range(5):
        acc_c, y_c = refimpl.lut_conv_numpy(table, x[..., c:c + 1], f[:, :, c:c + 1, :],
                                            _qparams(oracle, mm), (2, 2), "SAME", (1, 1))
        assert np.array_equal(acc[..., c].astype(np.int64), acc_c[..., 0])
        assert refimpl.linf_rel(y[..., c], y_c[..., 0]) < 2e-6


def test_geometry_closed_forms(oracle):
    for in_size in (1, 2, 5, 7, 8, 32, 56, 224):
        for k in (1, 2, 3, 5, 7, 8):
            for s in (1, 2, 3):
                for d in (1, 2):
                    for padding in ("SAME", "VALID"):
                        rc, g = oracle.geometry((1, in_size, in_size, 1), (k, k, 1, 1), (s, s), padding, (d, d))
                        eff = (k - 1) * d + 1
                        if padding == "VALID":
                            expect = (in_size - eff + s) // s if in_size - eff + s >= 0 else None
                            # C division truncates toward zero: (in - eff + s) / s is 0 for small negatives
                            num = in_size - eff + s
                            expect = int(num / s)
                            if expect < 0:
                                assert rc != 0
                                continue
                            assert rc == 0 and g.out_rows == expect and g.pad_rows_before == 0
                        else:
                            assert rc == 0 and g.out_rows == -(-in_size // s)
                            pad = max(0, (g.out_rows - 1) * s + eff - in_size)
                            assert g.pad_rows_before == pad // 2 and g.pad_rows_after == pad - pad // 2


def test_dispatch_restrictions(oracle, pkg):
    table = pkg.synth.table_exact()
    x = np.zeros((1, 4, 4, 4), np.float32)
    rc, _, _ = oracle.conv2d(table, x, np.zeros((3, 3, 2, 4), np.float32), *MM)       # grouped
    assert rc == oracle.UNIMPLEMENTED
    rc, _, _ = oracle.conv2d(table, x, np.zeros((3, 3, 3, 4), np.float32), *MM)       # 4 % 3 != 0
    assert rc == oracle.INVALID_ARGUMENT
    rc, y, _ = oracle.conv2d(table, np.zeros((0, 4, 4, 4), np.float32), np.zeros((3, 3, 4, 4), np.float32), *MM)
    assert rc == 0 and y.size == 0


def test_committed_config1_vectors(oracle, pkg, golden_dir):
    z = np.load(os.path.join(golden_dir, "config1_oracle.npz"))
    case = pkg.synth.config1(seed=1)
    assert np.array_equal(case["x"], z["x"]) and np.array_equal(case["f"], z["f"])
    for tname, table in (("exact", pkg.synth.table_exact()), ("noisy", pkg.synth.table_noisy(seed=7))):
        rc, y, acc = oracle.conv2d(table, z["x"], z["f"], *[float(v) for v in z["minmax"]])
        assert rc == 0
        assert np.array_equal(acc, z["acc_" + tname])
        assert np.array_equal(y, z["y_" + tname])
    # K = 144 fp32 terms in the epilogue: a few 1e-6 of the output maximum
    assert refimpl.linf_rel(z["y_exact"], refimpl.torch_conv2d_f64(z["x"], z["f"])) < 1e-5


# ---- tf1 AxConv2D functor and AxTune ---------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [((2, 7, 6, 3), (3, 3, 3, 4), 1, "SAME"), ((1, 9, 9, 2), (3, 2, 2, 5), 2, "SAME"),
                                   ((1, 8, 10, 3), (3, 3, 3, 2), 2, "VALID"), ((1, 5, 5, 1), (1, 1, 1, 3), 1, "VALID")])
def test_tf1_axconv2d_exact_table_is_integer_convolution(oracle, shape):
    """With t[a][b] = a*b every product term collapses to (a - offset_input) * (b - offset_filter), taps outside
    the image contribute 0: the plain zero-padded integer convolution, computed here by a library routine."""
    import torch
    xs, fs, stride, padding = shape
    rng = np.random.default_rng(sum(xs) + sum(fs))
    x = rng.integers(0, 256, size=xs).astype(np.uint8)
    f = rng.integers(0, 256, size=fs).astype(np.uint8)
    off_in, off_f = 117, 131
    got = oracle.axconv2d_tf1(oracle.table_exact(), x, f, off_in, off_f, stride, padding)
    want = refimpl.torch_conv2d_f64(x.astype(np.float64) - off_in, f.astype(np.float64) - off_f, (stride, stride), padding)
    assert got.shape == want.shape
    assert np.array_equal(got.astype(np.int64), np.rint(want).astype(np.int64))


def test_tf1_axconv2d_brute_force_with_noisy_table(oracle, pkg):
    rng = np.random.default_rng(4)
    x = rng.integers(0, 256, size=(1, 4, 5, 2)).astype(np.uint8)
    f = rng.integers(0, 256, size=(3, 3, 2, 3)).astype(np.uint8)
    table = pkg.synth.table_noisy(7).reshape(256, 256).astype(np.int64)
    off_in, off_f = 3, 200
    got = oracle.axconv2d_tf1(table.astype(np.uint16), x, f, off_in, off_f, 1, "SAME")
    want = np.zeros((1, 4, 5, 3), np.int64)
    for oy in range(4):
        for ox in range(5):
            for oc in range(3):
                for fy in range(3):
                    for fx in range(3):
                        for ic in range(2):
                            iy, ix = oy + fy - 1, ox + fx - 1
                            a = int(x[0, iy, ix, ic]) if 0 <= iy < 4 and 0 <= ix < 5 else off_in
                            b = int(f[fy, fx, ic, oc])
                            want[0, oy, ox, oc] += table[a, b] - a * off_f - b * off_in + off_in * off_f
    assert np.array_equal(got.astype(np.int64), want)


def test_tf1_table_tuning(oracle, pkg):
    exact = oracle.table_exact()
    assert np.array_equal(oracle.table_tune_weights(exact), np.asarray(exact).reshape(-1))  # nothing beats exact columns
    noisy = pkg.synth.table_truncated(4).reshape(256, 256).astype(np.int64)
    i = np.arange(256, dtype=np.int64)
    err = np.abs(i[None, :, None] * i[:, None, None] - noisy[None, :, :]).sum(axis=1)   # err[w][w2]
    tuned = oracle.table_tune_weights(noisy.astype(np.uint16)).reshape(256, 256)
    for w in range(256):
        best = err[w].min()
        w2 = w if err[w][w] == best else int(np.argmax(err[w] == best))                 # ties: w itself, else the first
        assert np.array_equal(tuned[:, w], noisy[:, w2]), w
