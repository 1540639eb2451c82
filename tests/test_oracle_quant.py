"""Pins the oracle's quantization parameters and quantize expression (reference:
tf2/src/approx_ops_types.h:29-49,135-197; approx_nn_conv_kernels.cpp:293) by closed forms,
golden float bit patterns and grid invariants -- none of which retype the oracle's code."""
import numpy as np
import pytest

RANGES = [(-1.0, 1.0), (-0.3, 0.3), (0.0, 1.0), (-0.5, 1.5), (0.0, 6.0), (-2.5, 0.0), (-0.017, 0.093)]


def test_nudge_golden_bit_patterns(oracle):
    # scale = (max-min)/255 rounded to fp32; zero point = round(-min/scale) clamped; nudged_min = -zp*scale
    nmin, nmax, scale = oracle.nudge(-1.0, 1.0)
    assert float(scale).hex() == "0x1.0101020000000p-7"
    assert float(nmin).hex() == "-0x1.fdfe000000000p-1"      # zero point 127: fp32 gives 127.49999
    nmin, nmax, scale = oracle.nudge(-0.3, 0.3)
    assert float(scale).hex() == "0x1.34679c0000000p-9"
    assert float(nmin).hex() == "-0x1.34679c0000000p-2"      # zero point 128
    nmin, nmax, scale = oracle.nudge(0.0, 1.0)
    assert float(scale).hex() == "0x1.0101020000000p-8" and nmin == 0.0 and nmax == 1.0


@pytest.mark.parametrize("vmin,vmax", RANGES)
def test_nudge_closed_form(oracle, vmin, vmax):
    nmin, nmax, scale = oracle.nudge(vmin, vmax)
    f32 = np.float32
    s = f32((f32(vmax) - f32(vmin)) / f32(255.0))
    assert f32(scale) == s
    zp = -np.float64(f32(f32(vmin) / s))  # 0 - min/scale, exact in float64 after the fp32 division
    zp = int(min(max(np.floor(zp + 0.5), 0), 255))
    assert f32(nmin) == f32(f32(-zp) * s)
    assert f32(nmax) == f32(f32(255 - zp) * s)
    # the nudged range always contains 0 exactly on the grid
    assert 0 <= zp <= 255


def test_zero_range_gives_zero_props(oracle):
    qp = oracle.quant_props(0.0, 0.0, -1.0, 1.0)
    assert qp.in_scale == 0.0 and qp.in_inv_scale == 0.0 and qp.in_offset == 0.0
    assert qp.s1xs2 == 0.0 and qp.m1 == 0.0 and qp.m1xm2 == 0.0


def test_op_quant_props_products(oracle):
    qp = oracle.quant_props(-1.0, 1.0, -0.3, 0.3)
    f32 = np.float32
    assert f32(qp.s1xs2) == f32(f32(qp.in_scale) * f32(qp.f_scale))
    assert f32(qp.m1xm2) == f32(f32(qp.in_offset) * f32(qp.f_offset))
    assert qp.m1 == qp.in_offset and qp.m2 == qp.f_offset
    assert f32(qp.in_inv_scale) == f32(f32(1.0) / f32(qp.in_scale))


@pytest.mark.parametrize("vmin,vmax", RANGES)
def test_quantize_grid_invariant(oracle, vmin, vmax):
    """q(nudged_min + i*scale) == i for every code, and q(0) is the zero point."""
    nmin, nmax, scale = oracle.nudge(vmin, vmax)
    inv = np.float32(np.float32(1.0) / np.float32(scale))
    codes = np.arange(256, dtype=np.float32)
    grid = (codes * np.float32(scale)).astype(np.float32) + np.float32(nmin)
    q = oracle.quantize(grid.astype(np.float32), nmin, float(inv))
    assert np.array_equal(q, np.arange(256, dtype=np.uint8))
    zp = int(round(-nmin / scale))
    assert oracle.quantize(np.zeros(1, np.float32), nmin, float(inv))[0] == zp


def test_quantize_truncates_not_rounds_to_even(oracle):
    # offset 0, inv_scale 1: q(v) = trunc(v + 0.5): 0.5 -> 1, 1.5 -> 2, 2.5 -> 3 (round-half-even would give 0, 2, 2)
    v = np.array([0.49, 0.5, 1.5, 2.5, 2.49, 254.5, 254.49], np.float32)
    assert oracle.quantize(v, 0.0, 1.0).tolist() == [0, 1, 2, 3, 2, 255, 254]


def test_quantize_out_of_range_clamps(oracle):
    v = np.array([-5.0, -0.6, 255.6, 300.0, 1e9, -1e9], np.float32)
    assert oracle.quantize(v, 0.0, 1.0).tolist() == [0, 0, 255, 255, 255, 0]


def test_fake_quant_lands_on_grid_and_is_idempotent(pkg, oracle):
    rng = np.random.default_rng(0)
    for vmin, vmax in RANGES:
        x = rng.uniform(vmin - 0.2, vmax + 0.2, size=4096).astype(np.float32)
        fq = pkg.fake_quant.fake_quant_with_min_max_vars(x, vmin, vmax)
        nmin, nmax, scale = oracle.nudge(vmin, vmax)
        assert fq.min() >= np.float32(nmin) and fq.max() <= np.float32(nmax)
        inv = float(np.float32(1.0) / np.float32(scale))
        codes = oracle.quantize(fq, nmin, inv)
        back = pkg.fake_quant.grid_value(codes, vmin, vmax)
        assert np.array_equal(back, fq)                       # every value is nudged_min + code*scale
        assert np.array_equal(pkg.fake_quant.fake_quant_with_min_max_vars(fq, vmin, vmax), fq)
        # host mirror of Nudge agrees with the oracle's
        hmin, hmax, hscale, hzp = pkg.fake_quant.nudge(vmin, vmax)
        assert (np.float32(nmin), np.float32(nmax), np.float32(scale)) == (hmin, hmax, hscale)


def test_fake_quant_ties_clamp_edges_and_one_sided_ranges(pkg):
    """Fixed vectors worked out by hand from Nudge and the fake-quant formula
    floor((clamp(x) - nudged_min) / scale + 0.5) * scale + nudged_min, on ranges whose scale is a power of two so
    that every float operation is exact: ties round half UP (not to even, not away from zero), values at and
    beyond both nudged ends clamp, and ranges that do not contain zero are nudged until they do."""
    fq = pkg.fake_quant.fake_quant_with_min_max_vars
    f32 = np.float32
    # (0, 255): scale 1, zero point 0, grid = the integers 0..255
    x = np.array([0.0, 0.49, 0.5, 1.5, 2.5, 3.5, 254.5, 255.0, 255.49, 300.0, -0.3, -7.0], f32)
    want = np.array([0.0, 0.0, 1.0, 2.0, 3.0, 4.0, 255.0, 255.0, 255.0, 255.0, 0.0, 0.0], f32)
    assert np.array_equal(fq(x, 0.0, 255.0), want)
    # (-64, 63.5): scale 0.5, zero point 128, grid = -64 + i/2; ties sit at odd quarters
    x = np.array([-64.0, -63.75, -63.76, -63.5, -0.25, 0.25, 63.25, 63.5, 63.74, 99.0, -64.2, -1e9], f32)
    want = np.array([-64.0, -63.5, -64.0, -63.5, 0.0, 0.5, 63.5, 63.5, 63.5, 63.5, -64.0, -64.0], f32)
    assert np.array_equal(fq(x, -64.0, 63.5), want)
    # min > 0: (32, 96) has scale 64/255 and a zero point below 0 -> nudged to [0, 255 * scale]
    nmin, nmax, scale, zp = pkg.fake_quant.nudge(32.0, 96.0)
    assert zp == 0 and nmin == 0.0 and nmax == f32(f32(255.0) * scale)
    assert np.array_equal(fq(np.array([-5.0, 0.0, 1000.0], f32), 32.0, 96.0), np.array([0.0, 0.0, nmax], f32))
    # max < 0: (-96, -32) -> zero point 255, nudged to [-255 * scale, 0]
    nmin, nmax, scale, zp = pkg.fake_quant.nudge(-96.0, -32.0)
    assert zp == 255 and nmax == 0.0 and nmin == f32(f32(-255.0) * scale)
    assert np.array_equal(fq(np.array([-1000.0, 0.0, 5.0], f32), -96.0, -32.0), np.array([nmin, 0.0, 0.0], f32))
    # min == max == 0: the op's quantization constants are all zero (approx_ops_types.h:142-151) and every value maps to 0
    assert np.array_equal(fq(np.array([-1.0, 0.0, 2.0], f32), 0.0, 0.0), np.zeros(3, f32))
