"""Seeded synthetic layers, networks and truth tables for the measured configurations.

All tensors are float32 NHWC / HWIO and are passed through fake quantization, as the
reference's callers do (tf2/test/test_table_approx_conv_2d.py:39-49), so every value the op
sees lies on its 8-bit grid.
"""
import numpy as np

from .fake_quant import fake_quant_with_min_max_vars, grid_value


# ---- truth tables: uint16[65536], index (a << 8) | b, a = input code, b = filter code -------

def _ab():
    a = np.arange(256, dtype=np.int64)[:, None]
    b = np.arange(256, dtype=np.int64)[None, :]
    return a, b


def table_exact():
    a, b = _ab()
    return (a * b).astype(np.uint16).reshape(-1)


def table_noisy(seed=7, rel=0.02):
    """t = clamp(a*b + round(N(0, rel*a*b)), 0, 65535)"""
    a, b = _ab()
    rng = np.random.default_rng(seed)
    ab = (a * b).astype(np.float64)
    t = ab + np.rint(rng.standard_normal(ab.shape) * rel * ab)
    return np.clip(t, 0, 65535).astype(np.uint16).reshape(-1)


def table_truncated(k):
    """t = a*b - (a*b mod 2^k): error biased toward small operands"""
    a, b = _ab()
    ab = a * b
    return (ab - (ab % (1 << k))).astype(np.uint16).reshape(-1)


def table_uniform_error(seed=11, amp=64):
    """t = clamp(a*b + U(-amp, amp), 0, 65535)"""
    a, b = _ab()
    rng = np.random.default_rng(seed)
    t = a * b + rng.integers(-amp, amp + 1, size=(256, 256))
    return np.clip(t, 0, 65535).astype(np.uint16).reshape(-1)


def table_random(seed=13):
    """fully random uint16: worst case for LDS bank conflicts and for the fp32 accumulator"""
    rng = np.random.default_rng(seed)
    return rng.integers(0, 65536, size=65536, dtype=np.uint32).astype(np.uint16)


def table_asymmetric(seed=17):
    """t[a][b] != t[b][a] almost everywhere, and t[0][b] != 0: catches operand swaps and skipped padding taps"""
    a, b = _ab()
    return ((a * b + 3 * a + 7 * b + 5) % 65536).astype(np.uint16).reshape(-1)


# ---- tensors --------------------------------------------------------------------------------

def uniform_input(shape, lo, hi, seed):
    rng = np.random.default_rng(seed)
    x = rng.uniform(lo, hi, size=shape).astype(np.float32)
    return fake_quant_with_min_max_vars(x, lo, hi)


def normal_filter(shape, std, lim, seed):
    rng = np.random.default_rng(seed)
    f = (rng.standard_normal(shape) * std).astype(np.float32)
    return fake_quant_with_min_max_vars(f, -lim, lim)


def he_normal_filter(shape, seed):
    kh, kw, c, co = shape
    rng = np.random.default_rng(seed)
    f = (rng.standard_normal(shape) * np.sqrt(2.0 / (kh * kw * c))).astype(np.float32)
    fmin, fmax = float(f.min()), float(f.max())
    return fake_quant_with_min_max_vars(f, fmin, fmax), fmin, fmax


def half_normal_codes(shape, seed, sigma=48.0):
    rng = np.random.default_rng(seed)
    c = np.abs(rng.standard_normal(shape) * sigma)
    return np.clip(np.rint(c), 0, 255).astype(np.uint8)


def uniform_codes(shape, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 256, size=shape, dtype=np.uint32).astype(np.uint8)


def codes_to_grid(codes, vmin, vmax):
    return grid_value(codes, vmin, vmax)


# ---- configurations -------------------------------------------------------------------------

def config1(seed=1):
    """1x32x32x16 U[-1,1] (min/max -1/1); filter 3x3x16x32 N(0,0.1) (min/max -0.3/0.3); stride 1, SAME."""
    x = uniform_input((1, 32, 32, 16), -1.0, 1.0, seed)
    f = normal_filter((3, 3, 16, 32), 0.1, 0.3, seed + 100)
    return {"x": x, "f": f, "minmax": (-1.0, 1.0, -0.3, 0.3), "strides": (1, 1), "padding": "SAME"}


def north_star_layer(seed=3, batch=64, hw=56, cin=64, cout=64, codes="uniform"):
    """3x3, batch x hw x hw x cin -> cout, stride 1, SAME: the layer the headline metric is quoted on."""
    in_min, in_max, f_min, f_max = -1.0, 1.0, -0.5, 0.5
    shape = (batch, hw, hw, cin)
    qa = uniform_codes(shape, seed) if codes == "uniform" else half_normal_codes(shape, seed)
    qb = uniform_codes((3, 3, cin, cout), seed + 100)
    x = codes_to_grid(qa, in_min, in_max)
    f = codes_to_grid(qb, f_min, f_max)
    return {"x": x, "f": f, "minmax": (in_min, in_max, f_min, f_max), "strides": (1, 1), "padding": "SAME"}
