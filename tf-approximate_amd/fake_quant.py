"""Host-side fake quantization: the pre-step the reference's callers apply before the op.

The reference's test (tf2/test/test_table_approx_conv_2d.py:39-44) and its Keras layer
(tf2/python/keras/layers/fake_approx_convolutional.py:233-242) pass both operands through
tf.quantization.fake_quant_with_min_max_vars, so the op only ever sees values that lie on the
8-bit grid nudged_min + i * scale.  TensorFlow is not available here; this restates the
published algorithm of that op (clamp to the nudged range, round half up to the grid) in
float32 numpy.  Parity with TensorFlow's own implementation is unpinned: nothing in the
reference holds an input/output pair for it.
"""
import numpy as np

_f32 = np.float32


def nudge(vmin, vmax, quant_min=0, quant_max=255):
    """float32 mirror of Nudge (tf2/src/approx_ops_types.h:29-49). Returns (nudged_min, nudged_max, scale, zero_point)."""
    vmin, vmax = _f32(vmin), _f32(vmax)
    qmin, qmax = _f32(quant_min), _f32(quant_max)
    scale = _f32((vmax - vmin) / (qmax - qmin))
    zp_from_min = _f32(qmin - _f32(vmin / scale))
    if zp_from_min < qmin:
        zp = int(quant_min)
    elif zp_from_min > qmax:
        zp = int(quant_max)
    else:
        # std::round: half away from zero
        zp = int(np.floor(np.float64(zp_from_min) + 0.5)) if zp_from_min >= 0 else -int(np.floor(-np.float64(zp_from_min) + 0.5))
    nmin = _f32(_f32(qmin - _f32(zp)) * scale)
    nmax = _f32(_f32(qmax - _f32(zp)) * scale)
    return nmin, nmax, scale, zp


def fake_quant_with_min_max_vars(x, vmin, vmax, num_bits=8):
    """Clamp to the nudged range and snap to the grid; float32 in, float32 out."""
    if num_bits != 8:
        raise ValueError("only num_bits=8 is supported")
    x = np.asarray(x, np.float32)
    if _f32(vmin) == 0 and _f32(vmax) == 0:
        return np.zeros_like(x)
    nmin, nmax, scale, _ = nudge(vmin, vmax)
    inv = _f32(_f32(1.0) / scale)
    clamped = np.minimum(np.maximum(x, nmin), nmax).astype(np.float32)
    shifted = (clamped - nmin).astype(np.float32)
    q = np.floor((shifted * inv).astype(np.float32) + _f32(0.5)).astype(np.float32)
    return ((q * scale).astype(np.float32) + nmin).astype(np.float32)


def grid_value(code, vmin, vmax):
    """The float the grid holds for an integer code: nudged_min + code * scale (float32 ops)."""
    nmin, _, scale, _ = nudge(vmin, vmax)
    return ((np.asarray(code, np.float32) * scale).astype(np.float32) + nmin).astype(np.float32)
