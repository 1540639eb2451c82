"""ctypes front end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this
module; the product path never does.  The arithmetic lives in axconv_oracle.c, whose
functions cite the reference lines they restate.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libaxconv_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libaxmult_ref.so")

PAD_VALID, PAD_SAME, PAD_EXPLICIT = 0, 1, 2
OK, INVALID_ARGUMENT, UNIMPLEMENTED = 0, 1, 2

MULTIPLIER_NAMES = [
    "125K", "12N4", "13QR", "1446", "14VP", "150Q", "17C8", "17KS", "17QU", "185Q", "18DU", "199Z",
    "19DB", "1AGV", "1JFF", "2AC", "2HH", "2P7", "7C1", "96D", "CK5", "DM1", "EXZ", "FTA", "GS2",
    "JQQ", "JV3", "KEM", "L40", "NGR", "PKY", "QJD", "QKX", "Y48", "YX7", "ZFB",
]


class QuantProps(ctypes.Structure):
    _fields_ = [(n, ctypes.c_float) for n in (
        "in_scale", "in_inv_scale", "in_offset", "f_scale", "f_inv_scale", "f_offset",
        "s1xs2", "m1", "m2", "m1xm2")]


class ConvDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in (
        "batch", "in_rows", "in_cols", "in_depth", "filter_rows", "filter_cols", "patch_depth",
        "out_depth", "stride_rows", "stride_cols", "dilation_rows", "dilation_cols", "padding")] + [
        (n, ctypes.c_int64) for n in (
            "out_rows", "out_cols", "pad_rows_before", "pad_rows_after", "pad_cols_before", "pad_cols_after")]


def build():
    """Compile the oracle (and the reference multiplier models when the reference tree exists)."""
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        f32p = ctypes.POINTER(ctypes.c_float)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        u8p = ctypes.POINTER(ctypes.c_uint8)
        i32p = ctypes.POINTER(ctypes.c_int32)
        L.axo_nudge.argtypes = [ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_int, f32p, f32p, f32p]
        L.axo_nudge.restype = None
        L.axo_update_quant_props.argtypes = [ctypes.c_float] * 4 + [ctypes.POINTER(QuantProps)]
        L.axo_update_quant_props.restype = None
        L.axo_table_exact.argtypes = [u16p]
        L.axo_table_load.argtypes = [ctypes.c_char_p, u16p]
        L.axo_table_load.restype = ctypes.c_int
        L.axo_quantize.argtypes = [ctypes.c_float] * 3
        L.axo_quantize.restype = ctypes.c_uint8
        L.axo_quantize_array.argtypes = [f32p, ctypes.c_int64, ctypes.c_float, ctypes.c_float, u8p]
        L.axo_conv_geometry.argtypes = [ctypes.POINTER(ConvDesc)]
        L.axo_conv_geometry.restype = ctypes.c_int
        conv_args = [u16p, ctypes.POINTER(ConvDesc), f32p, f32p] + [ctypes.c_float] * 4
        L.axo_conv2d.argtypes = conv_args + [f32p, i32p]
        L.axo_conv2d.restype = ctypes.c_int
        L.axo_conv2d_direct.argtypes = conv_args + [f32p]
        L.axo_conv2d_direct.restype = ctypes.c_int
        L.axo_conv2d_fast.argtypes = conv_args + [f32p, i32p, ctypes.c_int]
        L.axo_conv2d_fast.restype = ctypes.c_int
        L.axo_depthwise_conv2d.argtypes = conv_args + [f32p, i32p]
        L.axo_depthwise_conv2d.restype = ctypes.c_int
        L.axo_lut_gemm_codes.argtypes = [u16p, ctypes.c_int, ctypes.c_int, ctypes.c_int, u8p, u8p, i32p]
        L.axo_lut_gemm_codes.restype = None
        L.axo_time_reference_chunk.argtypes = conv_args + [ctypes.c_int, f32p]
        L.axo_time_reference_chunk.restype = ctypes.c_double
        _lib = L
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def nudge(vmin, vmax, qmin=0, qmax=255):
    a, b, c = ctypes.c_float(), ctypes.c_float(), ctypes.c_float()
    lib().axo_nudge(vmin, vmax, qmin, qmax, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
    return a.value, b.value, c.value  # nudged_min, nudged_max, scale


def quant_props(in_min, in_max, f_min, f_max):
    qp = QuantProps()
    lib().axo_update_quant_props(in_min, in_max, f_min, f_max, ctypes.byref(qp))
    return qp


def table_exact():
    t = np.zeros(65536, np.uint16)
    lib().axo_table_exact(_p(t, ctypes.c_uint16))
    return t


def table_load(path):
    t = np.zeros(65536, np.uint16)
    rc = lib().axo_table_load(os.fsencode(path), _p(t, ctypes.c_uint16))
    if rc != OK:
        raise ValueError("ApproxTF: Couldn't read the lookup table!")
    return t


def quantize(values, offset, inv_scale):
    v = np.ascontiguousarray(values, np.float32)
    out = np.zeros(v.shape, np.uint8)
    lib().axo_quantize_array(_p(v, ctypes.c_float), v.size, offset, inv_scale, _p(out, ctypes.c_uint8))
    return out


def make_desc(x_shape, f_shape, strides=(1, 1), padding="SAME", dilations=(1, 1), depthwise=False):
    n, h, w, c = x_shape
    kh, kw, fc, co = f_shape
    d = ConvDesc()
    d.batch, d.in_rows, d.in_cols, d.in_depth = n, h, w, c
    d.filter_rows, d.filter_cols = kh, kw
    d.patch_depth = fc
    d.out_depth = c if depthwise else co
    d.stride_rows, d.stride_cols = strides
    d.dilation_rows, d.dilation_cols = dilations
    d.padding = {"VALID": PAD_VALID, "SAME": PAD_SAME, "EXPLICIT": PAD_EXPLICIT}[padding]
    return d


def geometry(x_shape, f_shape, strides=(1, 1), padding="SAME", dilations=(1, 1)):
    d = make_desc(x_shape, f_shape, strides, padding, dilations)
    rc = lib().axo_conv_geometry(ctypes.byref(d))
    return rc, d


def _run(fn, table, x, f, mins, strides, padding, dilations, want_acc, extra=(), depthwise=False, want_out=True):
    x = np.ascontiguousarray(x, np.float32)
    f = np.ascontiguousarray(f, np.float32)
    table = np.ascontiguousarray(table, np.uint16)
    d = make_desc(x.shape, f.shape, strides, padding, dilations, depthwise)
    g = make_desc(x.shape, f.shape, strides, padding, dilations, depthwise)
    rc = lib().axo_conv_geometry(ctypes.byref(g))
    if rc != OK:
        return rc, None, None
    oshape = (g.batch, int(g.out_rows), int(g.out_cols), g.out_depth)
    out = np.zeros(oshape, np.float32) if want_out else None
    acc = np.zeros(oshape, np.int32) if want_acc else None
    args = [_p(table, ctypes.c_uint16), ctypes.byref(d), _p(x, ctypes.c_float), _p(f, ctypes.c_float)]
    args += [ctypes.c_float(v) for v in mins]
    args.append(_p(out, ctypes.c_float) if out is not None else None)
    if want_acc is not None:
        args.append(_p(acc, ctypes.c_int32) if acc is not None else None)
    args += list(extra)
    rc = fn(*args)
    return rc, out, acc


def conv2d(table, x, f, in_min, in_max, f_min, f_max, strides=(1, 1), padding="SAME", dilations=(1, 1)):
    """Reference-faithful path (dispatch, chunking, j->i->l loops, fp32 accumulate). Returns (rc, out, acc_i32)."""
    return _run(lib().axo_conv2d, table, x, f, (in_min, in_max, f_min, f_max), strides, padding, dilations, True)


def conv2d_direct(table, x, f, in_min, in_max, f_min, f_max, strides=(1, 1), padding="SAME"):
    rc, out, _ = _run(lib().axo_conv2d_direct, table, x, f, (in_min, in_max, f_min, f_max), strides, padding,
                      (1, 1), None)
    return rc, out


def conv2d_fast(table, x, f, in_min, in_max, f_min, f_max, strides=(1, 1), padding="SAME", dilations=(1, 1),
                threads=8):
    return _run(lib().axo_conv2d_fast, table, x, f, (in_min, in_max, f_min, f_max), strides, padding, dilations,
                True, extra=(ctypes.c_int(threads),))


def depthwise_conv2d(table, x, f, in_min, in_max, f_min, f_max, strides=(1, 1), padding="SAME",
                     dilations=(1, 1)):
    return _run(lib().axo_depthwise_conv2d, table, x, f, (in_min, in_max, f_min, f_max), strides, padding,
                dilations, True, depthwise=True)


def lut_gemm_codes(table, a, b):
    a = np.ascontiguousarray(a, np.uint8)
    b = np.ascontiguousarray(b, np.uint8)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    acc = np.zeros((m, n), np.int32)
    table = np.ascontiguousarray(table, np.uint16)
    lib().axo_lut_gemm_codes(_p(table, ctypes.c_uint16), m, n, k, _p(a, ctypes.c_uint8), _p(b, ctypes.c_uint8),
                             _p(acc, ctypes.c_int32))
    return acc


def axconv2d_tf1(table, input_codes, filter_codes, input_offset, filter_offset, stride=1, padding="SAME"):
    """tf1 AxConv2D reference functor; output shape by TensorFlow's GetWindowedOutputSize."""
    x = np.ascontiguousarray(input_codes, np.uint8)
    f = np.ascontiguousarray(filter_codes, np.uint8)
    table = np.ascontiguousarray(table, np.uint16)
    n, h, w, c = x.shape
    kh, kw, c2, co = f.shape
    assert c == c2
    if padding == "SAME":
        oh, ow = -(-h // stride), -(-w // stride)
    else:
        oh, ow = (h - kh + stride) // stride, (w - kw + stride) // stride
    out = np.zeros((n, oh, ow, co), np.int32)
    lib().axo_axconv2d_tf1(_p(table, ctypes.c_uint16), _p(x, ctypes.c_uint8), n, h, w, c, int(input_offset),
                           _p(f, ctypes.c_uint8), kh, kw, co, int(filter_offset), int(stride),
                           1 if padding == "SAME" else 0, _p(out, ctypes.c_int32), oh, ow)
    return out


def table_tune_weights(table):
    table = np.ascontiguousarray(table, np.uint16).reshape(-1)
    tuned = np.zeros(65536, np.uint16)
    lib().axo_table_tune_weights(_p(table, ctypes.c_uint16), _p(tuned, ctypes.c_uint16))
    return tuned


def time_reference_chunk(table, x, f, in_min, in_max, f_min, f_max, patches, strides=(1, 1), padding="SAME",
                         dilations=(1, 1)):
    """Seconds the reference-faithful single-thread path needs for the first `patches` output pixels."""
    x = np.ascontiguousarray(x, np.float32)
    f = np.ascontiguousarray(f, np.float32)
    table = np.ascontiguousarray(table, np.uint16)
    d = make_desc(x.shape, f.shape, strides, padding, dilations)
    out = np.zeros((patches, f.shape[3]), np.float32)
    secs = lib().axo_time_reference_chunk(
        _p(table, ctypes.c_uint16), ctypes.byref(d), _p(x, ctypes.c_float), _p(f, ctypes.c_float),
        in_min, in_max, f_min, f_max, patches, _p(out, ctypes.c_float))
    return secs, out


# ---- the reference's own C multiplier models (built by the Makefile into _ref/) -------------

def have_ref_models():
    return os.path.exists(_REF_PATH)


def ref_model_table(name):
    """256x256 table produced by calling the reference's C model mul8u_<name>(a, b), a outer, b inner."""
    L = ctypes.CDLL(_REF_PATH)
    fn = getattr(L, "mul8u_" + name)
    if name == "1JFF":
        fn.argtypes = [ctypes.c_uint8, ctypes.c_uint8]
        fn.restype = ctypes.c_uint16
    else:
        fn.argtypes = [ctypes.c_uint64, ctypes.c_uint64]
        fn.restype = ctypes.c_uint64
    t = np.zeros(65536, np.uint16)
    for a in range(256):
        for b in range(256):
            t[a * 256 + b] = fn(a, b) & 0xFFFF
    return t
