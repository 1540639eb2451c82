"""ctypes binding of libaxconv_hip.so (the C ABI declared in include/axconv.h).

There is no fallback: if the library is missing or a symbol is absent, loading fails loudly.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libaxconv_hip.so")

OK, INVALID_ARGUMENT, UNIMPLEMENTED, RUNTIME_ERROR = 0, 1, 2, 3
PAD_VALID, PAD_SAME, PAD_EXPLICIT = 0, 1, 2
FORMAT_NHWC, FORMAT_NCHW = 0, 1


class ConvDesc(ctypes.Structure):
    _fields_ = [
        ("input_shape", ctypes.c_int64 * 4),
        ("filter_shape", ctypes.c_int64 * 4),
        ("strides", ctypes.c_int32 * 4),
        ("dilations", ctypes.c_int32 * 4),
        ("padding", ctypes.c_int32),
        ("data_format", ctypes.c_int32),
        ("num_bits", ctypes.c_int32),
        ("explicit_paddings", ctypes.c_int64 * 8),
    ]


class ConvDims(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "batch", "input_rows", "input_cols", "in_depth", "filter_rows", "filter_cols", "patch_depth",
        "out_depth", "stride_rows", "stride_cols", "dilation_rows", "dilation_cols")] + [
        (n, ctypes.c_int64) for n in (
            "out_rows", "out_cols", "pad_rows_before", "pad_rows_after", "pad_cols_before", "pad_cols_after")]


class QuantProps(ctypes.Structure):
    _fields_ = [(n, ctypes.c_float) for n in (
        "input_scale", "input_inv_scale", "input_offset", "filter_scale", "filter_inv_scale", "filter_offset",
        "s1xs2", "m1", "m2", "m1xm2")] + [("input_zero_code", ctypes.c_int32)]


# every symbol include/axconv.h declares: (name, restype, argtypes)
_vp, _sz, _i64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int64
_f = ctypes.c_float
_desc = ctypes.POINTER(ConvDesc)
_launch_tail = [_f, _f, _f, _f, _vp, _vp, _sz, _vp]
SYMBOLS = [
    ("axc_status_string", ctypes.c_char_p, [ctypes.c_int]),
    ("axc_last_error", ctypes.c_char_p, []),
    ("axc_table_create", ctypes.c_int, [_vp, ctypes.POINTER(_vp)]),
    ("axc_table_create_from_file", ctypes.c_int, [ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(_vp)]),
    ("axc_table_destroy", ctypes.c_int, [_vp]),
    ("axc_quant_props_compute", ctypes.c_int, [_f, _f, _f, _f, ctypes.POINTER(QuantProps)]),
    ("axc_conv2d_geometry", ctypes.c_int, [_desc, ctypes.POINTER(ConvDims)]),
    ("axc_conv2d_workspace_bytes", ctypes.c_int, [_desc, ctypes.POINTER(_sz)]),
    ("axc_conv2d_tile_plan", ctypes.c_int, [_desc, ctypes.POINTER(ctypes.c_int32)]),
    ("axc_set_tile_columns", ctypes.c_int, [ctypes.c_int]),
    ("axc_set_preexpand", ctypes.c_int, [ctypes.c_int]),
    ("axc_set_wait_limit", ctypes.c_int, [ctypes.c_uint32]),
    ("axc_depthwise_conv2d_workspace_bytes", ctypes.c_int, [_desc, ctypes.POINTER(_sz)]),
    ("axc_conv2d_minmax", ctypes.c_int, [_vp, _desc, _vp, _vp] + _launch_tail),
    ("axc_depthwise_conv2d_minmax", ctypes.c_int, [_vp, _desc, _vp, _vp] + _launch_tail),
    ("axc_conv2d_minmax_bias_act", ctypes.c_int, [_vp, _desc, _vp, _vp, _f, _f, _f, _f, _vp, ctypes.c_int, _vp, _vp, _sz, _vp]),
    ("axc_depthwise_conv2d_minmax_bias_act", ctypes.c_int,
     [_vp, _desc, _vp, _vp, _f, _f, _f, _f, _vp, ctypes.c_int, _vp, _vp, _sz, _vp]),
    ("axc_conv2d_static_workspace_limit", ctypes.c_int, [ctypes.POINTER(_sz)]),
    ("axc_conv2d_minmax_static", ctypes.c_int, [_vp, _desc, _vp, _vp, _f, _f, _f, _f, _vp, _vp]),
    ("axc_fake_approx_conv2d", ctypes.c_int, [_vp, _desc, _vp, _vp, _vp, ctypes.c_int, _vp, _vp, _sz, _vp]),
    ("axc_fake_approx_depthwise_conv2d", ctypes.c_int, [_vp, _desc, _vp, _vp, _vp, ctypes.c_int, _vp, _vp, _sz, _vp]),
    ("axc_axconv2d_quint8", ctypes.c_int, [_vp, _desc, _vp, _vp, ctypes.c_int32, ctypes.c_int32, _vp, _vp, _sz, _vp]),
    ("axc_table_tune_weights", ctypes.c_int, [_vp, _vp]),
    ("axc_quint8_zero_point", ctypes.c_int, [_f, _f, ctypes.POINTER(ctypes.c_int32)]),
    ("axc_qint32_range_for_multiplication", ctypes.c_int, [_f, _f, _f, _f, ctypes.POINTER(_f), ctypes.POINTER(_f)]),
    ("axc_quantize", ctypes.c_int, [_vp, _i64, _f, _f, _vp, _vp]),
    ("axc_conv2d_minmax_acc_i32", ctypes.c_int, [_vp, _desc, _vp, _vp] + _launch_tail),
    ("axc_depthwise_conv2d_minmax_acc_i32", ctypes.c_int, [_vp, _desc, _vp, _vp] + _launch_tail),
    ("axc_conv2d_codes_acc_i32", ctypes.c_int, [_vp, _desc, _vp, _vp, ctypes.c_int, _vp, _vp, _sz, _vp]),
    ("axc_profile_enable", ctypes.c_int, [ctypes.c_int]),
    ("axc_profile_reset", ctypes.c_int, []),
    ("axc_profile_read", ctypes.c_int, [ctypes.c_int, ctypes.c_char_p, _sz, ctypes.POINTER(ctypes.c_double),
                                        ctypes.POINTER(_i64)]),
    ("axc_lds_gather_peak", ctypes.c_int, [ctypes.POINTER(ctypes.c_double), _vp]),
    ("axc_lds_read_peak", ctypes.c_int, [ctypes.POINTER(ctypes.c_double), _vp]),
    ("axc_valu_issue_peak", ctypes.c_int, [ctypes.POINTER(ctypes.c_double), _vp]),
    ("axc_lookup_mix_peak", ctypes.c_int, [ctypes.POINTER(ctypes.c_double), _vp]),
    ("axc_dense_accumulate_ops_per_lookup", ctypes.c_int, [ctypes.POINTER(ctypes.c_double)]),
    ("axc_device_info", ctypes.c_int, [ctypes.POINTER(ctypes.c_int)] * 3),
]

_lib = None


def load():
    """Loads the HIP library; raises if it has not been built (python tf-approximate_amd/build.py)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libaxconv_hip.so is not built: run `python tf-approximate_amd/build.py` "
                "(there is no CPU fallback for this op)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, restype, argtypes in SYMBOLS:
            fn = getattr(lib, name)  # AttributeError if the library does not export it
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib
