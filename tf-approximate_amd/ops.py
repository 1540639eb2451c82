"""Python face of the op, mirroring the wrapper TensorFlow generates for the reference's
REGISTER_OP("ApproxConv2DWithMinMaxVars") (tf2/src/approx_nn_ops.cpp:38-54): same argument names,
order and meaning as the call in tf2/test/test_table_approx_conv_2d.py:47-49.

Tensors are torch tensors on a ROCm device (torch is only the owner of device memory and of the
stream); all arithmetic happens in libaxconv_hip.so.
"""
import ctypes

import numpy as np

import torch

from . import _lib


class InvalidArgumentError(ValueError):
    """tensorflow::errors::InvalidArgument in the reference."""


class UnimplementedError(NotImplementedError):
    """tensorflow::errors::Unimplemented in the reference."""


def _check(rc):
    if rc == _lib.OK:
        return
    msg = _lib.load().axc_last_error().decode()
    if rc == _lib.INVALID_ARGUMENT:
        raise InvalidArgumentError(msg)
    if rc == _lib.UNIMPLEMENTED:
        raise UnimplementedError(msg)
    raise RuntimeError(msg)


_PADDING = {"VALID": _lib.PAD_VALID, "SAME": _lib.PAD_SAME, "EXPLICIT": _lib.PAD_EXPLICIT}
_FORMAT = {"NHWC": _lib.FORMAT_NHWC, "NCHW": _lib.FORMAT_NCHW}


def make_desc(input_shape, filter_shape, strides, padding, explicit_paddings=(), data_format="NHWC",
              dilations=(1, 1, 1, 1), num_bits=8):
    if len(input_shape) != 4:
        raise InvalidArgumentError("input must be 4-dimensional")
    if len(filter_shape) != 4:
        raise InvalidArgumentError("filter must be 4-dimensional")
    if len(strides) != 4:
        raise InvalidArgumentError("Sliding window strides must specify 4 dimensions")
    if len(dilations) != 4:
        raise InvalidArgumentError("Sliding window dilations field must specify 4 dimensions")
    if isinstance(padding, bytes):
        padding = padding.decode()
    if padding not in _PADDING:
        raise InvalidArgumentError("Invalid padding")
    if data_format not in _FORMAT:
        raise InvalidArgumentError("Invalid data format")
    d = _lib.ConvDesc()
    for i in range(4):
        d.input_shape[i] = int(input_shape[i])
        d.filter_shape[i] = int(filter_shape[i])
        d.strides[i] = int(strides[i])
        d.dilations[i] = int(dilations[i])
    d.padding = _PADDING[padding]
    d.data_format = _FORMAT[data_format]
    d.num_bits = int(num_bits)
    ep = list(explicit_paddings) + [0] * 8
    for i in range(8):
        d.explicit_paddings[i] = int(ep[i])
    return d


def conv2d_geometry(desc):
    dims = _lib.ConvDims()
    _check(_lib.load().axc_conv2d_geometry(ctypes.byref(desc), ctypes.byref(dims)))
    return dims


def quant_props(input_min, input_max, filter_min, filter_max):
    qp = _lib.QuantProps()
    _check(_lib.load().axc_quant_props_compute(float(input_min), float(input_max), float(filter_min),
                                               float(filter_max), ctypes.byref(qp)))
    return qp


class TruthTable:
    """Device-resident 256x256 uint16 truth table (the op's `mul_map_file` attr, loaded once)."""

    def __init__(self, source="", num_bits=8):
        lib = _lib.load()
        handle = ctypes.c_void_p()
        if isinstance(source, (str, bytes)):
            name = source.encode() if isinstance(source, str) else source
            _check(lib.axc_table_create_from_file(name, int(num_bits), ctypes.byref(handle)))
        else:
            import numpy as np
            if int(num_bits) != 8:
                raise InvalidArgumentError("only num_bits = 8 is supported")
            host = np.ascontiguousarray(source, dtype=np.uint16).reshape(-1)
            if host.size != 65536:
                raise InvalidArgumentError("truth table must hold 65536 uint16 entries")
            _check(lib.axc_table_create(host.ctypes.data, ctypes.byref(handle)))
        self.handle = handle

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                _lib.load().axc_table_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


_workspaces = {}


def _workspace(device, nbytes):
    """Scratch memory of a call, cached per (device, current stream): calls issued on one stream run in order and
    may share it; calls on different streams may overlap and must not."""
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def _scalar(v):
    if torch.is_tensor(v):
        return float(v.item())
    return float(v)


def _stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require_device_f32(t, what):
    if not torch.is_tensor(t) or not t.is_cuda:
        raise InvalidArgumentError("%s must be a tensor on the GPU" % what)
    if t.dtype != torch.float32:
        raise UnimplementedError("%s: only float32 is registered for this op" % what)
    return t.contiguous()


class ApproxConv2DWithMinMaxVars:
    """One op instance: attrs fixed at construction, like the reference's OpKernel
    (ApproxConv2DOp, tf2/src/approx_nn_conv_ops.cpp:411-468)."""

    def __init__(self, strides, num_bits, mul_map_file, padding, explicit_paddings=(), data_format="NHWC",
                 dilations=(1, 1, 1, 1), depthwise=False):
        self.strides = list(strides)
        self.num_bits = int(num_bits)
        self.padding = padding
        self.explicit_paddings = list(explicit_paddings)
        self.data_format = data_format
        self.dilations = list(dilations)
        self.depthwise = depthwise
        self.table = mul_map_file if isinstance(mul_map_file, TruthTable) else TruthTable(mul_map_file, num_bits)
        # attr checks the reference performs at construction (InitApproxConv2DParameters)
        make_desc((1, 1, 1, 1), (1, 1, 1, 1), self.strides, self.padding, self.explicit_paddings,
                  self.data_format, self.dilations, self.num_bits)

    def _desc(self, input, filter):
        return make_desc(tuple(input.shape), tuple(filter.shape), self.strides, self.padding,
                         self.explicit_paddings, self.data_format, self.dilations, self.num_bits)

    def _out_shape(self, dims):
        depth = dims.in_depth if self.depthwise else dims.out_depth
        return (dims.batch, int(dims.out_rows), int(dims.out_cols), depth)

    def _run(self, input, filter, mins, acc_i32):
        lib = _lib.load()
        input = _require_device_f32(input, "input")
        filter = _require_device_f32(filter, "filter")
        desc = self._desc(input, filter)
        dims = conv2d_geometry(desc)
        nbytes = ctypes.c_size_t()
        ws_fn = lib.axc_depthwise_conv2d_workspace_bytes if self.depthwise else lib.axc_conv2d_workspace_bytes
        _check(ws_fn(ctypes.byref(desc), ctypes.byref(nbytes)))
        ws = _workspace(input.device, nbytes.value)
        out = torch.empty(self._out_shape(dims), dtype=torch.int32 if acc_i32 else torch.float32,
                          device=input.device)
        if self.depthwise:
            fn = lib.axc_depthwise_conv2d_minmax_acc_i32 if acc_i32 else lib.axc_depthwise_conv2d_minmax
        else:
            fn = lib.axc_conv2d_minmax_acc_i32 if acc_i32 else lib.axc_conv2d_minmax
        with torch.cuda.device(input.device):
            _check(fn(self.table.handle, ctypes.byref(desc), input.data_ptr(), filter.data_ptr(),
                      *[_scalar(m) for m in mins], out.data_ptr(), ws.data_ptr(), ws.numel(),
                      _stream_ptr(input.device)))
        return out

    def __call__(self, input, filter, input_min, input_max, filter_min, filter_max, bias=None, activation=None):
        """The op.  With `bias` and / or `activation` ("relu"): the op followed by bias_add and the activation, fused
        into its store (the tail of the Keras layer's call, fake_approx_convolutional.py:261)."""
        if bias is None and activation is None:
            return self._run(input, filter, (input_min, input_max, filter_min, filter_max), False)
        if activation not in (None, "relu"):
            raise InvalidArgumentError("activation must be None or 'relu'")
        lib = _lib.load()
        input = _require_device_f32(input, "input")
        filter = _require_device_f32(filter, "filter")
        desc = self._desc(input, filter)
        dims = conv2d_geometry(desc)
        out_shape = self._out_shape(dims)
        if bias is not None:
            bias = _require_device_f32(bias, "bias")
            if bias.numel() != out_shape[3]:
                raise InvalidArgumentError("bias must have one value per output channel")
        nbytes = ctypes.c_size_t()
        ws_fn = lib.axc_depthwise_conv2d_workspace_bytes if self.depthwise else lib.axc_conv2d_workspace_bytes
        _check(ws_fn(ctypes.byref(desc), ctypes.byref(nbytes)))
        ws = _workspace(input.device, nbytes.value)
        out = torch.empty(out_shape, dtype=torch.float32, device=input.device)
        fn = lib.axc_depthwise_conv2d_minmax_bias_act if self.depthwise else lib.axc_conv2d_minmax_bias_act
        with torch.cuda.device(input.device):
            _check(fn(self.table.handle, ctypes.byref(desc), input.data_ptr(), filter.data_ptr(),
                      *[_scalar(m) for m in (input_min, input_max, filter_min, filter_max)],
                      bias.data_ptr() if bias is not None else None, 1 if activation == "relu" else 0,
                      out.data_ptr(), ws.data_ptr(), ws.numel(), _stream_ptr(input.device)))
        return out

    def accumulators(self, input, filter, input_min, input_max, filter_min, filter_max):
        """int32 sums of table entries before the epilogue (parity entry point)."""
        return self._run(input, filter, (input_min, input_max, filter_min, filter_max), True)


class FakeApproxConv2D:
    """The reference's Keras layer around the op (FakeApproxConv2D.call,
    tf2/python/keras/layers/fake_approx_convolutional.py:223-261) as one device-side call: min/max of the batch
    and of the kernel, fake quantization of both, the op, bias_add, activation.  No host synchronisation."""

    def __init__(self, strides, mul_map_file, padding="SAME", dilation_rate=(1, 1), activation=None, num_bits=8,
                 depthwise=False):
        """depthwise: the layer wraps the depthwise variant (kernel [rows, cols, C, 1], bias one value per channel)."""
        if activation not in (None, "relu"):
            raise UnimplementedError("activation %r: only None and 'relu' are fused" % (activation,))
        self.op = ApproxConv2DWithMinMaxVars([1, strides[0], strides[1], 1], num_bits, mul_map_file, padding.upper(),
                                             dilations=[1, dilation_rate[0], dilation_rate[1], 1], depthwise=depthwise)
        self.depthwise = depthwise
        self.activation = 1 if activation == "relu" else 0

    def __call__(self, inputs, kernel, bias=None):
        lib = _lib.load()
        inputs = _require_device_f32(inputs, "input")
        kernel = _require_device_f32(kernel, "filter")
        if bias is not None:
            bias = _require_device_f32(bias, "bias")
            if bias.numel() != (kernel.shape[2] if self.depthwise else kernel.shape[3]):
                raise InvalidArgumentError("bias must have one value per output channel")
        desc = self.op._desc(inputs, kernel)
        dims = conv2d_geometry(desc)
        nbytes = ctypes.c_size_t()
        ws_fn = lib.axc_depthwise_conv2d_workspace_bytes if self.depthwise else lib.axc_conv2d_workspace_bytes
        _check(ws_fn(ctypes.byref(desc), ctypes.byref(nbytes)))
        ws = _workspace(inputs.device, nbytes.value)
        out = torch.empty(self.op._out_shape(dims), dtype=torch.float32, device=inputs.device)
        fn = lib.axc_fake_approx_depthwise_conv2d if self.depthwise else lib.axc_fake_approx_conv2d
        with torch.cuda.device(inputs.device):
            _check(fn(self.op.table.handle, ctypes.byref(desc), inputs.data_ptr(),
                                              kernel.data_ptr(), bias.data_ptr() if bias is not None else None,
                                              self.activation, out.data_ptr(), ws.data_ptr(), ws.numel(),
                                              _stream_ptr(inputs.device)))
        return out


# ---- tf1 AxConv2D (tf1/axqconv/axqconv.cc) ----------------------------------------------------------------------
def float_to_quantized_unclamped_quint8(value, range_min, range_max):
    """FloatToQuantizedUnclamped<quint8> for the value 0.0f (tf1/axqconv/quantization_utils.h:49-64): the zero
    point the reference derives per tensor (tf1/axqconv/axqconv.cc:364-367).  Computed by the library."""
    if float(value) != 0.0:
        raise UnimplementedError("only the code of 0.0f is needed by AxConv2D")
    zp = ctypes.c_int32()
    _check(_lib.load().axc_quint8_zero_point(float(range_min), float(range_max), ctypes.byref(zp)))
    return zp.value


def quantization_range_for_multiplication(min_a, max_a, min_b, max_b):
    """QuantizationRangeForMultiplication<quint8, quint8, qint32> (tf1/axqconv/quantization_utils.h:114-140): the
    float range the qint32 output of AxConv2D stands for (tf1/axqconv/axqconv.cc:427-431)."""
    lo, hi = ctypes.c_float(), ctypes.c_float()
    _check(_lib.load().axc_qint32_range_for_multiplication(float(min_a), float(max_a), float(min_b), float(max_b),
                                                           ctypes.byref(lo), ctypes.byref(hi)))
    return lo.value, hi.value


def tune_table(table):
    """AxTune of the tf1 op (tf1/axqconv/approximate_selector.h:52-85) applied to a uint16[65536] table."""
    lib = _lib.load()
    src = np.ascontiguousarray(table, np.uint16).reshape(-1)
    if src.size != 65536:
        raise InvalidArgumentError("table must hold 65536 entries")
    out = np.zeros(65536, np.uint16)
    _check(lib.axc_table_tune_weights(src.ctypes.data, out.ctypes.data))
    return out


def ax_conv2d(input, filter, min_input, max_input, min_filter, max_filter, strides, padding, table):
    """The tf1 op AxConv2D (registration tf1/axqconv/axqconv.cc:66-94): quint8 codes in (uint8 tensors on the GPU),
    (qint32 output, min_output, max_output) out.  `table` is a TruthTable (AxMult / AxTune already applied)."""
    lib = _lib.load()
    if input.dtype != torch.uint8 or filter.dtype != torch.uint8:
        raise UnimplementedError("AxConv2D: only quint8 input and filter are registered")
    if not input.is_cuda or not filter.is_cuda:
        raise InvalidArgumentError("input and filter must be tensors on the GPU")
    input, filter = input.contiguous(), filter.contiguous()
    desc = make_desc(tuple(input.shape), tuple(filter.shape), list(strides), padding, (), "NHWC", (1, 1, 1, 1), 8)
    dims = conv2d_geometry(desc)
    nbytes = ctypes.c_size_t()
    _check(lib.axc_conv2d_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)))
    ws = _workspace(input.device, nbytes.value)
    out = torch.empty((dims.batch, int(dims.out_rows), int(dims.out_cols), dims.out_depth), dtype=torch.int32,
                      device=input.device)
    off_in = float_to_quantized_unclamped_quint8(0.0, min_input, max_input)
    off_f = float_to_quantized_unclamped_quint8(0.0, min_filter, max_filter)
    with torch.cuda.device(input.device):
        _check(lib.axc_axconv2d_quint8(table.handle, ctypes.byref(desc), input.data_ptr(), filter.data_ptr(), off_in, off_f,
                                       out.data_ptr(), ws.data_ptr(), ws.numel(), _stream_ptr(input.device)))
    lo, hi = quantization_range_for_multiplication(min_input, max_input, min_filter, max_filter)
    return out, lo, hi


def conv2d_tile_plan(input_shape, filter_shape, strides=(1, 1, 1, 1), padding="SAME", dilations=(1, 1, 1, 1)):
    """The dense kernel's tile plan for a layer on the current device, as a dict."""
    lib = _lib.load()
    desc = make_desc(tuple(input_shape), tuple(filter_shape), list(strides), padding, (), "NHWC", list(dilations), 8)
    plan = (ctypes.c_int32 * 8)()
    _check(lib.axc_conv2d_tile_plan(ctypes.byref(desc), plan))
    # preexpanded_rows: 0 = rows expanded inside every tile, 1 = pre-expanded rows, 2 = pre-expanded rows read by the
    # kernel without a barrier between fills
    keys = ("columns_per_tile", "rows_per_tile", "row_tiles", "column_tiles", "k_splits", "workgroups",
            "fills_per_split", "preexpanded_rows")
    return dict(zip(keys, [int(v) for v in plan]))


def set_tile_columns(columns):
    """Pins the dense kernel's tile width (16 / 32 / 64 columns; 0 = the planner's choice) for the whole process."""
    _check(_lib.load().axc_set_tile_columns(int(columns)))


def set_preexpand(mode):
    """Which dense layers run out of pre-expanded rows: 0 = the planner's choice, 1 = all that can, -1 = none."""
    _check(_lib.load().axc_set_preexpand(int(mode)))


def set_wait_limit(polls):
    """Polls a wavefront of the barrier-free LUT-GEMM kernel makes in one wait before it gives up (tests of the
    report; the default is 2**20)."""
    _check(_lib.load().axc_set_wait_limit(int(polls)))


_table_cache = {}


def _cached_table(mul_map_file, num_bits):
    if isinstance(mul_map_file, TruthTable):
        return mul_map_file
    if not isinstance(mul_map_file, (str, bytes)):
        return TruthTable(mul_map_file, num_bits)
    key = (mul_map_file, int(num_bits))
    if key not in _table_cache:
        _table_cache[key] = TruthTable(mul_map_file, num_bits)
    return _table_cache[key]


def approx_conv2d_with_min_max_vars(input, filter, input_min, input_max, filter_min, filter_max, strides,
                                    num_bits, mul_map_file, padding, explicit_paddings=(), data_format="NHWC",
                                    dilations=(1, 1, 1, 1), name=None):
    """Drop-in for the generated wrapper of the reference op (argument order of
    tf2/test/test_table_approx_conv_2d.py:47-49).  mul_map_file may also be a TruthTable or a
    uint16[65536] array, so seeded synthetic tables need no file."""
    op = ApproxConv2DWithMinMaxVars(strides, num_bits, _cached_table(mul_map_file, num_bits), padding,
                                    explicit_paddings, data_format, dilations)
    return op(input, filter, input_min, input_max, filter_min, filter_max)


def approx_depthwise_conv2d_with_min_max_vars(input, filter, input_min, input_max, filter_min, filter_max,
                                              strides, num_bits, mul_map_file, padding, explicit_paddings=(),
                                              data_format="NHWC", dilations=(1, 1, 1, 1), name=None):
    """Depthwise variant (filter [rows, cols, C, 1]); the reference has no such op."""
    op = ApproxConv2DWithMinMaxVars(strides, num_bits, _cached_table(mul_map_file, num_bits), padding,
                                    explicit_paddings, data_format, dilations, depthwise=True)
    return op(input, filter, input_min, input_max, filter_min, filter_max)


def quantize(values, vmin, vmax):
    """uint8 codes of a float32 device tensor (parity entry point for the quantize expression)."""
    values = _require_device_f32(values, "values")
    codes = torch.empty(values.shape, dtype=torch.uint8, device=values.device)
    with torch.cuda.device(values.device):
        _check(_lib.load().axc_quantize(values.data_ptr(), values.numel(), float(vmin), float(vmax),
                                        codes.data_ptr(), _stream_ptr(values.device)))
    return codes


def conv2d_codes_acc_i32(table, input_codes, filter_codes, input_zero_code, strides=(1, 1, 1, 1),
                         padding="SAME", dilations=(1, 1, 1, 1)):
    """int32 LUT-GEMM sums on caller-supplied uint8 codes (NHWC / HWIO device tensors)."""
    lib = _lib.load()
    if input_codes.dtype != torch.uint8 or filter_codes.dtype != torch.uint8:
        raise InvalidArgumentError("codes must be uint8")
    input_codes = input_codes.contiguous()
    filter_codes = filter_codes.contiguous()
    desc = make_desc(tuple(input_codes.shape), tuple(filter_codes.shape), strides, padding, (), "NHWC", dilations)
    dims = conv2d_geometry(desc)
    nbytes = ctypes.c_size_t()
    _check(lib.axc_conv2d_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)))
    ws = _workspace(input_codes.device, nbytes.value)
    out = torch.empty((dims.batch, int(dims.out_rows), int(dims.out_cols), dims.out_depth), dtype=torch.int32,
                      device=input_codes.device)
    with torch.cuda.device(input_codes.device):
        _check(lib.axc_conv2d_codes_acc_i32(table.handle, ctypes.byref(desc), input_codes.data_ptr(),
                                            filter_codes.data_ptr(), int(input_zero_code), out.data_ptr(),
                                            ws.data_ptr(), ws.numel(), _stream_ptr(input_codes.device)))
    return out


# ---- measurement helpers ---------------------------------------------------------------------

def profile_enable(on=True):
    _check(_lib.load().axc_profile_enable(1 if on else 0))


def profile_reset():
    _check(_lib.load().axc_profile_reset())


def profile_read():
    """{kernel name: (total_ms, launches)} since the last reset."""
    lib = _lib.load()
    out = {}
    i = 0
    while True:
        name = ctypes.create_string_buffer(64)
        ms = ctypes.c_double()
        n = ctypes.c_int64()
        if lib.axc_profile_read(i, name, 64, ctypes.byref(ms), ctypes.byref(n)) != _lib.OK:
            break
        out[name.value.decode()] = (ms.value, n.value)
        i += 1
    return out


def lds_gather_peak():
    v = ctypes.c_double()
    _check(_lib.load().axc_lds_gather_peak(ctypes.byref(v), None))
    return v.value


def lds_read_peak():
    """Streaming ds_read_b128 rate in bytes/s over all CUs (measured)."""
    v = ctypes.c_double()
    _check(_lib.load().axc_lds_read_peak(ctypes.byref(v), None))
    return v.value


def valu_issue_peak():
    """Issue rate of the LUT-GEMM's accumulate instruction mix in lane operations per second (measured)."""
    v = ctypes.c_double()
    _check(_lib.load().axc_valu_issue_peak(ctypes.byref(v), None))
    return v.value


def lookup_mix_peak():
    """Table entries per second of a kernel made of nothing but the LUT-GEMM's per-lookup instructions (address,
    16-byte LDS read, accumulate), in its occupancy (measured)."""
    v = ctypes.c_double()
    _check(_lib.load().axc_lookup_mix_peak(ctypes.byref(v), None))
    return v.value


def dense_accumulate_ops_per_lookup():
    v = ctypes.c_double()
    _check(_lib.load().axc_dense_accumulate_ops_per_lookup(ctypes.byref(v)))
    return v.value


def device_info():
    a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    _check(_lib.load().axc_device_info(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
    return {"compute_units": a.value, "lds_bytes_per_workgroup": b.value, "clock_khz": c.value}
