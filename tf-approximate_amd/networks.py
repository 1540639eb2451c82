"""Seeded synthetic networks whose every convolution is the approximate op (measurement harness).

The reference evaluates its op inside Keras models (tf2/examples/*.py) whose layers do, per batch,
fake-quantization with the tensor's own min/max and then the op
(tf2/python/keras/layers/fake_approx_convolutional.py:233-258).  This module builds the same kind of
forward pass from layer lists, random He-normal weights and synthetic inputs:

    cifar_resnet   3-stage residual CNN on 32x32x3 inputs (16 / 32 / 64 channels, stride-2 between stages)
    resnet50       ResNet-50 shaped: 7x7/2 stem, bottlenecks 1x1 / 3x3 / 1x1, stage widths 256/512/1024/2048
    inverted_residual  MobileNetV2-style block: 1x1 expand (x6), depthwise 3x3 (stride 1 or 2), 1x1 project

Only the convolutions run through the library (with the ReLU that directly follows one fused into its store);
residual adds with their ReLU (one elementwise kernel built by torch.cuda.jiterator, or torch's add and relu where
that is not available) and the max-pool are torch glue.  The
min/max of every layer input and filter are taken from the tensors in a calibration pass (the Keras wrapper's
policy) and then held fixed, so the timed pass has no host synchronisation.
"""
import math

import numpy as np
import torch

from . import ops


_ADD_RELU = None


def add_relu(a, b):
    """relu(a + b) as one elementwise kernel: torch compiles the functor at its first use (hiprtc) and caches it.
    Same values as torch.relu(a + b), NaNs included; falls back to torch's two kernels where the JIT is unavailable."""
    global _ADD_RELU
    if _ADD_RELU is None:
        try:
            fn = torch.cuda.jiterator._create_jit_fn(
                "template <typename T> T add_relu(T a, T b) { T s = a + b; return s > T(0) ? s : (s == s ? T(0) : s); }")
            fn(a, b)
            _ADD_RELU = fn
        except Exception:   # no JIT on this build: torch's own kernels
            _ADD_RELU = False
    if _ADD_RELU is False:
        return torch.relu_(a.add_(b))
    return _ADD_RELU(a, b)


class ConvSpec:
    def __init__(self, kh, kw, cin, cout, stride=1, depthwise=False, relu=True):
        self.kh, self.kw, self.cin, self.cout = kh, kw, cin, cout
        self.stride, self.depthwise, self.relu = stride, depthwise, relu

    def filter_shape(self):
        return (self.kh, self.kw, self.cin, 1 if self.depthwise else self.cout)

    def macs(self, oh, ow, n):
        per_out = self.kh * self.kw * (1 if self.depthwise else self.cin)
        return n * oh * ow * (self.cin if self.depthwise else self.cout) * per_out


def _he_normal(rng, shape):
    fan_in = shape[0] * shape[1] * shape[2]
    return (rng.standard_normal(shape) * math.sqrt(2.0 / fan_in)).astype(np.float32)


class ApproxNetwork:
    """A forward pass described as a small program over named tensors:
    ("conv", dst, src, ConvSpec) | ("add_relu", dst, a, b) | ("maxpool", dst, src)"""

    def __init__(self, program, input_shape, table, seed=0, device="cuda:0", fused_layers=False, fuse_relu=True):
        """fused_layers: run every convolution, dense or depthwise, through the layer entry point (min/max of each batch and
        fake quantization computed on the device, ReLU fused), as the reference's Keras layer does per call;
        otherwise ranges come from a calibration pass and the plain op runs."""
        self.fused_layers = fused_layers
        self.fuse_relu = fuse_relu   # calibrated mode: conv + ReLU as one call (axc_conv2d_minmax_bias_act)
        self.program = program
        self.input_shape = tuple(input_shape)
        self.device = torch.device(device)
        self.table = table if isinstance(table, ops.TruthTable) else ops.TruthTable(table, 8)
        rng = np.random.default_rng(seed)
        self.weights, self.ops, self.ranges = {}, {}, {}
        for i, step in enumerate(program):
            if step[0] != "conv":
                continue
            spec = step[3]
            w = _he_normal(rng, spec.filter_shape())
            self.weights[i] = torch.from_numpy(w).to(self.device)
            if fused_layers:
                self.ops[i] = ops.FakeApproxConv2D((spec.stride, spec.stride), self.table, "SAME",
                                                   activation="relu" if spec.relu else None,
                                                   depthwise=spec.depthwise)
            else:
                self.ops[i] = ops.ApproxConv2DWithMinMaxVars([1, spec.stride, spec.stride, 1], 8, self.table, "SAME",
                                                             depthwise=spec.depthwise)

    def conv_count(self):
        return len(self.ops)

    def unfused_layers(self):
        """With fused_layers: program indices of the convolutions that still run through the calibrated op."""
        return [i for i, op in self.ops.items() if not isinstance(op, ops.FakeApproxConv2D)]

    def forward(self, x, calibrate=False, trace=None):
        """Returns (output tensor, total approximate MACs).  With a list as `trace`, every convolution appends
        (spec, input, filter, (min/max x4), raw output) as host arrays, for layer-by-layer checks."""
        t = {"input": x}
        macs = 0
        for i, step in enumerate(self.program):
            kind, dst = step[0], step[1]
            if kind == "conv":
                src, spec = t[step[2]], step[3]
                w = self.weights[i]
                if self.fused_layers:
                    y = self.ops[i](src, w)
                    if trace is not None:
                        trace.append((spec, src.cpu().numpy(), w.cpu().numpy(), None, y.cpu().numpy()))
                    macs += spec.macs(y.shape[1], y.shape[2], y.shape[0])
                    t[dst] = y
                    continue
                if calibrate or i not in self.ranges:
                    lo, hi = torch.aminmax(src)
                    wlo, whi = torch.aminmax(w)
                    self.ranges[i] = (float(lo), float(hi), float(wlo), float(whi))
                if trace is not None or not self.fuse_relu:
                    y = self.ops[i](src, w, *self.ranges[i])
                    if trace is not None:
                        trace.append((spec, src.cpu().numpy(), w.cpu().numpy(), self.ranges[i], y.cpu().numpy()))
                    y = torch.relu_(y) if spec.relu else y
                else:   # a ReLU that directly follows the convolution goes into its store
                    y = self.ops[i](src, w, *self.ranges[i], activation="relu" if spec.relu else None)
                macs += spec.macs(y.shape[1], y.shape[2], y.shape[0])
                t[dst] = y
            elif kind == "add_relu":
                t[dst] = add_relu(t[step[2]], t[step[3]])
            elif kind == "maxpool":
                nchw = t[step[2]].permute(0, 3, 1, 2)
                t[dst] = torch.nn.functional.max_pool2d(nchw, 3, 2, 1).permute(0, 2, 3, 1).contiguous()
            else:
                raise ValueError(kind)
        return t[self.program[-1][1]], macs


def cifar_resnet_program(blocks_per_stage=3):
    prog = [("conv", "x", "input", ConvSpec(3, 3, 3, 16))]
    cin = 16
    for stage, width in enumerate((16, 32, 64)):
        for b in range(blocks_per_stage):
            stride = 2 if (stage > 0 and b == 0) else 1
            prog.append(("conv", "a", "x", ConvSpec(3, 3, cin, width, stride)))
            prog.append(("conv", "b", "a", ConvSpec(3, 3, width, width, 1, relu=False)))
            if stride != 1 or cin != width:
                prog.append(("conv", "s", "x", ConvSpec(1, 1, cin, width, stride, relu=False)))
                prog.append(("add_relu", "x", "b", "s"))
            else:
                prog.append(("add_relu", "x", "b", "x"))
            cin = width
    return prog


def resnet50_program():
    prog = [("conv", "x", "input", ConvSpec(7, 7, 3, 64, 2)), ("maxpool", "x", "x")]
    cin = 64
    for stage, (width, blocks) in enumerate(((64, 3), (128, 4), (256, 6), (512, 3))):
        for b in range(blocks):
            stride = 2 if (stage > 0 and b == 0) else 1
            prog.append(("conv", "a", "x", ConvSpec(1, 1, cin, width)))
            prog.append(("conv", "b", "a", ConvSpec(3, 3, width, width, stride)))
            prog.append(("conv", "c", "b", ConvSpec(1, 1, width, width * 4, relu=False)))
            if b == 0:
                prog.append(("conv", "s", "x", ConvSpec(1, 1, cin, width * 4, stride, relu=False)))
                prog.append(("add_relu", "x", "c", "s"))
            else:
                prog.append(("add_relu", "x", "c", "x"))
            cin = width * 4
    return prog


def inverted_residual_program(cin=32, expand=6, stride=1):
    mid = cin * expand
    prog = [("conv", "e", "input", ConvSpec(1, 1, cin, mid)),
            ("conv", "d", "e", ConvSpec(3, 3, mid, mid, stride, depthwise=True)),
            ("conv", "p", "d", ConvSpec(1, 1, mid, cin, relu=False))]
    return prog


NETWORKS = {
    # name: (program builder, input shape, input range)
    "cifar_resnet_b128": (cifar_resnet_program, (128, 32, 32, 3), (0.0, 1.0)),
    "resnet50_b64": (resnet50_program, (64, 224, 224, 3), (0.0, 1.0)),
    "resnet50_b8": (resnet50_program, (8, 224, 224, 3), (0.0, 1.0)),
    "resnet50_b1": (resnet50_program, (1, 224, 224, 3), (0.0, 1.0)),
    "inverted_residual_b64_s1": (lambda: inverted_residual_program(32, 6, 1), (64, 112, 112, 32), (-1.0, 1.0)),
    "inverted_residual_b64_s2": (lambda: inverted_residual_program(32, 6, 2), (64, 112, 112, 32), (-1.0, 1.0)),
}


def build(name, table, seed=0, device="cuda:0", fused_layers=False):
    builder, shape, (lo, hi) = NETWORKS[name]
    net = ApproxNetwork(builder(), shape, table, seed=seed, device=device, fused_layers=fused_layers)
    rng = np.random.default_rng(seed + 1)
    x = torch.from_numpy(rng.uniform(lo, hi, size=shape).astype(np.float32)).to(net.device)
    return net, x
