"""Every distinct convolution of the ResNet-50-shaped network at its full batch of 64, and the layers of the
inverted-residual block at 64x112x112, through the op with oracle evaluation of sampled output pixels (the
tensors are too large for the CPU oracle to recompute whole).  Covers the shapes the per-layer tests leave out:
the 1x1 stride-2 projections, the stem at batch 64, every stage's 1x1 and 3x3 shapes."""
import numpy as np
import pytest
import torch

import bench

pytestmark = pytest.mark.gpu

MM = (-1.0, 1.0, -0.5, 0.5)


def _distinct_convs(program, input_shape):
    """Walks a network program and returns the distinct (input shape, filter shape, stride, depthwise) of its
    convolutions, in order of first appearance."""
    shapes = {"input": tuple(input_shape)}
    seen, out = set(), []
    for step in program:
        kind, dst = step[0], step[1]
        if kind == "conv":
            n, h, w, c = shapes[step[2]]
            spec = step[3]
            assert c == spec.cin
            oh, ow = -(-h // spec.stride), -(-w // spec.stride)
            key = ((n, h, w, c), spec.filter_shape(), spec.stride, spec.depthwise)
            if key not in seen:
                seen.add(key)
                out.append(key)
            shapes[dst] = (n, oh, ow, spec.cin if spec.depthwise else spec.cout)
        elif kind == "add_relu":
            shapes[dst] = shapes[step[2]]
        elif kind == "maxpool":
            n, h, w, c = shapes[step[2]]
            shapes[dst] = (n, -(-h // 2), -(-w // 2), c)
    return out


def _layers():
    import __graft_entry__ as entry
    entry.load_package()
    from tf_approximate_amd import networks
    convs = [("resnet50",) + k for k in _distinct_convs(networks.resnet50_program(), (64, 224, 224, 3))]
    for stride in (1, 2):
        convs += [("inverted_residual_s%d" % stride,) + k
                  for k in _distinct_convs(networks.inverted_residual_program(32, 6, stride), (64, 112, 112, 32))]
    return convs


def _id(case):
    net, xs, fs, stride, dw = case
    return "%s-%dx%dx%d-%dx%d-%dto%d-s%d%s" % (net, xs[1], xs[2], xs[3], fs[0], fs[1], fs[2], xs[3] if dw else fs[3],
                                                stride, "-dw" if dw else "")


def test_the_walk_finds_the_shapes_it_is_for():
    cases = _layers()
    keys = {(c[1][1:], c[2], c[3]) for c in cases}
    assert ((224, 224, 3), (7, 7, 3, 64), 2) in keys                      # stem at batch 64
    assert ((56, 56, 256), (1, 1, 256, 512), 2) in keys                   # 1x1 stride-2 projection
    assert ((7, 7, 512), (1, 1, 512, 2048), 1) in keys and ((7, 7, 2048), (1, 1, 2048, 512), 1) in keys
    assert ((28, 28, 128), (3, 3, 128, 128), 1) in keys and ((14, 14, 256), (3, 3, 256, 256), 1) in keys
    assert ((112, 112, 32), (1, 1, 32, 192), 1) in keys and ((112, 112, 192), (1, 1, 192, 32), 1) in keys
    assert all(c[1][0] == 64 for c in cases) and len(cases) >= 25


@pytest.mark.parametrize("case", _layers(), ids=_id)
def test_network_layer_at_full_batch_sampled_pixels(pkg, oracle, case):
    net, xs, fs, stride, depthwise = case
    print("layer", _id(case), flush=True)
    table_host = pkg.synth.table_uniform_error(11) if net == "resnet50" else pkg.synth.table_truncated(4)
    xd, fd = bench.device_tensors(pkg, xs, fs, "halfnormal" if xs[3] >= 256 else "uniform", seed=sum(xs) + sum(fs))
    op = pkg.ApproxConv2DWithMinMaxVars([1, stride, stride, 1], 8, table_host, "SAME", depthwise=depthwise)
    y = op(xd, fd, *MM)
    exact, linf = bench.sampled_oracle_check(oracle, table_host, op, xd, fd, (stride, stride), depthwise, y,
                                             n_samples=16, seed=len(_id(case)))
    assert exact, "int32 accumulators differ from the oracle on sampled pixels"
    assert linf <= 1e-5
    assert torch.isfinite(y).all()
