"""Every distinct convolution of the ResNet-50-shaped network at its full batch of 64, of the CIFAR-style residual
network at its full batch of 128, and the layers of the inverted-residual block at 64x112x112, through the op.

Two checks per layer.  Sampled pixels against the CPU oracle, with any table (the tensors are too large for the
oracle to recompute whole), in the planner's own choice of kernel and in the other one where the layer can run
both.  And the WHOLE output with the exact table against the integer convolution of the codes, computed in fp64 by
torch on the GPU (every partial sum is an integer below 2^53, so fp64 is exact in any order): every tile of every
layer's tile walk, every K-split seam and every staggered start group is compared.  Covers the shapes the per-layer
tests leave out: the 1x1 stride-2 projections, the stem at batch 64, every stage's 1x1 and 3x3 shapes, the small
tiles of the 32x32 layers at batch 128."""
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
    convs += [("cifar_resnet",) + k for k in _distinct_convs(networks.cifar_resnet_program(), (128, 32, 32, 3))]
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
    assert ((32, 32, 3), (3, 3, 3, 16), 1) in keys and ((32, 32, 16), (3, 3, 16, 16), 1) in keys   # CIFAR-size, batch 128
    assert ((32, 32, 16), (3, 3, 16, 32), 2) in keys and ((8, 8, 64), (3, 3, 64, 64), 1) in keys
    assert all(c[1][0] == (128 if c[0] == "cifar_resnet" else 64) for c in cases) and len(cases) >= 35


def _table_for(pkg, net):
    return pkg.synth.table_uniform_error(11) if net == "resnet50" else (
        pkg.synth.table_noisy(7) if net == "cifar_resnet" else pkg.synth.table_truncated(4))


def _sampled(pkg, oracle, case):
    net, xs, fs, stride, depthwise = case
    table_host = _table_for(pkg, net)
    xd, fd = bench.device_tensors(pkg, xs, fs, "halfnormal" if xs[3] >= 256 else "uniform", seed=sum(xs) + sum(fs))
    op = pkg.ApproxConv2DWithMinMaxVars([1, stride, stride, 1], 8, table_host, "SAME", depthwise=depthwise)
    y = op(xd, fd, *MM)
    exact, linf = bench.sampled_oracle_check(oracle, table_host, op, xd, fd, (stride, stride), depthwise, y,
                                             n_samples=16, seed=len(_id(case)))
    assert exact, "int32 accumulators differ from the oracle on sampled pixels"
    assert linf <= 1e-5


@pytest.mark.parametrize("case", _layers(), ids=_id)
def test_network_layer_at_full_batch_sampled_pixels(pkg, oracle, case):
    print("layer", _id(case), flush=True)
    _sampled(pkg, oracle, case)


def _plan_uses_preexpanded_rows(pkg, case, mode):
    _, xs, fs, stride, _ = case
    pkg.ops.set_preexpand(mode)
    try:
        return bool(pkg.ops.conv2d_tile_plan(xs, fs, (1, stride, stride, 1))["preexpanded_rows"])
    finally:
        pkg.ops.set_preexpand(0)


@pytest.mark.parametrize("case", [c for c in _layers() if not c[4]], ids=_id)
def test_network_layer_sampled_pixels_in_the_kernel_the_planner_did_not_pick(pkg, oracle, case):
    """Each dense layer once more with the other LUT-GEMM kernel: out of pre-expanded rows where the planner expands
    inside the tiles, and the other way round.  Layers that can only run one way are skipped."""
    own = _plan_uses_preexpanded_rows(pkg, case, 0)
    other_mode = -1 if own else 1
    if _plan_uses_preexpanded_rows(pkg, case, other_mode) == own:
        pytest.skip("only one kernel can run this layer")
    print("layer", _id(case), "preexpand", other_mode, flush=True)
    pkg.ops.set_preexpand(other_mode)
    try:
        _sampled(pkg, oracle, case)
    finally:
        pkg.ops.set_preexpand(0)


def exact_conv_of_codes(qa, qb, zp, geom, stride, depthwise):
    """Integer convolution of uint8 codes in fp64 on the device: qa NHWC, qb HWIO (HWC1 for depthwise), taps outside
    the image read the zero-point code zp.  geom = (OH, OW, pad_rows_before, pad_cols_before)."""
    OH, OW, ph, pw = geom
    N, H, W, C = qa.shape
    KH, KW = qb.shape[0], qb.shape[1]
    pad_h_after = max(0, (OH - 1) * stride + KH - H - ph)
    pad_w_after = max(0, (OW - 1) * stride + KW - W - pw)
    a = torch.nn.functional.pad(qa.double(), (0, 0, pw, pad_w_after, ph, pad_h_after), value=float(zp))
    b = qb.double()
    Cout = C if depthwise else qb.shape[3]
    total = torch.zeros((N, OH, OW, Cout), dtype=torch.float64, device=qa.device)
    for kh in range(KH):
        for kw in range(KW):
            win = a[:, kh:kh + (OH - 1) * stride + 1:stride, kw:kw + (OW - 1) * stride + 1:stride, :]
            if depthwise:
                total += win * b[kh, kw, :, 0]
            else:
                total += (win.reshape(-1, C) @ b[kh, kw]).reshape(N, OH, OW, Cout)
    return total


@pytest.mark.parametrize("case", _layers(), ids=_id)
def test_network_layer_exact_table_whole_output(pkg, case):
    net, xs, fs, stride, depthwise = case
    print("layer", _id(case), flush=True)
    from tf_approximate_amd import ops
    xd, fd = bench.device_tensors(pkg, xs, fs, "halfnormal" if xs[3] >= 256 else "uniform", seed=sum(xs) + sum(fs) + 1)
    op = pkg.ApproxConv2DWithMinMaxVars([1, stride, stride, 1], 8, pkg.synth.table_exact(), "SAME", depthwise=depthwise)
    acc = op.accumulators(xd, fd, *MM)
    dims = ops.conv2d_geometry(op._desc(xd, fd))
    qa = ops.quantize(xd, MM[0], MM[1])
    qb = ops.quantize(fd, MM[2], MM[3])
    zp = ops.quant_props(*MM).input_zero_code
    want = exact_conv_of_codes(qa, qb, zp, (int(dims.out_rows), int(dims.out_cols), int(dims.pad_rows_before),
                                            int(dims.pad_cols_before)), stride, depthwise)
    assert acc.shape == want.shape
    bad = (acc.double() != want)
    assert not bool(bad.any()), "%d of %d sums differ, first at %s" % (
        int(bad.sum()), bad.numel(), tuple(int(v) for v in bad.nonzero()[0]))
