"""The LUT-GEMM kernel that reads pre-expanded rows without a barrier between fills (lutgemm_pxf_kernel in
tf-approximate_amd/csrc/lutgemm_px_kernel.hip): its wavefronts are held together by two LDS counters only.

The planner picks it for tiles of 16 to 63 wavefront-rows with 16 fills or more (32 for a 1x1 filter), so the cases
here are full-size layers, each asserted to get that kernel (tile plan code 2).  Every case is checked three ways:
the whole tensor of int32 sums and the whole float output bit for bit against the kernel that expands inside its tiles
(itself pinned against the oracle by the per-layer tests), sampled pixels against the CPU oracle, and, where torch can
restate the layer, the whole tensor of sums with the exact table against an fp64 convolution of the codes.  Shapes
cover even and odd fill counts (a tile that starts in LDS buffer 1), a K split, ragged last row tiles, a column count
that is no multiple of 16, stride, dilation, the flat 7x7x3 layout, both paddings, tiles of every row count the
kernel divides differently between its wavefronts, and a layer whose pre-expanded rows
(1.2 GB) are larger than any cache.  The last test forces the kernel's
bounded waits to run out and checks the report."""
import numpy as np
import pytest
import torch

import bench
import gpu_util
import refimpl
from test_gpu_networks import exact_conv_of_codes

pytestmark = pytest.mark.gpu

MM = (-1.0, 1.0, -0.5, 0.5)

CASES = [
    # input, filter, stride, dilation, padding
    ((16, 64, 64, 16), (3, 3, 16, 64), 1, 1, "SAME"),       # 18 fills, 16 wavefront-rows per tile (the smallest)
    ((33, 57, 55, 24), (3, 3, 24, 64), 1, 1, "SAME"),       # 27 fills (odd): every other tile starts in buffer 1; ragged
    ((33, 57, 55, 24), (3, 3, 24, 64), 1, 1, "VALID"),
    ((32, 112, 112, 16), (3, 3, 16, 40), 2, 1, "SAME"),     # stride 2, 40 columns: a column tile of 8
    ((16, 64, 64, 16), (3, 3, 16, 64), 1, 2, "SAME"),       # dilation 2
    ((20, 61, 67, 32), (3, 3, 32, 72), 1, 1, "VALID"),      # five column tiles (two blocks of the tile order), ragged
    ((32, 56, 56, 64), (3, 3, 64, 20), 1, 1, "SAME"),       # K split in four, 18 fills each
    ((16, 64, 64, 264), (1, 1, 264, 64), 1, 1, "SAME"),     # 1x1, 33 fills (odd)
    ((64, 112, 112, 3), (7, 7, 3, 64), 2, 1, "VALID"),      # flat layout of a 3-channel input, 44-row tiles
    ((32, 28, 28, 512), (3, 3, 512, 512), 1, 1, "SAME"),    # 1.2 GB of rows: read from memory, not from a cache
]
# tiles of 29 to 48 wavefront-rows, which the kernel divides between its older and younger wavefronts by a rule of its
# own (a second instantiation): 31 rows (20 + 11), 36 (20 + 16; also under a K split), 37 (24 + 13) with a ragged last tile
# of 19, 47 (28 + 19);
# the 7x7 stem above has 44 (28 + 16)
OWN_SPLIT_CASES = [
    ((64, 31, 64, 16), (3, 3, 16, 64), 1, 1, "SAME"),
    ((64, 36, 64, 16), (3, 3, 16, 64), 1, 1, "SAME"),
    ((31, 77, 63, 16), (3, 3, 16, 64), 1, 1, "SAME"),
    ((64, 47, 64, 16), (3, 3, 16, 64), 1, 1, "SAME"),
    ((64, 36, 64, 64), (3, 3, 64, 16), 1, 1, "SAME"),   # 36-row tiles with K split in four
]
CASES += OWN_SPLIT_CASES


def _id(case):
    xs, fs, stride, dil, padding = case
    return "%dx%dx%dx%d-%dx%d-to%d-s%d-d%d-%s" % (xs + (fs[0], fs[1], fs[3], stride, dil, padding))


def _plan(pkg, case):
    xs, fs, stride, dil, padding = case
    return pkg.ops.conv2d_tile_plan(xs, fs, (1, stride, stride, 1), padding, (1, dil, dil, 1))


def test_own_split_cases_have_such_tiles(pkg):
    rows = [_plan(pkg, case)["rows_per_tile"] // 64 for case in OWN_SPLIT_CASES]
    assert rows == [31, 36, 37, 47, 36], rows
    assert _plan(pkg, OWN_SPLIT_CASES[4])["k_splits"] == 4


@pytest.mark.parametrize("case", CASES, ids=_id)
def test_barrier_free_kernel_whole_output_and_oracle(pkg, oracle, case):
    print("case", _id(case), flush=True)
    xs, fs, stride, dil, padding = case
    ops = pkg.ops
    plan = _plan(pkg, case)
    assert plan["preexpanded_rows"] == 2, plan
    table = pkg.synth.table_random(sum(xs) + fs[3])
    xd, fd = bench.device_tensors(pkg, xs, fs, "uniform", seed=sum(xs) + 3 * sum(fs))
    op = pkg.ApproxConv2DWithMinMaxVars([1, stride, stride, 1], 8, table, padding, dilations=[1, dil, dil, 1])
    ops.profile_enable(True)
    ops.profile_reset()
    try:
        y = op(xd, fd, *MM)
        acc = op.accumulators(xd, fd, *MM)
        torch.cuda.synchronize()
        prof = ops.profile_read()
        assert "lutgemm_px" in prof and "lutgemm_expand" not in prof, prof
        # rows beyond 512 MiB get a launch of their own, the others ride in a pre-pass launch
        assert ("px_expand_rows" in prof) == (fs[3] * fs[0] * fs[1] * xs[3] * 512 > 512 << 20), prof   # 512 bytes per filter element
        ops.set_preexpand(-1)
        ops.profile_reset()
        y0 = op(xd, fd, *MM)
        acc0 = op.accumulators(xd, fd, *MM)
        torch.cuda.synchronize()
        assert "lutgemm_px" not in ops.profile_read()
    finally:
        ops.set_preexpand(0)
        ops.profile_enable(False)
    bad = acc != acc0
    assert not bool(bad.any()), "%d of %d sums differ from the other kernel's, first at %s" % (
        int(bad.sum()), bad.numel(), tuple(int(v) for v in bad.nonzero()[0]))
    assert torch.equal(y.view(torch.int32), y0.view(torch.int32))
    if dil == 1:
        exact, linf = bench.sampled_oracle_check(oracle, table, op, xd, fd, (stride, stride), False, y,
                                                 n_samples=12, seed=len(_id(case)))
        assert exact, "int32 accumulators differ from the oracle on sampled pixels"
        assert linf <= 1e-5
        op_exact = pkg.ApproxConv2DWithMinMaxVars([1, stride, stride, 1], 8, pkg.synth.table_exact(), padding)
        acc = op_exact.accumulators(xd, fd, *MM)
        dims = ops.conv2d_geometry(op_exact._desc(xd, fd))
        want = exact_conv_of_codes(ops.quantize(xd, MM[0], MM[1]), ops.quantize(fd, MM[2], MM[3]),
                                   ops.quant_props(*MM).input_zero_code,
                                   (int(dims.out_rows), int(dims.out_cols), int(dims.pad_rows_before),
                                    int(dims.pad_cols_before)), stride, False)
        bad = acc.double() != want
        assert not bool(bad.any()), "%d of %d exact sums differ, first at %s" % (
            int(bad.sum()), bad.numel(), tuple(int(v) for v in bad.nonzero()[0]))


def _random_layers(pkg, count, seed):
    """Seeded random layers that the planner gives to the kernel (plan code 2)."""
    ops = pkg.ops
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        k = int(rng.choice([1, 3, 3, 5]))
        c = int(rng.choice([16, 24, 32, 48, 64, 96, 128]))
        co = int(rng.integers(1, 13)) * int(rng.choice([8, 16, 20]))
        xs = (int(rng.integers(8, 49)), int(rng.integers(20, 70)), int(rng.integers(20, 70)), c)
        stride, padding = int(rng.choice([1, 1, 2])), str(rng.choice(["SAME", "VALID"]))
        if xs[0] * xs[1] * xs[2] * max(c, co) > 30e6:
            continue
        case = (xs, (k, k, c, co), stride, 1, padding)
        plan = ops.conv2d_tile_plan(xs, case[1], (1, stride, stride, 1), padding, (1, 1, 1, 1))
        if plan["preexpanded_rows"] == 2:
            out.append(case)
    return out


def test_random_full_size_layers_equal_the_expanding_kernel(pkg):
    """Ninety-six seeded random layers (tile heights, K splits, strides, paddings as the planner makes them): whole sums
    and whole float outputs bit for bit against the kernel that expands inside its tiles."""
    ops = pkg.ops
    heights = set()
    for i, case in enumerate(_random_layers(pkg, 96, seed=2024)):
        print("case", _id(case), flush=True)
        xs, fs, stride, dil, padding = case
        heights.add(_plan(pkg, case)["rows_per_tile"] // 64)
        table = pkg.synth.table_random(i)
        xd, fd = bench.device_tensors(pkg, xs, fs, "uniform", seed=i)
        op = pkg.ApproxConv2DWithMinMaxVars([1, stride, stride, 1], 8, table, padding)
        try:
            acc, y = op.accumulators(xd, fd, *MM), op(xd, fd, *MM)
            ops.set_preexpand(-1)
            acc0, y0 = op.accumulators(xd, fd, *MM), op(xd, fd, *MM)
        finally:
            ops.set_preexpand(0)
        assert torch.equal(acc, acc0), _id(case)
        assert torch.equal(y.view(torch.int32), y0.view(torch.int32)), _id(case)
    assert len(heights) >= 24, heights


def test_dilated_case_against_the_oracle_on_a_crop(pkg, oracle):
    """The dilated case above only compares the two kernels; here the oracle recomputes one whole image of it."""
    xs, fs, stride, dil, padding = CASES[4]
    assert dil == 2 and _plan(pkg, CASES[4])["preexpanded_rows"] == 2
    table = pkg.synth.table_noisy(9)
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=12)
    y, acc = gpu_util.run_op(pkg, table, x, f, MM, (stride, stride), padding, (dil, dil))
    for n in (0, xs[0] - 1):
        rc, y_ref, acc_ref = oracle.conv2d_fast(table, x[n:n + 1], f, *MM, strides=(stride, stride), padding=padding,
                                                dilations=(dil, dil))
        assert rc == 0
        assert np.array_equal(acc[n:n + 1], acc_ref)
        assert refimpl.linf_rel(y[n:n + 1], y_ref) <= 1e-5


def test_layer_entry_point_on_the_barrier_free_kernel(pkg, oracle):
    """Per-batch min/max, fake quantization, bias and ReLU around the kernel, against the oracle on the first image."""
    rng = np.random.default_rng(5)
    xs, fs = (16, 64, 64, 16), (3, 3, 16, 64)
    assert _plan(pkg, (xs, fs, 1, 1, "SAME"))["preexpanded_rows"] == 2
    x = rng.uniform(-2.0, 1.0, size=xs).astype(np.float32)
    w = (rng.standard_normal(fs) * 0.3).astype(np.float32)
    bias = rng.uniform(-1, 1, size=fs[3]).astype(np.float32)
    table = pkg.synth.table_noisy(5)
    dev = gpu_util.dev()
    layer = pkg.FakeApproxConv2D((1, 1), table, "SAME", activation="relu")
    y = layer(torch.from_numpy(x).to(dev), torch.from_numpy(w).to(dev), torch.from_numpy(bias).to(dev)).cpu().numpy()
    r = (float(x.min()), float(x.max()), float(w.min()), float(w.max()))
    fq = pkg.fake_quant.fake_quant_with_min_max_vars
    rc, y_ref, _ = oracle.conv2d_fast(table, fq(x[:1], r[0], r[1]), fq(w, r[2], r[3]), *r, strides=(1, 1),
                                      padding="SAME")
    assert rc == 0
    y_ref = np.maximum((y_ref + bias).astype(np.float32), 0.0)
    assert refimpl.linf_rel(y[:1], y_ref) <= 1e-5


def test_a_wait_that_runs_out_is_reported_by_the_next_call(pkg):
    """With a wait limit of zero polls the first wavefront to look at a counter before its time gives up, the others
    follow when they next wait, and every wavefront leaves the kernel.  The launch itself returns as usual (it is
    asynchronous); the next call on the device reports it, once; with the limit restored the layer is right again."""
    case = CASES[0]
    xs, fs, stride, dil, padding = case
    ops = pkg.ops
    assert _plan(pkg, case)["preexpanded_rows"] == 2
    table = pkg.synth.table_random(2)
    xd, fd = bench.device_tensors(pkg, xs, fs, "uniform", seed=1)
    op = pkg.ApproxConv2DWithMinMaxVars([1, stride, stride, 1], 8, table, padding)
    good = op.accumulators(xd, fd, *MM).clone()
    torch.cuda.synchronize()
    ops.set_wait_limit(0)
    try:
        print("launch with a wait limit of 0 polls", flush=True)
        op.accumulators(xd, fd, *MM)
        torch.cuda.synchronize()
    finally:
        ops.set_wait_limit(1 << 20)
    with pytest.raises(RuntimeError, match="gave up a wait"):
        op.accumulators(xd, fd, *MM)
    again = op.accumulators(xd, fd, *MM)      # reported once
    torch.cuda.synchronize()
    assert torch.equal(again, good)
