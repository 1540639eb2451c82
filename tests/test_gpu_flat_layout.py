"""Layers whose channel count is no multiple of four run on a flat layout of the quantized input: the codes of a
row of pixels lie one after the other (horizontal padding written out), the KW * C codes under one filter row are cut
into quads as one run, and the kernels read their activation dwords at byte granularity.  Every case checks, from the
library's kernel timers, that this layout was used, and compares whole outputs with the oracle."""
import numpy as np
import pytest
import torch

import gpu_util
import refimpl

pytestmark = pytest.mark.gpu

MM = (-1.0, 1.0, -0.5, 0.5)

CASES = [
    # input, filter, strides, dilations, padding
    ((2, 20, 23, 3), (7, 7, 3, 16), (2, 2), (1, 1), "SAME"),     # a stem: 21 codes per filter row in 6 quads
    ((1, 9, 40, 1), (3, 5, 1, 8), (1, 1), (1, 1), "SAME"),       # one channel
    ((2, 11, 13, 2), (3, 3, 2, 20), (1, 2), (2, 1), "VALID"),    # two channels, rows dilated, columns strided
    ((3, 8, 9, 5), (2, 4, 5, 33), (1, 1), (1, 1), "SAME"),       # even filter width: more padding right than left
    ((1, 6, 30, 5), (1, 3, 5, 16), (1, 3), (1, 1), "SAME"),      # stride 3 along the row
    ((2, 7, 7, 3), (5, 5, 3, 64), (1, 1), (1, 1), "SAME"),       # small image under a wide filter
    ((1, 5, 5, 3), (7, 7, 3, 8), (1, 1), (1, 1), "SAME"),        # filter larger than the image
    ((1, 6, 6, 3), (7, 7, 3, 16), (1, 1), (1, 1), "SAME"),       # few pixels, long K: split over tiles
    ((5, 30, 30, 3), (7, 7, 3, 64), (2, 2), (1, 1), "SAME"),     # several row tiles
    ((2, 12, 12, 6), (3, 3, 6, 24), (1, 1), (1, 1), "SAME"),     # 18 codes per row in 5 quads (6 as quads per pixel)
]


def _ran_flat(prof):
    """The float entry points time their patch sums under a name of its own on this layout (they write the rows too
    where the band of input rows fits the LDS); the other entry points run the pass that only writes the rows."""
    return "patch_sums_flat" in prof or "quantize_flat_rows" in prof


@pytest.fixture()
def timers(pkg):
    from tf_approximate_amd import ops
    ops.profile_enable(True)
    ops.profile_reset()
    yield ops
    ops.profile_enable(False)


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_flat_layout_vs_oracle(pkg, oracle, timers, case):
    xs, fs, strides, dil, padding = case
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=len(str(case)))
    table = pkg.synth.table_random(4) if xs[0] % 2 else pkg.synth.table_asymmetric()
    y, acc = gpu_util.run_op(pkg, table, x, f, MM, strides, padding, dil)
    assert _ran_flat(timers.profile_read()), case
    rc, y_ref, acc_ref = oracle.conv2d_fast(table, x, f, *MM, strides=strides, padding=padding, dilations=dil, threads=8)
    assert rc == 0
    assert np.array_equal(acc, acc_ref), case
    assert refimpl.linf_rel(y, y_ref) <= 1e-5, case


def test_flat_layout_with_zero_point_that_is_not_zero_code(pkg, oracle, timers):
    """Input range [0, max]: the padding bytes hold code 0, and a table with T[0][b] != 0 makes them count."""
    xs, fs = (2, 10, 11, 3), (5, 5, 3, 16)
    mm = (0.0, 2.0, -0.5, 0.5)
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, mm, seed=5)
    table = pkg.synth.table_random(12)
    y, acc = gpu_util.run_op(pkg, table, x, f, mm, (1, 1), "SAME")
    assert _ran_flat(timers.profile_read())
    rc, y_ref, acc_ref = oracle.conv2d_fast(table, x, f, *mm, strides=(1, 1), padding="SAME")
    assert rc == 0 and np.array_equal(acc, acc_ref)
    assert refimpl.linf_rel(y, y_ref) <= 1e-5


def test_layer_and_codes_entry_points_on_the_flat_layout(pkg, oracle, timers):
    from tf_approximate_amd import ops
    rng = np.random.default_rng(31)
    # the layer call: per-batch min/max, fake quantization inside the flat quantize pass, bias, ReLU
    xs, fs = (2, 19, 17, 3), (7, 7, 3, 24)
    x = rng.uniform(-1.5, 2.0, size=xs).astype(np.float32)
    w = (rng.standard_normal(fs) * 0.2).astype(np.float32)
    bias = rng.uniform(-1, 1, size=fs[3]).astype(np.float32)
    table = pkg.synth.table_noisy(3)
    dev = gpu_util.dev()
    layer = pkg.FakeApproxConv2D((2, 2), table, "SAME", activation="relu")
    y = layer(torch.from_numpy(x).to(dev), torch.from_numpy(w).to(dev), torch.from_numpy(bias).to(dev)).cpu().numpy()
    assert _ran_flat(timers.profile_read())
    r = (float(x.min()), float(x.max()), float(w.min()), float(w.max()))
    fq = pkg.fake_quant.fake_quant_with_min_max_vars
    rc, y_ref, _ = oracle.conv2d_fast(table, fq(x, r[0], r[1]), fq(w, r[2], r[3]), *r, strides=(2, 2), padding="SAME")
    assert rc == 0
    assert refimpl.linf_rel(y, np.maximum((y_ref + bias).astype(np.float32), 0.0)) <= 1e-5
    # uint8 codes in, int32 sums out
    table_np = pkg.synth.table_random(21)
    xs, fs, strides, padding, zp = (2, 9, 8, 5), (3, 3, 5, 11), (1, 1), "SAME", 17
    qa = rng.integers(0, 256, xs).astype(np.uint8)
    qb = rng.integers(0, 256, fs).astype(np.uint8)
    timers.profile_reset()
    acc = ops.conv2d_codes_acc_i32(pkg.TruthTable(table_np), torch.from_numpy(qa).to(dev), torch.from_numpy(qb).to(dev),
                                   zp, (1, 1, 1, 1), padding).cpu().numpy()
    assert _ran_flat(timers.profile_read())
    patches = refimpl.gather_patches(qa, zp, fs[0], fs[1], strides, padding, (1, 1))
    n, oh, ow = patches.shape[:3]
    want = oracle.lut_gemm_codes(table_np, patches.reshape(n * oh * ow, -1), qb.reshape(-1, fs[3]))
    assert np.array_equal(acc.reshape(n * oh * ow, fs[3]), want)


def test_stem_runs_flat_and_out_of_preexpanded_rows(pkg, timers):
    """The ResNet-50 stem at batch 32: 7 taps x 6 quads, an even count, so the planner can pre-expand its rows; a dilated
    row filter cannot use the flat layout."""
    table = pkg.synth.table_random(2)
    dev = gpu_util.dev()
    x = torch.zeros((32, 224, 224, 3), dtype=torch.float32, device=dev)
    f = torch.zeros((7, 7, 3, 64), dtype=torch.float32, device=dev)
    op = pkg.ApproxConv2DWithMinMaxVars([1, 2, 2, 1], 8, table, "SAME")
    op(x, f, *MM)
    torch.cuda.synchronize()
    prof = timers.profile_read()
    assert _ran_flat(prof) and "quantize_flat_rows" not in prof and "lutgemm_px" in prof
    timers.profile_reset()
    op = pkg.ApproxConv2DWithMinMaxVars([1, 1, 1, 1], 8, table, "SAME", dilations=[1, 1, 2, 1])
    op(torch.zeros((4, 40, 40, 3), dtype=torch.float32, device=dev), f, *MM)
    torch.cuda.synchronize()
    assert not _ran_flat(timers.profile_read())
