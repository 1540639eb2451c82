"""Full-size layers (the ResNet-50-shaped and the large GEMM-dominated benchmark layers): too large for the CPU oracle to recompute whole,
so checked through size-independent properties and through oracle evaluation of sampled output pixels."""
import numpy as np
import pytest
import torch

import gpu_util
import refimpl

pytestmark = pytest.mark.gpu

MM = (-1.0, 1.0, -0.5, 0.5)


def _sampled_rows_check(pkg, oracle, table, x, f, mm, strides, acc, y, n_samples, seed):
    """Oracle LUT-GEMM + epilogue on randomly chosen output pixels (patches gathered with numpy)."""
    KH, KW, C, Co = f.shape
    N, OH, OW, _ = acc.shape
    rng = np.random.default_rng(seed)
    qp = oracle.quant_props(*mm)
    qa = oracle.quantize(x, qp.in_offset, qp.in_inv_scale)
    qb = oracle.quantize(f, qp.f_offset, qp.f_inv_scale).reshape(-1, Co)
    zp = int(oracle.quantize(np.zeros(1, np.float32), qp.in_offset, qp.in_inv_scale)[0])
    _, ph = refimpl.same_or_valid_geometry(x.shape[1], KH, strides[0], 1, "SAME")
    _, pw = refimpl.same_or_valid_geometry(x.shape[2], KW, strides[1], 1, "SAME")
    picks = [(0, 0, 0), (N - 1, OH - 1, OW - 1), (0, 0, OW - 1), (N - 1, OH - 1, 0)]
    picks += [(int(rng.integers(N)), int(rng.integers(OH)), int(rng.integers(OW))) for _ in range(n_samples)]
    patches = np.full((len(picks), KH, KW, C), zp, np.uint8)
    psum = np.zeros(len(picks), np.float32)
    for i, (n, oh, ow) in enumerate(picks):
        s = np.float32(0)
        for kh in range(KH):
            for kw in range(KW):
                ih, iw = oh * strides[0] - ph + kh, ow * strides[1] - pw + kw
                if 0 <= ih < x.shape[1] and 0 <= iw < x.shape[2]:
                    patches[i, kh, kw] = qa[n, ih, iw]
                    for v in x[n, ih, iw]:
                        s = np.float32(s + v)
        psum[i] = s
    want = oracle.lut_gemm_codes(table, patches.reshape(len(picks), -1), qb)
    got = np.stack([acc[n, oh, ow] for n, oh, ow in picks])
    assert np.array_equal(got, want)
    fsum = np.zeros(Co, np.float32)
    for row in f.reshape(-1, Co):
        fsum = (fsum + row).astype(np.float32)
    K = KH * KW * C
    f32 = np.float32
    out = (want.astype(f32) * f32(qp.s1xs2)).astype(f32) + (f32(qp.m2) * psum)[:, None].astype(f32)
    out = (out.astype(f32) + (f32(qp.m1) * fsum)[None, :].astype(f32)).astype(f32)
    out = (out - f32(f32(K) * f32(qp.m1xm2))).astype(f32)
    got_y = np.stack([y[n, oh, ow] for n, oh, ow in picks])
    assert refimpl.linf_rel(got_y, out) <= 1e-5


@pytest.fixture(scope="module")
def north_star(pkg):
    return pkg.synth.north_star_layer(seed=3)


def test_north_star_layer_sampled_pixels(pkg, oracle, north_star):
    table = pkg.synth.table_uniform_error(11)
    y, acc = gpu_util.run_op(pkg, table, north_star["x"], north_star["f"], north_star["minmax"])
    assert acc.shape == (64, 56, 56, 64)
    _sampled_rows_check(pkg, oracle, table, north_star["x"], north_star["f"], north_star["minmax"], (1, 1),
                        acc, y, n_samples=60, seed=1)


def test_north_star_layer_exact_table_is_integer_conv(pkg, north_star):
    """With the exact table the sums are the integer convolution of the codes; checked against an fp64
    matmul of the zero-point-padded im2col matrix on the GPU (exact: all values are integers < 2^53)."""
    from tf_approximate_amd import ops
    x, f, mm = north_star["x"], north_star["f"], north_star["minmax"]
    _, acc = gpu_util.run_op(pkg, pkg.synth.table_exact(), x, f, mm)
    d = gpu_util.dev()
    qa = ops.quantize(torch.from_numpy(x).to(d), mm[0], mm[1]).double()
    qb = ops.quantize(torch.from_numpy(f).to(d), mm[2], mm[3]).double().reshape(-1, 64)
    zp = float(ops.quant_props(*mm).input_zero_code)
    qa_p = torch.nn.functional.pad(qa.permute(0, 3, 1, 2), (1, 1, 1, 1), value=zp)         # N,C,H+2,W+2
    total = torch.zeros((64, 56, 56, 64), dtype=torch.float64, device=d)
    for kh in range(3):
        for kw in range(3):
            a = qa_p[:, :, kh:kh + 56, kw:kw + 56].permute(0, 2, 3, 1).reshape(-1, 64)
            b = qb[(kh * 3 + kw) * 64:(kh * 3 + kw + 1) * 64]
            total += (a @ b).reshape(64, 56, 56, 64)
    assert torch.equal(total.cpu(), torch.from_numpy(acc).double())


def test_north_star_layer_table_plus_one_identity(pkg, north_star):
    """acc[T + 1] - acc[T] == K for every output, padding taps included (they are looked up, not skipped)."""
    base = pkg.synth.table_truncated(4)
    plus1 = (base.astype(np.int64) + 1).astype(np.uint16)
    _, acc0 = gpu_util.run_op(pkg, base, north_star["x"], north_star["f"], north_star["minmax"])
    _, acc1 = gpu_util.run_op(pkg, plus1, north_star["x"], north_star["f"], north_star["minmax"])
    assert np.array_equal(acc1 - acc0, np.full(acc0.shape, 576, np.int32))


def test_north_star_layer_is_deterministic(pkg, north_star):
    table = pkg.synth.table_random(13)
    y0, acc0 = gpu_util.run_op(pkg, table, north_star["x"], north_star["f"], north_star["minmax"])
    y1, acc1 = gpu_util.run_op(pkg, table, north_star["x"], north_star["f"], north_star["minmax"])
    assert np.array_equal(acc0, acc1) and np.array_equal(y0, y1)


@pytest.mark.parametrize("name", ["A_1x1_256_1024", "B_3x3_512_512", "stem_7x7", "stage4_3x3", "reduce_1x1_256_64"])
@pytest.mark.parametrize("tname", ["random", "exact"])
def test_stress_layers_sampled_pixels(pkg, oracle, name, tname):
    """The large GEMM-dominated stress layers (A: 1x1 32x56x56x256->1024; B: 3x3 64x28x28x512->512, K = 4608) and the
    ResNet-50 stem / stage-4 shapes, half-normal activation codes, fully random and exact tables."""
    shapes = {
        "A_1x1_256_1024": ((32, 56, 56, 256), (1, 1, 256, 1024), (1, 1)),
        "B_3x3_512_512": ((64, 28, 28, 512), (3, 3, 512, 512), (1, 1)),
        "stem_7x7": ((16, 224, 224, 3), (7, 7, 3, 64), (2, 2)),
        "stage4_3x3": ((64, 7, 7, 512), (3, 3, 512, 512), (1, 1)),
        "reduce_1x1_256_64": ((64, 56, 56, 256), (1, 1, 256, 64), (1, 1)),   # flat pre-pass, 256 pixels per workgroup
    }
    xs, fs, strides = shapes[name]
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=len(name), codes="halfnormal")
    table = pkg.synth.table_random(13) if tname == "random" else pkg.synth.table_exact()
    y, acc = gpu_util.run_op(pkg, table, x, f, MM, strides)
    _sampled_rows_check(pkg, oracle, table, x, f, MM, strides, acc, y, n_samples=24, seed=2)


@pytest.mark.parametrize("stride", [1, 2])
def test_depthwise_benchmark_shape_vs_oracle(pkg, oracle, stride):
    """The depthwise benchmark layer's geometry (3x3 over 112x112x192, both strides) at batch 4, whole output against
    the oracle: the runs of 32 / 16 output pixels per thread, the image borders and all three channel groups."""
    xs, fs = (4, 112, 112, 192), (3, 3, 192, 1)
    x, f, _, _ = refimpl.grid_case(pkg, xs, fs, MM, seed=31 + stride)
    x = x + np.float32(0.0017)          # off the quantization grid: patch sums differ from the dequantized codes
    table = pkg.synth.table_random(17)
    y, acc = gpu_util.run_op(pkg, table, x, f, MM, (stride, stride), depthwise=True)
    rc, y_ref, acc_ref = oracle.depthwise_conv2d(table, x, f, *MM, strides=(stride, stride), padding="SAME",
                                                  dilations=(1, 1))
    assert rc == 0
    assert np.array_equal(acc, acc_ref)
    assert np.max(np.abs(y - y_ref)) <= 1e-5 * max(np.max(np.abs(y_ref)), 1e-30)


def test_lds_probes_report_plausible_rates(pkg):
    """The two measured ceilings of the bench line: the per-entry gather rate and the streaming 16-byte read rate.
    A 16-byte read moves 8 entries, so the read port in entries/s must come out well above the gather rate."""
    gather = pkg.ops.lds_gather_peak()
    port = pkg.ops.lds_read_peak()
    assert 1e12 < gather < 1e14
    assert port / 2.0 > 2.0 * gather
