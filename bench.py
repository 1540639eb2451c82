#!/usr/bin/env python3
"""Benchmark of the ApproxConv2DWithMinMaxVars hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

One step = one full invocation of the op (input quantize/relayout, patch sums, filter pack, LUT-GEMM with
fused epilogue) on seeded synthetic tensors that are already resident in HBM.  Prints ONE JSON line.

  value        approximate GMAC/s of the whole op (1 MAC = 1 truth-table lookup) on the headline layer, wall clock
               over K steps
  roofline     the LUT-GEMM kernel alone: algorithmic lookups per launch / its mean launch duration (HIP events on
               the launch stream, recorded inside the library), as a fraction of the two ceilings that can bind it:
               the LDS read port (a lookup moves its 2-byte entry through it) and the issue rate of the kernel's
               accumulate instructions, each the larger of its nominal value (CUs x 256 B x clock, CUs x 64 lanes x
               clock) and what a probe kernel measures in this run.  `frac` is the larger of the two fractions,
               `peak` the ceiling it belongs to; `frac_nominal_gather` is the same rate against the nominal
               one-entry-per-bank-slot gather ceiling 256 CU x 32 lookups/clk x 2.4 GHz = 19.66 T/s.
  layers       the same measurement for the layer shapes of the other benchmark configurations (fewer steps each),
               every one with an oracle check of sampled output pixels; depthwise layers against HBM bandwidth
  networks     images/s of the two synthetic ResNet-shaped networks, every convolution through the op
  cpu_baseline the CPU oracle's reference-faithful single-thread path timed on this host on a bounded sample
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

NOMINAL_LDS_LOOKUPS_PER_S = 256 * 32 * 2.4e9
HBM_PEAK_GBPS = 8000.0
PREROLL_S = 0.3
MM = (-1.0, 1.0, -0.5, 0.5)

WORKLOADS = {
    # name: (x_shape, f_shape, strides, depthwise)
    "conv3x3_b64_56x56x64_to_64_s1_same": ((64, 56, 56, 64), (3, 3, 64, 64), (1, 1), False),
    "conv1x1_b32_56x56x256_to_1024": ((32, 56, 56, 256), (1, 1, 256, 1024), (1, 1), False),
    "conv3x3_b64_28x28x512_to_512": ((64, 28, 28, 512), (3, 3, 512, 512), (1, 1), False),
    "conv7x7s2_b64_224x224x3_to_64": ((64, 224, 224, 3), (7, 7, 3, 64), (2, 2), False),
    "conv1x1_b64_112x112x32_to_192": ((64, 112, 112, 32), (1, 1, 32, 192), (1, 1), False),
    "conv1x1_b64_112x112x192_to_32": ((64, 112, 112, 192), (1, 1, 192, 32), (1, 1), False),
    "conv1x1_b64_56x56x64_to_256": ((64, 56, 56, 64), (1, 1, 64, 256), (1, 1), False),
    "dw3x3_b64_112x112x192_s1": ((64, 112, 112, 192), (3, 3, 192, 1), (1, 1), True),
    "dw3x3_b64_112x112x192_s2": ((64, 112, 112, 192), (3, 3, 192, 1), (2, 2), True),
    "conv3x3_b128_32x32x16_to_16": ((128, 32, 32, 16), (3, 3, 16, 16), (1, 1), False),
    "conv3x3_b64_28x28x128_to_128": ((64, 28, 28, 128), (3, 3, 128, 128), (1, 1), False),   # K cut in two, pre-expanded rows
    "conv3x3_b64_7x7x512_to_512": ((64, 7, 7, 512), (3, 3, 512, 512), (1, 1), False),       # K cut over tiles, rows expanded in the tiles
}
DEFAULT = "conv3x3_b64_56x56x64_to_64_s1_same"

# The layer shapes of the other benchmark configurations, reported in the `layers` array.
# (config, layer, x_shape, f_shape, strides, depthwise, activation codes, table)
LAYERS = [
    ("cfg2_cifar_resnet", "stem_3x3_3_16", (128, 32, 32, 3), (3, 3, 3, 16), (1, 1), False, "uniform", "noisy"),
    ("cfg2_cifar_resnet", "conv3x3_16_16", (128, 32, 32, 16), (3, 3, 16, 16), (1, 1), False, "uniform", "noisy"),
    ("cfg2_cifar_resnet", "conv3x3_32_32", (128, 16, 16, 32), (3, 3, 32, 32), (1, 1), False, "uniform", "noisy"),
    ("cfg2_cifar_resnet", "conv3x3_64_64", (128, 8, 8, 64), (3, 3, 64, 64), (1, 1), False, "uniform", "noisy"),
    ("cfg3_inverted_residual", "expand_1x1_32_192", (64, 112, 112, 32), (1, 1, 32, 192), (1, 1), False, "uniform", "trunc2"),
    ("cfg3_inverted_residual", "dw3x3_192_s1", (64, 112, 112, 192), (3, 3, 192, 1), (1, 1), True, "uniform", "trunc4"),
    ("cfg3_inverted_residual", "dw3x3_192_s2", (64, 112, 112, 192), (3, 3, 192, 1), (2, 2), True, "uniform", "trunc2"),
    # a depthwise filter that is not 3x3 runs the generic kernel (whole table in LDS, one-entry gathers)
    ("cfg3_inverted_residual", "dw5x5_192_s1_generic", (64, 56, 56, 192), (5, 5, 192, 1), (1, 1), True, "uniform", "trunc4"),
    ("cfg3_inverted_residual", "project_1x1_192_32", (64, 112, 112, 192), (1, 1, 192, 32), (1, 1), False, "uniform", "trunc4"),
    ("cfg4_resnet50", "stem_7x7s2_3_64", (64, 224, 224, 3), (7, 7, 3, 64), (2, 2), False, "uniform", "uniform_error"),
    ("cfg4_resnet50", "stage1_1x1_64_256", (64, 56, 56, 64), (1, 1, 64, 256), (1, 1), False, "uniform", "uniform_error"),
    ("cfg4_resnet50", "stage1_1x1_256_64", (64, 56, 56, 256), (1, 1, 256, 64), (1, 1), False, "uniform", "uniform_error"),
    ("cfg4_resnet50", "stage2_3x3_128_128", (64, 28, 28, 128), (3, 3, 128, 128), (1, 1), False, "uniform", "uniform_error"),
    ("cfg4_resnet50", "stage2_1x1s2_256_512", (64, 56, 56, 256), (1, 1, 256, 512), (2, 2), False, "uniform", "uniform_error"),
    ("cfg4_resnet50", "stage3_3x3_256_256", (64, 14, 14, 256), (3, 3, 256, 256), (1, 1), False, "uniform", "uniform_error"),
    ("cfg4_resnet50", "stage4_3x3_512_512", (64, 7, 7, 512), (3, 3, 512, 512), (1, 1), False, "uniform", "uniform_error"),
    ("cfg4_resnet50", "stage4_1x1_512_2048", (64, 7, 7, 512), (1, 1, 512, 2048), (1, 1), False, "uniform", "uniform_error"),
    ("cfg5_stress", "A_1x1_256_1024", (32, 56, 56, 256), (1, 1, 256, 1024), (1, 1), False, "halfnormal", "random"),
    ("cfg5_stress", "B_3x3_512_512", (64, 28, 28, 512), (3, 3, 512, 512), (1, 1), False, "halfnormal", "random"),
    ("cfg5_stress", "A_1x1_256_1024", (32, 56, 56, 256), (1, 1, 256, 1024), (1, 1), False, "halfnormal", "exact"),
    ("cfg5_stress", "B_3x3_512_512", (64, 28, 28, 512), (3, 3, 512, 512), (1, 1), False, "halfnormal", "exact"),
]
CPU_SAMPLE_S = 0.5      # single-thread reference sample per `layers` record

# Bytes per launch that the main kernel moves between its L2s and the memory side (Infinity Cache or HBM), from
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, each scaled by what the same counter reads for the
# device copy of known size inside the same run.  Keyed by (workload, kernel); not measured in the run that prints
# them: the bench line says which profile they come from.
PROFILED_TRAFFIC = {
    ("conv3x3_b64_56x56x64_to_64_s1_same", "lutgemm_px"): (2.000 * 81258.0 * 1024 + 1.000 * 64419.8 * 1024,
                                                           "profiles/lutgemm_px_conv3x3_b64_56x56x64.md"),
    ("conv3x3_b64_56x56x64_to_64_s1_same", "lutgemm_expand"): (2.000 * 8312.5 * 1024 + 1.000 * 61656.5 * 1024,
                                                               "profiles/lutgemm_expand_conv3x3_b64_56x56x64.md"),
    ("conv1x1_b64_112x112x32_to_192", "lutgemm_px"): (2.000 * 48266.1 * 1024 + 1.000 * 792178.1 * 1024,
                                                      "profiles/lutgemm_px_conv1x1_b64_112x112x32_to_192.md"),
    ("conv1x1_b64_56x56x64_to_256", "lutgemm_px"): (2.000 * 37216.1 * 1024 + 1.000 * 266473.4 * 1024,
                                                    "profiles/lutgemm_px_conv1x1_b64_56x56x64_to_256.md"),
    ("conv1x1_b32_56x56x256_to_1024", "lutgemm_px"): (2.000 * 471685.9 * 1024 + 1.000 * 470379.1 * 1024,
                                                      "profiles/lutgemm_px_conv1x1_b32_56x56x256_to_1024.md"),
    ("conv7x7s2_b64_224x224x3_to_64", "lutgemm_px"): (2.000 * 94083.4 * 1024 + 1.000 * 244689.7 * 1024,
                                                      "profiles/lutgemm_px_conv7x7s2_b64_224x224x3_to_64.md"),
    ("conv3x3_b64_28x28x512_to_512", "lutgemm_px"): (2.000 * 2065967.7 * 1024 + 1.000 * 106108.0 * 1024,
                                                     "profiles/lutgemm_px_conv3x3_b64_28x28x512_to_512.md"),
    ("conv3x3_b128_32x32x16_to_16", "lutgemm_px"): (2.050 * 6113.0 * 1024 + 1.025 * 8192.0 * 1024,
                                                    "profiles/lutgemm_px_conv3x3_b128_32x32x16_to_16.md"),
    ("conv1x1_b64_112x112x192_to_32", "lutgemm_px"): (2.000 * 101823.7 * 1024 + 1.000 * 130117.9 * 1024,
                                                      "profiles/lutgemm_px_conv1x1_b64_112x112x192_to_32.md"),
    ("conv3x3_b64_28x28x128_to_128", "lutgemm_px"): (2.000 * 130204.7 * 1024 + 1.000 * 54284.1 * 1024,
                                                     "profiles/lutgemm_px_conv3x3_b64_28x28x128_to_128.md"),
    ("conv3x3_b64_7x7x512_to_512", "lutgemm_expand"): (2.000 * 8874.8 * 1024 + 1.000 * 55210.4 * 1024,
                                                       "profiles/lutgemm_expand_conv3x3_b64_7x7x512_to_512.md"),
    ("dw3x3_b64_112x112x192_s1", "depthwise_lut"): (2.000 * 360914 * 1024 + 1.000 * 602112 * 1024,
                                                    "profiles/depthwise_lut3x3_dw3x3_b64_112x112x192.md"),
    ("dw3x3_b64_112x112x192_s2", "depthwise_lut"): (2.000 * 314820 * 1024 + 1.000 * 150528 * 1024,
                                                    "profiles/depthwise_lut3x3_dw3x3_b64_112x112x192.md"),
}


def measured_copy_bandwidth(mib=512, reps=30):
    """Bytes per second (read + written) of a plain device-to-device copy: what HBM sustains for a streaming kernel
    that reads one buffer and writes another, the depthwise kernels' access pattern."""
    import torch
    n = mib * (1 << 20) // 4
    a = torch.ones(n, dtype=torch.float32, device="cuda:0")
    b = torch.empty_like(a)
    for _ in range(10):
        b.copy_(a)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        b.copy_(a)
    torch.cuda.synchronize()
    return 2.0 * n * 4 * reps / (time.perf_counter() - t0)


class Ceilings:
    """The ceilings of the dense kernel: measured once per run by probe kernels of the library, and nominal from the
    device's CU count and clock.  A fraction is taken against the LARGER of the two, so a probe that falls short of
    what the hardware is specified for does not flatter the kernel."""

    def __init__(self, ops):
        self.copy_bytes = measured_copy_bandwidth()
        self.gather = ops.lds_gather_peak()                     # conflict-free ds_read_u16 lookups/s
        self.port_bytes = max(ops.lds_read_peak(), 1.0)         # streaming ds_read_b128 bytes/s
        self.valu_lane_ops = max(ops.valu_issue_peak(), 1.0)    # accumulate-instruction lane operations/s
        self.ops_per_lookup = ops.dense_accumulate_ops_per_lookup()
        self.mix = max(ops.lookup_mix_peak(), 1.0)              # the whole per-lookup instruction mix, lookups/s
        info = ops.device_info()
        self.cus, self.clock_hz = info["compute_units"], info["clock_khz"] * 1e3
        self.valu_nominal = self.cus * 64.0 * self.clock_hz     # 4 SIMDs x 16 lanes per clock and CU
        self.port_nominal = self.cus * 256.0 * self.clock_hz    # 64 banks x 4 bytes per clock and CU

    def fractions(self, lookups_per_s):
        valu_ceiling = max(self.valu_nominal, self.valu_lane_ops)
        port_ceiling = max(self.port_nominal, self.port_bytes)
        f_port = 2.0 * lookups_per_s / port_ceiling
        f_valu = lookups_per_s * self.ops_per_lookup / valu_ceiling
        bound = "lds" if f_port >= f_valu else "valu"
        peak = port_ceiling / 2.0 if bound == "lds" else valu_ceiling / self.ops_per_lookup
        return {"bound": bound, "frac": round(max(f_port, f_valu), 4), "frac_lds_port": round(f_port, 4),
                "frac_valu": round(f_valu, 4),
                "frac_lds_port_measured": round(2.0 * lookups_per_s / self.port_bytes, 4),
                "frac_valu_measured": round(lookups_per_s * self.ops_per_lookup / self.valu_lane_ops, 4),
                "frac_lookup_mix_measured": round(lookups_per_s / self.mix, 4),
                "frac_nominal_gather": round(lookups_per_s / NOMINAL_LDS_LOOKUPS_PER_S, 4)}, peak

    def report(self):
        return {"compute_units": self.cus, "clock_ghz": round(self.clock_hz / 1e9, 3),
                "valu_nominal_glane_ops_per_s": round(self.valu_nominal / 1e9, 1),
                "lds_port_nominal_gbytes_per_s": round(self.port_nominal / 1e9, 1),
                "lds_read_port_gbytes_per_s": round(self.port_bytes / 1e9, 1),
                "lds_read_port_glookups_per_s": round(self.port_bytes / 2e9, 1),
                "valu_accumulate_glane_ops_per_s": round(self.valu_lane_ops / 1e9, 1),
                "valu_ops_per_lookup": self.ops_per_lookup,
                "valu_glookups_per_s": round(self.valu_lane_ops / self.ops_per_lookup / 1e9, 1),
                "lookup_mix_glookups_per_s": round(self.mix / 1e9, 1),
                "valu_nominal_glookups_per_s": round(self.valu_nominal / self.ops_per_lookup / 1e9, 1),
                "nominal_gather_glookups_per_s": round(NOMINAL_LDS_LOOKUPS_PER_S / 1e9, 1),
                "measured_ds_read_u16_glookups_per_s": round(self.gather / 1e9, 1),
                "hbm_device_copy_gbytes_per_s": round(self.copy_bytes / 1e9, 1)}


def make_table(synth, kind):
    return {"noisy": lambda: synth.table_noisy(7), "trunc2": lambda: synth.table_truncated(2),
            "trunc4": lambda: synth.table_truncated(4), "uniform_error": lambda: synth.table_uniform_error(11),
            "random": lambda: synth.table_random(13), "exact": synth.table_exact}[kind]()


def device_tensors(pkg, xs, fs, codes, seed, mm=MM):
    """Seeded on-grid input and filter, generated on the device (the float of code q is nudged_min + q * scale)."""
    import torch
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    if codes == "uniform":
        qa = torch.randint(0, 256, xs, generator=g, device=dev, dtype=torch.int32)
    else:   # half-normal histogram
        qa = torch.randn(xs, generator=g, device=dev).mul_(48.0).abs_().round_().clamp_(0, 255).to(torch.int32)
    qb = torch.randint(0, 256, fs, generator=g, device=dev, dtype=torch.int32)
    out = []
    for q, lo, hi in ((qa, mm[0], mm[1]), (qb, mm[2], mm[3])):
        nmin, _, scale, _ = pkg.fake_quant.nudge(lo, hi)
        out.append(q.to(torch.float32).mul_(float(scale)).add_(float(nmin)))
    return out[0], out[1]


def time_op(op, xd, fd, steps, preroll_s):
    import torch
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < preroll_s:
        for _ in range(5):
            y = op(xd, fd, *MM)
        torch.cuda.synchronize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        y = op(xd, fd, *MM)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps, y


def kernel_times(ops, op, xd, fd, steps):
    """Mean launch duration per kernel over `steps` calls, from HIP events on the launch stream."""
    import torch
    ops.profile_enable(True)
    ops.profile_reset()
    for _ in range(steps):
        op(xd, fd, *MM)
    torch.cuda.synchronize()
    prof = ops.profile_read()
    ops.profile_enable(False)
    return {k: v[0] / max(v[1], 1) for k, v in prof.items()}


def sampled_oracle_check(oracle, table, op, xd, fd, strides, depthwise, y, n_samples=12, seed=5, mm=MM):
    """The oracle's quantize + LUT-GEMM + epilogue on sampled output pixels (corners included) against the int32
    accumulators and the float output of the GPU.  Returns (acc_bit_exact, linf_rel)."""
    import numpy as np
    import torch
    acc = op.accumulators(xd, fd, *mm)
    N, OH, OW, Cout = acc.shape
    _, H, W, C = xd.shape
    KH, KW = fd.shape[0], fd.shape[1]
    desc = op._desc(xd, fd)
    from tf_approximate_amd import ops as _ops
    dims = _ops.conv2d_geometry(desc)
    ph, pw = int(dims.pad_rows_before), int(dims.pad_cols_before)
    rng = np.random.default_rng(seed)
    picks = [(0, 0, 0), (N - 1, OH - 1, OW - 1), (0, 0, OW - 1), (N - 1, OH - 1, 0)]
    picks += [(int(rng.integers(N)), int(rng.integers(OH)), int(rng.integers(OW))) for _ in range(n_samples)]
    P = len(picks)
    n_i = np.array([p[0] for p in picks])
    ih = np.array([p[1] for p in picks])[:, None] * strides[0] - ph + np.arange(KH)[None, :]      # [P, KH]
    iw = np.array([p[2] for p in picks])[:, None] * strides[1] - pw + np.arange(KW)[None, :]      # [P, KW]
    inb = ((ih >= 0) & (ih < H))[:, :, None] & ((iw >= 0) & (iw < W))[:, None, :]                  # [P, KH, KW]
    dev = xd.device
    idx = lambda a: torch.from_numpy(a).to(dev)
    vals = xd[idx(n_i)[:, None, None], idx(np.clip(ih, 0, H - 1))[:, :, None], idx(np.clip(iw, 0, W - 1))[:, None, :]]
    vals = (vals * idx(inb)[..., None]).cpu().numpy()                                              # [P, KH, KW, C], 0 outside
    got_acc = acc[idx(n_i), idx(np.array([p[1] for p in picks])), idx(np.array([p[2] for p in picks]))].cpu().numpy()
    got_y = y[idx(n_i), idx(np.array([p[1] for p in picks])), idx(np.array([p[2] for p in picks]))].cpu().numpy()
    f = fd.cpu().numpy()

    qp = oracle.quant_props(*mm)
    f32 = np.float32
    qa = oracle.quantize(vals, qp.in_offset, qp.in_inv_scale)      # taps outside hold 0.0f -> the zero-point code
    qb = oracle.quantize(f, qp.f_offset, qp.f_inv_scale)
    if depthwise:
        taps = KH * KW
        a_rows = qa.reshape(P, taps, C).transpose(0, 2, 1).reshape(P * C, taps)
        full = oracle.lut_gemm_codes(table, np.ascontiguousarray(a_rows), np.ascontiguousarray(qb.reshape(taps, C)))
        want = full.reshape(P, C, C)[:, np.arange(C), np.arange(C)]
        vflat = vals.reshape(P, taps, C)
        psum = np.zeros((P, C), f32)
        for t in range(taps):
            psum = (psum + vflat[:, t]).astype(f32)
        fflat = f.reshape(taps, C)
        fsum = np.zeros(C, f32)
        for t in range(taps):
            fsum = (fsum + fflat[t]).astype(f32)
        K = taps
        t1 = (f32(qp.m2) * psum).astype(f32)
    else:
        K = KH * KW * C
        want = oracle.lut_gemm_codes(table, qa.reshape(P, K), qb.reshape(K, Cout))
        vflat = vals.reshape(P, K)
        psum = np.zeros(P, f32)
        for k in range(K):
            psum = (psum + vflat[:, k]).astype(f32)
        fflat = f.reshape(K, Cout)
        fsum = np.zeros(Cout, f32)
        for k in range(K):
            fsum = (fsum + fflat[k]).astype(f32)
        t1 = (f32(qp.m2) * psum).astype(f32)[:, None]
    bit_exact = bool(np.array_equal(got_acc, want))
    out = ((want.astype(f32) * f32(qp.s1xs2)).astype(f32) + t1).astype(f32)
    out = (out + (f32(qp.m1) * fsum).astype(f32)[None, :]).astype(f32)
    out = (out - f32(f32(K) * f32(qp.m1xm2))).astype(f32)
    linf = float(np.max(np.abs(got_y - out)) / max(float(np.max(np.abs(out))), 1e-30))
    return bit_exact, linf


def dense_kernel_name(kernels_ms):
    """The LUT-GEMM kernel a dense layer ran: out of pre-expanded rows, or expanding inside every tile."""
    return "lutgemm_px" if "lutgemm_px" in kernels_ms else "lutgemm_expand"


def cpu_reference_sample(oracle, table, xd, fd, strides, depthwise, seconds=CPU_SAMPLE_S):
    """The oracle's reference-faithful single-thread path on the first output pixels of the first image, sized for
    about `seconds` of work, and its OpenMP variant on the first image; GMAC/s each.  The reference has no depthwise
    op: there the oracle's definition (the dense path per channel) runs on the first rows of the first image."""
    x1 = xd[:1].cpu().numpy()
    f = fd.cpu().numpy()
    cores = max(1, min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "64"))))
    if depthwise:
        rows = min(x1.shape[1], 8 * strides[0])
        t0 = time.perf_counter()
        rc, y, _ = oracle.depthwise_conv2d(table, x1[:, :rows], f, *MM, strides=strides, padding="SAME")
        secs = time.perf_counter() - t0
        macs = y.size * f.shape[0] * f.shape[1]
        return {"cpu_ref_1t_gmacs": round(macs / secs / 1e9, 4), "cpu_omp_gmacs": None, "host_cores": cores,
                "cpu_sample": "first %d input rows of image 0, the dense reference path per channel" % rows}
    kh, kw, c, co = f.shape
    per_pixel = co * kh * kw * c
    _, d = oracle.geometry(x1.shape, f.shape, strides, "SAME")
    pixels_image = int(d.out_rows) * int(d.out_cols)
    patches = int(max(4, min(pixels_image, seconds * 0.4e9 / per_pixel)))
    secs, _ = oracle.time_reference_chunk(table, x1, f, *MM, patches, strides=strides, padding="SAME")
    t0 = time.perf_counter()
    rc, _, _ = oracle.conv2d_fast(table, x1, f, *MM, strides=strides, padding="SAME", threads=cores)
    t_omp = time.perf_counter() - t0
    return {"cpu_ref_1t_gmacs": round(patches * per_pixel / secs / 1e9, 4),
            "cpu_omp_gmacs": round(pixels_image * per_pixel / t_omp / 1e9, 3) if rc == 0 else None, "host_cores": cores,
            "cpu_sample": "first %d output pixels of image 0 (1 thread, extrapolates to the layer); image 0 (OpenMP)" % patches}


def measure_layer(pkg, ops, oracle, ceil, spec, steps=None, preroll_s=0.08):
    config, name, xs, fs, strides, depthwise, codes, tkind = spec
    table = make_table(pkg.synth, tkind)
    xd, fd = device_tensors(pkg, xs, fs, codes, seed=len(name) * 7 + 1)
    op = pkg.ApproxConv2DWithMinMaxVars([1, strides[0], strides[1], 1], 8, table, "SAME", depthwise=depthwise)
    ms_est, _ = time_op(op, xd, fd, 3, 0.0)
    n = steps or int(min(200, max(20, 0.04 / max(ms_est * 1e-3, 1e-6))))
    ms, y = time_op(op, xd, fd, n, preroll_s)
    kms = kernel_times(ops, op, xd, fd, n)
    N, OH, OW, Cout = y.shape
    taps_c = fs[0] * fs[1] * (1 if depthwise else fs[2])
    lookups = N * OH * OW * Cout * taps_c
    main = "depthwise_lut" if depthwise else dense_kernel_name(kms)
    kernel_ms = kms[main]
    rec = {"config": config, "layer": name, "input": list(xs), "filter": list(fs), "strides": list(strides),
           "codes": codes, "table": tkind, "M": N * OH * OW, "K": taps_c, "N": Cout, "lookups": lookups,
           "steps": n, "gpu_ms": round(ms, 4), "gpu_gmacs": round(lookups / (ms * 1e-3) / 1e9, 1),
           "kernel": main, "kernel_ms": round(kernel_ms, 4)}
    if depthwise:
        nbytes = 4 * (xd.numel() + y.numel()) + 4 * fd.numel() + 131072
        gbps = nbytes / (kernel_ms * 1e-3) / 1e9
        rec.update({"bound": "hbm", "frac": round(gbps / HBM_PEAK_GBPS, 4), "hbm_algorithmic_gbytes_per_s": round(gbps, 1),
                    "frac_of_device_copy": round(gbps * 1e9 / ceil.copy_bytes, 4), "algorithmic_bytes": nbytes})
    else:
        fr, _ = ceil.fractions(lookups / (kernel_ms * 1e-3))
        rec.update(fr)
    if oracle is not None:
        exact, linf = sampled_oracle_check(oracle, table, op, xd, fd, strides, depthwise, y)
        rec["acc_bit_exact"] = exact
        rec["linf_rel"] = linf
        rec.update(cpu_reference_sample(oracle, table, xd, fd, strides, depthwise))
    rec["kernels_ms"] = {k: round(v, 4) for k, v in sorted(kms.items())}
    del xd, fd, y
    return rec


def measure_network(pkg, name, steps, warmup, fused_layers=False, graph=False):
    import torch
    from tf_approximate_amd import networks
    synth = pkg.synth
    table = synth.table_uniform_error(11) if name.startswith("resnet50") else synth.table_noisy(7)
    net, xin = networks.build(name, table, fused_layers=fused_layers)
    _, macs = net.forward(xin, calibrate=True)          # fixes every layer's min/max from its own tensors
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < PREROLL_S:      # settle the clocks
        net.forward(xin)
        torch.cuda.synchronize()
    for _ in range(max(warmup, 1)):
        net.forward(xin)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        net.forward(xin)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    rec = {"network": name, "input": list(xin.shape), "convolutions": net.conv_count(), "steps": steps,
           "ms_per_pass": round(ms, 4), "images_per_s": round(xin.shape[0] / (ms * 1e-3), 1),
           "approx_macs_per_pass": macs, "approx_gmac_per_s": round(macs / (ms * 1e-3) / 1e9, 1),
           "fused_layers": bool(fused_layers), "layers_not_fused": net.unfused_layers() if fused_layers else [],
           "note": "convolutions through the op, a ReLU that directly follows one fused into its store; each add with its "
                   "ReLU as one torch elementwise kernel (torch.cuda.jiterator) and the max-pool in torch"}
    if graph:
        rec["hip_graph"] = graph_replay(net, xin, steps)
    return rec


def graph_replay(net, xin, steps):
    """The same pass recorded once into a HIP graph and replayed: the library allocates nothing and never waits for the
    device inside a call, so a whole network is one graph launch and the host's per-call work (about as long as a
    small layer's kernels) drops out.  Every checked replay must reproduce the eager output bit for bit, with eager
    passes and synchronizations between the replays.  A failure is reported, not raised: the eager figures stand."""
    import torch
    try:
        want = net.forward(xin)[0].clone()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):      # first calls on the capture stream: its workspace, lazily set attributes
            for _ in range(2):
                net.forward(xin)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            out = net.forward(xin)[0]
        exact = True
        for _ in range(3):
            out.zero_()
            g.replay()
            torch.cuda.synchronize()
            exact = exact and bool(torch.equal(out, want))
            net.forward(xin)               # eager work between the replays
            torch.cuda.synchronize()
        for _ in range(3):
            g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            g.replay()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        g.replay()
        torch.cuda.synchronize()
        exact = exact and bool(torch.equal(out, want))
        return {"ms_per_pass": round(ms, 4), "images_per_s": round(xin.shape[0] / (ms * 1e-3), 1),
                "replays_equal_eager_bitwise": exact}
    except Exception as e:   # noqa: BLE001
        try:
            torch.cuda.synchronize()
        except Exception:   # noqa: BLE001
            pass
        return {"error": "%s: %s" % (type(e).__name__, str(e)[:300])}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    # the GPU clocks take a few hundred milliseconds of load to settle: the first launches run ~10 % slower
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default=DEFAULT, choices=sorted(WORKLOADS))
    ap.add_argument("--codes", default="uniform", choices=["uniform", "halfnormal"])
    ap.add_argument("--preexpand", type=int, default=0, choices=[-1, 0, 1],
                    help="which dense layers run out of pre-expanded rows (axc_set_preexpand): 0 = the planner's "
                         "choice, 1 = all that can, -1 = none (every layer expands its table rows inside every tile)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-layers", action="store_true", help="leave the `layers` array out (profiler runs)")
    ap.add_argument("--no-networks", action="store_true", help="leave the `networks` array out (profiler runs)")
    ap.add_argument("--only", action="store_true", help="short for --no-layers --no-networks --no-cpu-baseline")
    ap.add_argument("--network", default=None,
                    help="instead of the single layer, time a whole synthetic network whose convolutions all run "
                         "through the op (tf-approximate_amd/networks.py: cifar_resnet_b128, resnet50_b64, "
                         "inverted_residual_b64_s1, inverted_residual_b64_s2) and report images/s")
    ap.add_argument("--fused-layers", action="store_true",
                    help="with --network: every convolution through the layer entry point (per-batch min/max "
                         "and fake quantization on the device, ReLU fused) instead of the op with calibrated ranges")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="instead of the benchmark, run a plain device copy of MIB MiB five times: the known-size "
                         "kernel that scales the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path has no cross-GPU step (output pixels shard without "
                 "communication); run with --gpus 1")
    if args.only:
        args.no_layers = args.no_networks = args.no_cpu_baseline = True

    import numpy as np
    import torch
    if args.copy_calibration:
        n = args.copy_calibration * (1 << 20) // 4
        src = torch.ones(n, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_read": n * 4, "copy_calibration_bytes_written": n * 4, "launches": 5}))
        return
    import __graft_entry__ as entry
    pkg = entry.load_package()
    from tf_approximate_amd import ops, synth
    ops.set_preexpand(args.preexpand)

    if args.network:
        r = measure_network(pkg, args.network, args.steps, args.warmup, args.fused_layers, graph=True)
        print(json.dumps({
            "metric": "images_per_s", "value": r["images_per_s"], "unit": "images/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "preroll_s": PREROLL_S, "ms_per_step": r["ms_per_pass"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int32", "data": "synthetic",
            "config": {"workload": args.network, "input": r["input"], "convolutions": r["convolutions"],
                       "approx_macs_per_pass": r["approx_macs_per_pass"], "fused_layers": r["fused_layers"],
                       "layers_not_fused": r["layers_not_fused"], "note": r["note"]},
            "approx_gmac_per_s": r["approx_gmac_per_s"], "hip_graph": r.get("hip_graph")}))
        return

    xs, fs, strides, depthwise = WORKLOADS[args.workload]
    if args.codes == "uniform":
        qa = synth.uniform_codes(xs, 3)
    else:
        qa = synth.half_normal_codes(xs, 3)
    qb = synth.uniform_codes(fs, 103)
    x = synth.codes_to_grid(qa, MM[0], MM[1])
    f = synth.codes_to_grid(qb, MM[2], MM[3])
    table = synth.table_uniform_error(11)          # the ResNet-50 configuration's table: clamp(a*b + U(-64, 64))

    dev = torch.device("cuda:0")
    xd = torch.from_numpy(x).to(dev)
    fd = torch.from_numpy(f).to(dev)
    op = pkg.ApproxConv2DWithMinMaxVars([1, strides[0], strides[1], 1], 8, table, "SAME", depthwise=depthwise)

    # Settle the clocks first, whatever W is: the GPU needs a few hundred milliseconds of load before it runs at its
    # sustained frequency (the first calls are ~10 % slower).  Not counted as warm-up steps; reported as preroll_s.
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < PREROLL_S:
        for _ in range(20):
            y = op(xd, fd, *MM)
        torch.cuda.synchronize()
    for _ in range(max(args.warmup, 1)):
        y = op(xd, fd, *MM)
    torch.cuda.synchronize()

    # the timed region: exactly K steps, inputs resident, no per-kernel events
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        y = op(xd, fd, *MM)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps

    # the same K steps once more with HIP events around every kernel (on the launch stream), for the roofline:
    # the event bracketing costs a little launch overhead, so it stays out of the timed region
    kms = kernel_times(ops, op, xd, fd, args.steps)

    n, oh, ow, co = y.shape
    taps_c = fs[0] * fs[1] * (1 if depthwise else fs[2])
    lookups = n * oh * ow * co * taps_c
    gmacs = lookups / (ms_per_step * 1e-3) / 1e9

    main_kernel = "depthwise_lut" if depthwise else dense_kernel_name(kms)
    main_ms = kms[main_kernel]
    achieved = lookups / (main_ms * 1e-3)
    ceil = Ceilings(ops)
    hbm_bytes = 4 * (x.size + y.numel()) + 4 * f.size + 131072
    traffic, traffic_source = PROFILED_TRAFFIC.get((args.workload, main_kernel), (None, None))
    if depthwise:
        # K = kh*kw is too small for LDS reuse: 8 bytes of HBM per output element against 9 lookups, HBM-bound
        roofline = {
            "bound": "hbm",
            "kernel": main_kernel,
            "achieved": round(hbm_bytes / (main_ms * 1e-3) / 1e9, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(hbm_bytes / (main_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "frac_of_device_copy": round(hbm_bytes / (main_ms * 1e-3) / ceil.copy_bytes, 4),
            "device_copy_gbytes_per_s": round(ceil.copy_bytes / 1e9, 1),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel_ms": round(main_ms, 4),
            "algorithmic_bytes_per_launch": hbm_bytes,
            "lookups_per_launch": lookups,
            "glookups_per_s": round(achieved / 1e9, 1),
        }
    else:
        fr, peak = ceil.fractions(achieved)
        roofline = {
            "bound": fr["bound"],
            "kernel": main_kernel,
            "achieved": round(achieved / 1e9, 1),
            "peak": round(peak / 1e9, 1),
            "unit": "Glookup/s",
            "frac": fr["frac"],
            "frac_lds_port": fr["frac_lds_port"],
            "frac_valu": fr["frac_valu"],
            "frac_lds_port_measured": fr["frac_lds_port_measured"],
            "frac_valu_measured": fr["frac_valu_measured"],
            "frac_lookup_mix_measured": fr["frac_lookup_mix_measured"],
            "frac_nominal_gather": fr["frac_nominal_gather"],
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel_ms": round(main_ms, 4),
            "lookups_per_launch": lookups,
            "ceilings": ceil.report(),
            "note": "frac = the larger of frac_lds_port (2 bytes per lookup against the LDS read port) and frac_valu "
                    "(accumulate instructions per lookup against the vector ALUs' issue rate), each against the larger "
                    "of its nominal ceiling (CUs x 256 B x clock; CUs x 64 lanes x clock) and the rate a probe kernel "
                    "measured in this run; the *_measured figures are against the probes alone; "
                    "frac_lookup_mix_measured is against a probe made of the kernel's whole per-lookup instruction mix "
                    "(address, 16-byte LDS read, accumulate) and nothing else, which neither of the two ceilings "
                    "contains; frac_nominal_gather "
                    "is against 256 CU x 32 lookups/clk x 2.4 GHz, a ceiling for one-entry gathers that a kernel "
                    "reading 8 entries per access can pass",
            "hbm_algorithmic_bytes": hbm_bytes,
            "hbm_gbps_whole_op": round(hbm_bytes / (ms_per_step * 1e-3) / 1e9, 1),
            "hbm_frac_whole_op": round(hbm_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        }

    oracle = None if args.no_cpu_baseline and args.no_layers else entry.load_oracle()
    cpu = None
    if not args.no_cpu_baseline and not depthwise:
        # calibrate on 256 output pixels, then size the sample for ~cpu_seconds of single-thread work
        secs, _ = oracle.time_reference_chunk(table, x, f, *MM, 256, strides=strides, padding="SAME")
        per_pixel = max(secs / 256, 1e-9)
        patches = int(min(n * oh * ow, max(256, args.cpu_seconds / per_pixel)))
        secs, out_chunk = oracle.time_reference_chunk(table, x, f, *MM, patches, strides=strides, padding="SAME")
        cpu_gmacs = patches * co * taps_c / secs / 1e9
        got = y.reshape(-1, co)[:patches].cpu().numpy()
        linf = float(np.max(np.abs(got - out_chunk)) / max(np.max(np.abs(out_chunk)), 1e-30))
        cpu = {
            "value": round(cpu_gmacs, 4),
            "unit": "GMAC/s",
            "cores": 1,
            "kind": "port",
            "sample": "first %d output pixels (%d MACs), reference loop order j->i->l with the filter "
                      "re-quantized in the inner loop, fp32 accumulate, gcc -O2; the reference CPU op is "
                      "single-threaded" % (patches, patches * co * taps_c),
            "seconds": round(secs, 2),
            "gpu_vs_sample_linf": linf,
        }
        # Not the reference's behaviour (its CPU op is single-threaded): the oracle's pre-quantized int32 loop with
        # OpenMP over the output pixels on the host cores this process may use, on the first images of the batch.
        cores = max(1, min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "64"))))
        images = max(1, min(n, 16))
        t_omp = time.perf_counter()
        rc, _, _ = oracle.conv2d_fast(table, x[:images], f, *MM, strides=strides, padding="SAME", threads=cores)
        t_omp = time.perf_counter() - t_omp
        if rc == 0:
            cpu["openmp_variant"] = {"value": round(images * oh * ow * co * taps_c / t_omp / 1e9, 3), "unit": "GMAC/s",
                                     "cores": cores, "sample": "first %d images, int32 accumulate, filter quantized "
                                     "once, OpenMP over output pixels" % images, "seconds": round(t_omp, 2)}

    result = {
        "metric": "approx_gmac_per_s",
        "value": round(gmacs, 1),
        "unit": "GMAC/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "preroll_s": PREROLL_S,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int32",
        "data": "synthetic",
        "config": {"workload": args.workload, "input": list(xs), "filter": list(fs), "strides": list(strides),
                   "padding": "SAME", "activation_codes": args.codes, "table": "clamp(a*b+U(-64,64))",
                   "lookups": lookups, "preexpand": args.preexpand},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "kernels_ms": {k: round(v, 4) for k, v in sorted(kms.items())},
    }
    del xd, fd, y
    torch.cuda.empty_cache()
    if not args.no_layers:
        t_l = time.perf_counter()
        result["layers"] = [measure_layer(pkg, ops, oracle, ceil, spec) for spec in LAYERS]
        result["layers_seconds"] = round(time.perf_counter() - t_l, 1)
    if not args.no_networks:
        t_n = time.perf_counter()
        result["networks"] = [measure_network(pkg, "cifar_resnet_b128", 40, 10, graph=True),
                              measure_network(pkg, "resnet50_b64", 12, 3, graph=True),
                              measure_network(pkg, "cifar_resnet_b128", 40, 10, fused_layers=True),
                              measure_network(pkg, "resnet50_b64", 12, 3, fused_layers=True)]
        result["networks_seconds"] = round(time.perf_counter() - t_n, 1)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
