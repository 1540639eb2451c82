#!/usr/bin/env python3
"""Benchmark of the ApproxConv2DWithMinMaxVars hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

One step = one full invocation of the op (input quantize/relayout, patch sums, filter pack, LUT-GEMM with
fused epilogue) on seeded synthetic tensors that are already resident in HBM.  Prints ONE JSON line.

  value        approximate GMAC/s of the whole op (1 MAC = 1 truth-table lookup), wall clock over K steps
  roofline     the LUT-GEMM kernel alone: algorithmic lookups per launch / its mean launch duration (HIP events
               on the launch stream, recorded inside the library), against the LDS-lookup ceiling
               256 CU x 32 lookups/clk x 2.4 GHz = 19.66 T lookups/s (or this GPU's measured conflict-free
               ds_read_u16 rate, whichever is larger)
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

WORKLOADS = {
    # name: (x_shape, f_shape, strides, depthwise)
    "conv3x3_b64_56x56x64_to_64_s1_same": ((64, 56, 56, 64), (3, 3, 64, 64), (1, 1), False),
    "conv1x1_b32_56x56x256_to_1024": ((32, 56, 56, 256), (1, 1, 256, 1024), (1, 1), False),
    "conv3x3_b64_28x28x512_to_512": ((64, 28, 28, 512), (3, 3, 512, 512), (1, 1), False),
    "conv7x7s2_b64_224x224x3_to_64": ((64, 224, 224, 3), (7, 7, 3, 64), (2, 2), False),
    "conv1x1_b64_112x112x32_to_192": ((64, 112, 112, 32), (1, 1, 32, 192), (1, 1), False),
    "dw3x3_b64_112x112x192_s1": ((64, 112, 112, 192), (3, 3, 192, 1), (1, 1), True),
    "dw3x3_b64_112x112x192_s2": ((64, 112, 112, 192), (3, 3, 192, 1), (2, 2), True),
    "conv3x3_b128_32x32x16_to_16": ((128, 32, 32, 16), (3, 3, 16, 16), (1, 1), False),
}
DEFAULT = "conv3x3_b64_56x56x64_to_64_s1_same"

# HBM bytes per launch of the main kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, each
# scaled by what the same counter reads for --copy-calibration (profiles/lutgemm_expand_conv3x3_b64_56x56x64.md).
MEASURED_TRAFFIC_BYTES = {
    "conv3x3_b64_56x56x64_to_64_s1_same": 2.000 * 13465.0 * 1024 + 1.000 * 72175.1 * 1024,
    # profiles/depthwise_lut3x3_dw3x3_b64_112x112x192_s1.md
    "dw3x3_b64_112x112x192_s1": 2.000 * 838534 * 1024 + 1.000 * 602112 * 1024,
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    # the GPU clocks take a few hundred milliseconds of load to settle: the first launches run ~10 % slower
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default=DEFAULT, choices=sorted(WORKLOADS))
    ap.add_argument("--codes", default="uniform", choices=["uniform", "halfnormal"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--network", default=None,
                    help="instead of the single layer, time a whole synthetic network whose convolutions all run "
                         "through the op (tf-approximate_amd/networks.py: cifar_resnet_b128, resnet50_b64, "
                         "inverted_residual_b64_s1, inverted_residual_b64_s2) and report images/s")
    ap.add_argument("--fused-layers", action="store_true",
                    help="with --network: every dense convolution through the layer entry point (per-batch min/max "
                         "and fake quantization on the device, ReLU fused) instead of the op with calibrated ranges")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="instead of the benchmark, run a plain device copy of MIB MiB five times: the known-size "
                         "kernel that scales the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path has no cross-GPU step (output pixels shard without "
                 "communication); run with --gpus 1")

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

    if args.network:
        from tf_approximate_amd import networks
        table = synth.table_uniform_error(11) if args.network.startswith("resnet50") else synth.table_noisy(7)
        net, xin = networks.build(args.network, table, fused_layers=args.fused_layers)
        _, macs = net.forward(xin, calibrate=True)          # fixes every layer's min/max from its own tensors
        t_pre = time.perf_counter()
        while time.perf_counter() - t_pre < PREROLL_S:      # settle the clocks (see below)
            net.forward(xin)
            torch.cuda.synchronize()
        for _ in range(max(args.warmup, 1)):
            net.forward(xin)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            net.forward(xin)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        print(json.dumps({
            "metric": "images_per_s", "value": round(xin.shape[0] / (ms * 1e-3), 1), "unit": "images/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "preroll_s": PREROLL_S, "ms_per_step": round(ms, 4),
            "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "int32", "data": "synthetic",
            "config": {"workload": args.network, "input": list(xin.shape), "convolutions": net.conv_count(),
                       "approx_macs_per_pass": macs, "fused_layers": bool(args.fused_layers), "note": "convolutions through the op; ReLU, adds, max-pool in torch"},
            "approx_gmac_per_s": round(macs / (ms * 1e-3) / 1e9, 1)}))
        return

    xs, fs, strides, depthwise = WORKLOADS[args.workload]
    mm = (-1.0, 1.0, -0.5, 0.5)
    rng = np.random.default_rng(3)
    if args.codes == "uniform":
        qa = synth.uniform_codes(xs, 3)
    else:
        qa = synth.half_normal_codes(xs, 3)
    qb = synth.uniform_codes(fs, 103)
    x = synth.codes_to_grid(qa, mm[0], mm[1])
    f = synth.codes_to_grid(qb, mm[2], mm[3])
    table = synth.table_uniform_error(11)          # config 4's table: clamp(a*b + U(-64, 64))

    dev = torch.device("cuda:0")
    xd = torch.from_numpy(x).to(dev)
    fd = torch.from_numpy(f).to(dev)
    op = pkg.ApproxConv2DWithMinMaxVars([1, strides[0], strides[1], 1], 8, table, "SAME", depthwise=depthwise)

    # Settle the clocks first, whatever W is: the GPU needs a few hundred milliseconds of load before it runs at its
    # sustained frequency (the first calls are ~10 % slower).  Not counted as warm-up steps; reported as preroll_s.
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < PREROLL_S:
        for _ in range(20):
            y = op(xd, fd, *mm)
        torch.cuda.synchronize()
    for _ in range(max(args.warmup, 1)):
        y = op(xd, fd, *mm)
    torch.cuda.synchronize()

    # the timed region: exactly K steps, inputs resident, no per-kernel events
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        y = op(xd, fd, *mm)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps

    # the same K steps once more with HIP events around every kernel (on the launch stream), for the roofline:
    # the event bracketing costs a little launch overhead, so it stays out of the timed region
    ops.profile_enable(True)
    ops.profile_reset()
    for _ in range(args.steps):
        y = op(xd, fd, *mm)
    torch.cuda.synchronize()
    prof = ops.profile_read()
    ops.profile_enable(False)

    n, oh, ow, co = y.shape
    taps_c = fs[0] * fs[1] * (1 if depthwise else fs[2])
    lookups = n * oh * ow * co * taps_c
    gmacs = lookups / (ms_per_step * 1e-3) / 1e9

    main_kernel = "depthwise_lut" if depthwise else "lutgemm_expand"
    kms = {k: v[0] / max(v[1], 1) for k, v in prof.items()}
    main_ms = kms[main_kernel]
    achieved = lookups / (main_ms * 1e-3)
    measured_peak = ops.lds_gather_peak()
    port_bytes = max(ops.lds_read_peak(), 1.0)
    peak = max(NOMINAL_LDS_LOOKUPS_PER_S, measured_peak)
    hbm_bytes = 4 * (x.size + y.numel()) + 4 * f.size + 131072
    if depthwise:
        # K = kh*kw is too small for LDS reuse: 8 bytes of HBM per output element against 9 lookups, HBM-bound
        dw_bytes = 4 * (x.size + y.numel()) + f.size * 4 + 131072
        roofline = {
            "bound": "hbm",
            "kernel": main_kernel,
            "achieved": round(dw_bytes / (main_ms * 1e-3) / 1e9, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(dw_bytes / (main_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
            "kernel_ms": round(main_ms, 4),
            "algorithmic_bytes_per_launch": dw_bytes,
            "lookups_per_launch": lookups,
            "glookups_per_s": round(achieved / 1e9, 1),
        }
    else:
        roofline = {
            "bound": "lds",
            "kernel": main_kernel,
            "achieved": round(achieved / 1e9, 1),
            "peak": round(peak / 1e9, 1),
            "unit": "Glookup/s",
            "frac": round(achieved / peak, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
            "kernel_ms": round(main_ms, 4),
            "lookups_per_launch": lookups,
            "peak_nominal": round(NOMINAL_LDS_LOOKUPS_PER_S / 1e9, 1),
            "peak_measured_ds_read_u16": round(measured_peak / 1e9, 1),
            # `peak` is the gather ceiling (one 2-byte entry per bank slot).  The kernel reads 16 bytes = 8 entries
            # per lane access out of per-fill expanded rows, so it is not bound by it and `frac` can pass 1; the
            # physical bound behind it is the LDS read port, measured with streaming ds_read_b128:
            "lds_read_port": {
                "peak_gbytes_per_s": round(port_bytes / 1e9, 1),
                "achieved_gbytes_per_s": round(2.0 * achieved / 1e9, 1),
                "frac": round(2.0 * achieved / port_bytes, 4),
                "note": "2 bytes per lookup; the kernel's other LDS traffic (staging and expanding the rows, "
                        "about a quarter on top) is not counted as achieved",
            },
            "hbm_algorithmic_bytes": hbm_bytes,
            "hbm_gbps_whole_op": round(hbm_bytes / (ms_per_step * 1e-3) / 1e9, 1),
            "hbm_frac_whole_op": round(hbm_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        }

    cpu = None
    if not args.no_cpu_baseline and not depthwise:
        oracle = entry.load_oracle()
        # calibrate on 256 output pixels, then size the sample for ~cpu_seconds of single-thread work
        secs, _ = oracle.time_reference_chunk(table, x, f, *mm, 256, strides=strides, padding="SAME")
        per_pixel = max(secs / 256, 1e-9)
        patches = int(min(n * oh * ow, max(256, args.cpu_seconds / per_pixel)))
        secs, out_chunk = oracle.time_reference_chunk(table, x, f, *mm, patches, strides=strides, padding="SAME")
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
        rc, _, _ = oracle.conv2d_fast(table, x[:images], f, *mm, strides=strides, padding="SAME", threads=cores)
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
                   "lookups": lookups},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "kernels_ms": {k: round(v, 4) for k, v in sorted(kms.items())},
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
