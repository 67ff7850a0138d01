#!/usr/bin/env python3
"""Headline benchmark: decode a 4096x4096, 16-channel texture set with its full 13-level mip
chain (22 369 621 texels; 2x2-concat 8x2-bit high-res grid + bilinear 16x4-bit low-res grid,
MLP 64-48-32 int8, fp16 output) on one MI355X, bit-exact arithmetic, one launch per step.

Prints ONE JSON line.  A step = one full decode of the set; inputs (latents, weights) are
resident in HBM before the timed region.  `roofline` is for the decode kernel (the only
kernel of the path), timed with HIP events on the library's own stream; `cpu_baseline` is the
CPU checker on a bounded sample of the same workload, on this machine's host cores.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0        # MI355X dense int8 MFMA


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--size", type=int, default=4096)
    ap.add_argument("--format", choices=["fp16", "unorm8"], default="fp16")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target CPU-baseline sample time")
    ap.add_argument("--no-cpu", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this decoder runs on one GPU; texture sets shard with no exchange step, "
              "so multi-GPU figures are not measured here (--gpus must be 1).", file=sys.stderr)
        sys.exit(2)

    ntc = importlib.import_module("rtxntc-library_amd")
    from cases import cfg_case

    dev = ntc.Device(0)
    size = args.size
    spec = ntc.presets.spec_cfg01()
    num_mips = ntc.presets.full_mip_count(size, size)
    fmt = ntc.abi.OUT_FP16_PLANAR_PAIRS if args.format == "fp16" else ntc.abi.OUT_UNORM8_PIXELS
    case = cfg_case(ntc, spec, size, size, num_mips, 16, fmt, seed=0)
    dset = case.device_set(dev)
    texels = case.texels
    out_bytes_per_texel = 32 if args.format == "fp16" else 16
    # algorithmic HBM bytes per texel: output + latent bits amortised (HR 16 b per 4 texels, LR 64 b per 16)
    bytes_per_texel = out_bytes_per_texel + (16 / 4 + 64 / 16) / 8.0
    ops_per_texel = 2 * (64 * 64 + 64 * 48 + 48 * 32 + 32 * 16)

    sets = dev.pack_sets([dset])
    for _ in range(args.warmup):
        dev.decode(sets)
    dev.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        dev.decode(sets)
    dev.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3

    kernel_ms = dev.decode_timed(sets, args.steps)      # HIP events on the launch stream
    gtexels = texels / (ms_per_step * 1e-3) / 1e9
    achieved_gbs = texels * bytes_per_texel / (kernel_ms * 1e-3) / 1e9
    achieved_tops = texels * ops_per_texel / (kernel_ms * 1e-3) / 1e12

    cpu = None
    if not args.no_cpu:
        # The CPU checker (scalar C++ restatement, oracle/ntc_oracle.cpp) on this machine's host
        # cores, over the WHOLE set when that fits the time budget, else over leading rows of mip 0.
        cores = min(16, os.cpu_count() or 1)
        host = case.host_set()
        from oracle_lib import load_oracle
        orc = load_oracle()
        rows = min(256, size)
        t = orc.ntc_oracle_decode_rows(host.desc, 0, 0, rows, cores)          # calibrate
        est_full = t * texels / (rows * size)
        if est_full <= args.cpu_seconds:
            best = min(orc.ntc_oracle_decode(host.desc, cores) for _ in range(2))
            cpu = {"value": texels / best / 1e9, "unit": "Gtexels/s", "cores": cores, "kind": "port",
                   "sample": f"the whole set ({texels} texels), best of 2, {best:.2f} s"}
        else:
            rows = int(max(rows, min(size, args.cpu_seconds * rows / t)))
            t = orc.ntc_oracle_decode_rows(host.desc, 0, 0, rows, cores)
            cpu = {"value": rows * size / t / 1e9, "unit": "Gtexels/s", "cores": cores, "kind": "port",
                   "sample": f"rows 0..{rows} of mip 0 ({rows * size} texels) of the same set, {t:.1f} s"}

    line = {
        "metric": "decoded Gtexels/s, 4096^2 16-ch set, 64-48-32 int8; % of int8-MFMA/HBM roof",
        "value": gtexels, "unit": "Gtexels/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": f"cfg1 headline: {size}x{size} set, {num_mips} mips, 16 channels, MLP 64-64-48-32-16 int8, "
                               f"HR 2x2x8 f@2b + LR 16 f@4b, {args.format} output, {texels} texels per step",
                   "device": dev.name, "compute_units": dev.compute_units},
        "roofline": {"bound": "hbm", "achieved": achieved_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved_gbs / HBM_PEAK_GBS, "traffic": None,
                     "kernel_ms": kernel_ms, "bytes_per_texel": bytes_per_texel,
                     "mfma_achieved_tops": achieved_tops, "mfma_frac": achieved_tops / INT8_PEAK_TOPS},
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
