#!/usr/bin/env python3
"""Benchmark of the texture-set decode path on one MI355X.

Default (the headline configuration): decode a 4096x4096, 16-channel texture set with its
full 13-level mip chain (22 369 621 texels; 2x2-concat 8x2-bit high-res grid + bilinear 16x4-bit
low-res grid, MLP 64-48-32 int8, fp16 output), bit-exact arithmetic, ONE launch per step.

Prints ONE JSON line.  A step = one full decode of the workload; inputs (latents, weights,
queries) are resident in HBM before the timed region.  `roofline` is for the decode kernel (the
only kernel of the path), timed with HIP events on the library's own launch stream;
`cpu_baseline` is the CPU checker on the same workload (or a bounded sample of it) on this
machine's host cores.  Other --workload values measure the other configurations and kernels.
"""
import argparse
import ctypes as C
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
# Per-launch hardware counters of the decode kernel (rocprofv3 --pmc runs of this file), keyed by workload.
COUNTERS_FILE = os.path.join(ROOT, "profiles", "decode_kernel_counters.json")


def cpu_threads():
    """Threads for the CPU baseline: this job's share of the host (OMP_NUM_THREADS where the box sets one
    below the machine's core count), else every hardware thread."""
    total = os.cpu_count() or 1
    try:
        share = int(os.environ.get("OMP_NUM_THREADS", "0"))
    except ValueError:
        share = 0
    return (min(share, total) if share > 0 else total), total


KERNEL_SOURCES = ("rtxntc-library_amd/csrc/ntc_decode_kernel.hip", "rtxntc-library_amd/csrc/ntc_decode_device.h")


def kernel_source_digest():
    """sha256 over the sources of the decode kernel: the counters file records the one it was measured on."""
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def measured_counters(workload, fmt_name):
    """Counter figures for this workload from profiles/decode_kernel_counters.json, or None.  `stale` is set when the
    kernel's sources are not the ones the counters were taken on."""
    try:
        with open(COUNTERS_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    entry = table.get("workloads", {}).get(f"{workload}_{fmt_name}")
    if entry:
        try:
            stale = table.get("kernel_source_sha256") != kernel_source_digest()
        except OSError:
            stale = True
        entry = dict(entry, source=f"profiles/{os.path.basename(COUNTERS_FILE)}", stale=stale)
    return entry


def macs(widths):
    return sum(a * b for a, b in zip(widths[:-1], widths[1:]))


def bench_copy_kernels(args, ntc, dev):
    """The streaming kernels around the decoder on one 4096x4096, 16-channel mip in the internal fp16
    layout: read = ReadChannels to UNORM8 pixels, write = WriteChannels from UNORM8 pixels, loss =
    per-channel squared error of two images.  Wall-clock per call, synchronised at both ends."""
    import numpy as np
    A = ntc.abi
    size = args.size or 4096
    w = h = size
    channels = 16
    rng = np.random.default_rng(0)
    planar = rng.integers(0, 0x3C00, w * h * channels, dtype=np.uint16)          # halves in [0, 1)
    d_planar = dev.upload(planar)
    wl = args.workload
    if wl == "read":
        d_pixels = dev.alloc(w * h * channels)
        rc = A.ReadChannels()
        rc.planarPairs, rc.planarBytes = d_planar.ptr, d_planar.nbytes
        rc.width, rc.height, rc.setChannels, rc.firstChannel, rc.numChannels = w, h, channels, 0, channels
        rc.dst, rc.dstBytes, rc.format, rc.pixelStride, rc.rowPitch = d_pixels.ptr, d_pixels.nbytes, 1, channels, w * channels
        run = lambda: A.check(dev.lib.ntc_hip_read_channels(rc))
        bytes_per_texel, what = 2 * channels + channels, "ReadChannels, internal fp16 -> UNORM8 pixels"
    elif wl == "write":
        d_pixels = dev.upload(rng.integers(0, 256, w * h * channels, dtype=np.uint8))
        wc = A.WriteChannels()
        wc.src, wc.srcBytes, wc.format, wc.pixelStride, wc.rowPitch = d_pixels.ptr, d_pixels.nbytes, 1, channels, w * channels
        wc.planarPairs, wc.planarBytes = d_planar.ptr, d_planar.nbytes
        wc.width, wc.height, wc.setChannels, wc.firstChannel, wc.numChannels = w, h, channels, 0, channels
        run = lambda: A.check(dev.lib.ntc_hip_write_channels(wc))
        bytes_per_texel, what = channels + 2 * channels, "WriteChannels, UNORM8 pixels -> internal fp16"
    elif wl in ("bc1", "bc3", "bc5", "bc6", "bc7", "bc7m"):
        # RGBA8 image (smooth + noise, a tenth of the pixels transparent) -> blocks
        xs, ys = np.meshgrid(np.arange(w, dtype=np.float32), np.arange(h, dtype=np.float32))
        img = np.stack([127 + 100 * np.sin(xs / (9 + 4 * c) + ys / (17 - 3 * c)) + rng.normal(0, 4, (h, w)) for c in range(4)], axis=2)
        if wl != "bc5":
            img[:, :, 3] = np.where(rng.random((h, w)) < 0.1, 0, 255)
        d_pixels = dev.upload(np.clip(np.rint(img), 0, 255).astype(np.uint8).reshape(-1))
        block_bytes = 8 if wl == "bc1" else 16
        d_blocks = dev.alloc((w // 4) * (h // 4) * block_bytes)
        bc = A.BlockCompress()
        bc.src.data, bc.src.bytes, bc.src.pixelStride, bc.src.rowPitch = d_pixels.ptr, d_pixels.nbytes, 4, 4 * w
        bc.src.width, bc.src.height, bc.src.format, bc.src.numChannels = w, h, 1, 4
        bc.widthInBlocks, bc.heightInBlocks, bc.dstFormat, bc.alphaThreshold = w // 4, h // 4, int(wl[2]), 1.0 / 255.0
        bc.dst, bc.dstBytes, bc.dstRowPitch = d_blocks.ptr, d_blocks.nbytes, (w // 4) * block_bytes
        run = lambda: A.check(dev.lib.ntc_hip_block_compress(bc))
        if wl in ("bc7", "bc7m"):
            img[:, : w // 2, 3] = 255                            # left half opaque: every mode takes part there
            d_pixels = dev.upload(np.clip(np.rint(img), 0, 255).astype(np.uint8).reshape(-1))
            bc.src.data = d_pixels.ptr
        if wl == "bc7m":
            # the full search once; its modes and partitions, packed as MakeBC7ModeBuffer packs them (9 bits per
            # block), then drive the timed single-mode encodes
            run()
            dev.synchronize()
            first = d_blocks.download().view(np.uint32).reshape(-1, 4)[:, 0].astype(np.int64)
            mode = np.minimum(7, np.log2(first & -first).astype(np.int64))
            partition = (first >> (mode + 1)) & np.array([15, 63, 63, 63, 7, 3, 0, 63])[mode]
            entry = (mode << 6) | partition
            entry[entry == 0] = 0x1BF
            bits = ((entry[:, None] >> np.arange(9)) & 1).astype(np.uint8).reshape(-1)
            packed = np.packbits(bits, bitorder="little")
            packed = np.concatenate([packed, np.zeros((-len(packed)) % 4 + 4, dtype=np.uint8)])
            d_modes = dev.upload(packed)
            bc.modeBuffer, bc.modeBufferBytes, bc.modeMapWidthInBlocks, bc.modeMapHeightInBlocks = d_modes.ptr, d_modes.nbytes, w // 4, h // 4
        if wl == "bc5":
            channels = 2
            bytes_per_texel, what = 2 + 1, "BC5 compression of the R and G channels of an RGBA8 image (2 B read, 1 B written per texel)"
        else:
            channels = 4
            bytes_per_texel = 4 + block_bytes / 16
            what = f"{wl.upper()} compression of an RGBA8 image (4 B read, {block_bytes / 16:g} B written per texel)"
            if wl == "bc7m":
                what = "BC7 compression of an RGBA8 image with a mode buffer (each block's mode and partition given)"
    else:
        d_other = dev.upload(rng.integers(0, 0x3C00, w * h * channels, dtype=np.uint16))
        mse = (C.c_float * 16)()
        run = lambda: A.check(dev.lib.ntc_hip_image_loss(d_planar.ptr, d_other.ptr, d_planar.nbytes, w, h, channels, 0xFFFF, -1, 0, mse))
        bytes_per_texel, what = 4 * channels, "per-channel squared error of two images in the internal fp16 layout"
    for _ in range(args.warmup):
        run()
    dev.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    dev.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    gbs = w * h * bytes_per_texel / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "Gtexels/s of a streaming kernel around the decoder", "value": w * h / (ms * 1e-3) / 1e9, "unit": "Gtexels/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"{what}, {w}x{h}, {channels} channels", "device": dev.name, "compute_units": dev.compute_units},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None,
                     "bytes_per_texel": bytes_per_texel},
        "cpu_baseline": None}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=30)   # the GPU clock takes ~30 launches to settle
    ap.add_argument("--workload", default="cfg1", choices=["cfg0", "cfg1", "cfg2", "cfg3", "cfg4", "cfg4fp8", "ref092", "ref092fp8", "read", "write", "loss", "bc1", "bc3", "bc5", "bc6", "bc7", "bc7m"])
    ap.add_argument("--size", type=int, default=0, help="override the texture size of the workload")
    ap.add_argument("--settle-ms", type=float, default=60.0,
                    help="untimed decode steps for this long before the warm-up, so that clocks have ramped (0 = none)")
    ap.add_argument("--format", choices=["fp16", "unorm8"], default=None)
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="time budget of the CPU-baseline sample")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--fp8-weight-sigma", type=float, default=0.35,
                    help="FP8-network workloads: spread of the hidden-layer weights (synth.make_fp8_weights); 0.35 lets every "
                         "layer run on one weight plane, 1.5 needs two, 300 three")
    ap.add_argument("--file-order-latents", action="store_true",
                    help="cfg4: gather from the grids as the file stores them instead of the query-ordered copy")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this decoder runs on one GPU; texture sets shard with no exchange step, "
              "so multi-GPU figures are not measured here (--gpus must be 1).", file=sys.stderr)
        sys.exit(2)

    ntc = importlib.import_module("rtxntc-library_amd")
    from cases import cfg_case, ref_case
    A, P = ntc.abi, ntc.presets

    dev = ntc.Device(0)
    wl = args.workload
    if wl in ("read", "write", "loss", "bc1", "bc3", "bc5", "bc6", "bc7", "bc7m"):
        return bench_copy_kernels(args, ntc, dev)
    fmt_name = args.format or {"cfg2": "unorm8"}.get(wl, "fp16")
    fmt = A.OUT_FP16_PLANAR_PAIRS if fmt_name == "fp16" else A.OUT_UNORM8_PIXELS
    queries = None
    if wl == "cfg0":
        size = args.size or 512
        cases = [cfg_case(ntc, P.spec_cfg01(), size, size, 1, 8, fmt, seed=0)]
        widths, channels, latent_b = (64, 64, 48, 32, 16), 8, 1.0
        what = f"cfg0 plumbing: {size}x{size}, 1 mip, 8 channels, MLP 64-64-48-32-16 int8"
    elif wl == "cfg1":
        size = args.size or 4096
        cases = [cfg_case(ntc, P.spec_cfg01(), size, size, P.full_mip_count(size, size), 16, fmt, seed=0)]
        widths, channels, latent_b = (64, 64, 48, 32, 16), 16, 1.0
        what = (f"cfg1 headline: {size}x{size} set, {P.full_mip_count(size, size)} mips, 16 channels, "
                "MLP 64-64-48-32-16 int8, HR 2x2x8 f@2b + LR 16 f@4b")
    elif wl == "cfg2":
        size = args.size or 2048
        cases = [cfg_case(ntc, P.spec_cfg2(), size, size, P.full_mip_count(size, size), 12, fmt, seed=100 + i) for i in range(8)]
        widths, channels, latent_b = (56, 48, 48, 32, 16), 12, 0.875
        what = f"cfg2 batch: 8 sets of {size}x{size}, full mip chains, 12 channels, MLP 64(56)-48-48-32-16 int8, one launch"
    elif wl == "cfg3":
        size = args.size or 4096
        cases = [cfg_case(ntc, P.spec_cfg3(), size, size, 1, 16, fmt, seed=3)]
        widths, channels, latent_b = (46, 64, 64, 64, 16), 16, 2.5
        what = f"cfg3 wide: {size}x{size}, 1 mip, 16 channels, MLP 48(46)-64-64-64-16, e4m3 hidden-layer weights, both grids bilinear 16 f@4b"
    elif wl == "ref092":
        size = args.size or 4096
        cases = [ref_case(ntc, P.spec_ref092(16), size, size, P.full_mip_count(size, size), 2, 16, fmt, seed=5)]
        widths, channels, latent_b = (46, 64, 48, 32, 16), 16, 44738560 / 22369621.0
        what = f"LibNTC 0.9.2 geometry: {size}x{size}, full mip chain, grid scale 2, 16 features, MLP 48(46)-64-48-32-16 int8"
    elif wl == "ref092fp8":
        from cases import Case
        size = args.size or 4096
        spec = P.spec_ref092_fp8(16)
        mips, latent_bytes = P.mips_ref092(spec, size, size, P.full_mip_count(size, size), 2)
        cases = [Case(ntc, spec, mips, latent_bytes, 16, fmt, seed=5, weights=ntc.synth.make_fp8_weights(spec, 6, weight_sigma=args.fp8_weight_sigma))]
        widths, channels, latent_b = (46, 64, 48, 32, 16), 16, 44738560 / 22369621.0
        planes = "one weight plane per hidden layer" if args.fp8_weight_sigma <= 0.5 else ("two weight planes per hidden layer" if args.fp8_weight_sigma <= 20 else "three weight planes per hidden layer")
        what = (f"LibNTC 0.9.2 geometry with the FP8 network: {size}x{size}, full mip chain, grid scale 2, 16 features, "
                f"MLP 48(46)-64-48-32-16, e4m3 hidden layers (GenericFP8 blob), weights drawn with sigma {args.fp8_weight_sigma:g}: {planes}")
    else:
        size = args.size or 8192
        if wl == "cfg4fp8":
            from cases import Case
            spec = P.spec_ref092_fp8(16)
            mips, latent_bytes = P.mips_ref092(spec, size, size, P.full_mip_count(size, size), 2)
            cases = [Case(ntc, spec, mips, latent_bytes, 16, fmt, seed=4, weights=ntc.synth.make_fp8_weights(spec, 6, weight_sigma=args.fp8_weight_sigma))]
            widths, channels, latent_b = (46, 64, 48, 32, 16), 16, 0.0
        else:
            cases = [cfg_case(ntc, P.spec_cfg01(), size, size, P.full_mip_count(size, size), 16, fmt, seed=4)]
            widths, channels, latent_b = (64, 64, 48, 32, 16), 16, 0.0
        import numpy as np
        n = 1 << 24
        rng = np.random.default_rng(4)
        queries = np.zeros(n, dtype=[("u", np.float32), ("v", np.float32), ("mip", np.int32)])
        queries["u"], queries["v"] = rng.random(n, dtype=np.float32), rng.random(n, dtype=np.float32)
        queries["mip"] = rng.integers(0, len(cases[0].mips), n)
        what = f"cfg4 random access: {size}x{size} set, {len(cases[0].mips)} mips, 2^24 (u,v,mip) queries, 16 x fp16 per query"
        if wl == "cfg4fp8":
            what = "FP8 network of the LibNTC 0.9.2 geometry (grid scale 2, 16 features in both grids), " + what
        fmt_name = "fp16"

    dsets = [c.device_set(dev) for c in cases]
    sets = dev.pack_sets(dsets)
    if queries is None:
        texels = sum(c.texels for c in cases)
        out_b = channels * (2 if fmt_name == "fp16" else 1)
        bytes_per_texel = out_b + latent_b            # algorithmic HBM bytes: output + latent bits amortised
        run = lambda: dev.decode(sets)
        run_timed = lambda k: dev.decode_timed(sets, k)
    else:
        texels = queries.size
        bytes_per_texel = 32 + 12 + (64 if wl == "cfg4fp8" else 40)   # output + the query + 4 HR cells (2 B; 8 B in the 0.9.2 geometry) + 4 LR cells x 8 B
        d_q = dev.upload(queries.view("u1"))
        d_out = dev.alloc(queries.size * 32)
        if not args.file_order_latents:
            # one-time preparation, outside the timed region: the grids once more in query order
            d_bricks = dev.alloc(dev.lib.ntc_hip_query_latents_bytes(sets))
            t_build = time.perf_counter()
            A.check(dev.lib.ntc_hip_build_query_latents(sets, d_bricks.ptr, d_bricks.nbytes))
            dev.synchronize()
            t_build = (time.perf_counter() - t_build) * 1e3
            sets[0].queryLatents, sets[0].queryLatentsBytes = d_bricks.ptr, d_bricks.nbytes
            what += f", latents in query order (built once in {t_build:.2f} ms, not timed)"

        def run():
            A.check(dev.lib.ntc_hip_decode_queries(sets, d_q.ptr, queries.size, d_out.ptr, d_out.nbytes))

        def run_timed(k):
            ms = C.c_float()
            A.check(dev.lib.ntc_hip_decode_queries_timed(sets, d_q.ptr, queries.size, d_out.ptr, d_out.nbytes, k, C.byref(ms)))
            return ms.value
    ops_per_texel = 2 * macs(widths)

    # An idle GPU runs its first few dozen launches below its sustained clock.  Untimed steps, for `--settle-ms`
    # of wall time, come before the W warm-up steps so that a short warm-up does not time the ramp.
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for _ in range(4):
            run()
        dev.synchronize()

    for _ in range(args.warmup):
        run()
    dev.synchronize()
    # The timed region: K calls of the entry point between two synchronisations (wall clock), and HIP events on the
    # launch stream around the same K calls (device time; the first event goes in front of the first call's work).
    t0 = time.perf_counter()
    dev.timer_begin()
    for _ in range(args.steps):
        run()
    kernel_ms = dev.timer_end() / args.steps          # waits for the last launch
    dev.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3

    singles = sorted(run_timed(1) for _ in range(min(args.steps, 100)))     # launches timed one at a time: median and minimum
    median_ms, min_ms = singles[len(singles) // 2], singles[0]
    gtexels = texels / (ms_per_step * 1e-3) / 1e9
    achieved_gbs = texels * bytes_per_texel / (kernel_ms * 1e-3) / 1e9
    achieved_tops = texels * ops_per_texel / (kernel_ms * 1e-3) / 1e12

    cpu = None
    if not args.no_cpu:
        # The CPU checker (scalar C++ restatement, oracle/ntc_oracle.cpp) on this machine's host
        # cores, over the whole workload when that fits the time budget, else over a leading part.
        cores, host_cpus = cpu_threads()
        from oracle_lib import load_oracle
        orc = load_oracle()
        host = cases[0].host_set()
        if queries is None:
            mip0 = cases[0].mips[0]
            rows = min(256, mip0.height)
            t = orc.ntc_oracle_decode_rows(host.desc, 0, 0, rows, cores)          # calibrate
            per_texel = t / (rows * mip0.width)
            if per_texel * texels <= args.cpu_seconds:
                hosts = [host] + [c.host_set() for c in cases[1:]]
                best = None
                for _ in range(2):
                    total = sum(orc.ntc_oracle_decode(h.desc, cores) for h in hosts)
                    best = total if best is None else min(best, total)
                cpu = {"value": texels / best / 1e9, "unit": "Gtexels/s", "cores": cores, "host_cpus": host_cpus, "kind": "port",
                       "sample": f"the whole workload ({texels} texels), best of 2, {best:.2f} s"}
            else:
                rows = int(max(rows, min(mip0.height, args.cpu_seconds / (per_texel * mip0.width))))
                t = orc.ntc_oracle_decode_rows(host.desc, 0, 0, rows, cores)
                cpu = {"value": rows * mip0.width / t / 1e9, "unit": "Gtexels/s", "cores": cores, "host_cpus": host_cpus, "kind": "port",
                       "sample": f"rows 0..{rows} of mip 0 of the first set ({rows * mip0.width} texels), {t:.1f} s"}
        else:
            import numpy as np
            n = min(queries.size, 1 << 21)
            out = np.zeros((n, 16), dtype=np.uint16)
            t0 = time.perf_counter()
            orc.ntc_oracle_decode_queries(host.desc, queries.ctypes.data, n, out.ctypes.data, cores)
            t = time.perf_counter() - t0
            cpu = {"value": n / t / 1e9, "unit": "Gtexels/s", "cores": cores, "host_cpus": host_cpus, "kind": "port",
                   "sample": f"the first {n} queries of the same list, {t:.1f} s"}

    # Two roofs, both from algorithmic work over the kernel's HIP-event time: HBM (output bytes + latent bits) and dense
    # int8 MFMA (operations of the un-padded network).  `bound` names the lower roof, the one that binds; `frac` is the
    # fraction of it.  Instruction counts per texel come from the counters file when it matches the kernel's sources.
    counters = None if args.size else measured_counters(wl, fmt_name)
    fracs = {"hbm": achieved_gbs / HBM_PEAK_GBS, "mfma": achieved_tops / INT8_PEAK_TOPS}
    roofs = {"hbm": HBM_PEAK_GBS * 1e9 / bytes_per_texel / 1e9, "mfma": INT8_PEAK_TOPS * 1e12 / ops_per_texel / 1e9}   # Gtexels/s
    bound = min(roofs, key=roofs.get)
    issue = {}
    if counters and not counters["stale"]:
        issue = {k: counters[k] for k in ("valu_ops_per_texel", "mfma_per_wave_tile", "slow_valu_per_wave_tile",
                                          "SQ_ACTIVE_INST_VALU2_per_VALU", "summary") if k in counters}
    line = {
        "metric": "decoded Gtexels/s, 4096^2 16-ch set, 64-48-32 int8; % of int8-MFMA/HBM roof",
        "value": gtexels, "unit": "Gtexels/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_median": median_ms, "ms_per_step_min": min_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": f"{what}, {fmt_name} output, {texels} texels per step",
                   "device": dev.name, "compute_units": dev.compute_units, "settle_ms": args.settle_ms},
        "roofline": {"bound": bound, "achieved": achieved_gbs if bound == "hbm" else achieved_tops, "peak": HBM_PEAK_GBS if bound == "hbm" else INT8_PEAK_TOPS,
                     "unit": "GB/s" if bound == "hbm" else "TOP/s", "frac": fracs[bound],
                     # HBM bytes per launch from the FETCH_SIZE + WRITE_SIZE counters (null when the kernel's sources
                     # have changed since they were taken)
                     "traffic": counters.get("hbm_traffic_bytes") if counters and not counters["stale"] else None,
                     "counters_stale": bool(counters and counters["stale"]),
                     "kernel_ms": kernel_ms, "bytes_per_texel": bytes_per_texel, "roof_gtexels": roofs,
                     "hbm_achieved_gbs": achieved_gbs, "hbm_frac": fracs["hbm"],
                     "mfma_achieved_tops": achieved_tops, "mfma_frac": fracs["mfma"], **issue},
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
