"""Seeded random sweep over what the decode entry points accept: every compiled network (the two Int8 geometries of
the benchmark, the wide e4m3-weight one, the LibNTC 0.9.2 geometry with 4 - 16 features and grid scales 1 - 4 in its
Int8 and FP8 versions), sizes that are and are not powers of two down to one texel, partial mip chains, 1 - 16
channels, the three output formats, batches of up to five sets - each decoded through ntc_hip_decode and queried
through ntc_hip_decode_queries (file-ordered and query-ordered latents, sample points outside [0, 1) and mips
outside the set), byte for byte against the CPU checker."""
import random

import numpy as np
import pytest

from cases import Case, cfg_case, ref_case, first_mismatch

pytestmark = pytest.mark.gpu


def random_size(rnd):
    k = rnd.random()
    if k < 0.4:
        return 1 << rnd.randint(0, 9), 1 << rnd.randint(0, 9)
    if k < 0.7:
        return rnd.randint(1, 400), rnd.randint(1, 300)
    return rnd.choice([64, 128, 192, 256, 320, 512]), rnd.choice([4, 8, 60, 128, 256])


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_sets_and_queries_equal_checker(ntc, device, oracle, seed):
    A, P = ntc.abi, ntc.presets
    rnd = random.Random(seed)
    for i in range(40):
        kind = rnd.choice(["cfg01", "cfg2", "cfg3", "ref", "ref", "fp8", "fp8", "fp8"])
        fmt = rnd.choice([A.OUT_FP16_PLANAR_PAIRS, A.OUT_FP16_PIXELS, A.OUT_UNORM8_PIXELS])
        features, grid_scale = rnd.choice([4, 8, 12, 16]), rnd.randint(1, 4)
        cases, described = [], []
        for _ in range(rnd.choice([1, 1, 1, 2, 3, 5])):
            w, h = random_size(rnd)
            if kind in ("ref", "fp8"):
                w, h = max(w, grid_scale), max(h, grid_scale)
            mips = rnd.randint(1, P.full_mip_count(w, h))
            s = rnd.randint(0, 1 << 30)
            if kind == "cfg01":
                c = cfg_case(ntc, P.spec_cfg01(), w, h, mips, rnd.randint(1, 16), fmt, s, scale_log2_range=(-17.0, -12.0))
            elif kind == "cfg2":
                c = cfg_case(ntc, P.spec_cfg2(), w, h, mips, rnd.randint(1, 12), fmt, s, scale_log2_range=(-17.0, -12.0))
            elif kind == "cfg3":
                c = cfg_case(ntc, P.spec_cfg3(), w, h, mips, rnd.randint(1, 16), fmt, s, scale_log2_range=(-17.0, -13.0))
            elif kind == "ref":
                c = ref_case(ntc, P.spec_ref092(features), w, h, mips, grid_scale, rnd.randint(1, 16), fmt, s, scale_log2_range=(-17.0, -12.0))
            else:
                spec = P.spec_ref092_fp8(features)
                mip_list, latent_bytes = P.mips_ref092(spec, w, h, mips, grid_scale)
                sigma = rnd.choice([0.35, 0.35, 0.1, 1.5, (0.35, 1.5, 0.35), (1.5, 0.35, 300.0), (0.35, 40.0, 0.35), 300.0])   # one, two, three weight planes per layer
                c = Case(ntc, spec, mip_list, latent_bytes, rnd.randint(1, 16), fmt, s, weights=ntc.synth.make_fp8_weights(spec, s + 1, weight_sigma=sigma))
            cases.append(c)
            described.append((w, h, mips, c.num_channels))
        what = f"seed {seed} case {i}: {kind}, {features} features, grid scale {grid_scale}, format {fmt}, sets {described}"
        hosts = [c.host_set() for c in cases]
        for hset in hosts:
            hset.decode(threads=8)
        dsets = [c.device_set(device) for c in cases]
        device.decode(dsets)
        device.synchronize()
        for k, (c, hset) in enumerate(zip(cases, hosts)):
            assert first_mismatch(hset.output, c.d_output.download()) is None, f"{what}: set {k}"

        c, hset, dset = cases[0], hosts[0], dsets[0]
        n = rnd.choice([1, 63, 64, 65, 767, 768, 769, 3000])
        q = np.zeros(n, dtype=[("u", np.float32), ("v", np.float32), ("mip", np.int32)])
        rng = np.random.default_rng(rnd.randint(0, 1 << 30))
        q["u"] = rng.random(n, dtype=np.float32) * 1.2 - 0.1
        q["v"] = rng.random(n, dtype=np.float32) * 1.2 - 0.1
        q["mip"] = rng.integers(-1, len(c.mips) + 1, n)
        want = np.zeros((n, 16), dtype=np.uint16)
        assert oracle.ntc_oracle_decode_queries(hset.desc, q.ctypes.data, n, want.ctypes.data, 8) == 0
        d_q = device.upload(q.view(np.uint8))
        d_out = device.alloc(n * 32)
        d_bricks = device.alloc(max(device.lib.ntc_hip_query_latents_bytes(dset), 128))
        A.check(device.lib.ntc_hip_build_query_latents(dset, d_bricks.ptr, d_bricks.nbytes))
        for use_bricks in (False, True):
            dset.queryLatents, dset.queryLatentsBytes = (d_bricks.ptr, d_bricks.nbytes) if use_bricks else (None, 0)
            d_out.fill(0xCD)
            A.check(device.lib.ntc_hip_decode_queries(dset, d_q.ptr, n, d_out.ptr, d_out.nbytes))
            device.synchronize()
            got = d_out.download(np.uint16).reshape(n, 16)
            bad = np.nonzero((got != want).any(axis=1))[0]
            assert bad.size == 0, f"{what}: {bad.size} of {n} queries differ (query-ordered latents: {use_bricks}), first {q[bad[0]]}"
