"""Random-access decode (a list of (u, v, mip) sample points): oracle pin on the CPU and
GPU parity through ntc_hip_decode_queries."""
import ctypes as C

import numpy as np
import pytest

import np_decoder
import oracle_lib
from cases import cfg_case, ref_case

ACTIVE = (-17.0, -12.0)


def make_queries(rng, n, num_mips, with_edges=True):
    q = np.zeros(n, dtype=[("u", np.float32), ("v", np.float32), ("mip", np.int32)])
    q["u"] = rng.random(n, dtype=np.float32)
    q["v"] = rng.random(n, dtype=np.float32)
    q["mip"] = rng.integers(0, num_mips, n)
    if with_edges and n >= 12:
        q["u"][:6] = [0.0, np.nextafter(np.float32(1), np.float32(0)), 1.0, 1.5, -0.25, 0.5]
        q["v"][:6] = [0.0, np.nextafter(np.float32(1), np.float32(0)), 2.0, -3.0, 0.999, 0.5]
        q["mip"][6:9] = [-1, num_mips, 99]             # outside the set: zeros
        q["mip"][9:12] = [num_mips - 1, 0, 0]
    return q


def oracle_queries(oracle, host, q):
    out = np.zeros((q.size, 16), dtype=np.uint16)
    assert oracle.ntc_oracle_decode_queries(host.desc, q.ctypes.data, q.size, out.ctypes.data, 8) == 0
    return out


def test_checker_queries_against_numpy_decoder(ntc, oracle):
    case = cfg_case(ntc, ntc.presets.spec_cfg01(), 64, 32, 7, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, 31, scale_log2_range=ACTIVE)
    host = case.host_set()
    q = make_queries(np.random.default_rng(1), 300, 7)
    got = oracle_queries(oracle, host, q)
    layout = ntc.synth.weight_layout(case.spec)
    mips = [np_decoder.to_half_bits(np_decoder.decode_mip(case.spec, layout, case.weights, case.latents, m)[1]) for m in case.mips]
    for i in range(q.size):
        m = int(q["mip"][i])
        if m < 0 or m >= 7:
            assert not got[i].any()
            continue
        W, H = case.mips[m].width, case.mips[m].height
        x = int(np.clip(np.floor(np.float32(q["u"][i]) * np.float32(W)), 0, W - 1))
        y = int(np.clip(np.floor(np.float32(q["v"][i]) * np.float32(H)), 0, H - 1))
        assert np.array_equal(got[i], mips[m][y, x]), (i, m, x, y)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,n", [("cfg01", 5000), ("cfg01", 1), ("cfg01", 256), ("ref8", 3001), ("cfg2", 777), ("cfg3", 2049)])
def test_gpu_queries_match_checker(ntc, device, oracle, kind, n):
    A = ntc.abi
    if kind == "cfg01":
        case = cfg_case(ntc, ntc.presets.spec_cfg01(), 512, 256, 10, 16, A.OUT_FP16_PLANAR_PAIRS, 41, scale_log2_range=ACTIVE)
    elif kind == "cfg3":
        case = cfg_case(ntc, ntc.presets.spec_cfg3(), 256, 256, 9, 16, A.OUT_FP16_PLANAR_PAIRS, 44, scale_log2_range=(-17.0, -13.0))
    elif kind == "cfg2":
        case = cfg_case(ntc, ntc.presets.spec_cfg2(), 200, 120, 8, 12, A.OUT_FP16_PLANAR_PAIRS, 42, scale_log2_range=ACTIVE)
    else:
        case = ref_case(ntc, ntc.presets.spec_ref092(8), 320, 320, 9, 3, 16, A.OUT_FP16_PLANAR_PAIRS, 43, scale_log2_range=ACTIVE)
    host = case.host_set()
    q = make_queries(np.random.default_rng(n), n, len(case.mips))
    want = oracle_queries(oracle, host, q)
    dset = case.device_set(device)
    d_q = device.upload(q.view(np.uint8))
    d_out = device.alloc(n * 32)
    d_out.fill(0xCD)
    A.check(device.lib.ntc_hip_decode_queries(dset, d_q.ptr, n, d_out.ptr, d_out.nbytes))
    device.synchronize()
    got = d_out.download(np.uint16).reshape(n, 16)
    bad = np.nonzero((got != want).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} of {n} queries differ, first {bad[0]}: {q[bad[0]]} gpu {got[bad[0]]} oracle {want[bad[0]]}"
    ms = C.c_float()
    A.check(device.lib.ntc_hip_decode_queries_timed(dset, d_q.ptr, n, d_out.ptr, d_out.nbytes, 2, C.byref(ms)))
    assert ms.value > 0 and np.array_equal(d_out.download(np.uint16).reshape(n, 16), want)
    # too small an output buffer is refused before launch
    assert device.lib.ntc_hip_decode_queries(dset, d_q.ptr, n, d_out.ptr, n * 32 - 1) == A.ERR_INVALID_ARG


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["cfg01", "cfg2", "cfg3", "ref16", "ref12", "ref8", "ref4", "cfg01-odd", "ref8-odd"])
def test_gpu_queries_from_query_ordered_latents(ntc, device, oracle, kind):
    """ntc_hip_build_query_latents + set.queryLatents: the same bits as without it and as the checker,
    for every compiled geometry (1 to 4 layers per grid), tiny mips (grids narrower than a brick)
    included; sizes that are not powers of two keep using the file-ordered grids."""
    A = ntc.abi
    P = ntc.presets
    if kind.startswith("cfg01"):
        w, h = (512, 256) if kind == "cfg01" else (200, 120)
        case = cfg_case(ntc, P.spec_cfg01(), w, h, P.full_mip_count(w, h), 16, A.OUT_FP16_PLANAR_PAIRS, 51, scale_log2_range=ACTIVE)
    elif kind == "cfg2":
        case = cfg_case(ntc, P.spec_cfg2(), 256, 512, 10, 12, A.OUT_FP16_PLANAR_PAIRS, 52, scale_log2_range=ACTIVE)
    elif kind == "cfg3":
        case = cfg_case(ntc, P.spec_cfg3(), 256, 256, 9, 16, A.OUT_FP16_PLANAR_PAIRS, 53, scale_log2_range=(-17.0, -13.0))
    else:
        features = int(kind[3:].split("-")[0])
        size, grid_scale = (512, 2) if not kind.endswith("odd") else (320, 3)
        case = ref_case(ntc, P.spec_ref092(features), size, size, P.full_mip_count(size, size), grid_scale, 16, A.OUT_FP16_PLANAR_PAIRS, 54 + features, scale_log2_range=ACTIVE)
    n = 6000
    host = case.host_set()
    q = make_queries(np.random.default_rng(len(kind) + n), n, len(case.mips))
    want = oracle_queries(oracle, host, q)
    dset = case.device_set(device)
    d_q = device.upload(q.view(np.uint8))
    d_out = device.alloc(n * 32)
    need = device.lib.ntc_hip_query_latents_bytes(dset)
    assert need >= case.latents.nbytes                      # every grid once more, bricks rounded up
    d_bricks = device.alloc(need)
    A.check(device.lib.ntc_hip_build_query_latents(dset, d_bricks.ptr, d_bricks.nbytes))
    for use_bricks in (False, True):
        dset.queryLatents, dset.queryLatentsBytes = (d_bricks.ptr, d_bricks.nbytes) if use_bricks else (None, 0)
        d_out.fill(0xCD)
        A.check(device.lib.ntc_hip_decode_queries(dset, d_q.ptr, n, d_out.ptr, d_out.nbytes))
        device.synchronize()
        got = d_out.download(np.uint16).reshape(n, 16)
        bad = np.nonzero((got != want).any(axis=1))[0]
        assert bad.size == 0, f"bricks={use_bricks}: {bad.size} of {n} queries differ, first {bad[0]}: {q[bad[0]]} gpu {got[bad[0]]} oracle {want[bad[0]]}"
    # the raster decode does not look at the copy
    dset.queryLatents, dset.queryLatentsBytes = d_bricks.ptr, 1
    A.check(device.lib.ntc_hip_decode(dset, 1))
    # too small or misaligned a copy is refused
    assert device.lib.ntc_hip_decode_queries(dset, d_q.ptr, n, d_out.ptr, d_out.nbytes) == A.ERR_INVALID_ARG
    dset.queryLatents, dset.queryLatentsBytes = d_bricks.ptr + 64, d_bricks.nbytes
    assert device.lib.ntc_hip_decode_queries(dset, d_q.ptr, n, d_out.ptr, d_out.nbytes) == A.ERR_INVALID_ARG
    assert device.lib.ntc_hip_build_query_latents(dset, d_bricks.ptr, need - 1) == A.ERR_INVALID_ARG
    device.synchronize()
