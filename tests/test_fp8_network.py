"""The FP8 version of the network (what ITextureSet::Decompress decodes with unless asked for Int8 weights):
reference include/libntc/shaders/InferenceCoopVec.hlsli:22-124,127-160,235-398 over the weight blob of
src/WeightLayout.cpp:51-71.

The reference leaves the arithmetic of its e4m3 matrix-vector products to the graphics driver, so parity with
the reference's own bits is UNPINNED by construction.  The checker implements one deterministic reading
(oracle/ntc_oracle.cpp); what pins IT:
 * rounding to e4m3: brute force over the format's 127 non-negative values, for every half bit pattern;
 * double -> half: numpy's IEEE conversion;
 * the fp16 HGELU-clamp: numpy float64 evaluation with one rounding per operation over every half, closed-form
   values (0 below -1.5, the identity's neighbourhood above 1.5, 3 from 3 up);
 * an e4m3 layer: the exact rational dot product (python integers) - the fp16 result lies within one rounding
   of it, and equals the correctly rounded value whenever one weight plane carries the whole sum;
 * the input vector: closed forms (constant grids, the positional encoding at texel 0);
 * end to end: an independent vectorised numpy restatement (tests/np_decoder.py) on small sets.
GPU: the kernel's two fp16 primitives against the checker over every half; the matrix instruction's exactness on
operands shaped like the three weight planes; decodes byte-equal to the checker (all feature counts, ragged
sizes, the three output formats, through the C ABI and through libntc.so's Decompress default).
"""
import ctypes as C
from fractions import Fraction

import numpy as np
import pytest

import np_decoder as nd
import oracle_lib
from cases import Case, first_mismatch

ALL_HALVES = np.arange(65536, dtype=np.uint16)


def fp8_case(ntc, features, width, height, mips, grid_scale, channels, fmt, seed, **weights_kw):
    spec = ntc.presets.spec_ref092_fp8(features)
    mip_list, latent_bytes = ntc.presets.mips_ref092(spec, width, height, mips, grid_scale)
    weights = ntc.synth.make_fp8_weights(spec, seed + 1, **weights_kw)
    return Case(ntc, spec, mip_list, latent_bytes, channels, fmt, seed, weights=weights)


@pytest.fixture(scope="module")
def orc():
    lib = oracle_lib.load_oracle()
    lib.ntc_oracle_half_to_e4m3_times_512.restype = C.c_int32
    lib.ntc_oracle_half_to_e4m3_times_512.argtypes = [C.c_uint16]
    lib.ntc_oracle_hgelu_half.restype = C.c_uint16
    lib.ntc_oracle_hgelu_half.argtypes = [C.c_uint16]
    lib.ntc_oracle_double_to_half.restype = C.c_uint16
    lib.ntc_oracle_double_to_half.argtypes = [C.c_double]
    lib.ntc_oracle_layer_e4m3.restype = None
    lib.ntc_oracle_layer_e4m3.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.ntc_oracle_fp8_inputs.restype = C.c_int
    lib.ntc_oracle_fp8_inputs.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    return lib


def test_checker_e4m3_rounding_of_every_half_is_the_nearest_value(orc):
    got = np.array([orc.ntc_oracle_half_to_e4m3_times_512(int(h)) for h in ALL_HALVES], dtype=np.int64)
    values = ALL_HALVES.view(np.float16).astype(np.float64)
    want = np.rint(nd.round_to_e4m3(values) * 512.0).astype(np.int64)
    assert np.array_equal(got, want)
    assert got.max() == 448 * 512 and got.min() == -448 * 512 and len(np.unique(np.abs(got))) == 127


def test_checker_double_to_half_is_one_ieee_rounding(orc):
    rng = np.random.default_rng(2)
    with np.errstate(invalid="ignore"):
        samples = np.concatenate([rng.normal(0, 1, 4000), rng.normal(0, 1e-6, 2000), rng.normal(0, 3e4, 2000),
                                  ALL_HALVES[::37].view(np.float16).astype(np.float64) * (1 + 2.0 ** -12),      # just off a half: no tie
                                  (ALL_HALVES[:0x7bff:29].view(np.float16).astype(np.float64) + ALL_HALVES[1:0x7c00:29].view(np.float16).astype(np.float64)) / 2])   # exact ties
    samples = samples[np.isfinite(samples)]
    with np.errstate(over="ignore"):
        want = samples.astype(np.float16).view(np.uint16)
    got = np.array([orc.ntc_oracle_double_to_half(float(v)) for v in samples], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_checker_fp16_hgelu_of_every_half(orc):
    got = np.array([orc.ntc_oracle_hgelu_half(int(h)) for h in ALL_HALVES], dtype=np.uint16)
    want = nd.hgelu_half(ALL_HALVES.view(np.float16)).view(np.uint16)
    nonzero = (want & 0x7fff) != 0
    assert np.array_equal(got[nonzero], want[nonzero]) and np.all((got[~nonzero] & 0x7fff) == 0)
    x = ALL_HALVES.view(np.float16).astype(np.float64)
    y = got.view(np.float16).astype(np.float64)
    finite = np.isfinite(x)
    assert np.all(y[finite & (x <= -1.5009)] == 0) and np.all(y[x >= 3] == 3) and np.all(y[np.isnan(x)] == 0)
    mid = finite & (x > -1.5) & (x < 3)
    exact = np.minimum(x[mid], 3) * np.clip(x[mid] / 3 + 0.5, 0, 1)
    assert np.abs(y[mid] - exact).max() < 2e-3 and y.min() >= -0.1877 and y.max() == 3          # (half(1/3) < 1/3 lets the minimum dip a hair below -3/16)


def test_checker_e4m3_layer_against_exact_rational_arithmetic(orc):
    rng = np.random.default_rng(3)
    import importlib
    synth = importlib.import_module("rtxntc-library_amd").synth
    close = 0
    for trial in range(40):
        n_in, n_out = (48, 64) if trial % 2 else (64, 48)
        w = synth.e4m3_encode(rng.normal(0, 0.5 if trial < 30 else 40.0, (n_out, n_in)))
        a = nd.round_to_e4m3(rng.uniform(-0.1875, 3.0, n_in))
        if trial % 5 == 0:
            a = nd.round_to_e4m3(rng.uniform(-2.0 ** -6, 2.0 ** -6, n_in))       # subnormal inputs
        bias = rng.normal(0, 0.3, n_out).astype(np.float16)
        a512 = np.rint(a * 512).astype(np.int32)
        x = np.zeros(n_out, dtype=np.uint16)
        orc.ntc_oracle_layer_e4m3(w.ctypes.data, bias.ctypes.data, n_in, n_out, a512.ctypes.data, x.ctypes.data)
        assert np.array_equal(x, nd.layer_e4m3(w, bias, a[None, :])[0].view(np.uint16))
        w512 = nd.e4m3_times_512(w)
        for c in range(n_out):
            exact = Fraction(int(np.dot(w512[c].astype(object), a512.astype(object))), 1 << 18) + Fraction(float(bias[c]))
            got = Fraction(float(x[c:c + 1].view(np.float16)[0]))
            correctly_rounded = float(np.float64(exact.numerator / exact.denominator).astype(np.float16)) if abs(exact) < 60000 else None
            ulp = Fraction(float(np.spacing(np.float16(abs(float(exact))) if abs(exact) < 60000 else np.float16(60000))))
            assert abs(got - exact) <= ulp * Fraction(501, 1000), (trial, c, float(exact), float(got))      # one half rounding + 3 fp32 roundings
            close += correctly_rounded is not None and float(got) == correctly_rounded
    assert close > 0.995 * 40 * 56


def test_checker_fp8_input_vector_closed_forms(ntc, orc):
    """A grid whose cells all hold code q samples to q exactly: input = half(fma(q, 2/15, -1)); texel 0 encodes
    position 0: -1 and -1/2 in every wave; lod inputs hold the mip's positionLod."""
    spec = ntc.presets.spec_ref092_fp8(8)
    mips, latent_bytes = ntc.presets.mips_ref092(spec, 64, 32, 3, 2)
    for code in (0, 5, 15):
        word = code * 0x1111
        case = Case(ntc, spec, mips, latent_bytes, 8, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=1,
                    latents=np.full(latent_bytes // 2, word, dtype=np.uint16), weights=ntc.synth.make_fp8_weights(spec, 1))
        host = case.host_set()
        halves, in512 = np.zeros(48, dtype=np.uint16), np.zeros(48, dtype=np.int32)
        for (m, x, y) in ((0, 0, 0), (1, 7, 3), (2, 15, 7)):
            assert orc.ntc_oracle_fp8_inputs(C.byref(host.desc), m, x, y, halves.ctypes.data, in512.ctypes.data) == 0
            h = halves.view(np.float16).astype(np.float64)
            want = float(np.float16(np.float32(np.float32(code) * np.float32(2.0 / 15.0) - np.float32(1))))    # exact product here: one rounding either way
            assert np.all(h[:8] == want) and np.all(h[16:24] == want) and np.all(h[8:16] == 0) and np.all(h[24:32] == 0)
            assert np.all(h[44:46] == float(np.float16(np.float32(mips[m].positionLod)))) and np.all(h[46:] == 0)
            if (x, y) == (0, 0):
                assert list(h[32:44]) == [-1, -1, -0.5, -0.5] * 3
            assert np.array_equal(in512, np.rint(nd.round_to_e4m3(h) * 512).astype(np.int32))


@pytest.mark.parametrize("features,width,height,grid_scale", [(16, 64, 32, 2), (8, 40, 24, 3), (4, 16, 16, 1)])
def test_checker_fp8_decode_equals_the_numpy_restatement(ntc, oracle, features, width, height, grid_scale):
    mips = ntc.presets.full_mip_count(width, height)
    case = fp8_case(ntc, features, width, height, mips, grid_scale, 10, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=features)
    host = case.host_set()
    host.decode(threads=4)
    layout = ntc.synth.weight_layout(case.spec)
    want = np.full(case.output_bytes, 0xCD, dtype=np.uint8)
    for mip in case.mips:
        outputs = nd.decode_mip_fp8(case.spec, layout, case.weights, case.latents, mip)
        nd.store_mip(want, mip, outputs, 10, ntc.abi.OUT_FP16_PLANAR_PAIRS, 0)
    assert first_mismatch(want, host.output) is None
    assert len(np.unique(host.output.view(np.uint16))) > 200          # a real image


# ---- GPU ------------------------------------------------------------------------------------------------------

@pytest.mark.gpu
def test_gpu_fp16_activation_primitives_of_every_half(ntc, device, orc):
    out = np.zeros(3 * 65536, dtype=np.uint16)
    ntc.abi.check(device.lib.ntc_hip_selftest_fp8_activation(ALL_HALVES.ctypes.data, 65536, out.ctypes.data))
    hgelu, e4m3, quant = out[:65536], out[65536:2 * 65536], out[2 * 65536:]
    x = ALL_HALVES.view(np.float16).astype(np.float64)
    notnan = ~np.isnan(x)
    want_hgelu = np.array([orc.ntc_oracle_hgelu_half(int(h)) for h in ALL_HALVES], dtype=np.uint16)
    zero = (want_hgelu & 0x7fff) == 0
    assert np.array_equal(hgelu[notnan & ~zero], want_hgelu[notnan & ~zero]) and np.all((hgelu[notnan & zero] & 0x7fff) == 0)
    # e4m3 rounding: what the network feeds it lies in [-3, 3]; checked over the format's whole range
    inside = notnan & (np.abs(x) <= 448)
    want_e4m3 = np.array([orc.ntc_oracle_half_to_e4m3_times_512(int(h)) for h in ALL_HALVES], dtype=np.int64)
    got_e4m3 = np.rint(e4m3.view(np.float16).astype(np.float64) * 512).astype(np.int64)
    assert np.array_equal(got_e4m3[inside], want_e4m3[inside])
    # int8 quantisation of the last hidden layer's activations, which lie in [-0.1877, 3]
    act = notnan & (x >= -0.1877) & (x <= 3)
    assert np.array_equal(quant[act].view(np.float16).astype(np.float64), np.rint(80.0 * x[act] - 113.0))


@pytest.mark.gpu
@pytest.mark.parametrize("depth", [16, 32])
def test_gpu_matrix_instruction_is_exact_on_weight_planes(ntc, device, depth):
    """Operands shaped like the three planes of an e4m3 matrix times e4m3 inputs: every partial sum is
    representable in fp32, so the accumulated result must be the exact sum, from a zero accumulator."""
    rng = np.random.default_rng(40 + depth)
    units = (2.0 ** -9, 2.0 ** -2, 2.0 ** 5)
    tops = (127, 127, 14)
    for plane in range(3):
        for trial in range(4):
            a = (rng.integers(-tops[plane], tops[plane] + 1, (16, depth)) * units[plane])
            b = nd.round_to_e4m3(rng.uniform(-0.1875, 3.0, (depth, 16)))
            if trial == 0:
                a[:], b[:] = tops[plane] * units[plane], 3.0                 # largest magnitudes, one sign
            ah, bh = a.astype(np.float16), b.astype(np.float16)
            assert np.array_equal(ah.astype(np.float64), a) and np.array_equal(bh.astype(np.float64), b)
            c, d = np.zeros((16, 16), dtype=np.float32), np.zeros((16, 16), dtype=np.float32)
            ntc.abi.check(device.lib.ntc_hip_selftest_mfma_f16(ah.ctypes.data, bh.ctypes.data, c.ctypes.data, d.ctypes.data, depth))
            assert np.array_equal(d.astype(np.float64), a @ b), (plane, trial)


@pytest.mark.gpu
@pytest.mark.parametrize("depth", [16, 32])
def test_gpu_matrix_instruction_is_exact_on_whole_weights_within_the_one_plane_limit(ntc, device, depth):
    """What lets a layer run on one plane, the e4m3 weights themselves: while sum |512 w| * 1536 stays below 2^24
    for a channel, every partial sum of its products with inputs of at most 3 is a multiple of 2^-18 that fp32
    holds exactly, although the products span 2^-18 .. 2^6.  Operands of that kind - one large weight among tiny
    ones, alternating signs, inputs at the two ends of their range - and an accumulator input that uses up the
    rest of the limit, as the second and third instruction of a chain see it."""
    rng = np.random.default_rng(140 + depth)
    grid = np.unique(np.abs(nd.round_to_e4m3(np.concatenate([np.arange(8) * 2.0 ** -9] + [np.arange(8, 16) * 2.0 ** (e - 10) for e in range(1, 16)]))))
    limit = ((1 << 24) - 1) // 1536                                          # of sum |512 w|
    assert limit == 10922 and len(grid) == 127
    for trial in range(60):
        kind = trial % 4
        if kind == 0:
            a = rng.choice(grid[grid < 1.0], (16, depth)) * rng.choice([-1, 1], (16, depth))
        elif kind == 1:                                                      # one large weight per channel, the rest tiny
            a = rng.choice(grid[grid < 2.0 ** -6], (16, depth)) * rng.choice([-1, 1], (16, depth))
            a[np.arange(16), rng.integers(0, depth, 16)] = rng.choice(grid[(grid >= 4) & (grid <= 8)], 16)
        elif kind == 2:                                                      # alternating signs: large sums cancel
            a = rng.choice(grid[grid < 0.6], (16, depth)) * np.where(np.arange(depth) % 2 == 0, 1, -1)
        else:
            a = rng.choice(grid[grid < 1.3], (16, depth)) * rng.choice([-1, 1], (16, depth))
        for r in range(16):                                                  # this instruction takes at most half of the limit
            while np.abs(a[r] * 512).sum() > limit // 2:
                a[r, rng.integers(0, depth)] = 0
        b = nd.round_to_e4m3(rng.uniform(-3.0, 3.0, (depth, 16)))
        if trial % 3 == 0:
            b = np.where(rng.random((depth, 16)) < 0.5, 2.0 ** -9, 3.0) * rng.choice([-1, 1], (depth, 16))
        room = (limit - limit // 2) * 1536                                   # the accumulator input: the rest of it
        c = rng.integers(-room, room + 1, (16, 16)).astype(np.float64) * 2.0 ** -18
        if trial == 1:
            a[:], b[:], c[:] = 0, 3.0, room * 2.0 ** -18                     # everything at the limit, one sign
            a[:, :6] = [8.0, 2.0, 0.5, 0.125, 0.03125, 5.0 / 512]            # 512 w = 4096 + 1024 + 256 + 64 + 16 + 5 = 5461 = limit // 2
        ah, bh, cf = a.astype(np.float16), b.astype(np.float16), c.astype(np.float32)
        assert np.array_equal(ah.astype(np.float64), a) and np.array_equal(bh.astype(np.float64), b) and np.array_equal(cf.astype(np.float64), c)
        assert (np.abs(a * 512).sum(axis=1) <= limit // 2).all()
        d = np.zeros((16, 16), dtype=np.float32)
        ntc.abi.check(device.lib.ntc_hip_selftest_mfma_f16(ah.ctypes.data, bh.ctypes.data, cf.ctypes.data, d.ctypes.data, depth))
        assert np.array_equal(d.astype(np.float64), a @ b + c), trial


def run_both(device, case):
    host = case.host_set()
    host.decode(threads=8)
    dset = case.device_set(device)
    device.decode([dset])
    device.synchronize()
    return host.output, case.d_output.download()


@pytest.mark.gpu
@pytest.mark.parametrize("features,grid_scale", [(16, 2), (12, 3), (8, 4), (4, 1)])
def test_gpu_fp8_decode_equals_checker(ntc, device, features, grid_scale):
    case = fp8_case(ntc, features, 192, 128, 8, grid_scale, 10, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=60 + features)
    expected, got = run_both(device, case)
    mm = first_mismatch(expected, got)
    assert mm is None, f"{mm[1]} of {expected.size} bytes differ, first at {mm[0]}"
    assert len(np.unique(got.view(np.uint16))) > 1000


@pytest.mark.gpu
@pytest.mark.parametrize("w,h,ch", [(100, 36, 7), (67, 5, 16), (6, 4, 3), (256, 256, 16)])
def test_gpu_fp8_decode_ragged_sizes_and_formats(ntc, device, w, h, ch):
    for fmt in (ntc.abi.OUT_FP16_PLANAR_PAIRS, ntc.abi.OUT_FP16_PIXELS, ntc.abi.OUT_UNORM8_PIXELS):
        case = fp8_case(ntc, 16, w, h, ntc.presets.full_mip_count(w, h), 2, ch, fmt, seed=w + h)
        expected, got = run_both(device, case)
        assert first_mismatch(expected, got) is None, (w, h, ch, fmt)


@pytest.mark.gpu
def test_gpu_fp8_decode_with_extreme_weights(ntc, device):
    """Weights over the whole e4m3 range (sums far beyond fp16) and large biases: the three-plane sums stay
    exact and saturating activations behave as in the checker."""
    case = fp8_case(ntc, 16, 128, 64, 5, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=9, weight_sigma=300.0, bias_sigma=2000.0)
    expected, got = run_both(device, case)
    assert first_mismatch(expected, got) is None


@pytest.mark.gpu
@pytest.mark.parametrize("sigmas", [(300.0, 0.35, 0.35), (0.35, 300.0, 0.35), (0.35, 0.35, 300.0), (40.0, 0.35, 40.0)])
def test_gpu_fp8_decode_with_large_weights_in_some_layers(ntc, device, sigmas):
    """A hidden layer whose weights all stay below 32 runs without its top weight plane; layers are decided one
    by one.  Power-of-two sizes, so the integer input stage runs as well."""
    case = fp8_case(ntc, 16, 128, 64, 8, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=31, weight_sigma=sigmas, bias_sigma=1.0)
    expected, got = run_both(device, case)
    assert first_mismatch(expected, got) is None, sigmas


@pytest.mark.gpu
@pytest.mark.parametrize("sigmas", [(1.5, 1.5, 1.5), (0.35, 1.5, 300.0), (1.5, 300.0, 0.35), (300.0, 0.35, 1.5), (0.1, 0.1, 0.1)])
def test_gpu_fp8_decode_with_one_two_and_three_planes_in_some_layers(ntc, device, sigmas):
    """How many weight planes a hidden layer's matrix instructions go through is decided layer by layer from its
    weights: one where sum |w| of every channel is small enough for the whole dot product to be exact in fp32
    (sigma 0.35 and below here), two while all weights stay below 32 (sigma 1.5: sums of 30 and more), else three.
    The bytes must not depend on it."""
    case = fp8_case(ntc, 16, 128, 64, 8, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=47, weight_sigma=sigmas, bias_sigma=1.0)
    spec = ntc.presets.spec_ref092_fp8(16)
    layout = ntc.synth.weight_layout(spec)
    for layer, sigma in enumerate(sigmas):                                   # the networks are what the test says they are
        n_in, n_out = spec.layer_inputs(layer), spec.layer_outputs(layer)
        w512 = np.abs(nd.e4m3_times_512(case.weights[layout.weightOffset[layer]:layout.weightOffset[layer] + n_in * n_out])).reshape(n_out, n_in)
        planes = 3 if w512.max() >= 32 * 512 else (2 if w512.sum(axis=1).max() > 10922 else 1)
        assert planes == {300.0: 3, 1.5: 2, 0.35: 1, 0.1: 1}[sigma], (layer, sigma, planes)
    expected, got = run_both(device, case)
    assert first_mismatch(expected, got) is None, sigmas
    assert len(np.unique(got.view(np.uint16))) > 500


@pytest.mark.gpu
@pytest.mark.parametrize("layer", [0, 1, 2])
@pytest.mark.parametrize("planes", [1, 2, 3])
def test_gpu_fp8_every_form_of_every_layer(ntc, device, layer, planes):
    """Every (hidden layer, number of weight planes) form of the network on its own: the layer under test runs on
    `planes` planes, the two others on one.  planes = 1 is the instantiation for one-plane sets; 2 and 3 take the
    general one, where the layer's form differs from its neighbours'.  Each form has its own chain of matrix
    instructions (16-deep or 32-deep, one chain per plane): a wrong sum in any of them shows here."""
    sigma = {1: 0.35, 2: 1.5, 3: 300.0}[planes]
    sigmas = tuple(sigma if l == layer else 0.35 for l in range(3))
    case = fp8_case(ntc, 16, 128, 64, 8, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=90 + 3 * layer + planes, weight_sigma=sigmas, bias_sigma=1.0)
    spec = ntc.presets.spec_ref092_fp8(16)
    layout = ntc.synth.weight_layout(spec)
    n_in, n_out = spec.layer_inputs(layer), spec.layer_outputs(layer)
    w512 = np.abs(nd.e4m3_times_512(case.weights[layout.weightOffset[layer]:layout.weightOffset[layer] + n_in * n_out])).reshape(n_out, n_in)
    assert planes == (3 if w512.max() >= 32 * 512 else (2 if w512.sum(axis=1).max() > 10922 else 1))
    expected, got = run_both(device, case)
    assert first_mismatch(expected, got) is None, (layer, planes)
    assert len(np.unique(got.view(np.uint16))) > 500


@pytest.mark.gpu
@pytest.mark.parametrize("layer", [0, 1, 2])
def test_gpu_fp8_decode_at_the_one_plane_limit(ntc, device, layer):
    """One channel of one hidden layer with sum |512 w| = 10922 (the largest sum whose products with inputs of 3
    stay below 2^24 units of 2^-18: one plane) and with 10923 (two planes), the large weights on the channel's
    first inputs; both sides of the limit give the checker's bytes."""
    spec = ntc.presets.spec_ref092_fp8(16)
    layout = ntc.synth.weight_layout(spec)
    n_in, n_out = spec.layer_inputs(layer), spec.layer_outputs(layer)
    for last in (10, 11):                                                    # 7168 + 3584 + 160 + 10 = 10922
        case = fp8_case(ntc, 16, 64, 64, 4, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=300 + layer, weight_sigma=0.1, bias_sigma=0.5)
        w = case.weights[layout.weightOffset[layer]:layout.weightOffset[layer] + n_in * n_out].reshape(n_out, n_in)
        row = np.zeros(n_in)
        row[:4] = np.array([7168, -3584, 160, last]) / 512.0
        w[9] = ntc.synth.e4m3_encode(row)
        assert np.abs(nd.e4m3_times_512(w[9])).sum() == 10912 + last
        assert np.abs(nd.e4m3_times_512(w.reshape(-1))).reshape(n_out, n_in).sum(axis=1).max() == 10912 + last
        expected, got = run_both(device, case)
        assert first_mismatch(expected, got) is None, (layer, last)
        assert len(np.unique(got.view(np.uint16))) > 500


@pytest.mark.gpu
@pytest.mark.parametrize("scale", [0.107, 0.1072, 0.5, 40.0])
def test_gpu_fp8_outputs_near_and_beyond_the_fp16_range(ntc, device, scale):
    """An output whose half would be an infinity is stored as zero (IsHalfSpecial).  The stores skip that check
    when (|bias| + 32 * 127 * 128) * |scale| < 60000 holds for every channel of the output layer: with biases of
    +-40000 that is scale < 0.10711.  Either side of it, and scales with which outputs do overflow (zeros must
    appear, as in the checker)."""
    spec = ntc.presets.spec_ref092_fp8(16)
    layout = ntc.synth.weight_layout(spec)
    last = ntc.abi.MLP_LAYERS - 1
    case = fp8_case(ntc, 16, 128, 64, 4, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=401, bias_sigma=0.5)
    case.weights[layout.scaleOffset[last]:layout.scaleOffset[last] + 64] = np.full(16, scale, dtype=np.float32).view(np.uint8)
    bias = np.where(np.arange(16) % 2 == 0, 40000, -40000).astype(np.int32)
    case.weights[layout.biasOffset[last]:layout.biasOffset[last] + 64] = bias.view(np.uint8)
    expected, got = run_both(device, case)
    assert first_mismatch(expected, got) is None, scale
    halves = got.view(np.uint16)
    assert not np.any((halves & 0x7fff) >= 0x7c00)                           # no infinity, no NaN is ever stored
    if scale >= 40.0:
        assert np.count_nonzero(halves == 0) > 1000                          # overflowing outputs became zeros


@pytest.mark.gpu
def test_gpu_fp8_level_of_detail_input_up_to_three(ntc, device):
    """The exactness of the layer sums is proven for inputs of at most 3 in magnitude.  Features and positional
    encoding lie in [-1, 1]; the level-of-detail input comes from the caller's descriptor: +-3 decodes to the
    checker's bytes (layer 0 on one plane, its largest channel sum just inside the limit), anything beyond - and
    a NaN - is refused."""
    spec = ntc.presets.spec_ref092_fp8(16)
    layout = ntc.synth.weight_layout(spec)
    for lod in (3.0, -3.0, 2.75):
        case = fp8_case(ntc, 16, 64, 64, 3, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=71, weight_sigma=0.1, bias_sigma=0.5)
        w = case.weights[layout.weightOffset[0]:layout.weightOffset[0] + 48 * 64].reshape(64, 48)
        row = np.zeros(48)
        row[44:46] = np.array([7168, 3584]) / 512.0                          # the two level-of-detail inputs
        row[:2] = np.array([160, 10]) / 512.0                                # sum |512 w| = 10922
        w[3] = ntc.synth.e4m3_encode(row)
        for d in case.mips:
            d.positionLod = lod
        expected, got = run_both(device, case)
        assert first_mismatch(expected, got) is None, lod
    for lod in (3.0001, -4.0, float("nan"), float("inf")):
        case = fp8_case(ntc, 16, 64, 64, 3, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=71)
        case.mips[1].positionLod = lod
        with pytest.raises(ntc.NtcHipError) as e:
            device.decode([case.device_set(device)])
        assert e.value.code == ntc.abi.ERR_INVALID_ARG and "positionLod" in e.value.message, lod


@pytest.mark.gpu
@pytest.mark.parametrize("layer", [0, 1, 2])
def test_gpu_fp8_decode_with_biases_at_and_beyond_the_finite_range(ntc, device, layer):
    """A hidden layer with small weights and biases of at most 57344 in magnitude cannot leave the finite halves
    and runs without the activation's lower clamp; one bias beyond that (the next half, an infinity, a NaN) sends
    the layer through the general evaluation.  Both sides of the limit, in every hidden layer."""
    spec = ntc.presets.spec_ref092_fp8(16)
    layout = ntc.synth.weight_layout(spec)
    for trial, specials in enumerate([(0x7B00, 0xFB00, 0x7AFF), (0x7B01,), (0xFB01,), (0x7C00, 0xFC00), (0x7E00, 0xFB00), (0xFBFF, 0x7BFF)]):
        case = fp8_case(ntc, 16, 64, 32, 3, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=200 + 10 * layer + trial, bias_sigma=0.5)
        bias = case.weights[layout.biasOffset[layer]:layout.biasOffset[layer] + 2 * spec.layer_outputs(layer)].view(np.uint16)
        for i, bits in enumerate(specials):
            bias[5 + 7 * i] = bits
        expected, got = run_both(device, case)
        assert first_mismatch(expected, got) is None, (layer, specials)
        assert len(np.unique(got.view(np.uint16))) > 500


@pytest.mark.gpu
@pytest.mark.parametrize("features,grid_scale,w,h", [(16, 1, 256, 64), (16, 2, 64, 256), (12, 4, 512, 128), (8, 2, 128, 128), (4, 4, 256, 256)])
def test_gpu_fp8_integer_input_stage_equals_checker(ntc, device, features, grid_scale, w, h):
    """Power-of-two mips, grids and position scales take the all-integer input stage (and the positional table);
    every mip down to 1 x 1, where footprints wrap around grids one or two cells wide."""
    case = fp8_case(ntc, features, w, h, ntc.presets.full_mip_count(w, h), grid_scale, 16, ntc.abi.OUT_FP16_PIXELS, seed=7 * features + grid_scale)
    expected, got = run_both(device, case)
    mm = first_mismatch(expected, got)
    assert mm is None, f"{mm[1]} of {expected.size} bytes differ, first at {mm[0]}"


@pytest.mark.gpu
def test_gpu_fp8_batch_mixes_sets_with_and_without_top_planes(ntc, device):
    """One launch over sets whose weights need three planes, two planes, three again: the plane choice follows the
    staged set."""
    sigmas = [300.0, 0.35, (0.35, 300.0, 0.35), 0.35]
    cases = [fp8_case(ntc, 8, 64, 32, 6, 2, 8, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=90 + i, weight_sigma=s) for i, s in enumerate(sigmas)]
    hosts = [c.host_set() for c in cases]
    for hset in hosts:
        hset.decode(threads=8)
    device.decode([c.device_set(device) for c in cases])
    device.synchronize()
    for i, (c, hset) in enumerate(zip(cases, hosts)):
        assert first_mismatch(hset.output, c.d_output.download()) is None, i


@pytest.mark.gpu
def test_gpu_fp8_batch_with_set_boundaries_inside_the_rounds_of_a_workgroup(ntc, device):
    """More tiles than resident workgroups take three at a time: every workgroup walks a share of several tiles in
    rounds of up to three that stop at the next set (other weights), so sets begin in the middle of a share, at
    every position of a round.  Sizes chosen so that the sets' tile counts are not multiples of three."""
    sizes = [(256, 256), (320, 192), (256, 128), (192, 320), (256, 256), (64, 448)]
    cases = [fp8_case(ntc, 16, w, h, ntc.presets.full_mip_count(w, h), 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=300 + i,
                      weight_sigma=(0.35 if i % 2 else (0.35, 40.0, 0.35))) for i, (w, h) in enumerate(sizes)]
    hosts = [c.host_set() for c in cases]
    for hset in hosts:
        hset.decode(threads=8)
    device.decode([c.device_set(device) for c in cases])
    device.synchronize()
    for i, (c, hset) in enumerate(zip(cases, hosts)):
        mm = first_mismatch(hset.output, c.d_output.download())
        assert mm is None, (i, mm)


@pytest.mark.gpu
def test_gpu_fp8_batch_of_sets_and_static_table(ntc, device):
    cases = [fp8_case(ntc, 8, 64, 64, 7, 2, 8, ntc.abi.OUT_UNORM8_PIXELS, seed=80 + i) for i in range(3)]
    hosts = [c.host_set() for c in cases]
    for hset in hosts:
        hset.decode(threads=8)
    dsets = [c.device_set(device) for c in cases]
    device.decode(dsets)
    device.synchronize()
    for c, hset in zip(cases, hosts):
        assert first_mismatch(hset.output, c.d_output.download()) is None
        c.d_output.fill(0xCD)
    device.decode_static(dsets)
    device.synchronize()
    for c, hset in zip(cases, hosts):
        assert first_mismatch(hset.output, c.d_output.download()) is None


@pytest.mark.gpu
def test_gpu_fp8_network_is_not_offered_for_other_geometries(ntc, device):
    spec = ntc.presets.spec_cfg01()
    spec.weightType = ntc.abi.WEIGHTS_FP8
    case = Case(ntc, spec, *ntc.presets.mips_private_grids(spec, 64, 64, 1), 8, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=1,
                weights=np.zeros(ntc.synth.weight_layout(spec).bufferSize, dtype=np.uint8))
    with pytest.raises(ntc.NtcHipError) as e:
        device.decode([case.device_set(device)])
    assert e.value.code == ntc.abi.ERR_UNSUPPORTED
    q = device.upload(np.zeros(3 * 4, dtype=np.float32))
    out = device.alloc(4 * 32)
    assert device.lib.ntc_hip_decode_queries(case.device_set(device), q.ptr, 4, out.ptr, out.nbytes) == ntc.abi.ERR_UNSUPPORTED


def fp8_queries(rng, n, num_mips):
    q = np.zeros(n, dtype=[("u", np.float32), ("v", np.float32), ("mip", np.int32)])
    q["u"] = rng.random(n, dtype=np.float32)
    q["v"] = rng.random(n, dtype=np.float32)
    q["mip"] = rng.integers(0, num_mips, n)
    if n >= 12:
        q["u"][:6] = [0.0, np.nextafter(np.float32(1), np.float32(0)), 1.0, 1.5, -0.25, 0.5]
        q["v"][:6] = [0.0, np.nextafter(np.float32(1), np.float32(0)), 2.0, -3.0, 0.999, 0.5]
        q["mip"][6:9] = [-1, num_mips, 99]                 # outside the set: zeros
        q["mip"][9:12] = [num_mips - 1, 0, 0]
    return q


def test_checker_fp8_queries_are_its_raster_decode_at_the_texels_hit(ntc, oracle):
    case = fp8_case(ntc, 16, 48, 40, 6, 2, 16, ntc.abi.OUT_FP16_PIXELS, seed=77)
    host = case.host_set()
    host.decode(threads=8)
    n = 400
    q = fp8_queries(np.random.default_rng(5), n, len(case.mips))
    got = np.zeros((n, 16), dtype=np.uint16)
    assert oracle.ntc_oracle_decode_queries(host.desc, q.ctypes.data, n, got.ctypes.data, 4) == 0
    raster = host.output.view(np.uint16)
    for i in range(n):
        m = int(q["mip"][i])
        if m < 0 or m >= len(case.mips):
            assert not got[i].any()
            continue
        d = case.mips[m]
        x = int(np.clip(np.floor(np.float32(q["u"][i]) * np.float32(d.width)), 0, d.width - 1))
        y = int(np.clip(np.floor(np.float32(q["v"][i]) * np.float32(d.height)), 0, d.height - 1))
        start = (d.outOffset + y * d.outRowPitch + x * case.pixel_stride) // 2
        assert np.array_equal(got[i], raster[start:start + 16]), (i, m, x, y)


@pytest.mark.gpu
@pytest.mark.parametrize("features,size,grid_scale,n,sigma", [(16, 512, 2, 6000, 0.35), (12, 256, 4, 3001, 0.35), (8, 512, 1, 777, 0.35), (4, 256, 2, 1, 0.35),
                                                         (16, 320, 3, 4000, 0.35), (8, 200, 2, 2049, 0.35), (16, 256, 2, 5000, (0.35, 40.0, 300.0))])
def test_gpu_fp8_queries_match_checker(ntc, device, oracle, features, size, grid_scale, n, sigma):
    """Random-access decode with the FP8 network: sample points over every mip of a set (edges, mips outside the
    set), from the file-ordered grids and from the query-ordered copy, against the checker's decode of the texels
    they hit.  Sizes that are not powers of two take the float input stage; one case has layers with large weights
    (three weight planes)."""
    A = ntc.abi
    case = fp8_case(ntc, features, size, size, ntc.presets.full_mip_count(size, size), grid_scale, 16, A.OUT_FP16_PLANAR_PAIRS,
                    seed=400 + features + n, weight_sigma=sigma)
    host = case.host_set()
    q = fp8_queries(np.random.default_rng(n + features), n, len(case.mips))
    want = np.zeros((n, 16), dtype=np.uint16)
    assert oracle.ntc_oracle_decode_queries(host.desc, q.ctypes.data, n, want.ctypes.data, 8) == 0
    assert len(np.unique(want)) > min(n, 300)
    dset = case.device_set(device)
    d_q = device.upload(q.view(np.uint8))
    d_out = device.alloc(n * 32)
    need = device.lib.ntc_hip_query_latents_bytes(dset)
    d_bricks = device.alloc(need)
    A.check(device.lib.ntc_hip_build_query_latents(dset, d_bricks.ptr, d_bricks.nbytes))
    for use_bricks in (False, True):
        dset.queryLatents, dset.queryLatentsBytes = (d_bricks.ptr, d_bricks.nbytes) if use_bricks else (None, 0)
        d_out.fill(0xCD)
        A.check(device.lib.ntc_hip_decode_queries(dset, d_q.ptr, n, d_out.ptr, d_out.nbytes))
        device.synchronize()
        got = d_out.download(np.uint16).reshape(n, 16)
        bad = np.nonzero((got != want).any(axis=1))[0]
        assert bad.size == 0, f"bricks={use_bricks}: {bad.size} of {n} queries differ, first {bad[0]}: {q[bad[0]]} gpu {got[bad[0]]} checker {want[bad[0]]}"
    ms = C.c_float()
    A.check(device.lib.ntc_hip_decode_queries_timed(dset, d_q.ptr, n, d_out.ptr, d_out.nbytes, 2, C.byref(ms)))
    assert ms.value > 0 and np.array_equal(d_out.download(np.uint16).reshape(n, 16), want)


@pytest.mark.gpu
def test_gpu_fp8_launch_pairs_of_one_context_do_not_inherit_each_others_hand_off(ntc, device):
    """The network's two launches talk through one dword of the context (and another behind the per-device table):
    the second leaves at once unless the first met a set that is not its own.  Sets of either kind decoded in turn
    through one context, by both entry points, with the output cleared before each decode: a launch that believed
    the previous pair's word would leave its set undecoded."""
    kinds = [0.35, 1.5, 0.35, 0.35, 300.0, 1.5, 0.35]
    cases = [fp8_case(ntc, 16, 96, 40, 3, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=400 + i, weight_sigma=s) for i, s in enumerate(kinds)]
    hosts = [c.host_set() for c in cases]
    for hset in hosts:
        hset.decode(threads=8)
    dsets = [c.device_set(device) for c in cases]
    for static in (False, True, False):
        for i, (c, hset) in enumerate(zip(cases, hosts)):
            c.d_output.fill(0xCD)
            (device.decode_static if static else device.decode)([dsets[i]])
            device.synchronize()
            assert first_mismatch(hset.output, c.d_output.download()) is None, (static, i)
