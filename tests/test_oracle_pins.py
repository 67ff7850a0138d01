"""Pins the CPU checker (oracle/ntc_oracle.cpp) before anything is compared with it.

The reference ships no tests, golden vectors or sample files for the decode path, so each
function of the checker is pinned by something it did not come from: the reference's own
host code where that compiles (oracle/_ref), fixtures written from it, exact rational
arithmetic, exhaustive enumeration, numpy's IEEE types, and an independent numpy decoder.
"""
import ctypes as C
import json
import os
from fractions import Fraction

import numpy as np
import pytest

import np_decoder
import oracle_lib
from cases import cfg_case, ref_case

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ---------------------------------------------------------------------------------------
# exact helpers
# ---------------------------------------------------------------------------------------
def round_to_f32(fr):
    """Round an exact Fraction to the nearest float32 (ties to even), returned as np.float32."""
    if fr == 0:
        return np.float32(0.0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -126)                               # subnormals share the exponent -126
    scaled = a / Fraction(2) ** (e - 23)           # value in units of one ulp
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    return np.float32(sign * float(Fraction(n) * Fraction(2) ** (e - 23)))


def hgelu_exact(x32):
    """Inference.hlsli:36-39,123-131 in exact arithmetic with explicit float32 roundings."""
    x = Fraction(float(x32))
    t = round_to_f32(x * Fraction(float(np.float32(0.333333))) + Fraction(1, 2))      # fused mad
    t = min(max(Fraction(float(t)), Fraction(0)), Fraction(1))
    y = round_to_f32(min(x, Fraction(3)) * t)
    z = Fraction(float(round_to_f32(Fraction(float(y)) * 80)))
    n = z.numerator // z.denominator                                                  # floor
    rem = z - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    return n - 113


# ---------------------------------------------------------------------------------------
# weight-blob layout and neural-LOD geometry: against the reference's own host code
# ---------------------------------------------------------------------------------------
def test_weight_layout_closed_form_and_fixture(ntc, oracle):
    with open(os.path.join(GOLDEN, "ref_layout.json")) as f:
        fixture = json.load(f)
    for name, weight_type in (("GenericInt8", ntc.abi.WEIGHTS_INT8), ("GenericFP8", ntc.abi.WEIGHTS_FP8)):
        spec = ntc.presets.spec_ref092()
        spec.weightType = weight_type
        layout = ntc.abi.WeightLayout()
        assert oracle.ntc_oracle_weight_layout(spec, layout) == 0
        fx = fixture[name]
        assert list(layout.weightOffset) == fx["weightOffset"]
        assert layout.bufferSize == fx["bufferSize"]
        for layer in range(4):
            if fx["scaleSize"][layer]:
                assert layout.scaleOffset[layer] == fx["scaleOffset"][layer]
            assert layout.biasOffset[layer] == fx["biasOffset"][layer]
    # totals from src/WeightLayout.cpp:184-265 for 48-64-48-32-16
    assert fixture["GenericInt8"]["bufferSize"] == 8192 + 4 * 160 + 4 * 160 == 9472
    assert fixture["GenericFP8"]["bufferSize"] == 7680 + 512 + 2 * 144 + 64 + 64 == 8608


def test_weight_layout_against_reference_build(ntc, oracle):
    ref = oracle_lib.load_ref()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    geo = (C.c_int * 8)()
    ref.ntc_ref_mlp_geometry(geo)
    spec = ntc.presets.spec_ref092()
    assert [geo[2 * i] for i in range(4)] == [spec.layer_inputs(i) for i in range(4)]
    assert [geo[2 * i + 1] for i in range(4)] == [spec.layer_outputs(i) for i in range(4)]
    for ref_type, weight_type in ((1, ntc.abi.WEIGHTS_INT8), (2, ntc.abi.WEIGHTS_FP8)):
        out = (C.c_uint64 * 25)()
        assert ref.ntc_ref_weight_layout(ref_type, out) == 0
        spec.weightType = weight_type
        layout = ntc.abi.WeightLayout()
        assert oracle.ntc_oracle_weight_layout(spec, layout) == 0
        assert list(layout.weightOffset) == list(out[0:4])
        assert layout.bufferSize == out[12]
        for layer in range(4):
            if out[17 + layer]:
                assert layout.scaleOffset[layer] == out[4 + layer]
            if out[21 + layer]:
                assert layout.biasOffset[layer] == out[8 + layer]


def test_product_layout_helper_matches_checker(ntc, oracle):
    lib = ntc.load_library()
    for spec in (ntc.presets.spec_ref092(), ntc.presets.spec_cfg01(), ntc.presets.spec_cfg2()):
        for wt in (ntc.abi.WEIGHTS_INT8, ntc.abi.WEIGHTS_FP8):
            spec.weightType = wt
            a, b = ntc.abi.WeightLayout(), ntc.abi.WeightLayout()
            assert oracle.ntc_oracle_weight_layout(spec, a) == 0
            assert lib.ntc_hip_weight_layout(spec, b) == 0
            assert bytes(a) == bytes(b)
    spec = ntc.presets.spec_cfg01()
    layout = ntc.synth.weight_layout(spec)
    assert layout.bufferSize == 9216 + 640 + 640 == 10496
    layout = ntc.synth.weight_layout(ntc.presets.spec_cfg2())
    assert layout.bufferSize == 7424 + 576 + 576 == 8576


GEOMETRY_CASES = [(4096, 4096, 13, 2), (4096, 4096, 13, 4), (2048, 1024, 12, 3), (1000, 600, 10, 5),
                  (512, 512, 1, 1), (64, 64, 7, 6), (8192, 8192, 14, 2), (300, 200, 4, 2), (16, 16, 5, 4)]


def _oracle_geometry(ntc, oracle, w, h, mips, gs, features=16):
    arr = (ntc.abi.MipDesc * 16)()
    total = C.c_uint64(0)
    n = oracle.ntc_oracle_ref_geometry(w, h, mips, gs, features, arr, C.byref(total))
    return n, arr, total.value


def test_ref_geometry_against_reference_build(ntc, oracle):
    ref = oracle_lib.load_ref()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    for (w, h, mips, gs) in GEOMETRY_CASES:
        n, arr, total = _oracle_geometry(ntc, oracle, w, h, mips, gs)
        # same neural-LOD count as FeatureGrid::Initialize (src/FeatureGridHost.cpp:34-38)
        n_ref = min(ref.ntc_ref_num_neural_mips(w, h, gs), ref.ntc_ref_lod_to_neural_lod(mips - 1, gs, 8) + 2)
        assert n == n_ref
        assert total == ref.ntc_ref_quantized_latents_size(w, h, mips, gs, 16)
        for m in range(mips):
            nlod = ref.ntc_ref_lod_to_neural_lod(m, gs, n_ref)
            assert arr[m].hrWidth == ref.ntc_ref_grid_dimension(w, nlod, gs)
            assert arr[m].hrHeight == ref.ntc_ref_grid_dimension(h, nlod, gs)
            assert arr[m].lrWidth == max(arr[m].hrWidth >> 1, 1)


def test_ref_geometry_fixture_and_product_host(ntc, oracle):
    with open(os.path.join(GOLDEN, "ref_geometry.json")) as f:
        fixture = json.load(f)
    for entry in fixture["cases"]:
        w, h, mips, gs = entry["width"], entry["height"], entry["mips"], entry["gridSizeScale"]
        n, arr, total = _oracle_geometry(ntc, oracle, w, h, mips, gs)
        assert n == entry["numNeuralMips"] and total == entry["latentBytes16"]
        pm, ptotal = ntc.presets.mips_ref092(ntc.presets.spec_ref092(), w, h, mips, gs)
        assert ptotal == total
        for m in range(mips):
            assert [arr[m].hrWidth, arr[m].hrHeight] == entry["hrDims"][m]
            for field in ("width", "height", "hrWidth", "hrHeight", "lrWidth", "lrHeight", "hrOffset", "lrOffset"):
                assert getattr(pm[m], field) == getattr(arr[m], field), (entry, m, field)
            assert np.float32(pm[m].positionScale) == np.float32(arr[m].positionScale)
            # log2f is not correctly rounded in every libm: numpy and glibc may differ by one ulp
            assert abs(pm[m].positionLod - arr[m].positionLod) <= 2e-7
    # the 4096^2, grid scale 2 table: mips 0-2 share neural LOD 0 with positionScale 1/4, 1/2, 1
    n, arr, _ = _oracle_geometry(ntc, oracle, 4096, 4096, 13, 2)
    assert [arr[m].hrWidth for m in range(13)] == [2048] * 3 + [512] * 2 + [128] * 2 + [32] * 6
    assert [arr[m].positionScale for m in range(4)] == [0.25, 0.5, 1.0, 0.5]
    assert arr[12].positionScale == 16.0 and arr[12].positionLod == 1.0


# ---------------------------------------------------------------------------------------
# latent fields
# ---------------------------------------------------------------------------------------
def test_unpack_is_inverse_of_pack_for_every_word(oracle):
    words = np.arange(65536, dtype=np.uint32)
    for bits in (4, 2):
        per = 16 // bits
        repacked = np.zeros_like(words)
        for i in range(per):
            field = np.array([oracle.ntc_oracle_unpack_field(int(w), i, bits) for w in words[::257]])   # sparse C check
            assert np.array_equal(field, (words[::257] >> (bits * i)) & ((1 << bits) - 1))
            repacked |= ((words >> (bits * i)) & ((1 << bits) - 1)) << (bits * i)
        assert np.array_equal(repacked, words)
    # one-hot: feature i of a BGRA4 word is nibble i (src/Quantizer.cu:520-523)
    for i in range(4):
        assert oracle.ntc_oracle_unpack_field(0xF << (4 * i), i, 4) == 15
        assert sum(oracle.ntc_oracle_unpack_field(0xF << (4 * i), j, 4) for j in range(4)) == 15
    # QuantizeValue o UnquantizeValue = id on every code (src/Quantizer.cu:482-495)
    for bits in (2, 4):
        levels = (1 << bits) - 1
        for q in range(levels + 1):
            assert oracle.ntc_oracle_quantize_value(np.float32(q) * (np.float32(1) / np.float32(levels)), bits) == q


# ---------------------------------------------------------------------------------------
# half / unorm8 conversions against numpy's IEEE float16
# ---------------------------------------------------------------------------------------
def test_half_conversions_exhaustive(oracle):
    all_bits = np.arange(65536, dtype=np.uint16)
    as_f32 = all_bits.view(np.float16).astype(np.float32)
    for b in range(0, 65536, 7):
        f = oracle.ntc_oracle_half_to_float(int(all_bits[b]))
        if np.isnan(as_f32[b]):
            assert np.isnan(f)
        else:
            assert np.float32(f) == as_f32[b] and np.signbit(np.float32(f)) == np.signbit(as_f32[b])
    rng = np.random.default_rng(1)
    samples = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10),
        np.exp2(rng.uniform(-30, 17, 20000)).astype(np.float32) * rng.choice([-1, 1], 20000).astype(np.float32),
        # exact ties between neighbouring halves and their float32 neighbours
        np.concatenate([[(a + b) / 2, np.nextafter(np.float32((a + b) / 2), np.float32(np.inf)),
                         np.nextafter(np.float32((a + b) / 2), np.float32(-np.inf))]
                        for a, b in zip(as_f32[1:2000:3].astype(np.float64), as_f32[2:2001:3].astype(np.float64))]).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, np.inf, -np.inf, 5.9604645e-08, 2.9802322e-08,
                  2.9802326e-08, 6.097555e-05, 6.1035156e-05], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        want = samples.astype(np.float16).view(np.uint16)
    got = np.array([oracle.ntc_oracle_float_to_half(float(s)) for s in samples], dtype=np.uint16)
    assert np.array_equal(got, want)
    # network outputs: Inf/NaN become zero (src/Inference.cu:125-126)
    for special in (np.inf, -np.inf, np.nan, 1e9):
        assert oracle.ntc_oracle_output_to_half(float(special)) == 0
    assert oracle.ntc_oracle_output_to_half(1.0) == 0x3C00


def test_unorm8_exhaustive_over_halves(oracle):
    all_bits = np.arange(65536, dtype=np.uint16)
    finite = (all_bits & 0x7C00) != 0x7C00
    want = np_decoder.half_bits_to_unorm8(all_bits[finite])
    got = np.array([oracle.ntc_oracle_half_to_unorm8(int(b)) for b in all_bits[finite]], dtype=np.uint8)
    assert np.array_equal(got, want)
    # ties k + 1/2 round away from zero (roundf), negatives clamp to 0, > 1 clamps to 255
    assert oracle.ntc_oracle_half_to_unorm8(int(np.float16(0.5 / 255).view(np.uint16))) in (0, 1)
    assert oracle.ntc_oracle_half_to_unorm8(int(np.float16(-3.0).view(np.uint16))) == 0
    assert oracle.ntc_oracle_half_to_unorm8(int(np.float16(7.0).view(np.uint16))) == 255
    assert oracle.ntc_oracle_half_to_unorm8(int(np.float16(1.0).view(np.uint16))) == 255


def test_unorm8_round_half_even_equals_roundf_on_every_half(oracle):
    """The decode kernel converts with the hardware's saturating round-to-nearest-EVEN conversion of the exact
    product v * 255; the definition rounds half away from zero.  They agree on every finite half: inside
    [0, 255] the only tie is v = 1/2 -> 127.5 -> 128 under both rules."""
    all_bits = np.arange(65536, dtype=np.uint16)
    finite = all_bits[(all_bits & 0x7C00) != 0x7C00]
    product = finite.view(np.float16).astype(np.float32) * np.float32(255.0)
    assert np.array_equal(product.astype(np.float64), finite.view(np.float16).astype(np.float64) * 255.0)   # exact in fp32
    half_even = np.clip(np.rint(product), 0, 255).astype(np.uint8)
    want = np.array([oracle.ntc_oracle_half_to_unorm8(int(b)) for b in finite], dtype=np.uint8)
    assert np.array_equal(half_even, want)
    ties = product[(product > 0) & (product < 255) & (product - np.floor(product) == 0.5)]
    assert ties.tolist() == [127.5]


# ---------------------------------------------------------------------------------------
# HGELU-clamp quantiser
# ---------------------------------------------------------------------------------------
def test_hgelu_constants_two_derivations():
    # constexpr chain of src/tin/tin_activation.h:112-121
    minval, maxval, bins = -3.0 / 16, 3.0, 256
    step = (maxval - minval) / (bins - 1)
    qmax = int(maxval / step)
    qmin = qmax - bins + 1
    bias = -(bins // 2) - qmin
    # literals of include/libntc/shaders/Inference.hlsli:37-39
    assert abs(1 / step - 80) < 1e-9 and qmax == 240 and qmin == -15 and bias == -113 and maxval == 3


def test_hgelu_quantize_exact_rational(oracle):
    rng = np.random.default_rng(2)
    xs = np.concatenate([
        rng.uniform(-2.0, 3.5, 3000), rng.standard_normal(1000) * 100, np.linspace(-1.6, -1.4, 201),
        np.array([-1.5, -0.75, 0.0, 1.5, 3.0, 2.9999998, 3.0000002, 1e30, -1e30, 1e-30, -1e-30]),
        # inputs whose y*80 lands on or next to a .5 tie
        np.array([np.sqrt(3 * (k + 0.5) / 80 + 9 / 16) - 0.75 for k in range(0, 30)]),
    ]).astype(np.float32)
    for x in xs:
        assert oracle.ntc_oracle_hgelu_quantize(float(x)) == hgelu_exact(x), x
    got = np.array([oracle.ntc_oracle_hgelu_quantize(float(x)) for x in np.linspace(-4, 5, 20001, dtype=np.float32)])
    assert got.min() == -128 and got.max() == 127                       # fits int8 exactly
    assert oracle.ntc_oracle_hgelu_quantize(-0.75) == -15 - 113         # minimum of HGELU: -3/16 -> -15
    assert oracle.ntc_oracle_hgelu_quantize(3.0) == 127 and oracle.ntc_oracle_hgelu_quantize(100.0) == 127
    assert oracle.ntc_oracle_hgelu_quantize(-1.5) == -113 and oracle.ntc_oracle_hgelu_quantize(-50.0) == -113
    assert oracle.ntc_oracle_hgelu_quantize(0.0) == -113
    up = got[np.linspace(-4, 5, 20001) >= -0.75]
    assert np.all(np.diff(up) >= 0)                                      # monotone right of the minimum
    assert np.array_equal(np_decoder.hgelu_quantize(xs), np.array([hgelu_exact(x) for x in xs], dtype=np.int8))


# ---------------------------------------------------------------------------------------
# positional encoding
# ---------------------------------------------------------------------------------------
def test_positional_encoding_closed_form(oracle):
    out = (C.c_int8 * 14)()
    for scale in (0.25, 0.5, 1.0, 2.0, 16.0, 0.3):
        for x in range(0, 40):
            for y in (0, 3, 17):
                oracle.ntc_oracle_encode_position(np.float32(x * scale), np.float32(y * scale), 0.75, 3, 2, out)
                px, py = Fraction(float(np.float32(x * scale))), Fraction(float(np.float32(y * scale)))
                for w in range(3):
                    for i, p in enumerate((px, py, px + Fraction(1, 4), py + Fraction(1, 4))):
                        p32 = Fraction(float(round_to_f32(p)))
                        fr = p32 - (p32.numerator // p32.denominator)
                        e = Fraction(float(round_to_f32(fr * 2 - 1)))
                        v = Fraction(float(round_to_f32(e * Fraction(255, 2))))
                        want = int(v) if v >= 0 else -int(-v)           # truncation toward zero
                        assert out[4 * w + i] == want, (scale, x, y, w, i)
                    px, py = px * 2, py * 2
                assert out[12] == out[13] == int(0.75 * 127.5)
    # period 1/positionScale texels for the first wave; all values inside [-127, 127]
    a, b = (C.c_int8 * 12)(), (C.c_int8 * 12)()
    oracle.ntc_oracle_encode_position(np.float32(5 * 0.25), np.float32(9 * 0.25), 0.0, 3, 0, a)
    oracle.ntc_oracle_encode_position(np.float32(9 * 0.25), np.float32(13 * 0.25), 0.0, 3, 0, b)
    assert list(a) == list(b)
    assert all(-127 <= v <= 127 for v in a)


# ---------------------------------------------------------------------------------------
# bilinear footprint
# ---------------------------------------------------------------------------------------
def test_bilinear_footprint_exact_and_wrap(oracle):
    xy, w = (C.c_int * 4)(), (C.c_float * 4)()
    for (W, gw) in ((64, 16), (64, 32), (8, 8), (4, 1), (1, 1), (100, 50), (30, 7)):
        for x in list(range(min(W, 6))) + [W - 1]:
            u = np.float32(np.float32(x) + np.float32(0.5)) / np.float32(W)
            oracle.ntc_oracle_bilinear_footprint(u, u, gw, gw, xy, w)
            p = Fraction(float(round_to_f32(Fraction(float(round_to_f32(Fraction(float(u)) * gw))) - Fraction(1, 2))))
            b = p.numerator // p.denominator
            d = Fraction(float(round_to_f32(p - b)))
            dn = Fraction(float(round_to_f32(1 - d)))
            assert xy[0] == b % gw and xy[2] == (b + 1) % gw and xy[1] == xy[0] and xy[3] == xy[2]
            want = [round_to_f32(dn * dn), round_to_f32(d * dn), round_to_f32(dn * d), round_to_f32(d * d)]
            assert [np.float32(v) for v in w] == want
            assert 0 <= xy[0] < gw and 0 <= xy[2] < gw
    # first texel of a 64-wide mip over a 16-wide grid: left tap wraps to the last column
    oracle.ntc_oracle_bilinear_footprint(np.float32(0.5 / 64), np.float32(0.5 / 64), 16, 16, xy, w)
    assert (xy[0], xy[2]) == (15, 0) and abs(sum(w) - 1.0) < 1e-6
    # same-size grid: texel centres coincide with cell centres, weight one on tap 00
    oracle.ntc_oracle_bilinear_footprint(np.float32(3.5 / 8), np.float32(5.5 / 8), 8, 8, xy, w)
    assert (xy[0], xy[1]) == (3, 5) and list(w) == [1.0, 0.0, 0.0, 0.0]


# ---------------------------------------------------------------------------------------
# end to end against the independent numpy decoder
# ---------------------------------------------------------------------------------------
ACTIVE = (-17.0, -12.0)


def _np_decode_case(ntc, case):
    layout = ntc.synth.weight_layout(case.spec)
    out = np.full(case.output_bytes, oracle_lib.HostSet.FILL, dtype=np.uint8)
    inputs = []
    for mip in case.mips:
        ins, outs = np_decoder.decode_mip(case.spec, layout, case.weights, case.latents, mip)
        np_decoder.store_mip(out, mip, outs, case.num_channels, case.output_format, case.pixel_stride)
        inputs.append(ins)
    return inputs, out


def test_e4m3_decode_exhaustive(oracle):
    all_bytes = np.arange(256, dtype=np.uint8)
    got = np.array([oracle.ntc_oracle_e4m3_times_512(int(b)) for b in all_bytes], dtype=np.int64)
    assert np.array_equal(got, np_decoder.e4m3_times_512(all_bytes))
    # known values of the OCP e4m3 grid: 1.0, largest finite 448, smallest subnormal 2^-9, smallest normal 2^-6
    assert got[0x38] == 512 and got[0x7E] == 448 * 512 and got[0x01] == 1 and got[0x08] == 8
    assert got[0xB8] == -512 and got[0x7F] == 0 and got[0xFF] == 0 and got[0x00] == 0 and got[0x80] == 0
    finite = np.delete(got, [0x7F, 0xFF])
    assert np.unique(finite).size == 253                      # 254 finite patterns, +0 and -0 coincide
    assert np.all(np.diff(got[:0x7F]) > 0)                    # positive half is strictly increasing
    # three 6-bit planes reassemble every weight exactly (what the device stages into LDS)
    c0, c1, c2 = got & 63, (got >> 6) & 63, got >> 12
    assert np.array_equal(4096 * c2 + 64 * c1 + c0, got) and c2.min() >= -64 and c2.max() <= 63


@pytest.mark.parametrize("name", ["cfg3_fp8_planar", "cfg3_fp8_ragged_unorm8", "cfg01_planar", "cfg01_fp16px", "cfg01_unorm8", "cfg2_unorm8", "ref16_gs2", "ref8_gs4",
                                  "ref12_gs3_ragged", "cfg01_ragged", "cfg01_default_scales"])
def test_oracle_against_numpy_decoder(ntc, oracle, name):
    A = ntc.abi
    make = {
        "cfg3_fp8_planar": lambda: cfg_case(ntc, ntc.presets.spec_cfg3(), 64, 64, 7, 16, A.OUT_FP16_PLANAR_PAIRS, 9, scale_log2_range=(-17.0, -13.0)),
        "cfg3_fp8_ragged_unorm8": lambda: cfg_case(ntc, ntc.presets.spec_cfg3(), 50, 30, 3, 11, A.OUT_UNORM8_PIXELS, 10, scale_log2_range=(-17.0, -13.0)),
        "cfg01_planar": lambda: cfg_case(ntc, ntc.presets.spec_cfg01(), 64, 64, 7, 16, A.OUT_FP16_PLANAR_PAIRS, 1, scale_log2_range=ACTIVE),
        "cfg01_fp16px": lambda: cfg_case(ntc, ntc.presets.spec_cfg01(), 64, 32, 7, 9, A.OUT_FP16_PIXELS, 2, scale_log2_range=ACTIVE),
        "cfg01_unorm8": lambda: cfg_case(ntc, ntc.presets.spec_cfg01(), 32, 64, 7, 16, A.OUT_UNORM8_PIXELS, 3, scale_log2_range=ACTIVE),
        "cfg2_unorm8": lambda: cfg_case(ntc, ntc.presets.spec_cfg2(), 64, 64, 3, 12, A.OUT_UNORM8_PIXELS, 4, scale_log2_range=ACTIVE),
        "ref16_gs2": lambda: ref_case(ntc, ntc.presets.spec_ref092(16), 128, 128, 8, 2, 16, A.OUT_FP16_PLANAR_PAIRS, 5, scale_log2_range=ACTIVE),
        "ref8_gs4": lambda: ref_case(ntc, ntc.presets.spec_ref092(8), 128, 64, 8, 4, 6, A.OUT_FP16_PLANAR_PAIRS, 6, scale_log2_range=ACTIVE),
        "ref12_gs3_ragged": lambda: ref_case(ntc, ntc.presets.spec_ref092(12), 100, 75, 5, 3, 8, A.OUT_UNORM8_PIXELS, 7, scale_log2_range=ACTIVE),
        "cfg01_ragged": lambda: cfg_case(ntc, ntc.presets.spec_cfg01(), 37, 21, 6, 5, A.OUT_FP16_PLANAR_PAIRS, 8, scale_log2_range=ACTIVE),
        "cfg01_default_scales": lambda: cfg_case(ntc, ntc.presets.spec_cfg01(), 64, 64, 2, 16, A.OUT_FP16_PLANAR_PAIRS, 0),
    }
    case = make[name]()
    host = case.host_set()
    host.decode(threads=4)
    inputs, want = _np_decode_case(ntc, case)
    # the int8 input vectors of a few texels per mip, then every output byte
    got_in = (C.c_int8 * 64)()
    got_out = (C.c_float * 64)()
    for m, mip in enumerate(case.mips):
        for (x, y) in {(0, 0), (mip.width - 1, mip.height - 1), (mip.width // 2, mip.height // 3)}:
            assert oracle.ntc_oracle_decode_texel(host.desc, m, x, y, got_out, got_in) == 0
            assert list(got_in[: case.spec.inputChannels]) == list(inputs[m][y, x]), (name, m, x, y)
    assert np.array_equal(host.output, want), name


def test_numpy_fma_is_single_rounding():
    rng = np.random.default_rng(3)
    a = rng.standard_normal(300).astype(np.float32)
    b = rng.standard_normal(300).astype(np.float32)
    c = (-(a.astype(np.float64) * b.astype(np.float64))).astype(np.float32) * np.float32(1.0000001)
    got = np_decoder.fma32(a, b, c)
    want = np.array([round_to_f32(Fraction(float(x)) * Fraction(float(y)) + Fraction(float(z))) for x, y, z in zip(a, b, c)])
    assert np.array_equal(got, want)
