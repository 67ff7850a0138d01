"""What scale and bias in an int8 weight blob MEAN.

The decoder only sees the blob; the reference's encoder-side quantiser
(QuantizeColumnInt8, src/Quantizer.cu:88-208) defines how a float layer (weights w, bias b, inputs in
[-1, 1] quantised by tin::InputQuant, hidden activations quantised by ActHGELUClamp to steps of 1/80
starting at -15/80) turns into (W_q, scale, bias_i32).  This test restates that quantiser in numpy,
quantises random float layers with it, and checks that the checker's integer layer
    r = float(bias_i32 + sum W_q * a) * scale                       (Inference.hlsli:148-165)
reproduces the float layer evaluated on the de-quantised operands,
    r = b + sum w~ * a~,   a~ = a/127.5 (inputs) or (a + 113)/80 (hidden activations),
to within the rounding of the stored bias (half a scale step).  A dropped -113 offset, a wrong
activation step or input scale, a bias added after scaling, or a transposed weight matrix all fail it.
"""
import numpy as np
import pytest


def quantize_layer_int8(w, b, input_layer):
    """w: float32 [in][out], b: float32 [out] -> (W_q int8 [out][in], scale f32 [out], bias_i32 [out], w~ [in][out])."""
    n_in, n_out = w.shape
    wq = np.zeros((n_out, n_in), dtype=np.int8)
    scale = np.zeros(n_out, dtype=np.float32)
    bias_i = np.zeros(n_out, dtype=np.int32)
    w_deq = np.zeros_like(w)
    for c in range(n_out):
        col = w[:, c].astype(np.float32)
        limit = np.float32(max(abs(col.max()), abs(col.min())))                # Quantizer.cu:99-111
        # even input indices: (w * 127.5) * (1 / limit); odd ones: w * (127.5 / limit)   (Quantizer.cu:125-133)
        q = np.empty(n_in, dtype=np.float32)
        q[0::2] = (col[0::2] * np.float32(127.5)).astype(np.float32) * (np.float32(1) / limit)
        q[1::2] = col[1::2] * (np.float32(127.5) / limit)
        q = np.where(q >= 0, np.floor(q + np.float32(0.5)), np.ceil(q - np.float32(0.5)))   # round(): half away from zero
        q = np.clip(q, -127, 127)                                              # Quantizer.cu:116-131
        wq[c] = q.astype(np.int8)
        iscale = np.float32(1) / np.float32(127.5)                             # `1 / scale`, a float constant (:117)
        w_deq[:, c] = ((q.astype(np.float32) * limit).astype(np.float32) * iscale).astype(np.float32)
        layer_scale = limit * iscale
        layer_bias = np.float32(b[c])
        if input_layer:
            layer_scale = layer_scale / np.float32(127.5)                      # tin::InputQuant::scale, :157-160
        else:
            layer_scale = layer_scale * np.float32(3.1875 / 255)               # ActHGELUClamp::step = 1/80
            layer_bias = layer_bias - np.float32(int(q.sum()) * -113) * layer_scale      # :163-164
        scale[c] = layer_scale
        t = np.float64(np.float32(layer_bias) / np.float32(layer_scale))       # float division, then roundf (:202)
        bias_i[c] = int(np.floor(t + 0.5) if t >= 0 else np.ceil(t - 0.5))
    return wq, scale, bias_i, w_deq


@pytest.mark.parametrize("n_in,n_out,input_layer", [(64, 64, True), (48, 64, True), (64, 48, False), (48, 32, False), (32, 16, False)])
def test_integer_layer_equals_dequantised_float_layer(oracle, n_in, n_out, input_layer):
    rng = np.random.default_rng(n_in * 100 + n_out)
    w = (rng.standard_normal((n_in, n_out)) * 0.3).astype(np.float16).astype(np.float32)
    b = (rng.standard_normal(n_out) * 0.2).astype(np.float16).astype(np.float32)
    wq, scale, bias_i, w_deq = quantize_layer_int8(w, b, input_layer)
    assert np.abs(wq).max() == 127
    for trial in range(50):
        if input_layer:
            a = rng.integers(-127, 128, n_in).astype(np.int8)
            a_real = a.astype(np.float64) / 127.5
        else:
            a = rng.integers(-128, 128, n_in).astype(np.int8)
            a_real = (a.astype(np.float64) + 113) / 80.0
            assert a_real.min() >= -15 / 80 and a_real.max() <= 3.0
        r = np.zeros(n_out, dtype=np.float32)
        wq_c, scale_c, bias_c = np.ascontiguousarray(wq), np.ascontiguousarray(scale), np.ascontiguousarray(bias_i)
        oracle.ntc_oracle_layer_int8(wq_c.ctypes.data, scale_c.ctypes.data, bias_c.ctypes.data, n_in, n_out, a.ctypes.data, r.ctypes.data)
        want = b.astype(np.float64) + a_real @ w_deq.astype(np.float64)
        tol = 0.5 * scale.astype(np.float64) * 1.001 + 2e-6 * (1 + np.abs(want))
        assert np.all(np.abs(r.astype(np.float64) - want) <= tol), (trial, np.abs(r - want).max(), tol.min())


# ---- the host library's quantiser (rtxntc-library_amd/host/NtcQuantize.cpp) ------------------------

import ctypes as C
import os

HOST_LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "rtxntc-library_amd", "host", "libntc.so")


class FloatLayerDesc(C.Structure):
    _fields_ = [("inputChannels", C.c_int), ("outputChannels", C.c_int), ("weights", C.c_void_p), ("bias", C.c_void_p)]


class OutputChannelTransform(C.Structure):
    _fields_ = [("scale", C.c_float), ("bias", C.c_float)]


def host_lib():
    lib = C.CDLL(HOST_LIB)
    lib.QuantizeNetworkInt8.restype = C.c_int
    lib.QuantizeNetworkInt8.argtypes = [C.POINTER(FloatLayerDesc), C.c_int, C.POINTER(OutputChannelTransform), C.c_void_p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.GetLastErrorMessage.restype = C.c_char_p
    return lib


def float_network(rng, widths):
    """Random float MLP with fp16-representable values: [(w [in][out], b [out])]."""
    layers = []
    for n_in, n_out in zip(widths[:-1], widths[1:]):
        w = (rng.standard_normal((n_in, n_out)) * (1.5 / np.sqrt(n_in))).astype(np.float16).astype(np.float32)
        b = (rng.standard_normal(n_out) * 0.2).astype(np.float16).astype(np.float32)
        layers.append((w, b))
    return layers


def quantize_with_host_library(lib, layers, transforms=None):
    descs = (FloatLayerDesc * len(layers))()
    keep = []
    for d, (w, b) in zip(descs, layers):
        rows = np.ascontiguousarray(w.T)                  # the library takes weights[out][in]
        bias = np.ascontiguousarray(b)
        keep += [rows, bias]
        d.inputChannels, d.outputChannels, d.weights, d.bias = w.shape[0], w.shape[1], rows.ctypes.data, bias.ctypes.data
    size = C.c_size_t(0)
    t = None
    if transforms is not None:
        t = (OutputChannelTransform * len(transforms))(*[OutputChannelTransform(s, o) for s, o in transforms])
    assert lib.QuantizeNetworkInt8(descs, len(layers), t, None, 0, C.byref(size)) == 10      # InvalidArgument, size reported
    blob = np.zeros(size.value, dtype=np.uint8)
    assert lib.QuantizeNetworkInt8(descs, len(layers), t, blob.ctypes.data, blob.size, None) == 0, lib.GetLastErrorMessage()
    return blob


@pytest.mark.parametrize("widths", [(64, 64, 48, 32, 16), (48, 64, 48, 32, 16), (64, 48, 48, 32, 16)])
def test_host_quantiser_equals_the_numpy_restatement(widths):
    """Bit equality: both follow src/Quantizer.cu:88-208 operation by operation in IEEE binary32."""
    lib = host_lib()
    rng = np.random.default_rng(sum(widths))
    layers = float_network(rng, widths)
    blob = quantize_with_host_library(lib, layers)
    weight_bytes = sum(a * b for a, b in zip(widths[:-1], widths[1:]))
    channels = sum(widths[1:])
    assert blob.size == weight_bytes + 8 * channels
    w_at, c_at = 0, 0
    for index, (w, b) in enumerate(layers):
        wq, scale, bias_i, _ = quantize_layer_int8(w, b, index == 0)
        n_in, n_out = w.shape
        assert np.array_equal(blob[w_at: w_at + n_in * n_out].view(np.int8).reshape(n_out, n_in), wq), index
        assert np.array_equal(blob[weight_bytes + 4 * c_at: weight_bytes + 4 * (c_at + n_out)].view(np.float32), scale), index
        assert np.array_equal(blob[weight_bytes + 4 * channels + 4 * c_at: weight_bytes + 4 * channels + 4 * (c_at + n_out)].view(np.int32), bias_i), index
        w_at += n_in * n_out
        c_at += n_out


def test_host_quantiser_special_cases_and_errors():
    lib = host_lib()
    rng = np.random.default_rng(3)
    widths = (64, 64, 48, 32, 16)
    layers = float_network(rng, widths)
    layers[3][0][:, 5] = 0.0                                     # a constant output channel: zero scale
    layers[3][1][5] = 0.25
    transforms = [(1.0, 0.0)] * 16
    transforms[2] = (0.5, 0.125)                                 # optimal-to-linear mapping of channel 2
    transforms[7] = (0.0, 0.75)                                  # a constant image channel maps with scale 0
    blob = quantize_with_host_library(lib, layers, transforms)
    plain = quantize_with_host_library(lib, layers)
    weight_bytes, channels = 9216, 160
    scale = blob[weight_bytes: weight_bytes + 4 * channels].view(np.float32)
    bias = blob[weight_bytes + 4 * channels:].view(np.int32)
    w3 = blob[64 * 64 + 64 * 48 + 48 * 32: weight_bytes].view(np.int8).reshape(16, 32)
    assert scale[144 + 5] == np.float32(1 / 65536) and bias[144 + 5] == 16384 and not w3[5].any()     # Quantizer.cu:181-198
    assert scale[144 + 7] == np.float32(1 / 65536) and bias[144 + 7] == 49152 and not w3[7].any()
    plain_scale = plain[weight_bytes: weight_bytes + 4 * channels].view(np.float32)
    assert scale[144 + 2] == np.float32(plain_scale[144 + 2] * np.float32(0.5))
    # (x + bias_i) * scale of the transformed channel = 0.5 * (plain value) + 0.125 at x = 0, to half a step
    plain_bias = plain[weight_bytes + 4 * channels:].view(np.int32)
    assert abs(bias[144 + 2] * float(scale[144 + 2]) - (0.5 * plain_bias[144 + 2] * float(plain_scale[144 + 2]) + 0.125)) <= float(scale[144 + 2])
    # argument errors
    descs = (FloatLayerDesc * 4)()
    assert lib.QuantizeNetworkInt8(descs, 3, None, None, 0, None) == 16 and b"numLayers" in lib.GetLastErrorMessage()
    assert lib.QuantizeNetworkInt8(None, 4, None, None, 0, None) == 10
    assert lib.QuantizeNetworkInt8(descs, 4, None, None, 0, None) == 10 and b"NULL" in lib.GetLastErrorMessage()


def test_quantised_network_tracks_the_float_network(ntc, oracle):
    """End to end on the checker: quantise a float MLP with the host library, decode a small texture
    set with the blob, and compare with the float MLP evaluated on the same (de-quantised) inputs.
    Quantisation noise only: a few steps of 1/80 through three hidden layers."""
    lib = host_lib()
    rng = np.random.default_rng(11)
    widths = (64, 64, 48, 32, 16)
    layers = float_network(rng, widths)
    blob = quantize_with_host_library(lib, layers)
    from cases import cfg_case
    spec = ntc.presets.spec_cfg01()
    case = cfg_case(ntc, spec, 32, 32, 1, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=12, weights=blob)
    host = case.host_set()
    host.decode(threads=4)
    got = host.output.view(np.float16).astype(np.float64).reshape(32, 8, 32, 2).transpose(0, 2, 1, 3).reshape(32, 32, 16)
    # float network on the same int8 inputs
    import np_decoder
    layout = ntc.synth.weight_layout(spec)
    inputs, _ = np_decoder.decode_mip(spec, layout, blob, case.latents.view(np.uint16), case.mips[0])
    x = inputs.reshape(-1, 64).astype(np.float64) / 127.5
    for index, (w, b) in enumerate(layers):
        x = x @ w.astype(np.float64) + b.astype(np.float64)
        if index < 3:
            x = np.minimum(x, 3.0) * np.clip(x / 3.0 + 0.5, 0.0, 1.0)
    want = x.reshape(32, 32, 16)
    err = np.abs(got - want)
    assert err.max() < 0.15 and err.mean() < 0.02, (err.max(), err.mean())


@pytest.mark.gpu
@pytest.mark.parametrize("preset", ["cfg01", "ref092"])
def test_gpu_decode_with_a_quantised_float_network(ntc, device, preset):
    """A blob produced by the host quantiser (realistic scales and biases, unlike the synthetic
    blobs of the other tests) decodes bit-exactly."""
    from cases import cfg_case, ref_case, first_mismatch
    lib = host_lib()
    rng = np.random.default_rng(21)
    if preset == "cfg01":
        blob = quantize_with_host_library(lib, float_network(rng, (64, 64, 48, 32, 16)))
        case = cfg_case(ntc, ntc.presets.spec_cfg01(), 512, 256, 6, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=22, weights=blob)
    else:
        blob = quantize_with_host_library(lib, float_network(rng, (48, 64, 48, 32, 16)))
        case = ref_case(ntc, ntc.presets.spec_ref092(16), 512, 256, 6, 2, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=23, weights=blob)
    host = case.host_set()
    host.decode(threads=8)
    dset = case.device_set(device)
    device.decode([dset])
    device.synchronize()
    assert first_mismatch(host.output, case.d_output.download()) is None


def test_half_to_e4m3_is_round_to_nearest_even_saturating(oracle):
    """Every half against the textbook statement: the nearest of the 253 distinct finite e4m3 values
    (decoded by the checker's table, itself pinned against the OCP definition), ties to the even
    code, magnitudes from 448 up and infinities to +-448, NaN to the NaN code."""
    lib = host_lib()
    lib.HalfToE4M3.restype = C.c_uint8
    lib.HalfToE4M3.argtypes = [C.c_uint16]
    codes = np.arange(0x7F, dtype=np.int64)                                  # 0x00 .. 0x7E: non-negative finite codes, ascending
    values = np.array([oracle.ntc_oracle_e4m3_times_512(int(c)) for c in codes], dtype=np.float64) / 512.0
    assert np.all(np.diff(values) > 0) and values[-1] == 448.0
    halves = np.arange(0x7C01, dtype=np.uint16)                              # 0 .. +inf
    x = halves.view(np.float16).astype(np.float64)
    hi = np.clip(np.searchsorted(values, x, side="left"), 0, len(values) - 1)   # first code with value >= x
    lo = np.clip(hi - 1, 0, len(values) - 1)
    d_lo, d_hi = np.abs(x - values[lo]), np.abs(values[hi] - x)
    want = np.where(d_lo < d_hi, lo, np.where(d_hi < d_lo, hi, np.where(lo % 2 == 0, lo, hi)))
    want = np.where(x >= 448.0, 0x7E, want)
    got = np.array([lib.HalfToE4M3(int(h)) for h in halves], dtype=np.int64)
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:10]
    # sign symmetry, NaN
    for h in (0x0001, 0x1400, 0x3C00, 0x5EFF, 0x5F00, 0x7BFF, 0x7C00):
        assert lib.HalfToE4M3(h | 0x8000) == (lib.HalfToE4M3(h) | 0x80)
    assert lib.HalfToE4M3(0x7E00) == 0x7F and lib.HalfToE4M3(0xFE00) == 0xFF


@pytest.mark.parametrize("widths", [(48, 64, 48, 32, 16), (64, 64, 48, 32, 16)])
def test_host_fp8_quantiser_blob(widths, oracle):
    """GenericFP8 blob: e4m3 weights + fp16 biases for the hidden layers, the Int8 blob's output layer;
    layout sizes against the reference's own WeightLayout (oracle/_ref) for the 48-64-48-32-16 network."""
    import oracle_lib
    lib = host_lib()
    lib.QuantizeNetworkFP8.restype = C.c_int
    lib.QuantizeNetworkFP8.argtypes = lib.QuantizeNetworkInt8.argtypes
    lib.HalfToE4M3.restype = C.c_uint8
    lib.HalfToE4M3.argtypes = [C.c_uint16]
    rng = np.random.default_rng(sum(widths) + 1)
    layers = float_network(rng, widths)
    layers[1][0][0, :4] = [500.0, -1000.0, 447.9, 2.0 ** -11]               # saturation and underflow
    int8_blob = quantize_with_host_library(lib, layers)
    descs = (FloatLayerDesc * 4)()
    keep = []
    for d, (w, b) in zip(descs, layers):
        wt = np.ascontiguousarray(w.T, dtype=np.float32)
        bb = np.ascontiguousarray(b, dtype=np.float32)
        keep += [wt, bb]
        d.inputChannels, d.outputChannels, d.weights, d.bias = w.shape[0], w.shape[1], wt.ctypes.data, bb.ctypes.data
    size = C.c_size_t()
    assert lib.QuantizeNetworkFP8(descs, 4, None, None, 0, size) == 10       # InvalidArgument: no blob, but the size is reported
    weight_bytes = sum(a * b for a, b in zip(widths[:-1], widths[1:]))
    hidden = sum(widths[1:-1])
    assert size.value == weight_bytes + 2 * hidden + 8 * widths[-1]
    ref = oracle_lib.load_ref()
    if ref is not None and widths[0] == 48:
        out = (C.c_uint64 * 25)()
        assert ref.ntc_ref_weight_layout(2, out) == 0                        # InferenceWeightType::GenericFP8
        assert size.value == out[12] == 8608
    blob = np.zeros(size.value, dtype=np.uint8)
    assert lib.QuantizeNetworkFP8(descs, 4, None, blob.ctypes.data, blob.size, None) == 0, lib.GetLastErrorMessage()
    w_at, b_at = 0, weight_bytes
    for index, (w, b) in enumerate(layers[:-1]):
        n_in, n_out = w.shape
        halves = np.ascontiguousarray(w.T).astype(np.float16).view(np.uint16).reshape(-1)
        want = np.array([lib.HalfToE4M3(int(h)) for h in halves], dtype=np.uint8)
        assert np.array_equal(blob[w_at: w_at + n_in * n_out], want), index
        # and what the bytes mean: within half an e4m3 step of the weight (relative 1/16 for normal values)
        decoded = np.array([oracle.ntc_oracle_e4m3_times_512(int(c)) for c in want], dtype=np.float64) / 512.0
        exact = np.clip(np.ascontiguousarray(w.T).reshape(-1).astype(np.float64), -448, 448)
        assert np.all(np.abs(decoded - exact) <= np.maximum(np.abs(exact) / 16, 2.0 ** -10) + 1e-12), index
        assert np.array_equal(blob[b_at: b_at + 2 * n_out].view(np.float16), b.astype(np.float16)), index
        w_at += n_in * n_out
        b_at += 2 * n_out
    # output layer: the Int8 blob's weights, scales and biases
    n_in, n_out = layers[-1][0].shape
    channels = sum(widths[1:])
    assert np.array_equal(blob[w_at: w_at + n_in * n_out], int8_blob[w_at: w_at + n_in * n_out])
    int8_scales = int8_blob[weight_bytes + 4 * (channels - n_out): weight_bytes + 4 * channels]
    int8_biases = int8_blob[weight_bytes + 4 * channels + 4 * (channels - n_out):]
    assert np.array_equal(blob[b_at: b_at + 4 * n_out], int8_scales)
    assert np.array_equal(blob[b_at + 4 * n_out:], int8_biases)
