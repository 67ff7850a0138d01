"""Seeded synthetic latents and weight blobs (there are no .ntc sample files to decode).

Distributions follow the benchmark description: latent codes uniform over the code range;
int8 weights uniform in [-127, 127]; per-channel fp32 scale log-uniform in [2^-10, 2^-4];
fp32 bias ~ N(0, 0.1), stored the way the reference's quantiser stores a float bias:
bias_i32 = roundf(bias / scale) (src/Quantizer.cu:202).
"""
import numpy as np

from . import abi


def make_latents(total_bytes, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 65536, size=total_bytes // 2, dtype=np.uint16)


def weight_layout(spec):
    """Offsets of the blob pieces, from the library's own host-side layout helper."""
    lib = abi.load_library()
    layout = abi.WeightLayout()
    abi.check(lib.ntc_hip_weight_layout(spec, layout))
    return layout


def e4m3_encode(values):
    """float array -> OCP e4m3 bytes, round to nearest (ties to even), saturating at +-448; no NaNs produced."""
    v = np.asarray(values, dtype=np.float64)
    a = np.minimum(np.abs(v), 448.0)
    exponent = np.maximum(np.floor(np.log2(np.maximum(a, 2.0 ** -20))), -6.0)
    quantum = np.exp2(exponent - 3.0)
    a = np.minimum(np.rint(a / quantum) * quantum, 448.0)          # rint: ties to even on the 3-bit grid
    exponent = np.maximum(np.floor(np.log2(np.maximum(a, 2.0 ** -20))), -6.0)      # rounding may have reached the next binade
    normal = a >= 2.0 ** -6
    e = np.where(normal, exponent + 7, 0).astype(np.int64)
    m = np.where(normal, a / np.exp2(exponent) * 8.0 - 8.0, a * 512.0).astype(np.int64)
    return ((np.signbit(v).astype(np.int64) << 7) | (e << 3) | m).astype(np.uint8)


def make_fp8_weights(spec, seed, weight_sigma=0.35, bias_sigma=0.3, out_scale_log2_range=(-14.0, -11.0)):
    """The GenericFP8 blob (reference src/WeightLayout.cpp:51-71) for `spec` (weightType FP8): e4m3 hidden-layer
    weights ~ N(0, weight_sigma / sqrt(fan-in) * 4) (weight_sigma: one value, or one per hidden layer), fp16
    biases ~ N(0, bias_sigma), and an int8 output layer."""
    assert spec.weightType == abi.WEIGHTS_FP8
    layout = weight_layout(spec)
    rng = np.random.default_rng(seed)
    blob = np.zeros(layout.bufferSize, dtype=np.uint8)
    last = abi.MLP_LAYERS - 1
    for layer in range(abi.MLP_LAYERS):
        n_in, n_out = spec.layer_inputs(layer), spec.layer_outputs(layer)
        at = layout.weightOffset[layer]
        if layer < last:
            sigma = weight_sigma[layer] if isinstance(weight_sigma, (tuple, list)) else weight_sigma
            w = rng.normal(0.0, sigma * 4.0 / np.sqrt(n_in), size=(n_out, n_in))
            blob[at:at + n_in * n_out] = e4m3_encode(w).reshape(-1)
            bias = rng.normal(0.0, bias_sigma, size=n_out).astype(np.float16)
            blob[layout.biasOffset[layer]:layout.biasOffset[layer] + 2 * n_out] = bias.view(np.uint8)
        else:
            w = rng.integers(-127, 128, size=(n_out, n_in), dtype=np.int8)
            scale = np.exp2(rng.uniform(out_scale_log2_range[0], out_scale_log2_range[1], size=n_out)).astype(np.float32)
            bias = rng.integers(-40000, 40000, size=n_out).astype(np.int32)
            blob[at:at + n_in * n_out] = w.reshape(-1).view(np.uint8)
            blob[layout.scaleOffset[layer]:layout.scaleOffset[layer] + 4 * n_out] = scale.view(np.uint8)
            blob[layout.biasOffset[layer]:layout.biasOffset[layer] + 4 * n_out] = bias.view(np.uint8)
    return blob


def make_weights(spec, seed, scale_log2_range=(-10.0, -4.0), bias_sigma=0.1, layout=None):
    """Returns the int8 weight blob (uint8 array) for `spec`."""
    assert spec.weightType in (abi.WEIGHTS_INT8, abi.WEIGHTS_FP8_SCALED)
    fp8 = spec.weightType == abi.WEIGHTS_FP8_SCALED
    layout = layout or weight_layout(spec)
    rng = np.random.default_rng(seed)
    blob = np.zeros(layout.bufferSize, dtype=np.uint8)
    for layer in range(abi.MLP_LAYERS):
        n_in, n_out = spec.layer_inputs(layer), spec.layer_outputs(layer)
        if fp8 and layer < abi.MLP_LAYERS - 1:
            # uniform over the 254 finite e4m3 bit patterns; the blob's scale is per unit of w/512
            w = rng.integers(0, 254, size=(n_out, n_in)).astype(np.uint8)
            w = (w + (w >= 127)).astype(np.uint8).view(np.int8)       # skip 0x7f; 0xff is never reached
            unit = np.float32(1.0 / 512.0)
        else:
            w = rng.integers(-127, 128, size=(n_out, n_in), dtype=np.int8)
            unit = np.float32(1.0)
        scale = np.exp2(rng.uniform(scale_log2_range[0], scale_log2_range[1], size=n_out)).astype(np.float32) * unit
        bias = rng.normal(0.0, bias_sigma, size=n_out).astype(np.float32)
        q = (bias / scale).astype(np.float32).astype(np.float64)
        bias_i32 = np.trunc(q + np.copysign(0.5, q)).astype(np.int32)      # roundf
        blob[layout.weightOffset[layer]:layout.weightOffset[layer] + n_in * n_out] = w.reshape(-1).view(np.uint8)
        blob[layout.scaleOffset[layer]:layout.scaleOffset[layer] + 4 * n_out] = scale.view(np.uint8)
        blob[layout.biasOffset[layer]:layout.biasOffset[layer] + 4 * n_out] = bias_i32.view(np.uint8)
    return blob
