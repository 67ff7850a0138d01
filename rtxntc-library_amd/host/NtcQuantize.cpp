// NtcQuantize.cpp - turns a float MLP into the GenericInt8 weight blob the decoder consumes, or into
// the GenericFP8 blob LibNTC stores beside it.
//
// Host-side counterpart of cuda::QuantizeNetwork / QuantizeColumnInt8 (reference
// src/Quantizer.cu:88-208,266-283): per output channel, symmetric 8-bit weights scaled by the
// channel's largest magnitude, and a (scale, integer bias) pair such that
//     float(bias_i32 + sum W_q * a) * scale
// equals the float layer on de-quantised operands, where layer-0 inputs are a/127.5
// (tin::InputQuant::scale, src/tin/tin_mlp.h:42) and hidden activations (a + 113)/80
// (ActHGELUClamp::step and ::bias, src/tin/tin_activation.h:112-121).
//
// The arithmetic below is IEEE binary32 in the order the reference writes it, including its use of
// two different but equivalent expressions for even and odd input indices.  The reference runs
// this under nvcc --use_fast_math, whose approximate reciprocal and division can differ in the
// last bit, so bit equality with the CUDA quantiser is not claimed; the meaning of the result is
// what the tests check.
#include "ntc_decode.h"

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <limits>
#include <vector>

namespace ntc
{
void SetQuantizeError(char const* fmt, ...);      // NtcHost.cpp: writes the thread's error message

namespace amd
{
namespace
{
float RoundHalfAway(float v) { return std::round(v); }      // CUDA round(): half away from zero

// One output channel of an int8 layer: weights, scale and integer bias (src/Quantizer.cu:88-208).
void QuantizeColumnInt8(FloatLayerDesc const& L, int l, int numLayers, int c, OutputChannelTransform const* outputTransforms,
                        int8_t* q, float& outScale, int32_t& outBias)
{
    int const rows = L.inputChannels;
    float const* w = L.weights + size_t(c) * size_t(rows);

    // src/Quantizer.cu:96-111
    float elemMin = std::numeric_limits<float>::max();
    float elemMax = std::numeric_limits<float>::min();
    for (int r = 0; r < rows; ++r) { elemMin = std::min(elemMin, w[r]); elemMax = std::max(elemMax, w[r]); }
    float const limit = std::max(std::fabs(elemMax), std::fabs(elemMin));
    float const ilimit = 1.f / limit;

    // src/Quantizer.cu:113-148
    float const scale = 127.5f, iscale = 1.f / 127.5f, qmin = -127.f, qmax = 127.f;
    int integerWeightSum = 0;
    for (int r = 0; r < rows; r += 2) {
        float x = RoundHalfAway(w[r] * scale * ilimit);
        x = std::max(std::min(x, qmax), qmin);
        float y = RoundHalfAway(w[r + 1] * (scale / limit));
        y = std::max(std::min(y, qmax), qmin);
        q[r] = int8_t(x);
        q[r + 1] = int8_t(y);
        integerWeightSum += int(q[r]) + int(q[r + 1]);
    }

    // src/Quantizer.cu:150-176
    float layerScale = limit * iscale;
    float layerBias = L.bias[c];
    if (l == 0) {
        layerScale /= 127.5f;
    } else {
        float const activationStep = (3.f - (-3.f / 16)) / 255.f;     // ActHGELUClamp::step = 1/80
        layerScale *= activationStep;
        layerBias -= float(integerWeightSum * -113) * layerScale;
        if (l == numLayers - 1 && outputTransforms) {
            layerScale *= outputTransforms[c].scale;
            layerBias = layerBias * outputTransforms[c].scale + outputTransforms[c].bias;
        }
    }

    // src/Quantizer.cu:178-206: (x * scale + bias) -> (x + int(bias/scale)) * scale; a zero scale
    // (constant channel) becomes 2^-16 with zero weights.
    // The reference computes with flush-to-zero (nvcc --use_fast_math): a scale below the smallest
    // normal float -- an all-zero weight row gives limit = FLT_MIN, see elemMax above -- counts as zero.
    if (std::fabs(layerScale) < std::numeric_limits<float>::min()) layerScale = 0.f;
    if (layerScale == 0.f) {
        layerScale = 1.f / 65536.f;
        outBias = int32_t(roundf(layerBias * 65536.f));
        std::memset(q, 0, size_t(rows));
    } else {
        outBias = int32_t(roundf(layerBias / layerScale));
    }
    outScale = layerScale;
}

// float -> IEEE binary16 bits, round to nearest even, overflow to infinity.
uint16_t FloatToHalfBits(float value)
{
    uint32_t f;
    std::memcpy(&f, &value, 4);
    uint32_t const sign = (f >> 16) & 0x8000u, magnitude = f & 0x7fffffffu;
    if (magnitude > 0x7f800000u) return uint16_t(sign | 0x7e00u);            // NaN
    if (magnitude >= 0x47800000u) return uint16_t(sign | 0x7c00u);           // 65536 and above, infinity
    if (magnitude < 0x33000000u) return uint16_t(sign);                      // below 2^-25: zero
    int const exponent = int(magnitude >> 23) - 127;
    uint32_t mantissa = (magnitude & 0x7fffffu) | 0x800000u;
    int const shift = exponent < -14 ? 13 + (-14 - exponent) : 13;           // subnormal halves lose more bits
    uint32_t const kept = mantissa >> shift, rest = mantissa & ((1u << shift) - 1u), half = 1u << (shift - 1);
    uint32_t bits = exponent < -14 ? kept : (uint32_t(exponent + 15) << 10) + (kept - 0x400u);
    if (rest > half || (rest == half && (bits & 1u))) ++bits;                // a carry into the exponent (or to infinity) is right
    return uint16_t(sign | bits);
}

bool ValidateLayers(FloatLayerDesc const* layers, int numLayers, size_t& weightBytes, size_t& channels)
{
    if (!layers) { SetQuantizeError("layers is NULL."); return false; }
    weightBytes = 0; channels = 0;
    for (int l = 0; l < numLayers; ++l) {
        FloatLayerDesc const& L = layers[l];
        if (!L.weights || !L.bias) { SetQuantizeError("Layer %d has a NULL weights or bias pointer.", l); return false; }
        weightBytes += size_t(std::max(L.inputChannels, 0)) * size_t(std::max(L.outputChannels, 0));
        channels += size_t(std::max(L.outputChannels, 0));
    }
    return true;
}
Status ValidateLayerShapes(FloatLayerDesc const* layers, int numLayers)
{
    for (int l = 0; l < numLayers; ++l) {
        FloatLayerDesc const& L = layers[l];
        if (L.inputChannels < 1 || L.outputChannels < 1 || (L.inputChannels & 1)) {
            SetQuantizeError("Layer %d: inputChannels (%d) must be positive and even, outputChannels (%d) positive.", l, L.inputChannels, L.outputChannels);
            return Status::OutOfRange;
        }
        if (l > 0 && L.inputChannels != layers[l - 1].outputChannels) {
            SetQuantizeError("Layer %d takes %d inputs but layer %d produces %d outputs.", l, L.inputChannels, l - 1, layers[l - 1].outputChannels);
            return Status::InvalidArgument;
        }
    }
    return Status::Ok;
}
} // namespace

// IEEE half -> OCP e4m3 byte, round to nearest even, saturating: magnitudes from 448 up (infinity
// included) become +-448, NaN becomes 0x7F | sign.  This is the conversion the reference's FP8
// quantiser applies to every hidden-layer weight (__nv_fp8x2_e4m3 of a half2: src/Quantizer.cu:225-229).
extern "C" uint8_t HalfToE4M3(uint16_t halfBits)
{
    uint32_t const sign = (halfBits >> 8) & 0x80u, magnitude = halfBits & 0x7fffu;
    if (magnitude > 0x7c00u) return uint8_t(sign | 0x7fu);                   // NaN
    if (magnitude >= 0x5f00u) return uint8_t(sign | 0x7eu);                  // 448 and above
    // e4m3: exponent bias 7, 3 mantissa bits; normal from 2^-6, subnormal step 2^-9.  Half: bias 15, 10 bits.
    int const exponent = int(magnitude >> 10) - 15;                          // unbiased; -15 marks a half subnormal (below 2^-14: far below e4m3's step)
    if (exponent < -10) return uint8_t(sign);                                // below 2^-10 = half of the smallest e4m3 step: zero
    uint32_t const mantissa = (magnitude & 0x3ffu) | 0x400u;                 // 11 bits, value = mantissa * 2^(exponent - 10)
    int const shift = exponent < -6 ? 7 + (-6 - exponent) : 7;               // bits dropped
    uint32_t const kept = mantissa >> shift, rest = mantissa & ((1u << shift) - 1u), half = 1u << (shift - 1);
    uint32_t bits = exponent < -6 ? kept : (uint32_t(exponent + 7) << 3) + (kept - 8u);
    if (rest > half || (rest == half && (bits & 1u))) ++bits;
    return uint8_t(sign | bits);
}

extern "C" Status QuantizeNetworkInt8(FloatLayerDesc const* layers, int numLayers, OutputChannelTransform const* outputTransforms,
    void* pOutBlob, size_t blobSize, size_t* pOutSize)
{
    if (numLayers != 4) { SetQuantizeError("numLayers (%d) must be 4.", numLayers); return Status::OutOfRange; }
    size_t weightBytes = 0, channels = 0;
    if (!ValidateLayers(layers, numLayers, weightBytes, channels)) return Status::InvalidArgument;
    if (Status st = ValidateLayerShapes(layers, numLayers); st != Status::Ok) return st;
    size_t const total = weightBytes + channels * 8;         // int8 weights, then fp32 scales, then int32 biases
    if (pOutSize) *pOutSize = total;
    if (!pOutBlob) { SetQuantizeError("pOutBlob is NULL."); return Status::InvalidArgument; }
    if (blobSize < total) { SetQuantizeError("The blob needs %zu bytes, %zu were provided.", total, blobSize); return Status::OutOfRange; }

    int8_t* weightOut = static_cast<int8_t*>(pOutBlob);
    std::vector<float> scales(channels);
    std::vector<int32_t> biases(channels);
    size_t channelBase = 0;
    for (int l = 0; l < numLayers; ++l) {
        FloatLayerDesc const& L = layers[l];
        for (int c = 0; c < L.outputChannels; ++c)
            QuantizeColumnInt8(L, l, numLayers, c, outputTransforms, weightOut + size_t(c) * size_t(L.inputChannels),
                               scales[channelBase + size_t(c)], biases[channelBase + size_t(c)]);
        weightOut += size_t(L.inputChannels) * size_t(L.outputChannels);
        channelBase += size_t(L.outputChannels);
    }
    std::memcpy(static_cast<uint8_t*>(pOutBlob) + weightBytes, scales.data(), channels * 4);
    std::memcpy(static_cast<uint8_t*>(pOutBlob) + weightBytes + channels * 4, biases.data(), channels * 4);
    return Status::Ok;
}

// GenericFP8 blob (src/WeightLayout.cpp:51-71,249-262): the matrices of all layers, one byte per weight
// (e4m3 for the hidden layers, int8 for the output layer), then the fp16 biases of the hidden layers,
// then the output layer's fp32 scales and int32 biases.  Hidden layers as QuantizeColumnFP8 does them
// (src/Quantizer.cu:210-252): each weight rounded to half and on to e4m3, the bias stored as half; the
// output layer exactly as in the Int8 blob (its inputs are int8 activations in both modes).
extern "C" Status QuantizeNetworkFP8(FloatLayerDesc const* layers, int numLayers, OutputChannelTransform const* outputTransforms,
    void* pOutBlob, size_t blobSize, size_t* pOutSize)
{
    if (numLayers != 4) { SetQuantizeError("numLayers (%d) must be 4.", numLayers); return Status::OutOfRange; }
    size_t weightBytes = 0, channels = 0;
    if (!ValidateLayers(layers, numLayers, weightBytes, channels)) return Status::InvalidArgument;
    if (Status st = ValidateLayerShapes(layers, numLayers); st != Status::Ok) return st;
    FloatLayerDesc const& last = layers[numLayers - 1];
    size_t const hiddenChannels = channels - size_t(last.outputChannels);
    size_t const total = weightBytes + hiddenChannels * 2 + size_t(last.outputChannels) * 8;
    if (pOutSize) *pOutSize = total;
    if (!pOutBlob) { SetQuantizeError("pOutBlob is NULL."); return Status::InvalidArgument; }
    if (blobSize < total) { SetQuantizeError("The blob needs %zu bytes, %zu were provided.", total, blobSize); return Status::OutOfRange; }

    uint8_t* const blob = static_cast<uint8_t*>(pOutBlob);
    uint8_t* weightOut = blob;
    uint8_t* biasOut = blob + weightBytes;
    for (int l = 0; l < numLayers - 1; ++l) {
        FloatLayerDesc const& L = layers[l];
        size_t const count = size_t(L.inputChannels) * size_t(L.outputChannels);
        for (size_t i = 0; i < count; ++i) weightOut[i] = HalfToE4M3(FloatToHalfBits(L.weights[i]));
        weightOut += count;
        for (int c = 0; c < L.outputChannels; ++c) {
            uint16_t const h = FloatToHalfBits(L.bias[c]);
            std::memcpy(biasOut, &h, 2);
            biasOut += 2;
        }
    }
    std::vector<float> scales(size_t(last.outputChannels));
    std::vector<int32_t> biases(size_t(last.outputChannels));
    for (int c = 0; c < last.outputChannels; ++c)
        QuantizeColumnInt8(last, numLayers - 1, numLayers, c, outputTransforms, reinterpret_cast<int8_t*>(weightOut) + size_t(c) * size_t(last.inputChannels),
                           scales[size_t(c)], biases[size_t(c)]);
    std::memcpy(biasOut, scales.data(), scales.size() * 4);
    std::memcpy(biasOut + scales.size() * 4, biases.data(), biases.size() * 4);
    return Status::Ok;
}

} // namespace amd
} // namespace ntc
