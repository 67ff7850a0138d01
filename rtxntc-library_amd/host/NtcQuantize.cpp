// NtcQuantize.cpp - turns a float MLP into the GenericInt8 weight blob the decoder consumes.
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

namespace
{
float RoundHalfAway(float v) { return std::round(v); }      // CUDA round(): half away from zero
}

extern "C" Status QuantizeNetworkInt8(FloatLayerDesc const* layers, int numLayers, OutputChannelTransform const* outputTransforms,
    void* pOutBlob, size_t blobSize, size_t* pOutSize)
{
    if (!layers) { SetQuantizeError("layers is NULL."); return Status::InvalidArgument; }
    if (numLayers != 4) { SetQuantizeError("numLayers (%d) must be 4.", numLayers); return Status::OutOfRange; }
    size_t weightBytes = 0, channels = 0;
    for (int l = 0; l < numLayers; ++l) {
        FloatLayerDesc const& L = layers[l];
        if (!L.weights || !L.bias) { SetQuantizeError("Layer %d has a NULL weights or bias pointer.", l); return Status::InvalidArgument; }
        if (L.inputChannels < 1 || L.outputChannels < 1 || (L.inputChannels & 1)) {
            SetQuantizeError("Layer %d: inputChannels (%d) must be positive and even, outputChannels (%d) positive.", l, L.inputChannels, L.outputChannels);
            return Status::OutOfRange;
        }
        if (l > 0 && L.inputChannels != layers[l - 1].outputChannels) {
            SetQuantizeError("Layer %d takes %d inputs but layer %d produces %d outputs.", l, L.inputChannels, l - 1, layers[l - 1].outputChannels);
            return Status::InvalidArgument;
        }
        weightBytes += size_t(L.inputChannels) * size_t(L.outputChannels);
        channels += size_t(L.outputChannels);
    }
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
        int const rows = L.inputChannels;
        for (int c = 0; c < L.outputChannels; ++c) {
            float const* w = L.weights + size_t(c) * size_t(rows);
            int8_t* q = weightOut + size_t(c) * size_t(rows);

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
            int32_t integerLayerBias;
            if (layerScale == 0.f) {
                layerScale = 1.f / 65536.f;
                integerLayerBias = int32_t(roundf(layerBias * 65536.f));
                std::memset(q, 0, size_t(rows));
            } else {
                integerLayerBias = int32_t(roundf(layerBias / layerScale));
            }
            scales[channelBase + size_t(c)] = layerScale;
            biases[channelBase + size_t(c)] = integerLayerBias;
        }
        weightOut += size_t(rows) * size_t(L.outputChannels);
        channelBase += size_t(L.outputChannels);
    }
    std::memcpy(static_cast<uint8_t*>(pOutBlob) + weightBytes, scales.data(), channels * 4);
    std::memcpy(static_cast<uint8_t*>(pOutBlob) + weightBytes + channels * 4, biases.data(), channels * 4);
    return Status::Ok;
}

} // namespace ntc
