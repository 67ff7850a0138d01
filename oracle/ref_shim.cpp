/*
 * ref_shim.cpp - C entry points over the host-only pieces of the real LibNTC sources.
 *
 * TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/libntc_ref_host.so
 * together with the reference's own src/FeatureGridMath.cpp, src/WeightLayout.cpp and
 * src/CoopVecWeightConverter.cpp, compiled where they lie (nothing is copied).  It lets the
 * tests compare the restated layout / geometry code with what the reference computes, and
 * lets tests/golden/make_ref_fixtures.py write those answers down as fixtures.
 *
 * The CUDA kernels (src/Inference.cu and what it includes) need nvcc, CUDA headers and
 * tensor-core PTX and are not buildable here; only these two host files are.
 */
#include "WeightLayout.h"
#include "FeatureGridMath.h"
#include "MlpDesc.h"
#include <cstdint>

namespace {
// CalculateNumNeuralMipLevels is protected in the reference class.
struct GridMathAccess : ntc::FeatureGridMath {
    static int NumNeuralMips(int w, int h, int gs) { return CalculateNumNeuralMipLevels(w, h, gs); }
};
}

extern "C" {

// weightType: 1 = GenericInt8, 2 = GenericFP8 (ntc::InferenceWeightType).
// out[0..3] weight offsets, [4..7] scale offsets, [8..11] bias offsets, [12] buffer size,
// [13..16] weight sizes, [17..20] scale sizes, [21..24] bias sizes.
int ntc_ref_weight_layout(int weightType, uint64_t* out)
{
    ntc::WeightLayout layout;
    if (!ntc::MakeQuantizedWeightLayout(nullptr, ntc::InferenceWeightType(weightType), layout))
        return -1;
    for (int l = 0; l < NTC_MLP_LAYERS; ++l) {
        out[l]      = layout.weights[l].offset;
        out[4 + l]  = layout.scales[l].offset;
        out[8 + l]  = layout.biases[l].offset;
        out[13 + l] = layout.weights[l].size;
        out[17 + l] = layout.scales[l].size;
        out[21 + l] = layout.biases[l].size;
    }
    out[12] = layout.bufferSize;
    return 0;
}

void ntc_ref_mlp_geometry(int* out)
{
    for (int l = 0; l < NTC_MLP_LAYERS; ++l) {
        out[2 * l]     = ntc::MlpDesc::GetLayerInputChannels(l);
        out[2 * l + 1] = ntc::MlpDesc::GetLayerOutputChannels(l);
    }
}

int ntc_ref_lod_to_neural_lod(int lod, int gridScale, int neuralLods)
{
    return ntc::FeatureGridMath::LodToNeuralLod(lod, gridScale, neuralLods);
}

int ntc_ref_grid_dimension(int imageDimension, int neuralLod, int gridScale)
{
    return ntc::FeatureGridMath::GetGridDimension(imageDimension, neuralLod, gridScale);
}

int ntc_ref_num_neural_mips(int w, int h, int gridScale)
{
    return GridMathAccess::NumNeuralMips(w, h, gridScale);
}

uint64_t ntc_ref_quantized_latents_size(int w, int h, int mips, int gridScale, int numFeatures)
{
    return ntc::FeatureGridMath::CalculateQuantizedLatentsSize(w, h, mips, gridScale, numFeatures);
}

} // extern "C"
