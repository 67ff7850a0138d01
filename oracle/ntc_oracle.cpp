/*
 * ntc_oracle.cpp - CPU restatement of LibNTC's texture-set decode arithmetic (Int8 and FP8 networks).
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP decoder is compared
 * against; nothing in the shipped library links, loads or calls it.  Only tests, the
 * smoke check and the CPU-baseline leg of the benchmark may use it.
 *
 * It is scalar, one texel at a time, and follows the reference line by line in
 * meaning (not in code).  Each function names the reference lines it restates.
 * All paths are relative to the LibNTC 0.9.2 tree.
 *
 * Arithmetic contract (what "bit-exact" means for the GPU path):
 *   - every float operation is IEEE binary32, round-to-nearest-even, evaluated in the
 *     order written here; a fused multiply-add happens exactly where fmaf() is written
 *     (build with -ffp-contract=off);
 *   - integer accumulation is exact int32;
 *   - float -> int conversions say which rounding they use (floor / trunc / nearest-even).
 *
 * Pinning status of each function is listed in the table at the end of this header.
 *
 *   function                 pinned by (tests/test_oracle_pins.py unless another file is named)
 *   -----------------------  -----------------------------------------------------------
 *   weight_layout            reference build oracle/_ref (MakeQuantizedWeightLayout) +
 *                            committed fixture tests/golden/ref_layout.json + closed-form totals
 *   ref_geometry             reference build oracle/_ref (FeatureGridMath) + fixture
 *                            tests/golden/ref_geometry.json
 *   unpack (latent fields)   Pack o Unpack = id over all 65536 words; bit positions by one-hot
 *   bilinear / concat        integer cross-check in exact rational arithmetic for dyadic
 *                            positions; d = 0 special case; wrap at both borders enumerated
 *   pos-enc                  closed form, periodicity, range
 *   hgelu_quantize           constants re-derived two ways (constexpr chain of
 *                            src/tin/tin_activation.h:112-121 vs literals of
 *                            Inference.hlsli:37-39); exhaustive monotone pieces and range checks
 *   layer matmul             numpy int64 GEMM
 *   half / unorm8 convert    numpy float16 (IEEE RNE) over all 2^16 halves and a dense fp32 sweep
 *   e4m3_times_512           the OCP e4m3 definition evaluated in numpy over all 256 bytes
 *   layer_fp8_weights        numpy int64 GEMM on the decoded weights (tests/np_decoder.py)
 *   scale/bias semantics     a numpy restatement of QuantizeColumnInt8 (src/Quantizer.cu:88-208)
 *   (layer_int8)             must be reproduced by layer_int8 to quantisation error
 *                            (tests/test_quantizer_semantics.py)
 *   end-to-end decode        an independent numpy restatement (tests/np_decoder.py) on small sets
 *   decode_queries           the raster decode of the texels the queries hit (tests/test_queries.py)
 *   read_channels,           numpy models of the 1:1 branch of cuda::CopyImage, five channel
 *   write_channels           formats, padded rows, vertical flip (tests/test_host_api.py)
 *   resampling copies        numpy float64 bilinear resampling with clamped edges (to fp32 rounding);
 *   (read/write_channels_    exact cases: a 2x reduction is the mean of each 2x2 block added in
 *   resized, resize_planar)  tap order, same-size calls equal the 1:1 functions, a constant image
 *                            stays constant (tests/test_resampling.py)
 *   image_loss,              numpy float64 mean squared error, with the mask options restated from
 *   image_loss_masked        src/Inference.cu:80-112 in numpy and three special cases: no zero in the
 *                            mask = no mask, all masked = mask channel only, clamp idempotent
 *                            (tests/test_host_api.py)
 *   image_difference         numpy float64 mean squared error / mean squared log error over the
 *                            extent, to the fp32 accumulation error; the fixed-point split on
 *                            values with an exact binary expansion (tests/test_image_difference.py).
 *                            The reference does not define the order of a workgroup's additions,
 *                            so its exact low bits are parity unpinned by construction.
 *   block_compress (BC4/5)   the format's standard decoder in numpy: blocks of at most two distinct
 *                            values and exact ramps decode exactly, the decoded error of random
 *                            blocks never exceeds that of the start endpoints and stays within
 *                            half a palette step + 1 (tests/test_block_compress.py).  The choices
 *                            of the reference's shader compiler (fused multiply-adds in the
 *                            least-squares fit) are not known: parity with its exact blocks is
 *                            unpinned; blocks are valid BC4 by construction.
 *   block_compress (BC1/2/3) the single-colour endpoint tables, regenerated from their rule, equal
 *                            the reference's literal tables entry by entry; the BC1 decoder in
 *                            numpy: constant blocks within 2.6/255, blocks of two 5:6:5 colours
 *                            exact, transparent texels decode transparent, smaller error than a
 *                            plain bounding-box encoder; BC2 alpha against its closed form, BC3
 *                            alpha against the BC4 encoder (tests/test_block_compress_color.py).
 *                            HLSL leaves dot / lerp / fusion to the shader compiler: the float
 *                            operation order here is a choice, parity with the reference's exact
 *                            blocks is unpinned.
 *   block_compress (BC6H)    its deterministic log2 / exp2 against numpy's (2.5e-7 relative); a BC6H
 *                            decoder written from the specification for the three modes emitted:
 *                            constant blocks within one 10-bit endpoint step, 4-bit ramps to 2 %,
 *                            two-region blocks in the two-subset modes, out-of-range texels clamped
 *                            (tests/test_block_compress_bc6.py).  The shader's transcendental
 *                            functions are hardware approximations: parity with its exact blocks is
 *                            unpinned.
 *   block_compress (BC7)     partition and anchor tables, typed from the BPTC specification, equal
 *                            the reference's; a BC7 decoder written from the specification in
 *                            numpy: every emitted block is valid and decodes close to its source
 *                            (constant colours, alpha 0 / 1, one- / two- / three-region blocks,
 *                            against BC1), each mode decodable when forced, and the single-mode
 *                            path reproduces the full search's blocks
 *                            (tests/test_block_compress_bc7.py).  Float operation order as for
 *                            BC1: parity with the reference's exact blocks is unpinned.
 *   FP8 network              parity with the reference's own bits is UNPINNED by construction: its e4m3
 *   (decode_texel_fp8,       matrix-vector products are left to the graphics driver (cooperative vectors) or run
 *   layer_e4m3, hgelu_half,  as FP16 WMMA with half accumulation in CUDA.  The deterministic reading implemented
 *   half_to_e4m3, inputs)    here is pinned by: brute force over the 127 non-negative e4m3 values for every half;
 *                            numpy's IEEE double -> half conversion; the fp16 activation in numpy float64 with one
 *                            rounding per operation over every half plus closed forms; exact rational dot products
 *                            (python integers) for the layer; closed forms of the input vector; an independent
 *                            numpy restatement end to end (tests/test_fp8_network.py, tests/np_decoder.py).
 *   The exact bits of the reference's FP16-WMMA CUDA kernel (half accumulation order,
 *   --use_fast_math) and of a hardware bilinear sampler are NOT reproduced: parity unpinned
 *   for those two, by construction; the integer contract of Inference.hlsli is what is pinned.
 */
#include "../include/ntc_hip.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

namespace {

// ---------------------------------------------------------------------------------------
// Half-precision conversions (IEEE 754 binary16, round-to-nearest-even), done on the bits
// so the result does not depend on the host's conversion instructions.
// Reference use: __float22half2_rn stores of src/Inference.cu:121-135.
// ---------------------------------------------------------------------------------------
inline uint32_t f32_bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float bits_f32(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

uint16_t float_to_half_rne(float f)
{
    uint32_t const x = f32_bits(f);
    uint32_t const sign = (x >> 16) & 0x8000u;
    uint32_t const absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u)                       // Inf or NaN
        return uint16_t(sign | 0x7c00u | (absx > 0x7f800000u ? 0x200u : 0u));
    if (absx >= 0x477ff000u)                       // >= 65520 rounds to Inf
        return uint16_t(sign | 0x7c00u);
    if (absx < 0x33000001u)                        // <= 2^-25 rounds to zero (tie goes to even = 0)
        return uint16_t(sign);
    int32_t const exp = int32_t(absx >> 23) - 127;
    uint32_t mant = (absx & 0x7fffffu) | 0x800000u; // 24-bit significand
    int shift;                                      // bits dropped from the significand
    uint32_t halfExpField;
    if (exp < -14) { shift = 13 + (-14 - exp); halfExpField = 0; }   // subnormal half
    else           { shift = 13;               halfExpField = uint32_t(exp + 15); }
    uint32_t const kept = mant >> shift;
    uint32_t const rem  = mant & ((1u << shift) - 1u);
    uint32_t const halfway = 1u << (shift - 1);
    uint32_t r = kept;
    if (rem > halfway || (rem == halfway && (kept & 1u))) r += 1;
    // For normals `kept` still holds the implicit bit (0x400); adding the exponent field
    // shifted makes a mantissa carry bump the exponent correctly.
    uint32_t out;
    if (halfExpField == 0) out = r;                                  // may carry into exp=1: correct
    else                   out = ((halfExpField - 1) << 10) + r;     // r includes the 0x400 bit
    return uint16_t(sign | out);
}

float half_to_float(uint16_t h)
{
    uint32_t const sign = uint32_t(h & 0x8000u) << 16;
    uint32_t const exp = (h >> 10) & 0x1fu;
    uint32_t const mant = h & 0x3ffu;
    if (exp == 0) {
        if (mant == 0) return bits_f32(sign);
        float const v = float(mant) * 0x1p-24f;   // exact
        return (sign ? -v : v);
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (mant << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (mant << 13));
}

// IsHalfSpecial, src/CudaUtils.h:30-35: exponent field all ones.
inline bool half_is_special(uint16_t h) { return (h & 0x7c00u) == 0x7c00u; }

// The value Inference.cu stores for one output: network output as fp16, Inf/NaN replaced
// by zero (src/Inference.cu:123-126).  Channel scale/bias are identity on the decode
// path (src/TextureSet.cpp:1726-1729).
inline uint16_t output_to_half(float o)
{
    uint16_t h = float_to_half_rne(o);
    if (half_is_special(h)) h = 0;
    return h;
}

// WriteImageChannel, UNORM8 case, no dithering, linear colour space
// (src/ImageProcessing.cu:146-149): roundf = round half away from zero, then clamp.
// The source of that copy is the fp16 image Decompress wrote, so the value is rounded
// to half first.
inline uint8_t half_to_unorm8(uint16_t h)
{
    float const v = half_to_float(h) * 255.f;     // exact: 11-bit x 8-bit significands
    float r = std::trunc(v);
    float const frac = v - r;                     // exact
    if (frac >= 0.5f) r += 1.f; else if (frac <= -0.5f) r -= 1.f;
    r = std::max(0.f, std::min(255.f, r));
    return uint8_t(r);
}

// ---------------------------------------------------------------------------------------
// Weight blob layout: MakeQuantizedWeightLayout for GenericInt8 and GenericFP8
// (src/WeightLayout.cpp:142-268; prose :42-71).
// ---------------------------------------------------------------------------------------
int layer_inputs(NtcHipDecoderSpec const& s, int layer)
{
    return layer == 0 ? s.inputChannels : s.hiddenChannels[layer - 1];   // src/MlpDesc.h:57-75
}
int layer_outputs(NtcHipDecoderSpec const& s, int layer)
{
    return layer == NTC_HIP_MLP_LAYERS - 1 ? s.outputChannels : s.hiddenChannels[layer]; // src/MlpDesc.h:78-99
}

bool weight_layout(NtcHipDecoderSpec const& s, NtcHipWeightLayout& L)
{
    std::memset(&L, 0, sizeof(L));
    uint32_t off = 0;
    for (int l = 0; l < NTC_HIP_MLP_LAYERS; ++l) {           // all matrices, 1 byte per weight, back to back
        L.weightOffset[l] = off;
        off += uint32_t(layer_inputs(s, l) * layer_outputs(s, l));
    }
    if (s.weightType == NTC_HIP_WEIGHTS_INT8 || s.weightType == NTC_HIP_WEIGHTS_FP8_SCALED) {
        for (int l = 0; l < NTC_HIP_MLP_LAYERS; ++l) {       // all fp32 scale vectors ...
            L.scaleOffset[l] = off;
            off += 4u * uint32_t(layer_outputs(s, l));
        }
        for (int l = 0; l < NTC_HIP_MLP_LAYERS; ++l) {       // ... then all int32 bias vectors
            L.biasOffset[l] = off;
            off += 4u * uint32_t(layer_outputs(s, l));
        }
    } else if (s.weightType == NTC_HIP_WEIGHTS_FP8) {
        for (int l = 0; l < NTC_HIP_MLP_LAYERS - 1; ++l) {   // fp16 bias of the fp8 layers, no scale
            L.biasOffset[l] = off;
            off += 2u * uint32_t(layer_outputs(s, l));
        }
        int const last = NTC_HIP_MLP_LAYERS - 1;             // int8 output layer: fp32 scale, int32 bias
        L.scaleOffset[last] = off; off += 4u * uint32_t(layer_outputs(s, last));
        L.biasOffset[last]  = off; off += 4u * uint32_t(layer_outputs(s, last));
    } else {
        return false;
    }
    L.bufferSize = off;
    return true;
}

// ---------------------------------------------------------------------------------------
// Latent fields.  PackLatentsKernel stores feature i of a layer at bits [4i, 4i+4) of a
// u16 (src/Quantizer.cu:519-523); UnquantizeValue(q, bits) = q / (2^bits - 1)
// (src/Quantizer.cu:490-495) takes the width as a parameter, so a 2-bit grid holds 8
// features per u16, feature i at bits [2i, 2i+2).
// ---------------------------------------------------------------------------------------
inline int unpack_field(uint16_t word, int index, int bits)
{
    return (word >> (index * bits)) & ((1 << bits) - 1);
}

struct Grid {
    uint16_t const* base; int width, height, features, bits;
    int fetch(int x, int y, int f) const
    {
        int const perWord = 16 / bits;
        size_t const layer = size_t(f / perWord);
        uint16_t const w = base[(layer * size_t(height) + size_t(y)) * size_t(width) + size_t(x)];
        return unpack_field(w, f % perWord, bits);
    }
};

struct Footprint { int x0, y0, x1, y1; float w00, w10, w01, w11; };

// FeatureGrid::SetupBilinearFilter, src/FeatureGridDevice.h:33-58 (weights kept in fp32:
// the int8 contract samples in float, Inference.hlsli:62-87).
Footprint bilinear_footprint(float u, float v, int gw, int gh)
{
    float const x = u * float(gw) - 0.5f;
    float const y = v * float(gh) - 0.5f;
    float const fx = std::floor(x), fy = std::floor(y);
    float const dx = x - fx, dy = y - fy;
    float const dxn = 1.f - dx, dyn = 1.f - dy;
    Footprint fp;
    fp.w00 = dxn * dyn; fp.w10 = dx * dyn; fp.w01 = dxn * dy; fp.w11 = dx * dy;
    int xb = int(fx), yb = int(fy);
    if (xb < 0) xb += gw;                      // wrap addressing
    if (yb < 0) yb += gh;
    fp.x0 = xb % gw;       fp.y0 = yb % gh;
    fp.x1 = (xb + 1) % gw; fp.y1 = (yb + 1) % gh;
    return fp;
}

// One grid's contribution to the int8 input vector.
//  bilinear: Inference.hlsli:72-82 - the sampler returns s = t/(2^bits-1) with t the
//    filtered code; the shader takes floor(s*255 - 128).  With t kept un-normalised that
//    is floor(t * 255/(2^bits-1)) - 128 (255/15 = 17, 255/3 = 85, both exact).
//  concat 2x2: the four taps a00,a01,a10,a11 of FeatureGridDevice.h:67-70, unfiltered,
//    each code mapped by the same affine map (a tap with weight one).
// Slots beyond `features` stay zero (mask of Inference.hlsli:76-80).
void sample_grid(Grid const& g, int mode, int slots, float u, float v, int8_t* out)
{
    Footprint const fp = bilinear_footprint(u, v, g.width, g.height);
    float const codeScale = 255.f / float((1 << g.bits) - 1);
    if (mode == NTC_HIP_GRID_BILINEAR) {
        for (int f = 0; f < g.features; ++f) {
            float const q00 = float(g.fetch(fp.x0, fp.y0, f));
            float const q10 = float(g.fetch(fp.x1, fp.y0, f));
            float const q01 = float(g.fetch(fp.x0, fp.y1, f));
            float const q11 = float(g.fetch(fp.x1, fp.y1, f));
            float t = fp.w00 * q00;
            t = std::fmaf(fp.w10, q10, t);
            t = std::fmaf(fp.w01, q01, t);
            t = std::fmaf(fp.w11, q11, t);
            out[f] = int8_t(int(std::floor(t * codeScale)) - 128);
        }
    } else {
        int const xs[4] = { fp.x0, fp.x1, fp.x0, fp.x1 };
        int const ys[4] = { fp.y0, fp.y0, fp.y1, fp.y1 };
        for (int tap = 0; tap < 4; ++tap)
            for (int f = 0; f < g.features; ++f)
                out[tap * slots + f] = int8_t(g.fetch(xs[tap], ys[tap], f) * int(codeScale) - 128);
    }
}

// NtcEvaluatePositionalEncoding + NtcEncodeSamplePosition, Inference.hlsli:89-120
// (CUDA twin: src/RegressionKernels.h:59-85).  int(float) truncates toward zero.
inline float frac_hlsl(float x) { return x - std::floor(x); }

void encode_position(float px, float py, float lod, int waves, int lodInputs, int8_t* out)
{
    int idx = 0;
    for (int w = 0; w < waves; ++w) {
        float const e[4] = {
            frac_hlsl(px) * 2.f - 1.f, frac_hlsl(py) * 2.f - 1.f,
            frac_hlsl(px + 0.25f) * 2.f - 1.f, frac_hlsl(py + 0.25f) * 2.f - 1.f };
        for (int i = 0; i < 4; ++i) out[idx++] = int8_t(int(e[i] * 127.5f));
        px *= 2.f; py *= 2.f;
    }
    for (int i = 0; i < lodInputs; ++i) out[idx++] = int8_t(int(lod * 127.5f));
}

// NtcHGELUClamp_ForwardFloat + _QuantizeFloat, Inference.hlsli:36-39,123-131:
//   y = min(x,3) * saturate(mad(x, 0.333333, 0.5));  q = int(round(y*80) + (-113)).
// HLSL round() is round-half-to-even; mad is taken as fused.
inline int hgelu_quantize(float x)
{
    float t = std::fmaf(x, 0.333333f, 0.5f);
    t = std::min(std::max(t, 0.f), 1.f);
    float const y = std::min(x, 3.f) * t;
    float const r = std::nearbyintf(y * 80.f);   // default rounding mode = nearest-even
    return int(r + -113.f);
}

// NtcEvaluateLayerINT8, Inference.hlsli:133-182: acc starts at the int32 bias, adds
// dot4add_i8packed products, then float(acc) * scale.  W is [out][in] row-major
// (Inference.hlsli:153, src/Quantizer.cu:144).
void layer_int8(int8_t const* W, float const* scale, int32_t const* bias,
                int in, int out, int8_t const* x, float* r)
{
    for (int c = 0; c < out; ++c) {
        int32_t acc = bias[c];
        for (int k = 0; k < in; ++k) acc += int32_t(x[k]) * int32_t(W[c * in + k]);
        r[c] = float(acc) * scale[c];
    }
}

// OCP FP8 e4m3 (sign, 4 exponent bits with bias 7, 3 mantissa bits; no infinities, the all-ones
// pattern is NaN): the weight format of the reference's FP8 layers (src/Quantizer.cu:210-252 stores
// __nv_fp8_e4m3 bytes; src/tin/tin_activation.h:44-81 describes the same grid, max 448).
// Returned as the exact integer 512*value (smallest subnormal 2^-9 -> 1, largest 448 -> 229376).
int32_t e4m3_times_512(uint8_t byte)
{
    int const e = (byte >> 3) & 15, m = byte & 7;
    if ((byte & 0x7f) == 0x7f) return 0;                       // NaN encodings decode as zero
    int32_t const mag = (e == 0) ? m : ((8 + m) << (e - 1));
    return (byte & 0x80) ? -mag : mag;
}

// A hidden layer with e4m3 weights: the dot product of an fp32-accumulating implementation,
// taken without accumulation noise - the exact sum of (512 w)*x in int32 (wrapping like the
// device's accumulators), converted to float once, times the per-channel scale.
void layer_fp8_weights(int32_t const* W512 /* 512*w, decoded once per set */, float const* scale, int32_t const* bias,
                       int in, int out, int8_t const* x, float* r)
{
    for (int c = 0; c < out; ++c) {
        int64_t acc = bias[c];
        for (int k = 0; k < in; ++k) acc += int64_t(x[k]) * int64_t(W512[c * in + k]);
        r[c] = float(int32_t(uint32_t(uint64_t(acc)))) * scale[c];
    }
}

// ---------------------------------------------------------------------------------------
// The FP8 network: NtcSampleTextureSet_CoopVec_FP8 and what it calls
// (include/libntc/shaders/InferenceCoopVec.hlsli:22-124,127-160,235-309,312-398), with the weight blob of
// src/WeightLayout.cpp:51-71 (e4m3 matrices and fp16 biases for the three hidden layers, the int8 output
// layer).  The shader hands e4m3 matrix-vector products to the driver ("cooperative vectors"): rounding of
// the inputs to e4m3, accumulation order and precision, fusion inside the fp16 activation are NOT defined
// by the reference - parity with any particular driver is unpinned by construction.  What is implemented
// here is one deterministic reading, stated operation by operation:
//   inputs   latent feature: t = the fp32 bilinear filter of the codes (the same chain as the int8
//            contract), v = fma(t, 2/15, -1) (the sampler's t/15, then *2 - 1 of hlsli:40), half(v);
//            positional encoding and lod: half of the fp32 values of Inference.hlsli:89-120; every input
//            is then rounded to e4m3 (round-to-nearest-even, the grid of src/tin/tin_activation.h:44-81
//            including its subnormals, saturating at 448), which is how the driver reads an fp16 vector
//            as FloatE4M3 (hlsli:244,266);
//   layer    the exact dot product of e4m3 weights and e4m3 inputs is accumulated in three parts by the
//            bits of |512 w| (bits 14.., 7..13, 0..6: each part's sum is exactly representable in fp32),
//            r = ((s2 + s1) + s0) + float(bias_fp16) with three fp32 additions, x = half(r);
//   HGELU    in fp16 as NtcHGELUClamp_Forward_CoopVec writes it: t = sat(fma(x, half(1/3), 1/2)) (one
//            rounding), y = half(clamp(x, -3, 3) * t) - the lower clamp changes nothing where t > 0 and
//            keeps -inf * 0 out; a NaN x gives 0;
//   between  hidden layers: y rounded to e4m3; after the last one: q = rne(80 y - 113), the int8 input of
//            the output layer (hlsli:143-148,333-334), computed exactly and rounded once;
//   output   acc = bias_i32 + sum W_i8 q exactly, o = float(acc) * scale (hlsli:333-345).
// ---------------------------------------------------------------------------------------
uint16_t double_to_half_rne(double d)                        // one rounding, ties to even, overflow to infinity
{
    if (std::isnan(d)) return 0x7e00;
    uint16_t const sign = std::signbit(d) ? 0x8000 : 0;
    double const a = std::fabs(d);
    if (a >= 65520.0) return uint16_t(sign | 0x7c00);
    if (a == 0.0) return sign;
    int e;
    (void)std::frexp(a, &e);                                 // a = m * 2^e, m in [0.5, 1)
    int const exponent = std::max(e - 1, -14);               // of the half's binade (subnormals share -14)
    double const quantum = std::ldexp(1.0, exponent - 10);
    double const q = std::nearbyint(a / quantum);            // exact division, default rounding = nearest-even
    return uint16_t(sign | float_to_half_rne(float(q * quantum)));       // q * quantum has at most 12 bits: exact
}
inline double half_value(uint16_t h) { return double(half_to_float(h)); }
uint16_t half_fma(uint16_t a, uint16_t b, uint16_t c) { return double_to_half_rne(half_value(a) * half_value(b) + half_value(c)); }   // exact in double

// IEEE half -> the integer 512 * (nearest e4m3 value): round to nearest, ties to even, on the e4m3 grid
// (3 mantissa bits from 2^-6 up, steps of 2^-9 below), magnitudes from 464 up (and infinities) saturate
// at 448; NaN gives 0.
int32_t half_to_e4m3_times_512(uint16_t h)
{
    if ((h & 0x7fffu) > 0x7c00u) return 0;
    double const a = std::fabs(half_value(h));
    double r;
    if (a >= 464.0) r = 448.0;                               // 464 = midpoint of 448 and the absent 480: ties go to the even 448... and beyond saturates
    else {
        int e;
        (void)std::frexp(a, &e);
        int const exponent = a == 0.0 ? -6 : std::max(e - 1, -6);
        double const quantum = std::ldexp(1.0, exponent - 3);
        r = std::min(std::nearbyint(a / quantum) * quantum, 448.0);
    }
    int32_t const v = int32_t(r * 512.0);
    return (h & 0x8000u) ? -v : v;
}

constexpr uint16_t kHalfThird = 0x3555, kHalfOneHalf = 0x3800;     // half(1/3) = 0.33325195, 1/2

// x (fp16 layer output) -> y (fp16): NtcHGELUClamp_Forward_CoopVec, hlsli:150-153
uint16_t hgelu_half(uint16_t x)
{
    if ((x & 0x7fffu) > 0x7c00u) return 0;
    double t = half_value(half_fma(x, kHalfThird, kHalfOneHalf));      // +-inf stay +-inf, then saturate
    t = std::min(std::max(t, 0.0), 1.0);
    double const xc = std::min(std::max(half_value(x), -3.0), 3.0);
    return double_to_half_rne(xc * t);
}

struct Fp8Layers {                                           // decoded once per set
    std::vector<int32_t> w512;                               // 512 * w of the three e4m3 matrices, blob order
    void prepare(NtcHipTextureSet const& set, NtcHipWeightLayout const& layout)
    {
        uint8_t const* blob = static_cast<uint8_t const*>(set.weights);
        w512.resize(layout.weightOffset[NTC_HIP_MLP_LAYERS - 1]);
        for (size_t i = 0; i < w512.size(); ++i) w512[i] = e4m3_times_512(blob[i]);
    }
};

// One e4m3 layer: inputs a512 = 512 * a, result the fp16 layer output x (before the activation).
void layer_e4m3(int32_t const* W512, uint16_t const* biasHalf, int in, int out, int32_t const* a512, uint16_t* x)
{
    for (int c = 0; c < out; ++c) {
        int64_t s[3] = { 0, 0, 0 };
        for (int k = 0; k < in; ++k) {
            int32_t const w = W512[c * in + k];
            int64_t const mag = w < 0 ? -int64_t(w) : w, sign = w < 0 ? -1 : 1;
            s[0] += sign * (mag & 127) * a512[k];
            s[1] += sign * ((mag >> 7) & 127) * a512[k];
            s[2] += sign * (mag >> 14) * a512[k];
        }
        // each part is an integer below 2^24 in units of 2^-18, 2^-11 and 2^-4: exact in fp32
        float const f0 = float(s[0]) * 0x1p-18f, f1 = float(s[1]) * 0x1p-11f, f2 = float(s[2]) * 0x1p-4f;
        float r = f2 + f1;
        r = r + f0;
        r = r + half_to_float(biasHalf[c]);
        x[c] = float_to_half_rne(r);
    }
}

struct SetView {
    NtcHipTextureSet const* set;
    NtcHipWeightLayout layout;
    std::vector<int32_t> fp8Weights;       // 512*w of every e4m3 weight, blob order (hidden layers)
    Fp8Layers fp8;
    void prepare()
    {
        if (set->spec.weightType == NTC_HIP_WEIGHTS_FP8) fp8.prepare(*set, layout);
        if (set->spec.weightType != NTC_HIP_WEIGHTS_FP8_SCALED) return;
        uint8_t const* blob = static_cast<uint8_t const*>(set->weights);
        fp8Weights.resize(layout.weightOffset[NTC_HIP_MLP_LAYERS - 1]);
        for (size_t i = 0; i < fp8Weights.size(); ++i) fp8Weights[i] = e4m3_times_512(blob[i]);
    }
};

void prepare_inputs(NtcHipTextureSet const& set, NtcHipMipDesc const& mip, int x, int y, int8_t* in)
{
    NtcHipDecoderSpec const& s = set.spec;
    std::memset(in, 0, size_t(s.inputChannels));               // Inference.hlsli:221-224
    // src/Inference.cu:52-53
    float const u = (float(x) + 0.5f) / float(mip.width);
    float const v = (float(y) + 0.5f) / float(mip.height);
    uint8_t const* lat = static_cast<uint8_t const*>(set.latents);
    Grid const hr{ reinterpret_cast<uint16_t const*>(lat + mip.hrOffset), mip.hrWidth, mip.hrHeight, s.hrFeatures, s.hrBits };
    Grid const lr{ reinterpret_cast<uint16_t const*>(lat + mip.lrOffset), mip.lrWidth, mip.lrHeight, s.lrFeatures, s.lrBits };
    int const hrInputs = (s.hrMode == NTC_HIP_GRID_CONCAT2X2 ? 4 : 1) * s.hrFeatureSlots;
    int const lrInputs = (s.lrMode == NTC_HIP_GRID_CONCAT2X2 ? 4 : 1) * s.lrFeatureSlots;
    sample_grid(hr, s.hrMode, s.hrFeatureSlots, u, v, in);               // Inference.hlsli:229-230
    sample_grid(lr, s.lrMode, s.lrFeatureSlots, u, v, in + hrInputs);    // Inference.hlsli:232-234
    encode_position(float(x) * mip.positionScale, float(y) * mip.positionScale, mip.positionLod,
                    s.posEncWaves, s.lodInputs, in + hrInputs + lrInputs);   // Inference.hlsli:237-238
}

inline bool decodable(NtcHipDecoderSpec const& s)
{
    if (s.weightType == NTC_HIP_WEIGHTS_FP8)                 // the FP8 network exists for bilinear 4-bit grids (the reference's geometry)
        return s.hrMode == NTC_HIP_GRID_BILINEAR && s.lrMode == NTC_HIP_GRID_BILINEAR && s.hrBits == 4 && s.lrBits == 4;
    return s.weightType == NTC_HIP_WEIGHTS_INT8 || s.weightType == NTC_HIP_WEIGHTS_FP8_SCALED;
}

// The input vector of the FP8 network as 512 * (e4m3 value) per input: NtcPrepareNetworkInputsInternal_FP16,
// InferenceCoopVec.hlsli:77-107, then the e4m3 reading of the vector.
void prepare_inputs_fp8(NtcHipTextureSet const& set, NtcHipMipDesc const& mip, int x, int y, int32_t* in512, uint16_t* halvesOut)
{
    NtcHipDecoderSpec const& s = set.spec;
    uint16_t h[NTC_HIP_MAX_LAYER_WIDTH] = {};
    float const u = (float(x) + 0.5f) / float(mip.width);
    float const v = (float(y) + 0.5f) / float(mip.height);
    uint8_t const* lat = static_cast<uint8_t const*>(set.latents);
    Grid const grids[2] = {
        { reinterpret_cast<uint16_t const*>(lat + mip.hrOffset), mip.hrWidth, mip.hrHeight, s.hrFeatures, s.hrBits },
        { reinterpret_cast<uint16_t const*>(lat + mip.lrOffset), mip.lrWidth, mip.lrHeight, s.lrFeatures, s.lrBits } };
    int const base[2] = { 0, s.hrFeatureSlots };
    for (int g = 0; g < 2; ++g) {
        Footprint const fp = bilinear_footprint(u, v, grids[g].width, grids[g].height);
        for (int f = 0; f < grids[g].features; ++f) {
            float t = fp.w00 * float(grids[g].fetch(fp.x0, fp.y0, f));
            t = std::fmaf(fp.w10, float(grids[g].fetch(fp.x1, fp.y0, f)), t);
            t = std::fmaf(fp.w01, float(grids[g].fetch(fp.x0, fp.y1, f)), t);
            t = std::fmaf(fp.w11, float(grids[g].fetch(fp.x1, fp.y1, f)), t);
            h[base[g] + f] = float_to_half_rne(std::fmaf(t, 0.13333334f, -1.f));     // hlsli:38-45
        }
    }
    int idx = s.hrFeatureSlots + s.lrFeatureSlots;           // hlsli:51-75
    float px = float(x) * mip.positionScale, py = float(y) * mip.positionScale;
    for (int w = 0; w < s.posEncWaves; ++w) {
        h[idx++] = float_to_half_rne(frac_hlsl(px) * 2.f - 1.f);
        h[idx++] = float_to_half_rne(frac_hlsl(py) * 2.f - 1.f);
        h[idx++] = float_to_half_rne(frac_hlsl(px + 0.25f) * 2.f - 1.f);
        h[idx++] = float_to_half_rne(frac_hlsl(py + 0.25f) * 2.f - 1.f);
        px *= 2.f; py *= 2.f;
    }
    for (int i = 0; i < s.lodInputs; ++i) h[idx++] = float_to_half_rne(mip.positionLod);
    for (int k = 0; k < s.inputChannels; ++k) in512[k] = half_to_e4m3_times_512(h[k]);
    if (halvesOut) std::memcpy(halvesOut, h, size_t(s.inputChannels) * 2);
}

// One texel through the FP8 network: NtcEvaluateMLP_CoopVec_FP8, InferenceCoopVec.hlsli:348-398.
void decode_texel_fp8(SetView const& sv, NtcHipMipDesc const& mip, int x, int y, float* outputs)
{
    NtcHipTextureSet const& set = *sv.set;
    NtcHipDecoderSpec const& s = set.spec;
    uint8_t const* blob = static_cast<uint8_t const*>(set.weights);
    int32_t a512[NTC_HIP_MAX_LAYER_WIDTH];
    prepare_inputs_fp8(set, mip, x, y, a512, nullptr);
    uint16_t xh[NTC_HIP_MAX_LAYER_WIDTH];
    int8_t q[NTC_HIP_MAX_LAYER_WIDTH];
    constexpr int last = NTC_HIP_MLP_LAYERS - 1;
    for (int l = 0; l < last; ++l) {
        int const in = layer_inputs(s, l), out = layer_outputs(s, l);
        layer_e4m3(sv.fp8.w512.data() + sv.layout.weightOffset[l], reinterpret_cast<uint16_t const*>(blob + sv.layout.biasOffset[l]), in, out, a512, xh);
        for (int c = 0; c < out; ++c) {
            uint16_t const yh = hgelu_half(xh[c]);
            if (l < last - 1) a512[c] = half_to_e4m3_times_512(yh);
            else q[c] = int8_t(int(std::nearbyint(80.0 * half_value(yh) - 113.0)));    // hlsli:155-158: y*80 + (-113), in [-128, 127]
        }
    }
    float r[NTC_HIP_MAX_LAYER_WIDTH];
    layer_int8(reinterpret_cast<int8_t const*>(blob + sv.layout.weightOffset[last]),
               reinterpret_cast<float const*>(blob + sv.layout.scaleOffset[last]),
               reinterpret_cast<int32_t const*>(blob + sv.layout.biasOffset[last]),
               layer_inputs(s, last), layer_outputs(s, last), q, r);
    for (int c = 0; c < s.outputChannels; ++c) outputs[c] = r[c];
}

// One texel through the int8 network: NtcSampleTextureSet, Inference.hlsli:282-357.
void decode_texel_int8(SetView const& sv, NtcHipMipDesc const& mip, int x, int y, float* outputs, int8_t* inputsOut)
{
    NtcHipTextureSet const& set = *sv.set;
    NtcHipDecoderSpec const& s = set.spec;
    uint8_t const* blob = static_cast<uint8_t const*>(set.weights);
    int8_t act[NTC_HIP_MAX_LAYER_WIDTH];
    prepare_inputs(set, mip, x, y, act);
    if (inputsOut) std::memcpy(inputsOut, act, size_t(s.inputChannels));
    float r[NTC_HIP_MAX_LAYER_WIDTH];
    for (int l = 0; l < NTC_HIP_MLP_LAYERS; ++l) {
        int const in = layer_inputs(s, l), out = layer_outputs(s, l);
        if (s.weightType == NTC_HIP_WEIGHTS_FP8_SCALED && l < NTC_HIP_MLP_LAYERS - 1)
            layer_fp8_weights(sv.fp8Weights.data() + sv.layout.weightOffset[l],
                              reinterpret_cast<float const*>(blob + sv.layout.scaleOffset[l]),
                              reinterpret_cast<int32_t const*>(blob + sv.layout.biasOffset[l]),
                              in, out, act, r);
        else
            layer_int8(reinterpret_cast<int8_t const*>(blob + sv.layout.weightOffset[l]),
                       reinterpret_cast<float const*>(blob + sv.layout.scaleOffset[l]),
                       reinterpret_cast<int32_t const*>(blob + sv.layout.biasOffset[l]),
                       in, out, act, r);
        if (l == NTC_HIP_MLP_LAYERS - 1) break;
        for (int c = 0; c < out; ++c) act[c] = int8_t(hgelu_quantize(r[c]));   // NtcPackInt8x4: & 0xff
    }
    for (int c = 0; c < s.outputChannels; ++c) outputs[c] = r[c];
}

// One texel through the network the set's weight type selects.  inputsOut (optional) receives the int8
// input vector; the FP8 network has none.
void decode_texel(SetView const& sv, NtcHipMipDesc const& mip, int x, int y, float* outputs, int8_t* inputsOut)
{
    if (sv.set->spec.weightType == NTC_HIP_WEIGHTS_FP8) decode_texel_fp8(sv, mip, x, y, outputs);
    else decode_texel_int8(sv, mip, x, y, outputs, inputsOut);
}

// Output addressing.  Planar pairs: GetPixelBaseAddress/GetChannelAddress,
// src/RegressionKernels.h:36-45; channel count rounded up to even, src/TextureSet.cpp:86.
void store_texel(NtcHipTextureSet const& set, NtcHipMipDesc const& mip, int x, int y, float const* o)
{
    uint8_t* out = static_cast<uint8_t*>(set.output) + mip.outOffset;
    if (set.outputFormat == NTC_HIP_OUT_FP16_PLANAR_PAIRS) {
        int const C = (set.numChannels + 1) & ~1;
        uint16_t* img = reinterpret_cast<uint16_t*>(out);
        for (int ch = 0; ch < set.numChannels; ++ch) {
            size_t const a = size_t(y) * size_t(mip.width) * size_t(C) + size_t(x) * 2
                           + size_t(ch & ~1) * size_t(mip.width) + size_t(ch & 1);
            img[a] = output_to_half(o[ch]);
        }
        // An odd channel count still stores whole half2 pairs (Inference.cu:131-134).
        if (set.numChannels & 1) {
            int const ch = set.numChannels;
            size_t const a = size_t(y) * size_t(mip.width) * size_t(C) + size_t(x) * 2
                           + size_t(ch & ~1) * size_t(mip.width) + size_t(ch & 1);
            img[a] = output_to_half(o[ch]);
        }
    } else {
        uint8_t* px = out + size_t(y) * mip.outRowPitch + size_t(x) * size_t(set.outPixelStride);
        for (int ch = 0; ch < set.numChannels; ++ch) {
            uint16_t const h = output_to_half(o[ch]);
            if (set.outputFormat == NTC_HIP_OUT_FP16_PIXELS) std::memcpy(px + 2 * ch, &h, 2);
            else px[ch] = half_to_unorm8(h);
        }
    }
}

} // namespace

// =========================================================================================
// C entry points (loaded by the tests through ctypes)
// =========================================================================================
extern "C" {

int ntc_oracle_weight_layout(const NtcHipDecoderSpec* spec, NtcHipWeightLayout* out)
{
    return weight_layout(*spec, *out) ? 0 : -1;
}

uint16_t ntc_oracle_float_to_half(float f) { return float_to_half_rne(f); }
float    ntc_oracle_half_to_float(uint16_t h) { return half_to_float(h); }
uint16_t ntc_oracle_output_to_half(float f) { return output_to_half(f); }
uint8_t  ntc_oracle_half_to_unorm8(uint16_t h) { return half_to_unorm8(h); }
int      ntc_oracle_hgelu_quantize(float x) { return hgelu_quantize(x); }
int      ntc_oracle_unpack_field(uint16_t w, int index, int bits) { return unpack_field(w, index, bits); }
int32_t  ntc_oracle_e4m3_times_512(uint8_t byte) { return e4m3_times_512(byte); }
void     ntc_oracle_layer_int8(const int8_t* W, const float* scale, const int32_t* bias, int in, int out,
                               const int8_t* x, float* r) { layer_int8(W, scale, bias, in, out, x, r); }

// PackLatentsKernel's QuantizeValue, src/Quantizer.cu:482-488 (encoder side; here only so
// the tests can check Pack o Unpack = id).
uint32_t ntc_oracle_quantize_value(float value, int bits)
{
    float const step = 1.f / float((1 << bits) - 1);
    value = std::max(0.f, std::min(1.f, value));
    return uint32_t(std::round(value / step));
}

void ntc_oracle_encode_position(float px, float py, float lod, int waves, int lodInputs, int8_t* out)
{
    encode_position(px, py, lod, waves, lodInputs, out);
}

void ntc_oracle_bilinear_footprint(float u, float v, int gw, int gh, int* xy, float* w)
{
    Footprint const fp = bilinear_footprint(u, v, gw, gh);
    xy[0] = fp.x0; xy[1] = fp.y0; xy[2] = fp.x1; xy[3] = fp.y1;
    w[0] = fp.w00; w[1] = fp.w10; w[2] = fp.w01; w[3] = fp.w11;
}

// Inputs (int8, spec.inputChannels of them) and raw fp32 outputs of one texel.
int ntc_oracle_decode_texel(const NtcHipTextureSet* set, int mip, int x, int y, float* outputs, int8_t* inputs)
{
    SetView sv{ set, {}, {}, {} };
    if (!decodable(set->spec) || !weight_layout(set->spec, sv.layout)) return -1;
    sv.prepare();
    decode_texel(sv, set->mips[mip], x, y, outputs, inputs);
    return 0;
}

// Pieces of the FP8 network, for the tests that pin them.
int32_t  ntc_oracle_half_to_e4m3_times_512(uint16_t h) { return half_to_e4m3_times_512(h); }
uint16_t ntc_oracle_hgelu_half(uint16_t x) { return hgelu_half(x); }
uint16_t ntc_oracle_double_to_half(double d) { return double_to_half_rne(d); }
void     ntc_oracle_layer_e4m3(const uint8_t* weightsE4M3, const uint16_t* biasHalf, int in, int out, const int32_t* a512, uint16_t* x)
{
    std::vector<int32_t> w512(size_t(in) * size_t(out));
    for (size_t i = 0; i < w512.size(); ++i) w512[i] = e4m3_times_512(weightsE4M3[i]);
    layer_e4m3(w512.data(), biasHalf, in, out, a512, x);
}
int ntc_oracle_fp8_inputs(const NtcHipTextureSet* set, int mip, int x, int y, uint16_t* halves, int32_t* in512)
{
    if (!set || mip < 0 || mip >= set->numMips || set->spec.weightType != NTC_HIP_WEIGHTS_FP8 || !decodable(set->spec)) return -1;
    prepare_inputs_fp8(*set, set->mips[mip], x, y, in512, halves);
    return 0;
}

// Neural-LOD geometry of the reference, for a texture set of the given size:
//  LodToNeuralLod / GetGridDimension / CalculateNumNeuralMipLevels, src/FeatureGridMath.cpp:47-77;
//  colour-mip constants, src/TextureSet.cpp:441-463; low-res dims, src/TextureSet.cpp:1816-1817;
//  grids stored neural LOD after neural LOD, layers inside (src/FeatureGridHost.cpp:140-161).
// Fills width/height/grid dims/positionScale/positionLod/hrOffset/lrOffset of mips[0..numMips).
// Returns the number of neural LODs, or -1.
int ntc_oracle_ref_geometry(int width, int height, int numMips, int gridSizeScale, int numFeatures,
                            NtcHipMipDesc* mips, uint64_t* outLatentBytes)
{
    static int const sharedMipsForGridScale[] = { 2, 3, 3, 3, 4, 4 };
    if (gridSizeScale < 1 || gridSizeScale > 6 || numMips < 1 || numMips > NTC_HIP_MAX_MIPS) return -1;
    int const minGrid = int(float(std::min(width, height)) / float(gridSizeScale));
    int numNeural = std::max(2, int(1.f + std::floor(std::log2(float(minGrid))))) & ~1;
    auto lodToNeural = [&](int lod, int neuralLods) {
        int n = (lod - sharedMipsForGridScale[gridSizeScale - 1] + 2) & ~1;
        return std::max(0, std::min(n, neuralLods - 2));
    };
    // Clamp as CalculateQuantizedLatentsSize does (src/FeatureGridMath.cpp:27-33); the host
    // grid applies the same clamp when it is sized (src/FeatureGridHost.cpp:27-79).
    int const lastNeural = lodToNeural(numMips - 1, 8 /* NTC_MAX_NEURAL_MIPS */) + 1;
    numNeural = std::min(numNeural, lastNeural + 1);
    auto gridDim = [&](int dim, int nlod) { return std::max((dim / gridSizeScale) >> nlod, 1); };
    int const layers = (numFeatures + 3) / 4;
    std::vector<uint64_t> offs(size_t(numNeural) + 1, 0);
    for (int n = 0; n < numNeural; ++n)
        offs[size_t(n) + 1] = offs[size_t(n)] + uint64_t(gridDim(width, n)) * uint64_t(gridDim(height, n)) * 2u * uint64_t(layers);
    if (outLatentBytes) *outLatentBytes = offs[size_t(numNeural)];
    for (int m = 0; m < numMips; ++m) {
        NtcHipMipDesc& d = mips[m];
        int const nlod = lodToNeural(m, numNeural);
        d.width = std::max(1, width >> m);
        d.height = std::max(1, height >> m);
        d.hrWidth = gridDim(width, nlod);  d.hrHeight = gridDim(height, nlod);
        d.lrWidth = std::max(d.hrWidth >> 1, 1); d.lrHeight = std::max(d.hrHeight >> 1, 1);
        float const ws = float(d.hrWidth) / float(d.width), hs = float(d.hrHeight) / float(d.height);
        d.positionScale = 0.5f * std::max(ws, hs);
        d.positionLod = std::max(-1.f, std::min(1.f, 0.25f * std::log2(d.positionScale)));
        d.hrOffset = offs[size_t(nlod)];
        d.lrOffset = offs[size_t(nlod) + 1];
    }
    return numNeural;
}

// Transfer functions of the colour spaces (src/CudaUtils.h:61-114): sRGB and Hybrid Log-Gamma,
// with the host math library's powf / expf / logf / sqrtf -- results agree with the device's to a few
// units in the last place, not bit for bit, and the tests that use them say so.
static float decode_color_space(int cs, float v)
{
    if (cs == 1) return (v <= 0.04045f) ? v / 12.92f : std::pow((v + 0.055f) / 1.055f, 2.4f);
    if (cs == 2) {
        float const sign = (v < 0.f) ? -1.f : 1.f;
        float const h = std::fabs(v);
        return (h < 0.5f) ? 4.f * h * h * sign : (std::exp((h - 0.55991073f) / 0.17883277f) + 0.28466892f) * sign;
    }
    return v;
}
static float encode_color_space(int cs, float v)
{
    if (cs == 1) return (v <= 0.0031308f) ? v * 12.92f : 1.055f * std::pow(v, 1.0f / 2.4f) - 0.055f;
    if (cs == 2) {
        float const sign = (v < 0.f) ? -1.f : 1.f;
        float const e = std::fabs(v);
        return (e < 1.f) ? 0.5f * std::sqrt(e) * sign : (0.17883277f * std::log(e - 0.28466892f) + 0.55991073f) * sign;
    }
    return v;
}

// HashBasedRNG (src/CudaUtils.h:117-184): the seed is a Jenkins hash of the pixel's linear index,
// every draw is one Murmur3 round over a running counter that starts at 1; the float takes the low
// 23 bits as a mantissa in [1, 2) and subtracts 1.
struct HashRng {
    uint32_t seed, index = 1;
    explicit HashRng(uint32_t linearIndex)
    {
        uint32_t a = linearIndex;
        a = (a + 0x7ed55d16u) + (a << 12);
        a = (a ^ 0xc761c23cu) ^ (a >> 19);
        a = (a + 0x165667b1u) + (a << 5);
        a = (a + 0xd3a2646cu) ^ (a << 9);
        a = (a + 0xfd7046c5u) + (a << 3);
        a = (a ^ 0xb55a4f09u) ^ (a >> 16);
        seed = a;
    }
    static uint32_t rotl(uint32_t x, int n) { return (x << n) | (x >> (32 - n)); }
    uint32_t next_uint()
    {
        uint32_t k = index * 0xcc9e2d51u;
        k = rotl(k, 15) * 0x1b873593u;
        uint32_t h = rotl(seed ^ k, 13) * 5u + 0xe6546b64u;
        h ^= 4u;
        h ^= h >> 16; h *= 0x85ebca6bu;
        h ^= h >> 13; h *= 0xc2b2ae35u;
        h ^= h >> 16;
        ++index;
        return h;
    }
    float next_float() { return bits_f32((next_uint() & 0x7fffffu) | 0x3f800000u) - 1.f; }
};

// Draw number `draw` (0-based) of the dithering generator of pixel `linearIndex`, in [0, 1).
float ntc_oracle_dither_float(uint32_t linearIndex, int draw)
{
    HashRng rng(linearIndex);
    float v = 0.f;
    for (int i = 0; i <= draw; ++i) v = rng.next_float();
    return v;
}

// ITextureSet::ReadChannels' copy, 1:1 branch: CopyImageKernel + ReadImageChannel (FLOAT16 source)
// + WriteImageChannel (src/ImageProcessing.cu:86-164,220-265) reading the internal planar-pair
// layout (GetTextureDataSlice, src/TextureSet.cpp:1958-1983).  Destination channels beyond
// numChannels get GetDefaultChannelValue (src/ImageProcessing.cu:166-170); with useDithering every
// destination channel draws one number, in channel order.
// format: 1 UNORM8, 2 UNORM16, 3 FLOAT16, 4 FLOAT32, 5 UINT32 (include/libntc/ntc.h:227-236).
int ntc_oracle_read_channels_ex(const uint16_t* planarPairs, int width, int height, int setChannels,
                                int firstChannel, int numChannels, uint8_t* dst, int format,
                                uint64_t pixelStride, uint64_t rowPitch, int useDithering,
                                const uint8_t* srcColorSpaces /* 16 or null */, const uint8_t* dstColorSpaces /* 16 or null */)
{
    int const bpc = (format == 1) ? 1 : (format == 2 || format == 3) ? 2 : (format == 4 || format == 5) ? 4 : 0;
    if (!bpc) return -1;
    int const dstChannels = int(pixelStride / uint64_t(bpc));
    auto roundHalfAway = [](float v) {                       // roundf
        float r = std::trunc(v);
        float const fr = v - r;
        if (fr >= 0.5f) r += 1.f; else if (fr <= -0.5f) r -= 1.f;
        return r;
    };
    for (int y = 0; y < height; ++y)
        for (int x = 0; x < width; ++x) {
            uint8_t* px = dst + size_t(y) * rowPitch + size_t(x) * pixelStride;
            HashRng rng(uint32_t(x) + uint32_t(y) * uint32_t(width));
            for (int ch = 0; ch < dstChannels; ++ch) {
                float value;
                if (ch < numChannels) {
                    int const c = firstChannel + ch;
                    size_t const a = size_t(y) * size_t(width) * size_t(setChannels) + size_t(x) * 2
                                   + size_t(c & ~1) * size_t(width) + size_t(c & 1);
                    value = decode_color_space(srcColorSpaces ? srcColorSpaces[ch] : 0, half_to_float(planarPairs[a]));
                } else {
                    value = (ch == 3) ? 1.f : 0.f;
                }
                float const dither = useDithering ? rng.next_float() - 0.5f : 0.f;
                value = encode_color_space((dstColorSpaces && ch < 16) ? dstColorSpaces[ch] : 0, value);
                switch (format) {
                case 1: value += dither / 255.f; px[ch] = uint8_t(std::max(0.f, std::min(255.f, roundHalfAway(value * 255.f)))); break;
                case 2: { value += dither / 65535.f; uint16_t v = uint16_t(std::max(0.f, std::min(65535.f, roundHalfAway(value * 65535.f)))); std::memcpy(px + 2 * ch, &v, 2); break; }
                case 3: { uint16_t v = float_to_half_rne(std::max(-65504.f, std::min(65504.f, value))); std::memcpy(px + 2 * ch, &v, 2); break; }
                case 4: std::memcpy(px + 4 * ch, &value, 4); break;
                case 5: { uint32_t v = uint32_t(std::max(value, 0.f)); std::memcpy(px + 4 * ch, &v, 4); break; }
                }
            }
        }
    return 0;
}

int ntc_oracle_read_channels(const uint16_t* planarPairs, int width, int height, int setChannels,
                             int firstChannel, int numChannels, uint8_t* dst, int format,
                             uint64_t pixelStride, uint64_t rowPitch)
{
    return ntc_oracle_read_channels_ex(planarPairs, width, height, setChannels, firstChannel, numChannels, dst, format,
                                       pixelStride, rowPitch, 0, nullptr, nullptr);
}

// ITextureSet::WriteChannels' copy (1:1): ReadImageChannel in the user's format and colour space,
// WriteImageChannel FLOAT16 in the storage colour space into the internal planar-pair layout
// (src/ImageProcessing.cu:86-164,220-265), with the optional vertical flip of SetupBilinearFilter
// (src/ImageProcessing.cu:36-37).
int ntc_oracle_write_channels_ex(const uint8_t* src, int format, int verticalFlip, uint64_t pixelStride, uint64_t rowPitch,
                                 uint16_t* planarPairs, int width, int height, int setChannels, int firstChannel, int numChannels,
                                 const uint8_t* srcColorSpaces, const uint8_t* dstColorSpaces)
{
    for (int y = 0; y < height; ++y)
        for (int x = 0; x < width; ++x) {
            int const srcY = verticalFlip ? height - 1 - y : y;
            uint8_t const* px = src + size_t(srcY) * rowPitch + size_t(x) * pixelStride;
            for (int ch = 0; ch < numChannels; ++ch) {
                float v;
                switch (format) {
                case 1: v = float(px[ch]) / 255.f; break;
                case 2: { uint16_t t; std::memcpy(&t, px + 2 * ch, 2); v = float(t) / 65535.f; break; }
                case 3: { uint16_t t; std::memcpy(&t, px + 2 * ch, 2); v = half_to_float(t); break; }
                case 4: std::memcpy(&v, px + 4 * ch, 4); break;
                case 5: { uint32_t t; std::memcpy(&t, px + 4 * ch, 4); v = float(t); break; }
                default: return -1;
                }
                v = decode_color_space(srcColorSpaces ? srcColorSpaces[ch] : 0, v);
                v = encode_color_space(dstColorSpaces ? dstColorSpaces[ch] : 0, v);
                v = std::max(-65504.f, std::min(65504.f, v));
                int const c = firstChannel + ch;
                planarPairs[size_t(y) * size_t(width) * size_t(setChannels) + size_t(x) * 2
                            + size_t(c & ~1) * size_t(width) + size_t(c & 1)] = float_to_half_rne(v);
            }
        }
    return 0;
}

int ntc_oracle_write_channels(const uint8_t* src, int format, int verticalFlip, uint64_t pixelStride, uint64_t rowPitch,
                              uint16_t* planarPairs, int width, int height, int setChannels, int firstChannel, int numChannels)
{
    return ntc_oracle_write_channels_ex(src, format, verticalFlip, pixelStride, rowPitch, planarPairs, width, height, setChannels,
                                        firstChannel, numChannels, nullptr, nullptr);
}

// ---- resampling copies: SetupBilinearFilter (src/ImageProcessing.cu:24-72) ---------------------------
// Destination pixel (x, y) looks at ((x + 1/2) / dstW) * srcW - 1/2 in the source, clamped to the image;
// four taps, bilinear weights, taps of zero weight not read (:232-237).  The blend
// a*w0 + b*w1 + c*w2 + d*w3 is evaluated as one multiply and three fused multiply-adds (the
// contraction a CUDA compiler applies to that expression); the reference's fast-math division in
// the position is an IEEE division here, so its last bits are parity unpinned.
struct ResampleTaps { int x0, y0, x1, y1; float w[4]; };

static ResampleTaps resample_taps(int srcW, int srcH, int dstW, int dstH, int x, int y)
{
    if (srcW == dstW && srcH == dstH) return ResampleTaps{ x, y, x, y, { 1.f, 0.f, 0.f, 0.f } };    // the 1:1 shortcut, :39-45
    float const u = (float(x) + 0.5f) / float(dstW), v = (float(y) + 0.5f) / float(dstH);
    float const px = std::max(0.f, std::min(float(srcW) - 1.f, u * float(srcW) - 0.5f));
    float const py = std::max(0.f, std::min(float(srcH) - 1.f, v * float(srcH) - 0.5f));
    float const fx = px - std::floor(px), fy = py - std::floor(py);
    ResampleTaps t;
    t.x0 = int(std::floor(px)); t.y0 = int(std::floor(py));
    t.x1 = std::min(t.x0 + 1, srcW - 1); t.y1 = std::min(t.y0 + 1, srcH - 1);
    t.w[0] = (1.f - fx) * (1.f - fy); t.w[1] = fx * (1.f - fy); t.w[2] = (1.f - fx) * fy; t.w[3] = fx * fy;
    return t;
}

static float resample_blend(ResampleTaps const& t, float a, float b, float c, float d)
{
    a = t.w[0] > 0.f ? a : 0.f; b = t.w[1] > 0.f ? b : 0.f; c = t.w[2] > 0.f ? c : 0.f; d = t.w[3] > 0.f ? d : 0.f;
    return std::fmaf(d, t.w[3], std::fmaf(c, t.w[2], std::fmaf(b, t.w[1], a * t.w[0])));
}

static float planar_value(const uint16_t* image, int width, int setChannels, int x, int y, int c)
{
    return half_to_float(image[size_t(y) * size_t(width) * size_t(setChannels) + size_t(c & ~1) * size_t(width) + size_t(x) * 2 + size_t(c & 1)]);
}

static float user_value(const uint8_t* px, int format, int ch)
{
    switch (format) {
    case 1: return float(px[ch]) / 255.f;
    case 2: { uint16_t t; std::memcpy(&t, px + 2 * ch, 2); return float(t) / 65535.f; }
    case 3: { uint16_t t; std::memcpy(&t, px + 2 * ch, 2); return half_to_float(t); }
    case 4: { float t; std::memcpy(&t, px + 4 * ch, 4); return t; }
    default: { uint32_t t; std::memcpy(&t, px + 4 * ch, 4); return float(t); }
    }
}

// ReadChannels into an image of another size (CopyImageKernel, src/ImageProcessing.cu:220-265).
int ntc_oracle_read_channels_resized(const uint16_t* planarPairs, int width, int height, int setChannels,
                                     int firstChannel, int numChannels, uint8_t* dst, int format,
                                     uint64_t pixelStride, uint64_t rowPitch, int dstWidth, int dstHeight, int useDithering,
                                     const uint8_t* srcColorSpaces, const uint8_t* dstColorSpaces)
{
    int const bpc = (format == 1) ? 1 : (format == 2 || format == 3) ? 2 : (format == 4 || format == 5) ? 4 : 0;
    if (!bpc) return -1;
    int const dstChannels = int(pixelStride / uint64_t(bpc));
    auto roundHalfAway = [](float v) {
        float r = std::trunc(v);
        float const fr = v - r;
        if (fr >= 0.5f) r += 1.f; else if (fr <= -0.5f) r -= 1.f;
        return r;
    };
    for (int y = 0; y < dstHeight; ++y)
        for (int x = 0; x < dstWidth; ++x) {
            ResampleTaps const t = resample_taps(width, height, dstWidth, dstHeight, x, y);
            uint8_t* px = dst + size_t(y) * rowPitch + size_t(x) * pixelStride;
            HashRng rng(uint32_t(x) + uint32_t(y) * uint32_t(dstWidth));
            for (int ch = 0; ch < dstChannels; ++ch) {
                float value;
                if (ch < numChannels) {
                    int const c = firstChannel + ch, space = srcColorSpaces ? srcColorSpaces[ch] : 0;
                    value = resample_blend(t, decode_color_space(space, planar_value(planarPairs, width, setChannels, t.x0, t.y0, c)),
                                              decode_color_space(space, planar_value(planarPairs, width, setChannels, t.x1, t.y0, c)),
                                              decode_color_space(space, planar_value(planarPairs, width, setChannels, t.x0, t.y1, c)),
                                              decode_color_space(space, planar_value(planarPairs, width, setChannels, t.x1, t.y1, c)));
                } else {
                    value = (ch == 3) ? 1.f : 0.f;
                }
                float const dither = useDithering ? rng.next_float() - 0.5f : 0.f;
                value = encode_color_space((dstColorSpaces && ch < 16) ? dstColorSpaces[ch] : 0, value);
                switch (format) {
                case 1: value += dither / 255.f; px[ch] = uint8_t(std::max(0.f, std::min(255.f, roundHalfAway(value * 255.f)))); break;
                case 2: { value += dither / 65535.f; uint16_t v = uint16_t(std::max(0.f, std::min(65535.f, roundHalfAway(value * 65535.f)))); std::memcpy(px + 2 * ch, &v, 2); break; }
                case 3: { uint16_t v = float_to_half_rne(std::max(-65504.f, std::min(65504.f, value))); std::memcpy(px + 2 * ch, &v, 2); break; }
                case 4: std::memcpy(px + 4 * ch, &value, 4); break;
                case 5: { uint32_t v = uint32_t(std::max(value, 0.f)); std::memcpy(px + 4 * ch, &v, 4); break; }
                }
            }
        }
    return 0;
}

// WriteChannels from an image of another size.  With verticalFlip the destination row is mirrored
// before the source position is computed (src/ImageProcessing.cu:36-37).
int ntc_oracle_write_channels_resized(const uint8_t* src, int format, int verticalFlip, uint64_t pixelStride, uint64_t rowPitch,
                                      int srcWidth, int srcHeight, uint16_t* planarPairs, int width, int height, int setChannels,
                                      int firstChannel, int numChannels, const uint8_t* srcColorSpaces, const uint8_t* dstColorSpaces)
{
    if (format < 1 || format > 5) return -1;
    for (int y = 0; y < height; ++y)
        for (int x = 0; x < width; ++x) {
            ResampleTaps const t = resample_taps(srcWidth, srcHeight, width, height, x, verticalFlip ? height - 1 - y : y);
            auto at = [&](int sx, int sy) { return src + size_t(sy) * rowPitch + size_t(sx) * pixelStride; };
            for (int ch = 0; ch < numChannels; ++ch) {
                int const space = srcColorSpaces ? srcColorSpaces[ch] : 0;
                float v = resample_blend(t, decode_color_space(space, user_value(at(t.x0, t.y0), format, ch)), decode_color_space(space, user_value(at(t.x1, t.y0), format, ch)),
                                            decode_color_space(space, user_value(at(t.x0, t.y1), format, ch)), decode_color_space(space, user_value(at(t.x1, t.y1), format, ch)));
                v = encode_color_space(dstColorSpaces ? dstColorSpaces[ch] : 0, v);
                v = std::max(-65504.f, std::min(65504.f, v));
                int const c = firstChannel + ch;
                planarPairs[size_t(y) * size_t(width) * size_t(setChannels) + size_t(x) * 2 + size_t(c & ~1) * size_t(width) + size_t(c & 1)] = float_to_half_rne(v);
            }
        }
    return 0;
}

// ResizeMultichannelImage (src/ImageProcessing.cu:178-218): what GenerateMips runs from mip to mip.
void ntc_oracle_resize_planar(const uint16_t* src, int srcWidth, int srcHeight, uint16_t* dst, int dstWidth, int dstHeight,
                              int setChannels, const uint8_t* colorSpaces /* 16 or null */)
{
    for (int y = 0; y < dstHeight; ++y)
        for (int x = 0; x < dstWidth; ++x) {
            ResampleTaps const t = resample_taps(srcWidth, srcHeight, dstWidth, dstHeight, x, y);
            for (int c = 0; c < setChannels; ++c) {
                int const space = colorSpaces ? colorSpaces[c] : 0;
                float v = resample_blend(t, decode_color_space(space, planar_value(src, srcWidth, setChannels, t.x0, t.y0, c)),
                                            decode_color_space(space, planar_value(src, srcWidth, setChannels, t.x1, t.y0, c)),
                                            decode_color_space(space, planar_value(src, srcWidth, setChannels, t.x0, t.y1, c)),
                                            decode_color_space(space, planar_value(src, srcWidth, setChannels, t.x1, t.y1, c)));
                v = std::max(-65504.f, std::min(65504.f, encode_color_space(space, v)));
                dst[size_t(y) * size_t(dstWidth) * size_t(setChannels) + size_t(c & ~1) * size_t(dstWidth) + size_t(x) * 2 + size_t(c & 1)] = float_to_half_rne(v);
            }
        }
}

// Per-channel mean squared error between a decoded mip and its reference, both in the internal
// layout: what InferenceKernel's loss branch and ReduceLoss add up (src/Inference.cu:96-115,142-156,
// src/Optimizer.cu:335-390), here in double.
void ntc_oracle_image_loss(const uint16_t* a, const uint16_t* b, int width, int height, int setChannels,
                           uint32_t validChannelMask, double* outMse /* 16 */)
{
    for (int c = 0; c < 16; ++c) outMse[c] = 0.0;
    for (int y = 0; y < height; ++y)
        for (int c = 0; c < setChannels; ++c) {
            if (!((validChannelMask >> c) & 1u)) continue;
            size_t const base = size_t(y) * size_t(width) * size_t(setChannels) + size_t(c & ~1) * size_t(width) + size_t(c & 1);
            double acc = 0.0;
            for (int x = 0; x < width; ++x) {
                double const d = double(half_to_float(a[base + size_t(x) * 2])) - double(half_to_float(b[base + size_t(x) * 2]));
                acc += d * d;
            }
            outMse[c] += acc;
        }
    for (int c = 0; c < 16; ++c) outMse[c] /= double(width) * double(height);
}

// The same with the alpha-mask options of the loss branch (src/Inference.cu:80-84,96-97,107-108,112):
// the decoded mask channel is clamped to [0, 1] IN PLACE (a negative zero becomes +0: the device
// max(0.f, x) of the reference returns +0 for x = -0), and with discardMaskedOut a texel whose
// reference mask value is +-0 counts on the mask channel only.
void ntc_oracle_image_loss_masked(uint16_t* a, const uint16_t* b, int width, int height, int setChannels,
                                  uint32_t validChannelMask, int maskChannel, int discardMaskedOut, double* outMse /* 16 */)
{
    for (int c = 0; c < 16; ++c) outMse[c] = 0.0;
    auto at = [&](int x, int y, int c) {
        return size_t(y) * size_t(width) * size_t(setChannels) + size_t(c & ~1) * size_t(width) + size_t(x) * 2 + size_t(c & 1);
    };
    for (int y = 0; y < height; ++y)
        for (int x = 0; x < width; ++x) {
            bool maskedOut = false;
            if (maskChannel >= 0 && maskChannel < setChannels) {
                uint16_t& m = a[at(x, y, maskChannel)];
                float const v = half_to_float(m);
                m = float_to_half_rne(v > 0.f ? std::min(v, 1.f) : 0.f);
                maskedOut = discardMaskedOut && half_to_float(b[at(x, y, maskChannel)]) == 0.f;
            }
            for (int c = 0; c < setChannels; ++c) {
                if (!((validChannelMask >> c) & 1u) || (maskedOut && c != maskChannel)) continue;
                double const d = double(half_to_float(a[at(x, y, c)])) - double(half_to_float(b[at(x, y, c)]));
                outMse[c] += d * d;
            }
        }
    for (int c = 0; c < 16; ++c) outMse[c] /= double(width) * double(height);
}

// Image-difference pass (src/shaders/ImageDifference.hlsl): per-channel squared differences of two
// RGBA images over an extent, summed per 64 x 64 workgroup in fp32, normalised, converted to 16.48
// fixed point and accumulated as integers (hlsl:103-127).  The reference leaves the order of a
// workgroup's additions to the wave intrinsics; the order restated here is the one the HIP kernel
// documents: lane = column, wave w takes rows 16w..16w+15 in order, lanes are combined by an xor
// butterfly with offsets 32..1, the four waves are added in order.  `images` hold host pointers.
// MSLE uses the host logf; the device's differs in the last places.
static float diff_channel(NtcHipImage const& im, uint8_t const* px, int c)
{
    if (c >= im.numChannels) return c == 3 ? 1.f : 0.f;
    switch (im.format) {
    case 1: return float(px[c]) / 255.f;
    case 2: { uint16_t v; std::memcpy(&v, px + 2 * c, 2); return float(v) / 65535.f; }
    case 3: { uint16_t v; std::memcpy(&v, px + 2 * c, 2); return half_to_float(v); }
    case 4: { float v; std::memcpy(&v, px + 4 * c, 4); return v; }
    default: { uint32_t v; std::memcpy(&v, px + 4 * c, 4); return float(v); }
    }
}

static uint32_t saturating_u32(float v)
{
    if (!(v > 0.f)) return 0u;                               // negatives and NaN
    return v >= 4294967296.f ? 0xffffffffu : uint32_t(v);
}

void ntc_oracle_image_difference(const NtcHipImageDifference* p, uint64_t* out /* 4, added to */)
{
    for (int by = 0; by < (p->height + 63) / 64; ++by)
        for (int bx = 0; bx < (p->width + 63) / 64; ++bx) {
            float waveSum[4][4];
            for (int wave = 0; wave < 4; ++wave) {
                float lanes[64][4];
                for (int lane = 0; lane < 64; ++lane) {
                    float mse[4] = { 0.f, 0.f, 0.f, 0.f };
                    int const x = bx * 64 + lane;
                    for (int r = 0; r < 16; ++r) {
                        int const y = by * 64 + wave * 16 + r;
                        if (x >= p->width || y >= p->height) continue;
                        uint8_t const* pa = static_cast<uint8_t const*>(p->a.data) + size_t(y + p->top) * p->a.rowPitch + size_t(x + p->left) * p->a.pixelStride;
                        uint8_t const* pb = static_cast<uint8_t const*>(p->b.data) + size_t(y + p->top) * p->b.rowPitch + size_t(x + p->left) * p->b.pixelStride;
                        float t1[4], t2[4], diff[4];
                        for (int c = 0; c < 4; ++c) { t1[c] = diff_channel(p->a, pa, c); t2[c] = diff_channel(p->b, pb, c); }
                        for (int c = 0; c < 4; ++c)
                            diff[c] = p->useMSLE ? logf(fabsf(t1[c]) + 1.f) - logf(fabsf(t2[c]) + 1.f) : t1[c] - t2[c];
                        if (p->useAlphaThreshold && t1[3] < p->alphaThreshold && t2[3] < p->alphaThreshold) diff[0] = diff[1] = diff[2] = 0.f;
                        for (int c = 0; c < 4; ++c) { float const sq = diff[c] * diff[c]; mse[c] = mse[c] + sq; }
                    }
                    for (int c = 0; c < 4; ++c) lanes[lane][c] = mse[c];
                }
                for (int off = 32; off >= 1; off >>= 1) {
                    float next[64][4];
                    for (int lane = 0; lane < 64; ++lane)
                        for (int c = 0; c < 4; ++c) next[lane][c] = lanes[lane][c] + lanes[lane ^ off][c];
                    std::memcpy(lanes, next, sizeof lanes);
                }
                for (int c = 0; c < 4; ++c) waveSum[wave][c] = lanes[0][c];
            }
            for (int c = 0; c < 4; ++c) {
                float total = ((waveSum[0][c] + waveSum[1][c]) + waveSum[2][c]) + waveSum[3][c];
                total = total / float(p->width * p->height);
                total = total * 65536.f;
                float const whole = floorf(total);
                uint64_t const high = saturating_u32(whole), low = saturating_u32(floorf((total - whole) * 4294967296.f));
                out[c] += (high << 32) | low;
            }
        }
}

// ---- BC4 / BC5 encoder (BC4_* of src/shaders/BlockCompressCommon.hlsli:510-796, CompressBC4.hlsl,
// CompressBC5.hlsl) --------------------------------------------------------------------------------------
// Both palettes of the format are tried: from start endpoints (the block's extremes moved inwards by
// range / 34; for the six-value palette the extremes that are not 0 / 255) texels are assigned to their
// nearest palette entry, then at most eight rounds of least-squares endpoints + re-assignment, ending
// when the error stops falling or the assignment repeats (hlsli:710-795).  HLSL round() is taken as
// round-half-even, clamp() as min(max()) (a NaN becomes the lower bound).
namespace bc4 {

void palette(uint32_t e0, uint32_t e1, uint32_t p[8])       // hlsli:563-603
{
    p[0] = e0; p[1] = e1;
    if (e0 > e1) {
        p[2] = (6 * e0 + 1 * e1 + 3) / 7; p[3] = (5 * e0 + 2 * e1 + 3) / 7; p[4] = (4 * e0 + 3 * e1 + 3) / 7;
        p[5] = (3 * e0 + 4 * e1 + 3) / 7; p[6] = (2 * e0 + 5 * e1 + 3) / 7; p[7] = (1 * e0 + 6 * e1 + 3) / 7;
    } else {
        p[2] = (4 * e0 + 1 * e1 + 2) / 5; p[3] = (3 * e0 + 2 * e1 + 2) / 5; p[4] = (2 * e0 + 3 * e1 + 2) / 5; p[5] = (1 * e0 + 4 * e1 + 2) / 5;
        p[6] = 0; p[7] = 255;
    }
}

struct Block {
    uint32_t e0 = 0, e1 = 0;
    uint32_t index[16] = {};
    bool same_indices(Block const& o) const { return std::memcmp(index, o.index, sizeof index) == 0; }
    uint64_t bits() const
    {
        uint64_t v = uint64_t(e0 & 0xffu) | (uint64_t(e1 & 0xffu) << 8);
        for (int t = 0; t < 16; ++t) v |= uint64_t(index[t] & 7u) << (16 + 3 * t);
        return v;
    }
};

float assign(const uint32_t values[16], Block& b)           // hlsli:605-632
{
    uint32_t pal[8];
    palette(b.e0 & 0xffu, b.e1 & 0xffu, pal);
    float total = 0.f;
    for (int t = 0; t < 16; ++t) {
        int best = 0x7fffffff;
        uint32_t pick = 8;
        for (uint32_t k = 0; k < 8; ++k) {
            int d = int(values[t]) - int(pal[k]);
            d *= d;
            if (d < best) { best = d; pick = k; }
        }
        total += float(best);
        b.index[t] = pick;
    }
    return total;
}

uint32_t endpoint(float v) { return uint32_t(std::nearbyint(std::fmin(std::fmax(v, 0.f), 255.f))); }

void refit8(const uint32_t values[16], Block& b, bool zeroE1, bool oneE0)     // hlsli:634-670
{
    float aa = 0, bb = 0, ab = 0, ax = 0, bx = 0;
    for (int t = 0; t < 16; ++t) {
        uint32_t const k = b.index[t];
        float const alpha = k < 2 ? 1.f - float(k) : (8.f - float(k)) / 7.f;
        float const beta = 1.f - alpha;
        aa += alpha * alpha; bb += beta * beta; ab += alpha * beta;
        ax += alpha * float(values[t]); bx += beta * float(values[t]);
    }
    float const factor = 1.f / (aa * bb - ab * ab);
    float const a = (ax * bb - bx * ab) * factor, c = (bx * aa - ax * ab) * factor;
    uint32_t e0 = oneE0 ? 255u : endpoint(a), e1 = zeroE1 ? 0u : endpoint(c);
    if (e0 < e1) std::swap(e0, e1);
    b.e0 = e0; b.e1 = e1;
}

void refit6(const uint32_t values[16], Block& b)            // hlsli:672-708
{
    float aa = 0, bb = 0, ab = 0, ax = 0, bx = 0;
    for (int t = 0; t < 16; ++t) {
        uint32_t const k = b.index[t];
        float alpha;
        if (k < 2) alpha = 1.f - float(k);
        else if (k < 6) alpha = (6.f - float(k)) / 5.f;
        else continue;
        float const beta = 1.f - alpha;
        aa += alpha * alpha; bb += beta * beta; ab += alpha * beta;
        ax += alpha * float(values[t]); bx += beta * float(values[t]);
    }
    float const factor = aa * bb - ab * ab;
    if (factor == 0.f) return;
    b.e0 = endpoint((ax * bb - bx * ab) / factor);
    b.e1 = endpoint((bx * aa - ax * ab) / factor);
}

uint64_t encode(const float texels[16])                     // hlsli:710-795
{
    uint32_t values[16], mina = 255, maxa = 0, minaInner = 255, maxaInner = 0;
    for (int t = 0; t < 16; ++t) {
        float const s = std::fmin(std::fmax(texels[t], 0.f), 1.f);
        values[t] = uint32_t(std::nearbyint(s * 255.f));
        mina = std::min(mina, values[t]); maxa = std::max(maxa, values[t]);
        if (values[t] != 0) minaInner = std::min(minaInner, values[t]);
        if (values[t] != 255) maxaInner = std::max(maxaInner, values[t]);
    }
    bool const zeroE1 = mina == 0, oneE0 = maxa == 255;

    Block block;
    block.e0 = oneE0 ? 255u : maxa - (maxa - mina) / 34u;
    block.e1 = zeroE1 ? 0u : mina + (maxa - mina) / 34u;
    float bestError = assign(values, block);
    Block best = block;
    for (int i = 0; i < 8; ++i) {
        refit8(values, block, zeroE1, oneE0);
        float const error = assign(values, block);
        if (error >= bestError) break;
        if (block.same_indices(best)) { best = block; break; }
        best = block; bestError = error;
    }

    block.e0 = (minaInner + (maxaInner - minaInner) / 34u) & 0xffu;     // uint32 arithmetic, wraps when there are no inner values
    block.e1 = (maxaInner - (maxaInner - minaInner) / 34u) & 0xffu;
    float bestError2 = assign(values, block);
    Block best2 = block;
    for (int i = 0; i < 8; ++i) {
        refit6(values, block);
        float const error = assign(values, block);
        if (error >= bestError2) break;
        if (block.same_indices(best2)) { best2 = block; break; }
        best2 = block; bestError2 = error;
    }
    return (bestError2 < bestError ? best2 : best).bits();
}

} // namespace bc4

// BC1 colour blocks: CompressBC1.hlsl, BC1_* of BlockCompressCommon.hlsli:36-493.  HLSL leaves the
// evaluation of dot / lerp / fused operations to the shader compiler; here every operation is a
// separate IEEE binary32 one, dot products add left to right, lerp(a, b, t) = a + (b - a) * t,
// round() is to nearest even.
namespace bc1 {
namespace {         // internal linkage: this file's functions sit in an extern "C" block

// hlsli:36-78: the two tables are the single-colour tables of NVTT.  Their rule, as published with
// stb_dxt / NVTT: for every 8-bit value, over endpoint pairs (first, second) with `second` in the outer
// loop, minimise 100 * |(2 * expand(first) + expand(second)) / 3 - value| + 3 * |first - second|
// (integer division), keeping the first minimum.  tests/ compares the result with the reference's
// literal tables.
struct MatchTables {
    uint16_t five[256], six[256];
    MatchTables()
    {
        for (int bits = 5; bits <= 6; ++bits)
            for (int value = 0; value < 256; ++value) {
                int best = INT32_MAX, pick = 0;
                for (int second = 0; second < (1 << bits); ++second)
                    for (int first = 0; first < (1 << bits); ++first) {
                        int const a = bits == 5 ? (first << 3) | (first >> 2) : (first << 2) | (first >> 4);
                        int const b = bits == 5 ? (second << 3) | (second >> 2) : (second << 2) | (second >> 4);
                        int const cost = 100 * std::abs((2 * a + b) / 3 - value) + 3 * std::abs(first - second);
                        if (cost < best) { best = cost; pick = first | (second << 8); }
                    }
                (bits == 5 ? five : six)[value] = uint16_t(pick);
            }
    }
};
MatchTables const& match_tables() { static MatchTables const t; return t; }

float sat(float v) { return std::fmin(std::fmax(v, 0.f), 1.f); }
float dist2(const float a[3], const float b[3])
{
    float const d0 = a[0] - b[0], d1 = a[1] - b[1], d2 = a[2] - b[2];
    return d0 * d0 + d1 * d1 + d2 * d2;
}
void lerp3(const float a[3], const float b[3], float t, float out[3]) { for (int c = 0; c < 3; ++c) out[c] = a[c] + (b[c] - a[c]) * t; }
void expand565(uint32_t w, float out[3])                                 // hlsli:181-188
{
    out[0] = float((w >> 11) & 0x1f) / 31.f; out[1] = float((w >> 5) & 0x3f) / 63.f; out[2] = float(w & 0x1f) / 31.f;
}
uint32_t round565(float v[3])                                            // hlsli:190-203, v becomes the rounded colour
{
    uint32_t const x = uint32_t(std::nearbyint(sat(v[0]) * 31.f)), y = uint32_t(std::nearbyint(sat(v[1]) * 63.f)), z = uint32_t(std::nearbyint(sat(v[2]) * 31.f));
    v[0] = float(x) / 31.f; v[1] = float(y) / 63.f; v[2] = float(z) / 31.f;
    return (x << 11) | (y << 5) | z;
}
uint32_t select_index(const float d[4], float& error)                    // hlsli:116-144
{
    uint32_t k;
    if (std::fmin(d[0], d[1]) < std::fmin(d[2], d[3])) k = d[0] < d[1] ? 0 : 1;
    else k = d[2] < d[3] ? 2 : 3;
    error = d[k];
    return k;
}
uint32_t index4(const float px[4], const float hi[3], const float lo[3], float& error)      // hlsli:146-159
{
    float c2[3], c3[3], d[4];
    lerp3(hi, lo, 1.f / 3.f, c2); lerp3(hi, lo, 2.f / 3.f, c3);
    float const alphaDistance = (1.f - px[3]) * (1.f - px[3]);
    d[0] = dist2(hi, px) + alphaDistance; d[1] = dist2(lo, px) + alphaDistance;
    d[2] = dist2(c2, px) + alphaDistance; d[3] = dist2(c3, px) + alphaDistance;
    return select_index(d, error);
}
uint32_t index3(const float px[4], const float hi[3], const float lo[3], float threshold, float& error)     // hlsli:161-179
{
    if (px[3] <= threshold) { error = 0.f; return 3; }
    float c2[3], d[4];
    lerp3(hi, lo, 0.5f, c2);
    float const alphaDistance = (1.f - px[3]) * (1.f - px[3]);
    d[0] = dist2(hi, px) + alphaDistance; d[1] = dist2(lo, px) + alphaDistance; d[2] = dist2(c2, px) + alphaDistance;
    d[3] = px[0] * px[0] + px[1] * px[1] + px[2] * px[2] + px[3] * px[3];
    return select_index(d, error);
}

struct Result { uint32_t x, y; float error; };

Result transparent_block(const float px[16][4], float threshold)        // hlsli:99-109
{
    Result r{ 0u, 0xffffffffu, 0.f };
    for (int t = 0; t < 16; ++t)
        if (!(px[t][3] <= threshold)) r.error += px[t][0] * px[t][0] + px[t][1] * px[t][1] + px[t][2] * px[t][2] + px[t][3] * px[t][3];
    return r;
}

Result single_color(const float px[16][4])                               // hlsli:205-247
{
    float avg[3] = { 0.f, 0.f, 0.f };
    for (int t = 0; t < 16; ++t) for (int c = 0; c < 3; ++c) avg[c] += px[t][c];
    uint32_t m[3];
    for (int c = 0; c < 3; ++c) {
        // the reference indexes its table with the rounded mean unchecked; outside [0, 255] (inputs outside
        // [0, 1]) that read is undefined there and clamped here
        float const i = std::fmin(std::fmax(std::nearbyint(avg[c] / 16.f * 255.f), 0.f), 255.f);
        m[c] = (c == 1 ? match_tables().six : match_tables().five)[int(i)];
    }
    uint32_t const color0 = ((m[0] & 0x1f) << 11) | ((m[1] & 0x3f) << 5) | (m[2] & 0x1f);
    uint32_t const color1 = (((m[0] >> 8) & 0x1f) << 11) | (((m[1] >> 8) & 0x3f) << 5) | ((m[2] >> 8) & 0x1f);
    Result r;
    if (color0 < color1) { r.x = (color0 << 16) | color1; r.y = 0xffffffffu; }
    else                 { r.x = (color1 << 16) | color0; r.y = 0xaaaaaaaau; }
    float e0[3], e1[3], enc[3];
    expand565(color0, e0); expand565(color1, e1); lerp3(e0, e1, 1.f / 3.f, enc);
    r.error = 0.f;
    for (int t = 0; t < 16; ++t) {
        float const d0 = px[t][0] - enc[0], d1 = px[t][1] - enc[1], d2 = px[t][2] - enc[2], d3 = px[t][3] - 1.f;
        r.error += d0 * d0 + d1 * d1 + d2 * d2 + d3 * d3;
    }
    return r;
}

// Shared start of both fitted modes (hlsli:251-290, 380-424): bounding box of the texels in `use`,
// component ends swapped by covariance sign, inset by extent / divisor.
void start_box(const float px[16][4], const bool use[16], float divisor, int count, float lo[3], float hi[3])
{
    float sums[3] = { 0, 0, 0 };
    for (int c = 0; c < 3; ++c) { lo[c] = 1.f; hi[c] = 0.f; }
    for (int t = 0; t < 16; ++t) if (use[t])
        for (int c = 0; c < 3; ++c) { sums[c] += px[t][c]; lo[c] = std::fmin(lo[c], px[t][c]); hi[c] = std::fmax(hi[c], px[t][c]); }
    float center[3] = { 0, 0, 0 };
    if (count > 0) for (int c = 0; c < 3; ++c) center[c] = sums[c] / float(count);
    float rg = 0, rb = 0, gb = 0;
    for (int t = 0; t < 16; ++t) if (use[t]) {
        float const r = px[t][0] - center[0], g = px[t][1] - center[1], b = px[t][2] - center[2];
        rg += r * g; rb += r * b; gb += g * b;
    }
    if (lo[0] != hi[0]) {
        if (rg < 0) std::swap(lo[1], hi[1]);
        if (rb < 0) std::swap(lo[2], hi[2]);
    } else if (lo[1] != hi[1]) {
        if (gb < 0) std::swap(lo[2], hi[2]);
    }
    for (int c = 0; c < 3; ++c) {
        float const inset = (hi[c] - lo[c]) / divisor;
        hi[c] = sat(hi[c] - inset);
        lo[c] = sat(lo[c] + inset);
    }
}

struct Sums { float a2 = 0, b2 = 0, ab = 0, ax[3] = { 0, 0, 0 }, bx[3] = { 0, 0, 0 }; };
void accumulate(Sums& s, float beta, const float px[4])
{
    float const alpha = 1.f - beta;
    s.a2 += alpha * alpha; s.b2 += beta * beta; s.ab += alpha * beta;
    for (int c = 0; c < 3; ++c) { s.ax[c] += alpha * px[c]; s.bx[c] += beta * px[c]; }
}
bool solve(Sums const& s, float a[3], float b[3])
{
    float const denom = s.a2 * s.b2 - s.ab * s.ab;
    if (!(std::fabs(denom) > 0.0001f)) return false;
    float const factor = 1.f / denom;
    for (int c = 0; c < 3; ++c) {
        a[c] = (s.ax[c] * s.b2 - s.bx[c] * s.ab) * factor;
        b[c] = (s.bx[c] * s.a2 - s.ax[c] * s.ab) * factor;
    }
    return true;
}
void keep_extremes(float cur[3], const float fitted[3])                 // "preserve 0 and 1 cases"
{
    for (int c = 0; c < 3; ++c) if (!(cur[c] == 0.f || cur[c] == 1.f)) cur[c] = sat(fitted[c]);
}

Result compress_fast(const float px[16][4])                              // hlsli:249-376
{
    bool all[16]; for (bool& u : all) u = true;
    float lo[3], hi[3];
    start_box(px, all, 16.f, 16, lo, hi);
    uint32_t color0 = 0, color1 = 0;
    for (int pass = 0; pass < 4; ++pass) {
        Sums s;
        for (int t = 0; t < 16; ++t) {
            float e;
            uint32_t const index = index4(px[t], hi, lo, e);
            float beta = float(index & 1);
            if (index & 2) beta = (1 + beta) / 3.0f;
            accumulate(s, beta, px[t]);
        }
        float a[3], b[3];
        if (solve(s, a, b)) { keep_extremes(lo, b); keep_extremes(hi, a); }
        uint32_t const new0 = round565(hi), new1 = round565(lo);
        if (new0 == color0 && new1 == color1) break;
        color0 = new0; color1 = new1;
    }
    if (color0 == color1) {
        if (color0 == 0) { color0 = 1; expand565(color0, hi); }
        else { color1 = color0 - 1; expand565(color1, lo); }
    } else if (color0 < color1) {
        for (int c = 0; c < 3; ++c) std::swap(hi[c], lo[c]);
        std::swap(color0, color1);
    }
    Result r{ (color1 << 16) | color0, 0u, 0.f };
    for (int t = 0; t < 16; ++t) {
        float e;
        r.y |= index4(px[t], hi, lo, e) << (2 * t);
        r.error += e;
    }
    return r;
}

Result compress_fast_alpha(const float px[16][4], float threshold)       // hlsli:378-493
{
    bool opaque[16]; int count = 0;
    for (int t = 0; t < 16; ++t) { opaque[t] = !(px[t][3] <= threshold); count += opaque[t]; }
    float lo[3], hi[3];
    start_box(px, opaque, float(count), count, lo, hi);
    Sums s;
    for (int t = 0; t < 16; ++t) {
        float e;
        uint32_t const index = index3(px[t], hi, lo, threshold, e);
        if (index != 3) accumulate(s, (index & 2) ? 0.5f : float(index & 1), px[t]);
    }
    float a[3], b[3];
    if (solve(s, a, b)) { keep_extremes(lo, a); keep_extremes(hi, b); }     // a -> min, b -> max: as written at hlsli:453-455
    uint32_t color0 = round565(hi), color1 = round565(lo);
    if (color0 > color1) {
        for (int c = 0; c < 3; ++c) std::swap(hi[c], lo[c]);
        std::swap(color0, color1);
    }
    Result r{ (color1 << 16) | color0, 0u, 0.f };
    for (int t = 0; t < 16; ++t) {
        float e;
        uint32_t const index = index3(px[t], hi, lo, threshold, e);
        r.y |= index << (2 * t);
        if (index != 3 || opaque[t]) r.error += e;
    }
    return r;
}

// CompressBC1.hlsl:31-63 (withAlpha) / CompressBC2.hlsl, CompressBC3.hlsl:32-43 (alpha forced to 1 by the caller)
uint64_t encode_color(const float px[16][4], bool withAlpha, float threshold)
{
    Result best;
    if (withAlpha) {
        best = transparent_block(px, threshold);
        Result const one = single_color(px);
        if (one.error < best.error) best = one;
    } else best = single_color(px);
    Result const four = compress_fast(px);
    if (four.error < best.error) best = four;
    if (withAlpha) {
        Result const three = compress_fast_alpha(px, threshold);
        if (three.error < best.error) best = three;
    }
    return uint64_t(best.x) | (uint64_t(best.y) << 32);
}

uint64_t bc2_alpha(const float alpha[16])                                // hlsli:495-508
{
    uint64_t v = 0;
    for (int t = 0; t < 16; ++t) v |= uint64_t(uint32_t(std::nearbyint(sat(alpha[t]) * 15.f))) << (4 * t);
    return v;
}

} // namespace
} // namespace bc1

// ---- BC7 encoder (src/shaders/CompressBC7.hlsl) --------------------------------------------------------
// The reference tries, per block: for opaque blocks the three-subset modes 0 / 2 and the two-subset
// modes 1 / 3 (partition chosen by an estimated error over all 64 partitions), then for every block
// modes 4 and 5 in all four channel rotations, mode 6 and mode 7; a candidate replaces the current
// block when its error is not larger.  With a mode buffer (one 9-bit mode + partition entry per
// block, MakeBC7ModeBuffer) only that mode and partition are encoded and no error is computed.
// Same float conventions as for BC1: separate IEEE binary32 operations, dot products left to right,
// round() to nearest even.
extern "C++" {      // templates: not inside this file's extern "C" block
namespace bc7 {
namespace {

// Table.P2 and Table.P3 of the BPTC format specification (ARB_texture_compression_bptc): the subset of
// each of the 16 texels, texel 0 first; anchor tables A2, A3a, A3b of the same specification.
const char* const kTwoSubsets[64] = {
    "0011001100110011", "0001000100010001", "0111011101110111", "0001001100110111",
    "0000000100010011", "0011011101111111", "0001001101111111", "0000000100110111",
    "0000000000010011", "0011011111111111", "0000000101111111", "0000000000010111",
    "0001011111111111", "0000000011111111", "0000111111111111", "0000000000001111",
    "0000100011101111", "0111000100000000", "0000000010001110", "0111001100010000",
    "0011000100000000", "0000100011001110", "0000000010001100", "0111001100110001",
    "0011000100010000", "0000100010001100", "0110011001100110", "0011011001101100",
    "0001011111101000", "0000111111110000", "0111000110001110", "0011100110011100",
    "0101010101010101", "0000111100001111", "0101101001011010", "0011001111001100",
    "0011110000111100", "0101010110101010", "0110100101101001", "0101101010100101",
    "0111001111001110", "0001001111001000", "0011001001001100", "0011101111011100",
    "0110100110010110", "0011110011000011", "0110011010011001", "0000011001100000",
    "0100111001000000", "0010011100100000", "0000001001110010", "0000010011100100",
    "0110110010010011", "0011011011001001", "0110001110011100", "0011100111000110",
    "0110110011001001", "0110001100111001", "0111111010000001", "0001100011100111",
    "0000111100110011", "0011001111110000", "0010001011101110", "0100010001110111",
};
const char* const kThreeSubsets[64] = {
    "0011001102212222", "0001001122112221", "0000200122112211", "0222002200110111",
    "0000000011221122", "0011001100220022", "0022002211111111", "0011001122112211",
    "0000000011112222", "0000111111112222", "0000111122222222", "0012001200120012",
    "0112011201120112", "0122012201220122", "0011011211221222", "0011200122002220",
    "0001001101121122", "0111001120012200", "0000112211221122", "0022002200221111",
    "0111011102220222", "0001000122212221", "0000001101220122", "0000110022102210",
    "0122012200110000", "0012001211222222", "0110122112210110", "0000011012211221",
    "0022110211020022", "0110011020022222", "0011012201220011", "0000200022112221",
    "0000000211221222", "0222002200120011", "0011001200220222", "0120012001200120",
    "0000111122220000", "0120120120120120", "0120201212010120", "0011220011220011",
    "0011112222000011", "0101010122222222", "0000000021212121", "0022112200221122",
    "0022001100220011", "0220122102201221", "0101222222220101", "0000212121212121",
    "0101010101012222", "0222011102220111", "0002111200021112", "0000211221122112",
    "0222011101110222", "0002111211120002", "0110011001102222", "0000000021122112",
    "0110011022222222", "0022001100110022", "0022112211220022", "0000000000002112",
    "0002000100020001", "0222122202221222", "0101222222222222", "0111201122012220",
};
const uint8_t kAnchorSecondOfTwo[64] = {
    15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15,
    15,  2,  8,  2,  2,  8,  8, 15,  2,  8,  2,  2,  8,  8,  2,  2,
    15, 15,  6,  8,  2,  8, 15, 15,  2,  8,  2,  2,  2, 15, 15,  6,
     6,  2,  6,  8, 15, 15,  2,  2, 15, 15, 15, 15, 15,  2,  2, 15,
};
const uint8_t kAnchorSecondOfThree[64] = {
     3,  3, 15, 15,  8,  3, 15, 15,  8,  8,  6,  6,  6,  5,  3,  3,
     3,  3,  8, 15,  3,  3,  6, 10,  5,  8,  8,  6,  8,  5, 15, 15,
     8, 15,  3,  5,  6, 10,  8, 15, 15,  3, 15,  5, 15, 15, 15, 15,
     3, 15,  5,  5,  5,  8,  5, 10,  5, 10,  8, 13, 15, 12,  3,  3,
};
const uint8_t kAnchorThirdOfThree[64] = {
    15,  8,  8,  3, 15, 15,  3,  8, 15, 15, 15, 15, 15, 15, 15,  8,
    15,  8, 15,  3, 15,  8, 15,  8,  3, 15,  6, 10, 15, 15, 10,  8,
    15,  3, 15, 10, 10,  8,  9, 10,  6, 15,  8, 15,  3,  6,  6,  8,
    15,  3, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15,  3, 15, 15,  8,
};
struct Masks {
    uint32_t two[64][2], three[64][3];
    Masks()
    {
        for (int p = 0; p < 64; ++p) {
            two[p][0] = two[p][1] = three[p][0] = three[p][1] = three[p][2] = 0;
            for (int t = 0; t < 16; ++t) {
                two[p][kTwoSubsets[p][t] - '0'] |= 1u << t;
                three[p][kThreeSubsets[p][t] - '0'] |= 1u << t;
            }
        }
    }
};
Masks const& masks() { static Masks const m; return m; }

uint32_t subset_mask(int subsets, int partition, int s) { return subsets == 1 ? 0xffffu : subsets == 2 ? masks().two[partition][s] : masks().three[partition][s]; }
int subset_anchor(int subsets, int partition, int s)
{
    if (s == 0) return 0;
    if (subsets == 2) return kAnchorSecondOfTwo[partition];
    return s == 1 ? kAnchorSecondOfThree[partition] : kAnchorThirdOfThree[partition];
}

template <int C> struct Color { float c[C]; };
float sat(float v) { return std::fmin(std::fmax(v, 0.f), 1.f); }
template <int C> float dot(Color<C> const& a, Color<C> const& b) { float s = a.c[0] * b.c[0]; for (int k = 1; k < C; ++k) s += a.c[k] * b.c[k]; return s; }
template <int C> Color<C> sub(Color<C> const& a, Color<C> const& b) { Color<C> r; for (int k = 0; k < C; ++k) r.c[k] = a.c[k] - b.c[k]; return r; }
int popcount16(uint32_t m) { int n = 0; for (int t = 0; t < 16; ++t) n += (m >> t) & 1; return n; }

template <int C> void min_max(const Color<C> px[16], uint32_t mask, Color<C>& lo, Color<C>& hi)          // hlsl:175-189
{
    for (int k = 0; k < C; ++k) { lo.c[k] = FLT_MAX; hi.c[k] = -FLT_MAX; }
    for (int t = 0; t < 16; ++t) if (mask & (1u << t))
        for (int k = 0; k < C; ++k) { lo.c[k] = std::fmin(lo.c[k], px[t].c[k]); hi.c[k] = std::fmax(hi.c[k], px[t].c[k]); }
}

// hlsl:243-343: with the first component whose ends differ as the axis, later components' ends are swapped
// where their covariance with the axis is negative.
template <int C> void orient(const Color<C> px[16], uint32_t mask, Color<C>& e0, Color<C>& e1)
{
    Color<C> center;
    for (int k = 0; k < C; ++k) center.c[k] = 0.f;
    for (int t = 0; t < 16; ++t) if (mask & (1u << t)) for (int k = 0; k < C; ++k) center.c[k] += px[t].c[k];
    float const count = float(popcount16(mask));
    for (int k = 0; k < C; ++k) center.c[k] /= count;
    float cov[C][C] = {};
    for (int t = 0; t < 16; ++t) if (mask & (1u << t)) {
        Color<C> const d = sub(px[t], center);
        for (int a = 0; a < C; ++a) for (int b = a + 1; b < C; ++b) cov[a][b] += d.c[a] * d.c[b];
    }
    for (int a = 0; a + 1 < C; ++a)
        if (e0.c[a] != e1.c[a]) {
            for (int b = a + 1; b < C; ++b) if (cov[a][b] < 0.f) std::swap(e0.c[b], e1.c[b]);
            break;
        }
}

template <int C> void refine(const Color<C> px[16], uint32_t mask, Color<C>& e0, Color<C>& e1, int indexBits)     // hlsl:191-241
{
    for (int iter = 0; iter < 2; ++iter) {
        Color<C> const axis = sub(e1, e0);
        float mul = dot(axis, axis);
        if (mul > 0.f) mul = 1.f / mul;
        float const scale = float((1u << indexBits) - 1), iscale = 1.f / scale;
        float a2 = 0, b2 = 0, ab = 0;
        Color<C> ax, bx;
        for (int k = 0; k < C; ++k) ax.c[k] = bx.c[k] = 0.f;
        for (int t = 0; t < 16; ++t) if (mask & (1u << t)) {
            float const f = sat(dot(sub(px[t], e0), axis) * mul);
            float const beta = std::nearbyint(f * scale) * iscale, alpha = 1.f - beta;
            a2 += alpha * alpha; b2 += beta * beta; ab += alpha * beta;
            for (int k = 0; k < C; ++k) { ax.c[k] += alpha * px[t].c[k]; bx.c[k] += beta * px[t].c[k]; }
        }
        float const denom = a2 * b2 - ab * ab;
        if (!(std::fabs(denom) > 0.0001f)) break;
        float const factor = 1.f / denom;
        for (int k = 0; k < C; ++k) {
            float const a = sat((ax.c[k] * b2 - bx.c[k] * ab) * factor), b = sat((bx.c[k] * a2 - ax.c[k] * ab) * factor);
            if (!(e0.c[k] == 0.f || e0.c[k] == 1.f)) e0.c[k] = a;
            if (!(e1.c[k] == 0.f || e1.c[k] == 1.f)) e1.c[k] = b;
        }
    }
}

template <int C> float estimate(const Color<C> px[16], uint32_t mask, Color<C> const& e0, Color<C> const& e1, int indexBits)     // hlsl:345-373
{
    Color<C> const axis = sub(e1, e0);
    float mul = dot(axis, axis);
    if (mul > 0.f) mul = 1.f / mul;
    float const maxIndex = float((1u << indexBits) - 1), indexScale = 1.f / maxIndex;
    float error = 0.f;
    for (int t = 0; t < 16; ++t) if (mask & (1u << t)) {
        Color<C> const p = sub(px[t], e0);
        float f = dot(p, axis) * mul;
        f = std::nearbyint(f * maxIndex) * indexScale;
        Color<C> diff;
        for (int k = 0; k < C; ++k) diff.c[k] = f * axis.c[k] - p.c[k];
        error += dot(diff, diff);
    }
    return error;
}

int quantize(float v, int bits) { return int(std::nearbyint(sat(v) * float((1u << bits) - 1))); }         // hlsl:131-135
int expand8(int q, int bits) { return (q << (8 - bits)) | (q >> (2 * bits - 8)); }                       // hlsl:154-157

template <int C> struct Quantized { int c[C]; };

template <int C> float decoded_error(const Color<C> px[16], const int index[16], uint32_t mask, Quantized<C> q0, Quantized<C> q1,
                                     int indexBits, int endpointBits)                                    // hlsl:375-405
{
    for (int k = 0; k < C; ++k) { q0.c[k] = expand8(q0.c[k], endpointBits); q1.c[k] = expand8(q1.c[k], endpointBits); }
    float const indexScale = 64.f / float((1u << indexBits) - 1);
    float error = 0.f;
    for (int t = 0; t < 16; ++t) if (mask & (1u << t)) {
        int const w = int(std::nearbyint(float(index[t]) * indexScale));
        Color<C> diff;
        for (int k = 0; k < C; ++k) diff.c[k] = float((q0.c[k] * (64 - w) + q1.c[k] * w + 32) >> 6) / 255.f - px[t].c[k];
        error += dot(diff, diff);
    }
    return error;
}

// Indices of a subset's texels along the dequantised endpoints; when the anchor texel's index has its
// top bit set all of the subset's indices are complemented and true is returned (the caller then
// swaps the endpoints).  hlsl:445-527
template <int C> bool assign(const Color<C> px[16], uint32_t mask, int anchor, int indexBits, int endpointBits,
                             Quantized<C> const& q0, Quantized<C> const& q1, int index[16])
{
    Color<C> e0, e1;
    for (int k = 0; k < C; ++k) { e0.c[k] = float(expand8(q0.c[k], endpointBits)) / 255.f; e1.c[k] = float(expand8(q1.c[k], endpointBits)) / 255.f; }
    Color<C> const axis = sub(e1, e0);
    float mul = dot(axis, axis);
    if (mul > 0.f) mul = 1.f / mul;
    for (int t = 0; t < 16; ++t) if (mask & (1u << t)) index[t] = quantize(dot(sub(px[t], e0), axis) * mul, indexBits);
    bool const flip = (index[anchor] >> (indexBits - 1)) & 1;
    if (flip) for (int t = 0; t < 16; ++t) if (mask & (1u << t)) index[t] ^= (1 << indexBits) - 1;
    return flip;
}

struct Bits {
    uint64_t lo = 0, hi = 0;
    int at = 0;
    void put(int length, uint32_t value)
    {
        uint64_t const v = value & ((1u << length) - 1u);
        if (at < 64) { lo |= v << at; if (at + length > 64) hi |= v >> (64 - at); }
        else hi |= v << (at - 64);
        at += length;
    }
};

struct Best { float error = FLT_MAX; uint64_t lo = 0, hi = 0; bool fixedMode = false; };

enum PBit { kNoPBit, kPBitPerEndpoint, kPBitPerSubset };
struct Mode { int id, subsets, partitionBits, endpointBits /* with the p-bit */, indexBits; PBit pbit; };
const Mode kMode0{ 0, 3, 4, 5, 3, kPBitPerEndpoint }, kMode1{ 1, 2, 6, 7, 3, kPBitPerSubset }, kMode2{ 2, 3, 6, 5, 2, kNoPBit },
           kMode3{ 3, 2, 6, 8, 2, kPBitPerEndpoint }, kMode6{ 6, 1, 0, 8, 4, kPBitPerEndpoint }, kMode7{ 7, 2, 6, 6, 2, kPBitPerEndpoint };

// hlsl:407-443: endpoint quantisation with the mode's p-bit rule.
template <int C> void quantize_endpoints(Mode const& m, const Color<C> e[6], Quantized<C> q[6])
{
    int const n = 2 * m.subsets;
    for (int i = 0; i < n; ++i) for (int k = 0; k < C; ++k) q[i].c[k] = quantize(e[i].c[k], m.endpointBits);
    if (m.pbit == kPBitPerEndpoint) {
        for (int i = 0; i < n; ++i) {
            int odd = 0;
            for (int k = 0; k < C; ++k) odd += q[i].c[k] & 1;
            int lsb = odd >= 2 ? 1 : 0;
            if (C == 4) lsb = ((odd >= 2 && q[i].c[3] != 0) || e[i].c[3] == 1.f) ? 1 : 0;      // keeps alpha 0 and alpha 1 exact
            for (int k = 0; k < C; ++k) q[i].c[k] = (q[i].c[k] & 0xFE) | lsb;
        }
    } else if (m.pbit == kPBitPerSubset) {
        for (int i = 0; i < n; i += 2) {
            int odd = 0;
            for (int k = 0; k < C; ++k) odd += (q[i].c[k] & 1) + (q[i + 1].c[k] & 1);
            int const lsb = odd >= 4 ? 1 : 0;
            for (int k = 0; k < C; ++k) { q[i].c[k] = (q[i].c[k] & 0xFE) | lsb; q[i + 1].c[k] = (q[i + 1].c[k] & 0xFE) | lsb; }
        }
    }
}

// Refines the start endpoints of every subset, quantises, assigns indices and, if the result is not
// worse than the best so far, encodes the block (hlsl:570-726, 787-928, 1247-1407).
template <int C> void finish(Mode const& m, const Color<C> px[16], int partition, const Color<C> start[6], Best& best)
{
    Color<C> e[6];
    Quantized<C> q[6];
    for (int i = 0; i < 2 * m.subsets; ++i) e[i] = start[i];
    for (int s = 0; s < m.subsets; ++s) refine(px, subset_mask(m.subsets, partition, s), e[2 * s], e[2 * s + 1], m.indexBits);
    quantize_endpoints(m, e, q);
    int index[16] = {};
    float error = 0.f;
    for (int s = 0; s < m.subsets; ++s) {
        uint32_t const mask = subset_mask(m.subsets, partition, s);
        if (assign(px, mask, subset_anchor(m.subsets, partition, s), m.indexBits, m.endpointBits, q[2 * s], q[2 * s + 1], index))
            std::swap(q[2 * s], q[2 * s + 1]);
        if (!best.fixedMode) {
            float const e2 = decoded_error(px, index, mask, q[2 * s], q[2 * s + 1], m.indexBits, m.endpointBits);
            error = s == 0 ? e2 : error + e2;
        }
    }
    if (error > best.error) return;
    Bits b;
    b.put(m.id + 1, 1u << m.id);
    b.put(m.partitionBits, uint32_t(partition));
    int const drop = m.pbit == kNoPBit ? 0 : 1;
    for (int k = 0; k < C; ++k) for (int i = 0; i < 2 * m.subsets; ++i) b.put(m.endpointBits - drop, uint32_t(q[i].c[k]) >> drop);
    if (m.pbit == kPBitPerEndpoint) for (int i = 0; i < 2 * m.subsets; ++i) b.put(1, uint32_t(q[i].c[0]));
    if (m.pbit == kPBitPerSubset) for (int s = 0; s < m.subsets; ++s) b.put(1, uint32_t(q[2 * s].c[0]));
    for (int t = 0; t < 16; ++t) {
        bool anchor = t == 0;
        for (int s = 1; s < m.subsets; ++s) anchor = anchor || t == subset_anchor(m.subsets, partition, s);
        b.put(anchor ? m.indexBits - 1 : m.indexBits, uint32_t(index[t]));
    }
    best.error = error; best.lo = b.lo; best.hi = b.hi;
}

// Start endpoints (bounding box per subset, oriented) for one partition, and their estimated error.
template <int C> float start_endpoints(const Color<C> px[16], int subsets, int partition, bool orientEnds, int searchIndexBits, bool wantError, Color<C> e[6])
{
    float error = 0.f;
    for (int s = 0; s < subsets; ++s) min_max(px, subset_mask(subsets, partition, s), e[2 * s], e[2 * s + 1]);
    if (orientEnds) for (int s = 0; s < subsets; ++s) orient(px, subset_mask(subsets, partition, s), e[2 * s], e[2 * s + 1]);
    if (wantError)
        for (int s = 0; s < subsets; ++s) {
            float const e2 = estimate(px, subset_mask(subsets, partition, s), e[2 * s], e[2 * s + 1], searchIndexBits);
            error = s == 0 ? e2 : error + e2;
        }
    return error;
}

// The partition with the smallest estimated error (the first of equals) and its start endpoints; with a
// fixed partition just that one's endpoints (hlsl:728-785, 930-983, 1296-1345).
template <int C> int pick_partition(const Color<C> px[16], int subsets, bool orientEnds, int searchIndexBits, int fixedPartition, Color<C> bestEnds[6])
{
    if (fixedPartition >= 0) { start_endpoints(px, subsets, fixedPartition, orientEnds, searchIndexBits, false, bestEnds); return fixedPartition; }
    int bestPartition = 0;
    float bestError = FLT_MAX;
    // a NaN texel makes every estimate NaN and no partition "best": the reference then goes on with
    // uninitialised endpoints, here they are zero (and the partition 0)
    for (int i = 0; i < 2 * subsets; ++i) for (int k = 0; k < C; ++k) bestEnds[i].c[k] = 0.f;
    for (int p = 0; p < 64; ++p) {
        Color<C> e[6];
        float const error = start_endpoints(px, subsets, p, orientEnds, searchIndexBits, true, e);
        if (error < bestError) { bestPartition = p; bestError = error; for (int i = 0; i < 2 * subsets; ++i) bestEnds[i] = e[i]; }
    }
    return bestPartition;
}

// Modes 4 and 5: a colour plane of three channels and a scalar plane, each with its own endpoints and
// indices; `px` is already rotated so that the scalar channel is the fourth (hlsl:985-1148).
void dual_plane(int mode, bool wideColorIndex, const Color<4> px[16], uint32_t rotation, Best& best)
{
    int const colorIndexBits = mode == 5 ? 2 : (wideColorIndex ? 3 : 2), alphaIndexBits = mode == 5 ? 2 : (wideColorIndex ? 2 : 3);
    int const colorBits = mode == 5 ? 7 : 5, alphaBits = mode == 5 ? 8 : 6;
    Color<3> rgb[16];
    Color<1> a[16];
    for (int t = 0; t < 16; ++t) { rgb[t] = Color<3>{ { px[t].c[0], px[t].c[1], px[t].c[2] } }; a[t] = Color<1>{ { px[t].c[3] } }; }
    Color<1> a0, a1;
    min_max(a, 0xffffu, a0, a1);
    refine(a, 0xffffu, a0, a1, alphaIndexBits);
    Color<3> e0, e1;
    min_max(rgb, 0xffffu, e0, e1);
    orient(rgb, 0xffffu, e0, e1);
    refine(rgb, 0xffffu, e0, e1, colorIndexBits);
    Quantized<3> q0, q1;
    for (int k = 0; k < 3; ++k) { q0.c[k] = quantize(e0.c[k], colorBits); q1.c[k] = quantize(e1.c[k], colorBits); }
    Quantized<1> qa0{ { quantize(a0.c[0], alphaBits) } }, qa1{ { quantize(a1.c[0], alphaBits) } };
    int colorIndex[16], alphaIndex[16];
    float error = 0.f;
    if (assign(rgb, 0xffffu, 0, colorIndexBits, colorBits, q0, q1, colorIndex)) std::swap(q0, q1);
    if (!best.fixedMode) error = decoded_error(rgb, colorIndex, 0xffffu, q0, q1, colorIndexBits, colorBits);
    if (assign(a, 0xffffu, 0, alphaIndexBits, alphaBits, qa0, qa1, alphaIndex)) std::swap(qa0, qa1);
    if (!best.fixedMode) error += decoded_error(a, alphaIndex, 0xffffu, qa0, qa1, alphaIndexBits, alphaBits);
    if (error > best.error) return;
    Bits b;
    b.put(mode + 1, 1u << mode);
    b.put(2, rotation);
    if (mode == 4) b.put(1, wideColorIndex ? 1u : 0u);
    for (int k = 0; k < 3; ++k) { b.put(colorBits, uint32_t(q0.c[k])); b.put(colorBits, uint32_t(q1.c[k])); }
    b.put(alphaBits, uint32_t(qa0.c[0])); b.put(alphaBits, uint32_t(qa1.c[0]));
    // mode 4 stores its 2-bit indices first, then the 3-bit ones; mode 5 colour first, then the scalar
    bool const alphaFirst = mode == 4 && wideColorIndex;
    const int* first = alphaFirst ? alphaIndex : colorIndex;
    const int* second = alphaFirst ? colorIndex : alphaIndex;
    int const firstBits = alphaFirst ? alphaIndexBits : colorIndexBits, secondBits = alphaFirst ? colorIndexBits : alphaIndexBits;
    for (int t = 0; t < 16; ++t) b.put(t == 0 ? firstBits - 1 : firstBits, uint32_t(first[t]));
    for (int t = 0; t < 16; ++t) b.put(t == 0 ? secondBits - 1 : secondBits, uint32_t(second[t]));
    best.error = error; best.lo = b.lo; best.hi = b.hi;
}

// Channel order for rotation r: the scalar plane takes channel {A, R, G, B}[r], alpha takes its place.
void rotate(const Color<4> px[16], uint32_t rotation, Color<4> out[16])
{
    for (int t = 0; t < 16; ++t) {
        out[t] = px[t];
        if (rotation) std::swap(out[t].c[rotation - 1], out[t].c[3]);
    }
}

// One block.  fixedMode < 0: every mode is tried (CompressBC7.hlsl:1575-1587); otherwise only that
// mode with that partition (for modes 4 / 5: rotation in bits 0-1, "wide colour index" in bit 2).
void encode(const Color<4> px[16], int fixedMode, int fixedPartition, uint64_t out[2])
{
    Best best;
    best.fixedMode = fixedMode >= 0;
    Color<3> rgb[16];
    bool opaque = true;
    for (int t = 0; t < 16; ++t) { rgb[t] = Color<3>{ { px[t].c[0], px[t].c[1], px[t].c[2] } }; if (px[t].c[3] < 1.f) opaque = false; }
    auto three_subsets = [&](bool mode0, bool mode2, int partition) {
        Color<3> ends[6];
        int const p = pick_partition(rgb, 3, true, 3, partition, ends);
        if (mode0 && (partition >= 0 || p < 16)) finish(kMode0, rgb, p, ends, best);
        if (mode2) finish(kMode2, rgb, p, ends, best);
    };
    auto two_subsets = [&](bool mode1, bool mode3, int partition) {
        Color<3> ends[6];
        int const p = pick_partition(rgb, 2, true, 3, partition, ends);
        if (mode1) finish(kMode1, rgb, p, ends, best);
        if (mode3) finish(kMode3, rgb, p, ends, best);
    };
    auto mode6 = [&]() {
        Color<4> ends[6];
        start_endpoints(px, 1, 0, true, 4, false, ends);
        finish(kMode6, px, 0, ends, best);
    };
    auto mode7 = [&](int partition) {
        Color<4> ends[6];
        int const p = pick_partition(px, 2, false, 2, partition, ends);
        finish(kMode7, px, p, ends, best);
    };
    if (fixedMode < 0) {
        if (opaque) { three_subsets(true, true, -1); two_subsets(true, true, -1); }
        for (uint32_t rotation = 0; rotation < 4; ++rotation) {
            Color<4> r[16];
            rotate(px, rotation, r);
            dual_plane(4, false, r, rotation, best);
            dual_plane(4, true, r, rotation, best);
            dual_plane(5, false, r, rotation, best);
        }
        mode6();
        mode7(-1);
    } else {
        switch (fixedMode) {
        case 0: three_subsets(true, false, fixedPartition); break;
        case 2: three_subsets(false, true, fixedPartition); break;
        case 1: two_subsets(true, false, fixedPartition); break;
        case 3: two_subsets(false, true, fixedPartition); break;
        case 4: case 5: {
            Color<4> r[16];
            rotate(px, uint32_t(fixedPartition) & 3u, r);
            dual_plane(fixedMode, fixedMode == 4 && (fixedPartition & 4), r, uint32_t(fixedPartition) & 3u, best);
            break;
        }
        case 6: mode6(); break;
        default: mode7(fixedPartition); break;
        }
    }
    out[0] = best.lo; out[1] = best.hi;
}

} // namespace
} // namespace bc7
} // extern "C++"

// ---- BC6H encoder, unsigned half floats (src/shaders/CompressBC6.hlsl) ----------------------------------
// Two candidates per block, the smaller mean squared logarithmic error (luminance-weighted) wins:
//   * one subset, 10-bit endpoints, 4-bit indices (mode 11): bounding box, inset in log2 space by at most 1/32
//     of its extent towards the second-smallest / second-largest values, one least-squares refit;
//   * two subsets, 3-bit indices, on the partition (of the format's first 32) whose texels lie closest to the
//     two bounding-box diagonals: endpoints as 7-bit base + 6-bit deltas (mode 2) or 9-bit base + 5-bit deltas
//     (mode 6), whichever decodes with the smaller error.
// The shader's log2 / exp2 / rcp / normalize are hardware approximations there; here they are the
// deterministic functions below (plain binary32 operations, so that checker and kernel agree bit for bit),
// correct to a few units in the last place.  f32tof16 rounds to nearest even.  Texels are clamped to
// [0, 65504] first (a NaN becomes 0): the shader feeds other values into conversions that are undefined.
extern "C++" {
namespace bc6 {
namespace {

float bits_to_float(uint32_t b) { float f; std::memcpy(&f, &b, 4); return f; }
uint32_t float_to_bits(float f) { uint32_t b; std::memcpy(&b, &f, 4); return b; }

// log2 for x >= 0 (0 -> -inf), NaN for negative or NaN input.
float det_log2(float x)
{
    if (!(x >= 0.f)) return bits_to_float(0x7fc00000u);
    if (x == 0.f) return bits_to_float(0xff800000u);
    uint32_t b = float_to_bits(x);
    if (b >= 0x7f800000u) return x;                                      // +inf
    int e = 0;
    if (b < 0x00800000u) { x *= 8388608.f; b = float_to_bits(x); e = -23; }      // subnormal
    e += int(b >> 23) - 127;
    float m = bits_to_float((b & 0x007fffffu) | 0x3f800000u);            // [1, 2)
    if (m > 1.41421354f) { m *= 0.5f; e += 1; }
    float const t = (m - 1.f) / (m + 1.f), t2 = t * t;
    float p = t2 * (1.f / 9.f) + (1.f / 7.f);
    p = p * t2 + 0.2f;
    p = p * t2 + (1.f / 3.f);
    p = p * t2 + 1.f;
    return float(e) + p * t * 2.88539004f;                               // 2 / ln 2
}

// 2^x; overflows to +inf from 128, underflows to 0 below -150.
float det_exp2(float x)
{
    if (x != x) return x;
    if (x >= 128.f) return bits_to_float(0x7f800000u);
    if (x < -150.f) return 0.f;
    float const n = std::nearbyint(x), g = (x - n) * 0.693147182f;
    float p = g * (1.f / 5040.f) + (1.f / 720.f);
    p = p * g + (1.f / 120.f);
    p = p * g + (1.f / 24.f);
    p = p * g + (1.f / 6.f);
    p = p * g + 0.5f;
    p = p * g + 1.f;
    p = p * g + 1.f;
    int k = int(n);
    if (k > 127) { p *= 2.f; k -= 1; }
    if (k < -126) { p *= 5.96046448e-08f; k += 24; }                     // 2^-24
    return p * bits_to_float(uint32_t(k + 127) << 23);
}

struct V3 { float x, y, z; };
V3 operator+(V3 a, V3 b) { return { a.x + b.x, a.y + b.y, a.z + b.z }; }
V3 operator-(V3 a, V3 b) { return { a.x - b.x, a.y - b.y, a.z - b.z }; }
V3 operator*(V3 a, float s) { return { a.x * s, a.y * s, a.z * s }; }
V3 operator*(V3 a, V3 b) { return { a.x * b.x, a.y * b.y, a.z * b.z }; }
float dot(V3 a, V3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
V3 vmin(V3 a, V3 b) { return { std::fmin(a.x, b.x), std::fmin(a.y, b.y), std::fmin(a.z, b.z) }; }
V3 vmax(V3 a, V3 b) { return { std::fmax(a.x, b.x), std::fmax(a.y, b.y), std::fmax(a.z, b.z) }; }
template <class F> V3 map(V3 a, F f) { return { f(a.x), f(a.y), f(a.z) }; }
float clampf(float v, float lo, float hi) { return std::fmin(std::fmax(v, lo), hi); }
float to_half_bits(float v) { return v != v ? 32256.f : float(float_to_half_rne(v)); }     // f32tof16 as a number; any NaN -> 0x7e00
float from_half_bits(float v) { return half_to_float(uint16_t(uint32_t(v))); }

constexpr float kHalfMax = 65504.f;

float msle(V3 a, V3 b)                                                   // hlsl:62-73
{
    V3 const d = map(V3{ (b.x + 1.f) / (a.x + 1.f), (b.y + 1.f) / (a.y + 1.f), (b.z + 1.f) / (a.z + 1.f) }, det_log2);
    V3 const sq = d * d * V3{ 0.299f, 0.587f, 0.114f };
    return sq.x + sq.y + sq.z;
}

// Partitions: the format's first 32 two-subset partitions (the same table as BC7) and their anchors.
uint32_t subset_of(int pattern, int t) { return (bc7::masks().two[pattern][1] >> t) & 1u; }
int fixup_of(int pattern) { return bc7::kAnchorSecondOfTwo[pattern]; }

V3 quantize(V3 v, float levels) { return map(v, [&](float c) { return (to_half_bits(c) * levels) / 31744.f; }); }      // hlsl:111-124 (0x7bff + 1)
V3 unquantize(V3 v, float levels) { return map(v, [&](float c) { return (c * 65536.f + 32768.f) / levels; }); }        // hlsl:126-139
V3 interpolate(V3 e0, V3 e1, float weight)                              // hlsl:141-145
{
    return map((e0 * (64.f - weight) + e1 * weight + V3{ 32.f, 32.f, 32.f }) * (31.f / 4096.f), from_half_bits);
}
uint32_t index_of(float pos, float e0, float e1, float scale, float bias, float top)           // hlsl:161-171
{
    float const r = (pos - e0) / (e1 - e0);
    return uint32_t(clampf(r * scale + bias + 0.5f, 0.f, top));
}
uint32_t index3(float pos, float e0, float e1) { return index_of(pos, e0, e1, 6.98182f, 0.00909f, 7.f); }
uint32_t index4(float pos, float e0, float e1) { return index_of(pos, e0, e1, 14.93333f, 0.03333f, 15.f); }
V3 direction(V3 lo, V3 hi) { V3 const d = hi - lo; float const s = d.x + d.y + d.z; return { d.x / s, d.y / s, d.z / s }; }

void inset_box(const V3 px[16], V3& lo, V3& hi)                         // hlsl:183-207
{
    V3 innerLo = hi, innerHi = lo;
    for (int t = 0; t < 16; ++t) {
        V3 const p = px[t];
        innerLo = vmin(innerLo, V3{ p.x == lo.x ? innerLo.x : p.x, p.y == lo.y ? innerLo.y : p.y, p.z == lo.z ? innerLo.z : p.z });
        innerHi = vmax(innerHi, V3{ p.x == hi.x ? innerHi.x : p.x, p.y == hi.y ? innerHi.y : p.y, p.z == hi.z ? innerHi.z : p.z });
    }
    auto lg = [](float c) { return det_log2(c + 1.f); };
    V3 const logInnerHi = map(innerHi, lg), logInnerLo = map(innerLo, lg);
    V3 logHi = map(hi, lg), logLo = map(lo, lg);
    V3 const ext = (logHi - logLo) * (1.f / 32.f);
    logLo = logLo + vmin(logInnerLo - logLo, ext);
    logHi = logHi - vmin(logHi - logInnerHi, ext);
    lo = map(logLo, [](float c) { return det_exp2(c) - 1.f; });
    hi = map(logHi, [](float c) { return det_exp2(c) - 1.f; });
}

// Least-squares endpoints (in half-bit space) for the indices the current endpoints give; `member` selects
// the subset.  Returns false when the system is singular.  hlsl:239-326
template <class Member> bool refit(const V3 px[16], Member member, bool fourBit, V3 lo, V3 hi, V3& outLo, V3& outHi)
{
    V3 const dir = direction(lo, hi);
    float const e0 = to_half_bits(dot(lo, dir)), e1 = to_half_bits(dot(hi, dir));
    V3 alphaSum{ 0, 0, 0 }, betaSum{ 0, 0, 0 };
    float ab = 0, aa = 0, bb = 0;
    for (int t = 0; t < 16; ++t) if (member(t)) {
        float const pos = to_half_bits(dot(px[t], dir));
        uint32_t const index = fourBit ? index4(pos, e0, e1) : index3(pos, e0, e1);
        float const beta = clampf(float(index) / (fourBit ? 15.f : 7.f), 0.f, 1.f), alpha = 1.f - beta;
        V3 const h = map(px[t], to_half_bits);
        alphaSum = alphaSum + h * alpha; betaSum = betaSum + h * beta;
        ab += alpha * beta; aa += alpha * alpha; bb += beta * beta;
    }
    float const det = aa * bb - ab * ab;
    if (!(std::fabs(det) > 0.00001f)) return false;
    float const rcp = 1.f / det;
    // (the shader clamps these codes to 65504, which lets the codes of infinities and NaNs through; here to 0x7bff)
    auto finish = [&](V3 v) { return map(v * rcp, [](float c) { return from_half_bits(clampf(c, 0.f, 31743.f)); }); };
    outLo = finish(alphaSum * bb - betaSum * ab);
    outHi = finish(betaSum * aa - alphaSum * ab);
    return true;
}

struct Block { uint32_t w[4] = { 0, 0, 0, 0 }; float error = 0.f; };

void encode_one_subset(const V3 px[16], Block& out)                     // hlsl:328-419
{
    V3 lo = px[0], hi = px[0];
    for (int t = 1; t < 16; ++t) { lo = vmin(lo, px[t]); hi = vmax(hi, px[t]); }
    V3 const boxLo = lo, boxHi = hi;
    inset_box(px, lo, hi);
    V3 fitLo, fitHi;
    if (refit(px, [](int) { return true; }, true, lo, hi, fitLo, fitHi)) {
        lo = vmin(vmax(fitLo, boxLo), boxHi);
        hi = vmin(vmax(fitHi, boxLo), boxHi);
    }
    V3 const dir = direction(lo, hi);
    V3 q0 = quantize(lo, 1024.f), q1 = quantize(hi, 1024.f);
    float e0 = to_half_bits(dot(lo, dir)), e1 = to_half_bits(dot(hi, dir));
    if (index4(to_half_bits(dot(px[0], dir)), e0, e1) > 7) { std::swap(e0, e1); std::swap(q0, q1); }
    uint32_t index[16];
    for (int t = 0; t < 16; ++t) index[t] = index4(to_half_bits(dot(px[t], dir)), e0, e1);
    V3 const u0 = unquantize(q0, 1024.f), u1 = unquantize(q1, 1024.f);
    float error = 0.f;
    for (int t = 0; t < 16; ++t) error += msle(px[t], interpolate(u0, u1, std::floor((float(index[t]) * 64.f) / 15.f + 0.5f)));
    out = Block();
    out.error = error;
    uint32_t const e[6] = { uint32_t(q0.x), uint32_t(q0.y), uint32_t(q0.z), uint32_t(q1.x), uint32_t(q1.y), uint32_t(q1.z) };
    // mode 11: six 10-bit endpoint components from bit 5, then 4-bit indices (the first with 3 bits) from bit 65
    unsigned __int128 bits = 0x03;
    for (int i = 0; i < 6; ++i) bits |= (unsigned __int128)(e[i] & 0x3ffu) << (5 + 10 * i);
    int at = 65;
    for (int t = 0; t < 16; ++t) { int const n = t == 0 ? 3 : 4; bits |= (unsigned __int128)(index[t] & ((1u << n) - 1u)) << at; at += n; }
    out.w[0] = uint32_t(bits); out.w[1] = uint32_t(bits >> 32); out.w[2] = uint32_t(bits >> 64); out.w[3] = uint32_t(bits >> 96);
}

float distance_to_line2(V3 origin, V3 dir, V3 p)                        // hlsl:421-426
{
    V3 const w = p - origin, x = w - dir * dot(w, dir);
    return dot(x, x);
}
V3 normalized(V3 v) { float const len = std::sqrt(dot(v, v)); return { v.x / len, v.y / len, v.z / len }; }

void subset_boxes(const V3 px[16], int pattern, V3 lo[2], V3 hi[2])
{
    for (int s = 0; s < 2; ++s) { lo[s] = V3{ kHalfMax, kHalfMax, kHalfMax }; hi[s] = V3{ 0, 0, 0 }; }
    for (int t = 0; t < 16; ++t) { uint32_t const s = subset_of(pattern, t); lo[s] = vmin(lo[s], px[t]); hi[s] = vmax(hi[s], px[t]); }
}

float pattern_score(const V3 px[16], int pattern)                       // hlsl:428-470
{
    V3 lo[2], hi[2];
    subset_boxes(px, pattern, lo, hi);
    V3 const dir[2] = { normalized(hi[0] - lo[0]), normalized(hi[1] - lo[1]) };
    float total = 0.f;
    for (int t = 0; t < 16; ++t) { uint32_t const s = subset_of(pattern, t); total += distance_to_line2(lo[s], dir[s], px[t]); }
    return total;
}

int as_int(float v) { return int(v); }
// Two's complement field of `bits` bits of a small signed integer held in a float (hlsl:173-181).
uint32_t field(float v, int bits) { return uint32_t(as_int(v)) & ((1u << bits) - 1u); }

void encode_two_subsets(const V3 px[16], int pattern, Block& best)      // hlsl:472-733
{
    V3 lo[2], hi[2];
    subset_boxes(px, pattern, lo, hi);
    for (uint32_t s = 0; s < 2; ++s) {
        V3 fitLo, fitHi;
        if (refit(px, [&](int t) { return subset_of(pattern, t) == s; }, false, lo[s], hi[s], fitLo, fitHi)) { lo[s] = fitLo; hi[s] = fitHi; }
    }
    V3 const dir[2] = { direction(lo[0], hi[0]), direction(lo[1], hi[1]) };
    float e0[2], e1[2];
    for (int s = 0; s < 2; ++s) { e0[s] = to_half_bits(dot(lo[s], dir[s])); e1[s] = to_half_bits(dot(hi[s], dir[s])); }
    int const anchor[2] = { 0, fixup_of(pattern) };
    for (int s = 0; s < 2; ++s)
        if (index3(to_half_bits(dot(px[anchor[s]], dir[s])), e0[s], e1[s]) > 3) { std::swap(e0[s], e1[s]); std::swap(lo[s], hi[s]); }
    uint32_t index[16];
    for (int t = 0; t < 16; ++t) {
        uint32_t const s = subset_of(pattern, t);
        index[t] = index3(to_half_bits(dot(px[t], dir[s])), e0[s], e1[s]);
    }
    // endpoints: base + three signed deltas, as 7 + 6 bits and as 9 + 5 bits
    V3 const ends[4] = { lo[0], hi[0], lo[1], hi[1] };
    V3 q7[4], q9[4], u7[4], u9[4];
    auto fl = [](float c) { return std::floor(c); };
    for (int i = 0; i < 4; ++i) { q7[i] = map(quantize(ends[i], 128.f), fl); q9[i] = map(quantize(ends[i], 512.f), fl); }
    for (int i = 1; i < 4; ++i) {
        q7[i] = map(q7[i] - q7[0], [](float c) { return clampf(c, -31.f, 31.f); });
        q9[i] = map(q9[i] - q9[0], [](float c) { return clampf(c, -15.f, 15.f); });
    }
    u7[0] = unquantize(q7[0], 128.f); u9[0] = unquantize(q9[0], 512.f);
    for (int i = 1; i < 4; ++i) { u7[i] = unquantize(q7[0] + q7[i], 128.f); u9[i] = unquantize(q9[0] + q9[i], 512.f); }
    float error7 = 0.f, error9 = 0.f;
    for (int t = 0; t < 16; ++t) {
        uint32_t const s = subset_of(pattern, t);
        float const weight = std::floor((float(index[t]) * 64.f) / 7.f + 0.5f);
        error7 += msle(px[t], interpolate(u7[2 * s], u7[2 * s + 1], weight));
        error9 += msle(px[t], interpolate(u9[2 * s], u9[2 * s + 1], weight));
    }
    float const error = std::fmin(error7, error9);
    if (!(error < best.error)) return;
    bool const sevenSix = error == error7;
    V3 const* q = sevenSix ? q7 : q9;
    int const baseBits = sevenSix ? 7 : 9, deltaBits = sevenSix ? 6 : 5;
    // w = base, x / y / z = deltas of the first subset's second end and of the second subset's ends
    uint32_t const rw = field(q[0].x, baseBits), gw = field(q[0].y, baseBits), bw = field(q[0].z, baseBits);
    uint32_t const rx = field(q[1].x, deltaBits), gx = field(q[1].y, deltaBits), bx = field(q[1].z, deltaBits);
    uint32_t const ry = field(q[2].x, deltaBits), gy = field(q[2].y, deltaBits), by = field(q[2].z, deltaBits);
    uint32_t const rz = field(q[3].x, deltaBits), gz = field(q[3].y, deltaBits), bz = field(q[3].z, deltaBits);
    unsigned __int128 bits = 0;
    auto put = [&](int at, uint32_t value, int n) { bits |= (unsigned __int128)(value & ((1u << n) - 1u)) << at; };
    auto bit = [](uint32_t v, int i) { return (v >> i) & 1u; };
    if (sevenSix) {         // mode 2 of the format: 7.666
        put(0, 0x01, 5);
        put(2, bit(gy, 5), 1); put(3, bit(gz, 4), 1); put(4, bit(gz, 5), 1);
        put(5, rw, 7); put(12, bit(bz, 0), 1); put(13, bit(bz, 1), 1); put(14, bit(by, 4), 1);
        put(15, gw, 7); put(22, bit(by, 5), 1); put(23, bit(bz, 2), 1); put(24, bit(gy, 4), 1);
        put(25, bw, 7); put(32, bit(bz, 3), 1); put(33, bit(bz, 5), 1); put(34, bit(bz, 4), 1);
        put(35, rx, 6); put(41, gy, 4); put(45, gx, 6); put(51, gz, 4); put(55, bx, 6); put(61, by, 4);
        put(65, ry, 6); put(71, rz, 6);
    } else {                // mode 6 of the format: 9.555
        put(0, 0x0E, 5);
        put(5, rw, 9); put(14, bit(by, 4), 1); put(15, gw, 9); put(24, bit(gy, 4), 1); put(25, bw, 9); put(34, bit(bz, 4), 1);
        put(35, rx, 5); put(40, bit(gz, 4), 1); put(41, gy, 4); put(45, gx, 5); put(50, bit(bz, 0), 1); put(51, gz, 4);
        put(55, bx, 5); put(60, bit(bz, 1), 1); put(61, by, 4); put(65, ry, 5); put(70, bit(bz, 2), 1); put(71, rz, 5); put(76, bit(bz, 3), 1);
    }
    put(77, uint32_t(pattern), 5);
    int at = 82;
    for (int t = 0; t < 16; ++t) { int const n = (t == 0 || t == anchor[1]) ? 2 : 3; put(at, index[t], n); at += n; }
    best.error = error;
    best.w[0] = uint32_t(bits); best.w[1] = uint32_t(bits >> 32); best.w[2] = uint32_t(bits >> 64); best.w[3] = uint32_t(bits >> 96);
}

void encode(const float rgb[16][3], uint64_t out[2])                    // hlsl:735-778
{
    V3 px[16];
    for (int t = 0; t < 16; ++t) px[t] = V3{ clampf(rgb[t][0], 0.f, kHalfMax), clampf(rgb[t][1], 0.f, kHalfMax), clampf(rgb[t][2], 0.f, kHalfMax) };
    Block best;
    encode_one_subset(px, best);
    float bestScore = pattern_score(px, 0);
    int bestPattern = 0;
    for (int p = 1; p < 32; ++p) {
        float const score = pattern_score(px, p);
        if (score < bestScore) { bestPattern = p; bestScore = score; }
    }
    encode_two_subsets(px, bestPattern, best);
    out[0] = uint64_t(best.w[0]) | (uint64_t(best.w[1]) << 32);
    out[1] = uint64_t(best.w[2]) | (uint64_t(best.w[3]) << 32);
}

} // namespace
} // namespace bc6
} // extern "C++"

// For tests: the deterministic log2 / exp2 of the BC6H encoder.
float ntc_oracle_bc6_log2(float x) { return bc6::det_log2(x); }
float ntc_oracle_bc6_exp2(float x) { return bc6::det_exp2(x); }

// For tests: the single-colour tables (256 entries each, first endpoint | second << 8).
void ntc_oracle_bc1_match_tables(uint16_t* five, uint16_t* six)
{
    std::memcpy(five, bc1::match_tables().five, 512);
    std::memcpy(six, bc1::match_tables().six, 512);
}

// For tests: the subset masks the BC7 encoder derives from the specification's tables (two-subset:
// 64 x 2, three-subset: 64 x 3) and the three anchor tables.
void ntc_oracle_bc7_tables(uint32_t* two, uint32_t* three, uint8_t* anchors)
{
    for (int p = 0; p < 64; ++p) {
        for (int s = 0; s < 2; ++s) two[2 * p + s] = bc7::masks().two[p][s];
        for (int s = 0; s < 3; ++s) three[3 * p + s] = bc7::masks().three[p][s];
        anchors[p] = bc7::kAnchorSecondOfTwo[p]; anchors[64 + p] = bc7::kAnchorSecondOfThree[p]; anchors[128 + p] = bc7::kAnchorThirdOfThree[p];
    }
}

// dstFormat 1..7 (BC1, BC2, BC3, BC4: channel R, BC5: R then G, BC6H unsigned, BC7); host pointers in `p`.
// Returns -1 for other values.
int ntc_oracle_block_compress(const NtcHipBlockCompress* p)
{
    if (p->dstFormat < 1 || p->dstFormat > 7) return -1;
    auto fetch = [&](int x, int y, int c) -> float {
        if (x < 0 || y < 0 || x >= p->src.width || y >= p->src.height) return 0.f;
        // "+ 0.f": a stored -0 becomes +0 (minima and maxima of +0 and -0 depend on the operand order otherwise)
        return diff_channel(p->src, static_cast<uint8_t const*>(p->src.data) + size_t(y) * p->src.rowPitch + size_t(x) * p->src.pixelStride, c) + 0.f;
    };
    size_t const blockBytes = (p->dstFormat == 1 || p->dstFormat == 4) ? 8 : 16;
    for (int by = 0; by < p->heightInBlocks; ++by)
        for (int bx = 0; bx < p->widthInBlocks; ++bx) {
            uint64_t words[2] = { 0, 0 };
            if (p->dstFormat == 4 || p->dstFormat == 5) {
                for (int c = 0; c < p->dstFormat - 3; ++c) {
                    float texels[16];
                    for (int t = 0; t < 16; ++t) texels[t] = fetch(p->srcLeft + bx * 4 + (t & 3), p->srcTop + by * 4 + (t >> 2), c);
                    words[c] = bc4::encode(texels);
                }
            } else if (p->dstFormat == 6) {
                float rgb[16][3];
                for (int t = 0; t < 16; ++t)
                    for (int c = 0; c < 3; ++c) rgb[t][c] = fetch(p->srcLeft + bx * 4 + (t & 3), p->srcTop + by * 4 + (t >> 2), c);
                bc6::encode(rgb, words);
            } else if (p->dstFormat == 7) {
                bc7::Color<4> px[16];
                for (int t = 0; t < 16; ++t)
                    for (int c = 0; c < 4; ++c) px[t].c[c] = fetch(p->srcLeft + bx * 4 + (t & 3), p->srcTop + by * 4 + (t >> 2), c);
                int mode = -1, partition = -1;
                bool valid = true;
                if (p->modeBuffer) {
                    // CompressBC7.hlsl:1409-1443: 9 bits per block of the mode map, 0 = no entry, 0x1BF = mode 0 partition 0
                    int64_t const mx = int64_t(bx) + p->modeMapOffsetX, my = int64_t(by) + p->modeMapOffsetY;
                    valid = mx >= 0 && my >= 0 && mx < p->modeMapWidthInBlocks && my < p->modeMapHeightInBlocks;
                    if (valid) {
                        uint64_t const bit = (uint64_t(my) * uint64_t(p->modeMapWidthInBlocks) + uint64_t(mx)) * 9u;
                        uint8_t const* bytes = static_cast<uint8_t const*>(p->modeBuffer) + p->modeBufferByteOffset;
                        uint32_t entry = 0;
                        for (uint64_t b = 0; b < 9; ++b) entry |= uint32_t((bytes[(bit + b) >> 3] >> ((bit + b) & 7)) & 1u) << b;
                        valid = entry != 0;
                        if (entry == 0x1BF) entry = 0;
                        mode = int((entry >> 6) & 7u); partition = int(entry & 63u);
                    }
                }
                if (valid) bc7::encode(px, mode, partition, words);
                else { words[0] = 0x0001f00000f80004ull; words[1] = 0x1f9e00003ff0001full; }      // hlsl:1541-1548: four coloured squares
            } else {
                float px[16][4], alpha[16];
                for (int t = 0; t < 16; ++t) {
                    for (int c = 0; c < 4; ++c) px[t][c] = fetch(p->srcLeft + bx * 4 + (t & 3), p->srcTop + by * 4 + (t >> 2), c);
                    if (p->dstFormat != 1) { alpha[t] = px[t][3]; px[t][3] = 1.f; }
                }
                uint64_t const color = bc1::encode_color(px, p->dstFormat == 1, p->alphaThreshold);
                if (p->dstFormat == 1) words[0] = color;
                else { words[0] = p->dstFormat == 2 ? bc1::bc2_alpha(alpha) : bc4::encode(alpha); words[1] = color; }
            }
            std::memcpy(static_cast<uint8_t*>(p->dst) + size_t(by + p->dstOffsetY) * p->dstRowPitch + size_t(bx + p->dstOffsetX) * blockBytes, words, blockBytes);
        }
    return 0;
}

// Random-access decode of a list of (u, v, mip) sample points: NtcSampleTextureSet
// (Inference.hlsli:282-357) evaluated at texel (floor(u*W), floor(v*H)) clamped to the mip,
// 16 outputs per query as fp16 (Inf/NaN -> 0 as in the raster path).  Mips outside the set give zeros.
int ntc_oracle_decode_queries(const NtcHipTextureSet* set, const float* uvmip /* 3 words per query: u, v, int32 mip */,
                              uint64_t numQueries, uint16_t* out, int threads)
{
    SetView sv{ set, {}, {}, {} };
    if (!decodable(set->spec) || !weight_layout(set->spec, sv.layout)) return -1;
    sv.prepare();
    if (threads < 1) threads = 1;
    std::atomic<uint64_t> next{0};
    auto work = [&]() {
        float o[NTC_HIP_MAX_LAYER_WIDTH];
        for (;;) {
            uint64_t const q0 = next.fetch_add(1024);
            if (q0 >= numQueries) break;
            for (uint64_t q = q0; q < std::min(numQueries, q0 + 1024); ++q) {
                float const u = uvmip[3 * q], v = uvmip[3 * q + 1];
                int32_t mipIndex; std::memcpy(&mipIndex, &uvmip[3 * q + 2], 4);
                if (mipIndex < 0 || mipIndex >= set->numMips) { std::memset(out + 16 * q, 0, 32); continue; }
                NtcHipMipDesc const& mip = set->mips[mipIndex];
                int x = int(std::floor(u * float(mip.width))), y = int(std::floor(v * float(mip.height)));
                x = std::max(0, std::min(x, mip.width - 1));
                y = std::max(0, std::min(y, mip.height - 1));
                decode_texel(sv, mip, x, y, o, nullptr);
                for (int c = 0; c < 16; ++c) out[16 * q + uint64_t(c)] = output_to_half(o[c]);
            }
        }
    };
    std::vector<std::thread> pool;
    for (int i = 0; i < threads; ++i) pool.emplace_back(work);
    for (auto& t : pool) t.join();
    return 0;
}

// Decodes every mip of one set into set->output (host memory).  Rows of each mip are handed
// out in bands to `threads` workers.  Returns seconds spent decoding (steady clock), < 0 on error.
double ntc_oracle_decode(const NtcHipTextureSet* set, int threads)
{
    SetView sv{ set, {}, {}, {} };
    if (!decodable(set->spec) || !weight_layout(set->spec, sv.layout)) return -1.0;
    sv.prepare();
    if (threads < 1) threads = 1;
    auto const t0 = std::chrono::steady_clock::now();
    for (int m = 0; m < set->numMips; ++m) {
        NtcHipMipDesc const& mip = set->mips[m];
        std::atomic<int> nextRow{0};
        int const band = 4;
        auto work = [&]() {
            float o[NTC_HIP_MAX_LAYER_WIDTH];
            for (;;) {
                int const y0 = nextRow.fetch_add(band);
                if (y0 >= mip.height) break;
                int const y1 = std::min(mip.height, y0 + band);
                for (int y = y0; y < y1; ++y)
                    for (int x = 0; x < mip.width; ++x) {
                        decode_texel(sv, mip, x, y, o, nullptr);
                        store_texel(*set, mip, x, y, o);
                    }
            }
        };
        int const n = std::min(threads, std::max(1, (mip.height + band - 1) / band));
        if (n == 1) work();
        else {
            std::vector<std::thread> pool;
            for (int i = 0; i < n; ++i) pool.emplace_back(work);
            for (auto& t : pool) t.join();
        }
    }
    return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

// Decodes only rows [y0, y1) of mip `mipIndex` (bounded CPU-baseline samples).
double ntc_oracle_decode_rows(const NtcHipTextureSet* set, int mipIndex, int y0, int y1, int threads)
{
    SetView sv{ set, {}, {}, {} };
    if (!decodable(set->spec) || !weight_layout(set->spec, sv.layout)) return -1.0;
    sv.prepare();
    NtcHipMipDesc const& mip = set->mips[mipIndex];
    y0 = std::max(0, y0); y1 = std::min(mip.height, y1);
    if (threads < 1) threads = 1;
    auto const t0 = std::chrono::steady_clock::now();
    std::atomic<int> nextRow{y0};
    auto work = [&]() {
        float o[NTC_HIP_MAX_LAYER_WIDTH];
        for (;;) {
            int const y = nextRow.fetch_add(1);
            if (y >= y1) break;
            for (int x = 0; x < mip.width; ++x) {
                decode_texel(sv, mip, x, y, o, nullptr);
                store_texel(*set, mip, x, y, o);
            }
        }
    };
    std::vector<std::thread> pool;
    for (int i = 0; i < threads; ++i) pool.emplace_back(work);
    for (auto& t : pool) t.join();
    return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

} // extern "C"
