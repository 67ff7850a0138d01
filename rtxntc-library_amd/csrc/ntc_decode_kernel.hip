// ntc_decode_kernel.hip - texture-set decode for gfx950 (MI355X), int8 network.
//
// One persistent launch decodes every colour mip of every texture set handed to it.
// Work unit: a workgroup tile of 64x4 texels = four wave64 tiles of 16x4 texels.
//
// Per wave tile:
//   1. input stage, one texel per lane: latent fetch (2x2 concat or bilinear, wrap
//      addressing), unpack of the 2/4-bit fields in registers, positional encoding -> the
//      texel's int8 input vector (what FeatureGrid::Sample x2 + EncodeSamplePosition do in
//      reference src/Inference.cu:52-59, in the integer form of
//      include/libntc/shaders/Inference.hlsli:62-120);
//   2. a transpose through LDS into the B-operand layout of v_mfma_i32_16x16x64_i8
//      (lane = (texel column j = lane%16, k-group g = lane/16), 16 bytes of K per lane);
//   3. four layers of D = W * X as int8 MFMA tiles: A = 16 output channels x 64 K from
//      the weight copy in LDS, B = 64 K x 16 texels, C = int32 bias.  D comes back with
//      lane (j, g) holding channels 16t+4g..+3 of texel j, so the requantised bytes of the
//      four M-tiles t ARE the lane's 16 bytes of K for the next layer: k-slot (g, 4t+r)
//      means channel 16t+4g+r, and the weight copy in LDS is permuted to match.  No
//      cross-lane traffic between layers.
//   4. epilogue per D value in fp32 exactly as NtcEvaluateLayerINT8 + NtcHGELUClamp_*
//      (Inference.hlsli:36-39,123-182) prescribe; output layer -> fp16 / unorm8 stores.
//
// Float code here must be compiled with -ffp-contract=off: fused multiply-adds happen only
// where __builtin_fmaf is written, so results match the CPU checker bit for bit.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ntc_decode_kernel.h"

namespace ntc_hip_dev {

typedef int   v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWaves       = 4;     // waves per workgroup
constexpr int kWaveTexels  = 64;
constexpr int kInStride    = 20;    // dwords per texel row in the transpose buffer (16 + pad)

// ---- small device helpers -----------------------------------------------------------

__device__ __forceinline__ uint32_t spread2(uint32_t byte)     // 4 x 2-bit fields -> 4 bytes
{
    uint32_t x = byte & 0xffu;
    x = (x | (x << 12)) & 0x000f000fu;
    x = (x | (x << 6))  & 0x03030303u;
    return x;
}
__device__ __forceinline__ uint32_t spread4(uint32_t word)     // 4 x 4-bit fields -> 4 bytes
{
    uint32_t x = word & 0xffffu;
    x = (x | (x << 8)) & 0x00ff00ffu;
    x = (x | (x << 4)) & 0x0f0f0f0fu;
    return x;
}

// Wrap addressing of FeatureGrid::SetupBilinearFilter (src/FeatureGridDevice.h:51-57).
struct Taps { int x0, y0, x1, y1; float w00, w10, w01, w11; };

__device__ __forceinline__ Taps footprint(float u, float v, int gw, int gh)
{
    float const x = u * float(gw) - 0.5f;
    float const y = v * float(gh) - 0.5f;
    float const fx = floorf(x), fy = floorf(y);
    float const dx = x - fx, dy = y - fy;
    float const dxn = 1.f - dx, dyn = 1.f - dy;
    Taps t;
    t.w00 = dxn * dyn; t.w10 = dx * dyn; t.w01 = dxn * dy; t.w11 = dx * dy;
    // u, v lie in (0, 1), so floor() lands in [-1, g-1] (g itself only through rounding): the
    // reference's "add g if negative, then mod g" is a conditional add / subtract here.
    int xb = int(fx), yb = int(fy);
    if (xb < 0) xb += gw;
    if (yb < 0) yb += gh;
    if (xb >= gw) xb -= gw;
    if (yb >= gh) yb -= gh;
    t.x0 = xb; t.y0 = yb;
    t.x1 = (xb + 1 >= gw) ? xb + 1 - gw : xb + 1;
    t.y1 = (yb + 1 >= gh) ? yb + 1 - gh : yb + 1;
    return t;
}

// floor(t * codeScale) - 128 for four features at once, returned as four packed bytes.
__device__ __forceinline__ uint32_t bilinear4(Taps const& tp, uint32_t s00, uint32_t s10, uint32_t s01, uint32_t s11,
                                              float codeScale)
{
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float const q00 = float((s00 >> (8 * i)) & 0xffu);
        float const q10 = float((s10 >> (8 * i)) & 0xffu);
        float const q01 = float((s01 >> (8 * i)) & 0xffu);
        float const q11 = float((s11 >> (8 * i)) & 0xffu);
        float t = tp.w00 * q00;
        t = __builtin_fmaf(tp.w10, q10, t);
        t = __builtin_fmaf(tp.w01, q01, t);
        t = __builtin_fmaf(tp.w11, q11, t);
        int const c = int(floorf(t * codeScale));          // 0..255
        packed |= (uint32_t(c) & 0xffu) << (8 * i);
    }
    return packed ^ 0x80808080u;                            // -128 on every byte
}

// HGELU-clamp + requantise of four D values of one lane (Inference.hlsli:36-39,123-131,164-179).
// round-half-even of y*80 is taken from the low mantissa bits of y*80 + 1.5*2^23.
__device__ __forceinline__ uint32_t activate4(v4i acc, v4f scale)
{
    uint32_t packed = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float const x = float(acc[r]) * scale[r];
        float t = __builtin_fmaf(x, 0.333333f, 0.5f);
        t = fminf(fmaxf(t, 0.f), 1.f);
        float const y = fminf(x, 3.f) * t;
        float const z = y * 80.f;
        uint32_t const q = __float_as_uint(z + 12582912.f);  // low byte = rne(z) mod 256
        packed |= ((q + 143u) & 0xffu) << (8 * r);           // -113 mod 256
    }
    return packed;
}

__device__ __forceinline__ uint32_t to_half_bits(float o)
{
    // The network output is an fp32 product that is THEN rounded to half.  Without this
    // barrier the compiler folds multiply + convert into v_fma_mixlo_f16, which rounds the
    // exact product once, straight to half, and differs in rare double-rounding cases.
    asm volatile("" : "+v"(o));
    _Float16 const h = (_Float16)o;                          // v_cvt_f16_f32, round-nearest-even
    uint32_t bits = uint32_t(__builtin_bit_cast(uint16_t, h));
    if ((bits & 0x7c00u) == 0x7c00u) bits = 0;               // IsHalfSpecial -> 0 (Inference.cu:125-126)
    return bits;
}

// WriteImageChannel UNORM8 (src/ImageProcessing.cu:146-149): roundf, clamp.
__device__ __forceinline__ uint32_t half_bits_to_unorm8(uint32_t hbits)
{
    float const v = float(__builtin_bit_cast(_Float16, uint16_t(hbits))) * 255.f;
    float r = truncf(v);
    float const fr = v - r;
    if (fr >= 0.5f) r += 1.f; else if (fr <= -0.5f) r -= 1.f;
    r = fminf(fmaxf(r, 0.f), 255.f);
    return uint32_t(r);
}

// ---- decoder variants -----------------------------------------------------------------

template <int HR_MODE_, int HR_F_, int HR_BITS_, int HR_SLOTS_, int LR_F_, int LR_SLOTS_, int LOD_,
          int IN_, int H0_, int H1_, int H2_>
struct Variant {
    static constexpr int HR_MODE = HR_MODE_, HR_F = HR_F_, HR_BITS = HR_BITS_, HR_SLOTS = HR_SLOTS_;
    static constexpr int LR_F = LR_F_, LR_SLOTS = LR_SLOTS_, LOD = LOD_;
    static constexpr int IN = IN_, H0 = H0_, H1 = H1_, H2 = H2_, OUT = 16;
    static constexpr int HR_INPUTS = (HR_MODE == 1 ? 4 : 1) * HR_SLOTS;
    static constexpr int LR_INPUTS = LR_SLOTS;
    static constexpr int POS_BASE = HR_INPUTS + LR_INPUTS;
    static constexpr int T0 = H0 / 16, T1 = H1 / 16, T2 = H2 / 16, T3 = 1;
    static constexpr int NTILES = T0 + T1 + T2 + T3;
    static constexpr int W1_OFF = IN * H0, W2_OFF = W1_OFF + H0 * H1, W3_OFF = W2_OFF + H1 * H2;
    static constexpr int WEIGHT_BYTES = W3_OFF + H2 * OUT;
    static constexpr int TOTAL_OUT = H0 + H1 + H2 + OUT;
    static constexpr int SCALE_OFF = WEIGHT_BYTES, BIAS_OFF = WEIGHT_BYTES + 4 * TOTAL_OUT;
    static_assert(POS_BASE + 12 + LOD <= IN, "input vector does not fit");
    static_assert(IN % 16 == 0 && IN <= 64 && H0 <= 64 && H1 <= 64 && H2 <= 64, "layer widths");
    static_assert(HR_INPUTS % 4 == 0 && LR_INPUTS % 4 == 0, "grid blocks are dword aligned");
};

struct alignas(16) Lds {
    uint32_t w[10][64][4];            // A operands: [M-tile][lane][4 dwords]; 10 = max tiles (64+48+32+16)/16
    float    scale[10][4][4];         // [M-tile][k-group g][r]  -> channel 16t+4g+r
    int32_t  bias[10][4][4];
    uint32_t in[kWaves][kWaveTexels][kInStride];
};

// Copies the int8 blob (src/WeightLayout.cpp:42-49: matrices, then fp32 scales, then int32
// biases; W[c*IN + k]) into LDS in MFMA operand order.
template <class V>
__device__ void stage_weights(Lds& lds, uint8_t const* __restrict__ blob)
{
    constexpr int ins[4]   = { V::IN, V::H0, V::H1, V::H2 };
    constexpr int tiles[4] = { V::T0, V::T1, V::T2, V::T3 };
    constexpr int woff[4]  = { 0, V::W1_OFF, V::W2_OFF, V::W3_OFF };
    uint32_t const* blob32 = reinterpret_cast<uint32_t const*>(blob);
    int tileBase = 0, chanBase = 0;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        int const in = ins[l];
        for (int e = threadIdx.x; e < tiles[l] * 64 * 4; e += blockDim.x) {
            int const d = e & 3, lane = (e >> 2) & 63, t = e >> 8;
            int const i = lane & 15, g = lane >> 4;
            int const row = 16 * t + i;
            // layer 0: k-slot (g, 4d+r) = input 16g+4d+r.  layers >= 1: = channel 16d+4g+r.
            int const k = (l == 0) ? (16 * g + 4 * d) : (16 * d + 4 * g);
            uint32_t v = 0;
            if (k < in) v = blob32[(woff[l] + row * in + k) >> 2];
            lds.w[tileBase + t][lane][d] = v;
        }
        for (int e = threadIdx.x; e < tiles[l] * 16; e += blockDim.x) {
            int const r = e & 3, g = (e >> 2) & 3, t = e >> 4;
            int const c = chanBase + 16 * t + 4 * g + r;
            lds.scale[tileBase + t][g][r] = reinterpret_cast<float const*>(blob + V::SCALE_OFF)[c];
            lds.bias[tileBase + t][g][r]  = reinterpret_cast<int32_t const*>(blob + V::BIAS_OFF)[c];
        }
        tileBase += tiles[l];
        chanBase += tiles[l] * 16;
    }
}

// Input vector of one texel as 16 dwords (int8 x 64, zero padded).
template <class V>
__device__ __forceinline__ void prepare_inputs(DevMip const& m, int x, int y, uint32_t (&in)[16])
{
#pragma unroll
    for (int i = 0; i < 16; ++i) in[i] = 0;

    float const u = (float(x) + 0.5f) / float(m.width);      // src/Inference.cu:52-53
    float const v = (float(y) + 0.5f) / float(m.height);

    // ---- high-res grid
    {
        Taps const tp = footprint(u, v, m.hrWidth, m.hrHeight);
        uint16_t const* __restrict__ g = m.hr;
        size_t const layerStride = size_t(m.hrWidth) * size_t(m.hrHeight);
        size_t const a00 = size_t(tp.y0) * m.hrWidth + tp.x0, a10 = size_t(tp.y0) * m.hrWidth + tp.x1;
        size_t const a01 = size_t(tp.y1) * m.hrWidth + tp.x0, a11 = size_t(tp.y1) * m.hrWidth + tp.x1;
        constexpr int perWord = 16 / V::HR_BITS;
        constexpr int layers = (V::HR_F + perWord - 1) / perWord;
        if constexpr (V::HR_MODE == 1) {
            // 2x2 concat: taps a00,a01,a10,a11 of FeatureGridDevice.h:67-70 = (x0,y0),(x1,y0),(x0,y1),(x1,y1)
            size_t const addr[4] = { a00, a10, a01, a11 };
#pragma unroll
            for (int tap = 0; tap < 4; ++tap) {
#pragma unroll
                for (int L = 0; L < layers; ++L) {
                    uint32_t const w = g[addr[tap] + L * layerStride];
#pragma unroll
                    for (int q = 0; q < perWord / 4; ++q) {
                        int const f0 = L * perWord + 4 * q;          // first feature of this dword
                        if (f0 < V::HR_F) {
                            uint32_t s, b;
                            if constexpr (V::HR_BITS == 2) { s = spread2(w >> (8 * q));  b = s * 85u; }
                            else                           { s = spread4(w >> (16 * q)); b = s * 17u; }
                            b ^= 0x80808080u;
                            if (f0 + 4 > V::HR_F) b &= (1u << (8 * (V::HR_F - f0))) - 1u;   // masked features stay 0
                            in[(tap * V::HR_SLOTS + f0) / 4] = b;
                        }
                    }
                }
            }
        } else {
            static_assert(V::HR_MODE == 1 || V::HR_BITS == 4, "bilinear grids are 4-bit");
#pragma unroll
            for (int L = 0; L < layers; ++L) {
                uint32_t const s00 = spread4(g[a00 + L * layerStride]);
                uint32_t const s10 = spread4(g[a10 + L * layerStride]);
                uint32_t const s01 = spread4(g[a01 + L * layerStride]);
                uint32_t const s11 = spread4(g[a11 + L * layerStride]);
                uint32_t b = bilinear4(tp, s00, s10, s01, s11, 17.f);
                if (4 * L + 4 > V::HR_F) b &= (1u << (8 * (V::HR_F - 4 * L))) - 1u;
                in[L] = b;
            }
        }
    }
    // ---- low-res grid: bilinear, 4-bit
    {
        Taps const tp = footprint(u, v, m.lrWidth, m.lrHeight);
        uint16_t const* __restrict__ g = m.lr;
        size_t const layerStride = size_t(m.lrWidth) * size_t(m.lrHeight);
        size_t const a00 = size_t(tp.y0) * m.lrWidth + tp.x0, a10 = size_t(tp.y0) * m.lrWidth + tp.x1;
        size_t const a01 = size_t(tp.y1) * m.lrWidth + tp.x0, a11 = size_t(tp.y1) * m.lrWidth + tp.x1;
        constexpr int layers = (V::LR_F + 3) / 4;
#pragma unroll
        for (int L = 0; L < layers; ++L) {
            uint32_t const s00 = spread4(g[a00 + L * layerStride]);
            uint32_t const s10 = spread4(g[a10 + L * layerStride]);
            uint32_t const s01 = spread4(g[a01 + L * layerStride]);
            uint32_t const s11 = spread4(g[a11 + L * layerStride]);
            uint32_t b = bilinear4(tp, s00, s10, s01, s11, 17.f);
            if (4 * L + 4 > V::LR_F) b &= (1u << (8 * (V::LR_F - 4 * L))) - 1u;
            in[V::HR_INPUTS / 4 + L] = b;
        }
    }
    // ---- positional encoding (Inference.hlsli:89-120); int() truncates
    {
        float px = float(x) * m.positionScale, py = float(y) * m.positionScale;
#pragma unroll
        for (int w = 0; w < 3; ++w) {
            float const e0 = (px - floorf(px)) * 2.f - 1.f;
            float const e1 = (py - floorf(py)) * 2.f - 1.f;
            float const qx = px + 0.25f, qy = py + 0.25f;
            float const e2 = (qx - floorf(qx)) * 2.f - 1.f;
            float const e3 = (qy - floorf(qy)) * 2.f - 1.f;
            uint32_t const p = (uint32_t(int(e0 * 127.5f)) & 0xffu)
                             | ((uint32_t(int(e1 * 127.5f)) & 0xffu) << 8)
                             | ((uint32_t(int(e2 * 127.5f)) & 0xffu) << 16)
                             | ((uint32_t(int(e3 * 127.5f)) & 0xffu) << 24);
            in[V::POS_BASE / 4 + w] = p;
            px *= 2.f; py *= 2.f;
        }
        if constexpr (V::LOD == 2) {
            uint32_t const l = uint32_t(int(m.positionLod * 127.5f)) & 0xffu;
            in[V::POS_BASE / 4 + 3] = l | (l << 8);
        }
    }
}

template <class V>
__global__ void __launch_bounds__(256, 2)
decode_kernel(DevMip const* __restrict__ mips, int numMips, int totalTiles)
{
    __shared__ Lds lds;
    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const j = lane & 15, g = lane >> 4;

    // contiguous share of the tile list for this workgroup
    int const per = (totalTiles + gridDim.x - 1) / gridDim.x;
    int const tileBegin = blockIdx.x * per;
    int const tileEnd = min(totalTiles, tileBegin + per);

    uint8_t const* stagedBlob = nullptr;
    int entry = 0;

    for (int tile = tileBegin; tile < tileEnd; ++tile) {
        while (entry + 1 < numMips && mips[entry + 1].tileStart <= tile) ++entry;
        DevMip const& m = mips[entry];

        if (m.weights != stagedBlob) {                       // uniform across the workgroup
            __syncthreads();
            stage_weights<V>(lds, m.weights);
            stagedBlob = m.weights;
            __syncthreads();
        }

        int const local = tile - m.tileStart;
        int const tileY = local / m.tilesX, tileX = local - tileY * m.tilesX;
        int const x0 = tileX * 64 + wave * 16;
        int const y0 = tileY * 4;
        if (x0 >= m.width) continue;                         // whole wave tile outside the image

        // ---- 1. input stage: lane = texel (tx = lane%16, ty = lane/16)
        {
            int const x = min(x0 + j, m.width - 1), y = min(y0 + g, m.height - 1);
            uint32_t in[16];
            prepare_inputs<V>(m, x, y, in);
            uint4* dst = reinterpret_cast<uint4*>(&lds.in[wave][lane][0]);
            dst[0] = make_uint4(in[0], in[1], in[2], in[3]);
            dst[1] = make_uint4(in[4], in[5], in[6], in[7]);
            dst[2] = make_uint4(in[8], in[9], in[10], in[11]);
            dst[3] = make_uint4(in[12], in[13], in[14], in[15]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // ---- 2. B operands of layer 0: block b = tile row b, column j, k-group g
        v4i X[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            uint4 const t = *reinterpret_cast<uint4 const*>(&lds.in[wave][b * 16 + j][4 * g]);
            X[b] = v4i{ int(t.x), int(t.y), int(t.z), int(t.w) };
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();

        // ---- 3. hidden layers
        constexpr int tiles[3] = { V::T0, V::T1, V::T2 };
        int tb = 0;
#pragma unroll
        for (int l = 0; l < 3; ++l) {
            uint32_t Y[4][4];
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int d = 0; d < 4; ++d) Y[b][d] = 0;
#pragma unroll
            for (int t = 0; t < tiles[l]; ++t) {
                uint4 const wa = *reinterpret_cast<uint4 const*>(&lds.w[tb + t][lane][0]);
                v4i const A = v4i{ int(wa.x), int(wa.y), int(wa.z), int(wa.w) };
                v4i const C = *reinterpret_cast<v4i const*>(&lds.bias[tb + t][g][0]);
                v4f const S = *reinterpret_cast<v4f const*>(&lds.scale[tb + t][g][0]);
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    v4i const D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, X[b], C, 0, 0, 0);
                    Y[b][t] = activate4(D, S);
                }
            }
#pragma unroll
            for (int b = 0; b < 4; ++b) X[b] = v4i{ int(Y[b][0]), int(Y[b][1]), int(Y[b][2]), int(Y[b][3]) };
            tb += tiles[l];
        }

        // ---- 4. output layer + stores: lane (j, g) holds channels 4g..4g+3 of texel (x0+j, y0+b)
        {
            uint4 const wa = *reinterpret_cast<uint4 const*>(&lds.w[tb][lane][0]);
            v4i const A = v4i{ int(wa.x), int(wa.y), int(wa.z), int(wa.w) };
            v4i const C = *reinterpret_cast<v4i const*>(&lds.bias[tb][g][0]);
            v4f const S = *reinterpret_cast<v4f const*>(&lds.scale[tb][g][0]);
            int const x = x0 + j;
            int const chBase = 4 * g;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                v4i const D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, X[b], C, 0, 0, 0);
                int const y = y0 + b;
                if (x >= m.width || y >= m.height || chBase >= m.numChannels) continue;
                uint32_t h[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) h[r] = to_half_bits(float(D[r]) * S[r]);
                int const nch = min(4, m.numChannels - chBase);
                if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS) {
                    // src/RegressionKernels.h:36-45; whole half2 pairs (Inference.cu:131-134)
                    size_t const C2 = size_t((m.numChannels + 1) & ~1);
                    uint16_t* img = reinterpret_cast<uint16_t*>(m.out);
                    size_t const a = size_t(y) * size_t(m.width) * C2 + size_t(chBase) * size_t(m.width) + size_t(x) * 2;
                    *reinterpret_cast<uint32_t*>(img + a) = h[0] | (h[1] << 16);
                    if (nch > 2)
                        *reinterpret_cast<uint32_t*>(img + a + 2 * size_t(m.width)) = h[2] | (h[3] << 16);
                } else if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PIXELS) {
                    uint8_t* px = m.out + size_t(y) * m.outRowPitch + size_t(x) * size_t(m.outPixelStride) + 2 * chBase;
                    if (nch == 4 && ((reinterpret_cast<uintptr_t>(px) & 7u) == 0)) {
                        *reinterpret_cast<uint2*>(px) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
                    } else {
                        for (int r = 0; r < nch; ++r) reinterpret_cast<uint16_t*>(px)[r] = uint16_t(h[r]);
                    }
                } else {
                    uint8_t* px = m.out + size_t(y) * m.outRowPitch + size_t(x) * size_t(m.outPixelStride) + chBase;
                    uint32_t u8[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) u8[r] = half_bits_to_unorm8(h[r]);
                    if (nch == 4 && ((reinterpret_cast<uintptr_t>(px) & 3u) == 0)) {
                        *reinterpret_cast<uint32_t*>(px) = u8[0] | (u8[1] << 8) | (u8[2] << 16) | (u8[3] << 24);
                    } else {
                        for (int r = 0; r < nch; ++r) px[r] = uint8_t(u8[r]);
                    }
                }
            }
        }
    }
}

// 16x64 by 64x16 int8 product with the operand layout the decode kernel assumes.
__global__ void selftest_mfma_kernel(int8_t const* __restrict__ a, int8_t const* __restrict__ b, int32_t* __restrict__ d)
{
    int const lane = threadIdx.x & 63;
    int const ij = lane & 15, g = lane >> 4;
    v4i A, B;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        uint32_t pa = 0, pb = 0;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            int const k = 16 * g + 4 * w + r;
            pa |= (uint32_t(uint8_t(a[ij * 64 + k]))) << (8 * r);      // A[i][k], row-major 16x64
            pb |= (uint32_t(uint8_t(b[k * 16 + ij]))) << (8 * r);      // B[k][j], row-major 64x16
        }
        A[w] = int(pa); B[w] = int(pb);
    }
    v4i const D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, B, v4i{0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) d[(4 * g + r) * 16 + ij] = D[r];      // D[i = 4g+r][j]
}

// ---- host-callable launchers ------------------------------------------------------------

using VCfg01  = Variant<1, 8, 2, 8, 16, 16, 0, 64, 64, 48, 32>;   // 2x2 concat 8x2-bit + bilinear 16x4-bit
using VCfg2   = Variant<1, 8, 2, 8, 12, 12, 0, 64, 48, 48, 32>;   // faster decoder, 12 low-res features
using VRef16  = Variant<0, 16, 4, 16, 16, 16, 2, 48, 64, 48, 32>; // LibNTC 0.9.2 geometry, 16 features
using VRef12  = Variant<0, 12, 4, 16, 12, 16, 2, 48, 64, 48, 32>;
using VRef8   = Variant<0, 8, 4, 16, 8, 16, 2, 48, 64, 48, 32>;
using VRef4   = Variant<0, 4, 4, 16, 4, 16, 2, 48, 64, 48, 32>;

template <class V>
static hipError_t launch_variant(DevMip const* mips, int numMips, int totalTiles, int gridSize, hipStream_t stream)
{
    hipLaunchKernelGGL(decode_kernel<V>, dim3(gridSize), dim3(256), 0, stream, mips, numMips, totalTiles);
    return hipGetLastError();
}

hipError_t launch_decode(int variant, DevMip const* mips, int numMips, int totalTiles, int gridSize, hipStream_t stream)
{
    switch (variant) {
    case NTC_HIP_VARIANT_CFG01: return launch_variant<VCfg01>(mips, numMips, totalTiles, gridSize, stream);
    case NTC_HIP_VARIANT_CFG2:  return launch_variant<VCfg2>(mips, numMips, totalTiles, gridSize, stream);
    case NTC_HIP_VARIANT_REF16: return launch_variant<VRef16>(mips, numMips, totalTiles, gridSize, stream);
    case NTC_HIP_VARIANT_REF12: return launch_variant<VRef12>(mips, numMips, totalTiles, gridSize, stream);
    case NTC_HIP_VARIANT_REF8:  return launch_variant<VRef8>(mips, numMips, totalTiles, gridSize, stream);
    case NTC_HIP_VARIANT_REF4:  return launch_variant<VRef4>(mips, numMips, totalTiles, gridSize, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_selftest_mfma(int8_t const* a, int8_t const* b, int32_t* d, hipStream_t stream)
{
    hipLaunchKernelGGL(selftest_mfma_kernel, dim3(1), dim3(64), 0, stream, a, b, d);
    return hipGetLastError();
}

} // namespace ntc_hip_dev
