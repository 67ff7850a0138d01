// ntc_bc_kernel.hip - BC4 / BC5 block compression of a decoded image (gfx950).
//
// The step after decode in a load path that hands block-compressed textures to a renderer:
// the reference runs it as a graphics compute pass (IContext::MakeBlockCompressionComputePass,
// src/shaders/CompressBC4.hlsl, CompressBC5.hlsl, BC4_* of src/shaders/BlockCompressCommon.hlsli:510-796).
// One lane encodes one 4 x 4 block of one channel, as one thread does there.
//
// The encoder tries both BC4 palettes.  Eight-value palette (endpoint 0 > endpoint 1): start from the
// block's extremes pulled inwards by 1/34 of the range (extremes of exactly 0 or 255 stay), assign
// every texel its nearest palette entry, then up to eight rounds of "least-squares endpoints for
// the current assignment, re-assign", stopping when the error no longer falls or the assignment
// repeats.  Six-value palette (endpoint 0 <= endpoint 1, entries 6 and 7 are 0 and 255): the same
// from the extremes that are not 0 / 255.  The candidate with the smaller squared error wins, the
// eight-value one on a tie.  All float arithmetic is IEEE binary32 in the order written here.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ntc_decode_kernel.h"

namespace ntc_hip_dev {

namespace {

// The eight values a block's two endpoints stand for (integer interpolation with the reference's
// rounding bias: +3 before /7, +2 before /5).
__device__ __forceinline__ void bc4_palette(uint32_t e0, uint32_t e1, uint32_t (&p)[8])
{
    p[0] = e0; p[1] = e1;
    if (e0 > e1) {
#pragma unroll
        for (uint32_t k = 1; k < 7; ++k) p[k + 1] = ((7 - k) * e0 + k * e1 + 3) / 7;
    } else {
#pragma unroll
        for (uint32_t k = 1; k < 5; ++k) p[k + 1] = ((5 - k) * e0 + k * e1 + 2) / 5;
        p[6] = 0; p[7] = 255;
    }
}

// Block = endpoint 0 | endpoint 1 << 8 | sixteen 3-bit indices from bit 16 up.
__device__ __forceinline__ uint64_t bc4_with_endpoints(uint64_t block, uint32_t e0, uint32_t e1)
{
    return (block & ~uint64_t(0xffff)) | uint64_t(e0 & 0xffu) | (uint64_t(e1 & 0xffu) << 8);
}
__device__ __forceinline__ uint32_t bc4_index(uint64_t block, int texel) { return uint32_t(block >> (16 + 3 * texel)) & 7u; }

// Nearest palette entry for every texel (the first of equally near ones); returns the summed squared error.
__device__ __forceinline__ float bc4_assign(uint32_t const (&values)[16], uint64_t& block)
{
    uint32_t palette[8];
    bc4_palette(uint32_t(block) & 0xffu, (uint32_t(block) >> 8) & 0xffu, palette);
    block &= 0xffff;
    float total = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        int best = 0x7fffffff;
        uint32_t pick = 0;
#pragma unroll
        for (uint32_t k = 0; k < 8; ++k) {
            int const d = int(values[t]) - int(palette[k]);
            if (d * d < best) { best = d * d; pick = k; }
        }
        total += float(best);
        block |= uint64_t(pick) << (16 + 3 * t);
    }
    return total;
}

__device__ __forceinline__ uint32_t bc4_endpoint(float v) { return uint32_t(rintf(fminf(fmaxf(v, 0.f), 255.f))); }   // a NaN becomes 0

// Least-squares endpoints for the block's current assignment.  With `eightValues` every texel takes
// part and weights are 1, 0, 6/7 ... 1/7; otherwise indices 6 and 7 (the fixed 0 and 255) are left
// out and weights are 1, 0, 4/5 ... 1/5, and a singular system leaves the endpoints alone.
__device__ __forceinline__ uint64_t bc4_refit(uint32_t const (&values)[16], uint64_t block, bool eightValues, bool keep255, bool keep0)
{
    float aa = 0.f, bb = 0.f, ab = 0.f, ax = 0.f, bx = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        uint32_t const k = bc4_index(block, t);
        float alpha;
        if (k < 2) alpha = 1.f - float(k);
        else if (eightValues) alpha = (8.f - float(k)) / 7.f;
        else if (k < 6) alpha = (6.f - float(k)) / 5.f;
        else continue;
        float const beta = 1.f - alpha, x = float(values[t]);
        aa += alpha * alpha; bb += beta * beta; ab += alpha * beta;
        ax += alpha * x; bx += beta * x;
    }
    if (eightValues) {
        float const factor = 1.f / (aa * bb - ab * ab);
        uint32_t e0 = keep255 ? 255u : bc4_endpoint((ax * bb - bx * ab) * factor);
        uint32_t e1 = keep0 ? 0u : bc4_endpoint((bx * aa - ax * ab) * factor);
        if (e0 < e1) { uint32_t const t = e0; e0 = e1; e1 = t; }
        return bc4_with_endpoints(block, e0, e1);
    }
    float const det = aa * bb - ab * ab;
    if (det == 0.f) return block;
    return bc4_with_endpoints(block, bc4_endpoint((ax * bb - bx * ab) / det), bc4_endpoint((bx * aa - ax * ab) / det));
}

// Up to eight rounds of refit + re-assign from a starting block; returns the best block and its error.
__device__ __forceinline__ uint64_t bc4_refine(uint32_t const (&values)[16], uint64_t block, bool eightValues, bool keep255, bool keep0, float& bestError)
{
    bestError = bc4_assign(values, block);
    uint64_t best = block;
    for (int round = 0; round < 8; ++round) {
        block = bc4_refit(values, block, eightValues, keep255, keep0);
        float const error = bc4_assign(values, block);
        if (error >= bestError) break;
        bool const repeated = (block >> 16) == (best >> 16);
        best = block;
        if (repeated) break;
        bestError = error;
    }
    return best;
}

__device__ uint64_t bc4_encode(float const (&texels)[16])
{
    uint32_t values[16];
    uint32_t lo = 255, hi = 0, loInner = 255, hiInner = 0;      // extremes; extremes among values that are not 0 / not 255
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        float const s = fminf(fmaxf(texels[t], 0.f), 1.f);     // saturate: a NaN becomes 0
        values[t] = uint32_t(rintf(s * 255.f));
        lo = min(lo, values[t]); hi = max(hi, values[t]);
        if (values[t] != 0) loInner = min(loInner, values[t]);
        if (values[t] != 255) hiInner = max(hiInner, values[t]);
    }
    bool const keep0 = lo == 0, keep255 = hi == 255;
    float error8, error6;
    uint64_t const block8 = bc4_refine(values, bc4_with_endpoints(0, keep255 ? 255u : hi - (hi - lo) / 34u, keep0 ? 0u : lo + (hi - lo) / 34u),
                                       true, keep255, keep0, error8);
    // unsigned arithmetic on purpose: with no inner values (all texels 0 or 255) the difference wraps, as in the reference
    uint32_t const inset = (hiInner - loInner) / 34u;
    uint64_t const block6 = bc4_refine(values, bc4_with_endpoints(0, loInner + inset, hiInner - inset), false, false, false, error6);
    return error6 < error8 ? block6 : block8;
}

// Channel c of the pixel at (x, y) of the source image; outside the image everything reads as 0,
// like a texture load there.
__device__ __forceinline__ float source_channel(BlockCompressArgs const& a, int x, int y, int c)
{
    if (x < 0 || y < 0 || x >= a.srcWidth || y >= a.srcHeight) return 0.f;
    if (c >= a.numChannels) return c == 3 ? 1.f : 0.f;
    uint8_t const* px = a.src + size_t(y) * a.rowPitch + size_t(x) * a.pixelStride;
    switch (a.format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  return float(px[c]) / 255.f;
    case NTC_HIP_DEV_FORMAT_UNORM16: return float(reinterpret_cast<uint16_t const*>(px)[c]) / 65535.f;
    case NTC_HIP_DEV_FORMAT_FLOAT16: return float(reinterpret_cast<_Float16 const*>(px)[c]);
    case NTC_HIP_DEV_FORMAT_FLOAT32: return reinterpret_cast<float const*>(px)[c];
    default:                         return float(reinterpret_cast<uint32_t const*>(px)[c]);
    }
}

} // namespace

// Thread groups of 16 x 8 blocks as in the reference (BLOCK_COMPRESS_CS_GROUP_WIDTH / HEIGHT).
template <int CHANNELS>
__global__ void __launch_bounds__(128)
bc4_compress_kernel(BlockCompressArgs a)
{
    int const bx = blockIdx.x * 16 + (threadIdx.x & 15), by = blockIdx.y * 8 + (threadIdx.x >> 4);
    if (bx >= a.widthInBlocks || by >= a.heightInBlocks) return;
    uint64_t out[CHANNELS];
#pragma unroll
    for (int c = 0; c < CHANNELS; ++c) {
        float texels[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) texels[t] = source_channel(a, a.srcLeft + bx * 4 + (t & 3), a.srcTop + by * 4 + (t >> 2), c);
        out[c] = bc4_encode(texels);
    }
    uint64_t* const dst = reinterpret_cast<uint64_t*>(a.dst + size_t(by + a.dstOffsetY) * a.dstRowPitch) + size_t(bx + a.dstOffsetX) * CHANNELS;
#pragma unroll
    for (int c = 0; c < CHANNELS; ++c) dst[c] = out[c];
}

hipError_t launch_block_compress(BlockCompressArgs const& a, int channels, hipStream_t stream)
{
    dim3 const grid((a.widthInBlocks + 15) / 16, (a.heightInBlocks + 7) / 8);
    if (channels == 1) hipLaunchKernelGGL(bc4_compress_kernel<1>, grid, dim3(128), 0, stream, a);
    else               hipLaunchKernelGGL(bc4_compress_kernel<2>, grid, dim3(128), 0, stream, a);
    return hipGetLastError();
}

} // namespace ntc_hip_dev
