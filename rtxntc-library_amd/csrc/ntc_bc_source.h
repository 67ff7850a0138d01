// ntc_bc_source.h - how the block-compression kernels read their source image.
#ifndef NTC_BC_SOURCE_H
#define NTC_BC_SOURCE_H
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ntc_decode_kernel.h"

namespace ntc_hip_dev {

// fminf / fmaxf as single instructions.  The compiler brackets the library functions with two
// canonicalising instructions (it cannot know that its operands are already quiet); v_min_f32 /
// v_max_f32 themselves return the other operand when one is a NaN, which is all fminf / fmaxf promise.
__device__ __forceinline__ float min_f32(float a, float b) { float r; asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b)); return r; }
__device__ __forceinline__ float max_f32(float a, float b) { float r; asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b)); return r; }

// k / d for an integer k in [0, d], d = 255 or 65535, r = 1 / d rounded: one Newton step on k * r gives the
// correctly rounded quotient for every such k (all 256 + 65536 cases are checked in the tests with exact
// rational arithmetic) at a third of the instructions of a division.
__device__ __forceinline__ float unorm_quotient(float k, float d, float r)
{
    float const q = k * r;
    return __builtin_fmaf(__builtin_fmaf(-q, d, k), r, q);
}

// Channel c of the pixel at (x, y) of the source image, as a texture load gives it: outside the image
// everything reads as 0; channels the image does not have read as 0, alpha as 1.  A stored -0 becomes
// +0 (the "+ 0.f"): minima and maxima of +0 and -0 depend on the operand order otherwise.
__device__ __forceinline__ float source_channel(BlockCompressArgs const& a, int x, int y, int c)
{
    if (x < 0 || y < 0 || x >= a.srcWidth || y >= a.srcHeight) return 0.f;
    if (c >= a.numChannels) return c == 3 ? 1.f : 0.f;
    uint8_t const* px = a.src + size_t(y) * a.rowPitch + size_t(x) * a.pixelStride;
    switch (a.format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  return unorm_quotient(float(px[c]), 255.f, 1.f / 255.f);
    case NTC_HIP_DEV_FORMAT_UNORM16: return unorm_quotient(float(reinterpret_cast<uint16_t const*>(px)[c]), 65535.f, 1.f / 65535.f);
    case NTC_HIP_DEV_FORMAT_FLOAT16: return float(reinterpret_cast<_Float16 const*>(px)[c]) + 0.f;
    case NTC_HIP_DEV_FORMAT_FLOAT32: return reinterpret_cast<float const*>(px)[c] + 0.f;
    default:                         return float(reinterpret_cast<uint32_t const*>(px)[c]);
    }
}

// All four channels of a pixel.  The common source, four UNORM8 channels with every pixel on a 4-byte
// boundary (args.packedRgba8, set by the host), takes one 32-bit load per pixel.
__device__ __forceinline__ void source_pixel(BlockCompressArgs const& a, int x, int y, float (&rgba)[4])
{
    if (a.packedRgba8) {
        uint32_t v = 0;
        if (x >= 0 && y >= 0 && x < a.srcWidth && y < a.srcHeight)
            v = *reinterpret_cast<uint32_t const*>(a.src + size_t(y) * a.rowPitch + size_t(x) * a.pixelStride);
#pragma unroll
        for (int c = 0; c < 4; ++c) rgba[c] = unorm_quotient(float((v >> (8 * c)) & 0xffu), 255.f, 1.f / 255.f);
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) rgba[c] = source_channel(a, x, y, c);
    }
}

} // namespace ntc_hip_dev
#endif
