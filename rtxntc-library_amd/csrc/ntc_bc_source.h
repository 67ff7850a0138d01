// ntc_bc_source.h - how the block-compression kernels read their source image.
#ifndef NTC_BC_SOURCE_H
#define NTC_BC_SOURCE_H
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ntc_decode_kernel.h"

namespace ntc_hip_dev {

// Channel c of the pixel at (x, y) of the source image, as a texture load gives it: outside the image
// everything reads as 0; channels the image does not have read as 0, alpha as 1.  A stored -0 becomes
// +0 (the "+ 0.f"): minima and maxima of +0 and -0 depend on the operand order otherwise.
__device__ __forceinline__ float source_channel(BlockCompressArgs const& a, int x, int y, int c)
{
    if (x < 0 || y < 0 || x >= a.srcWidth || y >= a.srcHeight) return 0.f;
    if (c >= a.numChannels) return c == 3 ? 1.f : 0.f;
    uint8_t const* px = a.src + size_t(y) * a.rowPitch + size_t(x) * a.pixelStride;
    switch (a.format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  return float(px[c]) / 255.f;
    case NTC_HIP_DEV_FORMAT_UNORM16: return float(reinterpret_cast<uint16_t const*>(px)[c]) / 65535.f;
    case NTC_HIP_DEV_FORMAT_FLOAT16: return float(reinterpret_cast<_Float16 const*>(px)[c]) + 0.f;
    case NTC_HIP_DEV_FORMAT_FLOAT32: return reinterpret_cast<float const*>(px)[c] + 0.f;
    default:                         return float(reinterpret_cast<uint32_t const*>(px)[c]);
    }
}

} // namespace ntc_hip_dev
#endif
