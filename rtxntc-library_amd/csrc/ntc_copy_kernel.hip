// ntc_copy_kernel.hip - internal fp16 texture layout -> user pitch-linear image (gfx950).
//
// The 1:1 branch of the reference's CopyImageKernel as ITextureSet::ReadChannels uses it
// (src/ImageProcessing.cu:141-164,220-265, src/TextureSet.cpp:948-967): no resize, no
// dithering, linear colour spaces.  One lane per pixel; source reads are the half2 pairs of
// the planar-pair layout (coalesced across x), destination writes are the pixel's bytes.
// HBM-bound: 2 bytes read and 1-4 bytes written per channel.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ntc_decode_kernel.h"

namespace ntc_hip_dev {

// WriteImageChannel, src/ImageProcessing.cu:141-164.  roundf = round half away from zero,
// written as trunc + exact fraction test so that host and device agree on every input.
__device__ __forceinline__ float round_half_away(float v)
{
    float r = truncf(v);
    float const fr = v - r;                                  // exact
    if (fr >= 0.5f) r += 1.f; else if (fr <= -0.5f) r -= 1.f;
    return r;
}

__device__ __forceinline__ void write_channel(uint8_t* px, uint32_t ch, int format, float value)
{
    switch (format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:
        px[ch] = uint8_t(fmaxf(0.f, fminf(255.f, round_half_away(value * 255.f))));
        break;
    case NTC_HIP_DEV_FORMAT_UNORM16:
        reinterpret_cast<uint16_t*>(px)[ch] = uint16_t(fmaxf(0.f, fminf(65535.f, round_half_away(value * 65535.f))));
        break;
    case NTC_HIP_DEV_FORMAT_FLOAT16: {
        float v = fmaxf(-65504.f, fminf(65504.f, value));
        asm volatile("" : "+v"(v));
        reinterpret_cast<_Float16*>(px)[ch] = (_Float16)v;
        break;
    }
    case NTC_HIP_DEV_FORMAT_FLOAT32:
        reinterpret_cast<float*>(px)[ch] = value;
        break;
    case NTC_HIP_DEV_FORMAT_UINT32:
        reinterpret_cast<uint32_t*>(px)[ch] = uint32_t(fmaxf(value, 0.f));
        break;
    default:
        break;
    }
}

__global__ void __launch_bounds__(256)
read_channels_kernel(ReadChannelsArgs a)
{
    int const x = blockIdx.x * 64 + (threadIdx.x & 63);
    int const y = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (x >= a.width || y >= a.height) return;
    // GetPixelBaseAddress / GetChannelAddress, src/RegressionKernels.h:36-45
    uint16_t const* src = a.planarPairs + size_t(y) * size_t(a.width) * size_t(a.setChannels) + size_t(x) * 2;
    uint8_t* px = a.dst + size_t(y) * a.rowPitch + size_t(x) * a.pixelStride;
    for (int ch = 0; ch < a.dstChannels; ++ch) {
        float value;
        if (ch < a.numChannels) {
            int const c = a.firstChannel + ch;
            uint16_t const bits = src[size_t(c & ~1) * size_t(a.width) + size_t(c & 1)];
            value = float(__builtin_bit_cast(_Float16, bits));
        } else {
            value = (ch == 3) ? 1.f : 0.f;                   // GetDefaultChannelValue, src/ImageProcessing.cu:166-170
        }
        write_channel(px, uint32_t(ch), a.format, value);
    }
}

hipError_t launch_read_channels(ReadChannelsArgs const& a, hipStream_t stream)
{
    dim3 const grid((a.width + 63) / 64, (a.height + 3) / 4);
    hipLaunchKernelGGL(read_channels_kernel, grid, dim3(256), 0, stream, a);
    return hipGetLastError();
}

} // namespace ntc_hip_dev
