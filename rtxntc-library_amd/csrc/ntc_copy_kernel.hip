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

// ReadImageChannel, src/ImageProcessing.cu:107-139 (linear colour space).
__device__ __forceinline__ float read_channel(uint8_t const* px, uint32_t ch, int format)
{
    switch (format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  return float(px[ch]) / 255.f;
    case NTC_HIP_DEV_FORMAT_UNORM16: return float(reinterpret_cast<uint16_t const*>(px)[ch]) / 65535.f;
    case NTC_HIP_DEV_FORMAT_FLOAT16: return float(reinterpret_cast<_Float16 const*>(px)[ch]);
    case NTC_HIP_DEV_FORMAT_FLOAT32: return reinterpret_cast<float const*>(px)[ch];
    case NTC_HIP_DEV_FORMAT_UINT32:  return float(reinterpret_cast<uint32_t const*>(px)[ch]);
    default: return 0.f;
    }
}

// User image -> internal fp16 planar pairs: ITextureSet::WriteChannels through CopyImageKernel's 1:1
// branch (src/TextureSet.cpp:829-913, src/ImageProcessing.cu:220-265), optional vertical flip.
__global__ void __launch_bounds__(256)
write_channels_kernel(WriteChannelsArgs a)
{
    int const x = blockIdx.x * 64 + (threadIdx.x & 63);
    int const y = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (x >= a.width || y >= a.height) return;
    int const srcY = a.verticalFlip ? a.height - 1 - y : y;          // SetupBilinearFilter flips the read position
    uint8_t const* px = a.src + size_t(srcY) * a.rowPitch + size_t(x) * a.pixelStride;
    uint16_t* dst = a.planarPairs + size_t(y) * size_t(a.width) * size_t(a.setChannels) + size_t(x) * 2;
    for (int ch = 0; ch < a.numChannels; ++ch) {
        float v = read_channel(px, uint32_t(ch), a.format);
        v = fmaxf(-65504.f, fminf(65504.f, v));                      // WriteImageChannel FLOAT16, src/ImageProcessing.cu:154-156
        asm volatile("" : "+v"(v));
        int const c = a.firstChannel + ch;
        dst[size_t(c & ~1) * size_t(a.width) + size_t(c & 1)] = __builtin_bit_cast(uint16_t, (_Float16)v);
    }
}

hipError_t launch_write_channels(WriteChannelsArgs const& a, hipStream_t stream)
{
    dim3 const grid((a.width + 63) / 64, (a.height + 3) / 4);
    hipLaunchKernelGGL(write_channels_kernel, grid, dim3(256), 0, stream, a);
    return hipGetLastError();
}

// Per-channel sum of squared differences between a decoded mip and its reference image, both in the
// internal layout: the loss branch of InferenceKernel (src/Inference.cu:77-118) without its masking
// options.  Each workgroup covers 64 x 16 texels and writes 16 double partial sums; the host adds the
// partials (as ReduceLoss finishes its reduction on the host in double, src/Optimizer.cu:382-387).
__global__ void __launch_bounds__(256)
image_loss_kernel(uint16_t const* __restrict__ a, uint16_t const* __restrict__ b, int width, int height, int setChannels,
                  uint32_t validChannelMask, double* __restrict__ partials)
{
    __shared__ double sums[4][NTC_HIP_DEV_MAX_CHANNELS];
    int const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int const x = blockIdx.x * 64 + lane;
    float acc[NTC_HIP_DEV_MAX_CHANNELS];
#pragma unroll
    for (int c = 0; c < NTC_HIP_DEV_MAX_CHANNELS; ++c) acc[c] = 0.f;
    for (int r = 0; r < 4; ++r) {
        int const y = blockIdx.y * 16 + wave * 4 + r;
        if (x < width && y < height) {
            size_t const base = size_t(y) * size_t(width) * size_t(setChannels) + size_t(x) * 2;
#pragma unroll
            for (int p = 0; p < NTC_HIP_DEV_MAX_CHANNELS / 2; ++p) {
                if (2 * p < setChannels) {
                    uint32_t const va = *reinterpret_cast<uint32_t const*>(a + base + size_t(2 * p) * size_t(width));
                    uint32_t const vb = *reinterpret_cast<uint32_t const*>(b + base + size_t(2 * p) * size_t(width));
                    float const d0 = float(__builtin_bit_cast(_Float16, uint16_t(va))) - float(__builtin_bit_cast(_Float16, uint16_t(vb)));
                    float const d1 = float(__builtin_bit_cast(_Float16, uint16_t(va >> 16))) - float(__builtin_bit_cast(_Float16, uint16_t(vb >> 16)));
                    acc[2 * p] += d0 * d0;
                    acc[2 * p + 1] += d1 * d1;
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < NTC_HIP_DEV_MAX_CHANNELS; ++c) {
        double v = ((validChannelMask >> c) & 1u) ? double(acc[c]) : 0.0;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
        if (lane == 0) sums[wave][c] = v;
    }
    __syncthreads();
    if (threadIdx.x < NTC_HIP_DEV_MAX_CHANNELS) {
        int const c = threadIdx.x;
        size_t const block = size_t(blockIdx.y) * gridDim.x + blockIdx.x;
        partials[block * NTC_HIP_DEV_MAX_CHANNELS + c] = sums[0][c] + sums[1][c] + sums[2][c] + sums[3][c];
    }
}

hipError_t launch_image_loss(uint16_t const* a, uint16_t const* b, int width, int height, int setChannels,
                             uint32_t validChannelMask, double* partials, hipStream_t stream)
{
    dim3 const grid((width + 63) / 64, (height + 15) / 16);
    hipLaunchKernelGGL(image_loss_kernel, grid, dim3(256), 0, stream, a, b, width, height, setChannels, validChannelMask, partials);
    return hipGetLastError();
}

hipError_t launch_read_channels(ReadChannelsArgs const& a, hipStream_t stream)
{
    dim3 const grid((a.width + 63) / 64, (a.height + 3) / 4);
    hipLaunchKernelGGL(read_channels_kernel, grid, dim3(256), 0, stream, a);
    return hipGetLastError();
}

} // namespace ntc_hip_dev
