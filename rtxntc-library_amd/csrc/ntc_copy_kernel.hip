// ntc_copy_kernel.hip - internal fp16 texture layout <-> user pitch-linear image, image loss (gfx950).
//
// The 1:1 branch of the reference's CopyImageKernel as ITextureSet::ReadChannels / WriteChannels
// use it (src/ImageProcessing.cu:86-164,220-265, src/TextureSet.cpp:835-985): no resize; colour
// space decode/encode and dithering as the reference defines them.  One lane per pixel; source reads are the half2 pairs of
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

// Transfer functions, src/CudaUtils.h:61-114 (sRGB, Hybrid Log-Gamma) and src/ImageProcessing.cu:86-111.
// The transcendental parts are the device math library's, so results agree with a CPU
// evaluation to a few units in the last place, not bit for bit.
__device__ __forceinline__ float decode_color_space(int colorSpace, float v)
{
    if (colorSpace == 1) return (v <= 0.04045f) ? v / 12.92f : powf((v + 0.055f) / 1.055f, 2.4f);
    if (colorSpace == 2) {
        float const sign = (v < 0.f) ? -1.f : 1.f;
        float const h = fabsf(v);
        return (h < 0.5f) ? 4.f * h * h * sign : (expf((h - 0.55991073f) / 0.17883277f) + 0.28466892f) * sign;
    }
    return v;
}
__device__ __forceinline__ float encode_color_space(int colorSpace, float v)
{
    if (colorSpace == 1) return (v <= 0.0031308f) ? v * 12.92f : 1.055f * powf(v, 1.0f / 2.4f) - 0.055f;
    if (colorSpace == 2) {
        float const sign = (v < 0.f) ? -1.f : 1.f;
        float const e = fabsf(v);
        return (e < 1.f) ? 0.5f * sqrtf(e) * sign : (0.17883277f * logf(e - 0.28466892f) + 0.55991073f) * sign;
    }
    return v;
}

// HashBasedRNG, src/CudaUtils.h:117-184: Jenkins hash of the pixel index seeds a Murmur3 round per draw.
struct DitherRng {
    uint32_t seed, index;
    __device__ explicit DitherRng(uint32_t linearIndex) : index(1)
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
    __device__ float next_float()                            // [0, 1)
    {
        uint32_t k = index++ * 0xcc9e2d51u;
        k = (k << 15) | (k >> 17);
        k *= 0x1b873593u;
        uint32_t h = seed ^ k;
        h = ((h << 13) | (h >> 19)) * 5u + 0xe6546b64u;
        h ^= 4u;
        h ^= h >> 16; h *= 0x85ebca6bu;
        h ^= h >> 13; h *= 0xc2b2ae35u;
        h ^= h >> 16;
        return __builtin_bit_cast(float, (h & 0x7fffffu) | 0x3f800000u) - 1.f;
    }
};

__device__ __forceinline__ void write_channel(uint8_t* px, uint32_t ch, int format, int colorSpace, float value, float dither)
{
    value = encode_color_space(colorSpace, value);
    switch (format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:
        value += dither / 255.f;
        px[ch] = uint8_t(fmaxf(0.f, fminf(255.f, round_half_away(value * 255.f))));
        break;
    case NTC_HIP_DEV_FORMAT_UNORM16:
        value += dither / 65535.f;
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
    DitherRng rng(uint32_t(x) + uint32_t(y) * uint32_t(a.width));
    for (int ch = 0; ch < a.dstChannels; ++ch) {
        float value;
        if (ch < a.numChannels) {
            int const c = a.firstChannel + ch;
            uint16_t const bits = src[size_t(c & ~1) * size_t(a.width) + size_t(c & 1)];
            value = decode_color_space(a.srcColorSpaces[ch], float(__builtin_bit_cast(_Float16, bits)));
        } else {
            value = (ch == 3) ? 1.f : 0.f;                   // GetDefaultChannelValue, src/ImageProcessing.cu:166-170
        }
        float const dither = a.useDithering ? rng.next_float() - 0.5f : 0.f;      // one draw per destination channel
        write_channel(px, uint32_t(ch), a.format, ch < 16 ? a.dstColorSpaces[ch] : 0, value, dither);
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
        float v = decode_color_space(a.srcColorSpaces[ch], read_channel(px, uint32_t(ch), a.format));
        v = encode_color_space(a.dstColorSpaces[ch], v);
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
