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

// u(clamp(roundf(p), 0, top)) of WriteImageChannel (src/ImageProcessing.cu:141-152) for the UNORM formats.
// roundf rounds halves away from zero; for |p| < 2^23 it equals trunc(p + copysign(c, p)) with c the
// largest float below 1/2 (the sum rounds up to the next integer exactly when the fraction is at
// least 1/2), and negative p end at 0 either way, so: max with 0, add c, cap, truncating conversion.
__device__ __forceinline__ uint32_t unorm_code(float p, float top)
{
    return uint32_t(fminf(fmaxf(p, 0.f) + 0.49999997f, top));
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

constexpr int kRowsPerGroup = 4;       // image rows one workgroup of the copy kernels covers (more rows per workgroup measured slower)

constexpr int bytes_per_channel(int format)
{
    return format == NTC_HIP_DEV_FORMAT_UNORM8 ? 1 : (format == NTC_HIP_DEV_FORMAT_UNORM16 || format == NTC_HIP_DEV_FORMAT_FLOAT16) ? 2 : 4;
}

// WriteImageChannel (src/ImageProcessing.cu:141-164): the channel's bits in the destination format.
template <int FORMAT>
__device__ __forceinline__ uint32_t encode_channel(int colorSpace, float value, bool dithering, float dither)
{
    value = encode_color_space(colorSpace, value);
    if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_UNORM8) {
        if (dithering) value += dither / 255.f;
        return unorm_code(value * 255.f, 255.f);
    } else if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_UNORM16) {
        if (dithering) value += dither / 65535.f;
        return unorm_code(value * 65535.f, 65535.f);
    } else if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_FLOAT16) {
        float v = fmaxf(-65504.f, fminf(65504.f, value));
        asm volatile("" : "+v"(v));                          // round the clamped value, not a fused expression
        return uint32_t(__builtin_bit_cast(uint16_t, (_Float16)v));
    } else if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_FLOAT32) {
        return __builtin_bit_cast(uint32_t, value);
    } else {
        return uint32_t(fmaxf(value, 0.f));
    }
}

// One lane per pixel.  The pixel is produced 16 bytes at a time (16 / 8 / 4 channels for 1 / 2 / 4-byte
// formats) and stored with the widest access the image's alignment allows (a.vectorBytes, decided
// on the host from base, pitch and stride); source halves come in as the dword pairs of the
// planar-pair layout, coalesced across the lanes of a row.
template <int FORMAT>
__global__ void __launch_bounds__(256)
read_channels_kernel(ReadChannelsArgs a)
{
    constexpr int BPC = bytes_per_channel(FORMAT), PER = 16 / BPC;
    int const x = blockIdx.x * 64 + (threadIdx.x & 63);
    if (x >= a.width) return;
    for (int y = blockIdx.y * kRowsPerGroup + (threadIdx.x >> 6); y < min(a.height, int(blockIdx.y + 1) * kRowsPerGroup); y += 4) {
    // GetPixelBaseAddress / GetChannelAddress, src/RegressionKernels.h:36-45
    uint16_t const* src = a.planarPairs + size_t(y) * size_t(a.width) * size_t(a.setChannels) + size_t(x) * 2;
    uint8_t* px = a.dst + size_t(y) * a.rowPitch + size_t(x) * a.pixelStride;
    DitherRng rng(uint32_t(x) + uint32_t(y) * uint32_t(a.width));
    int loadedPair = -1;
    uint32_t pairBits = 0;
    for (int base = 0; base < a.dstChannels; base += PER) {
        uint32_t words[4] = { 0u, 0u, 0u, 0u };
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            int const ch = base + k;
            if (ch >= a.dstChannels) continue;               // uniform
            float value;
            if (ch < a.numChannels) {
                int const c = a.firstChannel + ch;
                if ((c >> 1) != loadedPair) {
                    loadedPair = c >> 1;
                    pairBits = *reinterpret_cast<uint32_t const*>(src + size_t(c & ~1) * size_t(a.width));
                }
                uint16_t const bits = uint16_t((c & 1) ? pairBits >> 16 : pairBits);
                value = decode_color_space(a.srcColorSpaces[ch], float(__builtin_bit_cast(_Float16, bits)));
            } else {
                value = (ch == 3) ? 1.f : 0.f;               // GetDefaultChannelValue, src/ImageProcessing.cu:166-170
            }
            float const dither = a.useDithering ? rng.next_float() - 0.5f : 0.f;      // one draw per destination channel
            uint32_t const bits = encode_channel<FORMAT>(ch < 16 ? a.dstColorSpaces[ch] : 0, value, a.useDithering != 0, dither);
            words[(k * BPC) >> 2] |= bits << (8 * ((k * BPC) & 3));
        }
        int const bytes = min(PER, a.dstChannels - base) * BPC;
        uint8_t* const out = px + base * BPC;
        if (bytes == 16 && a.vectorBytes >= 16) {
            *reinterpret_cast<uint4*>(out) = make_uint4(words[0], words[1], words[2], words[3]);
        } else if ((bytes & 7) == 0 && a.vectorBytes >= 8) {
            for (int q = 0; q < bytes / 8; ++q) reinterpret_cast<uint2*>(out)[q] = make_uint2(words[2 * q], words[2 * q + 1]);
        } else if ((bytes & 3) == 0 && a.vectorBytes >= 4) {
            for (int q = 0; q < bytes / 4; ++q) reinterpret_cast<uint32_t*>(out)[q] = words[q];
        } else if constexpr (BPC == 1) {
            for (int q = 0; q < bytes; ++q) out[q] = uint8_t(words[q >> 2] >> (8 * (q & 3)));
        } else if constexpr (BPC == 2) {
            for (int q = 0; q < bytes / 2; ++q) reinterpret_cast<uint16_t*>(out)[q] = uint16_t(words[q >> 1] >> (16 * (q & 1)));
        } else {
            for (int q = 0; q < bytes / 4; ++q) reinterpret_cast<uint32_t*>(out)[q] = words[q];
        }
    }
    }
}

// ReadImageChannel, src/ImageProcessing.cu:113-139: channel k of a 16-byte piece of the pixel.
template <int FORMAT>
__device__ __forceinline__ float decode_channel(uint32_t const (&words)[4], int k, float const* unorm8Table)
{
    constexpr int BPC = bytes_per_channel(FORMAT);
    uint32_t const w = words[(k * BPC) >> 2] >> (8 * ((k * BPC) & 3));
    if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_UNORM8)       return unorm8Table[w & 0xffu];          // = float(code) / 255.f
    else if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_UNORM16) return float(w & 0xffffu) / 65535.f;
    else if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_FLOAT16) return float(__builtin_bit_cast(_Float16, uint16_t(w)));
    else if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_FLOAT32) return __builtin_bit_cast(float, w);
    else                                                     return float(w);
}

// User image -> internal fp16 planar pairs: ITextureSet::WriteChannels through CopyImageKernel's 1:1
// branch (src/TextureSet.cpp:835-913, src/ImageProcessing.cu:220-265), optional vertical flip.
// The pixel is read 16 bytes at a time with the widest loads its alignment allows; channel pairs
// that fall on a half2 of the internal layout are written as one dword.
template <int FORMAT>
__global__ void __launch_bounds__(256)
write_channels_kernel(WriteChannelsArgs a)
{
    constexpr int BPC = bytes_per_channel(FORMAT), PER = 16 / BPC;
    __shared__ float unorm8Table[FORMAT == NTC_HIP_DEV_FORMAT_UNORM8 ? 256 : 1];
    if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_UNORM8) {     // one correctly rounded division per code instead of per channel
        unorm8Table[threadIdx.x & 255] = float(threadIdx.x & 255) / 255.f;
        __syncthreads();
    }
    int const x = blockIdx.x * 64 + (threadIdx.x & 63);
    if (x >= a.width) return;
    for (int y = blockIdx.y * kRowsPerGroup + (threadIdx.x >> 6); y < min(a.height, int(blockIdx.y + 1) * kRowsPerGroup); y += 4) {
    int const srcY = a.verticalFlip ? a.height - 1 - y : y;          // SetupBilinearFilter flips the read position
    uint8_t const* px = a.src + size_t(srcY) * a.rowPitch + size_t(x) * a.pixelStride;
    uint16_t* dst = a.planarPairs + size_t(y) * size_t(a.width) * size_t(a.setChannels) + size_t(x) * 2;
    uint32_t pending = 0;                                            // low half of a pair waiting for its partner
    for (int base = 0; base < a.numChannels; base += PER) {
        int const bytes = min(PER, a.numChannels - base) * BPC;
        uint8_t const* const in = px + base * BPC;
        uint32_t words[4] = { 0u, 0u, 0u, 0u };
        if (bytes == 16 && a.vectorBytes >= 16) {
            uint4 const v = *reinterpret_cast<uint4 const*>(in);
            words[0] = v.x; words[1] = v.y; words[2] = v.z; words[3] = v.w;
        } else if ((bytes & 3) == 0 && a.vectorBytes >= 4) {
            for (int q = 0; q < bytes / 4; ++q) words[q] = reinterpret_cast<uint32_t const*>(in)[q];
        } else if constexpr (BPC == 1) {
            for (int q = 0; q < bytes; ++q) words[q >> 2] |= uint32_t(in[q]) << (8 * (q & 3));
        } else if constexpr (BPC == 2) {
            for (int q = 0; q < bytes / 2; ++q) words[q >> 1] |= uint32_t(reinterpret_cast<uint16_t const*>(in)[q]) << (16 * (q & 1));
        } else {
            for (int q = 0; q < bytes / 4; ++q) words[q] = reinterpret_cast<uint32_t const*>(in)[q];
        }
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            int const ch = base + k;
            if (ch >= a.numChannels) continue;                       // uniform
            float v = decode_color_space(a.srcColorSpaces[ch], decode_channel<FORMAT>(words, k, unorm8Table));
            v = encode_color_space(a.dstColorSpaces[ch], v);
            v = fmaxf(-65504.f, fminf(65504.f, v));                  // WriteImageChannel FLOAT16, src/ImageProcessing.cu:154-156
            asm volatile("" : "+v"(v));
            uint32_t const half = __builtin_bit_cast(uint16_t, (_Float16)v);
            int const c = a.firstChannel + ch;
            uint16_t* const at = dst + size_t(c & ~1) * size_t(a.width);
            if ((c & 1) == 0) {
                if (ch + 1 < a.numChannels) pending = half;          // partner follows: store both together
                else at[0] = uint16_t(half);
            } else {
                if (ch > 0) *reinterpret_cast<uint32_t*>(at) = pending | (half << 16);
                else at[1] = uint16_t(half);
            }
        }
    }
    }
}

hipError_t launch_write_channels(WriteChannelsArgs const& a, hipStream_t stream)
{
    dim3 const grid((a.width + 63) / 64, (a.height + kRowsPerGroup - 1) / kRowsPerGroup);
    switch (a.format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  hipLaunchKernelGGL(write_channels_kernel<NTC_HIP_DEV_FORMAT_UNORM8>, grid, dim3(256), 0, stream, a); break;
    case NTC_HIP_DEV_FORMAT_UNORM16: hipLaunchKernelGGL(write_channels_kernel<NTC_HIP_DEV_FORMAT_UNORM16>, grid, dim3(256), 0, stream, a); break;
    case NTC_HIP_DEV_FORMAT_FLOAT16: hipLaunchKernelGGL(write_channels_kernel<NTC_HIP_DEV_FORMAT_FLOAT16>, grid, dim3(256), 0, stream, a); break;
    case NTC_HIP_DEV_FORMAT_FLOAT32: hipLaunchKernelGGL(write_channels_kernel<NTC_HIP_DEV_FORMAT_FLOAT32>, grid, dim3(256), 0, stream, a); break;
    case NTC_HIP_DEV_FORMAT_UINT32:  hipLaunchKernelGGL(write_channels_kernel<NTC_HIP_DEV_FORMAT_UINT32>, grid, dim3(256), 0, stream, a); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// Per-channel sum of squared differences between a decoded mip and its reference image, both in the
// internal layout: the loss branch of InferenceKernel (src/Inference.cu:77-118) as a pass of its own.
// With maskChannel >= 0 the decoded mask channel is first clamped to [0, 1] and stored back clamped
// (Inference.cu:96-97,112; a negative zero becomes +0 as the device max() of the reference returns),
// and with discardMaskedOut set a texel whose REFERENCE mask value is zero counts on the mask channel
// only (Inference.cu:80-84,107-108).  Each workgroup covers 64 x 16 texels and writes 16 double partial
// sums (channel-major, so that the second stage reads them coalesced); ReduceLoss likewise finishes in
// double (src/Optimizer.cu:382-387).
__global__ void __launch_bounds__(256)
image_loss_kernel(uint16_t* __restrict__ a, uint16_t const* __restrict__ b, int width, int height, int setChannels,
                  uint32_t validChannelMask, int maskChannel, int discardMaskedOut, double* __restrict__ partials)
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
            bool maskedOut = false;
            if (maskChannel >= 0 && discardMaskedOut) {
                uint16_t const m = b[base + size_t(maskChannel & ~1) * size_t(width) + size_t(maskChannel & 1)];
                maskedOut = (m & 0x7FFFu) == 0;
            }
#pragma unroll
            for (int p = 0; p < NTC_HIP_DEV_MAX_CHANNELS / 2; ++p) {
                if (2 * p < setChannels) {
                    uint32_t* const pa = reinterpret_cast<uint32_t*>(a + base + size_t(2 * p) * size_t(width));
                    uint32_t const va = *pa;
                    uint32_t const vb = *reinterpret_cast<uint32_t const*>(b + base + size_t(2 * p) * size_t(width));
                    float a0 = float(__builtin_bit_cast(_Float16, uint16_t(va)));
                    float a1 = float(__builtin_bit_cast(_Float16, uint16_t(va >> 16)));
                    if ((maskChannel >> 1) == p) {      // never true for a negative maskChannel
                        if (maskChannel & 1) a1 = a1 > 0.f ? fminf(a1, 1.f) : 0.f;
                        else                 a0 = a0 > 0.f ? fminf(a0, 1.f) : 0.f;
                        uint32_t const clamped = uint32_t(__builtin_bit_cast(uint16_t, _Float16(a0)))
                                               | uint32_t(__builtin_bit_cast(uint16_t, _Float16(a1))) << 16;
                        if (clamped != va) *pa = clamped;
                    }
                    float d0 = a0 - float(__builtin_bit_cast(_Float16, uint16_t(vb)));
                    float d1 = a1 - float(__builtin_bit_cast(_Float16, uint16_t(vb >> 16)));
                    if (maskedOut && maskChannel != 2 * p) d0 = 0.f;
                    if (maskedOut && maskChannel != 2 * p + 1) d1 = 0.f;
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
        size_t const block = size_t(blockIdx.y) * gridDim.x + blockIdx.x, blocks = size_t(gridDim.x) * gridDim.y;
        partials[size_t(c) * blocks + block] = sums[0][c] + sums[1][c] + sums[2][c] + sums[3][c];
    }
}

// Second stage: workgroup c adds the partial sums of channel c, in double and in a fixed order
// (thread t takes entries t, t + 256, ...; then one thread adds the 256 sub-totals), and writes the
// total behind the partials.
__global__ void __launch_bounds__(256)
image_loss_reduce_kernel(double const* __restrict__ partials, size_t blocks, double* __restrict__ totals)
{
    __shared__ double sums[256];
    int const c = blockIdx.x;
    double acc = 0.0;
    for (size_t b = threadIdx.x; b < blocks; b += 256) acc += partials[size_t(c) * blocks + b];
    sums[threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double total = 0.0;
        for (int t = 0; t < 256; ++t) total += sums[t];
        totals[c] = total;
    }
}

hipError_t launch_image_loss(uint16_t* a, uint16_t const* b, int width, int height, int setChannels,
                             uint32_t validChannelMask, int maskChannel, int discardMaskedOut, double* partials, hipStream_t stream)
{
    dim3 const grid((width + 63) / 64, (height + 15) / 16);
    size_t const blocks = size_t(grid.x) * size_t(grid.y);
    hipLaunchKernelGGL(image_loss_kernel, grid, dim3(256), 0, stream, a, b, width, height, setChannels, validChannelMask,
                       maskChannel, discardMaskedOut, partials);
    hipLaunchKernelGGL(image_loss_reduce_kernel, dim3(NTC_HIP_DEV_MAX_CHANNELS), dim3(256), 0, stream, partials, blocks, partials + blocks * NTC_HIP_DEV_MAX_CHANNELS);
    return hipGetLastError();
}

hipError_t launch_read_channels(ReadChannelsArgs const& a, hipStream_t stream)
{
    dim3 const grid((a.width + 63) / 64, (a.height + kRowsPerGroup - 1) / kRowsPerGroup);
    switch (a.format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  hipLaunchKernelGGL(read_channels_kernel<NTC_HIP_DEV_FORMAT_UNORM8>, grid, dim3(256), 0, stream, a); break;
    case NTC_HIP_DEV_FORMAT_UNORM16: hipLaunchKernelGGL(read_channels_kernel<NTC_HIP_DEV_FORMAT_UNORM16>, grid, dim3(256), 0, stream, a); break;
    case NTC_HIP_DEV_FORMAT_FLOAT16: hipLaunchKernelGGL(read_channels_kernel<NTC_HIP_DEV_FORMAT_FLOAT16>, grid, dim3(256), 0, stream, a); break;
    case NTC_HIP_DEV_FORMAT_FLOAT32: hipLaunchKernelGGL(read_channels_kernel<NTC_HIP_DEV_FORMAT_FLOAT32>, grid, dim3(256), 0, stream, a); break;
    case NTC_HIP_DEV_FORMAT_UINT32:  hipLaunchKernelGGL(read_channels_kernel<NTC_HIP_DEV_FORMAT_UINT32>, grid, dim3(256), 0, stream, a); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

} // namespace ntc_hip_dev
