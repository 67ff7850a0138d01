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

constexpr int bytes_per_channel(int format)
{
    return format == NTC_HIP_DEV_FORMAT_UNORM8 ? 1 : (format == NTC_HIP_DEV_FORMAT_UNORM16 || format == NTC_HIP_DEV_FORMAT_FLOAT16) ? 2 : 4;
}

// Lane -> pixel of the copy kernels: a workgroup covers 256 pixels of one row, or 64 pixels of four
// rows for images narrower than 256 (xShift = 8 or 6, chosen on the host).
struct CopyGrid {
    int x, y;
    __device__ explicit CopyGrid(int xShift)
        : x((int(blockIdx.x) << xShift) + (int(threadIdx.x) & ((1 << xShift) - 1))),
          y(int(blockIdx.y) * (256 >> xShift) + (int(threadIdx.x) >> xShift)) {}
};
inline dim3 copy_grid(int width, int height, int& xShift, bool wide = true)
{
    xShift = (wide && width >= 256) ? 8 : 6;
    int const rows = 256 >> xShift;
    return dim3((width + (1 << xShift) - 1) >> xShift, (height + rows - 1) / rows);
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

// One lane per pixel.  All the half2 pairs the pixel needs are loaded before any arithmetic (the
// loads of a lane overlap; issued one by one behind their uses the kernel ran at half the rate),
// coalesced across the lanes of a row.  The pixel is produced 16 bytes at a time (16 / 8 / 4
// channels for 1 / 2 / 4-byte formats) and stored with the widest access the image's alignment allows
// (a.vectorBytes, decided on the host from base, pitch and stride).  PLAIN = every colour space
// linear and no dithering: the transfer functions and the generator are compiled out.
template <int FORMAT, bool PLAIN>
__global__ void __launch_bounds__(256)
read_channels_kernel(ReadChannelsArgs a)
{
    constexpr int BPC = bytes_per_channel(FORMAT), PER = 16 / BPC;
    CopyGrid const at(a.xShift);
    int const x = at.x, y = at.y;
    if (x >= a.width || y >= a.height) return;
    // GetPixelBaseAddress / GetChannelAddress, src/RegressionKernels.h:36-45
    uint16_t const* src = a.planarPairs + size_t(y) * size_t(a.width) * size_t(a.setChannels) + size_t(x) * 2;
    uint8_t* px = a.dst + size_t(y) * a.rowPitch + size_t(x) * a.pixelStride;
    int const firstPair = a.firstChannel >> 1;
    bool const odd = (a.firstChannel & 1) != 0;
    int const pairs = ((a.firstChannel + a.numChannels + 1) >> 1) - firstPair;     // at most 8
    uint32_t pr[NTC_HIP_DEV_MAX_CHANNELS / 2];
#pragma unroll
    for (int p = 0; p < NTC_HIP_DEV_MAX_CHANNELS / 2; ++p) {
        pr[p] = 0u;
        if (p < pairs) pr[p] = *reinterpret_cast<uint32_t const*>(src + size_t(2 * (firstPair + p)) * size_t(a.width));     // uniform
    }
    auto half_of = [&](int k) -> uint32_t {                  // half k of the loaded pairs, k a compile-time constant after unrolling
        return k < NTC_HIP_DEV_MAX_CHANNELS ? ((k & 1) ? pr[(k >> 1) & 7] >> 16 : pr[(k >> 1) & 7] & 0xffffu) : 0u;
    };
    [[maybe_unused]] DitherRng rng(uint32_t(x) + uint32_t(y) * uint32_t(a.width));
#pragma unroll
    for (int piece = 0; piece < NTC_HIP_DEV_MAX_CHANNELS / PER; ++piece) {
        int const base = piece * PER;
        if (base >= a.dstChannels) break;                    // uniform
        uint32_t words[4] = { 0u, 0u, 0u, 0u };
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            int const ch = base + k;
            if (ch >= a.dstChannels) continue;               // uniform
            float value;
            if (ch < a.numChannels) {
                uint32_t const bits = odd ? half_of(ch + 1) : half_of(ch);
                value = float(__builtin_bit_cast(_Float16, uint16_t(bits)));
                if constexpr (!PLAIN) value = decode_color_space(a.srcColorSpaces[ch], value);
            } else {
                value = (ch == 3) ? 1.f : 0.f;               // GetDefaultChannelValue, src/ImageProcessing.cu:166-170
            }
            uint32_t bits;
            if constexpr (PLAIN) {
                bits = encode_channel<FORMAT>(0, value, false, 0.f);
            } else {
                float const dither = a.useDithering ? rng.next_float() - 0.5f : 0.f;  // one draw per destination channel
                bits = encode_channel<FORMAT>(a.dstColorSpaces[ch], value, a.useDithering != 0, dither);
            }
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
    // Destination channels beyond the sixteen a set can hold (a pixel stride of more than 16 components): the
    // default value 0 in every format and colour space, dithered or not (|noise| < 1/2 step rounds to 0).
    int const tailBegin = NTC_HIP_DEV_MAX_CHANNELS * BPC, tailEnd = a.dstChannels * BPC;      // bytes; uniform
    if (tailEnd > tailBegin) {
        if (((tailEnd - tailBegin) & 3) == 0 && a.vectorBytes >= 4) {
            for (int b = tailBegin; b < tailEnd; b += 4) *reinterpret_cast<uint32_t*>(px + b) = 0u;
        } else if constexpr (BPC == 2) {
            for (int b = tailBegin; b < tailEnd; b += 2) *reinterpret_cast<uint16_t*>(px + b) = uint16_t(0);
        } else {
            for (int b = tailBegin; b < tailEnd; ++b) px[b] = uint8_t(0);
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
// that fall on a half2 of the internal layout are written as one dword.  PLAIN as above.
template <int FORMAT, bool PLAIN>
__global__ void __launch_bounds__(256)
write_channels_kernel(WriteChannelsArgs a)
{
    constexpr int BPC = bytes_per_channel(FORMAT), PER = 16 / BPC;
    __shared__ float unorm8Table[FORMAT == NTC_HIP_DEV_FORMAT_UNORM8 ? 256 : 1];
    if constexpr (FORMAT == NTC_HIP_DEV_FORMAT_UNORM8) {     // one correctly rounded division per code instead of per channel
        unorm8Table[threadIdx.x & 255] = float(threadIdx.x & 255) / 255.f;
        __syncthreads();
    }
    CopyGrid const at(a.xShift);
    int const x = at.x, y = at.y;
    if (x >= a.width || y >= a.height) return;
    int const srcY = a.verticalFlip ? a.height - 1 - y : y;          // SetupBilinearFilter flips the read position
    uint8_t const* px = a.src + size_t(srcY) * a.rowPitch + size_t(x) * a.pixelStride;
    uint16_t* dst = a.planarPairs + size_t(y) * size_t(a.width) * size_t(a.setChannels) + size_t(x) * 2;
    uint32_t pending = 0;                                            // low half of a pair waiting for its partner
#pragma unroll
    for (int piece = 0; piece < NTC_HIP_DEV_MAX_CHANNELS / PER; ++piece) {
        int const base = piece * PER;
        if (base >= a.numChannels) break;                            // uniform
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
            float v = decode_channel<FORMAT>(words, k, unorm8Table);
            if constexpr (!PLAIN) v = encode_color_space(a.dstColorSpaces[ch], decode_color_space(a.srcColorSpaces[ch], v));
            v = fmaxf(-65504.f, fminf(65504.f, v));                  // WriteImageChannel FLOAT16, src/ImageProcessing.cu:154-156
            asm volatile("" : "+v"(v));
            uint32_t const half = __builtin_bit_cast(uint16_t, (_Float16)v);
            int const c = a.firstChannel + ch;
            uint16_t* const to = dst + size_t(c & ~1) * size_t(a.width);
            if ((c & 1) == 0) {
                if (ch + 1 < a.numChannels) pending = half;          // partner follows: store both together
                else to[0] = uint16_t(half);
            } else {
                if (ch > 0) *reinterpret_cast<uint32_t*>(to) = pending | (half << 16);
                else to[1] = uint16_t(half);
            }
        }
    }
}

// ---- resampling copies (src/ImageProcessing.cu:24-72: SetupBilinearFilter) -------------------------
//
// The position of destination pixel (x, y) in the source is ((x + 1/2) / dstW) * srcW - 1/2, clamped
// to the source image; the four taps around it are weighted bilinearly, and a tap whose weight is
// zero is not used (at the right and bottom edges it would lie outside the image; here its index is
// clamped and its value dropped).  The blend is a * w0 + b * w1 + c * w2 + d * w3 evaluated as one
// multiply and three fused multiply-adds, which is what the reference's compiler makes of that
// expression.  These kernels are general rather than fast: one lane per destination pixel, one
// channel at a time.
struct BilinearTaps { int x0, y0, x1, y1; float w[4]; };

__device__ __forceinline__ BilinearTaps setup_bilinear(int srcW, int srcH, int dstW, int dstH, int x, int y)
{
    if (srcW == dstW && srcH == dstH) return BilinearTaps{ x, y, x, y, { 1.f, 0.f, 0.f, 0.f } };   // the reference's 1:1 shortcut
    float const u = (float(x) + 0.5f) / float(dstW), v = (float(y) + 0.5f) / float(dstH);
    float const px = fmaxf(0.f, fminf(float(srcW) - 1.f, u * float(srcW) - 0.5f));
    float const py = fmaxf(0.f, fminf(float(srcH) - 1.f, v * float(srcH) - 0.5f));
    float const fx = px - floorf(px), fy = py - floorf(py);
    BilinearTaps t;
    t.x0 = int(floorf(px)); t.y0 = int(floorf(py));
    t.x1 = min(t.x0 + 1, srcW - 1); t.y1 = min(t.y0 + 1, srcH - 1);
    t.w[0] = (1.f - fx) * (1.f - fy); t.w[1] = fx * (1.f - fy); t.w[2] = (1.f - fx) * fy; t.w[3] = fx * fy;
    return t;
}

__device__ __forceinline__ float blend_taps(BilinearTaps const& t, float a, float b, float c, float d)
{
    a = t.w[0] > 0.f ? a : 0.f; b = t.w[1] > 0.f ? b : 0.f; c = t.w[2] > 0.f ? c : 0.f; d = t.w[3] > 0.f ? d : 0.f;
    return __builtin_fmaf(d, t.w[3], __builtin_fmaf(c, t.w[2], __builtin_fmaf(b, t.w[1], a * t.w[0])));
}

__device__ __forceinline__ float planar_half(uint16_t const* image, int width, int setChannels, int x, int y, int c)
{
    uint16_t const bits = image[size_t(y) * size_t(width) * size_t(setChannels) + size_t(c & ~1) * size_t(width) + size_t(x) * 2 + size_t(c & 1)];
    return float(__builtin_bit_cast(_Float16, bits));
}

// Channel `k` of a pixel of the user image, any format and alignment the format allows.
__device__ __forceinline__ float user_channel(uint8_t const* px, int format, int k)
{
    switch (format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  return float(px[k]) / 255.f;
    case NTC_HIP_DEV_FORMAT_UNORM16: return float(reinterpret_cast<uint16_t const*>(px)[k]) / 65535.f;
    case NTC_HIP_DEV_FORMAT_FLOAT16: return float(reinterpret_cast<_Float16 const*>(px)[k]);
    case NTC_HIP_DEV_FORMAT_FLOAT32: return reinterpret_cast<float const*>(px)[k];
    default:                         return float(reinterpret_cast<uint32_t const*>(px)[k]);
    }
}

__device__ __forceinline__ uint16_t stored_half(float v)     // WriteImageChannel FLOAT16, src/ImageProcessing.cu:154-156
{
    v = fmaxf(-65504.f, fminf(65504.f, v));
    asm volatile("" : "+v"(v));
    return __builtin_bit_cast(uint16_t, (_Float16)v);
}

template <int FORMAT>
__global__ void __launch_bounds__(256)
read_channels_resize_kernel(ReadChannelsArgs a)
{
    constexpr int BPC = bytes_per_channel(FORMAT);
    int const x = blockIdx.x * 64 + (threadIdx.x & 63), y = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (x >= a.dstWidth || y >= a.dstHeight) return;
    BilinearTaps const t = setup_bilinear(a.width, a.height, a.dstWidth, a.dstHeight, x, y);
    uint8_t* const px = a.dst + size_t(y) * a.rowPitch + size_t(x) * a.pixelStride;
    DitherRng rng(uint32_t(x) + uint32_t(y) * uint32_t(a.dstWidth));
    for (int ch = 0; ch < a.dstChannels; ++ch) {
        float value;
        if (ch < a.numChannels) {
            int const c = a.firstChannel + ch, space = a.srcColorSpaces[ch];
            value = blend_taps(t, decode_color_space(space, planar_half(a.planarPairs, a.width, a.setChannels, t.x0, t.y0, c)),
                                  decode_color_space(space, planar_half(a.planarPairs, a.width, a.setChannels, t.x1, t.y0, c)),
                                  decode_color_space(space, planar_half(a.planarPairs, a.width, a.setChannels, t.x0, t.y1, c)),
                                  decode_color_space(space, planar_half(a.planarPairs, a.width, a.setChannels, t.x1, t.y1, c)));
        } else {
            value = (ch == 3) ? 1.f : 0.f;
        }
        float const dither = a.useDithering ? rng.next_float() - 0.5f : 0.f;
        uint32_t const bits = encode_channel<FORMAT>(ch < 16 ? a.dstColorSpaces[ch] : 0, value, a.useDithering != 0, dither);
        if constexpr (BPC == 1) px[ch] = uint8_t(bits);
        else if constexpr (BPC == 2) reinterpret_cast<uint16_t*>(px)[ch] = uint16_t(bits);
        else reinterpret_cast<uint32_t*>(px)[ch] = bits;
    }
}

__global__ void __launch_bounds__(256)
write_channels_resize_kernel(WriteChannelsArgs a)
{
    int const x = blockIdx.x * 64 + (threadIdx.x & 63), y = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (x >= a.width || y >= a.height) return;
    BilinearTaps const t = setup_bilinear(a.srcWidth, a.srcHeight, a.width, a.height, x, a.verticalFlip ? a.height - 1 - y : y);
    uint8_t const* const p00 = a.src + size_t(t.y0) * a.rowPitch + size_t(t.x0) * a.pixelStride;
    uint8_t const* const p10 = a.src + size_t(t.y0) * a.rowPitch + size_t(t.x1) * a.pixelStride;
    uint8_t const* const p01 = a.src + size_t(t.y1) * a.rowPitch + size_t(t.x0) * a.pixelStride;
    uint8_t const* const p11 = a.src + size_t(t.y1) * a.rowPitch + size_t(t.x1) * a.pixelStride;
    uint16_t* const dst = a.planarPairs + size_t(y) * size_t(a.width) * size_t(a.setChannels) + size_t(x) * 2;
    for (int ch = 0; ch < a.numChannels; ++ch) {
        int const space = a.srcColorSpaces[ch];
        float const value = blend_taps(t, decode_color_space(space, user_channel(p00, a.format, ch)), decode_color_space(space, user_channel(p10, a.format, ch)),
                                          decode_color_space(space, user_channel(p01, a.format, ch)), decode_color_space(space, user_channel(p11, a.format, ch)));
        int const c = a.firstChannel + ch;
        dst[size_t(c & ~1) * size_t(a.width) + size_t(c & 1)] = stored_half(encode_color_space(a.dstColorSpaces[ch], value));
    }
}

// ResizeMultichannelImageKernel (src/ImageProcessing.cu:178-207): every channel of one image of the
// internal layout resampled into another; a channel pair is read as dwords and written as one.
struct ResizePlanarArgs {
    uint16_t const* src; uint16_t* dst;
    int32_t srcWidth, srcHeight, dstWidth, dstHeight, setChannels;
    uint8_t colorSpaces[16];
};

__global__ void __launch_bounds__(256)
resize_planar_kernel(ResizePlanarArgs a)
{
    int const x = blockIdx.x * 64 + (threadIdx.x & 63), y = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (x >= a.dstWidth || y >= a.dstHeight) return;
    BilinearTaps const t = setup_bilinear(a.srcWidth, a.srcHeight, a.dstWidth, a.dstHeight, x, y);
    size_t const srcRow = size_t(a.srcWidth) * size_t(a.setChannels), pairStride = size_t(a.srcWidth) * 2;
    uint16_t const* const r0 = a.src + size_t(t.y0) * srcRow;
    uint16_t const* const r1 = a.src + size_t(t.y1) * srcRow;
    uint32_t* const out = reinterpret_cast<uint32_t*>(a.dst + size_t(y) * size_t(a.dstWidth) * size_t(a.setChannels) + size_t(x) * 2);
    for (int p = 0; p < a.setChannels / 2; ++p) {
        uint32_t const v00 = *reinterpret_cast<uint32_t const*>(r0 + p * pairStride + size_t(t.x0) * 2);
        uint32_t const v10 = *reinterpret_cast<uint32_t const*>(r0 + p * pairStride + size_t(t.x1) * 2);
        uint32_t const v01 = *reinterpret_cast<uint32_t const*>(r1 + p * pairStride + size_t(t.x0) * 2);
        uint32_t const v11 = *reinterpret_cast<uint32_t const*>(r1 + p * pairStride + size_t(t.x1) * 2);
        uint32_t packed = 0;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            int const space = a.colorSpaces[2 * p + k];
            auto half_of = [&](uint32_t v) { return decode_color_space(space, float(__builtin_bit_cast(_Float16, uint16_t(v >> (16 * k))))); };
            float const value = blend_taps(t, half_of(v00), half_of(v10), half_of(v01), half_of(v11));
            packed |= uint32_t(stored_half(encode_color_space(space, value))) << (16 * k);
        }
        out[size_t(p) * size_t(a.dstWidth)] = packed;
    }
}

hipError_t launch_resize_planar(uint16_t const* src, int srcWidth, int srcHeight, uint16_t* dst, int dstWidth, int dstHeight,
                                int setChannels, uint8_t const* colorSpaces, hipStream_t stream)
{
    ResizePlanarArgs a{};
    a.src = src; a.dst = dst; a.srcWidth = srcWidth; a.srcHeight = srcHeight; a.dstWidth = dstWidth; a.dstHeight = dstHeight; a.setChannels = setChannels;
    for (int i = 0; i < 16; ++i) a.colorSpaces[i] = colorSpaces ? colorSpaces[i] : 0;
    hipLaunchKernelGGL(resize_planar_kernel, dim3((dstWidth + 63) / 64, (dstHeight + 3) / 4), dim3(256), 0, stream, a);
    return hipGetLastError();
}

static bool plain_copy(uint8_t const* srcSpaces, uint8_t const* dstSpaces, int useDithering)
{
    bool plain = useDithering == 0;
    for (int i = 0; i < 16; ++i) plain = plain && srcSpaces[i] == 0 && dstSpaces[i] == 0;
    return plain;
}

template <int FORMAT>
static void launch_write_format(WriteChannelsArgs const& a, dim3 grid, bool plain, hipStream_t stream)
{
    if (plain) hipLaunchKernelGGL((write_channels_kernel<FORMAT, true>), grid, dim3(256), 0, stream, a);
    else       hipLaunchKernelGGL((write_channels_kernel<FORMAT, false>), grid, dim3(256), 0, stream, a);
}

hipError_t launch_write_channels(WriteChannelsArgs const& args, hipStream_t stream)
{
    WriteChannelsArgs a = args;
    if (a.srcWidth > 0) {                                    // resampling copy
        hipLaunchKernelGGL(write_channels_resize_kernel, dim3((a.width + 63) / 64, (a.height + 3) / 4), dim3(256), 0, stream, a);
        return hipGetLastError();
    }
    dim3 const grid = copy_grid(a.width, a.height, a.xShift, false);
    bool const plain = plain_copy(a.srcColorSpaces, a.dstColorSpaces, 0);
    switch (a.format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  launch_write_format<NTC_HIP_DEV_FORMAT_UNORM8>(a, grid, plain, stream); break;
    case NTC_HIP_DEV_FORMAT_UNORM16: launch_write_format<NTC_HIP_DEV_FORMAT_UNORM16>(a, grid, plain, stream); break;
    case NTC_HIP_DEV_FORMAT_FLOAT16: launch_write_format<NTC_HIP_DEV_FORMAT_FLOAT16>(a, grid, plain, stream); break;
    case NTC_HIP_DEV_FORMAT_FLOAT32: launch_write_format<NTC_HIP_DEV_FORMAT_FLOAT32>(a, grid, plain, stream); break;
    case NTC_HIP_DEV_FORMAT_UINT32:  launch_write_format<NTC_HIP_DEV_FORMAT_UINT32>(a, grid, plain, stream); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// Per-channel sum of squared differences between a decoded mip and its reference image, both in the
// internal layout: the loss branch of InferenceKernel (src/Inference.cu:77-118) as a pass of its own.
// MASKED (maskChannel >= 0): the decoded mask channel is first clamped to [0, 1] and stored back
// clamped (Inference.cu:96-97,112; a negative zero becomes +0 as the device max() of the reference
// returns), and with discardMaskedOut a texel whose REFERENCE mask value is zero counts on the mask
// channel only (Inference.cu:80-84,107-108).
// A lane takes PX adjacent texels (2 when the width is even: 8-byte loads) of kLossRowsPerWave rows; all
// loads of a row are issued before its arithmetic.  Squares are fp32 as in the reference; their sum over the
// lane's texels of a row goes into a double accumulator, and the workgroup writes 16 double partial sums
// (channel-major, so that the second stage reads them coalesced); ReduceLoss likewise finishes in
// double (src/Optimizer.cu:382-387).
template <int PX, bool MASKED>
__global__ void __launch_bounds__(256)
image_loss_kernel(uint16_t* __restrict__ a, uint16_t const* __restrict__ b, int width, int height, int setChannels,
                  uint32_t validChannelMask, int maskChannel, int discardMaskedOut, double* __restrict__ partials)
{
    constexpr int PAIRS = NTC_HIP_DEV_MAX_CHANNELS / 2;
    __shared__ double sums[4][NTC_HIP_DEV_MAX_CHANNELS];
    int const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int const x = (blockIdx.x * 64 + lane) * PX;
    int const pairs = setChannels >> 1;
    double acc[NTC_HIP_DEV_MAX_CHANNELS];
#pragma unroll
    for (int c = 0; c < NTC_HIP_DEV_MAX_CHANNELS; ++c) acc[c] = 0.0;
    for (int r = 0; r < kLossRowsPerWave; ++r) {
        int const y = (blockIdx.y * 4 + wave) * kLossRowsPerWave + r;
        if (x >= width || y >= height) continue;             // width is a multiple of PX
        size_t const base = size_t(y) * size_t(width) * size_t(setChannels) + size_t(x) * 2;
        uint32_t va[PAIRS][PX], vb[PAIRS][PX];
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
            // no branch around a load (the loads of a row must all be in flight together): pairs the
            // set does not have re-read its last pair, and their sums are dropped at the end
            size_t const at = base + size_t(2 * min(p, pairs - 1)) * size_t(width);
            if constexpr (PX == 2) {
                uint2 const u = *reinterpret_cast<uint2 const*>(a + at), v = *reinterpret_cast<uint2 const*>(b + at);
                va[p][0] = u.x; va[p][1] = u.y; vb[p][0] = v.x; vb[p][1] = v.y;
            } else {
                va[p][0] = *reinterpret_cast<uint32_t const*>(a + at);
                vb[p][0] = *reinterpret_cast<uint32_t const*>(b + at);
            }
        }
        __builtin_amdgcn_sched_barrier(0);                   // keep the loads ahead of the arithmetic
        [[maybe_unused]] bool maskedOut[PX];
        if constexpr (MASKED) {
#pragma unroll
            for (int k = 0; k < PX; ++k) maskedOut[k] = false;
#pragma unroll
            for (int p = 0; p < PAIRS; ++p) {
                if ((maskChannel >> 1) != p || !discardMaskedOut) continue;          // uniform
#pragma unroll
                for (int k = 0; k < PX; ++k) maskedOut[k] = (((maskChannel & 1) ? vb[p][k] >> 16 : vb[p][k]) & 0x7FFFu) == 0;
            }
        }
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int k = 0; k < PX; ++k) {
                float a0 = float(__builtin_bit_cast(_Float16, uint16_t(va[p][k])));
                float a1 = float(__builtin_bit_cast(_Float16, uint16_t(va[p][k] >> 16)));
                if constexpr (MASKED) {
                    if ((maskChannel >> 1) == p) {              // uniform; the mask channel is below setChannels
                        if (maskChannel & 1) a1 = a1 > 0.f ? fminf(a1, 1.f) : 0.f;
                        else                 a0 = a0 > 0.f ? fminf(a0, 1.f) : 0.f;
                        uint32_t const clamped = uint32_t(__builtin_bit_cast(uint16_t, _Float16(a0)))
                                               | uint32_t(__builtin_bit_cast(uint16_t, _Float16(a1))) << 16;
                        if (clamped != va[p][k]) *reinterpret_cast<uint32_t*>(a + base + size_t(2 * p) * size_t(width) + size_t(2 * k)) = clamped;
                    }
                }
                float d0 = a0 - float(__builtin_bit_cast(_Float16, uint16_t(vb[p][k])));
                float d1 = a1 - float(__builtin_bit_cast(_Float16, uint16_t(vb[p][k] >> 16)));
                if constexpr (MASKED) {
                    if (maskedOut[k] && maskChannel != 2 * p) d0 = 0.f;
                    if (maskedOut[k] && maskChannel != 2 * p + 1) d1 = 0.f;
                }
                s0 += d0 * d0;
                s1 += d1 * d1;
            }
            acc[2 * p] += double(s0);
            acc[2 * p + 1] += double(s1);
        }
    }
#pragma unroll
    for (int c = 0; c < NTC_HIP_DEV_MAX_CHANNELS; ++c) {
        double v = (c < setChannels && ((validChannelMask >> c) & 1u)) ? acc[c] : 0.0;
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
// (thread t takes entries t, t + 256, ... into four interleaved sub-totals; then one thread adds the
// 256 thread totals), and writes the total behind the partials.
__global__ void __launch_bounds__(256)
image_loss_reduce_kernel(double const* __restrict__ partials, size_t blocks, double* __restrict__ totals)
{
    __shared__ double sums[256];
    double const* const mine = partials + size_t(blockIdx.x) * blocks;
    double acc[4] = { 0.0, 0.0, 0.0, 0.0 };
    size_t b = threadIdx.x;
    for (; b + 768 < blocks; b += 1024) {
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[k] += mine[b + size_t(k) * 256];
    }
#pragma unroll
    for (int k = 0; k < 3; ++k)
        if (b + size_t(k) * 256 < blocks) acc[k] += mine[b + size_t(k) * 256];
    sums[threadIdx.x] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    __syncthreads();
    if (threadIdx.x == 0) {
        double total = 0.0;
        for (int t = 0; t < 256; ++t) total += sums[t];
        totals[blockIdx.x] = total;
    }
}

hipError_t launch_image_loss(uint16_t* a, uint16_t const* b, int width, int height, int setChannels,
                             uint32_t validChannelMask, int maskChannel, int discardMaskedOut, double* partials, hipStream_t stream)
{
    dim3 const grid = image_loss_grid(width, height);
    size_t const blocks = size_t(grid.x) * size_t(grid.y);
    bool const two = (width & 1) == 0, masked = maskChannel >= 0;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, a, b, width, height, setChannels, validChannelMask,
                           maskChannel, discardMaskedOut, partials);
    };
    if (two) { if (masked) launch(image_loss_kernel<2, true>); else launch(image_loss_kernel<2, false>); }
    else     { if (masked) launch(image_loss_kernel<1, true>); else launch(image_loss_kernel<1, false>); }
    hipLaunchKernelGGL(image_loss_reduce_kernel, dim3(NTC_HIP_DEV_MAX_CHANNELS), dim3(256), 0, stream, partials, blocks, partials + blocks * NTC_HIP_DEV_MAX_CHANNELS);
    return hipGetLastError();
}

// ---- image difference (src/shaders/ImageDifference.hlsl) -------------------------------------------
//
// A workgroup covers 64 x 64 pixels of the extent, as the reference's does (16 x 16 threads of 4 x 4
// pixels); here lane = column and each wave walks 16 rows, so that the loads of a wave are one
// contiguous row piece.  Every thread adds its 16 squared differences in row order, the 64 lanes
// of a wave are combined by an xor butterfly (offsets 32 ... 1), the four waves in order.  Squares
// and sums are separate fp32 operations (no fused multiply-add).  The workgroup's sums are divided
// by width * height, scaled by 2^16, split into floor and fraction * 2^32 and added to the 64-bit
// accumulators (ImageDifference.hlsl:103-127; the integer atomics make the total independent of
// the order in which workgroups finish).
__device__ __forceinline__ float diff_channel(DiffImageArgs const& im, uint8_t const* px, int c)
{
    if (c >= im.numChannels) return c == 3 ? 1.f : 0.f;
    switch (im.format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  return float(px[c]) / 255.f;
    case NTC_HIP_DEV_FORMAT_UNORM16: return float(reinterpret_cast<uint16_t const*>(px)[c]) / 65535.f;
    case NTC_HIP_DEV_FORMAT_FLOAT16: return float(reinterpret_cast<_Float16 const*>(px)[c]);
    case NTC_HIP_DEV_FORMAT_FLOAT32: return reinterpret_cast<float const*>(px)[c];
    default:                         return float(reinterpret_cast<uint32_t const*>(px)[c]);
    }
}

__global__ void __launch_bounds__(256)
image_difference_kernel(ImageDifferenceArgs a)
{
    __shared__ float sums[4][4];
    int const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int const x = blockIdx.x * 64 + lane;
    float mse[4] = { 0.f, 0.f, 0.f, 0.f };
    for (int r = 0; r < 16; ++r) {
        int const y = blockIdx.y * 64 + wave * 16 + r;
        if (x >= a.width || y >= a.height) continue;
        uint8_t const* const pa = a.a.data + size_t(y + a.top) * a.a.rowPitch + size_t(x + a.left) * a.a.pixelStride;
        uint8_t const* const pb = a.b.data + size_t(y + a.top) * a.b.rowPitch + size_t(x + a.left) * a.b.pixelStride;
        float t1[4], t2[4], diff[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) { t1[c] = diff_channel(a.a, pa, c); t2[c] = diff_channel(a.b, pb, c); }
#pragma unroll
        for (int c = 0; c < 4; ++c)
            diff[c] = a.useMSLE ? __fsub_rn(logf(fabsf(t1[c]) + 1.f), logf(fabsf(t2[c]) + 1.f)) : __fsub_rn(t1[c], t2[c]);
        if (a.useAlphaThreshold && t1[3] < a.alphaThreshold && t2[3] < a.alphaThreshold) { diff[0] = 0.f; diff[1] = 0.f; diff[2] = 0.f; }
#pragma unroll
        for (int c = 0; c < 4; ++c) mse[c] = __fadd_rn(mse[c], __fmul_rn(diff[c], diff[c]));
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float v = mse[c];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) v = __fadd_rn(v, __shfl_xor(v, off, 64));
        if (lane == 0) sums[wave][c] = v;
    }
    __syncthreads();
    if (threadIdx.x < 4) {
        int const c = threadIdx.x;
        float total = __fadd_rn(__fadd_rn(__fadd_rn(sums[0][c], sums[1][c]), sums[2][c]), sums[3][c]);
        total = __fdiv_rn(total, float(a.width * a.height));
        total = __fmul_rn(total, 65536.f);
        float const whole = floorf(total);
        // float -> uint32 conversions saturate; a NaN (from NaN pixels) adds nothing
        unsigned long long const high = uint32_t(whole), low = uint32_t(floorf(__fmul_rn(__fsub_rn(total, whole), 4294967296.f)));
        unsigned long long const fixed = (high << 32) | low;
        if (fixed) atomicAdd(a.output + c, fixed);
    }
}

hipError_t launch_image_difference(ImageDifferenceArgs const& a, hipStream_t stream)
{
    dim3 const grid((a.width + 63) / 64, (a.height + 63) / 64);
    hipLaunchKernelGGL(image_difference_kernel, grid, dim3(256), 0, stream, a);
    return hipGetLastError();
}

template <int FORMAT>
static void launch_read_format(ReadChannelsArgs const& a, dim3 grid, bool plain, hipStream_t stream)
{
    if (plain) hipLaunchKernelGGL((read_channels_kernel<FORMAT, true>), grid, dim3(256), 0, stream, a);
    else       hipLaunchKernelGGL((read_channels_kernel<FORMAT, false>), grid, dim3(256), 0, stream, a);
}

hipError_t launch_read_channels(ReadChannelsArgs const& args, hipStream_t stream)
{
    ReadChannelsArgs a = args;
    if (a.dstWidth > 0) {                                    // resampling copy
        dim3 const grid((a.dstWidth + 63) / 64, (a.dstHeight + 3) / 4);
        switch (a.format) {
        case NTC_HIP_DEV_FORMAT_UNORM8:  hipLaunchKernelGGL(read_channels_resize_kernel<NTC_HIP_DEV_FORMAT_UNORM8>, grid, dim3(256), 0, stream, a); break;
        case NTC_HIP_DEV_FORMAT_UNORM16: hipLaunchKernelGGL(read_channels_resize_kernel<NTC_HIP_DEV_FORMAT_UNORM16>, grid, dim3(256), 0, stream, a); break;
        case NTC_HIP_DEV_FORMAT_FLOAT16: hipLaunchKernelGGL(read_channels_resize_kernel<NTC_HIP_DEV_FORMAT_FLOAT16>, grid, dim3(256), 0, stream, a); break;
        case NTC_HIP_DEV_FORMAT_FLOAT32: hipLaunchKernelGGL(read_channels_resize_kernel<NTC_HIP_DEV_FORMAT_FLOAT32>, grid, dim3(256), 0, stream, a); break;
        case NTC_HIP_DEV_FORMAT_UINT32:  hipLaunchKernelGGL(read_channels_resize_kernel<NTC_HIP_DEV_FORMAT_UINT32>, grid, dim3(256), 0, stream, a); break;
        default: return hipErrorInvalidValue;
        }
        return hipGetLastError();
    }
    dim3 const grid = copy_grid(a.width, a.height, a.xShift);
    bool const plain = plain_copy(a.srcColorSpaces, a.dstColorSpaces, a.useDithering);
    switch (a.format) {
    case NTC_HIP_DEV_FORMAT_UNORM8:  launch_read_format<NTC_HIP_DEV_FORMAT_UNORM8>(a, grid, plain, stream); break;
    case NTC_HIP_DEV_FORMAT_UNORM16: launch_read_format<NTC_HIP_DEV_FORMAT_UNORM16>(a, grid, plain, stream); break;
    case NTC_HIP_DEV_FORMAT_FLOAT16: launch_read_format<NTC_HIP_DEV_FORMAT_FLOAT16>(a, grid, plain, stream); break;
    case NTC_HIP_DEV_FORMAT_FLOAT32: launch_read_format<NTC_HIP_DEV_FORMAT_FLOAT32>(a, grid, plain, stream); break;
    case NTC_HIP_DEV_FORMAT_UINT32:  launch_read_format<NTC_HIP_DEV_FORMAT_UINT32>(a, grid, plain, stream); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Byte fill (what a memset does, as a kernel: the library clears memory only this way).  The
// 16-byte-aligned middle goes out as uint4 stores, the unaligned ends byte by byte.
__global__ void __launch_bounds__(256)
fill_kernel(uint8_t* dst, uint32_t pattern, uint64_t headBytes, uint64_t vectors, uint64_t tailBytes)
{
    uint64_t const stride = uint64_t(gridDim.x) * blockDim.x, first = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    uint4* const body = reinterpret_cast<uint4*>(dst + headBytes);
    for (uint64_t i = first; i < vectors; i += stride) body[i] = make_uint4(pattern, pattern, pattern, pattern);
    if (first < headBytes) dst[first] = uint8_t(pattern);
    if (first < tailBytes) dst[headBytes + vectors * 16u + first] = uint8_t(pattern);
}

hipError_t launch_fill(uint8_t* dst, uint8_t value, uint64_t bytes, hipStream_t stream)
{
    if (bytes == 0) return hipSuccess;
    uint64_t const misaligned = reinterpret_cast<uintptr_t>(dst) & 15u;
    uint64_t const headBytes = misaligned ? (16u - misaligned < bytes ? 16u - misaligned : bytes) : 0u;
    uint64_t const vectors = (bytes - headBytes) / 16u, tailBytes = bytes - headBytes - vectors * 16u;
    uint64_t const groups = (vectors + 255u) / 256u;
    uint32_t const grid = uint32_t(groups < 1u ? 1u : (groups > 16384u ? 16384u : groups));
    hipLaunchKernelGGL(fill_kernel, dim3(grid), dim3(256), 0, stream, dst, uint32_t(value) * 0x01010101u, headBytes, vectors, tailBytes);
    return hipGetLastError();
}

} // namespace ntc_hip_dev
