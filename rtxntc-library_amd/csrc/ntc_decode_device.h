// ntc_decode_device.h - device helpers shared by the decode kernels (int8 network: ntc_decode_kernel.hip,
// FP8 network: ntc_decode_fp8_kernel.hip): vector types, latent loads, the float sampling footprint, output
// conversion and the stores of one wave tile.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ntc_decode_kernel.h"

namespace ntc_hip_dev {

typedef int   v4i __attribute__((ext_vector_type(4)));
// Latent grids live in global memory; saying so lets loads use "scalar base + 32-bit lane offset"
// addressing instead of 64-bit flat addresses built per lane.
typedef __attribute__((address_space(1))) uint16_t const* GlobalU16Ptr;
typedef __attribute__((address_space(1))) uint8_t const*  GlobalU8Ptr;

// One u16 at a uniform base plus a 32-bit byte offset per lane (global_load_ushort v, v_off, s[base]).
__device__ __forceinline__ uint32_t load_u16(GlobalU8Ptr base, uint32_t byteOffset)
{
    return *reinterpret_cast<GlobalU16Ptr>(base + byteOffset);
}

// 24-bit multiply, full rate.  Inline assembly because the compiler turns the builtin back into the
// quarter-rate 32-bit multiply in places.  Only for the input stages: the compiler inserts the wait states that
// matrix instructions in flight need around instructions it can see, and an assembly statement is opaque to it.
// The input stage of a tile runs when none is in flight - after the previous tile's results were read for
// its stores and before this tile's first matrix instruction, in a basic block of its own.
__device__ __forceinline__ uint32_t mul24(uint32_t a, uint32_t b)
{
    uint32_t r;
    asm("v_mul_u32_u24 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
// Footprint of one axis of a bilinear tap pair in integers, for power-of-two sizes: with
// p = u*grid - 1/2 = N / 2^n, N = ((2x+1) << shl) - (1 << sublog) (the packed axis word of DevMip),
// floor and fraction are a shift and a mask, and the two cells wrap by masking.
struct AxisFoot { uint32_t c0, c1, f; };

__device__ __forceinline__ AxisFoot axis_fast(int x, uint32_t packedAxis, int gridSize)
{
    int const shl = int(packedAxis & 0xffu), n = int((packedAxis >> 8) & 0xffu), sublog = int((packedAxis >> 16) & 0xffu);
    int const N = ((2 * x + 1) << shl) - (1 << sublog);
    int const b = N >> n;                                    // arithmetic shift = floor
    AxisFoot a;
    a.f = uint32_t(N) & ((1u << n) - 1u);
    a.c0 = uint32_t(b) & uint32_t(gridSize - 1);             // wrap addressing
    a.c1 = uint32_t(b + 1) & uint32_t(gridSize - 1);
    return a;
}

// 24-bit multiply-add, full rate: a * b + c.  Input stages only, like mul24.
__device__ __forceinline__ uint32_t mad24(uint32_t a, uint32_t b, uint32_t c)
{
    uint32_t r;
    asm("v_mad_u32_u24 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWaveTexels  = 64;

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
        // 0..255, integer-valued after the floor: the conversion is exact and drops the byte into its slot
        packed = __builtin_amdgcn_cvt_pk_u8_f32(floorf(t * codeScale), uint32_t(i), packed);
    }
    return packed ^ 0x80808080u;                            // -128 on every byte
}

typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float    v2f __attribute__((ext_vector_type(2)));

// Two network outputs -> two fp16 in one dword.  The output is an fp32 product that is THEN
// rounded to half (round-nearest-even); a half that would be Inf/NaN is stored as zero
// (IsHalfSpecial, Inference.cu:125-126).  |o| >= 65520 is exactly the set that rounds to
// Inf.  The empty asm keeps the compiler from folding multiply + convert into
// v_fma_mixlo_f16, which rounds the exact product once, straight to half.
// CHECKED = false is for callers that know |a|, |b| stay far below 65520.
template <bool CHECKED = true>
__device__ __forceinline__ uint32_t to_half2_bits(float a, float b)
{
    asm("" : "+v"(a));
    asm("" : "+v"(b));
    if constexpr (CHECKED) {
        a = (__builtin_fabsf(a) < 65520.f) ? a : 0.f;
        b = (__builtin_fabsf(b) < 65520.f) ? b : 0.f;
    }
    v2h const h = __builtin_convertvector(v2f{a, b}, v2h);
    return __builtin_bit_cast(uint32_t, h);
}

// WriteImageChannel UNORM8 (src/ImageProcessing.cu:146-149): u8(clamp(roundf(v * 255), 0, 255)) of
// the stored half.  v*255 is exact in fp32 (11-bit x 8-bit significands).  v_cvt_pk_u8_f32 rounds to nearest
// even and saturates to [0, 255]; that equals roundf (half away from zero) here because the only tie inside
// the range is v = 1/2 (v*255 = k + 1/2 needs 255 | 2k + 1 for a dyadic v): 127.5 -> 128 under both rules.
// The result drops into byte `slot` of `packed`.
__device__ __forceinline__ uint32_t pack_unorm8(_Float16 h, uint32_t slot, uint32_t packed)
{
    return __builtin_amdgcn_cvt_pk_u8_f32(float(h) * 255.f, slot, packed);
}

typedef __attribute__((address_space(1))) uint8_t* GlobalOutPtr;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// A uniform 64-bit address, pinned to scalar registers so that stores take the "scalar base + 32-bit lane
// offset" form instead of a 64-bit address computed per lane.
__device__ __forceinline__ GlobalOutPtr uniform_pointer(uint64_t address)
{
    uint32_t const lo = __builtin_amdgcn_readfirstlane(uint32_t(address));
    uint32_t const hi = __builtin_amdgcn_readfirstlane(uint32_t(address >> 32));
    return (GlobalOutPtr)((uint64_t(hi) << 32) | lo);
}

// Stores of one 16-texel block row.  `row` is uniform (start of image row y in the output), `laneOff` the
// lane's byte offset inside the row (`laneOff2` that of the second channel pair of planar output), h01/h23 the
// lane's four channels as halves.  `vectorStores` (uniform; RunMip) says that every lane's four channels of a
// pixel format start at a multiple of their size and can go out as one store; otherwise channels go out one by
// one (a per-lane look at the address as second chance cost every instantiation registers: 8 to 110 spilled).
template <int FORMAT>
__device__ __forceinline__ void store_channels(GlobalOutPtr row, uint32_t laneOff, uint32_t laneOff2,
                                               uint32_t h01, uint32_t h23, int nch, bool vectorStores)
{
    GlobalOutPtr const dst = row + laneOff;
    if constexpr (FORMAT == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS) {
        // src/RegressionKernels.h:36-45; whole half2 pairs (Inference.cu:131-134)
        *reinterpret_cast<__attribute__((address_space(1))) uint32_t*>(dst) = h01;
        if (nch > 2) *reinterpret_cast<__attribute__((address_space(1))) uint32_t*>(row + laneOff2) = h23;
    } else if constexpr (FORMAT == NTC_HIP_DEV_OUT_FP16_PIXELS) {
        if (nch == 4 && vectorStores) {
            *reinterpret_cast<__attribute__((address_space(1))) u32x2*>(dst) = u32x2{ h01, h23 };
        } else {
            uint32_t const h[4] = { h01 & 0xffffu, h01 >> 16, h23 & 0xffffu, h23 >> 16 };
            for (int r = 0; r < nch; ++r) reinterpret_cast<__attribute__((address_space(1))) uint16_t*>(dst)[r] = uint16_t(h[r]);
        }
    } else {
        v2h const a = __builtin_bit_cast(v2h, h01), b = __builtin_bit_cast(v2h, h23);
        uint32_t const u8 = pack_unorm8(b[1], 3, pack_unorm8(b[0], 2, pack_unorm8(a[1], 1, pack_unorm8(a[0], 0, 0u))));
        if (nch == 4 && vectorStores) {
            *reinterpret_cast<__attribute__((address_space(1))) uint32_t*>(dst) = u8;
        } else {
            for (int r = 0; r < nch; ++r) dst[r] = uint8_t(u8 >> (8 * r));
        }
    }
}

// What the tile loop and the stores need of a mip for every tile, held by value (in scalar registers) for a run
// of tiles of one mip; the input stages read the rest through `full`.
struct RunMip {
    DevMip const& full;
    uint8_t* out;
    uint64_t outRowPitch;
    int32_t width, height, numChannels, outPixelStride, outFormat;
    uint32_t fast;
    // Pixel formats: every lane's group of four channels (8 bytes of fp16, 4 of unorm8; the groups of a pixel
    // follow each other) starts at a multiple of its size - decided once here from the mip's start, row pitch and
    // pixel stride, not per lane and store from a 64-bit address (headline -0.4 %, batch of sets -0.9 %).
    bool vectorStores;
    __device__ __forceinline__ explicit RunMip(DevMip const& m)
        : full(m), out(m.out), outRowPitch(m.outRowPitch), width(m.width), height(m.height), numChannels(m.numChannels),
          outPixelStride(m.outPixelStride), outFormat(m.outFormat), fast(m.fast),
          vectorStores(((reinterpret_cast<uint64_t>(m.out) | m.outRowPitch | uint64_t(uint32_t(m.outPixelStride)))
                        & (m.outFormat == NTC_HIP_DEV_OUT_FP16_PIXELS ? 7u : 3u)) == 0) {}
};

// Look-ups in the table of a decode call (one entry per mip of every set, sorted by tileStart).  Both go through
// the table a wave at a time - one load per lane and a ballot - where a loop over the entries pays a memory round
// trip for each: a workgroup does this once per segment of its share, twelve entries further for a full mip chain.
// Every wave computes the same, uniform, result.  Used by decode_fp8_kernel (-0.6 % on a 4096 x 4096 decode);
// decode_kernel keeps the plain loops: there the same change took 1.3 % off a batch of eight sets and added
// 0.3 - 3 % to single sets, through the tile loop's register allocation.

// The last entry at or after `entry` whose tiles begin at or before `tile`.
__device__ __forceinline__ int table_entry_of(DevMip const* __restrict__ mips, int numMips, int entry, int tile)
{
    int const lane = threadIdx.x & 63;
    for (int base = entry + 1; base < numMips; base += 64) {
        int const k = base + lane;
        bool const before = k < numMips && mips[k].tileStart <= tile;
        int const n = __popcll(__ballot(before));
        entry += n;
        if (n < 64) break;
    }
    return entry;
}

// Where the tiles that use `blob` (the weights of entry `entry`) end: the first tile of the next entry with other
// weights, at most tileEnd.
__device__ __forceinline__ int segment_end(DevMip const* __restrict__ mips, int numMips, int entry, int tileEnd, uint8_t const* blob)
{
    int const lane = threadIdx.x & 63;
    for (int base = entry + 1; base < numMips; base += 64) {
        int const k = base + lane;
        int start = 0x7fffffff;
        bool other = false;
        if (k < numMips) { start = mips[k].tileStart; other = mips[k].weights != blob; }
        uint64_t const hit = __ballot(other || start >= tileEnd);       // another set's entry, or one beyond the share
        if (hit) return min(tileEnd, __builtin_amdgcn_readlane(start, __ffsll((unsigned long long)hit) - 1));
    }
    return tileEnd;
}

// What a lane's stores of one wave tile share: channel count, byte offsets inside an output row, row size.
template <int FORMAT, class Mip>
struct StorePlace {
    int nch;
    uint32_t laneOff, laneOff2;
    size_t rowBytes;
    __device__ __forceinline__ StorePlace(Mip const& m, int x, int chBase)
    {
        nch = (x < m.width) ? min(4, m.numChannels - chBase) : 0;
        uint32_t const C2 = uint32_t((m.numChannels + 1) & ~1);
        laneOff = (FORMAT == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS)
            ? (uint32_t(chBase) * uint32_t(m.width) + uint32_t(x) * 2u) * 2u
            : uint32_t(x) * uint32_t(m.outPixelStride) + uint32_t(chBase) * (FORMAT == NTC_HIP_DEV_OUT_FP16_PIXELS ? 2u : 1u);
        laneOff2 = laneOff + uint32_t(m.width) * 4u;
        rowBytes = (FORMAT == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS) ? size_t(m.width) * C2 * 2 : size_t(m.outRowPitch);
    }
};

// The lane's four channels of one texel of image row y (uniform, inside the image): outputs = accumulators times
// scales, rounded to half.
template <int FORMAT, bool CHECKED, class AccV, class Mip>
__device__ __forceinline__ void store_row(Mip const& m, StorePlace<FORMAT, Mip> const& at, AccV D, v4f S, int y)
{
    uint32_t const h01 = to_half2_bits<CHECKED>(float(D[0]) * S[0], float(D[1]) * S[1]);
    uint32_t const h23 = to_half2_bits<CHECKED>(float(D[2]) * S[2], float(D[3]) * S[3]);
    GlobalOutPtr const row = uniform_pointer(reinterpret_cast<uint64_t>(m.out) + size_t(y) * at.rowBytes);
    store_channels<FORMAT>(row, at.laneOff, at.laneOff2, h01, h23, at.nch, m.vectorStores);
}

// The stores of one wave tile: D[b] holds the lane's four channels of the texel in column `x` of block b, where block
// b of 16 texels begins 16 * (b & 1) texels further right, in row y0 + (b >> 1).
template <int FORMAT, bool CHECKED = true, class Acc, class Mip>
__device__ __forceinline__ void store_tile(Mip const& m, Acc const (&D)[4], v4f S, int x, int y0, int chBase)
{
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        int const y = y0 + (b >> 1);
        if (y >= m.height) break;                            // uniform
        StorePlace<FORMAT, Mip> const at(m, x + 16 * (b & 1), chBase);
        if (at.nch > 0) store_row<FORMAT, CHECKED>(m, at, D[b], S, y);
    }
}

// The stores of a wave tile at an image edge, of a mip with fewer than sixteen channels or of a pixel format that
// needs channel-by-channel stores: the general form above, in the mip's format, with the checked conversion (it
// equals the unchecked one wherever that is allowed).  Not inlined: tiles like these are few, and inlined next to
// the fast form the six instantiations cost the kernels registers.
template <class Acc>
__device__ __attribute__((noinline)) void store_tile_general(DevMip const* mip, Acc D0, Acc D1, Acc D2, Acc D3, v4f S, int x, int y0, int chBase)
{
    RunMip const m(*mip);
    Acc const D[4] = { D0, D1, D2, D3 };
    if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS)  store_tile<NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS, true>(m, D, S, x, y0, chBase);
    else if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PIXELS)   store_tile<NTC_HIP_DEV_OUT_FP16_PIXELS, true>(m, D, S, x, y0, chBase);
    else                                                   store_tile<NTC_HIP_DEV_OUT_UNORM8_PIXELS, true>(m, D, S, x, y0, chBase);
}

// The stores of a wave tile that lies inside the image of a mip whose channel count is a multiple of four (the common
// case): no bounds to test, every lane stores its four channels of all four blocks (block b: 16 texels from
// x0 + 16 * (b & 1) in row y0 + (b >> 1)), and the row addresses are one uniform
// base plus multiples of the row size - a handful of scalar additions instead of a 64-bit product, a test and a
// branch per row.  x0, y0: first texel of the wave tile; lane = (j, g) holds channels 4g..4g+3 of texel column j.
template <int FORMAT, bool CHECKED, class Acc, class Mip>
__device__ __forceinline__ void store_tile_inside(Mip const& m, Acc const (&D)[4], v4f S, int x0, int y0, int j, int g)
{
    typedef __attribute__((address_space(1))) uint32_t* DwordPtr;
    size_t rowBytes;
    uint32_t laneOff;
    GlobalOutPtr tile;
    if (4 * g >= m.numChannels) return;                                          // lanes of channel groups the mip does not have
    if constexpr (FORMAT == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS) {
        rowBytes = size_t(m.width) * size_t(m.numChannels) * 2;                  // fp16, a multiple of four channels
        laneOff = uint32_t(g) * (uint32_t(m.width) * 8u) + uint32_t(j) * 4u;     // (4g * width + 2j) halves
        tile = (GlobalOutPtr)m.out + (size_t(y0) * rowBytes + size_t(x0) * 4);
    } else {
        rowBytes = size_t(m.outRowPitch);
        laneOff = uint32_t(j) * uint32_t(m.outPixelStride) + uint32_t(g) * (FORMAT == NTC_HIP_DEV_OUT_FP16_PIXELS ? 8u : 4u);
        tile = (GlobalOutPtr)m.out + (size_t(y0) * rowBytes + size_t(x0) * size_t(m.outPixelStride));
    }
    uint32_t laneOff2 = laneOff + uint32_t(m.width) * 4u;                        // planar: the lane's second channel pair
    // The offsets stay 32-bit values of this tile (hoisted out of the tile loop they become 64-bit lane addresses, and
    // the stores lose their "scalar base + 32-bit lane offset" form).
    asm volatile("" : "+v"(laneOff), "+v"(laneOff2));
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        uint32_t const h01 = to_half2_bits<CHECKED>(float(D[b][0]) * S[0], float(D[b][1]) * S[1]);
        uint32_t const h23 = to_half2_bits<CHECKED>(float(D[b][2]) * S[2], float(D[b][3]) * S[3]);
        GlobalOutPtr const row = tile + size_t(b >> 1) * rowBytes
                               + ((b & 1) ? size_t(16) * (FORMAT == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS ? size_t(4) : size_t(m.outPixelStride)) : size_t(0));
        if constexpr (FORMAT == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS) {
            *reinterpret_cast<DwordPtr>(row + laneOff) = h01;
            *reinterpret_cast<DwordPtr>(row + laneOff2) = h23;
        } else if constexpr (FORMAT == NTC_HIP_DEV_OUT_FP16_PIXELS) {
            *reinterpret_cast<__attribute__((address_space(1))) u32x2*>(row + laneOff) = u32x2{ h01, h23 };
        } else {
            v2h const a = __builtin_bit_cast(v2h, h01), c = __builtin_bit_cast(v2h, h23);
            *reinterpret_cast<DwordPtr>(row + laneOff) = pack_unorm8(c[1], 3, pack_unorm8(c[0], 2, pack_unorm8(a[1], 1, pack_unorm8(a[0], 0, 0u))));
        }
    }
}

// One row of a wave tile in the mip's own format (checked conversion): the stores of the int8-only network path,
// which produces the wave's four blocks of 16 texels one after the other.
template <class AccV, class Mip>
__device__ __forceinline__ void store_row_any_format(Mip const& m, AccV D, v4f S, int x, int y, int chBase)
{
    if (y >= m.height) return;
    if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS) {
        StorePlace<NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS, Mip> const at(m, x, chBase);
        if (at.nch > 0) store_row<NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS, true>(m, at, D, S, y);
    } else if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PIXELS) {
        StorePlace<NTC_HIP_DEV_OUT_FP16_PIXELS, Mip> const at(m, x, chBase);
        if (at.nch > 0) store_row<NTC_HIP_DEV_OUT_FP16_PIXELS, true>(m, at, D, S, y);
    } else {
        StorePlace<NTC_HIP_DEV_OUT_UNORM8_PIXELS, Mip> const at(m, x, chBase);
        if (at.nch > 0) store_row<NTC_HIP_DEV_OUT_UNORM8_PIXELS, true>(m, at, D, S, y);
    }
}

// ---- random-access decode: pieces shared by the query kernels ----------------------------------

// Two adjacent u16 cells as one 32-bit load (2-byte aligned).
typedef uint32_t __attribute__((aligned(2))) u32_align2;
typedef __attribute__((address_space(1))) u32_align2 const* GlobalU32A2Ptr;

// The query-ordered copy of a grid: bricks of T x T cells (T = 4, or 8 for a one-layer grid),
// [brick row][brick column][cell row][cell column][layer], so that all layers of a cell are one load of 2, 4,
// 6 or 8 bytes and a 2 x 2 footprint usually lies in one or two cache lines.
typedef __attribute__((address_space(1))) u32x2 const* GlobalU32x2Ptr;

template <int LAYERS>
__device__ __forceinline__ uint32_t brick_offset(uint32_t cx, uint32_t cy, uint32_t log2GridWidth)
{
    constexpr uint32_t T = brick_side_log2(LAYERS), MASK = (1u << T) - 1u;
    uint32_t const lgBricksX = log2GridWidth > T ? log2GridWidth - T : 0u;
    uint32_t const brick = ((cy >> T) << lgBricksX) + (cx >> T);
    uint32_t const cell = ((cy & MASK) << T) + (cx & MASK);
    return brick * uint32_t(brick_bytes(LAYERS)) + cell * uint32_t(2 * LAYERS);     // below 2^32: a grid holds less than 2^31 bytes
}

// All layers of one cell: layer L in the low or high half of out[L / 2].
template <int LAYERS>
__device__ __forceinline__ void load_brick_cell(GlobalU8Ptr base, uint32_t off, uint32_t (&out)[2])
{
    out[0] = 0; out[1] = 0;
    if constexpr (LAYERS == 1) {
        out[0] = load_u16(base, off);
    } else if constexpr (LAYERS == 2) {
        out[0] = *reinterpret_cast<GlobalU32A2Ptr>(base + off);
    } else if constexpr (LAYERS == 3) {
        out[0] = *reinterpret_cast<GlobalU32A2Ptr>(base + off);
        out[1] = load_u16(base, off + 4u);
    } else {
        u32x2 const v = *reinterpret_cast<GlobalU32x2Ptr>(base + off);
        out[0] = v[0]; out[1] = v[1];
    }
}

// What a query needs of its mip, kept in LDS: every lane of a wave may address another mip, and
// fetching these fields per lane from the table in global memory put a long dependent load in
// front of the latent gathers.
struct QueryMip {
    uint16_t const* hr;
    uint16_t const* lr;
    uint32_t hrAxisX, hrAxisY, lrAxisX, lrAxisY;
    int32_t hrWidth, hrHeight, lrWidth, lrHeight;
    int32_t width, height;
    uint32_t posMask, fast;
    float positionLod;
    uint32_t pad[3];
    uint8_t const* hrBricks;
    uint8_t const* lrBricks;
};
static_assert(sizeof(QueryMip) == 96, "QueryMip layout");

} // namespace ntc_hip_dev
