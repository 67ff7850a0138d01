// ntc_decode_kernel.hip - texture-set decode for gfx950 (MI355X), int8 network.
//
// One persistent launch decodes every colour mip of every texture set handed to it.
// Work unit: a workgroup tile of 64x4 texels = four wave64 tiles of 32x2 texels (four blocks of 16 texels: two side
// by side in each of two rows, so that a wave writes whole 128-byte lines of a row).
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
#include "ntc_decode_device.h"
#include <type_traits>

namespace ntc_hip_dev {

// HGELU-clamp + requantise of four D values of one lane (Inference.hlsli:36-39,123-131,164-179).
// round-half-even of y*80 is taken from the low mantissa bits of y*80 + 1.5*2^23; the four low bytes are
// gathered with byte permutes and the "-113" (= +143 mod 256) is one add on all four bytes at once, with the
// carries kept inside each byte.  No inline assembly here: the compiler adds the wait states that matrix
// instructions in flight require only around instructions it can see.
__device__ __forceinline__ uint32_t activate4(v4i acc, v4f scale)
{
    uint32_t z[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float const x = float(acc[r]) * scale[r];
        float t = __builtin_fmaf(x, 0.333333f, 0.5f);
        t = fminf(fmaxf(t, 0.f), 1.f);
        float const y = fminf(x, 3.f) * t;
        z[r] = __builtin_bit_cast(uint32_t, y * 80.f + 12582912.f);     // low byte = rne(y*80) mod 256
    }
    uint32_t const lo = __builtin_amdgcn_perm(z[1], z[0], 0x0c0c0400u);  // bytes [z0.0, z1.0, 0, 0]
    uint32_t const hi = __builtin_amdgcn_perm(z[3], z[2], 0x04000c0cu);  // bytes [0, 0, z2.0, z3.0]
    uint32_t const p = lo | hi;
    // p + 0x8f8f8f8f byte by byte: low seven bits added with room for the carry, top bits combined by xor
    return ((p & 0x7f7f7f7fu) + 0x0f0f0f0fu) ^ (~p & 0x80808080u);
}

// ---- all-integer input stage (power-of-two mip and grid sizes) --------------------------
//
// With W and the grid size powers of two, u*Wg - 1/2 = ((2x+1)*2^e - 1)/2 with e = log2(Wg/W):
// floor and fraction are shifts and masks, the bilinear weights are small integers, and
// every float operation of the general path is exact, so both paths give the same bytes.

// Four 4-bit features of the four taps, filtered: ((17 * sum w*q) >> n) - 128 per byte; the weights w sum to 2^n
// (n <= 8).  A cell c = f0 | f1<<4 | f2<<8 | f3<<12 is spread to P = byte0 | byte1<<16 (16-bit lanes holding
// f0 + 16 f1 and f2 + 16 f3); E = P & 0x000f000f holds the even features alone.  S = sum w*P and T = sum w*E stay
// below 2^16 per lane (255 * 2^n), so lanes never mix, and (S - T) / 16 is sum w*f for the odd features, exactly.
// Times 17 (T + 16 T, and D/16 + D for the odd ones) is at most 17 * 15 * 2^8 < 2^16: still inside the lane.
__device__ __forceinline__ uint32_t bilinear4_int(uint32_t c00, uint32_t c10, uint32_t c01, uint32_t c11,
                                                  uint32_t w00, uint32_t w10, uint32_t w01, uint32_t w11, uint32_t n)
{
    uint32_t const m = 0x000f000fu;
    uint32_t const sel = 0x0c010c00u;                        // v_perm_b32: bytes [0, zero, 1, zero] of the cell
    uint32_t const p00 = __builtin_amdgcn_perm(0u, c00, sel), p10 = __builtin_amdgcn_perm(0u, c10, sel);
    uint32_t const p01 = __builtin_amdgcn_perm(0u, c01, sel), p11 = __builtin_amdgcn_perm(0u, c11, sel);
    uint32_t const S = mad24(w11, p11, mad24(w01, p01, mad24(w10, p10, mul24(w00, p00))));
    uint32_t const T = mad24(w11, p11 & m, mad24(w01, p01 & m, mad24(w10, p10 & m, mul24(w00, p00 & m))));
    uint32_t const D = S - T;                                // 16 * sum w*f of features 1 and 3
    uint32_t const ve = (((T << 4) + T) >> n) & 0x00ff00ffu; // features 0 and 2 in bytes 0 and 2
    uint32_t const vo = ((D + (D >> 4)) >> n) & 0x00ff00ffu; // 17 * (D / 16): features 1 and 3
    return (ve | (vo << 8)) ^ 0x80808080u;
}

// ---- decoder variants -----------------------------------------------------------------

template <int HR_MODE_, int HR_F_, int HR_BITS_, int HR_SLOTS_, int LR_F_, int LR_SLOTS_, int LOD_,
          int IN_, int H0_, int H1_, int H2_, bool FP8_WEIGHTS_ = false>
struct Variant {
    // e4m3 weights in the three hidden layers: each weight w is the integer 512*w (at most 18 bits
    // plus sign).  On the int8 matrix instruction it is split into three 6-bit planes,
    // 512*w = 4096*c2 + 64*c1 + c0, and a layer runs as three passes whose int32 results are recombined
    // exactly; on the fp16 matrix instruction (layers 1 and 2) into two planes, 512*w = 1024*hi + lo with
    // 0 <= lo < 1024, whose fp32 sums are exact integers and recombine with one fused multiply-add.
    static constexpr bool FP8_WEIGHTS = FP8_WEIGHTS_;
    static constexpr int PLANES = FP8_WEIGHTS_ ? 3 : 1;
    static constexpr int F16_PLANES = FP8_WEIGHTS_ ? 2 : 1;
    // Waves per workgroup: four (a quartet) cover one 64 x 4 tile.  A workgroup has two quartets around one copy
    // of the weights, two workgroups fit a CU (the e4m3 variants keep so many weight planes in LDS that no more
    // would fit anyway): four waves on every SIMD to overlap matrix and vector work.
    static constexpr int WAVES = 8;
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int RESIDENT = 2;                         // workgroups per CU
    static constexpr int WAVES_PER_SIMD = RESIDENT * WAVES / 4; // what the register budget is set for
    // Dwords per texel in the transpose buffer in front of the network: 16 + 4 of padding, or 12 without
    // padding for 48 inputs (rows then still start in distinct banks: 12 j mod 64 differ for j = 0..15).
    static constexpr int IN_STRIDE = (FP8_WEIGHTS_ && IN_ <= 48) ? 12 : 20;
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
    // Layers 1..3 can also run on the fp16 matrix instruction (see mlp_forward_f16).  Their A operands
    // then take, per output tile, one 1024-byte block for every pair of input tiles (K = 32) and one
    // 512-byte block for an odd last input tile (K = 16); sizes below are in 16-byte units.
    // (Layers 1 and 2 of an e4m3 variant hold F16_PLANES such sets of blocks, plane after plane.)
    static constexpr bool F16_LAYERS = true;
    static constexpr int f16_units(int inTiles) { return (inTiles / 2) * 64 + (inTiles % 2) * 32; }
    static constexpr int F16_L1 = 0;
    static constexpr int F16_L2 = F16_L1 + F16_PLANES * T1 * f16_units(T0);
    static constexpr int F16_L3 = F16_L2 + F16_PLANES * T2 * f16_units(T1);
    static constexpr int F16_END = F16_L3 + T3 * f16_units(T2);
    // The same layers as int8 tiles: [plane][tile of layers 1..3][lane], one 16-byte unit each.
    static constexpr int LATE_TILES = T1 + T2 + T3;
    static constexpr int LATE_INT8_UNITS = PLANES * LATE_TILES * 64;
    static constexpr int LATE_UNITS = F16_END > LATE_INT8_UNITS ? F16_END : LATE_INT8_UNITS;
    // A operands kept in `w`: layer 0 (the later layers live in `late`, as int8 or as fp16).
    static constexpr int W_TILES = T0;
    static constexpr int LATE_CHANNELS = H1 + H2 + OUT;
    static_assert(POS_BASE + 12 + LOD <= IN, "input vector does not fit");
    static_assert(IN % 16 == 0 && IN <= 64 && H0 <= 64 && H1 <= 64 && H2 <= 64, "layer widths");
    static_assert(HR_INPUTS % 4 == 0 && LR_INPUTS % 4 == 0, "grid blocks are dword aligned");
};

// Low part of the start value of two-plane fp16 layers ([M-tile][g][r] like `bias`): e4m3 variants only, so
// that the others keep their LDS footprint (the query kernel's is exactly a quarter of a CU's LDS).
template <bool ENABLED, int TILES> struct BiasLoT { float biasLo[TILES][4][4]; };
template <int TILES> struct BiasLoT<false, TILES> {};

template <class V>
struct alignas(16) LdsT : BiasLoT<V::FP8_WEIGHTS, V::NTILES> {
    uint32_t w[V::PLANES][V::W_TILES][64][4];  // int8 A operands: [plane][M-tile][lane][4 dwords]
    uint4    late[V::LATE_UNITS];              // A operands of layers 1..3: int8 tiles or fp16 blocks
    float    scale[V::NTILES][4][4];           // [M-tile][k-group g][r]  -> channel 16t+4g+r
    int32_t  bias[V::NTILES][4][4];
    uint32_t in[V::WAVES][kWaveTexels][V::IN_STRIDE];
    uint32_t lut2[256];               // byte of four 2-bit codes -> four input bytes 85*q - 128
    // Positional encoding for every power-of-two positionScale 2^-k, k = 0..5: the entry for phase p of
    // scale 2^-k sits at index (2^k - 1) + p; dword w = enc(px*2^w) | enc(px*2^w + 1/4) << 16, px = p*2^-k.
    uint32_t xtab[64][4];
    uint32_t ytab[64][4];             // same for y, one byte up
};

// OCP e4m3 (1-4-3, bias 7, no infinities) byte -> the integer 512*value: subnormals m * 2^-9,
// normals (8+m) * 2^(e-10).  The two NaN encodings decode as 0.
__device__ __forceinline__ int32_t e4m3_times_512(uint32_t byte)
{
    uint32_t const e = (byte >> 3) & 15u, m = byte & 7u;
    int32_t mag = (e == 0) ? int32_t(m) : int32_t((8u + m) << (e - 1u));
    if ((byte & 0x7fu) == 0x7fu) mag = 0;
    return (byte & 0x80u) ? -mag : mag;
}

// A operand dword of an int8 layer: four consecutive weights of one row (0 beyond the layer's inputs).
__device__ __forceinline__ uint32_t weight_dword(uint32_t const* blob32, int woff, int row, int in, int k)
{
    return (k < in) ? blob32[(woff + row * in + k) >> 2] : 0u;
}

__device__ __forceinline__ uint32_t halves_of_ints(int a, int b)                   // two integers of at most 11 bits -> two fp16 (exact)
{
    v2h const h = { _Float16(a), _Float16(b) };
    return __builtin_bit_cast(uint32_t, h);
}

// Four e4m3 bytes -> the three int8 planes of their 512-fold values: 6 bits, 6 bits, signed rest.
__device__ __forceinline__ void int8_planes(uint32_t v, uint32_t (&planes)[3])
{
    planes[0] = planes[1] = planes[2] = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        int32_t const W = e4m3_times_512((v >> (8 * r)) & 0xffu);
        planes[0] |= uint32_t(W & 63) << (8 * r);
        planes[1] |= uint32_t((W >> 6) & 63) << (8 * r);
        planes[2] |= (uint32_t(W >> 12) & 0xffu) << (8 * r);
    }
}

__device__ __forceinline__ uint32_t halves_of_bytes(uint32_t v, int firstByte)     // two int8 -> two fp16 (exact)
{
    v2h const h = { _Float16(int(int8_t(v >> (8 * firstByte)))), _Float16(int(int8_t(v >> (8 * firstByte + 8)))) };
    return __builtin_bit_cast(uint32_t, h);
}

// The lane's number in its wave from the execution mask: no register has to keep the thread id alive for it.
__device__ __forceinline__ int lane_id()
{
    return int(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)));
}

// Copies the int8 blob (src/WeightLayout.cpp:42-49: matrices, then fp32 scales, then int32
// biases; W[c*IN + k]) into LDS in MFMA operand order.  Returns kStagedF16 when layers 1..3 were
// staged for the fp16 matrix instruction (see mlp_forward_f16): that needs, for every channel of
// those layers, |bias - 113*sum(W)| + 240*sum|W| < 2^24 (for e4m3 rows: the same for either plane, and
// |bias| + 128*sum|512 w| < 2^31); otherwise they are staged as int8 tiles.
// With kStagedF16, kOutputsBounded says that no output can come near the fp16 overflow threshold
// (the same bound times the channel's scale stays below 60000), so stores may skip that check.
// kL0Magic (with kStagedF16, variants without e4m3 weights): layer 0's accumulators start at bias + 0x4B400000,
// so that the int32 result, read as a float, is 1.5 * 2^23 + acc and one fp32 subtraction replaces the conversion
// (needs |acc| < 2^22: |bias| <= 3 100 000 for every channel, the inputs add at most 64 * 128 * 127).
constexpr int kStagedF16 = 1, kOutputsBounded = 2, kL0Magic = 4;
constexpr int32_t kMagicBits = 0x4B400000;                   // 12582912.0f = 1.5 * 2^23
template <class V>
__device__ __attribute__((noinline)) int stage_weights(LdsT<V>& lds, uint8_t const* __restrict__ blob, int const tid)
{
    constexpr int ins[4]   = { V::IN, V::H0, V::H1, V::H2 };
    constexpr int tiles[4] = { V::T0, V::T1, V::T2, V::T3 };
    constexpr int woff[4]  = { 0, V::W1_OFF, V::W2_OFF, V::W3_OFF };
    // The blob first goes into LDS as it is (the transposition buffers are idle now), in one pass of coalesced loads:
    // everything below - the row sums above all, one thread per channel walking its row - then reads LDS instead of
    // following a chain of loads from memory.
    constexpr int kBlobDwords = (V::BIAS_OFF + 4 * V::TOTAL_OUT) / 4;
    static_assert(sizeof(lds.in) >= size_t(kBlobDwords + 4) * 4, "the blob fits the transposition buffers");
    uint32_t* const flags = &lds.in[0][0][0];                  // one word for the workgroup's flags, then the blob
    uint32_t* const raw32 = flags + 4;
    {
        uint32_t const* const src = reinterpret_cast<uint32_t const*>(blob);
        for (int e = tid; e < kBlobDwords; e += V::THREADS) raw32[e] = src[e];
        if (tid == 0) *flags = 7u;
    }
    __syncthreads();
    uint32_t const* const blob32 = raw32;
    uint8_t const* const blobBytes = reinterpret_cast<uint8_t const*>(raw32);

    // scales and biases of every layer, in D-register order
    {
        int tileBase = 0, chanBase = 0;
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            for (int e = tid; e < tiles[l] * 16; e += V::THREADS) {
                int const r = e & 3, g = (e >> 2) & 3, t = e >> 4;
                int const c = chanBase + 16 * t + 4 * g + r;
                lds.scale[tileBase + t][g][r] = reinterpret_cast<float const*>(blobBytes + V::SCALE_OFF)[c];
                lds.bias[tileBase + t][g][r]  = reinterpret_cast<int32_t const*>(blobBytes + V::BIAS_OFF)[c];
            }
            tileBase += tiles[l];
            chanBase += tiles[l] * 16;
        }
    }

    // int8 tiles of layer 0 (three planes for e4m3 weights)
    for (int e = tid; e < V::T0 * 64 * 4; e += V::THREADS) {
        int const d = e & 3, lane = (e >> 2) & 63, t = e >> 8;
        int const i = lane & 15, g = lane >> 4;
        // k-slot (g, 4d+r) = input 16g+4d+r
        uint32_t const v = weight_dword(blob32, 0, 16 * t + i, V::IN, 16 * g + 4 * d);
        if constexpr (V::FP8_WEIGHTS) {
            uint32_t planes[3];
            int8_planes(v, planes);
#pragma unroll
            for (int q = 0; q < V::PLANES; ++q) lds.w[q][t][lane][d] = planes[q];
        } else {
            lds.w[0][t][lane][d] = v;
        }
    }

    // Four threads per channel of layers 1..3 (two or one where the workgroup has not that many), a part of the row
    // each: row sums decide whether the fp16 path is exact.  (The sums fit 32 bits: at most 64 weights of at most
    // 448 * 512 in magnitude.)  After the exchange all of them hold the totals; the first writes the channel's
    // constants further down.
    bool fits = true, bounded = true;
    int64_t shifted = 0;
    bool twoPlanes = false;
    int slotTile = 0, slotG = 0, slotR = 0;
    constexpr int kSplit = 4 * V::LATE_CHANNELS <= V::THREADS ? 4 : (2 * V::LATE_CHANNELS <= V::THREADS ? 2 : 1);
    static_assert(V::LATE_CHANNELS <= V::THREADS, "a thread per channel at least");
    bool const rowThread = tid < kSplit * V::LATE_CHANNELS;
    bool const rowWriter = rowThread && tid % kSplit == 0;
    int const c = tid / kSplit;                              // the thread's channel among those of layers 1..3
    if (rowThread) {
        int const part = tid % kSplit;
        int const l = c < V::H1 ? 1 : (c < V::H1 + V::H2 ? 2 : 3);
        int const row = c - (l == 1 ? 0 : (l == 2 ? V::H1 : V::H1 + V::H2));
        int const in = l == 1 ? V::H0 : (l == 2 ? V::H1 : V::H2);
        int const off = l == 1 ? V::W1_OFF : (l == 2 ? V::W2_OFF : V::W3_OFF);
        twoPlanes = V::FP8_WEIGHTS && l < 3;
        static_assert(V::H0 % 16 == 0 && V::H1 % 16 == 0 && V::H2 % 16 == 0, "a part of a row is whole dwords");
        int32_t sum = 0, sumAbs = 0, sumAbsHi = 0, sumLo = 0;
        for (int k = part * (in / kSplit); k < (part + 1) * (in / kSplit); k += 4) {
            uint32_t const v = blob32[(off + row * in + k) >> 2];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                uint32_t const byte = (v >> (8 * r)) & 0xffu;
                int const w = twoPlanes ? e4m3_times_512(byte) : int(int8_t(byte));
                int const hi = w >> 10;
                sum += w;
                sumAbs += w < 0 ? -w : w;
                sumAbsHi += hi < 0 ? -hi : hi;
                sumLo += w & 1023;
            }
        }
#pragma unroll
        for (int step = 1; step < kSplit; step *= 2) {        // the parts sit in neighbouring lanes of one wave
            sum += __shfl_xor(sum, step, 64);
            sumAbs += __shfl_xor(sumAbs, step, 64);
            if constexpr (V::FP8_WEIGHTS) {
                sumAbsHi += __shfl_xor(sumAbsHi, step, 64);
                sumLo += __shfl_xor(sumLo, step, 64);
            }
        }
        int32_t const bias = reinterpret_cast<int32_t const*>(blobBytes + V::BIAS_OFF)[V::H0 + c];
        shifted = int64_t(bias) - 113 * int64_t(sum);     // activations enter as q + 113 in [-15, 240]
        int64_t const absBias = bias < 0 ? -int64_t(bias) : int64_t(bias);
        int64_t const absShifted = shifted < 0 ? -shifted : shifted;
        if (twoPlanes) {
            // Exact when the int32 accumulator the result is defined by cannot wrap (inputs in [-128, 127])
            // and both fp32 partial sums, started at floor(shifted / 1024) and shifted mod 1024, stay integers.
            int64_t const startHi = shifted >> 10;
            fits = absBias + 128 * int64_t(sumAbs) < (int64_t(1) << 31)
                && (startHi < 0 ? -startHi : startHi) + 240 * int64_t(sumAbsHi) < (int64_t(1) << 24)
                && 1023 + 240 * int64_t(sumLo) < (int64_t(1) << 24);
        } else {
            int64_t const bound = absShifted + 240 * int64_t(sumAbs);
            fits = bound < (int64_t(1) << 24);
            if (l == 3) bounded = float(bound) * fabsf(reinterpret_cast<float const*>(blobBytes + V::SCALE_OFF)[V::H0 + c]) < 60000.f;
        }
        // the channel's scale gets multiplied by 2^24 (activations enter as (q + 113) * 2^-24): must stay finite
        fits = fits && fabsf(reinterpret_cast<float const*>(blobBytes + V::SCALE_OFF)[V::H0 + c]) < 0x1p100f;
        slotTile = V::T0 + (l == 1 ? 0 : (l == 2 ? V::T1 : V::T1 + V::T2)) + row / 16;
        slotG = (row >> 2) & 3;
        slotR = row & 3;
    }
    bool small = true;
    if constexpr (!V::FP8_WEIGHTS) {
        if (tid < V::H0) {
            int32_t const b = reinterpret_cast<int32_t const*>(blobBytes + V::BIAS_OFF)[tid];
            small = b >= -3100000 && b <= 3100000;
        }
    }
    // The three conditions, each over every thread of the workgroup: a ballot per wave, one LDS atomic per wave on a
    // word of the (idle) transposition buffer.  The barriers also order the bias writes above.  (The runtime's
    // workgroup reduction would do, but as a library call it needs the caller's thread ids kept in a vector register
    // for the whole kernel.)
    {
        uint32_t const mine = (__all(fits ? 1 : 0) ? 1u : 0u) | (__all(bounded ? 1 : 0) ? 2u : 0u) | (__all(small ? 1 : 0) ? 4u : 0u);
        if ((tid & 63) == 0) atomicAnd(flags, mine);
    }
    __syncthreads();
    uint32_t const all = __builtin_amdgcn_readfirstlane(*flags);
    __syncthreads();                                         // every wave has read the word before the buffer is used again
    bool const useF16 = (all & 1u) != 0, outputsBounded = (all & 2u) != 0;
    bool l0Magic = false;
    if constexpr (!V::FP8_WEIGHTS) {
        l0Magic = (all & 4u) != 0 && useF16;
        if (l0Magic && tid < V::H0) {
            int const c = tid;
            lds.bias[c >> 4][(c >> 2) & 3][c & 3] += kMagicBits;
        }
    }
    constexpr int base[4] = { 0, V::F16_L1, V::F16_L2, V::F16_L3 };
    uint32_t* const late32 = reinterpret_cast<uint32_t*>(lds.late);
    if (useF16) {
        if (rowWriter) {
            if constexpr (V::FP8_WEIGHTS) {
                if (twoPlanes) lds.biasLo[slotTile][slotG][slotR] = float(shifted & 1023) * 0x1p-24f;
            }
            // sums run over (q + 113) * 2^-24 (see activate_scale4): every term, this start value included, is an
            // integer below 2^24 times 2^-24, exact in fp32; the scale takes the 2^24 back
            lds.bias[slotTile][slotG][slotR] = __builtin_bit_cast(int32_t, float(twoPlanes ? (shifted >> 10) : shifted) * 0x1p-24f);
            lds.scale[slotTile][slotG][slotR] = reinterpret_cast<float const*>(blobBytes + V::SCALE_OFF)[V::H0 + c] * 0x1p24f;
        }
        // fp16 blocks.  Lane (i, kg) of the block of output tile t and input-tile pair p holds
        // W[16t + i][16*(2p + e/4) + 4*kg + e%4], e = 0..7: the channels lane (j, kg) of the
        // previous layer's D registers owns, in register order.
#pragma unroll
        for (int l = 1; l < 4; ++l) {
            int const in = ins[l];
            int const inTiles = tiles[l - 1], pairs = inTiles / 2, per = V::f16_units(inTiles);
            int const planeDwords = tiles[l] * per * 4;
            // one work item = one (output tile, input tile, lane): 4 weights -> 2 dwords (per plane)
            for (int e = tid; e < tiles[l] * inTiles * 64; e += V::THREADS) {
                int const lane = e & 63, rest = e >> 6;
                int const ti = rest % inTiles, t = rest / inTiles;
                int const i = lane & 15, kg = lane >> 4;
                uint32_t const v = blob32[(woff[l] + (16 * t + i) * in + 16 * ti + 4 * kg) >> 2];
                int const p = ti >> 1;
                // dword index inside `late`: paired blocks hold 4 dwords per lane, the tail block 2
                int const at = (p < pairs) ? ((base[l] + t * per + p * 64 + lane) * 4 + (ti & 1) * 2)
                                           : ((base[l] + t * per + pairs * 64) * 4 + lane * 2);
                if (V::FP8_WEIGHTS && l < 3) {
                    int32_t W[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) W[r] = e4m3_times_512((v >> (8 * r)) & 0xffu);
                    late32[at]     = halves_of_ints(W[0] >> 10, W[1] >> 10);
                    late32[at + 1] = halves_of_ints(W[2] >> 10, W[3] >> 10);
                    late32[at + planeDwords]     = halves_of_ints(W[0] & 1023, W[1] & 1023);
                    late32[at + planeDwords + 1] = halves_of_ints(W[2] & 1023, W[3] & 1023);
                } else {
                    late32[at]     = halves_of_bytes(v, 0);
                    late32[at + 1] = halves_of_bytes(v, 2);
                }
            }
        }
    } else {
        int tileBase = 0;
#pragma unroll
        for (int l = 1; l < 4; ++l) {
            int const in = ins[l];
            for (int e = tid; e < tiles[l] * 64 * 4; e += V::THREADS) {
                int const d = e & 3, lane = (e >> 2) & 63, t = e >> 8;
                int const i = lane & 15, g = lane >> 4;
                // k-slot (g, 4d+r) = channel 16d+4g+r of the previous layer
                uint32_t const v = weight_dword(blob32, woff[l], 16 * t + i, in, 16 * d + 4 * g);
                int const at = ((tileBase + t) * 64 + lane) * 4 + d;
                if (V::FP8_WEIGHTS && l < 3) {
                    uint32_t planes[3];
                    int8_planes(v, planes);
#pragma unroll
                    for (int q = 0; q < V::PLANES; ++q) late32[q * V::LATE_TILES * 256 + at] = planes[q];
                } else {
                    late32[at] = v;
                }
            }
            tileBase += tiles[l];
        }
    }
    return useF16 ? (kStagedF16 | (outputsBounded ? kOutputsBounded : 0) | (l0Magic ? kL0Magic : 0)) : 0;
}

template <class V>
__device__ __forceinline__ void prepare_inputs_general(DevMip const& m, int x, int y, uint32_t (&in)[16])
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

// Input vector of one texel from integer arithmetic only (see axis_fast above).  All gathers of both grids are
// issued before any of them is waited for (the scheduling barrier keeps the compiler from sinking the last of them
// below the first wait): one memory round trip per tile, not two.
template <class V, class Mip = DevMip>
__device__ __forceinline__ void prepare_inputs_fast(Mip const& m, LdsT<V> const& lds, int x, int y, uint32_t (&in)[16])
{
    constexpr int HL = V::HR_MODE == 1 ? 1 : (V::HR_F + 3) / 4, LL = (V::LR_F + 3) / 4;
#pragma unroll
    for (int i = 0; i < 16; ++i) in[i] = 0;

    AxisFoot const hx = axis_fast(x, m.hrAxisX, m.hrWidth), hy = axis_fast(y, m.hrAxisY, m.hrHeight);
    AxisFoot const lx = axis_fast(x, m.lrAxisX, m.lrWidth), ly = axis_fast(y, m.lrAxisY, m.lrHeight);
    uint32_t hv[HL][4], lv[LL][4];                           // [layer][tap 00, 10, 01, 11]
    {
        GlobalU8Ptr const g = (GlobalU8Ptr)m.hr;
        uint32_t const lgw = ((m.hrAxisX >> 24) & 0xffu) + 1u;   // log2(bytes per grid row)
        uint32_t const layerStride = uint32_t(m.hrWidth) * uint32_t(m.hrHeight) * 2u;   // bytes
        uint32_t const r0 = hy.c0 << lgw, r1 = hy.c1 << lgw, c0 = hx.c0 << 1, c1 = hx.c1 << 1;
        uint32_t const a00 = r0 + c0, a10 = r0 + c1, a01 = r1 + c0, a11 = r1 + c1;   // byte offsets
#pragma unroll
        for (int L = 0; L < HL; ++L) {
            GlobalU8Ptr const gl = g + size_t(L) * layerStride;
            hv[L][0] = load_u16(gl, a00); hv[L][1] = load_u16(gl, a10); hv[L][2] = load_u16(gl, a01); hv[L][3] = load_u16(gl, a11);
        }
    }
    {
        GlobalU8Ptr const g = (GlobalU8Ptr)m.lr;
        uint32_t const lgw = ((m.lrAxisX >> 24) & 0xffu) + 1u;
        uint32_t const layerStride = uint32_t(m.lrWidth) * uint32_t(m.lrHeight) * 2u;
        uint32_t const r0 = ly.c0 << lgw, r1 = ly.c1 << lgw, c0 = lx.c0 << 1, c1 = lx.c1 << 1;
        uint32_t const a00 = r0 + c0, a10 = r0 + c1, a01 = r1 + c0, a11 = r1 + c1;
#pragma unroll
        for (int L = 0; L < LL; ++L) {
            GlobalU8Ptr const gl = g + size_t(L) * layerStride;
            lv[L][0] = load_u16(gl, a00); lv[L][1] = load_u16(gl, a10); lv[L][2] = load_u16(gl, a01); lv[L][3] = load_u16(gl, a11);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- high-res grid
    if constexpr (V::HR_MODE == 1) {
        static_assert(V::HR_MODE != 1 || (V::HR_BITS == 2 && V::HR_F == 8 && V::HR_SLOTS == 8), "concat grids: 8 x 2-bit");
#pragma unroll
        for (int tap = 0; tap < 4; ++tap) {
            in[2 * tap]     = lds.lut2[hv[0][tap] & 0xffu];
            in[2 * tap + 1] = lds.lut2[hv[0][tap] >> 8];
        }
    } else {
        uint32_t const nx = (m.hrAxisX >> 8) & 0xffu, ny = (m.hrAxisY >> 8) & 0xffu;
        uint32_t const wx1 = hx.f, wx0 = (1u << nx) - hx.f, wy1 = hy.f, wy0 = (1u << ny) - hy.f;
        uint32_t const w00 = mul24(wx0, wy0), w10 = mul24(wx1, wy0), w01 = mul24(wx0, wy1), w11 = mul24(wx1, wy1);
#pragma unroll
        for (int L = 0; L < HL; ++L) {
            uint32_t b = bilinear4_int(hv[L][0], hv[L][1], hv[L][2], hv[L][3], w00, w10, w01, w11, nx + ny);
            if (4 * L + 4 > V::HR_F) b &= (1u << (8 * (V::HR_F - 4 * L))) - 1u;
            in[L] = b;
        }
    }
    // ---- low-res grid: bilinear, 4-bit
    {
        uint32_t const nx = (m.lrAxisX >> 8) & 0xffu, ny = (m.lrAxisY >> 8) & 0xffu;
        uint32_t const wx1 = lx.f, wx0 = (1u << nx) - lx.f, wy1 = ly.f, wy0 = (1u << ny) - ly.f;
        uint32_t const w00 = mul24(wx0, wy0), w10 = mul24(wx1, wy0), w01 = mul24(wx0, wy1), w11 = mul24(wx1, wy1);
#pragma unroll
        for (int L = 0; L < LL; ++L) {
            uint32_t b = bilinear4_int(lv[L][0], lv[L][1], lv[L][2], lv[L][3], w00, w10, w01, w11, nx + ny);
            if (4 * L + 4 > V::LR_F) b &= (1u << (8 * (V::LR_F - 4 * L))) - 1u;
            in[V::HR_INPUTS / 4 + L] = b;
        }
    }
    // ---- positional encoding from the per-mip phase tables
    {
        uint4 const ex = *reinterpret_cast<uint4 const*>(&lds.xtab[m.posMask + (uint32_t(x) & m.posMask)][0]);
        uint4 const ey = *reinterpret_cast<uint4 const*>(&lds.ytab[m.posMask + (uint32_t(y) & m.posMask)][0]);
        in[V::POS_BASE / 4 + 0] = ex.x | ey.x;
        in[V::POS_BASE / 4 + 1] = ex.y | ey.y;
        in[V::POS_BASE / 4 + 2] = ex.z | ey.z;
        if constexpr (V::LOD == 2) {
            uint32_t const l = uint32_t(int(m.positionLod * 127.5f)) & 0xffu;
            in[V::POS_BASE / 4 + 3] = l | (l << 8);
        }
    }
}

// The same input vector for scattered sample points (random-access queries), where what costs is
// the memory round trip of each gather, not vector issue.  Three steps:
//   1. one dword load per pair of horizontally adjacent taps (cells are 2 bytes, so the dword may sit
//      on a 2-byte boundary; global memory takes such loads) for every row and layer of both grids,
//      all issued back to back.  A footprint that wraps around the grid edge, or a grid one cell wide,
//      has no such dword: those lanes load from `safe` (any readable 4 bytes) instead, so that the
//      step has no branch and every lane's loads are in flight together;
//   2. the lanes without adjacent taps (few, except on the smallest mips) fetch their two cells with
//      16-bit loads in one divergent region;
//   3. arithmetic.
// Issued behind their uses, with a branch per pair, the gathers of a lane ran one after the other:
// about ten round trips per query instead of one.

template <class V, class Mip>
__device__ __forceinline__ void prepare_inputs_scattered(Mip const& m, LdsT<V> const& lds, int x, int y, GlobalU8Ptr safe,
                                                         uint32_t (&in)[16])
{
    constexpr int HL = V::HR_MODE == 1 ? 1 : (V::HR_F + 3) / 4, LL = (V::LR_F + 3) / 4;
#pragma unroll
    for (int i = 0; i < 16; ++i) in[i] = 0;

    AxisFoot const hx = axis_fast(x, m.hrAxisX, m.hrWidth), hy = axis_fast(y, m.hrAxisY, m.hrHeight);
    AxisFoot const lx = axis_fast(x, m.lrAxisX, m.lrWidth), ly = axis_fast(y, m.lrAxisY, m.lrHeight);
    GlobalU8Ptr const gh = (GlobalU8Ptr)m.hr, gl = (GlobalU8Ptr)m.lr;
    uint32_t const hlgw = ((m.hrAxisX >> 24) & 0xffu) + 1u, llgw = ((m.lrAxisX >> 24) & 0xffu) + 1u;
    uint32_t const hStride = uint32_t(m.hrWidth) * uint32_t(m.hrHeight) * 2u, lStride = uint32_t(m.lrWidth) * uint32_t(m.lrHeight) * 2u;
    uint32_t const hc0 = hx.c0 << 1, hc1 = hx.c1 << 1, lc0 = lx.c0 << 1, lc1 = lx.c1 << 1;
    uint32_t const hrow[2] = { hy.c0 << hlgw, hy.c1 << hlgw }, lrow[2] = { ly.c0 << llgw, ly.c1 << llgw };
    bool const hAdj = hc1 == hc0 + 2u, lAdj = lc1 == lc0 + 2u;

    uint32_t hp[HL][2], lp[LL][2];                           // [layer][row]: left cell in the low half
#pragma unroll
    for (int L = 0; L < HL; ++L)
#pragma unroll
        for (int r = 0; r < 2; ++r)
            hp[L][r] = *reinterpret_cast<GlobalU32A2Ptr>(hAdj ? gh + size_t(L) * hStride + (hrow[r] + hc0) : safe);
#pragma unroll
    for (int L = 0; L < LL; ++L)
#pragma unroll
        for (int r = 0; r < 2; ++r)
            lp[L][r] = *reinterpret_cast<GlobalU32A2Ptr>(lAdj ? gl + size_t(L) * lStride + (lrow[r] + lc0) : safe);
    __builtin_amdgcn_sched_barrier(0);
    if (!(hAdj && lAdj)) {
        if (!hAdj) {
#pragma unroll
            for (int L = 0; L < HL; ++L)
#pragma unroll
                for (int r = 0; r < 2; ++r)
                    hp[L][r] = load_u16(gh + size_t(L) * hStride, hrow[r] + hc0) | (load_u16(gh + size_t(L) * hStride, hrow[r] + hc1) << 16);
        }
        if (!lAdj) {
#pragma unroll
            for (int L = 0; L < LL; ++L)
#pragma unroll
                for (int r = 0; r < 2; ++r)
                    lp[L][r] = load_u16(gl + size_t(L) * lStride, lrow[r] + lc0) | (load_u16(gl + size_t(L) * lStride, lrow[r] + lc1) << 16);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    if constexpr (V::HR_MODE == 1) {
        static_assert(V::HR_MODE != 1 || (V::HR_BITS == 2 && V::HR_F == 8 && V::HR_SLOTS == 8), "concat grids: 8 x 2-bit");
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            in[4 * r]     = lds.lut2[hp[0][r] & 0xffu];
            in[4 * r + 1] = lds.lut2[(hp[0][r] >> 8) & 0xffu];
            in[4 * r + 2] = lds.lut2[(hp[0][r] >> 16) & 0xffu];
            in[4 * r + 3] = lds.lut2[hp[0][r] >> 24];
        }
    } else {
        uint32_t const nx = (m.hrAxisX >> 8) & 0xffu, ny = (m.hrAxisY >> 8) & 0xffu;
        uint32_t const wx1 = hx.f, wx0 = (1u << nx) - hx.f, wy1 = hy.f, wy0 = (1u << ny) - hy.f;
        uint32_t const w00 = mul24(wx0, wy0), w10 = mul24(wx1, wy0), w01 = mul24(wx0, wy1), w11 = mul24(wx1, wy1);
#pragma unroll
        for (int L = 0; L < HL; ++L) {
            uint32_t b = bilinear4_int(hp[L][0] & 0xffffu, hp[L][0] >> 16, hp[L][1] & 0xffffu, hp[L][1] >> 16, w00, w10, w01, w11, nx + ny);
            if (4 * L + 4 > V::HR_F) b &= (1u << (8 * (V::HR_F - 4 * L))) - 1u;
            in[L] = b;
        }
    }
    {
        uint32_t const nx = (m.lrAxisX >> 8) & 0xffu, ny = (m.lrAxisY >> 8) & 0xffu;
        uint32_t const wx1 = lx.f, wx0 = (1u << nx) - lx.f, wy1 = ly.f, wy0 = (1u << ny) - ly.f;
        uint32_t const w00 = mul24(wx0, wy0), w10 = mul24(wx1, wy0), w01 = mul24(wx0, wy1), w11 = mul24(wx1, wy1);
#pragma unroll
        for (int L = 0; L < LL; ++L) {
            uint32_t b = bilinear4_int(lp[L][0] & 0xffffu, lp[L][0] >> 16, lp[L][1] & 0xffffu, lp[L][1] >> 16, w00, w10, w01, w11, nx + ny);
            if (4 * L + 4 > V::LR_F) b &= (1u << (8 * (V::LR_F - 4 * L))) - 1u;
            in[V::HR_INPUTS / 4 + L] = b;
        }
    }
    {
        uint4 const ex = *reinterpret_cast<uint4 const*>(&lds.xtab[m.posMask + (uint32_t(x) & m.posMask)][0]);
        uint4 const ey = *reinterpret_cast<uint4 const*>(&lds.ytab[m.posMask + (uint32_t(y) & m.posMask)][0]);
        in[V::POS_BASE / 4 + 0] = ex.x | ey.x;
        in[V::POS_BASE / 4 + 1] = ex.y | ey.y;
        in[V::POS_BASE / 4 + 2] = ex.z | ey.z;
        if constexpr (V::LOD == 2) {
            uint32_t const l = uint32_t(int(m.positionLod * 127.5f)) & 0xffu;
            in[V::POS_BASE / 4 + 3] = l | (l << 8);
        }
    }
}

// The same input vector from the query-ordered copy of the grids: bricks of T x T cells (T = 4, or 8
// for a one-layer grid), [brick row][brick column][cell row][cell column][layer], so that all layers
// of a cell are one load of 2, 4, 6 or 8 bytes and the 2 x 2 footprint usually lies in one or two
// cache lines.  Every tap is addressed on its own (wrap included), so there is no branch at all:
// eight loads per sample point for the 8 x 2-bit + 16 x 4-bit geometry, all in flight together.
template <class V, class Mip>
__device__ __forceinline__ void prepare_inputs_bricked(Mip const& m, LdsT<V> const& lds, int x, int y, uint32_t (&in)[16])
{
    constexpr int HL = V::HR_MODE == 1 ? 1 : (V::HR_F + 3) / 4, LL = (V::LR_F + 3) / 4;
#pragma unroll
    for (int i = 0; i < 16; ++i) in[i] = 0;

    AxisFoot const hx = axis_fast(x, m.hrAxisX, m.hrWidth), hy = axis_fast(y, m.hrAxisY, m.hrHeight);
    AxisFoot const lx = axis_fast(x, m.lrAxisX, m.lrWidth), ly = axis_fast(y, m.lrAxisY, m.lrHeight);
    GlobalU8Ptr const gh = (GlobalU8Ptr)m.hrBricks, gl = (GlobalU8Ptr)m.lrBricks;
    uint32_t const hlg = (m.hrAxisX >> 24) & 0xffu, llg = (m.lrAxisX >> 24) & 0xffu;     // log2(grid width)

    // taps in the order a00 (x0, y0), a10 (x1, y0), a01 (x0, y1), a11 (x1, y1)
    uint32_t hc[4][2], lc[4][2];
    load_brick_cell<HL>(gh, brick_offset<HL>(hx.c0, hy.c0, hlg), hc[0]);
    load_brick_cell<HL>(gh, brick_offset<HL>(hx.c1, hy.c0, hlg), hc[1]);
    load_brick_cell<HL>(gh, brick_offset<HL>(hx.c0, hy.c1, hlg), hc[2]);
    load_brick_cell<HL>(gh, brick_offset<HL>(hx.c1, hy.c1, hlg), hc[3]);
    load_brick_cell<LL>(gl, brick_offset<LL>(lx.c0, ly.c0, llg), lc[0]);
    load_brick_cell<LL>(gl, brick_offset<LL>(lx.c1, ly.c0, llg), lc[1]);
    load_brick_cell<LL>(gl, brick_offset<LL>(lx.c0, ly.c1, llg), lc[2]);
    load_brick_cell<LL>(gl, brick_offset<LL>(lx.c1, ly.c1, llg), lc[3]);
    __builtin_amdgcn_sched_barrier(0);                       // all loads before any arithmetic

    auto layer_of = [](uint32_t const (&cell)[2], int L) -> uint32_t { return (L & 1) ? cell[L >> 1] >> 16 : cell[L >> 1] & 0xffffu; };
    if constexpr (V::HR_MODE == 1) {
        static_assert(V::HR_MODE != 1 || (V::HR_BITS == 2 && V::HR_F == 8 && V::HR_SLOTS == 8), "concat grids: 8 x 2-bit");
#pragma unroll
        for (int tap = 0; tap < 4; ++tap) {
            in[2 * tap]     = lds.lut2[hc[tap][0] & 0xffu];
            in[2 * tap + 1] = lds.lut2[(hc[tap][0] >> 8) & 0xffu];
        }
    } else {
        uint32_t const nx = (m.hrAxisX >> 8) & 0xffu, ny = (m.hrAxisY >> 8) & 0xffu;
        uint32_t const wx1 = hx.f, wx0 = (1u << nx) - hx.f, wy1 = hy.f, wy0 = (1u << ny) - hy.f;
        uint32_t const w00 = mul24(wx0, wy0), w10 = mul24(wx1, wy0), w01 = mul24(wx0, wy1), w11 = mul24(wx1, wy1);
#pragma unroll
        for (int L = 0; L < HL; ++L) {
            uint32_t b = bilinear4_int(layer_of(hc[0], L), layer_of(hc[1], L), layer_of(hc[2], L), layer_of(hc[3], L), w00, w10, w01, w11, nx + ny);
            if (4 * L + 4 > V::HR_F) b &= (1u << (8 * (V::HR_F - 4 * L))) - 1u;
            in[L] = b;
        }
    }
    {
        uint32_t const nx = (m.lrAxisX >> 8) & 0xffu, ny = (m.lrAxisY >> 8) & 0xffu;
        uint32_t const wx1 = lx.f, wx0 = (1u << nx) - lx.f, wy1 = ly.f, wy0 = (1u << ny) - ly.f;
        uint32_t const w00 = mul24(wx0, wy0), w10 = mul24(wx1, wy0), w01 = mul24(wx0, wy1), w11 = mul24(wx1, wy1);
#pragma unroll
        for (int L = 0; L < LL; ++L) {
            uint32_t b = bilinear4_int(layer_of(lc[0], L), layer_of(lc[1], L), layer_of(lc[2], L), layer_of(lc[3], L), w00, w10, w01, w11, nx + ny);
            if (4 * L + 4 > V::LR_F) b &= (1u << (8 * (V::LR_F - 4 * L))) - 1u;
            in[V::HR_INPUTS / 4 + L] = b;
        }
    }
    {
        uint4 const ex = *reinterpret_cast<uint4 const*>(&lds.xtab[m.posMask + (uint32_t(x) & m.posMask)][0]);
        uint4 const ey = *reinterpret_cast<uint4 const*>(&lds.ytab[m.posMask + (uint32_t(y) & m.posMask)][0]);
        in[V::POS_BASE / 4 + 0] = ex.x | ey.x;
        in[V::POS_BASE / 4 + 1] = ex.y | ey.y;
        in[V::POS_BASE / 4 + 2] = ex.z | ey.z;
        if constexpr (V::LOD == 2) {
            uint32_t const l = uint32_t(int(m.positionLod * 127.5f)) & 0xffu;
            in[V::POS_BASE / 4 + 3] = l | (l << 8);
        }
    }
}

// One byte of the positional encoding (Inference.hlsli:89-113): int(enc * 127.5), truncating.
__device__ __forceinline__ uint32_t posenc_byte(float p)
{
    float const e = (p - floorf(p)) * 2.f - 1.f;
    return uint32_t(int(e * 127.5f)) & 0xffu;
}

// Fills the phase tables.  For positionScale = 2^-k the encoding of texel x depends only on
// x mod 2^k, and all arithmetic involved is exact, so table and per-lane evaluation agree; scales of
// 1 and above have period 1 (k = 0).  One entry per thread, threads 0..62 fill both tables.
template <class V>
__device__ void build_posenc_tables(LdsT<V>& lds)
{
    int const t = threadIdx.x;
    if (t < 63) {
        int const k = 31 - __builtin_clz(uint32_t(t + 1));   // floor(log2(t + 1))
        int const phase = t + 1 - (1 << k);
        float p = float(phase) * __builtin_ldexpf(1.f, -k);
        uint32_t e[3];
#pragma unroll
        for (int w = 0; w < 3; ++w) {
            e[w] = posenc_byte(p) | (posenc_byte(p + 0.25f) << 16);
            p *= 2.f;
        }
        lds.xtab[t][0] = e[0];      lds.xtab[t][1] = e[1];      lds.xtab[t][2] = e[2];      lds.xtab[t][3] = 0;
        lds.ytab[t][0] = e[0] << 8; lds.ytab[t][1] = e[1] << 8; lds.ytab[t][2] = e[2] << 8; lds.ytab[t][3] = 0;
    }
}

// Input vectors of the wave's 64 texels (lane = texel 16*b + j holds its own in `in`) -> B operands of
// layer 0: X[b] = the four input dwords of k-group g = lane/16 of texel 16b + lane%16.
template <class V>
__device__ __forceinline__ void write_inputs(LdsT<V>& lds, int wave, int lane, uint32_t const (&in)[16])
{
    uint4* dst = reinterpret_cast<uint4*>(&lds.in[wave][lane][0]);
    dst[0] = make_uint4(in[0], in[1], in[2], in[3]);
    dst[1] = make_uint4(in[4], in[5], in[6], in[7]);
    dst[2] = make_uint4(in[8], in[9], in[10], in[11]);
    if constexpr (V::IN_STRIDE >= 16) dst[3] = make_uint4(in[12], in[13], in[14], in[15]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <class V>
__device__ __forceinline__ v4i read_input_block(LdsT<V> const& lds, int wave, int lane, int b)
{
    int const j = lane & 15, g = lane >> 4;
    // a row of 12 dwords has no k-group 3: those inputs are the zero padding
    int const gRead = V::IN_STRIDE >= 16 ? g : min(g, 2);
    uint4 t = *reinterpret_cast<uint4 const*>(&lds.in[wave][b * 16 + j][4 * gRead]);
    if (V::IN_STRIDE < 16 && g == 3) t = make_uint4(0u, 0u, 0u, 0u);
    return v4i{ int(t.x), int(t.y), int(t.z), int(t.w) };
}

template <class V>
__device__ __forceinline__ void transpose_inputs(LdsT<V>& lds, int wave, int lane, uint32_t const (&in)[16], v4i (&X)[4])
{
    write_inputs<V>(lds, wave, lane, in);
#pragma unroll
    for (int b = 0; b < 4; ++b) X[b] = read_input_block<V>(lds, wave, lane, b);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// The network with every layer on the int8 matrix instruction, for ONE 16-texel block of the wave (X = its B
// operand of layer 0).  This is the path of weights whose sums do not fit the fp16 form (see stage_weights): rare, so
// the wave's four blocks go through it one after the other in a loop that is not unrolled - a quarter of the code and
// of the registers of the unrolled form, which had cost the fp16 path of the widest variant its registers.
// On return D holds, for lane (j = lane%16, g = lane/16), the int32 accumulators of output channels 4g..4g+3 of
// texel j of the block, and S their scales.
template <class V>
__device__ __forceinline__ void mlp_forward_block(LdsT<V> const& lds, int lane, v4i X, v4i& D, v4f& S)
{
    int const g = lane >> 4;
    constexpr int tiles[3] = { V::T0, V::T1, V::T2 };
    int tb = 0;
#pragma unroll
    for (int l = 0; l < 3; ++l) {
        uint32_t Y[4] = { 0, 0, 0, 0 };
#pragma unroll
        for (int t = 0; t < tiles[l]; ++t) {
            // A operand of plane q: layer 0 from `w`, later layers from the int8 tiles in `late`
            auto const operand = [&](int q) {
                uint4 const wq = l > 0 ? lds.late[(q * V::LATE_TILES + tb - V::T0 + t) * 64 + lane]
                                       : *reinterpret_cast<uint4 const*>(&lds.w[q][t][lane][0]);
                return v4i{ int(wq.x), int(wq.y), int(wq.z), int(wq.w) };
            };
            v4i const C = *reinterpret_cast<v4i const*>(&lds.bias[tb + t][g][0]);
            v4f const Sc = *reinterpret_cast<v4f const*>(&lds.scale[tb + t][g][0]);
            v4i Dh = __builtin_amdgcn_mfma_i32_16x16x64_i8(operand(0), X, C, 0, 0, 0);
            if constexpr (V::FP8_WEIGHTS) {
                v4i const Z = v4i{ 0, 0, 0, 0 };
                v4i const D1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(operand(1), X, Z, 0, 0, 0);
                v4i const D2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(operand(2), X, Z, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r)                    // 4096*D2 + 64*D1 + D0, wrapping like int32
                    Dh[r] = int((((uint32_t(D2[r]) << 6) + uint32_t(D1[r])) << 6) + uint32_t(Dh[r]));
            }
            Y[t] = activate4(Dh, Sc);
        }
        X = v4i{ int(Y[0]), int(Y[1]), int(Y[2]), int(Y[3]) };
        tb += tiles[l];
    }

    // output layer
    uint4 const wa = lds.late[(tb - V::T0) * 64 + lane];
    v4i const A = v4i{ int(wa.x), int(wa.y), int(wa.z), int(wa.w) };
    v4i const C = *reinterpret_cast<v4i const*>(&lds.bias[tb][g][0]);
    S = *reinterpret_cast<v4f const*>(&lds.scale[tb][g][0]);
    D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, X, C, 0, 0, 0);
}

// ---- layers 1..3 on the fp16 matrix instruction --------------------------------------------
//
// Same integers, fewer vector operations.  The int8 matrix instruction returns int32, which costs a
// conversion per activation, and its operands are signed bytes, which forces the "- 113" and the
// clamp of min(x, 3) into fp32.  Here the previous layer's activations enter as fp16 numbers
// proportional to u = q + 113 in [-15, 240] (u * 2^-24, see activate_scale4) and the weights as fp16 integers;
// products and every partial sum are integers below 2^24 (stage_weights checked that) times 2^-24, so the
// fp32 accumulator of v_mfma_f32_16x16x32_f16 holds exactly 2^-24 * (bias + sum W*(u - 113)) once it starts
// at 2^-24 * (bias - 113*sum(W)), and the channel's scale times 2^24 gives the same product the definition
// rounds.  The epilogue is then 5 operations per activation:
//   v_mul (scale), v_fma clamp, v_mul (x*t), v_mul (80 * 2^-24), and half each of v_cvt_pk_f16_f32 and
//   v_pk_min_i16 (the cap at 240 = the min(x, 3) of the definition: below 3 both agree term by term, from 3
//   on t = 1 and x*80 >= 240).

// HGELU-clamp + requantise of four accumulators to n = q + 113, two dwords of fp16 SUBNORMALS n * 2^-24.
// Subnormal halves are spaced 2^-24 apart from zero on, so the round-to-nearest-even conversion of
// fl32(y * 80) * 2^-24 to half IS rint(fl32(y * 80)) (in sign-magnitude: bit pattern |n|, sign bit for n < 0),
// and the power of two folds into the multiplier: fl32(y * (80 * 2^-24)) = fl32(y * 80) * 2^-24 exactly.
// That saves the separate v_rndne_f32.  Anything above 240 * 2^-24, normal halves and +Inf included, has a
// larger bit pattern as a signed 16-bit integer and negatives a smaller one, so the cap is v_pk_min_i16.
// The fp16 matrix instruction takes subnormal operands as they are (checked by the unit test of the
// instruction); the layers that consume these values hold their biases times 2^-24 and their scales times 2^24.
// The empty asm keeps multiply and conversion apart: fused (v_fma_mixlo_f16) they would round once.
//
// In two parts, because the SIMD treats them differently.  The fp32 part (activate_scale4: four multiplies / fused
// multiply-adds per value) is made of instructions that issue two at a time, one from each of two waves; the packed
// conversion and minimum (activate_pack4) issue alone, and so does everything while a matrix instruction executes.
// The layers below therefore hold a tile's conversions back until the NEXT tile's matrix instructions are in flight
// and put them between those (slots that would be single anyway), and run a tile's fp32 part as a stretch of its own.
typedef short v2s __attribute__((ext_vector_type(2)));
template <class Acc>
__device__ __forceinline__ void activate_scale4(Acc acc, v4f scale, float (&v)[4])
{
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float const x = float(acc[r]) * scale[r];
        float t = __builtin_fmaf(x, 0.333333f, 0.5f);
        t = fminf(fmaxf(t, 0.f), 1.f);
        float const y = x * t;
        v[r] = y * (80.f * 0x1p-24f);
        asm("" : "+v"(v[r]));
    }
}

__device__ __forceinline__ void activate_pack4(float const (&v)[4], uint32_t (&out)[2])
{
    v2s const cap = { 240, 240 };
    v2s const lo = __builtin_bit_cast(v2s, __builtin_convertvector(v2f{ v[0], v[1] }, v2h));
    v2s const hi = __builtin_bit_cast(v2s, __builtin_convertvector(v2f{ v[2], v[3] }, v2h));
    out[0] = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(lo, cap));
    out[1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(hi, cap));
}

// The wave's priority with the SIMD's arbiter, per kind of section.  Without it the four waves of a SIMD take turns
// instruction by instruction, so at any moment some wave is usually inside a matrix section - and while a matrix
// instruction is in flight no two vector instructions share an issue slot.  With matrix sections above everything
// else a wave runs through its matrix instructions (and the packed conversions between them) without waiting for
// its turn, the matrix sections of the four waves bunch up, and the fp32 stretches, lowest of all, meet each other
// in the time that is left: headline -6.4 %, cfg2 -9.3 %, the 0.9.2 geometry -8.5 %, e4m3 weights -5.1 %.  The other
// way round (fp32 stretches above matrix sections) is 5 % slower than no priorities at all.  Input stage, output
// layer's tail and stores sit between the two (at the bottom: 2 % worse; at the top: 1 % worse).
constexpr int kPrioMatrix = 2, kPrioOther = 1, kPrioPlain = 0;
template <int PRIORITY> __device__ __forceinline__ void wave_priority() { __builtin_amdgcn_s_setprio(PRIORITY); }

// A section boundary for the instruction scheduler: vector and matrix instructions stay on their side, scalar and LDS
// instructions may cross (so that operand reads still go out ahead of their use).
__device__ __forceinline__ void section_end() { __builtin_amdgcn_sched_barrier(0x4 | 0x80 | 0x100 | 0x200); }

// Inside a section: `groups` times { `matrix` matrix instructions, then `vector` vector instructions }.
template <int GROUPS, int MATRIX, int VECTOR>
__device__ __forceinline__ void interleave()
{
#pragma unroll
    for (int i = 0; i < GROUPS; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x8, MATRIX, 0);
        __builtin_amdgcn_sched_group_barrier(0x2, VECTOR, 0);
    }
}

// The scaled outputs of one output tile whose conversion is pending, [block b][r].
struct PendingTile {
    float z[4][4];
    template <int FIRST = 0, int COUNT = 4>
    __device__ __forceinline__ void convert_into(uint32_t (&H)[4][4][2], int tile) const
    {
#pragma unroll
        for (int b = FIRST; b < FIRST + COUNT; ++b) activate_pack4(z[b], H[b][tile]);
    }
};

// A use of tile `tile` of H (blocks FIRST .. FIRST + COUNT - 1) at this place, the end of the section that converted
// it: without one the compiler sinks the conversions to their first real use, the next layer.
template <int FIRST = 0, int COUNT = 4>
__device__ __forceinline__ void keep_here(uint32_t (&H)[4][4][2], int tile)
{
#pragma unroll
    for (int b = FIRST; b < FIRST + COUNT; ++b) asm volatile("" : "+v"(H[b][tile][0]), "+v"(H[b][tile][1]));
}

// acc[b - FIRST] += W(tile t of the layer at `base`) * H[b] for the 16-texel blocks b = FIRST .. FIRST + COUNT - 1 of the wave.
template <class V, int IN_TILES, int FIRST = 0, int COUNT = 4>
__device__ __forceinline__ void f16_tile(LdsT<V> const& lds, int base, int t, int lane, uint32_t const (&H)[4][4][2], v4f (&acc)[COUNT])
{
    constexpr int PAIRS = IN_TILES / 2, PER = V::f16_units(IN_TILES);
    uint4 const* const block = lds.late + base + t * PER;
#pragma unroll
    for (int p = 0; p < PAIRS; ++p) {
        v8h const A = __builtin_bit_cast(v8h, block[p * 64 + lane]);
#pragma unroll
        for (int b = FIRST; b < FIRST + COUNT; ++b) {
            uint4 const h = make_uint4(H[b][2 * p][0], H[b][2 * p][1], H[b][2 * p + 1][0], H[b][2 * p + 1][1]);
            acc[b - FIRST] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, __builtin_bit_cast(v8h, h), acc[b - FIRST], 0, 0, 0);
        }
    }
    if constexpr (IN_TILES % 2 != 0) {
        // An odd number of input tiles: the last one goes through the same 32-deep instruction with zeros in the
        // upper half of both operands (its block in LDS holds four halves per lane).  32-deep and 16-deep instructions
        // are never mixed in one accumulator's chain: in either order that gave wrong sums with some instruction
        // schedules (the wait between the two was not always there), while chains of one kind are reliable.  (The
        // whole layer on 16-deep instructions - three per output tile and texel block instead of two - was 0.5 to
        // 0.9 % slower: every matrix instruction in flight keeps the SIMD from issuing two vector instructions a slot.)
        uint2 const a = reinterpret_cast<uint2 const*>(block + PAIRS * 64)[lane];
        v8h const A = __builtin_bit_cast(v8h, make_uint4(a.x, a.y, 0u, 0u));
#pragma unroll
        for (int b = FIRST; b < FIRST + COUNT; ++b) {
            uint4 const h = make_uint4(H[b][2 * PAIRS][0], H[b][2 * PAIRS][1], 0u, 0u);
            acc[b - FIRST] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, __builtin_bit_cast(v8h, h), acc[b - FIRST], 0, 0, 0);
        }
    }
}

// One hidden layer on the fp16 matrix instruction (e4m3 variants: weights as two fp16 planes, 512 w = 1024 hi + lo;
// both sums are exact integers in fp32, and fma(hi, 1024, lo) rounds their exact combination once - the value a
// conversion of the int32 accumulator to float gives).  On entry `pending` holds the scaled outputs of the LAST tile of
// Hin, not yet converted; on return those of this layer's last tile.  Per output tile: section A = the tile's matrix
// instructions with the pending conversions between them, section B = the fp32 part of the tile.  In the first tile
// the pending tile is an input: its conversions come first in program order, and the matrix instructions that read
// it are the last ones.
template <class V, int IN_TILES, int OUT_TILES, bool TWO_PLANES>
__device__ __forceinline__ void f16_hidden_layer(LdsT<V> const& lds, int base, int tileBase, int lane,
                                                 uint32_t (&Hin)[4][4][2], uint32_t (&Hout)[4][4][2], PendingTile& pending)
{
    constexpr int PLANE = OUT_TILES * V::f16_units(IN_TILES);
    constexpr int MATRIX = (TWO_PLANES ? 2 : 1) * 4 * ((IN_TILES + 1) / 2);   // matrix instructions per tile
    int const g = lane >> 4;
#pragma unroll
    for (int t = 0; t < OUT_TILES; ++t) {
        v4f const C = *reinterpret_cast<v4f const*>(&lds.bias[tileBase + t][g][0]);
        v4f const Sc = *reinterpret_cast<v4f const*>(&lds.scale[tileBase + t][g][0]);
        if constexpr (TWO_PLANES) {
            // The upper plane's matrix instructions carry the pending conversions; the lower plane's follow in a section
            // of their own, so that its accumulators take the registers the converted values have left.
            if constexpr (V::FP8_WEIGHTS) {                  // (biasLo exists in those variants only)
                v4f const Clo = *reinterpret_cast<v4f const*>(&lds.biasLo[tileBase + t][g][0]);
                wave_priority<kPrioMatrix>();
                if (t == 0) pending.convert_into(Hin, IN_TILES - 1);
                else        pending.convert_into(Hout, t - 1);
                v4f acc[4] = { C, C, C, C };
                f16_tile<V, IN_TILES>(lds, base, t, lane, Hin, acc);
                interleave<8, MATRIX / 16, 2>();
                if (t > 0) keep_here(Hout, t - 1);
                section_end();
                v4f lo[4] = { Clo, Clo, Clo, Clo };
                f16_tile<V, IN_TILES>(lds, base + PLANE, t, lane, Hin, lo);
                section_end();
                wave_priority<kPrioPlain>();
#pragma unroll
                for (int b = 0; b < 4; ++b) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[b][r] = __builtin_fmaf(acc[b][r], 1024.f, lo[b][r]);
                    activate_scale4(acc[b], Sc, pending.z[b]);
                }
                section_end();
            }
        } else {
            wave_priority<kPrioMatrix>();
            if (t == 0) pending.convert_into(Hin, IN_TILES - 1);
            else        pending.convert_into(Hout, t - 1);
            v4f acc[4] = { C, C, C, C };
            f16_tile<V, IN_TILES>(lds, base, t, lane, Hin, acc);
            interleave<8, (MATRIX >= 8 ? MATRIX / 8 : 1), 2>();
            if (t > 0) keep_here(Hout, t - 1);
            section_end();
            wave_priority<kPrioPlain>();
#pragma unroll
            for (int b = 0; b < 4; ++b) activate_scale4(acc[b], Sc, pending.z[b]);
            section_end();
        }
    }
}

// Layer 0: int8 inputs, int32 accumulators.  MAGIC (variants without e4m3 weights, decided at staging): the
// accumulators started at bias + 0x4B400000, so their bits are the float 1.5 * 2^23 + acc, exactly, and a subtraction
// replaces the conversion.  e4m3 variants: three planes, recombined wrapping like int32.  Same sections as above.
template <class V, bool MAGIC>
__device__ __forceinline__ void first_layer(LdsT<V> const& lds, int lane, v4i const (&X)[4], uint32_t (&Hout)[4][4][2], PendingTile& pending)
{
    int const g = lane >> 4;
#pragma unroll
    for (int t = 0; t < V::T0; ++t) {
        auto const operand = [&](int q) {
            uint4 const wq = *reinterpret_cast<uint4 const*>(&lds.w[q][t][lane][0]);
            return v4i{ int(wq.x), int(wq.y), int(wq.z), int(wq.w) };
        };
        v4i const A = operand(0);
        v4i const C = *reinterpret_cast<v4i const*>(&lds.bias[t][g][0]);
        v4f const Sc = *reinterpret_cast<v4f const*>(&lds.scale[t][g][0]);
        if constexpr (V::FP8_WEIGHTS) {
            // three planes: two blocks at a time, so that twenty-four accumulator registers are live, not forty-eight
            v4i const A1 = operand(V::PLANES > 1 ? 1 : 0), A2 = operand(V::PLANES > 2 ? 2 : 0);
            v4i const Z = v4i{ 0, 0, 0, 0 };
            auto const half = [&](auto first) __attribute__((always_inline)) {
                constexpr int FIRST = decltype(first)::value;
                wave_priority<kPrioMatrix>();
                if (t > 0) pending.template convert_into<FIRST, 2>(Hout, t - 1);
                v4i D0[2], D1[2], D2[2];
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    D0[k] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, X[FIRST + k], C, 0, 0, 0);
                    D1[k] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A1, X[FIRST + k], Z, 0, 0, 0);
                    D2[k] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A2, X[FIRST + k], Z, 0, 0, 0);
                }
                if (t > 0) { interleave<2, 3, 4>(); keep_here<FIRST, 2>(Hout, t - 1); }
                section_end();
                wave_priority<kPrioPlain>();
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    v4i Dh;
#pragma unroll
                    for (int r = 0; r < 4; ++r)                // 4096*D2 + 64*D1 + D0, wrapping like int32
                        Dh[r] = int((((uint32_t(D2[k][r]) << 6) + uint32_t(D1[k][r])) << 6) + uint32_t(D0[k][r]));
                    activate_scale4(Dh, Sc, pending.z[FIRST + k]);
                }
                section_end();
            };
            half(std::integral_constant<int, 0>{});
            half(std::integral_constant<int, 2>{});
            continue;
        }
        wave_priority<kPrioMatrix>();
        if (t > 0) pending.convert_into(Hout, t - 1);
        v4i Dh[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) Dh[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, X[b], C, 0, 0, 0);
        if (t > 0) { interleave<4, 1, 4>(); keep_here(Hout, t - 1); }
        section_end();
        wave_priority<kPrioPlain>();
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            if constexpr (MAGIC) {
                v4f acc;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    int32_t const bits = Dh[b][r];               // (a copy: bit_cast of a vector element expression reads element 0)
                    acc[r] = __builtin_bit_cast(float, bits) - 12582912.f;
                }
                activate_scale4(acc, Sc, pending.z[b]);
            } else {
                activate_scale4(Dh[b], Sc, pending.z[b]);
            }
        }
        section_end();
    }
}

// The network for the 64 texels of one wave with layers 1..3 on the fp16 matrix instruction.  `in` is the lane's own
// texel (lane = 16*b + j).  On return D[b] holds, for lane (j = lane%16, g = lane/16), the accumulators of output
// channels 4g..4g+3 of texel 16*b + j as floats (exact integers), and S their scales.
template <class V>
__device__ __forceinline__ void mlp_forward_f16(LdsT<V>& lds, int wave, int lane, bool l0Magic, uint32_t const (&in)[16], v4f (&D)[4], v4f& S)
{
    int const g = lane >> 4;
    v4i X[4];
    transpose_inputs<V>(lds, wave, lane, in, X);
    section_end();

    uint32_t Ha[4][4][2], Hb[4][4][2];
    PendingTile pending;
    if constexpr (V::FP8_WEIGHTS) {
        first_layer<V, false>(lds, lane, X, Ha, pending);
    } else {
        if (l0Magic) first_layer<V, true>(lds, lane, X, Ha, pending);      // uniform
        else         first_layer<V, false>(lds, lane, X, Ha, pending);
    }
    f16_hidden_layer<V, V::T0, V::T1, V::FP8_WEIGHTS>(lds, V::F16_L1, V::T0, lane, Ha, Hb, pending);
    f16_hidden_layer<V, V::T1, V::T2, V::FP8_WEIGHTS>(lds, V::F16_L2, V::T0 + V::T1, lane, Hb, Ha, pending);

    constexpr int outTile = V::T0 + V::T1 + V::T2;
    v4f const C = *reinterpret_cast<v4f const*>(&lds.bias[outTile][g][0]);
    S = *reinterpret_cast<v4f const*>(&lds.scale[outTile][g][0]);
    wave_priority<kPrioMatrix>();
    pending.convert_into(Ha, V::T2 - 1);
#pragma unroll
    for (int b = 0; b < 4; ++b) D[b] = C;
    f16_tile<V, V::T2>(lds, V::F16_L3, 0, lane, Ha, D);
    section_end();
    wave_priority<kPrioOther>();
}

// Two workgroups of eight waves per CU: sixteen waves, 128 VGPRs each, four to a SIMD.
template <class V>
__global__ void __launch_bounds__(V::THREADS, V::WAVES_PER_SIMD)
decode_kernel(DevMip const* __restrict__ mips, int numMips, int totalTiles)
{
    __shared__ LdsT<V> lds;
    constexpr int GROUP = V::WAVES / 4;                      // quartets of a workgroup
    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const member = wave >> 2;                            // which quartet this wave belongs to
    int const j = lane & 15, g = lane >> 4;

    // Contiguous share of the tile list for this workgroup.  Workgroups are dealt to the eight dies (XCDs) of the
    // device in turn, and each die has a cache of its own: the shares are numbered so that a die's workgroups hold
    // neighbouring shares - one eighth of the list per die - and the grid rows that vertically adjacent shares both
    // read come from memory once per die, not once per share.
    int const per = (totalTiles + gridDim.x - 1) / gridDim.x;
    constexpr int kDies = 8;
    int const share = (gridDim.x % kDies == 0) ? int(blockIdx.x % kDies) * int(gridDim.x / kDies) + int(blockIdx.x / kDies) : int(blockIdx.x);
    int const tileBegin = share * per;
    int const tileEnd = min(totalTiles, tileBegin + per);

    {   // 2-bit code bytes -> input bytes: code q maps to 85*q - 128 (255/3 = 85)
        uint32_t x = threadIdx.x & 0xffu;
        x = (x | (x << 12)) & 0x000f000fu;
        x = (x | (x << 6))  & 0x03030303u;
        lds.lut2[threadIdx.x & 0xffu] = (x * 85u) ^ 0x80808080u;
    }

    build_posenc_tables<V>(lds);

    uint8_t const* stagedBlob = nullptr;
    int staged = 0;                                          // uniform: how layers 1..3 of the staged set run (kStagedF16, ...)
    int entry = 0;

    // One wave tile: the 32 x 2 texels of this wave in tile (tileX, tileY) of mip m: block b of 16 texels begins at
    // (x0 + 16 * (b & 1), y0 + (b >> 1)).  (With 16 x 4 texels per wave the two 64-byte halves of an output line came
    // from two waves, at different times, and the L2 wrote 5 - 10 % of the halves back twice; so each line now comes
    // from one wave's consecutive stores and the write traffic is exactly the output's size.)
    auto decode_wave_tile = [&](RunMip const& m, int tileX, int tileY, int sub) __attribute__((always_inline)) {
        int const x0 = tileX * 64 + (sub & 1) * 32;
        int const y0 = tileY * 4 + (sub >> 1) * 2;
        if (x0 >= m.width || y0 >= m.height) return;         // whole wave tile outside the image

        // ---- 1. input stage: lane = texel (block g = lane/16, column j = lane%16 of the block)
        wave_priority<kPrioOther>();
        uint32_t in[16];
        {
            int const x = min(x0 + j + 16 * (g & 1), m.width - 1), y = min(y0 + (g >> 1), m.height - 1);
            if (m.fast) prepare_inputs_fast<V>(m.full, lds, x, y, in);
            else        prepare_inputs_general<V>(m.full, x, y, in);
        }
        // ---- 2.-4. transpose, hidden layers, output layer
        if (V::F16_LAYERS && (staged & kStagedF16)) {
            v4f D[4];
            v4f S;
            mlp_forward_f16<V>(lds, wave, lane, (staged & kL0Magic) != 0, in, D, S);
            // a wave tile inside the image, channels in whole groups of four (pixel formats: vector stores possible),
            // takes the stores without tests
            bool const inside = x0 + 32 <= m.width && y0 + 2 <= m.height && (m.numChannels & 3) == 0
                             && (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS || m.vectorStores);
            if (!inside) {
                store_tile_general(&m.full, D[0], D[1], D[2], D[3], S, x0 + j, y0, 4 * g);
            } else if (staged & kOutputsBounded) {
                if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS)  store_tile_inside<NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS, false>(m, D, S, x0, y0, j, g);
                else if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PIXELS)   store_tile_inside<NTC_HIP_DEV_OUT_FP16_PIXELS, false>(m, D, S, x0, y0, j, g);
                else                                                   store_tile_inside<NTC_HIP_DEV_OUT_UNORM8_PIXELS, false>(m, D, S, x0, y0, j, g);
            } else {
                if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS)  store_tile_inside<NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS, true>(m, D, S, x0, y0, j, g);
                else if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PIXELS)   store_tile_inside<NTC_HIP_DEV_OUT_FP16_PIXELS, true>(m, D, S, x0, y0, j, g);
                else                                                   store_tile_inside<NTC_HIP_DEV_OUT_UNORM8_PIXELS, true>(m, D, S, x0, y0, j, g);
            }
        } else {
            // every layer on the int8 matrix instruction: one 16-texel block at a time
            write_inputs<V>(lds, wave, lane, in);
#pragma unroll 1
            for (int b = 0; b < 4; ++b) {
                v4i D;
                v4f S;
                int laneB = lane;
                asm volatile("" : "+v"(laneB));                  // keeps the weight reads inside the loop (hoisted, they take every register)
                mlp_forward_block<V>(lds, laneB, read_input_block<V>(lds, wave, lane, b), D, S);
                store_row_any_format(m, D, S, x0 + j + 16 * (b & 1), y0 + (b >> 1), 4 * g);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    };

    // The workgroup walks its share in segments of tiles that use one weight blob (a single segment, unless sets of
    // a batch meet inside the share); inside a segment each quartet walks a contiguous part, so that its next tile
    // is a neighbour of its last one and finds the cache lines they share in place, and the four waves of a quartet
    // write whole lines together.  (Quartets that took alternate tiles of one sequence drifted apart in time, and
    // latent reads from memory doubled; waves that each walked wave tiles of their own wrote 12 % more bytes to
    // memory, half lines at a time.)
    for (int segBegin = tileBegin; segBegin < tileEnd; ) {
        while (entry + 1 < numMips && mips[entry + 1].tileStart <= segBegin) ++entry;
        uint8_t const* const blob = mips[entry].weights;
        int segEnd = tileEnd;
        for (int k = entry + 1; k < numMips && mips[k].tileStart < tileEnd; ++k)
            if (mips[k].weights != blob) { segEnd = mips[k].tileStart; break; }
        if (blob != stagedBlob) {                            // uniform across the workgroup
            __syncthreads();                                 // every wave has left the previous segment's weights
            staged = __builtin_amdgcn_readfirstlane(stage_weights<V>(lds, blob, wave * 64 + lane_id()));
            stagedBlob = blob;
            __syncthreads();                                 // also publishes the tables built above
        }
        int const part = (segEnd - segBegin + GROUP - 1) / GROUP;
        int const myBegin = segBegin + member * part, myEnd = min(segEnd, myBegin + part);
        // The quartet steps through its tiles mip by mip, keeping the tile's place in the mip in registers: no
        // look-up in the table (a vector load and a wait for every outstanding store, per tile) and no division.
        int mine = entry, nextStart = 0, tilesX = 1, tileX = 0, tileY = 0;
        auto enter_mip_of = [&](int tile) {
            while (mine + 1 < numMips && mips[mine + 1].tileStart <= tile) ++mine;
            nextStart = mine + 1 < numMips ? mips[mine + 1].tileStart : 0x7fffffff;
            tilesX = mips[mine].tilesX;
            int const local = tile - mips[mine].tileStart;
            tileY = local / tilesX; tileX = local - tileY * tilesX;
        };
        for (int tile = myBegin; tile < myEnd; ) {           // one run of tiles per mip: the mip's fields stay in registers
            enter_mip_of(tile);
            RunMip const m(mips[mine]);
            int const runEnd = min(myEnd, nextStart);
            for (; tile < runEnd; ++tile) {
                decode_wave_tile(m, tileX, tileY, wave & 3);
                if (++tileX == tilesX) { tileX = 0; ++tileY; }
            }
        }
        segBegin = segEnd;
    }
}

// Random-access decode ("inference on sample", NtcSampleTextureSet of Inference.hlsli:282-357):
// one query = (u, v, mip) -> the 16 outputs of texel (floor(u*W), floor(v*H)) of that mip, clamped to
// the image, as 16 fp16.  Lane = query in the input stage (each lane carries its own mip, so the
// per-lane form of either input stage is used); the network is the same 64-column tile as in raster decode.
// A query whose mip is out of range writes zeros.
template <class V>
__global__ void __launch_bounds__(V::THREADS, V::WAVES_PER_SIMD)
query_kernel(DevMip const* __restrict__ mips, int numMips, DevQuery const* __restrict__ queries, uint64_t numQueries,
             uint16_t* __restrict__ out)
{
    __shared__ LdsT<V> lds;
    __shared__ QueryMip qmips[16];
    if (threadIdx.x < 16) {
        DevMip const& d = mips[min(int(threadIdx.x), numMips - 1)];
        QueryMip& q = qmips[threadIdx.x];
        q.hr = d.hr; q.lr = d.lr;
        q.hrAxisX = d.hrAxisX; q.hrAxisY = d.hrAxisY; q.lrAxisX = d.lrAxisX; q.lrAxisY = d.lrAxisY;
        q.hrWidth = d.hrWidth; q.hrHeight = d.hrHeight; q.lrWidth = d.lrWidth; q.lrHeight = d.lrHeight;
        q.width = d.width; q.height = d.height;
        q.posMask = d.posMask; q.fast = d.fast; q.positionLod = d.positionLod;
        q.hrBricks = d.hrBricks; q.lrBricks = d.lrBricks;
    }
    bool const bricked = mips[0].hrBricks != nullptr;          // a set has the query-ordered copy for all of its mips or for none
    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const j = lane & 15, g = lane >> 4;


    {   // 2-bit code bytes -> input bytes (see decode_kernel)
        uint32_t x = threadIdx.x & 0xffu;
        x = (x | (x << 12)) & 0x000f000fu;
        x = (x | (x << 6))  & 0x03030303u;
        lds.lut2[threadIdx.x & 0xffu] = (x * 85u) ^ 0x80808080u;
    }
    build_posenc_tables<V>(lds);
    int const staged = __builtin_amdgcn_readfirstlane(stage_weights<V>(lds, mips[0].weights, wave * 64 + lane_id()));
    bool const useF16 = (staged & kStagedF16) != 0;
    __syncthreads();

    uint64_t const numBlocks = (numQueries + V::THREADS - 1) / V::THREADS;
    for (uint64_t block = blockIdx.x; block < numBlocks; block += gridDim.x) {
        uint64_t const q0 = block * V::THREADS + uint64_t(wave) * 64;
        if (q0 >= numQueries) continue;
        uint64_t const qi = min(q0 + uint64_t(lane), numQueries - 1);
        DevQuery const query = queries[qi];
        bool const validMip = query.mip >= 0 && query.mip < numMips;
        QueryMip const& m = qmips[validMip ? query.mip : 0];
        int x = int(floorf(query.u * float(m.width)));
        int y = int(floorf(query.v * float(m.height)));
        x = max(0, min(x, m.width - 1));
        y = max(0, min(y, m.height - 1));
        uint32_t in[16];
        if (__all(m.fast != 0)) {                                // every lane's mip is power-of-two sized
            if (bricked) prepare_inputs_bricked<V>(m, lds, x, y, in);
            else         prepare_inputs_scattered<V>(m, lds, x, y, (GlobalU8Ptr)mips, in);
        }
        else                    prepare_inputs_general<V>(mips[validMip ? query.mip : 0], x, y, in);

        // lane (j, g) holds channels 4g..4g+3 of query q0 + 16b + j; validity travels by shuffle
        auto store_outputs = [&](auto checked, int b, v4f Fb, v4f S) __attribute__((always_inline)) {
            constexpr bool CHECKED = decltype(checked)::value;
            uint64_t const q = q0 + uint64_t(16 * b + j);
            int const ok = __shfl(validMip ? 1 : 0, 16 * b + j, 64);
            if (q >= numQueries) return;
            uint32_t h01 = to_half2_bits<CHECKED>(Fb[0] * S[0], Fb[1] * S[1]);
            uint32_t h23 = to_half2_bits<CHECKED>(Fb[2] * S[2], Fb[3] * S[3]);
            if (!ok) { h01 = 0; h23 = 0; }
            *reinterpret_cast<u32x2*>(out + q * 16 + 4 * g) = u32x2{ h01, h23 };
        };
        if (V::F16_LAYERS && useF16) {
            // output-layer accumulators as floats: exact integers below 2^24
            v4f F[4];
            v4f S;
            mlp_forward_f16<V>(lds, wave, lane, (staged & kL0Magic) != 0, in, F, S);
            if (staged & kOutputsBounded) {                                                  // as in decode_kernel
#pragma unroll
                for (int b = 0; b < 4; ++b) store_outputs(std::false_type{}, b, F[b], S);
            } else {
#pragma unroll
                for (int b = 0; b < 4; ++b) store_outputs(std::true_type{}, b, F[b], S);
            }
        } else {
            // every layer on the int8 matrix instruction, one 16-query block at a time; the int32 -> float
            // conversion of the accumulators is the definition's
            write_inputs<V>(lds, wave, lane, in);
#pragma unroll 1
            for (int b = 0; b < 4; ++b) {
                v4i D;
                v4f S;
                int laneB = lane;
                asm volatile("" : "+v"(laneB));                  // keeps the weight reads inside the loop
                mlp_forward_block<V>(lds, laneB, read_input_block<V>(lds, wave, lane, b), D, S);
                store_outputs(std::true_type{}, b, v4f{ float(D[0]), float(D[1]), float(D[2]), float(D[3]) }, S);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
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

// D = A * B + C with the fp16 MFMA and the operand layouts the decode kernel assumes: for K = 32,
// A[i][k] sits in lane i + 16*(k/8), element k%8 (B alike with column j), for K = 16 in lane
// i + 16*(k/4), element k%4; D[i][j] in lane j + 16*(i/4), element i%4.
__global__ void selftest_mfma_f16_kernel(_Float16 const* __restrict__ a, _Float16 const* __restrict__ b,
                                         float const* __restrict__ c, float* __restrict__ d, int depth)
{
    int const lane = threadIdx.x & 63;
    int const ij = lane & 15, g = lane >> 4;
    v4f C;
#pragma unroll
    for (int r = 0; r < 4; ++r) C[r] = c[(4 * g + r) * 16 + ij];
    v4f D;
    if (depth == 32) {
        v8h A, B;
#pragma unroll
        for (int e = 0; e < 8; ++e) { A[e] = a[ij * 32 + 8 * g + e]; B[e] = b[(8 * g + e) * 16 + ij]; }
        D = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, C, 0, 0, 0);
    } else {
        v4h A, B;
#pragma unroll
        for (int e = 0; e < 4; ++e) { A[e] = a[ij * 16 + 4 * g + e]; B[e] = b[(4 * g + e) * 16 + ij]; }
        D = __builtin_amdgcn_mfma_f32_16x16x16f16(A, B, C, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) d[(4 * g + r) * 16 + ij] = D[r];
}

// ---- host-callable launchers ------------------------------------------------------------

using VCfg01  = Variant<1, 8, 2, 8, 16, 16, 0, 64, 64, 48, 32>;   // 2x2 concat 8x2-bit + bilinear 16x4-bit
using VCfg2   = Variant<1, 8, 2, 8, 12, 12, 0, 64, 48, 48, 32>;   // faster decoder, 12 low-res features
using VRef16  = Variant<0, 16, 4, 16, 16, 16, 2, 48, 64, 48, 32>; // LibNTC 0.9.2 geometry, 16 features
using VRef12  = Variant<0, 12, 4, 16, 12, 16, 2, 48, 64, 48, 32>;
using VRef8   = Variant<0, 8, 4, 16, 8, 16, 2, 48, 64, 48, 32>;
using VRef4   = Variant<0, 4, 4, 16, 4, 16, 2, 48, 64, 48, 32>;
using VCfg3   = Variant<0, 16, 4, 16, 16, 16, 2, 48, 64, 64, 64, true>;   // wide decoder, e4m3 hidden-layer weights

template <class V>
static hipError_t launch_variant(DevMip const* mips, int numMips, int totalTiles, int gridSize, hipStream_t stream)
{
    hipLaunchKernelGGL(decode_kernel<V>, dim3(gridSize), dim3(V::THREADS), 0, stream, mips, numMips, totalTiles);
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
    case NTC_HIP_VARIANT_CFG3_FP8: return launch_variant<VCfg3>(mips, numMips, totalTiles, gridSize, stream);
    default: return hipErrorInvalidValue;
    }
}

template <class V>
static hipError_t launch_query_variant(DevMip const* mips, int numMips, DevQuery const* queries, uint64_t numQueries,
                                       uint16_t* out, int gridSize, hipStream_t stream)
{
    hipLaunchKernelGGL(query_kernel<V>, dim3(gridSize), dim3(V::THREADS), 0, stream, mips, numMips, queries, numQueries, out);
    return hipGetLastError();
}

// Plain grid ([layer][row][column] u16) -> bricks; one thread per stored u16, reads coalesced.
__global__ void __launch_bounds__(256)
build_bricks_kernel(uint16_t const* __restrict__ src, uint16_t* __restrict__ dst, int width, int height, int layers, int sideLog2)
{
    size_t const cells = size_t(width) * size_t(height);
    size_t const i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= cells * size_t(layers)) return;
    int const layer = int(i / cells);
    size_t const cell = i - size_t(layer) * cells;
    uint32_t const cy = uint32_t(cell / size_t(width)), cx = uint32_t(cell - size_t(cy) * size_t(width));
    uint32_t const side = 1u << sideLog2, bricksX = (uint32_t(width) + side - 1u) >> sideLog2;
    size_t const brick = size_t(cy >> sideLog2) * bricksX + (cx >> sideLog2);
    size_t const inBrick = ((cy & (side - 1u)) << sideLog2) + (cx & (side - 1u));
    dst[(brick * (size_t(1) << (2 * sideLog2)) + inBrick) * size_t(layers) + size_t(layer)] = src[i];
}

hipError_t launch_build_bricks(uint16_t const* src, uint8_t* dst, int width, int height, int layers, hipStream_t stream)
{
    size_t const count = size_t(width) * size_t(height) * size_t(layers);
    hipLaunchKernelGGL(build_bricks_kernel, dim3(unsigned((count + 255) / 256)), dim3(256), 0, stream,
                       src, reinterpret_cast<uint16_t*>(dst), width, height, layers, brick_side_log2(layers));
    return hipGetLastError();
}

hipError_t launch_queries(int variant, DevMip const* mips, int numMips, DevQuery const* queries, uint64_t numQueries,
                          uint16_t* out, int gridSize, hipStream_t stream)
{
    switch (variant) {
    case NTC_HIP_VARIANT_CFG01: return launch_query_variant<VCfg01>(mips, numMips, queries, numQueries, out, gridSize, stream);
    case NTC_HIP_VARIANT_CFG2:  return launch_query_variant<VCfg2>(mips, numMips, queries, numQueries, out, gridSize, stream);
    case NTC_HIP_VARIANT_REF16: return launch_query_variant<VRef16>(mips, numMips, queries, numQueries, out, gridSize, stream);
    case NTC_HIP_VARIANT_REF12: return launch_query_variant<VRef12>(mips, numMips, queries, numQueries, out, gridSize, stream);
    case NTC_HIP_VARIANT_REF8:  return launch_query_variant<VRef8>(mips, numMips, queries, numQueries, out, gridSize, stream);
    case NTC_HIP_VARIANT_REF4:  return launch_query_variant<VRef4>(mips, numMips, queries, numQueries, out, gridSize, stream);
    case NTC_HIP_VARIANT_CFG3_FP8: return launch_query_variant<VCfg3>(mips, numMips, queries, numQueries, out, gridSize, stream);
    default: return hipErrorInvalidValue;
    }
}

template <class V>
static int occupancy_variant()
{
    int blocks = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, decode_kernel<V>, V::THREADS, 0) != hipSuccess || blocks < 1) blocks = 2;
    return blocks;
}

// Workgroups of the variant's kernel that fit on one compute unit (registers and LDS).
int resident_workgroups_per_cu(int variant)
{
    switch (variant) {
    case NTC_HIP_VARIANT_CFG01: return occupancy_variant<VCfg01>();
    case NTC_HIP_VARIANT_CFG2:  return occupancy_variant<VCfg2>();
    case NTC_HIP_VARIANT_REF16: return occupancy_variant<VRef16>();
    case NTC_HIP_VARIANT_REF12: return occupancy_variant<VRef12>();
    case NTC_HIP_VARIANT_REF8:  return occupancy_variant<VRef8>();
    case NTC_HIP_VARIANT_REF4:  return occupancy_variant<VRef4>();
    case NTC_HIP_VARIANT_CFG3_FP8: return occupancy_variant<VCfg3>();
    default: return 2;
    }
}

int tiles_per_round(int) { return VCfg01::WAVES / 4; }
int threads_per_workgroup(int) { return VCfg01::THREADS; }

hipError_t launch_selftest_mfma(int8_t const* a, int8_t const* b, int32_t* d, hipStream_t stream)
{
    hipLaunchKernelGGL(selftest_mfma_kernel, dim3(1), dim3(64), 0, stream, a, b, d);
    return hipGetLastError();
}

hipError_t launch_selftest_mfma_f16(uint16_t const* a, uint16_t const* b, float const* c, float* d, int depth, hipStream_t stream)
{
    hipLaunchKernelGGL(selftest_mfma_f16_kernel, dim3(1), dim3(64), 0, stream,
                       reinterpret_cast<_Float16 const*>(a), reinterpret_cast<_Float16 const*>(b), c, d, depth);
    return hipGetLastError();
}

} // namespace ntc_hip_dev
