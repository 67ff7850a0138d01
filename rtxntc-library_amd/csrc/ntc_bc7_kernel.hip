// ntc_bc7_kernel.hip - BC7 block compression of a decoded image (gfx950).
//
// The reference's BC7 pass (IContext::MakeBlockCompressionComputePass with BlockCompressedFormat::BC7,
// src/shaders/CompressBC7.hlsl) as a compute kernel: one lane encodes one 4 x 4 block.
//
// Full search, per block: opaque blocks try the three-subset modes 0 and 2 and the two-subset modes
// 1 and 3, each on the partition whose bounding-box endpoints give the smallest estimated error over
// all 64 partitions; every block then tries modes 4 and 5 in the four channel rotations, mode 6 and
// mode 7.  A candidate = bounding-box endpoints per subset (ends paired by covariance sign), two
// rounds of least-squares refinement, quantisation with the mode's p-bit rule, indices along the
// dequantised endpoints; its error is measured on what a decoder will show, and it replaces the
// current block when the error is not larger.  With a mode buffer (9 bits per block: mode and
// partition, MakeBC7ModeBuffer) only that candidate is encoded and no error is computed.
//
// All float arithmetic is IEEE binary32, unfused, in the order written here.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <float.h>
#include "ntc_decode_kernel.h"
#include "ntc_bc_source.h"

namespace ntc_hip_dev {

namespace {

#define BC7_INLINE __device__ __forceinline__

// Table.P2 and Table.P3 of the BPTC format specification (ARB_texture_compression_bptc), packed: the
// subset of texel t in bits 2t, 2t+1.  Anchor tables A2, A3a, A3b of the same specification.
__constant__ uint32_t kTwoSubsets[64] = {
    0x50505050u, 0x40404040u, 0x54545454u, 0x54505040u, 0x50404000u, 0x55545450u, 0x55545040u, 0x54504000u,
    0x50400000u, 0x55555450u, 0x55544000u, 0x54400000u, 0x55555440u, 0x55550000u, 0x55555500u, 0x55000000u,
    0x55150100u, 0x00004054u, 0x15010000u, 0x00405054u, 0x00004050u, 0x15050100u, 0x05010000u, 0x40505054u,
    0x00404050u, 0x05010100u, 0x14141414u, 0x05141450u, 0x01155440u, 0x00555500u, 0x15014054u, 0x05414150u,
    0x44444444u, 0x55005500u, 0x11441144u, 0x05055050u, 0x05500550u, 0x11114444u, 0x41144114u, 0x44111144u,
    0x15055054u, 0x01055040u, 0x05041050u, 0x05455150u, 0x14414114u, 0x50050550u, 0x41411414u, 0x00141400u,
    0x00041504u, 0x00105410u, 0x10541000u, 0x04150400u, 0x50410514u, 0x41051450u, 0x05415014u, 0x14054150u,
    0x41050514u, 0x41505014u, 0x40011554u, 0x54150140u, 0x50505500u, 0x00555050u, 0x15151010u, 0x54540404u,
};
__constant__ uint32_t kThreeSubsets[64] = {
    0xaa685050u, 0x6a5a5040u, 0x5a5a4200u, 0x5450a0a8u, 0xa5a50000u, 0xa0a05050u, 0x5555a0a0u, 0x5a5a5050u,
    0xaa550000u, 0xaa555500u, 0xaaaa5500u, 0x90909090u, 0x94949494u, 0xa4a4a4a4u, 0xa9a59450u, 0x2a0a4250u,
    0xa5945040u, 0x0a425054u, 0xa5a5a500u, 0x55a0a0a0u, 0xa8a85454u, 0x6a6a4040u, 0xa4a45000u, 0x1a1a0500u,
    0x0050a4a4u, 0xaaa59090u, 0x14696914u, 0x69691400u, 0xa08585a0u, 0xaa821414u, 0x50a4a450u, 0x6a5a0200u,
    0xa9a58000u, 0x5090a0a8u, 0xa8a09050u, 0x24242424u, 0x00aa5500u, 0x24924924u, 0x24499224u, 0x50a50a50u,
    0x500aa550u, 0xaaaa4444u, 0x66660000u, 0xa5a0a5a0u, 0x50a050a0u, 0x69286928u, 0x44aaaa44u, 0x66666600u,
    0xaa444444u, 0x54a854a8u, 0x95809580u, 0x96969600u, 0xa85454a8u, 0x80959580u, 0xaa141414u, 0x96960000u,
    0xaaaa1414u, 0xa05050a0u, 0xa0a5a5a0u, 0x96000000u, 0x40804080u, 0xa9a8a9a8u, 0xaaaaaa44u, 0x2a4a5254u,
};
__constant__ uint8_t kAnchorSecondOfTwo[64] = {
    15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15,
    15,  2,  8,  2,  2,  8,  8, 15,  2,  8,  2,  2,  8,  8,  2,  2,
    15, 15,  6,  8,  2,  8, 15, 15,  2,  8,  2,  2,  2, 15, 15,  6,
     6,  2,  6,  8, 15, 15,  2,  2, 15, 15, 15, 15, 15,  2,  2, 15,
};
__constant__ uint8_t kAnchorSecondOfThree[64] = {
     3,  3, 15, 15,  8,  3, 15, 15,  8,  8,  6,  6,  6,  5,  3,  3,
     3,  3,  8, 15,  3,  3,  6, 10,  5,  8,  8,  6,  8,  5, 15, 15,
     8, 15,  3,  5,  6, 10,  8, 15, 15,  3, 15,  5, 15, 15, 15, 15,
     3, 15,  5,  5,  5,  8,  5, 10,  5, 10,  8, 13, 15, 12,  3,  3,
};
__constant__ uint8_t kAnchorThirdOfThree[64] = {
    15,  8,  8,  3, 15, 15,  3,  8, 15, 15, 15, 15, 15, 15, 15,  8,
    15,  8, 15,  3, 15,  8, 15,  8,  3, 15,  6, 10, 15, 15, 10,  8,
    15,  3, 15, 10, 10,  8,  9, 10,  6, 15,  8, 15,  3,  6,  6,  8,
    15,  3, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15,  3, 15, 15,  8,
};
// Subset masks in "spread" form: bit 2t set when texel t belongs to the subset.
constexpr uint32_t kAllTexels = 0x55555555u;
BC7_INLINE uint32_t spread_mask(uint32_t partitionWord, uint32_t subset)
{
    uint32_t const x = partitionWord ^ (subset * kAllTexels);
    return ~(x | (x >> 1)) & kAllTexels;
}
BC7_INLINE bool has_texel(uint32_t mask, int t) { return (mask >> (2 * t)) & 1u; }

template <int SUBSETS> BC7_INLINE uint32_t partition_word(int partition)
{
    if constexpr (SUBSETS == 1) return 0u;
    else if constexpr (SUBSETS == 2) return kTwoSubsets[partition];
    else return kThreeSubsets[partition];
}
template <int SUBSETS> BC7_INLINE int subset_anchor(int partition, int s)
{
    if (s == 0) return 0;
    if constexpr (SUBSETS == 2) return kAnchorSecondOfTwo[partition];
    else if constexpr (SUBSETS == 3) return s == 1 ? kAnchorSecondOfThree[partition] : kAnchorThirdOfThree[partition];
    else return 0;
}

template <int C> struct Color { float c[C]; };
template <int C> struct Quantized { int c[C]; };

BC7_INLINE float saturate(float v) { return fminf(fmaxf(v, 0.f), 1.f); }        // a NaN becomes 0
template <int C> BC7_INLINE float dot(Color<C> const& a, Color<C> const& b)
{
    float s = a.c[0] * b.c[0];
#pragma unroll
    for (int k = 1; k < C; ++k) s += a.c[k] * b.c[k];
    return s;
}
template <int C> BC7_INLINE Color<C> sub(Color<C> const& a, Color<C> const& b)
{
    Color<C> r;
#pragma unroll
    for (int k = 0; k < C; ++k) r.c[k] = a.c[k] - b.c[k];
    return r;
}

template <int C> BC7_INLINE void min_max(Color<C> const (&px)[16], uint32_t mask, Color<C>& lo, Color<C>& hi)
{
#pragma unroll
    for (int k = 0; k < C; ++k) { lo.c[k] = FLT_MAX; hi.c[k] = -FLT_MAX; }
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if (has_texel(mask, t)) {
#pragma unroll
            for (int k = 0; k < C; ++k) { lo.c[k] = min_f32(lo.c[k], px[t].c[k]); hi.c[k] = max_f32(hi.c[k], px[t].c[k]); }
        }
}

// With the first component whose ends differ as the axis, the ends of later components are swapped
// where their covariance with the axis is negative.
template <int C> BC7_INLINE void orient(Color<C> const (&px)[16], uint32_t mask, Color<C>& e0, Color<C>& e1)
{
    Color<C> center;
#pragma unroll
    for (int k = 0; k < C; ++k) center.c[k] = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if (has_texel(mask, t)) {
#pragma unroll
            for (int k = 0; k < C; ++k) center.c[k] += px[t].c[k];
        }
    float const count = float(__popc(mask));
#pragma unroll
    for (int k = 0; k < C; ++k) center.c[k] /= count;
    float cov[C][C];
#pragma unroll
    for (int a = 0; a < C; ++a)
#pragma unroll
        for (int b = 0; b < C; ++b) cov[a][b] = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if (has_texel(mask, t)) {
            Color<C> const d = sub(px[t], center);
#pragma unroll
            for (int a = 0; a < C; ++a)
#pragma unroll
                for (int b = a + 1; b < C; ++b) cov[a][b] += d.c[a] * d.c[b];
        }
    bool done = false;
#pragma unroll
    for (int a = 0; a + 1 < C; ++a) {
        if (!done && e0.c[a] != e1.c[a]) {
#pragma unroll
            for (int b = a + 1; b < C; ++b)
                if (cov[a][b] < 0.f) { float const t = e0.c[b]; e0.c[b] = e1.c[b]; e1.c[b] = t; }
            done = true;
        }
    }
}

// Two rounds of: project the texels on the endpoint axis, snap to the index grid, solve the
// least-squares problem for new endpoints.  Components sitting exactly on 0 or 1 stay.
template <int C> BC7_INLINE void refine(Color<C> const (&px)[16], uint32_t mask, Color<C>& e0, Color<C>& e1, int indexBits)
{
    float const scale = float((1u << indexBits) - 1u), iscale = 1.f / scale;
#pragma unroll 1
    for (int iter = 0; iter < 2; ++iter) {
        Color<C> const axis = sub(e1, e0);
        float mul = dot(axis, axis);
        if (mul > 0.f) mul = 1.f / mul;
        float a2 = 0.f, b2 = 0.f, ab = 0.f;
        Color<C> ax, bx;
#pragma unroll
        for (int k = 0; k < C; ++k) ax.c[k] = bx.c[k] = 0.f;
#pragma unroll
        for (int t = 0; t < 16; ++t)
            if (has_texel(mask, t)) {
                float const f = saturate(dot(sub(px[t], e0), axis) * mul);
                float const beta = rintf(f * scale) * iscale, alpha = 1.f - beta;
                a2 += alpha * alpha; b2 += beta * beta; ab += alpha * beta;
#pragma unroll
                for (int k = 0; k < C; ++k) { ax.c[k] += alpha * px[t].c[k]; bx.c[k] += beta * px[t].c[k]; }
            }
        float const denom = a2 * b2 - ab * ab;
        if (!(fabsf(denom) > 0.0001f)) break;
        float const factor = 1.f / denom;
#pragma unroll
        for (int k = 0; k < C; ++k) {
            float const a = saturate((ax.c[k] * b2 - bx.c[k] * ab) * factor), b = saturate((bx.c[k] * a2 - ax.c[k] * ab) * factor);
            if (!(e0.c[k] == 0.f || e0.c[k] == 1.f)) e0.c[k] = a;
            if (!(e1.c[k] == 0.f || e1.c[k] == 1.f)) e1.c[k] = b;
        }
    }
}

// Squared error of the subset if every texel took the nearest of the 2^indexBits points between the
// (unquantised) endpoints.
template <int C> BC7_INLINE float estimate(Color<C> const (&px)[16], uint32_t mask, Color<C> const& e0, Color<C> const& e1, int indexBits)
{
    Color<C> const axis = sub(e1, e0);
    float mul = dot(axis, axis);
    if (mul > 0.f) mul = 1.f / mul;
    float const maxIndex = float((1u << indexBits) - 1u), indexScale = 1.f / maxIndex;
    float error = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if (has_texel(mask, t)) {
            Color<C> const p = sub(px[t], e0);
            float f = dot(p, axis) * mul;
            f = rintf(f * maxIndex) * indexScale;
            Color<C> diff;
#pragma unroll
            for (int k = 0; k < C; ++k) diff.c[k] = f * axis.c[k] - p.c[k];
            error += dot(diff, diff);
        }
    return error;
}

BC7_INLINE int quantize(float v, int bits) { return int(rintf(saturate(v) * float((1u << bits) - 1u))); }
BC7_INLINE int expand8(int q, int bits) { return (q << (8 - bits)) | (q >> (2 * bits - 8)); }

// Squared error of the subset as a decoder reconstructs it (integer interpolation with 6-bit weights).
template <int C> BC7_INLINE float decoded_error(Color<C> const (&px)[16], int const (&index)[16], uint32_t mask, Quantized<C> q0, Quantized<C> q1,
                                                int indexBits, int endpointBits)
{
#pragma unroll
    for (int k = 0; k < C; ++k) { q0.c[k] = expand8(q0.c[k], endpointBits); q1.c[k] = expand8(q1.c[k], endpointBits); }
    float const indexScale = 64.f / float((1u << indexBits) - 1u);
    float error = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if (has_texel(mask, t)) {
            int const w = int(rintf(float(index[t]) * indexScale));
            Color<C> diff;
#pragma unroll
            for (int k = 0; k < C; ++k) diff.c[k] = float((q0.c[k] * (64 - w) + q1.c[k] * w + 32) >> 6) / 255.f - px[t].c[k];
            error += dot(diff, diff);
        }
    return error;
}

// Indices of the subset's texels along the dequantised endpoints.  A decoder assumes the top index bit
// of the anchor texel to be 0: if it is 1 all indices of the subset are complemented and true is
// returned (the caller swaps the endpoints).
template <int C> BC7_INLINE bool assign(Color<C> const (&px)[16], uint32_t mask, int anchor, int indexBits, int endpointBits,
                                        Quantized<C> const& q0, Quantized<C> const& q1, int (&index)[16])
{
    Color<C> e0, e1;
#pragma unroll
    for (int k = 0; k < C; ++k) { e0.c[k] = float(expand8(q0.c[k], endpointBits)) / 255.f; e1.c[k] = float(expand8(q1.c[k], endpointBits)) / 255.f; }
    Color<C> const axis = sub(e1, e0);
    float mul = dot(axis, axis);
    if (mul > 0.f) mul = 1.f / mul;
    bool flip = false;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if (has_texel(mask, t)) {
            index[t] = quantize(dot(sub(px[t], e0), axis) * mul, indexBits);
            if (t == anchor) flip = (index[t] >> (indexBits - 1)) & 1;
        }
    int const all = (1 << indexBits) - 1;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if (flip && has_texel(mask, t)) index[t] ^= all;
    return flip;
}

struct Bits {
    uint64_t lo = 0, hi = 0;
    int at = 0;
    BC7_INLINE void put(int length, uint32_t value)
    {
        uint64_t const v = value & ((1u << length) - 1u);
        if (at < 64) { lo |= v << at; if (at + length > 64) hi |= v >> (64 - at); }
        else hi |= v << (at - 64);
        at += length;
    }
};

struct Best { float error; uint64_t lo, hi; };

enum { kNoPBit = 0, kPBitPerEndpoint = 1, kPBitPerSubset = 2 };
template <int ID, int SUBSETS_, int PARTITION_BITS, int ENDPOINT_BITS /* with the p-bit */, int INDEX_BITS, int PBIT>
struct Mode {
    static constexpr int id = ID, subsets = SUBSETS_, partitionBits = PARTITION_BITS, endpointBits = ENDPOINT_BITS, indexBits = INDEX_BITS, pbit = PBIT;
};
using Mode0 = Mode<0, 3, 4, 5, 3, kPBitPerEndpoint>;
using Mode1 = Mode<1, 2, 6, 7, 3, kPBitPerSubset>;
using Mode2 = Mode<2, 3, 6, 5, 2, kNoPBit>;
using Mode3 = Mode<3, 2, 6, 8, 2, kPBitPerEndpoint>;
using Mode6 = Mode<6, 1, 0, 8, 4, kPBitPerEndpoint>;
using Mode7 = Mode<7, 2, 6, 6, 2, kPBitPerEndpoint>;

// Endpoint quantisation with the mode's p-bit rule: the shared lowest bit is the majority of the
// components' lowest bits; with alpha, an alpha of exactly 1 forces it to 1 and a quantised alpha of 0
// to 0, which keeps both exact.
template <class M, int C> BC7_INLINE void quantize_endpoints(Color<C> const (&e)[2 * M::subsets], Quantized<C> (&q)[2 * M::subsets])
{
    constexpr int N = 2 * M::subsets;
#pragma unroll
    for (int i = 0; i < N; ++i)
#pragma unroll
        for (int k = 0; k < C; ++k) q[i].c[k] = quantize(e[i].c[k], M::endpointBits);
    if constexpr (M::pbit == kPBitPerEndpoint) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            int odd = 0;
#pragma unroll
            for (int k = 0; k < C; ++k) odd += q[i].c[k] & 1;
            int lsb = odd >= 2 ? 1 : 0;
            if constexpr (C == 4) lsb = ((odd >= 2 && q[i].c[3] != 0) || e[i].c[3] == 1.f) ? 1 : 0;
#pragma unroll
            for (int k = 0; k < C; ++k) q[i].c[k] = (q[i].c[k] & 0xFE) | lsb;
        }
    } else if constexpr (M::pbit == kPBitPerSubset) {
#pragma unroll
        for (int i = 0; i < N; i += 2) {
            int odd = 0;
#pragma unroll
            for (int k = 0; k < C; ++k) odd += (q[i].c[k] & 1) + (q[i + 1].c[k] & 1);
            int const lsb = odd >= 4 ? 1 : 0;
#pragma unroll
            for (int k = 0; k < C; ++k) { q[i].c[k] = (q[i].c[k] & 0xFE) | lsb; q[i + 1].c[k] = (q[i + 1].c[k] & 0xFE) | lsb; }
        }
    }
}

// Refines the start endpoints of every subset, quantises, assigns indices and, if the result is not
// worse than the best so far (always, with a fixed mode), encodes the block.
template <class M, int C> BC7_INLINE void finish(Color<C> const (&px)[16], int partition, Color<C> const (&start)[2 * M::subsets], bool fixedMode, Best& best)
{
    constexpr int N = 2 * M::subsets;
    uint32_t const word = partition_word<M::subsets>(partition);
    Color<C> e[N];
    Quantized<C> q[N];
#pragma unroll
    for (int i = 0; i < N; ++i) e[i] = start[i];
#pragma unroll
    for (int s = 0; s < M::subsets; ++s) refine(px, spread_mask(word, s), e[2 * s], e[2 * s + 1], M::indexBits);
    quantize_endpoints<M, C>(e, q);
    int index[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) index[t] = 0;
    int anchors[M::subsets];
    float error = 0.f;
#pragma unroll
    for (int s = 0; s < M::subsets; ++s) {
        uint32_t const mask = spread_mask(word, s);
        anchors[s] = subset_anchor<M::subsets>(partition, s);
        if (assign(px, mask, anchors[s], M::indexBits, M::endpointBits, q[2 * s], q[2 * s + 1], index)) {
            Quantized<C> const t = q[2 * s]; q[2 * s] = q[2 * s + 1]; q[2 * s + 1] = t;
        }
        if (!fixedMode) {
            float const e2 = decoded_error(px, index, mask, q[2 * s], q[2 * s + 1], M::indexBits, M::endpointBits);
            error = s == 0 ? e2 : error + e2;
        }
    }
    if (error > best.error) return;
    Bits b;
    b.put(M::id + 1, 1u << M::id);
    b.put(M::partitionBits, uint32_t(partition));
    constexpr int drop = M::pbit == kNoPBit ? 0 : 1;
#pragma unroll
    for (int k = 0; k < C; ++k)
#pragma unroll
        for (int i = 0; i < N; ++i) b.put(M::endpointBits - drop, uint32_t(q[i].c[k]) >> drop);
    if constexpr (M::pbit == kPBitPerEndpoint) {
#pragma unroll
        for (int i = 0; i < N; ++i) b.put(1, uint32_t(q[i].c[0]));
    }
    if constexpr (M::pbit == kPBitPerSubset) {
#pragma unroll
        for (int s = 0; s < M::subsets; ++s) b.put(1, uint32_t(q[2 * s].c[0]));
    }
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        bool anchor = t == 0;
#pragma unroll
        for (int s = 1; s < M::subsets; ++s) anchor = anchor || t == anchors[s];
        b.put(anchor ? M::indexBits - 1 : M::indexBits, uint32_t(index[t]));
    }
    best.error = error; best.lo = b.lo; best.hi = b.hi;
}

// The partition with the smallest estimated error (the first of equals) over [first, last) and its
// start endpoints: per subset the bounding box, oriented if asked.  A range of one partition is taken
// as it is.
template <int SUBSETS, int C> BC7_INLINE int pick_partition(Color<C> const (&px)[16], bool orientEnds, int searchIndexBits, int first, int last,
                                                            Color<C> (&bestEnds)[2 * SUBSETS])
{
    int bestPartition = first;
    float bestError = FLT_MAX;
    bool const single = last - first == 1;
    // a NaN texel makes every estimate NaN and no partition "best": the endpoints are then zero
#pragma unroll
    for (int i = 0; i < 2 * SUBSETS; ++i)
#pragma unroll
        for (int k = 0; k < C; ++k) bestEnds[i].c[k] = 0.f;
#pragma unroll 1
    for (int p = first; p < last; ++p) {
        uint32_t const word = partition_word<SUBSETS>(p);
        Color<C> e[2 * SUBSETS];
        float error = 0.f;
#pragma unroll
        for (int s = 0; s < SUBSETS; ++s) {
            uint32_t const mask = spread_mask(word, s);
            min_max(px, mask, e[2 * s], e[2 * s + 1]);
            if (orientEnds) orient(px, mask, e[2 * s], e[2 * s + 1]);
        }
        if (!single) {
#pragma unroll
            for (int s = 0; s < SUBSETS; ++s) {
                float const e2 = estimate(px, spread_mask(word, s), e[2 * s], e[2 * s + 1], searchIndexBits);
                error = s == 0 ? e2 : error + e2;
            }
        }
        if (single || error < bestError) {
            bestPartition = p; bestError = error;
#pragma unroll
            for (int i = 0; i < 2 * SUBSETS; ++i) bestEnds[i] = e[i];
        }
    }
    return bestPartition;
}

// Modes 4 and 5: a colour plane of three channels and a scalar plane, each with its own endpoints and
// indices; the scalar plane takes channel {A, R, G, B}[rotation] and alpha takes its place.
BC7_INLINE void dual_plane(int mode, bool wideColorIndex, Color<4> const (&rgba)[16], uint32_t rotation, bool fixedMode, Best& best)
{
    int const colorIndexBits = mode == 5 ? 2 : (wideColorIndex ? 3 : 2), alphaIndexBits = mode == 5 ? 2 : (wideColorIndex ? 2 : 3);
    int const colorBits = mode == 5 ? 7 : 5, alphaBits = mode == 5 ? 8 : 6;
    Color<3> rgb[16];
    Color<1> a[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        Color<4> const& p = rgba[t];
        rgb[t].c[0] = rotation == 1 ? p.c[3] : p.c[0];
        rgb[t].c[1] = rotation == 2 ? p.c[3] : p.c[1];
        rgb[t].c[2] = rotation == 3 ? p.c[3] : p.c[2];
        a[t].c[0] = rotation == 0 ? p.c[3] : rotation == 1 ? p.c[0] : rotation == 2 ? p.c[1] : p.c[2];
    }
    Color<1> a0, a1;
    min_max(a, kAllTexels, a0, a1);
    refine(a, kAllTexels, a0, a1, alphaIndexBits);
    Color<3> e0, e1;
    min_max(rgb, kAllTexels, e0, e1);
    orient(rgb, kAllTexels, e0, e1);
    refine(rgb, kAllTexels, e0, e1, colorIndexBits);
    Quantized<3> q0, q1;
#pragma unroll
    for (int k = 0; k < 3; ++k) { q0.c[k] = quantize(e0.c[k], colorBits); q1.c[k] = quantize(e1.c[k], colorBits); }
    Quantized<1> qa0, qa1;
    qa0.c[0] = quantize(a0.c[0], alphaBits); qa1.c[0] = quantize(a1.c[0], alphaBits);
    int colorIndex[16], alphaIndex[16];
    float error = 0.f;
    if (assign(rgb, kAllTexels, 0, colorIndexBits, colorBits, q0, q1, colorIndex)) { Quantized<3> const t = q0; q0 = q1; q1 = t; }
    if (!fixedMode) error = decoded_error(rgb, colorIndex, kAllTexels, q0, q1, colorIndexBits, colorBits);
    if (assign(a, kAllTexels, 0, alphaIndexBits, alphaBits, qa0, qa1, alphaIndex)) { Quantized<1> const t = qa0; qa0 = qa1; qa1 = t; }
    if (!fixedMode) error += decoded_error(a, alphaIndex, kAllTexels, qa0, qa1, alphaIndexBits, alphaBits);
    if (error > best.error) return;
    Bits b;
    b.put(mode + 1, 1u << mode);
    b.put(2, rotation);
    if (mode == 4) b.put(1, wideColorIndex ? 1u : 0u);
#pragma unroll
    for (int k = 0; k < 3; ++k) { b.put(colorBits, uint32_t(q0.c[k])); b.put(colorBits, uint32_t(q1.c[k])); }
    b.put(alphaBits, uint32_t(qa0.c[0])); b.put(alphaBits, uint32_t(qa1.c[0]));
    // mode 4 stores its 2-bit indices first, then the 3-bit ones; mode 5 colour first, then the scalar
    bool const alphaFirst = mode == 4 && wideColorIndex;
    int const firstBits = alphaFirst ? alphaIndexBits : colorIndexBits, secondBits = alphaFirst ? colorIndexBits : alphaIndexBits;
#pragma unroll
    for (int t = 0; t < 16; ++t) b.put(t == 0 ? firstBits - 1 : firstBits, uint32_t(alphaFirst ? alphaIndex[t] : colorIndex[t]));
#pragma unroll
    for (int t = 0; t < 16; ++t) b.put(t == 0 ? secondBits - 1 : secondBits, uint32_t(alphaFirst ? colorIndex[t] : alphaIndex[t]));
    best.error = error; best.lo = b.lo; best.hi = b.hi;
}

// One block.  FIXED false: every mode is tried; true: only fixedMode with fixedPartition (for modes 4 / 5:
// rotation in bits 0-1 of the partition, "wide colour index" in bit 2).  Both cases run through the same
// code, the fixed one with every range narrowed to one candidate.  (Two instantiations because in the
// full search every lane of a wave walks the same partitions, so the subset masks are uniform and the
// texel loops branch on scalar bits instead of being predicated per lane.)
template <bool FIXED>
BC7_INLINE void bc7_encode(Color<4> const (&px)[16], int fixedMode, int fixedPartition, uint64_t& lo, uint64_t& hi)
{
    constexpr bool fixed = FIXED;
    Best best{ FLT_MAX, 0, 0 };
    bool opaque = true;
#pragma unroll
    for (int t = 0; t < 16; ++t) if (px[t].c[3] < 1.f) opaque = false;
    int const firstPartition = fixed ? fixedPartition : 0, lastPartition = fixed ? fixedPartition + 1 : 64;

    if (fixed ? (fixedMode <= 3) : opaque) {
        Color<3> rgb[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) { rgb[t].c[0] = px[t].c[0]; rgb[t].c[1] = px[t].c[1]; rgb[t].c[2] = px[t].c[2]; }
        if (!fixed || fixedMode == 0 || fixedMode == 2) {
            Color<3> ends[6];
            int const p = pick_partition<3>(rgb, true, 3, firstPartition, lastPartition, ends);
            if (fixed ? fixedMode == 0 : p < 16) finish<Mode0>(rgb, p, ends, fixed, best);
            if (!fixed || fixedMode == 2) finish<Mode2>(rgb, p, ends, fixed, best);
        }
        if (!fixed || fixedMode == 1 || fixedMode == 3) {
            Color<3> ends[4];
            int const p = pick_partition<2>(rgb, true, 3, firstPartition, lastPartition, ends);
            if (!fixed || fixedMode == 1) finish<Mode1>(rgb, p, ends, fixed, best);
            if (!fixed || fixedMode == 3) finish<Mode3>(rgb, p, ends, fixed, best);
        }
    }
    if (!fixed || fixedMode == 4 || fixedMode == 5) {
        uint32_t const firstRotation = fixed ? uint32_t(fixedPartition) & 3u : 0u, lastRotation = fixed ? firstRotation + 1u : 4u;
#pragma unroll 1
        for (uint32_t rotation = firstRotation; rotation < lastRotation; ++rotation) {
            if (!fixed || (fixedMode == 4 && !(fixedPartition & 4))) dual_plane(4, false, px, rotation, fixed, best);
            if (!fixed || (fixedMode == 4 && (fixedPartition & 4))) dual_plane(4, true, px, rotation, fixed, best);
            if (!fixed || fixedMode == 5) dual_plane(5, false, px, rotation, fixed, best);
        }
    }
    if (!fixed || fixedMode == 6) {
        Color<4> ends[2];
        pick_partition<1>(px, true, 4, 0, 1, ends);
        finish<Mode6>(px, 0, ends, fixed, best);
    }
    if (!fixed || fixedMode == 7) {
        Color<4> ends[4];
        int const p = pick_partition<2>(px, false, 2, firstPartition, lastPartition, ends);
        finish<Mode7>(px, p, ends, fixed, best);
    }
    lo = best.lo; hi = best.hi;
}

BC7_INLINE void load_block(BlockCompressArgs const& a, int bx, int by, Color<4> (&px)[16])
{
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        int const x = a.srcLeft + bx * 4 + (t & 3), y = a.srcTop + by * 4 + (t >> 2);
        source_pixel(a, x, y, px[t].c);
    }
}
BC7_INLINE void store_block(BlockCompressArgs const& a, int bx, int by, uint64_t lo, uint64_t hi)
{
    uint64_t* const dst = reinterpret_cast<uint64_t*>(a.dst + size_t(by + a.dstOffsetY) * a.dstRowPitch) + size_t(bx + a.dstOffsetX) * 2;
    dst[0] = lo; dst[1] = hi;
}

} // namespace

// Full search.  8 x 8 blocks per 64-thread group, registers capped at 256 so that two waves share a SIMD:
// the search is a long chain of scalar branches over uniform subset masks, and a second wave fills the
// issue slots the first one leaves (1.7 times faster than one wave with 263 registers; three waves
// with 168 registers spill and gain nothing more).
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2)))
bc7_compress_kernel(BlockCompressArgs a)
{
    int const bx = blockIdx.x * 8 + (threadIdx.x & 7), by = blockIdx.y * 8 + (threadIdx.x >> 3);
    if (bx >= a.widthInBlocks || by >= a.heightInBlocks) return;
    Color<4> px[16];
    load_block(a, bx, by, px);
    uint64_t lo, hi;
    bc7_encode<false>(px, -1, 0, lo, hi);
    store_block(a, bx, by, lo, hi);
}

// With a mode buffer.  A workgroup covers 16 x 16 blocks; its threads first read their blocks' entries,
// then trade blocks through LDS so that thread i takes the i-th block in order of mode: the waves of the
// group then run (nearly) one mode each instead of every mode some lane of theirs happens to have
// (the reference's ReorderThreadsByMode, CompressBC7.hlsl:1445-1509).  Which thread encodes which block
// depends on the order the LDS counters are hit in; what is written for a block does not.
// Three waves per SIMD (168 registers) serve this kernel best: 0.40 ms with two, 0.34 ms with three, 0.48 ms with four.
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3)))
bc7_compress_modes_kernel(BlockCompressArgs a)
{
    __shared__ uint32_t counts[8];
    __shared__ uint32_t tasks[8][256];
    if (threadIdx.x < 8) counts[threadIdx.x] = 0;
    __syncthreads();
    {
        int const bx = blockIdx.x * 16 + (threadIdx.x & 15), by = blockIdx.y * 16 + (threadIdx.x >> 4);
        if (bx < a.widthInBlocks && by < a.heightInBlocks) {
            // 9 bits per block of the mode map; 0 = no entry, 0x1BF stands for mode 0 partition 0
            int64_t const mx = int64_t(bx) + a.modeMapOffsetX, my = int64_t(by) + a.modeMapOffsetY;
            uint32_t entry = 0;
            if (mx >= 0 && my >= 0 && mx < a.modeMapWidthInBlocks && my < a.modeMapHeightInBlocks) {
                uint64_t const bit = (uint64_t(my) * uint64_t(a.modeMapWidthInBlocks) + uint64_t(mx)) * 9u;
                uint32_t const* words = a.modeBuffer + (bit >> 5);
                uint32_t const shift = uint32_t(bit & 31u);
                entry = words[0] >> shift;
                if (shift > 23u) entry |= words[1] << (32u - shift);
                entry &= 0x1FFu;
            }
            if (entry == 0u) {
                store_block(a, bx, by, 0x0001f00000f80004ull, 0x1f9e00003ff0001full);     // the reference's marker: black, red, green and blue squares
            } else {
                if (entry == 0x1BFu) entry = 0u;
                uint32_t const mode = (entry >> 6) & 7u;
                uint32_t const slot = atomicAdd(&counts[mode], 1u);
                tasks[mode][slot] = ((entry & 63u) << 8) | threadIdx.x;
            }
        }
    }
    __syncthreads();
    uint32_t rank = threadIdx.x, task = 0;
    int mode = -1;
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        uint32_t const n = counts[m];
        if (mode < 0) {
            if (rank < n) { mode = m; task = tasks[m][rank]; }
            else rank -= n;
        }
    }
    if (mode < 0) return;
    int const bx = blockIdx.x * 16 + int(task & 15u), by = blockIdx.y * 16 + int((task >> 4) & 15u);
    Color<4> px[16];
    load_block(a, bx, by, px);
    uint64_t lo, hi;
    bc7_encode<true>(px, mode, int(task >> 8), lo, hi);
    store_block(a, bx, by, lo, hi);
}

hipError_t launch_bc7_compress(BlockCompressArgs const& a, hipStream_t stream)
{
    if (a.modeBuffer) {
        dim3 const grid((a.widthInBlocks + 15) / 16, (a.heightInBlocks + 15) / 16);
        hipLaunchKernelGGL(bc7_compress_modes_kernel, grid, dim3(256), 0, stream, a);
    } else {
        dim3 const grid((a.widthInBlocks + 7) / 8, (a.heightInBlocks + 7) / 8);
        hipLaunchKernelGGL(bc7_compress_kernel, grid, dim3(64), 0, stream, a);
    }
    return hipGetLastError();
}

} // namespace ntc_hip_dev
