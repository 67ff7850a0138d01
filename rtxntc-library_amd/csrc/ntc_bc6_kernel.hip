// ntc_bc6_kernel.hip - BC6H (unsigned half float) block compression of a decoded image (gfx950).
//
// The reference's BC6 pass (IContext::MakeBlockCompressionComputePass with BlockCompressedFormat::BC6,
// src/shaders/CompressBC6.hlsl) as a compute kernel: one lane encodes one 4 x 4 block.  Two candidates,
// the smaller luminance-weighted mean squared log2 error wins:
//   * one subset, 10-bit endpoints, 4-bit indices (mode 11 of the format): bounding box, pulled inwards in
//     log2 space by at most 1/32 of its extent, one least-squares refit in half-code space;
//   * two subsets with 3-bit indices on the partition (of the format's first 32) whose texels lie closest
//     to the diagonals of the subsets' bounding boxes; endpoints stored as 7-bit base + 6-bit deltas (mode
//     2) or 9-bit base + 5-bit deltas (mode 6), whichever decodes closer.
// Where the shader uses the hardware's log2 / exp2 / rcp / rsqrt, this kernel uses the functions below,
// built from plain binary32 operations (and correctly rounded division and square root), so that the CPU
// checker can reproduce every bit.  Half conversion rounds to nearest even.  Texels are clamped to
// [0, 65504] (a NaN becomes 0).  All float arithmetic is unfused, in the order written here.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ntc_decode_kernel.h"
#include "ntc_bc_source.h"

namespace ntc_hip_dev {

namespace {

#define BC6_INLINE __device__ __forceinline__

// The format's first 32 two-subset partitions (Table.P2 of the BPTC specification): bit t = subset of
// texel t; and the anchor texel of the second subset (table A2).
__constant__ uint16_t kSecondSubset[32] = {
    0xcccc, 0x8888, 0xeeee, 0xecc8, 0xc880, 0xfeec, 0xfec8, 0xec80, 0xc800, 0xffec, 0xfe80, 0xe800, 0xffe8, 0xff00, 0xfff0, 0xf000,
    0xf710, 0x008e, 0x7100, 0x08ce, 0x008c, 0x7310, 0x3100, 0x8cce, 0x088c, 0x3110, 0x6666, 0x366c, 0x17e8, 0x0ff0, 0x718e, 0x399c,
};
__constant__ uint8_t kSecondAnchor[32] = { 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 15, 2, 8, 2, 2, 8, 8, 15, 2, 8, 2, 2, 8, 8, 2, 2 };

// log2 for x >= 0 (0 -> -inf); NaN for a negative or NaN argument.  Argument reduction to [sqrt(1/2), sqrt 2),
// then the series of atanh; a few units in the last place.
BC6_INLINE float det_log2(float x)
{
    if (!(x >= 0.f)) return __uint_as_float(0x7fc00000u);
    if (x == 0.f) return __uint_as_float(0xff800000u);
    uint32_t b = __float_as_uint(x);
    if (b >= 0x7f800000u) return x;
    int e = 0;
    if (b < 0x00800000u) { x *= 8388608.f; b = __float_as_uint(x); e = -23; }
    e += int(b >> 23) - 127;
    float m = __uint_as_float((b & 0x007fffffu) | 0x3f800000u);
    if (m > 1.41421354f) { m *= 0.5f; e += 1; }
    float const t = (m - 1.f) / (m + 1.f), t2 = t * t;
    float p = t2 * (1.f / 9.f) + (1.f / 7.f);
    p = p * t2 + 0.2f;
    p = p * t2 + (1.f / 3.f);
    p = p * t2 + 1.f;
    return float(e) + p * t * 2.88539004f;
}

// 2^x: +inf from 128, 0 below -150.
BC6_INLINE float det_exp2(float x)
{
    if (x != x) return x;
    if (x >= 128.f) return __uint_as_float(0x7f800000u);
    if (x < -150.f) return 0.f;
    float const n = rintf(x), g = (x - n) * 0.693147182f;
    float p = g * (1.f / 5040.f) + (1.f / 720.f);
    p = p * g + (1.f / 120.f);
    p = p * g + (1.f / 24.f);
    p = p * g + (1.f / 6.f);
    p = p * g + 0.5f;
    p = p * g + 1.f;
    p = p * g + 1.f;
    int k = int(n);
    if (k > 127) { p *= 2.f; k -= 1; }
    if (k < -126) { p *= 5.96046448e-08f; k += 24; }
    return p * __uint_as_float(uint32_t(k + 127) << 23);
}

struct V3 { float x, y, z; };
BC6_INLINE V3 operator+(V3 a, V3 b) { return { a.x + b.x, a.y + b.y, a.z + b.z }; }
BC6_INLINE V3 operator-(V3 a, V3 b) { return { a.x - b.x, a.y - b.y, a.z - b.z }; }
BC6_INLINE V3 operator*(V3 a, float s) { return { a.x * s, a.y * s, a.z * s }; }
BC6_INLINE V3 operator*(V3 a, V3 b) { return { a.x * b.x, a.y * b.y, a.z * b.z }; }
BC6_INLINE float dot(V3 a, V3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
BC6_INLINE V3 vmin(V3 a, V3 b) { return { min_f32(a.x, b.x), min_f32(a.y, b.y), min_f32(a.z, b.z) }; }
BC6_INLINE V3 vmax(V3 a, V3 b) { return { max_f32(a.x, b.x), max_f32(a.y, b.y), max_f32(a.z, b.z) }; }
BC6_INLINE float clampf(float v, float lo, float hi) { return fminf(fmaxf(v, lo), hi); }
// A float as the number of its half-precision bit pattern, and back (the latter truncates to an integer first).
// (a NaN always gives the code 0x7e00, whatever its sign and payload)
BC6_INLINE float to_half_bits(float v) { return v != v ? 32256.f : float(__builtin_bit_cast(uint16_t, _Float16(v))); }
BC6_INLINE float from_half_bits(float v) { return float(__builtin_bit_cast(_Float16, uint16_t(uint32_t(v)))); }
BC6_INLINE V3 to_half_bits(V3 v) { return { to_half_bits(v.x), to_half_bits(v.y), to_half_bits(v.z) }; }

constexpr float kHalfMax = 65504.f;
constexpr float kHalfMaxCode = 31743.f;         // 0x7bff, the code of 65504

BC6_INLINE float msle(V3 a, V3 b)
{
    V3 const d{ det_log2((b.x + 1.f) / (a.x + 1.f)), det_log2((b.y + 1.f) / (a.y + 1.f)), det_log2((b.z + 1.f) / (a.z + 1.f)) };
    V3 const sq = d * d * V3{ 0.299f, 0.587f, 0.114f };
    return sq.x + sq.y + sq.z;
}

BC6_INLINE V3 quantize(V3 v, float levels)
{
    V3 const h = to_half_bits(v);
    return { (h.x * levels) / 31744.f, (h.y * levels) / 31744.f, (h.z * levels) / 31744.f };
}
BC6_INLINE V3 unquantize(V3 v, float levels)
{
    return { (v.x * 65536.f + 32768.f) / levels, (v.y * 65536.f + 32768.f) / levels, (v.z * 65536.f + 32768.f) / levels };
}
BC6_INLINE V3 interpolate(V3 e0, V3 e1, float weight)
{
    V3 const c = (e0 * (64.f - weight) + e1 * weight + V3{ 32.f, 32.f, 32.f }) * (31.f / 4096.f);
    return { from_half_bits(c.x), from_half_bits(c.y), from_half_bits(c.z) };
}
BC6_INLINE uint32_t index_of(float pos, float e0, float e1, float scale, float bias, float top)
{
    float const r = (pos - e0) / (e1 - e0);
    return uint32_t(clampf(r * scale + bias + 0.5f, 0.f, top));      // a NaN (coinciding ends) gives 0
}
BC6_INLINE uint32_t index3(float pos, float e0, float e1) { return index_of(pos, e0, e1, 6.98182f, 0.00909f, 7.f); }
BC6_INLINE uint32_t index4(float pos, float e0, float e1) { return index_of(pos, e0, e1, 14.93333f, 0.03333f, 15.f); }
BC6_INLINE V3 direction(V3 lo, V3 hi) { V3 const d = hi - lo; float const s = d.x + d.y + d.z; return { d.x / s, d.y / s, d.z / s }; }

BC6_INLINE float log1(float c) { return det_log2(c + 1.f); }
BC6_INLINE float exp1(float c) { return det_exp2(c) - 1.f; }

// Pulls the box inwards in log2(1 + x) space: towards the smallest / largest values that are not the
// extremes themselves, by at most 1/32 of the extent.
BC6_INLINE void inset_box(V3 const (&px)[16], V3& lo, V3& hi)
{
    V3 innerLo = hi, innerHi = lo;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        V3 const p = px[t];
        innerLo = vmin(innerLo, V3{ p.x == lo.x ? innerLo.x : p.x, p.y == lo.y ? innerLo.y : p.y, p.z == lo.z ? innerLo.z : p.z });
        innerHi = vmax(innerHi, V3{ p.x == hi.x ? innerHi.x : p.x, p.y == hi.y ? innerHi.y : p.y, p.z == hi.z ? innerHi.z : p.z });
    }
    V3 const logInnerHi{ log1(innerHi.x), log1(innerHi.y), log1(innerHi.z) }, logInnerLo{ log1(innerLo.x), log1(innerLo.y), log1(innerLo.z) };
    V3 logHi{ log1(hi.x), log1(hi.y), log1(hi.z) }, logLo{ log1(lo.x), log1(lo.y), log1(lo.z) };
    V3 const ext = (logHi - logLo) * (1.f / 32.f);
    logLo = logLo + vmin(logInnerLo - logLo, ext);
    logHi = logHi - vmin(logHi - logInnerHi, ext);
    lo = V3{ exp1(logLo.x), exp1(logLo.y), exp1(logLo.z) };
    hi = V3{ exp1(logHi.x), exp1(logHi.y), exp1(logHi.z) };
}

// Least-squares endpoints, in half-code space, for the indices the current endpoints give to the texels
// of `members` (bit t = texel t takes part).  False when the system is singular.
template <bool FOUR_BIT>
BC6_INLINE bool refit(V3 const (&px)[16], uint32_t members, V3 lo, V3 hi, V3& outLo, V3& outHi)
{
    V3 const dir = direction(lo, hi);
    float const e0 = to_half_bits(dot(lo, dir)), e1 = to_half_bits(dot(hi, dir));
    V3 alphaSum{ 0.f, 0.f, 0.f }, betaSum{ 0.f, 0.f, 0.f };
    float ab = 0.f, aa = 0.f, bb = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if ((members >> t) & 1u) {
            float const pos = to_half_bits(dot(px[t], dir));
            uint32_t const index = FOUR_BIT ? index4(pos, e0, e1) : index3(pos, e0, e1);
            float const beta = clampf(float(index) / (FOUR_BIT ? 15.f : 7.f), 0.f, 1.f), alpha = 1.f - beta;
            V3 const h = to_half_bits(px[t]);
            alphaSum = alphaSum + h * alpha; betaSum = betaSum + h * beta;
            ab += alpha * beta; aa += alpha * alpha; bb += beta * beta;
        }
    float const det = aa * bb - ab * ab;
    if (!(fabsf(det) > 0.00001f)) return false;
    float const rcp = 1.f / det;
    V3 const a = (alphaSum * bb - betaSum * ab) * rcp, b = (betaSum * aa - alphaSum * ab) * rcp;
    // (the shader clamps these codes to 65504, which lets the codes of infinities and NaNs through)
    outLo = V3{ from_half_bits(clampf(a.x, 0.f, kHalfMaxCode)), from_half_bits(clampf(a.y, 0.f, kHalfMaxCode)), from_half_bits(clampf(a.z, 0.f, kHalfMaxCode)) };
    outHi = V3{ from_half_bits(clampf(b.x, 0.f, kHalfMaxCode)), from_half_bits(clampf(b.y, 0.f, kHalfMaxCode)), from_half_bits(clampf(b.z, 0.f, kHalfMaxCode)) };
    return true;
}

struct Block { uint64_t lo, hi; float error; };

// 128-bit field writer for constant positions.
struct Bits {
    uint64_t lo = 0, hi = 0;
    BC6_INLINE void put(int at, uint32_t value, int n)
    {
        uint64_t const v = value & ((1u << n) - 1u);
        if (at < 64) { lo |= v << at; if (at + n > 64) hi |= v >> (64 - at); }
        else hi |= v << (at - 64);
    }
};

BC6_INLINE Block encode_one_subset(V3 const (&px)[16])
{
    V3 lo = px[0], hi = px[0];
#pragma unroll
    for (int t = 1; t < 16; ++t) { lo = vmin(lo, px[t]); hi = vmax(hi, px[t]); }
    V3 const boxLo = lo, boxHi = hi;
    inset_box(px, lo, hi);
    V3 fitLo, fitHi;
    if (refit<true>(px, 0xffffu, lo, hi, fitLo, fitHi)) {
        lo = vmin(vmax(fitLo, boxLo), boxHi);
        hi = vmin(vmax(fitHi, boxLo), boxHi);
    }
    V3 const dir = direction(lo, hi);
    V3 q0 = quantize(lo, 1024.f), q1 = quantize(hi, 1024.f);
    float e0 = to_half_bits(dot(lo, dir)), e1 = to_half_bits(dot(hi, dir));
    if (index4(to_half_bits(dot(px[0], dir)), e0, e1) > 7) {
        float const t = e0; e0 = e1; e1 = t;
        V3 const q = q0; q0 = q1; q1 = q;
    }
    V3 const u0 = unquantize(q0, 1024.f), u1 = unquantize(q1, 1024.f);
    Bits b;
    b.put(0, 0x03, 5);
    b.put(5, uint32_t(q0.x), 10); b.put(15, uint32_t(q0.y), 10); b.put(25, uint32_t(q0.z), 10);
    b.put(35, uint32_t(q1.x), 10); b.put(45, uint32_t(q1.y), 10); b.put(55, uint32_t(q1.z), 10);
    float error = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        uint32_t const index = index4(to_half_bits(dot(px[t], dir)), e0, e1);
        error += msle(px[t], interpolate(u0, u1, floorf((float(index) * 64.f) / 15.f + 0.5f)));
        b.put(t == 0 ? 65 : 64 + 4 * t, index, t == 0 ? 3 : 4);
    }
    return Block{ b.lo, b.hi, error };
}

BC6_INLINE void subset_boxes(V3 const (&px)[16], uint32_t second, V3 (&lo)[2], V3 (&hi)[2])
{
#pragma unroll
    for (int s = 0; s < 2; ++s) { lo[s] = V3{ kHalfMax, kHalfMax, kHalfMax }; hi[s] = V3{ 0.f, 0.f, 0.f }; }
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        if ((second >> t) & 1u) { lo[1] = vmin(lo[1], px[t]); hi[1] = vmax(hi[1], px[t]); }
        else                    { lo[0] = vmin(lo[0], px[t]); hi[0] = vmax(hi[0], px[t]); }
    }
}

BC6_INLINE V3 normalized(V3 v) { float const len = sqrtf(dot(v, v)); return { v.x / len, v.y / len, v.z / len }; }
BC6_INLINE float distance_to_line2(V3 origin, V3 dir, V3 p)
{
    V3 const w = p - origin, x = w - dir * dot(w, dir);
    return dot(x, x);
}

// Sum of the texels' squared distances from the diagonal of their subset's bounding box.
BC6_INLINE float pattern_score(V3 const (&px)[16], uint32_t second)
{
    V3 lo[2], hi[2];
    subset_boxes(px, second, lo, hi);
    V3 const dir0 = normalized(hi[0] - lo[0]), dir1 = normalized(hi[1] - lo[1]);
    float total = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        total += ((second >> t) & 1u) ? distance_to_line2(lo[1], dir1, px[t]) : distance_to_line2(lo[0], dir0, px[t]);
    return total;
}

BC6_INLINE uint32_t field(float v, int bits) { return uint32_t(int(v)) & ((1u << bits) - 1u); }      // two's complement of a small integer
BC6_INLINE V3 floor3(V3 v) { return { floorf(v.x), floorf(v.y), floorf(v.z) }; }
BC6_INLINE V3 clamp3(V3 v, float limit) { return { clampf(v.x, -limit, limit), clampf(v.y, -limit, limit), clampf(v.z, -limit, limit) }; }

BC6_INLINE void encode_two_subsets(V3 const (&px)[16], int pattern, Block& best)
{
    uint32_t const second = kSecondSubset[pattern];
    int const anchor1 = kSecondAnchor[pattern];
    V3 lo[2], hi[2];
    subset_boxes(px, second, lo, hi);
    {
        V3 fitLo, fitHi;
        if (refit<false>(px, ~second & 0xffffu, lo[0], hi[0], fitLo, fitHi)) { lo[0] = fitLo; hi[0] = fitHi; }
        if (refit<false>(px, second, lo[1], hi[1], fitLo, fitHi)) { lo[1] = fitLo; hi[1] = fitHi; }
    }
    V3 const dir0 = direction(lo[0], hi[0]), dir1 = direction(lo[1], hi[1]);
    float e00 = to_half_bits(dot(lo[0], dir0)), e01 = to_half_bits(dot(hi[0], dir0));
    float e10 = to_half_bits(dot(lo[1], dir1)), e11 = to_half_bits(dot(hi[1], dir1));
    V3 anchorTexel = px[0];
#pragma unroll
    for (int t = 1; t < 16; ++t) if (t == anchor1) anchorTexel = px[t];
    if (index3(to_half_bits(dot(px[0], dir0)), e00, e01) > 3) { float const t = e00; e00 = e01; e01 = t; V3 const v = lo[0]; lo[0] = hi[0]; hi[0] = v; }
    if (index3(to_half_bits(dot(anchorTexel, dir1)), e10, e11) > 3) { float const t = e10; e10 = e11; e11 = t; V3 const v = lo[1]; lo[1] = hi[1]; hi[1] = v; }

    // endpoints: base + three signed deltas, as 7 + 6 bits and as 9 + 5 bits
    V3 const ends[4] = { lo[0], hi[0], lo[1], hi[1] };
    V3 q7[4], q9[4], u7[4], u9[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { q7[i] = floor3(quantize(ends[i], 128.f)); q9[i] = floor3(quantize(ends[i], 512.f)); }
#pragma unroll
    for (int i = 1; i < 4; ++i) { q7[i] = clamp3(q7[i] - q7[0], 31.f); q9[i] = clamp3(q9[i] - q9[0], 15.f); }
    u7[0] = unquantize(q7[0], 128.f); u9[0] = unquantize(q9[0], 512.f);
#pragma unroll
    for (int i = 1; i < 4; ++i) { u7[i] = unquantize(q7[0] + q7[i], 128.f); u9[i] = unquantize(q9[0] + q9[i], 512.f); }
    float error7 = 0.f, error9 = 0.f;
    uint32_t index[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        bool const s = (second >> t) & 1u;
        index[t] = s ? index3(to_half_bits(dot(px[t], dir1)), e10, e11) : index3(to_half_bits(dot(px[t], dir0)), e00, e01);
        float const weight = floorf((float(index[t]) * 64.f) / 7.f + 0.5f);
        error7 += msle(px[t], interpolate(s ? u7[2] : u7[0], s ? u7[3] : u7[1], weight));
        error9 += msle(px[t], interpolate(s ? u9[2] : u9[0], s ? u9[3] : u9[1], weight));
    }
    float const error = fminf(error7, error9);
    if (!(error < best.error)) return;
    bool const sevenSix = error == error7;
    int const baseBits = sevenSix ? 7 : 9, deltaBits = sevenSix ? 6 : 5;
    V3 const w = sevenSix ? q7[0] : q9[0], x = sevenSix ? q7[1] : q9[1], y = sevenSix ? q7[2] : q9[2], z = sevenSix ? q7[3] : q9[3];
    uint32_t const rw = field(w.x, baseBits), gw = field(w.y, baseBits), bw = field(w.z, baseBits);
    uint32_t const rx = field(x.x, deltaBits), gx = field(x.y, deltaBits), bx = field(x.z, deltaBits);
    uint32_t const ry = field(y.x, deltaBits), gy = field(y.y, deltaBits), by = field(y.z, deltaBits);
    uint32_t const rz = field(z.x, deltaBits), gz = field(z.y, deltaBits), bz = field(z.z, deltaBits);
    Bits b;
    if (sevenSix) {         // mode 2 of the format: 7.666
        b.put(0, 0x01, 2);
        b.put(2, gy >> 5, 1); b.put(3, gz >> 4, 1); b.put(4, gz >> 5, 1);
        b.put(5, rw, 7); b.put(12, bz, 1); b.put(13, bz >> 1, 1); b.put(14, by >> 4, 1);
        b.put(15, gw, 7); b.put(22, by >> 5, 1); b.put(23, bz >> 2, 1); b.put(24, gy >> 4, 1);
        b.put(25, bw, 7); b.put(32, bz >> 3, 1); b.put(33, bz >> 5, 1); b.put(34, bz >> 4, 1);
        b.put(35, rx, 6); b.put(41, gy, 4); b.put(45, gx, 6); b.put(51, gz, 4); b.put(55, bx, 6); b.put(61, by, 4);
        b.put(65, ry, 6); b.put(71, rz, 6);
    } else {                // mode 6 of the format: 9.555
        b.put(0, 0x0E, 5);
        b.put(5, rw, 9); b.put(14, by >> 4, 1); b.put(15, gw, 9); b.put(24, gy >> 4, 1); b.put(25, bw, 9); b.put(34, bz >> 4, 1);
        b.put(35, rx, 5); b.put(40, gz >> 4, 1); b.put(41, gy, 4); b.put(45, gx, 5); b.put(50, bz, 1); b.put(51, gz, 4);
        b.put(55, bx, 5); b.put(60, bz >> 1, 1); b.put(61, by, 4); b.put(65, ry, 5); b.put(70, bz >> 2, 1); b.put(71, rz, 5); b.put(76, bz >> 3, 1);
    }
    b.put(77, uint32_t(pattern), 5);
    int at = 82;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        int const n = (t == 0 || t == anchor1) ? 2 : 3;
        uint64_t const v = index[t] & ((1u << n) - 1u);
        b.hi |= v << (at - 64);
        at += n;
    }
    best = Block{ b.lo, b.hi, error };
}

} // namespace

// Registers capped at 168 so that three waves share a SIMD: the encoder is long chains of dependent divisions
// and logarithms, and the other waves fill the issue slots one leaves (4096^2: 1.77 ms with one wave and 256
// registers, 1.05 ms with two, 0.98 ms with three in spite of 175 spilled registers, 1.02 ms with four).
__global__ void __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(3)))
bc6_compress_kernel(BlockCompressArgs a)
{
    int const bx = blockIdx.x * 16 + (threadIdx.x & 15), by = blockIdx.y * 8 + (threadIdx.x >> 4);
    if (bx >= a.widthInBlocks || by >= a.heightInBlocks) return;
    V3 px[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        int const x = a.srcLeft + bx * 4 + (t & 3), y = a.srcTop + by * 4 + (t >> 2);
        float c[4];
        source_pixel(a, x, y, c);
        px[t] = V3{ clampf(c[0], 0.f, kHalfMax), clampf(c[1], 0.f, kHalfMax), clampf(c[2], 0.f, kHalfMax) };
    }
    Block best = encode_one_subset(px);
    float bestScore = pattern_score(px, kSecondSubset[0]);
    int bestPattern = 0;
#pragma unroll 1
    for (int p = 1; p < 32; ++p) {
        float const score = pattern_score(px, kSecondSubset[p]);
        if (score < bestScore) { bestPattern = p; bestScore = score; }
    }
    encode_two_subsets(px, bestPattern, best);
    uint64_t* const dst = reinterpret_cast<uint64_t*>(a.dst + size_t(by + a.dstOffsetY) * a.dstRowPitch) + size_t(bx + a.dstOffsetX) * 2;
    dst[0] = best.lo; dst[1] = best.hi;
}

hipError_t launch_bc6_compress(BlockCompressArgs const& a, hipStream_t stream)
{
    dim3 const grid((a.widthInBlocks + 15) / 16, (a.heightInBlocks + 7) / 8);
    hipLaunchKernelGGL(bc6_compress_kernel, grid, dim3(128), 0, stream, a);
    return hipGetLastError();
}

} // namespace ntc_hip_dev
