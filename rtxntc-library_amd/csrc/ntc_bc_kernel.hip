// ntc_bc_kernel.hip - BC1 .. BC5 block compression of a decoded image (gfx950).
//
// The step after decode in a load path that hands block-compressed textures to a renderer:
// the reference runs it as a graphics compute pass (IContext::MakeBlockCompressionComputePass,
// src/shaders/CompressBC1.hlsl .. CompressBC5.hlsl, src/shaders/BlockCompressCommon.hlsli).
// One lane encodes one 4 x 4 block, as one thread does there.
//
// BC4 (one channel; BC5 = two of them, BC3 = one for alpha).  The encoder tries both BC4 palettes.
// Eight-value palette (endpoint 0 > endpoint 1): start from the
// block's extremes pulled inwards by 1/34 of the range (extremes of exactly 0 or 255 stay), assign
// every texel its nearest palette entry, then up to eight rounds of "least-squares endpoints for
// the current assignment, re-assign", stopping when the error no longer falls or the assignment
// repeats.  Six-value palette (endpoint 0 <= endpoint 1, entries 6 and 7 are 0 and 255): the same
// from the extremes that are not 0 / 255.  The candidate with the smaller squared error wins, the
// eight-value one on a tie.
//
// BC1 colour (also the colour half of BC2 and BC3).  Candidates, the first of the smallest squared
// error (over r, g, b and alpha against 1) wins:
//   * BC1 only: the all-transparent block;
//   * one colour: the block's mean, each component through a table of the endpoint pair whose
//     1/3 : 2/3 mix comes nearest to it;
//   * four-colour mode: endpoints from the bounding box of the block (corners paired by the sign of
//     the covariances, pulled inwards by 1/16), then up to four rounds of nearest-entry assignment
//     + least-squares endpoints + rounding to 5:6:5;
//   * BC1 only: three-colour mode with transparent texels (alpha <= threshold) left out, one round.
// BC2 alpha is 4 bits per texel.
//
// All float arithmetic is IEEE binary32, unfused, in the order written here.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include "ntc_decode_kernel.h"
#include "ntc_bc_source.h"

namespace ntc_hip_dev {

namespace {

// The eight values a block's two endpoints stand for (integer interpolation with the reference's
// rounding bias: +3 before /7, +2 before /5).
__device__ __forceinline__ void bc4_palette(uint32_t e0, uint32_t e1, uint32_t (&p)[8])
{
    p[0] = e0; p[1] = e1;
    if (e0 > e1) {
#pragma unroll
        for (uint32_t k = 1; k < 7; ++k) p[k + 1] = ((7 - k) * e0 + k * e1 + 3) / 7;
    } else {
#pragma unroll
        for (uint32_t k = 1; k < 5; ++k) p[k + 1] = ((5 - k) * e0 + k * e1 + 2) / 5;
        p[6] = 0; p[7] = 255;
    }
}

// Block = endpoint 0 | endpoint 1 << 8 | sixteen 3-bit indices from bit 16 up.
__device__ __forceinline__ uint64_t bc4_with_endpoints(uint64_t block, uint32_t e0, uint32_t e1)
{
    return (block & ~uint64_t(0xffff)) | uint64_t(e0 & 0xffu) | (uint64_t(e1 & 0xffu) << 8);
}
__device__ __forceinline__ uint32_t bc4_index(uint64_t block, int texel) { return uint32_t(block >> (16 + 3 * texel)) & 7u; }

// Nearest palette entry for every texel (the first of equally near ones); returns the summed squared error.
__device__ __forceinline__ float bc4_assign(uint32_t const (&values)[16], uint64_t& block)
{
    uint32_t palette[8];
    bc4_palette(uint32_t(block) & 0xffu, (uint32_t(block) >> 8) & 0xffu, palette);
    block &= 0xffff;
    float total = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        // key = distance * 8 + entry: the smallest key is the nearest entry, the first among equally near ones
        uint32_t key[8];
#pragma unroll
        for (uint32_t k = 0; k < 8; ++k) key[k] = (__sad(int(values[t]), int(palette[k]), 0u) << 3) + k;
        uint32_t const best = min(min(min(key[0], key[1]), min(key[2], key[3])), min(min(key[4], key[5]), min(key[6], key[7])));
        uint32_t const distance = best >> 3;
        total += float(distance * distance);
        block |= uint64_t(best & 7u) << (16 + 3 * t);
    }
    return total;
}

__device__ __forceinline__ uint32_t bc4_endpoint(float v) { return uint32_t(rintf(fminf(fmaxf(v, 0.f), 255.f))); }   // a NaN becomes 0

// Weight of endpoint 0 in palette entry k, for the eight-value and the six-value palette (entries 6 and 7
// of the latter are the constants 0 and 255 and take no part in a fit): the quotients the fit divides
// out, (8 - k) / 7 and (6 - k) / 5, evaluated once by the compiler.
__constant__ float kWeight8[8] = { 1.f, 0.f, 6.f / 7.f, 5.f / 7.f, 4.f / 7.f, 3.f / 7.f, 2.f / 7.f, 1.f / 7.f };
__constant__ float kWeight6[8] = { 1.f, 0.f, 4.f / 5.f, 3.f / 5.f, 2.f / 5.f, 1.f / 5.f, 0.f, 0.f };

// Least-squares endpoints for the block's current assignment.  With `eightValues` every texel takes
// part and weights are 1, 0, 6/7 ... 1/7; otherwise indices 6 and 7 (the fixed 0 and 255) are left
// out and weights are 1, 0, 4/5 ... 1/5, and a singular system leaves the endpoints alone.
__device__ __forceinline__ uint64_t bc4_refit(uint32_t const (&values)[16], uint64_t block, bool eightValues, bool keep255, bool keep0)
{
    float aa = 0.f, bb = 0.f, ab = 0.f, ax = 0.f, bx = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        uint32_t const k = bc4_index(block, t);
        if (!eightValues && k >= 6) continue;
        float const alpha = eightValues ? kWeight8[k] : kWeight6[k];
        float const beta = 1.f - alpha, x = float(values[t]);
        aa += alpha * alpha; bb += beta * beta; ab += alpha * beta;
        ax += alpha * x; bx += beta * x;
    }
    if (eightValues) {
        float const factor = 1.f / (aa * bb - ab * ab);
        uint32_t e0 = keep255 ? 255u : bc4_endpoint((ax * bb - bx * ab) * factor);
        uint32_t e1 = keep0 ? 0u : bc4_endpoint((bx * aa - ax * ab) * factor);
        if (e0 < e1) { uint32_t const t = e0; e0 = e1; e1 = t; }
        return bc4_with_endpoints(block, e0, e1);
    }
    float const det = aa * bb - ab * ab;
    if (det == 0.f) return block;
    return bc4_with_endpoints(block, bc4_endpoint((ax * bb - bx * ab) / det), bc4_endpoint((bx * aa - ax * ab) / det));
}

// Up to eight rounds of refit + re-assign from a starting block; returns the best block and its error.
__device__ __forceinline__ uint64_t bc4_refine(uint32_t const (&values)[16], uint64_t block, bool eightValues, bool keep255, bool keep0, float& bestError)
{
    bestError = bc4_assign(values, block);
    uint64_t best = block;
    for (int round = 0; round < 8; ++round) {
        block = bc4_refit(values, block, eightValues, keep255, keep0);
        float const error = bc4_assign(values, block);
        if (error >= bestError) break;
        bool const repeated = (block >> 16) == (best >> 16);
        best = block;
        if (repeated) break;
        bestError = error;
    }
    return best;
}

__device__ uint64_t bc4_encode(float const (&texels)[16])
{
    uint32_t values[16];
    uint32_t lo = 255, hi = 0, loInner = 255, hiInner = 0;      // extremes; extremes among values that are not 0 / not 255
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        float const s = fminf(fmaxf(texels[t], 0.f), 1.f);     // saturate: a NaN becomes 0
        values[t] = uint32_t(rintf(s * 255.f));
        lo = min(lo, values[t]); hi = max(hi, values[t]);
        if (values[t] != 0) loInner = min(loInner, values[t]);
        if (values[t] != 255) hiInner = max(hiInner, values[t]);
    }
    bool const keep0 = lo == 0, keep255 = hi == 255;
    float error8, error6;
    uint64_t const block8 = bc4_refine(values, bc4_with_endpoints(0, keep255 ? 255u : hi - (hi - lo) / 34u, keep0 ? 0u : lo + (hi - lo) / 34u),
                                       true, keep255, keep0, error8);
    // unsigned arithmetic on purpose: with no inner values (all texels 0 or 255) the difference wraps, as in the reference
    uint32_t const inset = (hiInner - loInner) / 34u;
    uint64_t const block6 = bc4_refine(values, bc4_with_endpoints(0, loInner + inset, hiInner - inset), false, false, false, error6);
    return error6 < error8 ? block6 : block8;
}

// ---------------------------------------------------------------------------------------------
// BC1 colour blocks (BlockCompressCommon.hlsli:36-493)

// For every 8-bit value the pair of 5-bit (6-bit) endpoints (a | b << 8) whose mix (2*A + B) / 3 of
// the expanded endpoints A, B (integer division) is nearest, with 3 % of |a - b| added so that close
// endpoints win among equals; pairs are tried with b in the outer loop, a in the inner one, and the
// first best is kept.  This regenerates the reference's c_ColorMatch5bit / c_ColorMatch6bit
// (hlsli:40-78), the single-colour tables of NVTT.
__device__ uint16_t g_match5[256];
__device__ uint16_t g_match6[256];

__device__ __forceinline__ uint32_t nearest_pair(int value, int bits)
{
    int const n = 1 << bits;
    int best = 0x7fffffff;
    uint32_t pick = 0;
    for (int b = 0; b < n; ++b)
        for (int a = 0; a < n; ++a) {
            int const A = bits == 5 ? (a << 3) | (a >> 2) : (a << 2) | (a >> 4);
            int const B = bits == 5 ? (b << 3) | (b >> 2) : (b << 2) | (b >> 4);
            int const cost = abs((2 * A + B) / 3 - value) * 100 + abs(a - b) * 3;
            if (cost < best) { best = cost; pick = uint32_t(a) | (uint32_t(b) << 8); }
        }
    return pick;
}

struct Rgb { float r, g, b; };
struct Rgba { float r, g, b, a; };

__device__ __forceinline__ float saturate(float v) { return fminf(fmaxf(v, 0.f), 1.f); }      // a NaN becomes 0
__device__ __forceinline__ Rgb rgb_of(Rgba const& p) { return Rgb{ p.r, p.g, p.b }; }
__device__ __forceinline__ float distance2(Rgb const& a, Rgb const& b)
{
    float const dr = a.r - b.r, dg = a.g - b.g, db = a.b - b.b;
    return dr * dr + dg * dg + db * db;
}
__device__ __forceinline__ Rgb mix(Rgb const& a, Rgb const& b, float t)
{
    return Rgb{ a.r + (b.r - a.r) * t, a.g + (b.g - a.g) * t, a.b + (b.b - a.b) * t };
}
__device__ __forceinline__ Rgb expand565(uint32_t w)
{
    return Rgb{ float((w >> 11) & 31u) / 31.f, float((w >> 5) & 63u) / 63.f, float(w & 31u) / 31.f };
}
__device__ __forceinline__ Rgb round565(Rgb const& v, uint32_t& w)
{
    uint32_t const r = uint32_t(rintf(saturate(v.r) * 31.f)), g = uint32_t(rintf(saturate(v.g) * 63.f)), b = uint32_t(rintf(saturate(v.b) * 31.f));
    w = (r << 11) | (g << 5) | b;
    return Rgb{ float(r) / 31.f, float(g) / 63.f, float(b) / 31.f };
}

// Of four distances the smallest; pairs (0, 1) and (2, 3) are compared first, ties go to the later
// pair and, inside a pair, to its second member (hlsli:116-144).
__device__ __forceinline__ uint32_t nearest_of_four(float d0, float d1, float d2, float d3, float& error)
{
    if (fminf(d0, d1) < fminf(d2, d3)) {
        if (d0 < d1) { error = d0; return 0; }
        error = d1; return 1;
    }
    if (d2 < d3) { error = d2; return 2; }
    error = d3; return 3;
}

// Palette index of a texel in four-colour mode: entries hi, lo, 1/3 and 2/3 of the way from hi to lo.
__device__ __forceinline__ uint32_t index_of_four(Rgba const& p, Rgb const& hi, Rgb const& lo, float& error)
{
    Rgb const c = rgb_of(p), third = mix(hi, lo, 1.f / 3.f), twoThirds = mix(hi, lo, 2.f / 3.f);
    float const alphaTerm = (1.f - p.a) * (1.f - p.a);
    return nearest_of_four(distance2(hi, c) + alphaTerm, distance2(lo, c) + alphaTerm,
                           distance2(third, c) + alphaTerm, distance2(twoThirds, c) + alphaTerm, error);
}

// Three-colour mode: entries hi, lo, their midpoint and transparent black; texels at or below the
// alpha threshold take the last at no cost.
__device__ __forceinline__ uint32_t index_of_three(Rgba const& p, Rgb const& hi, Rgb const& lo, float alphaThreshold, float& error)
{
    if (p.a <= alphaThreshold) { error = 0.f; return 3; }
    Rgb const c = rgb_of(p), middle = mix(hi, lo, 0.5f);
    float const alphaTerm = (1.f - p.a) * (1.f - p.a);
    return nearest_of_four(distance2(hi, c) + alphaTerm, distance2(lo, c) + alphaTerm, distance2(middle, c) + alphaTerm,
                           p.r * p.r + p.g * p.g + p.b * p.b + p.a * p.a, error);
}

struct ColorBlock { uint32_t endpoints, indices; float error; };

__device__ __forceinline__ uint32_t table_index(float mean)     // values outside [0, 1] use the table's ends (the reference reads outside its table there)
{
    return uint32_t(fminf(fmaxf(rintf(mean * 255.f), 0.f), 255.f));
}

__device__ ColorBlock bc1_single_color(Rgba const (&px)[16])
{
    Rgb sum{ 0.f, 0.f, 0.f };
#pragma unroll
    for (int t = 0; t < 16; ++t) { sum.r += px[t].r; sum.g += px[t].g; sum.b += px[t].b; }
    uint32_t const mr = g_match5[table_index(sum.r / 16.f)], mg = g_match6[table_index(sum.g / 16.f)], mb = g_match5[table_index(sum.b / 16.f)];
    uint32_t const c0 = ((mr & 31u) << 11) | ((mg & 63u) << 5) | (mb & 31u);
    uint32_t const c1 = (((mr >> 8) & 31u) << 11) | (((mg >> 8) & 63u) << 5) | ((mb >> 8) & 31u);
    ColorBlock out;
    // c0 carries weight 2/3: index 3 when the larger word has to come first (four-colour mode), else index 2
    if (c0 < c1) { out.endpoints = (c0 << 16) | c1; out.indices = 0xffffffffu; }
    else         { out.endpoints = (c1 << 16) | c0; out.indices = 0xaaaaaaaau; }
    Rgb const shown = mix(expand565(c0), expand565(c1), 1.f / 3.f);
    out.error = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        float const dr = px[t].r - shown.r, dg = px[t].g - shown.g, db = px[t].b - shown.b, da = px[t].a - 1.f;
        out.error += dr * dr + dg * dg + db * db + da * da;
    }
    return out;
}

// Bounding box of the texels that take part, its corners paired along the block's main direction:
// with red (or, if red is constant, green) as the axis, the other components' ends are swapped where
// their covariance with the axis is negative.  Then both ends move inwards by extent / divisor.
struct Box { Rgb lo, hi; };
__device__ __forceinline__ void orient_and_inset(Box& box, float covRG, float covRB, float covGB, float divisor)
{
    if (box.lo.r != box.hi.r) {
        if (covRG < 0.f) { float const t = box.lo.g; box.lo.g = box.hi.g; box.hi.g = t; }
        if (covRB < 0.f) { float const t = box.lo.b; box.lo.b = box.hi.b; box.hi.b = t; }
    } else if (box.lo.g != box.hi.g) {
        if (covGB < 0.f) { float const t = box.lo.b; box.lo.b = box.hi.b; box.hi.b = t; }
    }
    Rgb const inset{ (box.hi.r - box.lo.r) / divisor, (box.hi.g - box.lo.g) / divisor, (box.hi.b - box.lo.b) / divisor };
    box.hi = Rgb{ saturate(box.hi.r - inset.r), saturate(box.hi.g - inset.g), saturate(box.hi.b - inset.b) };
    box.lo = Rgb{ saturate(box.lo.r + inset.r), saturate(box.lo.g + inset.g), saturate(box.lo.b + inset.b) };
}

// Sums of the least-squares problem "texel = alpha * A + beta * B".
struct Fit {
    float aa = 0.f, bb = 0.f, ab = 0.f;
    Rgb ax{ 0.f, 0.f, 0.f }, bx{ 0.f, 0.f, 0.f };
    __device__ __forceinline__ void add(float beta, Rgba const& p)
    {
        float const alpha = 1.f - beta;
        aa += alpha * alpha; bb += beta * beta; ab += alpha * beta;
        ax.r += alpha * p.r; ax.g += alpha * p.g; ax.b += alpha * p.b;
        bx.r += beta * p.r;  bx.g += beta * p.g;  bx.b += beta * p.b;
    }
    // false when the system is (nearly) singular
    __device__ __forceinline__ bool solve(Rgb& A, Rgb& B) const
    {
        float const det = aa * bb - ab * ab;
        if (!(fabsf(det) > 0.0001f)) return false;
        float const factor = 1.f / det;
        A = Rgb{ (ax.r * bb - bx.r * ab) * factor, (ax.g * bb - bx.g * ab) * factor, (ax.b * bb - bx.b * ab) * factor };
        B = Rgb{ (bx.r * aa - ax.r * ab) * factor, (bx.g * aa - ax.g * ab) * factor, (bx.b * aa - ax.b * ab) * factor };
        return true;
    }
};
// An endpoint component that sits exactly on 0 or 1 stays there.
__device__ __forceinline__ float unless_pinned(float current, float fitted) { return (current == 0.f || current == 1.f) ? current : saturate(fitted); }
__device__ __forceinline__ Rgb unless_pinned(Rgb const& current, Rgb const& fitted)
{
    return Rgb{ unless_pinned(current.r, fitted.r), unless_pinned(current.g, fitted.g), unless_pinned(current.b, fitted.b) };
}

__device__ ColorBlock bc1_four_colors(Rgba const (&px)[16])
{
    Rgb sum{ 0.f, 0.f, 0.f };
    Box box{ Rgb{ 1.f, 1.f, 1.f }, Rgb{ 0.f, 0.f, 0.f } };
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        sum.r += px[t].r; sum.g += px[t].g; sum.b += px[t].b;
        box.lo = Rgb{ fminf(box.lo.r, px[t].r), fminf(box.lo.g, px[t].g), fminf(box.lo.b, px[t].b) };
        box.hi = Rgb{ fmaxf(box.hi.r, px[t].r), fmaxf(box.hi.g, px[t].g), fmaxf(box.hi.b, px[t].b) };
    }
    Rgb const center{ sum.r / 16.f, sum.g / 16.f, sum.b / 16.f };
    float covRG = 0.f, covRB = 0.f, covGB = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        float const r = px[t].r - center.r, g = px[t].g - center.g, b = px[t].b - center.b;
        covRG += r * g; covRB += r * b; covGB += g * b;
    }
    orient_and_inset(box, covRG, covRB, covGB, 16.f);

    uint32_t c0 = 0, c1 = 0;
    for (int round = 0; round < 4; ++round) {
        Fit fit;
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            float unused;
            uint32_t const k = index_of_four(px[t], box.hi, box.lo, unused);
            float beta = float(k & 1u);
            if (k & 2u) beta = (1.f + beta) / 3.f;
            fit.add(beta, px[t]);
        }
        Rgb A, B;
        if (fit.solve(A, B)) {
            box.lo = unless_pinned(box.lo, B);
            box.hi = unless_pinned(box.hi, A);
        }
        uint32_t n0, n1;
        box.hi = round565(box.hi, n0);
        box.lo = round565(box.lo, n1);
        if (n0 == c0 && n1 == c1) break;
        c0 = n0; c1 = n1;
    }
    // the first word must be the larger one, or a decoder takes the block for three-colour mode
    if (c0 == c1) {
        if (c0 == 0) { c0 = 1; box.hi = expand565(c0); }
        else         { c1 = c0 - 1; box.lo = expand565(c1); }
    } else if (c0 < c1) {
        Rgb const t = box.hi; box.hi = box.lo; box.lo = t;
        uint32_t const w = c0; c0 = c1; c1 = w;
    }
    ColorBlock out{ (c1 << 16) | c0, 0u, 0.f };
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        float e;
        out.indices |= index_of_four(px[t], box.hi, box.lo, e) << (2 * t);
        out.error += e;
    }
    return out;
}

__device__ ColorBlock bc1_three_colors(Rgba const (&px)[16], float alphaThreshold)
{
    Rgb sum{ 0.f, 0.f, 0.f };
    Box box{ Rgb{ 1.f, 1.f, 1.f }, Rgb{ 0.f, 0.f, 0.f } };
    int opaque = 0;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if (!(px[t].a <= alphaThreshold)) {
            sum.r += px[t].r; sum.g += px[t].g; sum.b += px[t].b;
            box.lo = Rgb{ fminf(box.lo.r, px[t].r), fminf(box.lo.g, px[t].g), fminf(box.lo.b, px[t].b) };
            box.hi = Rgb{ fmaxf(box.hi.r, px[t].r), fmaxf(box.hi.g, px[t].g), fmaxf(box.hi.b, px[t].b) };
            ++opaque;
        }
    float const count = float(opaque);
    Rgb const center = opaque > 0 ? Rgb{ sum.r / count, sum.g / count, sum.b / count } : Rgb{ 0.f, 0.f, 0.f };
    float covRG = 0.f, covRB = 0.f, covGB = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        if (!(px[t].a <= alphaThreshold)) {
            float const r = px[t].r - center.r, g = px[t].g - center.g, b = px[t].b - center.b;
            covRG += r * g; covRB += r * b; covGB += g * b;
        }
    orient_and_inset(box, covRG, covRB, covGB, count);      // no opaque texel: -1 / 0, the ends saturate to hi = 1, lo = 0

    Fit fit;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        float unused;
        uint32_t const k = index_of_three(px[t], box.hi, box.lo, alphaThreshold, unused);
        if (k != 3) fit.add((k & 2u) ? 0.5f : float(k & 1u), px[t]);
    }
    Rgb A, B;
    if (fit.solve(A, B)) {
        // as in the reference (hlsli:453-455): the solution for the entry-0 end goes to `lo` and vice versa
        box.lo = unless_pinned(box.lo, A);
        box.hi = unless_pinned(box.hi, B);
    }
    uint32_t c0, c1;
    box.hi = round565(box.hi, c0);
    box.lo = round565(box.lo, c1);
    if (c0 > c1) {              // first word <= second word selects three-colour mode
        Rgb const t = box.hi; box.hi = box.lo; box.lo = t;
        uint32_t const w = c0; c0 = c1; c1 = w;
    }
    ColorBlock out{ (c1 << 16) | c0, 0u, 0.f };
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        float e;
        out.indices |= index_of_three(px[t], box.hi, box.lo, alphaThreshold, e) << (2 * t);
        out.error += e;         // 0 for transparent texels
    }
    return out;
}

// Colour block of BC1 (withAlpha: the transparent and three-colour candidates take part) or of BC2 / BC3.
__device__ __forceinline__ uint64_t bc1_encode(Rgba const (&px)[16], bool withAlpha, float alphaThreshold)
{
    ColorBlock best = bc1_single_color(px);
    if (withAlpha) {
        float transparentError = 0.f;
#pragma unroll
        for (int t = 0; t < 16; ++t)
            if (!(px[t].a <= alphaThreshold)) transparentError += px[t].r * px[t].r + px[t].g * px[t].g + px[t].b * px[t].b + px[t].a * px[t].a;
        if (!(best.error < transparentError)) best = ColorBlock{ 0u, 0xffffffffu, transparentError };
    }
    ColorBlock const four = bc1_four_colors(px);
    if (four.error < best.error) best = four;
    if (withAlpha) {
        ColorBlock const three = bc1_three_colors(px, alphaThreshold);
        if (three.error < best.error) best = three;
    }
    return uint64_t(best.endpoints) | (uint64_t(best.indices) << 32);
}

// BC2 alpha: 4 bits per texel, texel 0 in the lowest bits.
__device__ __forceinline__ uint64_t bc2_alpha(float const (&alpha)[16])
{
    uint64_t bits = 0;
#pragma unroll
    for (int t = 0; t < 16; ++t) bits |= uint64_t(uint32_t(rintf(saturate(alpha[t]) * 15.f))) << (4 * t);
    return bits;
}

} // namespace

// Thread groups of 16 x 8 blocks as in the reference (BLOCK_COMPRESS_CS_GROUP_WIDTH / HEIGHT).
template <int CHANNELS>
__global__ void __launch_bounds__(128)
bc4_compress_kernel(BlockCompressArgs a)
{
    int const bx = blockIdx.x * 16 + (threadIdx.x & 15), by = blockIdx.y * 8 + (threadIdx.x >> 4);
    if (bx >= a.widthInBlocks || by >= a.heightInBlocks) return;
    uint64_t out[CHANNELS];
#pragma unroll
    for (int c = 0; c < CHANNELS; ++c) {
        float texels[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) texels[t] = source_channel(a, a.srcLeft + bx * 4 + (t & 3), a.srcTop + by * 4 + (t >> 2), c);
        out[c] = bc4_encode(texels);
    }
    uint64_t* const dst = reinterpret_cast<uint64_t*>(a.dst + size_t(by + a.dstOffsetY) * a.dstRowPitch) + size_t(bx + a.dstOffsetX) * CHANNELS;
#pragma unroll
    for (int c = 0; c < CHANNELS; ++c) dst[c] = out[c];
}

// BC1 (8 bytes per block), BC2 and BC3 (alpha block, then colour block).  At least three waves per SIMD: the BC1
// instance would otherwise take 203 registers and run two (4096^2: 0.22 ms with two, 0.19 ms with three, 0.26 ms with four).
template <int FORMAT>
__global__ void __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(3)))
bc1_compress_kernel(BlockCompressArgs a)
{
    int const bx = blockIdx.x * 16 + (threadIdx.x & 15), by = blockIdx.y * 8 + (threadIdx.x >> 4);
    if (bx >= a.widthInBlocks || by >= a.heightInBlocks) return;
    Rgba px[16];
    float alpha[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        int const x = a.srcLeft + bx * 4 + (t & 3), y = a.srcTop + by * 4 + (t >> 2);
        float c[4];
        source_pixel(a, x, y, c);
        px[t] = Rgba{ c[0], c[1], c[2], c[3] };
        if constexpr (FORMAT != 1) { alpha[t] = px[t].a; px[t].a = 1.f; }
    }
    uint64_t const color = bc1_encode(px, FORMAT == 1, a.alphaThreshold);
    constexpr int WORDS = FORMAT == 1 ? 1 : 2;
    uint64_t* const dst = reinterpret_cast<uint64_t*>(a.dst + size_t(by + a.dstOffsetY) * a.dstRowPitch) + size_t(bx + a.dstOffsetX) * WORDS;
    if constexpr (FORMAT == 1) dst[0] = color;
    else {
        dst[0] = FORMAT == 2 ? bc2_alpha(alpha) : bc4_encode(alpha);
        dst[1] = color;
    }
}

__global__ void __launch_bounds__(256)
bc1_tables_kernel()
{
    g_match5[threadIdx.x] = uint16_t(nearest_pair(int(threadIdx.x), 5));
    g_match6[threadIdx.x] = uint16_t(nearest_pair(int(threadIdx.x), 6));
}

hipError_t launch_block_compress(BlockCompressArgs const& a, int dstFormat, hipStream_t stream)
{
    dim3 const grid((a.widthInBlocks + 15) / 16, (a.heightInBlocks + 7) / 8);
    if (dstFormat <= 3) {
        // the single-colour tables are computed on the device the first time each device needs them
        // (every launch of the library is on one stream per device, so the order is given)
        static std::atomic<uint64_t> tablesBuilt{0};
        int device = 0;
        if (hipError_t const e = hipGetDevice(&device); e != hipSuccess) return e;
        uint64_t const bit = uint64_t(1) << (device & 63);
        if (!(tablesBuilt.load(std::memory_order_acquire) & bit)) {
            hipLaunchKernelGGL(bc1_tables_kernel, dim3(1), dim3(256), 0, stream);
            if (hipError_t const e = hipGetLastError(); e != hipSuccess) return e;
            tablesBuilt.fetch_or(bit, std::memory_order_release);
        }
    }
    switch (dstFormat) {
    case 1: hipLaunchKernelGGL(bc1_compress_kernel<1>, grid, dim3(128), 0, stream, a); break;
    case 2: hipLaunchKernelGGL(bc1_compress_kernel<2>, grid, dim3(128), 0, stream, a); break;
    case 3: hipLaunchKernelGGL(bc1_compress_kernel<3>, grid, dim3(128), 0, stream, a); break;
    case 4: hipLaunchKernelGGL(bc4_compress_kernel<1>, grid, dim3(128), 0, stream, a); break;
    case 5: hipLaunchKernelGGL(bc4_compress_kernel<2>, grid, dim3(128), 0, stream, a); break;
    case 6: return launch_bc6_compress(a, stream);
    case 7: return launch_bc7_compress(a, stream);
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

} // namespace ntc_hip_dev
