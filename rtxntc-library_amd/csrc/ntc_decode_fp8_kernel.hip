// ntc_decode_fp8_kernel.hip - texture-set decode for gfx950 with the FP8 version of the network: what
// ITextureSet::Decompress(stats, useInt8Weights = false) asks for (reference src/TextureSet.cpp:1664-1682,
// 1812,1826), evaluated as NtcSampleTextureSet_CoopVec_FP8 describes it
// (include/libntc/shaders/InferenceCoopVec.hlsli:22-124,127-160,235-398) from the weight blob of
// src/WeightLayout.cpp:51-71: three hidden layers with e4m3 weights, e4m3-rounded fp16 inputs and
// activations, fp16 biases and the HGELU-clamp activation in fp16; the int8 output layer.
//
// The shader leaves the arithmetic of its matrix-vector products to the driver.  Here every product sum is
// EXACT, so the result is a function of the inputs alone and a CPU restatement can match it bit for bit:
// e4m3 values are fp16 values, their products are exact in fp32, and a weight matrix is held as three fp16
// planes by the bits of |512 w| (bits 14.., 7..13, 0..6 - values up to 448, 31.75 and 0.248) so that every
// partial sum a plane's v_mfma_f32_16x16x32_f16 accumulates is exactly representable whatever the summation
// order: with |inputs| <= 3 (HGELU's range; 1 for layer 0) and 64 terms the sums stay below 2^24 units of
// each plane's smallest product (2^-4, 2^-11, 2^-18).  A layer output is then
//     x = half(((s2 + s1) + s0) + float(bias))          three fp32 additions, one conversion
// and the activation runs on packed halves:
//     t = sat(fma(x, half(1/3), 1/2));  y = clamp(x, -3, 3) * t;  next input = e4m3(y)
// (hardware fp16 -> e4m3 -> fp16 conversion, round-to-nearest-even), or after the last hidden layer
//     q = rne(80 y - 113) as one fp16 fma against 1423 = 1536 - 113 (fp16 integers from 1024 to 2048 are
//     one apart), minus 1536,
// the int8 input of the output layer, which is acc = bias + sum W q in exact fp32 / int32, o = float(acc) * scale.
//
// Work distribution, tiles and stores are those of decode_kernel (ntc_decode_kernel.hip): one persistent
// launch, a workgroup tile of 64 x 4 texels = four wave tiles of 16 x 4; lane = texel in the input stage,
// lane (j = lane%16, g = lane/16) = channels 16t+4g..+3 of texel j in the matrix stages.
#include "ntc_decode_device.h"

namespace ntc_hip_dev {

typedef short v2s __attribute__((ext_vector_type(2)));

// Two halves -> the nearest e4m3 values (as halves): v_cvt_scalef32_pk_fp8_f16 and back, scale 1.
__device__ __forceinline__ uint32_t round_e4m3_pk(uint32_t halves)
{
    v2s const bytes = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(v2s{ 0, 0 }, __builtin_bit_cast(v2h, halves), 1.0f, false);
    v2h const back = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(__builtin_bit_cast(uint32_t, bytes), 1.0f, false);
    return __builtin_bit_cast(uint32_t, back);
}

// Two fp32 values -> two halves, round-to-nearest-even.  The empty asm keeps a producing multiply-add from
// being folded into a conversion that rounds once (v_fma_mix*).
__device__ __forceinline__ uint32_t halves_rne(float a, float b)
{
    asm("" : "+v"(a));
    asm("" : "+v"(b));
    v2h const h = __builtin_convertvector(v2f{ a, b }, v2h);
    return __builtin_bit_cast(uint32_t, h);
}

// HGELU-clamp on two fp16 layer outputs (NtcHGELUClamp_Forward_CoopVec, InferenceCoopVec.hlsli:150-153).
__device__ __forceinline__ uint32_t hgelu_pk(uint32_t x)
{
    uint32_t const third = 0x35553555u, half = 0x38003800u, three = 0x42004200u, minusThree = 0xc200c200u;
    uint32_t t, xc, y;
    asm("v_pk_fma_f16 %0, %1, %2, %3 clamp" : "=v"(t) : "v"(x), "v"(third), "v"(half));
    asm("v_pk_max_f16 %0, %1, %2" : "=v"(xc) : "v"(x), "v"(minusThree));
    asm("v_pk_min_f16 %0, %1, %2" : "=v"(xc) : "v"(xc), "v"(three));
    asm("v_pk_mul_f16 %0, %1, %2" : "=v"(y) : "v"(xc), "v"(t));
    return y;
}

// After the last hidden layer: q = rne(80 y - 113) as fp16 integers in [-128, 127] (hlsli:155-158).
__device__ __forceinline__ uint32_t quantize_int8_pk(uint32_t y)
{
    uint32_t const eighty = 0x55005500u, c1423 = 0x658f658fu, minus1536 = 0xe600e600u;
    uint32_t z, q;
    asm("v_pk_fma_f16 %0, %1, %2, %3" : "=v"(z) : "v"(y), "v"(eighty), "v"(c1423));
    asm("v_pk_add_f16 %0, %1, %2" : "=v"(q) : "v"(z), "v"(minus1536));
    return q;
}

template <int FEATURES_>
struct Fp8Variant {
    static constexpr int F = FEATURES_;                      // features stored per cell of either grid (slots: 16)
    static constexpr int IN = 48, H0 = 64, H1 = 48, H2 = 32, OUT = 16;      // InferenceConstants.h:28-40
    static constexpr int T0 = H0 / 16, T1 = H1 / 16, T2 = H2 / 16;
    static constexpr int PLANES = 3;
    static constexpr int W1_OFF = IN * H0, W2_OFF = W1_OFF + H0 * H1, W3_OFF = W2_OFF + H1 * H2;
    static constexpr int WEIGHT_BYTES = W3_OFF + H2 * OUT;
    // src/WeightLayout.cpp:249-262: fp16 biases of the three e4m3 layers, then scale and bias of the output layer
    static constexpr int BIAS_OFF = WEIGHT_BYTES, SCALE3_OFF = BIAS_OFF + 2 * (H0 + H1 + H2), BIAS3_OFF = SCALE3_OFF + 4 * OUT;
    static constexpr int WAVES = 4, THREADS = 256;
    static constexpr int IN_STRIDE = 28;                     // dwords per texel in the transpose buffer: 24 + 4 of padding
};

// A operands in LDS, in 16-byte units.  A block for 32 inputs holds one unit per lane (8 halves), a block for
// 16 inputs half a unit per lane (4 halves, 32 units).
struct alignas(16) Fp8Lds {
    uint4 w0[3][4][96];        // layer 0, inputs in their natural order: [plane][output tile][K32 block | K16 block]
    uint4 w1[3][3][128];       // layer 1: two blocks of 32 (input-tile pairs 0-1, 2-3)
    uint4 w2[3][2][96];        // layer 2: input-tile pair 0-1, then input tile 2
    uint4 w3[64];              // output layer (int8 weights as halves): input-tile pair 0-1
    float bias[9][4][4];       // hidden layers: [output tile of layers 0..2][g][r] -> channel 16t+4g+r
    float outScale[4][4];      // output layer: [g][r]
    int32_t outBias[4][4];
    uint32_t in[4][kWaveTexels][28];
};

// OCP e4m3 byte -> the integer 512 * value (NaN encodings decode as 0).
__device__ __forceinline__ int32_t fp8_times_512(uint32_t byte)
{
    uint32_t const e = (byte >> 3) & 15u, m = byte & 7u;
    int32_t mag = (e == 0) ? int32_t(m) : int32_t((8u + m) << (e - 1u));
    if ((byte & 0x7fu) == 0x7fu) mag = 0;
    return (byte & 0x80u) ? -mag : mag;
}

// Plane p of an e4m3 weight as an fp16 value: bits [7p, 7p+7) (the top plane: the rest) of |512 w|, with w's
// sign, in units of 2^(7p - 9).
__device__ __forceinline__ _Float16 plane_value(int32_t w512, int plane)
{
    int32_t const mag = w512 < 0 ? -w512 : w512;
    int32_t const bits = plane == 2 ? mag >> 14 : (mag >> (7 * plane)) & 127;
    float const unit = plane == 0 ? 0x1p-9f : (plane == 1 ? 0x1p-2f : 0x1p5f);
    float const v = float(bits) * unit;
    return _Float16(w512 < 0 ? -v : v);
}

// Stores the 8 (or 4) halves of one lane of an A block: weights W[row][k[e]] of one plane.
template <class V>
__device__ __forceinline__ void stage_plane_halves(uint32_t* dst, uint8_t const* __restrict__ matrix, int in, int row, int const* k, int count, int plane)
{
    for (int e = 0; e < count; e += 2) {
        _Float16 const a = plane_value(fp8_times_512(matrix[row * in + k[e]]), plane);
        _Float16 const b = plane_value(fp8_times_512(matrix[row * in + k[e + 1]]), plane);
        v2h const h = { a, b };
        dst[e >> 1] = __builtin_bit_cast(uint32_t, h);
    }
}

// Copies the FP8 blob into LDS in matrix-instruction operand order.  Layer 0 takes its inputs in their
// natural order (lane (i, kg) of a block of 32 holds inputs 8kg..8kg+7, of a block of 16 inputs 32+4kg..+3);
// layers 1..3 take theirs in the order the previous layer's result registers hold them: lane (i, kg) of the
// block for input tiles (2p, 2p+1) holds inputs 16*(2p + e/4) + 4kg + e%4, e = 0..7.
template <class V>
__device__ void stage_fp8_weights(Fp8Lds& lds, uint8_t const* __restrict__ blob)
{
    int const tid = threadIdx.x;
    // biases of the hidden layers (fp16 in the blob), scale and bias of the output layer
    for (int e = tid; e < 9 * 16; e += V::THREADS) {
        int const r = e & 3, g = (e >> 2) & 3, t = e >> 4;
        int const c = 16 * t + 4 * g + r;                    // layers 0..2 back to back: 64 + 48 + 32 channels
        lds.bias[t][g][r] = float(reinterpret_cast<_Float16 const*>(blob + V::BIAS_OFF)[c]);
    }
    if (tid < 16) {
        lds.outScale[tid >> 2][tid & 3] = reinterpret_cast<float const*>(blob + V::SCALE3_OFF)[tid];
        lds.outBias[tid >> 2][tid & 3] = reinterpret_cast<int32_t const*>(blob + V::BIAS3_OFF)[tid];
    }
    // layer 0: (plane, tile, lane) -> one K32 unit and half a K16 unit
    for (int e = tid; e < 3 * V::T0 * 64; e += V::THREADS) {
        int const lane = e & 63, t = (e >> 6) % V::T0, p = e / (64 * V::T0);
        int const i = lane & 15, kg = lane >> 4;
        int k32[8], k16[4];
        for (int q = 0; q < 8; ++q) k32[q] = 8 * kg + q;
        for (int q = 0; q < 4; ++q) k16[q] = 32 + 4 * kg + q;
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w0[p][t][lane]), blob, V::IN, 16 * t + i, k32, 8, p);
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w0[p][t][64]) + 2 * lane, blob, V::IN, 16 * t + i, k16, 4, p);
    }
    // layer 1: 64 inputs = two blocks of 32
    for (int e = tid; e < 3 * V::T1 * 2 * 64; e += V::THREADS) {
        int const lane = e & 63, pair = (e >> 6) & 1, t = (e >> 7) % V::T1, p = e / (128 * V::T1);
        int const i = lane & 15, kg = lane >> 4;
        int k[8];
        for (int q = 0; q < 8; ++q) k[q] = 16 * (2 * pair + q / 4) + 4 * kg + q % 4;
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w1[p][t][pair * 64 + lane]), blob + V::W1_OFF, V::H0, 16 * t + i, k, 8, p);
    }
    // layer 2: 48 inputs = one block of 32 and one of 16
    for (int e = tid; e < 3 * V::T2 * 64; e += V::THREADS) {
        int const lane = e & 63, t = (e >> 6) % V::T2, p = e / (64 * V::T2);
        int const i = lane & 15, kg = lane >> 4;
        int k32[8], k16[4];
        for (int q = 0; q < 8; ++q) k32[q] = 16 * (q / 4) + 4 * kg + q % 4;
        for (int q = 0; q < 4; ++q) k16[q] = 32 + 4 * kg + q;
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w2[p][t][lane]), blob + V::W2_OFF, V::H1, 16 * t + i, k32, 8, p);
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w2[p][t][64]) + 2 * lane, blob + V::W2_OFF, V::H1, 16 * t + i, k16, 4, p);
    }
    // output layer: int8 weights as halves, 32 inputs = one block
    if (tid < 64) {
        int const lane = tid, i = lane & 15, kg = lane >> 4;
        uint32_t* dst = reinterpret_cast<uint32_t*>(&lds.w3[lane]);
        int8_t const* W = reinterpret_cast<int8_t const*>(blob + V::W3_OFF);
        for (int q = 0; q < 8; q += 2) {
            int const ka = 16 * (q / 4) + 4 * kg + q % 4;
            v2h const h = { _Float16(int(W[i * V::H2 + ka])), _Float16(int(W[i * V::H2 + ka + 1])) };
            dst[q >> 1] = __builtin_bit_cast(uint32_t, h);
        }
    }
}

// The 48 inputs of one texel as 24 dwords of e4m3-rounded halves (NtcPrepareNetworkInputsInternal_FP16,
// InferenceCoopVec.hlsli:22-107): [high-res features 0..15 | low-res features 0..15 | 12 x positional encoding |
// lod, lod | 0, 0].  Features a grid does not store stay zero (hlsli:36-40).
template <class V>
__device__ __forceinline__ void prepare_inputs_fp8(DevMip const& m, int x, int y, uint32_t (&in)[24])
{
#pragma unroll
    for (int i = 0; i < 24; ++i) in[i] = 0;
    float const u = (float(x) + 0.5f) / float(m.width);      // hlsli:117-118
    float const v = (float(y) + 0.5f) / float(m.height);
    constexpr int layers = (V::F + 3) / 4;
#pragma unroll
    for (int grid = 0; grid < 2; ++grid) {
        int const gw = grid == 0 ? m.hrWidth : m.lrWidth, gh = grid == 0 ? m.hrHeight : m.lrHeight;
        uint16_t const* __restrict__ g = grid == 0 ? m.hr : m.lr;
        Taps const tp = footprint(u, v, gw, gh);
        size_t const layerStride = size_t(gw) * size_t(gh);
        size_t const a00 = size_t(tp.y0) * gw + tp.x0, a10 = size_t(tp.y0) * gw + tp.x1;
        size_t const a01 = size_t(tp.y1) * gw + tp.x0, a11 = size_t(tp.y1) * gw + tp.x1;
#pragma unroll
        for (int L = 0; L < layers; ++L) {
            uint32_t const s00 = spread4(g[a00 + L * layerStride]), s10 = spread4(g[a10 + L * layerStride]);
            uint32_t const s01 = spread4(g[a01 + L * layerStride]), s11 = spread4(g[a11 + L * layerStride]);
            float value[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float t = tp.w00 * float((s00 >> (8 * i)) & 0xffu);
                t = __builtin_fmaf(tp.w10, float((s10 >> (8 * i)) & 0xffu), t);
                t = __builtin_fmaf(tp.w01, float((s01 >> (8 * i)) & 0xffu), t);
                t = __builtin_fmaf(tp.w11, float((s11 >> (8 * i)) & 0xffu), t);
                value[i] = (4 * L + i < V::F) ? __builtin_fmaf(t, 0.13333334f, -1.f) : 0.f;
            }
            in[8 * grid + 2 * L]     = round_e4m3_pk(halves_rne(value[0], value[1]));
            in[8 * grid + 2 * L + 1] = round_e4m3_pk(halves_rne(value[2], value[3]));
        }
    }
    float px = float(x) * m.positionScale, py = float(y) * m.positionScale;   // hlsli:51-75, Inference.hlsli:89-113
#pragma unroll
    for (int w = 0; w < 3; ++w) {
        float const e0 = (px - floorf(px)) * 2.f - 1.f;
        float const e1 = (py - floorf(py)) * 2.f - 1.f;
        float const qx = px + 0.25f, qy = py + 0.25f;
        float const e2 = (qx - floorf(qx)) * 2.f - 1.f;
        float const e3 = (qy - floorf(qy)) * 2.f - 1.f;
        in[16 + 2 * w]     = round_e4m3_pk(halves_rne(e0, e1));
        in[16 + 2 * w + 1] = round_e4m3_pk(halves_rne(e2, e3));
        px *= 2.f; py *= 2.f;
    }
    in[22] = round_e4m3_pk(halves_rne(m.positionLod, m.positionLod));
}

// One hidden layer's epilogue for the four channels a lane holds of one texel: sums of the three planes ->
// layer output -> activation -> the next layer's inputs (two dwords of halves).
template <bool LAST_HIDDEN>
__device__ __forceinline__ void fp8_epilogue(v4f s2, v4f s1, v4f s0, v4f bias, uint32_t (&out)[2])
{
    float r[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float a = s2[i] + s1[i];
        a = a + s0[i];
        r[i] = a + bias[i];
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        uint32_t const y = hgelu_pk(halves_rne(r[2 * h], r[2 * h + 1]));
        out[h] = LAST_HIDDEN ? quantize_int8_pk(y) : round_e4m3_pk(y);
    }
}

// acc[b] += A(block of 32 inputs) * X for the four 16-texel blocks of the wave.
__device__ __forceinline__ void mfma32(uint4 const& a, uint4 const (&x)[4], v4f (&acc)[4])
{
    v8h const A = __builtin_bit_cast(v8h, a);
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, __builtin_bit_cast(v8h, x[b]), acc[b], 0, 0, 0);
}
__device__ __forceinline__ void mfma16(uint2 const& a, uint2 const (&x)[4], v4f (&acc)[4])
{
    v4h const A = __builtin_bit_cast(v4h, a);
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[b] = __builtin_amdgcn_mfma_f32_16x16x16f16(A, __builtin_bit_cast(v4h, x[b]), acc[b], 0, 0, 0);
}

// The FP8 network for the 64 texels of one wave.  `in` is the lane's own texel.  On return D[b] holds, for
// lane (j, g), the int32 accumulators of output channels 4g..4g+3 of texel 16b + j, and S their scales.
template <class V>
__device__ __forceinline__ void mlp_forward_fp8(Fp8Lds& lds, int wave, int lane, uint32_t const (&in)[24], v4i (&D)[4], v4f& S)
{
    int const j = lane & 15, g = lane >> 4;
    // transpose: lane = texel -> lane (j, kg) holds inputs 8kg..8kg+7 (block of 32) and 32+4kg..+3 (block of 16)
    {
        uint4* dst = reinterpret_cast<uint4*>(&lds.in[wave][lane][0]);
#pragma unroll
        for (int q = 0; q < 6; ++q) dst[q] = make_uint4(in[4 * q], in[4 * q + 1], in[4 * q + 2], in[4 * q + 3]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    uint4 X32[4];
    uint2 X16[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        X32[b] = *reinterpret_cast<uint4 const*>(&lds.in[wave][16 * b + j][4 * g]);
        X16[b] = *reinterpret_cast<uint2 const*>(&lds.in[wave][16 * b + j][16 + 2 * g]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    v4f const zero = { 0.f, 0.f, 0.f, 0.f };
    // layer 0: 48 -> 64
    uint32_t Ha[4][4][2], Hb[4][4][2];                       // [texel block][tile of 16 channels][2 dwords = 4 halves]
#pragma unroll
    for (int t = 0; t < V::T0; ++t) {
        v4f acc[3][4];
#pragma unroll
        for (int p = 0; p < 3; ++p) {
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[p][b] = zero;
            mfma32(lds.w0[p][t][lane], X32, acc[p]);
            mfma16(reinterpret_cast<uint2 const*>(&lds.w0[p][t][64])[lane], X16, acc[p]);
        }
        v4f const bias = *reinterpret_cast<v4f const*>(&lds.bias[t][g][0]);
#pragma unroll
        for (int b = 0; b < 4; ++b) fp8_epilogue<false>(acc[2][b], acc[1][b], acc[0][b], bias, Ha[b][t]);
    }
    // layer 1: 64 -> 48
#pragma unroll
    for (int t = 0; t < V::T1; ++t) {
        v4f acc[3][4];
#pragma unroll
        for (int p = 0; p < 3; ++p) {
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[p][b] = zero;
#pragma unroll
            for (int pair = 0; pair < 2; ++pair) {
                uint4 x[4];
#pragma unroll
                for (int b = 0; b < 4; ++b) x[b] = make_uint4(Ha[b][2 * pair][0], Ha[b][2 * pair][1], Ha[b][2 * pair + 1][0], Ha[b][2 * pair + 1][1]);
                mfma32(lds.w1[p][t][pair * 64 + lane], x, acc[p]);
            }
        }
        v4f const bias = *reinterpret_cast<v4f const*>(&lds.bias[V::T0 + t][g][0]);
#pragma unroll
        for (int b = 0; b < 4; ++b) fp8_epilogue<false>(acc[2][b], acc[1][b], acc[0][b], bias, Hb[b][t]);
    }
    // layer 2: 48 -> 32, its activations quantised to the int8 inputs of the output layer
#pragma unroll
    for (int t = 0; t < V::T2; ++t) {
        v4f acc[3][4];
#pragma unroll
        for (int p = 0; p < 3; ++p) {
            uint4 x[4];
            uint2 xt[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                acc[p][b] = zero;
                x[b] = make_uint4(Hb[b][0][0], Hb[b][0][1], Hb[b][1][0], Hb[b][1][1]);
                xt[b] = make_uint2(Hb[b][2][0], Hb[b][2][1]);
            }
            mfma32(lds.w2[p][t][lane], x, acc[p]);
            mfma16(reinterpret_cast<uint2 const*>(&lds.w2[p][t][64])[lane], xt, acc[p]);
        }
        v4f const bias = *reinterpret_cast<v4f const*>(&lds.bias[V::T0 + V::T1 + t][g][0]);
#pragma unroll
        for (int b = 0; b < 4; ++b) fp8_epilogue<true>(acc[2][b], acc[1][b], acc[0][b], bias, Ha[b][t]);
    }
    // output layer: 32 -> 16, exact: |sum W q| <= 32 * 127 * 128 < 2^24
    {
        v4f acc[4] = { zero, zero, zero, zero };
        uint4 x[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) x[b] = make_uint4(Ha[b][0][0], Ha[b][0][1], Ha[b][1][0], Ha[b][1][1]);
        mfma32(lds.w3[lane], x, acc);
        v4i const bias = *reinterpret_cast<v4i const*>(&lds.outBias[g][0]);
        S = *reinterpret_cast<v4f const*>(&lds.outScale[g][0]);
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r) D[b][r] = int(uint32_t(int(acc[b][r])) + uint32_t(bias[r]));      // wraps like int32
    }
}

// 76.5 KB of LDS: two workgroups per CU.
template <class V>
__global__ void __launch_bounds__(V::THREADS, 2)
decode_fp8_kernel(DevMip const* __restrict__ mips, int numMips, int totalTiles)
{
    __shared__ Fp8Lds lds;
    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const j = lane & 15, g = lane >> 4;

    int const per = (totalTiles + gridDim.x - 1) / gridDim.x;
    int const tileBegin = blockIdx.x * per;
    int const tileEnd = min(totalTiles, tileBegin + per);

    uint8_t const* stagedBlob = nullptr;
    int entry = 0;
    for (int tile = tileBegin; tile < tileEnd; ++tile) {
        while (entry + 1 < numMips && mips[entry + 1].tileStart <= tile) ++entry;
        if (mips[entry].weights != stagedBlob) {             // uniform across the workgroup
            __syncthreads();
            stage_fp8_weights<V>(lds, mips[entry].weights);
            stagedBlob = mips[entry].weights;
            __syncthreads();
        }
        DevMip const& m = mips[entry];
        int const local = tile - m.tileStart;
        int const tileY = local / m.tilesX, tileX = local - tileY * m.tilesX;
        int const x0 = tileX * 64 + wave * 16;
        int const y0 = tileY * 4;
        if (x0 >= m.width) continue;                         // whole wave tile outside the image

        uint32_t in[24];
        prepare_inputs_fp8<V>(m, min(x0 + j, m.width - 1), min(y0 + g, m.height - 1), in);
        v4i D[4];
        v4f S;
        mlp_forward_fp8<V>(lds, wave, lane, in, D, S);
        if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS)      store_tile<NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS>(m, D, S, x0 + j, y0, 4 * g);
        else if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PIXELS)       store_tile<NTC_HIP_DEV_OUT_FP16_PIXELS>(m, D, S, x0 + j, y0, 4 * g);
        else                                                       store_tile<NTC_HIP_DEV_OUT_UNORM8_PIXELS>(m, D, S, x0 + j, y0, 4 * g);
    }
}

// The two fp16 primitives of the activation stage applied to a list of halves (for the tests): out[0..n) the
// HGELU-clamp result, out[n..2n) the input rounded to e4m3, out[2n..3n) the int8 quantisation of the input.
__global__ void selftest_fp8_activation_kernel(uint16_t const* __restrict__ in, uint16_t* __restrict__ out, int n)
{
    int const i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint32_t const pair = uint32_t(in[i]) | (uint32_t(in[i]) << 16);
    out[i] = uint16_t(hgelu_pk(pair) >> 16);
    out[n + i] = uint16_t(round_e4m3_pk(pair));
    out[2 * n + i] = uint16_t(quantize_int8_pk(pair) >> 16);
}

using VFp8_16 = Fp8Variant<16>;
using VFp8_12 = Fp8Variant<12>;
using VFp8_8  = Fp8Variant<8>;
using VFp8_4  = Fp8Variant<4>;

template <class V>
static hipError_t launch_fp8_variant(DevMip const* mips, int numMips, int totalTiles, int gridSize, hipStream_t stream)
{
    hipLaunchKernelGGL(decode_fp8_kernel<V>, dim3(gridSize), dim3(V::THREADS), 0, stream, mips, numMips, totalTiles);
    return hipGetLastError();
}

hipError_t launch_decode_fp8(int variant, DevMip const* mips, int numMips, int totalTiles, int gridSize, hipStream_t stream)
{
    switch (variant) {
    case NTC_HIP_VARIANT_REF16_FP8: return launch_fp8_variant<VFp8_16>(mips, numMips, totalTiles, gridSize, stream);
    case NTC_HIP_VARIANT_REF12_FP8: return launch_fp8_variant<VFp8_12>(mips, numMips, totalTiles, gridSize, stream);
    case NTC_HIP_VARIANT_REF8_FP8:  return launch_fp8_variant<VFp8_8>(mips, numMips, totalTiles, gridSize, stream);
    case NTC_HIP_VARIANT_REF4_FP8:  return launch_fp8_variant<VFp8_4>(mips, numMips, totalTiles, gridSize, stream);
    default: return hipErrorInvalidValue;
    }
}

int resident_fp8_workgroups_per_cu()
{
    int blocks = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, decode_fp8_kernel<VFp8_16>, VFp8_16::THREADS, 0) != hipSuccess || blocks < 1) blocks = 2;
    return blocks;
}

hipError_t launch_selftest_fp8_activation(uint16_t const* in, uint16_t* out, int n, hipStream_t stream)
{
    hipLaunchKernelGGL(selftest_fp8_activation_kernel, dim3(unsigned((n + 255) / 256)), dim3(256), 0, stream, in, out, n);
    return hipGetLastError();
}

} // namespace ntc_hip_dev
