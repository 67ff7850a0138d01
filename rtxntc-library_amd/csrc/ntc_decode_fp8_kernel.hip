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
// launch, a workgroup tile of 64 x 4 texels = four wave tiles of 32 x 2 (see decode_kernel); lane = texel in the input stage,
// lane (j = lane%16, g = lane/16) = channels 16t+4g..+3 of texel j in the matrix stages.
#include "ntc_decode_device.h"
#include <type_traits>

namespace ntc_hip_dev {

typedef short v2s __attribute__((ext_vector_type(2)));

// Two halves -> the nearest e4m3 values (as halves): v_cvt_scalef32_pk_fp8_f16 and back, scale 1.  The first
// instruction writes the two bytes into one half of its destination and keeps the other half; that other half
// is never read here, so the destination starts as the source itself and needs no clearing.
__device__ __forceinline__ uint32_t round_e4m3_pk(uint32_t halves)
{
    v2s const bytes = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(__builtin_bit_cast(v2s, halves), __builtin_bit_cast(v2h, halves), 1.0f, false);
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

// HGELU-clamp on two fp16 layer outputs (NtcHGELUClamp_Forward_CoopVec, InferenceCoopVec.hlsli:150-153):
// v_pk_fma_f16 with clamp, v_pk_max_f16, v_pk_min_f16, v_pk_mul_f16.  Written as vector arithmetic, not as
// inline assembly: these instructions are interleaved with matrix instructions, and the compiler inserts the
// wait states an in-flight matrix instruction needs (e.g. before one of its source registers is overwritten)
// only around instructions it can see.
// LOWER_CLAMP false leaves out max(x, -3).  For finite x < -3 that changes nothing: t is +0 from x = -1.5 down,
// and x * (+0) = -3 * (+0) = -0.  It differs for x = -Inf or NaN only (-Inf * 0 is NaN, -3 * 0 is not), so it is
// for layers whose outputs are known to be finite.
template <bool LOWER_CLAMP = true>
__device__ __forceinline__ uint32_t hgelu_pk(uint32_t xBits)
{
    v2h const x = __builtin_bit_cast(v2h, xBits);
    v2h const third = __builtin_bit_cast(v2h, 0x35553555u), half = { _Float16(0.5f), _Float16(0.5f) };
    v2h const zero = { _Float16(0.f), _Float16(0.f) }, one = { _Float16(1.f), _Float16(1.f) }, three = { _Float16(3.f), _Float16(3.f) };
    v2h t = __builtin_elementwise_fma(x, third, half);
    t = __builtin_elementwise_min(__builtin_elementwise_max(t, zero), one);
    v2h const xc = __builtin_elementwise_min(LOWER_CLAMP ? __builtin_elementwise_max(x, -three) : x, three);
    return __builtin_bit_cast(uint32_t, xc * t);
}

// After the last hidden layer: q = rne(80 y - 113) as fp16 integers in [-128, 127] (hlsli:155-158).
__device__ __forceinline__ uint32_t quantize_int8_pk(uint32_t yBits)
{
    v2h const y = __builtin_bit_cast(v2h, yBits);
    v2h const eighty = { _Float16(80.f), _Float16(80.f) }, c1423 = { _Float16(1423.f), _Float16(1423.f) };
    v2h const minus1536 = { _Float16(-1536.f), _Float16(-1536.f) };
    v2h z = __builtin_elementwise_fma(y, eighty, c1423);
    asm("" : "+v"(z));                                       // keeps the two roundings apart
    return __builtin_bit_cast(uint32_t, z + minus1536);
}

// ONE_: the instantiation for texture sets all of whose hidden layers run on one weight plane (see
// classify_fp8_weights): it holds one plane in LDS instead of three, which leaves room for the transposition
// buffers of sixteen waves, and its network has one form per layer, which fits the 128 registers four waves per
// SIMD leave a lane (108 used; the general form needs 150).  The two instantiations are launched one after the
// other; each decodes the sets that are its own.
template <int FEATURES_, bool ONE_ = false>
struct Fp8Variant {
    static constexpr bool ONE = ONE_;
    static constexpr int HELD = ONE_ ? 1 : 3;                // weight planes kept in LDS
    static constexpr int F = FEATURES_;                      // features stored per cell of either grid (slots: 16)
    static constexpr int IN = 48, H0 = 64, H1 = 48, H2 = 32, OUT = 16;      // InferenceConstants.h:28-40
    static constexpr int T0 = H0 / 16, T1 = H1 / 16, T2 = H2 / 16;
    static constexpr int PLANES = 3;
    static constexpr int W1_OFF = IN * H0, W2_OFF = W1_OFF + H0 * H1, W3_OFF = W2_OFF + H1 * H2;
    static constexpr int WEIGHT_BYTES = W3_OFF + H2 * OUT;
    // src/WeightLayout.cpp:249-262: fp16 biases of the three e4m3 layers, then scale and bias of the output layer
    static constexpr int BIAS_OFF = WEIGHT_BYTES, SCALE3_OFF = BIAS_OFF + 2 * (H0 + H1 + H2), BIAS3_OFF = SCALE3_OFF + 4 * OUT;
    // Twelve waves (sixteen with one plane) share one copy of the weight planes: one workgroup per CU, three (four)
    // waves per SIMD, working on GROUP tiles at a time.
    static constexpr int WAVES = ONE_ ? 16 : 12, THREADS = 64 * WAVES, GROUP = WAVES / 4;
    static constexpr int IN_STRIDE = 28;                     // dwords per texel in the transpose buffer: 24 + 4 of padding
};

// A operands in LDS, in 16-byte units.  A block for 32 inputs holds one unit per lane (8 halves), a block for
// 16 inputs half a unit per lane (4 halves, 32 units).
template <int HELD, int WAVES>
struct alignas(16) Fp8LdsT {
    uint4 w0[HELD][4][96];     // layer 0, inputs in their natural order: [plane][output tile][K32 block | K16 block]
    uint4 w1[HELD][3][128];    // layer 1: two blocks of 32 (input-tile pairs 0-1, 2-3)
    uint4 w2[HELD][2][96];     // layer 2: input-tile pair 0-1, then input tile 2
    uint4 w3[64];              // output layer (int8 weights as halves): input-tile pair 0-1
    float bias[9][4][4];       // hidden layers: [output tile of layers 0..2][g][r] -> channel 16t+4g+r
    float outScale[4][4];      // output layer: [g][r]
    int32_t outBias[4][4];
    uint32_t in[WAVES][kWaveTexels][28];
    // Positional encoding for every power-of-two positionScale 2^-k, k = 0..5: the entry for phase p of scale
    // 2^-k sits at index (2^k - 1) + p; dwords 0..2 hold enc(px * 2^w), dwords 3..5 enc(px * 2^w + 1/4), w = 0..2,
    // as e4m3-rounded halves in the low 16 bits (px = p * 2^-k).
    uint32_t postab[64][8];
    // Filtered feature -> network input, for the integer input stage: entry kFeatureLutBase(n) + T holds the
    // e4m3-rounded half of fma(float(T), (2/15) * 2^-n, -1) for T = 0 .. 15 * 2^n, n = 0, 2, 4, 6 (what square
    // power-of-two geometry produces; other n take the arithmetic).
    uint16_t featureLut[1280];
    // classify_fp8_weights: sum |512 w| of every output channel of the three hidden layers, and the flags it gathers
    int32_t channelSum[3][64];
    uint32_t classFlags;
};
template <class V> using Fp8Lds = Fp8LdsT<V::HELD, V::WAVES>;
__host__ __device__ constexpr int kFeatureLutBase(int n) { return n == 0 ? 0 : (n == 2 ? 16 : (n == 4 ? 77 : 318)); }   // 16 + 61 + 241 + 961 = 1279 entries

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
__device__ __forceinline__ _Float16 plane_value(int32_t w512, int plane, bool whole = false)
{
    if (whole) return _Float16(float(w512) * 0x1p-9f);       // the weight itself: every e4m3 value is a half
    int32_t const mag = w512 < 0 ? -w512 : w512;
    int32_t const bits = plane == 2 ? mag >> 14 : (mag >> (7 * plane)) & 127;
    float const unit = plane == 0 ? 0x1p-9f : (plane == 1 ? 0x1p-2f : 0x1p5f);
    float const v = float(bits) * unit;
    return _Float16(w512 < 0 ? -v : v);
}

// Stores the 8 (or 4) halves of one lane of an A block: weights W[row][k[e]] of one plane.
template <class V>
__device__ __forceinline__ void stage_plane_halves(uint32_t* dst, uint8_t const* __restrict__ matrix, int in, int row, int const* k, int count, int plane,
                                                   bool whole)
{
    for (int e = 0; e < count; e += 2) {
        _Float16 const a = plane_value(fp8_times_512(matrix[row * in + k[e]]), plane, whole);
        _Float16 const b = plane_value(fp8_times_512(matrix[row * in + k[e + 1]]), plane, whole);
        v2h const h = { a, b };
        dst[e >> 1] = __builtin_bit_cast(uint32_t, h);
    }
}

// Copies the FP8 blob into LDS in matrix-instruction operand order.  Layer 0 takes its inputs in their
// natural order (lane (i, kg) of a block of 32 holds inputs 8kg..8kg+7, of a block of 16 inputs 32+4kg..+3);
// layers 1..3 take theirs in the order the previous layer's result registers hold them: lane (i, kg) of the
// block for input tiles (2p, 2p+1) holds inputs 16*(2p + e/4) + 4kg + e%4, e = 0..7.
// stage_fp8_weights takes the layers' modes from classify_fp8_weights, which reads the blob only.  Bit l is set when hidden layer l needs the general evaluation (three planes, both
// clamps of the activation), i.e. when some weight of it has a non-zero top plane (|w| >= 32) or some bias is not
// a finite half of magnitude <= 57344.  The other layers (every layer of a trained network) are "tame": two
// planes, and since |sum| <= 64 * 31.75 * 3 = 6096 their outputs stay below 63440 + rounding < 65520, finite as
// halves.  Bit 4 + l is set when a tame layer needs ONE plane only, the weights themselves (stored in plane 0's
// place): when for every output channel  sum_k |512 w_k| * 1536 < 2^24.  Inputs are at most 3 in magnitude
// (1536 units of 2^-9), every product is a multiple of 2^-18, so every partial sum of a channel's dot product, in
// any order, is then a multiple of 2^-18 below 2^24 of them: exact in fp32.  The sums of the planes are such
// partial sums and so are (s2 + s1) and ((s2 + s1) + s0): the three-part evaluation the contract prescribes
// performs no rounding before the bias is added, and one matrix-instruction chain over the whole weights gives
// the same bits with half the matrix instructions and one addition less per activation.
constexpr int32_t kOnePlaneLimit = ((1 << 24) - 1) / 1536;   // largest sum_k |512 w_k| with sum * 1536 < 2^24: 10922
constexpr int kOnePlaneShift = 4;

constexpr int kAllOnePlane = 7 << kOnePlaneShift;         // every hidden layer runs on one plane
// Bit 8: no output can come near the fp16 overflow threshold, so stores may skip that check.  The output layer's
// int32 accumulator is at most 32 * 127 * 128 = 520192 in magnitude before the bias; bounded means
// (|bias| + 520192) * |scale| < 60000 for every channel (no wrap of the int32 sum either: that is far below 2^31
// unless the scale is tiny, and then |bias| itself must be checked).
constexpr int kFp8OutputsBounded = 1 << 8;

// Reads the blob a dword per thread (the api requires 4-byte alignment; rows of 48 or 64 bytes: a dword never
// straddles two channels) and gathers sums and flags in LDS: every workgroup of both instantiations does this for
// every set it meets, and the workgroups of the one that passes over the set do nothing else.
template <class V>
__device__ int classify_fp8_weights(Fp8Lds<V>& lds, uint8_t const* __restrict__ blob)
{
    int const tid = threadIdx.x;
    constexpr int rows[3] = { V::H0, V::H1, V::H2 }, ins[3] = { V::IN, V::H0, V::H1 };
    constexpr int dwords[3] = { V::W1_OFF / 4, (V::W2_OFF - V::W1_OFF) / 4, (V::W3_OFF - V::W2_OFF) / 4 };
    static_assert(V::IN % 4 == 0 && V::H0 % 4 == 0 && V::H1 % 4 == 0 && V::H0 <= 64, "a dword of weights belongs to one channel");
    if (tid == 0) lds.classFlags = 0;
    if (tid < 192) (&lds.channelSum[0][0])[tid] = 0;
    __syncthreads();                                         // also: every wave has left the previous set's tiles
    for (int e = tid; e < dwords[0] + dwords[1] + dwords[2]; e += V::THREADS) {
        int const l = e < dwords[0] ? 0 : (e < dwords[0] + dwords[1] ? 1 : 2);
        int const d = e - (l == 0 ? 0 : (l == 1 ? dwords[0] : dwords[0] + dwords[1]));
        uint32_t const four = reinterpret_cast<uint32_t const*>(blob)[e];      // the three matrices follow each other
        int32_t sum = 0, top = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            int32_t const w = fp8_times_512((four >> (8 * q)) & 0xffu);
            int32_t const mag = w < 0 ? -w : w;
            sum += mag;
            top |= mag >> 14;
        }
        atomicAdd(&lds.channelSum[l][(4 * d) / ins[l]], sum);
        if (top) atomicOr(&lds.classFlags, 1u << l);
    }
    if (tid < V::OUT) {
        float const bias = fabsf(float(reinterpret_cast<int32_t const*>(blob + V::BIAS3_OFF)[tid]));
        float const scale = fabsf(reinterpret_cast<float const*>(blob + V::SCALE3_OFF)[tid]);
        if (!((bias + 520192.f) * scale < 60000.f) || !(bias < 2.0e9f)) atomicOr(&lds.classFlags, 1u << 8);
    }
    if (tid < V::H0 + V::H1 + V::H2) {                       // a bias that is not a finite half of at most 57344
        int const l = tid < V::H0 ? 0 : (tid < V::H0 + V::H1 ? 1 : 2);
        if ((reinterpret_cast<uint16_t const*>(blob + V::BIAS_OFF)[tid] & 0x7fffu) > 0x7b00u) atomicOr(&lds.classFlags, 1u << l);
    }
    __syncthreads();
    if (tid < 192) {
        int const l = tid >> 6, r = tid & 63;
        if (r < rows[l] && lds.channelSum[l][r] > kOnePlaneLimit) atomicOr(&lds.classFlags, 16u << l);
    }
    __syncthreads();
    uint32_t const flags = lds.classFlags;
    __syncthreads();                                         // read by all before the next call clears it
    int const topMask = int(flags & 7u);
    int const oneMask = int(~(flags >> 4) & ~flags & 7u);
    return topMask | (oneMask << kOnePlaneShift) | ((flags & (1u << 8)) ? 0 : kFp8OutputsBounded);
}

template <class V>
__device__ void stage_fp8_weights(Fp8Lds<V>& lds, uint8_t const* __restrict__ blob, int modes)
{
    int const tid = threadIdx.x;
    int const oneMask = modes >> kOnePlaneShift;
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
    for (int e = tid; e < V::HELD * V::T0 * 64; e += V::THREADS) {
        int const lane = e & 63, t = (e >> 6) % V::T0, p = e / (64 * V::T0);
        int const i = lane & 15, kg = lane >> 4;
        int k32[8], k16[4];
        for (int q = 0; q < 8; ++q) k32[q] = 8 * kg + q;
        for (int q = 0; q < 4; ++q) k16[q] = 32 + 4 * kg + q;
        bool const whole = p == 0 && (oneMask & 1);
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w0[p][t][lane]), blob, V::IN, 16 * t + i, k32, 8, p, whole);
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w0[p][t][64]) + 2 * lane, blob, V::IN, 16 * t + i, k16, 4, p, whole);
    }
    // layer 1: 64 inputs = two blocks of 32
    for (int e = tid; e < V::HELD * V::T1 * 2 * 64; e += V::THREADS) {
        int const lane = e & 63, pair = (e >> 6) & 1, t = (e >> 7) % V::T1, p = e / (128 * V::T1);
        int const i = lane & 15, kg = lane >> 4;
        int k[8];
        for (int q = 0; q < 8; ++q) k[q] = 16 * (2 * pair + q / 4) + 4 * kg + q % 4;
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w1[p][t][pair * 64 + lane]), blob + V::W1_OFF, V::H0, 16 * t + i, k, 8, p, p == 0 && (oneMask & 2));
    }
    // layer 2: 48 inputs = one block of 32 and one of 16
    for (int e = tid; e < V::HELD * V::T2 * 64; e += V::THREADS) {
        int const lane = e & 63, t = (e >> 6) % V::T2, p = e / (64 * V::T2);
        int const i = lane & 15, kg = lane >> 4;
        int k32[8], k16[4];
        for (int q = 0; q < 8; ++q) k32[q] = 16 * (q / 4) + 4 * kg + q % 4;
        for (int q = 0; q < 4; ++q) k16[q] = 32 + 4 * kg + q;
        bool const whole = p == 0 && (oneMask & 4);
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w2[p][t][lane]), blob + V::W2_OFF, V::H1, 16 * t + i, k32, 8, p, whole);
        stage_plane_halves<V>(reinterpret_cast<uint32_t*>(&lds.w2[p][t][64]) + 2 * lane, blob + V::W2_OFF, V::H1, 16 * t + i, k16, 4, p, whole);
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

// The same 24 dwords from integer arithmetic, for mips whose sizes, grid sizes and positionScale are powers of
// two (DevMip::fast).  There every float operation of prepare_inputs_fp8 is exact up to the fused multiply-add:
// the filtered feature is t = T / 2^n with the integer T = sum w*q (weights w = products of the axis fractions,
// summing to 2^n, n <= 8), and fma(t, c, -1) = fma(float(T), c * 2^-n, -1) is the same real number rounded
// once.  T comes from the packed 16-bit-lane filter of the int8 kernel: a cell c = f0 | f1<<4 | f2<<8 | f3<<12
// is spread to P = byte0 | byte1<<16, E = P & 0x000f000f holds the even features, S = sum w*P and T = sum w*E
// stay below 2^16 per lane, and (S - T) / 16 holds the odd features.  The positional encoding of texel x depends
// only on x mod 2^k for positionScale = 2^-k and comes from a table in LDS.
//
// The stage comes in two halves so that a tile's latent loads can be in flight while the previous tile runs
// through the network: fetch_latents_fast issues the loads (four taps of every stored layer of both grids) and
// keeps the four axis fractions, finish_inputs_fast does the arithmetic.
template <class V>
struct Fp8Fetch {
    static constexpr int LAYERS = (V::F + 3) / 4;
    uint32_t cell[2][LAYERS][4];                             // [grid][layer][tap 00, 10, 01, 11]
    uint32_t fx[2], fy[2];                                   // axis fractions of the footprint, per grid
};

template <class V, class Mip>
__device__ __forceinline__ void fetch_latents_fast(Mip const& m, int x, int y, Fp8Fetch<V>& f)
{
#pragma unroll
    for (int grid = 0; grid < 2; ++grid) {
        uint32_t const axisX = grid == 0 ? m.hrAxisX : m.lrAxisX, axisY = grid == 0 ? m.hrAxisY : m.lrAxisY;
        int const gw = grid == 0 ? m.hrWidth : m.lrWidth, gh = grid == 0 ? m.hrHeight : m.lrHeight;
        AxisFoot const ax = axis_fast(x, axisX, gw), ay = axis_fast(y, axisY, gh);
        GlobalU8Ptr const g = (GlobalU8Ptr)(grid == 0 ? m.hr : m.lr);
        uint32_t const lgw = ((axisX >> 24) & 0xffu) + 1u;       // log2(bytes per grid row)
        uint32_t const layerStride = uint32_t(gw) * uint32_t(gh) * 2u;   // bytes
        uint32_t const r0 = ay.c0 << lgw, r1 = ay.c1 << lgw, c0 = ax.c0 << 1, c1 = ax.c1 << 1;
        uint32_t const a00 = r0 + c0, a10 = r0 + c1, a01 = r1 + c0, a11 = r1 + c1;   // byte offsets
        f.fx[grid] = ax.f; f.fy[grid] = ay.f;
#pragma unroll
        for (int L = 0; L < Fp8Fetch<V>::LAYERS; ++L) {
            GlobalU8Ptr const gl = g + size_t(L) * layerStride;
            f.cell[grid][L][0] = load_u16(gl, a00); f.cell[grid][L][1] = load_u16(gl, a10);
            f.cell[grid][L][2] = load_u16(gl, a01); f.cell[grid][L][3] = load_u16(gl, a11);
        }
    }
}

// The same cells from the query-ordered copy of the grids (bricks with all layers of a cell together): four
// loads per grid instead of four per layer.
template <class V, class Mip>
__device__ __forceinline__ void fetch_latents_bricked(Mip const& m, int x, int y, Fp8Fetch<V>& f)
{
    constexpr int LAYERS = Fp8Fetch<V>::LAYERS;
#pragma unroll
    for (int grid = 0; grid < 2; ++grid) {
        uint32_t const axisX = grid == 0 ? m.hrAxisX : m.lrAxisX, axisY = grid == 0 ? m.hrAxisY : m.lrAxisY;
        int const gw = grid == 0 ? m.hrWidth : m.lrWidth, gh = grid == 0 ? m.hrHeight : m.lrHeight;
        AxisFoot const ax = axis_fast(x, axisX, gw), ay = axis_fast(y, axisY, gh);
        GlobalU8Ptr const g = (GlobalU8Ptr)(grid == 0 ? m.hrBricks : m.lrBricks);
        uint32_t const lg = (axisX >> 24) & 0xffu;                // log2(grid width)
        f.fx[grid] = ax.f; f.fy[grid] = ay.f;
        uint32_t cell[4][2];                                      // taps 00, 10, 01, 11
        load_brick_cell<LAYERS>(g, brick_offset<LAYERS>(ax.c0, ay.c0, lg), cell[0]);
        load_brick_cell<LAYERS>(g, brick_offset<LAYERS>(ax.c1, ay.c0, lg), cell[1]);
        load_brick_cell<LAYERS>(g, brick_offset<LAYERS>(ax.c0, ay.c1, lg), cell[2]);
        load_brick_cell<LAYERS>(g, brick_offset<LAYERS>(ax.c1, ay.c1, lg), cell[3]);
#pragma unroll
        for (int L = 0; L < LAYERS; ++L)
#pragma unroll
            for (int tap = 0; tap < 4; ++tap)
                f.cell[grid][L][tap] = (L & 1) ? cell[tap][L >> 1] >> 16 : cell[tap][L >> 1] & 0xffffu;
    }
}

template <class V, class Mip>
__device__ __forceinline__ void finish_inputs_fast(Mip const& m, Fp8Lds<V> const& lds, int x, int y, Fp8Fetch<V> const& f, uint32_t (&in)[24])
{
#pragma unroll
    for (int i = 0; i < 24; ++i) in[i] = 0;
#pragma unroll
    for (int grid = 0; grid < 2; ++grid) {
        uint32_t const axisX = grid == 0 ? m.hrAxisX : m.lrAxisX, axisY = grid == 0 ? m.hrAxisY : m.lrAxisY;
        uint32_t const nx = (axisX >> 8) & 0xffu, ny = (axisY >> 8) & 0xffu;
        uint32_t const wx1 = f.fx[grid], wx0 = (1u << nx) - wx1, wy1 = f.fy[grid], wy0 = (1u << ny) - wy1;
        uint32_t const msk = 0x000f000fu, sel = 0x0c010c00u;     // v_perm_b32: bytes [0, zero, 1, zero] of the cell
        uint32_t const n = nx + ny;
        if (V::F % 4 == 0 && n <= 6u && !(n & 1u)) {             // (uniform in the raster kernel, per lane for queries)
            // Table form: with doubled weights and start values 2*base resp. 17 * 2*base the 16-bit lanes of T and
            // O come out as byte offsets into the table (S stays below 2^16: 2 * 255 * 64 + 34 * 318).
            uint32_t const w00 = mul24(2u * wx0, wy0), w10 = mul24(2u * wx1, wy0), w01 = mul24(2u * wx0, wy1), w11 = mul24(2u * wx1, wy1);
            uint32_t const base = uint32_t(n == 0u ? kFeatureLutBase(0) : (n == 2u ? kFeatureLutBase(2) : (n == 4u ? kFeatureLutBase(4) : kFeatureLutBase(6))));
            uint32_t const t0 = (2u * base) * 0x00010001u, s0 = 17u * t0;
            uint8_t const* const lut = reinterpret_cast<uint8_t const*>(lds.featureLut);
#pragma unroll
            for (int L = 0; L < Fp8Fetch<V>::LAYERS; ++L) {
                uint32_t const p00 = __builtin_amdgcn_perm(0u, f.cell[grid][L][0], sel), p10 = __builtin_amdgcn_perm(0u, f.cell[grid][L][1], sel);
                uint32_t const p01 = __builtin_amdgcn_perm(0u, f.cell[grid][L][2], sel), p11 = __builtin_amdgcn_perm(0u, f.cell[grid][L][3], sel);
                uint32_t const S = mad24(w11, p11, mad24(w01, p01, mad24(w10, p10, mad24(w00, p00, s0))));
                uint32_t const T = mad24(w11, p11 & msk, mad24(w01, p01 & msk, mad24(w10, p10 & msk, mad24(w00, p00 & msk, t0))));
                uint32_t const O = (S - T) >> 4;
                v2s const a = { short(*reinterpret_cast<uint16_t const*>(lut + (T & 0xffffu))), short(*reinterpret_cast<uint16_t const*>(lut + (O & 0xffffu))) };
                v2s const b = { short(*reinterpret_cast<uint16_t const*>(lut + (T >> 16))), short(*reinterpret_cast<uint16_t const*>(lut + (O >> 16))) };
                in[8 * grid + 2 * L]     = __builtin_bit_cast(uint32_t, a);
                in[8 * grid + 2 * L + 1] = __builtin_bit_cast(uint32_t, b);
            }
            continue;
        }
        uint32_t const w00 = mul24(wx0, wy0), w10 = mul24(wx1, wy0), w01 = mul24(wx0, wy1), w11 = mul24(wx1, wy1);
        float const k = __builtin_ldexpf(0.13333334f, -int(nx + ny));
#pragma unroll
        for (int L = 0; L < Fp8Fetch<V>::LAYERS; ++L) {
            uint32_t const p00 = __builtin_amdgcn_perm(0u, f.cell[grid][L][0], sel), p10 = __builtin_amdgcn_perm(0u, f.cell[grid][L][1], sel);
            uint32_t const p01 = __builtin_amdgcn_perm(0u, f.cell[grid][L][2], sel), p11 = __builtin_amdgcn_perm(0u, f.cell[grid][L][3], sel);
            uint32_t const S = mad24(w11, p11, mad24(w01, p01, mad24(w10, p10, mul24(w00, p00))));
            uint32_t const T = mad24(w11, p11 & msk, mad24(w01, p01 & msk, mad24(w10, p10 & msk, mul24(w00, p00 & msk))));
            uint32_t const O = (S - T) >> 4;                     // lanes: features 1 and 3; T: features 0 and 2
            float value[4] = { float(T & 0xffffu), float(O & 0xffffu), float(T >> 16), float(O >> 16) };
#pragma unroll
            for (int i = 0; i < 4; ++i) value[i] = (4 * L + i < V::F) ? __builtin_fmaf(value[i], k, -1.f) : 0.f;
            in[8 * grid + 2 * L]     = round_e4m3_pk(halves_rne(value[0], value[1]));
            in[8 * grid + 2 * L + 1] = round_e4m3_pk(halves_rne(value[2], value[3]));
        }
    }
    {
        uint32_t const* const ex = lds.postab[m.posMask + (uint32_t(x) & m.posMask)];
        uint32_t const* const ey = lds.postab[m.posMask + (uint32_t(y) & m.posMask)];
        uint4 const x0 = *reinterpret_cast<uint4 const*>(ex), y0 = *reinterpret_cast<uint4 const*>(ey);
        uint2 const x1 = *reinterpret_cast<uint2 const*>(ex + 4), y1 = *reinterpret_cast<uint2 const*>(ey + 4);
        in[16] = x0.x | (y0.x << 16);  in[17] = x0.w | (y0.w << 16);     // (e0, e1), (e2, e3) of wave 0
        in[18] = x0.y | (y0.y << 16);  in[19] = x1.x | (y1.x << 16);
        in[20] = x0.z | (y0.z << 16);  in[21] = x1.y | (y1.y << 16);
    }
    in[22] = round_e4m3_pk(halves_rne(m.positionLod, m.positionLod));
}

// Fills the positional table: one entry per thread, threads 0..62.
template <class Lds>
__device__ void build_fp8_posenc_table(Lds& lds)
{
    int const t = threadIdx.x;
    if (t < 63) {
        int const k = 31 - __builtin_clz(uint32_t(t + 1));   // floor(log2(t + 1))
        int const phase = t + 1 - (1 << k);
        float p = float(phase) * __builtin_ldexpf(1.f, -k);
#pragma unroll
        for (int w = 0; w < 3; ++w) {
            float const q = p + 0.25f;
            float const e0 = (p - floorf(p)) * 2.f - 1.f, e2 = (q - floorf(q)) * 2.f - 1.f;
            uint32_t const pair = round_e4m3_pk(halves_rne(e0, e2));
            lds.postab[t][w] = pair & 0xffffu;
            lds.postab[t][3 + w] = pair >> 16;
            p *= 2.f;
        }
        lds.postab[t][6] = lds.postab[t][7] = 0;
    }
}

// Fills the feature table with the same operations the arithmetic path applies per lane.
template <class Lds>
__device__ void build_fp8_feature_lut(Lds& lds)
{
    for (int e = threadIdx.x; e < 1279; e += blockDim.x) {
        int const n = e < 16 ? 0 : (e < 77 ? 2 : (e < 318 ? 4 : 6));
        int const T = e - kFeatureLutBase(n);
        float const v = __builtin_fmaf(float(T), __builtin_ldexpf(0.13333334f, -n), -1.f);
        lds.featureLut[e] = uint16_t(round_e4m3_pk(halves_rne(v, v)));
    }
}

// One hidden layer's epilogue for the four channels a lane holds of one texel: sums of the three planes ->
// layer output -> activation -> the next layer's inputs (two dwords of halves).
// With PLANES < 3 the layer is tame (see stage_fp8_weights): the top plane of its weights is all zero,
// s2 = +0 and (s2 + s1) = s1 exactly (a plane's sum is never -0: its accumulator starts at +0), so the first
// addition is left out; and its outputs are finite, so the activation's lower clamp is left out too.  With
// PLANES == 1, s0 is the sum over the whole weights, which is what ((s2 + s1) + s0) comes to there without rounding.
template <bool LAST_HIDDEN, int PLANES>
__device__ __forceinline__ void fp8_epilogue(v4f s2, v4f s1, v4f s0, v4f bias, uint32_t (&out)[2])
{
    float r[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float a = s0[i];
        if (PLANES == 3)      a = (s2[i] + s1[i]) + s0[i];
        else if (PLANES == 2) a = s1[i] + s0[i];
        r[i] = a + bias[i];
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        uint32_t const y = hgelu_pk<PLANES == 3>(halves_rne(r[2 * h], r[2 * h + 1]));
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
// The same for a block of 16 inputs.  32-deep and 16-deep instructions are never mixed in one accumulator's
// chain: in either order that gave wrong sums here with some instruction schedules (the wait between the two
// was not always there; compiling with padded matrix instructions made the same code correct), while chains of
// one kind are reliable.  Layers whose input count is not a multiple of 32 therefore split their 32-deep blocks
// with mfma32_as_two_16: a block's unit holds k-slots 8kg..8kg+7 of lane (i, kg) on both sides, so its first and
// last four halves are two valid 16-deep operands.  (The other way round - the block of 16 padded with zero
// weights to a 32-deep instruction, 148 instead of 196 matrix instructions per wave tile - measured 1.5 % slower:
// two 16-deep instructions cost this kernel no more than one 32-deep one.)
__device__ __forceinline__ void mfma16(uint2 const& a, uint2 const (&x)[4], v4f (&acc)[4])
{
    v4h const A = __builtin_bit_cast(v4h, a);
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[b] = __builtin_amdgcn_mfma_f32_16x16x16f16(A, __builtin_bit_cast(v4h, x[b]), acc[b], 0, 0, 0);
}
__device__ __forceinline__ void mfma32_as_two_16(uint4 const& a, uint4 const (&x)[4], v4f (&acc)[4])
{
    uint2 lo[4], hi[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) { lo[b] = make_uint2(x[b].x, x[b].y); hi[b] = make_uint2(x[b].z, x[b].w); }
    mfma16(make_uint2(a.x, a.y), lo, acc);
    mfma16(make_uint2(a.z, a.w), hi, acc);
}

// The wave's priority with the SIMD's arbiter, per part of a tile.  This network's activation stage is packed fp16
// arithmetic and conversions - instructions that take an issue slot alone - and it is what the SIMD's time goes to;
// the wave that has reached it goes first, matrix instructions (which then run in the shadow of other waves'
// activation stages) and the input stage and stores last: one-plane sets -6.3 %, two-plane sets -8.2 %.  Any setting
// with the activation stage above the rest measures the same; with the matrix instructions on top instead (what the
// Int8 network's kernel wants, whose fp32 requantiser pairs up between waves) nothing is gained, and with the input
// stage as high as the activation stage nothing either.
constexpr int kPrioMatrix = 0, kPrioEpilogue = 2, kPrioOther = 1;

// Hidden layers.  PLANES = 3, 2 for a tame layer, 1 where the whole weights sum exactly (see stage_fp8_weights).
template <int NK32, bool HAS16>
struct TileOperands { uint4 a32[3][NK32]; uint2 a16[3]; v4f bias; };     // one output tile's weight operands and bias

// One hidden layer: TILES output tiles of 16 channels; its inputs as NK32 blocks of 32 (B32[kb][b]) and, with
// HAS16, one block of 16 (B16[b]); load(t, operands) reads tile t's weight operands and bias.  A layer with a
// block of 16 runs on 16-deep instructions only (see mfma16).
template <int PLANES, int TILES, int NK32, bool HAS16, bool LAST_HIDDEN, class Load>
__device__ __forceinline__ void fp8_hidden_layer(Load&& load, uint4 const (&B32)[NK32][4], uint2 const (&B16)[4], uint32_t (&H)[4][4][2])
{
    v4f const zero = { 0.f, 0.f, 0.f, 0.f };
    // The operands of output tile t + 1 are loaded before the work on tile t (two sets of registers, alternating);
    // a scheduling barrier that only LDS reads may not cross keeps the compiler from moving those loads back down
    // to their uses.
    // (Not with three planes - a layer with a weight of 32 or more: that form's registers would set the kernel's
    // budget, and the kernel would spill in its prologue what every workgroup, also one that only passes over
    // sets, has to write out.)
    constexpr bool AHEAD = PLANES < 3;
    TileOperands<NK32, HAS16> ops[2];
    if (AHEAD) load(0, ops[0]);
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        if (!AHEAD) load(t, ops[t & 1]);
        if (AHEAD && t + 1 < TILES) {
            load(t + 1, ops[(t + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0x67f);           // everything but LDS instructions may cross
        }
        TileOperands<NK32, HAS16> const& o = ops[t & 1];
        __builtin_amdgcn_s_setprio(kPrioMatrix);
        v4f acc[3][4];
#pragma unroll
        for (int p = 0; p < 3; ++p) {
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[p][b] = zero;
            if (p >= PLANES) continue;
#pragma unroll
            for (int kb = 0; kb < NK32; ++kb) {
                if (HAS16) mfma32_as_two_16(o.a32[p][kb], B32[kb], acc[p]);
                else       mfma32(o.a32[p][kb], B32[kb], acc[p]);
            }
            if (HAS16) mfma16(o.a16[p], B16, acc[p]);
        }
        __builtin_amdgcn_s_setprio(kPrioEpilogue);
#pragma unroll
        for (int b = 0; b < 4; ++b) fp8_epilogue<LAST_HIDDEN, PLANES>(acc[2][b], acc[1][b], acc[0][b], o.bias, H[b][t]);
    }
}

template <class V, int PLANES>
__device__ __forceinline__ void fp8_layer0(Fp8Lds<V> const& lds, int lane, uint4 const (&X32)[4], uint2 const (&X16)[4], uint32_t (&H)[4][4][2])
{
    int const g = lane >> 4;
    uint4 B32[1][4];
#pragma unroll
    for (int b = 0; b < 4; ++b) B32[0][b] = X32[b];
    fp8_hidden_layer<PLANES, V::T0, 1, true, false>([&](int t, TileOperands<1, true>& o) {
#pragma unroll
        for (int p = 0; p < PLANES; ++p) {
            o.a32[p][0] = lds.w0[p][t][lane];
            o.a16[p] = reinterpret_cast<uint2 const*>(&lds.w0[p][t][64])[lane];
        }
        o.bias = *reinterpret_cast<v4f const*>(&lds.bias[t][g][0]);
    }, B32, X16, H);
}

template <class V, int PLANES>
__device__ __forceinline__ void fp8_layer1(Fp8Lds<V> const& lds, int lane, uint32_t const (&Hin)[4][4][2], uint32_t (&H)[4][4][2])
{
    int const g = lane >> 4;
    uint4 B32[2][4];
    uint2 B16[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        B32[0][b] = make_uint4(Hin[b][0][0], Hin[b][0][1], Hin[b][1][0], Hin[b][1][1]);
        B32[1][b] = make_uint4(Hin[b][2][0], Hin[b][2][1], Hin[b][3][0], Hin[b][3][1]);
        B16[b] = make_uint2(0u, 0u);
    }
    fp8_hidden_layer<PLANES, V::T1, 2, false, false>([&](int t, TileOperands<2, false>& o) {
#pragma unroll
        for (int p = 0; p < PLANES; ++p) {
            o.a32[p][0] = lds.w1[p][t][lane];
            o.a32[p][1] = lds.w1[p][t][64 + lane];
        }
        o.bias = *reinterpret_cast<v4f const*>(&lds.bias[V::T0 + t][g][0]);
    }, B32, B16, H);
}

// layer 2: its activations are quantised to the int8 inputs of the output layer
template <class V, int PLANES>
__device__ __forceinline__ void fp8_layer2(Fp8Lds<V> const& lds, int lane, uint32_t const (&Hin)[4][4][2], uint32_t (&H)[4][4][2])
{
    int const g = lane >> 4;
    uint4 B32[1][4];
    uint2 B16[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        B32[0][b] = make_uint4(Hin[b][0][0], Hin[b][0][1], Hin[b][1][0], Hin[b][1][1]);
        B16[b] = make_uint2(Hin[b][2][0], Hin[b][2][1]);
    }
    fp8_hidden_layer<PLANES, V::T2, 1, true, true>([&](int t, TileOperands<1, true>& o) {
#pragma unroll
        for (int p = 0; p < PLANES; ++p) {
            o.a32[p][0] = lds.w2[p][t][lane];
            o.a16[p] = reinterpret_cast<uint2 const*>(&lds.w2[p][t][64])[lane];
        }
        o.bias = *reinterpret_cast<v4f const*>(&lds.bias[V::T0 + V::T1 + t][g][0]);
    }, B32, B16, H);
}

// The FP8 network for the 64 texels of one wave.  `in` is the lane's own texel; `modes` (uniform) holds the hidden
// layers' modes as stage_fp8_weights returns them.  On return D[b] holds, for lane (j, g), the int32 accumulators of
// output channels 4g..4g+3 of texel 16b + j, and S their scales.
template <class V>
__device__ __forceinline__ void mlp_forward_fp8(Fp8Lds<V>& lds, int wave, int lane, int modes, uint32_t const (&in)[24], v4i (&D)[4], v4f& S)
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

    uint32_t Ha[4][4][2], Hb[4][4][2];                       // [texel block][tile of 16 channels][2 dwords = 4 halves]
    if constexpr (V::ONE) {
        fp8_layer0<V, 1>(lds, lane, X32, X16, Ha);                                                                 // 48 -> 64
        fp8_layer1<V, 1>(lds, lane, Ha, Hb);                                                                       // 64 -> 48
        fp8_layer2<V, 1>(lds, lane, Hb, Ha);                                                                       // 48 -> 32
    } else {
        int const one = modes >> kOnePlaneShift;
        if (one & 1)        fp8_layer0<V, 1>(lds, lane, X32, X16, Ha);
        else if (modes & 1) fp8_layer0<V, 3>(lds, lane, X32, X16, Ha);
        else                fp8_layer0<V, 2>(lds, lane, X32, X16, Ha);
        if (one & 2)        fp8_layer1<V, 1>(lds, lane, Ha, Hb);
        else if (modes & 2) fp8_layer1<V, 3>(lds, lane, Ha, Hb);
        else                fp8_layer1<V, 2>(lds, lane, Ha, Hb);
        if (one & 4)        fp8_layer2<V, 1>(lds, lane, Hb, Ha);
        else if (modes & 4) fp8_layer2<V, 3>(lds, lane, Hb, Ha);
        else                fp8_layer2<V, 2>(lds, lane, Hb, Ha);
    }
    // output layer: 32 -> 16, exact: |sum W q| <= 32 * 127 * 128 < 2^24
    {
        v4f const zero = { 0.f, 0.f, 0.f, 0.f };
        v4f acc[4] = { zero, zero, zero, zero };
        uint4 x[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) x[b] = make_uint4(Ha[b][0][0], Ha[b][0][1], Ha[b][1][0], Ha[b][1][1]);
        __builtin_amdgcn_s_setprio(kPrioMatrix);
        mfma32(lds.w3[lane], x, acc);
        __builtin_amdgcn_s_setprio(kPrioOther);
        v4i const bias = *reinterpret_cast<v4i const*>(&lds.outBias[g][0]);
        S = *reinterpret_cast<v4f const*>(&lds.outScale[g][0]);
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r) D[b][r] = int(uint32_t(int(acc[b][r])) + uint32_t(bias[r]));      // wraps like int32
    }
}

// 135 KB of LDS - three planes of every hidden layer's weights, shared by the twelve waves of the one workgroup
// a CU holds, and a transposition buffer per wave: three waves per SIMD, 168 registers per lane; the one-plane
// instantiation: one plane, sixteen waves, four per SIMD, 128 registers.  Each of the two decodes the segments
// whose set is its own (all hidden layers on one plane, or not) and passes over the others.
//
// A workgroup owns a contiguous share of the tile list.  It walks that share in segments of tiles that use the
// same weight blob (one segment, unless sets of a batch meet inside the share), and inside a segment each of its
// GROUP wave quartets walks a contiguous part, so that a quartet's consecutive tiles are neighbours in the image
// and find the cache lines they share with the previous tile still in place.  (Quartets taking every third tile
// of a common sequence drift apart in time, and the latent reads from memory doubled.)
template <class V>
__global__ void __launch_bounds__(V::THREADS, 1)
decode_fp8_kernel(DevMip const* __restrict__ mips, int numMips, int totalTiles, Fp8Handoff handoff)
{
    if (!V::ONE && *handoff.word != handoff.serial) return;  // the one-plane launch before this one met only its own sets
    __shared__ Fp8Lds<V> lds;
    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const member = wave >> 2;                            // which quartet of the workgroup
    int const j = lane & 15, g = lane >> 4;

    int const per = (totalTiles + gridDim.x - 1) / gridDim.x;
    int const tileBegin = blockIdx.x * per;
    int const tileEnd = min(totalTiles, tileBegin + per);
    if (tileBegin >= tileEnd) return;                        // uniform across the workgroup

    build_fp8_posenc_table(lds);
    build_fp8_feature_lut(lds);

    int modes = 7;                                           // uniform: the hidden layers' modes (stage_fp8_weights)

    // One wave tile: the 32 x 2 texels of this wave in tile (tileX, tileY) of mip m; block b of 16 texels begins at
    // (x0 + 16 * (b & 1), y0 + (b >> 1)), so that a wave's stores fill whole 128-byte lines of a row (store_tile).
    auto decode_wave_tile = [&](RunMip const& m, int tileX, int tileY) __attribute__((always_inline)) {
        int const x0 = tileX * 64 + (wave & 1) * 32, y0 = tileY * 4 + ((wave >> 1) & 1) * 2;
        if (x0 >= m.width || y0 >= m.height) return;         // whole wave tile outside the image
        uint32_t in[24];
        {
            int const x = min(x0 + j + 16 * (g & 1), m.width - 1), y = min(y0 + (g >> 1), m.height - 1);
            if (m.fast) {
                Fp8Fetch<V> fetch;
                fetch_latents_fast<V>(m.full, x, y, fetch);
                finish_inputs_fast<V>(m.full, lds, x, y, fetch, in);
            } else {
                prepare_inputs_fp8<V>(m.full, x, y, in);
            }
        }
        v4i D[4];
        v4f S;
        mlp_forward_fp8<V>(lds, wave, lane, modes, in, D, S);
        // a wave tile inside the image, channels in whole groups of four (pixel formats: vector stores possible), takes
        // the stores without tests; the one-plane instantiation also without the fp16-overflow check where no output
        // can come near it (the general instantiation keeps to the checked conversion)
        bool const inside = x0 + 32 <= m.width && y0 + 2 <= m.height && (m.numChannels & 3) == 0
                         && (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS || m.vectorStores);
        if (!inside) {
            store_tile_general(&m.full, D[0], D[1], D[2], D[3], S, x0 + j, y0, 4 * g);
        } else if (V::ONE && (modes & kFp8OutputsBounded)) {
            if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS)  store_tile_inside<NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS, false>(m, D, S, x0, y0, j, g);
            else if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PIXELS)   store_tile_inside<NTC_HIP_DEV_OUT_FP16_PIXELS, false>(m, D, S, x0, y0, j, g);
            else                                                   store_tile_inside<NTC_HIP_DEV_OUT_UNORM8_PIXELS, false>(m, D, S, x0, y0, j, g);
        } else {
            if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS)  store_tile_inside<NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS, true>(m, D, S, x0, y0, j, g);
            else if (m.outFormat == NTC_HIP_DEV_OUT_FP16_PIXELS)   store_tile_inside<NTC_HIP_DEV_OUT_FP16_PIXELS, true>(m, D, S, x0, y0, j, g);
            else                                                   store_tile_inside<NTC_HIP_DEV_OUT_UNORM8_PIXELS, true>(m, D, S, x0, y0, j, g);
        }
    };

    int entry = 0;
    for (int segBegin = tileBegin; segBegin < tileEnd; ) {   // uniform across the workgroup
        entry = table_entry_of(mips, numMips, entry, segBegin);
        uint8_t const* const blob = mips[entry].weights;
        int const segEnd = segment_end(mips, numMips, entry, tileEnd, blob);
        modes = classify_fp8_weights<V>(lds, blob);
        if (((modes & kAllOnePlane) == kAllOnePlane) != V::ONE) { // the other instantiation's segment
            if (V::ONE && threadIdx.x == 0) *handoff.word = handoff.serial;
            segBegin = segEnd;
            continue;
        }
        __syncthreads();                                     // every wave has left the previous segment's weights
        stage_fp8_weights<V>(lds, blob, modes);
        __syncthreads();                                     // also publishes the tables built above

        int const part = (segEnd - segBegin + V::GROUP - 1) / V::GROUP;
        int const myBegin = segBegin + member * part, myEnd = min(segEnd, myBegin + part);
        // The quartet steps through its tiles mip by mip, keeping the tile's place in the mip in registers: no
        // look-up in the table (a vector load and a wait for every outstanding store, per tile) and no division.
        int mine = entry;
        for (int tile = myBegin; tile < myEnd; ) {           // one run of tiles per mip
            while (mine + 1 < numMips && mips[mine + 1].tileStart <= tile) ++mine;
            RunMip const m(mips[mine]);
            int const runEnd = min(myEnd, mine + 1 < numMips ? mips[mine + 1].tileStart : 0x7fffffff);
            int const tilesX = m.full.tilesX, local = tile - m.full.tileStart;
            int tileY = local / tilesX, tileX = local - tileY * tilesX;
            for (; tile < runEnd; ++tile) {
                decode_wave_tile(m, tileX, tileY);
                if (++tileX == tilesX) { tileX = 0; ++tileY; }
            }
        }
        segBegin = segEnd;
    }
}

// Random-access decode with the FP8 network (NtcSampleTextureSet_CoopVec_FP8, InferenceCoopVec.hlsli:400-440,
// for a list of sample points): query_kernel of ntc_decode_kernel.hip with this file's input stage and network.  Lane = query in the input stage (each lane with its own mip, kept in LDS); one set, hence one
// weight blob, per launch.  A query whose mip is out of range writes zeros.
template <class V>
__global__ void __launch_bounds__(V::THREADS, 1)
query_fp8_kernel(DevMip const* __restrict__ mips, int numMips, DevQuery const* __restrict__ queries, uint64_t numQueries,
                 uint16_t* __restrict__ out, Fp8Handoff handoff)
{
    if (!V::ONE && *handoff.word != handoff.serial) return;  // the set went to the one-plane launch before this one
    __shared__ Fp8Lds<V> lds;
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

    int const modes = classify_fp8_weights<V>(lds, mips[0].weights);
    if (((modes & kAllOnePlane) == kAllOnePlane) != V::ONE) {            // the other instantiation's set (uniform over the grid)
        if (V::ONE && threadIdx.x == 0) *handoff.word = handoff.serial;
        return;
    }
    build_fp8_posenc_table(lds);
    build_fp8_feature_lut(lds);
    stage_fp8_weights<V>(lds, mips[0].weights, modes);
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
        uint32_t in[24];
        if (__all(m.fast != 0)) {                                // every lane's mip is power-of-two sized
            Fp8Fetch<V> fetch;
            if (bricked) fetch_latents_bricked<V>(m, x, y, fetch);
            else         fetch_latents_fast<V>(m, x, y, fetch);
            finish_inputs_fast<V>(m, lds, x, y, fetch, in);
        } else {
            prepare_inputs_fp8<V>(mips[validMip ? query.mip : 0], x, y, in);
        }
        v4i D[4];
        v4f S;
        mlp_forward_fp8<V>(lds, wave, lane, modes, in, D, S);

        // lane (j, g) holds channels 4g..4g+3 of query q0 + 16b + j; validity travels by shuffle
        auto store_outputs = [&](auto checked) __attribute__((always_inline)) {
            constexpr bool CHECKED = decltype(checked)::value;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                uint64_t const q = q0 + uint64_t(16 * b + j);
                int const ok = __shfl(validMip ? 1 : 0, 16 * b + j, 64);
                if (q >= numQueries) continue;
                uint32_t h01 = to_half2_bits<CHECKED>(float(D[b][0]) * S[0], float(D[b][1]) * S[1]);
                uint32_t h23 = to_half2_bits<CHECKED>(float(D[b][2]) * S[2], float(D[b][3]) * S[3]);
                if (!ok) { h01 = 0; h23 = 0; }
                *reinterpret_cast<u32x2*>(out + q * 16 + 4 * g) = u32x2{ h01, h23 };
            }
        };
        if (V::ONE && (modes & kFp8OutputsBounded)) store_outputs(std::false_type{});      // see decode_fp8_kernel
        else                                        store_outputs(std::true_type{});
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

// Both instantiations, the one-plane one first; a set is decoded by the one it belongs to (decided on the device
// from its weights).  A workgroup of the first launch that meets a set of the other kind writes the launch pair's
// serial number into the caller's hand-off word; the workgroups of the second launch leave at once unless they
// find that number there (nothing ever clears the word: a stale match only costs the second launch its look at
// the weights, after which it passes over the sets that are not its own as before).
template <int FEATURES>
static hipError_t launch_fp8_variant(DevMip const* mips, int numMips, int totalTiles, int gridSize, Fp8Handoff handoff, hipStream_t stream)
{
    using One = Fp8Variant<FEATURES, true>;
    using Any = Fp8Variant<FEATURES, false>;
    hipLaunchKernelGGL(decode_fp8_kernel<One>, dim3(gridSize), dim3(One::THREADS), 0, stream, mips, numMips, totalTiles, handoff);
    hipError_t const e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(decode_fp8_kernel<Any>, dim3(gridSize), dim3(Any::THREADS), 0, stream, mips, numMips, totalTiles, handoff);
    return hipGetLastError();
}

hipError_t launch_decode_fp8(int variant, DevMip const* mips, int numMips, int totalTiles, int gridSize, Fp8Handoff handoff, hipStream_t stream)
{
    switch (variant) {
    case NTC_HIP_VARIANT_REF16_FP8: return launch_fp8_variant<16>(mips, numMips, totalTiles, gridSize, handoff, stream);
    case NTC_HIP_VARIANT_REF12_FP8: return launch_fp8_variant<12>(mips, numMips, totalTiles, gridSize, handoff, stream);
    case NTC_HIP_VARIANT_REF8_FP8:  return launch_fp8_variant<8>(mips, numMips, totalTiles, gridSize, handoff, stream);
    case NTC_HIP_VARIANT_REF4_FP8:  return launch_fp8_variant<4>(mips, numMips, totalTiles, gridSize, handoff, stream);
    default: return hipErrorInvalidValue;
    }
}

template <int FEATURES>
static hipError_t launch_fp8_query_variant(DevMip const* mips, int numMips, DevQuery const* queries, uint64_t numQueries, uint16_t* out, int gridSize, Fp8Handoff handoff, hipStream_t stream)
{
    using One = Fp8Variant<FEATURES, true>;
    using Any = Fp8Variant<FEATURES, false>;
    hipLaunchKernelGGL(query_fp8_kernel<One>, dim3(gridSize), dim3(One::THREADS), 0, stream, mips, numMips, queries, numQueries, out, handoff);
    hipError_t const e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(query_fp8_kernel<Any>, dim3(gridSize), dim3(Any::THREADS), 0, stream, mips, numMips, queries, numQueries, out, handoff);
    return hipGetLastError();
}

hipError_t launch_queries_fp8(int variant, DevMip const* mips, int numMips, DevQuery const* queries, uint64_t numQueries,
                              uint16_t* out, int gridSize, Fp8Handoff handoff, hipStream_t stream)
{
    switch (variant) {
    case NTC_HIP_VARIANT_REF16_FP8: return launch_fp8_query_variant<16>(mips, numMips, queries, numQueries, out, gridSize, handoff, stream);
    case NTC_HIP_VARIANT_REF12_FP8: return launch_fp8_query_variant<12>(mips, numMips, queries, numQueries, out, gridSize, handoff, stream);
    case NTC_HIP_VARIANT_REF8_FP8:  return launch_fp8_query_variant<8>(mips, numMips, queries, numQueries, out, gridSize, handoff, stream);
    case NTC_HIP_VARIANT_REF4_FP8:  return launch_fp8_query_variant<4>(mips, numMips, queries, numQueries, out, gridSize, handoff, stream);
    default: return hipErrorInvalidValue;
    }
}

int fp8_threads_per_workgroup() { return VFp8_16::THREADS; }

int resident_fp8_workgroups_per_cu()
{
    int blocks = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, decode_fp8_kernel<VFp8_16>, VFp8_16::THREADS, 0) != hipSuccess || blocks < 1) blocks = 1;
    return blocks;
}

int fp8_tiles_per_round() { return VFp8_16::GROUP; }

hipError_t launch_selftest_fp8_activation(uint16_t const* in, uint16_t* out, int n, hipStream_t stream)
{
    hipLaunchKernelGGL(selftest_fp8_activation_kernel, dim3(unsigned((n + 255) / 256)), dim3(256), 0, stream, in, out, n);
    return hipGetLastError();
}

} // namespace ntc_hip_dev
