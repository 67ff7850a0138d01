// probe_issue_rates.hip - how fast one SIMD of a gfx950 compute unit issues the instructions the decode kernels
// are made of.  Not part of the library: a measurement behind the issue-rate figures quoted for the kernels.
//
// Every kernel runs one workgroup per compute unit with 1, 2 or 4 waves per SIMD; each wave executes a loop of
// independent (or, where said, dependent) instructions and times it with the constant 100 MHz counter
// (s_memrealtime).  Reported: nanoseconds per wave instruction per SIMD = loop time / (instructions * waves per SIMD).
// Findings on MI355X: plain fp32 add / mul / fma and 32-bit integer add / logic issue about 1.6 times faster than
// conversions, packed 16-bit, 24-bit multiplies, v_perm and other three-operand integer instructions; the fp16 ->
// fp8 conversion is twice as slow again; and the plain fp32 instructions do not overlap with matrix instructions
// in flight on the same SIMD (the loop time of "4 matrix + 32 v_mul" is the sum of the two), the slower ones partly.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <vector>

typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
constexpr int kIterations = 2048;

// Loop skeleton: r[8], q[8] are per-lane registers; `body` runs once per iteration.
#define PROBE(name, body) __global__ void __launch_bounds__(1024) name(uint32_t* out, long long* ticks, uint32_t seed) { \
    uint32_t r[8], q[8]; for (int i = 0; i < 8; ++i) { r[i] = seed * (i + 1) + threadIdx.x; q[i] = (seed * (i + 3)) ^ threadIdx.x; } \
    float const s = __builtin_bit_cast(float, 0x3f800100u + seed); \
    v4f acc[4]; for (int i = 0; i < 4; ++i) acc[i] = v4f{ s, s, s, s }; \
    v4i iacc[4]; for (int i = 0; i < 4; ++i) iacc[i] = v4i{ 1, 2, 3, 4 }; \
    v8h A, B; for (int i = 0; i < 8; ++i) { A[i] = _Float16(1.f + (threadIdx.x & 7)); B[i] = _Float16(2.f + (threadIdx.x & 3)); } \
    v4h const A4 = { A[0], A[1], A[2], A[3] }, B4 = { B[0], B[1], B[2], B[3] }; \
    v4i const Ai = { int(threadIdx.x), 2, 3, 4 }, Bi = { 5, int(threadIdx.x), 7, 8 }; \
    (void)A4; (void)B4; (void)Ai; (void)Bi; \
    __syncthreads(); long long const t0 = wall_clock64(); \
    for (int it = 0; it < kIterations; ++it) { body } \
    long long const t1 = wall_clock64(); \
    uint32_t x = 0; for (int i = 0; i < 8; ++i) x ^= r[i]; for (int i = 0; i < 4; ++i) x ^= uint32_t(acc[i][0] + acc[i][3]) ^ uint32_t(iacc[i][1]); \
    out[blockIdx.x * blockDim.x + threadIdx.x] = x; \
    if ((threadIdx.x & 63) == 0) ticks[blockIdx.x * 16 + threadIdx.x / 64] = t1 - t0; }
#define EACH8(text) _Pragma("unroll") for (int i = 0; i < 8; ++i) asm volatile(text : "+v"(r[i]) : "v"(q[i]));
#define MFMA4_F16K32 _Pragma("unroll") for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, acc[i], 0, 0, 0);

PROBE(p_mul_f32, EACH8("v_mul_f32 %0, %0, %1"))
PROBE(p_add_f32, EACH8("v_add_f32 %0, %0, %1"))
PROBE(p_fma_f32, EACH8("v_fma_f32 %0, %0, %1, %1"))
PROBE(p_fma_clamp, EACH8("v_fma_f32 %0, %0, %1, 0.5 clamp"))
PROBE(p_min_f32, EACH8("v_min_f32 %0, %0, %1"))
PROBE(p_add_u32, EACH8("v_add_u32 %0, %0, %1"))
PROBE(p_and_b32, EACH8("v_and_b32 %0, %0, %1"))
PROBE(p_lshrrev, EACH8("v_lshrrev_b32 %0, 4, %0"))
PROBE(p_lshlrev, EACH8("v_lshlrev_b32 %0, 1, %0"))
PROBE(p_mad_u24, EACH8("v_mad_u32_u24 %0, %0, %1, %1"))
PROBE(p_perm, EACH8("v_perm_b32 %0, %0, %1, %1"))
PROBE(p_and_or, EACH8("v_and_or_b32 %0, %0, %1, %1"))
PROBE(p_lshl_add, EACH8("v_lshl_add_u32 %0, %0, 1, %1"))
PROBE(p_cvt_f32_i32, EACH8("v_cvt_f32_i32 %0, %0"))
PROBE(p_cvt_pk_f16, EACH8("v_cvt_pk_f16_f32 %0, %0, %1"))
PROBE(p_cvt_pk_u8, EACH8("v_cvt_pk_u8_f32 %0, %0, 1, %1"))
PROBE(p_pk_min_i16, EACH8("v_pk_min_i16 %0, %0, %1"))
PROBE(p_pk_fma_f16, EACH8("v_pk_fma_f16 %0, %0, %1, %1"))
PROBE(p_pk_mul_f16, EACH8("v_pk_mul_f16 %0, %0, %1"))
PROBE(p_cvt_fp8_f16, EACH8("v_cvt_scalef32_pk_fp8_f16 %0, %1, 1.0"))
PROBE(p_cvt_f16_fp8, EACH8("v_cvt_scalef32_pk_f16_fp8 %0, %1, 1.0"))
PROBE(p_sdwa, EACH8("v_lshlrev_b32_sdwa %0, %1, %0 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1"))
PROBE(p_chain, _Pragma("unroll") for (int i = 0; i < 8; ++i) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(r[0]) : "v"(q[0]));)
// the requantiser of layers 1-2 of the int8 network for 8 activations: 4 dependent fp32 operations each, then
// a packed conversion and a packed minimum per pair (40 instructions); and layer 0's, with its conversion (48)
#define REQUANT(first) { float v[8]; _Pragma("unroll") for (int i = 0; i < 8; ++i) { float c = __builtin_bit_cast(float, r[i]), x, t, y; first \
        asm volatile("v_mul_f32 %0, %1, %2" : "=v"(x) : "v"(c), "v"(s)); asm volatile("v_fma_f32 %0, %1, %2, 0.5 clamp" : "=v"(t) : "v"(x), "v"(s)); \
        asm volatile("v_mul_f32 %0, %1, %2" : "=v"(y) : "v"(x), "v"(t)); asm volatile("v_mul_f32 %0, 0x36a00000, %1" : "=v"(v[i]) : "v"(y)); } \
    _Pragma("unroll") for (int i = 0; i < 8; i += 2) { uint32_t h; asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(h) : "v"(v[i]), "v"(v[i + 1])); \
        asm volatile("v_pk_min_i16 %0, %1, %2" : "=v"(r[i]) : "v"(h), "v"(q[i])); } }
PROBE(p_requant, REQUANT(;))
PROBE(p_requant_cvt, REQUANT(asm volatile("v_cvt_f32_i32 %0, %0" : "+v"(c));))
PROBE(p_mfma_f16_k32, MFMA4_F16K32)
PROBE(p_mfma_f16_k16, _Pragma("unroll") for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x16f16(A4, B4, acc[i], 0, 0, 0);)
PROBE(p_mfma_i8_k64, _Pragma("unroll") for (int i = 0; i < 4; ++i) iacc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Ai, Bi, iacc[i], 0, 0, 0);)
PROBE(p_mul32, EACH8("v_mul_f32 %0, %0, %1") EACH8("v_mul_f32 %0, %0, %1") EACH8("v_mul_f32 %0, %0, %1") EACH8("v_mul_f32 %0, %0, %1"))
PROBE(p_mfma_mul32, MFMA4_F16K32 EACH8("v_mul_f32 %0, %0, %1") EACH8("v_mul_f32 %0, %0, %1") EACH8("v_mul_f32 %0, %0, %1") EACH8("v_mul_f32 %0, %0, %1"))
PROBE(p_cvt32, EACH8("v_cvt_f32_i32 %0, %0") EACH8("v_cvt_f32_i32 %0, %0") EACH8("v_cvt_f32_i32 %0, %0") EACH8("v_cvt_f32_i32 %0, %0"))
PROBE(p_mfma_cvt32, MFMA4_F16K32 EACH8("v_cvt_f32_i32 %0, %0") EACH8("v_cvt_f32_i32 %0, %0") EACH8("v_cvt_f32_i32 %0, %0") EACH8("v_cvt_f32_i32 %0, %0"))

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("HIP error %s at line %d\n", hipGetErrorName(e_), __LINE__); return 1; } } while (0)

int main()
{
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    int const cus = prop.multiProcessorCount;
    uint32_t* out; long long* ticks;
    CHECK(hipMalloc(&out, size_t(cus) * 1024 * 4)); CHECK(hipMalloc(&ticks, size_t(cus) * 16 * 8));
    struct Probe { char const* what; void (*kernel)(uint32_t*, long long*, uint32_t); int instructions; };
    Probe const probes[] = {
        { "v_mul_f32", p_mul_f32, 8 }, { "v_add_f32", p_add_f32, 8 }, { "v_fma_f32", p_fma_f32, 8 }, { "v_fma_f32 clamp", p_fma_clamp, 8 }, { "v_min_f32", p_min_f32, 8 },
        { "v_add_u32", p_add_u32, 8 }, { "v_and_b32", p_and_b32, 8 }, { "v_lshrrev_b32", p_lshrrev, 8 }, { "v_lshlrev_b32", p_lshlrev, 8 },
        { "v_mad_u32_u24", p_mad_u24, 8 }, { "v_perm_b32", p_perm, 8 }, { "v_and_or_b32", p_and_or, 8 }, { "v_lshl_add_u32", p_lshl_add, 8 }, { "v_lshlrev_b32_sdwa", p_sdwa, 8 },
        { "v_cvt_f32_i32", p_cvt_f32_i32, 8 }, { "v_cvt_pk_f16_f32", p_cvt_pk_f16, 8 }, { "v_cvt_pk_u8_f32", p_cvt_pk_u8, 8 }, { "v_pk_min_i16", p_pk_min_i16, 8 },
        { "v_pk_fma_f16", p_pk_fma_f16, 8 }, { "v_pk_mul_f16", p_pk_mul_f16, 8 }, { "v_cvt_scalef32_pk_fp8_f16", p_cvt_fp8_f16, 8 }, { "v_cvt_scalef32_pk_f16_fp8", p_cvt_f16_fp8, 8 },
        { "v_mul_f32, one dependent chain", p_chain, 8 },
        { "requantiser of 8 activations (32 fp32 + 4 cvt_pk + 4 pk_min)", p_requant, 40 }, { "the same after v_cvt_f32_i32 (layer 0)", p_requant_cvt, 48 },
        { "v_mfma_f32_16x16x32_f16 x 4", p_mfma_f16_k32, 4 }, { "v_mfma_f32_16x16x16_f16 x 4 (same operands)", p_mfma_f16_k16, 4 }, { "v_mfma_i32_16x16x64_i8 x 4", p_mfma_i8_k64, 4 },
        { "32 v_mul_f32", p_mul32, 32 }, { "4 v_mfma_f32_16x16x32_f16 + 32 v_mul_f32", p_mfma_mul32, 36 },
        { "32 v_cvt_f32_i32", p_cvt32, 32 }, { "4 v_mfma_f32_16x16x32_f16 + 32 v_cvt_f32_i32", p_mfma_cvt32, 36 } };
    std::printf("%s, %d compute units; ns per wave instruction per SIMD (and per loop iteration) at 1 / 2 / 4 waves per SIMD\n", prop.name, cus);
    std::vector<long long> host(size_t(cus) * 16);
    for (Probe const& p : probes) {
        std::printf("%-62s", p.what);
        for (int wavesPerSimd : { 1, 2, 4 }) {
            int const waves = 4 * wavesPerSimd;
            for (int rep = 0; rep < 2; ++rep) { hipLaunchKernelGGL(p.kernel, dim3(cus), dim3(64 * waves), 0, 0, out, ticks, 7u); CHECK(hipDeviceSynchronize()); }
            CHECK(hipMemcpy(host.data(), ticks, host.size() * 8, hipMemcpyDeviceToHost));
            std::vector<double> t;
            for (int b = 0; b < cus; ++b) for (int w = 0; w < waves; ++w) t.push_back(double(host[size_t(b) * 16 + w]));
            std::sort(t.begin(), t.end());
            double const nsPerIteration = t[t.size() / 2] * 10.0 / (double(kIterations) * wavesPerSimd);     // 100 MHz counter
            std::printf("  %6.2f (%6.1f)", nsPerIteration / p.instructions, nsPerIteration);
        }
        std::printf("\n");
    }
    return 0;
}
