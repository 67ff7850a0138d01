// ntc_hip_api.cpp - the C ABI of include/ntc_hip.h: argument checks, the per-launch mip
// table, device memory and timing.  No CPU decode path exists here: without a HIP device
// every compute entry point fails with NTC_HIP_ERR_NO_DEVICE / NOT_INITIALIZED.
#include "../../include/ntc_hip.h"
#include "ntc_decode_kernel.h"

#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <algorithm>
#include <atomic>
#include <mutex>
#include <new>
#include <vector>

using namespace ntc_hip_dev;

namespace {

thread_local char t_error[1024] = "";

void set_error(char const* fmt, ...)
{
    va_list args;
    va_start(args, fmt);
    vsnprintf(t_error, sizeof(t_error), fmt, args);
    va_end(args);
}
void clear_error() { t_error[0] = 0; }

// Message shape of SetCudaErrorMessage (reference src/Errors.cpp:43-46).
int hip_fail(char const* call, hipError_t err)
{
    set_error("Call to %s failed, error code = %s.", call, hipGetErrorName(err));
    return int(err);
}
#define HIP_TRY(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) return hip_fail(#expr, e_); } while (0)

// Mip table of ntc_hip_decode_static: device memory that exists from the moment the library is loaded,
// so that entry point never allocates.  Each GPU holds its own copy of the array at its own address;
// on the host the array's NAME is only a stand-in for it, so every use below goes through the address
// hipGetSymbolAddress returned for the device (Library::staticTable), never through the name.
constexpr int kStaticTableEntries = NTC_HIP_STATIC_TABLE_MIPS;                      // 16 sets with a full mip chain each
constexpr int kTableChunkEntries = 16;                         // entries one table-writing launch carries
constexpr size_t kStaticTableBytes = (kStaticTableEntries * sizeof(DevMip) + 255) / 256 * 256;
static __device__ __align__(256) unsigned char scratch[kStaticTableBytes + 256];   // the table, then the FP8 hand-off word
constexpr int kMaxDevices = 64;
void* g_staticTable[kMaxDevices] = { nullptr };                // per device: address of `scratch` there

// Carries up to kTableChunkEntries table entries to the device as a kernel argument (no host-to-device
// copy, no staging memory) and stores them with ordinary vector stores.
struct TableChunk { DevMip entries[kTableChunkEntries]; };
static_assert(sizeof(TableChunk) <= 3072, "a table chunk must fit the kernel-argument segment");
static_assert(sizeof(DevMip) % 4 == 0, "table entries are copied as dwords");
__global__ void __launch_bounds__(256) write_table_kernel(uint32_t* dst, TableChunk chunk, int dwords)
{
    uint32_t const* src = reinterpret_cast<uint32_t const*>(&chunk);
    for (int i = threadIdx.x; i < dwords; i += blockDim.x) dst[i] = src[i];
}

} // namespace

// One device, one stream and the device-side working memory of the calls made through it: the mip table of
// the decode kernels with its pinned staging slots, the partial sums of the loss pass, two timing events.
// Contexts share nothing but the per-device table of ntc_hip_decode_static.
struct NtcHipContext {
    bool initialized = false;      // false again once destroyed
    int device = -1;
    int computeUnits = 0;
    int clockRateKHz = 0;
    char name[256] = "";
    hipStream_t stream = nullptr;
    hipEvent_t evStart = nullptr, evStop = nullptr;
    hipEvent_t evSpanStart = nullptr, evSpanStop = nullptr;    // ntc_hip_timer_begin / _end
    bool spanOpen = false;
    DevMip* tableDev = nullptr;        // device copy of the mip table
    DevMip* staticTable = nullptr;     // this device's `scratch` array (ntc_hip_decode_static)
    uint32_t* handoffDev = nullptr;    // the dword between the two launches of the FP8 network (launch_decode_fp8)
    uint32_t handoffSerial = 0;        // changes with every pair of such launches
    size_t tableCapacity = 0;          // entries
    std::vector<DevMip> lastTable;     // what tableDev currently holds (or will, in stream order)
    double* lossDev = nullptr;         // per-workgroup partial sums of the loss pass
    double* lossHost = nullptr;        // pinned copy of them
    size_t lossBytes = 0;
    static constexpr int kSlots = 4;
    struct Slot { DevMip* host = nullptr; size_t capacity = 0; hipEvent_t done = nullptr; bool inFlight = false; };
    Slot slots[kSlots];                // pinned staging for asynchronous table uploads
    int nextSlot = 0;
    DevMip staticBuild[NTC_HIP_STATIC_TABLE_MIPS];   // where ntc_hip_decode_static assembles its table (it allocates nothing)
};


namespace {
using Library = NtcHipContext;
Library* g_default = nullptr;          // the context behind the functions that take none (ntc_hip_init)

// Makes the context's device current for the duration of a call and restores the caller's afterwards, as the
// reference's CudaDeviceGuard does around every entry point (src/CudaDeviceGuard.cpp:21-62).
struct DeviceGuard {
    int previous = -1;
    bool changed = false;
    explicit DeviceGuard(int device)
    {
        if (hipGetDevice(&previous) == hipSuccess && previous != device) changed = hipSetDevice(device) == hipSuccess;
    }
    ~DeviceGuard() { if (changed) (void)hipSetDevice(previous); }
};

int not_initialized()
{
    set_error("ntc_hip_init has not been called (or found no HIP device), or the context is null or destroyed.");
    return NTC_HIP_ERR_NOT_INITIALIZED;
}
// The contexts that exist.  A handle is looked up here before it is dereferenced, so that a destroyed (freed) context
// is recognised by its address alone.
std::mutex g_liveMutex;
std::vector<NtcHipContext*> g_live;
bool is_live(NtcHipContext* ctx)
{
    if (!ctx) return false;
    std::lock_guard<std::mutex> lock(g_liveMutex);
    return std::find(g_live.begin(), g_live.end(), ctx) != g_live.end();
}
#define CTX_ENTER(ctx) if (!is_live(ctx)) return not_initialized(); Library& L = *(ctx); DeviceGuard deviceGuard_(L.device)

// Caller-given strides and offsets enter 64-bit size products: bounded so that none can wrap.
constexpr uint64_t kMaxRowPitch = uint64_t(1) << 40, kMaxPixelStride = uint64_t(1) << 20;
bool reaches_past(uint64_t offset, uint64_t bytes, uint64_t bufferBytes) { return bytes > bufferBytes || offset > bufferBytes - bytes; }

bool spec_equal(NtcHipDecoderSpec const& a, NtcHipDecoderSpec const& b) { return std::memcmp(&a, &b, sizeof(a)) == 0; }

int layer_in(NtcHipDecoderSpec const& s, int l) { return l == 0 ? s.inputChannels : s.hiddenChannels[l - 1]; }
int layer_out(NtcHipDecoderSpec const& s, int l) { return l == NTC_HIP_MLP_LAYERS - 1 ? s.outputChannels : s.hiddenChannels[l]; }

bool spec_sane(NtcHipDecoderSpec const& s)
{
    auto widthOk = [](int w) { return w >= 16 && w <= NTC_HIP_MAX_LAYER_WIDTH && (w % 16) == 0; };
    if (!widthOk(s.inputChannels) || s.outputChannels != 16) return false;
    for (int l = 0; l < NTC_HIP_MLP_LAYERS - 1; ++l) if (!widthOk(s.hiddenChannels[l])) return false;
    if ((s.hrBits != 2 && s.hrBits != 4) || (s.lrBits != 2 && s.lrBits != 4)) return false;
    if (s.hrFeatures < 1 || s.lrFeatures < 1 || s.hrFeatures > s.hrFeatureSlots || s.lrFeatures > s.lrFeatureSlots) return false;
    if (s.weightType < NTC_HIP_WEIGHTS_INT8 || s.weightType > NTC_HIP_WEIGHTS_FP8_SCALED) return false;
    return true;
}

// Which compiled kernel covers this spec.
int pick_variant(NtcHipDecoderSpec const& s)
{
    if (s.posEncWaves != 3 || s.outputChannels != 16) return NTC_HIP_VARIANT_NONE;
    if (s.lrMode != NTC_HIP_GRID_BILINEAR || s.lrBits != 4) return NTC_HIP_VARIANT_NONE;
    if (s.weightType == NTC_HIP_WEIGHTS_FP8_SCALED) {
        bool const wide = s.hrMode == NTC_HIP_GRID_BILINEAR && s.hrBits == 4 && s.hrFeatures == 16 && s.hrFeatureSlots == 16
            && s.lrFeatures == 16 && s.lrFeatureSlots == 16 && s.lodInputs == 2 && s.inputChannels == 48
            && s.hiddenChannels[0] == 64 && s.hiddenChannels[1] == 64 && s.hiddenChannels[2] == 64;
        return wide ? NTC_HIP_VARIANT_CFG3_FP8 : NTC_HIP_VARIANT_NONE;
    }
    if (s.weightType != NTC_HIP_WEIGHTS_INT8 && s.weightType != NTC_HIP_WEIGHTS_FP8) return NTC_HIP_VARIANT_NONE;
    bool const fp8 = s.weightType == NTC_HIP_WEIGHTS_FP8;    // the FP8 network exists for the LibNTC 0.9.2 geometry only
    bool const concat8x2 = s.hrMode == NTC_HIP_GRID_CONCAT2X2 && s.hrFeatures == 8 && s.hrBits == 2 && s.hrFeatureSlots == 8;
    if (!fp8 && concat8x2 && s.lodInputs == 0 && s.inputChannels == 64 && s.hiddenChannels[2] == 32) {
        if (s.lrFeatures == 16 && s.lrFeatureSlots == 16 && s.hiddenChannels[0] == 64 && s.hiddenChannels[1] == 48)
            return NTC_HIP_VARIANT_CFG01;
        if (s.lrFeatures == 12 && s.lrFeatureSlots == 12 && s.hiddenChannels[0] == 48 && s.hiddenChannels[1] == 48)
            return NTC_HIP_VARIANT_CFG2;
    }
    bool const ref = s.hrMode == NTC_HIP_GRID_BILINEAR && s.hrBits == 4 && s.hrFeatureSlots == 16 && s.lrFeatureSlots == 16
        && s.hrFeatures == s.lrFeatures && s.lodInputs == 2 && s.inputChannels == 48
        && s.hiddenChannels[0] == 64 && s.hiddenChannels[1] == 48 && s.hiddenChannels[2] == 32;
    if (ref) {
        switch (s.hrFeatures) {
        case 16: return fp8 ? NTC_HIP_VARIANT_REF16_FP8 : NTC_HIP_VARIANT_REF16;
        case 12: return fp8 ? NTC_HIP_VARIANT_REF12_FP8 : NTC_HIP_VARIANT_REF12;
        case 8:  return fp8 ? NTC_HIP_VARIANT_REF8_FP8 : NTC_HIP_VARIANT_REF8;
        case 4:  return fp8 ? NTC_HIP_VARIANT_REF4_FP8 : NTC_HIP_VARIANT_REF4;
        default: break;
        }
    }
    return NTC_HIP_VARIANT_NONE;
}

uint64_t grid_bytes(int32_t w, int32_t h, int32_t features, int32_t bits);

bool is_pow2(int32_t v) { return v > 0 && (v & (v - 1)) == 0; }
int log2i(int32_t v) { int l = 0; while ((1 << l) < v) ++l; return l; }

// Integer form of p = u*grid - 1/2 for power-of-two sizes: p = N / 2^n with
// N = ((2x+1) << shl) - (1 << sublog).  Returns false when the axis is not a power of two.
bool axis_params(int32_t size, int32_t grid, uint32_t& packed, int& n)
{
    if (!is_pow2(size) || !is_pow2(grid)) return false;
    int const e = log2i(grid) - log2i(size);
    int const shl = e > 0 ? e : 0, sublog = e < 0 ? -e : 0;
    n = 1 - e > 1 ? 1 - e : 1;
    if (shl > 12 || n > 16) return false;
    packed = uint32_t(shl) | (uint32_t(n) << 8) | (uint32_t(sublog) << 16) | (uint32_t(log2i(grid)) << 24);
    return true;
}

// Decides whether a mip may take the kernel's all-integer input stage and fills its parameters.
// Conditions: every size a power of two (then every float operation of the general stage is
// exact and the integer form gives the same bytes); bilinear weights of at most 8 fractional
// bits in total (16-bit lanes of the packed filter cannot overflow); positionScale a power of
// two, at least 2^-5 (the encoding has a period of at most 32 texels).
void fill_fast_path(NtcHipDecoderSpec const& spec, DevMip& e)
{
    e.fast = 0;
    int hx, hy, lx, ly;
    if (!axis_params(e.width, e.hrWidth, e.hrAxisX, hx) || !axis_params(e.height, e.hrHeight, e.hrAxisY, hy)) return;
    if (!axis_params(e.width, e.lrWidth, e.lrAxisX, lx) || !axis_params(e.height, e.lrHeight, e.lrAxisY, ly)) return;
    if (lx + ly > 8) return;
    if (spec.hrMode == NTC_HIP_GRID_BILINEAR && hx + hy > 8) return;
    if (grid_bytes(e.hrWidth, e.hrHeight, spec.hrFeatures, spec.hrBits) >= (1ull << 31)) return;
    if (grid_bytes(e.lrWidth, e.lrHeight, spec.lrFeatures, spec.lrBits) >= (1ull << 31)) return;
    int exp2 = 0;
    float const mant = std::frexp(e.positionScale, &exp2);      // scale = mant * 2^exp2, mant in [0.5, 1)
    if (!(mant == 0.5f) || exp2 - 1 < -5 || exp2 - 1 > 20) return;
    int const k = -(exp2 - 1);                                  // scale = 2^-k
    e.posMask = k > 0 ? (1u << k) - 1u : 0u;
    e.fast = 1;
}

uint64_t grid_bytes(int32_t w, int32_t h, int32_t features, int32_t bits)
{
    if (w <= 0 || h <= 0 || features <= 0 || (bits != 2 && bits != 4)) return 0;
    int const perWord = 16 / bits;
    return uint64_t(w) * uint64_t(h) * 2u * uint64_t((features + perWord - 1) / perWord);
}

// Where each grid of a set lives in the query-ordered copy (ntc_hip_build_query_latents).  Grids
// that several mips share (same offset and size in `latents`) are stored once; every grid starts
// on a 128-byte boundary.
struct BrickGrid { uint64_t srcOffset, dstOffset; int32_t width, height, layers; };
struct BrickPlan {
    std::vector<BrickGrid> grids;
    uint64_t hr[NTC_HIP_MAX_MIPS], lr[NTC_HIP_MAX_MIPS];
    uint64_t totalBytes = 0;
};

int grid_layers(int32_t features, int32_t bits) { return (features + 16 / bits - 1) / (16 / bits); }

uint64_t bricked_bytes(int32_t width, int32_t height, int layers)
{
    uint64_t const side = uint64_t(1) << brick_side_log2(layers);
    uint64_t const bytes = ((uint64_t(width) + side - 1) / side) * ((uint64_t(height) + side - 1) / side) * uint64_t(brick_bytes(layers));
    return (bytes + 127u) & ~uint64_t(127);
}

bool plan_bricks(NtcHipTextureSet const& set, BrickPlan& plan)
{
    if (!spec_sane(set.spec) || set.numMips < 1 || set.numMips > NTC_HIP_MAX_MIPS) return false;
    plan.grids.clear();
    plan.totalBytes = 0;
    auto place = [&](uint64_t srcOffset, int32_t w, int32_t h, int layers) -> uint64_t {
        for (BrickGrid const& g : plan.grids)
            if (g.srcOffset == srcOffset && g.width == w && g.height == h && g.layers == layers) return g.dstOffset;
        BrickGrid const g{ srcOffset, plan.totalBytes, w, h, layers };
        plan.grids.push_back(g);
        plan.totalBytes += bricked_bytes(w, h, layers);
        return g.dstOffset;
    };
    int const hrLayers = grid_layers(set.spec.hrFeatures, set.spec.hrBits), lrLayers = grid_layers(set.spec.lrFeatures, set.spec.lrBits);
    if (hrLayers < 1 || hrLayers > 4 || lrLayers < 1 || lrLayers > 4) return false;
    for (int m = 0; m < set.numMips; ++m) {
        NtcHipMipDesc const& d = set.mips[m];
        if (d.hrWidth < 1 || d.hrHeight < 1 || d.lrWidth < 1 || d.lrHeight < 1) return false;
        plan.hr[m] = place(d.hrOffset, d.hrWidth, d.hrHeight, hrLayers);
        plan.lr[m] = place(d.lrOffset, d.lrWidth, d.lrHeight, lrLayers);
    }
    return true;
}

// Validates the sets, builds the mip table (sorted by tileStart) and picks the kernel.
// Where build_table puts its entries: a vector, or (ntc_hip_decode_static, which may not allocate) a fixed array.
struct TableSink {
    std::vector<DevMip>* vector = nullptr;
    DevMip* fixed = nullptr;
    size_t capacity = 0, count = 0;
    void clear() { count = 0; if (vector) vector->clear(); }
    void push_back(DevMip const& e)
    {
        if (vector) vector->push_back(e);
        else if (count < capacity) fixed[count] = e;
        ++count;                                              // beyond the capacity entries are counted, not stored
    }
};

int build_table(NtcHipTextureSet const* sets, int32_t numSets, TableSink table, size_t& entries, int& variant, int& totalTiles,
                bool forQueries = false);
int build_table(NtcHipTextureSet const* sets, int32_t numSets, std::vector<DevMip>& table, int& variant, int& totalTiles,
                bool forQueries = false)
{
    TableSink sink;
    sink.vector = &table;
    size_t entries = 0;
    return build_table(sets, numSets, sink, entries, variant, totalTiles, forQueries);
}

int build_table(NtcHipTextureSet const* sets, int32_t numSets, TableSink table, size_t& entries, int& variant, int& totalTiles,
                bool forQueries)
{
    entries = 0;
    if (!sets || numSets < 1) { set_error("ntc_hip_decode: no texture sets given."); return NTC_HIP_ERR_INVALID_ARG; }
    table.clear();
    totalTiles = 0;
    for (int s = 0; s < numSets; ++s) {
        NtcHipTextureSet const& set = sets[s];
        if (!spec_sane(set.spec)) { set_error("ntc_hip_decode: set %d has a malformed decoder spec.", s); return NTC_HIP_ERR_INVALID_ARG; }
        if (!spec_equal(set.spec, sets[0].spec)) {
            set_error("ntc_hip_decode: all sets of one call must share one decoder spec (set %d differs).", s);
            return NTC_HIP_ERR_INVALID_ARG;
        }
        if (set.numMips < 1 || set.numMips > NTC_HIP_MAX_MIPS) { set_error("ntc_hip_decode: set %d: numMips %d out of range 1..%d.", s, set.numMips, NTC_HIP_MAX_MIPS); return NTC_HIP_ERR_INVALID_ARG; }
        if (set.numChannels < 1 || set.numChannels > NTC_HIP_MAX_CHANNELS) { set_error("ntc_hip_decode: set %d: numChannels %d out of range 1..%d.", s, set.numChannels, NTC_HIP_MAX_CHANNELS); return NTC_HIP_ERR_INVALID_ARG; }
        if (!set.latents || !set.weights || (!set.output && !forQueries)) { set_error("ntc_hip_decode: set %d: null latents / weights / output pointer.", s); return NTC_HIP_ERR_INVALID_ARG; }
        if (!forQueries && (set.outputFormat < NTC_HIP_OUT_FP16_PLANAR_PAIRS || set.outputFormat > NTC_HIP_OUT_UNORM8_PIXELS)) { set_error("ntc_hip_decode: set %d: unknown output format %d.", s, set.outputFormat); return NTC_HIP_ERR_INVALID_ARG; }
        if ((reinterpret_cast<uintptr_t>(set.weights) & 3u) || (reinterpret_cast<uintptr_t>(set.latents) & 1u)) { set_error("ntc_hip_decode: set %d: weights must be 4-byte and latents 2-byte aligned.", s); return NTC_HIP_ERR_INVALID_ARG; }
        BrickPlan bricks;
        bool const bricked = forQueries && set.queryLatents != nullptr;
        if (bricked) {
            if (!plan_bricks(set, bricks) || set.queryLatentsBytes < bricks.totalBytes || (reinterpret_cast<uintptr_t>(set.queryLatents) & 127u)) {
                set_error("ntc_hip_decode_queries: set %d: queryLatents must be 128-byte aligned and hold %llu bytes (ntc_hip_query_latents_bytes).",
                          s, (unsigned long long)bricks.totalBytes);
                return NTC_HIP_ERR_INVALID_ARG;
            }
        }
        NtcHipWeightLayout layout;
        if (ntc_hip_weight_layout(&set.spec, &layout) != 0) return NTC_HIP_ERR_INVALID_ARG;
        if (set.weightsBytes < layout.bufferSize) {
            set_error("ntc_hip_decode: set %d: weight blob holds %llu bytes, the spec needs %u.", s,
                      (unsigned long long)set.weightsBytes, layout.bufferSize);
            return NTC_HIP_ERR_INVALID_ARG;
        }
        int const bytesPerChannel = set.outputFormat == NTC_HIP_OUT_UNORM8_PIXELS ? 1 : 2;
        if (!forQueries && set.outputFormat != NTC_HIP_OUT_FP16_PLANAR_PAIRS
            && (set.outPixelStride < set.numChannels * bytesPerChannel || uint64_t(set.outPixelStride) > kMaxPixelStride)) {
            set_error("ntc_hip_decode: set %d: pixel stride %d is smaller than %d channels.", s, set.outPixelStride, set.numChannels);
            return NTC_HIP_ERR_INVALID_ARG;
        }
        // the kernel addresses a texel inside its row with 32 bits
        if (!forQueries && set.outputFormat != NTC_HIP_OUT_FP16_PLANAR_PAIRS)
            for (int m = 0; m < set.numMips; ++m)
                if (set.mips[m].width >= 1 && uint64_t(set.mips[m].width - 1) * uint64_t(set.outPixelStride) + uint64_t(set.numChannels * bytesPerChannel) >= (uint64_t(1) << 32)) {
                    set_error("ntc_hip_decode: set %d mip %d: a row of %d pixels with a stride of %d bytes reaches past 4 GiB.", s, m, set.mips[m].width, set.outPixelStride);
                    return NTC_HIP_ERR_INVALID_ARG;
                }
        for (int m = 0; m < set.numMips; ++m) {
            NtcHipMipDesc const& d = set.mips[m];
            if (d.width < 1 || d.height < 1 || d.hrWidth < 1 || d.hrHeight < 1 || d.lrWidth < 1 || d.lrHeight < 1
                || d.width > 65536 || d.height > 65536) {
                set_error("ntc_hip_decode: set %d mip %d: bad dimensions.", s, m);
                return NTC_HIP_ERR_INVALID_ARG;
            }
            if ((d.hrOffset & 1u) || (d.lrOffset & 1u)) { set_error("ntc_hip_decode: set %d mip %d: latent offsets must be even.", s, m); return NTC_HIP_ERR_INVALID_ARG; }
            // The FP8 network's exact sums are proven for inputs of at most 3 in magnitude; features and positional
            // encoding lie in [-1, 1], the level-of-detail input is the caller's (the reference's own: [-1, 1]).
            if (set.spec.weightType == NTC_HIP_WEIGHTS_FP8 && !(std::fabs(d.positionLod) <= 3.f)) {
                set_error("ntc_hip_decode: set %d mip %d: positionLod %g is outside [-3, 3] (FP8 network).", s, m, double(d.positionLod));
                return NTC_HIP_ERR_INVALID_ARG;
            }
            if (forQueries) {
                // no per-mip output
            } else if (set.outputFormat == NTC_HIP_OUT_FP16_PLANAR_PAIRS) {
                if (d.outOffset & 3u) { set_error("ntc_hip_decode: set %d mip %d: planar output offset must be 4-byte aligned.", s, m); return NTC_HIP_ERR_INVALID_ARG; }
            } else if (d.outRowPitch < uint64_t(d.width) * uint64_t(set.outPixelStride) || d.outRowPitch > kMaxRowPitch) {
                set_error("ntc_hip_decode: set %d mip %d: row pitch smaller than a row.", s, m);
                return NTC_HIP_ERR_INVALID_ARG;
            }
            uint64_t const hrBytes = grid_bytes(d.hrWidth, d.hrHeight, set.spec.hrFeatures, set.spec.hrBits);
            uint64_t const lrBytes = grid_bytes(d.lrWidth, d.lrHeight, set.spec.lrFeatures, set.spec.lrBits);
            if (reaches_past(d.hrOffset, hrBytes, set.latentsBytes) || reaches_past(d.lrOffset, lrBytes, set.latentsBytes)) {
                set_error("ntc_hip_decode: set %d mip %d: a latent grid reaches past the %llu-byte latent buffer.", s, m,
                          (unsigned long long)set.latentsBytes);
                return NTC_HIP_ERR_INVALID_ARG;
            }
            uint64_t outBytes;
            if (set.outputFormat == NTC_HIP_OUT_FP16_PLANAR_PAIRS)
                outBytes = uint64_t(d.width) * uint64_t(d.height) * uint64_t((set.numChannels + 1) & ~1) * 2u;
            else
                outBytes = uint64_t(d.height - 1) * d.outRowPitch + uint64_t(d.width - 1) * uint64_t(set.outPixelStride)
                         + uint64_t(set.numChannels * bytesPerChannel);
            if (!forQueries && reaches_past(d.outOffset, outBytes, set.outputBytes)) {
                set_error("ntc_hip_decode: set %d mip %d: output reaches past the %llu-byte output buffer.", s, m,
                          (unsigned long long)set.outputBytes);
                return NTC_HIP_ERR_INVALID_ARG;
            }
            DevMip e{};
            e.hr = reinterpret_cast<uint16_t const*>(static_cast<uint8_t const*>(set.latents) + d.hrOffset);
            e.lr = reinterpret_cast<uint16_t const*>(static_cast<uint8_t const*>(set.latents) + d.lrOffset);
            e.out = static_cast<uint8_t*>(set.output) + d.outOffset;
            e.weights = static_cast<uint8_t const*>(set.weights);
            e.outRowPitch = d.outRowPitch;
            e.width = d.width; e.height = d.height;
            e.hrWidth = d.hrWidth; e.hrHeight = d.hrHeight; e.lrWidth = d.lrWidth; e.lrHeight = d.lrHeight;
            e.positionScale = d.positionScale; e.positionLod = d.positionLod;
            e.outPixelStride = set.outPixelStride; e.numChannels = set.numChannels; e.outFormat = set.outputFormat;
            fill_fast_path(set.spec, e);
            if (bricked) {
                e.hrBricks = static_cast<uint8_t const*>(set.queryLatents) + bricks.hr[m];
                e.lrBricks = static_cast<uint8_t const*>(set.queryLatents) + bricks.lr[m];
            }
            e.tilesX = (d.width + kTileWidth - 1) / kTileWidth;
            e.tilesY = (d.height + kTileHeight - 1) / kTileHeight;
            e.tileStart = totalTiles;
            long long const next = (long long)totalTiles + (long long)e.tilesX * e.tilesY;
            if (next > 0x7fffffffLL) { set_error("ntc_hip_decode: too many tiles in one call."); return NTC_HIP_ERR_INVALID_ARG; }
            totalTiles = int(next);
            table.push_back(e);
        }
    }
    entries = table.count;
    variant = pick_variant(sets[0].spec);
    if (variant == NTC_HIP_VARIANT_NONE) {
        set_error("ntc_hip_decode: no compiled kernel covers this decoder spec "
                  "(weights %d, HR %dx%d-bit mode %d, LR %dx%d-bit mode %d, lod %d, MLP %d-%d-%d-%d-%d).",
                  sets[0].spec.weightType, sets[0].spec.hrFeatures, sets[0].spec.hrBits, sets[0].spec.hrMode,
                  sets[0].spec.lrFeatures, sets[0].spec.lrBits, sets[0].spec.lrMode, sets[0].spec.lodInputs,
                  sets[0].spec.inputChannels, sets[0].spec.hiddenChannels[0], sets[0].spec.hiddenChannels[1],
                  sets[0].spec.hiddenChannels[2], sets[0].spec.outputChannels);
        return NTC_HIP_ERR_UNSUPPORTED;
    }
    return 0;
}

// Makes the device table hold `table` (re-uploads only when it changed).  The copy is asynchronous
// from one of a few pinned staging slots; a slot is reused only after the copy that last read it
// has completed (its event), so back-to-back launches with different tables never wait on the GPU.
int upload_table(Library& L, std::vector<DevMip> const& table)
{
    bool const same = L.lastTable.size() == table.size()
        && std::memcmp(L.lastTable.data(), table.data(), table.size() * sizeof(DevMip)) == 0;
    if (same) return 0;
    if (table.size() > L.tableCapacity) {
        // The device table is read by kernels already queued on the stream: wait before replacing it.
        size_t const cap = table.size() * 2 + 16;
        HIP_TRY(hipStreamSynchronize(L.stream));
        if (L.tableDev) { HIP_TRY(hipFree(L.tableDev)); L.tableDev = nullptr; }
        L.tableCapacity = 0; L.lastTable.clear();
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&L.tableDev), cap * sizeof(DevMip)));
        L.tableCapacity = cap;
    }
    Library::Slot& slot = L.slots[L.nextSlot];
    L.nextSlot = (L.nextSlot + 1) % Library::kSlots;
    if (slot.inFlight) { HIP_TRY(hipEventSynchronize(slot.done)); slot.inFlight = false; }
    if (table.size() > slot.capacity) {
        if (slot.host) { HIP_TRY(hipHostFree(slot.host)); slot.host = nullptr; slot.capacity = 0; }
        HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&slot.host), L.tableCapacity * sizeof(DevMip), hipHostMallocDefault));
        slot.capacity = L.tableCapacity;
    }
    if (!slot.done) HIP_TRY(hipEventCreateWithFlags(&slot.done, hipEventDisableTiming));
    std::memcpy(slot.host, table.data(), table.size() * sizeof(DevMip));
    HIP_TRY(hipMemcpyAsync(L.tableDev, slot.host, table.size() * sizeof(DevMip), hipMemcpyHostToDevice, L.stream));
    HIP_TRY(hipEventRecord(slot.done, L.stream));
    slot.inFlight = true;
    L.lastTable = table;
    return 0;
}

int grid_size_for(Library const& L, int variant, int totalTiles)
{
    // Persistent workgroups: as many as stay resident at once, each walking a contiguous share of tiles.
    static std::atomic<int> perCu[NTC_HIP_VARIANT_COUNT];      // zero-initialised; every thread computes the same value
    int workgroups = perCu[variant].load(std::memory_order_relaxed);
    if (workgroups == 0) {
        workgroups = variant_is_fp8_network(variant) ? resident_fp8_workgroups_per_cu() : resident_workgroups_per_cu(variant);
        perCu[variant].store(workgroups, std::memory_order_relaxed);
    }
    int const resident = L.computeUnits * workgroups;
    // a workgroup takes tiles_per_round(variant) tiles at a time: fewer workgroups than that leaves waves idle
    int const group = variant_is_fp8_network(variant) ? fp8_tiles_per_round() : tiles_per_round(variant);
    int64_t const rounds = (int64_t(totalTiles) + group - 1) / group;
    return rounds < resident ? int(rounds) : resident;
}

// The hand-off word of a launch pair of the FP8 network over table `mips`: the context's own, or the one behind
// the per-device table when that is the table (then nothing of the context's device memory is used).
Fp8Handoff next_handoff(Library& L, DevMip const* mips)
{
    uint32_t* const word = mips == L.staticTable
        ? reinterpret_cast<uint32_t*>(reinterpret_cast<unsigned char*>(L.staticTable) + kStaticTableBytes) : L.handoffDev;
    return Fp8Handoff{ word, ++L.handoffSerial };
}

hipError_t launch_decode_any(Library& L, int variant, DevMip const* mips, int numMips, int totalTiles, int gridSize)
{
    return variant_is_fp8_network(variant) ? launch_decode_fp8(variant, mips, numMips, totalTiles, gridSize, next_handoff(L, mips), L.stream)
                                           : launch_decode(variant, mips, numMips, totalTiles, gridSize, L.stream);
}

} // namespace

extern "C" {

// Builds a context on `device`: cudaSetDevice + cudaInitDevice of CreateContext (src/PublicFunctions.cpp:84-112).
static int create_context(int device, NtcHipContext** outContext)
{
    clear_error();
    if (!outContext) { set_error("ntc_hip_create: null out-pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    *outContext = nullptr;
    int count = 0;
    hipError_t err = hipGetDeviceCount(&count);
    if (err != hipSuccess || count == 0) {
        set_error("No HIP device is available (hipGetDeviceCount: %s).", hipGetErrorName(err));
        return NTC_HIP_ERR_NO_DEVICE;
    }
    if (device < 0 || device >= count) { set_error("ntc_hip_init: device %d out of range 0..%d.", device, count - 1); return NTC_HIP_ERR_INVALID_ARG; }
    if (device >= kMaxDevices) { set_error("ntc_hip_init: device index %d is beyond the %d this library keeps state for.", device, kMaxDevices); return NTC_HIP_ERR_UNSUPPORTED; }
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("ntc_hip_init: device %d is %s; this library holds gfx950 code only.", device, prop.gcnArchName);
        return NTC_HIP_ERR_UNSUPPORTED;
    }
    DeviceGuard guard(device);
    {                                   // once per device, with that device current
        std::lock_guard<std::mutex> lock(g_liveMutex);
        if (!g_staticTable[device]) {
            void* address = nullptr;
            HIP_TRY(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
            g_staticTable[device] = address;
        }
    }
    NtcHipContext* L = new (std::nothrow) NtcHipContext();
    if (!L) { set_error("ntc_hip_create: out of host memory."); return NTC_HIP_ERR_INVALID_ARG; }
    L->device = device;
    L->computeUnits = prop.multiProcessorCount;
    L->clockRateKHz = prop.clockRate;
    // (some driver stacks report no marketing name)
    std::snprintf(L->name, sizeof(L->name), "%s (%s)", prop.name[0] ? prop.name : "AMD GPU", prop.gcnArchName);
    L->staticTable = static_cast<DevMip*>(g_staticTable[device]);
    hipError_t e = hipStreamCreate(&L->stream);
    if (e == hipSuccess) e = hipEventCreate(&L->evStart);
    if (e == hipSuccess) e = hipEventCreate(&L->evStop);
    if (e == hipSuccess) e = hipEventCreate(&L->evSpanStart);
    if (e == hipSuccess) e = hipEventCreate(&L->evSpanStop);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&L->handoffDev), 256);
    if (e != hipSuccess) {
        if (L->evSpanStop) (void)hipEventDestroy(L->evSpanStop);
        if (L->evSpanStart) (void)hipEventDestroy(L->evSpanStart);
        if (L->evStop) (void)hipEventDestroy(L->evStop);
        if (L->evStart) (void)hipEventDestroy(L->evStart);
        if (L->stream) (void)hipStreamDestroy(L->stream);
        delete L;
        return hip_fail("hipStreamCreate / hipEventCreate / hipMalloc", e);
    }
    L->initialized = true;
    {
        std::lock_guard<std::mutex> lock(g_liveMutex);
        g_live.push_back(L);
    }
    *outContext = L;
    return 0;
}

static void destroy_context(NtcHipContext* L)
{
    {                                   // a handle that is not (or no longer) a context's is ignored, never dereferenced
        std::lock_guard<std::mutex> lock(g_liveMutex);
        auto const at = std::find(g_live.begin(), g_live.end(), L);
        if (!L || at == g_live.end()) return;
        g_live.erase(at);
    }
    DeviceGuard guard(L->device);
    (void)hipStreamSynchronize(L->stream);
    if (L->tableDev) (void)hipFree(L->tableDev);
    if (L->handoffDev) (void)hipFree(L->handoffDev);
    if (L->lossDev) (void)hipFree(L->lossDev);
    if (L->lossHost) (void)hipHostFree(L->lossHost);
    for (Library::Slot& slot : L->slots) {
        if (slot.host) (void)hipHostFree(slot.host);
        if (slot.done) (void)hipEventDestroy(slot.done);
    }
    (void)hipEventDestroy(L->evStart);
    (void)hipEventDestroy(L->evStop);
    (void)hipEventDestroy(L->evSpanStart);
    (void)hipEventDestroy(L->evSpanStop);
    (void)hipStreamDestroy(L->stream);
    L->initialized = false;
    delete L;
}

int ntc_hip_create(int device, NtcHipContext** outContext) { return create_context(device, outContext); }
void ntc_hip_destroy(NtcHipContext* context) { if (context == g_default) g_default = nullptr; destroy_context(context); }

int ntc_hip_init(int device)
{
    if (is_live(g_default)) {
        if (g_default->device == device) { clear_error(); return 0; }
        ntc_hip_shutdown();
    }
    int const rc = create_context(device, &g_default);
    if (rc == 0) (void)hipSetDevice(device);      // callers of the context-free functions may use HIP themselves afterwards
    return rc;
}

void ntc_hip_shutdown(void)
{
    destroy_context(g_default);
    g_default = nullptr;
}

const char* ntc_hip_last_error(void) { return t_error; }

int ntc_hip_ctx_device_info(NtcHipContext* ctx, char* name, size_t nameSize, int* computeUnits)
{
    CTX_ENTER(ctx);
    if (name && nameSize) { std::snprintf(name, nameSize, "%s", L.name); }
    if (computeUnits) *computeUnits = L.computeUnits;
    return 0;
}

int ntc_hip_ctx_device_clock(NtcHipContext* ctx, int* clockRateKHz)
{
    CTX_ENTER(ctx);
    if (!clockRateKHz) { set_error("ntc_hip_device_clock: null out-pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    *clockRateKHz = L.clockRateKHz;
    return 0;
}

int ntc_hip_ctx_alloc(NtcHipContext* ctx, void** devPtr, size_t bytes)
{
    CTX_ENTER(ctx);
    if (!devPtr) { set_error("ntc_hip_alloc: null out-pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    *devPtr = nullptr;
    HIP_TRY(hipMalloc(devPtr, bytes ? bytes : 1));
    return 0;
}

int ntc_hip_ctx_free(NtcHipContext* ctx, void* devPtr)
{
    CTX_ENTER(ctx);
    if (!devPtr) return 0;
    HIP_TRY(hipStreamSynchronize(L.stream));
    HIP_TRY(hipFree(devPtr));
    return 0;
}

int ntc_hip_ctx_upload(NtcHipContext* ctx, void* dst, const void* src, size_t bytes)
{
    CTX_ENTER(ctx);
    if (bytes == 0) return 0;
    if (!dst || !src) { set_error("ntc_hip_upload: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, L.stream));
    HIP_TRY(hipStreamSynchronize(L.stream));
    return 0;
}

int ntc_hip_ctx_download(NtcHipContext* ctx, void* dst, const void* src, size_t bytes)
{
    CTX_ENTER(ctx);
    if (bytes == 0) return 0;
    if (!dst || !src) { set_error("ntc_hip_download: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, L.stream));
    HIP_TRY(hipStreamSynchronize(L.stream));
    return 0;
}

int ntc_hip_ctx_memset(NtcHipContext* ctx, void* dst, int value, size_t bytes)
{
    CTX_ENTER(ctx);
    if (bytes == 0) return 0;
    if (!dst) { set_error("ntc_hip_memset: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    HIP_TRY(launch_fill(static_cast<uint8_t*>(dst), uint8_t(value), bytes, L.stream));    // a kernel, not hipMemsetAsync
    return 0;
}

int ntc_hip_ctx_synchronize(NtcHipContext* ctx)
{
    CTX_ENTER(ctx);
    HIP_TRY(hipStreamSynchronize(L.stream));
    return 0;
}

int ntc_hip_weight_layout(const NtcHipDecoderSpec* spec, NtcHipWeightLayout* out)
{
    if (!spec || !out) { set_error("ntc_hip_weight_layout: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    if (!spec_sane(*spec)) { set_error("ntc_hip_weight_layout: malformed decoder spec."); return NTC_HIP_ERR_INVALID_ARG; }
    std::memset(out, 0, sizeof(*out));
    uint32_t cursor = 0;
    // Matrices first, one byte per weight, layer after layer (src/WeightLayout.cpp:157-176).
    for (int l = 0; l < NTC_HIP_MLP_LAYERS; ++l) {
        out->weightOffset[l] = cursor;
        cursor += uint32_t(layer_in(*spec, l)) * uint32_t(layer_out(*spec, l));
    }
    if (spec->weightType == NTC_HIP_WEIGHTS_INT8 || spec->weightType == NTC_HIP_WEIGHTS_FP8_SCALED) {
        // then every scale vector, then every bias vector (src/WeightLayout.cpp:229-247)
        for (int l = 0; l < NTC_HIP_MLP_LAYERS; ++l) { out->scaleOffset[l] = cursor; cursor += 4u * uint32_t(layer_out(*spec, l)); }
        for (int l = 0; l < NTC_HIP_MLP_LAYERS; ++l) { out->biasOffset[l] = cursor; cursor += 4u * uint32_t(layer_out(*spec, l)); }
    } else {
        // fp16 bias of the e4m3 layers, then scale and bias of the int8 output layer (src/WeightLayout.cpp:249-262)
        int const last = NTC_HIP_MLP_LAYERS - 1;
        for (int l = 0; l < last; ++l) { out->biasOffset[l] = cursor; cursor += 2u * uint32_t(layer_out(*spec, l)); }
        out->scaleOffset[last] = cursor; cursor += 4u * uint32_t(layer_out(*spec, last));
        out->biasOffset[last] = cursor;  cursor += 4u * uint32_t(layer_out(*spec, last));
    }
    out->bufferSize = cursor;
    return 0;
}

uint64_t ntc_hip_grid_bytes(int32_t width, int32_t height, int32_t features, int32_t bits)
{
    return grid_bytes(width, height, features, bits);
}

int ntc_hip_ctx_decode(NtcHipContext* ctx, const NtcHipTextureSet* sets, int32_t numSets)
{
    CTX_ENTER(ctx);
    std::vector<DevMip> table;
    int variant = NTC_HIP_VARIANT_NONE, totalTiles = 0;
    if (int r = build_table(sets, numSets, table, variant, totalTiles)) return r;
    if (int r = upload_table(L, table)) return r;
    HIP_TRY(launch_decode_any(L, variant, L.tableDev, int(table.size()), totalTiles, grid_size_for(L, variant, totalTiles)));
    clear_error();
    return 0;
}

int ntc_hip_ctx_decode_static(NtcHipContext* ctx, const NtcHipTextureSet* sets, int32_t numSets)
{
    CTX_ENTER(ctx);
    // No allocation on either side: the table is assembled in the context's own array (not in a vector) and
    // travels to the device as kernel arguments.
    TableSink sink;
    sink.fixed = L.staticBuild;
    sink.capacity = size_t(kStaticTableEntries);
    size_t entries = 0;
    int variant = NTC_HIP_VARIANT_NONE, totalTiles = 0;
    if (int r = build_table(sets, numSets, sink, entries, variant, totalTiles)) return r;
    if (entries > size_t(kStaticTableEntries)) {
        set_error("ntc_hip_decode_static: %zu mips in one call; the built-in table holds %d (use ntc_hip_decode).",
                  entries, kStaticTableEntries);
        return NTC_HIP_ERR_INVALID_ARG;
    }
    // A chunk per launch, into this device's built-in array.  Stream order keeps a decode that still reads the
    // previous table ahead of these stores.
    for (size_t first = 0; first < entries; first += kTableChunkEntries) {
        size_t const count = entries - first < size_t(kTableChunkEntries) ? entries - first : size_t(kTableChunkEntries);
        TableChunk chunk;
        std::memset(&chunk, 0, sizeof(chunk));
        std::memcpy(chunk.entries, L.staticBuild + first, count * sizeof(DevMip));
        write_table_kernel<<<1, 256, 0, L.stream>>>(reinterpret_cast<uint32_t*>(L.staticTable + first), chunk,
                                                    int(count * sizeof(DevMip) / 4));
        HIP_TRY(hipGetLastError());
    }
    HIP_TRY(launch_decode_any(L, variant, L.staticTable, int(entries), totalTiles, grid_size_for(L, variant, totalTiles)));
    clear_error();
    return 0;
}

int ntc_hip_ctx_decode_timed(NtcHipContext* ctx, const NtcHipTextureSet* sets, int32_t numSets, int32_t iterations, float* outMs)
{
    CTX_ENTER(ctx);
    if (iterations < 1 || !outMs) { set_error("ntc_hip_decode_timed: iterations must be >= 1 and the result pointer non-null."); return NTC_HIP_ERR_INVALID_ARG; }
    std::vector<DevMip> table;
    int variant = NTC_HIP_VARIANT_NONE, totalTiles = 0;
    if (int r = build_table(sets, numSets, table, variant, totalTiles)) return r;
    if (int r = upload_table(L, table)) return r;
    int const grid = grid_size_for(L, variant, totalTiles);
    HIP_TRY(hipEventRecord(L.evStart, L.stream));
    for (int i = 0; i < iterations; ++i)
        HIP_TRY(launch_decode_any(L, variant, L.tableDev, int(table.size()), totalTiles, grid));
    HIP_TRY(hipEventRecord(L.evStop, L.stream));
    HIP_TRY(hipEventSynchronize(L.evStop));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, L.evStart, L.evStop));
    *outMs = ms / float(iterations);
    clear_error();
    return 0;
}

int ntc_hip_ctx_timer_begin(NtcHipContext* ctx)
{
    CTX_ENTER(ctx);
    HIP_TRY(hipEventRecord(L.evSpanStart, L.stream));
    L.spanOpen = true;
    clear_error();
    return 0;
}

int ntc_hip_ctx_timer_end(NtcHipContext* ctx, float* outMilliseconds)
{
    CTX_ENTER(ctx);
    if (!outMilliseconds) { set_error("ntc_hip_timer_end: the result pointer is null."); return NTC_HIP_ERR_INVALID_ARG; }
    if (!L.spanOpen) { set_error("ntc_hip_timer_end: no ntc_hip_timer_begin before it on this context."); return NTC_HIP_ERR_INVALID_ARG; }
    L.spanOpen = false;
    HIP_TRY(hipEventRecord(L.evSpanStop, L.stream));
    HIP_TRY(hipEventSynchronize(L.evSpanStop));
    HIP_TRY(hipEventElapsedTime(outMilliseconds, L.evSpanStart, L.evSpanStop));
    clear_error();
    return 0;
}

static int run_queries(NtcHipContext* ctx, const NtcHipTextureSet* set, const NtcHipQuery* queries, uint64_t numQueries, void* out, uint64_t outBytes,
                       int iterations, float* outMs)
{
    CTX_ENTER(ctx);
    if (!set || !queries || !out) { set_error("ntc_hip_decode_queries: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    if (numQueries == 0) { if (outMs) *outMs = 0.f; return 0; }
    if (numQueries > (uint64_t(1) << 40)) { set_error("ntc_hip_decode_queries: too many queries in one call."); return NTC_HIP_ERR_INVALID_ARG; }
    if (outBytes < numQueries * 32u) { set_error("ntc_hip_decode_queries: the output buffer holds %llu bytes, %llu queries need %llu.", (unsigned long long)outBytes, (unsigned long long)numQueries, (unsigned long long)(numQueries * 32u)); return NTC_HIP_ERR_INVALID_ARG; }
    if ((reinterpret_cast<uintptr_t>(out) & 7u) || (reinterpret_cast<uintptr_t>(queries) & 3u)) { set_error("ntc_hip_decode_queries: output must be 8-byte and queries 4-byte aligned."); return NTC_HIP_ERR_INVALID_ARG; }
    std::vector<DevMip> table;
    int variant = NTC_HIP_VARIANT_NONE, totalTiles = 0;
    if (int r = build_table(set, 1, table, variant, totalTiles, true)) return r;
    bool const fp8 = variant_is_fp8_network(variant);
    if (int r = upload_table(L, table)) return r;
    uint64_t const perBlock = uint64_t(fp8 ? fp8_threads_per_workgroup() : threads_per_workgroup(variant));
    uint64_t const blocks = (numQueries + perBlock - 1) / perBlock;
    uint64_t const resident = uint64_t(L.computeUnits) * uint64_t(grid_size_for(L, variant, 0x7fffffff) / L.computeUnits);
    int const grid = int(blocks < resident ? blocks : resident);
    if (outMs) HIP_TRY(hipEventRecord(L.evStart, L.stream));
    for (int i = 0; i < iterations; ++i)
        HIP_TRY(fp8 ? launch_queries_fp8(variant, L.tableDev, int(table.size()), reinterpret_cast<DevQuery const*>(queries), numQueries,
                                         static_cast<uint16_t*>(out), grid, next_handoff(L, L.tableDev), L.stream)
                    : launch_queries(variant, L.tableDev, int(table.size()), reinterpret_cast<DevQuery const*>(queries), numQueries,
                                     static_cast<uint16_t*>(out), grid, L.stream));
    if (outMs) {
        HIP_TRY(hipEventRecord(L.evStop, L.stream));
        HIP_TRY(hipEventSynchronize(L.evStop));
        float ms = 0.f;
        HIP_TRY(hipEventElapsedTime(&ms, L.evStart, L.evStop));
        *outMs = ms / float(iterations);
    }
    clear_error();
    return 0;
}

uint64_t ntc_hip_query_latents_bytes(const NtcHipTextureSet* set)
{
    BrickPlan plan;
    if (!set || !plan_bricks(*set, plan)) { set_error("ntc_hip_query_latents_bytes: malformed texture set."); return 0; }
    return plan.totalBytes;
}

int ntc_hip_ctx_build_query_latents(NtcHipContext* ctx, const NtcHipTextureSet* set, void* dst, uint64_t dstBytes)
{
    CTX_ENTER(ctx);
    if (!set || !dst || !set->latents) { set_error("ntc_hip_build_query_latents: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    BrickPlan plan;
    if (!plan_bricks(*set, plan)) { set_error("ntc_hip_build_query_latents: malformed texture set."); return NTC_HIP_ERR_INVALID_ARG; }
    if (dstBytes < plan.totalBytes || (reinterpret_cast<uintptr_t>(dst) & 127u) || (reinterpret_cast<uintptr_t>(set->latents) & 1u)) {
        set_error("ntc_hip_build_query_latents: the destination must be 128-byte aligned and hold %llu bytes.", (unsigned long long)plan.totalBytes);
        return NTC_HIP_ERR_INVALID_ARG;
    }
    for (BrickGrid const& g : plan.grids) {
        uint64_t const srcBytes = uint64_t(g.width) * uint64_t(g.height) * 2u * uint64_t(g.layers);
        if ((g.srcOffset & 1u) || reaches_past(g.srcOffset, srcBytes, set->latentsBytes) || srcBytes >= (1ull << 32)) {
            set_error("ntc_hip_build_query_latents: a latent grid reaches past the %llu-byte latent buffer.", (unsigned long long)set->latentsBytes);
            return NTC_HIP_ERR_INVALID_ARG;
        }
    }
    // (bricks of grids narrower than a brick keep cells that nothing writes and no query reads)
    for (BrickGrid const& g : plan.grids)
        HIP_TRY(launch_build_bricks(reinterpret_cast<uint16_t const*>(static_cast<uint8_t const*>(set->latents) + g.srcOffset),
                                    static_cast<uint8_t*>(dst) + g.dstOffset, g.width, g.height, g.layers, L.stream));
    clear_error();
    return 0;
}

int ntc_hip_ctx_decode_queries(NtcHipContext* ctx, const NtcHipTextureSet* set, const NtcHipQuery* queries, uint64_t numQueries, void* out, uint64_t outBytes)
{
    return run_queries(ctx, set, queries, numQueries, out, outBytes, 1, nullptr);
}

int ntc_hip_ctx_decode_queries_timed(NtcHipContext* ctx, const NtcHipTextureSet* set, const NtcHipQuery* queries, uint64_t numQueries, void* out, uint64_t outBytes, int32_t iterations, float* outMillisecondsPerIteration)
{
    if (iterations < 1 || !outMillisecondsPerIteration) { set_error("ntc_hip_decode_queries_timed: iterations must be >= 1 and the result pointer non-null."); return NTC_HIP_ERR_INVALID_ARG; }
    return run_queries(ctx, set, queries, numQueries, out, outBytes, iterations, outMillisecondsPerIteration);
}

// Largest power of two up to 16 that divides the base address, the row pitch and the pixel stride:
// every pixel of the image starts on such a boundary.
static int32_t common_alignment(uintptr_t base, uint64_t rowPitch, uint64_t pixelStride)
{
    uint64_t const bits = uint64_t(base) | rowPitch | pixelStride | 16u;
    return int32_t(bits & (~bits + 1));
}

int ntc_hip_ctx_read_channels(NtcHipContext* ctx, const NtcHipReadChannels* p)
{
    CTX_ENTER(ctx);
    if (!p || !p->planarPairs || !p->dst) { set_error("ntc_hip_read_channels: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    int bpc = 0;
    switch (p->format) {
    case NTC_HIP_DEV_FORMAT_UNORM8: bpc = 1; break;
    case NTC_HIP_DEV_FORMAT_UNORM16: case NTC_HIP_DEV_FORMAT_FLOAT16: bpc = 2; break;
    case NTC_HIP_DEV_FORMAT_FLOAT32: case NTC_HIP_DEV_FORMAT_UINT32: bpc = 4; break;
    default: set_error("ntc_hip_read_channels: unknown channel format %d.", p->format); return NTC_HIP_ERR_INVALID_ARG;
    }
    if (p->width < 1 || p->height < 1 || p->setChannels < 2 || (p->setChannels & 1) || p->setChannels > NTC_HIP_MAX_CHANNELS
        || p->firstChannel < 0 || p->numChannels < 1 || p->firstChannel + p->numChannels > p->setChannels) {
        set_error("ntc_hip_read_channels: bad image or channel range.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    if ((p->dstWidth == 0) != (p->dstHeight == 0) || p->dstWidth < 0 || p->dstHeight < 0) {
        set_error("ntc_hip_read_channels: dstWidth and dstHeight must both be positive, or both 0 for the mip's size.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    bool const resample = p->dstWidth > 0 && (p->dstWidth != p->width || p->dstHeight != p->height);
    int const imageWidth = resample ? p->dstWidth : p->width, imageHeight = resample ? p->dstHeight : p->height;
    if (p->pixelStride < uint64_t(bpc) || p->pixelStride > kMaxPixelStride || p->rowPitch > kMaxRowPitch || p->rowPitch < p->pixelStride * uint64_t(imageWidth)
        || (p->pixelStride % uint64_t(bpc)) || (p->rowPitch % uint64_t(bpc)) || (reinterpret_cast<uintptr_t>(p->dst) % uintptr_t(bpc))) {
        set_error("ntc_hip_read_channels: pixel stride / row pitch do not fit the format.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    uint64_t const dstChannels = p->pixelStride / uint64_t(bpc);
    if (dstChannels > 64) { set_error("ntc_hip_read_channels: pixel stride too large."); return NTC_HIP_ERR_INVALID_ARG; }
    uint64_t const need = uint64_t(imageHeight - 1) * p->rowPitch + uint64_t(imageWidth) * p->pixelStride;
    uint64_t const srcNeed = uint64_t(p->width) * uint64_t(p->height) * uint64_t(p->setChannels) * 2u;
    if (need > p->dstBytes || srcNeed > p->planarBytes) {
        set_error("ntc_hip_read_channels: image reaches past the given buffer sizes.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    ReadChannelsArgs a{};
    a.planarPairs = static_cast<uint16_t const*>(p->planarPairs);
    a.dst = static_cast<uint8_t*>(p->dst);
    a.pixelStride = p->pixelStride; a.rowPitch = p->rowPitch;
    a.width = p->width; a.height = p->height; a.setChannels = p->setChannels;
    a.firstChannel = p->firstChannel; a.numChannels = p->numChannels;
    a.dstChannels = int32_t(dstChannels); a.format = p->format;
    a.useDithering = p->useDithering ? 1 : 0;
    a.vectorBytes = common_alignment(reinterpret_cast<uintptr_t>(p->dst), p->rowPitch, p->pixelStride);
    a.dstWidth = resample ? p->dstWidth : 0; a.dstHeight = resample ? p->dstHeight : 0;
    for (int i = 0; i < 16; ++i) {
        if (p->srcColorSpaces[i] > 2 || p->dstColorSpaces[i] > 2) { set_error("ntc_hip_read_channels: unknown colour space for channel %d.", i); return NTC_HIP_ERR_INVALID_ARG; }
        a.srcColorSpaces[i] = p->srcColorSpaces[i];
        a.dstColorSpaces[i] = p->dstColorSpaces[i];
    }
    HIP_TRY(launch_read_channels(a, L.stream));
    clear_error();
    return 0;
}

static int bytes_per_component(int format)
{
    switch (format) {
    case NTC_HIP_DEV_FORMAT_UNORM8: return 1;
    case NTC_HIP_DEV_FORMAT_UNORM16: case NTC_HIP_DEV_FORMAT_FLOAT16: return 2;
    case NTC_HIP_DEV_FORMAT_FLOAT32: case NTC_HIP_DEV_FORMAT_UINT32: return 4;
    default: return 0;
    }
}

int ntc_hip_ctx_write_channels(NtcHipContext* ctx, const NtcHipWriteChannels* p)
{
    CTX_ENTER(ctx);
    if (!p || !p->src || !p->planarPairs) { set_error("ntc_hip_write_channels: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    int const bpc = bytes_per_component(p->format);
    if (!bpc) { set_error("ntc_hip_write_channels: unknown channel format %d.", p->format); return NTC_HIP_ERR_INVALID_ARG; }
    if (p->width < 1 || p->height < 1 || p->setChannels < 2 || (p->setChannels & 1) || p->setChannels > NTC_HIP_MAX_CHANNELS
        || p->firstChannel < 0 || p->numChannels < 1 || p->firstChannel + p->numChannels > p->setChannels) {
        set_error("ntc_hip_write_channels: bad image or channel range.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    if ((p->srcWidth == 0) != (p->srcHeight == 0) || p->srcWidth < 0 || p->srcHeight < 0) {
        set_error("ntc_hip_write_channels: srcWidth and srcHeight must both be positive, or both 0 for the mip's size.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    bool const resample = p->srcWidth > 0 && (p->srcWidth != p->width || p->srcHeight != p->height);
    int const imageWidth = resample ? p->srcWidth : p->width, imageHeight = resample ? p->srcHeight : p->height;
    if (p->pixelStride < uint64_t(bpc) * uint64_t(p->numChannels) || p->pixelStride > kMaxPixelStride || p->rowPitch > kMaxRowPitch
        || p->rowPitch < p->pixelStride * uint64_t(imageWidth) || (p->pixelStride % uint64_t(bpc)) || (p->rowPitch % uint64_t(bpc)) || (reinterpret_cast<uintptr_t>(p->src) % uintptr_t(bpc))) {
        set_error("ntc_hip_write_channels: pixel stride / row pitch do not fit the format and channel count.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    uint64_t const srcNeed = uint64_t(imageHeight - 1) * p->rowPitch + uint64_t(imageWidth - 1) * p->pixelStride + uint64_t(bpc) * uint64_t(p->numChannels);
    uint64_t const dstNeed = uint64_t(p->width) * uint64_t(p->height) * uint64_t(p->setChannels) * 2u;
    if (srcNeed > p->srcBytes || dstNeed > p->planarBytes) { set_error("ntc_hip_write_channels: image reaches past the given buffer sizes."); return NTC_HIP_ERR_INVALID_ARG; }
    WriteChannelsArgs a{};
    a.src = static_cast<uint8_t const*>(p->src);
    a.planarPairs = static_cast<uint16_t*>(p->planarPairs);
    a.pixelStride = p->pixelStride; a.rowPitch = p->rowPitch;
    a.width = p->width; a.height = p->height; a.setChannels = p->setChannels;
    a.firstChannel = p->firstChannel; a.numChannels = p->numChannels; a.format = p->format; a.verticalFlip = p->verticalFlip ? 1 : 0;
    a.vectorBytes = common_alignment(reinterpret_cast<uintptr_t>(p->src), p->rowPitch, p->pixelStride);
    a.srcWidth = resample ? p->srcWidth : 0; a.srcHeight = resample ? p->srcHeight : 0;
    for (int i = 0; i < 16; ++i) {
        if (p->srcColorSpaces[i] > 2 || p->dstColorSpaces[i] > 2) { set_error("ntc_hip_write_channels: unknown colour space for channel %d.", i); return NTC_HIP_ERR_INVALID_ARG; }
        a.srcColorSpaces[i] = p->srcColorSpaces[i];
        a.dstColorSpaces[i] = p->dstColorSpaces[i];
    }
    HIP_TRY(launch_write_channels(a, L.stream));
    clear_error();
    return 0;
}

int ntc_hip_ctx_image_loss(NtcHipContext* ctx, void* decoded, const void* reference, uint64_t planarBytes, int32_t width, int32_t height, int32_t setChannels, uint32_t validChannelMask, int32_t maskChannelIndex, int32_t discardMaskedOutPixels, float* outMse)
{
    CTX_ENTER(ctx);
    if (!decoded || !reference || !outMse) { set_error("ntc_hip_image_loss: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    if (width < 1 || height < 1 || setChannels < 2 || (setChannels & 1) || setChannels > NTC_HIP_MAX_CHANNELS
        || uint64_t(width) * uint64_t(height) * uint64_t(setChannels) * 2u > planarBytes) {
        set_error("ntc_hip_image_loss: bad image shape or buffer size.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    if (maskChannelIndex >= setChannels) {      // src/TextureSet.cpp:1899-1902; negative = no mask channel
        set_error("ntc_hip_image_loss: maskChannelIndex (%d) must be below the channel count (%d).", maskChannelIndex, setChannels);
        return NTC_HIP_ERR_INVALID_ARG;
    }
    if (maskChannelIndex >= 0) {                // the decoded image is then written while the reference is read
        uintptr_t const d = reinterpret_cast<uintptr_t>(decoded), r = reinterpret_cast<uintptr_t>(reference);
        uint64_t const imageBytes = uint64_t(width) * uint64_t(height) * uint64_t(setChannels) * 2u;
        if (d < r + imageBytes && r < d + imageBytes) {
            set_error("ntc_hip_image_loss: with a mask channel the decoded and the reference image must not overlap.");
            return NTC_HIP_ERR_INVALID_ARG;
        }
    }
    size_t const blocks = image_loss_blocks(width, height);
    size_t const bytes = (blocks + 1) * NTC_HIP_DEV_MAX_CHANNELS * sizeof(double);    // partial sums, then the 16 totals
    if (bytes > L.lossBytes) {
        HIP_TRY(hipStreamSynchronize(L.stream));
        if (L.lossDev) { HIP_TRY(hipFree(L.lossDev)); L.lossDev = nullptr; }
        L.lossBytes = 0;
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&L.lossDev), bytes));
        if (!L.lossHost) HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&L.lossHost), NTC_HIP_DEV_MAX_CHANNELS * sizeof(double), hipHostMallocDefault));
        L.lossBytes = bytes;
    }
    HIP_TRY(launch_image_loss(static_cast<uint16_t*>(decoded), static_cast<uint16_t const*>(reference), width, height,
                              setChannels, validChannelMask, maskChannelIndex < 0 ? -1 : maskChannelIndex,
                              discardMaskedOutPixels ? 1 : 0, L.lossDev, L.stream));
    HIP_TRY(hipMemcpyAsync(L.lossHost, L.lossDev + blocks * NTC_HIP_DEV_MAX_CHANNELS, NTC_HIP_DEV_MAX_CHANNELS * sizeof(double),
                           hipMemcpyDeviceToHost, L.stream));
    HIP_TRY(hipStreamSynchronize(L.stream));
    double const norm = 1.0 / (double(width) * double(height));
    for (int c = 0; c < NTC_HIP_DEV_MAX_CHANNELS; ++c) outMse[c] = float(L.lossHost[c] * norm);
    clear_error();
    return 0;
}

int ntc_hip_ctx_resize_planar(NtcHipContext* ctx, const void* src, uint64_t srcBytes, int32_t srcWidth, int32_t srcHeight, void* dst, uint64_t dstBytes, int32_t dstWidth, int32_t dstHeight, int32_t setChannels, const uint8_t* channelColorSpaces)
{
    CTX_ENTER(ctx);
    if (!src || !dst) { set_error("ntc_hip_resize_planar: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    if (srcWidth < 1 || srcHeight < 1 || dstWidth < 1 || dstHeight < 1 || setChannels < 2 || (setChannels & 1) || setChannels > NTC_HIP_MAX_CHANNELS) {
        set_error("ntc_hip_resize_planar: bad image shape.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    uint64_t const srcNeed = uint64_t(srcWidth) * uint64_t(srcHeight) * uint64_t(setChannels) * 2u;
    uint64_t const dstNeed = uint64_t(dstWidth) * uint64_t(dstHeight) * uint64_t(setChannels) * 2u;
    if (srcNeed > srcBytes || dstNeed > dstBytes) { set_error("ntc_hip_resize_planar: image reaches past the given buffer sizes."); return NTC_HIP_ERR_INVALID_ARG; }
    uintptr_t const s = reinterpret_cast<uintptr_t>(src), d = reinterpret_cast<uintptr_t>(dst);
    if (s < d + dstNeed && d < s + srcNeed) { set_error("ntc_hip_resize_planar: source and destination overlap."); return NTC_HIP_ERR_INVALID_ARG; }
    if ((s | d) & 3u) { set_error("ntc_hip_resize_planar: images must be 4-byte aligned."); return NTC_HIP_ERR_INVALID_ARG; }
    if (channelColorSpaces)
        for (int i = 0; i < 16; ++i)
            if (channelColorSpaces[i] > 2) { set_error("ntc_hip_resize_planar: unknown colour space for channel %d.", i); return NTC_HIP_ERR_INVALID_ARG; }
    HIP_TRY(launch_resize_planar(static_cast<uint16_t const*>(src), srcWidth, srcHeight, static_cast<uint16_t*>(dst), dstWidth, dstHeight,
                                 setChannels, channelColorSpaces, L.stream));
    clear_error();
    return 0;
}

static int check_diff_image(NtcHipImage const& im, char const* which, int left, int top, int width, int height, DiffImageArgs& out)
{
    int const bpc = bytes_per_component(im.format);
    if (!im.data || !bpc) { set_error("ntc_hip_image_difference: image %s has no data or an unknown channel format (%d).", which, im.format); return NTC_HIP_ERR_INVALID_ARG; }
    if (im.numChannels < 1 || im.numChannels > 4 || im.width < 1 || im.height < 1) { set_error("ntc_hip_image_difference: image %s: 1..4 channels and a positive size are required.", which); return NTC_HIP_ERR_INVALID_ARG; }
    if (im.pixelStride < uint64_t(bpc) * uint64_t(im.numChannels) || im.pixelStride > kMaxPixelStride || im.rowPitch > kMaxRowPitch
        || im.rowPitch < im.pixelStride * uint64_t(im.width) || (im.pixelStride % uint64_t(bpc)) || (im.rowPitch % uint64_t(bpc)) || (reinterpret_cast<uintptr_t>(im.data) % uintptr_t(bpc))) {
        set_error("ntc_hip_image_difference: image %s: pixel stride / row pitch do not fit the format and channel count.", which);
        return NTC_HIP_ERR_INVALID_ARG;
    }
    if (uint64_t(im.height - 1) * im.rowPitch + uint64_t(im.width - 1) * im.pixelStride + uint64_t(bpc) * uint64_t(im.numChannels) > im.bytes) {
        set_error("ntc_hip_image_difference: image %s reaches past its buffer.", which);
        return NTC_HIP_ERR_INVALID_ARG;
    }
    if (int64_t(left) + width > im.width || int64_t(top) + height > im.height) {
        set_error("ntc_hip_image_difference: the extent (%d, %d, %d x %d) does not lie inside image %s (%d x %d).", left, top, width, height, which, im.width, im.height);
        return NTC_HIP_ERR_INVALID_ARG;
    }
    out.data = static_cast<uint8_t const*>(im.data);
    out.pixelStride = im.pixelStride; out.rowPitch = im.rowPitch; out.format = im.format; out.numChannels = im.numChannels;
    return 0;
}

int ntc_hip_ctx_image_difference(NtcHipContext* ctx, const NtcHipImageDifference* p)
{
    CTX_ENTER(ctx);
    if (!p || !p->output) { set_error("ntc_hip_image_difference: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    // src/Context.cpp:796-812
    if (p->left < 0 || p->top < 0) { set_error("ntc_hip_image_difference: left (%d) and top (%d) must be non-negative.", p->left, p->top); return NTC_HIP_ERR_INVALID_ARG; }
    if (p->width <= 0 || p->height <= 0 || int64_t(p->width) * int64_t(p->height) > INT32_MAX) {
        set_error("ntc_hip_image_difference: width (%d) and height (%d) must be positive (and their product below 2^31).", p->width, p->height);
        return NTC_HIP_ERR_INVALID_ARG;
    }
    if ((p->outputOffset & 7u) || (reinterpret_cast<uintptr_t>(p->output) & 7u) || uint64_t(p->outputOffset) + 32u > p->outputBytes) {
        set_error("ntc_hip_image_difference: the four 64-bit results at outputOffset (%u) must be 8-byte aligned and inside the output buffer.", p->outputOffset);
        return NTC_HIP_ERR_INVALID_ARG;
    }
    ImageDifferenceArgs a{};
    if (int r = check_diff_image(p->a, "A", p->left, p->top, p->width, p->height, a.a)) return r;
    if (int r = check_diff_image(p->b, "B", p->left, p->top, p->width, p->height, a.b)) return r;
    a.left = p->left; a.top = p->top; a.width = p->width; a.height = p->height;
    a.alphaThreshold = p->alphaThreshold; a.useAlphaThreshold = p->useAlphaThreshold ? 1 : 0; a.useMSLE = p->useMSLE ? 1 : 0;
    a.output = reinterpret_cast<unsigned long long*>(static_cast<uint8_t*>(p->output) + p->outputOffset);
    HIP_TRY(launch_image_difference(a, L.stream));
    clear_error();
    return 0;
}

int ntc_hip_ctx_block_compress(NtcHipContext* ctx, const NtcHipBlockCompress* p)
{
    CTX_ENTER(ctx);
    if (!p || !p->dst) { set_error("ntc_hip_block_compress: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    if (p->dstFormat < 1 || p->dstFormat > 7) { set_error("ntc_hip_block_compress: dstFormat (%d) is not a block-compressed format.", p->dstFormat); return NTC_HIP_ERR_INVALID_ARG; }
    if (p->srcLeft < 0 || p->srcTop < 0 || p->widthInBlocks < 1 || p->heightInBlocks < 1 || p->dstOffsetX < 0 || p->dstOffsetY < 0
        || p->widthInBlocks > (1 << 20) || p->heightInBlocks > (1 << 20) || p->dstOffsetX > (1 << 20) || p->dstOffsetY > (1 << 20)) {
        set_error("ntc_hip_block_compress: bad extent or destination offset.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    BlockCompressArgs a{};
    DiffImageArgs image{};
    if (int r = check_diff_image(p->src, "src", 0, 0, 1, 1, image)) return r;     // the extent may reach past the image: such pixels read as 0
    uint64_t const blockBytes = (p->dstFormat == 1 || p->dstFormat == 4) ? 8u : 16u;
    uint64_t const rowNeed = uint64_t(p->dstOffsetX + p->widthInBlocks) * blockBytes;
    if ((p->dstRowPitch & 7u) || p->dstRowPitch < rowNeed || p->dstRowPitch > kMaxRowPitch || (reinterpret_cast<uintptr_t>(p->dst) & 7u)
        || uint64_t(p->dstOffsetY + p->heightInBlocks - 1) * p->dstRowPitch + rowNeed > p->dstBytes) {
        set_error("ntc_hip_block_compress: the destination (8-byte aligned, row pitch a multiple of 8) does not hold the blocks.");
        return NTC_HIP_ERR_INVALID_ARG;
    }
    a.src = image.data; a.pixelStride = image.pixelStride; a.rowPitch = image.rowPitch; a.format = image.format; a.numChannels = image.numChannels;
    a.srcWidth = p->src.width; a.srcHeight = p->src.height;
    a.packedRgba8 = image.format == NTC_HIP_DEV_FORMAT_UNORM8 && image.numChannels == 4
        && ((reinterpret_cast<uintptr_t>(image.data) | image.pixelStride | image.rowPitch) & 3u) == 0;
    a.dst = static_cast<uint8_t*>(p->dst); a.dstRowPitch = p->dstRowPitch;
    a.srcLeft = p->srcLeft; a.srcTop = p->srcTop; a.widthInBlocks = p->widthInBlocks; a.heightInBlocks = p->heightInBlocks;
    a.dstOffsetX = p->dstOffsetX; a.dstOffsetY = p->dstOffsetY;
    a.alphaThreshold = p->alphaThreshold;
    if (p->dstFormat == 7 && p->modeBuffer) {
        if (p->modeMapWidthInBlocks < 1 || p->modeMapHeightInBlocks < 1 || p->modeMapWidthInBlocks > (1 << 20) || p->modeMapHeightInBlocks > (1 << 20)
            || p->modeMapOffsetX < -(1 << 20) || p->modeMapOffsetX > (1 << 20) || p->modeMapOffsetY < -(1 << 20) || p->modeMapOffsetY > (1 << 20)) {
            set_error("ntc_hip_block_compress: bad mode map size or offset.");
            return NTC_HIP_ERR_INVALID_ARG;
        }
        // size of MakeBC7ModeBuffer's output for the map: 9 bits per block, rounded up to whole 32-bit words
        uint64_t const mapBytes = ((uint64_t(p->modeMapWidthInBlocks) * uint64_t(p->modeMapHeightInBlocks) * 9u + 31u) >> 5) << 2;
        if ((p->modeBufferByteOffset & 3u) || (reinterpret_cast<uintptr_t>(p->modeBuffer) & 3u) || reaches_past(p->modeBufferByteOffset, mapBytes, p->modeBufferBytes)) {
            set_error("ntc_hip_block_compress: the mode buffer (4-byte aligned, offset a multiple of 4) does not hold the %llu bytes of a %d x %d mode map.",
                      (unsigned long long)mapBytes, p->modeMapWidthInBlocks, p->modeMapHeightInBlocks);
            return NTC_HIP_ERR_INVALID_ARG;
        }
        a.modeBuffer = reinterpret_cast<uint32_t const*>(static_cast<uint8_t const*>(p->modeBuffer) + p->modeBufferByteOffset);
        a.modeMapWidthInBlocks = p->modeMapWidthInBlocks; a.modeMapHeightInBlocks = p->modeMapHeightInBlocks;
        a.modeMapOffsetX = p->modeMapOffsetX; a.modeMapOffsetY = p->modeMapOffsetY;
    }
    HIP_TRY(launch_block_compress(a, p->dstFormat, L.stream));
    clear_error();
    return 0;
}

int ntc_hip_selftest_mfma(const int8_t* a16x64, const int8_t* b64x16, int32_t* d16x16)
{
    NtcHipContext* const ctx = g_default;
    CTX_ENTER(ctx);
    if (!a16x64 || !b64x16 || !d16x16) { set_error("ntc_hip_selftest_mfma: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    int8_t *a = nullptr, *b = nullptr; int32_t* d = nullptr;
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&a), 1024));
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b), 1024));
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&d), 1024));
    HIP_TRY(hipMemcpy(a, a16x64, 1024, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(b, b64x16, 1024, hipMemcpyHostToDevice));
    HIP_TRY(launch_selftest_mfma(a, b, d, L.stream));
    HIP_TRY(hipStreamSynchronize(L.stream));
    HIP_TRY(hipMemcpy(d16x16, d, 1024, hipMemcpyDeviceToHost));
    (void)hipFree(a); (void)hipFree(b); (void)hipFree(d);
    return 0;
}

int ntc_hip_selftest_fp8_activation(const uint16_t* halves, int32_t count, uint16_t* out)
{
    NtcHipContext* const ctx = g_default;
    CTX_ENTER(ctx);
    if (!halves || !out || count < 1 || count > (1 << 20)) { set_error("ntc_hip_selftest_fp8_activation: null pointer or count outside 1..2^20."); return NTC_HIP_ERR_INVALID_ARG; }
    uint16_t* dev = nullptr;
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&dev), size_t(count) * 8));
    hipError_t e = hipMemcpy(dev, halves, size_t(count) * 2, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = launch_selftest_fp8_activation(dev, dev + count, count, L.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(L.stream);
    if (e == hipSuccess) e = hipMemcpy(out, dev + count, size_t(count) * 6, hipMemcpyDeviceToHost);
    (void)hipFree(dev);
    HIP_TRY(e);
    return 0;
}

int ntc_hip_selftest_mfma_f16(const uint16_t* aHalves, const uint16_t* bHalves, const float* c16x16, float* d16x16, int32_t depth)
{
    NtcHipContext* const ctx = g_default;
    CTX_ENTER(ctx);
    if (!aHalves || !bHalves || !c16x16 || !d16x16) { set_error("ntc_hip_selftest_mfma_f16: null pointer."); return NTC_HIP_ERR_INVALID_ARG; }
    if (depth != 16 && depth != 32) { set_error("ntc_hip_selftest_mfma_f16: depth must be 16 or 32."); return NTC_HIP_ERR_INVALID_ARG; }
    size_t const operandBytes = size_t(16) * size_t(depth) * 2;
    uint8_t* dev = nullptr;
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&dev), 4096));
    uint16_t* a = reinterpret_cast<uint16_t*>(dev);
    uint16_t* b = reinterpret_cast<uint16_t*>(dev + 1024);
    float* c = reinterpret_cast<float*>(dev + 2048);
    float* d = reinterpret_cast<float*>(dev + 3072);
    hipError_t e = hipMemcpy(a, aHalves, operandBytes, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(b, bHalves, operandBytes, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(c, c16x16, 1024, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = launch_selftest_mfma_f16(a, b, c, d, depth, L.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(L.stream);
    if (e == hipSuccess) e = hipMemcpy(d16x16, d, 1024, hipMemcpyDeviceToHost);
    (void)hipFree(dev);
    HIP_TRY(e);
    return 0;
}

// ---- the same entry points on the context ntc_hip_init created
int ntc_hip_device_info(char* name, size_t nameSize, int* computeUnits) { return ntc_hip_ctx_device_info(g_default, name, nameSize, computeUnits); }
int ntc_hip_device_clock(int* clockRateKHz) { return ntc_hip_ctx_device_clock(g_default, clockRateKHz); }
int ntc_hip_alloc(void** devPtr, size_t bytes) { return ntc_hip_ctx_alloc(g_default, devPtr, bytes); }
int ntc_hip_free(void* devPtr) { return ntc_hip_ctx_free(g_default, devPtr); }
int ntc_hip_upload(void* dst, const void* src, size_t bytes) { return ntc_hip_ctx_upload(g_default, dst, src, bytes); }
int ntc_hip_download(void* dst, const void* src, size_t bytes) { return ntc_hip_ctx_download(g_default, dst, src, bytes); }
int ntc_hip_memset(void* dst, int value, size_t bytes) { return ntc_hip_ctx_memset(g_default, dst, value, bytes); }
int ntc_hip_synchronize(void) { return ntc_hip_ctx_synchronize(g_default); }
int ntc_hip_decode(const NtcHipTextureSet* sets, int32_t numSets) { return ntc_hip_ctx_decode(g_default, sets, numSets); }
int ntc_hip_decode_static(const NtcHipTextureSet* sets, int32_t numSets) { return ntc_hip_ctx_decode_static(g_default, sets, numSets); }
int ntc_hip_timer_begin(void) { return ntc_hip_ctx_timer_begin(g_default); }
int ntc_hip_timer_end(float* outMilliseconds) { return ntc_hip_ctx_timer_end(g_default, outMilliseconds); }
int ntc_hip_decode_timed(const NtcHipTextureSet* sets, int32_t numSets, int32_t iterations, float* outMs) { return ntc_hip_ctx_decode_timed(g_default, sets, numSets, iterations, outMs); }
int ntc_hip_build_query_latents(const NtcHipTextureSet* set, void* dst, uint64_t dstBytes) { return ntc_hip_ctx_build_query_latents(g_default, set, dst, dstBytes); }
int ntc_hip_decode_queries(const NtcHipTextureSet* set, const NtcHipQuery* queries, uint64_t numQueries, void* out, uint64_t outBytes) { return ntc_hip_ctx_decode_queries(g_default, set, queries, numQueries, out, outBytes); }
int ntc_hip_decode_queries_timed(const NtcHipTextureSet* set, const NtcHipQuery* queries, uint64_t numQueries, void* out, uint64_t outBytes, int32_t iterations, float* outMillisecondsPerIteration) { return ntc_hip_ctx_decode_queries_timed(g_default, set, queries, numQueries, out, outBytes, iterations, outMillisecondsPerIteration); }
int ntc_hip_read_channels(const NtcHipReadChannels* p) { return ntc_hip_ctx_read_channels(g_default, p); }
int ntc_hip_write_channels(const NtcHipWriteChannels* p) { return ntc_hip_ctx_write_channels(g_default, p); }
int ntc_hip_image_loss(void* decoded, const void* reference, uint64_t planarBytes, int32_t width, int32_t height, int32_t setChannels, uint32_t validChannelMask, int32_t maskChannelIndex, int32_t discardMaskedOutPixels, float* outMse) { return ntc_hip_ctx_image_loss(g_default, decoded, reference, planarBytes, width, height, setChannels, validChannelMask, maskChannelIndex, discardMaskedOutPixels, outMse); }
int ntc_hip_resize_planar(const void* src, uint64_t srcBytes, int32_t srcWidth, int32_t srcHeight, void* dst, uint64_t dstBytes, int32_t dstWidth, int32_t dstHeight, int32_t setChannels, const uint8_t* channelColorSpaces) { return ntc_hip_ctx_resize_planar(g_default, src, srcBytes, srcWidth, srcHeight, dst, dstBytes, dstWidth, dstHeight, setChannels, channelColorSpaces); }
int ntc_hip_image_difference(const NtcHipImageDifference* p) { return ntc_hip_ctx_image_difference(g_default, p); }
int ntc_hip_block_compress(const NtcHipBlockCompress* p) { return ntc_hip_ctx_block_compress(g_default, p); }

} // extern "C"
