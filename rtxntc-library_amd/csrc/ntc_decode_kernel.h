// ntc_decode_kernel.h - what the host side of the library knows about the device code.
#pragma once
#include <hip/hip_runtime_api.h>
#include <stdint.h>

namespace ntc_hip_dev {

enum {
    NTC_HIP_DEV_OUT_FP16_PLANAR_PAIRS = 0,
    NTC_HIP_DEV_OUT_FP16_PIXELS = 1,
    NTC_HIP_DEV_OUT_UNORM8_PIXELS = 2
};

// Compiled decoder variants (geometry is a template parameter of the kernel).
enum {
    NTC_HIP_VARIANT_NONE = -1,
    NTC_HIP_VARIANT_CFG01 = 0,  // HR 2x2 concat of 8 x 2-bit, LR bilinear 16 x 4-bit, IN 64, 64-48-32
    NTC_HIP_VARIANT_CFG2,       // HR 2x2 concat of 8 x 2-bit, LR bilinear 12 x 4-bit, IN 64, 48-48-32
    NTC_HIP_VARIANT_REF16,      // LibNTC 0.9.2: both grids bilinear 4-bit, (lod,lod), IN 48, 64-48-32
    NTC_HIP_VARIANT_REF12,
    NTC_HIP_VARIANT_REF8,
    NTC_HIP_VARIANT_REF4,
    NTC_HIP_VARIANT_CFG3_FP8,   // both grids bilinear 16 x 4-bit, (lod,lod), IN 48, 64-64-64, e4m3 hidden-layer weights
    // LibNTC 0.9.2 geometry with the FP8 version of the network (GenericFP8 blob): ntc_decode_fp8_kernel.hip
    NTC_HIP_VARIANT_REF16_FP8,
    NTC_HIP_VARIANT_REF12_FP8,
    NTC_HIP_VARIANT_REF8_FP8,
    NTC_HIP_VARIANT_REF4_FP8,
    NTC_HIP_VARIANT_COUNT
};
inline bool variant_is_fp8_network(int variant) { return variant >= NTC_HIP_VARIANT_REF16_FP8 && variant <= NTC_HIP_VARIANT_REF4_FP8; }

// One colour mip of one texture set, as the kernel sees it.  Entries are sorted by
// tileStart; a workgroup tile covers 64 x 4 texels.
struct DevMip {
    uint16_t const* hr;        // first u16 layer of the high-res grid
    uint16_t const* lr;
    uint8_t*        out;       // start of this mip in the output
    uint8_t const*  weights;   // weight blob of the set this mip belongs to
    uint64_t outRowPitch;
    int32_t width, height;
    int32_t hrWidth, hrHeight, lrWidth, lrHeight;
    float   positionScale, positionLod;
    int32_t outPixelStride, numChannels, outFormat;
    int32_t tileStart, tilesX, tilesY;
    // All-integer input stage, valid when `fast` is set (every size a power of two, positionScale
    // a power of two).  An axis word packs, for p = u*grid - 1/2 = N / 2^n with
    // N = ((2x+1) << shl) - (1 << sublog):  shl | n << 8 | sublog << 16 | log2(grid size) << 24.
    uint32_t fast;
    uint32_t hrAxisX, hrAxisY, lrAxisX, lrAxisY;
    uint32_t posMask;          // (texels per period of the positional encoding) - 1
    // The two grids once more in query order (bricks of 4 x 4 or 8 x 8 cells, all layers of a cell
    // together), or null; read by the query kernel only.
    uint8_t const* hrBricks;
    uint8_t const* lrBricks;
};

// Brick geometry of a grid with `layers` u16 layers: log2 of the brick's side in cells.
constexpr int brick_side_log2(int layers) { return layers == 1 ? 3 : 2; }
constexpr int brick_bytes(int layers) { return (1 << (2 * brick_side_log2(layers))) * layers * 2; }
hipError_t launch_build_bricks(uint16_t const* src, uint8_t* dst, int width, int height, int layers, hipStream_t stream);

// One random-access query (same layout as NtcHipQuery of the C ABI).
struct DevQuery { float u, v; int32_t mip; };

constexpr int kTileWidth = 64, kTileHeight = 4;

// ChannelFormat values of the reference (include/libntc/ntc.h:227-236)
enum {
    NTC_HIP_DEV_FORMAT_UNORM8 = 1, NTC_HIP_DEV_FORMAT_UNORM16 = 2, NTC_HIP_DEV_FORMAT_FLOAT16 = 3,
    NTC_HIP_DEV_FORMAT_FLOAT32 = 4, NTC_HIP_DEV_FORMAT_UINT32 = 5
};

struct ReadChannelsArgs {
    uint16_t const* planarPairs;   // start of the mip in the internal fp16 layout
    uint8_t* dst;
    uint64_t pixelStride, rowPitch;
    int32_t width, height, setChannels, firstChannel, numChannels, dstChannels, format;
    int32_t useDithering;
    int32_t vectorBytes;           // widest store every pixel start is aligned to: 16, 8, 4, 2 or 1
    int32_t xShift;                // set by the launcher: log2 of the pixels of a row one workgroup covers
    int32_t dstWidth, dstHeight;   // size of the user image when it differs from the mip's (resampling copy), else 0
    uint8_t srcColorSpaces[16], dstColorSpaces[16];   // per copied channel: 0 linear, 1 sRGB, 2 HLG
};
hipError_t launch_read_channels(ReadChannelsArgs const& args, hipStream_t stream);

constexpr int NTC_HIP_DEV_MAX_CHANNELS = 16;

struct WriteChannelsArgs {
    uint8_t const* src;
    uint16_t* planarPairs;
    uint64_t pixelStride, rowPitch;
    int32_t width, height, setChannels, firstChannel, numChannels, format, verticalFlip;
    int32_t vectorBytes;           // widest load every pixel start is aligned to
    int32_t xShift;                // set by the launcher
    int32_t srcWidth, srcHeight;   // size of the user image when it differs from the mip's (resampling copy), else 0
    uint8_t srcColorSpaces[16], dstColorSpaces[16];
};
hipError_t launch_write_channels(WriteChannelsArgs const& args, hipStream_t stream);

// Grid of the loss kernel: a workgroup (= one row of 16 double partial sums) covers 64 lanes x 1 or 2
// texels (2 when the width is even) by 4 waves x kLossRowsPerWave rows.
constexpr int kLossRowsPerWave = 8;
inline dim3 image_loss_grid(int width, int height)
{
    int const perLane = (width & 1) ? 1 : 2;
    return dim3((width + 64 * perLane - 1) / (64 * perLane), (height + 4 * kLossRowsPerWave - 1) / (4 * kLossRowsPerWave));
}
inline size_t image_loss_blocks(int width, int height)
{
    dim3 const grid = image_loss_grid(width, height);
    return size_t(grid.x) * size_t(grid.y);
}
hipError_t launch_image_loss(uint16_t* a, uint16_t const* b, int width, int height, int setChannels,
                             uint32_t validChannelMask, int maskChannel, int discardMaskedOut, double* partials, hipStream_t stream);

hipError_t launch_resize_planar(uint16_t const* src, int srcWidth, int srcHeight, uint16_t* dst, int dstWidth, int dstHeight,
                                int setChannels, uint8_t const* colorSpaces, hipStream_t stream);

struct DiffImageArgs {
    uint8_t const* data;
    uint64_t pixelStride, rowPitch;
    int32_t format, numChannels;
};
struct ImageDifferenceArgs {
    DiffImageArgs a, b;
    int32_t left, top, width, height;
    float alphaThreshold;
    int32_t useAlphaThreshold, useMSLE;
    unsigned long long* output;    // four 16.48 fixed-point accumulators
};
hipError_t launch_image_difference(ImageDifferenceArgs const& args, hipStream_t stream);

struct BlockCompressArgs {
    uint8_t const* src;
    uint8_t* dst;
    uint64_t pixelStride, rowPitch, dstRowPitch;
    int32_t srcWidth, srcHeight, format, numChannels;
    int32_t srcLeft, srcTop, widthInBlocks, heightInBlocks, dstOffsetX, dstOffsetY;
    float alphaThreshold;       // BC1: texels with alpha <= threshold are transparent
    // BC7: 9-bit (mode, partition) entries of a modeMapWidthInBlocks x modeMapHeightInBlocks map, or null
    uint32_t const* modeBuffer;
    int32_t modeMapWidthInBlocks, modeMapHeightInBlocks, modeMapOffsetX, modeMapOffsetY;
    int32_t packedRgba8;        // source = four UNORM8 channels, every pixel 4-byte aligned
};
// Sets `bytes` bytes at dst to `value` (any alignment).
hipError_t launch_fill(uint8_t* dst, uint8_t value, uint64_t bytes, hipStream_t stream);
hipError_t launch_block_compress(BlockCompressArgs const& args, int dstFormat /* 1..7 */, hipStream_t stream);
hipError_t launch_bc6_compress(BlockCompressArgs const& args, hipStream_t stream);
hipError_t launch_bc7_compress(BlockCompressArgs const& args, hipStream_t stream);

hipError_t launch_decode(int variant, DevMip const* mips, int numMips, int totalTiles, int gridSize, hipStream_t stream);
hipError_t launch_queries(int variant, DevMip const* mips, int numMips, DevQuery const* queries, uint64_t numQueries,
                          uint16_t* out, int gridSize, hipStream_t stream);
// The FP8 network is launched twice (weights of one plane per layer, then any weights); `word` is a dword of device
// memory through which the first launch tells the second whether any set is left for it, `serial` a number the
// caller changes with every pair of launches that shares the word.
struct Fp8Handoff { uint32_t* word; uint32_t serial; };
hipError_t launch_decode_fp8(int variant, DevMip const* mips, int numMips, int totalTiles, int gridSize, Fp8Handoff handoff, hipStream_t stream);
int resident_fp8_workgroups_per_cu();
int fp8_tiles_per_round();               // tiles a workgroup of decode_fp8_kernel works on at a time
int fp8_threads_per_workgroup();
hipError_t launch_queries_fp8(int variant, DevMip const* mips, int numMips, DevQuery const* queries, uint64_t numQueries,
                              uint16_t* out, int gridSize, Fp8Handoff handoff, hipStream_t stream);
hipError_t launch_selftest_fp8_activation(uint16_t const* in, uint16_t* out, int n, hipStream_t stream);
int resident_workgroups_per_cu(int variant);
int tiles_per_round(int variant);      // tiles a workgroup of the variant's decode kernel works on at a time
int threads_per_workgroup(int variant);
hipError_t launch_selftest_mfma(int8_t const* a, int8_t const* b, int32_t* d, hipStream_t stream);
hipError_t launch_selftest_mfma_f16(uint16_t const* a, uint16_t const* b, float const* c, float* d, int depth, hipStream_t stream);

} // namespace ntc_hip_dev
