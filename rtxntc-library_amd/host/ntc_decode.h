// ntc_decode.h - additions of the MI355X build of libntc to LibNTC's public interface.
//
// The library itself implements LibNTC's own header: it is compiled against the unmodified
// <libntc/ntc.h> of the LibNTC tree it is dropped into (-I<LibNTC>/include), its classes derive from
// the IContext / ITextureSet / ITextureSetMetadata / ITextureMetadata / IStream declared THERE, and it
// exports the free functions declared there.  An application built against LibNTC's header links
// against this libntc.so unchanged and never needs this file.
//
// What LibNTC's interface has no way to express is declared here, in namespace ntc::amd:
//   * raw latents and weights without an NTC file, and the decoder geometries of the benchmark
//     configurations (ITextureSetExtension);
//   * the image-difference and block-compression passes run on the device instead of being handed to
//     a graphics API as shader bytecode, and texture sets without a device for host-side tests
//     (IContextExtension);
//   * the host weight quantiser.
// An extension interface is reached from the LibNTC object with GetTextureSetExtension /
// GetContextExtension and lives exactly as long as that object.
#pragma once

#include <libntc/ntc.h>

namespace ntc
{
namespace amd
{

// Decoder families beyond the one compiled into LibNTC 0.9.2 (the reference changes decoders by editing
// InferenceConstants.h, README.md:32-36).
enum class DecoderPreset
{
    LibNTC092 = 0,      // both grids bilinear 4-bit, shared neural LODs, (lod, lod) inputs, MLP 48-64-48-32-16
    Concat2x2_64 = 1,   // per-mip grids: HR (W/2) 2x2-concat of 8 x 2-bit, LR (W/4) bilinear 16 x 4-bit, MLP 64-64-48-32-16
    Concat2x2_48 = 2    // same grids with 12 LR features, MLP 64-48-48-32-16
};

class ITextureSetExtension
{
public:
    virtual Status SetDecoderPreset(DecoderPreset preset) = 0;
    // Size in bytes of the latent buffer / Int8 weight blob / FP8 weight blob the current shape expects.
    virtual uint64_t GetLatentDataSize() const = 0;
    virtual uint64_t GetWeightDataSize() const = 0;
    virtual uint64_t GetFP8WeightDataSize() const = 0;
    // Latent grids exactly as stored in an NTC file (u16 layers, neural LOD after neural LOD) and the
    // GenericInt8 weight blob of src/WeightLayout.cpp:42-49.  Host memory.
    virtual Status SetLatentData(void const* data, size_t size) = 0;
    virtual Status SetWeightData(void const* data, size_t size) = 0;
    // The GenericFP8 weight blob of src/WeightLayout.cpp:51-71 (what ITextureSet::Decompress uses when
    // useInt8Weights is false); LibNTC092 preset only.  Host memory.
    virtual Status SetFP8WeightData(void const* data, size_t size) = 0;
protected:
    ~ITextureSetExtension() = default;
};

// One image of ComputeImageDifference / CompressBlocks: pitch-linear pixels of 1..4 channels (R, G, B, A)
// in device memory; channels a pixel does not store read as 0, 0, 0, 1.
struct ImageDesc
{
    unsigned char const* pData = nullptr;
    size_t dataSize = 0;
    int width = 0;
    int height = 0;
    size_t pixelStride = 0;
    size_t rowPitch = 0;
    ChannelFormat channelFormat = ChannelFormat::UNKNOWN;
    int numChannels = 4;
};

// The fields of MakeImageDifferenceComputePassParameters (include/libntc/ntc.h:1103-1121) plus what a
// graphics application binds to that pass: the two images and the output buffer.
struct ImageDifferenceParameters
{
    ImageDesc imageA, imageB;
    Rect extent;                        // compared in both images
    bool useAlphaThreshold = false;     // ignore colour differences where both alphas are below the threshold
    float alphaThreshold = 1.f / 255.f;
    bool useMSLE = false;               // mean squared log error of |values| instead of mean squared error
    void* pOutputBuffer = nullptr;      // device memory, cleared by the caller: four uint64 in 16.48 fixed point are ADDED
    size_t outputBufferSize = 0;
    uint32_t outputOffset = 0;          // bytes, multiple of 8
};

// The fields of MakeBlockCompressionComputePassParameters (include/libntc/ntc.h:1050-1100) that BC1 ..
// BC7 use, plus what a graphics application binds to that pass: the source image and the destination.
struct BlockCompressionParameters
{
    ImageDesc srcImage;                 // device memory
    Rect srcRect;                       // pixels to compress; width and height are rounded up to whole blocks
    Point dstOffsetInBlocks;
    BlockCompressedFormat dstFormat = BlockCompressedFormat::None;      // BC1 .. BC7
    float alphaThreshold = 1.f / 255.f; // BC1: pixels with alpha at or below it may become transparent
    void* pDstData = nullptr;           // device memory: rows of 8-byte (BC1, BC4) or 16-byte (all others) blocks
    size_t dstDataSize = 0;
    size_t dstRowPitch = 0;             // bytes per row of blocks
    // BC7 with a mode buffer (the reference's modeBufferSource == Custom): device memory holding
    // MakeBC7ModeBuffer's output for a map of modeMapWidthInBlocks x modeMapHeightInBlocks blocks; the block
    // (x, y) of srcRect uses the map entry (x + modeMapOffsetInBlocks.x, y + modeMapOffsetInBlocks.y).
    // Only the recorded mode and partition of each block are encoded then.  Null: every mode is tried.
    void const* pModeBuffer = nullptr;
    size_t modeBufferSize = 0;
    uint64_t modeBufferByteOffset = 0;  // multiple of 4
    Point modeMapOffsetInBlocks;
    int modeMapWidthInBlocks = 0;
    int modeMapHeightInBlocks = 0;
};

class IContextExtension
{
public:
    // Runs the image-difference pass that IContext::MakeImageDifferenceComputePass describes for a
    // graphics API (include/libntc/ntc.h:1227-1239, src/Context.cpp:781-860, src/shaders/ImageDifference.hlsl)
    // on the device, asynchronously; DecodeImageDifferenceResult converts the four results.
    virtual Status ComputeImageDifference(ImageDifferenceParameters const& params) const = 0;
    // Runs the block-compression pass that IContext::MakeBlockCompressionComputePass describes for a
    // graphics API (include/libntc/ntc.h:1213-1225, src/Context.cpp:630-779, src/shaders/CompressBC1.hlsl ..
    // CompressBC7.hlsl) on the device, asynchronously.  All seven formats; BC6 is the unsigned variant.
    virtual Status CompressBlocks(BlockCompressionParameters const& params) const = 0;
    // True when a gfx950 device was initialised for this context.
    virtual bool IsDeviceAvailable() const = 0;
    // Every context queues its device work (Decompress without statistics, ReadChannels into device memory, the two
    // passes above) on a stream of its own and returns.  Synchronize waits for all of it: call it before other
    // code - another context, the application's own streams - touches the memory that work reads or writes.
    virtual Status Synchronize() const = 0;
    // IContext::CreateTextureSet and CreateCompressedTextureSetFrom* refuse to work without a device, as the
    // reference's do (src/Context.cpp:187-191,311-315).  After AllowTextureSetsWithoutDevice(true) they create
    // the set regardless: everything that needs no device (shapes, sizes, validation, metadata, file parsing)
    // works, device work fails with CudaUnavailable.  For host-side tests; CreateContext switches it on by
    // itself when the environment variable LIBNTC_ALLOW_TEXTURE_SETS_WITHOUT_DEVICE is set.
    virtual void AllowTextureSetsWithoutDevice(bool allow) const = 0;
protected:
    ~IContextExtension() = default;
};

// One layer of a float MLP: weights[out][in] row-major, bias[out].
struct FloatLayerDesc
{
    int inputChannels = 0;
    int outputChannels = 0;
    float const* weights = nullptr;
    float const* bias = nullptr;
};
// Maps an output channel from the network's range to linear values: v * scale + bias
// (optimalToLinearScale / Bias of src/ChannelInfo.h, folded into the output layer by the quantiser).
struct OutputChannelTransform { float scale = 1.f; float bias = 0.f; };

extern "C" {
// Null when the object was not created by this library.
NTC_API ITextureSetExtension* GetTextureSetExtension(ITextureSetMetadata* textureSet);
NTC_API IContextExtension* GetContextExtension(IContext* context);

// Quantises a four-layer float MLP into the GenericInt8 weight blob (src/WeightLayout.cpp:42-49) as the
// reference's encoder does (cuda::QuantizeNetwork, src/Quantizer.cu:88-208,266-283), on the host.
// pOutSize (optional) receives the blob size; outputTransforms (optional) holds one entry per output channel.
NTC_API Status QuantizeNetworkInt8(FloatLayerDesc const* layers, int numLayers, OutputChannelTransform const* outputTransforms,
    void* pOutBlob, size_t blobSize, size_t* pOutSize);
// The same network as the GenericFP8 blob (src/WeightLayout.cpp:51-71): e4m3 weights and fp16 biases
// for the hidden layers (src/Quantizer.cu:210-252), the Int8 output layer.
NTC_API Status QuantizeNetworkFP8(FloatLayerDesc const* layers, int numLayers, OutputChannelTransform const* outputTransforms,
    void* pOutBlob, size_t blobSize, size_t* pOutSize);
// IEEE half bits -> OCP e4m3 byte: round to nearest even, saturating at +-448, NaN -> 0x7F | sign.
NTC_API uint8_t HalfToE4M3(uint16_t halfBits);
}

} // namespace amd
} // namespace ntc
