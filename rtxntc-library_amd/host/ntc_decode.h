// ntc_decode.h - C++ host interface of the MI355X texture-set decoder.
//
// It mirrors the part of LibNTC's public interface that the decompression path uses
// (reference include/libntc/ntc.h): the same names in namespace ntc, the same argument meaning,
// the same status codes and error-message convention, so code written against LibNTC's
//   CreateContext -> IContext::CreateCompressedTextureSetFromFile (or CreateTextureSet +
//   ITextureSet::LoadFromFile) -> ITextureSet::Decompress -> ITextureSet::ReadChannels
// sequence reads the same here.  Compression, saving files and graphics-API interop are not part
// of this library; the interface below simply does not declare them.
//
// Everything device-side goes through the C ABI of include/ntc_hip.h; this layer never
// includes a HIP header.
#pragma once

#include <cstddef>
#include <cstdint>

namespace ntc
{

// Same value as the reference's InterfaceVersion (include/libntc/ntc.h:40): applications pass
// it in ContextParameters and CreateContext rejects a mismatch (src/PublicFunctions.cpp:66-71).
constexpr uint32_t InterfaceVersion = 0x25121500;

// Numeric values follow include/libntc/ntc.h:53-74.
enum class Status
{
    Ok = 0, InterfaceMismatch = 1, CudaError = 2, CudaUnavailable = 3, FileUnavailable = 4,
    FileUnrecognized = 5, FileIncompatible = 6, Incomplete = 7, Unsupported = 8, InternalError = 9,
    InvalidArgument = 10, InvalidData = 11, InvalidState = 12, IOError = 13, NotImplemented = 14,
    OutOfMemory = 15, OutOfRange = 16, ShaderUnavailable = 17, UnknownError = 18
};

// include/libntc/ntc.h:227-236
enum class ChannelFormat { UNKNOWN = 0, UNORM8 = 1, UNORM16 = 2, FLOAT16 = 3, FLOAT32 = 4, UINT32 = 5 };
// include/libntc/ntc.h:238-256
enum class BlockCompressedFormat { None = 0, BC1 = 1, BC2 = 2, BC3 = 3, BC4 = 4, BC5 = 5, BC6 = 6, BC7 = 7 };
enum class ColorSpace { Linear = 0, sRGB = 1, HLG = 2 };

// include/libntc/ntc.h:285-293, 367-371
enum class InferenceWeightType { Unknown = 0, GenericInt8 = 1, GenericFP8 = 2, CoopVecFP8 = 3, Count };
enum class CompressionType { None = 0, GDeflate = 1 };
// Where a buffer lies in a stream such as an NTC file and how it is stored (include/libntc/ntc.h:116-122,373-387).
struct StreamRange { uint64_t offset = 0; uint64_t size = 0; };
struct BufferFootprint
{
    StreamRange rangeInStream;
    CompressionType compressionType = CompressionType::None;
    uint64_t uncompressedSize = 0;      // equals rangeInStream.size when not compressed
    uint32_t uncompressedCrc32 = 0;     // 0 = none recorded
};
struct LatentTextureFootprint
{
    BufferFootprint buffer;
    int width = 0;
    int height = 0;
    size_t rowPitch = 0;                // bytes
};

// What a shader (or any other kernel) that decodes single texels of a set needs besides the latents and the
// weight blob (include/libntc/shaders/InferenceConstants.h:43-85, include/libntc/ntc.h:359-365).
struct NtcColorMipConstants
{
    int neuralMip;          // latent image of the colour mip, counted from firstLatentMipInTexture
    float positionLod;
    float positionScale;
    int pad;
};
struct NtcTextureSetConstants
{
    NtcColorMipConstants colorMips[16];
    int networkWeightOffsets[4];
    int networkBiasOffsets[4];
    int networkScaleOffsets[4];
    int imageWidth;
    int imageHeight;
    int imageMips;
    int pad0;
    unsigned int validChannelMask;
    unsigned int channelColorSpaces;    // 2 bits per channel
    int pad1;
    int pad2;
};
struct InferenceData { NtcTextureSetConstants constants; };

// include/libntc/ntc.h:43-51
struct VersionInfo
{
    int major;
    int minor;
    int point;
    char const* branch;
    char const* commitHash;
};

// Source of one output channel in ITextureSet::ShuffleInferenceOutputs (include/libntc/ntc.h:459-517).
enum class ShuffleSourceType
{
    Undefined,   // the channel outputs zero and is not counted as valid
    Channel,     // the channel outputs what channel `channelIndex` used to output
    Constant     // the channel outputs `constantValue` and counts as valid
};
struct ShuffleSource
{
    ShuffleSourceType type = ShuffleSourceType::Undefined;
    union { int channelIndex; float constantValue; };
    ShuffleSource() : channelIndex(0) {}
    int GetChannelIndex() const { return type == ShuffleSourceType::Channel ? channelIndex : -1; }
    static ShuffleSource Undefined() { return ShuffleSource(); }
    static ShuffleSource Channel(int index) { ShuffleSource s; s.type = ShuffleSourceType::Channel; s.channelIndex = index; return s; }
    static ShuffleSource Constant(float value) { ShuffleSource s; s.type = ShuffleSourceType::Constant; s.constantValue = value; return s; }
};

// include/libntc/ntc.h:272-276
enum class AddressSpace { Host, Device };
enum class TextureDataPage { Reference, Output };
// Application-provided or library-provided byte streams (include/libntc/ntc.h:91-114).
class IStream
{
public:
    virtual bool Read(void* dst, size_t size) = 0;          // false on error or a short read
    virtual bool Write(const void* src, size_t size) = 0;
    virtual bool Seek(uint64_t offset) = 0;                 // from the beginning of the stream
    virtual uint64_t Tell() = 0;
    virtual uint64_t Size() = 0;
    virtual ~IStream() = default;
};

constexpr int DisableCudaDevice = -1;          // ContextParameters::cudaDevice: do not touch the GPU

// include/libntc/ntc.h:131-156
struct LatentShape
{
    int gridSizeScale = 4;
    int numFeatures = 16;
    bool operator==(LatentShape const& o) const { return gridSizeScale == o.gridSizeScale && numFeatures == o.numFeatures; }
    bool operator!=(LatentShape const& o) const { return !(*this == o); }
    static constexpr LatentShape Empty() { return LatentShape{ 0, 0 }; }
    bool IsEmpty() const { return *this == Empty(); }
};

// include/libntc/ntc.h:158-177
struct TextureSetDesc
{
    int width = 0;
    int height = 0;
    int channels = 0;
    int mips = 1;
};

// include/libntc/ntc.h:179-199 (the fields the decode path reads)
struct TextureSetFeatures
{
    int stagingBytesPerPixel = 4;   // staging buffer for ReadChannels into host memory; 0 = none
    int stagingWidth = 0;           // 0 = texture-set width
    int stagingHeight = 0;
    bool enableCompression = false; // accepted for source compatibility; compression is not available
    bool separateRefOutData = false;
};

// include/libntc/ntc.h:645-687
struct WriteChannelsParameters
{
    int mipLevel = 0;
    int firstChannel = 0;
    int numChannels = 0;
    unsigned char const* pData = nullptr;
    AddressSpace addressSpace = AddressSpace::Host;
    int width = 0;
    int height = 0;
    size_t pixelStride = 0;
    size_t rowPitch = 0;
    ChannelFormat channelFormat = ChannelFormat::UNKNOWN;
    ColorSpace const* srcColorSpaces = nullptr;   // per written channel; null = all linear
    ColorSpace const* dstColorSpaces = nullptr;   // storage colour spaces, recorded with the set; null = all linear
    bool verticalFlip = false;
};

// include/libntc/ntc.h:689-730
struct ReadChannelsParameters
{
    TextureDataPage page = TextureDataPage::Output;
    int mipLevel = 0;
    int firstChannel = 0;
    int numChannels = 0;
    unsigned char* pOutData = nullptr;
    AddressSpace addressSpace = AddressSpace::Host;
    int width = 0;
    int height = 0;
    size_t pixelStride = 0;
    size_t rowPitch = 0;
    ChannelFormat channelFormat = ChannelFormat::UNKNOWN;
    ColorSpace const* dstColorSpaces = nullptr;   // per read channel; null = all linear
    bool useDithering = false;                    // +-1/2 step of hash noise on UNORM outputs
};

// include/libntc/ntc.h:810-816.  Losses are mean squared errors against the image written with
// WriteChannels, over the channels that textures claim (GetValidChannelMask); with no texture
// registered they stay zero, as in the reference (src/Inference.cu:119-136, src/TextureSet.cpp:1833).
struct DecompressionStats
{
    float perChannelLoss[16];
    float perMipLoss[16];
    float overallLoss = 0;
    float gpuTimeMilliseconds = 0;
};

// include/libntc/ntc.h:1278-1305 (graphics-API fields left out)
// A custom CPU memory allocator (include/libntc/ntc.h:76-87).
class IAllocator
{
public:
    virtual void* Allocate(size_t size) = 0;
    virtual void Deallocate(void* ptr, size_t size) = 0;    // size: what Allocate was asked for
    virtual ~IAllocator() = default;
};

struct ContextParameters
{
    uint32_t interfaceVersion = InterfaceVersion;
    // Optional (include/libntc/ntc.h:1284-1287): where the context, its texture sets, texture metadata and
    // stream objects live; null = the C runtime's heap.  Must outlive the context.  Buffers inside those
    // objects (names, host copies of weights and mode maps) come from the C++ runtime either way.
    IAllocator* pAllocator = nullptr;
    int cudaDevice = 0;             // index of the HIP device; the name is kept for source compatibility
};

// include/libntc/ntc.h (Rect): a rectangle of pixels.
struct Rect { int left = 0; int top = 0; int width = 0; int height = 0; };

// The latent grids seen as one texture: width x height of the finest grid, one array layer per four
// features, one mip level per neural LOD (include/libntc/ntc.h:519-528).
struct LatentTextureDesc { int width = 0; int height = 0; int arraySize = 0; int mipLevels = 0; };

// One image of IContext::ComputeImageDifference: pitch-linear pixels of 1..4 channels (R, G, B, A) in
// device memory; channels a pixel does not store read as 0, 0, 0, 1.
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
struct Point { int x = 0; int y = 0; };
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

// Decoder families beyond the one compiled into LibNTC 0.9.2, selected with
// ITextureSet::SetDecoderPreset (an addition; the reference changes decoders by editing
// InferenceConstants.h, README.md:32-36).
enum class DecoderPreset
{
    LibNTC092 = 0,      // both grids bilinear 4-bit, shared neural LODs, (lod, lod) inputs, MLP 48-64-48-32-16
    Concat2x2_64 = 1,   // per-mip grids: HR (W/2) 2x2-concat of 8 x 2-bit, LR (W/4) bilinear 16 x 4-bit, MLP 64-64-48-32-16
    Concat2x2_48 = 2    // same grids with 12 LR features, MLP 64-48-48-32-16
};

// The slice of include/libntc/ntc.h:385-455 that decides which channels hold image data.
class ITextureMetadata
{
public:
    virtual void SetName(char const* name) = 0;
    virtual char const* GetName() const = 0;
    // Assigns the texture's channels inside the set; OutOfRange unless the range lies inside the
    // set's channels (src/TextureMetadata.cpp:48-69).
    virtual Status SetChannels(int firstChannel, int numChannels) = 0;
    virtual void GetChannels(int& outFirstChannel, int& outNumChannels) const = 0;
    virtual int GetFirstChannel() const = 0;
    virtual int GetNumChannels() const = 0;
    // Stored with the texture and read back from NTC files; the decoder itself does not use them.
    virtual void SetChannelFormat(ChannelFormat format) = 0;
    virtual ChannelFormat GetChannelFormat() const = 0;
    virtual void SetBlockCompressedFormat(BlockCompressedFormat format) = 0;
    virtual BlockCompressedFormat GetBlockCompressedFormat() const = 0;
    virtual void SetRgbColorSpace(ColorSpace colorSpace) = 0;
    virtual ColorSpace GetRgbColorSpace() const = 0;
    virtual void SetAlphaColorSpace(ColorSpace colorSpace) = 0;
    virtual ColorSpace GetAlphaColorSpace() const = 0;
    // BC7 acceleration data of one colour mip (include/libntc/ntc.h:437-453, src/TextureMetadata.cpp:96-223):
    // MakeAndStoreBC7ModeBuffer extracts mode and partition of every block of a BC7-compressed mip (host
    // memory; the block grid must be the mip's) and keeps them with the texture; GetBC7ModeBuffer returns the
    // stored map (host memory, null / 0 when there is none) - upload it and pass it to
    // IContext::CompressBlocks as pModeBuffer.  Maps stored uncompressed in an NTC file are loaded with the
    // file; GetBC7ModeBufferFootprint says where a mip's map lies in the file and how it is stored (a
    // GDeflate-compressed one is not loaded: GetBC7ModeBuffer then returns nothing).
    virtual Status MakeAndStoreBC7ModeBuffer(int mipLevel, int widthInBlocks, int heightInBlocks,
        void const* blockData, size_t blockDataSize, size_t rowPitch) = 0;
    virtual void GetBC7ModeBuffer(int mipLevel, void const** outData, size_t* outSize) const = 0;
    virtual BufferFootprint GetBC7ModeBufferFootprint(int mipLevel) const = 0;
    virtual ~ITextureMetadata() = default;
};

class ITextureSet
{
public:
    virtual TextureSetDesc const& GetDesc() const = 0;
    virtual LatentShape const& GetLatentShape() const = 0;

    // include/libntc/ntc.h:551-568
    virtual ITextureMetadata* AddTexture() = 0;
    virtual Status RemoveTexture(ITextureMetadata* texture) = 0;
    virtual void ClearTextureMetadata() = 0;
    virtual int GetTextureCount() const = 0;
    virtual ITextureMetadata* GetTexture(int textureIndex) = 0;

    // Changes the latent shape; all compressed data is lost (include/libntc/ntc.h:858-861).
    // Range rules follow src/TextureSetMetadata.cpp:1137-1159.
    virtual Status SetLatentShape(LatentShape const& newShape) = 0;

    // Loads latents, the Int8 MLP and texture metadata from an NTC file whose dimensions match
    // this set (include/libntc/ntc.h:871-889, src/TextureSet.cpp:154-294,718-800).  Views stored
    // with GDeflate compression are refused with Status::Unsupported.
    virtual Status LoadFromStream(IStream* stream) = 0;
    virtual Status LoadFromMemory(void const* pData, size_t size) = 0;
    virtual Status LoadFromFile(char const* fileName) = 0;
    // Storage colour space of a channel as recorded in the file (include/libntc/ntc.h:592-595).
    virtual ColorSpace GetChannelStorageColorSpace(int channel) const = 0;

    // Which colour mips share latent grids (include/libntc/ntc.h:572-591, src/TextureSetMetadata.cpp:109-228).
    // Meaningful for the LibNTC 0.9.2 geometry, where a neural LOD serves several colour mips; with the
    // other decoder presets every colour mip owns its grids and these return zeros / Status::Unsupported.
    virtual LatentTextureDesc GetLatentTextureDesc() const = 0;
    virtual int GetNumLatentImages() const = 0;
    // Where one layer (four features) of one latent image lies in the file the set was loaded from, and its
    // size (include/libntc/ntc.h:530-537,577-581, src/TextureSetMetadata.cpp:119-144): for callers that stream
    // latent layers themselves.  OutOfRange for indices outside the set; the footprint is empty (size 0) when
    // the set was not loaded from a file.
    virtual Status GetLatentTextureFootprint(int latentMipLevel, int arrayLayer, LatentTextureFootprint& outFootprint) const = 0;
    // The range of colour mips decoded from the same latent image as mipLevel.
    virtual Status GetFusedMipLevels(int mipLevel, int* pOutFirstFusedMip, int* pOutLastFusedMip) const = 0;
    // The range of colour mips whose high-resolution grid is latent image latentImageIndex.
    virtual Status GetMipLevelsForLatentImage(int latentImageIndex, int* pOutFirstColorMip, int* pOutLastColorMip) const = 0;
    virtual bool IsInferenceWeightTypeSupported(InferenceWeightType weightType) const = 0;
    // Accepted for source compatibility; has no effect (include/libntc/ntc.h:942-944).
    virtual void SetExperimentalKnob(float value) = 0;

    // --- additions: raw latents and weights without a file ---
    virtual Status SetDecoderPreset(DecoderPreset preset) = 0;
    // Size in bytes of the latent buffer / weight blob the current shape expects.
    virtual uint64_t GetLatentDataSize() const = 0;
    virtual uint64_t GetWeightDataSize() const = 0;
    // Latent grids exactly as stored in an NTC file (u16 layers, neural LOD after neural LOD)
    // and the GenericInt8 weight blob of src/WeightLayout.cpp:42-49.  Host memory.
    virtual Status SetLatentData(void const* data, size_t size) = 0;
    virtual Status SetWeightData(void const* data, size_t size) = 0;

    // Decompresses into the internal representation; ReadChannels extracts it
    // (include/libntc/ntc.h:929-933, src/TextureSet.cpp:1664-1897).  useInt8Weights is accepted
    // and ignored: the int8 weights are the only weights.
    virtual Status Decompress(DecompressionStats* pOutStats, bool useInt8Weights = false) = 0;

    // Stores a reference image (include/libntc/ntc.h:899, src/TextureSet.cpp:829-913): the data
    // Decompress measures its loss against.
    virtual Status WriteChannels(WriteChannelsParameters const& params) = 0;

    // include/libntc/ntc.h:902, src/TextureSet.cpp:915-985.  As in WriteChannels, an image whose size
    // differs from the mip's is resampled bilinearly (src/ImageProcessing.cu:24-72).
    virtual Status ReadChannels(ReadChannelsParameters const& params) = 0;

    // Fills mips 1.. of the reference page from mip 0 with a 2x2 box filter (include/libntc/ntc.h:910-912,
    // src/TextureSet.cpp:1121-1142).
    virtual Status GenerateMips() = 0;

    // Index of the channel that holds an alpha mask; negative = none (include/libntc/ntc.h:936-940,
    // src/TextureSet.cpp:1899-1907).  Decompress then clamps the decoded mask channel to [0, 1] when
    // it compares against a reference (valid channel mask != 0), and with discardMaskedOutPixels texels
    // whose reference mask is zero count in the loss of the mask channel only.  OutOfRange for an
    // index at or beyond the channel count.
    virtual Status SetMaskChannelIndex(int index, bool discardMaskedOutPixels) = 0;

    // The weight blob an application uploads for inference in its own shaders (include/libntc/ntc.h:596-605,
    // src/TextureSetMetadata.cpp:245-286): host memory owned by the set, valid until the weights
    // change.  Only InferenceWeightType::GenericInt8 exists here (others: Status::Unsupported);
    // *pOutConvertedSize is 0.
    virtual InferenceWeightType GetBestSupportedWeightType() const = 0;
    virtual Status GetInferenceWeights(InferenceWeightType weightType, void const** pOutData, size_t* pOutSize,
        size_t* pOutConvertedSize) = 0;

    // Rearranges the rows of the output layer in the weights GetInferenceWeights returns
    // (include/libntc/ntc.h:620-636, src/TextureSetMetadata.cpp:305-432): afterwards output `ch` is what
    // output mapping[ch].channelIndex used to be, a constant (zero weights, scale 2^-16, bias
    // round(c * 2^16)), or zero.  Storage colour spaces and the valid channel mask follow the mapping.
    // As in the reference, Decompress keeps using the weights as loaded; `mapping` has 16 entries.
    virtual Status ShuffleInferenceOutputs(ShuffleSource mapping[16]) = 0;

    // Union of the channel ranges of the registered textures, carried through the shuffle mapping;
    // constant outputs count as valid (include/libntc/ntc.h:638-640, src/TextureSetMetadata.cpp:807-832).
    virtual uint32_t GetValidChannelMask() const = 0;

    virtual ~ITextureSet() = default;
};

class IContext
{
public:
    // include/libntc/ntc.h:1149, src/Context.cpp:235-261
    virtual Status CreateTextureSet(TextureSetDesc const& desc, TextureSetFeatures const& features,
        ITextureSet** pOutTextureSet) const = 0;
    // include/libntc/ntc.h:1153
    virtual void DestroyTextureSet(ITextureSet* textureSet) const = 0;
    // Streams over files and memory (include/libntc/ntc.h:1127-1145, src/Context.cpp:80-176).
    virtual Status OpenFile(char const* fileName, bool write, IStream** pOutStream) const = 0;
    virtual void CloseFile(IStream* stream) const = 0;
    virtual Status OpenMemory(void* pData, size_t size, IStream** pOutStream) const = 0;
    virtual Status OpenReadOnlyMemory(void const* pData, size_t size, IStream** pOutStream) const = 0;
    virtual void CloseMemory(IStream* stream) const = 0;
    // Reads what an NTC file says about a set - descriptor, latent shape, textures, colour spaces, the Int8 weights
    // (GetInferenceWeights, MakeInferenceData), BC7 mode maps and where every latent layer lies in the file
    // (GetLatentTextureFootprint) - without reading the latents and without a device
    // (include/libntc/ntc.h:1158-1163, src/Context.cpp:263-293).  Latent layers stored with GDeflate are fine here:
    // their footprints say so.  Device work on the returned object fails with CudaUnavailable / InvalidState.
    virtual Status CreateTextureSetMetadataFromStream(IStream* inputStream, ITextureSet** pOutMetadata) const = 0;
    virtual void DestroyTextureSetMetadata(ITextureSet* textureSetMetadata) const = 0;
    // Creates a texture set with the dimensions found in an NTC file and loads it
    // (include/libntc/ntc.h:1166-1177, src/Context.cpp:296-376).
    virtual Status CreateCompressedTextureSetFromStream(IStream* inputStream, TextureSetFeatures const& features,
        ITextureSet** pOutTextureSet) const = 0;
    virtual Status CreateCompressedTextureSetFromMemory(void const* pData, size_t size, TextureSetFeatures const& features,
        ITextureSet** pOutTextureSet) const = 0;
    virtual Status CreateCompressedTextureSetFromFile(char const* fileName, TextureSetFeatures const& features,
        ITextureSet** pOutTextureSet) const = 0;
    // Runs the image-difference pass that IContext::MakeImageDifferenceComputePass describes for a
    // graphics API (include/libntc/ntc.h:1227-1239, src/Context.cpp:781-860, src/shaders/ImageDifference.hlsl)
    // on the device, asynchronously; DecodeImageDifferenceResult converts the four results.
    virtual Status ComputeImageDifference(ImageDifferenceParameters const& params) const = 0;
    // Runs the block-compression pass that IContext::MakeBlockCompressionComputePass describes for a
    // graphics API (include/libntc/ntc.h:1213-1225, src/Context.cpp:630-779, src/shaders/CompressBC1.hlsl ..
    // CompressBC7.hlsl) on the device, asynchronously.  All seven formats; BC6 is the unsigned variant.
    virtual Status CompressBlocks(BlockCompressionParameters const& params) const = 0;
    // Fills the constants for decoding single texels of a set outside this library (include/libntc/ntc.h:1251-1255,
    // src/Context.cpp:864-922): per colour mip the latent image and the position constants, the offsets of
    // every layer's weights, scales and biases in the blob GetInferenceWeights returns, the image size, the
    // valid-channel mask and the packed storage colour spaces.  Sets with shared latent images only.
    virtual Status MakeInferenceData(ITextureSet* textureSet, InferenceWeightType weightType, int firstLatentMipInTexture,
        InferenceData* pOutInferenceData) const = 0;
    // True when a gfx950 device was initialised (reference: IsCudaAvailable).
    virtual bool IsCudaAvailable() const = 0;
    virtual ~IContext() = default;
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
// An addition: quantises a four-layer float MLP into the GenericInt8 weight blob
// (src/WeightLayout.cpp:42-49) as the reference's encoder does (cuda::QuantizeNetwork,
// src/Quantizer.cu:88-208,266-283), on the host.  pOutSize (optional) receives the blob size;
// outputTransforms (optional) holds one entry per output channel.
Status QuantizeNetworkInt8(FloatLayerDesc const* layers, int numLayers, OutputChannelTransform const* outputTransforms,
    void* pOutBlob, size_t blobSize, size_t* pOutSize);
// The same network as the GenericFP8 blob (src/WeightLayout.cpp:51-71): e4m3 weights and fp16 biases
// for the hidden layers (src/Quantizer.cu:210-252), the Int8 output layer.  The decoder of this
// library does not consume that blob; it is what LibNTC stores as the second MLP version of a file.
Status QuantizeNetworkFP8(FloatLayerDesc const* layers, int numLayers, OutputChannelTransform const* outputTransforms,
    void* pOutBlob, size_t blobSize, size_t* pOutSize);
// IEEE half bits -> OCP e4m3 byte: round to nearest even, saturating at +-448, NaN -> 0x7F | sign.
uint8_t HalfToE4M3(uint16_t halfBits);

// include/libntc/ntc.h:1307-1331.  CreateContext returns CudaUnavailable together with a usable
// context when no device can be used (src/PublicFunctions.cpp:161).
uint32_t GetInterfaceVersion();
Status CreateContext(IContext** pOutContext, ContextParameters const& params);
void DestroyContext(IContext* context);
char const* GetLastErrorMessage();
char const* StatusToString(Status status);
char const* ChannelFormatToString(ChannelFormat format);
char const* BlockCompressedFormatToString(BlockCompressedFormat format);
char const* ColorSpaceToString(ColorSpace colorSpace);
char const* InferenceWeightTypeToString(InferenceWeightType weightType);
char const* CompressionTypeToString(CompressionType type);
size_t GetBytesPerPixelComponent(ChannelFormat format);
float LossToPSNR(float loss);

// include/libntc/ntc.h:1312-1313, 1352-1391 (src/PublicFunctions.cpp:36-45,354-557).
VersionInfo GetLibraryVersion();
// Size of the compressed data of a set: latent grids plus the Int8 network, without file headers.
Status EstimateCompressedTextureSetSize(TextureSetDesc const& textureSetDesc, LatentShape const& latentShape, size_t& outSize);
int GetKnownLatentShapeCount();
Status EnumerateKnownLatentShapes(int index, float& outBitsPerPixel, LatentShape& outShape);
// The known shape nearest to the requested bit rate within 25 %, else OutOfRange.
Status PickLatentShape(float requestedBitsPerPixel, float& outBitsPerPixel, LatentShape& outShape);
float GetLatentShapeBitsPerPixel(LatentShape const& shape);
// 16.48 fixed-point result of an image-difference pass -> mean squared error.
double DecodeImageDifferenceResult(uint64_t value);
size_t GetBC7ModeBufferSize(int widthInBlocks, int heightInBlocks);
Status MakeBC7ModeBuffer(int widthInBlocks, int heightInBlocks, void const* blockData, size_t blockDataSize,
    size_t rowPitch, void* modeBuffer, size_t modeBufferSize);
// Always 0: GDeflate-compressed views are not supported.
size_t GetGDeflateHeaderSize(size_t uncompressedSize);
}

} // namespace ntc
