// NtcHost.cpp - libntc.so: LibNTC's public interface (the unmodified <libntc/ntc.h> of the LibNTC tree,
// included through ntc_decode.h) implemented over the gfx950 decoder.
//
// Counterpart of the parts of reference src/Context.cpp, src/TextureSet.cpp,
// src/FeatureGridHost.cpp, src/FeatureGridMath.cpp and src/Errors.cpp that the decompression
// path goes through, src/TextureSetMetadata.cpp for loading NTC files and src/Stream.cpp.  The classes
// here derive from LibNTC's own IContext / ITextureSet (: virtual ITextureSetMetadata) / ITextureMetadata /
// IStream, so their vtables are the ones an application compiled against that header expects; entry points
// outside the decompression path (compression, saving files, graphics-API passes, shared textures) have
// bodies that set the error message and return Status::NotImplemented or Unsupported.
// All device work is done by libntc_hip.so through include/ntc_hip.h.
#include "ntc_decode.h"
#include "NtcFile.h"
#include "../../include/ntc_hip.h"

#include <algorithm>
#include <cerrno>
#include <cinttypes>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <new>
#include <string>
#include <utility>
#include <vector>

namespace ntc
{
using amd::DecoderPreset;
using amd::ImageDesc;
using amd::ImageDifferenceParameters;
using amd::BlockCompressionParameters;

// ---- errors: a thread-local message buffer, set on failure and cleared on success
// (src/Errors.cpp:21-52) -------------------------------------------------------------------
namespace
{
thread_local char t_message[1024] = "";

void SetErrorMessage(char const* fmt, ...)
{
    va_list args;
    va_start(args, fmt);
    vsnprintf(t_message, sizeof t_message, fmt, args);
    va_end(args);
}
void ClearErrorMessage() { t_message[0] = 0; }

// A failed C-ABI call: keep its message, classify it.
Status DeviceFailure(int code)
{
    SetErrorMessage("%s", ntc_hip_last_error());
    if (code > 0) return Status::CudaError;                  // a HIP runtime error
    switch (code) {
    case NTC_HIP_ERR_UNSUPPORTED: return Status::Unsupported;
    case NTC_HIP_ERR_NO_DEVICE:
    case NTC_HIP_ERR_NOT_INITIALIZED: return Status::CudaUnavailable;
    default: return Status::InvalidArgument;
    }
}

// Entry points of LibNTC's interface that lie outside the decompression path.
Status NotPartOfThisLibrary(char const* function, char const* what)
{
    SetErrorMessage("%s: %s is not part of this build of LibNTC (MI355X decompression path only).", function, what);
    return Status::NotImplemented;
}

enum class NetworkState { Empty, Initialized, Complete };
char const* NetworkStateToString(NetworkState s)
{
    switch (s) {
    case NetworkState::Empty: return "Empty";
    case NetworkState::Initialized: return "Initialized";
    case NetworkState::Complete: return "Complete";
    }
    return "Invalid";
}

NtcHipDecoderSpec MakeSpec(DecoderPreset preset, int numFeatures)
{
    NtcHipDecoderSpec s{};
    s.posEncWaves = 3;
    s.outputChannels = 16;
    s.weightType = NTC_HIP_WEIGHTS_INT8;
    if (preset == DecoderPreset::LibNTC092) {
        // include/libntc/shaders/InferenceConstants.h:26-40
        s.hrFeatures = s.lrFeatures = numFeatures;
        s.hrBits = s.lrBits = 4;
        s.hrMode = s.lrMode = NTC_HIP_GRID_BILINEAR;
        s.hrFeatureSlots = s.lrFeatureSlots = 16;
        s.lodInputs = 2;
        s.inputChannels = 48;
        s.hiddenChannels[0] = 64; s.hiddenChannels[1] = 48; s.hiddenChannels[2] = 32;
    } else {
        bool const wide = preset == DecoderPreset::Concat2x2_64;
        s.hrFeatures = 8; s.hrBits = 2; s.hrMode = NTC_HIP_GRID_CONCAT2X2; s.hrFeatureSlots = 8;
        s.lrFeatures = wide ? 16 : 12; s.lrBits = 4; s.lrMode = NTC_HIP_GRID_BILINEAR; s.lrFeatureSlots = s.lrFeatures;
        s.lodInputs = 0;
        s.inputChannels = 64;
        s.hiddenChannels[0] = wide ? 64 : 48; s.hiddenChannels[1] = 48; s.hiddenChannels[2] = 32;
    }
    return s;
}

// Neural-LOD geometry, src/FeatureGridMath.cpp:47-77.
int SharedMipCount(int gridSizeScale) { static int const table[] = { 2, 3, 3, 3, 4, 4 }; return table[gridSizeScale - 1]; }
int LodToNeuralLod(int lod, int gridSizeScale, int neuralLods) { return std::max(0, std::min((lod - SharedMipCount(gridSizeScale) + 2) & ~1, neuralLods - 2)); }
int GridDimension(int imageDimension, int neuralLod, int gridSizeScale) { return std::max((imageDimension / gridSizeScale) >> neuralLod, 1); }
int NeuralLodCount(int width, int height, int mips, int gridSizeScale)      // with src/FeatureGridHost.cpp:27-58
{
    int const minGrid = int(float(std::min(width, height)) / float(gridSizeScale));
    int const byGridSize = std::max(2, int(1.f + std::floor(std::log2(float(minGrid))))) & ~1;
    return std::min(byGridSize, LodToNeuralLod(mips - 1, gridSizeScale, 8) + 2);
}

// src/Stream.cpp:27-121
class FileStream final : public IStream
{
public:
    explicit FileStream(FILE* file) : m_file(file) {}
    ~FileStream() override { if (m_file) std::fclose(m_file); }
    bool Read(void* dst, size_t size) override { return size == 0 || std::fread(dst, size, 1, m_file) == 1; }
    bool Write(const void* src, size_t size) override { return size == 0 || std::fwrite(src, size, 1, m_file) == 1; }
    bool Seek(uint64_t offset) override { return fseeko(m_file, off_t(offset), SEEK_SET) == 0; }
    uint64_t Tell() override { return uint64_t(ftello(m_file)); }
    uint64_t Size() override
    {
        off_t const current = ftello(m_file);
        fseeko(m_file, 0, SEEK_END);
        off_t const size = ftello(m_file);
        fseeko(m_file, current, SEEK_SET);
        return uint64_t(size);
    }
private:
    FILE* m_file;
};

class MemoryStream final : public IStream
{
public:
    MemoryStream(uint8_t* data, size_t size, bool readonly) : m_data(data), m_size(size), m_readonly(readonly) {}
    bool Read(void* dst, size_t size) override
    {
        if (size > m_size - m_at) return false;
        std::memcpy(dst, m_data + m_at, size);
        m_at += size;
        return true;
    }
    bool Write(const void* src, size_t size) override
    {
        if (m_readonly || size > m_size - m_at) return false;
        std::memcpy(m_data + m_at, src, size);
        m_at += size;
        return true;
    }
    bool Seek(uint64_t offset) override { if (offset >= m_size) return false; m_at = size_t(offset); return true; }
    uint64_t Tell() override { return m_at; }
    uint64_t Size() override { return m_size; }
private:
    uint8_t* m_data;
    size_t m_size, m_at = 0;
    bool m_readonly;
};

// positionScale / positionLod of a colour mip, src/TextureSet.cpp:456-461
void PositionConstants(NtcHipMipDesc& d)
{
    float const widthScale = float(d.hrWidth) / float(d.width);
    float const heightScale = float(d.hrHeight) / float(d.height);
    d.positionScale = 0.5f * std::max(widthScale, heightScale);
    d.positionLod = std::max(-1.f, std::min(1.f, 0.25f * log2f(d.positionScale)));
}
} // namespace

// For the other translation units of this library.
void SetQuantizeError(char const* fmt, ...)
{
    va_list args;
    va_start(args, fmt);
    vsnprintf(t_message, sizeof t_message, fmt, args);
    va_end(args);
}

class Context;

// Public objects are constructed in memory from the context's allocator and destroyed through it
// (src/Context.cpp:201-233,263-293, src/PublicFunctions.cpp:46-60,164-172).
class DefaultAllocator final : public IAllocator
{
public:
    void* Allocate(size_t size) override { return std::malloc(size); }
    void Deallocate(void* ptr, size_t) override { std::free(ptr); }
};
DefaultAllocator g_defaultAllocator;

template <class T, class... Args> T* MakeObject(IAllocator* allocator, Args&&... args)
{
    void* const memory = allocator->Allocate(sizeof(T));
    return memory ? new (memory) T(std::forward<Args>(args)...) : nullptr;
}
template <class T> void DestroyObject(IAllocator* allocator, T* object)      // T: the object's own (final) class
{
    if (!object) return;
    object->~T();
    allocator->Deallocate(object, sizeof(T));
}

// src/TextureMetadata.cpp:30-75 (name and channel range only)
class TextureMetadata final : public ITextureMetadata
{
public:
    explicit TextureMetadata(TextureSetDesc const& setDesc) : m_setDesc(setDesc) {}
    void SetName(char const* name) override { m_name = name ? name : ""; }
    char const* GetName() const override { return m_name.c_str(); }
    Status SetChannels(int firstChannel, int numChannels) override
    {
        if (firstChannel < 0 || firstChannel >= m_setDesc.channels) {
            SetErrorMessage("firstChannel (%d) must be between 0 and %d.", firstChannel, m_setDesc.channels - 1);
            return Status::OutOfRange;
        }
        if (numChannels < 1 || numChannels + firstChannel > m_setDesc.channels) {
            SetErrorMessage("For the provided firstChannel (%d), numChannels (%d) must be between 1 and %d.",
                firstChannel, numChannels, m_setDesc.channels - firstChannel);
            return Status::OutOfRange;
        }
        m_firstChannel = firstChannel; m_numChannels = numChannels;
        return Status::Ok;
    }
    void GetChannels(int& outFirstChannel, int& outNumChannels) const override { outFirstChannel = m_firstChannel; outNumChannels = m_numChannels; }
    int GetFirstChannel() const override { return m_firstChannel; }
    int GetNumChannels() const override { return m_numChannels; }
    void SetChannelFormat(ChannelFormat format) override { m_channelFormat = format; }
    ChannelFormat GetChannelFormat() const override { return m_channelFormat; }
    void SetBlockCompressedFormat(BlockCompressedFormat format) override { m_bcFormat = format; }
    BlockCompressedFormat GetBlockCompressedFormat() const override { return m_bcFormat; }
    void SetRgbColorSpace(ColorSpace colorSpace) override { m_rgbColorSpace = colorSpace; }
    ColorSpace GetRgbColorSpace() const override { return m_rgbColorSpace; }
    void SetAlphaColorSpace(ColorSpace colorSpace) override { m_alphaColorSpace = colorSpace; }
    ColorSpace GetAlphaColorSpace() const override { return m_alphaColorSpace; }

    // src/TextureMetadata.cpp:96-135
    Status MakeAndStoreBC7ModeBuffer(int mipLevel, int widthInBlocks, int heightInBlocks,
        void const* blockData, size_t blockDataSize, size_t rowPitch) override
    {
        if (mipLevel < 0 || mipLevel >= m_setDesc.mips) {
            SetErrorMessage("mipLevel (%d) must be between 0 and %d.", mipLevel, m_setDesc.mips - 1);
            return Status::OutOfRange;
        }
        int const mipWidthInBlocks = (std::max(1, m_setDesc.width >> mipLevel) + 3) / 4;
        int const mipHeightInBlocks = (std::max(1, m_setDesc.height >> mipLevel) + 3) / 4;
        if (widthInBlocks != mipWidthInBlocks || heightInBlocks != mipHeightInBlocks) {
            SetErrorMessage("Provided widthInBlocks (%d) and heightInBlocks (%d) do not match the expected "
                "dimensions (%d x %d) for mip level %d.", widthInBlocks, heightInBlocks, mipWidthInBlocks, mipHeightInBlocks, mipLevel);
            return Status::InvalidArgument;
        }
        ModeBuffer& buffer = m_modeBuffers[size_t(mipLevel)];
        buffer = ModeBuffer();
        buffer.data.assign(GetBC7ModeBufferSize(mipWidthInBlocks, mipHeightInBlocks), 0);
        Status const status = MakeBC7ModeBuffer(widthInBlocks, heightInBlocks, blockData, blockDataSize, rowPitch, buffer.data.data(), buffer.data.size());
        if (status != Status::Ok) { buffer.data.clear(); return status; }
        ClearErrorMessage();
        return Status::Ok;
    }
    void GetBC7ModeBuffer(int mipLevel, void const** outData, size_t* outSize) const override
    {
        if (outData) *outData = nullptr;
        if (outSize) *outSize = 0;
        if (mipLevel < 0 || mipLevel >= NTC_HIP_MAX_MIPS || m_modeBuffers[size_t(mipLevel)].data.empty()) return;
        if (outData) *outData = m_modeBuffers[size_t(mipLevel)].data.data();
        if (outSize) *outSize = m_modeBuffers[size_t(mipLevel)].data.size();
    }
    BufferFootprint GetBC7ModeBufferFootprint(int mipLevel) const override
    {
        return (mipLevel < 0 || mipLevel >= NTC_HIP_MAX_MIPS) ? BufferFootprint() : m_modeBuffers[size_t(mipLevel)].footprint;
    }
    // Used by the file loader: where the file keeps the map of a mip, and the map itself once read.
    void SetBC7ModeBufferFromFile(int mipLevel, BufferFootprint const& footprint, std::vector<uint8_t>&& data)
    {
        if (mipLevel < 0 || mipLevel >= NTC_HIP_MAX_MIPS) return;
        m_modeBuffers[size_t(mipLevel)].footprint = footprint;
        m_modeBuffers[size_t(mipLevel)].data = std::move(data);
    }
private:
    struct ModeBuffer { std::vector<uint8_t> data; BufferFootprint footprint; };
    ModeBuffer m_modeBuffers[NTC_HIP_MAX_MIPS];
    TextureSetDesc const& m_setDesc;
    std::string m_name;
    int m_firstChannel = 0, m_numChannels = 0;
    ChannelFormat m_channelFormat = ChannelFormat::UNORM8;
    BlockCompressedFormat m_bcFormat = BlockCompressedFormat::None;
    ColorSpace m_rgbColorSpace = ColorSpace::Linear, m_alphaColorSpace = ColorSpace::Linear;
};

// Header + JSON chunk of an NTC file (src/TextureSetMetadata.cpp:1210-1264).
Status LoadFileHeadersFromStream(IStream* stream, file::Document& document, uint64_t& binaryChunkOffset, uint64_t& binaryChunkSize)
{
    unsigned char raw[40];
    if (!stream->Read(raw, sizeof raw)) {
        SetErrorMessage("Failed to read the file header - file smaller than %zu bytes?", sizeof raw);
        return Status::IOError;
    }
    file::Header const header = file::DecodeHeader(raw);
    if (header.signature != file::kSignature) { SetErrorMessage("Unrecognized file format."); return Status::FileUnrecognized; }
    if (header.version != file::kContainerVersion) {
        SetErrorMessage("Incompatible file format version: expected %d, got %d.", int(file::kContainerVersion), int(header.version));
        return Status::FileUnrecognized;
    }
    uint64_t const streamSize = stream->Size();
    uint64_t const expected = std::max(header.jsonChunkOffset + header.jsonChunkSize, header.binaryChunkOffset + header.binaryChunkSize);
    bool const wraps = header.jsonChunkOffset + header.jsonChunkSize < header.jsonChunkOffset
                    || header.binaryChunkOffset + header.binaryChunkSize < header.binaryChunkOffset;
    if (streamSize < expected) {
        SetErrorMessage("File incomplete: expected at least %" PRIu64 " bytes, actual size %" PRIu64 " bytes.", expected, streamSize);
        return Status::FileUnrecognized;
    }
    if (wraps) {        // a sum that wrapped slips through the test above (the reference then allocates a chunk of that size)
        SetErrorMessage("File header describes a chunk that reaches past the 64-bit offset range.");
        return Status::FileUnrecognized;
    }
    if (!stream->Seek(header.jsonChunkOffset)) return Status::IOError;
    std::vector<char> json(size_t(header.jsonChunkSize) + 1, 0);
    if (!stream->Read(json.data(), size_t(header.jsonChunkSize))) return Status::IOError;
    std::string error;
    if (!file::ParseDocument(json.data(), std::strlen(json.data()), document, error)) {
        SetErrorMessage("%s", error.c_str());
        return Status::FileUnrecognized;
    }
    binaryChunkOffset = header.binaryChunkOffset;
    binaryChunkSize = header.binaryChunkSize;
    return Status::Ok;
}

Status ValidateLatentShape(LatentShape const& shape)        // src/TextureSetMetadata.cpp:1137-1159
{
    if (shape.IsEmpty()) return Status::Ok;
    if (shape.numFeatures <= 0 || shape.numFeatures > 16 || (shape.numFeatures % 4) != 0) {
        SetErrorMessage("Invalid LatentShape: numFeatures (%d) must be a positive multiple of %d up to %d.", shape.numFeatures, 4, 16);
        return Status::OutOfRange;
    }
    if (shape.gridSizeScale < 1 || shape.gridSizeScale > 6) {
        SetErrorMessage("Invalid LatentShape: gridSizeScale (%d) must be between 1 and 6.", shape.gridSizeScale);
        return Status::OutOfRange;
    }
    return Status::Ok;
}

Status ValidateTextureSetDesc(TextureSetDesc const& desc)   // src/TextureSetMetadata.cpp:1161-1178
{
    if (desc.width <= 0 || desc.height <= 0 || desc.channels <= 0 || desc.mips <= 0) {
        SetErrorMessage("Invalid TextureSetDesc: width (%d), height (%d), channels (%d) and mips (%d) "
            "must be positive numbers.", desc.width, desc.height, desc.channels, desc.mips);
        return Status::OutOfRange;
    }
    if (desc.channels > NTC_HIP_MAX_CHANNELS) {
        SetErrorMessage("Invalid TextureSetDesc: too many channels (%d). Only up to %d channels are supported.", desc.channels, NTC_HIP_MAX_CHANNELS);
        return Status::OutOfRange;
    }
    if (desc.mips > NTC_HIP_MAX_MIPS) {
        SetErrorMessage("Invalid TextureSetDesc: too many mips (%d). Only up to %d mips are supported.", desc.mips, NTC_HIP_MAX_MIPS);
        return Status::OutOfRange;
    }
    return Status::Ok;
}

// src/TextureSetMetadata.cpp:1180-1208: the grid size scale is not stored, it follows from the
// size of the first latent image.
Status DeserializeTextureSetDesc(file::Document const& document, TextureSetDesc& desc, LatentShape& shape)
{
    desc.width = int(document.width);
    desc.height = int(document.height);
    desc.channels = int(document.numChannels);
    desc.mips = int(document.numColorMips.value_or(1));
    if (document.latentFeatures.has_value() && !document.latents.empty()) {
        shape.numFeatures = int(*document.latentFeatures);
        file::LatentImage const& first = document.latents[0];
        float const widthRatio = float(desc.width) / float(std::max(first.width, 1u));
        float const heightRatio = float(desc.height) / float(std::max(first.height, 1u));
        shape.gridSizeScale = int(roundf(std::min(widthRatio, heightRatio)));
    } else {
        shape = LatentShape::Empty();
    }
    if (Status st = ValidateTextureSetDesc(desc); st != Status::Ok) return st;
    return ValidateLatentShape(shape);
}

class TextureSet final : public ITextureSet, public amd::ITextureSetExtension
{
public:
    TextureSet(Context const* context, TextureSetDesc const& desc, TextureSetFeatures const& features)
        : m_context(context), m_desc(desc), m_features(features) { ResetShuffle(); }

    ~TextureSet() override
    {
        ClearTextureMetadata();
        ReleaseDevice(m_textureData);
        ReleaseDevice(m_textureDataOut);
        ReleaseDevice(m_staging);
        ReleaseDevice(m_latents);
        ReleaseDevice(m_weights);
        ReleaseDevice(m_weightsFP8);
    }

    // src/TextureSet.cpp:81-152: even channel count, per-mip offsets, texture and staging memory
    Status Initialize(bool deviceAvailable)
    {
        m_deviceAvailable = deviceAvailable;
        m_desc.channels = (m_desc.channels + 1) & ~1;
        uint64_t offset = 0;
        int w = m_desc.width, h = m_desc.height;
        for (int mip = 0; mip < m_desc.mips; ++mip) {
            m_mipOffsets[mip] = offset;
            offset += uint64_t(w) * uint64_t(h);
            w = std::max(1, w >> 1);
            h = std::max(1, h >> 1);
        }
        m_mipOffsets[m_desc.mips] = offset;
        m_textureBytes = offset * uint64_t(m_desc.channels) * 2u;
        int const stagingWidth = m_features.stagingWidth > 0 ? m_features.stagingWidth : m_desc.width;
        int const stagingHeight = m_features.stagingHeight > 0 ? m_features.stagingHeight : m_desc.height;
        m_stagingBytes = uint64_t(stagingWidth) * uint64_t(stagingHeight) * uint64_t(std::max(0, m_features.stagingBytesPerPixel));
        if (m_deviceAvailable) {
            if (int r = ntc_hip_ctx_alloc(Hip(), &m_textureData, m_textureBytes)) return AllocationFailure(r, "texture data", m_textureBytes);
            // A second page keeps the reference image apart from the decoded one (src/TextureSet.cpp:103-124).
            if (m_features.separateRefOutData)
                if (int r = ntc_hip_ctx_alloc(Hip(), &m_textureDataOut, m_textureBytes)) return AllocationFailure(r, "texture data (output)", m_textureBytes);
            if (m_stagingBytes)
                if (int r = ntc_hip_ctx_alloc(Hip(), &m_staging, m_stagingBytes)) return AllocationFailure(r, "staging", m_stagingBytes);
        }
        return Status::Ok;
    }

    TextureSetDesc const& GetDesc() const override { return m_desc; }
    LatentShape const& GetLatentShape() const override { return m_latentShape; }
    ITextureMetadata* AddTexture() override
    {
        TextureMetadata* t = MakeObject<TextureMetadata>(Allocator(), m_desc);
        if (t) m_textures.push_back(t);
        return t;
    }
    Status RemoveTexture(ITextureMetadata* texture) override
    {
        auto it = std::find(m_textures.begin(), m_textures.end(), texture);
        if (it == m_textures.end()) { SetErrorMessage("The texture does not belong to this texture set."); return Status::OutOfRange; }
        DestroyObject(Allocator(), *it);
        m_textures.erase(it);
        return Status::Ok;
    }
    void ClearTextureMetadata() override { for (TextureMetadata* t : m_textures) DestroyObject(Allocator(), t); m_textures.clear(); }
    int GetTextureCount() const override { return int(m_textures.size()); }
    ITextureMetadata* GetTexture(int index) override { return (index >= 0 && index < int(m_textures.size())) ? m_textures[size_t(index)] : nullptr; }
    ITextureMetadata const* GetTexture(int index) const override { return (index >= 0 && index < int(m_textures.size())) ? m_textures[size_t(index)] : nullptr; }

    // ---- outside the decompression path (include/libntc/ntc.h:863-867,873-894,904-908,914-927) ----
    uint64_t GetOutputStreamSize() override { (void)NotPartOfThisLibrary("GetOutputStreamSize", "saving texture sets"); return 0; }
    Status SaveToStream(IStream*, LosslessCompressionStats*) override { return NotPartOfThisLibrary("SaveToStream", "saving texture sets"); }
    Status SaveToMemory(void*, size_t*, LosslessCompressionStats*) override { return NotPartOfThisLibrary("SaveToMemory", "saving texture sets"); }
    Status SaveToFile(char const*, LosslessCompressionStats*) override { return NotPartOfThisLibrary("SaveToFile", "saving texture sets"); }
    Status ConfigureLosslessCompression(LosslessCompressionSettings const&) override { return NotPartOfThisLibrary("ConfigureLosslessCompression", "saving texture sets"); }
    Status WriteChannelsFromTexture(WriteChannelsFromTextureParameters const&) override { return NotPartOfThisLibrary("WriteChannelsFromTexture", "graphics-API texture sharing"); }
    Status ReadChannelsIntoTexture(ReadChannelsIntoTextureParameters const&) override { return NotPartOfThisLibrary("ReadChannelsIntoTexture", "graphics-API texture sharing"); }
    Status BeginCompression(CompressionSettings const&) override { return NotPartOfThisLibrary("BeginCompression", "compression (training)"); }
    Status RunCompressionSteps(CompressionStats*) override { return NotPartOfThisLibrary("RunCompressionSteps", "compression (training)"); }
    Status FinalizeCompression() override { return NotPartOfThisLibrary("FinalizeCompression", "compression (training)"); }
    void AbortCompression() override {}
    // src/TextureSetMetadata.cpp:607-658: the conversion is for cooperative-vector layouts of a graphics device
    Status ConvertInferenceWeights(InferenceWeightType weightType, void* commandList, void* srcBuffer, uint64_t, void* dstBuffer, uint64_t) override
    {
        if (!commandList) { SetErrorMessage("commandList is NULL"); return Status::InvalidArgument; }
        if (!srcBuffer) { SetErrorMessage("srcBuffer is NULL"); return Status::InvalidArgument; }
        if (!dstBuffer) { SetErrorMessage("dstBuffer is NULL"); return Status::InvalidArgument; }
        if (dstBuffer == srcBuffer) { SetErrorMessage("dstBuffer must not be the same as srcBuffer"); return Status::InvalidArgument; }
        if (weightType != InferenceWeightType::CoopVecFP8) {
            SetErrorMessage("Unsupported weightType (%s), must be one of the CoopVec types", InferenceWeightTypeToString(weightType));
            return Status::InvalidArgument;
        }
        SetErrorMessage("The requested conversion operation is not supported by the graphics device or disabled by the context settings.");
        return Status::Unsupported;
    }

    // src/TextureSetMetadata.cpp:807-832 (no output shuffling here)
    // src/TextureSet.cpp:1899-1907
    Status SetMaskChannelIndex(int index, bool discardMaskedOutPixels) override
    {
        if (index >= m_desc.channels) { SetErrorMessage("Mask channel index (%d) must be below the channel count (%d).", index, m_desc.channels); return Status::OutOfRange; }
        m_maskChannelIndex = index;
        m_discardMaskedOutPixels = discardMaskedOutPixels;
        ClearErrorMessage();
        return Status::Ok;
    }

    uint32_t GetValidChannelMask() const override
    {
        uint32_t mask = 0;
        for (TextureMetadata const* t : m_textures) {
            int first, count;
            t->GetChannels(first, count);
            mask |= ((1u << count) - 1u) << first;
        }
        // textures name un-shuffled channels: carry the mask through the mapping
        uint32_t shuffled = 0;
        for (int ch = 0; ch < NTC_HIP_MAX_CHANNELS; ++ch) {
            ShuffleSource const& src = m_shuffle[ch];
            if ((src.type == ShuffleSourceType::Channel && (mask & (1u << src.channelIndex))) || src.type == ShuffleSourceType::Constant)
                shuffled |= 1u << ch;
        }
        return shuffled;
    }

    // src/TextureSetMetadata.cpp:109-228.  m_neuralLodOfMip is filled for the shared-LOD geometry only.
    LatentTextureDesc GetLatentTextureDesc() const override
    {
        LatentTextureDesc desc;
        if (m_numNeuralLods == 0) return desc;
        desc.width = GridDimension(m_desc.width, 0, m_latentShape.gridSizeScale);
        desc.height = GridDimension(m_desc.height, 0, m_latentShape.gridSizeScale);
        desc.arraySize = (m_latentShape.numFeatures + 3) / 4;
        desc.mipLevels = m_numNeuralLods;
        return desc;
    }
    int GetNumLatentImages() const override { return m_numNeuralLods; }

    // src/TextureSetMetadata.cpp:119-144
    Status GetLatentTextureFootprint(int latentMipLevel, int arrayLayer, LatentTextureFootprint& outFootprint) const override
    {
        if (latentMipLevel < 0 || latentMipLevel >= m_numNeuralLods) {
            SetErrorMessage("latentMipLevel (%d) must be between 0 and %d", latentMipLevel, m_numNeuralLods - 1);
            return Status::OutOfRange;
        }
        int const arraySize = (m_latentShape.numFeatures + 3) / 4;
        if (arrayLayer < 0 || arrayLayer >= arraySize) {
            SetErrorMessage("arrayLayer (%d) must be between 0 and %d", arrayLayer, arraySize);
            return Status::OutOfRange;
        }
        outFootprint = LatentTextureFootprint();
        size_t const index = size_t(latentMipLevel) * size_t(arraySize) + size_t(arrayLayer);
        if (index < m_latentFootprints.size()) outFootprint.buffer = m_latentFootprints[index];
        outFootprint.width = GridDimension(m_desc.width, latentMipLevel, m_latentShape.gridSizeScale);
        outFootprint.height = GridDimension(m_desc.height, latentMipLevel, m_latentShape.gridSizeScale);
        outFootprint.rowPitch = size_t(outFootprint.width) * 2u;      // FeatureGridMath::BytesPerLatentPixel
        ClearErrorMessage();
        return Status::Ok;
    }

    Status GetFusedMipLevels(int mipLevel, int* pOutFirstFusedMip, int* pOutLastFusedMip) const override
    {
        if (m_numNeuralLods == 0) { SetErrorMessage("This decoder geometry has no shared latent images."); return Status::Unsupported; }
        if (mipLevel < 0 || mipLevel >= m_desc.mips) {
            SetErrorMessage("mipLevel (%d) must be between 0 and %d", mipLevel, m_desc.mips - 1);
            return Status::OutOfRange;
        }
        int first = mipLevel, last = mipLevel;
        while (first > 0 && m_neuralLodOfMip[first - 1] == m_neuralLodOfMip[mipLevel]) --first;
        while (last + 1 < m_desc.mips && m_neuralLodOfMip[last + 1] == m_neuralLodOfMip[mipLevel]) ++last;
        if (pOutFirstFusedMip) *pOutFirstFusedMip = first;
        if (pOutLastFusedMip) *pOutLastFusedMip = last;
        ClearErrorMessage();
        return Status::Ok;
    }

    Status GetMipLevelsForLatentImage(int latentImageIndex, int* pOutFirstColorMip, int* pOutLastColorMip) const override
    {
        if (latentImageIndex < 0 || latentImageIndex >= m_numNeuralLods) {
            SetErrorMessage("Invalid latentImageIndex (%d), it must be between 0 and %d", latentImageIndex, m_numNeuralLods);
            return m_numNeuralLods == 0 ? Status::Unsupported : Status::OutOfRange;
        }
        int first = -1, last = -1;
        for (int mip = 0; mip < m_desc.mips; ++mip)
            if (m_neuralLodOfMip[mip] == latentImageIndex) { if (first < 0) first = mip; last = mip; }
        if (first < 0) {                                     // the odd LODs are only ever the low-resolution partner
            SetErrorMessage("No color MIPs found that are represented by latent image %d", latentImageIndex);
            return Status::OutOfRange;
        }
        if (pOutFirstColorMip) *pOutFirstColorMip = first;
        if (pOutLastColorMip) *pOutLastColorMip = last;
        ClearErrorMessage();
        return Status::Ok;
    }

    // FillColorMipConstants, GetWeightOffsets, GetPackedColorSpaces (src/TextureSetMetadata.cpp:786-858)
    void FillInferenceConstants(InferenceWeightType weightType, int firstLatentMipInTexture, NtcTextureSetConstants& constants) const
    {
        NtcHipWeightLayout const& layout = weightType == InferenceWeightType::GenericInt8 ? m_weightLayout : m_weightLayoutFP8;
        for (int mip = 0; mip < m_desc.mips; ++mip) {
            NtcColorMipConstants& colorMip = constants.colorMips[mip];
            colorMip.neuralMip = m_neuralLodOfMip[mip] - firstLatentMipInTexture;
            colorMip.positionLod = m_mips[mip].positionLod;
            colorMip.positionScale = m_mips[mip].positionScale;
        }
        for (int layer = 0; layer < NTC_HIP_MLP_LAYERS; ++layer) {
            constants.networkWeightOffsets[layer] = int(layout.weightOffset[layer]);
            constants.networkBiasOffsets[layer] = int(layout.biasOffset[layer]);
            constants.networkScaleOffsets[layer] = int(layout.scaleOffset[layer]);
        }
        constants.imageWidth = m_desc.width;
        constants.imageHeight = m_desc.height;
        constants.imageMips = m_desc.mips;
        constants.validChannelMask = GetValidChannelMask();
        for (int channel = 0; channel < NTC_HIP_MAX_CHANNELS; ++channel)
            constants.channelColorSpaces |= uint32_t(GetChannelStorageColorSpace(channel)) << (2 * channel);
    }

    // src/TextureSetMetadata.cpp:288-303; no cooperative-vector layout exists without a graphics device
    bool IsInferenceWeightTypeSupported(InferenceWeightType weightType) const override
    {
        switch (weightType) {
        case InferenceWeightType::GenericInt8: return !m_hostWeights.empty();
        case InferenceWeightType::GenericFP8: return !m_hostWeightsFP8.empty();
        default: return false;
        }
    }
    void SetExperimentalKnob(float) override {}

    // src/TextureSetMetadata.cpp:233-243: CoopVecFP8 first (never available here), then GenericInt8
    InferenceWeightType GetBestSupportedWeightType() const override
    {
        return m_hostWeights.empty() ? InferenceWeightType::Unknown : InferenceWeightType::GenericInt8;
    }

    // src/TextureSetMetadata.cpp:245-286
    Status GetInferenceWeights(InferenceWeightType weightType, void const** pOutData, size_t* pOutSize, size_t* pOutConvertedSize) override
    {
        if (!IsInferenceWeightTypeSupported(weightType)) {
            SetErrorMessage("No weights available for weightType = %s.", InferenceWeightTypeToString(weightType));
            return Status::Unsupported;
        }
        std::vector<uint8_t> const& blob = weightType == InferenceWeightType::GenericInt8 ? m_hostWeights : m_hostWeightsFP8;
        if (pOutData) *pOutData = blob.data();
        if (pOutSize) *pOutSize = blob.size();
        if (pOutConvertedSize) *pOutConvertedSize = 0;
        ClearErrorMessage();
        return Status::Ok;
    }

    // src/TextureSetMetadata.cpp:305-432
    Status ShuffleInferenceOutputs(ShuffleSource mapping[16]) override
    {
        if (!mapping) { SetErrorMessage("mapping is NULL"); return Status::InvalidArgument; }
        for (int ch = 0; ch < NTC_HIP_MAX_CHANNELS; ++ch) {
            int const type = int(mapping[ch].type);
            if (type < int(ShuffleSourceType::Undefined) || type > int(ShuffleSourceType::Constant)) {
                SetErrorMessage("mapping[%d] has invalid type %d", ch, type);
                return Status::InvalidArgument;
            }
            if (mapping[ch].type == ShuffleSourceType::Channel && (mapping[ch].channelIndex < 0 || mapping[ch].channelIndex >= NTC_HIP_MAX_CHANNELS)) {
                SetErrorMessage("mapping[%d] is using invalid channel %d, must be between 0 and %d", ch, mapping[ch].channelIndex, NTC_HIP_MAX_CHANNELS - 1);
                return Status::OutOfRange;
            }
        }
        // the output layer is int8 with fp32 scale and int32 bias in both blobs (src/TextureSetMetadata.cpp:362-365)
        for (int version = 0; version < 2; ++version) {
            std::vector<uint8_t>& blob = version == 0 ? m_hostWeights : m_hostWeightsFP8;
            NtcHipWeightLayout const& layout = version == 0 ? m_weightLayout : m_weightLayoutFP8;
            if (blob.empty()) continue;
            constexpr int last = NTC_HIP_MLP_LAYERS - 1, outputs = NTC_HIP_MAX_CHANNELS;
            constexpr float constantUnit = 65536.f;          // constants are stored as bias = round(c * 2^16), scale = 2^-16
            int const inputs = m_spec.hiddenChannels[last - 1];
            uint8_t* const weights = blob.data() + layout.weightOffset[last];
            uint8_t* const scales = blob.data() + layout.scaleOffset[last];
            uint8_t* const biases = blob.data() + layout.biasOffset[last];
            std::vector<uint8_t> newWeights(size_t(inputs) * outputs, 0);
            float newScales[outputs];
            int32_t newBiases[outputs];
            for (int row = 0; row < outputs; ++row) {
                ShuffleSource const& src = mapping[row];
                if (src.type == ShuffleSourceType::Channel) {
                    std::memcpy(newWeights.data() + size_t(row) * inputs, weights + size_t(src.channelIndex) * inputs, size_t(inputs));
                    std::memcpy(&newScales[row], scales + 4 * src.channelIndex, 4);
                    std::memcpy(&newBiases[row], biases + 4 * src.channelIndex, 4);
                } else {
                    newScales[row] = 1.f / constantUnit;
                    newBiases[row] = src.type == ShuffleSourceType::Constant ? int32_t(roundf(src.constantValue * constantUnit)) : 0;
                }
            }
            std::memcpy(weights, newWeights.data(), newWeights.size());
            std::memcpy(scales, newScales, sizeof newScales);
            std::memcpy(biases, newBiases, sizeof newBiases);
        }
        ColorSpace newSpaces[NTC_HIP_MAX_CHANNELS];
        ShuffleSource newShuffle[NTC_HIP_MAX_CHANNELS];
        for (int ch = 0; ch < NTC_HIP_MAX_CHANNELS; ++ch) {
            if (mapping[ch].type == ShuffleSourceType::Channel) {
                newSpaces[ch] = m_channelColorSpaces[mapping[ch].channelIndex];
                newShuffle[ch] = m_shuffle[mapping[ch].channelIndex];
            } else {
                newSpaces[ch] = ColorSpace::Linear;
                newShuffle[ch] = mapping[ch];
            }
        }
        std::copy(newSpaces, newSpaces + NTC_HIP_MAX_CHANNELS, m_channelColorSpaces);
        std::copy(newShuffle, newShuffle + NTC_HIP_MAX_CHANNELS, m_shuffle);
        ClearErrorMessage();
        return Status::Ok;
    }

    // src/TextureSet.cpp:718-745
    Status LoadFromStream(IStream* stream) override
    {
        if (!stream) { SetErrorMessage("inputStream is NULL."); return Status::InvalidArgument; }
        file::Document document;
        uint64_t binaryChunkOffset = 0, binaryChunkSize = 0;
        if (Status st = LoadFileHeadersFromStream(stream, document, binaryChunkOffset, binaryChunkSize); st != Status::Ok) return st;
        TextureSetDesc desc;
        LatentShape shape;
        if (Status st = DeserializeTextureSetDesc(document, desc, shape); st != Status::Ok) return st;
        if (desc.width != m_desc.width || desc.height != m_desc.height || desc.channels != m_desc.channels || desc.mips != m_desc.mips) {
            SetErrorMessage("Incompatible texture set in the file - dimensions do not match.");
            return Status::FileIncompatible;
        }
        return LoadFromStreamPostHeader(document, binaryChunkOffset, binaryChunkSize, stream, shape);
    }
    Status LoadFromMemory(void const* pData, size_t size) override
    {
        if (!pData) { SetErrorMessage("pData is NULL."); return Status::InvalidArgument; }
        if (size == 0) { SetErrorMessage("size is 0."); return Status::InvalidArgument; }
        MemoryStream stream(const_cast<uint8_t*>(static_cast<uint8_t const*>(pData)), size, true);
        return LoadFromStream(&stream);
    }
    Status LoadFromFile(char const* fileName) override
    {
        if (!fileName) { SetErrorMessage("fileName is NULL."); return Status::InvalidArgument; }
        FILE* f = std::fopen(fileName, "rb");
        if (!f) { SetErrorMessage("Cannot open file '%s': %s.", fileName, std::strerror(errno)); return Status::FileUnavailable; }
        FileStream stream(f);
        return LoadFromStream(&stream);
    }
    ColorSpace GetChannelStorageColorSpace(int channel) const override
    {
        return (channel >= 0 && channel < NTC_HIP_MAX_CHANNELS) ? m_channelColorSpaces[channel] : ColorSpace::Linear;
    }

    // LoadMetadataFromStream + LoadFromStreamPostHeader + LoadWeightsFromStream
    // (src/TextureSetMetadata.cpp:434-581,676-784, src/TextureSet.cpp:154-294).  Everything is
    // validated and assembled in host memory first; the device is touched last.
    // With metadataOnly the latent layers are described (footprints) but neither read nor uploaded, so GDeflate
    // views are acceptable there, and the weights stay in host memory.
    Status LoadFromStreamPostHeader(file::Document const& document, uint64_t binaryChunkOffset, uint64_t binaryChunkSize,
        IStream* stream, LatentShape const& shape, bool metadataOnly = false)
    {
        ClearTextureMetadata();
        if (shape.IsEmpty()) { SetErrorMessage("The file does not describe a latent shape."); return Status::FileUnrecognized; }

        // MLP versions
        if (document.mlpVersions.empty()) { SetErrorMessage("File doesn't contain MLP information"); return Status::FileUnrecognized; }
        NtcHipDecoderSpec const spec = MakeSpec(DecoderPreset::LibNTC092, shape.numFeatures);
        for (file::Mlp const& mlp : document.mlpVersions)
            if (!ValidateMLP(document, mlp, spec, binaryChunkSize)) return Status::FileUnrecognized;

        // Texture headers
        for (file::Texture const& t : document.textures) {
            ITextureMetadata* texture = AddTexture();
            if (!texture) { SetErrorMessage("Failed to allocate a texture metadata object."); return Status::OutOfMemory; }
            texture->SetName(t.name.c_str());
            (void)texture->SetChannels(int(t.firstChannel), int(t.numChannels));
            texture->SetChannelFormat(ChannelFormat(t.channelFormat.value_or(int(ChannelFormat::UNORM8))));
            texture->SetBlockCompressedFormat(BlockCompressedFormat(t.bcFormat.value_or(0)));
            texture->SetRgbColorSpace(ColorSpace(t.rgbColorSpace.value_or(0)));
            texture->SetAlphaColorSpace(ColorSpace(t.alphaColorSpace.value_or(0)));
            // BC7 mode maps (src/TextureSetMetadata.cpp:470-476, src/TextureMetadata.cpp:151-213); a map stored with
            // GDeflate is described by its footprint but not loaded
            for (file::Texture::ModeBuffer const& ref : t.bcModeBuffers) {
                if (!ValidateBufferView(ref.view, 0, document, binaryChunkSize)) return Status::FileUnrecognized;
                file::BufferView const& view = document.views[ref.view];
                BufferFootprint footprint;
                footprint.rangeInStream = StreamRange{ view.offset + binaryChunkOffset, view.storedSize };
                footprint.compressionType = CompressionType(int(view.compression.value_or(file::Compression::None)));
                footprint.uncompressedSize = view.uncompressedSize.value_or(view.storedSize);
                footprint.uncompressedCrc32 = view.crc32.value_or(0);
                std::vector<uint8_t> data;
                if (footprint.compressionType == CompressionType::None && view.storedSize != 0) {
                    data.resize(size_t(view.storedSize));
                    if (!stream->Seek(footprint.rangeInStream.offset) || !stream->Read(data.data(), data.size())) {
                        SetErrorMessage("Failed to read BC7 mode buffer data of size %llu for mip level %u.",
                            (unsigned long long)view.storedSize, ref.mipLevel);
                        return Status::IOError;
                    }
                }
                static_cast<TextureMetadata*>(texture)->SetBC7ModeBufferFromFile(int(ref.mipLevel), footprint, std::move(data));
            }
        }

        // Channel headers
        std::fill_n(m_channelColorSpaces, NTC_HIP_MAX_CHANNELS, ColorSpace::Linear);
        if (!document.channelColorSpaces.empty()) {
            if (int(document.channelColorSpaces.size()) != m_desc.channels) {
                SetErrorMessage("The file describes %d texture channels while %d are expected", int(document.numChannels), m_desc.channels);
                return Status::FileUnrecognized;
            }
            for (size_t i = 0; i < document.channelColorSpaces.size(); ++i)
                m_channelColorSpaces[i] = ColorSpace(document.channelColorSpaces[i].value_or(0));
        }

        // Latent image headers
        int const numLayers = (shape.numFeatures + 3) / 4;
        for (size_t neuralLod = 0; neuralLod < document.latents.size(); ++neuralLod) {
            file::LatentImage const& image = document.latents[neuralLod];
            uint64_t const layerSize = uint64_t(image.width) * uint64_t(image.height) * 2u;
            if (int(image.layerViews.size()) != numLayers) {
                SetErrorMessage("Expected %d layers, got %d for the latent image in MIP %d", numLayers, int(image.layerViews.size()), int(neuralLod));
                return Status::FileUnrecognized;
            }
            for (uint32_t view : image.layerViews)
                if (!ValidateBufferView(view, layerSize, document, binaryChunkSize)) return Status::FileUnrecognized;
        }

        // Colour mips
        if (int(document.colorMips.size()) > m_desc.mips) {
            SetErrorMessage("The file describes %d color MIP levels while %d are expected", int(document.colorMips.size()), m_desc.mips);
            return Status::FileUnrecognized;
        }
        int fileNeuralLod[NTC_HIP_MAX_MIPS] = {};
        for (size_t mipLevel = 0; mipLevel < document.colorMips.size(); ++mipLevel) {
            file::ColorMip const& colorMip = document.colorMips[mipLevel];
            if (!colorMip.latentMip.has_value()) {
                SetErrorMessage("Color MIP %d doesn't have a mapping to a latent image, which is currently unsupported.", int(mipLevel));
                return Status::FileUnrecognized;
            }
            fileNeuralLod[mipLevel] = int(*colorMip.latentMip);
            if (!colorMip.positionLod.has_value() || !colorMip.positionScale.has_value()) {
                SetErrorMessage("Color MIP %d doesn't have the positionLod and positionScale parameters.", int(mipLevel));
                return Status::FileUnrecognized;
            }
            if (colorMip.width.has_value() && colorMip.height.has_value()) {
                int const mipWidth = std::max(m_desc.width >> mipLevel, 1), mipHeight = std::max(m_desc.height >> mipLevel, 1);
                if (int(*colorMip.width) != mipWidth || int(*colorMip.height) != mipHeight) {
                    SetErrorMessage("Color MIP %d specifies dimensions of %dx%d, but it is expected to be %dx%d.", int(mipLevel),
                        int(*colorMip.width), int(*colorMip.height), mipWidth, mipHeight);
                    return Status::FileUnrecognized;
                }
            }
        }

        // The decoder relies on one specific geometry (src/TextureSet.cpp:161-196).
        for (size_t neuralLod = 0; neuralLod < document.latents.size(); ++neuralLod) {
            file::LatentImage const& image = document.latents[neuralLod];
            int const width = GridDimension(m_desc.width, int(neuralLod), shape.gridSizeScale);
            int const height = GridDimension(m_desc.height, int(neuralLod), shape.gridSizeScale);
            if (int(image.width) != width || int(image.height) != height) {
                SetErrorMessage("Neural MIP %d dimensions (%dx%d) don't match the expected dimensions (%dx%d)", int(neuralLod),
                    int(image.width), int(image.height), width, height);
                return Status::FileUnrecognized;
            }
        }
        for (int mipLevel = 0; mipLevel < m_desc.mips; ++mipLevel) {
            int const expected = LodToNeuralLod(mipLevel, shape.gridSizeScale, int(document.latents.size()));
            if (fileNeuralLod[mipLevel] != expected) {
                SetErrorMessage("Color MIP %d specifies latent image index %d, but it is expected to be %d.", mipLevel, fileNeuralLod[mipLevel], expected);
                return Status::FileUnrecognized;
            }
        }
        int const neuralLods = NeuralLodCount(m_desc.width, m_desc.height, m_desc.mips, shape.gridSizeScale);
        if (int(document.latents.size()) < neuralLods) {
            SetErrorMessage("The file holds %d latent images while %d are expected", int(document.latents.size()), neuralLods);
            return Status::FileUnrecognized;
        }

        // MLP data: the Int8 and the FP8 version, each expanded to the layer sizes the decoder is built for
        // (LoadWeightsFromStream, src/TextureSetMetadata.cpp:675-784).
        NtcHipWeightLayout layout{}, layoutFP8{};
        NtcHipDecoderSpec specFP8 = spec;
        specFP8.weightType = NTC_HIP_WEIGHTS_FP8;
        if (ntc_hip_weight_layout(&spec, &layout) != 0 || ntc_hip_weight_layout(&specFP8, &layoutFP8) != 0) { SetErrorMessage("%s", ntc_hip_last_error()); return Status::InternalError; }
        std::vector<uint8_t> blob, blobFP8;
        for (file::Mlp const& mlp : document.mlpVersions) {
            if (mlp.layers.empty()) continue;
            if (mlp.layers[0].weightType == file::MlpDataType::Int8) {
                blob.assign(layout.bufferSize, 0);
                if (Status st = ReadMlpData(document, mlp, spec, layout, binaryChunkOffset, stream, blob); st != Status::Ok) return st;
            } else if (mlp.layers[0].weightType == file::MlpDataType::FloatE4M3) {
                blobFP8.assign(layoutFP8.bufferSize, 0);
                if (Status st = ReadMlpData(document, mlp, specFP8, layoutFP8, binaryChunkOffset, stream, blobFP8); st != Status::Ok) return st;
            }
        }

        // Latents: u16 layers, neural LOD after neural LOD (src/FeatureGridHost.cpp:140-161).
        std::vector<uint8_t> latents;
        std::vector<BufferFootprint> footprints;
        for (int neuralLod = 0; neuralLod < neuralLods; ++neuralLod) {
            file::LatentImage const& image = document.latents[size_t(neuralLod)];
            size_t const layerSize = size_t(image.width) * size_t(image.height) * 2u;
            for (uint32_t viewIndex : image.layerViews) {
                file::BufferView const& view = document.views[viewIndex];
                file::Compression const compression = view.compression.value_or(file::Compression::None);
                BufferFootprint footprint;
                footprint.rangeInStream = StreamRange{ view.offset + binaryChunkOffset, view.storedSize };
                footprint.compressionType = CompressionType(int(compression));
                footprint.uncompressedSize = view.uncompressedSize.value_or(view.storedSize);
                footprint.uncompressedCrc32 = view.crc32.value_or(0);
                footprints.push_back(footprint);
                if (metadataOnly) continue;
                if (compression != file::Compression::None) {
                    SetErrorMessage("Latent image view %d is stored with GDeflate compression, which this library does not decode.", int(viewIndex));
                    return Status::Unsupported;
                }
                size_t const at = latents.size();
                latents.resize(at + layerSize);
                if (!(stream->Seek(binaryChunkOffset + view.offset) && stream->Read(latents.data() + at, layerSize))) {
                    SetErrorMessage("Failed to read latent image view %d.", int(viewIndex));
                    return Status::IOError;
                }
            }
        }

        // Same order as the reference: the shape is (re)applied, then the data goes in.
        m_latentShape = LatentShape::Empty();
        if (Status st = SetLatentShape(shape); st != Status::Ok) return st;
        m_latentFootprints = std::move(footprints);     // file metadata: valid whether or not the uploads below succeed
        if ((!metadataOnly && latents.size() != m_latentBytes) || (!blob.empty() && blob.size() != m_weightLayout.bufferSize)
            || (!blobFP8.empty() && blobFP8.size() != m_weightLayoutFP8.bufferSize)) { SetErrorMessage("Inconsistent sizes for MLP or latent data"); return Status::InternalError; }
        if (metadataOnly) {
            // no device behind a metadata object: the host copies are what counts
            for (int version = 0; version < 2; ++version) {
                std::vector<uint8_t> const& data = version == 0 ? blob : blobFP8;
                if (data.empty()) continue;
                Status const st = version == 0 ? SetWeightData(data.data(), data.size()) : SetFP8WeightData(data.data(), data.size());
                if (st != Status::Ok && st != Status::CudaUnavailable) return st;
            }
            ClearErrorMessage();
            return Status::Ok;
        }
        if (!blob.empty())
            if (Status st = SetWeightData(blob.data(), blob.size()); st != Status::Ok) return st;
        if (!blobFP8.empty())
            if (Status st = SetFP8WeightData(blobFP8.data(), blobFP8.size()); st != Status::Ok) return st;
        if (Status st = SetLatentData(latents.data(), latents.size()); st != Status::Ok) return st;
        ClearErrorMessage();
        return Status::Ok;
    }

    Status SetDecoderPreset(DecoderPreset preset) override
    {
        if (int(preset) < 0 || int(preset) > int(DecoderPreset::Concat2x2_48)) {
            SetErrorMessage("Unknown decoder preset %d.", int(preset));
            return Status::OutOfRange;
        }
        m_preset = preset;
        if (preset == DecoderPreset::LibNTC092)
            return m_latentShape.IsEmpty() ? ResetShape() : Rebuild();
        return Rebuild();
    }

    // src/TextureSet.cpp:296-466 (decode-side part) with the range rules of
    // src/TextureSetMetadata.cpp:1137-1159
    Status SetLatentShape(LatentShape const& newShape) override
    {
        if (Status st = ValidateLatentShape(newShape); st != Status::Ok) return st;
        m_latentShape = newShape;
        if (newShape.IsEmpty()) return ResetShape();
        m_preset = DecoderPreset::LibNTC092;
        return Rebuild();
    }

    uint64_t GetLatentDataSize() const override { return m_state == NetworkState::Empty ? 0 : m_latentBytes; }
    uint64_t GetWeightDataSize() const override { return m_state == NetworkState::Empty ? 0 : m_weightLayout.bufferSize; }
    uint64_t GetFP8WeightDataSize() const override { return (m_state == NetworkState::Empty || m_preset != DecoderPreset::LibNTC092) ? 0 : m_weightLayoutFP8.bufferSize; }

    Status SetLatentData(void const* data, size_t size) override { return Upload(data, size, m_latentBytes, m_latents, "latent", m_haveLatents); }
    Status SetWeightData(void const* data, size_t size) override
    {
        Status const st = Upload(data, size, m_weightLayout.bufferSize, m_weights, "weight", m_haveWeights);
        // The copy GetInferenceWeights hands out; a new blob starts un-shuffled.  A context without a device keeps
        // it too (the blob passed every check but the upload), as the reference's metadata-only objects do.
        if (st == Status::Ok || st == Status::CudaUnavailable) {
            m_hostWeights.assign(static_cast<uint8_t const*>(data), static_cast<uint8_t const*>(data) + size);
            ResetShuffle();
        }
        return st;
    }

    Status SetFP8WeightData(void const* data, size_t size) override
    {
        if (m_state != NetworkState::Empty && m_preset != DecoderPreset::LibNTC092) {
            SetErrorMessage("FP8 weights exist for the LibNTC092 decoder preset only.");
            return Status::Unsupported;
        }
        Status const st = Upload(data, size, m_weightLayoutFP8.bufferSize, m_weightsFP8, "FP8 weight", m_haveWeightsFP8);
        if (st == Status::Ok || st == Status::CudaUnavailable)
            m_hostWeightsFP8.assign(static_cast<uint8_t const*>(data), static_cast<uint8_t const*>(data) + size);
        return st;
    }

    // useInt8Weights selects the MLP version, as in the reference (src/TextureSet.cpp:1664-1682,1812,1826):
    // false, the default, decodes with the FP8 version (e4m3 hidden layers), true with the Int8 version.
    Status Decompress(DecompressionStats* pOutStats, bool useInt8Weights) override
    {
        bool const complete = m_haveLatents && (useInt8Weights ? m_haveWeights : m_haveWeightsFP8);
        if (m_state == NetworkState::Empty || !complete) {
            if (m_state != NetworkState::Empty && m_haveLatents && (m_haveWeights || m_haveWeightsFP8))
                SetErrorMessage("The texture set holds no %s version of the MLP weights; call Decompress with useInt8Weights = %s.",
                    useInt8Weights ? "Int8" : "FP8", useInt8Weights ? "false" : "true");
            else
                SetErrorMessage("Invalid network state for Decompress (%s), must be Complete.", NetworkStateToString(m_state));
            return Status::InvalidState;
        }
        if (pOutStats) { *pOutStats = DecompressionStats(); std::fill_n(pOutStats->perChannelLoss, 16, 0.f); std::fill_n(pOutStats->perMipLoss, 16, 0.f); }
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }

        // Losses need the reference image to survive the decode: decode into a second page.
        uint32_t const validMask = GetValidChannelMask();
        // The loss branch runs whenever the valid mask is non-zero (src/Inference.cu:77); here it is a pass
        // of its own, needed for the statistics or for the clamp of the mask channel.
        bool const lossPass = validMask != 0 && (pOutStats || m_maskChannelIndex >= 0);
        bool const lazyOutPage = lossPass && !m_textureDataOut;
        if (lazyOutPage)
            if (int r = ntc_hip_ctx_alloc(Hip(), &m_textureDataOut, m_textureBytes)) return AllocationFailure(r, "texture data (output)", m_textureBytes);
        void* const outPage = m_textureDataOut ? m_textureDataOut : m_textureData;   // src/TextureSet.cpp:1799-1802

        NtcHipTextureSet set{};
        set.spec = m_spec;
        if (!useInt8Weights) set.spec.weightType = NTC_HIP_WEIGHTS_FP8;
        set.numMips = m_desc.mips;
        set.numChannels = m_desc.channels;
        set.outputFormat = NTC_HIP_OUT_FP16_PLANAR_PAIRS;
        set.latents = m_latents; set.latentsBytes = m_latentBytes;
        set.weights = useInt8Weights ? m_weights : m_weightsFP8;
        set.weightsBytes = useInt8Weights ? m_weightLayout.bufferSize : m_weightLayoutFP8.bufferSize;
        set.output = outPage; set.outputBytes = m_textureBytes;
        for (int mip = 0; mip < m_desc.mips; ++mip) {
            set.mips[mip] = m_mips[mip];
            set.mips[mip].outOffset = m_mipOffsets[mip] * uint64_t(m_desc.channels) * 2u;   // src/TextureSet.cpp:1804
        }
        // The reference brackets its per-mip loop with events only when statistics are asked
        // for, and otherwise returns without waiting (src/TextureSet.cpp:1772-1780,1866-1882).
        if (pOutStats) {
            float ms = 0.f;
            if (int r = ntc_hip_ctx_decode_timed(Hip(), &set, 1, 1, &ms)) return DeviceFailure(r);
            pOutStats->gpuTimeMilliseconds = ms;
        } else if (int r = ntc_hip_ctx_decode(Hip(), &set, 1)) {
            return DeviceFailure(r);
        }

        // Per-channel / per-mip / overall mean squared error, weighted by pixel count exactly as
        // src/TextureSet.cpp:1833-1863,1884-1892 combine them.
        if (lossPass) {
            int validChannels = 0;
            for (int ch = 0; ch < m_desc.channels; ++ch) if (validMask & (1u << ch)) ++validChannels;
            double perChannel[16] = {};
            double overall = 0.0, pixels = 0.0;
            for (int mip = 0; mip < m_desc.mips; ++mip) {
                uint64_t const offset = m_mipOffsets[mip] * uint64_t(m_desc.channels) * 2u;
                float mse[16];
                if (int r = ntc_hip_ctx_image_loss(Hip(), static_cast<uint8_t*>(outPage) + offset, static_cast<uint8_t const*>(m_textureData) + offset,
                                               m_textureBytes - offset, m_mips[mip].width, m_mips[mip].height, m_desc.channels, validMask,
                                               m_maskChannelIndex < 0 ? -1 : m_maskChannelIndex, m_discardMaskedOutPixels ? 1 : 0, mse))
                    return DeviceFailure(r);
                if (!pOutStats) continue;
                double const mipPixels = double(m_mips[mip].width) * double(m_mips[mip].height);
                double mean = 0.0;
                for (int ch = 0; ch < m_desc.channels; ++ch) {
                    if (!(validMask & (1u << ch))) continue;
                    mean += mse[ch];
                    perChannel[ch] += mipPixels * mse[ch];
                }
                mean /= double(validChannels);
                pOutStats->perMipLoss[mip] = float(mean);
                overall += mipPixels * mean;
                pixels += mipPixels;
            }
            if (pOutStats) {
                pOutStats->overallLoss = float(overall / pixels);
                for (int ch = 0; ch < 16; ++ch) pOutStats->perChannelLoss[ch] = float(perChannel[ch] / pixels);
            }
        }
        // Without separateRefOutData both pages are one memory in the reference and the decode
        // overwrites the reference image; keep that: the decoded page becomes the only page.
        if (lazyOutPage) {
            if (int r = ntc_hip_ctx_synchronize(Hip())) return DeviceFailure(r);
            std::swap(m_textureData, m_textureDataOut);
            ReleaseDevice(m_textureDataOut);
        }
        m_decompressed = true;
        ClearErrorMessage();
        return Status::Ok;
    }

    // src/TextureSet.cpp:829-913
    Status WriteChannels(WriteChannelsParameters const& params) override
    {
        if (!params.pData) { SetErrorMessage("pData is NULL."); return Status::InvalidArgument; }
        size_t const sizeToCopy = size_t(params.height) * params.rowPitch;
        bool const fromHost = params.addressSpace == AddressSpace::Host;
        if (Status st = ValidateReadWriteChannelsArgs(params.mipLevel, params.firstChannel, params.numChannels, params.width, params.height,
                params.pixelStride, params.rowPitch, fromHost ? sizeToCopy : 0, params.channelFormat, "writes"); st != Status::Ok)
            return st;
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }
        if (fromHost)
            if (int r = ntc_hip_ctx_upload(Hip(), m_staging, params.pData, sizeToCopy)) return DeviceFailure(r);
        int const mipWidth = std::max(m_desc.width >> params.mipLevel, 1), mipHeight = std::max(m_desc.height >> params.mipLevel, 1);
        NtcHipWriteChannels wc{};
        wc.src = fromHost ? m_staging : static_cast<void const*>(params.pData);
        wc.srcBytes = sizeToCopy;
        wc.format = int(params.channelFormat);
        wc.verticalFlip = params.verticalFlip ? 1 : 0;
        wc.pixelStride = params.pixelStride; wc.rowPitch = params.rowPitch;
        uint64_t const offset = m_mipOffsets[params.mipLevel] * uint64_t(m_desc.channels) * 2u;
        wc.planarPairs = static_cast<uint8_t*>(m_textureData) + offset;               // the reference page
        wc.planarBytes = m_textureBytes - offset;
        wc.width = mipWidth; wc.height = mipHeight; wc.setChannels = m_desc.channels;
        wc.srcWidth = params.width; wc.srcHeight = params.height;               // another size: resampled (src/ImageProcessing.cu:24-72)
        wc.firstChannel = params.firstChannel; wc.numChannels = params.numChannels;
        for (int channel = 0; channel < params.numChannels; ++channel) {
            ColorSpace const source = params.srcColorSpaces ? params.srcColorSpaces[channel] : ColorSpace::Linear;
            ColorSpace const storage = params.dstColorSpaces ? params.dstColorSpaces[channel] : ColorSpace::Linear;
            if (unsigned(source) > 2u || unsigned(storage) > 2u) { SetErrorMessage("Unknown colour space for channel %d.", channel); return Status::InvalidArgument; }
            wc.srcColorSpaces[channel] = uint8_t(source);
            wc.dstColorSpaces[channel] = uint8_t(storage);
            m_channelColorSpaces[channel + params.firstChannel] = storage;       // src/TextureSet.cpp:899-902
        }
        if (int r = ntc_hip_ctx_write_channels(Hip(), &wc)) return DeviceFailure(r);
        ClearErrorMessage();
        return Status::Ok;
    }

    // src/TextureSet.cpp:915-985 and :1914-1956
    Status ReadChannels(ReadChannelsParameters const& params) override
    {
        if (!params.pOutData) { SetErrorMessage("pOutData is NULL."); return Status::InvalidArgument; }
        size_t const sizeToCopy = size_t(params.height) * params.rowPitch;
        bool const toHost = params.addressSpace == AddressSpace::Host;
        if (Status st = ValidateReadWriteChannelsArgs(params.mipLevel, params.firstChannel, params.numChannels, params.width, params.height,
                params.pixelStride, params.rowPitch, toHost ? sizeToCopy : 0, params.channelFormat, "reads"); st != Status::Ok)
            return st;
        int const mipWidth = std::max(m_desc.width >> params.mipLevel, 1), mipHeight = std::max(m_desc.height >> params.mipLevel, 1);
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }

        // Rows the copy does not fully overwrite must not carry garbage to the client (src/TextureSet.cpp:936-946).
        if (toHost && params.rowPitch > params.pixelStride * size_t(params.width))
            if (int r = ntc_hip_ctx_memset(Hip(), m_staging, 0, sizeToCopy)) return DeviceFailure(r);

        NtcHipReadChannels rc{};
        // GetTextureDataSlice: the output page when it exists and is asked for (src/TextureSet.cpp:1961-1964)
        void const* const page = (params.page == TextureDataPage::Output && m_textureDataOut) ? m_textureDataOut : m_textureData;
        rc.planarPairs = static_cast<uint8_t const*>(page) + m_mipOffsets[params.mipLevel] * uint64_t(m_desc.channels) * 2u;
        rc.planarBytes = uint64_t(mipWidth) * uint64_t(mipHeight) * uint64_t(m_desc.channels) * 2u;
        rc.width = mipWidth; rc.height = mipHeight;
        rc.dstWidth = params.width; rc.dstHeight = params.height;               // another size: resampled
        rc.setChannels = m_desc.channels;
        rc.firstChannel = params.firstChannel; rc.numChannels = params.numChannels;
        rc.dst = toHost ? m_staging : params.pOutData;
        rc.dstBytes = toHost ? m_stagingBytes : sizeToCopy;
        rc.format = int(params.channelFormat);
        rc.pixelStride = params.pixelStride; rc.rowPitch = params.rowPitch;
        rc.useDithering = params.useDithering ? 1 : 0;
        for (int channel = 0; channel < params.numChannels; ++channel) {
            ColorSpace const wanted = params.dstColorSpaces ? params.dstColorSpaces[channel] : ColorSpace::Linear;
            if (unsigned(wanted) > 2u) { SetErrorMessage("Unknown colour space for channel %d.", channel); return Status::InvalidArgument; }
            rc.srcColorSpaces[channel] = uint8_t(m_channelColorSpaces[channel + params.firstChannel]);
            rc.dstColorSpaces[channel] = uint8_t(wanted);
        }
        if (int r = ntc_hip_ctx_read_channels(Hip(), &rc)) return DeviceFailure(r);
        if (toHost)
            if (int r = ntc_hip_ctx_download(Hip(), params.pOutData, m_staging, sizeToCopy)) return DeviceFailure(r);
        ClearErrorMessage();
        return Status::Ok;
    }

    // src/TextureSet.cpp:1121-1142: every mip of the reference page from the one above it, through the
    // storage colour spaces of the channels; a 2x reduction is a 2x2 box filter.
    Status GenerateMips() override
    {
        if (m_desc.mips <= 1) { ClearErrorMessage(); return Status::Ok; }
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }
        uint8_t spaces[NTC_HIP_MAX_CHANNELS];
        for (int ch = 0; ch < NTC_HIP_MAX_CHANNELS; ++ch) spaces[ch] = uint8_t(m_channelColorSpaces[ch]);
        for (int mip = 1; mip < m_desc.mips; ++mip) {
            uint64_t const srcOffset = m_mipOffsets[mip - 1] * uint64_t(m_desc.channels) * 2u, dstOffset = m_mipOffsets[mip] * uint64_t(m_desc.channels) * 2u;
            if (int r = ntc_hip_ctx_resize_planar(Hip(), static_cast<uint8_t const*>(m_textureData) + srcOffset, dstOffset - srcOffset,
                                              std::max(m_desc.width >> (mip - 1), 1), std::max(m_desc.height >> (mip - 1), 1),
                                              static_cast<uint8_t*>(m_textureData) + dstOffset, m_textureBytes - dstOffset,
                                              std::max(m_desc.width >> mip, 1), std::max(m_desc.height >> mip, 1), m_desc.channels, spaces))
                return DeviceFailure(r);
        }
        ClearErrorMessage();
        return Status::Ok;
    }

private:
    // src/TextureSet.cpp:1914-1956
    Status ValidateReadWriteChannelsArgs(int mipLevel, int firstChannel, int numChannels, int width, int height,
        size_t pixelStride, size_t rowPitch, size_t stagedBytes, ChannelFormat format, char const* what)
    {
        if (mipLevel < 0 || mipLevel >= m_desc.mips) {
            SetErrorMessage("mipLevel (%d) must be between 0 and %d.", mipLevel, m_desc.mips - 1);
            return Status::OutOfRange;
        }
        if (firstChannel < 0 || firstChannel >= m_desc.channels) {
            SetErrorMessage("firstChannel (%d) must be between 0 and %d.", firstChannel, m_desc.channels - 1);
            return Status::OutOfRange;
        }
        if (numChannels < 1 || numChannels + firstChannel > m_desc.channels) {
            SetErrorMessage("For the provided firstChannel (%d), numChannels (%d) must be between 1 and %d.",
                firstChannel, numChannels, m_desc.channels - firstChannel);
            return Status::OutOfRange;
        }
        if (width <= 0 || height <= 0) {
            SetErrorMessage("width (%d) and height (%d) must be positive.", width, height);
            return Status::OutOfRange;
        }
        if (pixelStride < 1 || rowPitch < pixelStride) {
            SetErrorMessage("pixelStride (%zu) must be between 1 and rowPitch (%zu).", pixelStride, rowPitch);
            return Status::InvalidArgument;
        }
        if (stagedBytes > m_stagingBytes) {
            SetErrorMessage("The operation requires copying too much data (%zu bytes), must fit into "
                "the staging buffer (%zu bytes).", stagedBytes, size_t(m_stagingBytes));
            return Status::OutOfRange;
        }
        if (GetBytesPerPixelComponent(format) == 0) { SetErrorMessage("Unknown channel format %d for %s.", int(format), what); return Status::InvalidArgument; }
        return Status::Ok;
    }

    // src/TextureSetMetadata.cpp:978-1016
    bool ValidateBufferView(uint32_t view, uint64_t minSize, file::Document const& document, uint64_t binaryChunkSize)
    {
        if (view >= document.views.size()) { SetErrorMessage("Invalid view index %u", view); return false; }
        file::BufferView const& desc = document.views[view];
        if ((desc.offset & 3) != 0) { SetErrorMessage("View %u offset %" PRIu64 " is not 4-byte aligned", view, desc.offset); return false; }
        uint64_t const uncompressedSize = desc.compression.value_or(file::Compression::None) != file::Compression::None
            ? desc.uncompressedSize.value_or(0) : desc.storedSize;
        if (uncompressedSize < minSize) {
            SetErrorMessage("View %u size %" PRIu64 " is less than minimum expected size %" PRIu64 ".", view, desc.storedSize, minSize);
            return false;
        }
        if (desc.offset + desc.storedSize < desc.offset || desc.offset + desc.storedSize > binaryChunkSize) {
            SetErrorMessage("View %u ends at byte offset %" PRIu64 " from the binary chunk start, "
                "which is outside of the chunk size %" PRIu64 ".", view, desc.offset + desc.storedSize, binaryChunkSize);
            return false;
        }
        return true;
    }

    static size_t MlpDataTypeSize(file::MlpDataType type)      // src/TextureSetMetadata.cpp:1018-1029
    {
        switch (type) {
        case file::MlpDataType::Int8: case file::MlpDataType::FloatE4M3: case file::MlpDataType::FloatE5M2: return 1;
        case file::MlpDataType::Float16: return 2;
        case file::MlpDataType::Float32: return 4;
        default: return 0;
        }
    }

    // src/TextureSetMetadata.cpp:1031-1135: four layers, row-major, one of the two known type
    // patterns, hidden layers no wider than the decoder's, views large enough.
    bool ValidateMLP(file::Document const& document, file::Mlp const& mlp, NtcHipDecoderSpec const& spec, uint64_t binaryChunkSize)
    {
        using T = file::MlpDataType;
        if (mlp.layers.size() != 4) {
            SetErrorMessage("File describes an MLP with %d layers, while only %d layers are supported", int(mlp.layers.size()), 4);
            return false;
        }
        if (mlp.weightLayout != file::MatrixLayout::RowMajor) { SetErrorMessage("Only row-major MLP weight layout is supported at this time."); return false; }
        bool int8Pattern = true, fp8Pattern = true;
        for (int l = 0; l < 4; ++l) {
            file::MlpLayer const& layer = mlp.layers[size_t(l)];
            bool const last = l == 3;
            int8Pattern = int8Pattern && layer.weightType == T::Int8 && layer.scaleType == T::Float32 && layer.biasType == T::Int32;
            fp8Pattern = fp8Pattern && (last ? (layer.weightType == T::Int8 && layer.scaleType == T::Float32 && layer.biasType == T::Int32)
                                             : (layer.weightType == T::FloatE4M3 && !layer.scaleType.has_value() && layer.biasType == T::Float16));
        }
        if (!int8Pattern && !fp8Pattern) {
            SetErrorMessage("Only Int8 weights + Float32 scale + Int32 bias or FloatE4M3 + Float16 bias MLP configurations are supported at this time.");
            return false;
        }
        for (int l = 0; l < 4; ++l) {
            file::MlpLayer const& layer = mlp.layers[size_t(l)];
            bool const smallerInputsAllowed = l > 0, smallerOutputsAllowed = l < 3;
            uint32_t const expectedInputs = uint32_t(LayerInputs(spec, l)), expectedOutputs = uint32_t(LayerOutputs(spec, l));
            bool const inputsFine = smallerInputsAllowed ? layer.inputChannels <= expectedInputs : layer.inputChannels == expectedInputs;
            bool const outputsFine = smallerOutputsAllowed ? layer.outputChannels <= expectedOutputs : layer.outputChannels == expectedOutputs;
            if (!inputsFine || !outputsFine) {
                SetErrorMessage("File describes MLP layer %d with %d inputs and %d outputs, but that layer should have %s%d inputs and %s%d outputs.",
                    l, int(layer.inputChannels), int(layer.outputChannels), smallerInputsAllowed ? "at most " : "", int(expectedInputs),
                    smallerOutputsAllowed ? "at most " : "", int(expectedOutputs));
                return false;
            }
            if (!ValidateBufferView(layer.weightView, uint64_t(layer.inputChannels) * layer.outputChannels * MlpDataTypeSize(layer.weightType), document, binaryChunkSize)) return false;
            if (layer.scaleType.has_value() && layer.scaleView.has_value())
                if (!ValidateBufferView(*layer.scaleView, uint64_t(layer.outputChannels) * MlpDataTypeSize(*layer.scaleType), document, binaryChunkSize)) return false;
            if (!ValidateBufferView(layer.biasView, uint64_t(layer.outputChannels) * MlpDataTypeSize(layer.biasType), document, binaryChunkSize)) return false;
        }
        return true;
    }

    static int LayerInputs(NtcHipDecoderSpec const& spec, int layer) { return layer == 0 ? spec.inputChannels : spec.hiddenChannels[layer - 1]; }
    static int LayerOutputs(NtcHipDecoderSpec const& spec, int layer) { return layer == 3 ? spec.outputChannels : spec.hiddenChannels[layer]; }

    // src/TextureSetMetadata.cpp:661-761: a narrower hidden layer lands in the top-left corner of
    // the zero-filled matrix, missing scales become 1, missing biases stay 0.
    Status ReadMlpData(file::Document const& document, file::Mlp const& mlp, NtcHipDecoderSpec const& spec, NtcHipWeightLayout const& layout,
        uint64_t binaryChunkOffset, IStream* stream, std::vector<uint8_t>& blob)
    {
        auto readView = [&](uint32_t view, void* dst, size_t size) {
            return size == 0 || (stream->Seek(binaryChunkOffset + document.views[view].offset) && stream->Read(dst, size));
        };
        std::vector<uint8_t> narrow;
        for (int l = 0; l < 4; ++l) {
            file::MlpLayer const& layer = mlp.layers[size_t(l)];
            size_t const expectedInputs = size_t(LayerInputs(spec, l)), expectedOutputs = size_t(LayerOutputs(spec, l));
            uint8_t* const weights = blob.data() + layout.weightOffset[l];
            if (layer.inputChannels < expectedInputs || layer.outputChannels < expectedOutputs) {
                narrow.resize(size_t(layer.inputChannels) * layer.outputChannels);
                if (!readView(layer.weightView, narrow.data(), narrow.size())) return ReadFailure("weights", l);
                for (size_t row = 0; row < layer.outputChannels; ++row)
                    std::memcpy(weights + row * expectedInputs, narrow.data() + row * layer.inputChannels, layer.inputChannels);
            } else if (!readView(layer.weightView, weights, expectedInputs * expectedOutputs)) {
                return ReadFailure("weights", l);
            }
            // e4m3 layers of the FP8 blob carry no scales and fp16 biases (src/WeightLayout.cpp:51-71)
            bool const e4m3Layer = spec.weightType == NTC_HIP_WEIGHTS_FP8 && l < 3;
            if (!e4m3Layer) {
                float* const scales = reinterpret_cast<float*>(blob.data() + layout.scaleOffset[l]);
                size_t const providedScales = layer.scaleView.has_value() ? layer.outputChannels : 0;
                if (providedScales && !readView(*layer.scaleView, scales, providedScales * sizeof(float))) return ReadFailure("scales", l);
                for (size_t i = providedScales; i < expectedOutputs; ++i) scales[i] = 1.0f;
            }
            size_t const biasElement = e4m3Layer ? sizeof(uint16_t) : sizeof(int32_t);
            if (!readView(layer.biasView, blob.data() + layout.biasOffset[l], size_t(layer.outputChannels) * biasElement)) return ReadFailure("biases", l);
        }
        return Status::Ok;
    }
    Status ReadFailure(char const* what, int layer) { SetErrorMessage("Failed to read the %s of MLP layer %d.", what, layer); return Status::IOError; }

    Status AllocationFailure(int code, char const* what, uint64_t bytes)
    {
        if (code > 0) { SetErrorMessage("Failed to allocate %llu bytes of device memory for the %s buffer.", (unsigned long long)bytes, what); return Status::OutOfMemory; }
        return DeviceFailure(code);
    }

    void ReleaseDevice(void*& p) { if (p) { (void)ntc_hip_ctx_free(Hip(), p); p = nullptr; } }

    Status ResetShape()
    {
        ReleaseDevice(m_latents); ReleaseDevice(m_weights); ReleaseDevice(m_weightsFP8);
        m_hostWeights.clear(); m_hostWeightsFP8.clear();
        m_latentFootprints.clear();
        m_latentBytes = 0; m_haveLatents = m_haveWeights = m_haveWeightsFP8 = false;
        m_numNeuralLods = 0;
        m_state = NetworkState::Empty;
        ClearErrorMessage();
        return Status::Ok;
    }

    // Recomputes the geometry of every colour mip and (re)allocates latent / weight memory.
    Status Rebuild()
    {
        m_spec = MakeSpec(m_preset, m_latentShape.IsEmpty() ? 16 : m_latentShape.numFeatures);
        if (m_preset == DecoderPreset::LibNTC092) {
            if (m_latentShape.IsEmpty()) { SetErrorMessage("SetLatentShape must be called before selecting the LibNTC092 preset."); return Status::InvalidState; }
            BuildSharedNeuralLods();
        } else {
            BuildPerMipGrids();
        }
        if (ntc_hip_weight_layout(&m_spec, &m_weightLayout) != 0) { SetErrorMessage("%s", ntc_hip_last_error()); return Status::InternalError; }
        m_weightLayoutFP8 = NtcHipWeightLayout{};
        if (m_preset == DecoderPreset::LibNTC092) {
            NtcHipDecoderSpec specFP8 = m_spec;
            specFP8.weightType = NTC_HIP_WEIGHTS_FP8;
            if (ntc_hip_weight_layout(&specFP8, &m_weightLayoutFP8) != 0) { SetErrorMessage("%s", ntc_hip_last_error()); return Status::InternalError; }
        }
        ReleaseDevice(m_latents); ReleaseDevice(m_weights); ReleaseDevice(m_weightsFP8);
        m_hostWeights.clear(); m_hostWeightsFP8.clear();
        m_latentFootprints.clear();
        m_haveLatents = m_haveWeights = m_haveWeightsFP8 = false;
        if (m_deviceAvailable) {
            if (int r = ntc_hip_ctx_alloc(Hip(), &m_latents, m_latentBytes)) return AllocationFailure(r, "latent", m_latentBytes);
            if (int r = ntc_hip_ctx_alloc(Hip(), &m_weights, m_weightLayout.bufferSize)) return AllocationFailure(r, "MLP weights", m_weightLayout.bufferSize);
            if (m_weightLayoutFP8.bufferSize)
                if (int r = ntc_hip_ctx_alloc(Hip(), &m_weightsFP8, m_weightLayoutFP8.bufferSize)) return AllocationFailure(r, "MLP weights (FP8)", m_weightLayoutFP8.bufferSize);
        }
        m_state = NetworkState::Initialized;
        ClearErrorMessage();
        return Status::Ok;
    }

    // LodToNeuralLod / GetGridDimension / CalculateNumNeuralMipLevels (src/FeatureGridMath.cpp:47-77),
    // neural-LOD count and offsets of FeatureGrid::Initialize (src/FeatureGridHost.cpp:27-58,140-146),
    // colour-mip constants (src/TextureSet.cpp:441-463), low-res dimensions (src/TextureSet.cpp:1816-1817).
    void BuildSharedNeuralLods()
    {
        int const gs = m_latentShape.gridSizeScale;
        auto neuralOf = [&](int lod, int count) { return LodToNeuralLod(lod, gs, count); };
        auto gridDim = [&](int dim, int nlod) { return GridDimension(dim, nlod, gs); };
        int const neuralLods = NeuralLodCount(m_desc.width, m_desc.height, m_desc.mips, gs);
        uint64_t const layers = uint64_t((m_latentShape.numFeatures + 3) / 4);
        std::vector<uint64_t> offset(size_t(neuralLods) + 1, 0);
        for (int n = 0; n < neuralLods; ++n)
            offset[size_t(n) + 1] = offset[size_t(n)] + uint64_t(gridDim(m_desc.width, n)) * uint64_t(gridDim(m_desc.height, n)) * 2u * layers;
        m_latentBytes = offset[size_t(neuralLods)];
        m_numNeuralLods = neuralLods;
        for (int mip = 0; mip < m_desc.mips; ++mip) {
            NtcHipMipDesc& d = m_mips[mip];
            d = NtcHipMipDesc{};
            int const nlod = neuralOf(mip, neuralLods);
            m_neuralLodOfMip[mip] = nlod;
            d.width = std::max(1, m_desc.width >> mip); d.height = std::max(1, m_desc.height >> mip);
            d.hrWidth = gridDim(m_desc.width, nlod); d.hrHeight = gridDim(m_desc.height, nlod);
            d.lrWidth = std::max(d.hrWidth >> 1, 1); d.lrHeight = std::max(d.hrHeight >> 1, 1);
            d.hrOffset = offset[size_t(nlod)]; d.lrOffset = offset[size_t(nlod) + 1];
            PositionConstants(d);
        }
    }

    // Every colour mip owns a high-res grid of half and a low-res grid of a quarter of its size.
    void BuildPerMipGrids()
    {
        m_numNeuralLods = 0;
        uint64_t cursor = 0;
        for (int mip = 0; mip < m_desc.mips; ++mip) {
            NtcHipMipDesc& d = m_mips[mip];
            d = NtcHipMipDesc{};
            d.width = std::max(1, m_desc.width >> mip); d.height = std::max(1, m_desc.height >> mip);
            d.hrWidth = std::max(d.width / 2, 1); d.hrHeight = std::max(d.height / 2, 1);
            d.lrWidth = std::max(d.width / 4, 1); d.lrHeight = std::max(d.height / 4, 1);
            d.hrOffset = cursor; cursor += ntc_hip_grid_bytes(d.hrWidth, d.hrHeight, m_spec.hrFeatures, m_spec.hrBits);
            d.lrOffset = cursor; cursor += ntc_hip_grid_bytes(d.lrWidth, d.lrHeight, m_spec.lrFeatures, m_spec.lrBits);
            PositionConstants(d);
        }
        m_latentBytes = cursor;
    }

    Status Upload(void const* data, size_t size, uint64_t expected, void* device, char const* what, bool& have)
    {
        if (m_state == NetworkState::Empty) { SetErrorMessage("Set a latent shape or decoder preset before providing %s data.", what); return Status::InvalidState; }
        if (!data) { SetErrorMessage("The %s data pointer is NULL.", what); return Status::InvalidArgument; }
        if (size != expected) { SetErrorMessage("The %s data must be %llu bytes, got %zu.", what, (unsigned long long)expected, size); return Status::InvalidArgument; }
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }
        if (int r = ntc_hip_ctx_upload(Hip(), device, data, size)) return DeviceFailure(r);
        have = true;
        if (m_haveLatents && (m_haveWeights || m_haveWeightsFP8)) m_state = NetworkState::Complete;
        ClearErrorMessage();
        return Status::Ok;
    }

    IAllocator* Allocator() const;      // the context's
    NtcHipContext* Hip() const;         // the context's device context (null without a device)

    Context const* m_context;
    TextureSetDesc m_desc;
    TextureSetFeatures m_features;
    LatentShape m_latentShape = LatentShape::Empty();
    DecoderPreset m_preset = DecoderPreset::LibNTC092;
    NetworkState m_state = NetworkState::Empty;
    NtcHipDecoderSpec m_spec{};
    NtcHipWeightLayout m_weightLayout{}, m_weightLayoutFP8{};
    NtcHipMipDesc m_mips[NTC_HIP_MAX_MIPS]{};
    uint64_t m_mipOffsets[NTC_HIP_MAX_MIPS + 1]{};
    uint64_t m_textureBytes = 0, m_stagingBytes = 0, m_latentBytes = 0;
    std::vector<TextureMetadata*> m_textures;
    ColorSpace m_channelColorSpaces[NTC_HIP_MAX_CHANNELS] = {};
    void* m_textureData = nullptr;      // reference page (and the only page without separateRefOutData)
    void* m_textureDataOut = nullptr;   // output page
    void* m_staging = nullptr;
    void* m_latents = nullptr;
    void* m_weights = nullptr;
    void* m_weightsFP8 = nullptr;
    int m_numNeuralLods = 0;                       // shared-LOD geometry only
    int m_neuralLodOfMip[NTC_HIP_MAX_MIPS] = {};
    std::vector<uint8_t> m_hostWeights, m_hostWeightsFP8;
    std::vector<BufferFootprint> m_latentFootprints;    // per (latent image, layer) of the file last loaded; empty otherwise
    ShuffleSource m_shuffle[NTC_HIP_MAX_CHANNELS];
    void ResetShuffle() { for (int ch = 0; ch < NTC_HIP_MAX_CHANNELS; ++ch) m_shuffle[ch] = ShuffleSource::Channel(ch); }
    int m_maskChannelIndex = -1;
    bool m_discardMaskedOutPixels = false;
    bool m_deviceAvailable = false, m_haveLatents = false, m_haveWeights = false, m_haveWeightsFP8 = false, m_decompressed = false;
};

class Context final : public IContext, public amd::IContextExtension
{
public:
    // `hip`: this context's device, stream and working memory (null: no device); owned.
    Context(IAllocator* allocator, NtcHipContext* hip) : m_allocator(allocator), m_hip(hip), m_deviceAvailable(hip != nullptr) {}
    ~Context() override { ntc_hip_destroy(m_hip); }
    IAllocator* GetAllocator() const { return m_allocator; }
    NtcHipContext* GetHip() const { return m_hip; }

    // src/Context.cpp:177-218 with the descriptor rules of src/TextureSetMetadata.cpp:1161-1178
    Status CreateTextureSet(TextureSetDesc const& desc, TextureSetFeatures const& features, ITextureSet** pOutTextureSet) const override
    {
        if (!pOutTextureSet) { SetErrorMessage("pOutTextureSet is NULL."); return Status::InvalidArgument; }
        *pOutTextureSet = nullptr;
        if (!m_deviceAvailable && !m_allowSetsWithoutDevice) {
            SetErrorMessage("Cannot create a TextureSet object when no suitable CUDA device is available.");
            return Status::CudaUnavailable;
        }
        if (Status st = ValidateTextureSetDesc(desc); st != Status::Ok) return st;
        TextureSet* set = MakeObject<TextureSet>(m_allocator, this, desc, features);
        if (!set) { SetErrorMessage("Failed to allocate the texture set object."); return Status::OutOfMemory; }
        Status const status = set->Initialize(m_deviceAvailable);
        if (status != Status::Ok) { DestroyObject(m_allocator, set); return status; }
        *pOutTextureSet = set;
        ClearErrorMessage();
        return Status::Ok;
    }

    void DestroyTextureSet(ITextureSet* textureSet) const override { DestroyObject(m_allocator, dynamic_cast<TextureSet*>(textureSet)); }
    bool IsDeviceAvailable() const override { return m_deviceAvailable; }
    Status Synchronize() const override
    {
        if (!m_deviceAvailable) { ClearErrorMessage(); return Status::Ok; }
        if (int r = ntc_hip_ctx_synchronize(m_hip)) return DeviceFailure(r);
        ClearErrorMessage();
        return Status::Ok;
    }
    void AllowTextureSetsWithoutDevice(bool allow) const override { m_allowSetsWithoutDevice = allow; }

    // ---- outside the decompression path ----
    // src/Context.cpp:380-415: sharing textures with a graphics API
    Status RegisterSharedTexture(SharedTextureDesc const&, ISharedTexture** pOutTexture) const override
    {
        if (!pOutTexture) { SetErrorMessage("pOutTexture is NULL."); return Status::InvalidArgument; }
        *pOutTexture = nullptr;
        return NotPartOfThisLibrary("RegisterSharedTexture", "graphics-API texture sharing");
    }
    void ReleaseSharedTexture(ISharedTexture*) const override {}
    // src/Context.cpp:432-451: the search over compression presets
    Status CreateAdaptiveCompressionSession(IAdaptiveCompressionSession** pOutSession) const override
    {
        if (!pOutSession) { SetErrorMessage("pOutSession is NULL"); return Status::InvalidArgument; }
        *pOutSession = nullptr;
        return NotPartOfThisLibrary("CreateAdaptiveCompressionSession", "compression (training)");
    }
    void DestroyAdaptiveCompressionSession(IAdaptiveCompressionSession*) const override {}
    // src/Context.cpp:453-464,630-643,781-794: the three passes are described for a graphics API, and a context
    // without one answers InvalidArgument.  On the device they run through ntc::amd::IContextExtension and
    // ITextureSet::Decompress.
    Status MakeDecompressionComputePass(MakeDecompressionComputePassParameters const&, ComputePassDesc* pOutComputePass) const override { return NoGraphicsApi(pOutComputePass); }
    Status MakeBlockCompressionComputePass(MakeBlockCompressionComputePassParameters const&, ComputePassDesc* pOutComputePass) const override { return NoGraphicsApi(pOutComputePass); }
    Status MakeImageDifferenceComputePass(MakeImageDifferenceComputePassParameters const&, ComputePassDesc* pOutComputePass) const override { return NoGraphicsApi(pOutComputePass); }
    bool IsCooperativeVectorSupported() const override { return false; }      // src/Context.cpp:924-930
    // src/Context.cpp:952-991.  GDeflate needs the reference's external codec, which its tree does not contain.
    Status DecompressBuffer(CompressionType compressionType, void const* pCompressedData, size_t compressedSize,
        void* pOutDecompressedData, size_t outputBufferSize, uint32_t /*expectedCrc32*/) const override
    {
        switch (compressionType) {
        case CompressionType::None:
            if (!pCompressedData) { SetErrorMessage("pCompressedData is NULL."); return Status::InvalidArgument; }
            if (!pOutDecompressedData) { SetErrorMessage("pOutDecompressedData is NULL."); return Status::InvalidArgument; }
            if (outputBufferSize < compressedSize) {
                SetErrorMessage("When compressionType == None, outputBufferSize (%zu) must be no less than compressedSize (%zu).", outputBufferSize, compressedSize);
                return Status::InvalidArgument;
            }
            std::memcpy(pOutDecompressedData, pCompressedData, compressedSize);
            ClearErrorMessage();
            return Status::Ok;
        case CompressionType::GDeflate:
            SetErrorMessage("GDeflate decompression is not part of this build of LibNTC.");
            return Status::Unsupported;
        default:
            SetErrorMessage("Unknown compressionType (%d).", int(compressionType));
            return Status::InvalidArgument;
        }
    }
    Status DecompressGDeflateOnVulkanGPU(void*, void const*, size_t, uint64_t, uint64_t) const override
    {
        SetErrorMessage("GDeflate decompression on a Vulkan device is not part of this build of LibNTC.");
        return Status::Unsupported;
    }

    Status CompressBlocks(BlockCompressionParameters const& params) const override
    {
        if (!params.pDstData || !params.srcImage.pData) { SetErrorMessage("Source or destination data is NULL"); return Status::InvalidArgument; }
        if (params.srcRect.left < 0 || params.srcRect.top < 0) {
            SetErrorMessage("Left (%d) and top (%d) must be non-negative", params.srcRect.left, params.srcRect.top);
            return Status::OutOfRange;
        }
        if (params.srcRect.width <= 0 || params.srcRect.height <= 0) {
            SetErrorMessage("Width (%d) and height (%d) must be positive", params.srcRect.width, params.srcRect.height);
            return Status::OutOfRange;
        }
        if (params.dstOffsetInBlocks.x < 0 || params.dstOffsetInBlocks.y < 0) {
            SetErrorMessage("dstOffsetInBlocks (%d, %d) must be non-negative", params.dstOffsetInBlocks.x, params.dstOffsetInBlocks.y);
            return Status::OutOfRange;
        }
        if (int(params.dstFormat) < int(BlockCompressedFormat::BC1) || int(params.dstFormat) > int(BlockCompressedFormat::BC7)) {
            SetErrorMessage("Invalid dstFormat (%s)", BlockCompressedFormatToString(params.dstFormat));
            return Status::OutOfRange;
        }
        if (params.pModeBuffer && params.dstFormat != BlockCompressedFormat::BC7) {     // src/Context.cpp:666-671
            SetErrorMessage("Mode buffer can only be used with BC7 compression");
            return Status::InvalidArgument;
        }
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }
        NtcHipBlockCompress p{};
        ImageDesc const& src = params.srcImage;
        p.src.data = src.pData; p.src.bytes = src.dataSize; p.src.pixelStride = src.pixelStride; p.src.rowPitch = src.rowPitch;
        p.src.width = src.width; p.src.height = src.height; p.src.format = int32_t(src.channelFormat); p.src.numChannels = src.numChannels;
        p.srcLeft = params.srcRect.left; p.srcTop = params.srcRect.top;
        p.widthInBlocks = (params.srcRect.width + 3) / 4; p.heightInBlocks = (params.srcRect.height + 3) / 4;
        p.dstFormat = int32_t(params.dstFormat);
        p.alphaThreshold = params.alphaThreshold;
        p.dstOffsetX = params.dstOffsetInBlocks.x; p.dstOffsetY = params.dstOffsetInBlocks.y;
        p.dst = params.pDstData; p.dstBytes = params.dstDataSize; p.dstRowPitch = params.dstRowPitch;
        p.modeBuffer = params.pModeBuffer; p.modeBufferBytes = params.modeBufferSize; p.modeBufferByteOffset = params.modeBufferByteOffset;
        p.modeMapWidthInBlocks = params.modeMapWidthInBlocks; p.modeMapHeightInBlocks = params.modeMapHeightInBlocks;
        p.modeMapOffsetX = params.modeMapOffsetInBlocks.x; p.modeMapOffsetY = params.modeMapOffsetInBlocks.y;
        if (int r = ntc_hip_ctx_block_compress(m_hip, &p)) return DeviceFailure(r);
        ClearErrorMessage();
        return Status::Ok;
    }

    // Argument rules and messages of src/Context.cpp:796-812; the pass itself is ntc_hip_image_difference.
    Status ComputeImageDifference(ImageDifferenceParameters const& params) const override
    {
        if (!params.pOutputBuffer) { SetErrorMessage("pOutputBuffer is NULL"); return Status::InvalidArgument; }
        if (!params.imageA.pData || !params.imageB.pData) { SetErrorMessage("Image data is NULL"); return Status::InvalidArgument; }
        if (params.extent.left < 0 || params.extent.top < 0) {
            SetErrorMessage("Left (%d) and top (%d) must be non-negative", params.extent.left, params.extent.top);
            return Status::OutOfRange;
        }
        if (params.extent.width <= 0 || params.extent.height <= 0) {
            SetErrorMessage("Width (%d) and height (%d) must be positive", params.extent.width, params.extent.height);
            return Status::OutOfRange;
        }
        if ((params.outputOffset & 7u) != 0) {
            SetErrorMessage("outputOffset (%d) must be aligned to 8 bytes", int(params.outputOffset));
            return Status::OutOfRange;
        }
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }
        NtcHipImageDifference p{};
        auto fill = [](NtcHipImage& dst, ImageDesc const& src) {
            dst.data = src.pData; dst.bytes = src.dataSize; dst.pixelStride = src.pixelStride; dst.rowPitch = src.rowPitch;
            dst.width = src.width; dst.height = src.height; dst.format = int32_t(src.channelFormat); dst.numChannels = src.numChannels;
        };
        fill(p.a, params.imageA);
        fill(p.b, params.imageB);
        p.left = params.extent.left; p.top = params.extent.top; p.width = params.extent.width; p.height = params.extent.height;
        p.alphaThreshold = params.alphaThreshold;
        p.useAlphaThreshold = params.useAlphaThreshold ? 1 : 0;
        p.useMSLE = params.useMSLE ? 1 : 0;
        p.outputOffset = params.outputOffset;
        p.output = params.pOutputBuffer; p.outputBytes = params.outputBufferSize;
        if (int r = ntc_hip_ctx_image_difference(m_hip, &p)) return DeviceFailure(r);
        ClearErrorMessage();
        return Status::Ok;
    }

    // src/Context.cpp:80-176
    Status OpenFile(char const* fileName, bool write, IStream** pOutStream) const override
    {
        if (!fileName) { SetErrorMessage("fileName is NULL."); return Status::InvalidArgument; }
        if (!pOutStream) { SetErrorMessage("pOutStream is NULL."); return Status::InvalidArgument; }
        FILE* file = std::fopen(fileName, write ? "wb" : "rb");
        if (!file) { SetErrorMessage("Cannot open file '%s': %s.", fileName, std::strerror(errno)); return Status::FileUnavailable; }
        *pOutStream = MakeObject<FileStream>(m_allocator, file);
        if (!*pOutStream) { std::fclose(file); SetErrorMessage("Failed to allocate the stream object."); return Status::OutOfMemory; }
        return Status::Ok;
    }
    void CloseFile(IStream* stream) const override { DestroyObject(m_allocator, static_cast<FileStream*>(stream)); }
    Status OpenMemory(void* pData, size_t size, IStream** pOutStream) const override { return OpenMemoryStream(pData, size, false, pOutStream); }
    Status OpenReadOnlyMemory(void const* pData, size_t size, IStream** pOutStream) const override
    {
        return OpenMemoryStream(const_cast<void*>(pData), size, true, pOutStream);
    }
    void CloseMemory(IStream* stream) const override { DestroyObject(m_allocator, static_cast<MemoryStream*>(stream)); }

    // src/Context.cpp:296-352
    // src/Context.cpp:864-922
    Status MakeInferenceData(ITextureSetMetadata* textureSet, InferenceWeightType weightType, int firstLatentMipInTexture,
        InferenceData* pOutInferenceData) const override
    {
        if (!pOutInferenceData) { SetErrorMessage("pOutInferenceData is NULL"); return Status::InvalidArgument; }
        TextureSet* const set = dynamic_cast<TextureSet*>(textureSet);
        if (!set) { SetErrorMessage("textureSetMetadata is NULL or points at a wrong object type"); return Status::InvalidArgument; }
        switch (weightType) {
        case InferenceWeightType::GenericInt8: case InferenceWeightType::GenericFP8: case InferenceWeightType::CoopVecFP8: break;
        default:
            SetErrorMessage("Unsupported weightType (%s)", InferenceWeightTypeToString(weightType));
            return Status::Unsupported;
        }
        if (!set->IsInferenceWeightTypeSupported(weightType)) {
            SetErrorMessage("The texture set does not provide %s weights", InferenceWeightTypeToString(weightType));
            return Status::Unsupported;
        }
        if (set->GetNumLatentImages() == 0) {
            SetErrorMessage("This decoder geometry has no shared latent images.");
            return Status::Unsupported;
        }
        std::memset(pOutInferenceData, 0, sizeof(InferenceData));
        set->FillInferenceConstants(weightType, firstLatentMipInTexture, pOutInferenceData->constants);
        ClearErrorMessage();
        return Status::Ok;
    }

    // src/Context.cpp:263-293: everything a file says about a set, without its latents and without a device.
    Status CreateTextureSetMetadataFromStream(IStream* inputStream, ITextureSetMetadata** pOutMetadata) const override
    {
        if (!pOutMetadata) { SetErrorMessage("pOutMetadata is NULL."); return Status::InvalidArgument; }
        *pOutMetadata = nullptr;
        if (!inputStream) { SetErrorMessage("inputStream is NULL."); return Status::InvalidArgument; }
        file::Document document;
        uint64_t binaryChunkOffset = 0, binaryChunkSize = 0;
        if (Status st = LoadFileHeadersFromStream(inputStream, document, binaryChunkOffset, binaryChunkSize); st != Status::Ok) return st;
        TextureSetDesc desc;
        LatentShape shape;
        if (Status st = DeserializeTextureSetDesc(document, desc, shape); st != Status::Ok) return st;
        TextureSet* set = MakeObject<TextureSet>(m_allocator, this, desc, TextureSetFeatures());
        if (!set) { SetErrorMessage("Failed to allocate the texture set object."); return Status::OutOfMemory; }
        Status status = set->Initialize(false);
        if (status == Status::Ok) status = set->LoadFromStreamPostHeader(document, binaryChunkOffset, binaryChunkSize, inputStream, shape, true);
        if (status != Status::Ok) { DestroyObject(m_allocator, set); return status; }
        *pOutMetadata = set;
        ClearErrorMessage();
        return Status::Ok;
    }
    void DestroyTextureSetMetadata(ITextureSetMetadata* textureSetMetadata) const override { DestroyObject(m_allocator, dynamic_cast<TextureSet*>(textureSetMetadata)); }

    Status CreateCompressedTextureSetFromStream(IStream* inputStream, TextureSetFeatures const& features, ITextureSet** pOutTextureSet) const override
    {
        if (!pOutTextureSet) { SetErrorMessage("pOutTextureSet is NULL."); return Status::InvalidArgument; }
        *pOutTextureSet = nullptr;
        if (!inputStream) { SetErrorMessage("inputStream is NULL."); return Status::InvalidArgument; }
        if (!m_deviceAvailable && !m_allowSetsWithoutDevice) {   // src/Context.cpp:311-315
            SetErrorMessage("Cannot create a TextureSet object when no suitable CUDA device is available.");
            return Status::CudaUnavailable;
        }
        file::Document document;
        uint64_t binaryChunkOffset = 0, binaryChunkSize = 0;
        if (Status st = LoadFileHeadersFromStream(inputStream, document, binaryChunkOffset, binaryChunkSize); st != Status::Ok) return st;
        TextureSetDesc desc;
        LatentShape shape;
        if (Status st = DeserializeTextureSetDesc(document, desc, shape); st != Status::Ok) return st;
        ITextureSet* created = nullptr;
        if (Status st = CreateTextureSet(desc, features, &created); st != Status::Ok) return st;
        Status const status = dynamic_cast<TextureSet*>(created)->LoadFromStreamPostHeader(document, binaryChunkOffset, binaryChunkSize, inputStream, shape);
        if (status != Status::Ok) { DestroyTextureSet(created); return status; }
        *pOutTextureSet = created;
        ClearErrorMessage();
        return Status::Ok;
    }
    Status CreateCompressedTextureSetFromMemory(void const* pData, size_t size, TextureSetFeatures const& features, ITextureSet** pOutTextureSet) const override
    {
        IStream* stream = nullptr;
        if (Status st = OpenReadOnlyMemory(pData, size, &stream); st != Status::Ok) return st;
        Status const status = CreateCompressedTextureSetFromStream(stream, features, pOutTextureSet);
        CloseMemory(stream);
        return status;
    }
    Status CreateCompressedTextureSetFromFile(char const* fileName, TextureSetFeatures const& features, ITextureSet** pOutTextureSet) const override
    {
        IStream* stream = nullptr;
        if (Status st = OpenFile(fileName, false, &stream); st != Status::Ok) return st;
        Status const status = CreateCompressedTextureSetFromStream(stream, features, pOutTextureSet);
        CloseFile(stream);
        return status;
    }

private:
    static Status NoGraphicsApi(ComputePassDesc* pOutComputePass)
    {
        if (!pOutComputePass) { SetErrorMessage("pOutComputePass is NULL"); return Status::InvalidArgument; }
        SetErrorMessage("The context was initialized with graphicsApi == None");
        return Status::InvalidArgument;
    }

    Status OpenMemoryStream(void* pData, size_t size, bool readonly, IStream** pOutStream) const
    {
        if (!pData) { SetErrorMessage("pData is NULL."); return Status::InvalidArgument; }
        if (size == 0) { SetErrorMessage("size is 0."); return Status::InvalidArgument; }
        if (!pOutStream) { SetErrorMessage("pOutStream is NULL."); return Status::InvalidArgument; }
        *pOutStream = MakeObject<MemoryStream>(m_allocator, static_cast<uint8_t*>(pData), size, readonly);
        if (!*pOutStream) { SetErrorMessage("Failed to allocate the stream object."); return Status::OutOfMemory; }
        return Status::Ok;
    }

    IAllocator* m_allocator;
    NtcHipContext* m_hip;
    bool m_deviceAvailable;
    mutable bool m_allowSetsWithoutDevice = false;
};

IAllocator* TextureSet::Allocator() const { return m_context->GetAllocator(); }
NtcHipContext* TextureSet::Hip() const { return m_context->GetHip(); }

namespace amd
{
extern "C" {
ITextureSetExtension* GetTextureSetExtension(ITextureSetMetadata* textureSet) { return dynamic_cast<TextureSet*>(textureSet); }
IContextExtension* GetContextExtension(IContext* context) { return dynamic_cast<Context*>(context); }
}
}

extern "C" {

uint32_t GetInterfaceVersion() { return InterfaceVersion; }

// src/PublicFunctions.cpp:62-176
Status CreateContext(IContext** pOutContext, ContextParameters const& params)
{
    ClearErrorMessage();
    if (params.interfaceVersion != InterfaceVersion) {
        SetErrorMessage("Invalid interface version: provided 0x%08x, expected 0x%08x.", params.interfaceVersion, InterfaceVersion);
        return Status::InterfaceMismatch;
    }
    if (!pOutContext) { SetErrorMessage("pOutContext is NULL."); return Status::InvalidArgument; }
    switch (params.graphicsApi) {                            // src/PublicFunctions.cpp:118-153: built without D3D12 and Vulkan
    case GraphicsAPI::None: break;
    case GraphicsAPI::D3D12: SetErrorMessage("This version of LibNTC doesn't support D3D12."); return Status::NotImplemented;
    case GraphicsAPI::Vulkan: SetErrorMessage("This version of LibNTC doesn't support Vulkan."); return Status::NotImplemented;
    default: SetErrorMessage("Invalid graphicsApi (%d).", int(params.graphicsApi)); return Status::InvalidArgument;
    }
    // every context has its own device context: device, stream, working memory (src/PublicFunctions.cpp:84-112)
    NtcHipContext* hip = nullptr;
    if (params.cudaDevice >= 0 && ntc_hip_create(params.cudaDevice, &hip) != 0) {
        SetErrorMessage("%s", ntc_hip_last_error());
        hip = nullptr;
    }
    bool const deviceAvailable = hip != nullptr;
    IAllocator* const allocator = params.pAllocator ? params.pAllocator : &g_defaultAllocator;
    Context* context = MakeObject<Context>(allocator, allocator, hip);
    if (!context) { ntc_hip_destroy(hip); SetErrorMessage("Failed to allocate the context object."); return Status::OutOfMemory; }
    // for host-side checks by programs that know LibNTC's header only (see ntc::amd::IContextExtension)
    if (std::getenv("LIBNTC_ALLOW_TEXTURE_SETS_WITHOUT_DEVICE")) context->AllowTextureSetsWithoutDevice(true);
    *pOutContext = context;
    return deviceAvailable ? Status::Ok : Status::CudaUnavailable;
}

void DestroyContext(IContext* context)
{
    if (!context) return;
    Context* const object = static_cast<Context*>(context);
    DestroyObject(object->GetAllocator(), object);
}

char const* GetLastErrorMessage() { return t_message; }

// Enum names as include/libntc/ntc.h spells them; a value outside the enum is printed as its number
// into a static buffer, as the reference does (src/PublicFunctions.cpp:177-327).
static char const* NameOrNumber(char const* const* names, int count, int value)
{
    static char number[16];
    if (value >= 0 && value < count) return names[value];
    snprintf(number, sizeof number, "%d", value);
    return number;
}

char const* StatusToString(Status status)
{
    static char const* const names[] = {
        "Ok", "InterfaceMismatch", "CudaError", "CudaUnavailable", "FileUnavailable", "FileUnrecognized",
        "FileIncompatible", "Incomplete", "Unsupported", "InternalError", "InvalidArgument", "InvalidData",
        "InvalidState", "IOError", "NotImplemented", "OutOfMemory", "OutOfRange", "ShaderUnavailable", "UnknownError" };
    return NameOrNumber(names, int(sizeof names / sizeof names[0]), int(status));
}

char const* ChannelFormatToString(ChannelFormat format)
{
    static char const* const names[] = { "UNKNOWN", "UNORM8", "UNORM16", "FLOAT16", "FLOAT32", "UINT32" };
    return NameOrNumber(names, 6, int(format));
}

char const* BlockCompressedFormatToString(BlockCompressedFormat format)
{
    static char const* const names[] = { "None", "BC1", "BC2", "BC3", "BC4", "BC5", "BC6", "BC7" };
    return NameOrNumber(names, 8, int(format));
}

char const* ColorSpaceToString(ColorSpace colorSpace)
{
    static char const* const names[] = { "Linear", "sRGB", "HLG" };
    return NameOrNumber(names, 3, int(colorSpace));
}

char const* InferenceWeightTypeToString(InferenceWeightType weightType)
{
    static char const* const names[] = { "Unknown", "GenericInt8", "GenericFP8", "CoopVecFP8" };
    return NameOrNumber(names, 4, int(weightType));
}

char const* CompressionTypeToString(CompressionType type)
{
    static char const* const names[] = { "None", "GDeflate" };
    return NameOrNumber(names, 2, int(type));
}

// src/PublicFunctions.cpp:329-344
size_t GetBytesPerPixelComponent(ChannelFormat format)
{
    switch (format) {
    case ChannelFormat::UNORM8: return 1;
    case ChannelFormat::UNORM16: case ChannelFormat::FLOAT16: return 2;
    case ChannelFormat::FLOAT32: case ChannelFormat::UINT32: return 4;
    default: return 0;
    }
}

// src/PublicFunctions.cpp:346-352
float LossToPSNR(float loss)
{
    return (loss == 0.f) ? std::numeric_limits<float>::infinity() : -10.f * log10f(loss);
}

// src/PublicFunctions.cpp:36-45.  The version of the interface this library follows; branch and
// commit describe this implementation.
VersionInfo GetLibraryVersion()
{
    VersionInfo info;
    info.major = 0; info.minor = 9; info.point = 2;
    info.branch = "mi355x";
    info.commitHash = "";
    return info;
}

// src/PublicFunctions.cpp:354-380: latent grids of every neural LOD plus the Int8 network of the
// 48-64-48-32-16 decoder (one byte per weight, fp32 scale and bias per output).
Status EstimateCompressedTextureSetSize(TextureSetDesc const& textureSetDesc, LatentShape const& latentShape, size_t& outSize)
{
    if (Status st = ValidateTextureSetDesc(textureSetDesc); st != Status::Ok) return st;
    if (Status st = ValidateLatentShape(latentShape); st != Status::Ok) return st;
    if (latentShape.IsEmpty()) { SetErrorMessage("latentShape is empty."); return Status::OutOfRange; }
    int const gs = latentShape.gridSizeScale;
    int const neuralLods = NeuralLodCount(textureSetDesc.width, textureSetDesc.height, textureSetDesc.mips, gs);
    size_t cells = 0;
    for (int lod = 0; lod < neuralLods; ++lod)
        cells += size_t(GridDimension(textureSetDesc.width, lod, gs)) * size_t(GridDimension(textureSetDesc.height, lod, gs));
    size_t const layers = size_t((latentShape.numFeatures + 3) / 4);
    size_t const weights = 48 * 64 + 64 * 48 + 48 * 32 + 32 * 16, outputs = 64 + 48 + 32 + 16;
    outSize = cells * 2 * layers + weights + outputs * 2 * sizeof(float);
    ClearErrorMessage();
    return Status::Ok;
}

// The latent shapes the reference recommends per bit rate (src/PublicFunctions.cpp:382-393), sorted by rate.
namespace
{
struct KnownLatentShape { float bitsPerPixel; LatentShape shape; };
KnownLatentShape const kKnownLatentShapes[] = {
    { 1.11f, { 6, 8 } }, { 1.67f, { 6, 12 } }, { 2.50f, { 4, 8 } }, { 3.75f, { 4, 12 } }, { 5.00f, { 4, 16 } },
    { 6.67f, { 3, 12 } }, { 10.0f, { 2, 8 } }, { 15.0f, { 2, 12 } }, { 20.0f, { 2, 16 } } };
constexpr int kKnownLatentShapeCount = int(sizeof kKnownLatentShapes / sizeof kKnownLatentShapes[0]);
}

int GetKnownLatentShapeCount() { return kKnownLatentShapeCount; }

Status EnumerateKnownLatentShapes(int index, float& outBitsPerPixel, LatentShape& outShape)
{
    if (index < 0 || index >= kKnownLatentShapeCount) {
        SetErrorMessage("Invalid index (%d), must be 0-%d.", index, kKnownLatentShapeCount - 1);
        return Status::OutOfRange;
    }
    outBitsPerPixel = kKnownLatentShapes[index].bitsPerPixel;
    outShape = kKnownLatentShapes[index].shape;
    ClearErrorMessage();
    return Status::Ok;
}

// The known shape nearest to the requested rate, if it lies within 25 % of the request
// (src/PublicFunctions.cpp:415-452).
Status PickLatentShape(float requestedBitsPerPixel, float& outBitsPerPixel, LatentShape& outShape)
{
    if (!(requestedBitsPerPixel > 0.f)) {
        SetErrorMessage("requestedBitsPerPixel (%f) must be positive.", requestedBitsPerPixel);
        return Status::OutOfRange;
    }
    int best = -1;
    float bestDiff = std::numeric_limits<float>::max();
    for (int i = 0; i < kKnownLatentShapeCount; ++i) {
        float const diff = fabsf(kKnownLatentShapes[i].bitsPerPixel - requestedBitsPerPixel);
        if (diff < requestedBitsPerPixel * 0.25f && diff < bestDiff) { best = i; bestDiff = diff; }
    }
    if (best < 0) {
        SetErrorMessage("The provided requestedBitsPerPixel (%f) is out of the supported range.", requestedBitsPerPixel);
        return Status::OutOfRange;
    }
    outBitsPerPixel = kKnownLatentShapes[best].bitsPerPixel;
    outShape = kKnownLatentShapes[best].shape;
    ClearErrorMessage();
    return Status::Ok;
}

// src/PublicFunctions.cpp:454-461: two adjacent neural LODs are read together, so a latent cell of
// `layers` x 2 bytes costs 16 bits x 1.25 per layer, spread over gridSizeScale^2 texels.
float GetLatentShapeBitsPerPixel(LatentShape const& shape)
{
    int const layers = (shape.numFeatures + 3) / 4;
    return float(layers) / float(shape.gridSizeScale * shape.gridSizeScale) * 2.f * 10.f;
}

// 16.48 fixed point -> double (src/PublicFunctions.cpp:463-467).
double DecodeImageDifferenceResult(uint64_t value) { return double(value) * 0x1p-48; }

// BC7 mode bitmap: 9 bits per block (3 bits mode, 6 bits partition), rounded up to whole dwords
// (src/PublicFunctions.cpp:469-473, include/libntc/shaders/BlockCompressConstants.h:24-27).
namespace { constexpr size_t kBc7ModeBits = 9; constexpr uint32_t kBc7Mode0Partition0 = 0x1BF; }

size_t GetBC7ModeBufferSize(int widthInBlocks, int heightInBlocks)
{
    size_t const blocks = size_t(widthInBlocks) * size_t(heightInBlocks);
    return ((blocks * kBc7ModeBits + 31) >> 5) << 2;
}

// src/PublicFunctions.cpp:475-557.  The mode of a BC7 block is the position of the lowest set bit of
// its first byte (8 and above: the reserved mode, treated as 7); the partition index follows the mode
// bit with 4, 6, 6, 6, 3 (rotation + index selector), 2, 0, 6 bits.  Entries are OR-ed into the
// buffer, which the caller provides zeroed.
Status MakeBC7ModeBuffer(int widthInBlocks, int heightInBlocks, void const* blockData, size_t blockDataSize,
    size_t rowPitch, void* modeBuffer, size_t modeBufferSize)
{
    if (!blockData) { SetErrorMessage("blockData is NULL."); return Status::InvalidArgument; }
    if (!modeBuffer) { SetErrorMessage("modeBuffer is NULL."); return Status::InvalidArgument; }
    size_t const bytesPerBlock = 16, minPitch = size_t(widthInBlocks) * bytesPerBlock;
    if (rowPitch < minPitch || rowPitch % bytesPerBlock != 0) {
        SetErrorMessage("Invalid rowPitch (%zu), must be at least %zu and a multiple of %zu.", rowPitch, minPitch, bytesPerBlock);
        return Status::InvalidArgument;
    }
    if (blockDataSize < size_t(heightInBlocks) * rowPitch) {
        SetErrorMessage("Size of BC7 block data (%zu bytes) does not match the expected size (%zu bytes).",
            blockDataSize, size_t(heightInBlocks) * rowPitch);
        return Status::InvalidArgument;
    }
    size_t const needed = GetBC7ModeBufferSize(widthInBlocks, heightInBlocks);
    if (modeBufferSize < needed) {
        SetErrorMessage("Size of BC7 mode buffer (%zu bytes) is smaller than the expected size (%zu bytes).", modeBufferSize, needed);
        return Status::InvalidArgument;
    }
    static uint32_t const partitionMask[8] = { 15, 63, 63, 63, 7, 3, 0, 63 };
    uint8_t const* const blocks = static_cast<uint8_t const*>(blockData);
    uint8_t* const bits = static_cast<uint8_t*>(modeBuffer);
    for (int row = 0; row < heightInBlocks; ++row)
        for (int col = 0; col < widthInBlocks; ++col) {
            uint32_t first;
            std::memcpy(&first, blocks + size_t(row) * rowPitch + size_t(col) * bytesPerBlock, 4);
            uint32_t const mode = first ? std::min(7u, uint32_t(__builtin_ctz(first))) : 7u;
            uint32_t const partition = (first >> (mode + 1)) & partitionMask[mode];
            uint32_t entry = (mode << 6) | partition;
            if (entry == 0) entry = kBc7Mode0Partition0;       // zero stays free to mean "not written"
            size_t const bit = (size_t(row) * size_t(widthInBlocks) + size_t(col)) * kBc7ModeBits;
            bits[bit / 8] |= uint8_t(entry << (bit & 7));
            bits[bit / 8 + 1] |= uint8_t(entry >> (8 - (bit & 7)));
        }
    ClearErrorMessage();
    return Status::Ok;
}

// GDeflate streams are not supported by this library (the reference's codec is an external
// dependency that its tree does not contain): no header.
size_t GetGDeflateHeaderSize(size_t /*uncompressedSize*/) { return 0; }

} // extern "C"

} // namespace ntc
