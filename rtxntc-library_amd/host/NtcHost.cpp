// NtcHost.cpp - host side of the decoder behind the interface of ntc_decode.h.
//
// Counterpart of the parts of reference src/Context.cpp, src/TextureSet.cpp,
// src/FeatureGridHost.cpp, src/FeatureGridMath.cpp and src/Errors.cpp that the decompression
// path goes through.  All device work is done by libntc_hip.so through include/ntc_hip.h.
#include "ntc_decode.h"
#include "../../include/ntc_hip.h"

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <limits>
#include <new>
#include <string>
#include <vector>

namespace ntc
{

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

// positionScale / positionLod of a colour mip, src/TextureSet.cpp:456-461
void PositionConstants(NtcHipMipDesc& d)
{
    float const widthScale = float(d.hrWidth) / float(d.width);
    float const heightScale = float(d.hrHeight) / float(d.height);
    d.positionScale = 0.5f * std::max(widthScale, heightScale);
    d.positionLod = std::max(-1.f, std::min(1.f, 0.25f * log2f(d.positionScale)));
}
} // namespace

class Context;

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
private:
    TextureSetDesc const& m_setDesc;
    std::string m_name;
    int m_firstChannel = 0, m_numChannels = 0;
};

class TextureSet final : public ITextureSet
{
public:
    TextureSet(Context const* context, TextureSetDesc const& desc, TextureSetFeatures const& features)
        : m_context(context), m_desc(desc), m_features(features) {}

    ~TextureSet() override
    {
        ClearTextureMetadata();
        ReleaseDevice(m_textureData);
        ReleaseDevice(m_textureDataOut);
        ReleaseDevice(m_staging);
        ReleaseDevice(m_latents);
        ReleaseDevice(m_weights);
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
            if (int r = ntc_hip_alloc(&m_textureData, m_textureBytes)) return AllocationFailure(r, "texture data", m_textureBytes);
            // A second page keeps the reference image apart from the decoded one (src/TextureSet.cpp:103-124).
            if (m_features.separateRefOutData)
                if (int r = ntc_hip_alloc(&m_textureDataOut, m_textureBytes)) return AllocationFailure(r, "texture data (output)", m_textureBytes);
            if (m_stagingBytes)
                if (int r = ntc_hip_alloc(&m_staging, m_stagingBytes)) return AllocationFailure(r, "staging", m_stagingBytes);
        }
        return Status::Ok;
    }

    TextureSetDesc const& GetDesc() const override { return m_desc; }
    LatentShape const& GetLatentShape() const override { return m_latentShape; }
    ITextureMetadata* AddTexture() override
    {
        TextureMetadata* t = new (std::nothrow) TextureMetadata(m_desc);
        if (t) m_textures.push_back(t);
        return t;
    }
    Status RemoveTexture(ITextureMetadata* texture) override
    {
        auto it = std::find(m_textures.begin(), m_textures.end(), texture);
        if (it == m_textures.end()) { SetErrorMessage("The texture does not belong to this texture set."); return Status::OutOfRange; }
        delete *it;
        m_textures.erase(it);
        return Status::Ok;
    }
    void ClearTextureMetadata() override { for (TextureMetadata* t : m_textures) delete t; m_textures.clear(); }
    int GetTextureCount() const override { return int(m_textures.size()); }
    ITextureMetadata* GetTexture(int index) override { return (index >= 0 && index < int(m_textures.size())) ? m_textures[size_t(index)] : nullptr; }

    // src/TextureSetMetadata.cpp:807-832 (no output shuffling here)
    uint32_t GetValidChannelMask() const override
    {
        uint32_t mask = 0;
        for (TextureMetadata const* t : m_textures) {
            int first, count;
            t->GetChannels(first, count);
            mask |= ((1u << count) - 1u) << first;
        }
        return mask;
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
        if (!newShape.IsEmpty()) {
            if (newShape.numFeatures <= 0 || newShape.numFeatures > 16 || (newShape.numFeatures % 4) != 0) {
                SetErrorMessage("Invalid LatentShape: numFeatures (%d) must be a positive multiple of %d up to %d.",
                    newShape.numFeatures, 4, 16);
                return Status::OutOfRange;
            }
            if (newShape.gridSizeScale < 1 || newShape.gridSizeScale > 6) {
                SetErrorMessage("Invalid LatentShape: gridSizeScale (%d) must be between 1 and 6.", newShape.gridSizeScale);
                return Status::OutOfRange;
            }
        }
        m_latentShape = newShape;
        if (newShape.IsEmpty()) return ResetShape();
        m_preset = DecoderPreset::LibNTC092;
        return Rebuild();
    }

    uint64_t GetLatentDataSize() const override { return m_state == NetworkState::Empty ? 0 : m_latentBytes; }
    uint64_t GetWeightDataSize() const override { return m_state == NetworkState::Empty ? 0 : m_weightLayout.bufferSize; }

    Status SetLatentData(void const* data, size_t size) override { return Upload(data, size, m_latentBytes, m_latents, "latent", m_haveLatents); }
    Status SetWeightData(void const* data, size_t size) override { return Upload(data, size, m_weightLayout.bufferSize, m_weights, "weight", m_haveWeights); }

    Status Decompress(DecompressionStats* pOutStats, bool /*useInt8Weights*/) override
    {
        if (m_state != NetworkState::Complete) {
            SetErrorMessage("Invalid network state for Decompress (%s), must be Complete.", NetworkStateToString(m_state));
            return Status::InvalidState;
        }
        if (pOutStats) { *pOutStats = DecompressionStats(); std::fill_n(pOutStats->perChannelLoss, 16, 0.f); std::fill_n(pOutStats->perMipLoss, 16, 0.f); }
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }

        // Losses need the reference image to survive the decode: decode into a second page.
        uint32_t const validMask = GetValidChannelMask();
        bool const lazyOutPage = validMask != 0 && !m_textureDataOut;
        if (lazyOutPage)
            if (int r = ntc_hip_alloc(&m_textureDataOut, m_textureBytes)) return AllocationFailure(r, "texture data (output)", m_textureBytes);
        void* const outPage = m_textureDataOut ? m_textureDataOut : m_textureData;   // src/TextureSet.cpp:1799-1802

        NtcHipTextureSet set{};
        set.spec = m_spec;
        set.numMips = m_desc.mips;
        set.numChannels = m_desc.channels;
        set.outputFormat = NTC_HIP_OUT_FP16_PLANAR_PAIRS;
        set.latents = m_latents; set.latentsBytes = m_latentBytes;
        set.weights = m_weights; set.weightsBytes = m_weightLayout.bufferSize;
        set.output = outPage; set.outputBytes = m_textureBytes;
        for (int mip = 0; mip < m_desc.mips; ++mip) {
            set.mips[mip] = m_mips[mip];
            set.mips[mip].outOffset = m_mipOffsets[mip] * uint64_t(m_desc.channels) * 2u;   // src/TextureSet.cpp:1804
        }
        // The reference brackets its per-mip loop with events only when statistics are asked
        // for, and otherwise returns without waiting (src/TextureSet.cpp:1772-1780,1866-1882).
        if (pOutStats) {
            float ms = 0.f;
            if (int r = ntc_hip_decode_timed(&set, 1, 1, &ms)) return DeviceFailure(r);
            pOutStats->gpuTimeMilliseconds = ms;
        } else if (int r = ntc_hip_decode(&set, 1)) {
            return DeviceFailure(r);
        }

        // Per-channel / per-mip / overall mean squared error, weighted by pixel count exactly as
        // src/TextureSet.cpp:1833-1863,1884-1892 combine them.
        if (validMask != 0 && pOutStats) {
            int validChannels = 0;
            for (int ch = 0; ch < m_desc.channels; ++ch) if (validMask & (1u << ch)) ++validChannels;
            double perChannel[16] = {};
            double overall = 0.0, pixels = 0.0;
            for (int mip = 0; mip < m_desc.mips; ++mip) {
                uint64_t const offset = m_mipOffsets[mip] * uint64_t(m_desc.channels) * 2u;
                float mse[16];
                if (int r = ntc_hip_image_loss(static_cast<uint8_t const*>(outPage) + offset, static_cast<uint8_t const*>(m_textureData) + offset,
                                               m_textureBytes - offset, m_mips[mip].width, m_mips[mip].height, m_desc.channels, validMask, mse))
                    return DeviceFailure(r);
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
            pOutStats->overallLoss = float(overall / pixels);
            for (int ch = 0; ch < 16; ++ch) pOutStats->perChannelLoss[ch] = float(perChannel[ch] / pixels);
        }
        // Without separateRefOutData both pages are one memory in the reference and the decode
        // overwrites the reference image; keep that: the decoded page becomes the only page.
        if (lazyOutPage) {
            if (int r = ntc_hip_synchronize()) return DeviceFailure(r);
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
        if (params.srcColorSpaces || params.dstColorSpaces) { SetErrorMessage("Non-linear colour spaces are not supported."); return Status::Unsupported; }
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }
        if (fromHost)
            if (int r = ntc_hip_upload(m_staging, params.pData, sizeToCopy)) return DeviceFailure(r);
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
        wc.firstChannel = params.firstChannel; wc.numChannels = params.numChannels;
        if (int r = ntc_hip_write_channels(&wc)) return DeviceFailure(r);
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
        if (params.useDithering || params.dstColorSpaces) {
            SetErrorMessage("Dithering and non-linear destination colour spaces are not supported.");
            return Status::Unsupported;
        }
        if (!m_deviceAvailable) { SetErrorMessage("No HIP device is available to this context."); return Status::CudaUnavailable; }

        // Rows the copy does not fully overwrite must not carry garbage to the client (src/TextureSet.cpp:936-946).
        if (toHost && params.rowPitch > params.pixelStride * size_t(params.width))
            if (int r = ntc_hip_memset(m_staging, 0, sizeToCopy)) return DeviceFailure(r);

        NtcHipReadChannels rc{};
        // GetTextureDataSlice: the output page when it exists and is asked for (src/TextureSet.cpp:1961-1964)
        void const* const page = (params.page == TextureDataPage::Output && m_textureDataOut) ? m_textureDataOut : m_textureData;
        rc.planarPairs = static_cast<uint8_t const*>(page) + m_mipOffsets[params.mipLevel] * uint64_t(m_desc.channels) * 2u;
        rc.planarBytes = uint64_t(mipWidth) * uint64_t(mipHeight) * uint64_t(m_desc.channels) * 2u;
        rc.width = mipWidth; rc.height = mipHeight;
        rc.setChannels = m_desc.channels;
        rc.firstChannel = params.firstChannel; rc.numChannels = params.numChannels;
        rc.dst = toHost ? m_staging : params.pOutData;
        rc.dstBytes = toHost ? m_stagingBytes : sizeToCopy;
        rc.format = int(params.channelFormat);
        rc.pixelStride = params.pixelStride; rc.rowPitch = params.rowPitch;
        if (int r = ntc_hip_read_channels(&rc)) return DeviceFailure(r);
        if (toHost)
            if (int r = ntc_hip_download(params.pOutData, m_staging, sizeToCopy)) return DeviceFailure(r);
        ClearErrorMessage();
        return Status::Ok;
    }

private:
    // src/TextureSet.cpp:1914-1956, plus what this library cannot do (resizing copies)
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
        if (GetBytesPerPixelComponent(format) == 0) { SetErrorMessage("Unknown channel format %d.", int(format)); return Status::InvalidArgument; }
        int const mipWidth = std::max(m_desc.width >> mipLevel, 1), mipHeight = std::max(m_desc.height >> mipLevel, 1);
        if (width != mipWidth || height != mipHeight) {
            SetErrorMessage("Resizing %s are not supported: the image must be %dx%d for mip %d.", what, mipWidth, mipHeight, mipLevel);
            return Status::Unsupported;
        }
        return Status::Ok;
    }

    Status AllocationFailure(int code, char const* what, uint64_t bytes)
    {
        if (code > 0) { SetErrorMessage("Failed to allocate %llu bytes of device memory for the %s buffer.", (unsigned long long)bytes, what); return Status::OutOfMemory; }
        return DeviceFailure(code);
    }

    void ReleaseDevice(void*& p) { if (p) { (void)ntc_hip_free(p); p = nullptr; } }

    Status ResetShape()
    {
        ReleaseDevice(m_latents); ReleaseDevice(m_weights);
        m_latentBytes = 0; m_haveLatents = m_haveWeights = false;
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
        ReleaseDevice(m_latents); ReleaseDevice(m_weights);
        m_haveLatents = m_haveWeights = false;
        if (m_deviceAvailable) {
            if (int r = ntc_hip_alloc(&m_latents, m_latentBytes)) return AllocationFailure(r, "latent", m_latentBytes);
            if (int r = ntc_hip_alloc(&m_weights, m_weightLayout.bufferSize)) return AllocationFailure(r, "MLP weights", m_weightLayout.bufferSize);
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
        static int const sharedMips[] = { 2, 3, 3, 3, 4, 4 };
        int const gs = m_latentShape.gridSizeScale;
        auto neuralOf = [&](int lod, int count) { return std::max(0, std::min((lod - sharedMips[gs - 1] + 2) & ~1, count - 2)); };
        auto gridDim = [&](int dim, int nlod) { return std::max((dim / gs) >> nlod, 1); };
        int const minGrid = int(float(std::min(m_desc.width, m_desc.height)) / float(gs));
        int neuralLods = std::max(2, int(1.f + std::floor(std::log2(float(minGrid))))) & ~1;
        neuralLods = std::min(neuralLods, neuralOf(m_desc.mips - 1, 8) + 2);
        uint64_t const layers = uint64_t((m_latentShape.numFeatures + 3) / 4);
        std::vector<uint64_t> offset(size_t(neuralLods) + 1, 0);
        for (int n = 0; n < neuralLods; ++n)
            offset[size_t(n) + 1] = offset[size_t(n)] + uint64_t(gridDim(m_desc.width, n)) * uint64_t(gridDim(m_desc.height, n)) * 2u * layers;
        m_latentBytes = offset[size_t(neuralLods)];
        for (int mip = 0; mip < m_desc.mips; ++mip) {
            NtcHipMipDesc& d = m_mips[mip];
            d = NtcHipMipDesc{};
            int const nlod = neuralOf(mip, neuralLods);
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
        if (int r = ntc_hip_upload(device, data, size)) return DeviceFailure(r);
        have = true;
        if (m_haveLatents && m_haveWeights) m_state = NetworkState::Complete;
        ClearErrorMessage();
        return Status::Ok;
    }

    Context const* m_context;
    TextureSetDesc m_desc;
    TextureSetFeatures m_features;
    LatentShape m_latentShape = LatentShape::Empty();
    DecoderPreset m_preset = DecoderPreset::LibNTC092;
    NetworkState m_state = NetworkState::Empty;
    NtcHipDecoderSpec m_spec{};
    NtcHipWeightLayout m_weightLayout{};
    NtcHipMipDesc m_mips[NTC_HIP_MAX_MIPS]{};
    uint64_t m_mipOffsets[NTC_HIP_MAX_MIPS + 1]{};
    uint64_t m_textureBytes = 0, m_stagingBytes = 0, m_latentBytes = 0;
    std::vector<TextureMetadata*> m_textures;
    void* m_textureData = nullptr;      // reference page (and the only page without separateRefOutData)
    void* m_textureDataOut = nullptr;   // output page
    void* m_staging = nullptr;
    void* m_latents = nullptr;
    void* m_weights = nullptr;
    bool m_deviceAvailable = false, m_haveLatents = false, m_haveWeights = false, m_decompressed = false;
};

class Context final : public IContext
{
public:
    explicit Context(bool deviceAvailable) : m_deviceAvailable(deviceAvailable) {}

    // src/Context.cpp:235-261 with the descriptor rules of src/TextureSetMetadata.cpp:1161-1178
    Status CreateTextureSet(TextureSetDesc const& desc, TextureSetFeatures const& features, ITextureSet** pOutTextureSet) const override
    {
        if (!pOutTextureSet) { SetErrorMessage("pOutTextureSet is NULL."); return Status::InvalidArgument; }
        *pOutTextureSet = nullptr;
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
        TextureSet* set = new (std::nothrow) TextureSet(this, desc, features);
        if (!set) { SetErrorMessage("Failed to allocate the texture set object."); return Status::OutOfMemory; }
        Status const status = set->Initialize(m_deviceAvailable);
        if (status != Status::Ok) { delete set; return status; }
        *pOutTextureSet = set;
        ClearErrorMessage();
        return Status::Ok;
    }

    void DestroyTextureSet(ITextureSet* textureSet) const override { delete textureSet; }
    bool IsCudaAvailable() const override { return m_deviceAvailable; }

private:
    bool m_deviceAvailable;
};

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
    bool deviceAvailable = false;
    if (params.cudaDevice >= 0) {
        if (ntc_hip_init(params.cudaDevice) == 0) deviceAvailable = true;
        else SetErrorMessage("%s", ntc_hip_last_error());
    }
    Context* context = new (std::nothrow) Context(deviceAvailable);
    if (!context) { SetErrorMessage("Failed to allocate the context object."); return Status::OutOfMemory; }
    *pOutContext = context;
    return deviceAvailable ? Status::Ok : Status::CudaUnavailable;
}

void DestroyContext(IContext* context) { delete context; }

char const* GetLastErrorMessage() { return t_message; }

char const* StatusToString(Status status)
{
    static char const* const names[] = {
        "Ok", "InterfaceMismatch", "CudaError", "CudaUnavailable", "FileUnavailable", "FileUnrecognized",
        "FileIncompatible", "Incomplete", "Unsupported", "InternalError", "InvalidArgument", "InvalidData",
        "InvalidState", "IOError", "NotImplemented", "OutOfMemory", "OutOfRange", "ShaderUnavailable", "UnknownError" };
    int const i = int(status);
    return (i >= 0 && i < int(sizeof names / sizeof names[0])) ? names[i] : "Invalid";
}

char const* ChannelFormatToString(ChannelFormat format)
{
    switch (format) {
    case ChannelFormat::UNORM8: return "UNORM8";
    case ChannelFormat::UNORM16: return "UNORM16";
    case ChannelFormat::FLOAT16: return "FLOAT16";
    case ChannelFormat::FLOAT32: return "FLOAT32";
    case ChannelFormat::UINT32: return "UINT32";
    default: return "UNKNOWN";
    }
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

} // extern "C"

} // namespace ntc
