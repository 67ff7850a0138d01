// libntc_dropin_test.cpp - an application written for LibNTC: it includes nothing but LibNTC's own
// <libntc/ntc.h> (which pulls in wrappers.h) and links against libntc.so.  Built by tests/Makefile against the
// header where it lies in the LibNTC tree, run by tests/test_libntc_dropin.py.
//   libntc_dropin_test walk <file.ntc>
//       no GPU: every virtual of IContext, ITextureSet, ITextureSetMetadata, ITextureMetadata and IStream is
//       called once through the interface pointers (a vtable that does not match the header's declaration
//       order would crash or return nonsense here), statuses checked
//   libntc_dropin_test decode <file.ntc> <outPrefix> <useInt8Weights 0|1>
//       CreateContext -> CreateCompressedTextureSetFromMemory -> Decompress -> ReadChannels of every mip
//       (FLOAT16 pixels, host memory) -> <outPrefix>_mip<N>.bin
#include <libntc/ntc.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#define CHECK(cond) do { if (!(cond)) { std::fprintf(stderr, "FAILED %s:%d: %s\n  last error: %s\n", __FILE__, __LINE__, #cond, ntc::GetLastErrorMessage()); return 1; } } while (0)

static std::vector<unsigned char> readFile(char const* path)
{
    std::vector<unsigned char> data;
    if (FILE* f = std::fopen(path, "rb")) {
        std::fseek(f, 0, SEEK_END); long n = std::ftell(f); std::fseek(f, 0, SEEK_SET);
        data.resize(size_t(n));
        if (std::fread(data.data(), 1, size_t(n), f) != size_t(n)) data.clear();
        std::fclose(f);
    }
    return data;
}

static int walkMetadata(ntc::IContext* ctx, ntc::ITextureSetMetadata* meta, bool fromFile)
{
    using namespace ntc;
    TextureSetDesc const& desc = meta->GetDesc();
    CHECK(desc.width > 0 && desc.height > 0 && desc.channels > 0 && desc.mips > 0);
    LatentShape const& shape = meta->GetLatentShape();
    CHECK(fromFile ? !shape.IsEmpty() : true);
    int const before = meta->GetTextureCount();
    ITextureMetadata* texture = meta->AddTexture();
    CHECK(texture != nullptr && meta->GetTextureCount() == before + 1);
    CHECK(meta->GetTexture(before) == texture);
    CHECK(static_cast<ITextureSetMetadata const*>(meta)->GetTexture(before) == texture);
    CHECK(meta->GetTexture(before + 1) == nullptr);
    {   // ITextureMetadata, every virtual
        texture->SetName("albedo");
        CHECK(std::strcmp(texture->GetName(), "albedo") == 0);
        CHECK(texture->SetChannels(0, 3) == Status::Ok);
        CHECK(texture->SetChannels(desc.channels, 1) == Status::OutOfRange);
        int first = -1, count = -1;
        texture->GetChannels(first, count);
        CHECK(first == 0 && count == 3 && texture->GetFirstChannel() == 0 && texture->GetNumChannels() == 3);
        texture->SetChannelFormat(ChannelFormat::UNORM16);
        CHECK(texture->GetChannelFormat() == ChannelFormat::UNORM16);
        texture->SetBlockCompressedFormat(BlockCompressedFormat::BC7);
        CHECK(texture->GetBlockCompressedFormat() == BlockCompressedFormat::BC7);
        texture->SetRgbColorSpace(ColorSpace::sRGB);
        CHECK(texture->GetRgbColorSpace() == ColorSpace::sRGB);
        texture->SetAlphaColorSpace(ColorSpace::HLG);
        CHECK(texture->GetAlphaColorSpace() == ColorSpace::HLG);
        int const wb = (desc.width + 3) / 4, hb = (desc.height + 3) / 4;
        std::vector<unsigned char> blocks(size_t(wb) * size_t(hb) * 16, 0x40);      // mode 6 everywhere
        CHECK(texture->MakeAndStoreBC7ModeBuffer(0, wb, hb, blocks.data(), blocks.size(), size_t(wb) * 16) == Status::Ok);
        CHECK(texture->MakeAndStoreBC7ModeBuffer(0, wb + 1, hb, blocks.data(), blocks.size(), size_t(wb) * 16) == Status::InvalidArgument);
        void const* modes = nullptr; size_t modesSize = 0;
        texture->GetBC7ModeBuffer(0, &modes, &modesSize);
        CHECK(modes != nullptr && modesSize == GetBC7ModeBufferSize(wb, hb));
        CHECK(texture->GetBC7ModeBufferFootprint(0).rangeInStream.size == 0);       // made here, not stored in a file
    }
    CHECK((meta->GetValidChannelMask() & 7u) == 7u);
    CHECK(meta->GetChannelStorageColorSpace(0) == ColorSpace::Linear || meta->GetChannelStorageColorSpace(0) == ColorSpace::sRGB);
    LatentTextureDesc const lt = meta->GetLatentTextureDesc();
    int const images = meta->GetNumLatentImages();
    CHECK(images == lt.mipLevels);
    LatentTextureFootprint fp;
    if (images > 0) {
        CHECK(lt.width > 0 && lt.height > 0 && lt.arraySize == (shape.numFeatures + 3) / 4);
        CHECK(meta->GetLatentTextureFootprint(0, 0, fp) == Status::Ok && fp.width == lt.width && fp.height == lt.height && fp.rowPitch == size_t(lt.width) * 2);
        CHECK(fromFile ? fp.buffer.rangeInStream.size == size_t(lt.width) * size_t(lt.height) * 2 : fp.buffer.rangeInStream.size == 0);
        int firstMip = -1, lastMip = -1;
        CHECK(meta->GetFusedMipLevels(0, &firstMip, &lastMip) == Status::Ok && firstMip == 0 && lastMip >= 0);
        CHECK(meta->GetMipLevelsForLatentImage(0, &firstMip, &lastMip) == Status::Ok && firstMip == 0);
    }
    CHECK(meta->GetLatentTextureFootprint(images, 0, fp) == Status::OutOfRange);
    CHECK(meta->GetFusedMipLevels(desc.mips, nullptr, nullptr) != Status::Ok);
    CHECK(meta->GetMipLevelsForLatentImage(-1, nullptr, nullptr) != Status::Ok);

    CHECK(meta->IsInferenceWeightTypeSupported(InferenceWeightType::GenericInt8) == fromFile);
    CHECK(!meta->IsInferenceWeightTypeSupported(InferenceWeightType::CoopVecFP8));
    CHECK(meta->GetBestSupportedWeightType() == (fromFile ? InferenceWeightType::GenericInt8 : InferenceWeightType::Unknown));
    void const* weights = nullptr; size_t weightSize = 0, convertedSize = 1;
    if (fromFile) {
        CHECK(meta->GetInferenceWeights(InferenceWeightType::GenericInt8, &weights, &weightSize, &convertedSize) == Status::Ok);
        CHECK(weights != nullptr && weightSize == 9472 && convertedSize == 0);      // src/WeightLayout.cpp:42-49 for 48-64-48-32-16
        CHECK(meta->GetInferenceWeights(InferenceWeightType::GenericFP8, &weights, &weightSize, &convertedSize) == Status::Ok);
        CHECK(weights != nullptr && weightSize == 8608 && convertedSize == 0);      // src/WeightLayout.cpp:51-71
        InferenceData data;
        CHECK(ctx->MakeInferenceData(meta, InferenceWeightType::GenericInt8, 0, &data) == Status::Ok);
        CHECK(data.constants.imageWidth == desc.width && data.constants.imageMips == desc.mips && data.constants.networkWeightOffsets[1] == 48 * 64);
        CHECK(data.constants.networkScaleOffsets[0] == 8192 && data.constants.networkBiasOffsets[0] == 8192 + 640);
        CHECK(ctx->MakeInferenceData(meta, InferenceWeightType::GenericFP8, 0, &data) == Status::Ok);
        CHECK(data.constants.networkBiasOffsets[0] == 8192 && data.constants.networkScaleOffsets[3] == 8192 + 288);
    }
    CHECK(meta->GetInferenceWeights(InferenceWeightType::CoopVecFP8, &weights, &weightSize, &convertedSize) == Status::Unsupported);
    CHECK(ctx->MakeInferenceData(meta, InferenceWeightType::CoopVecFP8, 0, nullptr) == Status::InvalidArgument);
    int dummy = 0, other = 0;
    CHECK(meta->ConvertInferenceWeights(InferenceWeightType::CoopVecFP8, nullptr, &dummy, 0, &other, 0) == Status::InvalidArgument);
    CHECK(meta->ConvertInferenceWeights(InferenceWeightType::CoopVecFP8, &dummy, &dummy, 0, &dummy, 0) == Status::InvalidArgument);
    CHECK(meta->ConvertInferenceWeights(InferenceWeightType::CoopVecFP8, &dummy, &dummy, 0, &other, 0) == Status::Unsupported);
    ShuffleSource mapping[NTC_MAX_CHANNELS];
    for (int ch = 0; ch < NTC_MAX_CHANNELS; ++ch) mapping[ch] = ShuffleSource::Channel(NTC_MAX_CHANNELS - 1 - ch);
    CHECK(meta->ShuffleInferenceOutputs(mapping) == Status::Ok);
    CHECK((meta->GetValidChannelMask() & 0xE000u) == 0xE000u);                      // channels 0..2 now come out as 15..13
    CHECK(meta->ShuffleInferenceOutputs(mapping) == Status::Ok);                    // and back
    CHECK(meta->ShuffleInferenceOutputs(nullptr) == Status::InvalidArgument);

    CHECK(meta->RemoveTexture(texture) == Status::Ok && meta->GetTextureCount() == before);
    CHECK(meta->RemoveTexture(texture) == Status::OutOfRange);
    return 0;
}

static int walk(int argc, char** argv)
{
    using namespace ntc;
    if (argc < 3) { std::fprintf(stderr, "usage: walk <file.ntc>\n"); return 2; }
    std::vector<unsigned char> image = readFile(argv[2]);
    CHECK(!image.empty());
    CHECK(GetInterfaceVersion() == InterfaceVersion);
    VersionInfo const version = GetLibraryVersion();
    CHECK(version.branch != nullptr && version.commitHash != nullptr);
    CHECK(std::strcmp(StatusToString(Status::ShaderUnavailable), "ShaderUnavailable") == 0);
    CHECK(std::strcmp(ChannelFormatToString(ChannelFormat::FLOAT32), "FLOAT32") == 0);
    CHECK(std::strcmp(BlockCompressedFormatToString(BlockCompressedFormat::BC6), "BC6") == 0);
    CHECK(std::strcmp(ColorSpaceToString(ColorSpace::HLG), "HLG") == 0);
    CHECK(std::strcmp(InferenceWeightTypeToString(InferenceWeightType::GenericFP8), "GenericFP8") == 0);
    CHECK(std::strcmp(CompressionTypeToString(CompressionType::GDeflate), "GDeflate") == 0);
    CHECK(GetBytesPerPixelComponent(ChannelFormat::UINT32) == 4 && LossToPSNR(0.1f) == 10.f);
    size_t estimated = 0; float bpp = 0.f; LatentShape picked;
    TextureSetDesc d4k; d4k.width = 4096; d4k.height = 4096; d4k.channels = 16; d4k.mips = 13;
    CHECK(EstimateCompressedTextureSetSize(d4k, LatentShape{ 2, 16 }, estimated) == Status::Ok && estimated > 44000000);
    CHECK(GetKnownLatentShapeCount() > 0 && EnumerateKnownLatentShapes(0, bpp, picked) == Status::Ok);
    CHECK(PickLatentShape(5.f, bpp, picked) == Status::Ok && GetLatentShapeBitsPerPixel(picked) == bpp);
    CHECK(DecodeImageDifferenceResult(1ull << 48) == 1.0 && GetGDeflateHeaderSize(1000) == 0);

    ContextParameters params;
    params.cudaDevice = DisableCudaDevice;
    params.graphicsApi = GraphicsAPI::Vulkan;
    IContext* none = nullptr;
    CHECK(CreateContext(&none, params) == Status::NotImplemented && none == nullptr);
    params.graphicsApi = GraphicsAPI::None;
    ContextWrapper ctx;                                           // wrappers.h
    CHECK(CreateContext(ctx.ptr(), params) == Status::CudaUnavailable && ctx.Get() != nullptr);

    // ---- IContext: streams
    MemoryStreamWrapper memory(ctx);
    CHECK(ctx->OpenReadOnlyMemory(image.data(), image.size(), memory.ptr()) == Status::Ok);
    {   // IStream, every virtual
        unsigned char four[4] = {};
        CHECK(memory->Size() == image.size() && memory->Tell() == 0);
        CHECK(memory->Read(four, 4) && std::memcmp(four, "NTEX", 4) == 0 && memory->Tell() == 4);
        CHECK(!memory->Write(four, 4));                           // read-only
        CHECK(memory->Seek(0) && !memory->Seek(image.size() + 1));
    }
    unsigned char scratch[64] = {};
    MemoryStreamWrapper writable(ctx);
    CHECK(ctx->OpenMemory(scratch, sizeof scratch, writable.ptr()) == Status::Ok && writable->Write("abcd", 4) && scratch[3] == 'd');
    writable.Close();                                             // IContext::CloseMemory
    FileStreamWrapper file(ctx);
    CHECK(ctx->OpenFile(argv[2], false, file.ptr()) == Status::Ok && file->Size() == image.size());
    file.Close();                                                 // IContext::CloseFile
    CHECK(ctx->OpenFile("/nonexistent/file.ntc", false, file.ptr()) == Status::FileUnavailable);

    // ---- IContext: metadata objects (no device needed)
    TextureSetMetadataWrapper meta(ctx);
    CHECK(ctx->CreateTextureSetMetadataFromStream(memory, meta.ptr()) == Status::Ok && meta.Get() != nullptr);
    CHECK(walkMetadata(ctx, meta, true) == 0);
    TextureSetDesc const desc = meta->GetDesc();
    LatentShape const fileShape = meta->GetLatentShape();
    meta.Close();                                                 // IContext::DestroyTextureSetMetadata

    // ---- IContext: texture sets.  Without a device LibNTC creates none (src/Context.cpp:187-191,311-315) ...
    TextureSetFeatures features;
    TextureSetWrapper set(ctx);
    bool const allowed = std::getenv("LIBNTC_ALLOW_TEXTURE_SETS_WITHOUT_DEVICE") != nullptr;
    Status const created = ctx->CreateTextureSet(desc, features, set.ptr());
    CHECK(allowed ? created == Status::Ok : (created == Status::CudaUnavailable && set.Get() == nullptr));
    TextureSetWrapper loaded(ctx);
    Status const fromMemory = ctx->CreateCompressedTextureSetFromMemory(image.data(), image.size(), features, loaded.ptr());
    CHECK(fromMemory == Status::CudaUnavailable && loaded.Get() == nullptr);       // allowed or not: the upload needs a device
    CHECK(ctx->CreateCompressedTextureSetFromFile(argv[2], features, loaded.ptr()) == Status::CudaUnavailable);
    CHECK(memory->Seek(0) && ctx->CreateCompressedTextureSetFromStream(memory, features, loaded.ptr()) == Status::CudaUnavailable);
    CHECK(ctx->CreateCompressedTextureSetFromStream(nullptr, features, loaded.ptr()) == Status::InvalidArgument);

    // ---- IContext: what lies outside the decompression path answers with a status, never a crash
    ISharedTexture* shared = nullptr;
    CHECK(ctx->RegisterSharedTexture(SharedTextureDesc(), &shared) == Status::NotImplemented && shared == nullptr);
    ctx->ReleaseSharedTexture(nullptr);
    IAdaptiveCompressionSession* session = nullptr;
    CHECK(ctx->CreateAdaptiveCompressionSession(&session) == Status::NotImplemented && session == nullptr);
    ctx->DestroyAdaptiveCompressionSession(nullptr);
    ComputePassDesc pass;
    CHECK(ctx->MakeDecompressionComputePass(MakeDecompressionComputePassParameters(), &pass) == Status::InvalidArgument);
    CHECK(std::strstr(GetLastErrorMessage(), "graphicsApi == None") != nullptr);   // src/Context.cpp:461-465
    CHECK(ctx->MakeBlockCompressionComputePass(MakeBlockCompressionComputePassParameters(), &pass) == Status::InvalidArgument);
    CHECK(ctx->MakeImageDifferenceComputePass(MakeImageDifferenceComputePassParameters(), nullptr) == Status::InvalidArgument);
    CHECK(!ctx->IsCooperativeVectorSupported());
    unsigned char copy[8] = {};
    CHECK(ctx->DecompressBuffer(CompressionType::None, "12345678", 8, copy, 8) == Status::Ok && std::memcmp(copy, "12345678", 8) == 0);
    CHECK(ctx->DecompressBuffer(CompressionType::None, "12345678", 8, copy, 4) == Status::InvalidArgument);
    CHECK(ctx->DecompressBuffer(CompressionType::GDeflate, "12345678", 8, copy, 8) == Status::Unsupported);
    CHECK(ctx->DecompressGDeflateOnVulkanGPU(nullptr, nullptr, 0, 0, 0) == Status::Unsupported);

    if (allowed) {
        // ---- ITextureSet, every virtual, on a set without a device
        CHECK(walkMetadata(ctx, set, false) == 0);                // the ITextureSetMetadata part, through the virtual base
        CHECK(set->SetLatentShape(LatentShape{ 7, 16 }) == Status::OutOfRange);
        CHECK(set->SetLatentShape(fileShape) == Status::Ok && set->GetLatentShape() == fileShape);
        CHECK(set->GetNumLatentImages() >= 2 && set->GetNumLatentImages() % 2 == 0);
        CHECK(set->GetOutputStreamSize() == 0);
        LosslessCompressionStats lossless;
        size_t size = sizeof scratch;
        CHECK(set->SaveToStream(memory, &lossless) == Status::NotImplemented);
        CHECK(set->SaveToMemory(scratch, &size, nullptr) == Status::NotImplemented);
        CHECK(set->SaveToFile("/tmp/never_written.ntc") == Status::NotImplemented);
        CHECK(set->ConfigureLosslessCompression(LosslessCompressionSettings()) == Status::NotImplemented);
        CHECK(memory->Seek(0) && set->LoadFromStream(memory) == Status::CudaUnavailable);      // parsed and validated; the upload needs a device
        CHECK(set->GetLatentShape() == fileShape && set->GetTextureCount() >= 0);
        CHECK(set->LoadFromMemory(image.data(), image.size()) == Status::CudaUnavailable);
        CHECK(set->LoadFromFile(argv[2]) == Status::CudaUnavailable);
        CHECK(set->LoadFromMemory(image.data(), 10) != Status::Ok);
        std::vector<unsigned char> pixels(size_t(desc.width) * size_t(desc.height) * 2);
        WriteChannelsParameters wp;
        wp.numChannels = 2; wp.pData = pixels.data(); wp.width = desc.width; wp.height = desc.height; wp.pixelStride = 2; wp.rowPitch = size_t(desc.width) * 2;
        wp.channelFormat = ChannelFormat::UNORM8;
        CHECK(set->WriteChannels(wp) == Status::CudaUnavailable);
        wp.mipLevel = desc.mips;
        CHECK(set->WriteChannels(wp) == Status::OutOfRange);
        ReadChannelsParameters rp;
        rp.numChannels = 2; rp.pOutData = pixels.data(); rp.width = desc.width; rp.height = desc.height; rp.pixelStride = 2; rp.rowPitch = size_t(desc.width) * 2;
        rp.channelFormat = ChannelFormat::UNORM8;
        CHECK(set->ReadChannels(rp) == Status::CudaUnavailable);
        rp.firstChannel = desc.channels;
        CHECK(set->ReadChannels(rp) == Status::OutOfRange);
        CHECK(set->WriteChannelsFromTexture(WriteChannelsFromTextureParameters()) == Status::NotImplemented);
        CHECK(set->ReadChannelsIntoTexture(ReadChannelsIntoTextureParameters()) == Status::NotImplemented);
        CHECK(set->GenerateMips() == Status::CudaUnavailable);
        CHECK(set->BeginCompression(CompressionSettings()) == Status::NotImplemented);
        CompressionStats stats;
        CHECK(set->RunCompressionSteps(&stats) == Status::NotImplemented);
        CHECK(set->FinalizeCompression() == Status::NotImplemented);
        set->AbortCompression();
        DecompressionStats dstats;
        CHECK(set->Decompress(&dstats) == Status::InvalidState);                   // the default asks for the FP8 weights
        CHECK(set->Decompress(&dstats, true) == Status::InvalidState);
        CHECK(set->SetMaskChannelIndex(desc.channels, false) == Status::OutOfRange && set->SetMaskChannelIndex(1, true) == Status::Ok);
        set->SetExperimentalKnob(1.f);
    }
    set.Close();                                                  // IContext::DestroyTextureSet
    std::printf("libntc drop-in walk OK (%s texture sets without a device)\n", allowed ? "with" : "without");
    return 0;
}

static int decode(int argc, char** argv)
{
    using namespace ntc;
    if (argc < 5) { std::fprintf(stderr, "usage: decode <file.ntc> <outPrefix> <useInt8Weights 0|1>\n"); return 2; }
    std::vector<unsigned char> image = readFile(argv[2]);
    std::string const prefix = argv[3];
    bool const useInt8Weights = std::atoi(argv[4]) != 0;
    CHECK(!image.empty());
    ContextWrapper ctx;
    ContextParameters params;
    CHECK(CreateContext(ctx.ptr(), params) == Status::Ok);
    TextureSetFeatures features;
    features.stagingBytesPerPixel = NTC_MAX_CHANNELS * 2;
    TextureSetWrapper set(ctx);
    CHECK(ctx->CreateCompressedTextureSetFromMemory(image.data(), image.size(), features, set.ptr()) == Status::Ok);
    TextureSetDesc const desc = set->GetDesc();
    DecompressionStats stats;
    CHECK(set->Decompress(&stats, useInt8Weights) == Status::Ok);
    CHECK(stats.gpuTimeMilliseconds > 0.f);
    for (int mip = 0; mip < desc.mips; ++mip) {
        ReadChannelsParameters rp;
        rp.page = TextureDataPage::Output;
        rp.mipLevel = mip; rp.firstChannel = 0; rp.numChannels = desc.channels;
        rp.width = std::max(desc.width >> mip, 1); rp.height = std::max(desc.height >> mip, 1);
        rp.pixelStride = size_t(desc.channels) * 2; rp.rowPitch = rp.pixelStride * size_t(rp.width);
        rp.channelFormat = ChannelFormat::FLOAT16;
        rp.addressSpace = AddressSpace::Host;
        std::vector<unsigned char> pixels(rp.rowPitch * size_t(rp.height));
        rp.pOutData = pixels.data();
        CHECK(set->ReadChannels(rp) == Status::Ok);
        FILE* f = std::fopen((prefix + "_mip" + std::to_string(mip) + ".bin").c_str(), "wb");
        CHECK(f != nullptr);
        bool const ok = std::fwrite(pixels.data(), 1, pixels.size(), f) == pixels.size();
        std::fclose(f);
        CHECK(ok);
    }
    {   // a second context in the same process: its own device context and stream; both decode interleaved, without
        // statistics (so without waiting), and read back the same pixels
        ContextWrapper other;
        CHECK(CreateContext(other.ptr(), params) == Status::Ok);
        TextureSetWrapper otherSet(other);
        CHECK(other->CreateCompressedTextureSetFromMemory(image.data(), image.size(), features, otherSet.ptr()) == Status::Ok);
        for (int round = 0; round < 3; ++round) {
            CHECK(set->Decompress(nullptr, useInt8Weights) == Status::Ok);
            CHECK(otherSet->Decompress(nullptr, useInt8Weights) == Status::Ok);
        }
        ReadChannelsParameters rp;
        rp.firstChannel = 0; rp.numChannels = desc.channels; rp.width = desc.width; rp.height = desc.height;
        rp.pixelStride = size_t(desc.channels) * 2; rp.rowPitch = rp.pixelStride * size_t(rp.width);
        rp.channelFormat = ChannelFormat::FLOAT16;
        std::vector<unsigned char> a(rp.rowPitch * size_t(rp.height)), b(a.size());
        rp.pOutData = a.data();
        CHECK(set->ReadChannels(rp) == Status::Ok);
        rp.pOutData = b.data();
        CHECK(otherSet->ReadChannels(rp) == Status::Ok);
        CHECK(a == b);
    }
    std::printf("libntc drop-in decode OK: %d x %d, %d channels, %d mips, %s weights, %.3f ms\n", desc.width, desc.height, desc.channels, desc.mips,
                useInt8Weights ? "Int8" : "FP8", stats.gpuTimeMilliseconds);
    return 0;
}

int main(int argc, char** argv)
{
    if (argc >= 2 && std::strcmp(argv[1], "walk") == 0) return walk(argc, argv);
    if (argc >= 2 && std::strcmp(argv[1], "decode") == 0) return decode(argc, argv);
    std::fprintf(stderr, "usage: libntc_dropin_test walk <file.ntc> | decode <file.ntc> <outPrefix> <useInt8Weights 0|1>\n");
    return 2;
}
