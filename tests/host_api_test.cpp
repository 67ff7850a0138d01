// host_api_test.cpp - drives the C++ host layer (rtxntc-library_amd/host/ntc_decode.h) the way an
// application drives LibNTC.  Built by tests/Makefile, run by tests/test_host_api.py.
//   host_api_test cpu
//       host-only checks (no GPU): status codes, messages, state machine, sizes
//   host_api_test decode <preset> <w> <h> <mips> <channels> <gridScale> <features> <latents> <weights> <outPrefix>
//       loads raw latents/weights, decompresses, reads every mip back as UNORM8 (host address
//       space) and FLOAT16 (device address space is exercised through a second read), writes files
//   host_api_test loss <preset> <w> <h> <mips> <channels> <gridScale> <features> <latents> <weights> <refPrefix> <separate 0|1>
//                      [<maskChannel> <discardMaskedOut 0|1> <withStats 0|1>]
//       registers two textures (channels 0..2 and 4..5), writes <refPrefix>_mip<N>.bin (FLOAT32 pixels,
//       all channels) as the reference image, decompresses twice and prints the loss statistics
//   host_api_test shuffle <preset> <w> <h> <channels> <gridScale> <features> <latents> <weights>
//       ShuffleInferenceOutputs / GetInferenceWeights: decodes with the loaded weights, shuffles, decodes
//       again with the weights GetInferenceWeights returns and compares the channels
//   host_api_test genmips <w> <h> <channels> <mips> <image> <outPrefix>
//       WriteChannels from an image of twice the size, GenerateMips, reference page of every mip to files
//   host_api_test imagediff
//       IContext::ComputeImageDifference on images with exactly known differences
//   host_api_test load <file> <device 0|1> [<w> <h> <channels> <mips>]
//       loads an NTC file: with dimensions through CreateTextureSet + LoadFromFile, without through
//       CreateCompressedTextureSetFromFile; prints the status, the message and what the set holds
//   host_api_test decodefile <file> <outPrefix>
//       CreateCompressedTextureSetFromMemory -> Decompress -> every mip as FLOAT16 pixels to files
#include "../rtxntc-library_amd/host/ntc_decode.h"     // LibNTC's own <libntc/ntc.h> plus the ntc::amd additions
#include "../include/ntc_hip.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

using namespace ntc;
using namespace ntc::amd;

// The ntc::amd additions of an object of this library.
static ITextureSetExtension* X(ITextureSetMetadata* set) { return GetTextureSetExtension(set); }
static IContextExtension* X(IContext* context) { return GetContextExtension(context); }

// This program's own device buffers live on the C ABI's default context; a libntc context works on a stream of
// its own, so its results are waited for before they are fetched.
static int syncedDownload(IContext* context, void* dst, void const* src, size_t bytes)
{
    if (X(context)->Synchronize() != Status::Ok) return -1;
    return ntc_hip_download(dst, src, bytes);
}

#define CHECK(cond) do { if (!(cond)) { std::fprintf(stderr, "FAILED %s:%d: %s\n  last error: %s\n", __FILE__, __LINE__, #cond, GetLastErrorMessage()); return 1; } } while (0)

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
static bool writeFile(std::string const& path, void const* p, size_t n)
{
    FILE* f = std::fopen(path.c_str(), "wb");
    if (!f) return false;
    bool ok = std::fwrite(p, 1, n, f) == n;
    std::fclose(f);
    return ok;
}

// Counts what the library takes from and returns to a caller's allocator.
struct CountingAllocator final : IAllocator
{
    size_t allocations = 0, releases = 0, liveBytes = 0;
    bool sizesMatch = true;
    std::vector<std::pair<void*, size_t>> live;
    void* Allocate(size_t size) override
    {
        void* const p = std::malloc(size);
        if (p) { ++allocations; liveBytes += size; live.emplace_back(p, size); }
        return p;
    }
    void Deallocate(void* ptr, size_t size) override
    {
        for (size_t i = 0; i < live.size(); ++i)
            if (live[i].first == ptr) {
                if (live[i].second != size) sizesMatch = false;
                liveBytes -= live[i].second;
                live.erase(live.begin() + long(i));
                ++releases;
                std::free(ptr);
                return;
            }
        sizesMatch = false;     // not ours
    }
};

// Public objects come from the allocator given in ContextParameters and go back to it with the size they
// were allocated with (include/libntc/ntc.h:76-87,1284-1287, src/Context.cpp:201-233,263-293).
static int allocatorChecks()
{
    CountingAllocator allocator;
    IContext* ctx = nullptr;
    ContextParameters params; params.cudaDevice = DisableCudaDevice; params.pAllocator = &allocator;
    CHECK(CreateContext(&ctx, params) == Status::CudaUnavailable && ctx != nullptr);
    CHECK(allocator.allocations == 1);
    TextureSetDesc desc; desc.width = 64; desc.height = 64; desc.channels = 4; desc.mips = 1;
    ITextureSet* set = nullptr;
    // without a device LibNTC creates no texture sets (src/Context.cpp:187-191) ...
    CHECK(ctx->CreateTextureSet(desc, TextureSetFeatures(), &set) == Status::CudaUnavailable && set == nullptr && allocator.allocations == 1);
    X(ctx)->AllowTextureSetsWithoutDevice(true);              // ... unless told to, for checks like these
    CHECK(ctx->CreateTextureSet(desc, TextureSetFeatures(), &set) == Status::Ok && allocator.allocations == 2);
    ITextureMetadata* a = set->AddTexture();
    ITextureMetadata* b = set->AddTexture();
    CHECK(a && b && allocator.allocations == 4 && allocator.releases == 0);
    CHECK(set->RemoveTexture(a) == Status::Ok && allocator.releases == 1);
    unsigned char bytes[16] = {};
    IStream* stream = nullptr;
    CHECK(ctx->OpenReadOnlyMemory(bytes, sizeof bytes, &stream) == Status::Ok && allocator.allocations == 5);
    ctx->CloseMemory(stream);
    CHECK(allocator.releases == 2);
    desc.width = 0;                                           // a set that fails validation leaves nothing behind
    ITextureSet* bad = nullptr;
    CHECK(ctx->CreateTextureSet(desc, TextureSetFeatures(), &bad) != Status::Ok && bad == nullptr);
    ctx->DestroyTextureSet(set);                              // takes texture b with it
    CHECK(allocator.releases == 4 && allocator.live.size() == 1);
    DestroyContext(ctx);
    CHECK(allocator.allocations == allocator.releases && allocator.liveBytes == 0 && allocator.live.empty() && allocator.sizesMatch);
    DestroyContext(nullptr);                                  // allowed (src/PublicFunctions.cpp:164-167)
    return 0;
}

static int cpuChecks()
{
    CHECK(allocatorChecks() == 0);
    {   // BC7 mode maps kept with a texture (include/libntc/ntc.h:437-453)
        IContext* c = nullptr; ContextParameters cp; cp.cudaDevice = DisableCudaDevice;
        (void)CreateContext(&c, cp);
        CHECK(c != nullptr);
        X(c)->AllowTextureSetsWithoutDevice(true);
        ITextureSet* set = nullptr;
        TextureSetDesc desc; desc.width = 64; desc.height = 40; desc.channels = 4; desc.mips = 3;
        CHECK(c->CreateTextureSet(desc, TextureSetFeatures(), &set) == Status::Ok);
        ITextureMetadata* t = set->AddTexture();
        CHECK(t != nullptr);
        void const* data = reinterpret_cast<void const*>(1); size_t size = 1;
        t->GetBC7ModeBuffer(1, &data, &size);
        CHECK(data == nullptr && size == 0 && t->GetBC7ModeBufferFootprint(1).rangeInStream.size == 0);
        // mip 1 is 32 x 20 pixels = 8 x 5 blocks; block n gets mode n % 8 and a partition from n
        std::vector<uint32_t> blocks(8 * 5 * 4 + 4, 0);
        for (uint32_t n = 0; n < 40; ++n) blocks[n * 4] = (1u << (n % 8)) | ((n * 7u % 64u) << (n % 8 + 1));
        CHECK(t->MakeAndStoreBC7ModeBuffer(1, 8, 5, blocks.data(), 40 * 16, 8 * 16) == Status::Ok);
        t->GetBC7ModeBuffer(1, &data, &size);
        std::vector<uint8_t> direct(GetBC7ModeBufferSize(8, 5), 0);
        CHECK(MakeBC7ModeBuffer(8, 5, blocks.data(), 40 * 16, 8 * 16, direct.data(), direct.size()) == Status::Ok);
        CHECK(data != nullptr && size == direct.size() && std::memcmp(data, direct.data(), size) == 0);
        CHECK(size == ((40 * 9 + 31) / 32) * 4);
        t->GetBC7ModeBuffer(0, &data, &size);
        CHECK(data == nullptr && size == 0);
        CHECK(t->MakeAndStoreBC7ModeBuffer(1, 8, 4, blocks.data(), 40 * 16, 8 * 16) == Status::InvalidArgument);
        CHECK(std::strstr(GetLastErrorMessage(), "do not match the expected dimensions (8 x 5)") != nullptr);
        CHECK(t->MakeAndStoreBC7ModeBuffer(3, 2, 2, blocks.data(), 40 * 16, 8 * 16) == Status::OutOfRange);
        CHECK(t->MakeAndStoreBC7ModeBuffer(1, 8, 5, blocks.data(), 39 * 16, 8 * 16) == Status::InvalidArgument);   // too little block data
        t->GetBC7ModeBuffer(1, &data, &size);
        CHECK(data == nullptr && size == 0);                                                                       // the failed call discarded the old map
        c->DestroyTextureSet(set);
        DestroyContext(c);
    }

    IContext* ctx = nullptr;
    ContextParameters params;
    params.interfaceVersion = 0x12345678;
    CHECK(CreateContext(&ctx, params) == Status::InterfaceMismatch);
    CHECK(std::strstr(GetLastErrorMessage(), "Invalid interface version") != nullptr);
    params = ContextParameters();
    CHECK(CreateContext(nullptr, params) == Status::InvalidArgument);
    params.cudaDevice = DisableCudaDevice;
    CHECK(CreateContext(&ctx, params) == Status::CudaUnavailable);     // ... and still a usable context
    CHECK(ctx != nullptr && !X(ctx)->IsDeviceAvailable());
    X(ctx)->AllowTextureSetsWithoutDevice(true);
    CHECK(GetInterfaceVersion() == InterfaceVersion);
    CHECK(std::strcmp(StatusToString(Status::OutOfRange), "OutOfRange") == 0);
    CHECK(std::strcmp(StatusToString(Status::CudaUnavailable), "CudaUnavailable") == 0);
    CHECK(GetBytesPerPixelComponent(ChannelFormat::FLOAT16) == 2 && GetBytesPerPixelComponent(ChannelFormat::UNKNOWN) == 0);
    CHECK(LossToPSNR(0.01f) == 20.f);

    ITextureSet* set = nullptr;
    TextureSetDesc desc;                       // all zero
    TextureSetFeatures features;
    CHECK(ctx->CreateTextureSet(desc, features, &set) == Status::OutOfRange && set == nullptr);
    desc.width = 4096; desc.height = 4096; desc.channels = 17; desc.mips = 13;
    CHECK(ctx->CreateTextureSet(desc, features, &set) == Status::OutOfRange);
    CHECK(std::strstr(GetLastErrorMessage(), "too many channels") != nullptr);
    desc.channels = 15;
    CHECK(ctx->CreateTextureSet(desc, features, nullptr) == Status::InvalidArgument);
    CHECK(ctx->CreateTextureSet(desc, features, &set) == Status::Ok && set != nullptr);
    CHECK(set->GetDesc().channels == 16);       // rounded up to even (src/TextureSet.cpp:86)
    CHECK(set->GetLatentShape().IsEmpty() && set->GetValidChannelMask() == 0);
    CHECK(X(set)->GetLatentDataSize() == 0);

    // Decompress on an empty set: InvalidState (src/TextureSet.cpp:1666-1673)
    CHECK(set->Decompress(nullptr, true) == Status::InvalidState);
    CHECK(std::strstr(GetLastErrorMessage(), "Invalid network state for Decompress") != nullptr);

    LatentShape shape; shape.gridSizeScale = 7; shape.numFeatures = 16;
    CHECK(set->SetLatentShape(shape) == Status::OutOfRange);
    CHECK(std::strstr(GetLastErrorMessage(), "gridSizeScale (7) must be between 1 and 6") != nullptr);
    shape.gridSizeScale = 2; shape.numFeatures = 10;
    CHECK(set->SetLatentShape(shape) == Status::OutOfRange);
    shape.numFeatures = 16;
    CHECK(set->SetLatentShape(shape) == Status::Ok);
    CHECK(X(set)->GetWeightDataSize() == 9472);                 // src/WeightLayout.cpp, 48-64-48-32-16
    CHECK(X(set)->GetLatentDataSize() == 44738560ull);          // 4096^2, grid scale 2, 16 features, 13 mips
    CHECK(set->Decompress(nullptr, true) == Status::InvalidState); // shape set, no data yet
    // which colour mips share latent images (4096^2, grid scale 2: mips 0-2 -> LOD 0, 3-4 -> 2, 5-6 -> 4, 7-12 -> 6;
    // eight neural LODs, the odd ones serve as the low-resolution partner only)
    {
        CHECK(set->GetNumLatentImages() == 8);
        LatentTextureDesc const lt = set->GetLatentTextureDesc();
        CHECK(lt.width == 2048 && lt.height == 2048 && lt.arraySize == 4 && lt.mipLevels == 8);
        int first = -1, last = -1;
        CHECK(set->GetFusedMipLevels(0, &first, &last) == Status::Ok && first == 0 && last == 2);
        CHECK(set->GetFusedMipLevels(4, &first, &last) == Status::Ok && first == 3 && last == 4);
        CHECK(set->GetFusedMipLevels(9, &first, nullptr) == Status::Ok && first == 7);
        CHECK(set->GetFusedMipLevels(12, nullptr, &last) == Status::Ok && last == 12);
        CHECK(set->GetFusedMipLevels(13, &first, &last) == Status::OutOfRange);
        CHECK(set->GetMipLevelsForLatentImage(0, &first, &last) == Status::Ok && first == 0 && last == 2);
        CHECK(set->GetMipLevelsForLatentImage(2, &first, &last) == Status::Ok && first == 3 && last == 4);
        CHECK(set->GetMipLevelsForLatentImage(6, &first, &last) == Status::Ok && first == 7 && last == 12);
        CHECK(set->GetMipLevelsForLatentImage(1, &first, &last) == Status::OutOfRange);
        CHECK(set->GetMipLevelsForLatentImage(8, &first, &last) == Status::OutOfRange);
        CHECK(!set->IsInferenceWeightTypeSupported(InferenceWeightType::GenericInt8));       // no weights yet
        set->SetExperimentalKnob(1.f);
    }
    std::vector<unsigned char> blob(9472);
    CHECK(X(set)->SetWeightData(blob.data(), 100) == Status::InvalidArgument);
    CHECK(X(set)->SetWeightData(nullptr, 9472) == Status::InvalidArgument);
    CHECK(X(set)->SetWeightData(blob.data(), blob.size()) == Status::CudaUnavailable);
    // constants for decoding single texels elsewhere (src/Context.cpp:864-922): the host copy of the blob is kept
    // without a device, so the offsets (src/WeightLayout.cpp:184-265) and per-mip constants
    // (src/TextureSet.cpp:450-463) can be had
    {
        InferenceData data;
        std::memset(&data, 0xff, sizeof(data));
        CHECK(ctx->MakeInferenceData(set, InferenceWeightType::GenericInt8, 0, nullptr) == Status::InvalidArgument);
        CHECK(ctx->MakeInferenceData(nullptr, InferenceWeightType::GenericInt8, 0, &data) == Status::InvalidArgument);
        CHECK(ctx->MakeInferenceData(set, InferenceWeightType::Unknown, 0, &data) == Status::Unsupported);
        CHECK(ctx->MakeInferenceData(set, InferenceWeightType::CoopVecFP8, 0, &data) == Status::Unsupported);
        CHECK(std::strstr(GetLastErrorMessage(), "does not provide CoopVecFP8 weights") != nullptr);
        CHECK(ctx->MakeInferenceData(set, InferenceWeightType::GenericInt8, 0, &data) == Status::Ok);
        NtcTextureSetConstants const& c = data.constants;
        static int const neural[13] = { 0, 0, 0, 2, 2, 4, 4, 6, 6, 6, 6, 6, 6 };
        static float const scale[13] = { .25f, .5f, 1.f, .5f, 1.f, .5f, 1.f, .5f, 1.f, 2.f, 4.f, 8.f, 16.f };
        static float const lod[13] = { -.5f, -.25f, 0.f, -.25f, 0.f, -.25f, 0.f, -.25f, 0.f, .25f, .5f, .75f, 1.f };
        for (int mip = 0; mip < 16; ++mip) {
            NtcColorMipConstants const& m = c.colorMips[mip];
            if (mip < 13) CHECK(m.neuralMip == neural[mip] && m.positionScale == scale[mip] && m.positionLod == lod[mip] && m.pad == 0);
            else CHECK(m.neuralMip == 0 && m.positionScale == 0.f && m.positionLod == 0.f && m.pad == 0);
        }
        static int const weights[4] = { 0, 3072, 6144, 7680 }, scales[4] = { 8192, 8448, 8640, 8768 }, biases[4] = { 8832, 9088, 9280, 9408 };
        for (int layer = 0; layer < 4; ++layer)
            CHECK(c.networkWeightOffsets[layer] == weights[layer] && c.networkScaleOffsets[layer] == scales[layer] && c.networkBiasOffsets[layer] == biases[layer]);
        CHECK(c.imageWidth == 4096 && c.imageHeight == 4096 && c.imageMips == 13 && c.pad0 == 0 && c.pad1 == 0 && c.pad2 == 0);
        CHECK(c.validChannelMask == 0 && c.channelColorSpaces == 0);        // no textures described yet
        CHECK(ctx->MakeInferenceData(set, InferenceWeightType::GenericInt8, 2, &data) == Status::Ok);
        CHECK(c.colorMips[0].neuralMip == -2 && c.colorMips[3].neuralMip == 0 && c.colorMips[12].neuralMip == 4);
    }
    CHECK(X(set)->SetDecoderPreset(DecoderPreset::Concat2x2_64) == Status::Ok);
    CHECK(X(set)->GetWeightDataSize() == 10496 && X(set)->GetLatentDataSize() == 22369636ull);
    CHECK(set->GetNumLatentImages() == 0 && set->GetFusedMipLevels(0, nullptr, nullptr) == Status::Unsupported);   // per-mip grids
    CHECK(X(set)->SetDecoderPreset(DecoderPreset::Concat2x2_48) == Status::Ok);
    CHECK(X(set)->GetWeightDataSize() == 8576);

    // texture metadata decides which channels count (src/TextureMetadata.cpp:48-69)
    ITextureMetadata* albedo = set->AddTexture();
    CHECK(albedo != nullptr && set->GetTextureCount() == 1 && set->GetTexture(0) == albedo && set->GetTexture(1) == nullptr);
    albedo->SetName("albedo");
    CHECK(std::strcmp(albedo->GetName(), "albedo") == 0);
    CHECK(albedo->SetChannels(-1, 3) == Status::OutOfRange && albedo->SetChannels(16, 1) == Status::OutOfRange);
    CHECK(albedo->SetChannels(14, 3) == Status::OutOfRange && albedo->SetChannels(0, 0) == Status::OutOfRange);
    CHECK(albedo->SetChannels(1, 3) == Status::Ok && set->GetValidChannelMask() == 0xEu);
    ITextureMetadata* height = set->AddTexture();
    CHECK(height->SetChannels(8, 1) == Status::Ok && set->GetValidChannelMask() == 0x10Eu);
    int first = -1, count = -1;
    height->GetChannels(first, count);
    CHECK(first == 8 && count == 1);
    CHECK(set->RemoveTexture(albedo) == Status::Ok && set->RemoveTexture(albedo) == Status::OutOfRange);
    CHECK(set->GetTextureCount() == 1 && set->GetValidChannelMask() == 0x100u);
    set->ClearTextureMetadata();
    CHECK(set->GetTextureCount() == 0 && set->GetValidChannelMask() == 0);

    // WriteChannels shares the argument checks of ReadChannels (src/TextureSet.cpp:829-850,1914-1956)
    WriteChannelsParameters wp;
    CHECK(set->WriteChannels(wp) == Status::InvalidArgument);                // pData NULL
    std::vector<unsigned char> source(64);
    wp.pData = source.data(); wp.mipLevel = -1;
    CHECK(set->WriteChannels(wp) == Status::OutOfRange);
    wp.mipLevel = 12; wp.firstChannel = 15; wp.numChannels = 2;
    CHECK(set->WriteChannels(wp) == Status::OutOfRange);
    wp.numChannels = 1; wp.width = 1; wp.height = 1; wp.pixelStride = 0; wp.rowPitch = 4;
    CHECK(set->WriteChannels(wp) == Status::InvalidArgument);
    wp.pixelStride = 4; wp.channelFormat = ChannelFormat::FLOAT32;
    CHECK(set->WriteChannels(wp) == Status::CudaUnavailable);

    // ReadChannels argument checks (src/TextureSet.cpp:1914-1956)
    std::vector<unsigned char> pixels(16);
    ReadChannelsParameters rp;
    CHECK(set->ReadChannels(rp) == Status::InvalidArgument);                 // pOutData NULL
    rp.pOutData = pixels.data(); rp.mipLevel = 13;
    CHECK(set->ReadChannels(rp) == Status::OutOfRange);
    rp.mipLevel = 12; rp.firstChannel = 16;
    CHECK(set->ReadChannels(rp) == Status::OutOfRange);
    rp.firstChannel = 14; rp.numChannels = 3;
    CHECK(set->ReadChannels(rp) == Status::OutOfRange);
    rp.numChannels = 2;
    CHECK(set->ReadChannels(rp) == Status::OutOfRange);                      // width/height 0
    rp.width = 1; rp.height = 1; rp.pixelStride = 4; rp.rowPitch = 2;
    CHECK(set->ReadChannels(rp) == Status::InvalidArgument);
    rp.rowPitch = 4; rp.channelFormat = ChannelFormat::UNORM8;
    CHECK(set->ReadChannels(rp) == Status::CudaUnavailable);                 // arguments fine, no device

    // image-difference pass: argument rules come first, then the missing device
    {
        unsigned char pixels[64] = {};
        uint64_t result[4] = {};
        ImageDifferenceParameters dp;
        dp.imageA.pData = pixels; dp.imageA.dataSize = sizeof pixels; dp.imageA.width = 4; dp.imageA.height = 4;
        dp.imageA.pixelStride = 4; dp.imageA.rowPitch = 16; dp.imageA.channelFormat = ChannelFormat::UNORM8;
        dp.imageB = dp.imageA;
        dp.extent.width = 4; dp.extent.height = 4;
        CHECK(X(ctx)->ComputeImageDifference(dp) == Status::InvalidArgument);       // no output buffer
        dp.pOutputBuffer = result; dp.outputBufferSize = sizeof result;
        dp.extent.left = -1;
        CHECK(X(ctx)->ComputeImageDifference(dp) == Status::OutOfRange);
        dp.extent.left = 0; dp.extent.height = 0;
        CHECK(X(ctx)->ComputeImageDifference(dp) == Status::OutOfRange);
        dp.extent.height = 4; dp.outputOffset = 4;
        CHECK(X(ctx)->ComputeImageDifference(dp) == Status::OutOfRange);
        dp.outputOffset = 0;
        CHECK(X(ctx)->ComputeImageDifference(dp) == Status::CudaUnavailable);
    }

    ctx->DestroyTextureSet(set);
    DestroyContext(ctx);
    std::printf("host cpu checks OK\n");
    return 0;
}

static int decode(int argc, char** argv)
{
    if (argc < 12) { std::fprintf(stderr, "usage: decode <preset> <w> <h> <mips> <channels> <gridScale> <features> <latents> <weights> <outPrefix>\n"); return 2; }
    int const preset = std::atoi(argv[2]), w = std::atoi(argv[3]), h = std::atoi(argv[4]), mips = std::atoi(argv[5]);
    int const channels = std::atoi(argv[6]), gridScale = std::atoi(argv[7]), features = std::atoi(argv[8]);
    std::vector<unsigned char> latents = readFile(argv[9]), weights = readFile(argv[10]);
    std::string const prefix = argv[11];

    IContext* ctx = nullptr;
    ContextParameters params;
    CHECK(CreateContext(&ctx, params) == Status::Ok);
    CHECK(ntc_hip_init(params.cudaDevice) == 0);              // the default context of the C ABI, for this program's own device buffers
    CHECK(X(ctx)->IsDeviceAvailable());
    TextureSetDesc desc; desc.width = w; desc.height = h; desc.channels = channels; desc.mips = mips;
    TextureSetFeatures features_;
    features_.stagingBytesPerPixel = 16 * 4;
    ITextureSet* set = nullptr;
    CHECK(ctx->CreateTextureSet(desc, features_, &set) == Status::Ok);
    if (preset == 0) { LatentShape shape; shape.gridSizeScale = gridScale; shape.numFeatures = features; CHECK(set->SetLatentShape(shape) == Status::Ok); }
    else CHECK(X(set)->SetDecoderPreset(DecoderPreset(preset)) == Status::Ok);
    CHECK(X(set)->GetLatentDataSize() == latents.size());
    CHECK(X(set)->GetWeightDataSize() == weights.size());
    CHECK(X(set)->SetLatentData(latents.data(), latents.size()) == Status::Ok);
    CHECK(set->Decompress(nullptr, true) == Status::InvalidState);                // weights still missing
    CHECK(X(set)->SetWeightData(weights.data(), weights.size()) == Status::Ok);
    DecompressionStats stats;
    CHECK(set->Decompress(&stats, true) == Status::Ok);
    CHECK(stats.gpuTimeMilliseconds > 0.f && stats.overallLoss == 0.f);
    CHECK(set->Decompress(nullptr, true) == Status::Ok);                           // asynchronous form, idempotent
    int const C = set->GetDesc().channels;
    for (int mip = 0; mip < mips; ++mip) {
        int const mw = std::max(w >> mip, 1), mh = std::max(h >> mip, 1);
        // UNORM8, all channels, host memory, padded rows
        ReadChannelsParameters rp;
        rp.mipLevel = mip; rp.firstChannel = 0; rp.numChannels = C;
        rp.width = mw; rp.height = mh; rp.pixelStride = size_t(C); rp.rowPitch = size_t(C) * size_t(mw) + 8;
        rp.channelFormat = ChannelFormat::UNORM8;
        std::vector<unsigned char> u8(rp.rowPitch * size_t(mh), 0xEE);
        rp.pOutData = u8.data();
        CHECK(set->ReadChannels(rp) == Status::Ok);
        CHECK(writeFile(prefix + "_mip" + std::to_string(mip) + "_unorm8.bin", u8.data(), u8.size()));
        // FLOAT16, channels 1..3 into an RGBA pixel (4th channel takes the default), device memory
        if (C >= 4) {
            void* dev = nullptr;
            size_t const bytes = size_t(mw) * size_t(mh) * 8;
            CHECK(ntc_hip_alloc(&dev, bytes) == 0);
            ReadChannelsParameters rd;
            rd.mipLevel = mip; rd.firstChannel = 1; rd.numChannels = 3;
            rd.width = mw; rd.height = mh; rd.pixelStride = 8; rd.rowPitch = size_t(mw) * 8;
            rd.channelFormat = ChannelFormat::FLOAT16; rd.addressSpace = AddressSpace::Device;
            rd.pOutData = static_cast<unsigned char*>(dev);
            CHECK(set->ReadChannels(rd) == Status::Ok);
            std::vector<unsigned char> f16(bytes);
            CHECK(syncedDownload(ctx, f16.data(), dev, bytes) == 0);
            CHECK(ntc_hip_free(dev) == 0);
            CHECK(writeFile(prefix + "_mip" + std::to_string(mip) + "_rgba16f.bin", f16.data(), f16.size()));
        }
    }
    // dithered read of mip 0 into sRGB for the first three channels
    {
        ColorSpace wanted[16];
        for (int c = 0; c < 16; ++c) wanted[c] = c < 3 ? ColorSpace::sRGB : ColorSpace::Linear;
        ReadChannelsParameters rp;
        rp.mipLevel = 0; rp.firstChannel = 0; rp.numChannels = C; rp.width = w; rp.height = h;
        rp.pixelStride = size_t(C); rp.rowPitch = size_t(C) * size_t(w);
        rp.channelFormat = ChannelFormat::UNORM8; rp.dstColorSpaces = wanted; rp.useDithering = true;
        std::vector<unsigned char> u8(rp.rowPitch * size_t(h));
        rp.pOutData = u8.data();
        CHECK(set->ReadChannels(rp) == Status::Ok);
        CHECK(writeFile(prefix + "_srgb_dither.bin", u8.data(), u8.size()));
    }
    // a read at another size resamples mip 0 (here: down to 2 x 2, channel 0)
    {
        ReadChannelsParameters small;
        std::vector<unsigned char> tmp(64, 0xEE);
        small.pOutData = tmp.data(); small.numChannels = 1; small.width = 2; small.height = 2; small.pixelStride = 1; small.rowPitch = 2;
        small.channelFormat = ChannelFormat::UNORM8;
        CHECK(set->ReadChannels(small) == Status::Ok);
        CHECK(writeFile(prefix + "_2x2.bin", tmp.data(), 4));
    }
    ctx->DestroyTextureSet(set);
    DestroyContext(ctx);
    std::printf("host decode OK, gpu %.3f ms\n", stats.gpuTimeMilliseconds);
    return 0;
}

// IEEE binary16 bits of a float in the normal half range, round to nearest even (expected constants)
static uint16_t halfBits(float v)
{
    uint32_t f;
    std::memcpy(&f, &v, 4);
    uint32_t const sign = (f >> 16) & 0x8000u, exponent = (f >> 23) & 0xffu, mantissa = f & 0x7fffffu;
    if (exponent == 0) return uint16_t(sign);
    uint32_t half = ((exponent - 112u) << 10) | (mantissa >> 13);      // exponent rebias 127 -> 15
    uint32_t const rest = mantissa & 0x1fffu;
    if (rest > 0x1000u || (rest == 0x1000u && (half & 1u))) ++half;     // a carry into the exponent is the right result
    return uint16_t(sign | half);
}

static int shuffle(int argc, char** argv)
{
    if (argc < 10) { std::fprintf(stderr, "usage: shuffle <preset> <w> <h> <channels> <gridScale> <features> <latents> <weights>\n"); return 2; }
    int const preset = std::atoi(argv[2]), w = std::atoi(argv[3]), h = std::atoi(argv[4]), channels = std::atoi(argv[5]);
    int const gridScale = std::atoi(argv[6]), features = std::atoi(argv[7]);
    std::vector<unsigned char> latents = readFile(argv[8]), weights = readFile(argv[9]);
    IContext* ctx = nullptr;
    ContextParameters params;
    CHECK(CreateContext(&ctx, params) == Status::Ok);
    CHECK(ntc_hip_init(params.cudaDevice) == 0);              // the default context of the C ABI, for this program's own device buffers
    TextureSetDesc desc; desc.width = w; desc.height = h; desc.channels = channels; desc.mips = 1;
    TextureSetFeatures features_;
    features_.stagingBytesPerPixel = 16 * 2;
    ITextureSet* set = nullptr;
    CHECK(ctx->CreateTextureSet(desc, features_, &set) == Status::Ok);
    void const* blob = nullptr; size_t blobSize = 0, converted = 1;
    CHECK(set->GetInferenceWeights(InferenceWeightType::GenericInt8, &blob, &blobSize, &converted) == Status::Unsupported);   // nothing loaded yet
    CHECK(set->GetBestSupportedWeightType() == InferenceWeightType::Unknown);
    if (preset == 0) { LatentShape shape; shape.gridSizeScale = gridScale; shape.numFeatures = features; CHECK(set->SetLatentShape(shape) == Status::Ok); }
    else CHECK(X(set)->SetDecoderPreset(DecoderPreset(preset)) == Status::Ok);
    CHECK(X(set)->SetLatentData(latents.data(), latents.size()) == Status::Ok);
    CHECK(X(set)->SetWeightData(weights.data(), weights.size()) == Status::Ok);
    CHECK(set->GetBestSupportedWeightType() == InferenceWeightType::GenericInt8);
    CHECK(set->GetInferenceWeights(InferenceWeightType::GenericFP8, &blob, &blobSize, &converted) == Status::Unsupported);
    CHECK(std::strstr(GetLastErrorMessage(), "GenericFP8") != nullptr);
    CHECK(set->GetInferenceWeights(InferenceWeightType::GenericInt8, &blob, &blobSize, &converted) == Status::Ok);
    CHECK(blobSize == weights.size() && converted == 0 && std::memcmp(blob, weights.data(), blobSize) == 0);
    ITextureMetadata* tex = set->AddTexture(); CHECK(tex->SetChannels(0, 4) == Status::Ok);
    CHECK(set->GetValidChannelMask() == 0xFu);

    auto decodeAll = [&](std::vector<uint16_t>& out) -> int {
        CHECK(set->Decompress(nullptr, true) == Status::Ok);
        ReadChannelsParameters rp;
        rp.mipLevel = 0; rp.firstChannel = 0; rp.numChannels = channels; rp.width = w; rp.height = h;
        rp.pixelStride = size_t(channels) * 2; rp.rowPitch = rp.pixelStride * size_t(w); rp.channelFormat = ChannelFormat::FLOAT16;
        out.assign(size_t(w) * size_t(h) * size_t(channels), 0);
        rp.pOutData = reinterpret_cast<unsigned char*>(out.data());
        CHECK(set->ReadChannels(rp) == Status::Ok);
        return 0;
    };
    std::vector<uint16_t> before, unchanged, after;
    if (decodeAll(before)) return 1;

    ShuffleSource mapping[16];
    for (int ch = 0; ch < 16; ++ch) mapping[ch] = ShuffleSource::Channel((ch * 7 + 3) % 16);
    mapping[0] = ShuffleSource::Channel(5);
    mapping[1] = ShuffleSource::Constant(0.625f);      // exactly representable
    mapping[2] = ShuffleSource::Undefined();
    mapping[3] = ShuffleSource::Channel(3);
    mapping[4] = ShuffleSource::Constant(0.1f);        // stored as round(0.1 * 2^16) / 2^16
    mapping[5] = ShuffleSource::Constant(-2.5f);
    ShuffleSource bad[16];
    for (int ch = 0; ch < 16; ++ch) bad[ch] = ShuffleSource::Channel(ch);
    bad[7] = ShuffleSource::Channel(16);
    CHECK(set->ShuffleInferenceOutputs(nullptr) == Status::InvalidArgument);
    CHECK(set->ShuffleInferenceOutputs(bad) == Status::OutOfRange);
    bad[7].type = ShuffleSourceType(9);
    CHECK(set->ShuffleInferenceOutputs(bad) == Status::InvalidArgument);
    CHECK(set->ShuffleInferenceOutputs(mapping) == Status::Ok);
    // valid mask: channels whose source lies in the texture's channels 0..3, and constants
    uint32_t wantMask = 0;
    for (int ch = 0; ch < 16; ++ch)
        if (mapping[ch].type == ShuffleSourceType::Constant || (mapping[ch].type == ShuffleSourceType::Channel && mapping[ch].channelIndex < 4)) wantMask |= 1u << ch;
    CHECK(set->GetValidChannelMask() == wantMask);
    // Decompress keeps the weights as loaded
    if (decodeAll(unchanged)) return 1;
    CHECK(unchanged == before);
    // the shuffled weights, used as the set's weights, give the shuffled channels
    CHECK(set->GetInferenceWeights(InferenceWeightType::GenericInt8, &blob, &blobSize, nullptr) == Status::Ok);
    std::vector<unsigned char> shuffled(static_cast<unsigned char const*>(blob), static_cast<unsigned char const*>(blob) + blobSize);
    CHECK(shuffled != weights);
    CHECK(X(set)->SetWeightData(shuffled.data(), shuffled.size()) == Status::Ok);
    CHECK(set->GetValidChannelMask() == 0xFu);         // a new blob starts un-shuffled
    if (decodeAll(after)) return 1;
    size_t mismatches = 0;
    for (size_t px = 0; px < size_t(w) * size_t(h); ++px)
        for (int ch = 0; ch < channels; ++ch) {
            uint16_t want = 0;
            if (mapping[ch].type == ShuffleSourceType::Channel) {
                int const src = mapping[ch].channelIndex;
                if (src >= channels) continue;             // the source was never stored by the first decode
                want = before[px * size_t(channels) + size_t(src)];
            } else if (mapping[ch].type == ShuffleSourceType::Constant) {
                want = halfBits(float(int32_t(roundf(mapping[ch].constantValue * 65536.f))) * (1.f / 65536.f));
            }
            if (after[px * size_t(channels) + size_t(ch)] != want) ++mismatches;
        }
    CHECK(mismatches == 0);
    // shuffling twice composes: the inverse permutation of a bijective mapping restores the blob
    ShuffleSource perm[16], inverse[16];
    for (int ch = 0; ch < 16; ++ch) { perm[ch] = ShuffleSource::Channel((ch * 5 + 2) % 16); inverse[(ch * 5 + 2) % 16] = ShuffleSource::Channel(ch); }
    CHECK(X(set)->SetWeightData(weights.data(), weights.size()) == Status::Ok);
    CHECK(set->ShuffleInferenceOutputs(perm) == Status::Ok);
    CHECK(set->ShuffleInferenceOutputs(inverse) == Status::Ok);
    CHECK(set->GetInferenceWeights(InferenceWeightType::GenericInt8, &blob, &blobSize, nullptr) == Status::Ok);
    CHECK(std::memcmp(blob, weights.data(), blobSize) == 0);
    CHECK(set->GetValidChannelMask() == 0xFu);
    ctx->DestroyTextureSet(set);
    DestroyContext(ctx);
    std::printf("host shuffle OK\n");
    return 0;
}

// IContext::ComputeImageDifference on two small images in device memory: every byte differs by 255
// in one image pair (mean squared error exactly 1 in all four channels), the alpha threshold removes
// the colour channels, and a sub-rectangle of identical pixels gives zero.
static int imageDifference()
{
    IContext* ctx = nullptr;
    ContextParameters params;
    CHECK(CreateContext(&ctx, params) == Status::Ok);
    CHECK(ntc_hip_init(params.cudaDevice) == 0);              // the default context of the C ABI, for this program's own device buffers
    int const w = 192, h = 80;
    std::vector<unsigned char> a(size_t(w) * h * 4, 0), b(size_t(w) * h * 4, 255);
    for (int y = 0; y < 16; ++y) for (int x = 0; x < 32; ++x) std::memcpy(&b[(size_t(y) * w + x) * 4], &a[(size_t(y) * w + x) * 4], 4);   // identical corner
    void *dA = nullptr, *dB = nullptr, *dOut = nullptr;
    CHECK(ntc_hip_alloc(&dA, a.size()) == 0 && ntc_hip_alloc(&dB, b.size()) == 0 && ntc_hip_alloc(&dOut, 64) == 0);
    CHECK(ntc_hip_upload(dA, a.data(), a.size()) == 0 && ntc_hip_upload(dB, b.data(), b.size()) == 0);
    uint64_t zeros[8] = {}, result[8] = {};
    CHECK(ntc_hip_upload(dOut, zeros, sizeof zeros) == 0);
    ImageDifferenceParameters dp;
    dp.imageA.pData = static_cast<unsigned char const*>(dA); dp.imageA.dataSize = a.size(); dp.imageA.width = w; dp.imageA.height = h;
    dp.imageA.pixelStride = 4; dp.imageA.rowPitch = size_t(w) * 4; dp.imageA.channelFormat = ChannelFormat::UNORM8;
    dp.imageB = dp.imageA; dp.imageB.pData = static_cast<unsigned char const*>(dB);
    dp.pOutputBuffer = dOut; dp.outputBufferSize = 64;
    dp.extent.left = 64; dp.extent.top = 16; dp.extent.width = 128; dp.extent.height = 64;     // all pixels differ
    CHECK(X(ctx)->ComputeImageDifference(dp) == Status::Ok);
    dp.outputOffset = 32; dp.extent = Rect{ 0, 0, 32, 16 };                                     // identical pixels
    CHECK(X(ctx)->ComputeImageDifference(dp) == Status::Ok);
    CHECK(syncedDownload(ctx, result, dOut, sizeof result) == 0);
    for (int c = 0; c < 4; ++c) CHECK(DecodeImageDifferenceResult(result[c]) == 1.0 && result[4 + c] == 0);
    // both alphas (0 and 1) below a threshold of 2: colour ignored, alpha still compared
    CHECK(ntc_hip_upload(dOut, zeros, sizeof zeros) == 0);
    dp.outputOffset = 0; dp.extent = Rect{ 64, 16, 128, 64 }; dp.useAlphaThreshold = true; dp.alphaThreshold = 2.f;
    CHECK(X(ctx)->ComputeImageDifference(dp) == Status::Ok);
    CHECK(syncedDownload(ctx, result, dOut, sizeof result) == 0);
    CHECK(result[0] == 0 && result[1] == 0 && result[2] == 0 && DecodeImageDifferenceResult(result[3]) == 1.0);
    dp.extent.width = 200;                                                                      // leaves the image
    CHECK(X(ctx)->ComputeImageDifference(dp) == Status::InvalidArgument);
    CHECK(std::strstr(GetLastErrorMessage(), "does not lie inside") != nullptr);
    // block compression of image B: constant 255 everywhere except the zero corner -> BC4 blocks 0xFF, 0xFF / 0, 0 with all indices 0
    {
        size_t const blocksX = size_t(w) / 4, blocksY = size_t(h) / 4;
        void* dBlocks = nullptr;
        CHECK(ntc_hip_alloc(&dBlocks, blocksX * blocksY * 16) == 0);
        BlockCompressionParameters bp;
        bp.srcImage = dp.imageB;
        bp.srcRect = Rect{ 0, 0, w, h };
        bp.dstFormat = BlockCompressedFormat::BC5;
        bp.pDstData = dBlocks; bp.dstDataSize = blocksX * blocksY * 16; bp.dstRowPitch = blocksX * 16;
        CHECK(X(ctx)->CompressBlocks(bp) == Status::Ok);
        std::vector<uint64_t> blocks(blocksX * blocksY * 2);
        CHECK(syncedDownload(ctx, blocks.data(), dBlocks, blocks.size() * 8) == 0);
        for (size_t by = 0; by < blocksY; ++by)
            for (size_t bx = 0; bx < blocksX; ++bx) {
                bool const corner = bx < 8 && by < 4;
                uint64_t const want = corner ? 0ull : 0xFFFFull;
                CHECK(blocks[(by * blocksX + bx) * 2] == want && blocks[(by * blocksX + bx) * 2 + 1] == want);
            }
        // BC1 of the same image: opaque white is the single-colour block of 0xFFFF twice with every index 2,
        // the zero corner (alpha 0) the all-transparent block
        bp.dstFormat = BlockCompressedFormat::BC1; bp.dstRowPitch = blocksX * 8;
        CHECK(X(ctx)->CompressBlocks(bp) == Status::Ok);
        CHECK(syncedDownload(ctx, blocks.data(), dBlocks, blocksX * blocksY * 8) == 0);
        for (size_t by = 0; by < blocksY; ++by)
            for (size_t bx = 0; bx < blocksX; ++bx)
                CHECK(blocks[by * blocksX + bx] == ((bx < 8 && by < 4) ? 0xFFFFFFFF00000000ull : 0xAAAAAAAAFFFFFFFFull));
        bp.dstRowPitch = blocksX * 16;
        // BC7 of the same image, then once more through the mode buffer made from those blocks: the same blocks.
        // Opaque white is exact in BC7; the zero corner has alpha 0.
        bp.dstFormat = BlockCompressedFormat::BC7;
        CHECK(X(ctx)->CompressBlocks(bp) == Status::Ok);
        CHECK(syncedDownload(ctx, blocks.data(), dBlocks, blocks.size() * 8) == 0);
        {
            std::vector<uint8_t> modes(GetBC7ModeBufferSize(int(blocksX), int(blocksY)), 0);
            CHECK(MakeBC7ModeBuffer(int(blocksX), int(blocksY), blocks.data(), blocks.size() * 8, blocksX * 16, modes.data(), modes.size()) == Status::Ok);
            void* dModes = nullptr;
            CHECK(ntc_hip_alloc(&dModes, modes.size()) == 0 && ntc_hip_upload(dModes, modes.data(), modes.size()) == 0);
            CHECK(ntc_hip_memset(dBlocks, 0, blocksX * blocksY * 16) == 0 && ntc_hip_synchronize() == 0);
            bp.pModeBuffer = dModes; bp.modeBufferSize = modes.size();
            bp.modeMapWidthInBlocks = int(blocksX); bp.modeMapHeightInBlocks = int(blocksY);
            CHECK(X(ctx)->CompressBlocks(bp) == Status::Ok);
            std::vector<uint64_t> again(blocks.size());
            CHECK(syncedDownload(ctx, again.data(), dBlocks, again.size() * 8) == 0);
            CHECK(again == blocks);
            bp.dstFormat = BlockCompressedFormat::BC3;
            CHECK(X(ctx)->CompressBlocks(bp) == Status::InvalidArgument);
            bp.pModeBuffer = nullptr;
            CHECK(ntc_hip_free(dModes) == 0);
        }
        // BC6H of the same image: the zero corner is the one-subset block with zero endpoints; the white blocks are
        // all the same block in one of the three modes the encoder emits
        bp.dstFormat = BlockCompressedFormat::BC6;
        CHECK(X(ctx)->CompressBlocks(bp) == Status::Ok);
        CHECK(syncedDownload(ctx, blocks.data(), dBlocks, blocks.size() * 8) == 0);
        {
            uint64_t const whiteLo = blocks[(blocksY - 1) * blocksX * 2], whiteHi = blocks[(blocksY - 1) * blocksX * 2 + 1];
            CHECK((whiteLo & 3u) == 1u || (whiteLo & 31u) == 0x0Eu || (whiteLo & 31u) == 0x03u);
            for (size_t by = 0; by < blocksY; ++by)
                for (size_t bx = 0; bx < blocksX; ++bx) {
                    bool const corner = bx < 8 && by < 4;
                    CHECK(blocks[(by * blocksX + bx) * 2] == (corner ? 0x03u : whiteLo) && blocks[(by * blocksX + bx) * 2 + 1] == (corner ? 0u : whiteHi));
                }
        }
        bp.dstFormat = BlockCompressedFormat::None;
        CHECK(X(ctx)->CompressBlocks(bp) == Status::OutOfRange);
        bp.dstFormat = BlockCompressedFormat::BC4; bp.dstDataSize = 8;
        CHECK(X(ctx)->CompressBlocks(bp) == Status::InvalidArgument);
        CHECK(ntc_hip_free(dBlocks) == 0);
    }
    CHECK(ntc_hip_free(dA) == 0 && ntc_hip_free(dB) == 0 && ntc_hip_free(dOut) == 0);
    DestroyContext(ctx);
    std::printf("host image difference OK\n");
    return 0;
}

// WriteChannels at twice the size of mip 0 (resampled down), GenerateMips, then every mip of the
// reference page read back as FLOAT16 pixels into <prefix>_mip<N>.bin for the test to compare.
static int generateMips(int argc, char** argv)
{
    if (argc < 8) { std::fprintf(stderr, "usage: genmips <w> <h> <channels> <mips> <image(FLOAT32 pixels, 2w x 2h)> <outPrefix>\n"); return 2; }
    int const w = std::atoi(argv[2]), h = std::atoi(argv[3]), channels = std::atoi(argv[4]), mips = std::atoi(argv[5]);
    std::vector<unsigned char> image = readFile(argv[6]);
    std::string const prefix = argv[7];
    IContext* ctx = nullptr;
    ContextParameters params;
    CHECK(CreateContext(&ctx, params) == Status::Ok);
    CHECK(ntc_hip_init(params.cudaDevice) == 0);              // the default context of the C ABI, for this program's own device buffers
    TextureSetDesc desc; desc.width = w; desc.height = h; desc.channels = channels; desc.mips = mips;
    TextureSetFeatures features_;
    features_.stagingBytesPerPixel = 16 * 4; features_.stagingWidth = 2 * w; features_.stagingHeight = 2 * h;
    ITextureSet* set = nullptr;
    CHECK(ctx->CreateTextureSet(desc, features_, &set) == Status::Ok);
    int const C = set->GetDesc().channels;
    CHECK(image.size() == size_t(2 * w) * size_t(2 * h) * size_t(C) * 4);
    ColorSpace source[16], storage[16];
    for (int c = 0; c < 16; ++c) { source[c] = ColorSpace::Linear; storage[c] = c == 1 ? ColorSpace::sRGB : ColorSpace::Linear; }
    WriteChannelsParameters wp;
    wp.mipLevel = 0; wp.firstChannel = 0; wp.numChannels = C; wp.pData = image.data();
    wp.width = 2 * w; wp.height = 2 * h; wp.pixelStride = size_t(C) * 4; wp.rowPitch = wp.pixelStride * size_t(2 * w);
    wp.channelFormat = ChannelFormat::FLOAT32; wp.srcColorSpaces = source; wp.dstColorSpaces = storage;
    CHECK(set->WriteChannels(wp) == Status::Ok);
    CHECK(set->GenerateMips() == Status::Ok);
    for (int mip = 0; mip < mips; ++mip) {
        int const mw = std::max(w >> mip, 1), mh = std::max(h >> mip, 1);
        ReadChannelsParameters rp;
        rp.page = TextureDataPage::Reference;
        rp.mipLevel = mip; rp.firstChannel = 0; rp.numChannels = C; rp.width = mw; rp.height = mh;
        rp.pixelStride = size_t(C) * 2; rp.rowPitch = rp.pixelStride * size_t(mw); rp.channelFormat = ChannelFormat::FLOAT16;
        rp.dstColorSpaces = storage;                         // read the stored values as they are
        std::vector<unsigned char> out(rp.rowPitch * size_t(mh));
        rp.pOutData = out.data();
        CHECK(set->ReadChannels(rp) == Status::Ok);
        CHECK(writeFile(prefix + "_mip" + std::to_string(mip) + ".bin", out.data(), out.size()));
    }
    ctx->DestroyTextureSet(set);
    DestroyContext(ctx);
    std::printf("host genmips OK\n");
    return 0;
}

static int loss(int argc, char** argv)
{
    if (argc < 13) { std::fprintf(stderr, "usage: loss <preset> <w> <h> <mips> <channels> <gridScale> <features> <latents> <weights> <refPrefix> <separate>\n"); return 2; }
    int const preset = std::atoi(argv[2]), w = std::atoi(argv[3]), h = std::atoi(argv[4]), mips = std::atoi(argv[5]);
    int const channels = std::atoi(argv[6]), gridScale = std::atoi(argv[7]), features = std::atoi(argv[8]);
    std::vector<unsigned char> latents = readFile(argv[9]), weights = readFile(argv[10]);
    std::string const prefix = argv[11];
    bool const separate = std::atoi(argv[12]) != 0;
    int const maskChannel = argc >= 16 ? std::atoi(argv[13]) : -1;
    bool const discard = argc >= 16 && std::atoi(argv[14]) != 0;
    bool const withStats = argc < 16 || std::atoi(argv[15]) != 0;

    IContext* ctx = nullptr;
    ContextParameters params;
    CHECK(CreateContext(&ctx, params) == Status::Ok);
    CHECK(ntc_hip_init(params.cudaDevice) == 0);              // the default context of the C ABI, for this program's own device buffers
    TextureSetDesc desc; desc.width = w; desc.height = h; desc.channels = channels; desc.mips = mips;
    TextureSetFeatures features_;
    features_.stagingBytesPerPixel = 16 * 4;
    features_.separateRefOutData = separate;
    ITextureSet* set = nullptr;
    CHECK(ctx->CreateTextureSet(desc, features_, &set) == Status::Ok);
    if (preset == 0) { LatentShape shape; shape.gridSizeScale = gridScale; shape.numFeatures = features; CHECK(set->SetLatentShape(shape) == Status::Ok); }
    else CHECK(X(set)->SetDecoderPreset(DecoderPreset(preset)) == Status::Ok);
    CHECK(X(set)->SetLatentData(latents.data(), latents.size()) == Status::Ok);
    CHECK(X(set)->SetWeightData(weights.data(), weights.size()) == Status::Ok);
    ITextureMetadata* a = set->AddTexture(); CHECK(a->SetChannels(0, 3) == Status::Ok);
    ITextureMetadata* b = set->AddTexture(); CHECK(b->SetChannels(4, 2) == Status::Ok);
    CHECK(set->GetValidChannelMask() == 0x37u);
    CHECK(set->SetMaskChannelIndex(set->GetDesc().channels, false) == Status::OutOfRange);
    CHECK(set->SetMaskChannelIndex(maskChannel, discard) == Status::Ok);
    int const C = set->GetDesc().channels;
    for (int mip = 0; mip < mips; ++mip) {
        int const mw = std::max(w >> mip, 1), mh = std::max(h >> mip, 1);
        std::vector<unsigned char> ref = readFile((prefix + "_mip" + std::to_string(mip) + ".bin").c_str());
        CHECK(ref.size() == size_t(mw) * size_t(mh) * size_t(C) * 4);
        WriteChannelsParameters wp;
        wp.mipLevel = mip; wp.firstChannel = 0; wp.numChannels = C; wp.pData = ref.data();
        wp.width = mw; wp.height = mh; wp.pixelStride = size_t(C) * 4; wp.rowPitch = wp.pixelStride * size_t(mw);
        wp.channelFormat = ChannelFormat::FLOAT32;
        CHECK(set->WriteChannels(wp) == Status::Ok);
    }
    auto printStats = [&](char const* tag, DecompressionStats const& st) {
        std::printf("%s overall %.9g\n%s mips", tag, st.overallLoss, tag);
        for (int m = 0; m < mips; ++m) std::printf(" %.9g", st.perMipLoss[m]);
        std::printf("\n%s channels", tag);
        for (int c = 0; c < 16; ++c) std::printf(" %.9g", st.perChannelLoss[c]);
        std::printf("\n");
    };
    DecompressionStats first{}, second{};
    CHECK(set->Decompress(withStats ? &first : nullptr, true) == Status::Ok);
    printStats("first", first);
    CHECK(set->Decompress(withStats ? &second : nullptr, true) == Status::Ok);
    printStats("second", second);
    // Reference page after the decode: the written image when the pages are separate, the
    // decoded image when they share memory (src/TextureSet.cpp:103-124).
    ReadChannelsParameters rp;
    rp.mipLevel = 0; rp.firstChannel = 0; rp.numChannels = C; rp.width = w; rp.height = h;
    rp.pixelStride = size_t(C) * 2; rp.rowPitch = rp.pixelStride * size_t(w); rp.channelFormat = ChannelFormat::FLOAT16;
    std::vector<unsigned char> page(rp.rowPitch * size_t(h));
    rp.pOutData = page.data();
    rp.page = TextureDataPage::Reference;
    CHECK(set->ReadChannels(rp) == Status::Ok);
    CHECK(writeFile(prefix + "_page_reference.bin", page.data(), page.size()));
    rp.page = TextureDataPage::Output;
    CHECK(set->ReadChannels(rp) == Status::Ok);
    CHECK(writeFile(prefix + "_page_output.bin", page.data(), page.size()));
    // storage colour spaces given to WriteChannels are recorded with the set (src/TextureSet.cpp:899-902)
    {
        CHECK(set->GetChannelStorageColorSpace(1) == ColorSpace::Linear);
        std::vector<unsigned char> one(size_t(w) * size_t(h), 128);
        ColorSpace const source = ColorSpace::Linear, storage = ColorSpace::sRGB;
        WriteChannelsParameters wp;
        wp.mipLevel = 0; wp.firstChannel = 1; wp.numChannels = 1; wp.pData = one.data();
        wp.width = w; wp.height = h; wp.pixelStride = 1; wp.rowPitch = size_t(w);
        wp.channelFormat = ChannelFormat::UNORM8; wp.srcColorSpaces = &source; wp.dstColorSpaces = &storage;
        CHECK(set->WriteChannels(wp) == Status::Ok);
        CHECK(set->GetChannelStorageColorSpace(1) == ColorSpace::sRGB && set->GetChannelStorageColorSpace(0) == ColorSpace::Linear);
        // reading it back as linear UNORM8 returns the written codes (sRGB there and back), to one code
        ReadChannelsParameters rb;
        rb.page = TextureDataPage::Reference;
        rb.mipLevel = 0; rb.firstChannel = 1; rb.numChannels = 1; rb.width = w; rb.height = h; rb.pixelStride = 1; rb.rowPitch = size_t(w);
        rb.channelFormat = ChannelFormat::UNORM8;
        std::vector<unsigned char> back(one.size());
        rb.pOutData = back.data();
        CHECK(set->ReadChannels(rb) == Status::Ok);
        for (unsigned char v : back) CHECK(v >= 127 && v <= 129);
    }
    ctx->DestroyTextureSet(set);
    DestroyContext(ctx);
    std::printf("host loss OK\n");
    return 0;
}

static int describe(ITextureSetMetadata* set)
{
    TextureSetDesc const& d = set->GetDesc();
    std::printf("desc %d %d %d %d\n", d.width, d.height, d.channels, d.mips);
    std::printf("shape %d %d\n", set->GetLatentShape().gridSizeScale, set->GetLatentShape().numFeatures);
    std::printf("sizes %llu %llu\n", (unsigned long long)X(set)->GetLatentDataSize(), (unsigned long long)X(set)->GetWeightDataSize());
    for (int i = 0; i < set->GetTextureCount(); ++i) {
        ITextureMetadata* t = set->GetTexture(i);
        std::printf("texture %s|%d|%d|%s|%d|%d|%d\n", t->GetName(), t->GetFirstChannel(), t->GetNumChannels(),
            ChannelFormatToString(t->GetChannelFormat()), int(t->GetBlockCompressedFormat()), int(t->GetRgbColorSpace()), int(t->GetAlphaColorSpace()));
        for (int mip = 0; mip < d.mips; ++mip) {
            BufferFootprint const fp = t->GetBC7ModeBufferFootprint(mip);
            if (fp.rangeInStream.size == 0) continue;
            void const* data = nullptr; size_t size = 0;
            t->GetBC7ModeBuffer(mip, &data, &size);
            unsigned long long sum = 0;
            for (size_t b = 0; b < size; ++b) sum = sum * 131 + static_cast<unsigned char const*>(data)[b];
            std::printf("modes %d %d %llu %llu %d %llu %zu %llu\n", i, mip, (unsigned long long)fp.rangeInStream.offset, (unsigned long long)fp.rangeInStream.size,
                int(fp.compressionType), (unsigned long long)fp.uncompressedSize, size, sum);
        }
    }
    LatentTextureDesc const lt = set->GetLatentTextureDesc();
    for (int level = 0; level < set->GetNumLatentImages(); ++level)
        for (int layer = 0; layer < lt.arraySize; ++layer) {
            LatentTextureFootprint fp;
            CHECK(set->GetLatentTextureFootprint(level, layer, fp) == Status::Ok);
            std::printf("latent %d %d %llu %llu %d %llu %u %d %d %zu\n", level, layer, (unsigned long long)fp.buffer.rangeInStream.offset,
                (unsigned long long)fp.buffer.rangeInStream.size, int(fp.buffer.compressionType), (unsigned long long)fp.buffer.uncompressedSize,
                fp.buffer.uncompressedCrc32, fp.width, fp.height, fp.rowPitch);
        }
    {
        LatentTextureFootprint fp;
        CHECK(set->GetLatentTextureFootprint(-1, 0, fp) == Status::OutOfRange);
        CHECK(set->GetLatentTextureFootprint(set->GetNumLatentImages(), 0, fp) == Status::OutOfRange);
        if (set->GetNumLatentImages() > 0) {
            CHECK(set->GetLatentTextureFootprint(0, -1, fp) == Status::OutOfRange);
            CHECK(set->GetLatentTextureFootprint(0, lt.arraySize, fp) == Status::OutOfRange);
        }
    }
    std::printf("colorspaces");
    for (int c = 0; c < d.channels; ++c) std::printf(" %d", int(set->GetChannelStorageColorSpace(c)));
    std::printf("\nmask 0x%x\n", set->GetValidChannelMask());
    return 0;
}

static int load(int argc, char** argv)
{
    if (argc < 4) { std::fprintf(stderr, "usage: load <file> <device 0|1> [<w> <h> <channels> <mips>]\n"); return 2; }
    IContext* ctx = nullptr;
    ContextParameters params;
    if (std::atoi(argv[3]) == 0) params.cudaDevice = DisableCudaDevice;
    Status const created = CreateContext(&ctx, params);
    CHECK(ctx != nullptr && (created == Status::Ok || created == Status::CudaUnavailable));
    if (created == Status::CudaUnavailable) X(ctx)->AllowTextureSetsWithoutDevice(true);
    ITextureSet* set = nullptr;
    Status status;
    if (argc >= 8) {
        TextureSetDesc desc; desc.width = std::atoi(argv[4]); desc.height = std::atoi(argv[5]); desc.channels = std::atoi(argv[6]); desc.mips = std::atoi(argv[7]);
        CHECK(ctx->CreateTextureSet(desc, TextureSetFeatures(), &set) == Status::Ok);
        status = set->LoadFromFile(argv[2]);
    } else {
        status = ctx->CreateCompressedTextureSetFromFile(argv[2], TextureSetFeatures(), &set);
        CHECK((status == Status::Ok) == (set != nullptr));
    }
    std::printf("status %d %s\nmessage %s\n", int(status), StatusToString(status), GetLastErrorMessage());
    if (set) { CHECK(describe(set) == 0); ctx->DestroyTextureSet(set); }
    DestroyContext(ctx);
    return 0;
}

// What a file says about its set, read without a device and without the latents.
static int metadata(int argc, char** argv)
{
    if (argc < 3) { std::fprintf(stderr, "usage: metadata <file>\n"); return 2; }
    IContext* ctx = nullptr;
    ContextParameters params; params.cudaDevice = DisableCudaDevice;
    CHECK(CreateContext(&ctx, params) == Status::CudaUnavailable && ctx != nullptr);
    IStream* stream = nullptr;
    CHECK(ctx->OpenFile(argv[2], false, &stream) == Status::Ok);
    ITextureSetMetadata* set = nullptr;
    CHECK(ctx->CreateTextureSetMetadataFromStream(stream, nullptr) == Status::InvalidArgument);
    CHECK(ctx->CreateTextureSetMetadataFromStream(nullptr, &set) == Status::InvalidArgument);
    Status const status = ctx->CreateTextureSetMetadataFromStream(stream, &set);
    ctx->CloseFile(stream);
    CHECK((status == Status::Ok) == (set != nullptr));
    std::printf("status %d %s\nmessage %s\n", int(status), StatusToString(status), GetLastErrorMessage());
    if (set) {
        CHECK(describe(set) == 0);
        CHECK(dynamic_cast<ITextureSet*>(set) == nullptr || dynamic_cast<ITextureSet*>(set)->Decompress(nullptr, true) != Status::Ok);   // nothing to decode with
        void const* weights = nullptr; size_t weightSize = 0;
        CHECK(set->GetInferenceWeights(InferenceWeightType::GenericInt8, &weights, &weightSize, nullptr) == Status::Ok);
        unsigned long long sum = 0;
        for (size_t b = 0; b < weightSize; ++b) sum = sum * 131 + static_cast<unsigned char const*>(weights)[b];
        InferenceData data;
        CHECK(ctx->MakeInferenceData(set, InferenceWeightType::GenericInt8, 0, &data) == Status::Ok);
        std::printf("weights %zu %llu\ninference 0x%x 0x%x %d", weightSize, sum, data.constants.validChannelMask, data.constants.channelColorSpaces,
            data.constants.imageMips);
        for (int mip = 0; mip < data.constants.imageMips; ++mip)
            std::printf(" %d:%g:%g", data.constants.colorMips[mip].neuralMip, data.constants.colorMips[mip].positionScale, data.constants.colorMips[mip].positionLod);
        std::printf("\n");
        ctx->DestroyTextureSetMetadata(set);
    }
    DestroyContext(ctx);
    return 0;
}

static int decodeFile(int argc, char** argv)
{
    if (argc < 4) { std::fprintf(stderr, "usage: decodefile <file> <outPrefix>\n"); return 2; }
    std::vector<unsigned char> image = readFile(argv[2]);
    std::string const prefix = argv[3];
    IContext* ctx = nullptr;
    ContextParameters params;
    CHECK(CreateContext(&ctx, params) == Status::Ok);
    CHECK(ntc_hip_init(params.cudaDevice) == 0);              // the default context of the C ABI, for this program's own device buffers
    TextureSetFeatures features;
    features.stagingBytesPerPixel = 16 * 2;
    ITextureSet* set = nullptr;
    CHECK(ctx->CreateCompressedTextureSetFromMemory(image.data(), image.size(), features, &set) == Status::Ok);
    CHECK(describe(set) == 0);
    CHECK(set->Decompress(nullptr, true) == Status::Ok);
    TextureSetDesc const desc = set->GetDesc();
    for (int mip = 0; mip < desc.mips; ++mip) {
        ReadChannelsParameters rp;
        rp.mipLevel = mip; rp.firstChannel = 0; rp.numChannels = desc.channels;
        rp.width = std::max(desc.width >> mip, 1); rp.height = std::max(desc.height >> mip, 1);
        rp.pixelStride = size_t(desc.channels) * 2; rp.rowPitch = rp.pixelStride * size_t(rp.width);
        rp.channelFormat = ChannelFormat::FLOAT16;
        std::vector<unsigned char> pixels(rp.rowPitch * size_t(rp.height));
        rp.pOutData = pixels.data();
        CHECK(set->ReadChannels(rp) == Status::Ok);
        CHECK(writeFile(prefix + "_mip" + std::to_string(mip) + ".bin", pixels.data(), pixels.size()));
    }
    // loading the same file again into the existing set, through a stream this time
    IStream* stream = nullptr;
    CHECK(ctx->OpenFile(argv[2], false, &stream) == Status::Ok);
    CHECK(set->LoadFromStream(stream) == Status::Ok);
    ctx->CloseFile(stream);
    CHECK(set->Decompress(nullptr, true) == Status::Ok);
    ctx->DestroyTextureSet(set);
    DestroyContext(ctx);
    std::printf("host decodefile OK\n");
    return 0;
}

int main(int argc, char** argv)
{
    if (argc >= 2 && std::strcmp(argv[1], "load") == 0) return load(argc, argv);
    if (argc >= 2 && std::strcmp(argv[1], "metadata") == 0) return metadata(argc, argv);
    if (argc >= 2 && std::strcmp(argv[1], "decodefile") == 0) return decodeFile(argc, argv);
    if (argc >= 2 && std::strcmp(argv[1], "loss") == 0) return loss(argc, argv);
    if (argc >= 2 && std::strcmp(argv[1], "shuffle") == 0) return shuffle(argc, argv);
    if (argc >= 2 && std::strcmp(argv[1], "imagediff") == 0) return imageDifference();
    if (argc >= 2 && std::strcmp(argv[1], "genmips") == 0) return generateMips(argc, argv);
    if (argc >= 2 && std::strcmp(argv[1], "cpu") == 0) return cpuChecks();
    if (argc >= 2 && std::strcmp(argv[1], "decode") == 0) return decode(argc, argv);
    std::fprintf(stderr, "usage: host_api_test cpu | decode ...\n");
    return 2;
}
