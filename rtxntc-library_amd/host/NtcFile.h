// NtcFile.h - reader of the NTC texture-set container ("NTEX" files), host side only.
//
// The container (reference src/JsonFileFormat.h:26-38,188-218): a 40-byte binary header, a JSON
// chunk describing the texture set, and a binary chunk that the JSON's "views" index into.
// This reader covers what the decompression path consumes: set dimensions, latent shape, the Int8
// version of the MLP, latent image layers, colour-mip mapping and texture metadata.  It is the
// counterpart of TextureSetMetadata::LoadFileHeadersFromStream / DeserializeTextureSetDesc
// (src/TextureSetMetadata.cpp:1180-1264) and of json::ParseDocument (src/JsonFileFormat.cpp:189-192).
#pragma once

#include <cstdint>
#include <optional>
#include <string>
#include <vector>

namespace ntc::file
{

constexpr uint32_t kSignature = 0x5845544E;      // "NTEX", src/JsonFileFormat.h:29
constexpr uint32_t kContainerVersion = 0x100;    // src/JsonFileFormat.h:30
constexpr uint32_t kSchemaVersion = 3;           // src/JsonFileFormat.h:190

struct Header                                     // src/JsonFileFormat.h:27-39, 40 bytes, little endian
{
    uint32_t signature = 0, version = 0;
    uint64_t jsonChunkOffset = 0, jsonChunkSize = 0, binaryChunkOffset = 0, binaryChunkSize = 0;
};

enum class Compression { None, GDeflate };
enum class MatrixLayout { RowMajor, ColumnMajor };
enum class MlpDataType { Int8, Int32, FloatE4M3, FloatE5M2, Float16, Float32 };

struct BufferView
{
    uint64_t offset = 0, storedSize = 0;
    std::optional<Compression> compression;
    std::optional<uint64_t> uncompressedSize;
    std::optional<uint32_t> crc32;
};

struct MlpLayer
{
    uint32_t inputChannels = 0, outputChannels = 0, weightView = 0, biasView = 0;
    std::optional<uint32_t> scaleView;
    MlpDataType weightType = MlpDataType::Int8, biasType = MlpDataType::Int8;
    std::optional<MlpDataType> scaleType;
};

struct Mlp
{
    std::vector<MlpLayer> layers;
    std::optional<MatrixLayout> weightLayout;
};

struct Texture
{
    std::string name;
    uint32_t firstChannel = 0, numChannels = 0;
    std::optional<int> channelFormat, rgbColorSpace, alphaColorSpace, bcFormat;   // values of the public enums
    struct ModeBuffer { uint32_t mipLevel = 0, view = 0; };
    std::vector<ModeBuffer> bcModeBuffers;              // BC7 acceleration data, one view per colour mip
};

struct LatentImage
{
    uint32_t width = 0, height = 0;
    std::vector<uint32_t> layerViews;
};

struct ColorMip
{
    std::optional<uint32_t> width, height, latentMip;
    std::optional<float> positionLod, positionScale;
};

struct Document                                   // src/JsonFileFormat.h:188-218
{
    uint32_t schemaVersion = 0, width = 0, height = 0, numChannels = 0;
    std::optional<uint32_t> numColorMips;
    std::optional<uint32_t> latentFeatures;       // latentShape.numFeatures
    std::vector<Mlp> mlpVersions;
    std::vector<Texture> textures;
    std::vector<std::optional<int>> channelColorSpaces;
    std::vector<LatentImage> latents;
    std::vector<ColorMip> colorMips;
    std::vector<BufferView> views;
};

// Parses the JSON chunk.  Unknown members are skipped, required members must be present and of
// the right type (src/JsonSerialization.cpp:310-930).  On failure `error` says what and where.
bool ParseDocument(char const* json, size_t length, Document& out, std::string& error);

// Decodes the 40-byte header from `bytes` (at least 40 of them).
Header DecodeHeader(unsigned char const* bytes);

} // namespace ntc::file
