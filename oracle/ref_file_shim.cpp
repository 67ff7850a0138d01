/*
 * ref_file_shim.cpp - C entry points over the reference's own NTC-file header and JSON code.
 *
 * TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/libntc_ref_file.so
 * together with the reference's src/JsonFileFormat.cpp, JsonSerialization.cpp, Stream.cpp,
 * Errors.cpp, TextureSetMetadata.cpp, TextureMetadata.cpp, FeatureGridMath.cpp, WeightLayout.cpp
 * and CoopVecWeightConverter.cpp, compiled where they lie (nothing is copied).  Only the static
 * entry points TextureSetMetadata::LoadFileHeadersFromStream / DeserializeTextureSetDesc and the
 * JSON (de)serialiser are reachable from here; the link drops every unreferenced section
 * (hidden visibility + --gc-sections), which is what removes the parts of those files that
 * need the CUDA context, the graphics back ends or GDeflate, none of which build here.
 *
 * It lets the tests check that (a) the files tests/ntex_writer.py produces are accepted by the
 * reference's loader front end with the same descriptor the host layer derives, (b) malformed
 * files are refused with the same status, and (c) the host layer reads JSON as the reference
 * itself serialises it.
 */
#include "TextureSetMetadata.h"
#include "JsonFileFormat.h"
#include "Stream.h"
#include "Errors.h"
#include <cstdint>
#include <cstdlib>
#include <cstring>

#define SHIM_API extern "C" __attribute__((visibility("default")))

namespace {
struct Mallocator final : ntc::IAllocator {
    void* Allocate(size_t size) override { return std::malloc(size); }
    void Deallocate(void* ptr, size_t) override { std::free(ptr); }
};
void copy_text(char* dst, int cap, char const* src)
{
    if (!dst || cap <= 0) return;
    std::strncpy(dst, src ? src : "", size_t(cap) - 1);
    dst[cap - 1] = 0;
}
}

// Runs LoadFileHeadersFromStream + DeserializeTextureSetDesc on a file image in memory.
// out[0..9] = width, height, channels, mips, gridSizeScale, numFeatures, #views, #latents,
// #colorMips, #textures; out64[0..1] = binary chunk offset and size.  Returns ntc::Status.
SHIM_API int ntc_ref_parse_file(void const* data, uint64_t size, int* out, uint64_t* out64, char* message, int messageCap)
{
    Mallocator allocator;
    ntc::MemoryStream stream(const_cast<uint8_t*>(static_cast<uint8_t const*>(data)), size, true);
    ntc::json::Document document(&allocator);
    uint64_t offset = 0, chunk = 0;
    ntc::ClearErrorMessage();
    ntc::Status status = ntc::TextureSetMetadata::LoadFileHeadersFromStream(&allocator, &stream, document, offset, chunk);
    ntc::TextureSetDesc desc{};
    ntc::LatentShape shape = ntc::LatentShape::Empty();
    if (status == ntc::Status::Ok)
        status = ntc::TextureSetMetadata::DeserializeTextureSetDesc(document, desc, shape);
    out[0] = desc.width; out[1] = desc.height; out[2] = desc.channels; out[3] = desc.mips;
    out[4] = shape.gridSizeScale; out[5] = shape.numFeatures;
    out[6] = int(document.views.size()); out[7] = int(document.latents.size());
    out[8] = int(document.colorMips.size()); out[9] = int(document.textures.size());
    out64[0] = offset; out64[1] = chunk;
    copy_text(message, messageCap, ntc::GetErrorBuffer());
    return int(status);
}

// Parses a JSON chunk with the reference's parser and writes it back with the reference's
// serialiser.  Returns 0, or 1 when parsing failed, 2 when serialising failed, 3 when the
// output does not fit; `error` receives the reference's message.
SHIM_API int ntc_ref_reserialize_json(char const* json, char* out, int outCap, char* error, int errorCap)
{
    Mallocator allocator;
    ntc::Vector<char> text(&allocator);
    text.assign(json, json + std::strlen(json) + 1);          // parsed in place, so on a copy
    ntc::json::Document document(&allocator);
    ntc::String message(&allocator);
    if (!ntc::json::ParseDocument(document, text.data(), message)) { copy_text(error, errorCap, message.c_str()); return 1; }
    ntc::String result(&allocator);
    if (!ntc::json::SerializeDocument(document, result, message)) { copy_text(error, errorCap, message.c_str()); return 2; }
    if (int(result.size()) + 1 > outCap) return 3;
    copy_text(out, outCap, result.c_str());
    copy_text(error, errorCap, "");
    return 0;
}
