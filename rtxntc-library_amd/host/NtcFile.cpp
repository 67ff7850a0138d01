// NtcFile.cpp - JSON chunk parser of the NTC container.  See NtcFile.h.
//
// Two stages: a small strict JSON reader builds a value tree (texts are a few kB), then typed
// extraction walks the tree member by member with the presence and type rules of the
// reference's schema tables (src/JsonFileFormat.cpp:25-186): plain scalars are required,
// optionals and arrays are not, unknown members are ignored, integers must fit their field.
#include "NtcFile.h"

#include <cinttypes>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <utility>

namespace ntc::file
{
namespace
{

struct Value
{
    enum Kind { Null, Bool, Integer, Real, String, Array, Object };
    Kind kind = Null;
    bool boolean = false;
    bool negative = false;          // Integer: sign, magnitude below
    uint64_t magnitude = 0;
    double real = 0.0;
    std::string text;
    // Where the reference's streaming reader stands when it rejects this value (it reports that offset and the
    // text that follows): the first character of a number; just behind a string, a literal, or the opening
    // bracket of an array or object.  closeAt: just behind the closing bracket, where missing members of an object
    // (closing bracket) are noticed.
    size_t at = 0, closeAt = 0;
    std::vector<Value> items;
    std::vector<std::pair<std::string, Value>> members;

    Value const* Find(char const* name) const
    {
        Value const* found = nullptr;       // the last of duplicate keys wins, as with a streaming reader
        for (auto const& m : members) if (m.first == name) found = &m.second;
        return found;
    }
};

char const* KindName(Value::Kind k)
{
    switch (k) {
    case Value::Null: return "null";
    case Value::Bool: return "bool";
    case Value::Integer: return "integer";
    case Value::Real: return "double";
    case Value::String: return "string";
    case Value::Array: return "array";
    default: return "object";
    }
}

class Reader
{
public:
    Reader(char const* text, size_t length, std::string& error) : m_p(text), m_end(text + length), m_begin(text), m_error(error) {}

    bool ParseRoot(Value& out)
    {
        SkipSpace();
        if (m_p == m_end) return Fail("The document is empty.");
        if (!ParseValue(out, 0)) return false;
        SkipSpace();
        if (m_p != m_end && *m_p != 0) return Fail("The document root must not be followed by other values.");
        return true;
    }

private:
    static constexpr int kMaxDepth = 32;

    bool Fail(char const* what)
    {
        char snippet[32];
        size_t const left = size_t(m_end - m_p);
        size_t const n = left < 28 ? left : 28;
        std::memcpy(snippet, m_p, n);
        snippet[n] = 0;
        char buf[256];
        std::snprintf(buf, sizeof buf, "Error at character %zu (%s%s): %s", size_t(m_p - m_begin), snippet, left > n ? "..." : "", what);
        m_error = buf;
        return false;
    }
    void SkipSpace() { while (m_p != m_end && (*m_p == ' ' || *m_p == '\t' || *m_p == '\n' || *m_p == '\r')) ++m_p; }
    bool Literal(char const* word)
    {
        size_t const n = std::strlen(word);
        if (size_t(m_end - m_p) < n || std::memcmp(m_p, word, n) != 0) return Fail("Invalid value.");
        m_p += n;
        return true;
    }

    bool ParseValue(Value& out, int depth)
    {
        if (depth > kMaxDepth) return Fail("The document is nested too deeply.");
        if (m_p == m_end) return Fail("Invalid value.");
        bool ok;
        switch (*m_p) {
        case '{': return ParseObject(out, depth);
        case '[': return ParseArray(out, depth);
        case '"': out.kind = Value::String; ok = ParseString(out.text); break;
        case 't': out.kind = Value::Bool; out.boolean = true; ok = Literal("true"); break;
        case 'f': out.kind = Value::Bool; out.boolean = false; ok = Literal("false"); break;
        case 'n': out.kind = Value::Null; ok = Literal("null"); break;
        default: out.at = size_t(m_p - m_begin); return ParseNumber(out);
        }
        out.at = size_t(m_p - m_begin);
        return ok;
    }

    bool ParseObject(Value& out, int depth)
    {
        out.kind = Value::Object;
        ++m_p;
        out.at = size_t(m_p - m_begin);
        SkipSpace();
        if (m_p != m_end && *m_p == '}') { ++m_p; out.closeAt = size_t(m_p - m_begin); return true; }
        for (;;) {
            SkipSpace();
            if (m_p == m_end || *m_p != '"') return Fail("Missing a name for object member.");
            std::string key;
            if (!ParseString(key)) return false;
            SkipSpace();
            if (m_p == m_end || *m_p != ':') return Fail("Missing a colon after a name of object member.");
            ++m_p;
            SkipSpace();
            out.members.emplace_back(std::move(key), Value());
            if (!ParseValue(out.members.back().second, depth + 1)) return false;
            SkipSpace();
            if (m_p != m_end && *m_p == ',') { ++m_p; continue; }
            if (m_p != m_end && *m_p == '}') { ++m_p; out.closeAt = size_t(m_p - m_begin); return true; }
            return Fail("Missing a comma or '}' after an object member.");
        }
    }

    bool ParseArray(Value& out, int depth)
    {
        out.kind = Value::Array;
        ++m_p;
        out.at = size_t(m_p - m_begin);
        SkipSpace();
        if (m_p != m_end && *m_p == ']') { ++m_p; out.closeAt = size_t(m_p - m_begin); return true; }
        for (;;) {
            SkipSpace();
            out.items.emplace_back();
            if (!ParseValue(out.items.back(), depth + 1)) return false;
            SkipSpace();
            if (m_p != m_end && *m_p == ',') { ++m_p; continue; }
            if (m_p != m_end && *m_p == ']') { ++m_p; out.closeAt = size_t(m_p - m_begin); return true; }
            return Fail("Missing a comma or ']' after an array element.");
        }
    }

    static void AppendUtf8(std::string& s, uint32_t cp)
    {
        if (cp < 0x80) s += char(cp);
        else if (cp < 0x800) { s += char(0xC0 | (cp >> 6)); s += char(0x80 | (cp & 0x3F)); }
        else if (cp < 0x10000) { s += char(0xE0 | (cp >> 12)); s += char(0x80 | ((cp >> 6) & 0x3F)); s += char(0x80 | (cp & 0x3F)); }
        else { s += char(0xF0 | (cp >> 18)); s += char(0x80 | ((cp >> 12) & 0x3F)); s += char(0x80 | ((cp >> 6) & 0x3F)); s += char(0x80 | (cp & 0x3F)); }
    }
    bool Hex4(uint32_t& out)
    {
        if (m_end - m_p < 4) return Fail("Incorrect hex digit after \\u escape in string.");
        out = 0;
        for (int i = 0; i < 4; ++i) {
            char const c = *m_p++;
            out <<= 4;
            if (c >= '0' && c <= '9') out |= uint32_t(c - '0');
            else if (c >= 'a' && c <= 'f') out |= uint32_t(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') out |= uint32_t(c - 'A' + 10);
            else { --m_p; return Fail("Incorrect hex digit after \\u escape in string."); }
        }
        return true;
    }

    bool ParseString(std::string& out)
    {
        ++m_p;      // opening quote
        for (;;) {
            if (m_p == m_end) return Fail("Missing a closing quotation mark in string.");
            unsigned char const c = static_cast<unsigned char>(*m_p);
            if (c == '"') { ++m_p; return true; }
            if (c < 0x20) return Fail("Invalid encoding in string.");
            if (c != '\\') { out += char(c); ++m_p; continue; }
            ++m_p;
            if (m_p == m_end) return Fail("Invalid escape character in string.");
            char const e = *m_p++;
            switch (e) {
            case '"': out += '"'; break;
            case '\\': out += '\\'; break;
            case '/': out += '/'; break;
            case 'b': out += '\b'; break;
            case 'f': out += '\f'; break;
            case 'n': out += '\n'; break;
            case 'r': out += '\r'; break;
            case 't': out += '\t'; break;
            case 'u': {
                uint32_t cp = 0;
                if (!Hex4(cp)) return false;
                if (cp >= 0xD800 && cp <= 0xDBFF) {
                    uint32_t low = 0;
                    if (m_end - m_p < 2 || m_p[0] != '\\' || m_p[1] != 'u') return Fail("The surrogate pair in string is invalid.");
                    m_p += 2;
                    if (!Hex4(low)) return false;
                    if (low < 0xDC00 || low > 0xDFFF) return Fail("The surrogate pair in string is invalid.");
                    cp = 0x10000 + ((cp - 0xD800) << 10) + (low - 0xDC00);
                } else if (cp >= 0xDC00 && cp <= 0xDFFF) {
                    return Fail("The surrogate pair in string is invalid.");
                }
                AppendUtf8(out, cp);
                break;
            }
            default: --m_p; return Fail("Invalid escape character in string.");
            }
        }
    }

    bool ParseNumber(Value& out)
    {
        char const* const start = m_p;
        bool negative = false;
        if (m_p != m_end && *m_p == '-') { negative = true; ++m_p; }
        if (m_p == m_end || *m_p < '0' || *m_p > '9') { m_p = start; return Fail("Invalid value."); }
        uint64_t magnitude = 0;
        bool overflow = false;
        if (*m_p == '0') ++m_p;
        else while (m_p != m_end && *m_p >= '0' && *m_p <= '9') {
            uint64_t const digit = uint64_t(*m_p - '0');
            if (magnitude > (UINT64_MAX - digit) / 10) overflow = true;
            else magnitude = magnitude * 10 + digit;
            ++m_p;
        }
        bool real = false;
        if (m_p != m_end && *m_p == '.') {
            real = true;
            ++m_p;
            if (m_p == m_end || *m_p < '0' || *m_p > '9') return Fail("Miss fraction part in number.");
            while (m_p != m_end && *m_p >= '0' && *m_p <= '9') ++m_p;
        }
        if (m_p != m_end && (*m_p == 'e' || *m_p == 'E')) {
            real = true;
            ++m_p;
            if (m_p != m_end && (*m_p == '+' || *m_p == '-')) ++m_p;
            if (m_p == m_end || *m_p < '0' || *m_p > '9') return Fail("Miss exponent in number.");
            while (m_p != m_end && *m_p >= '0' && *m_p <= '9') ++m_p;
        }
        if (real || overflow || (negative && magnitude > uint64_t(INT64_MAX) + 1)) {
            std::string const token(start, size_t(m_p - start));
            out.kind = Value::Real;
            out.real = std::strtod(token.c_str(), nullptr);
            if (!std::isfinite(out.real)) { m_p = start; return Fail("Number too big to be stored in double."); }
            return true;
        }
        out.kind = Value::Integer;
        out.negative = negative && magnitude != 0;
        out.magnitude = magnitude;
        return true;
    }

    char const* m_p;
    char const* m_end;
    char const* m_begin;
    std::string& m_error;
};

// A complaint about the value at text offset `at`, to be completed by ParseDocument, which has the text:
// marker, offset, marker, message.
constexpr char kLocated = '\x01';
std::string LocatedMessage(size_t at, char const* message)
{
    return std::string(1, kLocated) + std::to_string(at) + kLocated + message;
}

// "Error at character N (the 28 characters from there on, "..." when more follow): message", the form of the
// reference's reader (src/JsonSerialization.cpp:1040-1058).
std::string ExpandLocatedMessage(std::string const& error, char const* json, size_t length)
{
    if (error.empty() || error[0] != kLocated) return error;
    size_t const second = error.find(kLocated, 1);
    if (second == std::string::npos) return error;
    size_t at = size_t(std::strtoull(error.c_str() + 1, nullptr, 10));
    if (at > length) at = length;
    size_t left = 0;
    while (at + left < length && json[at + left] != 0) ++left;
    size_t const n = left < 28 ? left : 28;
    char buf[512];
    std::snprintf(buf, sizeof buf, "Error at character %zu (%.*s%s): %s", at, int(n), json + at, left > n ? "..." : "", error.c_str() + second + 1);
    return buf;
}

// Typed access to the members of one JSON object of schema type `typeName`.
class Members
{
public:
    Members(Value const& object, char const* typeName, std::string& error) : m_object(object), m_type(typeName), m_error(error) {}

    bool UInt(char const* name, uint32_t& out) { return !Required(name) || AsUnsigned(name, *m_found, UINT32_MAX, "uint", [&](uint64_t v) { out = uint32_t(v); }); }
    bool UInt64(char const* name, uint64_t& out) { return !Required(name) || AsUnsigned(name, *m_found, UINT64_MAX, "uint64", [&](uint64_t v) { out = v; }); }
    // To be called when every member has been read: fails if a required one was absent.
    bool Complete()
    {
        if (!m_missing) return true;
        Format(m_object.closeAt, "Missing value for required field '%s.%s'", m_type, m_missing);
        return false;
    }
    bool Has(char const* name) const { return m_object.Find(name) != nullptr; }
    bool OptionalUInt(char const* name, std::optional<uint32_t>& out)
    {
        if (!Optional(name)) return true;
        return AsUnsigned(name, *m_found, UINT32_MAX, "uint", [&](uint64_t v) { out = uint32_t(v); });
    }
    bool OptionalUInt64(char const* name, std::optional<uint64_t>& out)
    {
        if (!Optional(name)) return true;
        return AsUnsigned(name, *m_found, UINT64_MAX, "uint64", [&](uint64_t v) { out = v; });
    }
    bool OptionalFloat(char const* name, std::optional<float>& out)
    {
        if (!Optional(name)) return true;
        Value const& v = *m_found;
        if (v.kind == Value::Real) { out = float(v.real); return true; }
        if (v.kind == Value::Integer) { out = v.negative ? -float(v.magnitude) : float(v.magnitude); return true; }
        return WrongType(name, "float", v);
    }
    bool String(char const* name, std::string& out)
    {
        if (!Required(name)) return true;
        if (m_found->kind != Value::String) return WrongType(name, "string", *m_found);
        out = m_found->text;
        return true;
    }
    // names[i] is the spelling of enum value i
    template <typename E> bool Enum(char const* name, E& out, std::initializer_list<char const*> names)
    {
        if (!Required(name)) return true;
        int index;
        if (!AsEnum(name, *m_found, names, index)) return false;
        out = E(index);
        return true;
    }
    template <typename E> bool OptionalEnum(char const* name, std::optional<E>& out, std::initializer_list<char const*> names)
    {
        if (!Optional(name)) return true;
        int index;
        if (!AsEnum(name, *m_found, names, index)) return false;
        out = E(index);
        return true;
    }
    // Arrays are never required (src/JsonSerialization.h:262-282); returns null when absent.
    bool Array(char const* name, char const* expected, Value const*& out)
    {
        out = nullptr;
        if (!Optional(name)) return true;
        if (m_found->kind != Value::Array) return WrongType(name, expected, *m_found);
        out = m_found;
        return true;
    }
    // Hands the elements of an array of objects to `read`, one after the other in the order of the text, each
    // checked to be an object first.  Never required; a bare object counts as an array of one, as with the
    // reference's reader.
    template <typename Read> bool ForEachObject(char const* name, Read read)
    {
        if (!Optional(name)) return true;
        Value const& field = *m_found;
        if (field.kind == Value::Object) return read(field);
        if (field.kind != Value::Array) return WrongType(name, "array", field);
        for (Value const& item : field.items)
            if (!ElementMustBeObject(name, item, field) || !read(item)) return false;
        return true;
    }
    bool OptionalObject(char const* name, Value const*& out)
    {
        out = nullptr;
        if (!Optional(name)) return true;
        if (m_found->kind != Value::Object) return WrongType(name, "object", *m_found);
        out = m_found;
        return true;
    }
    bool ArrayOfUInt(char const* name, std::vector<uint32_t>& out)
    {
        if (!Optional(name)) return true;
        // a bare number counts as an array of one, as with the reference's reader
        if (m_found->kind == Value::Integer) return AsUnsigned(name, *m_found, UINT32_MAX, "uint", [&](uint64_t v) { out.push_back(uint32_t(v)); });
        if (m_found->kind != Value::Array) return WrongType(name, "uint", *m_found);
        return UIntElements(name, *m_found, nullptr, out);
    }
    // An element of an array of objects.  The reference's reader takes an array in that place for the start of the
    // field's own array once more: a scalar inside it is then the wrong thing in an array of objects, and when the
    // nested array closes, the field's array counts as closed, which its real end then trips over.
    bool ElementMustBeObject(char const* name, Value const& item, Value const& fieldArray)
    {
        if (item.kind == Value::Object) return true;
        Value const* inner = &item;
        while (inner->kind == Value::Array && !inner->items.empty() && inner->items.front().kind == Value::Array) inner = &inner->items.front();
        if (inner->kind != Value::Array) return WrongType(name, "array", item);
        if (!inner->items.empty() && inner->items.front().kind != Value::Object) return WrongType(name, "array", inner->items.front());
        m_error = LocatedMessage(fieldArray.closeAt, "End-of-array encountered outside of an array");
        return false;
    }

private:
    // The elements of an array of numbers.  A nested array is taken by the reference's reader for the start of the
    // field's array once more; when the first such array closes, the field's array counts as closed, the
    // elements that follow are skipped, and the next closing bracket (the parent's) is one too many.
    bool UIntElements(char const* name, Value const& array, Value const* parent, std::vector<uint32_t>& out)
    {
        for (Value const& item : array.items) {
            if (item.kind == Value::Array) return UIntElements(name, item, &array, out);
            if (!AsUnsigned(name, item, UINT32_MAX, "uint", [&](uint64_t v) { out.push_back(uint32_t(v)); })) return false;
        }
        if (!parent) return true;
        m_error = LocatedMessage(parent->closeAt, "End-of-array encountered outside of an array");
        return false;
    }
    bool Optional(char const* name) { m_found = m_object.Find(name); return m_found != nullptr; }
    // A required member that is absent is noticed where the object ends (Complete), after the members that are
    // there have had their say: the order in which a streaming reader meets the faults of a document.
    bool Required(char const* name)
    {
        if (Optional(name)) return true;
        if (!m_missing) m_missing = name;
        return false;
    }
    bool WrongType(char const* name, char const* expected, Value const& v)
    {
        Format(v.at, "Expected %s for '%s.%s', got %s", expected, m_type, name, KindName(v.kind));
        return false;
    }
    template <typename Store> bool AsUnsigned(char const* name, Value const& v, uint64_t limit, char const* expected, Store store)
    {
        if (v.kind != Value::Integer) return WrongType(name, expected, v);
        // a 64-bit field takes any integer, a negative one as its two's complement: the reference's reader stores
        // what it is given there (src/JsonSerialization.cpp:499-527); what such a value means is checked later
        if (limit == UINT64_MAX) { store(v.negative ? uint64_t(0) - v.magnitude : v.magnitude); return true; }
        if (v.negative || v.magnitude > limit) {
            char buf[256];
            // the reference prints the value through a signed 64-bit integer: 2^63 and above come out negative
            if (!v.negative && v.magnitude > uint64_t(INT64_MAX))
                std::snprintf(buf, sizeof buf, "Value %" PRId64 " is out of range for %s field '%s.%s'", int64_t(v.magnitude), expected, m_type, name);
            else
                std::snprintf(buf, sizeof buf, "Value %s%" PRIu64 " is out of range for %s field '%s.%s'", v.negative ? "-" : "", v.magnitude, expected, m_type, name);
            m_error = LocatedMessage(v.at, buf);
            return false;
        }
        store(v.magnitude);
        return true;
    }
    bool AsEnum(char const* name, Value const& v, std::initializer_list<char const*> names, int& index)
    {
        if (v.kind != Value::String) return WrongType(name, "enum", v);
        index = 0;
        for (char const* candidate : names) {
            if (v.text == candidate) return true;
            ++index;
        }
        Format(v.at, "Unknown value '%s' specified for '%s.%s'", v.text.c_str(), m_type, name);
        return false;
    }
    void Format(size_t at, char const* fmt, char const* a, char const* b, char const* c = nullptr, char const* d = nullptr)
    {
        char buf[320];
        std::snprintf(buf, sizeof buf, fmt, a, b, c, d);
        m_error = LocatedMessage(at, buf);
    }

    Value const& m_object;
    char const* m_type;
    std::string& m_error;
    Value const* m_found = nullptr;
    char const* m_missing = nullptr;        // the first required member found absent
};

// spellings in the order of the enums (src/JsonFileFormat.cpp:25-113)
#define NTC_FILE_MLP_TYPES { "Int8", "Int32", "FloatE4M3", "FloatE5M2", "Float16", "Float32" }
#define NTC_FILE_CHANNEL_FORMATS { "UNKNOWN", "UNORM8", "UNORM16", "FLOAT16", "FLOAT32", "UINT32" }
#define NTC_FILE_COLOR_SPACES { "Linear", "sRGB", "HLG" }
#define NTC_FILE_BC_FORMATS { "None", "BC1", "BC2", "BC3", "BC4", "BC5", "BC6", "BC7" }

bool ReadView(Value const& v, BufferView& out, std::string& error)
{
    Members m(v, "BufferView", error);
    return m.UInt64("offset", out.offset) && m.UInt64("storedSize", out.storedSize)
        && m.OptionalEnum("compression", out.compression, { "None", "GDeflate" })
        && m.OptionalUInt64("uncompressedSize", out.uncompressedSize) && m.OptionalUInt("crc32", out.crc32) && m.Complete();
}

bool ReadLayer(Value const& v, MlpLayer& out, std::string& error)
{
    Members m(v, "MLPLayer", error);
    return m.UInt("inputChannels", out.inputChannels) && m.UInt("outputChannels", out.outputChannels)
        && m.UInt("weightView", out.weightView) && m.OptionalUInt("scaleView", out.scaleView) && m.UInt("biasView", out.biasView)
        && m.Enum("weightType", out.weightType, NTC_FILE_MLP_TYPES)
        && m.OptionalEnum("scaleType", out.scaleType, NTC_FILE_MLP_TYPES)
        && m.Enum("biasType", out.biasType, NTC_FILE_MLP_TYPES) && m.Complete();
}

bool ReadMlp(Value const& v, Mlp& out, std::string& error)
{
    Members m(v, "MLP", error);
    if (!m.ForEachObject("layers", [&](Value const& item) { out.layers.emplace_back(); return ReadLayer(item, out.layers.back(), error); }))
        return false;
    std::optional<int> activation;
    return m.OptionalEnum("activation", activation, { "HGELUClamp" })
        && m.OptionalEnum("weightLayout", out.weightLayout, { "RowMajor", "ColumnMajor" }) && m.Complete();
}

bool ReadTexture(Value const& v, Texture& out, std::string& error)
{
    Members m(v, "Texture", error);
    if (!(m.String("name", out.name) && m.UInt("firstChannel", out.firstChannel) && m.UInt("numChannels", out.numChannels)
        && m.OptionalEnum("channelFormat", out.channelFormat, NTC_FILE_CHANNEL_FORMATS)
        && m.OptionalEnum("rgbColorSpace", out.rgbColorSpace, NTC_FILE_COLOR_SPACES)
        && m.OptionalEnum("alphaColorSpace", out.alphaColorSpace, NTC_FILE_COLOR_SPACES)
        && m.OptionalEnum("bcFormat", out.bcFormat, NTC_FILE_BC_FORMATS)))
        return false;
    // BC7 mode buffers: which view holds the (mode, partition) map of which colour mip
    return m.ForEachObject("bcModeBuffers", [&](Value const& item) {
        Members b(item, "BCModeBuffer", error);
        Texture::ModeBuffer ref;
        if (!(b.UInt("mipLevel", ref.mipLevel) && b.UInt("view", ref.view) && b.Complete())) return false;
        out.bcModeBuffers.push_back(ref);
        return true;
    }) && m.Complete();
}

bool ReadColorMip(Value const& v, ColorMip& out, std::string& error)
{
    Members m(v, "ColorMip", error);
    return m.OptionalUInt("width", out.width) && m.OptionalUInt("height", out.height) && m.OptionalUInt("latentMip", out.latentMip)
        && m.OptionalFloat("positionLod", out.positionLod) && m.OptionalFloat("positionScale", out.positionScale) && m.Complete();
}

template <typename T, typename ReadOne>
bool ReadObjectArray(Members& parent, char const* name, std::vector<T>& out, ReadOne readOne)
{
    return parent.ForEachObject(name, [&](Value const& item) { out.emplace_back(); return readOne(item, out.back()); });
}

} // namespace

namespace
{
bool ParseDocumentValues(char const* json, size_t length, Document& out, std::string& error);
}

bool ParseDocument(char const* json, size_t length, Document& out, std::string& error)
{
    if (ParseDocumentValues(json, length, out, error)) return true;
    error = ExpandLocatedMessage(error, json, length);
    return false;
}

namespace
{
bool ParseDocumentValues(char const* json, size_t length, Document& out, std::string& error)
{
    Value root;
    Reader reader(json, length, error);
    if (!reader.ParseRoot(root)) return false;
    if (root.kind != Value::Object) { error = LocatedMessage(root.at, (std::string("Expected object, got ") + KindName(root.kind)).c_str()); return false; }

    Members m(root, "Document", error);
    if (!m.UInt("schemaVersion", out.schemaVersion)) return false;
    if (m.Has("schemaVersion") && out.schemaVersion != kSchemaVersion) {      // src/JsonFileFormat.cpp:194-210
        char buf[128];
        std::snprintf(buf, sizeof buf, "Incompatible file schema version %u, expected %u", out.schemaVersion, kSchemaVersion);
        error = LocatedMessage(root.Find("schemaVersion")->at, buf);
        return false;
    }
    if (!(m.UInt("width", out.width) && m.UInt("height", out.height) && m.UInt("numChannels", out.numChannels)
        && m.OptionalUInt("numColorMips", out.numColorMips)))
        return false;
    Value const* latentShape;
    if (!m.OptionalObject("latentShape", latentShape)) return false;
    if (latentShape) {
        Members s(*latentShape, "LatentShape", error);
        uint32_t features = 0;
        if (!(s.UInt("numFeatures", features) && s.Complete())) return false;
        out.latentFeatures = features;
    }
    return ReadObjectArray(m, "mlpVersions", out.mlpVersions, [&](Value const& v, Mlp& o) { return ReadMlp(v, o, error); })
        && ReadObjectArray(m, "textures", out.textures, [&](Value const& v, Texture& o) { return ReadTexture(v, o, error); })
        && ReadObjectArray(m, "channels", out.channelColorSpaces, [&](Value const& v, std::optional<int>& o) {
               Members c(v, "Channel", error);
               return c.OptionalEnum("colorSpace", o, NTC_FILE_COLOR_SPACES) && c.Complete(); })
        && ReadObjectArray(m, "latents", out.latents, [&](Value const& v, LatentImage& o) {
               Members l(v, "LatentImage", error);
               return l.UInt("width", o.width) && l.UInt("height", o.height) && l.ArrayOfUInt("layerViews", o.layerViews) && l.Complete(); })
        && ReadObjectArray(m, "colorMips", out.colorMips, [&](Value const& v, ColorMip& o) { return ReadColorMip(v, o, error); })
        && ReadObjectArray(m, "views", out.views, [&](Value const& v, BufferView& o) { return ReadView(v, o, error); })
        && m.Complete();
}
} // namespace

Header DecodeHeader(unsigned char const* b)
{
    auto u32 = [&](int at) { return uint32_t(b[at]) | uint32_t(b[at + 1]) << 8 | uint32_t(b[at + 2]) << 16 | uint32_t(b[at + 3]) << 24; };
    auto u64 = [&](int at) { return uint64_t(u32(at)) | uint64_t(u32(at + 4)) << 32; };
    Header h;
    h.signature = u32(0); h.version = u32(4);
    h.jsonChunkOffset = u64(8); h.jsonChunkSize = u64(16); h.binaryChunkOffset = u64(24); h.binaryChunkSize = u64(32);
    return h;
}

} // namespace ntc::file
