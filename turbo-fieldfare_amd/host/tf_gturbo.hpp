// Reader of the `.gturbo` packed-experts layout (packed_experts/layout.json) and the glue that puts a layer file
// (packed_experts/layer_XX.bin: expertsPerLayer blobs of expertStride bytes) into an HBM-resident pool.
//
// Mirrors, over the C ABI: GTurboPackedExpertsLayoutCodec.decode + GTurboV1StructuralValidator.validate
// (Sources/TurboFieldfareFormat/GTurboPackedExpertsLayoutV1.swift:65-180), PackedExpertsLayoutReader.decode
// (Infrastructure/ModelIO/PackedExpertsLayout.swift:78-120) and Model.routedExpertOffsets
// (Runtime/Inference/ModelExpertIO.swift:20-43).  Where the reference streams experts from SSD into a slot cache, all
// experts of a layer are uploaded once, in LOGICAL order, so kernels address expert e at pool + e * expertStride.
//
// Also here: the resident index of model_weights.bin (everything that is not a routed expert: embedding / lm_head table,
// attention projections, router, shared expert, norms).  Mirrors GTurboResidentIndexCodec.decodeHeader / decodeRegion
// (Sources/TurboFieldfareFormat/GTurboResidentIndexV1.swift:42-171), ResidentIndexReader.load
// (Infrastructure/ModelIO/ResidentIndex.swift:44-141) and Model.resident(name:) with its named accessors
// (Runtime/Inference/Model.swift:88-233).  Where the reference maps the payload into one shared MTLBuffer
// (ResidentBuffer.swift:15-78), uploadResident() copies it into one device allocation; a TensorView's offsets are
// relative to that allocation.
#pragma once

#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include <stdint.h>

#include <algorithm>
#include <fstream>
#include <map>
#include <memory>
#include <set>
#include <sstream>
#include <string>
#include <vector>

#include "tf_host.hpp"

namespace tf {
namespace gturbo {

struct FormatError : std::runtime_error {
    std::string field;
    FormatError(const std::string &f, const std::string &reason) : std::runtime_error(f + ": " + reason), field(f) {}
};

// ---- a JSON value tree, just enough for layout.json (objects, arrays, strings, non-negative integers, null, booleans)
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    bool boolean = false;
    uint64_t number = 0;
    bool integral = true;      // false for negative, fractional or exponent forms (never valid in a layout)
    std::string string;
    std::vector<Json> array;
    std::map<std::string, Json> object;

    const Json *find(const std::string &key) const {
        if (kind != Object) return nullptr;
        const auto it = object.find(key);
        return it == object.end() ? nullptr : &it->second;
    }
};

class JsonParser {
public:
    explicit JsonParser(const std::string &text) : s_(text) {}
    Json parse() {
        Json v = value(0);
        skip();
        if (p_ != s_.size()) fail("trailing characters");
        return v;
    }

private:
    const std::string &s_;
    size_t p_ = 0;
    [[noreturn]] void fail(const std::string &why) const {
        throw FormatError("packed_experts/layout.json", "invalid JSON at byte " + std::to_string(p_) + ": " + why);
    }
    void skip() {
        while (p_ < s_.size() && (s_[p_] == ' ' || s_[p_] == '\n' || s_[p_] == '\t' || s_[p_] == '\r')) ++p_;
    }
    bool eat(const char *word) {
        const size_t n = std::char_traits<char>::length(word);
        if (s_.compare(p_, n, word) != 0) return false;
        p_ += n;
        return true;
    }
    std::string string_body() {
        std::string out;
        ++p_;   // opening quote
        while (true) {
            if (p_ >= s_.size()) fail("unterminated string");
            const char c = s_[p_++];
            if (c == '"') return out;
            if (c != '\\') {
                out.push_back(c);
                continue;
            }
            if (p_ >= s_.size()) fail("unterminated escape");
            const char e = s_[p_++];
            switch (e) {
                case '"': out.push_back('"'); break;
                case '\\': out.push_back('\\'); break;
                case '/': out.push_back('/'); break;
                case 'n': out.push_back('\n'); break;
                case 't': out.push_back('\t'); break;
                case 'r': out.push_back('\r'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'u': {
                    if (p_ + 4 > s_.size()) fail("short \\u escape");
                    unsigned code = 0;
                    for (int i = 0; i < 4; ++i) {
                        const char h = s_[p_++];
                        code <<= 4;
                        if (h >= '0' && h <= '9') code |= (unsigned)(h - '0');
                        else if (h >= 'a' && h <= 'f') code |= (unsigned)(h - 'a' + 10);
                        else if (h >= 'A' && h <= 'F') code |= (unsigned)(h - 'A' + 10);
                        else fail("bad \\u escape");
                    }
                    // names in a layout are ASCII; anything else is kept as UTF-8 of the BMP code point
                    if (code < 0x80) out.push_back((char)code);
                    else if (code < 0x800) {
                        out.push_back((char)(0xC0 | (code >> 6)));
                        out.push_back((char)(0x80 | (code & 0x3F)));
                    } else {
                        out.push_back((char)(0xE0 | (code >> 12)));
                        out.push_back((char)(0x80 | ((code >> 6) & 0x3F)));
                        out.push_back((char)(0x80 | (code & 0x3F)));
                    }
                    break;
                }
                default: fail("unknown escape");
            }
        }
    }
    Json value(int depth) {
        if (depth > 16) fail("nesting too deep");
        skip();
        if (p_ >= s_.size()) fail("unexpected end");
        Json v;
        const char c = s_[p_];
        if (c == '{') {
            v.kind = Json::Object;
            ++p_;
            skip();
            if (p_ < s_.size() && s_[p_] == '}') { ++p_; return v; }
            while (true) {
                skip();
                if (p_ >= s_.size() || s_[p_] != '"') fail("expected a key");
                const std::string key = string_body();
                skip();
                if (p_ >= s_.size() || s_[p_] != ':') fail("expected ':'");
                ++p_;
                if (!v.object.emplace(key, value(depth + 1)).second) fail("duplicate key " + key);
                skip();
                if (p_ < s_.size() && s_[p_] == ',') { ++p_; continue; }
                if (p_ < s_.size() && s_[p_] == '}') { ++p_; return v; }
                fail("expected ',' or '}'");
            }
        }
        if (c == '[') {
            v.kind = Json::Array;
            ++p_;
            skip();
            if (p_ < s_.size() && s_[p_] == ']') { ++p_; return v; }
            while (true) {
                v.array.push_back(value(depth + 1));
                skip();
                if (p_ < s_.size() && s_[p_] == ',') { ++p_; continue; }
                if (p_ < s_.size() && s_[p_] == ']') { ++p_; return v; }
                fail("expected ',' or ']'");
            }
        }
        if (c == '"') {
            v.kind = Json::String;
            v.string = string_body();
            return v;
        }
        if (eat("null")) return v;
        if (eat("true")) { v.kind = Json::Bool; v.boolean = true; return v; }
        if (eat("false")) { v.kind = Json::Bool; return v; }
        if (c == '-' || (c >= '0' && c <= '9')) {
            v.kind = Json::Number;
            if (c == '-') { v.integral = false; ++p_; }
            bool digits = false;
            while (p_ < s_.size() && s_[p_] >= '0' && s_[p_] <= '9') {
                const uint64_t d = (uint64_t)(s_[p_] - '0');
                if (v.number > (UINT64_MAX - d) / 10) fail("integer overflow");
                v.number = v.number * 10 + d;
                digits = true;
                ++p_;
            }
            if (!digits) fail("bad number");
            if (p_ < s_.size() && (s_[p_] == '.' || s_[p_] == 'e' || s_[p_] == 'E')) {
                v.integral = false;
                while (p_ < s_.size() && (s_[p_] == '.' || s_[p_] == 'e' || s_[p_] == 'E' || s_[p_] == '+' || s_[p_] == '-' ||
                                          (s_[p_] >= '0' && s_[p_] <= '9')))
                    ++p_;
            }
            return v;
        }
        fail("unexpected character");
    }
};

// ---- the layout (PackedExpertsLayout.swift:4-52)
struct SubTensorEntry {
    uint64_t offset = 0, size = 0;   // offset relative to the expert blob
    std::string dtype;               // "U32" | "BF16"
    std::vector<uint32_t> shape;
    int bits = 0;                    // 0: absent
    bool operator==(const SubTensorEntry &o) const {
        return offset == o.offset && size == o.size && dtype == o.dtype && shape == o.shape && bits == o.bits;
    }
};

struct ExpertEntry {
    int expert = 0, physicalRank = 0;
    uint64_t offset = 0, size = 0;   // offset inside the layer file
    std::map<std::string, SubTensorEntry> subTensors;
};

struct LayerLayout {
    int layer = 0;
    std::string file;                 // basename, e.g. "layer_00.bin"
    std::vector<ExpertEntry> experts; // sorted by logical expert id
};

struct PackedExpertsLayout {
    static constexpr uint64_t alignmentBytes = 16384;   // GTurboFormatV1.alignmentBytes
    uint64_t expertStride = 0;
    int numLayers = 0, expertsPerLayer = 0;
    std::vector<LayerLayout> layers;                     // sorted by layer

    const ExpertEntry &expert(int layer, int e) const { return layers.at((size_t)layer).experts.at((size_t)e); }

    // Model.routedExpertOffsets(layer:) plus the runtime schema rule that all experts of a layer share one metadata
    // record per role (Model.swift:676-722).
    MoEExpertOffsets routedExpertOffsets(int layer) const {
        const LayerLayout &l = layers.at((size_t)layer);
        const ExpertEntry &first = l.experts.at(0);
        static const char *roles[9] = {"gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales", "down_biases"};
        uint32_t off[9];
        for (int i = 0; i < 9; ++i) {
            const auto it = first.subTensors.find(roles[i]);
            if (it == first.subTensors.end()) throw FormatError(std::string("routed layer ") + std::to_string(layer), std::string("missing role ") + roles[i]);
            if (it->second.offset > UINT32_MAX) throw FormatError(roles[i], "offset does not fit 32 bits");
            for (const ExpertEntry &e : l.experts) {
                const auto other = e.subTensors.find(roles[i]);
                if (other == e.subTensors.end() || !(other->second == it->second))
                    throw FormatError(std::string("routed layer ") + std::to_string(layer), std::string("role ") + roles[i] + " metadata differs across experts");
            }
            off[i] = (uint32_t)it->second.offset;
        }
        return MoEExpertOffsets{off[0], off[1], off[2], off[3], off[4], off[5], off[6], off[7], off[8]};
    }

    // logical expert id -> position of its blob in the layer file
    std::vector<uint32_t> physicalRanks(int layer) const {
        std::vector<uint32_t> out;
        for (const ExpertEntry &e : layers.at((size_t)layer).experts) out.push_back((uint32_t)e.physicalRank);
        return out;
    }
};

namespace detail {

inline uint64_t need_uint(const Json &obj, const char *key, const std::string &where) {
    const Json *v = obj.find(key);
    if (!v || v->kind != Json::Number || !v->integral) throw FormatError(where + "." + key, "missing or not a non-negative integer");
    return v->number;
}

inline bool basename_ok(const std::string &name) {
    if (name.empty() || name == "." || name == ".." || name.size() > 255) return false;
    for (const char c : name)
        if (c == '/' || c == '\\' || c == '\0' || (unsigned char)c < 0x20) return false;
    return true;
}

inline std::string lower(std::string s) {
    std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return (char)std::tolower(c); });
    return s;
}

}  // namespace detail

// GTurboPackedExpertsLayoutCodec.decode + GTurboV1StructuralValidator.validate + PackedExpertsLayoutReader.decode.
inline PackedExpertsLayout decodeLayout(const std::string &json_text) {
    const Json root = JsonParser(json_text).parse();
    if (root.kind != Json::Object) throw FormatError("layout", "not an object");
    PackedExpertsLayout out;
    out.expertStride = detail::need_uint(root, "expertStride", "layout");
    const uint64_t nl = detail::need_uint(root, "numLayers", "layout"), ne = detail::need_uint(root, "expertsPerLayer", "layout");
    const Json *layers = root.find("layers");
    if (!layers || layers->kind != Json::Array) throw FormatError("layout.layers", "missing");
    if (nl == 0 || ne == 0 || nl > 1u << 20 || ne > 1u << 20 || out.expertStride == 0 || out.expertStride % PackedExpertsLayout::alignmentBytes != 0 ||
        layers->array.size() != nl)
        throw FormatError("layout", "invalid dimensions or stride");
    out.numLayers = (int)nl;
    out.expertsPerLayer = (int)ne;
    std::set<int> layer_ids;
    std::set<std::string> layer_files;
    for (const Json &jl : layers->array) {
        LayerLayout l;
        const uint64_t id = detail::need_uint(jl, "layer", "layout.layers");
        if (id >= nl || !layer_ids.insert((int)id).second) throw FormatError("layout.layers", "duplicate or invalid layer");
        l.layer = (int)id;
        const std::string where = "layout.layers[" + std::to_string(id) + "]";
        const Json *file = jl.find("file");
        if (!file || file->kind != Json::String || !detail::basename_ok(file->string)) throw FormatError(where + ".file", "not a plain file name");
        l.file = file->string;
        const std::string key = detail::lower(l.file);   // the reference compares names as a case-insensitive filesystem would
        if (key == "layout.json") throw FormatError(where + ".file", "reserved packed-expert filename");
        if (!layer_files.insert(key).second) throw FormatError(where + ".file", "duplicate layer filename");
        const Json *experts = jl.find("experts");
        if (!experts || experts->kind != Json::Array || experts->array.size() != ne) throw FormatError(where + ".experts", "wrong expert count");
        size_t explicit_ids = 0;
        for (const Json &je : experts->array) {
            const Json *e = je.find("expert");
            if (e && e->kind != Json::Null) ++explicit_ids;
        }
        if (explicit_ids != 0 && explicit_ids != ne) throw FormatError(where + ".experts", "expert ids must be either all explicit or all positional");
        std::set<int> logical_ids, physical_ranks;
        std::set<uint64_t> offsets;
        for (size_t position = 0; position < experts->array.size(); ++position) {
            const Json &je = experts->array[position];
            ExpertEntry e;
            const Json *jid = je.find("expert"), *jrank = je.find("physicalRank");
            const uint64_t logical = (jid && jid->kind != Json::Null) ? detail::need_uint(je, "expert", where) : position;
            const uint64_t physical = (jrank && jrank->kind != Json::Null) ? detail::need_uint(je, "physicalRank", where) : logical;
            e.offset = detail::need_uint(je, "offset", where + ".experts");
            e.size = detail::need_uint(je, "size", where + ".experts");
            if (logical >= ne || physical >= ne || !logical_ids.insert((int)logical).second || !physical_ranks.insert((int)physical).second ||
                !offsets.insert(e.offset).second)
                throw FormatError(where + ".experts", "duplicate or invalid expert mapping");
            e.expert = (int)logical;
            e.physicalRank = (int)physical;
            if (physical != 0 && out.expertStride > UINT64_MAX / physical) throw FormatError("expert.offset", "overflow");
            if (e.offset != physical * out.expertStride || e.size != out.expertStride)
                throw FormatError("expert[" + std::to_string(logical) + "]", "offset or size does not match physical rank");
            const Json *tensors = je.find("tensors");
            if (!tensors || tensors->kind != Json::Object) throw FormatError("expert[" + std::to_string(logical) + "].tensors", "missing");
            std::vector<std::pair<uint64_t, uint64_t>> ranges;
            for (const auto &kv : tensors->object) {
                const std::string tw = "expert[" + std::to_string(logical) + "].tensors." + kv.first;
                SubTensorEntry t;
                t.offset = detail::need_uint(kv.second, "offset", tw);
                t.size = detail::need_uint(kv.second, "size", tw);
                const Json *dtype = kv.second.find("dtype"), *shape = kv.second.find("shape"), *bits = kv.second.find("bits");
                if (!dtype || dtype->kind != Json::String || !shape || shape->kind != Json::Array) throw FormatError(tw, "invalid dtype or shape");
                t.dtype = dtype->string;
                bool ok = (t.dtype == "U32" || t.dtype == "BF16") && !kv.first.empty() && t.size > 0 && !shape->array.empty();
                for (const Json &dim : shape->array) {
                    ok = ok && dim.kind == Json::Number && dim.integral && dim.number > 0 && dim.number <= UINT32_MAX;
                    t.shape.push_back((uint32_t)dim.number);
                }
                if (bits && bits->kind != Json::Null) {
                    ok = ok && bits->kind == Json::Number && bits->integral && bits->number > 0 && bits->number <= 32;
                    t.bits = (int)bits->number;
                }
                if (!ok) throw FormatError(tw, "invalid dtype or shape");
                if (t.offset > UINT64_MAX - t.size) throw FormatError(tw + ".range", "overflow");
                if (t.offset + t.size > e.size) throw FormatError(tw, "range exceeds expert blob");
                ranges.emplace_back(t.offset, t.offset + t.size);
                e.subTensors.emplace(kv.first, std::move(t));
            }
            std::sort(ranges.begin(), ranges.end());
            for (size_t i = 1; i < ranges.size(); ++i)
                if (ranges[i - 1].second > ranges[i].first) throw FormatError("expert[" + std::to_string(logical) + "].tensors", "overlapping ranges");
            l.experts.push_back(std::move(e));
        }
        std::sort(l.experts.begin(), l.experts.end(), [](const ExpertEntry &a, const ExpertEntry &b) { return a.expert < b.expert; });
        out.layers.push_back(std::move(l));
    }
    std::sort(out.layers.begin(), out.layers.end(), [](const LayerLayout &a, const LayerLayout &b) { return a.layer < b.layer; });
    return out;
}

// PackedExpertsLayoutReader.load(directoryURL:): reads <directory>/packed_experts/layout.json (at most maxBytes).
inline PackedExpertsLayout loadLayout(const std::string &directory, uint64_t maxBytes = 16u * 1024 * 1024) {
    const std::string path = directory + "/packed_experts/layout.json";
    std::ifstream in(path, std::ios::binary);
    if (!in) throw FormatError("packed_experts/layout.json", "cannot open " + path);
    std::ostringstream text;
    text << in.rdbuf();
    if (text.str().size() > maxBytes) throw FormatError("packed_experts/layout.json", "larger than the metadata limit");
    return decodeLayout(text.str());
}

// A layer's experts resident in HBM in logical order: fills `device_pool` (expertsPerLayer * expertStride bytes, owned by
// the caller) from <directory>/packed_experts/<layer file>.  Enqueues on the context's stream and returns when the host
// side of the upload is done; synchronise the stream before the first use.
inline void uploadLayer(const Context &c, const PackedExpertsLayout &layout, const std::string &directory, int layer, void *device_pool) {
    const LayerLayout &l = layout.layers.at((size_t)layer);
    const std::vector<uint32_t> ranks = layout.physicalRanks(layer);
    const std::string path = directory + "/packed_experts/" + l.file;
    c.check(tf_upload_packed_experts_layer(c.raw(), c.stream(), path.c_str(), layout.expertStride, (uint32_t)layout.expertsPerLayer, ranks.data(),
                                           device_pool));
}

// ------------------------------------------------------------------------------------------------ resident index
constexpr uint64_t kAlignmentBytes = 16384;               // GTurboFormatV1.alignmentBytes
constexpr size_t kResidentHeaderBytes = 24;               // GTurboFormatV1.residentHeaderBytes
constexpr size_t kResidentEntryBytes = 72;                // GTurboFormatV1.residentEntryBytes
constexpr uint64_t kResidentIndexMaxBytes = 16ull * 1024 * 1024;   // GTurboFormatV1.residentIndexMaxBytes
enum class DType : uint8_t { u32 = 0, bf16 = 1, fp16 = 2, fp32 = 3 };   // GTurboFormatV1.DType

// What the model loader throws (ModelError.indexCorrupt / tensorNotFound / posixFailed)
struct ModelError : std::runtime_error {
    enum Kind { IndexCorrupt, TensorNotFound, PosixFailed } kind;
    ModelError(Kind k, const std::string &detail) : std::runtime_error(detail), kind(k) {}
};

struct ResidentIndexHeader {
    uint64_t indexSize = 0;      // bytes of the leading index region (header, entry table, string table, padding)
    uint64_t residentSize = 0;   // bytes of the tensor payload that follows it
    uint64_t entryCount = 0;
};

struct ResidentIndexEntry {
    std::string name;
    uint8_t dtype = 0;
    uint64_t fileOffset = 0, sizeBytes = 0;          // absolute file offset of the packed weights
    uint32_t shape[4] = {0, 0, 0, 0};
    uint64_t scaleOffset = 0, scaleSize = 0, biasOffset = 0, biasSize = 0;   // absent: offset 0, size 0
};

// ModelTypes.swift:164-196 without the buffer: offsets are relative to the start of the resident payload
struct TensorView {
    uint64_t offset = 0, length = 0, scaleOffset = 0, scaleLength = 0, biasOffset = 0, biasLength = 0;
    uint32_t shape[4] = {0, 0, 0, 0};
    uint8_t dtype = 0;
    // The view as an operand of the shared-expert / GEMV entry points, against the device copy of the payload.  For a
    // 4-bit tensor stored as U32 words, shape = [rows, cols / 8]; `cols` is passed by the caller who knows the bit width.
    SharedExpertProjection projection(const void *device_payload, uint32_t rows, uint32_t cols) const {
        return SharedExpertProjection{device_payload, offset, device_payload, scaleOffset, device_payload, biasOffset, rows, cols};
    }
};

namespace detail {
inline uint64_t le(const uint8_t *p, size_t off, int bytes) {
    uint64_t v = 0;
    for (int i = bytes - 1; i >= 0; --i) v = v << 8 | p[off + (size_t)i];
    return v;
}
// well-formed UTF-8 (no overlong forms, no surrogates, nothing above U+10FFFF), as String(bytes:encoding:.utf8) accepts
inline bool valid_utf8(const uint8_t *p, size_t n) {
    size_t i = 0;
    while (i < n) {
        const uint8_t c = p[i];
        size_t need;
        uint32_t cp, min;
        if (c < 0x80) { ++i; continue; }
        else if ((c & 0xE0) == 0xC0) { need = 1; cp = c & 0x1Fu; min = 0x80; }
        else if ((c & 0xF0) == 0xE0) { need = 2; cp = c & 0x0Fu; min = 0x800; }
        else if ((c & 0xF8) == 0xF0) { need = 3; cp = c & 0x07u; min = 0x10000; }
        else return false;
        if (i + need >= n) return false;   // the continuation bytes must exist
        for (size_t k = 1; k <= need; ++k) {
            if ((p[i + k] & 0xC0) != 0x80) return false;
            cp = cp << 6 | (p[i + k] & 0x3Fu);
        }
        if (cp < min || cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF)) return false;
        i += need + 1;
    }
    return true;
}
inline uint64_t checked_add(uint64_t a, uint64_t b, const std::string &field) {
    if (a > UINT64_MAX - b) throw FormatError(field, "overflow");
    return a + b;
}
}  // namespace detail

// GTurboResidentIndexCodec.decodeHeader: three little-endian u64
inline ResidentIndexHeader decodeResidentHeader(const uint8_t *bytes, size_t count) {
    if (count < kResidentHeaderBytes) throw FormatError("resident.header", "truncated");
    ResidentIndexHeader h;
    h.indexSize = detail::le(bytes, 0, 8);
    h.residentSize = detail::le(bytes, 8, 8);
    h.entryCount = detail::le(bytes, 16, 8);
    return h;
}

// GTurboResidentIndexCodec.decodeRegion: `bytes` holds the whole index region.  Entries come back in table order.
inline std::vector<ResidentIndexEntry> decodeResidentRegion(const uint8_t *bytes, size_t count, const ResidentIndexHeader &header) {
    if (header.indexSize > kResidentIndexMaxBytes) throw FormatError("resident.indexSize", "exceeds v1 metadata cap");
    if (header.indexSize > count || header.indexSize < kResidentHeaderBytes || header.indexSize % kAlignmentBytes != 0)
        throw FormatError("resident.index", "truncated");
    if (header.entryCount > UINT64_MAX / kResidentEntryBytes) throw FormatError("resident.entryTable", "overflow");
    const uint64_t tableEnd = detail::checked_add(kResidentHeaderBytes, header.entryCount * kResidentEntryBytes, "resident.entryTable");
    if (tableEnd > header.indexSize) throw FormatError("resident.entryTable", "outside index");
    const uint64_t residentEnd = detail::checked_add(header.indexSize, header.residentSize, "resident.payload");
    std::vector<ResidentIndexEntry> result;
    result.reserve((size_t)header.entryCount);
    std::set<std::string> names;
    struct Range {
        uint64_t start, end;
        std::string field;
    };
    std::vector<Range> ranges;
    auto contained = [&](uint64_t offset, uint64_t size, const std::string &field) {
        const uint64_t end = detail::checked_add(offset, size, field);
        if (offset < header.indexSize || end > residentEnd) throw FormatError(field, "range outside resident payload");
    };
    auto optional = [&](uint64_t offset, uint64_t size, const std::string &field) {
        if (size == 0) {
            if (offset != 0) throw FormatError(field, "absent payload offset must be zero");
            return;
        }
        contained(offset, size, field);
    };
    for (uint64_t index = 0; index < header.entryCount; ++index) {
        const std::string where = "resident.entries[" + std::to_string(index) + "]";
        const uint8_t *entry = bytes + kResidentHeaderBytes + (size_t)index * kResidentEntryBytes;
        const uint64_t nameOffset = detail::le(entry, 0, 4), nameLength = detail::le(entry, 4, 2);
        if (entry[7] != 0) throw FormatError(where + ".reserved", "must be zero");
        const uint64_t nameEnd = nameOffset + nameLength;
        if (nameOffset < tableEnd || nameEnd > header.indexSize) throw FormatError(where + ".name", "range outside string table");
        ResidentIndexEntry e;
        e.name.assign(reinterpret_cast<const char *>(bytes + nameOffset), (size_t)nameLength);
        if (e.name.empty() || !detail::valid_utf8(bytes + nameOffset, (size_t)nameLength) || !names.insert(e.name).second)
            throw FormatError(where + ".name", "invalid UTF-8 or duplicate");
        e.dtype = entry[6];
        if (e.dtype > (uint8_t)DType::fp32) throw FormatError(where + ".dtype", "unknown dtype");
        e.fileOffset = detail::le(entry, 8, 8);
        e.sizeBytes = detail::le(entry, 16, 8);
        for (int i = 0; i < 4; ++i) e.shape[i] = (uint32_t)detail::le(entry, 24 + 4 * (size_t)i, 4);
        e.scaleOffset = detail::le(entry, 40, 8);
        e.scaleSize = detail::le(entry, 48, 8);
        e.biasOffset = detail::le(entry, 56, 8);
        e.biasSize = detail::le(entry, 64, 8);
        if (e.shape[0] == 0) throw FormatError(where + ".shape", "first dimension must be positive");
        bool sawZero = false;
        for (int i = 0; i < 4; ++i) {
            if (e.shape[i] == 0) sawZero = true;
            else if (sawZero) throw FormatError(where + ".shape", "zero dimensions must be trailing");
        }
        if (e.sizeBytes == 0) throw FormatError(where + ".weights", "primary payload is empty");
        contained(e.fileOffset, e.sizeBytes, where + ".weights");
        optional(e.scaleOffset, e.scaleSize, where + ".scales");
        optional(e.biasOffset, e.biasSize, where + ".biases");
        ranges.push_back({e.fileOffset, e.fileOffset + e.sizeBytes, where + ".weights"});
        if (e.scaleSize > 0) ranges.push_back({e.scaleOffset, e.scaleOffset + e.scaleSize, where + ".scales"});
        if (e.biasSize > 0) ranges.push_back({e.biasOffset, e.biasOffset + e.biasSize, where + ".biases"});
        result.push_back(std::move(e));
    }
    std::sort(ranges.begin(), ranges.end(), [](const Range &a, const Range &b) { return a.start == b.start ? a.end < b.end : a.start < b.start; });
    for (size_t i = 1; i < ranges.size(); ++i)
        if (ranges[i].start < ranges[i - 1].end) throw FormatError(ranges[i].field, "overlaps " + ranges[i - 1].field);
    return result;
}

// Parsed resident index: header + name-keyed entries, with Model's accessors (Model.swift:88-233).
struct ResidentIndex {
    ResidentIndexHeader header;
    std::map<std::string, ResidentIndexEntry> entries;

    // Model.resident(name:): absolute file offsets -> offsets inside the resident payload
    TensorView resident(const std::string &name) const {
        const auto it = entries.find(name);
        if (it == entries.end()) throw ModelError(ModelError::TensorNotFound, "tensor not found: " + name);
        const ResidentIndexEntry &e = it->second;
        auto relative = [&](uint64_t absolute, uint64_t size, const char *field) -> uint64_t {
            if (size == 0) {
                if (absolute != 0) throw ModelError(ModelError::IndexCorrupt, name + "." + field + " has an absent nonzero offset");
                return 0;
            }
            if (absolute < header.indexSize) throw ModelError(ModelError::IndexCorrupt, name + "." + field + " precedes the resident payload");
            const uint64_t rel = absolute - header.indexSize;
            if (rel > header.residentSize || size > header.residentSize - rel)
                throw ModelError(ModelError::IndexCorrupt, name + "." + field + " exceeds the resident payload");
            return rel;
        };
        TensorView v;
        v.offset = relative(e.fileOffset, e.sizeBytes, "weights");
        v.length = e.sizeBytes;
        v.scaleOffset = relative(e.scaleOffset, e.scaleSize, "scales");
        v.scaleLength = e.scaleSize;
        v.biasOffset = relative(e.biasOffset, e.biasSize, "biases");
        v.biasLength = e.biasSize;
        for (int i = 0; i < 4; ++i) v.shape[i] = e.shape[i];
        v.dtype = e.dtype;
        return v;
    }
    static std::string layerName(int layer, const char *suffix) { return "language_model.model.layers." + std::to_string(layer) + "." + suffix; }
    TensorView embedding() const { return resident("language_model.model.embed_tokens.weight"); }
    TensorView lmHead() const { return embedding(); }   // tied
    TensorView finalNorm() const { return resident("language_model.model.norm.weight"); }
    TensorView qProj(int L) const { return resident(layerName(L, "self_attn.q_proj.weight")); }
    TensorView kProj(int L) const { return resident(layerName(L, "self_attn.k_proj.weight")); }
    TensorView vProj(int L) const { return resident(layerName(L, "self_attn.v_proj.weight")); }
    TensorView oProj(int L) const { return resident(layerName(L, "self_attn.o_proj.weight")); }
    TensorView router(int L) const { return resident(layerName(L, "router.proj.weight")); }
    TensorView routerScale(int L) const { return resident(layerName(L, "router.scale")); }
    TensorView routerPerExpertScale(int L) const { return resident(layerName(L, "router.per_expert_scale")); }
    TensorView sharedExpertGate(int L) const { return resident(layerName(L, "mlp.gate_proj.weight")); }
    TensorView sharedExpertUp(int L) const { return resident(layerName(L, "mlp.up_proj.weight")); }
    TensorView sharedExpertDown(int L) const { return resident(layerName(L, "mlp.down_proj.weight")); }
    TensorView inputNorm(int L) const { return resident(layerName(L, "input_layernorm.weight")); }
    TensorView postAttnNorm(int L) const { return resident(layerName(L, "post_attention_layernorm.weight")); }
    TensorView qNorm(int L) const { return resident(layerName(L, "self_attn.q_norm.weight")); }
    TensorView kNorm(int L) const { return resident(layerName(L, "self_attn.k_norm.weight")); }
    TensorView preFFN(int L) const { return resident(layerName(L, "pre_feedforward_layernorm.weight")); }
    TensorView preFFN2(int L) const { return resident(layerName(L, "pre_feedforward_layernorm_2.weight")); }
    TensorView postFFN1(int L) const { return resident(layerName(L, "post_feedforward_layernorm_1.weight")); }
    TensorView postFFN2(int L) const { return resident(layerName(L, "post_feedforward_layernorm_2.weight")); }
    TensorView postFFN(int L) const { return resident(layerName(L, "post_feedforward_layernorm.weight")); }
    TensorView layerScalar(int L) const { return resident(layerName(L, "layer_scalar")); }
};

// ResidentIndexReader.load(fileURL:maxBytes:): header + index region of model_weights.bin; the payload is not read.
inline ResidentIndex loadResidentIndex(const std::string &path, uint64_t maxBytes = kResidentIndexMaxBytes) {
    struct Fd {
        int fd;
        ~Fd() {
            if (fd >= 0) close(fd);
        }
    } file{open(path.c_str(), O_RDONLY | O_NONBLOCK | O_CLOEXEC)};
    if (file.fd < 0) throw ModelError(ModelError::PosixFailed, "open(" + path + "): " + strerror(errno));
    struct stat st;
    if (fstat(file.fd, &st) != 0) throw ModelError(ModelError::PosixFailed, "fstat(" + path + "): " + strerror(errno));
    if (!S_ISREG(st.st_mode)) throw ModelError(ModelError::IndexCorrupt, "resident index is not a regular file");
    auto readExactly = [&](uint8_t *dst, size_t n, uint64_t offset, const char *field) {
        size_t total = 0;
        while (total < n) {
            const ssize_t got = pread(file.fd, dst + total, n - total, (off_t)(offset + total));
            if (got < 0 && errno == EINTR) continue;
            if (got <= 0) throw ModelError(ModelError::IndexCorrupt, std::string("short read for ") + field + " (" + std::to_string(total) + "/" + std::to_string(n) + ")");
            total += (size_t)got;
        }
    };
    uint8_t headerBytes[kResidentHeaderBytes];
    readExactly(headerBytes, kResidentHeaderBytes, 0, "IndexHeader");
    ResidentIndex out;
    out.header = decodeResidentHeader(headerBytes, kResidentHeaderBytes);
    if (out.header.indexSize > maxBytes)
        throw ModelError(ModelError::IndexCorrupt, "indexSize " + std::to_string(out.header.indexSize) + " exceeds metadata cap " + std::to_string(maxBytes));
    if (out.header.indexSize < kResidentHeaderBytes) throw ModelError(ModelError::IndexCorrupt, "indexSize is smaller than the header");
    if (out.header.indexSize > (uint64_t)st.st_size) throw ModelError(ModelError::IndexCorrupt, "index region exceeds file size");
    std::vector<uint8_t> region((size_t)out.header.indexSize);
    memcpy(region.data(), headerBytes, kResidentHeaderBytes);
    readExactly(region.data() + kResidentHeaderBytes, region.size() - kResidentHeaderBytes, kResidentHeaderBytes, "index region");
    std::vector<ResidentIndexEntry> list;
    try {
        list = decodeResidentRegion(region.data(), region.size(), out.header);
    } catch (const FormatError &e) {
        throw ModelError(ModelError::IndexCorrupt, e.what());
    }
    for (ResidentIndexEntry &e : list) {
        const std::string name = e.name;
        out.entries.emplace(name, std::move(e));
    }
    return out;
}

// The resident payload of model_weights.bin ([indexSize, indexSize + residentSize) of the file) into `device_payload`
// (residentSize bytes, owned by the caller).  Returns when the copy is complete.
inline void uploadResident(const Context &c, const ResidentIndex &index, const std::string &path, void *device_payload) {
    c.check(tf_upload_file_region(c.raw(), c.stream(), path.c_str(), index.header.indexSize, index.header.residentSize, device_payload));
}

}  // namespace gturbo
}  // namespace tf
