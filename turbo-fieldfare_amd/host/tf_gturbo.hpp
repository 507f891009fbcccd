// Reader of the `.gturbo` packed-experts layout (packed_experts/layout.json) and the glue that puts a layer file
// (packed_experts/layer_XX.bin: expertsPerLayer blobs of expertStride bytes) into an HBM-resident pool.
//
// Mirrors, over the C ABI: GTurboPackedExpertsLayoutCodec.decode + GTurboV1StructuralValidator.validate
// (Sources/TurboFieldfareFormat/GTurboPackedExpertsLayoutV1.swift:65-180), PackedExpertsLayoutReader.decode
// (Infrastructure/ModelIO/PackedExpertsLayout.swift:78-120) and Model.routedExpertOffsets
// (Runtime/Inference/ModelExpertIO.swift:20-43).  Where the reference streams experts from SSD into a slot cache, all
// experts of a layer are uploaded once, in LOGICAL order, so kernels address expert e at pool + e * expertStride.
#pragma once

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

}  // namespace gturbo
}  // namespace tf
