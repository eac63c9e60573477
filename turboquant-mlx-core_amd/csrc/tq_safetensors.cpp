// safetensors reader / writer and the TQ8 file layout (include/turboquant/serialization.h).
// File format: u64 little-endian header length N, N bytes of JSON
//   { "<name>": {"dtype": "F32", "shape": [..], "data_offsets": [begin, end]}, ...,
//     "__metadata__": {"key": "value", ...} }
// followed by the tensor bytes; offsets are relative to the first byte after the header.
#include "turboquant/serialization.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <fstream>
#include <map>
#include <sstream>
#include <stdexcept>

namespace turboquant {

namespace {

// ---- a small JSON reader: enough for a safetensors header -------------------
struct Json {
    enum Kind { Null, Bool, Number, String, ArrayK, Object } kind = Null;
    bool b = false;
    double num = 0.0;
    std::string str;
    std::vector<Json> items;                              // ArrayK
    std::vector<std::pair<std::string, Json>> members;    // Object, file order

    const Json* find(const std::string& key) const {
        for (const auto& m : members)
            if (m.first == key) return &m.second;
        return nullptr;
    }
};

class JsonReader {
public:
    JsonReader(const char* p, size_t n) : p_(p), end_(p + n) {}

    Json parse_document() {
        Json v = value(0);
        skip_ws();
        if (p_ != end_) bad("trailing characters");
        return v;
    }

private:
    const char* p_;
    const char* end_;

    [[noreturn]] void bad(const char* what) { throw std::runtime_error(std::string("safetensors header: ") + what); }
    void skip_ws() { while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) ++p_; }
    bool eat(char c) { skip_ws(); if (p_ < end_ && *p_ == c) { ++p_; return true; } return false; }
    void expect(char c) { if (!eat(c)) bad("unexpected character"); }

    static void append_utf8(std::string& s, uint32_t cp) {
        if (cp < 0x80) s += (char)cp;
        else if (cp < 0x800) { s += (char)(0xC0 | (cp >> 6)); s += (char)(0x80 | (cp & 0x3F)); }
        else if (cp < 0x10000) {
            s += (char)(0xE0 | (cp >> 12)); s += (char)(0x80 | ((cp >> 6) & 0x3F)); s += (char)(0x80 | (cp & 0x3F));
        } else {
            s += (char)(0xF0 | (cp >> 18)); s += (char)(0x80 | ((cp >> 12) & 0x3F));
            s += (char)(0x80 | ((cp >> 6) & 0x3F)); s += (char)(0x80 | (cp & 0x3F));
        }
    }

    uint32_t hex4() {
        if (end_ - p_ < 4) bad("short \\u escape");
        uint32_t v = 0;
        for (int i = 0; i < 4; ++i) {
            const char c = *p_++;
            v <<= 4;
            if (c >= '0' && c <= '9') v |= (uint32_t)(c - '0');
            else if (c >= 'a' && c <= 'f') v |= (uint32_t)(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') v |= (uint32_t)(c - 'A' + 10);
            else bad("bad \\u escape");
        }
        return v;
    }

    std::string string() {
        expect('"');
        std::string s;
        while (true) {
            if (p_ >= end_) bad("unterminated string");
            const char c = *p_++;
            if (c == '"') break;
            if (c != '\\') { s += c; continue; }
            if (p_ >= end_) bad("unterminated escape");
            const char e = *p_++;
            switch (e) {
                case '"': s += '"'; break;
                case '\\': s += '\\'; break;
                case '/': s += '/'; break;
                case 'b': s += '\b'; break;
                case 'f': s += '\f'; break;
                case 'n': s += '\n'; break;
                case 'r': s += '\r'; break;
                case 't': s += '\t'; break;
                case 'u': {
                    uint32_t cp = hex4();
                    if (cp >= 0xD800 && cp < 0xDC00 && end_ - p_ >= 6 && p_[0] == '\\' && p_[1] == 'u') {
                        p_ += 2;
                        const uint32_t lo = hex4();
                        cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                    }
                    append_utf8(s, cp);
                    break;
                }
                default: bad("unknown escape");
            }
        }
        return s;
    }

    // A safetensors header nests three levels deep (entry -> shape / data_offsets); anything much deeper
    // is not a header, and unbounded recursion on "[[[[..." would overflow the stack.
    static constexpr int kMaxDepth = 8;

    Json value(int depth) {
        if (depth > kMaxDepth) bad("nested too deeply");
        skip_ws();
        if (p_ >= end_) bad("unexpected end");
        Json v;
        const char c = *p_;
        if (c == '{') {
            ++p_;
            v.kind = Json::Object;
            if (eat('}')) return v;
            do {
                skip_ws();
                std::string key = string();
                expect(':');
                v.members.emplace_back(std::move(key), value(depth + 1));
            } while (eat(','));
            expect('}');
        } else if (c == '[') {
            ++p_;
            v.kind = Json::ArrayK;
            if (eat(']')) return v;
            do { v.items.push_back(value(depth + 1)); } while (eat(','));
            expect(']');
        } else if (c == '"') {
            v.kind = Json::String;
            v.str = string();
        } else if (c == 't' && end_ - p_ >= 4 && std::string(p_, 4) == "true") {
            v.kind = Json::Bool; v.b = true; p_ += 4;
        } else if (c == 'f' && end_ - p_ >= 5 && std::string(p_, 5) == "false") {
            v.kind = Json::Bool; v.b = false; p_ += 5;
        } else if (c == 'n' && end_ - p_ >= 4 && std::string(p_, 4) == "null") {
            v.kind = Json::Null; p_ += 4;
        } else {
            const char* s = p_;
            while (p_ < end_ && (std::isdigit((unsigned char)*p_) || *p_ == '-' || *p_ == '+' || *p_ == '.' ||
                                 *p_ == 'e' || *p_ == 'E'))
                ++p_;
            if (s == p_) bad("unexpected token");
            v.kind = Json::Number;
            try { v.num = std::stod(std::string(s, p_)); }
            catch (const std::exception&) { bad("bad number"); }           // "-", "1e99999", ...
        }
        return v;
    }
};

std::string json_quote(const std::string& s) {
    std::string o = "\"";
    for (const unsigned char c : s) {
        switch (c) {
            case '"': o += "\\\""; break;
            case '\\': o += "\\\\"; break;
            case '\n': o += "\\n"; break;
            case '\r': o += "\\r"; break;
            case '\t': o += "\\t"; break;
            default:
                if (c < 0x20) { char buf[8]; std::snprintf(buf, sizeof buf, "\\u%04x", c); o += buf; }
                else o += (char)c;
        }
    }
    return o + "\"";
}

struct DtypeName { const char* name; Dtype dtype; };
const DtypeName kDtypes[] = {
    {"F32", Dtype::F32}, {"F16", Dtype::F16}, {"BF16", Dtype::BF16}, {"U8", Dtype::U8}, {"U32", Dtype::U32},
    {"F64", Dtype::F64}, {"I8", Dtype::I8}, {"I16", Dtype::I16}, {"I32", Dtype::I32}, {"I64", Dtype::I64},
    {"U16", Dtype::U16}, {"U64", Dtype::U64}, {"BOOL", Dtype::BOOL},
};

Dtype dtype_from_name(const std::string& n) {
    for (const auto& d : kDtypes)
        if (n == d.name) return d.dtype;
    throw std::runtime_error("safetensors: unsupported dtype " + n);
}

const char* dtype_name(Dtype t) {
    for (const auto& d : kDtypes)
        if (t == d.dtype) return d.name;
    return "U8";
}

// Read the header of a file; leaves `in` positioned at the first data byte.
Json read_header(std::ifstream& in, const std::string& path, uint64_t* header_len) {
    unsigned char len8[8];
    if (!in.read(reinterpret_cast<char*>(len8), 8)) throw std::runtime_error("safetensors: cannot read " + path);
    uint64_t n = 0;
    for (int i = 7; i >= 0; --i) n = (n << 8) | len8[i];
    if (n < 2 || n > 100000000ull) throw std::runtime_error("safetensors: bad header length in " + path);   // 100 MB, the format's own cap
    std::string text((size_t)n, '\0');
    if (!in.read(&text[0], (std::streamsize)n)) throw std::runtime_error("safetensors: truncated header in " + path);
    *header_len = n;
    Json root = JsonReader(text.data(), text.size()).parse_document();
    if (root.kind != Json::Object) throw std::runtime_error("safetensors: header is not an object");
    return root;
}

MetadataMap metadata_of(const Json& root) {
    MetadataMap md;
    if (const Json* m = root.find("__metadata__"))
        if (m->kind == Json::Object)
            for (const auto& kv : m->members)
                if (kv.second.kind == Json::String) md[kv.first] = kv.second.str;
    return md;
}

Codebook codebook_from_tensor(const Array& t, uint8_t bits) {
    if (t.dtype() != Dtype::F32) throw std::runtime_error("TQ8 file: codebook tensors must be float32");
    Codebook cb;
    cb.centroids.assign(t.data<float>(), t.data<float>() + t.size());
    for (size_t i = 0; i + 1 < cb.centroids.size(); ++i)
        cb.boundaries.push_back((cb.centroids[i] + cb.centroids[i + 1]) * 0.5f);
    cb.bits = bits;
    cb.origin = CodebookOrigin::Empirical;
    return cb;
}

Array centroid_tensor(const Codebook& cb) {
    return Array(cb.centroids.data(), {(int)cb.centroids.size()});
}

const Array& need(const TensorMap& tensors, const std::string& name) {
    auto it = tensors.find(name);
    if (it == tensors.end()) throw std::runtime_error("TQ8 file: missing tensor " + name);
    return it->second;
}

}  // namespace

std::pair<TensorMap, MetadataMap> load_safetensors(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) throw std::runtime_error("safetensors: cannot open " + path);
    uint64_t header_len = 0;
    const Json root = read_header(in, path, &header_len);
    in.seekg(0, std::ios::end);
    const std::streamoff file_end = in.tellg();
    if (file_end < 0 || (uint64_t)file_end < 8 + header_len) throw std::runtime_error("safetensors: truncated file " + path);
    const uint64_t data_bytes = (uint64_t)file_end - 8 - header_len;

    TensorMap tensors;
    for (const auto& kv : root.members) {
        if (kv.first == "__metadata__") continue;
        const Json& e = kv.second;
        const Json* dt = e.find("dtype");
        const Json* sh = e.find("shape");
        const Json* off = e.find("data_offsets");
        if (e.kind != Json::Object || !dt || !sh || !off || dt->kind != Json::String || sh->kind != Json::ArrayK ||
            off->kind != Json::ArrayK || off->items.size() != 2)
            throw std::runtime_error("safetensors: malformed entry " + kv.first);
        // Every number is checked before it is converted (a cast of a huge or negative double is undefined),
        // and the byte count is checked against the offsets and the file before anything is allocated.
        auto integral = [&](const Json& j, double max) {
            if (j.kind != Json::Number || !(j.num >= 0.0) || j.num > max || j.num != std::floor(j.num))
                throw std::runtime_error("safetensors: bad number in entry " + kv.first);
            return (uint64_t)j.num;
        };
        const Dtype dtype = dtype_from_name(dt->str);
        std::vector<int> shape;
        uint64_t count = 1;
        for (const Json& d : sh->items) {
            const uint64_t dim = integral(d, 2147483647.0);
            if (dim != 0 && count > (uint64_t(1) << 62) / dim) throw std::runtime_error("safetensors: shape too large for " + kv.first);
            count *= dim;
            shape.push_back((int)dim);
        }
        const uint64_t b = integral(off->items[0], 9007199254740992.0), e2 = integral(off->items[1], 9007199254740992.0);
        if (count > (uint64_t(1) << 62) / 8 || e2 < b || e2 > data_bytes || e2 - b != count * dtype_size(dtype))
            throw std::runtime_error("safetensors: bad data_offsets for " + kv.first);
        Array a(shape, dtype);
        in.seekg((std::streamoff)(8 + header_len + b));
        if (a.nbytes() && !in.read(a.data<char>(), (std::streamsize)a.nbytes()))
            throw std::runtime_error("safetensors: truncated data for " + kv.first);
        tensors.emplace(kv.first, std::move(a));
    }
    return {std::move(tensors), metadata_of(root)};
}

void save_safetensors(const std::string& path, const TensorMap& tensors, const MetadataMap& metadata) {
    std::map<std::string, const Array*> ordered;
    for (const auto& kv : tensors) ordered[kv.first] = &kv.second;

    std::ostringstream hdr;
    hdr << '{';
    bool first = true;
    if (!metadata.empty()) {
        const std::map<std::string, std::string> md(metadata.begin(), metadata.end());
        hdr << "\"__metadata__\":{";
        bool f2 = true;
        for (const auto& kv : md) {
            if (!f2) hdr << ',';
            f2 = false;
            hdr << json_quote(kv.first) << ':' << json_quote(kv.second);
        }
        hdr << '}';
        first = false;
    }
    uint64_t offset = 0;
    for (const auto& kv : ordered) {
        if (!first) hdr << ',';
        first = false;
        const Array& a = *kv.second;
        hdr << json_quote(kv.first) << ":{\"dtype\":\"" << dtype_name(a.dtype()) << "\",\"shape\":[";
        for (int i = 0; i < a.ndim(); ++i) hdr << (i ? "," : "") << a.shape(i);
        hdr << "],\"data_offsets\":[" << offset << ',' << offset + a.nbytes() << "]}";
        offset += a.nbytes();
    }
    hdr << '}';
    std::string text = hdr.str();
    while (text.size() % 8) text += ' ';

    std::ofstream out(path, std::ios::binary | std::ios::trunc);
    if (!out) throw std::runtime_error("safetensors: cannot create " + path);
    unsigned char len8[8];
    uint64_t n = text.size();
    for (int i = 0; i < 8; ++i) { len8[i] = (unsigned char)(n & 0xff); n >>= 8; }
    out.write(reinterpret_cast<const char*>(len8), 8);
    out.write(text.data(), (std::streamsize)text.size());
    for (const auto& kv : ordered)
        if (kv.second->nbytes()) out.write(kv.second->data<char>(), (std::streamsize)kv.second->nbytes());
    if (!out) throw std::runtime_error("safetensors: write failed for " + path);
}

MetadataMap read_tq_metadata(const std::string& path) {
    try {
        std::ifstream in(path, std::ios::binary);
        if (!in) return {};
        uint64_t header_len = 0;
        return metadata_of(read_header(in, path, &header_len));
    } catch (...) {
        return {};
    }
}

bool write_tq_safetensors(
    const std::string& path,
    const std::unordered_map<std::string, QuantizedWeight>& weights,
    const Codebook& primary_codebook,
    const Codebook& residual_codebook,
    const std::unordered_map<std::string, std::pair<Codebook, Codebook>>& per_layer_codebooks) {
    TensorMap tensors;
    for (const auto& kv : weights) {
        tensors.emplace(kv.first + ".packed_primary", kv.second.packed_primary);
        tensors.emplace(kv.first + ".packed_residual", kv.second.packed_residual);
        tensors.emplace(kv.first + ".norms", kv.second.norms);
        tensors.emplace(kv.first + ".seeds", kv.second.seeds);
    }
    for (const auto& kv : per_layer_codebooks) {
        tensors.emplace(kv.first + ".codebook_primary", centroid_tensor(kv.second.first));
        tensors.emplace(kv.first + ".codebook_residual", centroid_tensor(kv.second.second));
    }
    tensors.emplace("tq_codebook_primary", centroid_tensor(primary_codebook));
    tensors.emplace("tq_codebook_residual", centroid_tensor(residual_codebook));

    MetadataMap md;
    md["quantization_method"] = "turboquant";
    md["tq_version"] = "1";
    md["tq_primary_bits"] = std::to_string((int)primary_codebook.bits);
    md["tq_residual_bits"] = std::to_string((int)residual_codebook.bits);
    md["tq_total_bits"] = std::to_string((int)primary_codebook.bits + (int)residual_codebook.bits);
    if (!per_layer_codebooks.empty()) md["tq_per_layer_codebooks"] = "true";
    save_safetensors(path, tensors, md);
    return true;
}

std::unordered_map<std::string, TQLayer> read_tq_layers(const TensorMap& tensors, const MetadataMap& metadata) {
    auto bits_of = [&](const char* key, int fallback) {
        auto it = metadata.find(key);
        return (uint8_t)(it == metadata.end() ? fallback : std::atoi(it->second.c_str()));
    };
    const uint8_t pbits = bits_of("tq_primary_bits", 4), rbits = bits_of("tq_residual_bits", 4);
    const Codebook shared_p = codebook_from_tensor(need(tensors, "tq_codebook_primary"), pbits);
    const Codebook shared_r = codebook_from_tensor(need(tensors, "tq_codebook_residual"), rbits);
    auto pl = metadata.find("tq_per_layer_codebooks");
    const bool per_layer = pl != metadata.end() && pl->second == "true";

    static const std::string suffix = ".packed_primary";
    std::unordered_map<std::string, TQLayer> layers;
    for (const auto& kv : tensors) {
        const std::string& name = kv.first;
        if (name.size() < suffix.size() || name.compare(name.size() - suffix.size(), suffix.size(), suffix) != 0)
            continue;
        const std::string layer = name.substr(0, name.size() - suffix.size());
        TQLayer L;
        L.weights.packed_primary = kv.second;
        L.weights.packed_residual = need(tensors, layer + ".packed_residual");
        L.weights.norms = need(tensors, layer + ".norms");
        L.weights.seeds = need(tensors, layer + ".seeds");
        if (L.weights.seeds.dtype() != Dtype::U32) throw std::runtime_error("TQ8 file: seeds must be uint32");
        L.block_size = L.weights.seeds.size() > 2 ? L.weights.seeds.data<uint32_t>()[2] : 512u;
        L.primary_codebook = shared_p;
        L.residual_codebook = shared_r;
        if (per_layer) {
            auto p = tensors.find(layer + ".codebook_primary");
            auto r = tensors.find(layer + ".codebook_residual");
            if (p != tensors.end()) L.primary_codebook = codebook_from_tensor(p->second, pbits);
            if (r != tensors.end()) L.residual_codebook = codebook_from_tensor(r->second, rbits);
        }
        layers.emplace(layer, std::move(L));
    }
    return layers;
}

}  // namespace turboquant
