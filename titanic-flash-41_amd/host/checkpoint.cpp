#include "checkpoint.hpp"
#include "hip_rt.hpp"
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <memory>

namespace tf {
namespace {

constexpr uint64_t kHeaderLimit = 32ull * 1024 * 1024;                                            // src/checkpoint.rs:12

// The JSON subset a safetensors header and index hold: objects, arrays, strings, unsigned integers, literals.
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    double number = 0;
    std::string text;
    std::vector<Json> items;
    std::vector<std::pair<std::string, Json>> members;
    const Json* find(const std::string& key) const {
        for (const auto& m : members) if (m.first == key) return &m.second;
        return nullptr;
    }
};
class JsonParser {
public:
    JsonParser(const char* p, size_t n) : p_(p), end_(p + n) {}
    Json parse() { Json v = value(0); space(); ensure(p_ == end_, "trailing bytes after JSON value"); return v; }
private:
    void space() { while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) ++p_; }
    char peek() { space(); ensure(p_ < end_, "unexpected end of JSON"); return *p_; }
    void expect(char c) { ensure(peek() == c, "malformed JSON"); ++p_; }
    std::string string() {
        expect('"');
        std::string s;
        while (true) {
            ensure(p_ < end_, "unterminated JSON string");
            const char c = *p_++;
            if (c == '"') return s;
            if (c != '\\') { s.push_back(c); continue; }
            ensure(p_ < end_, "unterminated JSON escape");
            const char e = *p_++;
            switch (e) {
                case '"': case '\\': case '/': s.push_back(e); break;
                case 'n': s.push_back('\n'); break;
                case 't': s.push_back('\t'); break;
                case 'r': s.push_back('\r'); break;
                case 'b': s.push_back('\b'); break;
                case 'f': s.push_back('\f'); break;
                case 'u': {
                    ensure(end_ - p_ >= 4, "short JSON unicode escape");
                    unsigned code = 0;
                    for (int i = 0; i < 4; ++i) {
                        const char h = *p_++;
                        code = code * 16 + (h >= '0' && h <= '9' ? h - '0' : h >= 'a' && h <= 'f' ? h - 'a' + 10 : h >= 'A' && h <= 'F' ? h - 'A' + 10 : 256);
                    }
                    ensure(code < 0x80, "non-ASCII escape in a tensor name");     // names and dtypes are ASCII
                    s.push_back((char)code);
                    break;
                }
                default: ensure(false, "unknown JSON escape");
            }
        }
    }
    Json value(int depth) {
        ensure(depth < 16, "JSON nesting too deep");
        Json v;
        const char c = peek();
        if (c == '{') {
            v.kind = Json::Object; ++p_;
            if (peek() == '}') { ++p_; return v; }
            while (true) {
                std::string key = string();
                expect(':');
                v.members.emplace_back(std::move(key), value(depth + 1));
                if (peek() == ',') { ++p_; continue; }
                expect('}');
                return v;
            }
        }
        if (c == '[') {
            v.kind = Json::Array; ++p_;
            if (peek() == ']') { ++p_; return v; }
            while (true) {
                v.items.push_back(value(depth + 1));
                if (peek() == ',') { ++p_; continue; }
                expect(']');
                return v;
            }
        }
        if (c == '"') { v.kind = Json::String; v.text = string(); return v; }
        if (c == 't' && end_ - p_ >= 4 && !std::strncmp(p_, "true", 4)) { p_ += 4; v.kind = Json::Bool; v.number = 1; return v; }
        if (c == 'f' && end_ - p_ >= 5 && !std::strncmp(p_, "false", 5)) { p_ += 5; v.kind = Json::Bool; return v; }
        if (c == 'n' && end_ - p_ >= 4 && !std::strncmp(p_, "null", 4)) { p_ += 4; return v; }
        ensure((c >= '0' && c <= '9') || c == '-', "malformed JSON value");
        const char* start = p_;
        while (p_ < end_ && ((*p_ >= '0' && *p_ <= '9') || *p_ == '-' || *p_ == '+' || *p_ == '.' || *p_ == 'e' || *p_ == 'E')) ++p_;
        v.kind = Json::Number;
        v.text.assign(start, p_);
        v.number = std::strtod(v.text.c_str(), nullptr);
        return v;
    }
    const char* p_;
    const char* end_;
};
uint64_t as_u64(const Json& v, const char* what) {
    ensure(v.kind == Json::Number && !v.text.empty() && v.text.find_first_not_of("0123456789") == std::string::npos && v.text.size() <= 18, what);
    return std::strtoull(v.text.c_str(), nullptr, 10);
}

struct File {
    explicit File(const std::string& path) : f(std::fopen(path.c_str(), "rb")) { if (!f) throw Error("open " + path); }
    ~File() { if (f) std::fclose(f); }
    File(const File&) = delete;
    File& operator=(const File&) = delete;
    uint64_t size() { ensure(!std::fseek(f, 0, SEEK_END), "seek"); const long n = std::ftell(f); ensure(n >= 0, "tell"); return (uint64_t)n; }
    void read_at(uint64_t at, void* out, size_t n) {
        ensure(!std::fseek(f, (long)at, SEEK_SET) && std::fread(out, 1, n, f) == n, "short read from a checkpoint shard");
    }
    std::FILE* f;
};
void safe_filename(const std::string& name) {                                                    // src/checkpoint.rs safe_filename
    ensure(!name.empty() && name != "." && name != ".." && name.find('/') == std::string::npos && name.find('\\') == std::string::npos &&
               name.find('\0') == std::string::npos,
           "unsafe shard file name");
}
uint64_t dtype_bytes(const std::string& dtype) {                                                 // :28-36
    if (dtype == "F32") return 4;
    if (dtype == "BF16") return 2;
    if (dtype == "F8_E4M3" || dtype == "F8_E8M0" || dtype == "I8") return 1;
    throw Error("unsupported checkpoint dtype " + dtype);
}
void validate_tensor(const CheckpointTensor& t, const CheckpointShard& shard, const std::string& name) {   // :48-70
    ensure(!t.shape.empty() && t.shape.size() <= 4, "unsupported tensor rank");
    uint64_t elements = 1;
    for (uint64_t d : t.shape) {
        ensure(d == 0 || elements <= UINT64_MAX / (d ? d : 1), "shape overflow");
        elements *= d;
    }
    const uint64_t width = dtype_bytes(t.dtype);
    ensure(elements <= UINT64_MAX / width, "tensor size overflow");
    if (t.end < t.begin || t.end - t.begin != elements * width || t.end > shard.size - shard.data_start)
        throw Error("tensor bytes disagree with its shape: " + name);
}

}  // namespace

Checkpoint Checkpoint::scan(const std::string& root) {
    Checkpoint c;
    c.root_ = root;
    std::map<std::string, std::string> weight_map;
    {
        File index(root + "/model.safetensors.index.json");
        const uint64_t n = index.size();
        ensure(n > 1 && n <= kHeaderLimit, "invalid checkpoint index size");
        std::string text((size_t)n, '\0');
        index.read_at(0, text.data(), (size_t)n);
        const Json doc = JsonParser(text.data(), text.size()).parse();
        const Json* map = doc.kind == Json::Object ? doc.find("weight_map") : nullptr;
        ensure(map && map->kind == Json::Object && !map->members.empty(), "empty checkpoint");
        for (const auto& m : map->members) {
            ensure(m.second.kind == Json::String, "weight_map values are file names");
            ensure(weight_map.emplace(m.first, m.second.text).second, "duplicate tensor in the index");
        }
    }
    std::map<std::string, int> names;
    for (const auto& m : weight_map) names[m.second] = 0;
    for (const auto& entry : names) {
        const std::string& name = entry.first;
        safe_filename(name);
        File f(root + "/" + name);
        CheckpointShard shard;
        shard.size = f.size();
        ensure(shard.size >= 8, "invalid header size: shard shorter than its length field");
        uint8_t le[8];
        f.read_at(0, le, 8);
        uint64_t n = 0;
        for (int i = 7; i >= 0; --i) n = (n << 8) | le[i];
        if (!(n > 1 && n <= kHeaderLimit && n + 8 <= shard.size)) throw Error("invalid header size: " + name);
        shard.data_start = n + 8;
        std::string text((size_t)n, '\0');
        f.read_at(8, text.data(), (size_t)n);
        const Json header = JsonParser(text.data(), text.size()).parse();
        ensure(header.kind == Json::Object, "shard header is not an object");
        for (const auto& m : header.members) {
            if (m.first == "__metadata__") continue;
            const auto owner = weight_map.find(m.first);
            if (owner == weight_map.end() || owner->second != name) throw Error("index/header disagreement: " + m.first);
            const Json& v = m.second;
            const Json *dtype = v.find("dtype"), *shape = v.find("shape"), *offsets = v.find("data_offsets");
            ensure(v.kind == Json::Object && dtype && dtype->kind == Json::String && shape && shape->kind == Json::Array && offsets &&
                       offsets->kind == Json::Array && offsets->items.size() == 2,
                   "malformed tensor entry");
            CheckpointTensor t;
            t.file = name;
            t.dtype = dtype->text;
            for (const Json& d : shape->items) t.shape.push_back(as_u64(d, "tensor shape"));
            t.begin = as_u64(offsets->items[0], "data offset");
            t.end = as_u64(offsets->items[1], "data offset");
            validate_tensor(t, shard, m.first);
            if (!c.tensors_.emplace(m.first, std::move(t)).second) throw Error("duplicate tensor " + m.first);
        }
        c.files_[name] = shard;
    }
    ensure(c.tensors_.size() == weight_map.size(), "index tensor missing in headers");
    c.validate();
    return c;
}
void Checkpoint::validate() const {
    ensure(!files_.empty() && !tensors_.empty(), "empty manifest");
    std::map<std::string, std::vector<std::pair<uint64_t, uint64_t>>> ranges;
    for (const auto& f : files_) ensure(f.second.data_start >= 8 && f.second.data_start <= f.second.size, "invalid shard metadata");
    for (const auto& t : tensors_) {
        const auto shard = files_.find(t.second.file);
        ensure(shard != files_.end(), "unknown shard");
        validate_tensor(t.second, shard->second, t.first);
        ranges[t.second.file].emplace_back(t.second.begin, t.second.end);
    }
    for (auto& r : ranges) {
        std::sort(r.second.begin(), r.second.end());
        uint64_t end = 0;
        for (const auto& span : r.second) {
            if (span.first != end) throw Error("overlap or hole in " + r.first);
            end = span.second;
        }
        const CheckpointShard& s = files_.at(r.first);
        if (end != s.size - s.data_start) throw Error("unindexed trailing data in " + r.first);
    }
}
const CheckpointTensor& Checkpoint::tensor(const std::string& name) const {
    const auto t = tensors_.find(name);
    if (t == tensors_.end()) throw Error("missing tensor " + name);
    return t->second;
}
void Checkpoint::require(const std::string& name, const std::string& dtype, const std::vector<uint64_t>& shape) const {
    const CheckpointTensor& t = tensor(name);
    if (t.dtype != dtype || t.shape != shape) throw Error("tensor contract mismatch: " + name);
}
std::vector<uint8_t> Checkpoint::read(const std::string& name) const {
    const CheckpointTensor& t = tensor(name);
    const CheckpointShard& s = files_.at(t.file);
    std::vector<uint8_t> out((size_t)t.bytes());
    File f(root_ + "/" + t.file);
    f.read_at(s.data_start + t.begin, out.data(), out.size());
    return out;
}

std::vector<TensorContract> ffn_layer_contract(const std::string& p, const ca_geometry& g) {
    const uint64_t H = g.hidden, E = g.experts, I = g.intermediate, S = g.shared_intermediate, bn = g.shared_bn, bk = g.shared_bk;
    std::vector<TensorContract> c;
    for (uint64_t e = 0; e < E; ++e) {
        const std::string x = p + ".ffn.experts." + std::to_string(e) + ".";
        for (const char* name : {"w1", "w3"}) {
            c.push_back({x + name + ".weight", "I8", {I, H / 2}});
            c.push_back({x + name + ".scale", "F8_E8M0", {I, H / 32}});
        }
        c.push_back({x + "w2.weight", "I8", {H, I / 2}});
        c.push_back({x + "w2.scale", "F8_E8M0", {H, I / 32}});
    }
    for (const char* name : {"w1", "w3"}) {
        c.push_back({p + ".ffn.shared_experts." + name + ".weight", "F8_E4M3", {S, H}});
        c.push_back({p + ".ffn.shared_experts." + name + ".scale", "F8_E8M0", {S / bn, H / bk}});
    }
    c.push_back({p + ".ffn.shared_experts.w2.weight", "F8_E4M3", {H, S}});
    c.push_back({p + ".ffn.shared_experts.w2.scale", "F8_E8M0", {H / bn, S / bk}});
    c.push_back({p + ".ffn.gate.weight", "BF16", {E, H}});
    c.push_back({p + ".ffn.gate.bias", "F32", {E}});
    c.push_back({p + ".ffn.gate.bias_vl", "F32", {E}});
    return c;
}

LayerOperandsHost load_ffn_layer(const Checkpoint& cp, const std::string& p, const ca_geometry& g) {
    const uint64_t H = g.hidden, E = g.experts, I = g.intermediate;
    LayerOperandsHost out;
    // the contract first (src/layout.rs:247-275), then the bytes
    for (const TensorContract& t : ffn_layer_contract(p, g)) cp.require(t.name, t.dtype, t.shape);

    auto append = [&](std::vector<uint8_t>& to, const std::string& name, bool expert_scale) {
        const std::vector<uint8_t> bytes = cp.read(name);
        if (expert_scale)                                                                         // src/weights.rs:538-542
            for (uint8_t b : bytes) if (b > 247) throw Error("canonical expert scale exceeds lossless conversion range: " + name);
        to.insert(to.end(), bytes.begin(), bytes.end());
    };
    out.w13.reserve(E * 2 * I * H / 2); out.s13.reserve(E * 2 * I * H / 32); out.w2.reserve(E * H * I / 2); out.s2.reserve(E * H * I / 32);
    for (uint64_t e = 0; e < E; ++e) {                                                           // up (w3) precedes gate (w1): src/weights.rs:334-340
        const std::string x = p + ".ffn.experts." + std::to_string(e) + ".";
        append(out.w13, x + "w3.weight", false); append(out.w13, x + "w1.weight", false);
        append(out.s13, x + "w3.scale", true); append(out.s13, x + "w1.scale", true);
        append(out.w2, x + "w2.weight", false);
        append(out.s2, x + "w2.scale", true);
    }
    const std::string sh = p + ".ffn.shared_experts.";                                           // gate (w1) rows first: src/blockscaled.rs:132-133
    append(out.sh_w13, sh + "w1.weight", false); append(out.sh_w13, sh + "w3.weight", false);
    append(out.sh_s13, sh + "w1.scale", false); append(out.sh_s13, sh + "w3.scale", false);
    append(out.sh_w2, sh + "w2.weight", false);
    append(out.sh_s2, sh + "w2.scale", false);
    const std::vector<uint8_t> gate = cp.read(p + ".ffn.gate.weight"), bias = cp.read(p + ".ffn.gate.bias"), alt = cp.read(p + ".ffn.gate.bias_vl");
    out.gate_w.resize(gate.size() / 2); std::memcpy(out.gate_w.data(), gate.data(), gate.size());
    out.bias.resize(bias.size() / 4); std::memcpy(out.bias.data(), bias.data(), bias.size());
    out.bias_alt.resize(alt.size() / 4); std::memcpy(out.bias_alt.data(), alt.data(), alt.size());
    return out;
}

}  // namespace tf
