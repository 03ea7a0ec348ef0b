// Host mirror of the reference's Rust FFN operators: see ffn_host.hpp for the map of names.
#include "ffn_host.hpp"
#include <dlfcn.h>
#include <algorithm>
#include <cstdio>
#include <fstream>
#include <vector>

namespace tf {

namespace {
template <class F>
F symbol(void* lib, const char* name) {
    void* p = dlsym(lib, name);
    if (!p) throw Error(std::string("missing symbol ") + name);
    return reinterpret_cast<F>(p);
}
size_t align256(size_t n) { return (n + 255) / 256 * 256; }

// SHA-256 (FIPS 180-4) of a file, as lower-case hexadecimal; empty when the file cannot be read.
std::string sha256_file(const std::string& path) {
    static const uint32_t K[64] = {
        0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01, 0x243185be,
        0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa,
        0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967, 0x27b70a85,
        0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85, 0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3,
        0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f,
        0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
    std::ifstream in(path, std::ios::binary);
    if (!in) return std::string();
    std::vector<uint8_t> data((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    const uint64_t bits = (uint64_t)data.size() * 8;
    data.push_back(0x80);
    while (data.size() % 64 != 56) data.push_back(0);
    for (int i = 7; i >= 0; --i) data.push_back((uint8_t)(bits >> (8 * i)));
    uint32_t h[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
    auto rotr = [](uint32_t v, int n) { return (v >> n) | (v << (32 - n)); };
    for (size_t at = 0; at < data.size(); at += 64) {
        uint32_t w[64];
        for (int i = 0; i < 16; ++i) w[i] = (uint32_t)data[at + 4 * i] << 24 | (uint32_t)data[at + 4 * i + 1] << 16 | (uint32_t)data[at + 4 * i + 2] << 8 | data[at + 4 * i + 3];
        for (int i = 16; i < 64; ++i)
            w[i] = w[i - 16] + (rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3)) + w[i - 7] + (rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10));
        uint32_t v[8];
        for (int i = 0; i < 8; ++i) v[i] = h[i];
        for (int i = 0; i < 64; ++i) {
            const uint32_t t1 = v[7] + (rotr(v[4], 6) ^ rotr(v[4], 11) ^ rotr(v[4], 25)) + ((v[4] & v[5]) ^ (~v[4] & v[6])) + K[i] + w[i];
            const uint32_t t2 = (rotr(v[0], 2) ^ rotr(v[0], 13) ^ rotr(v[0], 22)) + ((v[0] & v[1]) ^ (v[0] & v[2]) ^ (v[1] & v[2]));
            v[7] = v[6]; v[6] = v[5]; v[5] = v[4]; v[4] = v[3] + t1; v[3] = v[2]; v[2] = v[1]; v[1] = v[0]; v[0] = t1 + t2;
        }
        for (int i = 0; i < 8; ++i) h[i] += v[i];
    }
    char hex[65];
    for (int i = 0; i < 8; ++i) std::snprintf(hex + 8 * i, 9, "%08x", h[i]);
    return std::string(hex, 64);
}
// The value of "library_sha256" in the manifest the build writes beside the library (manifest.json); empty when absent.
std::string manifest_sha256(const std::string& library) {
    const size_t slash = library.find_last_of('/');
    std::ifstream in((slash == std::string::npos ? std::string() : library.substr(0, slash + 1)) + "manifest.json");
    if (!in) return std::string();
    const std::string text((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    const size_t key = text.find("\"library_sha256\"");
    if (key == std::string::npos) return std::string();
    const size_t open = text.find('"', text.find(':', key) + 1);
    const size_t close = open == std::string::npos ? open : text.find('"', open + 1);
    return close == std::string::npos ? std::string() : text.substr(open + 1, close - open - 1);
}
}  // namespace

std::string library_sha256(const std::string& path) { return sha256_file(path); }

// ---- Native ---------------------------------------------------------------------------------------------------------
Native::Native(const std::string& library, const ca_geometry& geometry) : g_(geometry) {
    // the library is the one the build's manifest pins (src/ffn.rs:70-74, src/primitives.rs:75-79: "hash mismatch")
    const std::string pinned = manifest_sha256(library);
    if (!pinned.empty() && pinned != sha256_file(library)) throw Error("FFN native library hash mismatch: " + library);
    lib_ = dlopen(library.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!lib_) throw Error(std::string("load kernel library: ") + dlerror());
    ensure(symbol<int (*)()>(lib_, "ca_ffn_abi")() == 1, "FFN native ABI mismatch");                    // src/ffn.rs:76-77
    ensure(symbol<int32_t (*)()>(lib_, "ca_primitives_abi")() == 1, "primitive entrypoint ABI mismatch"); // src/primitives.rs:104-108
    // the geometry lives in this object's context, not in the library's process state: layers of different geometries
    // (the reference's target and drafter, src/layer_id.rs:39-47) keep a Native each
    router_logits_ = symbol<decltype(router_logits_)>(lib_, "ca_router_logits_in");
    router_logits_wide_ = symbol<decltype(router_logits_wide_)>(lib_, "ca_router_logits_wide_in");
    shared_swiglu_ = symbol<decltype(shared_swiglu_)>(lib_, "ca_shared_swiglu_in");
    ffn_add_ = symbol<decltype(ffn_add_)>(lib_, "ca_ffn_add_in");
    spin_limit_ = symbol<decltype(spin_limit_)>(lib_, "ca_primitives_spin_limit");
    shared_reserve_ = symbol<decltype(shared_reserve_)>(lib_, "ca_primitives_shared_reserve");
    kernel_launch_ = symbol<decltype(kernel_launch_)>(lib_, "ca_kernel_launch");
    close_ = symbol<decltype(close_)>(lib_, "ca_primitives_close");
    launch_ = symbol<decltype(launch_)>(lib_, "ca_primitives_launch");
    scratch_bytes_ = symbol<decltype(scratch_bytes_)>(lib_, "ca_primitives_scratch_bytes");
    marks_ = symbol<decltype(marks_)>(lib_, "ca_primitives_marks");
    encode_ = symbol<decltype(encode_)>(lib_, "ca_encode");                                              // src/ffn.rs:808-811
    decode_ = symbol<decltype(decode_)>(lib_, "ca_decode");
    local_live_ = symbol<decltype(local_live_)>(lib_, "ca_local_live");
    pack_bf16_ = symbol<decltype(pack_bf16_)>(lib_, "ca_pack_bf16");
    int32_t status = 0;
    ctx_ = symbol<void* (*)(const ca_geometry*, int32_t*)>(lib_, "ca_primitives_open_geometry")(&g_, &status);
    if (status == -4) throw Error("FFN native contract changed: geometry rejected (" + std::to_string(status) + ")");
    if (status != 0 || !ctx_) throw Error("initialize primitive library: " + std::to_string(status));   // src/primitives.rs:116-119
}
Native::~Native() {
    if (ctx_ && close_) close_(ctx_);
    if (lib_) dlclose(lib_);
}
void Native::marks(hipEvent_t* events, size_t count) const {
    ensure(marks_(ctx_, (void* const*)events, events ? count : 0) == 0, "profiling marks rejected");
}
void Native::codec_encode(uint64_t routed, uint64_t scales, uint64_t shared, uint64_t packed, int rows, int k, hipStream_t s) const {
    ensure(encode_((const uint8_t*)routed, (const uint8_t*)scales, (const uint8_t*)shared, (uint8_t*)packed, rows, k, s) == 0, "packed MoE encode launch");   // src/ffn.rs:856-858
}
void Native::codec_decode(uint64_t packed, uint64_t shared, uint64_t row_scales, uint64_t mma_scales, int rows, int k, hipStream_t s) const {
    ensure(decode_((const uint8_t*)packed, (uint8_t*)shared, (uint8_t*)row_scales, (uint8_t*)mma_scales, rows, k, s) == 0, "packed MoE shared decode launch");   // :872-874
}
void Native::codec_local_live(uint64_t global, uint64_t local, int rows, int rank, hipStream_t s) const {
    ensure(local_live_((const int*)global, (int*)local, rows, rank, s) == 0, "packed MoE local metadata launch");                   // :845-846
}
void Native::codec_pack_bf16(uint64_t input, uint64_t packed, int rows, int k, hipStream_t s) const {
    ensure(pack_bf16_((const void*)input, (uint8_t*)packed, rows, k, s) == 0, "fused packed MoE producer launch");                  // :849-850
}
void Native::router_logits(int rows, uint64_t x, uint64_t w, uint64_t out, hipStream_t s) const {
    ensure(router_logits_(ctx_, rows, (const void*)x, (const void*)w, (void*)out, s) == 0, "tiny router GPU launch failed");   // src/ffn.rs:352-363
}
void Native::router_logits_wide(int rows, uint64_t x, uint64_t w, uint64_t out, hipStream_t s) const {
    ensure(router_logits_wide_(ctx_, rows, (const void*)x, (const void*)w, (void*)out, s) == 0, "wide router GPU launch failed");
}
void Native::shared_swiglu(int rows, uint64_t in, uint64_t out, hipStream_t s) const {
    ensure(shared_swiglu_(ctx_, rows, (const void*)in, (void*)out, s) == 0, "shared SwiGLU launch failed");                    // src/ffn.rs:1108-1118
}
void Native::ffn_add(int rows, uint64_t routed, uint64_t shared, uint64_t out, hipStream_t s) const {
    ensure(ffn_add_(ctx_, rows, (const void*)routed, (const void*)shared, (void*)out, s) == 0, "FFN shared addition launch failed");   // src/ffn.rs:1071-1082
}
void Native::spin_limit(int limit) const { ensure(spin_limit_(ctx_, limit) == 0, "spin limit rejected"); }
int Native::compute_units() const {
    int device = 0, cus = 0;
    check(hipGetDevice(&device), "current device");
    check(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device), "compute unit count");
    return cus;
}
void Native::shared_reserve(int cus) const { ensure(shared_reserve_(ctx_, cus) == 0, "shared expert CU reserve rejected"); }
void Native::launch(const char* name, uint32_t grid_x, uint32_t grid_y, uint32_t block, uint32_t shared, void** args, hipStream_t s) const {
    const uint32_t grid[3] = {grid_x, grid_y, 1}, blk[3] = {block, 1, 1};
    const int status = kernel_launch_(name, grid, blk, shared, args, s);
    if (status != 0) throw Error(std::string("kernel launch failed: ") + name + " (" + std::to_string(status) + ")");
}
void Native::primitive(int index, const uint64_t* pointers, size_t np, const int32_t* scalars, size_t ns, hipStream_t s, const char* what) const {
    const int32_t status = launch_(ctx_, index, pointers, np, scalars, ns, s);
    if (status != 0) throw Error(std::string(what) + ": primitive launch status " + std::to_string(status));            // src/primitives.rs:150
}
int64_t Native::scratch_bytes(int index, int rows) const { return scratch_bytes_(ctx_, index, rows); }

// ---- Weights --------------------------------------------------------------------------------------------------------
void Weights::layout(const ca_geometry& g) {
    const size_t H = g.hidden, E = g.experts, I = g.intermediate, S = g.shared_intermediate;
    const size_t wb = I * H / 2, sb = I * H / 32;
    size_t at = 0;
    auto add = [&](const std::string& name, size_t bytes) { views_[name] = View{at, bytes}; at += align256(bytes); };
    add("ffn.gate.weight", E * H * 2);
    add("ffn.gate.bias", E * 4);
    add("ffn.gate.bias_vl", E * 4);
    // expert groups, contiguous and in the kernels' order (src/weights.rs:330-353): [e][w3 | w1], [e][w2], scales likewise
    add("ffn.experts.w13", E * 2 * wb);
    add("ffn.experts.w2", E * wb);
    add("ffn.experts.s13", E * 2 * sb);
    add("ffn.experts.s2", E * sb);
    add("ffn.shared_experts.w13.weight", 2 * S * H);
    add("ffn.shared_experts.w13.scale", (2 * S / g.shared_bn) * (H / g.shared_bk));
    add("ffn.shared_experts.w2.weight", H * S);
    add("ffn.shared_experts.w2.scale", (H / g.shared_bn) * (S / g.shared_bk));
    add("ffn.shared_experts.w13.prepared", 2 * S * H);
    add("ffn.shared_experts.w2.prepared", H * S);
    atlas_ = Buffer<uint8_t>(at);
}
ca_geometry padded_geometry(const ca_geometry& g) {
    ca_geometry p = g;
    p.intermediate = (g.intermediate + 511) / 512 * 512;
    p.shared_intermediate = (g.shared_intermediate + 511) / 512 * 512;
    return p;
}
void Weights::fill(const ca_geometry& g, const Host& src, hipMemcpyKind kind) {
    auto put = [&](const char* name, const void* from) {
        const View& v = view(name);
        check(hipMemcpy((void*)(atlas_.ptr() + v.offset), from, v.bytes, kind), "weight upload");
    };
    // `count` pieces of `piece` source bytes each, `stride` bytes apart in the (zeroed) view
    auto put_pieces = [&](const char* name, const void* from, size_t piece, size_t stride, size_t count) {
        const View& v = view(name);
        ensure(piece <= stride && stride * count == v.bytes, "padded weight view");
        check(hipMemset((void*)(atlas_.ptr() + v.offset), 0, v.bytes), "weight padding");
        check(hipMemcpy2D((void*)(atlas_.ptr() + v.offset), stride, from, piece, piece, count, kind), "weight upload");
    };
    const size_t H = g.hidden, E = g.experts, I = g.intermediate, S = g.shared_intermediate;
    const size_t Is = src.source_intermediate ? src.source_intermediate : I, Ss = src.source_shared_intermediate ? src.source_shared_intermediate : S;
    ensure(Is <= I && Ss <= S && Is % 32 == 0 && Is % (size_t)g.act_block == 0 && Ss % (size_t)g.act_block == 0 && Ss % (size_t)g.shared_bn == 0 &&
           Ss % (size_t)g.shared_bk == 0, "narrower expert operands must end on whole quantization blocks");
    put("ffn.gate.weight", src.gate_w); put("ffn.gate.bias", src.bias); put("ffn.gate.bias_vl", src.bias_alt);
    if (Is == I) {
        put("ffn.experts.w13", src.w13); put("ffn.experts.w2", src.w2); put("ffn.experts.s13", src.s13); put("ffn.experts.s2", src.s2);
    } else {
        put_pieces("ffn.experts.w13", src.w13, Is * H / 2, I * H / 2, 2 * E);          // per expert: up rows, gate rows
        put_pieces("ffn.experts.s13", src.s13, Is * H / 32, I * H / 32, 2 * E);
        put_pieces("ffn.experts.w2", src.w2, Is / 2, I / 2, E * H);                     // per output row: its K columns
        put_pieces("ffn.experts.s2", src.s2, Is / 32, I / 32, E * H);
    }
    if (Ss == S) {
        put("ffn.shared_experts.w13.weight", src.sh_w13); put("ffn.shared_experts.w13.scale", src.sh_s13);
        put("ffn.shared_experts.w2.weight", src.sh_w2); put("ffn.shared_experts.w2.scale", src.sh_s2);
    } else {
        const size_t bn = g.shared_bn, bk = g.shared_bk;
        put_pieces("ffn.shared_experts.w13.weight", src.sh_w13, Ss * H, S * H, 2);      // gate rows, up rows
        put_pieces("ffn.shared_experts.w13.scale", src.sh_s13, (Ss / bn) * (H / bk), (S / bn) * (H / bk), 2);
        put_pieces("ffn.shared_experts.w2.weight", src.sh_w2, Ss, S, H);
        put_pieces("ffn.shared_experts.w2.scale", src.sh_s2, Ss / bk, S / bk, H / bn);
    }
}
Weights::Weights(const ca_geometry& g, const Host& host) { layout(g); fill(g, host, hipMemcpyHostToDevice); }
Weights::Weights(const ca_geometry& g, const Host& device, bool) { layout(g); fill(g, device, hipMemcpyDeviceToDevice); }
const View& Weights::view(const std::string& name) const {
    auto it = views_.find(name);
    if (it == views_.end()) throw Error("unknown weight view " + name);
    return it->second;
}
uint64_t Weights::pointer_at(size_t offset, size_t bytes) const {
    ensure(offset + bytes <= atlas_.bytes(), "weight range outside the atlas");
    return atlas_.ptr() + offset;
}

// ---- expert preparation ---------------------------------------------------------------------------------------------------
// src/expert_packing.rs:46-207: validate the contiguous atlas, re-lay every matrix through a scratch buffer and copy it
// back in place (here: one launch per group, since the layouts tile by 16 rows and expert matrices are whole tiles).
Prepared prepare_layer(const Native& native, Weights& weights, size_t layer) {
    const ca_geometry& g = native.geometry();
    const size_t E = g.experts, n = g.intermediate, k = g.hidden;
    ensure(n > 0 && n <= 65536 && k > 0 && k <= 65536 && n % 64 == 0 && k % 64 == 0 && n % 512 == 0 && k % 512 == 0,
           "compact expert layout requires whole N64/K64 row groups");                                // :260-274 (+ the 512 scale words here)
    const size_t wb = n * k / 2, sb = n * k / 32;
    const View w13 = weights.view("ffn.experts.w13"), w2 = weights.view("ffn.experts.w2"), s13 = weights.view("ffn.experts.s13"),
               s2 = weights.view("ffn.experts.s2");
    ensure(w13.bytes == E * 2 * wb && w2.bytes == E * wb && s13.bytes == E * 2 * sb && s2.bytes == E * sb,
           "expert atlas is not the exact contiguous kernel layout");                                // :124-128
    ensure(!weights.expert_ready(), "expert layer already prepared");
    Stream stream;
    Buffer<uint8_t> scratch(E * 2 * wb);
    struct Job { const char* symbol; View view; int rows, cols; size_t unit; };
    const Job jobs[] = {
        {"ca_expert_compact_words", w13, (int)(E * 2 * n), (int)k, 32}, {"ca_expert_compact_scales", s13, (int)(E * 2 * n), (int)k, 32},
        {"ca_expert_compact_words", w2, (int)(E * k), (int)n, 32}, {"ca_expert_compact_scales", s2, (int)(E * k), (int)n, 32}};
    for (const Job& j : jobs) {
        uint64_t src = weights.pointer_at(j.view.offset, j.view.bytes), dst = scratch.ptr();
        int nr = j.rows, kr = j.cols, group = j.rows;
        void* args[] = {&src, &dst, &nr, &kr, &group};
        const size_t total = (size_t)j.rows * (j.cols / j.unit);
        native.launch(j.symbol, (uint32_t)((total + 255) / 256), 1, 256, 0, args, stream.raw());
        check(hipMemcpyAsync((void*)src, (void*)dst, j.view.bytes, hipMemcpyDeviceToDevice, stream.raw()), "prepared copy back");   // :170
    }
    stream.synchronize();
    weights.finish_expert_layer();
    Prepared p;
    p.layer = layer; p.experts = E; p.hidden = k; p.intermediate = n;
    p.w13_offset = w13.offset; p.w2_offset = w2.offset; p.s13_offset = s13.offset; p.s2_offset = s2.offset;
    p.resident_bytes = E * (3 * wb + 3 * sb); p.temporary_bytes = scratch.bytes();
    return p;
}
// src/expert_packing.rs:212-259 + src/config.rs:1365-1375
ScaleCodeReport code_layer_scales(const Native& native, Weights& weights, const Prepared& p) {
    const size_t E = p.experts, n = p.intermediate, k = p.hidden;
    const size_t t13 = (n + 127) / 128, s13 = (k + 127) / 128, t2 = (k + 127) / 128, s2 = (n / 32 + 3) / 4;
    const size_t u13 = t13 * s13, u2 = t2 * s2;
    const size_t f13 = E * 2 * u13 * 16, b13 = f13 + E * 2 * u13 * 4, c2 = b13 + (2 * E + 3) / 4 * 4, f2 = c2 + E * u2 * 16,
                 b2 = f2 + E * u2 * 4, words = b2 + E;
    Buffer<uint32_t> code(words), error(1);
    Buffer<unsigned long long> counts(1);
    code.zero(); error.zero(); counts.zero();
    Stream stream;
    struct Part { size_t offset, matrices, rows, columns, c, f, b; };
    const Part parts[] = {{p.s13_offset, 2 * E, n, k / 32, 0, f13, b13}, {p.s2_offset, E, k, n / 32, c2, f2, b2}};
    for (const Part& part : parts) {
        const size_t units = (part.rows + 127) / 128 * ((part.columns + 3) / 4);
        uint64_t src = weights.pointer_at(part.offset, part.matrices * part.rows * part.columns);
        uint64_t cp = code.ptr() + part.c * 4, fp = code.ptr() + part.f * 4, bp = code.ptr() + part.b * 4, status = error.ptr(), tally = counts.ptr();
        int nr = (int)part.rows, cols = (int)part.columns;
        void* a1[] = {&src, &cp, &fp, &bp, &nr, &cols};
        native.launch("ca_expert_scale_code1", (uint32_t)part.matrices, 1, 256, 0, a1, stream.raw());
        void* a2[] = {&src, &cp, &fp, &bp, &status, &nr, &cols};
        native.launch("ca_expert_scale_code1_check", (uint32_t)((units * 128 + 255) / 256), (uint32_t)part.matrices, 256, 0, a2, stream.raw());
        size_t flag_words = part.matrices * units * 4;
        void* a3[] = {&fp, &tally, &flag_words};
        native.launch("ca_expert_scale_code1_census", (uint32_t)((flag_words + 255) / 256), 1, 256, 0, a3, stream.raw());
    }
    stream.synchronize();
    const uint32_t status = error.download()[0];
    if (status != 0) throw Error("expert scale code failed its decode check (layer " + std::to_string(p.layer) + ", error " + std::to_string(status) + ")");
    ScaleCodeReport report;
    report.bytes = words * 4;
    report.raw_rows = (size_t)counts.download()[0];
    report.rows = E * (2 * u13 + u2) * 128;
    weights.install_expert_scale_code1(std::move(code));
    return report;
}

Expert::Expert(std::shared_ptr<Weights> weights, Prepared layout) : weights_(std::move(weights)), layout_(layout) {
    ensure(weights_->expert_ready(), "expert layer is not ready");                                        // src/moe.rs:128-131
}
std::pair<uint64_t, size_t> Expert::region(const std::string& role) const {                                // src/moe.rs:143-155
    const Prepared& l = layout_;
    const size_t wb = l.hidden * l.intermediate / 2, sb = l.hidden * l.intermediate / 32;
    size_t offset, bytes;
    if (role == "w13") { offset = l.w13_offset; bytes = 2 * l.experts * wb; }
    else if (role == "w2") { offset = l.w2_offset; bytes = l.experts * wb; }
    else if (role == "s13") { offset = l.s13_offset; bytes = 2 * l.experts * sb; }
    else if (role == "s2") { offset = l.s2_offset; bytes = l.experts * sb; }
    else throw Error("unknown expert operand");
    return {weights_->pointer_at(offset, bytes), bytes};
}

SharedMatrix prepare_shared(const Native& native, Weights& weights, const std::string& name, size_t n, size_t k) {
    const View src = weights.view(name + ".weight"), dst = weights.view(name + ".prepared");
    ensure(src.bytes == n * k && dst.bytes == n * k && n % 16 == 0 && k % 128 == 0, "shared matrix geometry mismatch");
    Stream stream;
    uint64_t from = weights.pointer_at(src.offset, src.bytes), to = weights.pointer_at(dst.offset, dst.bytes);
    int nr = (int)n, kr = (int)k, inverse = 0;
    void* args[] = {&from, &to, &nr, &kr, &inverse};
    native.launch("ca_dense_compact_fp8", (uint32_t)((n * (k / 16) + 255) / 256), 1, 256, 0, args, stream.raw());
    stream.synchronize();
    return SharedMatrix{to, weights.ptr(name + ".scale"), n, k};
}

// ---- TokenRows --------------------------------------------------------------------------------------------------------------
TokenRows::TokenRows(const int64_t* ids, size_t rows, size_t live) : ids_(rows), live_(1), padding_sources_(rows), rows_(rows) {
    ensure(rows > 0 && rows <= 65536, "token row capacity");                                                // src/ffn.rs:103
    std::vector<int32_t> none(rows, -1);
    padding_sources_.upload(none);
    update(ids, rows, live);
}
void TokenRows::update(const int64_t* ids, size_t rows, size_t live) {
    bool domain = rows == rows_ && live <= rows_;
    for (size_t i = 0; domain && i < rows; ++i) domain = ids[i] >= 0 && ids[i] < 129280;
    ensure(domain, "router token metadata domain");                                                          // src/ffn.rs:121-126
    ids_.upload(ids, rows);
    const int32_t n = (int32_t)live;
    live_.upload(&n, 1);
    active_rows_ = live;
    padding_active_ = false;                                                                                 // :132-133
}
void TokenRows::set_padding_sources(const int32_t* sources, size_t rows) {
    bool ok = rows == rows_;
    for (size_t r = 0; ok && r < rows; ++r) {
        const int32_t s = sources[r];
        ok = s < 0 || ((size_t)s < active_rows_ && (size_t)s != r && sources[s] < 0);
    }
    ensure(ok, "padding route sources must name live rows");                                                 // src/ffn.rs:139-141
    padding_sources_.upload(sources, rows);
    padding_active_ = true;
}

// ---- Router -----------------------------------------------------------------------------------------------------------------
Router::Router(std::shared_ptr<const Native> native, std::shared_ptr<Weights> weights, size_t rows)
    : native_(std::move(native)), weights_(std::move(weights)), rows_(rows), logits_(rows * native_->geometry().experts),
      routing_(rows * native_->geometry().topk), ids_(rows * native_->geometry().topk), census_(native_->geometry().experts) {
    const ca_geometry& g = native_->geometry();
    ensure(rows >= 1, "router row capacity");
    ensure(weights_->view("ffn.gate.weight").bytes == (size_t)g.experts * g.hidden * 2 && weights_->view("ffn.gate.bias").bytes == (size_t)g.experts * 4,
           "router checkpoint shape/dtype mismatch");                                                        // src/ffn.rs:225-228
    census_.zero();
}
std::optional<RouteOperands> Router::run_routed(uint64_t input, size_t input_len, const TokenRows& tokens, bool fused, const Stream& stream,
                                                bool gate_front) {
    const ca_geometry& g = native_->geometry();
    ensure(input_len == rows_ * (size_t)g.hidden && tokens.rows() == rows_, "router shape/context mismatch");   // src/ffn.rs:331-339
    ensure(!stream_set_ || stream_ == stream.raw(), "router needs one ordered stream");                        // :340-345
    stream_ = stream.raw(); stream_set_ = true;
    const uint64_t gate = weights_->ptr("ffn.gate.weight");
    const bool gate_in_front = fused && gate_front && rows_ <= 64;
    if (gate_in_front) {
    } else if (rows_ <= 64) {
        for (size_t offset = 0; offset < rows_; offset += 16)                                                  // :351-364
            native_->router_logits((int)std::min<size_t>(16, rows_ - offset), input + offset * g.hidden * 2, gate,
                                   logits_.ptr() + offset * g.experts * 4, stream.raw());
    } else {
        native_->router_logits_wide((int)rows_, input, gate, logits_.ptr(), stream.raw());                     // Scores::Vendor, :366
    }
    const uint64_t bias = weights_->ptr("ffn.gate.bias"), bias_alt = weights_->ptr("ffn.gate.bias_vl");
    if (fused) {
        ensure(rows_ * g.topk <= 1024, "fused routing owner");                                                 // :370-371
        return RouteOperands{logits_.ptr(), bias, bias_alt, tokens.ids().ptr(), tokens.live().ptr(),
                             tokens.padding_active() ? tokens.padding_sources().ptr() : 0, ids_.ptr(), routing_.ptr(), rows_,
                             gate_in_front ? gate : 0};
    }
    uint64_t lp = logits_.ptr(), tp = tokens.ids().ptr(), vp = tokens.live().ptr(), ip = ids_.ptr(), wp = routing_.ptr();
    uint64_t b = bias, ba = bias_alt;
    const uint32_t blocks = (uint32_t)((rows_ + 15) / 16);
    uint64_t pad = (tokens.padding_active() && blocks == 1) ? tokens.padding_sources().ptr() : 0;
    int rows = (int)rows_, experts = g.experts, topk = g.topk, scoring = g.scoring;
    float scale = g.route_scale;
    long long alt = g.alt_token;
    void* args[] = {&lp, &b, &ba, &tp, &vp, &pad, &ip, &wp, &rows, &experts, &topk, &scoring, &scale, &alt};
    native_->launch("ca_route_topk", blocks, 1, 1024, 0, args, stream.raw());                                  // :380-395
    if (tokens.padding_active() && blocks > 1) {                                                               // :396-409
        uint64_t source = tokens.padding_sources().ptr();
        void* pargs[] = {&ip, &wp, &source, &rows, &topk};
        native_->launch("ca_route_padding_rows", (uint32_t)((rows_ * g.topk + 127) / 128), 1, 128, 0, pargs, stream.raw());
    }
    return std::nullopt;
}
void Router::census(const TokenRows& tokens, const Stream& stream) {                                          // src/route_census.rs:63-76
    const ca_geometry& g = native_->geometry();
    uint64_t ip = ids_.ptr(), vp = tokens.live().ptr(), cp = census_.ptr();
    int rows = (int)rows_, topk = g.topk, experts = g.experts;
    void* args[] = {&ip, &vp, &rows, &topk, &cp, &experts};
    native_->launch("ca_route_census", (uint32_t)((rows_ * g.topk + 255) / 256), 1, 256, 0, args, stream.raw());
}

// ---- Workspace ----------------------------------------------------------------------------------------------------------------
// The runtime contract's scratch layout (src/moe.rs:34-68 Contract / Node pointer offsets), computed instead of read from
// JSON: the same table tools/contracts writes into contracts/runtime-contract-m<rows>.json.
Workspace::Workspace(std::shared_ptr<const Native> native, size_t rows) : native_(std::move(native)), rows_(rows) {
    const ca_geometry& g = native_->geometry();
    ensure(rows >= 1, "MoE workspace rows");
    tile_m_ = rows <= 64 ? 16 : 128;
    const size_t pairs = rows * g.topk;
    max_tiles_ = (pairs + tile_m_ - 1) / tile_m_ - 1 + std::min<size_t>(g.experts, pairs);   // the reference contracts' capacity (runtime-contract.json max_phys_tiles)
    const size_t padded = max_tiles_ * tile_m_, H = g.hidden, I = g.intermediate, B = g.act_block;
    size_t at = 0;
    auto add = [&](const char* name, size_t bytes) { regions_[name] = View{at, bytes}; at += align256(bytes); };
    add("packed_a_storage_ptr", rows * H); add("scale_storage_ptr", rows * H / B);
    add("shared_a_storage_ptr", rows * H); add("shared_scale_storage_ptr", rows * H / B);
    add("intermediate_ptr", padded * I * 2); add("intermediate_codes_ptr", padded * I); add("intermediate_scales_ptr", padded * I / B);
    add("task_expert_ptr", max_tiles_ * 4); add("task_valid_rows_ptr", max_tiles_ * 4); add("expert_tile_base", (g.experts + 1) * 4);
    add("token_map_ptr", padded * 4); add("token_weights_ptr", padded * 4);
    add("scatter_ptr", pairs * H * 2);
    add("plan_scratch_ptr", ((pairs + 63) / 64 * g.experts + pairs) * 4);
    add("sync_ptr", 4096 + 8 * 512 * 4);           // arrival counters + the front-end's logit mailbox (8 rows x 512 experts words)
    scratch_ = Buffer<uint8_t>(at);
    scratch_.zero();                                                                                          // scratch_initializer "zero", src/moe.rs:440
    output_ = Buffer<uint16_t>(rows * H);
    output_.zero();
}
uint64_t Workspace::at(const std::string& name) const {
    auto it = regions_.find(name);
    if (it == regions_.end()) throw Error("unknown MoE runtime pointer role");                                 // src/moe.rs:1214-1216
    return scratch_.ptr() + it->second.offset;
}
size_t Workspace::bytes_of(const std::string& name) const {
    auto it = regions_.find(name);
    if (it == regions_.end()) throw Error("unknown MoE runtime pointer role");
    return it->second.bytes;
}
void Workspace::guard_stream(const Stream& stream) {                                                           // src/moe.rs:584-595
    ensure(!stream_set_ || stream_ == stream.raw(), "MoE workspace needs one ordered stream");
    stream_ = stream.raw(); stream_set_ = true;
}
void Workspace::pointers(const Expert& expert, uint64_t input, const Buffer<int32_t>& ids, const Buffer<float>& routing_weights, uint64_t* p) const {
    const char* scratch_names[] = {"packed_a_storage_ptr", "scale_storage_ptr", "shared_a_storage_ptr", "shared_scale_storage_ptr",
                                   "intermediate_ptr", "intermediate_codes_ptr", "intermediate_scales_ptr", "task_expert_ptr",
                                   "task_valid_rows_ptr", "expert_tile_base", "token_map_ptr", "token_weights_ptr"};
    p[0] = input; p[1] = ids.ptr(); p[2] = routing_weights.ptr();
    for (int i = 0; i < 12; ++i) p[3 + i] = at(scratch_names[i]);
    if (!emit_shared_input_) p[5] = p[6] = 0;
    if (!keep_intermediate_ && rows_ > 64) p[7] = 0;
    p[15] = expert.region("w13").first; p[16] = expert.region("s13").first; p[17] = expert.region("w2").first; p[18] = expert.region("s2").first;
    p[19] = at("scatter_ptr"); p[20] = at("plan_scratch_ptr");
}
std::optional<std::pair<uint64_t, size_t>> Workspace::run_live_for_ffn(const Expert& expert, uint64_t input, size_t input_len, const Buffer<int32_t>& ids,
                                                                       const Buffer<float>& routing_weights, size_t live, bool fuse_sum,
                                                                       const std::optional<RouteOperands>& route, const Stream& stream,
                                                                       const SharedOperands* shared) {
    const ca_geometry& g = native_->geometry();
    ensure(live <= rows_, "MoE live row domain");                                                             // src/moe.rs:1045
    guard_stream(stream);
    ensure(input_len == rows_ * (size_t)g.hidden, "BF16 MoE operand");                                         // :1057-1058
    ensure(expert.layout().experts == (size_t)g.experts && expert.layout().hidden == (size_t)g.hidden &&
               expert.layout().intermediate == (size_t)g.intermediate && ids.len() == rows_ * g.topk && routing_weights.len() == rows_ * g.topk,
           "MoE input shape mismatch");                                                                       // :1103-1114
    uint64_t p[40];
    pointers(expert, input, ids, routing_weights, p);
    int32_t scalars[8] = {(int32_t)rows_, (int32_t)rows_, (int32_t)(max_tiles_ * tile_m_), (int32_t)max_tiles_, (int32_t)tile_m_, 1, (int32_t)rows_, (int32_t)live};
    if (shared) {
        ensure(rows_ <= 64 && p[5] && p[6], "folded shared expert is for few-row owners");
        for (int i = 21; i < 29; ++i) p[i] = 0;
        if (route) {
            ensure(route->ids == p[1] && route->weights == p[2] && route->owner_rows == rows_ && route->logits && route->bias && route->live,
                   "fused routing domain");
            p[21] = route->logits; p[22] = route->bias; p[23] = route->bias_alt; p[24] = route->tokens; p[25] = route->live; p[26] = route->padding;
            p[27] = route->gate_w;
        }
        p[28] = at("sync_ptr");
        const uint64_t sh[9] = {shared->w13, shared->s13, shared->w2, shared->s2, shared->activation, shared->activation_codes,
                                shared->activation_scales, shared->up_tap, shared->output};
        for (int i = 0; i < 9; ++i) p[29 + i] = sh[i];
        p[38] = shared->routed_output; p[39] = shared->layer_output;
        native_->primitive(9, p, 40, scalars, 8, stream.raw(), "ffn.experts_with_shared");
        if (shared->layer_output) return std::nullopt;      // summed and added inside the entry
    } else if (route) {
        ensure(route->ids == p[1] && route->weights == p[2] && route->owner_rows == rows_ && route->logits && route->bias && route->live,
               "fused routing domain");                                                                       // :1266-1269
        p[21] = route->logits; p[22] = route->bias; p[23] = route->bias_alt; p[24] = route->tokens; p[25] = route->live; p[26] = route->padding;
        p[27] = route->gate_w; p[28] = at("sync_ptr");
        scalars[6] = (int32_t)route->owner_rows;
        native_->primitive(1, p, 29, scalars, 7, stream.raw(), "integration.tp_moe.dynamic (route front)");
    } else {
        native_->primitive(0, p, 21, scalars, 6, stream.raw(), "integration.tp_moe.dynamic");
    }
    if (fuse_sum) return std::make_pair(at("scatter_ptr"), live);                                              // :1005-1008
    const uint64_t sp[3] = {at("scatter_ptr"), output_.ptr(), 0};
    const int32_t ss[3] = {(int32_t)live, 0, 0};                                                              // active_m patched to the live rows, :1229
    native_->primitive(2, sp, 3, ss, 3, stream.raw(), "moe.w4a16.topk_sum");
    return std::nullopt;
}
void Workspace::run_live(const Expert& expert, uint64_t input, size_t input_len, const Buffer<int32_t>& ids, const Buffer<float>& routing_weights,
                         size_t live, const Stream& stream) {                                                 // src/moe.rs:1011-1043
    const ca_geometry& g = native_->geometry();
    ensure(live >= 1 && live <= rows_, "MoE live row domain");
    guard_stream(stream);
    ensure(input_len == rows_ * (size_t)g.hidden && ids.len() == rows_ * g.topk && routing_weights.len() == rows_ * g.topk, "MoE input shape mismatch");
    uint64_t p[21];
    pointers(expert, input, ids, routing_weights, p);
    // num_tokens patched to the live prefix (:1221-1237): the rows past it are outside the launch
    const int32_t scalars[6] = {(int32_t)live, (int32_t)rows_, (int32_t)(max_tiles_ * tile_m_), (int32_t)max_tiles_, (int32_t)tile_m_, 1};
    native_->primitive(0, p, 21, scalars, 6, stream.raw(), "integration.tp_moe.dynamic");
    const uint64_t sp[3] = {at("scatter_ptr"), output_.ptr(), 0};
    const int32_t ss[3] = {(int32_t)live, 0, 0};
    native_->primitive(2, sp, 3, ss, 3, stream.raw(), "moe.w4a16.topk_sum");
}
void Workspace::run_packed(const Expert& expert, uint64_t packed, size_t packed_len, const Buffer<int32_t>& ids, const Buffer<float>& routing_weights,
                           const Stream& stream) {                                                             // src/moe.rs:571-577
    const ca_geometry& g = native_->geometry();
    guard_stream(stream);
    ensure(g.act_block == 32 && packed && packed_len == rows_ * (size_t)g.hidden * 37 / 32, "packed MoE operand");
    ensure(ids.len() == rows_ * g.topk && routing_weights.len() == rows_ * g.topk, "MoE input shape mismatch");
    uint64_t p[21];
    pointers(expert, packed, ids, routing_weights, p);
    const int32_t scalars[6] = {(int32_t)rows_, (int32_t)rows_, (int32_t)(max_tiles_ * tile_m_), (int32_t)max_tiles_, (int32_t)tile_m_, 1};
    native_->primitive(10, p, 21, scalars, 6, stream.raw(), "integration.tp_moe.dynamic (dual_quant_rows_v1)");
    const uint64_t sp[3] = {at("scatter_ptr"), output_.ptr(), 0};
    const int32_t ss[3] = {(int32_t)rows_, 0, 0};
    native_->primitive(2, sp, 3, ss, 3, stream.raw(), "moe.w4a16.topk_sum");
}
void Workspace::run_phase(int entry, const Expert& expert, uint64_t input, const Buffer<int32_t>& ids, const Buffer<float>& routing_weights,
                          const Stream& stream) {
    ensure(entry == 6 || entry == 7 || entry == 8, "phase entry");
    uint64_t p[21];
    pointers(expert, input, ids, routing_weights, p);
    const int32_t scalars[6] = {(int32_t)rows_, (int32_t)rows_, (int32_t)(max_tiles_ * tile_m_), (int32_t)max_tiles_, (int32_t)tile_m_, 1};
    native_->primitive(entry, p, 21, scalars, 6, stream.raw(), "expert phase");
}

// ---- LayerFfn -----------------------------------------------------------------------------------------------------------------
LayerFfn::LayerFfn(std::shared_ptr<const Native> native, std::shared_ptr<Weights> weights, Prepared layout, size_t rows, Options options)
    : native_(native), router_(native, weights, rows), expert_(weights, layout),
      shared_up_(rows * 2 * native->geometry().shared_intermediate), activation_(rows * native->geometry().shared_intermediate),
      shared_down_(rows * native->geometry().hidden), output_(rows * native->geometry().hidden),
      activation_codes_(rows * native->geometry().shared_intermediate),
      activation_scales_(rows * native->geometry().shared_intermediate / native->geometry().act_block), rows_(rows), options_(options) {
    const ca_geometry& g = native->geometry();
    ensure(layout.experts == (size_t)g.experts, "FFN namespace/expert geometry");                              // src/ffn.rs:617-620
    shared_w13_ = prepare_shared(*native, *weights, "ffn.shared_experts.w13", 2 * g.shared_intermediate, g.hidden);
    shared_w2_ = prepare_shared(*native, *weights, "ffn.shared_experts.w2", g.hidden, g.shared_intermediate);
    output_.zero();
    if (options_.overlap) {                                                                                    // :700-706 SharedBranch
        compute_units_ = native->compute_units();
        branch_stream_ = std::make_unique<Stream>();
        input_ready_ = std::make_unique<Event>();
        output_ready_ = std::make_unique<Event>();
    }
}
void LayerFfn::run_shared(const Workspace& workspace, uint64_t input, const Stream& stream) {                  // :1053-1124 run_shared / run_shared_quantized_input + finish_shared
    if (input) {   // Linear::run: this branch quantizes the BF16 input itself (src/fp8_linear.rs:782-806)
        const uint64_t q[5] = {input, 0, 0, workspace.at("shared_a_storage_ptr"), workspace.at("shared_scale_storage_ptr")};
        const int32_t qs[3] = {(int32_t)rows_, native_->geometry().hidden, 0};
        native_->primitive(3, q, 5, qs, 3, stream.raw(), "gemm.mxfp8_quant_cute");
    }
    run_shared_quantized(workspace.at("shared_a_storage_ptr"), workspace.at("shared_scale_storage_ptr"), stream);
}
void LayerFfn::run_shared_quantized(uint64_t codes, uint64_t scales, const Stream& stream) {
    ensure(codes && scales, "prequantized normalized shared input requires both operands");
    // many rows: the BF16 activation and the projections before it are taps (the second projection reads the codes)
    const bool taps = keep_intermediate_ || rows_ <= 64;
    const uint64_t p[11] = {codes, scales, shared_w13_.values, shared_w13_.scales, shared_w2_.values, shared_w2_.scales, taps ? activation_.ptr() : 0,
                            activation_codes_.ptr(), activation_scales_.ptr(), taps ? shared_up_.ptr() : 0, shared_down_.ptr()};
    const int32_t s[1] = {(int32_t)rows_};
    native_->primitive(5, p, 11, s, 1, stream.raw(), "ffn.shared_expert");
}
void LayerFfn::add_shared(const Workspace& workspace, const Stream& stream) {                                  // :1066-1084
    native_->ffn_add((int)rows_, workspace.output().ptr(), shared_down_.ptr(), output_.ptr(), stream.raw());
}
void LayerFfn::run_quantized_input(Workspace& workspace, uint64_t input, size_t input_len, const QuantizedInput* quantized, const TokenRows& tokens,
                                   const Stream& stream) {                                                      // :974-1047
    const ca_geometry& g = native_->geometry();
    ensure(workspace.rows() == rows_, "MoE workspace context mismatch");
    const bool fused = options_.route_front && rows_ * g.topk <= 1024;                                          // :988-990
    // Dual-stream schedule (:1007-1010, :1028-1036): the shared branch forks before routing, quantizes the input itself
    // and joins before the sum.  Without the branch the front-end emits the shared-flavour codes beside the routed ones.
    const bool fold = options_.fold_shared && rows_ <= 64 && !quantized;      // given codes: the shared expert runs from them, beside the routed launches
    const bool branch = branch_stream_ && !fold;
    workspace.emit_shared_input(!branch && !quantized);
    if (fold) {
        const SharedOperands shared{shared_w13_.values, shared_w13_.scales, shared_w2_.values, shared_w2_.scales, activation_.ptr(),
                                    activation_codes_.ptr(), activation_scales_.ptr(), shared_up_.ptr(), shared_down_.ptr(),
                                    options_.sum_shared ? workspace.output().ptr() : 0, options_.sum_shared ? output_.ptr() : 0};
        const std::optional<RouteOperands> route = router_.run_routed(input, input_len, tokens, fused, stream, options_.gate_front);
        const auto deferred = workspace.run_live_for_ffn(expert_, input, input_len, router_.ids(), router_.routing(), tokens.active_rows(),
                                                         options_.sum_shared, route, stream, &shared);
        if (options_.sum_shared) return;                    // the entry summed and added
        if (deferred) sum_shared(workspace, deferred->second, stream);
        else add_shared(workspace, stream);
        return;
    }
    if (branch) {
        input_ready_->record(stream.raw());
        input_ready_->wait(branch_stream_->raw());
        // The branch's first projection runs beside the router's launches (gate product, top-k, plan, quantizer: about 60 us +
        // 8 ns a row, on few CUs) and takes about 20 ns a row with one workgroup on every CU, which leaves the router no CU until
        // it ends.  Up to 6,144 rows a quarter of the CUs stays free for the router (the projection gets a third longer, the
        // router runs under it); beyond, the projection outlasts the router by more than that costs.
        const int reserve = rows_ > 64 && rows_ <= 6144 ? compute_units_ / 32 * 8 : 0;
        if (reserve) native_->shared_reserve(reserve);
        if (quantized) run_shared_quantized(quantized->codes, quantized->scales, *branch_stream_);              // :1058-1064
        else run_shared(workspace, input, *branch_stream_);
        if (reserve) native_->shared_reserve(0);
        output_ready_->record(branch_stream_->raw());
    }
    const std::optional<RouteOperands> route = router_.run_routed(input, input_len, tokens, fused, stream, options_.gate_front);
    const auto deferred = workspace.run_live_for_ffn(expert_, input, input_len, router_.ids(), router_.routing(), tokens.active_rows(),
                                                     options_.sum_shared, route, stream);
    if (branch) output_ready_->wait(stream.raw());
    else if (quantized) run_shared_quantized(quantized->codes, quantized->scales, stream);
    else run_shared(workspace, 0, stream);
    if (deferred) sum_shared(workspace, deferred->second, stream);
    else add_shared(workspace, stream);
}
void LayerFfn::enable_row_transport() {                                                                        // src/ffn.rs:789-822
    const ca_geometry& g = native_->geometry();
    ensure(g.act_block == 32 && rows_ % 128 == 0 && !row_transport_active(), "packed MoE transport requires the wide sequential profile");
    packed_ = Buffer<uint8_t>(rows_ * (size_t)g.hidden * 37 / 32);
    decoded_codes_ = Buffer<uint8_t>(rows_ * (size_t)g.hidden);
    decoded_scales_ = Buffer<uint8_t>(rows_ * (size_t)g.hidden / 32);
    local_live_ = Buffer<int32_t>(1);
}
void LayerFfn::run_row_transport(Workspace& workspace, uint64_t input, size_t input_len, const TokenRows& tokens, const Stream& stream) {   // :827-878
    const ca_geometry& g = native_->geometry();
    ensure(row_transport_active() && tokens.rows() == rows_ && input && input_len == rows_ * (size_t)g.hidden && workspace.rows() == rows_,
           "packed MoE transport input geometry/context");
    // one rank: its share is every row, its live count the batch's
    native_->codec_local_live(tokens.live().ptr(), local_live_.ptr(), (int)rows_, 0, stream.raw());
    router_.run(input, input_len, tokens, stream);
    native_->codec_pack_bf16(input, packed_.ptr(), (int)rows_, g.hidden, stream.raw());
    // (all-gather of packed rows, ids and routing weights over the ranks goes here)
    native_->codec_decode(packed_.ptr(), decoded_codes_.ptr(), decoded_scales_.ptr(), 0, (int)rows_, g.hidden, stream.raw());
    if (branch_stream_) {                                                                                      // :566-584 run_packed_and_shared
        input_ready_->record(stream.raw());
        workspace.run_packed(expert_, packed_.ptr(), packed_.len(), router_.ids(), router_.routing(), stream);
        input_ready_->wait(branch_stream_->raw());
        run_shared_quantized(decoded_codes_.ptr(), decoded_scales_.ptr(), *branch_stream_);
        output_ready_->record(branch_stream_->raw());
        output_ready_->wait(stream.raw());
    } else {
        workspace.run_packed(expert_, packed_.ptr(), packed_.len(), router_.ids(), router_.routing(), stream);
        run_shared_quantized(decoded_codes_.ptr(), decoded_scales_.ptr(), stream);
    }
    add_shared(workspace, stream);
}
void LayerFfn::sum_shared(const Workspace& workspace, size_t live_rows, const Stream& stream) {               // :1037-1046 ca_ffn_sum_shared
    const ca_geometry& g = native_->geometry();
    uint64_t routes = workspace.at("scatter_ptr"), shared = shared_down_.ptr(), routed = workspace.output().ptr(), output = output_.ptr();
    int n = (int)(rows_ * g.hidden), live = (int)live_rows, topk = g.topk, hidden = g.hidden;
    void* args[] = {&routes, &shared, &routed, &output, &n, &live, &topk, &hidden};
    native_->launch("ca_ffn_sum_shared", (uint32_t)((n / 8 + 255) / 256), 1, 256, 0, args, stream.raw());
}

// ---- Paired ------------------------------------------------------------------------------------------------------------------
Paired::Paired(std::shared_ptr<const Native> native, size_t owner_rows)
    : native_(native), rows_(owner_rows), workspace_(native, 2 * owner_rows), shared_scratch_{Workspace(native, owner_rows), Workspace(native, owner_rows)},
      shared_scratch_pool_(native, 2 * owner_rows),
      input_(2 * owner_rows * native->geometry().hidden), ids_(2 * owner_rows * native->geometry().topk),
      routing_(2 * owner_rows * native->geometry().topk) {
    ensure(owner_rows >= 1 && 2 * owner_rows <= 64, "paired owners pool into one few-row launch");
    input_.zero(); ids_.zero(); routing_.zero();                                                               // src/paired_ffn.rs:21-23
}
void Paired::run(LayerFfn& a, uint64_t a_input, const TokenRows& a_tokens, LayerFfn& b, uint64_t b_input, const TokenRows& b_tokens,
                 const Stream& stream, LayerFfn* pool) {                                                       // :65-120
    const ca_geometry& g = native_->geometry();
    const size_t a_live = a_tokens.active_rows(), b_live = b_tokens.active_rows(), H = g.hidden, K = g.topk;
    ensure(a.rows() == rows_ && b.rows() == rows_ && a_live >= 1 && a_live <= rows_ && b_live >= 1 && b_live <= rows_ && a_input && b_input &&
               a.expert().same_layer_weights(b.expert()),
           "paired FFN needs two live prefixes of one canonical layer");                                       // :70-75
    a.router().run(a_input, rows_ * H, a_tokens, stream);                                                      // :79-80: each owner routes privately
    b.router().run(b_input, rows_ * H, b_tokens, stream);
    struct Owner { size_t offset, live; LayerFfn* ffn; uint64_t input; };
    const Owner owners[2] = {{0, a_live, &a, a_input}, {a_live, b_live, &b, b_input}};
    for (const Owner& o : owners) {                                                                            // :84-90: six capturable copies on the one stream
        check(hipMemcpyAsync((void*)(input_.ptr() + o.offset * H * 2), (const void*)o.input, o.live * H * 2, hipMemcpyDeviceToDevice, stream.raw()), "pool rows");
        check(hipMemcpyAsync((void*)(ids_.ptr() + o.offset * K * 4), (const void*)o.ffn->router().ids().ptr(), o.live * K * 4, hipMemcpyDeviceToDevice, stream.raw()), "pool ids");
        check(hipMemcpyAsync((void*)(routing_.ptr() + o.offset * K * 4), (const void*)o.ffn->router().routing().ptr(), o.live * K * 4, hipMemcpyDeviceToDevice, stream.raw()), "pool weights");
    }
    workspace_.run_live(a.expert(), input_.ptr(), input_.len(), ids_, routing_, a_live + b_live, stream);      // :91
    if (pool != nullptr) {                                                                                     // :91-102: the shared expert once, over the pooled rows
        ensure(pool->rows() == 2 * rows_ && a.expert().same_layer_weights(pool->expert()), "pooled shared expert needs a layer of both owners' rows");
        pool->run_shared(shared_scratch_pool_, input_.ptr(), stream);
        for (const Owner& o : owners)
            native_->ffn_add((int)o.live, workspace_.output().ptr() + o.offset * H * 2, pool->shared_down().ptr() + o.offset * H * 2, o.ffn->output().ptr(),
                             stream.raw());
        return;
    }
    for (int i = 0; i < 2; ++i) {                                                                              // :108-115: every owner's shared expert on its own rows
        const Owner& o = owners[i];
        o.ffn->run_shared(shared_scratch_[i], o.input, stream);
        native_->ffn_add((int)o.live, workspace_.output().ptr() + o.offset * H * 2, o.ffn->shared_down().ptr(), o.ffn->output().ptr(), stream.raw());   // :116-121
    }
}

}  // namespace tf
