// Host mirror of the reference's Rust FFN operators above the C ABI of include/titanic_moe.h.
//
//   reference (Rust)                                   here (C++)
//   src/ffn.rs           Native / TokenRows / Router   tf::Native / tf::TokenRows / tf::Router
//   src/ffn.rs           LayerFfn                      tf::LayerFfn   (new_rows, run, output, taps)
//   src/moe.rs           Expert / Workspace            tf::Expert / tf::Workspace (scratch arena, launch plan)
//   src/expert_packing.rs Prepared / prepare_layer     tf::Prepared / tf::prepare_layer, tf::code_layer_scales
//   src/blockscaled.rs   Matrix::prepare_shared_named  tf::SharedMatrix
//   src/weights.rs       device atlas of named views   tf::Weights
//
// The classes keep the reference's names, argument meaning, call order and failure behaviour ("ensure" -> tf::Error with
// the reference's message).  They call the kernels only through the C ABI, loaded with dlopen as the Rust side loads
// its libraries, and own every device buffer; the kernel library never allocates.
#pragma once
#include "../../include/titanic_moe.h"
#include "hip_rt.hpp"
#include <map>
#include <memory>
#include <optional>
#include <string>

namespace tf {

// SHA-256 of a file as lower-case hexadecimal (empty: unreadable): what the build's manifest pins the kernel library with.
std::string library_sha256(const std::string& path);

// ---- loaded kernel library (src/ffn.rs:46-85 Native::open, src/primitives.rs:66-151 Primitives::open) --------------
class Native {
public:
    Native(const std::string& library, const ca_geometry& geometry);
    ~Native();
    Native(const Native&) = delete;
    Native& operator=(const Native&) = delete;
    const ca_geometry& geometry() const { return g_; }
    void router_logits(int rows, uint64_t x, uint64_t w, uint64_t out, hipStream_t s) const;
    void router_logits_wide(int rows, uint64_t x, uint64_t w, uint64_t out, hipStream_t s) const;
    void shared_swiglu(int rows, uint64_t in, uint64_t out, hipStream_t s) const;
    void ffn_add(int rows, uint64_t routed, uint64_t shared, uint64_t out, hipStream_t s) const;
    // Module::function(name)?.launch(grid, block, shared, stream, args)  (src/cuda.rs:199-226)
    void launch(const char* name, uint32_t grid_x, uint32_t grid_y, uint32_t block, uint32_t shared, void** args, hipStream_t s) const;
    // Primitives::launch (src/primitives.rs:122-151)
    void primitive(int index, const uint64_t* pointers, size_t np, const int32_t* scalars, size_t ns, hipStream_t s, const char* what) const;
    int64_t scratch_bytes(int index, int rows) const;
    // five events recorded around the launches of the dynamic entries (null: off)
    void marks(hipEvent_t* events, size_t count = 5) const;      // 5: between the launches; 7: + the FC1 kernel's own begin / end
    // polls a wait inside the front-end launch may take before the waiter does the work itself (0: no hand-off is waited for)
    void spin_limit(int limit) const;
    // CUs the many-row shared expert's first projection leaves free (ca_primitives_shared_reserve); holds for later launches
    void shared_reserve(int cus) const;
    int compute_units() const;          // of the current device
    // the wire row "dual_quant_rows_v1" (src/ffn.rs:805-811 RowTransport's functions)
    void codec_encode(uint64_t routed, uint64_t scales, uint64_t shared, uint64_t packed, int rows, int k, hipStream_t s) const;
    void codec_decode(uint64_t packed, uint64_t shared, uint64_t row_scales, uint64_t mma_scales, int rows, int k, hipStream_t s) const;
    void codec_local_live(uint64_t global, uint64_t local, int rows, int rank, hipStream_t s) const;
    void codec_pack_bf16(uint64_t input, uint64_t packed, int rows, int k, hipStream_t s) const;
private:
    void* lib_ = nullptr;
    void* ctx_ = nullptr;
    ca_geometry g_;
    int (*router_logits_)(void*, int, const void*, const void*, void*, void*) = nullptr;
    int (*router_logits_wide_)(void*, int, const void*, const void*, void*, void*) = nullptr;
    int (*shared_swiglu_)(void*, int, const void*, void*, void*) = nullptr;
    int (*ffn_add_)(void*, int, const void*, const void*, void*, void*) = nullptr;
    int32_t (*spin_limit_)(void*, int32_t) = nullptr;
    int32_t (*shared_reserve_)(void*, int32_t) = nullptr;
    int (*kernel_launch_)(const char*, const uint32_t*, const uint32_t*, uint32_t, void**, void*) = nullptr;
    void (*close_)(void*) = nullptr;
    int32_t (*launch_)(void*, int32_t, const uint64_t*, size_t, const int32_t*, size_t, void*) = nullptr;
    int64_t (*scratch_bytes_)(void*, int32_t, int32_t) = nullptr;
    int32_t (*marks_)(void*, void* const*, size_t) = nullptr;
    int (*encode_)(const uint8_t*, const uint8_t*, const uint8_t*, uint8_t*, int, int, void*) = nullptr;
    int (*decode_)(const uint8_t*, uint8_t*, uint8_t*, uint8_t*, int, int, void*) = nullptr;
    int (*local_live_)(const int*, int*, int, int, void*) = nullptr;
    int (*pack_bf16_)(const void*, uint8_t*, int, int, void*) = nullptr;
};

// The kernels take expert widths that are multiples of 512; the reference's are 2,304 (576 a tensor-parallel rank,
// src/expert_packing.rs:64-66).  Returns `g` with both intermediate widths rounded up to the next multiple of 512: a layer
// built for that geometry from operands of the narrower widths (Weights::Host::source_*) computes the same outputs, since the
// added up / gate rows are zero (their activation columns are exactly zero, as are their codes, and whole quantization
// blocks of them do not touch a real block's scale) and the added down-projection columns multiply those zeros.
ca_geometry padded_geometry(const ca_geometry& g);

// ---- device atlas (src/weights.rs:276-417: contiguous expert groups, 256-byte aligned views) --------------------------
struct View { size_t offset = 0, bytes = 0; };
class Weights {
public:
    // Canonical checkpoint-layout operands on the host; experts in numeric order, up (w3) before gate (w1).
    struct Host {
        const uint16_t* gate_w; const float* bias; const float* bias_alt;
        const uint8_t* w13; const uint8_t* s13; const uint8_t* w2; const uint8_t* s2;
        const uint8_t* sh_w13; const uint8_t* sh_s13; const uint8_t* sh_w2; const uint8_t* sh_s2;
        // Expert widths of the operands above when they are narrower than the geometry's (0: the same): the atlas is then
        // filled with zero weight rows (w13) and zero weight columns (w2) up to the geometry's widths, which changes no
        // result (see padded_geometry).
        size_t source_intermediate = 0, source_shared_intermediate = 0;
    };
    Weights(const ca_geometry& g, const Host& host);
    // Same, from device-resident canonical operands (copied device to device into the atlas).
    Weights(const ca_geometry& g, const Host& device, bool from_device);
    const View& view(const std::string& name) const;
    uint64_t ptr(const std::string& name) const { return atlas_.ptr() + view(name).offset; }
    uint64_t pointer_at(size_t offset, size_t bytes) const;
    bool expert_ready() const { return expert_ready_; }
    void finish_expert_layer() { expert_ready_ = true; }
    void install_expert_scale_code1(Buffer<uint32_t>&& code) { scale_code1_ = std::move(code); }
    const Buffer<uint32_t>* expert_scale_code1() const { return scale_code1_.len() ? &scale_code1_ : nullptr; }
    size_t bytes() const { return atlas_.bytes(); }
private:
    void layout(const ca_geometry& g);
    void fill(const ca_geometry& g, const Host& src, hipMemcpyKind kind);
    Buffer<uint8_t> atlas_;
    std::map<std::string, View> views_;
    bool expert_ready_ = false;
    Buffer<uint32_t> scale_code1_;
};

// ---- load-time expert preparation (src/expert_packing.rs) -------------------------------------------------------------
struct Prepared {
    size_t layer = 0, experts = 0, hidden = 0, intermediate = 0;
    size_t w13_offset = 0, w2_offset = 0, s13_offset = 0, s2_offset = 0, resident_bytes = 0, temporary_bytes = 0;
};
Prepared prepare_layer(const Native& native, Weights& weights, size_t layer);                       // :20-207
struct ScaleCodeReport { size_t bytes = 0, raw_rows = 0, rows = 0; };
ScaleCodeReport code_layer_scales(const Native& native, Weights& weights, const Prepared& p);       // :212-259

class Expert {                                                                                      // src/moe.rs:100-156
public:
    Expert(std::shared_ptr<Weights> weights, Prepared layout);
    std::pair<uint64_t, size_t> region(const std::string& role) const;
    const Prepared& layout() const { return layout_; }
    const Weights& weights() const { return *weights_; }
    // same_layer_weights (src/moe.rs:150-155): both views name the same prepared layer of the same atlas
    bool same_layer_weights(const Expert& other) const { return weights_ == other.weights_ && layout_.layer == other.layout_.layer; }
private:
    std::shared_ptr<Weights> weights_;
    Prepared layout_;
};

// Shared-expert matrices re-laid for the matrix instruction (src/blockscaled.rs:149-191 prepare_shared_named / prepare).
struct SharedMatrix { uint64_t values = 0, scales = 0; size_t n = 0, k = 0; };
SharedMatrix prepare_shared(const Native& native, Weights& weights, const std::string& name, size_t n, size_t k);

// ---- per-step metadata (src/ffn.rs:88-172) ----------------------------------------------------------------------------
class TokenRows {
public:
    TokenRows(const int64_t* ids, size_t rows, size_t live);
    void update(const int64_t* ids, size_t rows, size_t live);
    void set_padding_sources(const int32_t* sources, size_t rows);
    const Buffer<int64_t>& ids() const { return ids_; }
    const Buffer<int32_t>& live() const { return live_; }
    const Buffer<int32_t>& padding_sources() const { return padding_sources_; }
    bool padding_active() const { return padding_active_; }
    size_t rows() const { return rows_; }
    size_t active_rows() const { return active_rows_; }
private:
    Buffer<int64_t> ids_;
    Buffer<int32_t> live_, padding_sources_;
    size_t rows_, active_rows_ = 0;
    bool padding_active_ = false;
};

// Operands a router hands to the experts' front-end when its top-k runs there (src/moe.rs:181-200 RouteOperands).
// gate_w != 0: the gate product is left to the front-end too (owners of at most 64 rows).
struct RouteOperands { uint64_t logits, bias, bias_alt, tokens, live, padding, ids, weights; size_t owner_rows; uint64_t gate_w; };
// Operands of the shared expert when it is folded into the routed experts' launches (entry "ffn.experts_with_shared"):
// prepared w13 / scales / w2 / scales, activation (BF16), its codes and scales, the up-projection tap, the output.
// layer_output != 0: the entry also runs the ordered sum and the shared addition into routed_output / layer_output.
struct SharedOperands { uint64_t w13, s13, w2, s2, activation, activation_codes, activation_scales, up_tap, output, routed_output, layer_output; };

class Router {                                                                                      // src/ffn.rs:173-426
public:
    Router(std::shared_ptr<const Native> native, std::shared_ptr<Weights> weights, size_t rows);
    void run(uint64_t input, size_t input_len, const TokenRows& tokens, const Stream& stream) { run_routed(input, input_len, tokens, false, stream); }
    // fused: the gate product only; returns the operands for the front-end that will route.
    std::optional<RouteOperands> run_routed(uint64_t input, size_t input_len, const TokenRows& tokens, bool fused, const Stream& stream,
                                            bool gate_front = false);
    const Buffer<float>& logits() const { return logits_; }
    const Buffer<int32_t>& ids() const { return ids_; }
    const Buffer<float>& routing() const { return routing_; }
    void census(const TokenRows& tokens, const Stream& stream);
    std::vector<uint32_t> census_counts() const { return census_.download(); }
private:
    std::shared_ptr<const Native> native_;
    std::shared_ptr<Weights> weights_;
    size_t rows_;
    Buffer<float> logits_, routing_;
    Buffer<int32_t> ids_;
    Buffer<uint32_t> census_;
    hipStream_t stream_ = nullptr;
    bool stream_set_ = false;
};

// ---- routed-expert workspace (src/moe.rs:235-1289) --------------------------------------------------------------------
class Workspace {
public:
    Workspace(std::shared_ptr<const Native> native, size_t rows);
    const Buffer<uint16_t>& output() const { return output_; }
    size_t rows() const { return rows_; }
    size_t tile_m() const { return tile_m_; }
    size_t max_tiles() const { return max_tiles_; }
    // run_live_for_ffn (:997-1009): fuse_sum leaves the route outputs for the caller's fused sum and returns their address
    // and row count; otherwise the topk_sum node runs and output() holds the reduced rows.
    std::optional<std::pair<uint64_t, size_t>> run_live_for_ffn(const Expert& expert, uint64_t input, size_t input_len, const Buffer<int32_t>& ids,
                                                               const Buffer<float>& routing_weights, size_t live, bool fuse_sum,
                                                               const std::optional<RouteOperands>& route, const Stream& stream,
                                                               const SharedOperands* shared = nullptr);
    void run(const Expert& expert, uint64_t input, size_t input_len, const Buffer<int32_t>& ids, const Buffer<float>& routing_weights,
             const Stream& stream) { run_live_for_ffn(expert, input, input_len, ids, routing_weights, rows_, false, std::nullopt, stream); }
    // run_live (:1011-1043): only the first `live` rows are launched (ids / weights given); output() holds their reduced rows.
    void run_live(const Expert& expert, uint64_t input, size_t input_len, const Buffer<int32_t>& ids, const Buffer<float>& routing_weights,
                  size_t live, const Stream& stream);
    // run_packed (src/moe.rs:571-577): the routed experts from wire rows "dual_quant_rows_v1" (rows x hidden x 37 / 32 bytes,
    // 32-wide activation blocks) instead of BF16 rows; every row is launched.
    void run_packed(const Expert& expert, uint64_t packed, size_t packed_len, const Buffer<int32_t>& ids, const Buffer<float>& routing_weights,
                    const Stream& stream);
    // Phase nodes alone (for per-kernel timing): 8 = front-end (plan + quantize), 6 = FC1 + SwiGLU, 7 = FC2.
    void run_phase(int entry, const Expert& expert, uint64_t input, const Buffer<int32_t>& ids, const Buffer<float>& routing_weights, const Stream& stream);
    // scratch regions by role name (the runtime contract's pointer table)
    uint64_t at(const std::string& name) const;
    size_t bytes_of(const std::string& name) const;
    size_t scratch_bytes() const { return scratch_.bytes(); }
    void emit_shared_input(bool on) { emit_shared_input_ = on; }
    // many rows: whether FC1 also stores the BF16 intermediate (a tap: FC2 reads the codes).  Few rows always keep it.
    void keep_intermediate(bool on) { keep_intermediate_ = on; }
private:
    bool emit_shared_input_ = true, keep_intermediate_ = true;
    void pointers(const Expert& expert, uint64_t input, const Buffer<int32_t>& ids, const Buffer<float>& routing_weights, uint64_t* p) const;
    void guard_stream(const Stream& stream);
    std::shared_ptr<const Native> native_;
    size_t rows_, tile_m_, max_tiles_;
    Buffer<uint8_t> scratch_;
    Buffer<uint16_t> output_;
    std::map<std::string, View> regions_;
    hipStream_t stream_ = nullptr;
    bool stream_set_ = false;
};

// ---- the layer (src/ffn.rs:427-1165) ------------------------------------------------------------------------------------
class LayerFfn {
public:
    struct Options {
        bool overlap = true;        // FFN_OVERLAP: shared expert on an auxiliary stream beside the routed experts (:518-522)
        bool sum_shared = true;     // FFN_SUM_SHARED: fused route sum + shared addition (:1037-1046)
        bool route_front = true;    // MOE_ROUTE_FRONT: the router's top-k inside the experts' front-end (:986-990)
        bool gate_front = true;     // the gate product inside the front-end launch as well (owners of at most 64 rows)
        bool fold_shared = true;    // few rows: the shared expert's weights stream inside the routed experts' two launches
                                    // (one queue, no cross-stream join); takes precedence over `overlap`
    };
    LayerFfn(std::shared_ptr<const Native> native, std::shared_ptr<Weights> weights, Prepared layout, size_t rows, Options options);
    void run(Workspace& workspace, uint64_t input, size_t input_len, const TokenRows& tokens, const Stream& stream) {
        run_quantized_input(workspace, input, input_len, nullptr, tokens, stream);                             // src/ffn.rs:965-973
    }
    // run_quantized_input (:974-1047): `quantized` (may be null) = E4M3 codes and UE8M0 scales of the same rows in the shared
    // expert's quantizer flavour (amax floored at 1e-4), produced upstream with the normalized input; the shared expert then
    // consumes them instead of quantizing the BF16 rows again.
    struct QuantizedInput { uint64_t codes, scales; };
    void run_quantized_input(Workspace& workspace, uint64_t input, size_t input_len, const QuantizedInput* quantized, const TokenRows& tokens,
                             const Stream& stream);
    const Buffer<uint16_t>& output() const { return output_; }
    Router& router() { return router_; }
    const Buffer<uint16_t>& shared_up() const { return shared_up_; }
    const Buffer<uint16_t>& activation() const { return activation_; }
    const Buffer<uint16_t>& shared_down() const { return shared_down_; }
    const Buffer<uint8_t>& activation_codes() const { return activation_codes_; }
    const Buffer<uint8_t>& activation_scales() const { return activation_scales_; }
    const Expert& expert() const { return expert_; }
    const Native& native() const { return *native_; }
    size_t rows() const { return rows_; }
    // input != 0: quantize it first (the branch's own quantizer); 0: use the codes the front-end left in the workspace.
    void run_shared(const Workspace& workspace, uint64_t input, const Stream& stream);
    // the shared expert from given codes / scales (Linear::run_quantized, src/fp8_linear.rs:792-806)
    void run_shared_quantized(uint64_t codes, uint64_t scales, const Stream& stream);
    void sum_shared(const Workspace& workspace, size_t live_rows, const Stream& stream);
    // Row transport of the sequence-parallel prefill on one rank (src/ffn.rs:789-878): the rows are routed, packed into wire rows
    // by the fused producer, (gathered: with one rank the rows are already all here), the shared quantizer's codes are decoded
    // from them, the routed experts run from the packed rows and the shared expert from the decoded codes.
    // many rows: whether the shared expert also stores its BF16 taps (projections before the activation, the activation); the
    // second projection reads the FP8 codes.  Few rows always keep them (there the BF16 activation is the hand-over).
    void keep_intermediate(bool on) { keep_intermediate_ = on; }
    void enable_row_transport();
    bool row_transport_active() const { return packed_.len() != 0; }
    void run_row_transport(Workspace& workspace, uint64_t input, size_t input_len, const TokenRows& tokens, const Stream& stream);
    const Buffer<uint8_t>& packed_rows() const { return packed_; }
private:
    void add_shared(const Workspace& workspace, const Stream& stream);
    Buffer<uint8_t> packed_, decoded_codes_, decoded_scales_;
    Buffer<int32_t> local_live_;
    std::shared_ptr<const Native> native_;
    Router router_;
    Expert expert_;
    SharedMatrix shared_w13_, shared_w2_;
    Buffer<uint16_t> shared_up_, activation_, shared_down_, output_;
    Buffer<uint8_t> activation_codes_, activation_scales_;
    size_t rows_;
    Options options_;
    bool keep_intermediate_ = true;
    int compute_units_ = 0;
    std::unique_ptr<Stream> branch_stream_;
    std::unique_ptr<Event> input_ready_, output_ready_;
};

// ---- two owners pooled into one routed-experts launch (src/paired_ffn.rs:5-120) ---------------------------------------------
// Each owner routes privately; the live prefixes of both owners' rows, ids and routing weights are concatenated (device
// copies on the one ordered stream, capturable), one launch runs the pooled rows, every owner's shared expert runs on its own
// rows, and the routed sums are split back by the two shared additions.  No padding row of A becomes a live row of B.
class Paired {
public:
    Paired(std::shared_ptr<const Native> native, size_t owner_rows);
    // `pool` (may be null): a LayerFfn of the same layer for 2 x owner_rows rows.  With it the shared expert runs once over the
    // pooled rows (its weights stream once for both owners; the reference pools the owners' shared up-projection,
    // src/paired_ffn.rs:91-102, src/fp8_paired.rs:15-60) instead of once per owner; a row's result is the same bits either way.
    void run(LayerFfn& a, uint64_t a_input, const TokenRows& a_tokens, LayerFfn& b, uint64_t b_input, const TokenRows& b_tokens,
             const Stream& stream, LayerFfn* pool = nullptr);
    const Workspace& workspace() const { return workspace_; }
    const Buffer<int32_t>& ids() const { return ids_; }
private:
    std::shared_ptr<const Native> native_;
    size_t rows_;
    Workspace workspace_;
    Workspace shared_scratch_[2];      // the owners' shared-branch quantizer scratch
    Workspace shared_scratch_pool_;    // the same for the pooled rows
    Buffer<uint16_t> input_;
    Buffer<int32_t> ids_;
    Buffer<float> routing_;
};

}  // namespace tf
