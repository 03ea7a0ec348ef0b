// Flat C interface of the host mirror for the python tests and the benchmark (ctypes): one handle per layer instance.
// Every function returns 0 on success and -1 on failure with the message in the caller's buffer.
#include "ffn_host.hpp"
#include "checkpoint.hpp"
#include <cstdio>
#include <cstring>

namespace {
struct Handle {
    std::shared_ptr<tf::Native> native;
    std::shared_ptr<tf::Weights> weights;
    tf::Prepared prepared;
    std::unique_ptr<tf::LayerFfn> layer;
    std::unique_ptr<tf::Workspace> workspace;
    std::unique_ptr<tf::TokenRows> tokens;
    std::unique_ptr<tf::Stream> stream;
    std::vector<std::unique_ptr<tf::Graph>> graphs;
    tf::ScaleCodeReport scale_code;
    size_t rows = 0;
    tf::LayerFfn::Options options;
    // a second owner of the same layer and the pool both owners run through (src/paired_ffn.rs)
    std::unique_ptr<tf::LayerFfn> layer_b;
    std::unique_ptr<tf::LayerFfn> layer_pool;       // 2 x rows: the shared expert over both owners' pooled rows
    std::unique_ptr<tf::TokenRows> tokens_b;
    std::unique_ptr<tf::Paired> paired;
};
template <class F>
int guarded(char* error, size_t error_len, F&& body) {
    try { body(); return 0; }
    catch (const std::exception& e) { if (error && error_len) std::snprintf(error, error_len, "%s", e.what()); return -1; }
}
}  // namespace

extern "C" {

namespace {
void build_layer(Handle* h, const char* kernel_library, const ca_geometry* geometry, int rows, const tf::Weights::Host& src, bool on_device,
                 int overlap, int sum_shared, int route_front, int code_scales, int fold_shared, int gate_front) {
    // expert widths that are not multiples of 512 (the reference's 2,304 / 576) run zero-padded
    const ca_geometry run = tf::padded_geometry(*geometry);
    tf::Weights::Host padded = src;
    if (run.intermediate != geometry->intermediate) padded.source_intermediate = (size_t)geometry->intermediate;
    if (run.shared_intermediate != geometry->shared_intermediate) padded.source_shared_intermediate = (size_t)geometry->shared_intermediate;
    h->native = std::make_shared<tf::Native>(kernel_library, run);
    h->weights = on_device ? std::make_shared<tf::Weights>(run, padded, true) : std::make_shared<tf::Weights>(run, padded);
    h->prepared = tf::prepare_layer(*h->native, *h->weights, 0);
    if (code_scales) h->scale_code = tf::code_layer_scales(*h->native, *h->weights, h->prepared);
    tf::LayerFfn::Options options;
    options.overlap = overlap != 0; options.sum_shared = sum_shared != 0; options.route_front = route_front != 0; options.fold_shared = fold_shared != 0; options.gate_front = gate_front != 0;
    h->options = options;
    h->layer = std::make_unique<tf::LayerFfn>(h->native, h->weights, h->prepared, (size_t)rows, options);
    h->workspace = std::make_unique<tf::Workspace>(h->native, (size_t)rows);
    std::vector<int64_t> ids((size_t)rows, 0);
    h->tokens = std::make_unique<tf::TokenRows>(ids.data(), (size_t)rows, (size_t)rows);
    h->stream = std::make_unique<tf::Stream>();
    h->rows = (size_t)rows;
}
tf::Weights::Host host_view(const tf::LayerOperandsHost& o) {
    return tf::Weights::Host{o.gate_w.data(), o.bias.data(), o.bias_alt.data(), o.w13.data(), o.s13.data(), o.w2.data(), o.s2.data(),
                             o.sh_w13.data(), o.sh_s13.data(), o.sh_w2.data(), o.sh_s2.data()};
}
}  // namespace

// operands: gate_w, bias, bias_alt, w13, s13, w2, s2, sh_w13, sh_s13, sh_w2, sh_s2 (canonical checkpoint layout).
void* tfh_layer_create(const char* kernel_library, const ca_geometry* geometry, int rows, const void* const* operands, int operands_on_device,
                       int overlap, int sum_shared, int route_front, int code_scales, int fold_shared, int gate_front, char* error, size_t error_len) {
    Handle* h = new Handle;
    const int status = guarded(error, error_len, [&] {
        tf::Weights::Host src{(const uint16_t*)operands[0], (const float*)operands[1], (const float*)operands[2], (const uint8_t*)operands[3],
                              (const uint8_t*)operands[4], (const uint8_t*)operands[5], (const uint8_t*)operands[6], (const uint8_t*)operands[7],
                              (const uint8_t*)operands[8], (const uint8_t*)operands[9], (const uint8_t*)operands[10]};
        build_layer(h, kernel_library, geometry, rows, src, operands_on_device != 0, overlap, sum_shared, route_front, code_scales, fold_shared, gate_front);
    });
    if (status != 0) { delete h; return nullptr; }
    return h;
}
// The same layer with its operands read from a safetensors checkpoint directory (index + shards), layer prefix e.g. "layers.3".
void* tfh_layer_create_from_checkpoint(const char* kernel_library, const ca_geometry* geometry, int rows, const char* root, const char* prefix,
                                       int overlap, int sum_shared, int route_front, int code_scales, int fold_shared, int gate_front, char* error,
                                       size_t error_len) {
    Handle* h = new Handle;
    const int status = guarded(error, error_len, [&] {
        const tf::Checkpoint checkpoint = tf::Checkpoint::scan(root);
        const tf::LayerOperandsHost operands = tf::load_ffn_layer(checkpoint, prefix, *geometry);
        build_layer(h, kernel_library, geometry, rows, host_view(operands), false, overlap, sum_shared, route_front, code_scales, fold_shared, gate_front);
    });
    if (status != 0) { delete h; return nullptr; }
    return h;
}
// Checkpoint scan and operand assembly alone (no device): fills the caller's eleven host buffers (sizes in bytes, checked) in
// the order of tfh_layer_create's operands; counts[0] = tensors in the checkpoint, counts[1] = shards.
int tfh_checkpoint_layer(const char* root, const char* prefix, const ca_geometry* geometry, void* const* out, const size_t* sizes, size_t* counts,
                         char* error, size_t error_len) {
    return guarded(error, error_len, [&] {
        const tf::Checkpoint checkpoint = tf::Checkpoint::scan(root);
        const tf::LayerOperandsHost o = tf::load_ffn_layer(checkpoint, prefix, *geometry);
        const void* src[11] = {o.gate_w.data(), o.bias.data(), o.bias_alt.data(), o.w13.data(), o.s13.data(), o.w2.data(), o.s2.data(),
                               o.sh_w13.data(), o.sh_s13.data(), o.sh_w2.data(), o.sh_s2.data()};
        const size_t bytes[11] = {o.gate_w.size() * 2, o.bias.size() * 4, o.bias_alt.size() * 4, o.w13.size(), o.s13.size(), o.w2.size(), o.s2.size(),
                                  o.sh_w13.size(), o.sh_s13.size(), o.sh_w2.size(), o.sh_s2.size()};
        for (int i = 0; i < 11; ++i) {
            tf::ensure(sizes[i] == bytes[i], "operand buffer size");
            std::memcpy(out[i], src[i], bytes[i]);
        }
        counts[0] = checkpoint.tensors(); counts[1] = checkpoint.shards();
    });
}
// The loader's tensor contract for one layer as text, a tensor a line: "<name> <dtype> <d0>,<d1>".  Returns the length the
// text needs (with its terminator); fills `out` when `out_len` holds it.
long long tfh_checkpoint_contract(const char* prefix, const ca_geometry* geometry, char* out, size_t out_len) {
    std::string text;
    for (const tf::TensorContract& t : tf::ffn_layer_contract(prefix, *geometry)) {
        text += t.name + " " + t.dtype + " ";
        for (size_t i = 0; i < t.shape.size(); ++i) text += (i ? "," : "") + std::to_string(t.shape[i]);
        text += "\n";
    }
    if (out && out_len > text.size()) std::memcpy(out, text.c_str(), text.size() + 1);
    return (long long)text.size() + 1;
}
void tfh_layer_destroy(void* handle) { delete (Handle*)handle; }
// The geometry the layer runs with (the caller's, with the expert widths padded to multiples of 512): the widths of the taps.
void tfh_layer_geometry(void* handle, ca_geometry* out) { *out = ((Handle*)handle)->native->geometry(); }
// Test hooks of the front-end's in-launch hand-offs: the bound of its waits, and the host's reset of the `sync` region.
int tfh_layer_spin_limit(void* handle, int limit, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] { h->native->spin_limit(limit); });
}
int tfh_layer_zero_sync(void* handle, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        h->stream->synchronize();
        tf::check(hipMemset((void*)h->workspace->at("sync_ptr"), 0, h->workspace->bytes_of("sync_ptr")), "zero sync region");
    });
}
// Many rows: drop (0) or keep (1) the BF16 taps of the routed intermediate and of the shared expert (its projections before
// the activation, its activation): both second projections read the FP8 codes.
void tfh_layer_keep_intermediate(void* handle, int on) {
    Handle* h = (Handle*)handle;
    h->workspace->keep_intermediate(on != 0);
    h->layer->keep_intermediate(on != 0);
    if (h->layer_b) h->layer_b->keep_intermediate(on != 0);
    if (h->layer_pool) h->layer_pool->keep_intermediate(on != 0);
}

int tfh_layer_set_tokens(void* handle, const int64_t* ids, int live, const int32_t* padding, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        h->tokens->update(ids, h->rows, (size_t)live);
        if (padding) h->tokens->set_padding_sources(padding, h->rows);
    });
}
// One eager pass over the device-resident BF16 input [rows][hidden]; returns after the stream has drained.
int tfh_layer_run(void* handle, uint64_t input, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        h->layer->run(*h->workspace, input, h->rows * (size_t)h->native->geometry().hidden, *h->tokens, *h->stream);
        h->stream->synchronize();
    });
}
// One eager pass with the shared expert fed from pre-quantized input (LayerFfn::run_quantized_input): `codes` / `scales` are
// device addresses of the rows' E4M3 codes and UE8M0 scales in the shared expert's quantizer flavour.
int tfh_layer_run_quantized(void* handle, uint64_t input, uint64_t codes, uint64_t scales, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        const tf::LayerFfn::QuantizedInput q{codes, scales};
        h->layer->run_quantized_input(*h->workspace, input, h->rows * (size_t)h->native->geometry().hidden, &q, *h->tokens, *h->stream);
        h->stream->synchronize();
    });
}
// One eager pass through the row transport of the sequence-parallel prefill on one rank (LayerFfn::run_row_transport): the rows
// are packed into wire rows "dual_quant_rows_v1", the routed experts run from the packed rows, the shared expert from the codes
// decoded out of them.  `packed_out` (may be 0): device address that receives a copy of the packed rows (rows x hidden x 37 / 32).
int tfh_layer_run_row_transport(void* handle, uint64_t input, uint64_t packed_out, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        if (!h->layer->row_transport_active()) h->layer->enable_row_transport();
        h->layer->run_row_transport(*h->workspace, input, h->rows * (size_t)h->native->geometry().hidden, *h->tokens, *h->stream);
        if (packed_out)
            tf::check(hipMemcpyAsync((void*)packed_out, (const void*)h->layer->packed_rows().ptr(), h->layer->packed_rows().len(), hipMemcpyDeviceToDevice,
                                     h->stream->raw()), "copy packed rows");
        h->stream->synchronize();
    });
}
// Captures one pass over each of `count` inputs, in order, into one graph (the reference captures its whole forward, forty
// layers' passes, into one graph and replays it: src/probe.rs:1527-1542, src/cuda.rs:2068-2153); returns the graph's index.
int tfh_layer_capture(void* handle, const uint64_t* inputs, int count, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    int index = -1;
    const int status = guarded(error, error_len, [&] {
        tf::ensure(count >= 1, "capture needs an input");
        auto graph = std::make_unique<tf::Graph>();
        graph->capture(*h->stream, [&] {
            for (int i = 0; i < count; ++i)
                h->layer->run(*h->workspace, inputs[i], h->rows * (size_t)h->native->geometry().hidden, *h->tokens, *h->stream);
        });
        h->graphs.push_back(std::move(graph));
        index = (int)h->graphs.size() - 1;
    });
    return status == 0 ? index : -1;
}
// Replays graphs[order[i % n]] for `warmup` untimed and `steps` timed launches; milliseconds of the timed launches.
int tfh_layer_time(void* handle, const int* order, int n, int warmup, int steps, float* milliseconds, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        tf::ensure(n > 0 && steps > 0, "timing arguments");
        for (int i = 0; i < n; ++i) tf::ensure(order[i] >= 0 && (size_t)order[i] < h->graphs.size(), "graph index");
        tf::Event begin(true), end(true);
        for (int i = 0; i < warmup; ++i) h->graphs[order[i % n]]->launch(*h->stream);
        h->stream->synchronize();
        begin.record(h->stream->raw());
        for (int i = 0; i < steps; ++i) h->graphs[order[(warmup + i) % n]]->launch(*h->stream);
        end.record(h->stream->raw());
        end.synchronize();
        *milliseconds = end.elapsed_since(begin);
    });
}
// Times `iterations` back-to-back launches of one expert phase (6: FC1 + SwiGLU, 7: FC2, 5: shared expert) with events on
// the launch stream, using the routing the last pass left in the workspace.
int tfh_layer_time_phase(void* handle, int entry, uint64_t input, int iterations, float* milliseconds, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        tf::Event begin(true), end(true);
        auto once = [&] {
            if (entry == 5) h->layer->run_shared(*h->workspace, input, *h->stream);
            else h->workspace->run_phase(entry, h->layer->expert(), input, h->layer->router().ids(), h->layer->router().routing(), *h->stream);
        };
        once();
        h->stream->synchronize();
        begin.record(h->stream->raw());
        for (int i = 0; i < iterations; ++i) once();
        end.record(h->stream->raw());
        end.synchronize();
        *milliseconds = end.elapsed_since(begin);
    });
}
// One eager pass with HIP events on the launch stream around each part (no overlap, separate top-k): milliseconds of
// [0] gate product + top-k, [1] front-end, [2] FC1 + SwiGLU, [3] FC2, [4] shared expert, [5] sum + addition, [6] whole pass.
int tfh_layer_profile_step(void* handle, uint64_t input, float* milliseconds, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        std::vector<std::unique_ptr<tf::Event>> e;
        for (int i = 0; i < 7; ++i) e.push_back(std::make_unique<tf::Event>(true));
        tf::LayerFfn& l = *h->layer;
        tf::Workspace& w = *h->workspace;
        const tf::Stream& s = *h->stream;
        const ca_geometry& g = h->native->geometry();
        w.emit_shared_input(true);
        e[0]->record(s.raw());
        l.router().run(input, h->rows * (size_t)g.hidden, *h->tokens, s);
        e[1]->record(s.raw());
        w.run_phase(8, l.expert(), input, l.router().ids(), l.router().routing(), s);
        e[2]->record(s.raw());
        w.run_phase(6, l.expert(), input, l.router().ids(), l.router().routing(), s);
        e[3]->record(s.raw());
        w.run_phase(7, l.expert(), input, l.router().ids(), l.router().routing(), s);
        e[4]->record(s.raw());
        l.run_shared(w, 0, s);
        e[5]->record(s.raw());
        l.sum_shared(w, h->tokens->active_rows(), s);
        e[6]->record(s.raw());
        e[6]->synchronize();
        for (int i = 0; i < 6; ++i) milliseconds[i] = e[i + 1]->elapsed_since(*e[i]);
        milliseconds[6] = e[6]->elapsed_since(*e[0]);
    });
}
// `passes` eager passes of the layer's own schedule over the `count` inputs in turn, all enqueued before the first wait, with
// the library's marks around every launch of the dynamic entry: mean milliseconds of [0] front-end (gate product, top-k, plan,
// quantizers), [1] FC1 + SwiGLU, [2] FC2, [3] ordered sum + shared addition, [4] first mark to last.  Needs the schedule that
// keeps the shared expert inside the routed launches (otherwise there is no sum mark).
// `exact` != 0: the FC1 + SwiGLU kernel is launched with a pair of events that take its own start and completion
// (milliseconds[5]); that launch path costs a few microseconds more per pass, so the launch-to-launch intervals of such a
// run are not the schedule's.
int tfh_layer_profile_marks(void* handle, const uint64_t* inputs, int count, int passes, int exact, float* milliseconds, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        tf::ensure(count >= 1 && passes >= 1, "profile needs inputs and passes");
        if (h->rows > 64) exact = 0;          // the kernel's own events exist for the few-row FC1 launch only
        std::vector<std::unique_ptr<tf::Event>> events;
        for (int i = 0; i < 7 * passes; ++i) events.push_back(std::make_unique<tf::Event>(true));
        const size_t n = h->rows * (size_t)h->native->geometry().hidden;
        try {
            for (int pass = 0; pass < passes; ++pass) {
                hipEvent_t raw[7];
                for (int i = 0; i < 7; ++i) raw[i] = events[7 * pass + i]->raw();
                h->native->marks(raw, exact ? 7 : 5);
                h->layer->run(*h->workspace, inputs[pass % count], n, *h->tokens, *h->stream);
            }
        } catch (...) { h->native->marks(nullptr); throw; }
        h->native->marks(nullptr);
        h->stream->synchronize();
        // [0 .. 3]: front-end, FC1 + SwiGLU, FC2, sum (launch to launch); [4]: first mark to last; [5]: the FC1 + SwiGLU kernel alone
        double sum[6] = {0, 0, 0, 0, 0, 0};
        for (int pass = 0; pass < passes; ++pass) {
            for (int i = 0; i < 4; ++i) sum[i] += events[7 * pass + i + 1]->elapsed_since(*events[7 * pass + i]);
            sum[4] += events[7 * pass + 4]->elapsed_since(*events[7 * pass]);
            if (exact) sum[5] += events[7 * pass + 6]->elapsed_since(*events[7 * pass + 5]);
        }
        for (int i = 0; i < 6; ++i) milliseconds[i] = (float)(sum[i] / passes);
    });
}
// Paired owners: a second LayerFfn over the same prepared layer and the pooled workspace.  Runs owner A (the handle's layer,
// input `a_input`, token ids / live count as given) and owner B through Paired::run and copies both owners' layer outputs
// ([rows][hidden] BF16 each) to the host.  `pool_shared` != 0: the shared expert runs once over the pooled rows.
int tfh_layer_pair_run(void* handle, uint64_t a_input, const int64_t* a_ids, int a_live, uint64_t b_input, const int64_t* b_ids, int b_live,
                       int pool_shared, uint16_t* a_output, uint16_t* b_output, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        if (!h->paired) {
            h->layer_b = std::make_unique<tf::LayerFfn>(h->native, h->weights, h->prepared, h->rows, h->options);
            std::vector<int64_t> ids(h->rows, 0);
            h->tokens_b = std::make_unique<tf::TokenRows>(ids.data(), h->rows, h->rows);
            h->paired = std::make_unique<tf::Paired>(h->native, h->rows);
        }
        h->tokens->update(a_ids, h->rows, (size_t)a_live);
        h->tokens_b->update(b_ids, h->rows, (size_t)b_live);
        if (pool_shared && !h->layer_pool) h->layer_pool = std::make_unique<tf::LayerFfn>(h->native, h->weights, h->prepared, 2 * h->rows, h->options);
        h->paired->run(*h->layer, a_input, *h->tokens, *h->layer_b, b_input, *h->tokens_b, *h->stream, pool_shared ? h->layer_pool.get() : nullptr);
        h->stream->synchronize();
        h->layer->output().download(a_output, h->layer->output().len());
        h->layer_b->output().download(b_output, h->layer_b->output().len());
    });
}
// Copies a named tap to the host.  Returns the tap's size in bytes (or -1); copies min(bytes, size).
long long tfh_layer_tap(void* handle, const char* name, void* out, size_t bytes, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    long long size = -1;
    guarded(error, error_len, [&] {
        const std::string n(name);
        uint64_t p = 0;
        auto buf = [&](uint64_t ptr, size_t b) { p = ptr; size = (long long)b; };
        tf::LayerFfn& l = *h->layer;
        tf::Workspace& w = *h->workspace;
        if (n == "logits") buf(l.router().logits().ptr(), l.router().logits().bytes());
        else if (n == "ids") buf(l.router().ids().ptr(), l.router().ids().bytes());
        else if (n == "weights") buf(l.router().routing().ptr(), l.router().routing().bytes());
        else if (n == "shared_up") buf(l.shared_up().ptr(), l.shared_up().bytes());
        else if (n == "shared_act") buf(l.activation().ptr(), l.activation().bytes());
        else if (n == "shared_aq") buf(l.activation_codes().ptr(), l.activation_codes().bytes());
        else if (n == "shared_as") buf(l.activation_scales().ptr(), l.activation_scales().bytes());
        else if (n == "shared_down") buf(l.shared_down().ptr(), l.shared_down().bytes());
        else if (n == "out") buf(l.output().ptr(), l.output().bytes());
        else if (n == "routed") buf(w.output().ptr(), w.output().bytes());
        else {
            static const std::map<std::string, std::string> alias = {
                {"xq", "packed_a_storage_ptr"}, {"xs", "scale_storage_ptr"}, {"xq_min", "shared_a_storage_ptr"}, {"xs_min", "shared_scale_storage_ptr"},
                {"h", "intermediate_ptr"}, {"hq", "intermediate_codes_ptr"}, {"hs", "intermediate_scales_ptr"}, {"task_expert", "task_expert_ptr"},
                {"task_valid", "task_valid_rows_ptr"}, {"tile_base", "expert_tile_base"}, {"token_map", "token_map_ptr"},
                {"token_weights", "token_weights_ptr"}, {"route_out", "scatter_ptr"}, {"sync", "sync_ptr"}};
            auto it = alias.find(n);
            tf::ensure(it != alias.end(), "unknown tap");
            buf(w.at(it->second), w.bytes_of(it->second));
        }
        h->stream->synchronize();
        if (out && bytes) tf::check(hipMemcpy(out, (const void*)p, std::min<size_t>(bytes, (size_t)size), hipMemcpyDeviceToHost), "tap download");
    });
    return size;
}
int tfh_layer_census(void* handle, uint32_t* counts, char* error, size_t error_len) {
    Handle* h = (Handle*)handle;
    return guarded(error, error_len, [&] {
        h->layer->router().census(*h->tokens, *h->stream);
        h->stream->synchronize();
        const std::vector<uint32_t> c = h->layer->router().census_counts();
        std::memcpy(counts, c.data(), c.size() * 4);
    });
}
// info[0] tile_m, [1] max_tiles, [2] scratch bytes, [3] atlas bytes, [4] resident expert bytes, [5] scale-code bytes, [6] raw rows, [7] coded rows
void tfh_layer_info(void* handle, long long* info) {
    Handle* h = (Handle*)handle;
    info[0] = (long long)h->workspace->tile_m(); info[1] = (long long)h->workspace->max_tiles(); info[2] = (long long)h->workspace->scratch_bytes();
    info[3] = (long long)h->weights->bytes(); info[4] = (long long)h->prepared.resident_bytes; info[5] = (long long)h->scale_code.bytes;
    info[6] = (long long)h->scale_code.raw_rows; info[7] = (long long)h->scale_code.rows;
}

}  // extern "C"
