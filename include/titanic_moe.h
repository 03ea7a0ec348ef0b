/*
 * titanic_moe.h -- C ABI of libtitanic_moe_hip.so, the MI355X (gfx950) implementation of Titanic Flash's MoE FFN layer.
 *
 * The library is the drop-in for the native objects the reference's Rust FFN operators bind:
 *   libcanada_ffn.so              (src/ffn.rs:42-84:        ca_ffn_abi, ca_router_logits, ca_shared_swiglu, ca_ffn_add)
 *   libcanada_moe_primitives.so   (src/primitives.rs:45-182: ca_primitives_abi / open / close / launch / launch2)
 *   core.cubin / shared.cubin     (kernels resolved by name and launched through src/cuda.rs Function::launch)
 * Conventions are the reference's (runtime/kernels/moe-runtime-m6-cache-ca-v1/bridge.cc): 0 = success, negative =
 * argument validation (-1 null / range, -2 arity, -3 unknown index, -4 unsupported geometry), positive = hipError_t.
 * No entry point allocates, frees or synchronizes; every launch goes to the stream passed in (a hipStream_t as void*),
 * so calls can be captured into a HIP graph.  All pointers are device pointers unless stated otherwise.
 *
 * Shapes are not compiled in: ca_ffn_configure() sets the process geometry used by the fixed-signature entry points,
 * and ca_primitives_open() snapshots it into the context it returns; ca_primitives_open_geometry() and the *_in functions
 * keep a geometry per context, so that layers of different geometries live side by side in one process.
 */
#ifndef TITANIC_MOE_H
#define TITANIC_MOE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct ca_geometry {
    int32_t hidden;               /* H: multiple of 512 up to 4,096, or of 1,024 up to 8,192 */
    int32_t experts;              /* E <= 512 */
    int32_t topk;                 /* K <= 8 */
    int32_t intermediate;         /* routed expert intermediate I, multiple of 512 up to 4,096 */
    int32_t shared_intermediate;  /* shared expert intermediate, multiple of 512 up to 4,096 */
    int32_t scoring;              /* 0 sigmoid, 1 sqrt(softplus) (reference: 1, src/ffn.rs:249) */
    float route_scale;            /* routed_scaling_factor (reference: 1.5, src/ffn.rs:250) */
    int32_t act_block;            /* activation quantization block: 32 (reference) or 128 */
    int32_t shared_bn, shared_bk; /* shared-expert weight scale block (reference: 32 x 32, src/blockscaled.rs:161-171) */
    int64_t alt_token;            /* token id that selects the alternative bias (reference: 129264), -1 none */
    float swiglu_limit;           /* 10 (src/ffn.rs:66) */
} ca_geometry;

/* ---- libcanada_ffn.so surface (runtime/kernels/ffn-native-v1/ffn.cu:259-276) ----------------------------------- */
int ca_ffn_abi(void);                                   /* ffn.cu:259: returns 1 */
int ca_ffn_configure(const ca_geometry* geometry);      /* additive: replaces the reference's compiled-in 5120/384/576 */
int ca_ffn_geometry(ca_geometry* out);                  /* additive: reads the process geometry back */
/* ffn.cu:260-265.  logits[rows][E] (f32) = x[rows][H] (bf16) . w[E][H]^T (bf16), rows 1..16. */
int ca_router_logits(int rows, const void* x, const void* w, void* out, void* stream);
/* ffn.cu:266-271.  out[rows][Is] (bf16) = clipped SwiGLU of in[rows][gate | up] (bf16), rows 1..65536. */
int ca_shared_swiglu(int rows, const void* input, void* output, void* stream);
/* ffn.cu:272-276.  out = bf16(f32(routed) + f32(shared)) over rows x H, rows 1..65536. */
int ca_ffn_add(int rows, const void* routed, const void* shared, void* out, void* stream);
/* Additive: the gate product for any row count (rows > 16 use the matrix-core kernel, whose summation order differs). */
int ca_router_logits_wide(int rows, const void* x, const void* w, void* out, void* stream);
/* Additive: the same four functions with the geometry of a context of ca_primitives_open_geometry instead of the process
 * geometry, for hosts that keep layers of several geometries in one process (the reference's 384-expert target and
 * 128-expert drafter, src/layer_id.rs:39-47).  -1 for a null context. */
int ca_router_logits_in(void* context, int rows, const void* x, const void* w, void* out, void* stream);
int ca_router_logits_wide_in(void* context, int rows, const void* x, const void* w, void* out, void* stream);
int ca_shared_swiglu_in(void* context, int rows, const void* input, void* output, void* stream);
int ca_ffn_add_in(void* context, int rows, const void* routed, const void* shared, void* out, void* stream);

/* ---- the decoder's FFN boundary either side of the layer ------------------------------------------------------- */
/* Upstream, the reference's producer `hc_combine_norm_quant` (runtime/kernels/mhc-norm-quant-v1/mhc-norm-quant.py:15-44 and its
 * layout8 twin; loaded at src/mhc.rs:606-614, launched at :981-990): the row's `streams` residual streams x [rows][streams][H]
 * (BF16) are collapsed with the predecessor's pre-coefficients pre [rows][streams] (FP32; null: all 1) by ordered FP32 fused
 * multiply-adds and rounded to BF16; normed = bf16((value / sqrt(mean(value^2) + 1e-20)) * weight); then the shared-flavour
 * MXFP8 quantizer in the context's activation block width (amax floored at 1e-4): codes_min [rows][H] (the reference's Q),
 * scales_min [rows][H / block] (SR), and the same scale bytes at the reference's matrix-instruction offsets in mma_scales (SM:
 * ceil(rows / 128) * ceil(H / 128) * 512 bytes; 32-wide blocks only; bytes of absent rows are not written).  normed and the
 * (codes_min, scales_min) pair feed Layer::run_quantized_input (src/ffn.rs:974-975, 1053-1065; src/decoder.rs:1654-1656).
 * Additive: codes / scales, the routed experts' flavour of the same row (zero block -> scale byte 0).  Each of the two pairs and
 * mma_scales may be null.  The reference's approximate reciprocal root is replaced by a correctly rounded one.  H <= 8,192. */
int ca_hc_combine_norm_quant(void* context, int rows, int streams, const void* x, const float* pre, const void* weight, void* normed,
                             void* codes_min, void* scales_min, void* mma_scales, void* codes, void* scales, void* stream);
/* The single-stream case of the producer with a caller's eps (a plain RMS norm with a BF16 boundary), both flavours. */
int ca_ffn_norm_quant(void* context, int rows, const void* x, const void* weight, float eps, void* normed, void* codes, void* scales,
                      void* codes_min, void* scales_min, void* stream);
/* Downstream, the reference's `hc_post_tiles` (runtime/kernels/mhc-post-tiles-v1/mhc-post-tiles.py:11-27; launched at
 * src/mhc.rs:1223-1234 behind the layer, src/decoder.rs:1497-1543 `finish_ffn`): the layer's output mixed into the four
 * residual streams, y[row][c][h] = bf16(fma(C[3][c], r3, fma(C[2][c], r2, fma(C[1][c], r1, fma(post[c], a, C[0][c] * r0))))) with
 * a = sublayer [rows][H], r_s = residual [rows][4][H] (BF16), post [rows][4], C = comb [rows][4][4] (FP32).  y may alias
 * residual (a thread reads its columns of all four streams before it writes them). */
int ca_hc_post(void* context, int rows, const void* sublayer, const void* residual, const float* post, const float* comb, void* y, void* stream);
/* Additive: ca_ffn_sum_shared (src/ffn.rs:1041-1044) with ca_hc_post behind it in one pass: routed (rows < live) = ordered
 * FP32 sum of the top-k route outputs rounded to BF16; ffn = bf16(routed + shared) (flush-to-zero add), written to ffn_out
 * unless null; y = the post step of ffn. */
int ca_ffn_sum_hc_post(void* context, int rows, int live, const void* routes, const void* shared, const void* residual, const float* post,
                       const float* comb, void* routed, void* ffn_out, void* y, void* stream);
/* Additive: the single-stream form of the same pass (one residual stream, coefficients 1): routed and ffn as above,
 * residual_out = bf16(f32(ffn) + f32(residual)) (may alias residual). */
int ca_ffn_sum_residual(void* context, int rows, int live, const void* routes, const void* shared, const void* residual, void* routed,
                        void* ffn_out, void* residual_out, void* stream);

/* ---- kernels the reference resolves by name from a code module (src/cuda.rs:199-226 Module::function + launch) -- */
/* Launches the `extern "C" __global__` kernel `name` with the reference's launch tuple ([grid;3], [block;3], dynamic
 * shared bytes, stream, argument pointers).  -3 for an unknown name.  The same kernels are in titanic_moe_gfx950.hsaco
 * for hosts that load code objects with hipModuleLoadData / hipModuleGetFunction. */
int ca_kernel_launch(const char* name, const uint32_t grid[3], const uint32_t block[3], uint32_t shared_bytes, void** args,
                     void* stream);
int ca_kernel_count(void);
const char* ca_kernel_name(int index);

/* kernels/moe_nibble_layout_probe.cu:17-21 */
int ca_moe_nibble_permute(void* data, uint64_t bytes, int inverse, void* stream);

/* ---- libcanada_moe_input_codec.so surface: the wire row "dual_quant_rows_v1" of the sequence-parallel prefill ------
 * (runtime/kernels/moe-input-codec-coalesced-v1/moe-dual-quant-codec-fast.cu).  A row of k values is k routed E4M3 codes,
 * k / 32 UE8M0 scale bytes and k / 32 32-bit correction words: k * 37 / 32 bytes.  All pointers are device pointers, every
 * call only enqueues on `stream`; 0, -1 for an argument out of range (the reference's own checks), or a hipError_t. */
/* :81-87.  routed[rows][k], scales[rows][k/32] (routed quantizer), shared[rows][k] (shared quantizer's codes) -> packed. */
int ca_encode(const uint8_t* routed, const uint8_t* scales, const uint8_t* shared, uint8_t* packed, int rows, int k, void* stream);
/* :88-94.  packed -> shared[rows][k], row_scales[rows][k/32] and the same scale bytes at the reference's matrix-instruction
 * offsets in mma_scales (rows * k / 32 bytes; additive: may be null).  rows % 128 == 0. */
int ca_decode(const uint8_t* packed, uint8_t* shared, uint8_t* row_scales, uint8_t* mma_scales, int rows, int k, void* stream);
/* :99-105.  *local = min(rows, max(0, *global - rank * rows)), rank 0..3. */
int ca_local_live(const int* global, int* local, int rows, int rank, void* stream);
/* :138-144.  input[rows][k] (bf16) -> packed: both quantizers and the encoder in one pass. */
int ca_pack_bf16(const void* input, uint8_t* packed, int rows, int k, void* stream);

/* ---- operator ABI (src/primitives.rs:45-60, 91-182; bridge.cc) ------------------------------------------------- */
int32_t ca_primitives_abi(void);                /* returns 1 */
void* ca_primitives_open(int32_t* status);      /* host handle; snapshots the process geometry and the device's CU count */
/* Additive: a handle with a geometry of its own; the process geometry is neither read nor written.  -1 null, -4 unsupported. */
void* ca_primitives_open_geometry(const ca_geometry* geometry, int32_t* status);
int32_t ca_primitives_geometry(void* context, ca_geometry* out);      /* additive: the handle's geometry */
void ca_primitives_close(void* context);
/* Entries, pointer and scalar lists: titanic-flash-41_amd/contracts/bindings.json (same schema as the reference's). */
int32_t ca_primitives_launch(void* context, int32_t index, const uint64_t* pointers, size_t pointer_count,
                             const int32_t* scalars, size_t scalar_count, void* stream);
/* words = pointers followed by scalars widened to 64 bits (src/primitives.rs:153-182). */
int32_t ca_primitives_launch2(void* context, int32_t index, const uint64_t* words, size_t word_count, void* stream);
int32_t ca_primitives_entries(void);            /* additive: number of entries */
/* additive: scratch bytes entry `index` needs for `rows` token rows (the role "scratch" of the runtime contract). */
int64_t ca_primitives_scratch_bytes(void* context, int32_t index, int32_t rows);

/* No counterpart in the reference (its per-node timings come from CUDA events around whole graph launches,
 * src/moe.rs:1261-1300): a profiling aid.  With five hipEvent_t in `events`, every later launch of entries 0, 1 and 9 on this
 * context records them on the launch stream: [0] before the first kernel, [1] after the front-end, [2] after FC1 + SwiGLU,
 * [3] after FC2, [4] after the ordered sum (entry 9 with outputs only).  With seven, [5] and [6] also take the start and the
 * completion of the few-row FC1 + SwiGLU kernel itself (without the gap to its neighbours that [1] .. [2] includes).
 * count 0 turns it off.  Not for use while the stream is being captured.  0, or -1 for a null context / event or a count
 * other than 0, 5 or 7. */
int32_t ca_primitives_marks(void* context, void* const* events, size_t count);

/* No counterpart in the reference: for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid it).  The routed experts of entry 0 (`integration.tp_moe.dynamic`: plan, token
 * quantization, FC1 + SwiGLU, FC2 x routing weight) for at most 64 rows, with every scratch region of that entry (token
 * codes, plan tables, intermediate) in a static device array of the library instead of a caller's arena; the caller passes only
 * inputs (token rows BF16 [rows][H], top-k ids and weights [rows][K], the prepared expert weights and scales) and the output
 * (route outputs BF16 [rows][K][H], what entry 0 writes to its `scatter_ptr`).  Same kernels and bits as entry 0.  The array
 * (ca_moe_dynamic_static_capacity() bytes, 16 MiB) exists once a device and keeps the last call's contents; calls that
 * overlap on one device race.  Nothing is allocated, freed or synchronized.  0; -1 null / rows < 1 / a context opened on
 * another device than the current one; -5 more than 64 rows or a geometry whose regions exceed the array; -4; or a hipError_t. */
int32_t ca_moe_dynamic_static(void* context, const void* input, const int32_t* topk_ids, const float* topk_weights, const void* w13,
                              const void* s13, const void* w2, const void* s2, void* route_output, int32_t rows, void* stream);
int64_t ca_moe_dynamic_static_capacity(void);

/* No counterpart in the reference (its front-end has no waits inside a launch).  The front-end launch of entries 1 and 9 hands
 * data from some of its workgroups to others; every such wait is bounded by `limit` polls (default 262,144), after which the
 * waiter does the work it waited for itself and marks the `sync_ptr` region: later launches then take that path at once
 * (same results) until the host has zeroed the region again.  limit 0: no hand-off is ever waited for.  0, or -1 for a null
 * context or a negative limit. */
int32_t ca_primitives_spin_limit(void* context, int32_t limit);

/* No counterpart in the reference.  Entry 5 (`ffn.shared_expert`) above 64 rows runs persistent workgroups, one a CU, which leave
 * no room for other launches while they run.  A host that runs the router's small launches beside it on another stream (the
 * dual-stream schedule of src/ffn.rs:1000-1040) sets `cus` (a multiple of 8, at most half the part's CUs; 0, the default: none)
 * and the entry's first projection then leaves that many CUs without a workgroup.  The setting holds for the launches
 * enqueued after it.  0, or -1 for a null context or a count outside that range. */
int32_t ca_primitives_shared_reserve(void* context, int32_t cus);

#ifdef __cplusplus
}
#endif
#endif
