// C ABI of libtitanic_moe_hip.so: the entry points the reference's Rust FFN operators bind (see include/titanic_moe.h).
// Nothing here allocates, frees or synchronizes; every entry point only enqueues kernels on the caller's stream.
#include "../../include/titanic_moe.h"
#include "boundary.cuh"
#include "codec.cuh"
#include "combine.cuh"
#include "experts_gemm.cuh"
#include "experts_grouped.cuh"
#include "experts_stream.cuh"
#include "packing.cuh"
#include "shared.cuh"
#include <hip/hip_ext.h>
#include <cstdlib>
#include <cstring>

// Scratch of ca_moe_dynamic_static: one array a device, held from the library's load to the end of the process.  In host code
// the array's name stands for the symbol, not for device memory: its address on the current device is looked up once a device
// (ca_primitives_open*), and only that address is ever handed to kernels.
#define TF_STATIC_SCRATCH_BYTES (16u << 20)
static __device__ __align__(256) unsigned char scratch[TF_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
void* g_static_scratch[kMaxDevices] = {};

ca_geometry g_geometry = {5120, 384, 6, 576, 576, 1, 1.5f, 32, 32, 32, 129264, 10.f};   // src/ffn.rs:65-66, 245-258

// contraction lengths: multiples of 512 up to 4,096 everywhere; the token width (FC1) also multiples of 1,024 up to 8,192
bool supported_k(int k) { return k >= 512 && k <= 4096 && k % 512 == 0; }
bool supported_hidden(int k) { return supported_k(k) || (k > 4096 && k <= 8192 && k % 1024 == 0); }
int check_geometry(const ca_geometry& g) {
    if (g.hidden <= 0 || g.hidden % 512 || g.experts <= 0 || g.experts > 512 || g.topk <= 0 || g.topk > 8 ||
        g.topk > g.experts || g.intermediate <= 0 || g.intermediate % 512 || g.shared_intermediate <= 0 ||
        g.shared_intermediate % 512 || (g.scoring != 0 && g.scoring != 1) || (g.act_block != 32 && g.act_block != 128) ||
        g.shared_bn <= 0 || g.shared_bk <= 0 || g.shared_bk % 32 || g.hidden % g.shared_bk || g.shared_intermediate % g.shared_bk ||
        g.hidden % g.shared_bn || (2 * g.shared_intermediate) % g.shared_bn)
        return -4;
    if (!supported_hidden(g.hidden) || !supported_k(g.intermediate) || !supported_k(g.shared_intermediate)) return -4;
    return 0;
}
int launch_status() { return (int)hipGetLastError(); }

struct Context {
    ca_geometry g;
    int cus;
    int stream_wgs;    // persistent workgroups of the streaming kernels
    hipEvent_t marks[7];   // profiling aid: see ca_primitives_marks
    bool marking;
    bool kernel_marks;     // marks[5], marks[6]: begin and end of the FC1 + SwiGLU kernel itself
    int spin_limit;        // polls a wait inside the front-end launch may take before the waiter does the work itself
    int shared_reserve;    // CUs the shared expert's many-row first projection leaves without a workgroup (0: none)
    int device;            // the device the context was opened on
    uint8_t* static_scratch;   // that device's copy of `scratch`
};

// The regions of entry 0 / 1's scratch arena, in the runtime contract's order, each aligned to 256 bytes: token codes and
// scales (routed flavour, shared flavour), intermediate (BF16, codes, scales), tile tables, row maps, route outputs,
// wide-plan scratch, the front-end's sync region.
struct DynLayout {
    long long packed, scales, packed_min, scales_min, inter, inter_codes, inter_scales, task_expert, task_valid, tile_base, token_map,
        token_weights, scatter, plan_scratch, sync, total;
    int tile_m;
    long long tiles;
};
DynLayout dyn_layout(const ca_geometry& g, int rows) {
    DynLayout l{};
    const long long pairs = (long long)rows * g.topk;
    l.tile_m = rows <= TF_STREAM_MAX_ROWS ? 16 : TF_GEMM_TILE_M;
    l.tiles = (pairs + l.tile_m - 1) / l.tile_m - 1 + (g.experts < pairs ? g.experts : pairs);
    const long long padded = l.tiles * l.tile_m, H = g.hidden, I = g.intermediate, B = g.act_block;
    long long at = 0;
    auto add = [&](long long n) { const long long here = at; at += (n + 255) / 256 * 256; return here; };
    l.packed = add(rows * H); l.scales = add(rows * H / B); l.packed_min = add(rows * H); l.scales_min = add(rows * H / B);
    l.inter = add(padded * I * 2); l.inter_codes = add(padded * I); l.inter_scales = add(padded * I / B);
    l.task_expert = add(l.tiles * 4); l.task_valid = add(l.tiles * 4); l.tile_base = add((g.experts + 1) * 4ll);
    l.token_map = add(padded * 4); l.token_weights = add(padded * 4);
    l.scatter = add(pairs * H * 2);
    l.plan_scratch = add(((pairs + 63) / 64 * g.experts + pairs) * 4);
    l.sync = add(TF_SYNC_BYTES);
    l.total = at;
    return l;
}

// Records mark `i` on the launch stream when the caller asked for marks (never while a stream is captured: the caller's duty).
void mark(const Context& c, int i, hipStream_t s) {
    if (c.marking) (void)hipEventRecord(c.marks[i], s);
}

// Phase launches of the streaming kernels; either operand set may be absent (w == nullptr).
// `begin` / `end` (both or neither): events that take the kernel's own start and completion times (hipExtLaunchKernelGGL).
int launch_phase1(const StreamArgs& routed, const StreamArgs& shared, int wgs, hipStream_t s, hipEvent_t begin = nullptr, hipEvent_t end = nullptr) {
    const int k = routed.w ? routed.k : shared.k;
    if (routed.w && shared.w && routed.k != shared.k) return -4;
    const int wide = wgs >= 2 ? wgs / 2 : 1;       // eight-wave workgroups: one a CU
    auto go = [&](auto kernel, int grid, int block) {
        if (begin != nullptr && end != nullptr) hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, s, begin, end, 0, routed, shared);
        else kernel<<<grid, block, 0, s>>>(routed, shared);
    };
    switch (k) {
        case 512: go(tf_phase1_stream<1, 1, 4>, wgs, 256); break;
        case 1024: go(tf_phase1_stream<2, 2, 4>, wgs, 256); break;
        case 1536: go(tf_phase1_stream<3, 3, 4>, wgs, 256); break;
        case 2048: go(tf_phase1_stream<4, 4, 4>, wgs, 256); break;
        case 2560: go(tf_phase1_stream<5, 5, 4>, wgs, 256); break;
        case 3072: go(tf_phase1_stream<6, 6, 4>, wgs, 256); break;
        case 3584: go(tf_phase1_stream<7, 7, 4>, wgs, 256); break;
        case 4096: go(tf_phase1_stream<8, 8, 4>, wgs, 256); break;
        case 5120: go(tf_phase1_stream<5, 5, 8>, wide, 512); break;
        case 6144: go(tf_phase1_stream<6, 6, 8>, wide, 512); break;
        case 7168: go(tf_phase1_stream<7, 7, 8>, wide, 512); break;
        case 8192: go(tf_phase1_stream<8, 8, 8>, wide, 512); break;
        default: return -4;
    }
    return launch_status();
}
int launch_phase2(const StreamArgs& routed, const StreamArgs& shared, int wgs, hipStream_t s) {
    if (routed.w && shared.w && routed.k != shared.k) {       // different intermediate sizes: one launch each
        StreamArgs none{};
        const int status = launch_phase2(routed, none, wgs, s);
        return status ? status : launch_phase2(none, shared, wgs, s);
    }
    const int k = routed.w ? routed.k : shared.k, block = routed.w ? routed.act_block : shared.act_block;
    const size_t lds = 16 * (size_t)k + 16 * (size_t)(k / block);
    switch (k) {
        case 512: tf_phase2_stream<1, 1><<<wgs, 256, lds, s>>>(routed, shared); break;
        case 1024: tf_phase2_stream<2, 2><<<wgs, 256, lds, s>>>(routed, shared); break;
        case 1536: tf_phase2_stream<3, 3><<<wgs, 256, lds, s>>>(routed, shared); break;
        case 2048: tf_phase2_stream<4, 4><<<wgs, 256, lds, s>>>(routed, shared); break;
        case 2560: tf_phase2_stream<5, 5><<<wgs, 256, lds, s>>>(routed, shared); break;
        case 3072: tf_phase2_stream<6, 6><<<wgs, 256, lds, s>>>(routed, shared); break;
        case 3584: tf_phase2_stream<7, 7><<<wgs, 256, lds, s>>>(routed, shared); break;
        case 4096: tf_phase2_stream<8, 8><<<wgs, 256, lds, s>>>(routed, shared); break;
        default: return -4;
    }
    return launch_status();
}

// ---- entry 0 / 1: integration.tp_moe.dynamic -----------------------------------------------------------------------
enum DynPtr {
    P_A, P_IDS, P_WEIGHTS, P_PACKED, P_SCALES, P_PACKED_MIN, P_SCALES_MIN, P_INTER, P_INTER_CODES, P_INTER_SCALES,
    P_TASK_EXPERT, P_TASK_VALID, P_TILE_BASE, P_TOKEN_MAP, P_TOKEN_WEIGHTS, P_W13, P_S13, P_W2, P_S2, P_SCATTER,
    P_PLAN_SCRATCH, P_DYN_COUNT,
    P_LOGITS = P_DYN_COUNT, P_BIAS, P_BIAS_ALT, P_TOKENS, P_LIVE, P_PADDING, P_GATE_W, P_SYNC, P_ROUTE_COUNT
};
enum DynScalar { S_TOKENS, S_MAX_ROWS, S_ROWS_PADDED, S_MAX_TILES, S_TILE_M, S_GROUPS, S_DYN_COUNT, S_OWNER_ROWS = S_DYN_COUNT, S_ROUTE_COUNT };

enum SharedPtr { H_A, H_AS, H_W13, H_S13, H_W2, H_S2, H_ACT, H_ACT_CODES, H_ACT_SCALES, H_UP_TAP, H_OUT, H_COUNT };
// Streaming operands of the shared expert's two projections (few rows).
void shared_stream_args(const Context& c, const uint64_t* p, int m, StreamArgs& a, StreamArgs& b) {
    const ca_geometry& g = c.g;
    a = StreamArgs{};
    a.a_codes = (const uint8_t*)p[H_A]; a.a_scales = (const uint8_t*)p[H_AS];
    a.w = (const uint8_t*)p[H_W13]; a.ws = (const uint8_t*)p[H_S13]; a.bn = g.shared_bn; a.bk = g.shared_bk;
    a.dense_rows = m; a.k = g.hidden; a.inter = g.shared_intermediate; a.hidden = g.hidden; a.act_block = g.act_block;
    a.limit = g.swiglu_limit; a.out = (uint16_t*)p[H_ACT]; a.tap = (uint16_t*)p[H_UP_TAP];
    b = a;
    b.a_codes = nullptr; b.a_scales = nullptr; b.a_bf16 = (const uint16_t*)p[H_ACT];
    b.q_codes = (uint8_t*)p[H_ACT_CODES]; b.q_scales = (uint8_t*)p[H_ACT_SCALES]; b.min_amax = 1e-4f;
    b.w = (const uint8_t*)p[H_W2]; b.ws = (const uint8_t*)p[H_S2]; b.k = g.shared_intermediate; b.out = (uint16_t*)p[H_OUT];
    b.tap = nullptr;
}
// phases: 1 front-end (plan + quantize), 2 FC1 + SwiGLU, 4 FC2.  `sh` (may be null): the shared expert's operands (SharedPtr
// order, its input codes taken from the front-end's shared-flavour output), folded into the same phase launches.
// `sum` (may be null, needs `sh`): {routed output, layer output} device pointers and the live row count: the ordered sum and the
// shared addition run as well (inside the single streaming launch when the shapes allow it).
struct SumArgs { uint64_t routed_out, output; int live; };
int codec_blocks(const Context& c, long long rows, int k) {
    const long long blocks = (rows * (k >> 3) + 255) / 256;
    return (int)(blocks < (long long)c.cus * 16 ? blocks : (long long)c.cus * 16);
}
// `packed_input`: p[P_A] holds wire rows "dual_quant_rows_v1" (src/moe.rs:512-583) instead of BF16 rows.
int launch_dynamic(const Context& c, bool route, const uint64_t* p, const int32_t* sc, hipStream_t s, int phases = 7, const uint64_t* sh = nullptr,
                   const SumArgs* sum = nullptr, bool packed_input = false, float* projections = nullptr) {
    const ca_geometry& g = c.g;
    const int rows = sc[S_TOKENS], tile_m = sc[S_TILE_M], groups = sc[S_GROUPS], max_tiles = sc[S_MAX_TILES];
    if (rows < 1 || rows > sc[S_MAX_ROWS] || groups < 1 || max_tiles < 1 || sc[S_ROWS_PADDED] != max_tiles * tile_m) return -1;
    // many rows: the BF16 copy of the intermediate is a tap (FC2 reads the codes); few rows: it is what FC2 reads
    for (int i = 0; i < P_DYN_COUNT; ++i)
        if (!p[i] && i != P_PACKED_MIN && i != P_SCALES_MIN && i != P_INTER_CODES && i != P_INTER_SCALES && i != P_PLAN_SCRATCH &&
            !(i == P_INTER && rows > TF_STREAM_MAX_ROWS))
            return -1;
    if (!supported_hidden(g.hidden) || !supported_k(g.intermediate)) return -4;
    if (packed_input && g.act_block != 32) return -4;      // the wire row carries 32-wide blocks
    const long long pairs = (long long)rows * g.topk;
    // capacity of the reference's contracts (max_phys_tiles): A = min(E, pairs) experts open a tile each and the other routes fill
    // at most floor((pairs - A) / tile_m) <= ceil(pairs / tile_m) - 1 more
    const long long need_tiles = (pairs + tile_m - 1) / tile_m - 1 + (g.experts < pairs ? g.experts : pairs);
    if (need_tiles > max_tiles) return -1;
    const bool few = rows <= TF_STREAM_MAX_ROWS;
    if (few ? tile_m != 16 : tile_m != TF_GEMM_TILE_M) return -1;
    if (few && max_tiles > TF_LDS_TILES) return -1;

    StreamArgs sa{}, sb{};                 // few rows: the shared expert's two projections
    if (sh && few) {
        for (int i = 0; i < H_COUNT; ++i) if (!sh[i] && i != H_UP_TAP && i != H_ACT_CODES && i != H_ACT_SCALES) return -1;
        if (!supported_k(g.shared_intermediate)) return -4;
        shared_stream_args(c, sh, rows, sa, sb);
    }
    mark(c, 0, s);
    const uint16_t* x = (const uint16_t*)p[P_A];
    int32_t* ids = (int32_t*)p[P_IDS];
    float* weights = (float*)p[P_WEIGHTS];
    if (!(phases & 1)) {
    } else if (pairs <= 1024 && g.experts < 1024 && !packed_input) {
        const int quant_blocks = (int)((((long long)rows * (g.hidden >> 3)) + 1023) / 1024);
        if (route) {
            const int owner = sc[S_OWNER_ROWS];
            if (owner < rows || (long long)owner * g.topk > 1024) return -1;
            for (int i = P_LOGITS; i <= P_LIVE; ++i) if (!p[i] && i != P_BIAS_ALT && i != P_TOKENS) return -1;
            // with the gate weight (and a zeroed sync word) the gate product runs inside this launch too (owner rows <= 64)
            const bool gate = p[P_GATE_W] != 0;
            if (gate && (!p[P_SYNC] || owner > TF_STREAM_MAX_ROWS || g.hidden > 8192)) return -1;
            // per group of four rows: one expert a wave, eight waves a block (four for owners of at most eight rows)
            const int row_groups = (owner + 3) / 4;
            int logit_blocks = gate ? row_groups * (row_groups > 2 ? (g.experts + 7) / 8 : (g.experts + 3) / 4) : 0;
            // hidden <= 5,120: the shared expert's first projection streams in this launch, beside the front-end's chain of
            // dependent steps, instead of lengthening the routed experts' first launch
            const int shared_blocks = g.shared_intermediate / 16;          // one item (16 columns, every row tile) a block
            const int dense_logit_blocks = row_groups * ((g.experts + 7) / 8);
            const bool early_shared = sa.w != nullptr && gate && g.hidden <= TF_FRONT_SHARED_MAX_K && (g.hidden <= 4096 || g.hidden % 1024 == 0) && (phases & 3) == 3;
            if (early_shared) {
                logit_blocks = dense_logit_blocks;
                ca_moe_route_frontend_shared<<<quant_blocks + 1 + logit_blocks + shared_blocks, 512, 0, s>>>(
                    x, ids, weights, (uint8_t*)p[P_PACKED], (uint8_t*)p[P_SCALES], (int32_t*)p[P_TOKEN_MAP], (float*)p[P_TOKEN_WEIGHTS],
                    (int32_t*)p[P_TASK_EXPERT], (int32_t*)p[P_TASK_VALID], (int32_t*)p[P_TILE_BASE], (float*)p[P_LOGITS],
                    (const float*)p[P_BIAS], (const float*)p[P_BIAS_ALT], (const long long*)p[P_TOKENS], (const int32_t*)p[P_LIVE],
                    (const int32_t*)p[P_PADDING], rows, g.topk, g.experts, g.hidden, groups, tile_m, owner, g.act_block,
                    (uint8_t*)p[P_PACKED_MIN], (uint8_t*)p[P_SCALES_MIN], g.scoring, g.route_scale, (long long)g.alt_token,
                    (const uint16_t*)p[P_GATE_W], (uint32_t*)p[P_SYNC], logit_blocks, sa, shared_blocks, c.spin_limit);
                sa.w = nullptr;            // done: the routed experts' first launch runs without it
            } else
            ca_moe_route_frontend<<<quant_blocks + 1 + logit_blocks, 512, 0, s>>>(
                x, ids, weights, (uint8_t*)p[P_PACKED], (uint8_t*)p[P_SCALES], (int32_t*)p[P_TOKEN_MAP], (float*)p[P_TOKEN_WEIGHTS],
                (int32_t*)p[P_TASK_EXPERT], (int32_t*)p[P_TASK_VALID], (int32_t*)p[P_TILE_BASE], (float*)p[P_LOGITS],
                (const float*)p[P_BIAS], (const float*)p[P_BIAS_ALT], (const long long*)p[P_TOKENS], (const int32_t*)p[P_LIVE],
                (const int32_t*)p[P_PADDING], rows, g.topk, g.experts, g.hidden, groups, tile_m, owner, g.act_block,
                (uint8_t*)p[P_PACKED_MIN], (uint8_t*)p[P_SCALES_MIN], g.scoring, g.route_scale, (long long)g.alt_token,
                (const uint16_t*)p[P_GATE_W], (uint32_t*)p[P_SYNC], logit_blocks, c.spin_limit);
        } else {
            ca_moe_frontend<<<quant_blocks, 512, 0, s>>>(
                x, ids, weights, (uint8_t*)p[P_PACKED], (uint8_t*)p[P_SCALES], (int32_t*)p[P_TOKEN_MAP], (float*)p[P_TOKEN_WEIGHTS],
                (int32_t*)p[P_TASK_EXPERT], (int32_t*)p[P_TASK_VALID], (int32_t*)p[P_TILE_BASE], rows, g.topk, g.experts, g.hidden,
                groups, tile_m, g.act_block, (uint8_t*)p[P_PACKED_MIN], (uint8_t*)p[P_SCALES_MIN]);
        }
    } else {
        if (route || !p[P_PLAN_SCRATCH]) return -1;   // wide owners route with ca_route_topk first
        const int waves = (int)((pairs + 63) / 64);
        int32_t* wave_counts = (int32_t*)p[P_PLAN_SCRATCH];
        int32_t* local_rank = wave_counts + (size_t)waves * g.experts;
        ca_plan_wave_counts<<<(waves + 3) / 4, 256, 0, s>>>(ids, (int)pairs, g.experts, wave_counts, local_rank);
        ca_plan_scan<<<g.experts, 256, 0, s>>>(wave_counts, waves, g.experts, (int32_t*)p[P_TILE_BASE]);
        ca_plan_tiles<<<1, 512, 0, s>>>(g.experts, groups, tile_m, (int32_t*)p[P_TILE_BASE], (int32_t*)p[P_TASK_EXPERT], (int32_t*)p[P_TASK_VALID]);
        ca_plan_scatter<<<(int)((pairs + 255) / 256), 256, 0, s>>>(ids, weights, wave_counts, local_rank, (int32_t*)p[P_TILE_BASE],
                                                                    (int)pairs, g.experts, tile_m, (int32_t*)p[P_TOKEN_MAP],
                                                                    (float*)p[P_TOKEN_WEIGHTS]);
        const int blocks = codec_blocks(c, rows, g.hidden);
        if (packed_input)
            ca_codec_unpack_routed<<<blocks, 256, 0, s>>>((const uint8_t*)p[P_A], (uint8_t*)p[P_PACKED], (uint8_t*)p[P_SCALES], rows, g.hidden);
        else
            ca_quantize_rows<<<blocks, 256, 0, s>>>(x, (uint8_t*)p[P_PACKED], (uint8_t*)p[P_SCALES], (uint8_t*)p[P_PACKED_MIN],
                                                    (uint8_t*)p[P_SCALES_MIN], rows, g.hidden, g.act_block);
    }
    int status = launch_status();
    if (status) return status;
    mark(c, 1, s);

    const long long w13_stride = (long long)g.intermediate * g.hidden, s13_stride = w13_stride / 16;   // 2 I x H / 2, / 32
    const long long w2_stride = (long long)g.hidden * g.intermediate / 2, s2_stride = w2_stride / 16;
    if (few) {
        StreamArgs a{};
        a.a_codes = (const uint8_t*)p[P_PACKED]; a.a_scales = (const uint8_t*)p[P_SCALES];
        a.w = (const uint8_t*)p[P_W13]; a.ws = (const uint8_t*)p[P_S13];
        a.w_expert_stride = w13_stride; a.ws_expert_stride = s13_stride;
        a.expert_tile_base = (const int32_t*)p[P_TILE_BASE]; a.task_expert = (const int32_t*)p[P_TASK_EXPERT];
        a.task_valid_rows = (const int32_t*)p[P_TASK_VALID]; a.token_map = (const int32_t*)p[P_TOKEN_MAP];
        a.token_weights = (const float*)p[P_TOKEN_WEIGHTS];
        a.experts = g.experts; a.groups = groups; a.topk = g.topk;
        a.k = g.hidden; a.inter = g.intermediate; a.hidden = g.hidden; a.act_block = g.act_block; a.limit = g.swiglu_limit;
        a.out = (uint16_t*)p[P_INTER];
        a.table_tiles = max_tiles;
        StreamArgs b = a;
        a.proj = projections;
        b.a_codes = nullptr; b.a_scales = nullptr; b.a_bf16 = (const uint16_t*)p[P_INTER];
        b.q_codes = (uint8_t*)p[P_INTER_CODES]; b.q_scales = (uint8_t*)p[P_INTER_SCALES]; b.min_amax = 0.f;
        b.w = (const uint8_t*)p[P_W2]; b.ws = (const uint8_t*)p[P_S2];
        b.w_expert_stride = w2_stride; b.ws_expert_stride = s2_stride;
        b.k = g.intermediate; b.out = (uint16_t*)p[P_SCATTER];
        if (phases & 2) {
            status = c.marking && c.kernel_marks ? launch_phase1(a, sa, c.stream_wgs, s, c.marks[5], c.marks[6]) : launch_phase1(a, sa, c.stream_wgs, s);
            if (status) return status;
        }
        mark(c, 2, s);
        if (!(phases & 4)) return 0;
        status = launch_phase2(b, sb, c.stream_wgs, s);
        mark(c, 3, s);
        if (status || !sum) return status;
        const int n = rows * g.hidden;
        ca_ffn_sum_shared<<<(n / 8 + 255) / 256, 256, 0, s>>>((const uint16_t*)p[P_SCATTER], (const uint16_t*)sh[H_OUT], (uint16_t*)sum->routed_out,
                                                               (uint16_t*)sum->output, n, sum->live < rows ? sum->live : rows, g.topk, g.hidden);
        mark(c, 4, s);
        return launch_status();
    }
    if (sh || projections) return -4;   // many rows: the shared expert runs through its own entry; no FP32 projection tap
    if (!p[P_INTER_CODES] || !p[P_INTER_SCALES]) return -1;
    GemmArgs a{};
    a.a_codes = (const uint8_t*)p[P_PACKED]; a.a_scales = (const uint8_t*)p[P_SCALES];
    a.w = (const uint8_t*)p[P_W13]; a.ws = (const uint8_t*)p[P_S13];
    a.w_expert_stride = w13_stride; a.ws_expert_stride = s13_stride;
    a.expert_tile_base = (const int32_t*)p[P_TILE_BASE]; a.task_expert = (const int32_t*)p[P_TASK_EXPERT];
    a.task_valid_rows = (const int32_t*)p[P_TASK_VALID]; a.token_map = (const int32_t*)p[P_TOKEN_MAP];
    a.token_weights = (const float*)p[P_TOKEN_WEIGHTS];
    a.experts = g.experts; a.groups = groups; a.topk = g.topk; a.max_tiles = max_tiles;
    a.k = g.hidden; a.inter = g.intermediate; a.hidden = g.hidden; a.act_block = g.act_block; a.limit = g.swiglu_limit;
    a.h_bf16 = (uint16_t*)p[P_INTER]; a.h_codes = (uint8_t*)p[P_INTER_CODES]; a.h_scales = (uint8_t*)p[P_INTER_SCALES];
    a.out = (uint16_t*)p[P_SCATTER];
    if (phases & 2) {
        status = tf_launch_grouped<TF_GEMM_FC1_ROUTED>(a, pairs, c.cus, s);
        if (status) return status;
    }
    if (!(phases & 4)) return 0;
    GemmArgs b = a;
    b.a_codes = (const uint8_t*)p[P_INTER_CODES]; b.a_scales = (const uint8_t*)p[P_INTER_SCALES];
    b.w = (const uint8_t*)p[P_W2]; b.ws = (const uint8_t*)p[P_S2];
    b.w_expert_stride = w2_stride; b.ws_expert_stride = s2_stride;
    b.k = g.intermediate;
    return tf_launch_grouped<TF_GEMM_FC2_ROUTED>(b, pairs, c.cus, s);
}

// ---- entry 2: moe.w4a16.topk_sum -----------------------------------------------------------------------------------
int launch_topk_sum(const Context& c, const uint64_t* p, const int32_t* sc, hipStream_t s) {
    if (!p[0] || !p[1] || sc[0] < 0 || sc[1] != 0 || sc[2] != 0) return -1;
    if (sc[0] == 0) return 0;
    const long long n8 = (long long)sc[0] * (c.g.hidden >> 3);
    // the live rows arrive as active_m (the reference's host patches that scalar, src/moe.rs:1229); the third pointer is reserved
    // and never read: a contract may bind it to any operand
    ca_moe_topk_sum<<<(int)((n8 + 255) / 256), 256, 0, s>>>((const uint16_t*)p[0], (uint16_t*)p[1], sc[0], c.g.topk, c.g.hidden, nullptr, sc[0]);
    return launch_status();
}
// ---- entry 3: gemm.mxfp8_quant_cute --------------------------------------------------------------------------------
// pointers: input, values, scales (zero block -> scale 0), values_min, scales_min (amax floored at 1e-4); either pair may be null.
int launch_quant(const Context& c, const uint64_t* p, const int32_t* sc, hipStream_t s) {
    const int m = sc[0], k = sc[1];
    if (!p[0] || (!p[1] != !p[2]) || (!p[3] != !p[4]) || (!p[1] && !p[3]) || m < 1 || k < c.g.act_block || k % c.g.act_block || sc[2] != 0)
        return -1;
    const long long items = (long long)m * (k >> 3);
    int blocks = (int)((items + 255) / 256);
    if (blocks > c.cus * 16) blocks = c.cus * 16;
    ca_quantize_rows<<<blocks, 256, 0, s>>>((const uint16_t*)p[0], (uint8_t*)p[1], (uint8_t*)p[2], (uint8_t*)p[3], (uint8_t*)p[4], m, k,
                                            c.g.act_block);
    return launch_status();
}
// ---- entries 12, 13: gemm.mxfp8_quant_cute with the reference's own operand list (src/moe.rs:557-561, 573-575): source,
// values, row-major block scales, and a second scale buffer.  The reference's second buffer holds the scales in the order
// its matrix instructions read them; this library's kernels read the row-major ones, and the second buffer (may be null)
// receives the same bytes.  Entry 12: no amax floor (the routed experts' flavour); entry 13: amax floored at 1e-4 (the
// shared expert's).  `grid_x` is the reference kernel's launch width and is not used here.
int launch_quant_reference(const Context& c, const uint64_t* p, const int32_t* sc, hipStream_t s, bool floored) {
    const int m = sc[0], k = sc[1];
    if (!p[0] || !p[1] || !p[2] || m < 1 || k < c.g.act_block || k % c.g.act_block || sc[2] < 0) return -1;
    const long long items = (long long)m * (k >> 3);
    int blocks = (int)((items + 255) / 256);
    if (blocks > c.cus * 16) blocks = c.cus * 16;
    ca_quantize_rows<<<blocks, 256, 0, s>>>((const uint16_t*)p[0], floored ? nullptr : (uint8_t*)p[1], floored ? nullptr : (uint8_t*)p[2],
                                            floored ? (uint8_t*)p[1] : nullptr, floored ? (uint8_t*)p[2] : nullptr, m, k, c.g.act_block);
    int status = launch_status();
    if (status || !p[3]) return status;
    return (int)hipMemcpyAsync((void*)p[3], (const void*)p[2], (size_t)m * (k / c.g.act_block), hipMemcpyDeviceToDevice, s);
}
// ---- entry 11: moe.w4a8.compact_micro (src/moe.rs:379-393, 625-629; runtime/kernels/moe-runtime-m6-micro-fp32-v1) -----
// Both projections of the routed experts for a few rows whose token codes are already quantized (entry 12 before it), with
// the FP32 projections of FC1 kept: projections[pair][2 I] (up, then gate).  Pointers: the reference's fifteen (the four
// `ones` scale pointers are not read: E8M0 block scales carry every scale here), then this library's plan tables.  The
// routes are grouped by expert as in entry 0, so an expert chosen by several rows streams once; a pair's results do not
// depend on the grouping.  num_pairs = live rows x top-k.
enum MicroPtr { M_CODES, M_CODE_SCALES, M_W13, M_S13, M_INTER, M_PROJ, M_WEIGHTS, M_IDS, M_ALPHA1, M_INPUT_SCALE, M_W2, M_S2, M_OUT, M_ALPHA2,
                M_DOWN_SCALE, M_TASK_EXPERT, M_TASK_VALID, M_TILE_BASE, M_TOKEN_MAP, M_TILE_WEIGHTS, M_COUNT };
int launch_micro(const Context& c, const uint64_t* p, const int32_t* sc, hipStream_t s) {
    const ca_geometry& g = c.g;
    const int pairs = sc[0];
    for (int i = 0; i < M_COUNT; ++i)
        if (!p[i] && i != M_PROJ && i != M_ALPHA1 && i != M_INPUT_SCALE && i != M_ALPHA2 && i != M_DOWN_SCALE) return -1;
    if (pairs < 1 || pairs % g.topk || pairs / g.topk > TF_STREAM_MAX_ROWS || sc[1] < 0) return -1;
    const int rows = pairs / g.topk;
    const int tiles = (pairs + 15) / 16 - 1 + (g.experts < pairs ? g.experts : pairs);
    if (tiles > TF_LDS_TILES) return -1;
    // the plan alone: the front-end kernel with no columns to quantize
    ca_moe_frontend<<<1, 512, 0, s>>>(nullptr, (const int32_t*)p[M_IDS], (const float*)p[M_WEIGHTS], nullptr, nullptr, (int32_t*)p[M_TOKEN_MAP],
                                      (float*)p[M_TILE_WEIGHTS], (int32_t*)p[M_TASK_EXPERT], (int32_t*)p[M_TASK_VALID], (int32_t*)p[M_TILE_BASE],
                                      rows, g.topk, g.experts, 0, 1, 16, g.act_block, nullptr, nullptr);
    const int status = launch_status();
    if (status) return status;
    uint64_t q[P_DYN_COUNT] = {};
    q[P_A] = p[M_CODES]; q[P_IDS] = p[M_IDS]; q[P_WEIGHTS] = p[M_WEIGHTS]; q[P_PACKED] = p[M_CODES]; q[P_SCALES] = p[M_CODE_SCALES];
    q[P_INTER] = p[M_INTER]; q[P_TASK_EXPERT] = p[M_TASK_EXPERT]; q[P_TASK_VALID] = p[M_TASK_VALID]; q[P_TILE_BASE] = p[M_TILE_BASE];
    q[P_TOKEN_MAP] = p[M_TOKEN_MAP]; q[P_TOKEN_WEIGHTS] = p[M_TILE_WEIGHTS]; q[P_W13] = p[M_W13]; q[P_S13] = p[M_S13]; q[P_W2] = p[M_W2];
    q[P_S2] = p[M_S2]; q[P_SCATTER] = p[M_OUT];
    const int32_t scalars[S_DYN_COUNT] = {rows, rows, tiles * 16, tiles, 16, 1};
    return launch_dynamic(c, false, q, scalars, s, 6, nullptr, nullptr, false, (float*)p[M_PROJ]);
}
// ---- entry 4: gemm.dense (FP8 x FP8 block-scaled -> BF16) -----------------------------------------------------------
int launch_dense(const Context& c, const uint64_t* p, const int32_t* sc, hipStream_t s) {
    const int m = sc[0], n = sc[1], k = sc[2];
    for (int i = 0; i < 5; ++i) if (!p[i]) return -1;
    if (m < 1 || n < 64 || n % 64 || !supported_hidden(k)) return -1;
    if (m <= TF_STREAM_MAX_ROWS) {
        // few rows (src/fp8_linear.rs:883-897 launches this entry at 6 rows): the streaming kernel of the shared expert's first
        // projection, whose BF16 projections before the activation are this product; the activation itself is not stored.
        // Its items pair weight tile j with tile n / 32 + j, so n is a multiple of 32 (of 64 here).
        StreamArgs a{}, none{};
        a.a_codes = (const uint8_t*)p[0]; a.a_scales = (const uint8_t*)p[1];
        a.w = (const uint8_t*)p[2]; a.ws = (const uint8_t*)p[3]; a.bn = c.g.shared_bn; a.bk = c.g.shared_bk;
        a.dense_rows = m; a.k = k; a.inter = n / 2; a.hidden = k; a.act_block = c.g.act_block; a.limit = c.g.swiglu_limit;
        a.out = nullptr; a.tap = (uint16_t*)p[4];
        if (c.cus <= 0) return (int)hipErrorNoDevice;
        return launch_phase1(none, a, c.stream_wgs, s);
    }
    GemmArgs a{};
    a.a_codes = (const uint8_t*)p[0]; a.a_scales = (const uint8_t*)p[1];
    a.w = (const uint8_t*)p[2]; a.ws = (const uint8_t*)p[3]; a.bn = c.g.shared_bn; a.bk = c.g.shared_bk;
    a.dense_rows = m; a.k = k; a.hidden = n; a.act_block = c.g.act_block; a.out = (uint16_t*)p[4];
    if (tf_grouped_dense_shape_ok(a, false)) return tf_launch_grouped_dense<TF_GEMM_DENSE>(a, c.cus, s);
    return tf_launch_dense_gemm(a, c.cus, s);
}
// ---- entry 5: ffn.shared_expert (up + clipped SwiGLU + requant + down, from the quantized input) ---------------------
int launch_shared(const Context& c, const uint64_t* p, const int32_t* sc, hipStream_t s) {
    const ca_geometry& g = c.g;
    const int m = sc[0];
    // many rows: the second projection reads the FP8 codes, so the BF16 activation is a tap like the projections before it
    for (int i = 0; i < H_COUNT; ++i)
        if (!p[i] && i != H_UP_TAP && i != H_ACT_CODES && i != H_ACT_SCALES && !(i == H_ACT && m > TF_STREAM_MAX_ROWS)) return -1;
    if (m < 1 || !supported_hidden(g.hidden) || !supported_k(g.shared_intermediate)) return -4;
    if (m <= TF_STREAM_MAX_ROWS) {
        StreamArgs a, b, none{};
        shared_stream_args(c, p, m, a, b);
        const int status = launch_phase1(none, a, c.stream_wgs, s);
        return status ? status : launch_phase2(none, b, c.stream_wgs, s);
    }
    if (!p[H_ACT_CODES] || !p[H_ACT_SCALES]) return -1;
    GemmArgs a{};
    a.a_codes = (const uint8_t*)p[H_A]; a.a_scales = (const uint8_t*)p[H_AS];
    a.w = (const uint8_t*)p[H_W13]; a.ws = (const uint8_t*)p[H_S13]; a.bn = g.shared_bn; a.bk = g.shared_bk;
    a.dense_rows = m; a.k = g.hidden; a.inter = g.shared_intermediate; a.hidden = g.hidden; a.act_block = g.act_block;
    a.limit = g.swiglu_limit; a.h_bf16 = (uint16_t*)p[H_ACT]; a.h_codes = (uint8_t*)p[H_ACT_CODES]; a.h_scales = (uint8_t*)p[H_ACT_SCALES];
    a.tap = (uint16_t*)p[H_UP_TAP];
    // a host that runs the router beside this entry on another stream may keep some CUs free for it (ca_primitives_shared_reserve)
    int status = tf_grouped_dense_shape_ok(a, true) ? tf_launch_grouped_dense<TF_GEMM_FC1_SHARED>(a, c.cus - c.shared_reserve, s) : tf_launch_shared_fc1_gemm(a, c.cus, s);
    if (status) return status;
    GemmArgs b{};
    b.a_codes = (const uint8_t*)p[H_ACT_CODES]; b.a_scales = (const uint8_t*)p[H_ACT_SCALES];
    b.w = (const uint8_t*)p[H_W2]; b.ws = (const uint8_t*)p[H_S2]; b.bn = g.shared_bn; b.bk = g.shared_bk;
    b.dense_rows = m; b.k = g.shared_intermediate; b.hidden = g.hidden; b.act_block = g.act_block; b.out = (uint16_t*)p[H_OUT];
    if (tf_grouped_dense_shape_ok(b, false)) return tf_launch_grouped_dense<TF_GEMM_DENSE>(b, c.cus, s);
    return tf_launch_dense_gemm(b, c.cus, s);
}

struct EntryShape { const char* kernel_id; size_t pointers, scalars; };
const EntryShape kEntries[] = {
    {"integration.tp_moe.dynamic", P_DYN_COUNT, S_DYN_COUNT},
    {"integration.tp_moe.dynamic", P_ROUTE_COUNT, S_ROUTE_COUNT},
    {"moe.w4a16.topk_sum", 3, 3},
    {"gemm.mxfp8_quant_cute", 5, 3},
    {"gemm.dense", 5, 3},
    {"ffn.shared_expert", H_COUNT, 1},
    {"moe.w4a8.phase1", P_DYN_COUNT, S_DYN_COUNT},
    {"moe.w4a8.phase2", P_DYN_COUNT, S_DYN_COUNT},
    {"moe.front_end", P_DYN_COUNT, S_DYN_COUNT},
    {"ffn.experts_with_shared", P_ROUTE_COUNT + H_COUNT - 2 + 2, S_ROUTE_COUNT + 1},
    {"integration.tp_moe.dynamic", P_DYN_COUNT, S_DYN_COUNT},      // input_format dual_quant_rows_v1
    {"moe.w4a8.compact_micro", M_COUNT, 2},
    {"gemm.mxfp8_quant_cute", 4, 3},
    {"gemm.mxfp8_quant_cute", 4, 3},
};
constexpr int kEntryCount = sizeof(kEntries) / sizeof(kEntries[0]);

struct KernelName { const char* name; const void* function; };
#define TF_KERNEL(k) {#k, (const void*)k}
const KernelName kKernels[] = {
    TF_KERNEL(ca_router_logits_rows), TF_KERNEL(ca_route_topk), TF_KERNEL(ca_route_padding_rows), TF_KERNEL(ca_route_census),
    TF_KERNEL(ca_moe_frontend), TF_KERNEL(ca_moe_route_frontend), TF_KERNEL(ca_moe_route_frontend_shared), TF_KERNEL(ca_quantize_rows), TF_KERNEL(ca_plan_wave_counts),
    TF_KERNEL(ca_plan_scan), TF_KERNEL(ca_plan_tiles), TF_KERNEL(ca_plan_scatter), TF_KERNEL(ca_shared_swiglu_rows), TF_KERNEL(ca_shared_swiglu_quant),
    TF_KERNEL(ca_ffn_add_rows), TF_KERNEL(ca_moe_topk_sum), TF_KERNEL(ca_ffn_sum_shared), TF_KERNEL(ca_moe_group_sum_rows),
    TF_KERNEL(ca_expert_compact_words), TF_KERNEL(ca_expert_expand_words), TF_KERNEL(ca_expert_compact_scales),
    TF_KERNEL(ca_expert_expand_scales), TF_KERNEL(ca_dense_compact_fp8), TF_KERNEL(ca_moe_nibble_permute_words),
    TF_KERNEL(ca_expert_scale_code1), TF_KERNEL(ca_expert_scale_code1_check), TF_KERNEL(ca_expert_scale_code1_census),
    TF_KERNEL(ca_expert_scale_codes4), TF_KERNEL(ca_router_logits_mfma), TF_KERNEL(ca_codec_encode), TF_KERNEL(ca_codec_decode),
    TF_KERNEL(ca_codec_pack_bf16), TF_KERNEL(ca_codec_unpack_routed), TF_KERNEL(ca_codec_local_live), TF_KERNEL(ca_convert_formats),
    TF_KERNEL(ca_rmsnorm_quant), TF_KERNEL(ca_ffn_sum_shared_residual), TF_KERNEL(ca_hc_combine_norm_quant_rows), TF_KERNEL(ca_hc_post_rows),
    TF_KERNEL(ca_ffn_sum_shared_hc_post),
};
constexpr int kKernelCount = sizeof(kKernels) / sizeof(kKernels[0]);

}  // namespace

extern "C" {

int ca_ffn_abi(void) { return 1; }
int ca_ffn_configure(const ca_geometry* geometry) {
    if (!geometry) return -1;
    const int status = check_geometry(*geometry);
    if (status) return status;
    g_geometry = *geometry;
    return 0;
}
int ca_ffn_geometry(ca_geometry* out) {
    if (!out) return -1;
    *out = g_geometry;
    return 0;
}
// The four functions of the reference's libcanada_ffn.so keep its signatures, which carry no shapes: they take the process
// geometry of ca_ffn_configure.  A host that keeps layers of several geometries in one process (the reference's 384-expert
// target and 128-expert drafter, src/layer_id.rs:39-47) calls the *_in variants, which take the geometry of a context.
namespace {
int router_logits_of(const ca_geometry& g, int rows, const void* x, const void* w, void* out, void* stream) {
    if (rows < 1 || rows > 16 || !x || !w || !out) return -1;
    ca_router_logits_rows<<<g.experts, 64, 0, (hipStream_t)stream>>>((const uint16_t*)x, (const uint16_t*)w, (float*)out, rows, g.hidden, g.experts);
    return launch_status();
}
int router_logits_wide_of(const ca_geometry& g, int rows, const void* x, const void* w, void* out, void* stream) {
    if (rows < 1 || !x || !w || !out) return -1;
    if (rows <= 16) return router_logits_of(g, rows, x, w, out, stream);
    if (g.hidden % 64) return -4;
    // 128-row workgroup tiles once they give every CU of the part (256) a workgroup; 64-row tiles below that
    const dim3 grid((rows + 127) / 128, (g.experts + 255) / 256);
    if (grid.x * grid.y >= 256) {
        ca_router_logits_mfma<<<grid, 512, 0, (hipStream_t)stream>>>((const uint16_t*)x, (const uint16_t*)w, (float*)out, rows, g.hidden, g.experts);
    } else {
        const dim3 half((rows + 63) / 64, grid.y);
        tf_router_logits_mfma_64<<<half, 512, 0, (hipStream_t)stream>>>((const uint16_t*)x, (const uint16_t*)w, (float*)out, rows, g.hidden, g.experts);
    }
    return launch_status();
}
int shared_swiglu_of(const ca_geometry& g, int rows, const void* input, void* output, void* stream) {
    if (rows < 1 || rows > 65536 || !input || !output) return -1;
    const long long items = (long long)rows * (g.shared_intermediate >> 3);
    ca_shared_swiglu_rows<<<(int)((items + 255) / 256), 256, 0, (hipStream_t)stream>>>((const uint16_t*)input, (uint16_t*)output, rows,
                                                                                       g.shared_intermediate, g.swiglu_limit);
    return launch_status();
}
int ffn_add_of(const ca_geometry& g, int rows, const void* routed, const void* shared, void* out, void* stream) {
    if (rows < 1 || rows > 65536 || !routed || !shared || !out) return -1;
    const long long n8 = (long long)rows * (g.hidden >> 3);
    ca_ffn_add_rows<<<(int)((n8 + 255) / 256), 256, 0, (hipStream_t)stream>>>((const uint16_t*)routed, (const uint16_t*)shared, (uint16_t*)out, n8);
    return launch_status();
}
}  // namespace
int ca_router_logits(int rows, const void* x, const void* w, void* out, void* stream) { return router_logits_of(g_geometry, rows, x, w, out, stream); }
int ca_router_logits_wide(int rows, const void* x, const void* w, void* out, void* stream) { return router_logits_wide_of(g_geometry, rows, x, w, out, stream); }
int ca_shared_swiglu(int rows, const void* input, void* output, void* stream) { return shared_swiglu_of(g_geometry, rows, input, output, stream); }
int ca_ffn_add(int rows, const void* routed, const void* shared, void* out, void* stream) { return ffn_add_of(g_geometry, rows, routed, shared, out, stream); }
int ca_router_logits_in(void* context, int rows, const void* x, const void* w, void* out, void* stream) {
    return context ? router_logits_of(((const Context*)context)->g, rows, x, w, out, stream) : -1;
}
int ca_router_logits_wide_in(void* context, int rows, const void* x, const void* w, void* out, void* stream) {
    return context ? router_logits_wide_of(((const Context*)context)->g, rows, x, w, out, stream) : -1;
}
int ca_shared_swiglu_in(void* context, int rows, const void* input, void* output, void* stream) {
    return context ? shared_swiglu_of(((const Context*)context)->g, rows, input, output, stream) : -1;
}
int ca_ffn_add_in(void* context, int rows, const void* routed, const void* shared, void* out, void* stream) {
    return context ? ffn_add_of(((const Context*)context)->g, rows, routed, shared, out, stream) : -1;
}
// ---- the decoder's FFN boundary either side of the layer (boundary.cuh) -------------------------------------------------
int ca_ffn_norm_quant(void* context, int rows, const void* x, const void* weight, float eps, void* normed, void* codes, void* scales,
                      void* codes_min, void* scales_min, void* stream) {
    if (!context || !x || !weight || !normed || rows < 1 || (!codes != !scales) || (!codes_min != !scales_min) || !(eps >= 0.f)) return -1;
    const ca_geometry& g = ((const Context*)context)->g;
    if (g.hidden > 8192 || g.hidden % g.act_block) return -4;
    ca_rmsnorm_quant<<<rows, 256, 0, (hipStream_t)stream>>>((const uint16_t*)x, (const uint16_t*)weight, (uint16_t*)normed, (uint8_t*)codes,
                                                            (uint8_t*)scales, (uint8_t*)codes_min, (uint8_t*)scales_min, g.hidden, g.act_block, eps);
    return launch_status();
}
int ca_hc_combine_norm_quant(void* context, int rows, int streams, const void* x, const float* pre, const void* weight, void* normed,
                             void* codes_min, void* scales_min, void* mma_scales, void* codes, void* scales, void* stream) {
    if (!context || !x || !weight || !normed || rows < 1 || rows > 65536 || streams < 1 || streams > 8 || (!codes != !scales) ||
        (!codes_min != !scales_min))
        return -1;
    const ca_geometry& g = ((const Context*)context)->g;
    if (g.hidden > 8192 || g.hidden % g.act_block) return -4;
    if (mma_scales && g.act_block != 32) return -1;          // the reference's offsets are those of 32-wide blocks
    ca_hc_combine_norm_quant_rows<<<dim3(rows, 1, 1), 256, 0, (hipStream_t)stream>>>(
        (const uint16_t*)x, pre, (const uint16_t*)weight, (uint16_t*)normed, (uint8_t*)codes_min, (uint8_t*)scales_min, (uint8_t*)mma_scales,
        (uint8_t*)codes, (uint8_t*)scales, g.hidden, streams, g.act_block, 1.0e-20f);
    return launch_status();
}
int ca_hc_post(void* context, int rows, const void* sublayer, const void* residual, const float* post, const float* comb, void* y, void* stream) {
    if (!context || !sublayer || !residual || !post || !comb || !y || rows < 1) return -1;
    const ca_geometry& g = ((const Context*)context)->g;
    const long long n8 = (long long)rows * (g.hidden >> 3);
    if (n8 > 0x7fffffffll) return -1;
    ca_hc_post_rows<<<(int)((n8 + 255) / 256), 256, 0, (hipStream_t)stream>>>((const uint16_t*)sublayer, (const uint16_t*)residual, post, comb,
                                                                          (uint16_t*)y, rows, g.hidden);
    return launch_status();
}
int ca_ffn_sum_hc_post(void* context, int rows, int live, const void* routes, const void* shared, const void* residual, const float* post,
                       const float* comb, void* routed, void* ffn_out, void* y, void* stream) {
    if (!context || !routes || !shared || !residual || !post || !comb || !routed || !y || rows < 1 || live < 0) return -1;
    const ca_geometry& g = ((const Context*)context)->g;
    const long long n8 = (long long)rows * (g.hidden >> 3);
    if (n8 > 0x7fffffffll) return -1;
    ca_ffn_sum_shared_hc_post<<<(int)((n8 + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        (const uint16_t*)routes, (const uint16_t*)shared, (const uint16_t*)residual, post, comb, (uint16_t*)routed, (uint16_t*)ffn_out, (uint16_t*)y,
        rows, live < rows ? live : rows, g.topk, g.hidden);
    return launch_status();
}
int ca_ffn_sum_residual(void* context, int rows, int live, const void* routes, const void* shared, const void* residual, void* routed,
                        void* ffn_out, void* residual_out, void* stream) {
    if (!context || !routes || !shared || !residual || !routed || !residual_out || rows < 1 || live < 0) return -1;
    const ca_geometry& g = ((const Context*)context)->g;
    const long long n = (long long)rows * g.hidden;
    if (n > 0x7fffffffll) return -1;
    ca_ffn_sum_shared_residual<<<(int)((n / 8 + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        (const uint16_t*)routes, (const uint16_t*)shared, (const uint16_t*)residual, (uint16_t*)routed, (uint16_t*)ffn_out, (uint16_t*)residual_out,
        (int)n, live < rows ? live : rows, g.topk, g.hidden);
    return launch_status();
}
int ca_moe_nibble_permute(void* data, uint64_t bytes, int inverse, void* stream) {
    if (!data || bytes % 4 || (inverse != 0 && inverse != 1)) return -1;
    ca_moe_nibble_permute_words<<<256, 256, 0, (hipStream_t)stream>>>((uint32_t*)data, bytes / 4, inverse);
    return launch_status();
}

// ---- row codec (runtime/kernels/moe-input-codec-coalesced-v1/moe-dual-quant-codec-fast.cu:81-94, 99-105, 138-144) ----
namespace { int codec_grid(long long rows, int k) { const long long b = (rows * (k >> 3) + 255) / 256; return (int)(b < 4096 ? b : 4096); } }
int ca_encode(const uint8_t* routed, const uint8_t* scales, const uint8_t* shared, uint8_t* packed, int rows, int k, void* stream) {
    if (!routed || !scales || !shared || !packed || rows <= 0 || k <= 0 || k % 128) return -1;
    ca_codec_encode<<<codec_grid(rows, k), 256, 0, (hipStream_t)stream>>>(routed, scales, shared, packed, rows, k);
    return launch_status();
}
int ca_decode(const uint8_t* packed, uint8_t* shared, uint8_t* row_scales, uint8_t* mma_scales, int rows, int k, void* stream) {
    if (!packed || !shared || !row_scales || rows <= 0 || rows % 128 || k <= 0 || k % 128) return -1;
    ca_codec_decode<<<codec_grid(rows, k), 256, 0, (hipStream_t)stream>>>(packed, shared, row_scales, mma_scales, rows, k);
    return launch_status();
}
int ca_local_live(const int* global, int* local, int rows, int rank, void* stream) {
    if (!global || !local || rows <= 0 || rank < 0 || rank >= 4) return -1;
    ca_codec_local_live<<<1, 64, 0, (hipStream_t)stream>>>(global, local, rows, rank);
    return launch_status();
}
int ca_pack_bf16(const void* input, uint8_t* packed, int rows, int k, void* stream) {
    if (!input || !packed || rows <= 0 || k <= 0 || k % 128) return -1;
    ca_codec_pack_bf16<<<codec_grid(rows, k), 256, 0, (hipStream_t)stream>>>((const uint16_t*)input, packed, rows, k);
    return launch_status();
}

int ca_kernel_count(void) { return kKernelCount; }
const char* ca_kernel_name(int index) { return index >= 0 && index < kKernelCount ? kKernels[index].name : nullptr; }
int ca_kernel_launch(const char* name, const uint32_t grid[3], const uint32_t block[3], uint32_t shared_bytes, void** args, void* stream) {
    if (!name || !grid || !block || !args) return -1;
    if (!grid[0] || !grid[1] || !grid[2] || !block[0] || !block[1] || !block[2] || (uint64_t)block[0] * block[1] * block[2] > 1024) return -1;
    for (int i = 0; i < kKernelCount; ++i)
        if (!std::strcmp(name, kKernels[i].name))
            return (int)hipLaunchKernel(kKernels[i].function, dim3(grid[0], grid[1], grid[2]), dim3(block[0], block[1], block[2]), args,
                                        shared_bytes, (hipStream_t)stream);
    return -3;
}

int32_t ca_primitives_abi(void) { return 1; }
int32_t ca_primitives_entries(void) { return kEntryCount; }
void* ca_primitives_open_geometry(const ca_geometry* geometry, int32_t* status) {
    if (!status) return nullptr;
    if (!geometry) { *status = -1; return nullptr; }
    *status = check_geometry(*geometry);
    if (*status) return nullptr;
    int device = 0, cus = 0;
    hipError_t e = hipGetDevice(&device);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
    if (e != hipSuccess) { *status = (int32_t)e; return nullptr; }
    if (device < 0 || device >= kMaxDevices) { *status = -1; return nullptr; }
    if (!g_static_scratch[device]) {          // this device's copy of the static scratch array: looked up once, with the device current
        void* at = nullptr;
        e = hipGetSymbolAddress(&at, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !at) { *status = e != hipSuccess ? (int32_t)e : -1; return nullptr; }
        g_static_scratch[device] = at;
    }
    Context* c = new Context{};
    c->g = *geometry; c->cus = cus; c->stream_wgs = cus * 2; c->spin_limit = 1 << 18; c->shared_reserve = 0;
    c->device = device; c->static_scratch = (uint8_t*)g_static_scratch[device];
    return c;
}
void* ca_primitives_open(int32_t* status) { return ca_primitives_open_geometry(&g_geometry, status); }
int32_t ca_primitives_geometry(void* context, ca_geometry* out) {
    if (!context || !out) return -1;
    *out = ((const Context*)context)->g;
    return 0;
}
void ca_primitives_close(void* context) { delete (Context*)context; }
int32_t ca_primitives_marks(void* context, void* const* events, size_t count) {
    if (!context || (count != 0 && ((count != 5 && count != 7) || !events))) return -1;
    Context* c = (Context*)context;
    c->marking = count != 0;
    c->kernel_marks = count == 7;
    for (size_t i = 0; i < count; ++i) {
        if (!events[i]) { c->marking = c->kernel_marks = false; return -1; }
        c->marks[i] = (hipEvent_t)events[i];
    }
    return 0;
}
int32_t ca_primitives_spin_limit(void* context, int32_t limit) {
    if (!context || limit < 0) return -1;
    ((Context*)context)->spin_limit = limit;
    return 0;
}
int32_t ca_primitives_shared_reserve(void* context, int32_t cus) {
    if (!context || cus < 0 || cus % 8 || cus * 2 > ((Context*)context)->cus) return -1;
    ((Context*)context)->shared_reserve = cus;
    return 0;
}
int32_t ca_primitives_launch(void* context, int32_t index, const uint64_t* pointers, size_t np, const int32_t* scalars, size_t ns,
                             void* stream) {
    if (!context || !pointers || !scalars) return -1;
    if (index < 0 || index >= kEntryCount) return -3;
    if (np != kEntries[index].pointers || ns != kEntries[index].scalars) return -2;
    const Context& c = *(const Context*)context;
    hipStream_t s = (hipStream_t)stream;
    switch (index) {
        case 0: return launch_dynamic(c, false, pointers, scalars, s);
        case 1: return launch_dynamic(c, true, pointers, scalars, s);
        case 2: return launch_topk_sum(c, pointers, scalars, s);
        case 3: return launch_quant(c, pointers, scalars, s);
        case 4: return launch_dense(c, pointers, scalars, s);
        case 5: return launch_shared(c, pointers, scalars, s);
        case 6: return launch_dynamic(c, false, pointers, scalars, s, 2);
        case 7: return launch_dynamic(c, false, pointers, scalars, s, 4);
        case 8: return launch_dynamic(c, false, pointers, scalars, s, 1);
        case 9: {   // routed experts (top-k inside the front-end when logits are given) + shared expert in the same launches
            uint64_t sh[H_COUNT];
            sh[H_A] = pointers[P_PACKED_MIN]; sh[H_AS] = pointers[P_SCALES_MIN];
            for (int i = 2; i < H_COUNT; ++i) sh[i] = pointers[P_ROUTE_COUNT + i - 2];
            if (!sh[H_A] || !sh[H_AS]) return -1;
            // + routed output, layer output (both or neither) and the live row count: the sum and the shared addition run too
            const uint64_t routed_out = pointers[P_ROUTE_COUNT + H_COUNT - 2], output = pointers[P_ROUTE_COUNT + H_COUNT - 1];
            if (!routed_out != !output) return -1;
            const SumArgs sum{routed_out, output, scalars[S_ROUTE_COUNT]};
            return launch_dynamic(c, pointers[P_LOGITS] != 0, pointers, scalars, s, 7, sh, output ? &sum : nullptr);
        }
        case 10: return launch_dynamic(c, false, pointers, scalars, s, 7, nullptr, nullptr, true);
        case 11: return launch_micro(c, pointers, scalars, s);
        case 12: return launch_quant_reference(c, pointers, scalars, s, false);
        case 13: return launch_quant_reference(c, pointers, scalars, s, true);
        default: return -3;
    }
}
int32_t ca_primitives_launch2(void* context, int32_t index, const uint64_t* words, size_t n, void* stream) {
    if (!context || !words) return -1;
    if (index < 0 || index >= kEntryCount) return -3;
    const size_t np = kEntries[index].pointers, ns = kEntries[index].scalars;
    if (n != np + ns) return -2;
    int32_t scalars[16];
    for (size_t i = 0; i < ns; ++i) scalars[i] = (int32_t)words[np + i];
    return ca_primitives_launch(context, index, words, np, scalars, ns, stream);
}
int64_t ca_primitives_scratch_bytes(void* context, int32_t index, int32_t rows) {
    if (!context || rows < 1 || (index != 0 && index != 1)) return -1;
    return dyn_layout(((const Context*)context)->g, rows).total;
}
int64_t ca_moe_dynamic_static_capacity(void) { return (int64_t)TF_STATIC_SCRATCH_BYTES; }
int32_t ca_moe_dynamic_static(void* context, const void* input, const int32_t* topk_ids, const float* topk_weights, const void* w13,
                              const void* s13, const void* w2, const void* s2, void* route_output, int32_t rows, void* stream) {
    if (!context || !input || !topk_ids || !topk_weights || !w13 || !s13 || !w2 || !s2 || !route_output || rows < 1) return -1;
    const Context& c = *(const Context*)context;
    if (rows > TF_STREAM_MAX_ROWS) return -5;                  // few-row owners only: the many-row arena is far past the static array
    const DynLayout l = dyn_layout(c.g, rows);
    // everything but the route outputs, which the caller passes, lies in the static array
    const long long needed = l.scatter;
    if (needed > (long long)TF_STATIC_SCRATCH_BYTES || l.tiles > TF_LDS_TILES) return -5;
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device != c.device || !c.static_scratch) return -1;      // the array of the context's device
    const uint64_t base = (uint64_t)c.static_scratch;
    uint64_t p[P_DYN_COUNT] = {};
    p[P_A] = (uint64_t)input; p[P_IDS] = (uint64_t)topk_ids; p[P_WEIGHTS] = (uint64_t)topk_weights;
    p[P_PACKED] = base + l.packed; p[P_SCALES] = base + l.scales; p[P_PACKED_MIN] = 0; p[P_SCALES_MIN] = 0;
    p[P_INTER] = base + l.inter; p[P_INTER_CODES] = base + l.inter_codes; p[P_INTER_SCALES] = base + l.inter_scales;
    p[P_TASK_EXPERT] = base + l.task_expert; p[P_TASK_VALID] = base + l.task_valid; p[P_TILE_BASE] = base + l.tile_base;
    p[P_TOKEN_MAP] = base + l.token_map; p[P_TOKEN_WEIGHTS] = base + l.token_weights;
    p[P_W13] = (uint64_t)w13; p[P_S13] = (uint64_t)s13; p[P_W2] = (uint64_t)w2; p[P_S2] = (uint64_t)s2;
    p[P_SCATTER] = (uint64_t)route_output; p[P_PLAN_SCRATCH] = 0;
    const int32_t sc[S_DYN_COUNT] = {rows, rows, (int32_t)(l.tiles * l.tile_m), (int32_t)l.tiles, l.tile_m, 1};
    return launch_dynamic(c, false, p, sc, (hipStream_t)stream);
}

}  // extern "C"
