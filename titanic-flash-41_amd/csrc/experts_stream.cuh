// Few-row (decode / speculative verify) expert projections: a weight-streaming kernel family.
//
// Every active expert's prepared weights are read from HBM exactly once per step, in 1 KiB contiguous pieces (one
// 16-byte non-temporal load per lane), straight into the B operand of v_mfma_scale_f32_16x16x128_f8f6f4.  The matrix
// core decodes E2M1 / E4M3 and applies the UE8M0 block scales of both operands, so no VALU dequantization runs.  The
// activation tile (at most 16 token rows of one expert) stays in registers as the A operand for a whole tile of work.
// The hidden (K) dimension is split over the four waves of a workgroup; partial sums meet in LDS in a fixed order.
//
// Work is a flat list of items (tile, column group); the persistent grid takes equal contiguous shares, so each
// expert's weights stream once, expert-major, and consecutive items of a workgroup reuse the activation registers.
//
// Reference semantics (contract level; the reference's kernels are third-party binaries): FC1 + SwiGLU and FC2 of
// src/moe.rs:1098-1289 plan nodes, runtime/kernels/moe-runtime-m6-cache-ca-v1/manifest.json precision string.
#pragma once
#include "frontend.cuh"

#define TF_MFMA(A, B, C, BFMT, OPSEL, SA, SB) \
    __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, C, 0, BFMT, OPSEL, SA, OPSEL, SB)

struct StreamGeometry {
    int k;            // contraction length (hidden for FC1, intermediate for FC2)
    int n;            // weight rows per expert matrix that one item column group indexes into
    int act_block;    // activation scale block (32 or 128)
};

// A operand of one M tile for this wave's share of K: KS k-steps of 8 dwords, plus packed scale bytes (4 k-steps a dword).
template <int KS>
struct ATile {
    v8i a[KS];
    uint32_t scale[(KS + 3) / 4];
};

// Loads the A operand from row-major E4M3 codes [row][k] with UE8M0 scales [row][k / act_block].
// Lane (g = lane / 16, m = lane % 16): row m of the tile, bytes k = 128 ks + 64 half + 16 g ..; scale byte of K32 block
// 4 ks + g.  `row` < 0 marks an unused row (zeros).
template <int KS, int KSMAX = KS>
__device__ __forceinline__ void tf_load_a(ATile<KSMAX>& t, const uint8_t* codes, const uint8_t* scales, long long row, int k,
                                          int act_block, int ks_first, int lane) {
    const int g = lane >> 4;
#pragma unroll
    for (int q = 0; q < (KS + 3) / 4; ++q) t.scale[q] = 0x7f7f7f7fu;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int ks = ks_first + s;
        if (row >= 0) {
            const uint8_t* base = codes + row * k + ks * 128 + 16 * g;
            const u4v lo = *reinterpret_cast<const u4v*>(base);
            const u4v hi = *reinterpret_cast<const u4v*>(base + 64);
            t.a[s] = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
            const uint32_t byte = scales[row * (k / act_block) + (ks * 128 + 32 * g) / act_block];
            t.scale[s >> 2] = (t.scale[s >> 2] & ~(0xffu << (8 * (s & 3)))) | (byte << (8 * (s & 3)));
        } else {
            t.a[s] = v8i{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }
}

// One pipeline unit of streamed weights for this wave: N 16-byte loads a lane (N KiB a wave).
//   FP4 (routed): TILES weight tiles of 16 rows, KS k-steps each: d[t * KS + s].
//   FP8 (shared): TILES / 2 weight tiles, each k-step as two 16-byte planes: d[(t * KS + s) * 2 + half].
// Scale bytes travel as one dword per tile and four k-steps (byte q = k-step 4 i + q of the wave's share).
template <int TILES, int KS>
struct Unit {
    u4v d[TILES * KS];
    uint32_t scale[TILES * ((KS + 3) / 4)];
};
// FP4: words [n/16][k/128][lane][16 B], scales [n/16][k/512][lane][4 B] (byte q of a word = k-step 4 kq + q).
// A wave's k-steps start inside a scale word unless KS is a multiple of 4 (KS 1, 2: inside one word); for the other counts
// one more word is read and the two are funnel-shifted so that byte q of register i is k-step 4 i + q of the wave's share.
template <int TILES, int KS>
__device__ __forceinline__ void tf_load_fp4(Unit<TILES, KS>& u, const uint8_t* w, const uint8_t* scales, const int (&ntile)[TILES], int k,
                                            int ks_first, int lane) {
    constexpr int SW = (KS + 3) / 4;
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const u4v* src = reinterpret_cast<const u4v*>(w) + ((size_t)ntile[t] * (k / 128) + ks_first) * 64 + lane;
#pragma unroll
        for (int s = 0; s < KS; ++s) u.d[t * KS + s] = tf_stream_load(src + s * 64);
        if constexpr (KS <= 2 || KS % 4 == 0) {
            const uint32_t* sc = reinterpret_cast<const uint32_t*>(scales) + ((size_t)ntile[t] * (k / 512) + ks_first / 4) * 64 + lane;
#pragma unroll
            for (int q = 0; q < SW; ++q) u.scale[t * SW + q] = __builtin_nontemporal_load(sc + q * 64) >> (8 * (ks_first & 3));
        } else {
            const int words = k / 512, first = ks_first / 4;
            const uint32_t* sc = reinterpret_cast<const uint32_t*>(scales) + (size_t)ntile[t] * words * 64 + lane;
            uint32_t raw[SW + 1];
#pragma unroll
            for (int q = 0; q <= SW; ++q) raw[q] = __builtin_nontemporal_load(sc + (size_t)min(first + q, words - 1) * 64);   // past the row: unused
#pragma unroll
            for (int q = 0; q < SW; ++q) u.scale[t * SW + q] = __builtin_amdgcn_alignbyte(raw[q + 1], raw[q], (uint32_t)(ks_first & 3));
        }
    }
}
// FP8: bytes [n/16][k/128][half][lane][16 B]; scales row-major UE8M0 [n/bn][k/bk].  TILES counts 16-byte planes: tile = t / 2.
template <int TILES, int KS>
__device__ __forceinline__ void tf_load_fp8(Unit<TILES, KS>& u, const uint8_t* w, const uint8_t* scales, const int (&ntile)[TILES], int k,
                                            int ks_first, int lane, int bn, int bk) {
    constexpr int SW = (KS + 3) / 4;
    const int g = lane >> 4;
#pragma unroll
    for (int t = 0; t < TILES / 2; ++t) {
        const u4v* src = reinterpret_cast<const u4v*>(w) + (((size_t)ntile[t] * (k / 128) + ks_first) * 2) * 64 + lane;
#pragma unroll
        for (int s = 0; s < 2 * KS; ++s) u.d[t * 2 * KS + s] = tf_stream_load(src + s * 64);
        const uint8_t* sc = scales + (size_t)((ntile[t] * 16 + (lane & 15)) / bn) * (k / bk);
#pragma unroll
        for (int q = 0; q < SW; ++q) {
            uint32_t word = 0x7f7f7f7fu;
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (4 * q + b < KS) word = (word & ~(0xffu << (8 * b))) | ((uint32_t)sc[((ks_first + 4 * q + b) * 128 + 32 * g) / bk] << (8 * b));
            u.scale[t * SW + q] = word;
        }
    }
}
#define TF_MFMA4(A, B, C, FMT, S, SA, SB)                                              \
    switch ((S) & 3) {                                                                 \
        case 0: C = TF_MFMA(A, B, C, FMT, 0, SA, SB); break;                            \
        case 1: C = TF_MFMA(A, B, C, FMT, 1, SA, SB); break;                            \
        case 2: C = TF_MFMA(A, B, C, FMT, 2, SA, SB); break;                            \
        default: C = TF_MFMA(A, B, C, FMT, 3, SA, SB); break;                           \
    }
// Product of the A tile with weight tile `t` of a unit over the wave's k-steps.
template <bool FP8, int TILES, int KS>
__device__ __forceinline__ v4f tf_dot_unit(const ATile<KS>& a, const Unit<TILES, KS>& u, int t) {
    constexpr int SW = (KS + 3) / 4;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int sa = (int)a.scale[s >> 2], sb = (int)u.scale[t * SW + (s >> 2)];
        if constexpr (FP8) {
            const u4v lo = u.d[(t * KS + s) * 2], hi = u.d[(t * KS + s) * 2 + 1];
            const v8i bv = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
            TF_MFMA4(a.a[s], bv, acc, 0, s, sa, sb)
        } else {
            const u4v lo = u.d[t * KS + s];
            const v8i bv = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], 0, 0, 0, 0};
            TF_MFMA4(a.a[s], bv, acc, 4, s, sa, sb)
        }
    }
    return acc;
}

// Operands of one streamed projection (routed: FP4 weights through the plan; dense: FP8 weights over all rows).
struct StreamArgs {
    const uint8_t* a_codes;          // FC1: E4M3 token codes [rows][k]
    const uint8_t* a_scales;
    const uint16_t* a_bf16;          // FC2: BF16 intermediate rows [phys_row][k] (quantized in the tile prologue)
    uint8_t* q_codes;                // FC2: where the prologue stores the codes it used ([phys_row][k]), may be null
    uint8_t* q_scales;
    float min_amax;                  // quantizer flavour of the FC2 prologue
    const uint8_t* w;                // prepared weights, expert-major
    const uint8_t* ws;               // prepared scales (FP4) or row-major block scales (FP8)
    long long w_expert_stride, ws_expert_stride;
    int bn, bk;                      // FP8 weight scale block
    const int32_t* expert_tile_base; // routed: [experts + 1]; tiles = expert_tile_base[experts]
    const int32_t* task_expert;      // routed: [tile * groups]; null: dense (tile t covers rows 16 t ..)
    const int32_t* task_valid_rows;
    const int32_t* token_map;        // [tile * 16 + m] -> route index
    const float* token_weights;
    int experts, groups, topk;
    int dense_rows;
    int k, inter, hidden, act_block;
    float limit;
    uint16_t* out;                   // FC1: BF16 intermediate [phys_row][inter]; FC2: BF16 [route or row][hidden]
    uint16_t* tap;                   // FC1 dense: BF16 projections [row][2 inter] before the activation, may be null
    float* proj;                     // FC1 routed: FP32 projections [route][2 inter] (up, then gate) before the activation, may be null
    int table_tiles;                 // routed: capacity of the plan tables in tiles (phase kernels: at most TF_LDS_TILES)
};
// A workgroup walks the plan's tile table for every item; read in place that is three dependent round trips (tile count,
// the tile's expert, the tile's rows) before the first weight load can be issued.  The phase kernels copy the table into
// LDS with one round of independent loads instead (expert and row count packed in one word).
constexpr int TF_LDS_TILES = 576;       // rows <= 64, topk <= 8, experts <= 512: at most 32 + 512 tiles
struct PlanLds {
    int32_t tiles;
    uint32_t tile[TF_LDS_TILES];        // expert | valid rows << 16
};
// Block barrier inside.  `v` must be a routed operand set with table_tiles in [1, TF_LDS_TILES].
__device__ __forceinline__ void tf_plan_preload(const StreamArgs& v, PlanLds& t) {
    if (threadIdx.x == 0) t.tiles = v.expert_tile_base[v.experts];
    for (int i = threadIdx.x; i < v.table_tiles; i += blockDim.x)
        t.tile[i] = (uint32_t)v.task_expert[i * v.groups] | ((uint32_t)v.task_valid_rows[i * v.groups] << 16);
    __syncthreads();
}
struct ItemRef { int tile, j, expert, valid; };
__device__ __forceinline__ ItemRef tf_item(const StreamArgs& p, int item, int per_tile, const PlanLds& t) {
    ItemRef r;
    r.tile = item / per_tile;
    r.j = item - r.tile * per_tile;
    if (p.task_expert != nullptr) {
        const uint32_t word = t.tile[r.tile];
        r.expert = (int)(word & 0xffffu);
        r.valid = (int)(word >> 16);
    } else {
        r.expert = 0;
        r.valid = min(16, p.dense_rows - r.tile * 16);
    }
    return r;
}
__device__ __forceinline__ ItemRef tf_item(const StreamArgs& p, int item, int per_tile) {
    ItemRef r;
    r.tile = item / per_tile;
    r.j = item - r.tile * per_tile;
    if (p.task_expert != nullptr) {
        r.expert = p.task_expert[r.tile * p.groups];
        r.valid = p.task_valid_rows[r.tile * p.groups];
    } else {
        r.expert = 0;
        r.valid = min(16, p.dense_rows - r.tile * 16);
    }
    return r;
}
__device__ __forceinline__ int tf_tiles(const StreamArgs& p) {
    return p.task_expert != nullptr ? p.expert_tile_base[p.experts] : (p.dense_rows + 15) / 16;
}

// FC1 + SwiGLU.  Item = (tile, j): weight tiles j and inter / 16 + j of the expert's [2 inter][k] matrix; output
// intermediate columns 16 j .. 16 j + 15 of the tile's rows.  A pipeline unit is 2 KS KiB a wave: both tiles of an FP4
// item, or one tile of an FP8 item (units 2 item, 2 item + 1); the next unit's loads are issued before the current unit's
// products run.
// Routed (FP4): rows [0, inter) are up, [inter, 2 inter) gate; h = bf16((g * logistic(g)) * u), g = min(gate, limit),
// u = clamp(up) in FP32.  Shared (FP8): rows [0, inter) gate, then up; both rounded to BF16 first, clamped in BF16.
template <bool FP8, int KS, int WAVES = 4>
__device__ __forceinline__ void tf_fc1_items(const StreamArgs& p, int item_first, int item_last, float (*red)[2][4][64],
                                             const PlanLds& plan) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_tile = p.inter / 16, ks_first = wave * KS;
    if (item_first >= item_last) return;
    constexpr int PER_ITEM = FP8 ? 2 : 1;                    // units per item
    const int unit_first = item_first * PER_ITEM, unit_last = item_last * PER_ITEM;
    int loaded_tile = -1;
    ATile<KS> a;
    Unit<2, KS> cur, next;
    auto load_unit = [&](Unit<2, KS>& u, int unit) {
        const ItemRef r = tf_item(p, unit / PER_ITEM, per_tile, plan);
        const uint8_t* w = p.w + (size_t)r.expert * p.w_expert_stride;
        const uint8_t* ws = p.ws + (size_t)r.expert * p.ws_expert_stride;
        if constexpr (FP8) {
            const int nt[2] = {(unit & 1) * per_tile + r.j, 0};
            tf_load_fp8<2, KS>(u, w, ws, nt, p.k, ks_first, lane, p.bn, p.bk);
        } else {
            const int nt[2] = {r.j, per_tile + r.j};
            tf_load_fp4<2, KS>(u, w, ws, nt, p.k, ks_first, lane);
        }
    };
    load_unit(cur, unit_first);
    v4f first_acc = {0.f, 0.f, 0.f, 0.f};
    for (int unit = unit_first; unit < unit_last; ++unit) {
        const int item = unit / PER_ITEM;
        const ItemRef r = tf_item(p, item, per_tile, plan);
        if (r.tile != loaded_tile) {
            long long row = -1;
            if ((lane & 15) < r.valid)
                row = p.task_expert != nullptr ? p.token_map[r.tile * 16 + (lane & 15)] / p.topk : r.tile * 16 + (lane & 15);
            tf_load_a<KS>(a, p.a_codes, p.a_scales, row, p.k, p.act_block, ks_first, lane);
            loaded_tile = r.tile;
        }
        if (unit + 1 < unit_last) load_unit(next, unit + 1);
        v4f c0, c1;
        if constexpr (FP8) {
            const v4f c = tf_dot_unit<true, 2, KS>(a, cur, 0);
            if ((unit & 1) == 0) { first_acc = c; if (unit + 1 < unit_last) cur = next; continue; }
            c0 = first_acc; c1 = c;
        } else {
            c0 = tf_dot_unit<false, 2, KS>(a, cur, 0);
            c1 = tf_dot_unit<false, 2, KS>(a, cur, 1);
        }
        float (*slot)[2][4][64] = red + (item & 1) * WAVES;
#pragma unroll
        for (int i = 0; i < 4; ++i) { slot[wave][0][i][lane] = c0[i]; slot[wave][1][i][lane] = c1[i]; }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = 4 * (lane >> 4) + i;
                if (m < r.valid) {
                    float first = slot[0][0][i][lane], second = slot[0][1][i][lane];
#pragma unroll
                    for (int w2 = 1; w2 < WAVES; ++w2) {
                        first = __fadd_rn(first, slot[w2][0][i][lane]);
                        second = __fadd_rn(second, slot[w2][1][i][lane]);
                    }
                    float value;
                    const size_t row = (size_t)(r.tile * 16 + m);
                    if constexpr (FP8) {
                        const uint16_t gb = tf_to_bf16(first), ub = tf_to_bf16(second);
                        if (p.tap != nullptr) {
                            p.tap[row * 2 * p.inter + 16 * r.j + (lane & 15)] = gb;
                            p.tap[row * 2 * p.inter + p.inter + 16 * r.j + (lane & 15)] = ub;
                        }
                        const float hi = tf_bf16(tf_to_bf16(p.limit)), lo = tf_bf16(tf_to_bf16(-p.limit));
                        const float g = fminf(tf_bf16(gb), hi);
                        const float u = fminf(fmaxf(tf_bf16(ub), lo), hi);
                        value = __fmul_rn(g / __fadd_rn(1.0f, tf_exp(-g)), u);
                    } else {
                        if (p.proj != nullptr) {
                            float* at = p.proj + (size_t)p.token_map[row] * 2 * p.inter + 16 * r.j + (lane & 15);
                            at[0] = first;
                            at[p.inter] = second;
                        }
                        const float g = fminf(second, p.limit);
                        const float u = fminf(p.limit, fmaxf(-p.limit, first));
                        value = __fmul_rn(__fmul_rn(g, tf_logistic(g)), u);
                    }
                    if (!FP8 || p.out != nullptr) p.out[row * p.inter + 16 * r.j + (lane & 15)] = tf_to_bf16(value);      // dense product alone: only the tap
                }
            }
        }
        if (unit + 1 < unit_last) cur = next;
    }
}

// FC2.  Routed item = (tile, j): weight tiles 4 j .. 4 j + 3 of the expert's [hidden][k] FP4 matrix (64 output columns);
// shared item: tiles 2 j, 2 j + 1 of the FP8 matrix (32 columns): 4 KS KiB a wave either way.  The prologue of a tile
// quantizes its BF16 intermediate rows (MXFP8, `act_block` columns a block) into LDS; every wave then keeps its K share
// as the A operand.  Routed: out[route][c] = bf16(acc * token_weight); dense: out[row][c] = bf16(acc).
template <bool FP8, int KS>
__device__ __forceinline__ void tf_fc2_items(const StreamArgs& p, int item_first, int item_last, float (*red)[2][4][64],
                                             uint8_t* s_codes, uint8_t* s_scales, const PlanLds& plan) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int COLS = FP8 ? 32 : 64, NT = COLS / 16;
    const int per_tile = p.hidden / COLS, ks_first = wave * KS;
    if (item_first >= item_last) return;
    int loaded_tile = -1;
    int route[4] = {0, 0, 0, 0};
    float share[4] = {0.f, 0.f, 0.f, 0.f};
    ATile<KS> a;
    Unit<4, KS> cur, next;
    auto load_unit = [&](Unit<4, KS>& u, int item) {
        const ItemRef r = tf_item(p, item, per_tile, plan);
        const uint8_t* w = p.w + (size_t)r.expert * p.w_expert_stride;
        const uint8_t* ws = p.ws + (size_t)r.expert * p.ws_expert_stride;
        if constexpr (FP8) {
            const int nt[4] = {2 * r.j, 2 * r.j + 1, 0, 0};
            tf_load_fp8<4, KS>(u, w, ws, nt, p.k, ks_first, lane, p.bn, p.bk);
        } else {
            const int nt[4] = {4 * r.j, 4 * r.j + 1, 4 * r.j + 2, 4 * r.j + 3};
            tf_load_fp4<4, KS>(u, w, ws, nt, p.k, ks_first, lane);
        }
    };
    load_unit(cur, item_first);
    for (int item = item_first; item < item_last; ++item) {
        const ItemRef r = tf_item(p, item, per_tile, plan);
        if (r.tile != loaded_tile) {
            if (p.task_expert != nullptr) {      // where rows 4 (lane / 16) + i of the tile go, and their weights
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int m = 4 * (lane >> 4) + i;
                    if (m < r.valid) { route[i] = p.token_map[r.tile * 16 + m]; share[i] = p.token_weights[r.tile * 16 + m]; }
                }
            }
            __syncthreads();
            // quantize rows [0, valid) of the tile: 8 values a lane-step, groups of act_block / 8 lanes.  Four steps' loads are
            // requested together (a step at a time, each row would cost a round trip of its own); a wave's 64 steps are all
            // inside the tile's rows or all outside (k / 8 is a multiple of 64)
            const int per_row = p.k >> 3, group_lanes = p.act_block >> 3, total = r.valid * per_row;
            for (int q0 = threadIdx.x; q0 < total; q0 += 4 * blockDim.x) {
                u4v wv[4];
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int q = min(q0 + b * (int)blockDim.x, total - 1), m = q / per_row, c8 = q - m * per_row;
                    wv[b] = reinterpret_cast<const u4v*>(p.a_bf16 + (size_t)(r.tile * 16 + m) * p.k)[c8];
                }
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int q = q0 + b * (int)blockDim.x;
                    if (q >= total) break;
                    const int m = q / per_row, c8 = q - m * per_row;
                    float v[8];
#pragma unroll
                    for (int i = 0; i < 4; ++i) { v[2 * i] = tf_bf16_lo(wv[b][i]); v[2 * i + 1] = tf_bf16_hi(wv[b][i]); }
                    const float amax = tf_group_amax(v, group_lanes);
                    const Quant8 c = tf_quant8(v, amax, p.min_amax);
                    reinterpret_cast<u2v*>(s_codes + (size_t)m * p.k)[c8] = u2v{c.lo, c.hi};
                    if ((c8 & (group_lanes - 1)) == 0) s_scales[m * (p.k / p.act_block) + c8 / group_lanes] = (uint8_t)c.exponent;
                    if (p.q_codes != nullptr && r.j == 0) {
                        reinterpret_cast<u2v*>(p.q_codes + (size_t)(r.tile * 16 + m) * p.k)[c8] = u2v{c.lo, c.hi};
                        if ((c8 & (group_lanes - 1)) == 0)
                            p.q_scales[(size_t)(r.tile * 16 + m) * (p.k / p.act_block) + c8 / group_lanes] = (uint8_t)c.exponent;
                    }
                }
            }
            __syncthreads();
            tf_load_a<KS>(a, s_codes, s_scales, (lane & 15) < r.valid ? (lane & 15) : -1, p.k, p.act_block, ks_first, lane);
            loaded_tile = r.tile;
        }
        if (item + 1 < item_last) load_unit(next, item + 1);
        // the partial sums of consecutive items alternate between two sets of LDS slots, so one barrier an item is enough:
        // a set is written again two items later, behind the next item's barrier
        float (*set)[2][4][64] = red + (item & 1) * 8;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const v4f c = tf_dot_unit<FP8, 4, KS>(a, cur, t);
#pragma unroll
            for (int i = 0; i < 4; ++i) set[(t >> 1) * 4 + wave][t & 1][i][lane] = c[i];
        }
        __syncthreads();
        // wave w finishes 16-column tile w of the item (routed: 4 tiles; shared: 2)
        if (wave < NT) {
            float (*slot)[2][4][64] = set + (wave >> 1) * 4;
            const int which = wave & 1;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = 4 * (lane >> 4) + i;
                if (m < r.valid) {
                    float acc = slot[0][which][i][lane];
#pragma unroll
                    for (int w2 = 1; w2 < 4; ++w2) acc = __fadd_rn(acc, slot[w2][which][i][lane]);
                    const int col = COLS * r.j + 16 * wave + (lane & 15);
                    if (p.task_expert != nullptr) {
                        p.out[(size_t)route[i] * p.hidden + col] = tf_to_bf16(__fmul_rn(acc, share[i]));
                    } else {
                        p.out[(size_t)(r.tile * 16 + m) * p.hidden + col] = tf_to_bf16(acc);
                    }
                }
            }
        }
        if (item + 1 < item_last) cur = next;
    }
}

// Persistent launch of one phase over the routed experts and, optionally, the shared expert (`shared.w == nullptr`: routed
// only; `routed.w == nullptr`: dense only).  Every item costs the same bytes (a shared FC1 item counts twice), so workgroup
// b of G takes the cost range [b C / G, (b + 1) C / G) of the list "routed items, then shared items" (the second phase: shared first).  block = 64 WAVES:
// four waves, two workgroups a CU, for K <= 4,096; eight waves, one workgroup a CU, above (a wave's share of K stays at
// most eight k-steps: what the registers hold of the A tile and a unit of weights).
template <int KSR, int KSS, int WAVES = 4>
__global__ void __launch_bounds__(64 * WAVES, WAVES == 4 ? 2 : 1) tf_phase1_stream(const StreamArgs routed, const StreamArgs shared) {
    __shared__ float red[2 * WAVES][2][4][64];
    __shared__ PlanLds plan;
    if (routed.w) tf_plan_preload(routed, plan);
    const long long r_items = routed.w ? (long long)plan.tiles * (routed.inter / 16) : 0;
    const long long s_units = shared.w ? (long long)tf_tiles(shared) * (shared.inter / 16) * 2 : 0;
    const long long total = r_items + s_units;
    // equal shares for as many workgroups as fill whole rounds: with every workgroup of the grid taking floor or ceil of
    // total / grid items, the last round runs on a part of the chip that is too small to keep the memory system busy
    const long long rounds = (total + gridDim.x - 1) / gridDim.x, active = rounds > 0 ? (total + rounds - 1) / rounds : 0;
    if ((long long)blockIdx.x >= active) return;
    const long long lo = total * blockIdx.x / active, hi = total * (blockIdx.x + 1) / active;
    if (lo < r_items) tf_fc1_items<false, KSR, WAVES>(routed, (int)lo, (int)(hi < r_items ? hi : r_items), red, plan);
    if (hi > r_items) {
        const long long a = (lo > r_items ? lo - r_items : 0), b = hi - r_items;
        __syncthreads();
        tf_fc1_items<true, KSS, WAVES>(shared, (int)((a + 1) / 2), (int)((b + 1) / 2), red, plan);
    }
}
template <int KSR, int KSS>
__global__ void __launch_bounds__(256, 2) tf_phase2_stream(const StreamArgs routed, const StreamArgs shared) {
    __shared__ float red[16][2][4][64];
    extern __shared__ uint8_t dyn[];
    __shared__ PlanLds plan;
    if (routed.w) tf_plan_preload(routed, plan);
    const long long r_items = routed.w ? (long long)plan.tiles * (routed.hidden / 64) : 0;
    const long long s_items = shared.w ? (long long)tf_tiles(shared) * (shared.hidden / 32) : 0;
    // Equal cost shares of the list "shared items, then routed items", in quarter items.  Every item streams the same bytes; a
    // shared item of an owner with more than eight rows counts a quarter more: its workgroup quantizes a row tile that is full
    // or nearly so (four rounds of loads instead of one or two) for the four to six items it takes, and the launch ends with
    // the slowest workgroup.  An item belongs to the workgroup whose cost range holds its start.  (Dealing the last items out
    // by an atomic counter instead, to whichever workgroup is done first, was measured: the device-scope atomics travel the
    // same congested request path as the weights, and 512 of them at the workgroups' exits alone cost 1.5 us.)
    const long long cs = 4 + (shared.w && shared.dense_rows > 8 ? 1 : 0);
    const long long s_cost = cs * s_items, cost = s_cost + 4 * r_items;
    const long long lo = cost * blockIdx.x / gridDim.x, hi = cost * (blockIdx.x + 1) / gridDim.x;
    const long long s_lo = min(s_items, (lo + cs - 1) / cs), s_hi = min(s_items, (hi + cs - 1) / cs);
    const long long r_lo = lo > s_cost ? min(r_items, (lo - s_cost + 3) / 4) : 0, r_hi = hi > s_cost ? min(r_items, (hi - s_cost + 3) / 4) : 0;
    const int kmax = routed.w && (!shared.w || routed.k > shared.k) ? routed.k : shared.k;
    if (s_lo < s_hi) tf_fc2_items<true, KSS>(shared, (int)s_lo, (int)s_hi, red, dyn, dyn + 16 * (size_t)kmax, plan);
    if (r_lo < r_hi) tf_fc2_items<false, KSR>(routed, (int)r_lo, (int)r_hi, red, dyn, dyn + 16 * (size_t)kmax, plan);
}

// The experts' front-end with the shared expert's first projection in the same launch (few-row owners, hidden <= 5,120).
// The front-end proper keeps a handful of workgroups busy for its whole length (gate product, routing, plan: a chain of
// dependent steps) while the rest of the chip idles, or idles again once the logit blocks are done; the shared expert does
// not depend on the routing, so its up / gate weights (two thirds of its bytes) stream here instead of inside the routed
// experts' first launch, whose length they would add to.  `shared_blocks` = intermediate / 16 further blocks (the highest
// block ids: dispatched last; nothing waits for them), one item (16 intermediate columns, every row tile of the owner) each:
// waves 0 - 3 take the item's gate tile and waves 4 - 7 its up tile (a K quarter each), loaded once; per row tile the block
// takes the token rows' codes (shared flavour) -- one row tile: it quantizes the few rows itself, into LDS, and waits for
// nobody; more: from the launch's quantizer blocks -- and wave 0 finishes the tile as tf_fc1_items does (same summation
// order, same activation).
template <int KS, bool HANDOFF>
__device__ __forceinline__ void tf_front_shared_item(const StreamArgs& p, const uint16_t* __restrict__ all_rows, int all_row_count, uint8_t* s_pool,
                                                     int item, uint32_t* sync, int quant_blocks, int shared_blocks, int spin_limit) {
    const int k = p.k, per_row = k >> 3, group_lanes = p.act_block >> 3;
    const int per_tile = p.inter / 16, tiles = (all_row_count + 15) >> 4;
    uint8_t* s_codes = s_pool;                                        // [rows][k]             (at most 64 KiB)
    uint8_t* s_scales = s_pool + 16 * TF_FRONT_SHARED_MAX_K;          // [rows][k / act_block]
    // [row tile parity][gate / up][wave][i][lane]: 2 x 8 KiB; consecutive row tiles alternate, so one barrier a tile is enough
    float (*red)[2][4][4][64] = reinterpret_cast<float (*)[2][4][4][64]>(s_pool + 16 * TF_FRONT_SHARED_MAX_K + 16 * (TF_FRONT_SHARED_MAX_K / 32));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = wave >> 2, quarter = wave & 3, ks_first = quarter * KS;
    // `quant_blocks` > 0: the launch's quantizer blocks publish the rows' codes (shared flavour) and count themselves in; this
    // block waits for all of them (a bounded wait: they have lower block ids, none of them waits for anything) and reads its
    // operand from their output instead of quantizing every row again.  Should the bound expire, or have expired in an earlier
    // launch (the arrival word may then hold that launch's late arrivals), it quantizes them itself.
    // The wait comes before the first weight request: a workgroup barrier waits for every load in flight.
    bool ready = false;
    if constexpr (HANDOFF) {
        __shared__ int s_ready;
        if (threadIdx.x == 0) {
            int ok = 0;
            if (tf_sync_trusted(sync)) {
                for (int spin = 0; spin < spin_limit; ++spin) {
                    if (__hip_atomic_load(sync + 32 * TF_SYNC_QUANT_DONE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (uint32_t)quant_blocks) { ok = 1; break; }
                    __builtin_amdgcn_s_sleep(2);
                }
                if (!ok) tf_sync_give_up(sync);
            }
            s_ready = ok;
        }
        __syncthreads();
        ready = s_ready != 0;
    }
    // the weights first: they come from HBM, the rows from L2; every row tile of the owner uses them
    Unit<2, KS> u;
    const int nt[2] = {half * per_tile + item, 0};
    tf_load_fp8<2, KS>(u, p.w, p.ws, nt, k, ks_first, lane, p.bn, p.bk);
    for (int tile = 0; tile < tiles; ++tile) {
        const int rows = min(16, all_row_count - 16 * tile);                // of this tile
        ATile<KS> a;
        if (HANDOFF && ready) {
            // the tile's codes and scales, published by the quantizer blocks, through LDS: consecutive lanes take consecutive
            // 8-byte pieces (device-scope loads come from beyond this XCD's L2; as A-fragment gathers, 8 bytes from 64 places
            // an instruction, they took 20 us a block).  The previous tile's operand left LDS before that tile's barrier below.
            const unsigned long long* codes = reinterpret_cast<const unsigned long long*>(p.a_codes + (size_t)tile * 16 * k);
            const uint32_t* scale_words = reinterpret_cast<const uint32_t*>(p.a_scales + (size_t)tile * 16 * (k / p.act_block));
            const int pieces = rows * (k >> 3), words = rows * (k / p.act_block) >> 2;         // k / act_block is a multiple of 4
            for (int q = threadIdx.x; q < pieces; q += blockDim.x)
                reinterpret_cast<unsigned long long*>(s_codes)[q] = __hip_atomic_load(codes + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            for (int q = threadIdx.x; q < words; q += blockDim.x)
                reinterpret_cast<uint32_t*>(s_scales)[q] = __hip_atomic_load(scale_words + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            tf_load_a<KS>(a, s_codes, s_scales, (lane & 15) < rows ? (lane & 15) : -1, k, p.act_block, ks_first, lane);
        } else {
            // (the previous tile's operand left LDS before that tile's barrier below)
            const uint16_t* input = all_rows + (size_t)tile * 16 * k;
            const int total = rows * per_row, padded = (total + 63) & ~63;
            for (int q = threadIdx.x; q < padded; q += blockDim.x) {
                const bool on = q < total;
                float v[8];
                if (on) {
                    const u4v wv = reinterpret_cast<const u4v*>(input)[q];
#pragma unroll
                    for (int i = 0; i < 4; ++i) { v[2 * i] = tf_bf16_lo(wv[i]); v[2 * i + 1] = tf_bf16_hi(wv[i]); }
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[i] = 0.f;
                }
                const float amax = tf_group_amax(v, group_lanes);
                if (!on) continue;
                const Quant8 c = tf_quant8(v, amax, 1e-4f);
                reinterpret_cast<u2v*>(s_codes)[q] = u2v{c.lo, c.hi};
                if ((q & (group_lanes - 1)) == 0) s_scales[q / group_lanes] = (uint8_t)c.exponent;
            }
            __syncthreads();
            tf_load_a<KS>(a, s_codes, s_scales, (lane & 15) < rows ? (lane & 15) : -1, k, p.act_block, ks_first, lane);
        }
        const v4f c = tf_dot_unit<true, 2, KS>(a, u, 0);
        float (*set)[4][4][64] = red[tile & 1];
#pragma unroll
        for (int i = 0; i < 4; ++i) set[half][quarter][i][lane] = c[i];
        __syncthreads();
        if (wave != 0) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = 4 * (lane >> 4) + i;
            if (m < rows) {
                float first = set[0][0][i][lane], second = set[1][0][i][lane];
#pragma unroll
                for (int w2 = 1; w2 < 4; ++w2) {
                    first = __fadd_rn(first, set[0][w2][i][lane]);
                    second = __fadd_rn(second, set[1][w2][i][lane]);
                }
                const uint16_t gb = tf_to_bf16(first), ub = tf_to_bf16(second);
                const size_t row = (size_t)(tile * 16 + m);
                if (p.tap != nullptr) {
                    p.tap[row * 2 * p.inter + 16 * item + (lane & 15)] = gb;
                    p.tap[row * 2 * p.inter + p.inter + 16 * item + (lane & 15)] = ub;
                }
                const float hi = tf_bf16(tf_to_bf16(p.limit)), lo = tf_bf16(tf_to_bf16(-p.limit));
                const float g = fminf(tf_bf16(gb), hi);
                const float up = fminf(fmaxf(tf_bf16(ub), lo), hi);
                const float value = __fmul_rn(g / __fadd_rn(1.0f, tf_exp(-g)), up);
                p.out[row * p.inter + 16 * item + (lane & 15)] = tf_to_bf16(value);
            }
        }
    }
    // every wave's operands have been consumed (the last tile's barrier): the last item block to get here empties both arrival
    // words for the next launch
    if (HANDOFF && ready && threadIdx.x == 0 && atomicAdd(sync + 32 * TF_SYNC_SHARED_PASSED, 1u) == (uint32_t)(shared_blocks - 1)) {
        __hip_atomic_store(sync + 32 * TF_SYNC_QUANT_DONE, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(sync + 32 * TF_SYNC_SHARED_PASSED, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

extern "C" __global__ void __launch_bounds__(512) ca_moe_route_frontend_shared(
    const uint16_t* input, int32_t* ids, float* weights, uint8_t* packed, uint8_t* scales, int32_t* token_map,
    float* token_weights, int32_t* task_expert, int32_t* task_valid_rows, int32_t* expert_tile_base,
    float* logits, const float* bias, const float* bias_alt, const long long* tokens, const int32_t* live,
    const int32_t* padding, int32_t rows, int32_t topk, int32_t experts, int32_t cols, int32_t groups, int32_t tile_m,
    int32_t owner_rows, int32_t act_block, uint8_t* packed_min, uint8_t* scales_min, int32_t scoring,
    float route_scale, long long alt_token, const uint16_t* gate_w, uint32_t* sync, int32_t logit_blocks, const StreamArgs shared,
    int32_t shared_blocks, int32_t spin_limit) {
    __shared__ __attribute__((aligned(16))) uint8_t s_pool[TF_FRONT_POOL_BYTES];
    const int grid_blocks = (int)gridDim.x - shared_blocks;
    // more than one row tile: the item blocks take the rows' codes from the launch's quantizer blocks (one tile: they quantize the
    // few rows themselves and wait for nobody)
    const bool handoff = rows > 16 && packed_min != nullptr && scales_min != nullptr && shared.a_codes == packed_min && shared.a_scales == scales_min;
    if ((int)blockIdx.x >= grid_blocks) {
        const int block = (int)blockIdx.x - grid_blocks;
        const int quant_blocks = grid_blocks - logit_blocks - 1;
        if (handoff) {
            switch (shared.k) {
                case 512: tf_front_shared_item<1, true>(shared, input, rows, s_pool, block, sync, quant_blocks, shared_blocks, spin_limit); break;
                case 1024: tf_front_shared_item<2, true>(shared, input, rows, s_pool, block, sync, quant_blocks, shared_blocks, spin_limit); break;
                case 1536: tf_front_shared_item<3, true>(shared, input, rows, s_pool, block, sync, quant_blocks, shared_blocks, spin_limit); break;
                case 2048: tf_front_shared_item<4, true>(shared, input, rows, s_pool, block, sync, quant_blocks, shared_blocks, spin_limit); break;
                case 2560: tf_front_shared_item<5, true>(shared, input, rows, s_pool, block, sync, quant_blocks, shared_blocks, spin_limit); break;
                case 3072: tf_front_shared_item<6, true>(shared, input, rows, s_pool, block, sync, quant_blocks, shared_blocks, spin_limit); break;
                case 3584: tf_front_shared_item<7, true>(shared, input, rows, s_pool, block, sync, quant_blocks, shared_blocks, spin_limit); break;
                case 4096: tf_front_shared_item<8, true>(shared, input, rows, s_pool, block, sync, quant_blocks, shared_blocks, spin_limit); break;
                case 5120: tf_front_shared_item<10, true>(shared, input, rows, s_pool, block, sync, quant_blocks, shared_blocks, spin_limit); break;
                default: break;
            }
        } else {
            switch (shared.k) {
                case 512: tf_front_shared_item<1, false>(shared, input, rows, s_pool, block, sync, 0, shared_blocks, spin_limit); break;
                case 1024: tf_front_shared_item<2, false>(shared, input, rows, s_pool, block, sync, 0, shared_blocks, spin_limit); break;
                case 1536: tf_front_shared_item<3, false>(shared, input, rows, s_pool, block, sync, 0, shared_blocks, spin_limit); break;
                case 2048: tf_front_shared_item<4, false>(shared, input, rows, s_pool, block, sync, 0, shared_blocks, spin_limit); break;
                case 2560: tf_front_shared_item<5, false>(shared, input, rows, s_pool, block, sync, 0, shared_blocks, spin_limit); break;
                case 3072: tf_front_shared_item<6, false>(shared, input, rows, s_pool, block, sync, 0, shared_blocks, spin_limit); break;
                case 3584: tf_front_shared_item<7, false>(shared, input, rows, s_pool, block, sync, 0, shared_blocks, spin_limit); break;
                case 4096: tf_front_shared_item<8, false>(shared, input, rows, s_pool, block, sync, 0, shared_blocks, spin_limit); break;
                case 5120: tf_front_shared_item<10, false>(shared, input, rows, s_pool, block, sync, 0, shared_blocks, spin_limit); break;
                default: break;
            }
        }
        return;
    }
    tf_route_frontend(input, ids, weights, packed, scales, token_map, token_weights, task_expert, task_valid_rows, expert_tile_base, logits, bias,
                      bias_alt, tokens, live, padding, rows, topk, experts, cols, groups, tile_m, owner_rows, act_block, packed_min, scales_min,
                      scoring, route_scale, alt_token, gate_w, sync, logit_blocks, grid_blocks, s_pool, spin_limit, handoff);
}

