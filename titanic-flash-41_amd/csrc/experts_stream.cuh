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
template <int KS>
__device__ __forceinline__ void tf_load_a(ATile<KS>& t, const uint8_t* codes, const uint8_t* scales, long long row, int k,
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

// B operand of one 16-row weight tile for this wave's KS k-steps.
template <int KS, bool FP8>
struct BTile {
    u4v lo[KS];
    u4v hi[FP8 ? KS : 1];
    uint32_t scale[(KS + 3) / 4];
};
// FP4: words [n/16][k/128][lane][16 B], scales [n/16][k/512][lane][4 B] (byte q of a word = k-step 4 kq + q).
// FP8: bytes [n/16][k/128][half][lane][16 B]; scales row-major UE8M0 [n/bn][k/bk].
// KS is 1, 2 or a multiple of 4, so a wave's k-steps never straddle a scale word.
template <int KS, bool FP8>
__device__ __forceinline__ void tf_load_b(BTile<KS, FP8>& b, const uint8_t* w, const uint8_t* scales, int ntile, int k,
                                          int ks_first, int lane, int bn, int bk) {
    if constexpr (FP8) {
        const u4v* src = reinterpret_cast<const u4v*>(w) + (((size_t)ntile * (k / 128) + ks_first) * 2) * 64 + lane;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            b.lo[s] = tf_stream_load(src + (s * 2) * 64);
            b.hi[s] = tf_stream_load(src + (s * 2 + 1) * 64);
        }
        const int row = ntile * 16 + (lane & 15), g = lane >> 4;
#pragma unroll
        for (int q = 0; q < (KS + 3) / 4; ++q) b.scale[q] = 0x7f7f7f7fu;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const uint32_t byte = scales[(size_t)(row / bn) * (k / bk) + ((ks_first + s) * 128 + 32 * g) / bk];
            b.scale[s >> 2] = (b.scale[s >> 2] & ~(0xffu << (8 * (s & 3)))) | (byte << (8 * (s & 3)));
        }
    } else {
        const u4v* src = reinterpret_cast<const u4v*>(w) + ((size_t)ntile * (k / 128) + ks_first) * 64 + lane;
#pragma unroll
        for (int s = 0; s < KS; ++s) b.lo[s] = tf_stream_load(src + s * 64);
        const uint32_t* sc = reinterpret_cast<const uint32_t*>(scales) + ((size_t)ntile * (k / 512) + ks_first / 4) * 64 + lane;
#pragma unroll
        for (int q = 0; q < (KS + 3) / 4; ++q) b.scale[q] = __builtin_nontemporal_load(sc + q * 64) >> (8 * (ks_first & 3));
    }
}
template <int KS, bool FP8>
__device__ __forceinline__ v4f tf_dot_tile(const ATile<KS>& a, const BTile<KS, FP8>& b) {
    v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        v8i bv;
        if constexpr (FP8) bv = v8i{(int)b.lo[s][0], (int)b.lo[s][1], (int)b.lo[s][2], (int)b.lo[s][3], (int)b.hi[s][0],
                                    (int)b.hi[s][1], (int)b.hi[s][2], (int)b.hi[s][3]};
        else bv = v8i{(int)b.lo[s][0], (int)b.lo[s][1], (int)b.lo[s][2], (int)b.lo[s][3], 0, 0, 0, 0};
        const int sa = (int)a.scale[s >> 2], sb = (int)b.scale[s >> 2];
        constexpr int F = FP8 ? 0 : 4;
        switch (s & 3) {
            case 0: acc = TF_MFMA(a.a[s], bv, acc, F, 0, sa, sb); break;
            case 1: acc = TF_MFMA(a.a[s], bv, acc, F, 1, sa, sb); break;
            case 2: acc = TF_MFMA(a.a[s], bv, acc, F, 2, sa, sb); break;
            default: acc = TF_MFMA(a.a[s], bv, acc, F, 3, sa, sb); break;
        }
    }
    return acc;
}

// Description of one streamed projection over a list of M tiles.
struct StreamArgs {
    // activations: E4M3 codes [rows][k] + scales, or (FC2) BF16 rows to quantize first
    const uint8_t* a_codes;
    const uint8_t* a_scales;
    const uint16_t* a_bf16;          // FC2: BF16 intermediate rows [phys_row][k] (quantized in the prologue)
    uint8_t* q_codes;                // FC2: where the prologue stores the codes it used ([phys_row][k]), may be null
    uint8_t* q_scales;
    float min_amax;                  // quantizer flavour of the FC2 prologue
    // weights
    const uint8_t* w;                // prepared weights, expert-major
    const uint8_t* ws;               // prepared scales (FP4) or row-major block scales (FP8)
    long long w_expert_stride, ws_expert_stride;
    int bn, bk;                      // FP8 weight scale block
    // plan (routed) or null (dense: tile t covers rows 16 t ..)
    const int32_t* expert_tile_base; // [experts + 1]; tiles = expert_tile_base[experts]
    const int32_t* task_expert;      // [tile * groups]
    const int32_t* task_valid_rows;
    const int32_t* token_map;        // [tile * 16 + m] -> route index
    const float* token_weights;
    int experts, groups, topk;
    int dense_rows;                  // dense: number of rows
    // shapes
    int k, inter, hidden, act_block;
    float limit;
    // outputs
    uint16_t* out;                   // FC1: BF16 intermediate [phys_row][inter]; FC2: BF16 [route or row][hidden]
    uint16_t* tap;                   // FC1 dense: BF16 projections [row][2 inter] before the activation, may be null
};
struct ItemRef { int tile, j, expert, valid; };
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

// FC1 + SwiGLU.  Item = (tile, j): weight tiles j ("up" for routed, "gate" for shared) and inter / 16 + j of the
// expert's [2 inter][k] matrix; output intermediate columns 16 j .. 16 j + 15 of the tile's rows.
// Routed (FP4): rows [0, inter) are up, [inter, 2 inter) gate; h = bf16((g * logistic(g)) * u), g = min(gate, limit),
// u = clamp(up) in FP32.  Shared (FP8): rows [0, inter) gate, then up; both rounded to BF16 first, clamped in BF16.
// The weights of the next item are requested before the current item's products run.
template <bool FP8, int KS>
__device__ __forceinline__ void tf_fc1_items(const StreamArgs& p, int item_first, int item_last, float (*red)[2][4][64]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_tile = p.inter / 16, ks_first = wave * KS;
    if (item_first >= item_last) return;
    int loaded_tile = -1;
    ATile<KS> a;
    BTile<KS, FP8> b0, b1;
    ItemRef cur = tf_item(p, item_first, per_tile);
    tf_load_b<KS, FP8>(b0, p.w + (size_t)cur.expert * p.w_expert_stride, p.ws + (size_t)cur.expert * p.ws_expert_stride,
                       cur.j, p.k, ks_first, lane, p.bn, p.bk);
    tf_load_b<KS, FP8>(b1, p.w + (size_t)cur.expert * p.w_expert_stride, p.ws + (size_t)cur.expert * p.ws_expert_stride,
                       per_tile + cur.j, p.k, ks_first, lane, p.bn, p.bk);
    for (int item = item_first; item < item_last; ++item) {
        if (cur.tile != loaded_tile) {
            long long row = -1;
            if ((lane & 15) < cur.valid)
                row = p.task_expert != nullptr ? p.token_map[cur.tile * 16 + (lane & 15)] / p.topk : cur.tile * 16 + (lane & 15);
            tf_load_a<KS>(a, p.a_codes, p.a_scales, row, p.k, p.act_block, ks_first, lane);
            loaded_tile = cur.tile;
        }
        BTile<KS, FP8> n0, n1;
        ItemRef next = cur;
        if (item + 1 < item_last) {
            next = tf_item(p, item + 1, per_tile);
            const uint8_t* w = p.w + (size_t)next.expert * p.w_expert_stride;
            const uint8_t* ws = p.ws + (size_t)next.expert * p.ws_expert_stride;
            tf_load_b<KS, FP8>(n0, w, ws, next.j, p.k, ks_first, lane, p.bn, p.bk);
            tf_load_b<KS, FP8>(n1, w, ws, per_tile + next.j, p.k, ks_first, lane, p.bn, p.bk);
        }
        const v4f c0 = tf_dot_tile<KS, FP8>(a, b0), c1 = tf_dot_tile<KS, FP8>(a, b1);
        float (*slot)[2][4][64] = red + (item & 1) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) { slot[wave][0][i][lane] = c0[i]; slot[wave][1][i][lane] = c1[i]; }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = 4 * (lane >> 4) + i;
                if (m < cur.valid) {
                    float first = slot[0][0][i][lane], second = slot[0][1][i][lane];
#pragma unroll
                    for (int w2 = 1; w2 < 4; ++w2) {
                        first = __fadd_rn(first, slot[w2][0][i][lane]);
                        second = __fadd_rn(second, slot[w2][1][i][lane]);
                    }
                    float value;
                    const size_t row = (size_t)(cur.tile * 16 + m);
                    if constexpr (FP8) {
                        const uint16_t gb = tf_to_bf16(first), ub = tf_to_bf16(second);
                        if (p.tap != nullptr) {
                            p.tap[row * 2 * p.inter + 16 * cur.j + (lane & 15)] = gb;
                            p.tap[row * 2 * p.inter + p.inter + 16 * cur.j + (lane & 15)] = ub;
                        }
                        const float hi = tf_bf16(tf_to_bf16(p.limit)), lo = tf_bf16(tf_to_bf16(-p.limit));
                        const float g = fminf(tf_bf16(gb), hi);
                        const float u = fminf(fmaxf(tf_bf16(ub), lo), hi);
                        value = __fmul_rn(g / __fadd_rn(1.0f, tf_exp(-g)), u);
                    } else {
                        const float g = fminf(second, p.limit);
                        const float u = fminf(p.limit, fmaxf(-p.limit, first));
                        value = __fmul_rn(__fmul_rn(g, tf_logistic(g)), u);
                    }
                    p.out[row * p.inter + 16 * cur.j + (lane & 15)] = tf_to_bf16(value);
                }
            }
        }
        if (item + 1 < item_last) { b0 = n0; b1 = n1; }
        cur = next;
    }
}

// FC2.  Item = (tile, j): weight tiles 4 j .. 4 j + 3 of the expert's [hidden][k] matrix (64 output columns).  The
// prologue of a tile quantizes its BF16 intermediate rows (MXFP8, `act_block` columns a block) into LDS; every wave then
// keeps its K share as the A operand.  Routed: out[route][c] = bf16(acc * token_weight); dense: out[row][c] = bf16(acc).
template <bool FP8, int KS>
__device__ __forceinline__ void tf_fc2_items(const StreamArgs& p, int item_first, int item_last, float (*red)[2][4][64],
                                             uint8_t* s_codes, uint8_t* s_scales) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_tile = p.hidden / 64, ks_first = wave * KS;
    if (item_first >= item_last) return;
    int loaded_tile = -1;
    ATile<KS> a;
    BTile<KS, FP8> b[4];
    ItemRef cur = tf_item(p, item_first, per_tile);
#pragma unroll
    for (int t = 0; t < 4; ++t)
        tf_load_b<KS, FP8>(b[t], p.w + (size_t)cur.expert * p.w_expert_stride, p.ws + (size_t)cur.expert * p.ws_expert_stride,
                           4 * cur.j + t, p.k, ks_first, lane, p.bn, p.bk);
    for (int item = item_first; item < item_last; ++item) {
        if (cur.tile != loaded_tile) {
            __syncthreads();
            // quantize rows [0, valid) of the tile: 8 values a lane-step, groups of act_block / 8 lanes
            const int per_row = p.k >> 3, group_lanes = p.act_block >> 3;
            for (int q = threadIdx.x; q < cur.valid * per_row; q += blockDim.x) {
                const int m = q / per_row, c8 = q - m * per_row;
                const u4v wv = reinterpret_cast<const u4v*>(p.a_bf16 + (size_t)(cur.tile * 16 + m) * p.k)[c8];
                float v[8];
#pragma unroll
                for (int i = 0; i < 4; ++i) { v[2 * i] = tf_bf16_lo(wv[i]); v[2 * i + 1] = tf_bf16_hi(wv[i]); }
                const float amax = tf_group_amax(v, group_lanes);
                const Quant8 c = tf_quant8(v, amax, p.min_amax);
                reinterpret_cast<u2v*>(s_codes + (size_t)m * p.k)[c8] = u2v{c.lo, c.hi};
                if ((c8 & (group_lanes - 1)) == 0) s_scales[m * (p.k / p.act_block) + c8 / group_lanes] = (uint8_t)c.exponent;
                if (p.q_codes != nullptr && cur.j == 0) {
                    reinterpret_cast<u2v*>(p.q_codes + (size_t)(cur.tile * 16 + m) * p.k)[c8] = u2v{c.lo, c.hi};
                    if ((c8 & (group_lanes - 1)) == 0)
                        p.q_scales[(size_t)(cur.tile * 16 + m) * (p.k / p.act_block) + c8 / group_lanes] = (uint8_t)c.exponent;
                }
            }
            __syncthreads();
            tf_load_a<KS>(a, s_codes, s_scales, (lane & 15) < cur.valid ? (lane & 15) : -1, p.k, p.act_block, ks_first, lane);
            loaded_tile = cur.tile;
        }
        BTile<KS, FP8> n[4];
        ItemRef next = cur;
        if (item + 1 < item_last) {
            next = tf_item(p, item + 1, per_tile);
#pragma unroll
            for (int t = 0; t < 4; ++t)
                tf_load_b<KS, FP8>(n[t], p.w + (size_t)next.expert * p.w_expert_stride,
                                   p.ws + (size_t)next.expert * p.ws_expert_stride, 4 * next.j + t, p.k, ks_first, lane, p.bn, p.bk);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const v4f c = tf_dot_tile<KS, FP8>(a, b[t]);
#pragma unroll
            for (int i = 0; i < 4; ++i) red[(t >> 1) * 4 + wave][t & 1][i][lane] = c[i];
        }
        __syncthreads();
        // waves 0..3 each finish one of the four 16-column tiles
        {
            float (*slot)[2][4][64] = red + (wave >> 1) * 4;
            const int which = wave & 1;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = 4 * (lane >> 4) + i;
                if (m < cur.valid) {
                    float acc = slot[0][which][i][lane];
#pragma unroll
                    for (int w2 = 1; w2 < 4; ++w2) acc = __fadd_rn(acc, slot[w2][which][i][lane]);
                    const int col = 64 * cur.j + 16 * wave + (lane & 15);
                    if (p.task_expert != nullptr) {
                        const int phys = cur.tile * 16 + m;
                        p.out[(size_t)p.token_map[phys] * p.hidden + col] = tf_to_bf16(__fmul_rn(acc, p.token_weights[phys]));
                    } else {
                        p.out[(size_t)(cur.tile * 16 + m) * p.hidden + col] = tf_to_bf16(acc);
                    }
                }
            }
        }
        __syncthreads();
        if (item + 1 < item_last) {
#pragma unroll
            for (int t = 0; t < 4; ++t) b[t] = n[t];
        }
        cur = next;
    }
}

__device__ __forceinline__ int tf_tiles(const StreamArgs& p) {
    return p.task_expert != nullptr ? p.expert_tile_base[p.experts] : (p.dense_rows + 15) / 16;
}
// Persistent launch: workgroup b of G takes items [b W / G, (b + 1) W / G).  block = 256 threads (four waves).
template <bool FP8, int KS>
__global__ void __launch_bounds__(256) tf_fc1_stream(const StreamArgs p) {
    __shared__ float red[8][2][4][64];
    const long long items = (long long)tf_tiles(p) * (p.inter / 16);
    const int first = (int)(items * blockIdx.x / gridDim.x), last = (int)(items * (blockIdx.x + 1) / gridDim.x);
    tf_fc1_items<FP8, KS>(p, first, last, red);
}
template <bool FP8, int KS>
__global__ void __launch_bounds__(256) tf_fc2_stream(const StreamArgs p) {
    __shared__ float red[8][2][4][64];
    extern __shared__ uint8_t dyn[];
    const long long items = (long long)tf_tiles(p) * (p.hidden / 64);
    const int first = (int)(items * blockIdx.x / gridDim.x), last = (int)(items * (blockIdx.x + 1) / gridDim.x);
    tf_fc2_items<FP8, KS>(p, first, last, red, dyn, dyn + 16 * (size_t)p.k);
}
