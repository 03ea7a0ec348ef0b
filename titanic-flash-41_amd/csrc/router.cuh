// Router: gate product for few rows, top-k with renormalised weights, padding routes, census.
// Reference semantics: src/ffn.rs:330-413 (Router::run_routed), kernels/moe_frontend.cuh:85-157 (top-k),
// kernels/core.cu:1093-1097 (padding rows), kernels/core.cu:161-166 (census).
#pragma once
#include "common.cuh"

// logits[m][e] = sum_k x[m][k] * w[e][k], BF16 inputs, FP32 accumulate, for one expert by one wave.
// Fixed summation order: lane l accumulates the 8-element vectors at k = 512 j + 8 l (j ascending) with fma in k order,
// then the 64 partials are combined by the xor butterfly 32, 16, 8, 4, 2, 1.  hidden % 512 == 0, hidden <= 8192.
// Loads are issued sixteen at a time (four vectors of the expert's row, four of each of four token rows).
__device__ __forceinline__ void tf_logits_expert(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, float* __restrict__ out,
                                                 int rows, int hidden, int experts, int e, int lane) {
    const int nj = hidden >> 9;
    const u4v* wrow = reinterpret_cast<const u4v*>(w + (size_t)e * hidden);
    for (int m0 = 0; m0 < rows; m0 += 4) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int j0 = 0; j0 < nj; j0 += 4) {                 // four vectors of the expert and of four rows in flight
            u4v wv[4], xv[4][4];
#pragma unroll
            for (int j = 0; j < 4; ++j) if (j0 + j < nj) wv[j] = wrow[(j0 + j) * 64 + lane];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (m0 + r < rows && j0 + j < nj) xv[r][j] = reinterpret_cast<const u4v*>(x + (size_t)(m0 + r) * hidden)[(j0 + j) * 64 + lane];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (m0 + r < rows && j0 + j < nj) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            acc[r] = __fmaf_rn(tf_bf16_lo(xv[r][j][i]), tf_bf16_lo(wv[j][i]), acc[r]);
                            acc[r] = __fmaf_rn(tf_bf16_hi(xv[r][j][i]), tf_bf16_hi(wv[j][i]), acc[r]);
                        }
                    }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float v = acc[r];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v = __fadd_rn(v, __shfl_xor(v, o));
            if (lane == 0 && m0 + r < rows) tf_publish_f32(out + (size_t)(m0 + r) * experts + e, v);   // may be read by another block of the same launch
        }
    }
}
// The same product for one workgroup of the experts' front-end: wave `wave` takes expert `e`, all waves share at most four
// token rows.  One round trip: every lane requests its expert's whole row (hidden / 512 vectors) and the workgroup requests
// the token rows once (instead of once a wave), which then go through LDS.  Same summation order as tf_logits_expert.
// Block barrier inside; hidden <= 8192; `s_x` holds rows * hidden / 8 vectors (at most 4,096).
// `mailbox` (may be null): the consumer polls these words instead of waiting for a counter: a word is zero while empty and
// holds the complement of the logit's bits once written (no sum of BF16 products has all bits set: the low half of every
// widened BF16 operand is zero and a NaN keeps an operand's payload).
__device__ __forceinline__ void tf_logits_block(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, float* __restrict__ out,
                                                int rows, int hidden, int experts, int e, int lane, u4v* s_x, uint32_t* mailbox = nullptr) {
    const int nj = hidden >> 9, per_row = hidden >> 3, total = rows * per_row;
    const bool on = e < experts;
    u4v wv[16], xr[8];
    const u4v* wrow = reinterpret_cast<const u4v*>(w + (size_t)(on ? e : 0) * hidden);
#pragma unroll
    for (int j = 0; j < 16; ++j) if (on && j < nj) wv[j] = wrow[j * 64 + lane];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int v = (int)threadIdx.x + (int)blockDim.x * i;
        if (v < total) xr[i] = reinterpret_cast<const u4v*>(x)[v];           // the rows are consecutive: row v / per_row
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int v = (int)threadIdx.x + (int)blockDim.x * i;
        if (v < total) s_x[v] = xr[i];
    }
    __syncthreads();
    if (!on) return;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 16; ++j)
        if (j < nj) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (r < rows) {
                    const u4v xv = s_x[r * per_row + j * 64 + lane];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc[r] = __fmaf_rn(tf_bf16_lo(xv[i]), tf_bf16_lo(wv[j][i]), acc[r]);
                        acc[r] = __fmaf_rn(tf_bf16_hi(xv[i]), tf_bf16_hi(wv[j][i]), acc[r]);
                    }
                }
        }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float v = acc[r];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v = __fadd_rn(v, __shfl_xor(v, o));
        if (lane == 0 && r < rows) {
            if (mailbox != nullptr) {
                out[(size_t)r * experts + e] = v;
                tf_publish_u32(mailbox + (size_t)r * experts + e, ~__float_as_uint(v));
            } else {
                tf_publish_f32(out + (size_t)r * experts + e, v);   // read by another block of the same launch
            }
        }
    }
}
// One wave per expert, up to 16 rows a launch.
extern "C" __global__ void __launch_bounds__(64) ca_router_logits_rows(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, float* __restrict__ out, int rows, int hidden,
    int experts) {
    if ((int)blockIdx.x < experts) tf_logits_expert(x, w, out, rows, hidden, experts, blockIdx.x, threadIdx.x);
}

struct RouteParams {
    int experts, topk, scoring;   // scoring: 0 sigmoid, 1 sqrt(softplus)
    float route_scale;
    long long alt_token;          // token id that selects bias_alt, -1: none
};

// Maximum of 64-bit keys (hi, lo) over the 64 lanes of a wave, in every lane (data-parallel primitives, as tf_wave_max).
__device__ __forceinline__ void tf_wave_max_key(uint32_t& hi, uint32_t& lo) {
#define TF_KEY_STEP(CTRL, ROWS, ALL)                                                                                          \
    {                                                                                                                         \
        const uint32_t ohi = (uint32_t)__builtin_amdgcn_update_dpp((ALL) ? 0 : (int)hi, (int)hi, CTRL, ROWS, 0xf, ALL);       \
        const uint32_t olo = (uint32_t)__builtin_amdgcn_update_dpp((ALL) ? 0 : (int)lo, (int)lo, CTRL, ROWS, 0xf, ALL);       \
        const bool take = ohi > hi || (ohi == hi && olo > lo);                                                                \
        hi = take ? ohi : hi;                                                                                                 \
        lo = take ? olo : lo;                                                                                                 \
    }
    TF_KEY_STEP(0xb1, 0xf, true)       // quad_perm [1,0,3,2]
    TF_KEY_STEP(0x4e, 0xf, true)       // quad_perm [2,3,0,1]
    TF_KEY_STEP(0x141, 0xf, true)      // row_half_mirror
    TF_KEY_STEP(0x140, 0xf, true)      // row_mirror
    TF_KEY_STEP(0x142, 0xa, false)     // row_bcast15 -> rows 1, 3
    TF_KEY_STEP(0x143, 0xc, false)     // row_bcast31 -> rows 2, 3
#undef TF_KEY_STEP
    hi = (uint32_t)__builtin_amdgcn_readlane((int)hi, 63);
    lo = (uint32_t)__builtin_amdgcn_readlane((int)lo, 63);
}

// One wave routes one row.  Lane l holds experts l, l + 64, ... (at most 8 per lane: experts <= 512): `x` their logits,
// `b` their selection biases.  Every lane returns the same ids / weights in registers [k]; topk <= 8.
// Selection = the k largest biased scores, ties to the lowest expert id (a NaN counts as +inf): each candidate is one 64-bit
// key (the biased score's bits mapped to an unsigned order, then the complemented id), so a round is one wave maximum.
// SLOTS = 4 for at most 256 experts (half the scans of a round), else 8.
template <int SLOTS>
__device__ __forceinline__ void tf_route_row(const float (&x)[8], const float (&b)[8], int lane, const RouteParams& p,
                                             int32_t* out_ids, float* out_weights) {
    float score[SLOTS];
    uint32_t key[SLOTS];
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
        const int e = i * 64 + lane;
        score[i] = 0.f;
        key[i] = 0u;                                    // below every candidate: -inf maps to 0x007fffff
        if (e < p.experts) {
            float s;
            if (p.scoring == 1) s = __builtin_sqrtf(x[i] > 20.f ? x[i] : tf_log1p_pos(tf_exp(x[i])));
            else s = tf_logistic(x[i]);
            float v = __fadd_rn(s, b[i]);
            v = (v == v) ? __fadd_rn(v, 0.f) : INFINITY;              // -0 -> +0: equal scores must have equal keys
            const uint32_t u = __float_as_uint(v);
            score[i] = s;
            key[i] = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
        }
    }
    float w[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        w[k] = 0.f;
        if (k < p.topk) {
            uint32_t hi = 0u, lo = 0u;
#pragma unroll
            for (int i = 0; i < SLOTS; ++i) {           // ids ascend with i: a later slot wins only with a larger score
                const bool take = key[i] > hi;
                hi = take ? key[i] : hi;
                lo = take ? ~(uint32_t)(i * 64 + lane) : lo;
            }
            tf_wave_max_key(hi, lo);
            const int32_t winner = (int32_t)~lo;
            float mine = 0.f;
#pragma unroll
            for (int i = 0; i < SLOTS; ++i)
                if (i * 64 + lane == winner) { mine = score[i]; key[i] = 0u; }
            w[k] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mine), winner & 63));
            out_ids[k] = winner;
        }
    }
    float total;
    if (p.topk == 6) {
        total = __fadd_rn(__fadd_rn(__fadd_rn(w[3], __fadd_rn(w[2], __fadd_rn(w[0], w[1]))), __fadd_rn(w[4], w[5])), 1e-20f);
    } else {
        total = w[0];
#pragma unroll
        for (int k = 1; k < 8; ++k) if (k < p.topk) total = __fadd_rn(total, w[k]);
        total = __fadd_rn(total, 1e-20f);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) if (k < p.topk) out_weights[k] = __fmul_rn(w[k] / total, p.route_scale);
}

// Padding rows of a batched step take their source row's experts with zero weights; by one block, after the rows' routes
// are complete (in `ids` / `weights`, and in the LDS copy when there is one).  Ends with a block barrier.
__device__ __forceinline__ void tf_apply_padding(const int32_t* padding, int32_t* ids, float* weights, int rows, int topk, int32_t* s_ids,
                                                 float* s_weights) {
    if (padding != nullptr)
        for (int i = threadIdx.x; i < rows * topk; i += blockDim.x) {
            const int r = i / topk, s = padding[r];
            if (s >= 0) {
                const int32_t from = s_ids != nullptr ? s_ids[s * topk + (i - r * topk)] : ids[s * topk + (i - r * topk)];
                ids[i] = from;
                weights[i] = 0.f;
                if (s_ids != nullptr) { s_ids[i] = from; s_weights[i] = 0.f; }
            }
        }
    __syncthreads();
}

// Routes rows [first_row, first_row + waves of this block) of `rows`; rows at or past min(rows, live[0]) get ids -1 and
// weights 0.  `padding` (may be null) is applied only by a single-block launch, after a block barrier.  `leave_padded`: rows
// with a padding source are not written at all (another workgroup of the launch writes them, with their source's experts).
template <bool COHERENT = true>
__device__ __forceinline__ void tf_route_block(const float* logits, const float* bias, const float* bias_alt,
                                               const long long* tokens, const int32_t* live, const int32_t* padding,
                                               int32_t* ids, float* weights, int rows, const RouteParams& p,
                                               int first_row, int row_stride, bool apply_padding, int32_t* s_ids = nullptr,
                                               float* s_weights = nullptr, bool publish = false, bool leave_padded = false) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int live_count = live[0];
    const bool has_alt = bias_alt != nullptr && tokens != nullptr && p.alt_token >= 0;
    for (int row = first_row + wave; row < rows; row += row_stride) {
        // everything the row needs is requested at once (one round trip): its logits, both biases, its token id; the live
        // count requested above is first used below
        float x[8], b0[8], b1[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int e = i * 64 + lane;
            x[i] = 0.f; b0[i] = 0.f; b1[i] = 0.f;
            if (e < p.experts) {
                const float* at = logits + (size_t)row * p.experts + e;
                x[i] = COHERENT ? tf_acquire_f32(at) : *at;
                b0[i] = bias[e];
                if (has_alt) b1[i] = bias_alt[e];
            }
        }
        const long long token = has_alt ? tokens[row] : -1;
        const bool is_live = row < min(rows, live_count);
        if (leave_padded && padding != nullptr && padding[row] >= 0) continue;       // uniform over the wave: one row a wave
        int32_t chosen[8];
        float share[8];
        if (is_live) {
            if (has_alt && token == p.alt_token) {
#pragma unroll
                for (int i = 0; i < 8; ++i) b0[i] = b1[i];
            }
            if (p.experts <= 256) tf_route_row<4>(x, b0, lane, p, chosen, share);
            else tf_route_row<8>(x, b0, lane, p, chosen, share);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (k < p.topk && lane == k) {
                if (publish) {      // read next by another workgroup of the same launch
                    tf_publish_u32(reinterpret_cast<uint32_t*>(ids) + row * p.topk + k, (uint32_t)(is_live ? chosen[k] : -1));
                    tf_publish_f32(weights + row * p.topk + k, is_live ? share[k] : 0.f);
                } else {
                    ids[row * p.topk + k] = is_live ? chosen[k] : -1;
                    weights[row * p.topk + k] = is_live ? share[k] : 0.f;
                }
                if (s_ids != nullptr) {      // a copy in LDS for the plan that follows in the same block
                    s_ids[row * p.topk + k] = is_live ? chosen[k] : -1;
                    s_weights[row * p.topk + k] = is_live ? share[k] : 0.f;
                }
            }
    }
    if (apply_padding) {
        __threadfence_block();
        __syncthreads();
        tf_apply_padding(padding, ids, weights, rows, p.topk, s_ids, s_weights);
    }
}

// The router's top-k alone.  One block: routes every row and applies `padding`.  Several blocks: each block routes its
// waves' rows; the caller passes padding = null and launches ca_route_padding_rows afterwards.
extern "C" __global__ void ca_route_topk(const float* logits, const float* bias, const float* bias_alt,
                                         const long long* tokens, const int32_t* live, const int32_t* padding,
                                         int32_t* ids, float* weights, int32_t rows, int32_t experts, int32_t topk,
                                         int32_t scoring, float route_scale, long long alt_token) {
    const RouteParams p{experts, topk, scoring, route_scale, alt_token};
    const int waves = blockDim.x >> 6;
    tf_route_block<false>(logits, bias, bias_alt, tokens, live, padding, ids, weights, rows, p, blockIdx.x * waves,
                   gridDim.x * waves, gridDim.x == 1);
}

// Padding rows of a batched step take their source row's experts with zero weights.
extern "C" __global__ void ca_route_padding_rows(int32_t* ids, float* weights, const int32_t* source, int rows, int topk) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * topk) return;
    const int r = i / topk, s = source[r];
    if (s < 0) return;
    ids[i] = ids[s * topk + (i - r * topk)];
    weights[i] = 0.f;
}

// Diagnostic histogram of the routed slots of live rows.
extern "C" __global__ void ca_route_census(const int32_t* ids, const int32_t* live, int rows, int topk,
                                           uint32_t* counters, int experts) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * topk || i / topk >= live[0]) return;
    const int e = ids[i];
    if (e >= 0 && e < experts) atomicAdd(counters + e, 1u);
}
