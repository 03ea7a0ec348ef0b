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

// One wave routes one row.  Lane l holds experts l, l + 64, ... (at most 8 per lane: experts <= 512).  Every lane
// returns the same ids / weights in registers [k]; topk <= 8.  COHERENT: the logits were written by other workgroups of this
// launch (device-scope loads); otherwise by an earlier launch (plain loads).
template <bool COHERENT>
__device__ __forceinline__ void tf_route_row(const float* logits, const float* bias, int lane, const RouteParams& p,
                                             int32_t* out_ids, float* out_weights) {
    float score[8], biased[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int e = i * 64 + lane;
        score[i] = 0.f;
        biased[i] = -INFINITY;
        if (e < p.experts) {
            const float x = COHERENT ? tf_acquire_f32(logits + e) : logits[e];
            float s;
            if (p.scoring == 1) s = __builtin_sqrtf(x > 20.f ? x : tf_log1p_pos(tf_exp(x)));
            else s = tf_logistic(x);
            const float v = __fadd_rn(s, bias[e]);
            score[i] = s;
            biased[i] = (v == v) ? v : INFINITY;
        }
    }
    float w[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        w[k] = 0.f;
        if (k < p.topk) {
            float best = -INFINITY;
#pragma unroll
            for (int i = 0; i < 8; ++i) best = fmaxf(best, biased[i]);
            best = tf_wave_max(best);
            int32_t winner = 0x7fffffff;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (i * 64 + lane < p.experts && biased[i] == best) winner = min(winner, i * 64 + lane);
            winner = tf_wave_min(winner);
            float mine = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (i * 64 + lane == winner) { mine = score[i]; biased[i] = -INFINITY; }
            w[k] = __shfl(mine, winner & 63);
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
// weights 0.  `padding` (may be null) is applied only by a single-block launch, after a block barrier.
template <bool COHERENT = true>
__device__ __forceinline__ void tf_route_block(const float* logits, const float* bias, const float* bias_alt,
                                               const long long* tokens, const int32_t* live, const int32_t* padding,
                                               int32_t* ids, float* weights, int rows, const RouteParams& p,
                                               int first_row, int row_stride, bool apply_padding, int32_t* s_ids = nullptr,
                                               float* s_weights = nullptr, bool publish = false) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n_live = min(rows, live[0]);
    for (int row = first_row + wave; row < rows; row += row_stride) {
        const bool is_live = row < n_live;
        int32_t chosen[8];
        float share[8];
        if (is_live) {
            const bool alt = bias_alt != nullptr && tokens != nullptr && p.alt_token >= 0 && tokens[row] == p.alt_token;
            tf_route_row<COHERENT>(logits + (size_t)row * p.experts, alt ? bias_alt : bias, lane, p, chosen, share);
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
