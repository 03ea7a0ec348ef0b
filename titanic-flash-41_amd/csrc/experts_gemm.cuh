// Many-row (prefill) expert projections: grouped GEMM on the scaled FP8 x FP4 matrix instruction.
#pragma once
#include "experts_stream.cuh"

#define TF_STREAM_MAX_ROWS 64
#define TF_GEMM_TILE_M 128

struct GemmArgs {
    const uint8_t* a_codes;
    const uint8_t* a_scales;
    const uint8_t* w;
    const uint8_t* ws;
    long long w_expert_stride, ws_expert_stride;
    int bn, bk;
    const int32_t* expert_tile_base;
    const int32_t* task_expert;
    const int32_t* task_valid_rows;
    const int32_t* token_map;
    const float* token_weights;
    int experts, groups, topk, max_tiles;
    int dense_rows;
    int k, inter, hidden, act_block;
    float limit;
    uint16_t* h_bf16;
    uint8_t* h_codes;
    uint8_t* h_scales;
    uint16_t* out;
    uint16_t* tap;
};
inline int tf_launch_fc1_gemm(const GemmArgs&, int, hipStream_t) { return -4; }
inline int tf_launch_fc2_gemm(const GemmArgs&, int, hipStream_t) { return -4; }
inline int tf_launch_dense_gemm(const GemmArgs&, int, hipStream_t) { return -4; }
inline int tf_launch_shared_fc1_gemm(const GemmArgs&, int, hipStream_t) { return -4; }

// Gate product for many rows.  grid (ceil(rows / 64), experts / 32), block 128.
extern "C" __global__ void __launch_bounds__(128) ca_router_logits_mfma(const uint16_t* x, const uint16_t* w, float* out, int rows,
                                                                        int hidden, int experts) {
    // placeholder: scalar dot products, one thread per (row, expert) pair of the block's 64 x 32 tile
    for (int i = threadIdx.x; i < 64 * 32; i += blockDim.x) {
        const int row = blockIdx.x * 64 + i / 32, e = blockIdx.y * 32 + i % 32;
        if (row >= rows || e >= experts) continue;
        float acc = 0.f;
        for (int k = 0; k < hidden; ++k) acc = __fmaf_rn(tf_bf16(x[(size_t)row * hidden + k]), tf_bf16(w[(size_t)e * hidden + k]), acc);
        out[(size_t)row * experts + e] = acc;
    }
}
