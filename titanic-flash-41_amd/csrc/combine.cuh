// Combine: ordered per-token sum of the route outputs, shared-expert addition, and their fusion.
// Reference semantics: kernels/ffn_sum_shared.cuh:7-58, runtime/kernels/ffn-native-v1/ffn.cu:255-258.
#pragma once
#include "common.cuh"

// out = bf16(f32(a) + f32(b)), flush-to-zero add.  8 values a thread.
extern "C" __global__ void __launch_bounds__(256) ca_ffn_add_rows(const uint16_t* a, const uint16_t* b, uint16_t* out,
                                                                  long long n8) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    const u4v x = reinterpret_cast<const u4v*>(a)[i], y = reinterpret_cast<const u4v*>(b)[i];
    u4v o;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        o[j] = tf_pack_bf16(tf_ftz(__fadd_rn(tf_ftz(tf_bf16_lo(x[j])), tf_ftz(tf_bf16_lo(y[j])))),
                            tf_ftz(__fadd_rn(tf_ftz(tf_bf16_hi(x[j])), tf_ftz(tf_bf16_hi(y[j])))));
    reinterpret_cast<u4v*>(out)[i] = o;
}
// routed[row][c] = bf16(sum over slots, in slot order, of f32(routes[row][slot][c])) for rows < live (other rows keep
// their value).  routes [rows][topk][hidden].  8 columns a thread.
__device__ __forceinline__ void tf_sum_routes(const uint16_t* routes, long long row, int c8, int topk, int hidden, float (&sum)[8]) {
#pragma unroll
    for (int k = 0; k < 8; ++k) sum[k] = 0.f;
    // eight slots' loads are requested together and added in slot order (a slot at a time, a thread of a few-row launch would
    // wait for one round trip a slot)
    for (int first = 0; first < topk; first += 8) {
        u4v v[8];
#pragma unroll
        for (int s = 0; s < 8; ++s)
            if (first + s < topk) v[s] = reinterpret_cast<const u4v*>(routes + (row * topk + first + s) * hidden)[c8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            if (first + s >= topk) break;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sum[2 * j] = __fadd_rn(sum[2 * j], tf_bf16_lo(v[s][j]));
                sum[2 * j + 1] = __fadd_rn(sum[2 * j + 1], tf_bf16_hi(v[s][j]));
            }
        }
    }
}
extern "C" __global__ void __launch_bounds__(256) ca_moe_topk_sum(const uint16_t* routes, uint16_t* routed, int rows,
                                                                  int topk, int hidden, const int32_t* live_ptr, int live_value) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x, per_row = hidden >> 3;
    if (i >= rows * per_row) return;
    const long long row = i / per_row;
    const int live = live_ptr != nullptr ? live_ptr[0] : live_value;
    if (row >= live) return;
    float sum[8];
    tf_sum_routes(routes, row, (int)(i - row * per_row), topk, hidden, sum);
    u4v o;
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = tf_pack_bf16(sum[2 * j], sum[2 * j + 1]);
    reinterpret_cast<u4v*>(routed)[i] = o;
}
// The sum above fused with the shared addition; also writes the routed buffer (rows < live).
extern "C" __global__ void __launch_bounds__(256) ca_ffn_sum_shared(const uint16_t* routes, const uint16_t* shared,
                                                                    uint16_t* routed_out, uint16_t* output, int n, int live,
                                                                    int topk, int hidden) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x, per_row = hidden >> 3;
    if (i * 8 >= n) return;
    const long long row = i / per_row;
    const u4v y = reinterpret_cast<const u4v*>(shared)[i];          // requested with the routes, not after their sum
    u4v routed;
    if (row < live) {
        float sum[8];
        tf_sum_routes(routes, row, (int)(i - row * per_row), topk, hidden, sum);
#pragma unroll
        for (int j = 0; j < 4; ++j) routed[j] = tf_pack_bf16(sum[2 * j], sum[2 * j + 1]);
        reinterpret_cast<u4v*>(routed_out)[i] = routed;
    } else {
        routed = reinterpret_cast<const u4v*>(routed_out)[i];
    }
    u4v o;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        o[j] = tf_pack_bf16(tf_ftz(__fadd_rn(tf_ftz(tf_bf16_lo(routed[j])), tf_ftz(tf_bf16_lo(y[j])))),
                            tf_ftz(__fadd_rn(tf_ftz(tf_bf16_hi(routed[j])), tf_ftz(tf_bf16_hi(y[j])))));
    reinterpret_cast<u4v*>(output)[i] = o;
}
// The route sum for one row group of a sequence-parallel chunk, laid out for that group's own reduce-scatter:
// out[c][j][:] = sum of routes of row c * quarter + group * per + j (rows >= live are not written).
extern "C" __global__ void __launch_bounds__(256) ca_moe_group_sum_rows(const uint16_t* routes, uint16_t* out, int quarter,
                                                                        int per, int group, int live, int topk, int hidden) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x, per_row = hidden >> 3;
    const long long n = 4ll * per * per_row;
    if (i >= n) return;
    const int c8 = (int)(i % per_row);
    const long long t = i / per_row;
    const int j = (int)(t % per), c = (int)(t / per);
    const int row = c * quarter + group * per + j;
    if (row >= live) return;
    float sum[8];
    tf_sum_routes(routes, row, c8, topk, hidden, sum);
    u4v o;
#pragma unroll
    for (int k = 0; k < 4; ++k) o[k] = tf_pack_bf16(sum[2 * k], sum[2 * k + 1]);
    reinterpret_cast<u4v*>(out + ((long long)c * per + j) * hidden)[c8] = o;
}
