// Shared-expert activation: clipped SwiGLU in BF16, alone or fused with the MXFP8 requantization of its output.
// Reference semantics: runtime/kernels/ffn-native-v1/ffn.cu:173-243 (silu_mul_clamp_kernel),
// kernels/shared_swiglu_quant.cuh:11-81 (fused with the quantizer, amax floored at 1e-4).
#pragma once
#include "frontend.cuh"

// Clamp in BF16 (gate <= limit, -limit <= up <= limit), widen, silu(g) * u in FP32, round to BF16.
__device__ __forceinline__ float tf_shared_activation(float gate, float up, float limit_hi, float limit_lo) {
    const float g = fminf(gate, limit_hi);
    const float u = fminf(fmaxf(up, limit_lo), limit_hi);
    return tf_bf16(tf_to_bf16(__fmul_rn(g / __fadd_rn(1.0f, tf_exp(-g)), u)));
}
// in [rows][gate(0..inter) | up(inter..2 inter)] BF16 -> act [rows][inter] BF16.  One thread per 8 outputs.
extern "C" __global__ void __launch_bounds__(256) ca_shared_swiglu_rows(const uint16_t* in, uint16_t* act, int rows,
                                                                        int inter, float limit) {
    const long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x, per_row = inter >> 3;
    if (q >= rows * per_row) return;
    const long long row = q / per_row, c8 = q - row * per_row;
    const float hi = tf_bf16(tf_to_bf16(limit)), lo = tf_bf16(tf_to_bf16(-limit));
    const u4v g = reinterpret_cast<const u4v*>(in + row * 2 * inter)[c8];
    const u4v u = reinterpret_cast<const u4v*>(in + row * 2 * inter + inter)[c8];
    u4v o;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = tf_pack_bf16(tf_shared_activation(tf_bf16_lo(g[i]), tf_bf16_lo(u[i]), hi, lo),
                            tf_shared_activation(tf_bf16_hi(g[i]), tf_bf16_hi(u[i]), hi, lo));
    reinterpret_cast<u4v*>(act + row * inter)[c8] = o;
}
// The same activation, kept in BF16, then quantized (MXFP8, `act_block` columns a block, amax floored at 1e-4):
// act [rows][inter] BF16, values [rows][inter] E4M3, scale_rows [rows][inter / act_block] UE8M0.
extern "C" __global__ void __launch_bounds__(256) ca_shared_swiglu_quant(const uint16_t* in, uint16_t* act, uint8_t* values,
                                                                         uint8_t* scale_rows, int rows, int inter,
                                                                         int act_block, float limit) {
    const long long per_row = inter >> 3, total = rows * per_row, padded = (total + 63) & ~63ll;
    const int group_lanes = act_block >> 3;
    const float hi = tf_bf16(tf_to_bf16(limit)), lo = tf_bf16(tf_to_bf16(-limit));
    for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < padded; q += (long long)gridDim.x * blockDim.x) {
        const bool on = q < total;
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = 0.f;
        long long row = 0, c8 = 0;
        if (on) {
            row = q / per_row;
            c8 = q - row * per_row;
            const u4v g = reinterpret_cast<const u4v*>(in + row * 2 * inter)[c8];
            const u4v u = reinterpret_cast<const u4v*>(in + row * 2 * inter + inter)[c8];
            u4v o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[2 * i] = tf_shared_activation(tf_bf16_lo(g[i]), tf_bf16_lo(u[i]), hi, lo);
                v[2 * i + 1] = tf_shared_activation(tf_bf16_hi(g[i]), tf_bf16_hi(u[i]), hi, lo);
                o[i] = (__float_as_uint(v[2 * i]) >> 16) | (__float_as_uint(v[2 * i + 1]) & 0xffff0000u);
            }
            reinterpret_cast<u4v*>(act + row * inter)[c8] = o;
        }
        const float amax = tf_group_amax(v, group_lanes);
        if (!on) continue;
        const Quant8 c = tf_quant8(v, amax, 1e-4f);
        reinterpret_cast<u2v*>(values + row * inter)[c8] = u2v{c.lo, c.hi};
        if ((c8 & (group_lanes - 1)) == 0) scale_rows[row * (inter / act_block) + c8 / group_lanes] = (uint8_t)c.exponent;
    }
}
