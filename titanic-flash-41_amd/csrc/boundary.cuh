// The steps either side of the layer at the decoder's FFN boundary (src/decoder.rs:1497-1543, 1654-1656; src/ffn.rs:974-975,
// 1053-1065): upstream the boundary hands the layer a normalized BF16 row together with its MXFP8 codes (the layer then
// skips its own quantizer); downstream the layer's output is added to the residual.  The reference's boundary operators
// are binaries (src/mhc.rs loads them by name), so the arithmetic here is this library's own statement of an RMS norm with a
// BF16 boundary and of a BF16 residual addition, every rounding step fixed so that the host-side restatement gives the same
// bits.
#pragma once
#include "combine.cuh"
#include "frontend.cuh"

// One workgroup of 256 threads a row; cols a multiple of 8, at most 8,192.
//   ss       = sum of x^2 in FP32: every thread over its 8-value pieces in ascending order, value by value; the 64 threads of a
//              wave by a butterfly (xor 1, 2, 4, 8, 16, 32); the four waves in ascending order
//   inverse  = 1 / sqrt(ss / cols + eps), division and root correctly rounded
//   normed   = bf16((x * inverse) * weight), two FP32 products
// then both MXFP8 flavours of the normalized row: blocks of `act_block` columns, scale = amax / 448 rounded up to a power of
// two; `codes` / `scales`: an all-zero block has scale byte 0 (the routed experts' input); `codes_min` / `scales_min`: amax
// floored at 1e-4 (the shared expert's input).  Either pair may be null.
extern "C" __global__ void __launch_bounds__(256) ca_rmsnorm_quant(const uint16_t* __restrict__ x, const uint16_t* __restrict__ weight,
                                                                   uint16_t* __restrict__ normed, uint8_t* __restrict__ codes,
                                                                   uint8_t* __restrict__ scales, uint8_t* __restrict__ codes_min,
                                                                   uint8_t* __restrict__ scales_min, int cols, int act_block, float eps) {
    constexpr int MAX_PIECES = 4;                      // 8,192 columns
    __shared__ float s_wave[4];
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int per_row = cols >> 3, group_lanes = act_block >> 3;
    const u4v* src = reinterpret_cast<const u4v*>(x + (size_t)row * cols);
    u4v piece[MAX_PIECES];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAX_PIECES; ++i) {
        const int q = i * 256 + tid;
        piece[i] = q < per_row ? src[q] : u4v{0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float a = tf_bf16_lo(piece[i][j]), b = tf_bf16_hi(piece[i][j]);
            ss = __fadd_rn(ss, __fmul_rn(a, a));
            ss = __fadd_rn(ss, __fmul_rn(b, b));
        }
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) ss = __fadd_rn(ss, __shfl_xor(ss, o));
    if (lane == 0) s_wave[wave] = ss;
    __syncthreads();
    const float total = __fadd_rn(__fadd_rn(__fadd_rn(s_wave[0], s_wave[1]), s_wave[2]), s_wave[3]);
    const float inverse = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, (float)cols), eps)));
    const u4v* wsrc = reinterpret_cast<const u4v*>(weight);
#pragma unroll
    for (int i = 0; i < MAX_PIECES; ++i) {
        const int q = i * 256 + tid;
        const bool on = q < per_row;
        float v[8];
        u4v o = {0, 0, 0, 0};
        if (on) {
            const u4v w = wsrc[q];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint16_t a = tf_to_bf16(__fmul_rn(__fmul_rn(tf_bf16_lo(piece[i][j]), inverse), tf_bf16_lo(w[j])));
                const uint16_t b = tf_to_bf16(__fmul_rn(__fmul_rn(tf_bf16_hi(piece[i][j]), inverse), tf_bf16_hi(w[j])));
                v[2 * j] = tf_bf16(a);
                v[2 * j + 1] = tf_bf16(b);
                o[j] = (uint32_t)a | ((uint32_t)b << 16);
            }
            reinterpret_cast<u4v*>(normed + (size_t)row * cols)[q] = o;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = 0.f;
        }
        // whole groups of lanes are on or off together: per_row is a multiple of group_lanes
        const float amax = tf_group_amax(v, group_lanes);
        if (!on) continue;
        const size_t at = (size_t)row * per_row + q;
        if (codes != nullptr) {
            const Quant8 c = tf_quant8(v, amax, 0.f);
            reinterpret_cast<u2v*>(codes)[at] = u2v{c.lo, c.hi};
            if ((q & (group_lanes - 1)) == 0) scales[at / group_lanes] = (uint8_t)c.exponent;
        }
        if (codes_min != nullptr) {
            const Quant8 c = tf_quant8(v, amax, 1e-4f);
            reinterpret_cast<u2v*>(codes_min)[at] = u2v{c.lo, c.hi};
            if ((q & (group_lanes - 1)) == 0) scales_min[at / group_lanes] = (uint8_t)c.exponent;
        }
    }
}

// The ordered route sum and the shared addition of ca_ffn_sum_shared with the residual addition behind them, in one pass:
//   routed (rows < live) = bf16(sum of the row's route outputs, FP32 adds in route order); other rows keep `routed_out`
//   ffn      = bf16(routed + shared), the addition flushing subnormals to zero        (written to `ffn_out` unless null)
//   residual = bf16(f32(ffn) + f32(residual))                                         (in place or to another buffer)
// 8 values a thread.
extern "C" __global__ void __launch_bounds__(256) ca_ffn_sum_shared_residual(const uint16_t* routes, const uint16_t* shared, const uint16_t* residual,
                                                                             uint16_t* routed_out, uint16_t* ffn_out, uint16_t* residual_out,
                                                                             int n, int live, int topk, int hidden) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x, per_row = hidden >> 3;
    if (i * 8 >= n) return;
    const long long row = i / per_row;
    u4v routed = reinterpret_cast<const u4v*>(routed_out)[i];
    if (row < live) {
        float sum[8];
        tf_sum_routes(routes, row, (int)(i - row * per_row), topk, hidden, sum);
#pragma unroll
        for (int j = 0; j < 4; ++j) routed[j] = tf_pack_bf16(sum[2 * j], sum[2 * j + 1]);
        reinterpret_cast<u4v*>(routed_out)[i] = routed;
    }
    const u4v y = reinterpret_cast<const u4v*>(shared)[i], r = reinterpret_cast<const u4v*>(residual)[i];
    u4v f, o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f[j] = tf_pack_bf16(tf_ftz(__fadd_rn(tf_ftz(tf_bf16_lo(routed[j])), tf_ftz(tf_bf16_lo(y[j])))),
                            tf_ftz(__fadd_rn(tf_ftz(tf_bf16_hi(routed[j])), tf_ftz(tf_bf16_hi(y[j])))));
        o[j] = tf_pack_bf16(__fadd_rn(tf_bf16_lo(f[j]), tf_bf16_lo(r[j])), __fadd_rn(tf_bf16_hi(f[j]), tf_bf16_hi(r[j])));
    }
    if (ffn_out != nullptr) reinterpret_cast<u4v*>(ffn_out)[i] = f;
    reinterpret_cast<u4v*>(residual_out)[i] = o;
}
