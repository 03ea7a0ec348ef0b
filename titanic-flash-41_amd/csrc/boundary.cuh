// The steps either side of the layer at the decoder's FFN boundary (src/decoder.rs:1497-1543, 1654-1656; src/ffn.rs:974-975,
// 1053-1065; src/mhc.rs:981-990, 1223-1234).  Upstream the boundary collapses the row's residual streams with the predecessor's
// pre-coefficients, normalizes, and hands the layer the normalized BF16 row together with its MXFP8 codes (the layer then skips
// its own quantizer): runtime/kernels/mhc-norm-quant-v1/mhc-norm-quant.py:15-44.  Downstream the layer's output is mixed back
// into the residual streams: runtime/kernels/mhc-post-tiles-v1/mhc-post-tiles.py:11-27.  Every rounding step is fixed so that
// the host-side restatement gives the same bits; the two NVIDIA approximations of the reference's object code (reciprocal
// root, division) are replaced by correctly rounded operations.
#pragma once
#include "combine.cuh"
#include "frontend.cuh"

// One workgroup of 256 threads a row (blockIdx.x) and column part (blockIdx.y of gridDim.y: every part forms the whole row's
// statistics and writes its own columns, as the reference's grid (rows, PARTS) does); cols a multiple of 8, at most 8,192,
// cols / parts a multiple of the block width.
//   value    = bf16(fma(x[row][S-1], pre[S-1], ... fma(x[row][0], pre[0], 0)))      S = streams; pre == null: coefficients 1
//   ss       = sum of value^2 in FP32: every thread over its 8-value pieces in ascending order, one fused multiply-add a value;
//              the 64 threads of a wave by a butterfly (xor 1, 2, 4, 8, 16, 32); the four waves in ascending order
//   inverse  = 1 / sqrt(ss / cols + eps), divisions and root correctly rounded
//   normed   = bf16((value * inverse) * weight), two FP32 products
// then the MXFP8 flavours of the normalized row: blocks of `act_block` columns, scale = amax / 448 rounded up to a power of
// two; `codes` / `scales`: an all-zero block has scale byte 0 (the routed experts' input); `codes_min` / `scales_min`: amax
// floored at 1e-4 (the reference's Q / SR: the shared expert's input); `mma_scales`: the floored flavour's scale bytes once
// more at (row % 32) * 16 + ((row / 32) % 4) * 4 + (row / 128) * (ceil(groups / 4) * 512) + (group / 4) * 512 + group % 4 (the
// reference's SM).  Any of the three may be null.
__device__ __forceinline__ void tf_hc_norm_quant_row(const uint16_t* __restrict__ x, const float* __restrict__ pre, const uint16_t* __restrict__ weight,
                                                     uint16_t* __restrict__ normed, uint8_t* __restrict__ codes, uint8_t* __restrict__ scales,
                                                     uint8_t* __restrict__ codes_min, uint8_t* __restrict__ scales_min, uint8_t* __restrict__ mma_scales,
                                                     int cols, int streams, int act_block, float eps) {
    constexpr int MAX_PIECES = 4;                      // 8,192 columns
    __shared__ float s_wave[4];
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int per_row = cols >> 3, group_lanes = act_block >> 3;
    const int part_pieces = per_row / (int)gridDim.y, part_first = (int)blockIdx.y * part_pieces;
    float value[MAX_PIECES][8];
#pragma unroll
    for (int i = 0; i < MAX_PIECES; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) value[i][j] = 0.f;
    for (int c = 0; c < streams; ++c) {
        const u4v* src = reinterpret_cast<const u4v*>(x + ((size_t)row * streams + c) * cols);
        const float coefficient = pre != nullptr ? pre[(size_t)row * streams + c] : 1.0f;
#pragma unroll
        for (int i = 0; i < MAX_PIECES; ++i) {
            const int q = i * 256 + tid;
            if (q < per_row) {
                const u4v piece = src[q];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    value[i][2 * j] = __fmaf_rn(tf_bf16_lo(piece[j]), coefficient, value[i][2 * j]);
                    value[i][2 * j + 1] = __fmaf_rn(tf_bf16_hi(piece[j]), coefficient, value[i][2 * j + 1]);
                }
            }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAX_PIECES; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            value[i][j] = tf_bf16(tf_to_bf16(value[i][j]));
            ss = __fmaf_rn(value[i][j], value[i][j], ss);
        }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) ss = __fadd_rn(ss, __shfl_xor(ss, o));
    if (lane == 0) s_wave[wave] = ss;
    __syncthreads();
    const float total = __fadd_rn(__fadd_rn(__fadd_rn(s_wave[0], s_wave[1]), s_wave[2]), s_wave[3]);
    // __builtin_sqrtf and `/` are the correctly rounded forms (the __fsqrt_rn intrinsic is the hardware's approximate root here)
    const float inverse = 1.0f / __builtin_sqrtf(__fadd_rn(total / (float)cols, eps));
    const u4v* wsrc = reinterpret_cast<const u4v*>(weight);
    const int groups = cols / act_block;
#pragma unroll
    for (int i = 0; i < MAX_PIECES; ++i) {
        const int q = i * 256 + tid;
        const bool on = q >= part_first && q < part_first + part_pieces;
        float v[8];
        u4v o = {0, 0, 0, 0};
        if (on) {
            const u4v w = wsrc[q];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint16_t a = tf_to_bf16(__fmul_rn(__fmul_rn(value[i][2 * j], inverse), tf_bf16_lo(w[j])));
                const uint16_t b = tf_to_bf16(__fmul_rn(__fmul_rn(value[i][2 * j + 1], inverse), tf_bf16_hi(w[j])));
                v[2 * j] = tf_bf16(a);
                v[2 * j + 1] = tf_bf16(b);
                o[j] = (uint32_t)a | ((uint32_t)b << 16);
            }
            reinterpret_cast<u4v*>(normed + (size_t)row * cols)[q] = o;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = 0.f;
        }
        // whole groups of lanes are on or off together: the part's first piece and its piece count are multiples of group_lanes
        const float amax = tf_group_amax(v, group_lanes);
        if (!on) continue;
        const size_t at = (size_t)row * per_row + q;
        const int group = q / group_lanes;
        if (codes != nullptr) {
            const Quant8 c = tf_quant8(v, amax, 0.f);
            reinterpret_cast<u2v*>(codes)[at] = u2v{c.lo, c.hi};
            if ((q & (group_lanes - 1)) == 0) scales[(size_t)row * groups + group] = (uint8_t)c.exponent;
        }
        if (codes_min != nullptr || mma_scales != nullptr) {
            const Quant8 c = tf_quant8(v, amax, 1e-4f);
            if (codes_min != nullptr) reinterpret_cast<u2v*>(codes_min)[at] = u2v{c.lo, c.hi};
            if ((q & (group_lanes - 1)) == 0) {
                if (codes_min != nullptr) scales_min[(size_t)row * groups + group] = (uint8_t)c.exponent;
                if (mma_scales != nullptr)
                    mma_scales[(size_t)(row & 31) * 16 + (size_t)((row >> 5) & 3) * 4 + (size_t)(row >> 7) * ((size_t)((groups + 3) >> 2) * 512) +
                               (size_t)(group >> 2) * 512 + (size_t)(group & 3)] = (uint8_t)c.exponent;
            }
        }
    }
}
// The reference's producer with the dimensions as trailing arguments (grid (rows, parts), 256 threads).
extern "C" __global__ void __launch_bounds__(256) ca_hc_combine_norm_quant_rows(const uint16_t* x, const float* pre, const uint16_t* weight, uint16_t* normed,
                                                                           uint8_t* codes_min, uint8_t* scales_min, uint8_t* mma_scales,
                                                                           uint8_t* codes, uint8_t* scales, int cols, int streams, int act_block,
                                                                           float eps) {
    tf_hc_norm_quant_row(x, pre, weight, normed, codes, scales, codes_min, scales_min, mma_scales, cols, streams, act_block, eps);
}
// The single-stream case (a plain RMS norm with a BF16 boundary) with a caller's eps, both flavours.
extern "C" __global__ void __launch_bounds__(256) ca_rmsnorm_quant(const uint16_t* __restrict__ x, const uint16_t* __restrict__ weight,
                                                                   uint16_t* __restrict__ normed, uint8_t* __restrict__ codes,
                                                                   uint8_t* __restrict__ scales, uint8_t* __restrict__ codes_min,
                                                                   uint8_t* __restrict__ scales_min, int cols, int act_block, float eps) {
    tf_hc_norm_quant_row(x, nullptr, weight, normed, codes, scales, codes_min, scales_min, nullptr, cols, 1, act_block, eps);
}

// mhc-post-tiles.py:11-27 for 8 columns of one row: the layer's output `a` mixed into the S = 4 residual streams,
//   y[row][c][h] = bf16(fma(C[3][c], r3, fma(C[2][c], r2, fma(C[1][c], r1, fma(post[c], a, C[0][c] * r0)))))
// with C = comb[row] ([stream][c]), FP32 throughout and one BF16 rounding at the end.
__device__ __forceinline__ void tf_hc_post_piece(const u4v a, const uint16_t* __restrict__ residual, const float* __restrict__ post,
                                                 const float* __restrict__ comb, uint16_t* __restrict__ y, size_t row, int c8, int cols) {
    float av[8], r[4][8];
#pragma unroll
    for (int j = 0; j < 4; ++j) { av[2 * j] = tf_bf16_lo(a[j]); av[2 * j + 1] = tf_bf16_hi(a[j]); }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        const u4v v = reinterpret_cast<const u4v*>(residual + (row * 4 + s) * cols)[c8];
#pragma unroll
        for (int j = 0; j < 4; ++j) { r[s][2 * j] = tf_bf16_lo(v[j]); r[s][2 * j + 1] = tf_bf16_hi(v[j]); }
    }
    const float* C = comb + row * 16;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const float p = post[row * 4 + c], c0 = C[c], c1 = C[4 + c], c2 = C[8 + c], c3 = C[12 + c];
        float z[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float t = __fmaf_rn(p, av[j], __fmul_rn(c0, r[0][j]));
            t = __fmaf_rn(c1, r[1][j], t);
            t = __fmaf_rn(c2, r[2][j], t);
            z[j] = __fmaf_rn(c3, r[3][j], t);
        }
        u4v o;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = tf_pack_bf16(z[2 * j], z[2 * j + 1]);
        reinterpret_cast<u4v*>(y + (row * 4 + c) * cols)[c8] = o;
    }
}
// a [rows][cols], residual / y [rows][4][cols] BF16 (y may alias residual: a thread reads its columns of all four streams first);
// post [rows][4], comb [rows][4][4] FP32.  8 columns a thread.
extern "C" __global__ void __launch_bounds__(256) ca_hc_post_rows(const uint16_t* a, const uint16_t* residual, const float* post, const float* comb,
                                                             uint16_t* y, int rows, int cols) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x, per_row = cols >> 3;
    if (i >= rows * per_row) return;
    const long long row = i / per_row;
    tf_hc_post_piece(reinterpret_cast<const u4v*>(a)[i], residual, post, comb, y, (size_t)row, (int)(i - row * per_row), cols);
}
// ca_ffn_sum_shared with the post step behind it in one pass (the sum, the shared addition and the mix into the residual streams):
//   routed (rows < live) = bf16(sum of the row's route outputs, FP32 adds in route order); other rows keep `routed_out`
//   ffn = bf16(routed + shared), the addition flushing subnormals to zero              (written to `ffn_out` unless null)
//   y   = the post step of ffn
extern "C" __global__ void __launch_bounds__(256) ca_ffn_sum_shared_hc_post(const uint16_t* routes, const uint16_t* shared, const uint16_t* residual,
                                                                            const float* post, const float* comb, uint16_t* routed_out,
                                                                            uint16_t* ffn_out, uint16_t* y, int rows, int live, int topk, int hidden) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x, per_row = hidden >> 3;
    if (i >= rows * per_row) return;
    const long long row = i / per_row;
    u4v routed = reinterpret_cast<const u4v*>(routed_out)[i];
    if (row < live) {
        float sum[8];
        tf_sum_routes(routes, row, (int)(i - row * per_row), topk, hidden, sum);
#pragma unroll
        for (int j = 0; j < 4; ++j) routed[j] = tf_pack_bf16(sum[2 * j], sum[2 * j + 1]);
        reinterpret_cast<u4v*>(routed_out)[i] = routed;
    }
    const u4v s = reinterpret_cast<const u4v*>(shared)[i];
    u4v f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        f[j] = tf_pack_bf16(tf_ftz(__fadd_rn(tf_ftz(tf_bf16_lo(routed[j])), tf_ftz(tf_bf16_lo(s[j])))),
                            tf_ftz(__fadd_rn(tf_ftz(tf_bf16_hi(routed[j])), tf_ftz(tf_bf16_hi(s[j])))));
    if (ffn_out != nullptr) reinterpret_cast<u4v*>(ffn_out)[i] = f;
    tf_hc_post_piece(f, residual, post, comb, y, (size_t)row, (int)(i - row * per_row), hidden);
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
