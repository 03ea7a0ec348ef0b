// Code object for the reference's own layer: hidden 5,120, 384 experts, top 6, a shared-expert shard of 576 columns
// (640 with padding).  The reference's host code resolves a handful of kernels by name from its modules and launches them
// with fixed argument lists and grids in which those dimensions are not arguments (src/ffn.rs:728-732, 1041-1044,
// 1099-1102, 1228-1230; src/moe.rs:212-218; src/blockscaled.rs:54, 375; src/mhc.rs:79).  The kernels of the main code
// object carry the same names with the dimensions appended to their argument lists; the ones here take exactly the
// reference's arguments and are thin instantiations of the same device functions, so a host that launches by name with the
// reference's lists finds them in this module (titanic_moe_gfx950_reference_layer.hsaco).
#include <hip/hip_runtime.h>
// the general kernels of these names stay out of this module's symbol table
#define ca_ffn_sum_shared tf_general_ffn_sum_shared
#define ca_moe_frontend tf_general_moe_frontend
#define ca_moe_route_frontend tf_general_moe_route_frontend
#define ca_route_topk tf_general_route_topk
#define ca_moe_group_sum_rows tf_general_moe_group_sum_rows
#include "combine.cuh"
#include "frontend.cuh"
#include "shared.cuh"
#include "boundary.cuh"
#undef ca_ffn_sum_shared
#undef ca_moe_frontend
#undef ca_moe_route_frontend
#undef ca_route_topk
#undef ca_moe_group_sum_rows

namespace {
constexpr int RL_HIDDEN = 5120, RL_EXPERTS = 384, RL_TOPK = 6, RL_SHARED = 576, RL_SHARED_PADDED = 640;
constexpr int RL_SCORING = 1;                  // sqrt-softplus
constexpr float RL_ROUTE_SCALE = 1.5f;
constexpr long long RL_ALT_TOKEN = 129264;     // the image token, whose rows take the alternative selection bias
}  // namespace

// kernels/ffn_sum_shared.cuh:7-27; launched with ceil(n / 128) blocks of 128 threads (src/ffn.rs:1041-1044): an element a
// thread.  Rows below `live`: routed = bf16(sum of the row's six route outputs, FP32 adds in route order), written back;
// other rows keep what `routed_out` holds.  output = bf16(routed + shared), the addition flushing subnormals to zero.
extern "C" __global__ void __launch_bounds__(128) ca_ffn_sum_shared(const uint16_t* routes, const uint16_t* shared, uint16_t* routed_out,
                                                                    uint16_t* output, int n, int live) {
    const int i = blockIdx.x * 128 + threadIdx.x;
    if (i >= n) return;
    const int row = i / RL_HIDDEN, col = i - row * RL_HIDDEN;
    uint16_t routed = routed_out[i];
    if (row < live) {
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < RL_TOPK; ++r) sum = __fadd_rn(sum, tf_bf16(routes[((size_t)row * RL_TOPK + r) * RL_HIDDEN + col]));
        routed = tf_to_bf16(sum);
        routed_out[i] = routed;
    }
    output[i] = tf_to_bf16(tf_ftz(__fadd_rn(tf_ftz(tf_bf16(routed)), tf_ftz(tf_bf16(shared[i])))));
}

// kernels/shared_swiglu_quant.cuh:36-82.  x [rows][1,152] BF16 (gate columns, then up); a [rows][576] BF16 activation;
// q [rows][160] words of E4M3 codes (columns 576 - 639: zero); sr [rows][20] UE8M0 block scales (32 columns a block, amax
// floored at 1e-4; the two padding blocks: 0); sm: the same bytes at row * 16 + block % 4 + (block / 4) * 512.  Any grid
// of whole waves: a lane takes eight columns, four lanes a block.
__device__ __forceinline__ void rl_shared_swiglu_quant(const uint16_t* x, uint16_t* a, uint32_t* q, uint8_t* sr, uint8_t* sm, int rows) {
    constexpr int PER_ROW = RL_SHARED_PADDED / 8;
    const float hi = tf_bf16(tf_to_bf16(10.f)), lo = tf_bf16(tf_to_bf16(-10.f));
    const int total = rows * PER_ROW, padded = (total + 63) & ~63;
    for (int item = blockIdx.x * blockDim.x + threadIdx.x; item < padded; item += gridDim.x * blockDim.x) {
        const bool on = item < total;
        const int row = on ? item / PER_ROW : 0, c8 = on ? item - row * PER_ROW : 0;
        const bool real = on && c8 * 8 < RL_SHARED;
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = 0.f;
        if (real) {
            const u4v g = reinterpret_cast<const u4v*>(x + (size_t)row * 2 * RL_SHARED)[c8];
            const u4v u = reinterpret_cast<const u4v*>(x + (size_t)row * 2 * RL_SHARED + RL_SHARED)[c8];
            u4v o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[2 * i] = tf_shared_activation(tf_bf16_lo(g[i]), tf_bf16_lo(u[i]), hi, lo);
                v[2 * i + 1] = tf_shared_activation(tf_bf16_hi(g[i]), tf_bf16_hi(u[i]), hi, lo);
                o[i] = (__float_as_uint(v[2 * i]) >> 16) | (__float_as_uint(v[2 * i + 1]) & 0xffff0000u);
            }
            reinterpret_cast<u4v*>(a + (size_t)row * RL_SHARED)[c8] = o;
        }
        const float amax = tf_group_amax(v, 4);
        if (!on) continue;
        uint32_t lo_word = 0, hi_word = 0, exponent = 0;
        if (real) {
            const Quant8 c = tf_quant8(v, amax, 1e-4f);
            lo_word = c.lo; hi_word = c.hi; exponent = c.exponent;
        }
        reinterpret_cast<u2v*>(q + (size_t)row * (RL_SHARED_PADDED / 4))[c8] = u2v{lo_word, hi_word};
        if ((c8 & 3) == 0) {
            const int block = c8 >> 2;
            sr[row * (RL_SHARED_PADDED / 32) + block] = (uint8_t)exponent;
            sm[row * 16 + (block & 3) + (block >> 2) * 512] = (uint8_t)exponent;
        }
    }
}
// src/ffn.rs:1099-1102: 8 blocks of 128 threads.
extern "C" __global__ void __launch_bounds__(128) ca_shared_swiglu_quant128(const uint16_t* x, uint16_t* a, uint32_t* q, uint8_t* sr, uint8_t* sm,
                                                                            int rows) {
    rl_shared_swiglu_quant(x, a, q, sr, sm, rows);
}
// kernels/shared_swiglu_quant.cuh (the 64-thread form).
extern "C" __global__ void __launch_bounds__(64) ca_shared_swiglu_quant64(const uint16_t* x, uint16_t* a, uint32_t* q, uint8_t* sr, uint8_t* sm,
                                                                          int rows) {
    rl_shared_swiglu_quant(x, a, q, sr, sm, rows);
}
// src/ffn.rs:1228-1230: sixteen rows, 40 blocks of 64 threads.
extern "C" __global__ void __launch_bounds__(64) ca_shared_swiglu_quant16_64(const uint16_t* x, uint16_t* a, uint32_t* q, uint8_t* sr, uint8_t* sm,
                                                                             int rows) {
    rl_shared_swiglu_quant(x, a, q, sr, sm, rows);
}

// kernels/moe_frontend.cuh:154-157 (one block of 512 threads): every row's top six of 384 experts from the gate's logits.
extern "C" __global__ void __launch_bounds__(1024) ca_route_topk(const float* logits, const float* bias, const float* bias_alt, const long long* tokens,
                                                                 const int32_t* live, const int32_t* padding, int32_t* ids, float* weights,
                                                                 int32_t rows) {
    const RouteParams p{RL_EXPERTS, RL_TOPK, RL_SCORING, RL_ROUTE_SCALE, RL_ALT_TOKEN};
    const int waves = blockDim.x >> 6;
    tf_route_block<false>(logits, bias, bias_alt, tokens, live, padding, ids, weights, rows, p, blockIdx.x * waves, gridDim.x * waves,
                          gridDim.x == 1);
}
// The router operator `routing_vl` (src/ffn.rs:237, 380-395; runtime/kernels/routing-v1/manifest.json: symbol
// _router_triton_kernel, one block a row, arguments scores, bias, bias_alt, input ids, live count, out weights, out indices, M,
// then the two scratch words the reference's operator launcher appends, src/triton_ops.rs:141-142): the same top six of 384
// with the weights before the indices.  Any block of whole waves; the block's first wave routes its row.
extern "C" __global__ void __launch_bounds__(256) _router_triton_kernel(const float* scores, const float* bias, const float* bias_alt,
                                                                         const long long* input_ids, const int32_t* live, float* out_weights,
                                                                         int32_t* out_indices, int32_t M, const void*, const void*) {
    if (threadIdx.x >= 64) return;
    const RouteParams p{RL_EXPERTS, RL_TOPK, RL_SCORING, RL_ROUTE_SCALE, RL_ALT_TOKEN};
    tf_route_block<false>(scores, bias, bias_alt, input_ids, live, nullptr, out_indices, out_weights, M, p, blockIdx.x, gridDim.x, false);
}
// kernels/moe_frontend.cuh:243-252: block 0 plans, every block quantizes the rows (32 columns a block, no floor).
extern "C" __global__ void __launch_bounds__(512) ca_moe_frontend(const uint16_t* input, const int32_t* ids, const float* weights, uint8_t* packed,
                                                                  uint8_t* scales, int32_t* token_map, float* token_weights, int32_t* task_expert,
                                                                  int32_t* task_valid_rows, int32_t* expert_tile_base, int32_t rows, int32_t topk,
                                                                  int32_t experts, int32_t cols, int32_t groups, int32_t tile_m) {
    tf_frontend_run(input, ids, weights, packed, scales, nullptr, nullptr, token_map, token_weights, task_expert, task_valid_rows,
                    expert_tile_base, rows, topk, experts, cols, groups, tile_m, 32, 0);
}
// kernels/moe_frontend.cuh:256-266: block 0 routes the owner's rows from the logits, applies the padding routes and plans;
// the other blocks quantize (one block more than ca_moe_frontend's grid).
extern "C" __global__ void __launch_bounds__(512) ca_moe_route_frontend(
    const uint16_t* input, int32_t* ids, float* weights, uint8_t* packed, uint8_t* scales, int32_t* token_map, float* token_weights,
    int32_t* task_expert, int32_t* task_valid_rows, int32_t* expert_tile_base, const float* logits, const float* bias, const float* bias_alt,
    const long long* tokens, const int32_t* live, const int32_t* padding, int32_t rows, int32_t topk, int32_t experts, int32_t cols,
    int32_t groups, int32_t tile_m, int32_t owner_rows) {
    __shared__ __attribute__((aligned(16))) uint8_t s_pool[TF_FRONT_POOL_BYTES];
    tf_route_frontend(input, ids, weights, packed, scales, token_map, token_weights, task_expert, task_valid_rows, expert_tile_base,
                      const_cast<float*>(logits), bias, bias_alt, tokens, live, padding, rows, topk, experts, cols, groups, tile_m, owner_rows, 32,
                      nullptr, nullptr, RL_SCORING, RL_ROUTE_SCALE, RL_ALT_TOKEN, nullptr, nullptr, 0, (int)gridDim.x, s_pool, 0);
}

// kernels/ffn_sum_shared.cuh:35-58 (src/decoder.rs:717, 1000): the route sum of one row group of a sequence-parallel chunk, laid
// out for that group's own reduce-scatter: out[c][j][:] = bf16(ordered FP32 sum of the six route outputs of row
// c * quarter + group * per + j), c = 0..3, j < per; rows at or past `live` are not written.  Any grid that covers
// 4 * per * 5,120 / 8 threads; 8 columns a thread.
extern "C" __global__ void __launch_bounds__(256) ca_moe_group_sum_rows(const uint16_t* routes, uint16_t* out, int quarter, int per, int group,
                                                                        int live) {
    constexpr int PER_ROW = RL_HIDDEN / 8;
    const long long n = 4ll * per * PER_ROW;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const int c8 = (int)(i % PER_ROW);
        const long long t = i / PER_ROW;
        const int j = (int)(t % per), c = (int)(t / per);
        const int row = c * quarter + group * per + j;
        if (row >= live) continue;
        float sum[8];
        tf_sum_routes(routes, row, c8, RL_TOPK, RL_HIDDEN, sum);
        u4v o;
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = tf_pack_bf16(sum[2 * k], sum[2 * k + 1]);
        reinterpret_cast<u4v*>(out + ((long long)c * per + j) * RL_HIDDEN)[c8] = o;
    }
}

// The boundary operator `hc_norm_quant_p4` / `hc_norm_quant_p2` (symbol hc_combine_norm_quant;
// runtime/kernels/mhc-norm-quant-v1/mhc-norm-quant.py:15-44, src/mhc.rs:606-614, 981-990): four residual streams of 5,120
// columns, grid (rows, PARTS), 256 threads, arguments X, P, W, Y, Q, SR, SM and the two scratch words the operator launcher
// appends (src/triton_ops.rs:141-142).  eps 1e-20, 32-wide blocks.
extern "C" __global__ void __launch_bounds__(256) hc_combine_norm_quant(const uint16_t* X, const float* P, const uint16_t* W, uint16_t* Y, uint8_t* Q,
                                                                        uint8_t* SR, uint8_t* SM, const void*, const void*) {
    tf_hc_norm_quant_row(X, P, W, Y, nullptr, nullptr, Q, SR, SM, RL_HIDDEN, 4, 32, 1.0e-20f);
}
// The boundary operator `hc_post_b128_w1` (symbol hc_post_tiles; runtime/kernels/mhc-post-tiles-v1/mhc-post-tiles.py:11-27,
// src/mhc.rs:1223-1234): grid (rows, tiles), any block; a block takes 5,120 / tiles columns of its row, 8 a thread.
extern "C" __global__ void hc_post_tiles(const uint16_t* A, const uint16_t* R, const float* POST, const float* C, uint16_t* Y, const void*,
                                         const void*) {
    constexpr int PER_ROW = RL_HIDDEN / 8;
    const int tile_pieces = (PER_ROW + (int)gridDim.y - 1) / (int)gridDim.y, first = (int)blockIdx.y * tile_pieces;
    const size_t row = blockIdx.x;
    for (int q = first + (int)threadIdx.x; q < min(first + tile_pieces, PER_ROW); q += (int)blockDim.x)
        tf_hc_post_piece(reinterpret_cast<const u4v*>(A + row * RL_HIDDEN)[q], R, POST, C, Y, row, q, RL_HIDDEN);
}

// kernels/core.cu:25-28 (src/mhc.rs:79: one block of 32 threads with a stated amount of dynamic LDS): a launch that starts
// once a CU has that much LDS free, for work that should begin in the tail of the experts' launches.  Touches no model data.
extern "C" __global__ void ca_tail_gate() {
    extern __shared__ unsigned char gate[];
    if (threadIdx.x == 0) gate[0] = 1;
}
// kernels/core.cu:822-830 (src/blockscaled.rs:54; blocks of 256 threads): row-major block scales [n / 32][k / 32] spread
// to one byte a weight row and 32 columns in tiles of 128 rows x 128 columns, byte order (32-row quarter, row, block) within a tile:
// out[((nt * k_tiles + kt) * 32 + rl) * 16 + rh * 4 + kg] = scale of row nt * 128 + rh * 32 + rl, block kt * 4 + kg; 127 (2^0)
// outside the matrix.
extern "C" __global__ void __launch_bounds__(256) ca_block_scales_mma(const uint8_t* source, uint8_t* out, int n, int k, int padded_k) {
    const int index = blockIdx.x * blockDim.x + threadIdx.x;
    const int k_tiles = padded_k / 128, n_tiles = (n + 127) / 128;
    if (index >= n_tiles * 128 * (padded_k / 32)) return;
    const int kg = index & 3, rh = (index >> 2) & 3, rl = (index >> 4) & 31, tile = index >> 9;
    const int kt = tile % k_tiles, nt = tile / k_tiles;
    const int row = nt * 128 + rh * 32 + rl, block = kt * 4 + kg;
    out[index] = row < n && block < k / 32 ? source[(row / 32) * (k / 32) + block] : (uint8_t)127;
}
// kernels/core.cu:831-835 (src/blockscaled.rs:375): rows of k bytes padded with zeros to padded_k bytes.
extern "C" __global__ void __launch_bounds__(256) ca_pad_fp8_columns(const uint8_t* source, uint8_t* out, int n, int k, int padded_k) {
    const int index = blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= n * padded_k) return;
    const int row = index / padded_k, column = index - row * padded_k;
    out[index] = column < k ? source[(size_t)row * k + column] : (uint8_t)0;
}
