// Routed-expert front-end: route plan (counts, tiles, task tables, physical-row permutation) and the MXFP8
// quantization of the token rows, with the router's top-k optionally inside.
// Reference semantics: kernels/moe_frontend.cuh:158-265 (ca_moe_frontend / ca_moe_route_frontend).
#pragma once
#include "router.cuh"

// The front-end's `sync` region: 4 KiB of arrival counters (128 bytes apart) + a mailbox of 8 rows x 512 experts words.
#define TF_SYNC_BYTES (4096 + 8 * 512 * 4)

// Quantizes 8 consecutive BF16 values held by each lane of a group of `block / 8` adjacent lanes (one quantization
// block per group).  Returns the routed-flavour codes (zero block -> scale byte 0) and, when asked, the shared-flavour
// ones (amax floored at 1e-4).
struct Quant8 { uint32_t lo, hi, exponent; };
__device__ __forceinline__ Quant8 tf_quant8(const float (&v)[8], float amax, float min_amax) {
    if (min_amax > 0.f) amax = fmaxf(amax, min_amax);
    Quant8 q;
    q.exponent = tf_block_exponent(amax);
    const float inv = tf_block_inverse(q.exponent);
    q.lo = tf_pack_e4m3(__fmul_rn(v[0], inv), __fmul_rn(v[1], inv), __fmul_rn(v[2], inv), __fmul_rn(v[3], inv));
    q.hi = tf_pack_e4m3(__fmul_rn(v[4], inv), __fmul_rn(v[5], inv), __fmul_rn(v[6], inv), __fmul_rn(v[7], inv));
    return q;
}
__device__ __forceinline__ float tf_group_amax(const float (&v)[8], int group_lanes) {
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
    // groups are 4 lanes (32-wide blocks) or 16 lanes (128-wide blocks), aligned to their size
    if (group_lanes == 16) return tf_row16_max(amax);
    if (group_lanes == 4) return tf_quad_max(amax);
    for (int o = 1; o < group_lanes; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    return amax;
}
// Quantizes `rows` x `cols` BF16 values in blocks of `block` (32 or 128) columns.  Work item = 8 values; items are
// dealt to threads [first, first + count) of a virtual 1-D thread space with stride `stride`.
// `publish_min`: the floored flavour is written with device-scope stores, for readers in other workgroups of the same launch.
__device__ __forceinline__ void tf_quantize_span(const uint16_t* __restrict__ input, uint8_t* __restrict__ codes,
                                                 uint8_t* __restrict__ scales, uint8_t* __restrict__ codes_min,
                                                 uint8_t* __restrict__ scales_min, long long total_items,
                                                 int block, long long thread, long long stride, bool publish_min = false) {
    const int group_lanes = block >> 3;
    // Whole groups stay together: thread and stride are multiples of 64 apart across waves, group_lanes divides 64.
    const long long padded = (total_items + 63) & ~63ll;
    for (long long q = thread; q < padded; q += stride) {
        const bool on = q < total_items;
        float v[8];
        if (on) {
            const u4v w = reinterpret_cast<const u4v*>(input)[q];
#pragma unroll
            for (int i = 0; i < 4; ++i) { v[2 * i] = tf_bf16_lo(w[i]); v[2 * i + 1] = tf_bf16_hi(w[i]); }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = 0.f;
        }
        const float amax = tf_group_amax(v, group_lanes);
        if (!on) continue;
        if (codes != nullptr) {
            const Quant8 a = tf_quant8(v, amax, 0.f);
            reinterpret_cast<u2v*>(codes)[q] = u2v{a.lo, a.hi};
            if ((q & (group_lanes - 1)) == 0) scales[q / group_lanes] = (uint8_t)a.exponent;
        }
        if (codes_min != nullptr) {
            const Quant8 b = tf_quant8(v, amax, 1e-4f);
            if (publish_min) {
                __hip_atomic_store(reinterpret_cast<unsigned long long*>(codes_min) + q, (unsigned long long)b.lo | ((unsigned long long)b.hi << 32),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((q & (group_lanes - 1)) == 0) __hip_atomic_store(scales_min + q / group_lanes, (uint8_t)b.exponent, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                reinterpret_cast<u2v*>(codes_min)[q] = u2v{b.lo, b.hi};
                if ((q & (group_lanes - 1)) == 0) scales_min[q / group_lanes] = (uint8_t)b.exponent;
            }
        }
    }
}

// Route plan of at most 1,024 routes by one block (the block's first `experts` threads own one expert each).
__device__ __forceinline__ void tf_plan_block(const int32_t* ids, const float* weights, int32_t* token_map,
                                              float* token_weights, int32_t* task_expert, int32_t* task_valid_rows,
                                              int32_t* expert_tile_base, int pairs, int experts, int groups, int tile_m,
                                              int32_t* s_ids, float* s_weights, bool preloaded) {
    __shared__ int32_t s_base[513];
    __shared__ int32_t s_wave[16];   // blocks of at most 1,024 threads
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    if (!preloaded) {
        for (int p = t; p < pairs; p += blockDim.x) { s_ids[p] = ids[p]; s_weights[p] = weights[p]; }
        __syncthreads();
    }
    int count = 0;
    if (t < experts) for (int p = 0; p < pairs; ++p) count += s_ids[p] == t;
    const int tiles = (count + tile_m - 1) / tile_m;
    int prefix = tiles;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int below = __shfl_up(prefix, o);
        if (lane >= o) prefix += below;
    }
    if (lane == 63) s_wave[wave] = prefix;
    __syncthreads();
    int base = prefix - tiles;
    for (int w = 0; w < wave; ++w) base += s_wave[w];
    if (t == experts - 1) expert_tile_base[experts] = base + tiles;      // the total: written by the last expert's thread (experts may equal blockDim.x)
    if (t < experts) {
        expert_tile_base[t] = base;
        s_base[t] = base;
        for (int k = 0; k < tiles; ++k) {
            const int valid = min(tile_m, count - k * tile_m);
            for (int g = 0; g < groups; ++g) {
                task_expert[(base + k) * groups + g] = t;
                task_valid_rows[(base + k) * groups + g] = valid;
            }
        }
    }
    __syncthreads();
    for (int p = t; p < pairs; p += blockDim.x) {
        const int expert = s_ids[p];
        if (expert >= 0 && expert < experts) {
            int rank = 0;
            for (int q = 0; q < p; ++q) rank += s_ids[q] == expert;
            const int row = (s_base[expert] + rank / tile_m) * tile_m + rank % tile_m;
            token_map[row] = p;
            token_weights[row] = s_weights[p];
        }
    }
}

// Front-end of a few-row launch (rows * topk <= 1,024, experts < blockDim.x <= 1,024): block 0 plans the routes, the
// blocks from `first` on quantize (first = 1: block 0 only routes and plans).
__device__ __forceinline__ void tf_frontend_run(const uint16_t* input, const int32_t* ids, const float* weights,
                                                uint8_t* packed, uint8_t* scales, uint8_t* packed_min, uint8_t* scales_min,
                                                int32_t* token_map, float* token_weights, int32_t* task_expert,
                                                int32_t* task_valid_rows, int32_t* expert_tile_base, int rows, int topk,
                                                int experts, int cols, int groups, int tile_m, int act_block, int first) {
    __shared__ __attribute__((aligned(16))) int32_t s_ids[1024];
    __shared__ float s_weights[1024];
    if (blockIdx.x == 0)
        tf_plan_block(ids, weights, token_map, token_weights, task_expert, task_valid_rows, expert_tile_base,
                      rows * topk, experts, groups, tile_m, s_ids, s_weights, false);
    if ((int)blockIdx.x < first) return;
    const long long total = (long long)rows * (cols >> 3);
    tf_quantize_span(input, packed, scales, packed_min, scales_min, total, act_block,
                     (long long)(blockIdx.x - first) * blockDim.x + threadIdx.x,
                     (long long)(gridDim.x - first) * blockDim.x);
}
extern "C" __global__ void __launch_bounds__(512) ca_moe_frontend(
    const uint16_t* input, const int32_t* ids, const float* weights, uint8_t* packed, uint8_t* scales,
    int32_t* token_map, float* token_weights, int32_t* task_expert, int32_t* task_valid_rows,
    int32_t* expert_tile_base, int32_t rows, int32_t topk, int32_t experts, int32_t cols, int32_t groups,
    int32_t tile_m, int32_t act_block, uint8_t* packed_min, uint8_t* scales_min) {
    tf_frontend_run(input, ids, weights, packed, scales, packed_min, scales_min, token_map, token_weights, task_expert,
                    task_valid_rows, expert_tile_base, rows, topk, experts, cols, groups, tile_m, act_block, 0);
}
// The front-end with the router's top-k inside: block 0 first routes every owner row from the gate's logits (and
// applies padding routes), then plans; the other blocks quantize meanwhile (launch one block more).
// With `gate_w` the gate product runs here too: `logit_blocks` further blocks (one wave per expert and four rows) compute the
// logits.  Owners of at most eight rows: the logits are handed to block 0 through a mailbox of one word a logit (`sync` +
// 4 KiB: zero = empty; block 0 polls every word, takes the value and empties the word again), so neither side waits for a
// store to complete or for a counter.  Larger owners: the blocks publish the logits and count themselves in at `sync`
// (seventeen words, 128 bytes apart).  The whole `sync` region is zero before the first launch, and a launch whose waits all
// end in time leaves it zero.  Every wait is bounded by `spin_limit` polls: the waiter then does the work it waited for itself
// (block 0 forms the logits and routes every row; an item block quantizes its rows), so the kernel always ends, and sets the
// word TF_SYNC_DIRTY, which is never cleared by a kernel: what the late producers still post stays in the region, so from
// then on no launch trusts a hand-off (every waiter takes its own path at once, the results stay the same) until the host
// has zeroed the region again.  The blocks a waiter waits for need not all be resident with it: workgroups are dispatched in
// block order, the waited-for blocks wait for nothing themselves, and the blocks before them (quantizer blocks) end without
// waiting, so they reach a CU while the waiter polls; the bound covers whatever breaks that assumption.
#define TF_SYNC_QUANT_DONE 17             // arrival words (128 bytes apart) of the launch that also runs the shared expert's first projection:
#define TF_SYNC_SHARED_PASSED 18          // quantizer blocks that are done; item blocks that have read the quantizer's output
#define TF_SYNC_DIRTY 19                  // a bounded wait has expired since the host last zeroed the region
__device__ __forceinline__ bool tf_sync_trusted(const uint32_t* sync) {
    return __hip_atomic_load(sync + 32 * TF_SYNC_DIRTY, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u;
}
__device__ __forceinline__ void tf_sync_give_up(uint32_t* sync) {
    __hip_atomic_store(sync + 32 * TF_SYNC_DIRTY, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
#define TF_FRONT_SHARED_MAX_K 5120         // widest token row whose shared up / gate projection runs inside the front-end launch
// the shared expert's item blocks hold a 16-row tile's codes, its scales (32-wide blocks at most) and two sets of partial sums
#define TF_FRONT_POOL_BYTES (16 * TF_FRONT_SHARED_MAX_K + 16 * (TF_FRONT_SHARED_MAX_K / 32) + 16384)
// `grid_blocks`: the blocks of the launch that belong to the front-end (block ids [0, grid_blocks)); `s_pool`: TF_FRONT_POOL_BYTES
// of LDS (logit blocks: the token rows; block 0 of owners of at most eight rows: logits, biases, token ids, live count).
__device__ __forceinline__ void tf_route_frontend(
    const uint16_t* input, int32_t* ids, float* weights, uint8_t* packed, uint8_t* scales, int32_t* token_map,
    float* token_weights, int32_t* task_expert, int32_t* task_valid_rows, int32_t* expert_tile_base,
    float* logits, const float* bias, const float* bias_alt, const long long* tokens, const int32_t* live,
    const int32_t* padding, int32_t rows, int32_t topk, int32_t experts, int32_t cols, int32_t groups, int32_t tile_m,
    int32_t owner_rows, int32_t act_block, uint8_t* packed_min, uint8_t* scales_min, int32_t scoring,
    float route_scale, long long alt_token, const uint16_t* gate_w, uint32_t* sync, int32_t logit_blocks, int grid_blocks,
    uint8_t* s_pool, int32_t spin_limit, bool publish_min = false) {
    __shared__ __attribute__((aligned(16))) int32_t s_ids[1024];
    __shared__ float s_weights[1024];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int first_logit_block = grid_blocks - logit_blocks;
    const RouteParams p{experts, topk, scoring, route_scale, alt_token};
    // Logit blocks are group-major: block lb works on row group lb / per_group (four rows), experts 8 (lb % per_group) ..
    // More than two row groups: the last block of a group to finish routes the group's rows itself (one routing round for
    // the whole owner instead of one per eight rows in block 0) and block 0 only collects, applies padding and plans.
    const int row_groups = (owner_rows + 3) >> 2;
    const bool distributed = gate_w != nullptr && row_groups > 2;
    // experts a logit block takes: a wave each; owners of at most eight rows may use four of the eight waves (one a SIMD: the
    // product is bound by the vector pipe), when the launcher has the room for twice the blocks
    const int expert_waves = !distributed && logit_blocks == row_groups * ((experts + 3) >> 2) ? 4 : waves;      // the launcher's choice
    const int per_group = (experts + expert_waves - 1) / expert_waves;
    uint32_t* routed_groups = sync + 32 * 16;            // arrival words: 128 bytes apart; [0, 16) per row group, [16] routed groups
    uint32_t* mailbox = sync + 1024;                     // owners of at most eight rows: [row][expert], zero = empty
    if (gate_w != nullptr && (int)blockIdx.x >= first_logit_block) {
        const int lb = (int)blockIdx.x - first_logit_block, group = lb / per_group;
        const int e = wave < expert_waves ? (lb - group * per_group) * expert_waves + wave : experts;
        const int first_row = 4 * group;
        u4v* s_x = reinterpret_cast<u4v*>(s_pool);    // four token rows of at most 8,192 columns
        if (first_row < owner_rows)
            tf_logits_block(input + (size_t)first_row * cols, gate_w, logits + (size_t)first_row * experts, min(4, owner_rows - first_row), cols,
                            experts, e, lane, s_x, distributed ? nullptr : mailbox + (size_t)first_row * experts);
        if (!distributed) return;
        tf_stores_done();
        __syncthreads();
        __shared__ int last;
        if (threadIdx.x == 0) {
            last = atomicAdd(sync + 32 * group, 1u) == (uint32_t)(per_group - 1);
            if (last) __hip_atomic_store(sync + 32 * group, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);     // for the next launch
        }
        __syncthreads();
        if (!last) return;
        // rows with a padding source are block 0's to write (from their source's routes): a group router that is still running
        // after block 0's wait has expired must not write over them
        tf_route_block(logits, bias, bias_alt, tokens, live, padding, ids, weights, min(owner_rows, first_row + 4), p, first_row, waves, false,
                       nullptr, nullptr, true, true);
        tf_stores_done();
        __syncthreads();
        if (threadIdx.x == 0) atomicAdd(routed_groups, 1u);
        return;
    }
    if (blockIdx.x == 0) {
        bool routed = false;
        if (gate_w != nullptr) {
            __shared__ int arrived;
            float* s_logits = reinterpret_cast<float*>(s_pool);                       // [8][512]
            float* s_bias = s_logits + 8 * 512;                                       // [2][512]: bias, bias_alt
            long long* s_tokens = reinterpret_cast<long long*>(s_bias + 2 * 512);    // [8]
            int32_t* s_live = reinterpret_cast<int32_t*>(s_tokens + 8);
            // what routing needs besides the logits is requested now and lands while the logits are awaited
            const int t = threadIdx.x;
            float my_bias = 0.f, my_alt = 0.f;
            long long my_token = -1;
            int32_t my_live = 0;
            if (!distributed) {
                if (t < experts) { my_bias = bias[t]; if (bias_alt != nullptr) my_alt = bias_alt[t]; }
                if (t < owner_rows && tokens != nullptr) my_token = tokens[t];
                if (t == 0) my_live = live[0];
            }
            const bool trusted = tf_sync_trusted(sync);            // uniform: one word
            if (threadIdx.x == 0) arrived = trusted ? 1 : 0;
            __syncthreads();
            if (!trusted) {
                // a wait has expired in some earlier launch: the region may hold that launch's words; nothing of it is read
            } else if (distributed) {
                if (threadIdx.x < 64) {
                    int ok = 0;
                    for (int spin = 0; spin < spin_limit; ++spin) {
                        if (__hip_atomic_load(routed_groups, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (uint32_t)row_groups) { ok = 1; break; }
                        __builtin_amdgcn_s_sleep(2);
                    }
                    if (lane == 0 && ok) __hip_atomic_store(routed_groups, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (lane == 0 && !ok) { arrived = 0; tf_sync_give_up(sync); }
                }
            } else {
                // every thread takes its words of the mailbox as they arrive and empties them for the next launch
                for (int i = threadIdx.x; i < owner_rows * experts; i += blockDim.x) {
                    uint32_t word = 0;
                    for (int spin = 0; spin < spin_limit; ++spin) {
                        word = __hip_atomic_load(mailbox + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (word != 0u) break;
                        __builtin_amdgcn_s_sleep(1);
                    }
                    if (word != 0u) {
                        s_logits[i] = __uint_as_float(~word);
                        __hip_atomic_store(mailbox + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    } else {
                        arrived = 0;
                        tf_sync_give_up(sync);
                    }
                }
                if (t < experts) { s_bias[t] = my_bias; s_bias[512 + t] = my_alt; }
                if (t < owner_rows) s_tokens[t] = my_token;
                if (t == 0) *s_live = my_live;
            }
            __syncthreads();
            if (!arrived) {              // a bound expired (now or in an earlier launch): this block forms the logits (and routes) itself
                for (int e = wave; e < experts; e += waves) tf_logits_expert(input, gate_w, logits, owner_rows, cols, experts, e, lane);
                tf_stores_done();
                __syncthreads();
            } else if (distributed) {
                // collect the groups' routes (written by other workgroups of this launch), then padding rows
                for (int i = threadIdx.x; i < owner_rows * topk; i += blockDim.x) {
                    s_ids[i] = (int32_t)__hip_atomic_load(reinterpret_cast<const uint32_t*>(ids) + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    s_weights[i] = tf_acquire_f32(weights + i);
                }
                __syncthreads();
                tf_apply_padding(padding, ids, weights, owner_rows, topk, s_ids, s_weights);
                routed = true;
            } else {
                tf_route_block<false>(s_logits, s_bias, bias_alt != nullptr ? s_bias + 512 : nullptr, tokens != nullptr ? s_tokens : nullptr, s_live,
                                      padding, ids, weights, owner_rows, p, 0, waves, true, s_ids, s_weights);
                routed = true;
            }
        }
        if (!routed)
            tf_route_block(logits, bias, bias_alt, tokens, live, padding, ids, weights, owner_rows, p, 0, waves, true, s_ids, s_weights);
    }
    if ((int)blockIdx.x >= first_logit_block) return;
    // quantizer blocks are blocks [1, first_logit_block)
    if (blockIdx.x == 0) {
        // the executed rows are the owner's first `rows` rows, so their routes are the first rows * topk of the LDS copy
        tf_plan_block(ids, weights, token_map, token_weights, task_expert, task_valid_rows, expert_tile_base, rows * topk, experts, groups, tile_m,
                      s_ids, s_weights, true);
        return;
    }
    const long long total = (long long)rows * (cols >> 3);
    tf_quantize_span(input, packed, scales, packed_min, scales_min, total, act_block,
                     (long long)(blockIdx.x - 1) * blockDim.x + threadIdx.x, (long long)(first_logit_block - 1) * blockDim.x, publish_min);
    if (publish_min) {           // readers in this launch wait for every quantizer block (TF_SYNC_QUANT_DONE)
        tf_stores_done();
        __syncthreads();
        if (threadIdx.x == 0) atomicAdd(sync + 32 * TF_SYNC_QUANT_DONE, 1u);
    }
}
extern "C" __global__ void __launch_bounds__(512) ca_moe_route_frontend(
    const uint16_t* input, int32_t* ids, float* weights, uint8_t* packed, uint8_t* scales, int32_t* token_map,
    float* token_weights, int32_t* task_expert, int32_t* task_valid_rows, int32_t* expert_tile_base,
    float* logits, const float* bias, const float* bias_alt, const long long* tokens, const int32_t* live,
    const int32_t* padding, int32_t rows, int32_t topk, int32_t experts, int32_t cols, int32_t groups, int32_t tile_m,
    int32_t owner_rows, int32_t act_block, uint8_t* packed_min, uint8_t* scales_min, int32_t scoring,
    float route_scale, long long alt_token, const uint16_t* gate_w, uint32_t* sync, int32_t logit_blocks, int32_t spin_limit) {
    __shared__ __attribute__((aligned(16))) uint8_t s_pool[TF_FRONT_POOL_BYTES];
    tf_route_frontend(input, ids, weights, packed, scales, token_map, token_weights, task_expert, task_valid_rows, expert_tile_base, logits, bias,
                      bias_alt, tokens, live, padding, rows, topk, experts, cols, groups, tile_m, owner_rows, act_block, packed_min, scales_min,
                      scoring, route_scale, alt_token, gate_w, sync, logit_blocks, (int)gridDim.x, s_pool, spin_limit);
}
// Row quantizer alone (any number of rows).
extern "C" __global__ void __launch_bounds__(256) ca_quantize_rows(
    const uint16_t* input, uint8_t* packed, uint8_t* scales, uint8_t* packed_min, uint8_t* scales_min, long long rows,
    int32_t cols, int32_t act_block) {
    tf_quantize_span(input, packed, scales, packed_min, scales_min, rows * (cols >> 3), act_block,
                     (long long)blockIdx.x * blockDim.x + threadIdx.x, (long long)gridDim.x * blockDim.x);
}

// ---- Wide plan (any number of routes): four kernels, no atomics, same tables as the one-block plan. -----------------
// 1. One wave per 64 consecutive routes: each route's rank among the wave's earlier routes of its expert, and the wave's
//    per-expert counts.
extern "C" __global__ void __launch_bounds__(256) ca_plan_wave_counts(
    const int32_t* ids, int32_t pairs, int32_t experts, int32_t* wave_counts, int32_t* local_rank) {
    __shared__ int32_t s_count[4][512];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int wave = blockIdx.x * 4 + w, p = wave * 64 + lane;
    if (wave * 64 >= pairs) return;
    for (int e = lane; e < experts; e += 64) s_count[w][e] = 0;
    int id = p < pairs ? ids[p] : -1;
    if (id >= experts) id = -1;
    unsigned long long todo = __ballot(id >= 0);
    int rank = 0;
    while (todo) {
        const int leader = __ffsll((long long)todo) - 1;
        const int which = __shfl(id, leader);
        const unsigned long long same = __ballot(id == which);
        if (id == which) rank = __popcll(same & ((1ull << lane) - 1ull));
        if (lane == leader) s_count[w][which] = __popcll(same);
        todo &= ~same;
    }
    if (p < pairs) local_rank[p] = rank;
    __builtin_amdgcn_wave_barrier();
    for (int e = lane; e < experts; e += 64) wave_counts[(size_t)wave * experts + e] = s_count[w][e];
}
// 2a. One block per expert: exclusive prefix of the expert's wave counts (in place); the expert's route count goes to
//     expert_tile_base[expert] for step 2b.
extern "C" __global__ void __launch_bounds__(256) ca_plan_scan(int32_t* wave_counts, int32_t waves, int32_t experts, int32_t* expert_tile_base) {
    __shared__ int32_t s_wave[4];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, e = blockIdx.x;
    if (e >= experts) return;
    const int per = (waves + 255) >> 8, first = t * per, last = min(first + per, waves);
    int sum = 0;
    for (int w = first; w < last; ++w) sum += wave_counts[(size_t)w * experts + e];
    int prefix = sum;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int below = __shfl_up(prefix, o);
        if (lane >= o) prefix += below;
    }
    if (lane == 63) s_wave[wave] = prefix;
    __syncthreads();
    int run = prefix - sum;
    for (int w = 0; w < wave; ++w) run += s_wave[w];
    for (int w = first; w < last; ++w) {
        const int c = wave_counts[(size_t)w * experts + e];
        wave_counts[(size_t)w * experts + e] = run;
        run += c;
    }
    if (t == 255) expert_tile_base[e] = run;
}
// 2b. One block, one thread per expert: tiles from the counts step 2a left in expert_tile_base, tile bases, task tables.
extern "C" __global__ void __launch_bounds__(512) ca_plan_tiles(int32_t experts, int32_t groups, int32_t tile_m, int32_t* expert_tile_base,
                                                                int32_t* task_expert, int32_t* task_valid_rows) {
    __shared__ int32_t s_wave[8];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int count = t < experts ? expert_tile_base[t] : 0;
    __syncthreads();
    const int tiles = (count + tile_m - 1) / tile_m;
    int prefix = tiles;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int below = __shfl_up(prefix, o);
        if (lane >= o) prefix += below;
    }
    if (lane == 63) s_wave[wave] = prefix;
    __syncthreads();
    int base = prefix - tiles;
    for (int w = 0; w < wave; ++w) base += s_wave[w];
    if (t == experts - 1) expert_tile_base[experts] = base + tiles;      // the total: written by the last expert's thread (experts may equal blockDim.x)
    if (t < experts) expert_tile_base[t] = base;
    if (t < experts)
        for (int k = 0; k < tiles; ++k) {
            const int valid = min(tile_m, count - k * tile_m);
            for (int g = 0; g < groups; ++g) {
                task_expert[(base + k) * groups + g] = t;
                task_valid_rows[(base + k) * groups + g] = valid;
            }
        }
}
// 3. Every route: physical row from the expert's tile base and the route's rank.
extern "C" __global__ void __launch_bounds__(256) ca_plan_scatter(
    const int32_t* ids, const float* weights, const int32_t* wave_counts, const int32_t* local_rank,
    const int32_t* expert_tile_base, int32_t pairs, int32_t experts, int32_t tile_m, int32_t* token_map,
    float* token_weights) {
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= pairs) return;
    const int e = ids[p];
    if (e < 0 || e >= experts) return;
    const int rank = wave_counts[(size_t)(p >> 6) * experts + e] + local_rank[p];
    const int row = (expert_tile_base[e] + rank / tile_m) * tile_m + rank % tile_m;
    token_map[row] = p;
    token_weights[row] = weights[p];
}
