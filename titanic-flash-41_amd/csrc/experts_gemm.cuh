// Many-row (prefill) projections of the FP8 shared expert and the dense product: GEMM on v_mfma_scale_f32_16x16x128_f8f6f4
// (the kernel is written for routed FP4 experts as well; those run in experts_grouped.cuh and are not instantiated from here).
//
// One task = one M tile of 128 physical rows (one expert's rows, gathered through the permutation map) x one column
// group.  A workgroup of eight waves (512 threads, two waves a SIMD) keeps a 128 x 256 accumulator: wave nq holds all
// 128 rows (eight 16-row fragments) x 32 weight rows (two 16-row weight tiles), so every weight byte is requested by
// exactly one wave of the workgroup (the fetch path of a CU, not the matrix cores, bounds this kernel; the token tile is
// shared through LDS anyway):
//   FC1: 128 intermediate columns = 128 "up" + 128 "gate" weight rows (a wave: 16 + 16 of the same 16 columns), so SwiGLU
//        and the FP8 requantization of the result (one scale a row and `act_block` columns) run in the epilogue, from
//        registers;
//   FC2 / dense: 256 output columns; routed rows are scaled by their routing weight and scattered to route order.
// The E4M3 token tile goes through LDS (double-buffered, stored in matrix-instruction fragment order so every wave reads
// 1 KiB contiguous, conflict-free, per fragment; its scales are staged once a tile); the prepared weights go from global memory straight into the B operand
// (1 KiB contiguous per weight tile and k-step) through a ring of register sets, three k-steps ahead of their use.
// Workgroups are persistent and XCD-aware: workgroup b runs on XCD b % 8 and only ever touches 1/8 of the column groups,
// so every XCD's L2 holds its own slices of the expert's weights while the expert's tiles pass by; partially filled
// tiles skip the 16-row fragments past their last valid row.
//
// Reference semantics (contract level): the two phase kernels of the reference's dynamic MoE node
// (src/moe.rs:1098-1289; runtime/kernels/moe-runtime-*/manifest.json precision string) and its block-scaled dense GEMM
// for the shared expert (src/fp8_linear.rs:782-806).
#pragma once
#include "experts_stream.cuh"
#include <type_traits>

#define TF_STREAM_MAX_ROWS 64
#define TF_GEMM_TILE_M 128
#define TF_GEMM_MAX_SCALES_ROW 256                 // activation scales a row the tile table holds: k / act_block
#define TF_GEMM_SCALE_WORDS 8                       // words of that table a thread moves a pass: 128 rows x 128 bytes / 512 threads / 4 (wider rows: two passes)

struct GemmArgs {
    const uint8_t* a_codes;          // E4M3 [rows][k]: token rows (FC1), physical rows (routed FC2), dense rows
    const uint8_t* a_scales;         // UE8M0 [rows][k / act_block]
    const uint8_t* w;                // prepared weights, expert-major
    const uint8_t* ws;               // prepared scales (FP4) or row-major block scales (FP8)
    long long w_expert_stride, ws_expert_stride;
    int bn, bk;
    const int32_t* expert_tile_base; // routed: [experts + 1]
    const int32_t* task_expert;      // routed: [tile * groups]; null: dense
    const int32_t* task_valid_rows;
    const int32_t* token_map;
    const float* token_weights;
    int experts, groups, topk, max_tiles;
    int dense_rows;
    int k, inter, hidden, act_block;
    float limit;
    uint16_t* h_bf16;                // FC1: optional BF16 activation [phys_row][inter]
    uint8_t* h_codes;                // FC1: E4M3 activation codes [phys_row][inter]
    uint8_t* h_scales;               // FC1: UE8M0 [phys_row][inter / act_block]
    uint16_t* out;                   // FC2 / dense: BF16 [route or row][hidden]
    uint16_t* tap;                   // shared FC1: optional BF16 projections [row][2 inter]
};

enum { TF_GEMM_FC1_ROUTED = 0, TF_GEMM_FC1_SHARED = 1, TF_GEMM_FC2_ROUTED = 2, TF_GEMM_DENSE = 3 };

template <bool FP8>
struct BFrag { u4v lo; u4v hi; };

template <bool FP8, int MODE>
__global__ void __launch_bounds__(512) tf_gemm(const GemmArgs p) {
    constexpr bool FC1 = MODE == TF_GEMM_FC1_ROUTED || MODE == TF_GEMM_FC1_SHARED;
    constexpr bool ROUTED = MODE == TF_GEMM_FC1_ROUTED || MODE == TF_GEMM_FC2_ROUTED;
    constexpr int GROUP_COLS = FC1 ? 128 : 256;          // output columns a task covers
    __shared__ __attribute__((aligned(16))) uint8_t s_a[2][16384];     // [stage][m-frag 8][half 2][lane 64][16 B]
    __shared__ __attribute__((aligned(16))) uint8_t s_scale[128 * (TF_GEMM_MAX_SCALES_ROW + 16)];   // [row][k-block]: the tile's activation scales; the 16 rows a fragment reads at once fall into different banks
    __shared__ float s_amax[8][128];
    __shared__ long long s_row[128];                                    // source row of each tile row
    __shared__ int32_t s_route[128];                                    // routed FC2: route (output row) of each tile row
    __shared__ float s_weight[128];                                     // routed FC2: routing weight of each tile row
    // eight waves: wave nq takes 32 weight rows (two 16-row tiles) against every row fragment of the tile
    // the wave's index as a scalar: everything derived from it (weight tile addresses, LDS fragment offsets) stays out of the vector registers
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), nq = wave, g = lane >> 4, r16 = lane & 15;
    const int ksteps = p.k / 128;
    const int scales_row = p.k / p.act_block, scale_words_row = scales_row / 4, scale_stride = scales_row + 16;
    const int act_shift = p.act_block == 32 ? 5 : 7;
    const int n_cols = FC1 ? p.inter : p.hidden, groups = n_cols / GROUP_COLS;
    const int tiles = ROUTED ? p.expert_tile_base[p.experts] : (p.dense_rows + 127) / 128;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3, local_count = gridDim.x >> 3;
    const bool split = groups % 8 == 0;
    const int gpx = split ? groups / 8 : 0;
    const long long my_tasks = split ? (long long)tiles * gpx : ((long long)tiles * groups - xcd + 7) / 8;

    // What a tile needs from the plan tables is requested a whole tile ahead (with the previous tile's first operand loads), so
    // that no tile starts with a chain of dependent round trips: the tile's expert and row count, and per tile row its source
    // row (routed FC1: through the permutation map) or its route and routing weight (routed FC2).  The last tile requests
    // itself again: no load is conditional.
    struct TileRef { int tile, ng, expert, valid; long long src; int32_t route; float weight; };
    auto fetch = [&](long long q) {
        TileRef r;
        if (split) { r.tile = (int)(q / gpx); r.ng = xcd * gpx + (int)(q % gpx); }
        else { const long long id = q * 8 + xcd; r.tile = (int)(id / groups); r.ng = (int)(id % groups); }
        r.expert = 0;
        if (ROUTED) { r.expert = p.task_expert[r.tile * p.groups]; r.valid = p.task_valid_rows[r.tile * p.groups]; }
        else r.valid = min(128, p.dense_rows - r.tile * 128);
        const int at = r.tile * 128 + (tid & 127);
        r.src = at; r.route = 0; r.weight = 0.f;
        if (MODE == TF_GEMM_FC1_ROUTED) r.src = p.token_map[at];          // route index; rows past the valid ones: never looked up
        if (MODE == TF_GEMM_FC2_ROUTED) { r.route = p.token_map[at]; r.weight = p.token_weights[at]; }
        return r;
    };
    if (local >= my_tasks) return;
    TileRef next = fetch(local);
    for (long long q = local; q < my_tasks; q += local_count) {
        const TileRef cur = next;
        const int tile = cur.tile, ng = cur.ng, expert = cur.expert, valid = cur.valid;
        const uint8_t* w = p.w + (size_t)expert * p.w_expert_stride;
        const uint8_t* ws = p.ws + (size_t)expert * p.ws_expert_stride;
        __syncthreads();
        if (tid < 128) {
            s_row[tid] = MODE == TF_GEMM_FC1_ROUTED ? cur.src / p.topk : cur.src;
            if (MODE == TF_GEMM_FC2_ROUTED) { s_route[tid] = cur.route; s_weight[tid] = cur.weight; }
        }
        __syncthreads();
        next = fetch(min(q + local_count, my_tasks - 1));
        // rows past the last valid one re-read the last valid row (no load of the main loop is conditional); their products are
        // never stored
        // this thread's two 16-byte chunks of every k-step's A tile: chunk id c = tid + 512 i is LDS slot c (a wave fills one
        // 1 KiB fragment block with consecutive 16-byte slots: no bank conflicts), i.e. fragment c / 128, K half (c / 64) % 2,
        // row c % 16 of the fragment, 16-byte piece (c % 64) / 16 of the half
        const uint8_t* a_src[2];
        int a_dst[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + 512 * i, block = c >> 6, slot = c & 63;
            const int row = (block >> 1) * 16 + (slot & 15), piece = (block & 1) * 4 + (slot >> 4);
            a_src[i] = p.a_codes + s_row[min(row, valid - 1)] * p.k + piece * 16;
            a_dst[i] = c * 16;
        }
        // weight row tiles of this wave: FC1 routed: two "up" tiles then two "gate" tiles of the same 32 intermediate columns;
        // FC1 shared: gate tiles then up tiles; FC2 / dense: four tiles of 64 output columns
        int ntile[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (FC1) ntile[j] = j * (p.inter / 16) + (ng * 128 + nq * 16) / 16;
            else ntile[j] = (ng * 256 + nq * 32) / 16 + j;
        }
        auto load_a = [&](int ks, u4v (&ra)[2]) {
#pragma unroll
            for (int i = 0; i < 2; ++i) ra[i] = *reinterpret_cast<const u4v*>(a_src[i] + (size_t)ks * 128);
        };
        auto store_a = [&](int stage, const u4v (&ra)[2]) {
#pragma unroll
            for (int i = 0; i < 2; ++i) *reinterpret_cast<u4v*>(&s_a[stage][a_dst[i]]) = ra[i];
        };
        // The rows' activation scales of every k-step go to LDS once a tile (a byte a row and k-step fetched inside the main
        // loop costs a cache line request per row: as many requests as the tile's codes need).  Requested first, stored after
        // the main loop's first operand requests are out.
        uint32_t scale_regs[TF_GEMM_SCALE_WORDS];
        auto load_scales = [&](int pass) {
#pragma unroll
            for (int i = 0; i < TF_GEMM_SCALE_WORDS; ++i) {
                const int c = min(tid + 512 * (i + TF_GEMM_SCALE_WORDS * pass), 128 * scale_words_row - 1);            // word c % per_row of row c / per_row
                scale_regs[i] = *reinterpret_cast<const uint32_t*>(p.a_scales + s_row[min(c / scale_words_row, valid - 1)] * scales_row + (c % scale_words_row) * 4);
            }
        };
        auto store_scales = [&](int pass) {
#pragma unroll
            for (int i = 0; i < TF_GEMM_SCALE_WORDS; ++i) {
                const int c = tid + 512 * (i + TF_GEMM_SCALE_WORDS * pass);
                if (c < 128 * scale_words_row)
                    *reinterpret_cast<uint32_t*>(&s_scale[(c / scale_words_row) * scale_stride + (c % scale_words_row) * 4]) = scale_regs[i];
            }
        };
        load_scales(0);
        // B operand of one k-step: plain loads (an expert's weight slice is re-read by the expert's other tiles from this
        // XCD's L2).  FP8: with the lane's block scale of the k-step; FP4: scales come a word per four k-steps (load_b_scales).
        auto load_b = [&](int ks, BFrag<FP8> (&b)[2], uint32_t (&sb)[2]) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if constexpr (FP8) {
                    const u4v* src = reinterpret_cast<const u4v*>(w) + (((size_t)ntile[j] * ksteps + ks) * 2) * 64 + lane;
                    b[j].lo = src[0];
                    b[j].hi = src[64];
                    sb[j] = ws[(size_t)((ntile[j] * 16 + r16) / p.bn) * (p.k / p.bk) + (ks * 128 + 32 * g) / p.bk];
                } else {
                    b[j].lo = reinterpret_cast<const u4v*>(w)[((size_t)ntile[j] * ksteps + ks) * 64 + lane];
                }
            }
        };
        auto load_b_scales = [&](int ks, uint32_t (&sb)[2]) {
#pragma unroll
            for (int j = 0; j < 2; ++j) sb[j] = reinterpret_cast<const uint32_t*>(ws)[((size_t)ntile[j] * (p.k / 512) + ks / 4) * 64 + lane];
        };
        v4f acc[8][2];
#pragma unroll
        for (int f = 0; f < 8; ++f)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[f][j] = v4f{0.f, 0.f, 0.f, 0.f};
        const int my_frags = (valid + 15) >> 4;                    // 16-row fragments of the tile with valid rows: every wave runs them all

        // Main loop, compiled for 0, 2 or 4 row fragments of the wave's half so that its products sit under no branch (every
        // wave runs the same loads, LDS stores and barriers whatever its count).  Operands of k-step ks + D - 1 are requested
        // while k-step ks is multiplied (a ring of D register sets, indexed statically by unrolling D times): the token tile
        // goes registers -> LDS one k-step ahead of its use (two LDS stages, one barrier a k-step), the weights stay in
        // registers.  Two waves share a SIMD, so one wave's loads, LDS traffic and scalar work run under the other's products.
        auto main_loop = [&](auto fr_constant, auto words_constant) {
            constexpr int FR = decltype(fr_constant)::value;
            // 128-wide activation blocks: a k-step has one scale a row, so a word holds the scales of four k-steps (the
            // instruction selects the byte); 32-wide blocks: a byte a row, k-step and lane group
            constexpr bool WORDS = decltype(words_constant)::value;
            constexpr int U = 4;                   // k-steps an unrolled round
            constexpr int D = FP8 ? 2 : 4;         // ksteps % 4 == 0
            u4v ra[D][2];
            BFrag<FP8> b[D][2];
            uint32_t sbk[D][2];                  // FP8: the slot's scale bytes
            uint32_t sb[2] = {0, 0}, sb_next[2] = {0, 0};   // FP4: scale words of the current / next four k-steps
#pragma unroll
            for (int d = 0; d < D - 1; ++d) { load_a(d, ra[d]); load_b(d, b[d], sbk[d]); }
            if constexpr (!FP8) load_b_scales(0, sb);
            store_scales(0);
            if (scale_words_row > 4 * TF_GEMM_SCALE_WORDS) {       // more than 128 scale bytes a row (K above 4,096 with 32-wide blocks)
                load_scales(1);
                store_scales(1);
            }
            store_a(0, ra[0]);
            __syncthreads();
            int sw[FR];
            for (int ks0 = 0; ks0 < ksteps; ks0 += U) {
                if constexpr (WORDS) {
#pragma unroll
                    for (int f = 0; f < FR; ++f) sw[f] = *reinterpret_cast<const int*>(&s_scale[(f * 16 + r16) * scale_stride + ks0]);
                }
                // one k-step; its index within the round is a compile-time constant (it selects ring slots and scale bytes)
                auto k_step = [&](auto u_constant) {
                    constexpr int u = decltype(u_constant)::value;
                    const int ks = ks0 + u;
                    {
                        // No load sits under a condition (the last D - 1 k-steps request the last k-step again rather than
                        // nothing): the compiler counts outstanding loads statically, and a load that may or may not have been
                        // issued turns every wait behind it into a wait for all loads in flight.
                        const int stage = ks & 1, ahead = min(ks + D - 1, ksteps - 1);
                        load_a(ahead, ra[(u + D - 1) % D]);
                        load_b(ahead, b[(u + D - 1) % D], sbk[(u + D - 1) % D]);
                        if constexpr (!FP8) { if (u == 1) load_b_scales(ahead, sb_next); }           // ahead % 4 == 0 (D == 4)
                        if constexpr (!FP8) {
                            if (u == 0 && ks > 0) {
#pragma unroll
                                for (int j = 0; j < 2; ++j) sb[j] = sb_next[j];
                            }
                        }
                        // the next fragment's rows leave LDS while the current fragment's products run: two register sets
                        v8i av[2];
                        int sa[FR];
#pragma unroll
                        for (int f = 0; f < FR; ++f) sa[f] = WORDS ? sw[f] : s_scale[(f * 16 + r16) * scale_stride + ((ks * 128 + 32 * g) >> act_shift)];
                        constexpr int SEL = WORDS ? u : 0;        // byte of the activation scale register
                        auto read_frag = [&](int f, v8i& a) {
                            const int tf = f;                      // fragment of the tile
                            const u4v lo = *reinterpret_cast<const u4v*>(&s_a[stage][((tf * 2) * 64 + lane) * 16]);
                            const u4v hi = *reinterpret_cast<const u4v*>(&s_a[stage][((tf * 2 + 1) * 64 + lane) * 16]);
                            a = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
                        };
                        if constexpr (FR > 0) read_frag(0, av[0]);
#pragma unroll
                        for (int f = 0; f < FR; ++f) {
                            if (f + 1 < FR) read_frag(f + 1, av[(f + 1) & 1]);
                            const v8i a_now = av[f & 1];
#pragma unroll
                            for (int j = 0; j < 2; ++j) {
                                const BFrag<FP8>& bj = b[u % D][j];
                                if constexpr (FP8) {
                                    const v8i bv = v8i{(int)bj.lo[0], (int)bj.lo[1], (int)bj.lo[2], (int)bj.lo[3], (int)bj.hi[0], (int)bj.hi[1], (int)bj.hi[2], (int)bj.hi[3]};
                                    if constexpr (FC1) acc[f][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, a_now, acc[f][j], 0, 0, 0, (int)sbk[u % D][j], SEL, sa[f]);
                                    else acc[f][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a_now, bv, acc[f][j], 0, 0, SEL, sa[f], 0, (int)sbk[u % D][j]);
                                } else {
                                    const v8i bv = v8i{(int)bj.lo[0], (int)bj.lo[1], (int)bj.lo[2], (int)bj.lo[3], 0, 0, 0, 0};
                                    if constexpr (FC1) acc[f][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, a_now, acc[f][j], 4, 0, u, (int)sb[j], SEL, sa[f]);
                                    else acc[f][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a_now, bv, acc[f][j], 0, 4, SEL, sa[f], u, (int)sb[j]);
                                }
                            }
                            // a use the optimizer cannot move: without it every product of the unrolled k-steps is sunk below the
                            // barriers, the k-steps' A fragments stay alive until then and spill
#pragma unroll
                            for (int j = 0; j < 2; ++j) asm volatile("" :: "v"(acc[f][j]));
                        }
                        // issue order of the k-step: fragment f + 1's LDS reads go out before fragment f's four products
                        if constexpr (FR > 0) {
                            __builtin_amdgcn_sched_group_barrier(0x100, FR + 2, 0);
#pragma unroll
                            for (int f = 0; f < FR; ++f) {
                                if (f + 1 < FR) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                            }
                        }
                        store_a(stage ^ 1, ra[(u + 1) % D]);
                        __syncthreads();
                    }
                };
                k_step(std::integral_constant<int, 0>{});
                k_step(std::integral_constant<int, 1>{});
                k_step(std::integral_constant<int, 2>{});
                k_step(std::integral_constant<int, 3>{});
            }
        };
        if (p.act_block == 128) {
            if (my_frags > 6) main_loop(std::integral_constant<int, 8>{}, std::true_type{});
            else if (my_frags > 4) main_loop(std::integral_constant<int, 6>{}, std::true_type{});
            else if (my_frags > 2) main_loop(std::integral_constant<int, 4>{}, std::true_type{});
            else main_loop(std::integral_constant<int, 2>{}, std::true_type{});
        } else {
            if (my_frags > 6) main_loop(std::integral_constant<int, 8>{}, std::false_type{});
            else if (my_frags > 4) main_loop(std::integral_constant<int, 6>{}, std::false_type{});
            else if (my_frags > 2) main_loop(std::integral_constant<int, 4>{}, std::false_type{});
            else main_loop(std::integral_constant<int, 2>{}, std::false_type{});
        }

        // ---- epilogue --------------------------------------------------------------------------------------------------
        if constexpr (FC1) {
            // The weight tile is the instruction's first operand and the token fragment its second, so lane (g, r16) of product
            // (f, j) holds tile row 16 f + r16 and the four consecutive columns 4 g + i (i < 4) of weight tile j: a lane packs
            // its four values into one store (four E4M3 codes a word, four BF16 values a pair of words).  j = 0 / 1: the up and
            // gate tiles (shared expert: gate, up) of the wave's 16 intermediate columns.
            const float hi_lim = tf_bf16(tf_to_bf16(p.limit)), lo_lim = tf_bf16(tf_to_bf16(-p.limit));
            float hv[8][4];
            float amax[8];
#pragma unroll
            for (int f = 0; f < 8; ++f) {
                const int row = 16 * f + r16;
                float m = 0.f;
                if (MODE == TF_GEMM_FC1_SHARED) {
                    uint16_t gb[4], ub[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) { gb[i] = tf_to_bf16(acc[f][0][i]); ub[i] = tf_to_bf16(acc[f][1][i]); }
                    if (p.tap != nullptr && f < my_frags && row < valid) {
                        const size_t at = (size_t)(tile * 128 + row) * 2 * p.inter + ng * 128 + nq * 16 + 4 * g;
                        *reinterpret_cast<u2v*>(p.tap + at) = u2v{(uint32_t)gb[0] | ((uint32_t)gb[1] << 16), (uint32_t)gb[2] | ((uint32_t)gb[3] << 16)};
                        *reinterpret_cast<u2v*>(p.tap + at + p.inter) = u2v{(uint32_t)ub[0] | ((uint32_t)ub[1] << 16), (uint32_t)ub[2] | ((uint32_t)ub[3] << 16)};
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float gv = fminf(tf_bf16(gb[i]), hi_lim), uv = fminf(fmaxf(tf_bf16(ub[i]), lo_lim), hi_lim);
                        hv[f][i] = tf_bf16(tf_to_bf16(__fmul_rn(gv / __fadd_rn(1.0f, tf_exp(-gv)), uv)));
                    }
                } else {
                    // routed experts: no bit-level definition of this step exists (the reference's is inside a binary), the
                    // result is rounded to BF16 next; the many-row path takes the hardware exponential and reciprocal
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float gv = fminf(acc[f][1][i], p.limit), uv = fminf(p.limit, fmaxf(-p.limit, acc[f][0][i]));
                        hv[f][i] = tf_bf16(tf_to_bf16(__fmul_rn(__fmul_rn(gv, tf_logistic_fast(gv)), uv)));
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) m = fmaxf(m, fabsf(hv[f][i]));
                // the row's 16 columns of this wave sit in the four lanes r16 + 16 g
                m = fmaxf(m, __shfl_xor(m, 16));
                amax[f] = fmaxf(m, __shfl_xor(m, 32));
            }
            // one scale per row and 32 (two waves) or 128 (all eight waves) columns
#pragma unroll
            for (int f = 0; f < 8; ++f) if (g == 0) s_amax[nq][16 * f + r16] = amax[f];
            __syncthreads();
#pragma unroll
            for (int f = 0; f < 8; ++f) {
                const int row = 16 * f + r16;
                if (p.act_block == 128) {
                    float m = s_amax[0][row];
#pragma unroll
                    for (int w2 = 1; w2 < 8; ++w2) m = fmaxf(m, s_amax[w2][row]);
                    amax[f] = m;
                } else {
                    amax[f] = fmaxf(s_amax[nq & 6][row], s_amax[nq | 1][row]);
                }
            }
            const float min_amax = MODE == TF_GEMM_FC1_SHARED ? 1e-4f : 0.f;
#pragma unroll
            for (int f = 0; f < 8; ++f) {
                const int row = 16 * f + r16;
                if (f < my_frags && row < valid) {
                    const uint32_t exponent = tf_block_exponent(min_amax > 0.f ? fmaxf(amax[f], min_amax) : amax[f]);
                    const float inv = tf_block_inverse(exponent);
                    const size_t phys = (size_t)tile * 128 + row;
                    const int col = ng * 128 + nq * 16 + 4 * g;
                    *reinterpret_cast<uint32_t*>(p.h_codes + phys * p.inter + col) =
                        tf_pack_e4m3(__fmul_rn(hv[f][0], inv), __fmul_rn(hv[f][1], inv), __fmul_rn(hv[f][2], inv), __fmul_rn(hv[f][3], inv));
                    if (p.h_bf16 != nullptr)
                        *reinterpret_cast<u2v*>(p.h_bf16 + phys * p.inter + col) = u2v{tf_pack_bf16(hv[f][0], hv[f][1]), tf_pack_bf16(hv[f][2], hv[f][3])};
                    if (g == 0) {
                        if (p.act_block == 32) { if ((nq & 1) == 0) p.h_scales[phys * (p.inter / 32) + ng * 4 + (nq >> 1)] = (uint8_t)exponent; }
                        else if (nq == 0) p.h_scales[phys * (p.inter / 128) + ng] = (uint8_t)exponent;
                    }
                }
            }
        } else {
            // the token fragment is the first operand here: lane (g, r16) of product (f, j) holds tile rows 16 f + 4 g + i
            // (i < 4) and column r16 of weight tile j
#pragma unroll
            for (int f = 0; f < 8; ++f) {
                if (f < my_frags) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = 16 * f + 4 * g + i;
                        if (row < valid) {
                            size_t out_row = (size_t)tile * 128 + row;
                            float scale = 1.f;
                            if (MODE == TF_GEMM_FC2_ROUTED) { out_row = (size_t)s_route[row]; scale = s_weight[row]; }
#pragma unroll
                            for (int j = 0; j < 2; ++j) {
                                const float v = MODE == TF_GEMM_FC2_ROUTED ? __fmul_rn(acc[f][j][i], scale) : acc[f][j][i];
                                p.out[out_row * p.hidden + ng * 256 + nq * 32 + 16 * j + r16] = tf_to_bf16(v);
                            }
                        }
                    }
                }
            }
        }
    }
}

inline int tf_gemm_grid(int cus) { return cus >= 8 ? cus / 8 * 8 : 8; }
inline bool tf_gemm_shape_ok(const GemmArgs& a, bool fc1) {
    return a.k >= 512 && a.k % 512 == 0 && (a.act_block == 32 || a.act_block == 128) && a.k / a.act_block <= TF_GEMM_MAX_SCALES_ROW &&
           (fc1 ? (a.inter >= 128 && a.inter % 128 == 0) : (a.hidden >= 256 && a.hidden % 256 == 0));
}
// The routed experts' projections run in experts_grouped.cuh (tf_grouped_gemm); this kernel serves the FP8 shared expert and
// the dense product.
inline int tf_launch_dense_gemm(const GemmArgs& a, int cus, hipStream_t s) {
    if (!tf_gemm_shape_ok(a, false)) return -4;
    tf_gemm<true, TF_GEMM_DENSE><<<tf_gemm_grid(cus), 512, 0, s>>>(a);
    return (int)hipGetLastError();
}
inline int tf_launch_shared_fc1_gemm(const GemmArgs& a, int cus, hipStream_t s) {
    if (!tf_gemm_shape_ok(a, true)) return -4;
    tf_gemm<true, TF_GEMM_FC1_SHARED><<<tf_gemm_grid(cus), 512, 0, s>>>(a);
    return (int)hipGetLastError();
}

// Gate product for many rows: logits[rows][experts] = x . w^T, BF16 inputs, FP32 accumulate on the matrix cores
// (v_mfma_f32_32x32x16_bf16).  grid (ceil(rows / (32 XT)), ceil(experts / 256)), block 512: a workgroup keeps a 32 XT x 256 tile
// of logits, XT = 4 or 2 (wave (mr, nq): rows 16 XT mr .., experts 64 nq ..: XT / 2 x 2 accumulators of 32 x 32), so the rows
// are read from HBM once and the gate weight (2 MB) from L2 once per 32 XT rows.  Both operands go through LDS, 64 columns of K
// a step, double buffered, loaded as whole 128-byte row pieces (eight lanes a row) and stored in matrix-instruction fragment
// order: the 16-byte piece kc of row r of a 32-row tile sits in block (tile, kc / 2), half kc % 2, slot (r + 2 kc) % 32; the
// rotation by 2 kc keeps both the stores (two rows x eight pieces a phase) and the fragment reads free of bank conflicts.
// Every logit is the same sum in the same order for either tile height.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
template <int XT>
__device__ __forceinline__ void tf_router_logits_tile(const uint16_t* x, const uint16_t* w, float* out, int rows, int hidden, int experts) {
    static_assert(XT == 2 || XT == 4, "64 or 128 rows a workgroup");
    constexpr int X_TILES = XT, W_TILES = 8, STAGE = (X_TILES + W_TILES) * 4 * 1024;      // 32-row tiles; 4 KiB a tile and step
    constexpr int XA = XT / 2;                    // 32-row tiles of x a wave; also this thread's x pieces a step
    constexpr int NP = XA + 4;                    // this thread's pieces of a step: x: 32 XT rows x 8 pieces (XA a thread); w: 256 rows x 8 (4 a thread)
    __shared__ __attribute__((aligned(16))) uint8_t s_ops[2][STAGE];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), mr = wave >> 2, nq = wave & 3;
    const int r32 = lane & 31, kg = lane >> 5;
    const int row0 = blockIdx.x * (32 * XT), e0 = blockIdx.y * 256;
    const uint16_t* src[NP];
    int dst[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int is_w = i >= XA, local = tid + 512 * (is_w ? i - XA : i), r = local >> 3, kc = local & 7;
        const int tile = (is_w ? X_TILES : 0) + (r >> 5);
        const long long source_row = is_w ? min(e0 + r, experts - 1) : min(row0 + r, rows - 1);
        src[i] = (is_w ? w : x) + source_row * hidden + kc * 8;
        dst[i] = ((tile * 4 + (kc >> 1)) * 64 + (kc & 1) * 32 + ((r + 2 * kc) & 31)) * 16;
    }
    v16f acc[XA][2];
#pragma unroll
    for (int a = 0; a < XA; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;
    // operands of step s + 3 are requested while step s is multiplied: a ring of three register sets (indexed statically by
    // unrolling four steps; hidden % 256 == 0), one LDS stage ahead of the products
    constexpr int D = 4;
    u4v regs[D][NP];
    const int steps = hidden / 64;
#pragma unroll
    for (int d = 0; d < D - 1; ++d)
#pragma unroll
        for (int i = 0; i < NP; ++i) regs[d][i] = *reinterpret_cast<const u4v*>(src[i] + (size_t)min(d, steps - 1) * 64);
#pragma unroll
    for (int i = 0; i < NP; ++i) *reinterpret_cast<u4v*>(&s_ops[0][dst[i]]) = regs[0][i];
    __syncthreads();
    for (int step0 = 0; step0 < steps; step0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            const int step = step0 + u, stage = step & 1, ahead = min(step + D - 1, steps - 1);
#pragma unroll
            for (int i = 0; i < NP; ++i) regs[(u + D - 1) % D][i] = *reinterpret_cast<const u4v*>(src[i] + (size_t)ahead * 64);
#pragma unroll
            for (int sub = 0; sub < 4; ++sub) {
                const int slot = (r32 + 4 * sub + 2 * kg) & 31;                 // (r + 2 kc) % 32 with kc = 2 sub + kg
                u4v av[XA], bv[2];
#pragma unroll
                for (int a = 0; a < XA; ++a) av[a] = *reinterpret_cast<const u4v*>(&s_ops[stage][(((XA * mr + a) * 4 + sub) * 64 + kg * 32 + slot) * 16]);
#pragma unroll
                for (int b = 0; b < 2; ++b) bv[b] = *reinterpret_cast<const u4v*>(&s_ops[stage][(((X_TILES + 2 * nq + b) * 4 + sub) * 64 + kg * 32 + slot) * 16]);
#pragma unroll
                for (int a = 0; a < XA; ++a)
#pragma unroll
                    for (int b = 0; b < 2; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av[a]), __builtin_bit_cast(bf16x8, bv[b]), acc[a][b], 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < NP; ++i) *reinterpret_cast<u4v*>(&s_ops[stage ^ 1][dst[i]]) = regs[(u + 1) % D][i];
            __syncthreads();
        }
    }
#pragma unroll
    for (int a = 0; a < XA; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int e = e0 + (2 * nq + b) * 32 + r32;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = row0 + (XA * mr + a) * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);      // D[m][n = lane % 32]
                if (row < rows && e < experts) out[(size_t)row * experts + e] = acc[a][b][i];
            }
        }
}
extern "C" __global__ void __launch_bounds__(512) ca_router_logits_mfma(const uint16_t* x, const uint16_t* w, float* out, int rows,
                                                                        int hidden, int experts) {
    tf_router_logits_tile<4>(x, w, out, rows, hidden, experts);
}
// 64 rows a workgroup: twice the workgroups for the same rows (for row counts whose 128-row tiles leave CUs without one).
__global__ void __launch_bounds__(512) tf_router_logits_mfma_64(const uint16_t* x, const uint16_t* w, float* out, int rows, int hidden,
                                                                 int experts) {
    tf_router_logits_tile<2>(x, w, out, rows, hidden, experts);
}
