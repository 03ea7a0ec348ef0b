// Many-row (prefill) routed-expert projections: grouped GEMM with both operands streamed into LDS by the memory system.
//
// One task = one unit of an expert's physical rows x its column groups.  BM = 256: a unit is two consecutive plan tiles of
// the same expert and a task takes one column group (FC1: 128 intermediate columns = 128 "up" + 128 "gate" weight rows;
// FC2: 256 output columns).  BM = 128: a unit is one plan tile and a task takes two column groups, so that a wave's
// products a k-step are the same in both.  A workgroup of eight waves (two a SIMD): wave (wm, wn) holds token rows
// [wm BM/4, +BM/4) against weight rows [128 wn, +128) of each of the task's groups, i.e. 32 products of
// v_mfma_scale_f32_16x16x128_f8f6f4 a k-step of 128.
//
// No operand of the main loop passes through vector registers on its way in: token codes (E4M3, gathered through the
// permutation map), their UE8M0 scales, the prepared FP4 weights and their scales are written into LDS by
// global_load_lds (16 or 4 bytes a lane, a wave's 64 lanes land at consecutive LDS addresses), two k-steps ahead of
// their use, in a ring of three stages.  The loads are issued from inline assembly, so the compiler's own wait
// insertion does not know them (it would wait for every load in flight before each LDS read); the kernel counts them
// itself: loads complete in issue order, every wave issues the same number of them in every k-step, and a wait allows
// exactly the loads issued after the needed ones to stay in flight.
//
// The two waves of a SIMD run half a k-step apart (waves 0 - 3 "early", 4 - 7 "late"): a wave passes one barrier a k-step,
// the early waves at its top, the late waves in its middle.  Behind a barrier the next stage is whole and the previous
// one is free; while one wave of a SIMD waits at its barrier and for its first operands from LDS, the other multiplies.
//
// Token tile in LDS: row-major, 128 bytes a row and k-step, the 16-byte pieces of a row permuted by a function of the
// row so that the eight lanes that copy one row read one whole 128-byte line of global memory while the sixteen rows a
// matrix-instruction fragment reads at once fall into different banks.  Weights in LDS: as prepared (1 KiB a 16-row
// weight tile and k-step in fragment order).
//
// Workgroups are persistent; workgroup b runs on XCD b % 8.  The XCDs take contiguous runs of the units of equal cost
// (BM = 256; of equal count at BM = 128).  BM = 128: all column groups of a unit at about the same time on neighbouring
// CUs of an XCD, so a unit's token rows reach the XCD's L2 once while its workgroups pass.  BM = 256, where an expert has
// several units and its weights do not stay in the L2 from one to the next: four units of an expert side by side, column
// group by column group, so that neighbouring workgroups want the same weight columns at the same time; units of more
// than 128 rows first (one duration: the neighbours stay in step), the experts' short last units after them.  The next
// task's first operands are requested before the current task's epilogue (SwiGLU + FP8 requantization, or routing weight
// + scatter), which needs no registers for them.
//
// Reference semantics (contract level): the two phase kernels of the reference's dynamic MoE node
// (src/moe.rs:1098-1289; runtime/kernels/moe-runtime-*/manifest.json precision string).
#pragma once
#include "experts_gemm.cuh"

// Lane l of the wave copies 16 (4) bytes from global address base + offset (a scalar base, the lane's own 32-bit byte
// offset) to LDS byte address lds_base + 16 l (4 l).
__device__ __forceinline__ void tf_dma16(const uint8_t* base, uint32_t offset, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(offset), "s"(base), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void tf_dma4(const uint8_t* base, uint32_t offset, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(offset), "s"(base), "s"(lds_base) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void tf_wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// Workgroup barrier that orders LDS accesses only (no wait for loads from global memory in flight).
__device__ __forceinline__ void tf_lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
__device__ __forceinline__ uint32_t tf_lds_addr(const void* p) {
    return (uint32_t)(size_t)(const __attribute__((address_space(3))) uint8_t*)p;
}
// acc += weights (FP4, first operand) x tokens (FP8, second operand) with the accumulator held in place (written as
// assembly: the compiler's own form of this instruction writes a fresh destination for every product, and 128 accumulator
// registers a lane then no longer fit beside the operands).  SW / ST: which byte of the weight / token scale registers
// applies.  Lane (g, r) of the result holds weight rows 4 g .. 4 g + 3 of the 16-row weight tile for token row r of the
// fragment.  Hazards the compiler does not see: results are read by vector instructions only after tf_mfma_settle().
template <int SW, int ST>
__device__ __forceinline__ void tf_mfma_weights_first(v4f& acc, const u4v& weights, const v8i& tokens, uint32_t scale_w, uint32_t scale_t) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%8,0] cbsz:4"
                 : "+v"(acc) : "v"(weights), "v"(tokens), "v"(scale_w), "v"(scale_t), "n"(SW & 1), "n"(ST & 1), "n"(SW >> 1), "n"(ST >> 1));
}
// The same product with FP8 (E4M3) weights: eight registers a lane for the first operand too, no format modifier.
template <int SW, int ST>
__device__ __forceinline__ void tf_mfma_fp8_weights_first(v4f& acc, const v8i& weights, const v8i& tokens, uint32_t scale_w, uint32_t scale_t) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%8,0]"
                 : "+v"(acc) : "v"(weights), "v"(tokens), "v"(scale_w), "v"(scale_t), "n"(SW & 1), "n"(ST & 1), "n"(SW >> 1), "n"(ST >> 1));
}
// The matrix pipeline's last results have reached the registers (the longest product takes 8 passes of 4 cycles; 32 idle
// cycles follow the last product before any of these eight accumulators is read).
__device__ __forceinline__ void tf_mfma_settle(v4f (&acc)[8]) {
    asm volatile("s_nop 15\n\ts_nop 15"
                 : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7]));
}
// Requests that may still be in flight at the barrier of k-step `u` of an unrolled round of four: those issued in the
// LEAD - 1 k-steps before it.  Every k-step issues DATA requests, k-step EXTRA of a round MORE more (the next round's weight
// scales).  Requests the count does not know (the next tasks' permutation map, stores) only make the wait stricter: it
// lets the N youngest stay in flight, and whatever is younger than the k-step's own requests may.
template <int LEAD, int DATA, int EXTRA, int MORE>
constexpr int tf_loads_behind(int u) {
    int n = 0;
    for (int j = 1; j < LEAD; ++j) n += DATA + (((u - j) & 3) == EXTRA ? MORE : 0);
    return n;
}

// What a 256-row unit costs by its rows (more than 128 / more than 32 / fewer), for the XCDs' shares.
#ifndef TF_UNIT_COST
#define TF_UNIT_COST 5
#define TF_UNIT_COST_SHORT 3
#define TF_UNIT_COST_TINY 2
#endif
#ifndef TF_GROUPED_SHARE
#define TF_GROUPED_SHARE 4
#endif
// 256-row units: the prefix of the units' costs is held in 16 bits
#define TF_GROUPED_MAX_UNITS (65535 / TF_UNIT_COST)

template <int MODE, int BM, bool WORDS>
__global__ void __launch_bounds__(512) tf_grouped_gemm(const GemmArgs p) {
    constexpr bool FC1 = MODE == TF_GEMM_FC1_ROUTED || MODE == TF_GEMM_FC1_SHARED;
    // The FP8 shared expert and the dense product: rows in place (no plan, no permutation map: tile t holds rows 128 t ..),
    // one weight matrix, E4M3 weights (2 KiB a 16-row weight tile and k-step: two requests) with row-major block scales.
    constexpr bool FP8B = MODE == TF_GEMM_FC1_SHARED || MODE == TF_GEMM_DENSE;
    static_assert(!FP8B || BM == 128, "FP8 weights: a ring stage holds a 128-row unit and one column group");
    constexpr int BREQ = FP8B ? 2 : 1;       // 1 KiB requests a weight tile and k-step
    constexpr int NG = FP8B || BM == 256 ? 1 : 2;    // column groups a task: a 128-row unit of FP4 weights takes two, so that a wave's products a
                                             // k-step (and with them the k-step's fixed costs a product) are those of a 256-row unit
    constexpr int NS = 3, LEAD = NS - 1;
    constexpr int NA = BM / 64;              // 16-byte pieces of the token tile a thread requests a k-step
    constexpr int NF = BM / 64;              // 16-row fragments of a wave (BM / 4 rows)
    constexpr int NT = 8 * NG;               // weight tiles a wave multiplies its fragments with
    constexpr int NB = 2 * NG;               // weight tiles a wave requests a k-step
    constexpr int WROWS = BM / 4;
    constexpr int DATA = NA + 1 + NB * BREQ; // requests a wave issues a k-step: token pieces, token scales, weight tiles
    constexpr int MORE = FP8B ? 0 : NB;      // and once a round of four k-steps: the next round's prepared weight scale words
    constexpr int A_STAGE = BM * 128, B_STAGE = 16 * 1024 * NG * BREQ;
    constexpr int ROW_WAVES = BM / 64;       // waves whose 64 lanes cover the tile's rows once; the other waves repeat them
    __shared__ __attribute__((aligned(1024))) uint8_t s_a[NS * A_STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t s_b[NS * B_STAGE];
    __shared__ __attribute__((aligned(256))) uint32_t s_asc[NS][BM];
    __shared__ __attribute__((aligned(256))) uint32_t s_bsc[FP8B ? 64 : 16 * NG * 64];
    // FP8 weights: the block scales of the task's 256 weight rows, as they lie in memory ([row block][k / bk] bytes), for three tasks in turn
    __shared__ __attribute__((aligned(256))) uint32_t s_wsc[FP8B ? 3 : 1][FP8B ? 512 : 64];
    __shared__ __attribute__((aligned(256))) int32_t s_src[3][BM];   // the permutation map's entry (route index) of each tile row, for three tasks in turn
    __shared__ __attribute__((aligned(256))) float s_wgt[NG == 2 ? 4 : 3][BM];   // FC2: routing weight of each tile row (three tasks in turn); FC1: row maxima of the column halves
    __shared__ uint16_t s_ubase[BM == 256 ? 514 : 2], s_nbase[BM == 256 ? 514 : 2];      // units / short last units before expert e
    __shared__ int32_t s_part[8], s_cpart[8], s_npart[8], s_bound[9], s_nbound[9];
    constexpr int SHARE = TF_GROUPED_SHARE;  // BM == 256: units of an expert whose tasks of one column group run next to each other
    uint16_t* s_cbase = reinterpret_cast<uint16_t*>(s_a);      // prefix of the units' costs: needed before the ring starts only

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1, g = lane >> 4, r16 = lane & 15;
    const int KS = p.k / 128, scales_row = p.k / p.act_block;
    const int groups = (FC1 ? p.inter / 128 : p.hidden / 256) / NG;          // a task's column groups: ng NG .. ng NG + NG - 1
    const int total_tiles = FP8B ? (p.dense_rows + 127) / 128 : p.expert_tile_base[p.experts];
    int units = total_tiles;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3, local_count = gridDim.x >> 3;
    int u_lo, u_hi, n_lo = 0, n_hi = 0;      // the XCD's units; BM == 256: short last units before them
    if constexpr (BM == 256) {
        // units of two plan tiles: per expert ceil(tiles / 2); exclusive prefix over the experts (one thread an expert).  Beside
        // it a prefix of what the units cost: a unit with more than 128 rows keeps both waves of every SIMD multiplying (5), one
        // with fewer rows one wave a SIMD (3; up to 32 rows: half of that wave's fragments, 2).  The experts come in no
        // particular order of size, and where they come sorted (popular experts first) equal counts of units an XCD would leave
        // the XCDs with the small experts idle for a third of the launch: the XCDs take equal shares of the cost.
        const int e = tid;
        int tb = 0, tn = 0;
        if (e < p.experts) { tb = p.expert_tile_base[e]; tn = p.expert_tile_base[e + 1]; }
        const int mine = (tn - tb + 1) >> 1;
        int cost = 0, small_last = 0;        // small: the expert's last unit has at most 128 rows (one wave a SIMD multiplies: a shorter task)
        if (mine > 0) {
            const int last_rows = (tn - tb - 1) * 128 + p.task_valid_rows[(size_t)(tn - 1) * p.groups] - 256 * (mine - 1);
            cost = TF_UNIT_COST * (mine - 1) + (last_rows > 128 ? TF_UNIT_COST : last_rows > 32 ? TF_UNIT_COST_SHORT : TF_UNIT_COST_TINY);
            small_last = last_rows <= 128;
        }
        int prefix = mine, cprefix = cost, nprefix = small_last;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int below = __shfl_up(prefix, o), cbelow = __shfl_up(cprefix, o), nbelow = __shfl_up(nprefix, o);
            if (lane >= o) { prefix += below; cprefix += cbelow; nprefix += nbelow; }
        }
        if (lane == 63) { s_part[wave] = prefix; s_cpart[wave] = cprefix; s_npart[wave] = nprefix; }
        __syncthreads();
        for (int w = 0; w < wave; ++w) { prefix += s_part[w]; cprefix += s_cpart[w]; nprefix += s_npart[w]; }
        if (e < p.experts) { s_ubase[e + 1] = (uint16_t)prefix; s_nbase[e + 1] = (uint16_t)nprefix; s_cbase[e + 1] = (uint16_t)cprefix; }
        if (e == 0) { s_ubase[0] = 0; s_nbase[0] = 0; s_cbase[0] = 0; }
        __syncthreads();
        units = s_ubase[p.experts];
        if (tid <= 8) {             // boundary tid of the XCDs' shares: the first unit at or behind tid eighths of the cost
            const int total_cost = s_cbase[p.experts], target = (int)((long long)total_cost * tid / 8);
            int lo = 0, hi = p.experts;                     // the expert with s_cbase[lo] <= target < s_cbase[lo + 1]
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if ((int)s_cbase[mid] <= target) lo = mid; else hi = mid;
            }
            const int in_expert = (int)s_ubase[lo + 1] - (int)s_ubase[lo];
            const int bound = tid == 8 ? units : min((int)s_ubase[lo] + min((target - (int)s_cbase[lo]) / TF_UNIT_COST, in_expert), units);
            s_bound[tid] = tid == 0 ? 0 : bound;
            // short last units before the boundary
            s_nbound[tid] = tid == 0 ? 0 : tid == 8 ? (int)s_nbase[p.experts] : (int)s_nbase[bound >= (int)s_ubase[lo + 1] ? lo + 1 : lo];
        }
        __syncthreads();
        u_lo = s_bound[xcd];
        u_hi = s_bound[xcd + 1];
        n_lo = s_nbound[xcd];
        n_hi = s_nbound[xcd + 1];
    } else {
        u_lo = (int)((long long)units * xcd / 8);
        u_hi = (int)((long long)units * (xcd + 1) / 8);
    }
    const int my_tasks = (u_hi - u_lo) * groups;
    if (local >= my_tasks) return;

    // What a task needs from the plan is requested two tasks ahead, and not through vector registers either (a load the
    // compiler knows of makes it wait for every load in flight, the ring's requests included, before the loaded register's
    // next use): the tile rows' entries of the permutation map (and their routing weights) go to an LDS slot like every other
    // operand; the task's scalars (tile, expert, valid rows) are scalar loads.
    struct TaskRef { int ng, first_tile, rows, expert; };      // the same in every lane
    auto scalar_load = [](const int32_t* at) {
        int32_t v;
        asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(at) : "memory");
        return v;
    };
    const uint32_t lds_src = tf_lds_addr(&s_src[0][0]), lds_wgt = tf_lds_addr(&s_wgt[0][0]);
    // BM == 256: the XCD's tasks in two parts.  First the units of more than 128 rows (every unit but an expert's last, and
    // the last one too if it is that long: both waves of every SIMD multiply, one duration): within an expert the units
    // fastest, SHARE at a time, then the column groups, so that the workgroups next to each other in a round multiply SHARE
    // row blocks by the same weight columns at about the same time and those weights cross the fabric once for all of them
    // (an expert's weights do not stay in an XCD's L2 from one unit to the next; equal durations keep the neighbours in
    // step, and a workgroup that falls behind finds its weights in the L2 and catches up).  Then the experts' short last
    // units (s_nbase counts them), a unit's column groups next to each other.
    const int first_part = (u_hi - n_hi) - (u_lo - n_lo);          // units of the first part
    const int w_lo = u_lo - n_lo;                                   // units of the first part before this XCD's
    int walk = 0, walk_last = 0;             // the expert of the last unit looked up in either part (each asked for in ascending order)
    auto lds16 = [](const uint16_t* at) { return __builtin_amdgcn_readfirstlane((int)*at); };
    auto fetch = [&](int q, int slot) {
        TaskRef r;
        if constexpr (BM == 256) {
            int unit;
            if (q < first_part * groups) {
                // position w among the units of the first part; expert e holds [s_ubase[e] - s_nbase[e], s_ubase[e + 1] - s_nbase[e + 1])
                const int w = w_lo + q / groups;
                while (lds16(&s_ubase[walk + 1]) - lds16(&s_nbase[walk + 1]) <= w) ++walk;
                const int before = lds16(&s_nbase[walk]);
                const int a = max(lds16(&s_ubase[walk]) - before, w_lo), b = min(lds16(&s_ubase[walk + 1]) - lds16(&s_nbase[walk + 1]), w_lo + first_part);
                const int t = q - (a - w_lo) * groups, blk = t / (SHARE * groups);
                const int mb = min(SHARE, b - a - SHARE * blk), rem = t - blk * SHARE * groups;
                r.ng = rem / mb;
                unit = a + SHARE * blk + (rem - r.ng * mb) + before;
                r.expert = walk;
            } else {
                const int j = (q - first_part * groups) / groups;
                r.ng = q - first_part * groups - j * groups;
                while (lds16(&s_nbase[walk_last + 1]) <= n_lo + j) ++walk_last;      // the expert of the (n_lo + j)-th short last unit
                unit = lds16(&s_ubase[walk_last + 1]) - 1;
                r.expert = walk_last;
            }
            const int k2 = unit - lds16(&s_ubase[r.expert]);
            const int tb = scalar_load(p.expert_tile_base + r.expert), tn = scalar_load(p.expert_tile_base + r.expert + 1);
            r.first_tile = tb + 2 * k2;
            r.rows = min(BM, (tn - tb - 1) * 128 + scalar_load(p.task_valid_rows + (size_t)(tn - 1) * p.groups) - 256 * k2);
        } else if constexpr (FP8B) {
            const int un = q / groups, unit = u_lo + un;
            r.ng = q - un * groups;
            r.first_tile = unit;
            r.expert = 0;
            r.rows = min(BM, p.dense_rows - unit * BM);
            // the block scales of the task's weight rows: word i of the slot = word i % wpr of row block i / wpr of the task
            // (FC1: the column group's 128 "gate" rows, then its 128 "up" rows; otherwise 256 consecutive rows)
            const int per_block = p.k / p.bk, wpr = per_block >> 2, half_blocks = 128 / p.bn;
            const int i = min(wave * 64 + lane, 2 * half_blocks * wpr - 1), rb = i / wpr, j = i - rb * wpr;
            const int block = FC1 ? (rb < half_blocks ? (r.ng * 128) / p.bn + rb : (p.inter + r.ng * 128) / p.bn + rb - half_blocks)
                                  : (r.ng * 256) / p.bn + rb;
            tf_dma4(p.ws, (uint32_t)(block * per_block + j * 4), tf_lds_addr(&s_wsc[slot][0]) + wave * 256);
            return r;
        } else {
            const int un = q / groups, unit = u_lo + un;
            r.ng = q - un * groups;
            r.first_tile = unit;
            r.expert = scalar_load(p.task_expert + (size_t)unit * p.groups);
            r.rows = scalar_load(p.task_valid_rows + (size_t)unit * p.groups);
        }
        const uint32_t at = (uint32_t)min(r.first_tile * 128 + ((wave & (ROW_WAVES - 1)) * 64 + lane), total_tiles * 128 - 1) * 4u;
        tf_dma4(reinterpret_cast<const uint8_t*>(p.token_map), at, lds_src + slot * (BM * 4) + (wave & (ROW_WAVES - 1)) * 256);
        if constexpr (!FC1) tf_dma4(reinterpret_cast<const uint8_t*>(p.token_weights), at, lds_wgt + slot * (BM * 4) + (wave & (ROW_WAVES - 1)) * 256);
        return r;
    };

    // ---- request state: where this thread's pieces of a k-step come from, for the current task and the one after -----------
    // Every request is a scalar base (operand array + the k-step's offset, or the expert's weight tile) plus the lane's own
    // 32-bit byte offset, which stays the same for a whole task.
    struct Source {
        uint32_t a_off[NA], asc_off;
        const uint8_t* b_base[NB];
        const uint8_t* bsc_base[NB];
    };
    const uint32_t lds_a = tf_lds_addr(s_a), lds_b = tf_lds_addr(s_b), lds_asc = tf_lds_addr(&s_asc[0][0]), lds_bsc = tf_lds_addr(s_bsc);
    // The task's slot has landed and is visible (a wait for the requests and a barrier lie between its request and this).
    auto install = [&](Source& src, const TaskRef& task, int slot) {
        const int ng = task.ng, first_tile = task.first_tile, expert = task.expert, rows = task.rows;
        auto source_row = [&](int row) -> uint32_t {         // rows past the valid ones request the first row's bytes again
            if constexpr (FC1 && !FP8B) return (uint32_t)(s_src[slot][row < rows ? row : 0] / p.topk);
            else return (uint32_t)(first_tile * 128 + (row < rows ? row : 0));
        };
#pragma unroll
        for (int c = 0; c < NA; ++c) {
            const int row = (wave * NA + c) * 8 + (lane >> 3);
            const int piece = (lane & 7) ^ ((row & 7) ^ ((row >> 3) & 1));
            src.a_off[c] = source_row(row) * (uint32_t)p.k + piece * 16;
        }
        src.asc_off = source_row((wave & (ROW_WAVES - 1)) * 64 + lane) * (uint32_t)scales_row;
        const uint8_t* w = p.w + (size_t)expert * p.w_expert_stride;
        const uint8_t* ws = p.ws + (size_t)expert * p.ws_expert_stride;
#pragma unroll
        for (int c = 0; c < NB; ++c) {
            const int T = (wave * NB + c) & 15, cg = ng * NG + (wave * NB + c) / 16;       // tile within its column group, the group
            const int ntile = FC1 ? (T < 8 ? cg * 8 + T : p.inter / 16 + cg * 8 + T - 8) : cg * 16 + T;
            src.b_base[c] = w + (size_t)ntile * KS * (1024 * BREQ);
            src.bsc_base[c] = ws + (size_t)ntile * (p.k / 512) * 256;       // (FP4 weights: prepared scale words)
        }
    };
    const uint32_t lane16 = lane * 16, lane4 = lane * 4;
    // Request `op` of k-step `ks` of a task into ring stage `stage`: ops [0, NA): token pieces, NA: token scales, then NB weight
    // tiles; ops DATA .. DATA + NB - 1: those tiles' scales of round `ks / 4` (four k-steps a word).
    auto issue_op = [&](const Source& src, int op, int ks, int stage) {
        if (op < NA) tf_dma16(p.a_codes + (size_t)ks * 128, src.a_off[op], lds_a + stage * A_STAGE + (wave * NA + op) * 1024);
        else if (op == NA) tf_dma4(p.a_scales + (WORDS ? (ks >> 2) * 4 : ks * 4), src.asc_off, lds_asc + stage * (BM * 4) + (wave & (ROW_WAVES - 1)) * 256);
        else if (op < DATA) {
            // FP8 weights: request 2 c + half is the 1 KiB plane `half` of the wave's tile c (consecutive in memory and in the stage)
            const int c = (op - NA - 1) / BREQ, piece = op - NA - 1;
            tf_dma16(src.b_base[c] + (size_t)ks * (1024 * BREQ) + (piece - c * BREQ) * 1024, lane16, lds_b + stage * B_STAGE + (wave * NB * BREQ + piece) * 1024);
        }
        else tf_dma4(src.bsc_base[op - DATA] + (size_t)(ks >> 2) * 256, lane4, lds_bsc + (wave * NB + op - DATA) * 256);
    };

    // ---- this lane's fragment addresses ----------------------------------------------------------------------------------
    const int swz = (r16 & 7) ^ (r16 >> 3);
    // weight tiles of the wave within a stage: FC1: four "up" tiles 4 wn + t, then the four "gate" tiles 8 + 4 wn + t of the same
    // columns; FC2: tiles 8 wn + t.  One base a wave plus a constant a tile.
    const int b_first = FC1 ? wn * 4 : wn * 8;
    // Waves w and w + 4 share a SIMD.  Waves 4 - 7 ("late") run half a k-step behind waves 0 - 3 ("early"): a wave passes one
    // barrier a k-step, the early waves at its top, the late waves in its middle (and one more before their first k-step, as
    // the early waves do after their last), so the early waves' barrier of k-step b is the late waves' of k-step b - 1.
    // While one wave of a SIMD waits at its barrier and for its first operands from LDS, the other is in the middle of
    // its products.
    const bool late = wave >= 4;
    auto b_step = [](int t) constexpr { return FC1 ? (t < 4 ? t : 8 + t - 4) : t; };

    // ---- the first task's first k-steps, and the second task's slot ------------------------------------------------------------
    Source now, then;
    TaskRef cur = fetch(local, 0);
    tf_wait_vm<0>();
    tf_lds_barrier();
    install(now, cur, 0);
    if constexpr (!FP8B) {
#pragma unroll
        for (int c = 0; c < NB; ++c) issue_op(now, DATA + c, 0, 0);
    }
#pragma unroll
    for (int d = 0; d < LEAD; ++d)
#pragma unroll
        for (int op = 0; op < DATA; ++op) issue_op(now, op, d, d);
    if (late) {                             // the late waves request one k-step further ahead throughout
#pragma unroll
        for (int op = 0; op < DATA; ++op) issue_op(now, op, LEAD, LEAD);
    }
    TaskRef nxt = fetch(min(local + local_count, my_tasks - 1), 1);
    tf_wait_vm<0>();
    int cs = 0, ps = LEAD;                  // stage read in the current k-step; stage the k-step LEAD ahead is written to
    if (late) __builtin_amdgcn_s_barrier();
    int slot = 0, slot_next = 1, slot_after = 2;
    for (int q = local; q < my_tasks; q += local_count) {
        const int rows = cur.rows, first_tile = cur.first_tile, ng = cur.ng;
        // A unit of at most BM / 2 rows spreads them over all eight waves (wave row groups of BM / 8 rows, half the fragments
        // each) instead of leaving the upper row groups' waves without products: both waves of every SIMD then multiply, one
        // under the other's barrier and LDS latency.
        const int wbase = wm * (rows <= BM / 2 ? WROWS / 2 : WROWS);          // first tile row of this wave
        const int nf = max(0, min(rows <= BM / 2 ? NF / 2 : NF, (rows - wbase + 15) >> 4));     // fragments of this wave with valid rows
        const int a_lo = (wbase + r16) * 128 + ((g ^ swz) << 4), a_hi = a_lo ^ 64;     // + 2,048 a fragment
        TaskRef after = nxt;
        // FP8 weights: where the block scales of the wave's weight tile t start in the task's table (tile T of the stage: rows
        // 16 T .. of the task's first 128 weight rows, or 16 (T - 8) .. of its second)
        int wsc_row[8];
        const int bk_shift = p.bk == 32 ? 5 : p.bk == 64 ? 6 : 7;
        if constexpr (FP8B) {
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int T = b_first + b_step(t);
                wsc_row[t] = ((FC1 && T >= 8 ? 128 / p.bn + ((T - 8) * 16) / p.bn : (T * 16) / p.bn)) * (p.k / p.bk);
            }
        }

        // One task, compiled for 0, NF / 2 or NF fragments of the wave so that no product sits under a branch and the
        // accumulators are as many as the wave needs; every wave issues the same requests and passes the same barriers
        // whatever its count.
        auto run_task = [&](auto frags_constant) {
            constexpr int FR = decltype(frags_constant)::value, FRA = FR > 0 ? FR : 1;
            v4f acc[FRA][NT];
#pragma unroll
            for (int f = 0; f < FRA; ++f)
#pragma unroll
                for (int t = 0; t < NT; ++t) acc[f][t] = v4f{0.f, 0.f, 0.f, 0.f};
            uint32_t bsc[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) bsc[t] = 0;
            // One k-step.  FIRST / LAST: in the task's first / last round of four.  The requests of k-step ks + LEAD (the next
            // task's first k-steps in the last round: the ring runs on across tasks) are issued between the fragments' products,
            // so that their address arithmetic runs under the matrix pipeline.
            auto k_step = [&](auto u_constant, auto first_constant, auto last_constant, int ks) {
                constexpr int u = decltype(u_constant)::value;
                constexpr bool FIRST = decltype(first_constant)::value, LAST = decltype(last_constant)::value;
                // The k-step's barrier: at the top for the early waves, in the middle for the late waves, whose barrier of k-step
                // u is the early waves' of k-step u + 1.  Behind barrier b (the early waves' top of k-step b) the stage of k-step b
                // is whole (every wave waited for its share before it) and no wave reads the stage of k-step b - 1 any more (the
                // late waves have taken their last fragments of it into registers before their barrier), so every wave then
                // requests its share of k-step b + LEAD into it: the early waves in k-step b, the late waves in the second half
                // of their k-step b - 1.  A task's first k-steps landed before the previous task's stores went out (below).
                if (!late) {
                    if constexpr (!FIRST || u >= LEAD) tf_wait_vm<tf_loads_behind<LEAD, DATA, 1, MORE>(u)>();
                    __builtin_amdgcn_s_barrier();
                }
                asm volatile("" ::: "memory");
                if constexpr (FIRST && u == 0) install(then, nxt, slot_next);
                // requests of this k-step: `ahead` k-steps on (early waves LEAD, late waves LEAD + 1), the next task's in its last;
                // one k-step of a round (`extra`: the early waves' 1, the late waves' 0) first requests the next round's weight
                // scales: behind that k-step's barrier no wave reads this round's any more (they are in registers since the top
                // of k-step 0), and the early waves' top of the next round's k-step 0 finds them landed by either count
                auto issue_range = [&](auto ahead_constant, auto extra_constant) {
                    constexpr int AHEAD = decltype(ahead_constant)::value;
                    constexpr bool EXTRA = decltype(extra_constant)::value == u;
                    constexpr bool OVER = LAST && u + AHEAD >= 4;
                    const int ks_ahead = OVER ? u + AHEAD - 4 : ks + AHEAD;
                    const Source& from = OVER ? then : now;
                    const int stage = AHEAD == LEAD ? ps : (ps + 1 == NS ? 0 : ps + 1);
                    if constexpr (EXTRA && !FP8B) {
#pragma unroll
                        for (int i = 0; i < NB; ++i) issue_op(LAST ? then : now, DATA + i, LAST ? 0 : ks + 4 - u, 0);
                    }
#pragma unroll
                    for (int i = 0; i < DATA; ++i) issue_op(from, i, ks_ahead, stage);
                };
                const std::integral_constant<int, LEAD> early_ahead;
                const std::integral_constant<int, LEAD + 1> late_ahead;
                const std::integral_constant<int, 1> early_extra;
                const std::integral_constant<int, 0> late_extra;
                auto middle = [&]() {
                    if (late) {
                        // the late waves' share of the next k-step's stage (the next task's first, after a task's last k-step);
                        // what they requested for the task's first LEAD + 1 k-steps landed before their last stores
                        constexpr bool WAIT = u == 3 || !(FIRST && u + 1 <= LEAD);
                        if constexpr (WAIT) tf_wait_vm<tf_loads_behind<LEAD, DATA, 0, MORE>(u)>();
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // this k-step's last reads of its stage have returned
                        __builtin_amdgcn_s_barrier();
                        asm volatile("" ::: "memory");
                        issue_range(late_ahead, late_extra);
                    }
                };
                constexpr int HALF = (FR + 1) / 2;                     // fragments before the late waves' barrier
                if constexpr (FR == 0) {
                    if (!late) issue_range(early_ahead, early_extra);
                    middle();
                }
                if constexpr (FR > 0 && NG == 2) {
                    // Two column groups: the wave's (at most two) token fragments stay in registers for the whole k-step and
                    // the weights pass in four blocks of four tiles (group, then "up" / "gate" or lower / upper half), the next
                    // block leaving LDS under the current block's products.  The late waves' barrier stands before the last
                    // block's products: every read of the stage has been issued a block earlier.
                    const uint8_t* sa = s_a + cs * A_STAGE;
                    const uint8_t* sb = s_b + cs * B_STAGE + lane16;
                    const uint32_t* sc = &s_asc[cs][wbase + r16];
                    auto block_at = [&](int b) constexpr { return ((b >> 1) * 16 + (FC1 ? ((b & 1) ? 8 + 4 * wn : 4 * wn) : 8 * wn + 4 * (b & 1))) * 1024; };
                    u4v bf[2][4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) bf[0][t] = *reinterpret_cast<const u4v*>(sb + block_at(0) + t * 1024);
                    if constexpr (u == 0) {
#pragma unroll
                        for (int b = 0; b < 4; ++b)
#pragma unroll
                            for (int t = 0; t < 4; ++t) bsc[b * 4 + t] = s_bsc[block_at(b) / 16 + t * 64 + lane];
                    }
                    v8i av[FR];
                    uint32_t sca[FR];
#pragma unroll
                    for (int f = 0; f < FR; ++f) {
                        const u4v l = *reinterpret_cast<const u4v*>(sa + a_lo + f * 2048), h = *reinterpret_cast<const u4v*>(sa + a_hi + f * 2048);
                        av[f] = v8i{(int)l[0], (int)l[1], (int)l[2], (int)l[3], (int)h[0], (int)h[1], (int)h[2], (int)h[3]};
                        sca[f] = WORDS ? sc[f * 16] : sc[f * 16] >> (8 * g);
                    }
                    constexpr int SEL = WORDS ? u : 0;
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        if (b == 3) middle();
                        if (b + 1 < 4) {
#pragma unroll
                            for (int t = 0; t < 4; ++t) bf[(b + 1) & 1][t] = *reinterpret_cast<const u4v*>(sb + block_at(b + 1) + t * 1024);
                        }
#pragma unroll
                        for (int f = 0; f < FR; ++f)
#pragma unroll
                            for (int t = 0; t < 4; ++t) tf_mfma_weights_first<u, SEL>(acc[f][b * 4 + t], bf[b & 1][t], av[f], bsc[b * 4 + t], sca[f]);
                        if (b == 0) { if (!late) issue_range(early_ahead, early_extra); }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if constexpr (FR > 0 && NG == 1) {
                    const uint8_t* sa = s_a + cs * A_STAGE;
                    const uint8_t* sb = s_b + cs * B_STAGE + b_first * (1024 * BREQ) + lane16;
                    const uint32_t* sc = &s_asc[cs][wbase + r16];
                    u4v bf[8], bf_hi[FP8B ? 8 : 1];
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        bf[t] = *reinterpret_cast<const u4v*>(sb + b_step(t) * (1024 * BREQ));
                        if constexpr (FP8B) bf_hi[t] = *reinterpret_cast<const u4v*>(sb + b_step(t) * 2048 + 1024);
                    }
                    if constexpr (FP8B) {
                        // the weights' block scale of this k-step and lane group: byte (128 ks + 32 g) / bk of the tile's row block
                        const uint8_t* table = reinterpret_cast<const uint8_t*>(&s_wsc[slot][0]) + ((ks * 128 + 32 * g) >> bk_shift);
#pragma unroll
                        for (int t = 0; t < 8; ++t) bsc[t] = table[wsc_row[t]];
                    } else if constexpr (u == 0) {
#pragma unroll
                        for (int t = 0; t < 8; ++t) bsc[t] = s_bsc[b_first * 64 + lane + b_step(t) * 64];
                    }
                    // fragment f + 1 leaves LDS while fragment f is multiplied: two register sets
                    u4v lo[2], hi[2];
                    uint32_t word[2];
                    lo[0] = *reinterpret_cast<const u4v*>(sa + a_lo);
                    hi[0] = *reinterpret_cast<const u4v*>(sa + a_hi);
                    word[0] = sc[0];
#pragma unroll
                    for (int f = 0; f < FR; ++f) {
                        if (f == HALF) middle();
                        if (f + 1 < FR && f + 1 <= HALF) {
                            lo[(f + 1) & 1] = *reinterpret_cast<const u4v*>(sa + a_lo + (f + 1) * 2048);
                            hi[(f + 1) & 1] = *reinterpret_cast<const u4v*>(sa + a_hi + (f + 1) * 2048);
                            word[(f + 1) & 1] = sc[(f + 1) * 16];
                        }
                        const u4v l = lo[f & 1], h = hi[f & 1];
                        const uint32_t sca = WORDS ? word[f & 1] : word[f & 1] >> (8 * g);
                        constexpr int SEL = WORDS ? u : 0;
                        const v8i av = v8i{(int)l[0], (int)l[1], (int)l[2], (int)l[3], (int)h[0], (int)h[1], (int)h[2], (int)h[3]};
                        if constexpr (FP8B) {
#pragma unroll
                            for (int t = 0; t < 8; ++t) {
                                const v8i bv = v8i{(int)bf[t][0], (int)bf[t][1], (int)bf[t][2], (int)bf[t][3], (int)bf_hi[t][0], (int)bf_hi[t][1], (int)bf_hi[t][2], (int)bf_hi[t][3]};
                                tf_mfma_fp8_weights_first<0, SEL>(acc[f][t], bv, av, bsc[t], sca);
                            }
                        } else {
#pragma unroll
                            for (int t = 0; t < 8; ++t) tf_mfma_weights_first<u, SEL>(acc[f][t], bf[t], av, bsc[t], sca);
                        }
                        // the early waves' requests of the k-step behind their first fragment's products, so that their address
                        // arithmetic runs under the matrix pipeline (the late waves': behind their barrier, above)
                        if (f == 0) { if (!late) issue_range(early_ahead, early_extra); }
                        __builtin_amdgcn_sched_barrier(0);       // keeps fragment f + 2's reads behind these products: two register sets
                        // the fragment behind the middle barrier's first leaves LDS before that barrier too, into the registers
                        // these products have just read: behind the barrier no wave reads this stage
                        if (f == HALF - 1 && HALF + 1 < FR) {
                            static_assert(FR <= 4, "two register sets");
                            lo[(HALF + 1) & 1] = *reinterpret_cast<const u4v*>(sa + a_lo + (HALF + 1) * 2048);
                            hi[(HALF + 1) & 1] = *reinterpret_cast<const u4v*>(sa + a_hi + (HALF + 1) * 2048);
                            word[(HALF + 1) & 1] = sc[(HALF + 1) * 16];
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                    if constexpr (HALF == FR) middle();
                }
                cs = cs + 1 == NS ? 0 : cs + 1;
                ps = ps + 1 == NS ? 0 : ps + 1;
                // the plan's entries for the task after the next: a chain of dependent scalar steps, taken by the two waves of a
                // SIMD in different k-steps so that one of them always has products to issue
                if constexpr (FIRST && (u == 1 || u == 2)) {
                    if ((wave < 4) == (u == 1)) after = fetch(min(q + 2 * local_count, my_tasks - 1), slot_after);
                }
            };
            auto round = [&](auto first_constant, auto last_constant, int ks0) {
                k_step(std::integral_constant<int, 0>{}, first_constant, last_constant, ks0);
                k_step(std::integral_constant<int, 1>{}, first_constant, last_constant, ks0 + 1);
                k_step(std::integral_constant<int, 2>{}, first_constant, last_constant, ks0 + 2);
                k_step(std::integral_constant<int, 3>{}, first_constant, last_constant, ks0 + 3);
            };
            if (KS == 4) round(std::true_type{}, std::true_type{}, 0);
            else {
                round(std::true_type{}, std::false_type{}, 0);
                for (int ks0 = 4; ks0 < KS - 4; ks0 += 4) round(std::false_type{}, std::false_type{}, ks0);
                round(std::false_type{}, std::true_type{}, KS - 4);
            }
#pragma unroll
            for (int f = 0; f < FR; ++f)
#pragma unroll
                for (int gi = 0; gi < NG; ++gi) tf_mfma_settle(*reinterpret_cast<v4f (*)[8]>(&acc[f][gi * 8]));

            // ---- epilogue: values first, then a wait for every request in flight (the next task's first k-steps, long landed
            // by now: its first LEAD k-steps then wait for nothing, in particular not for the stores below), then the stores ---
            // Lane (g, r16) of product (f, t) holds tile row wbase + 16 f + r16 and the four consecutive columns 4 g + i of
            // weight tile t of column group `cg`; the task's column groups one after the other.
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                const int cg = ng * NG + gi;
                if constexpr (FC1) {
                    // t < 4: "up" tiles, t >= 4: the "gate" tiles of the same columns 64 wn + 16 (t % 4) + 4 g + i of the group
                    float hv[FRA][4][4];
                    float amax[FRA][2];
                    uint32_t codes[FRA][4], exponent[FRA][2];
                    float (*s_max)[BM] = s_wgt + 2 * gi;          // [wn][row]: FC1 keeps no routing weights here
                    // the shared expert: "gate" tiles first, then "up"; both projections are rounded to BF16 (and kept, where the caller
                    // asks for them), clamped in BF16, and the activation is the exact-sequence one (its bits are the oracle's)
                    u2v tap_gate[FP8B ? FRA : 1][4], tap_up[FP8B ? FRA : 1][4];
                    const float hi_lim = tf_bf16(tf_to_bf16(p.limit)), lo_lim = tf_bf16(tf_to_bf16(-p.limit));
#pragma unroll
                    for (int f = 0; f < FR; ++f) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            if constexpr (FP8B) {
                                const v4f gq = acc[f][j], uq = acc[f][4 + j];
                                tap_gate[f][j] = u2v{tf_pack_bf16(gq[0], gq[1]), tf_pack_bf16(gq[2], gq[3])};
                                tap_up[f][j] = u2v{tf_pack_bf16(uq[0], uq[1]), tf_pack_bf16(uq[2], uq[3])};
#pragma unroll
                                for (int i = 0; i < 4; ++i) {
                                    const uint32_t gw = tap_gate[f][j][i >> 1], uw = tap_up[f][j][i >> 1];
                                    const float gv = fminf((i & 1) ? tf_bf16_hi(gw) : tf_bf16_lo(gw), hi_lim);
                                    const float uv = fminf(fmaxf((i & 1) ? tf_bf16_hi(uw) : tf_bf16_lo(uw), lo_lim), hi_lim);
                                    hv[f][j][i] = tf_bf16(tf_to_bf16(__fmul_rn(gv / __fadd_rn(1.0f, tf_exp(-gv)), uv)));
                                }
                            } else {
#pragma unroll
                                for (int i = 0; i < 4; ++i) {
                                    const float gv = fminf(acc[f][gi * 8 + 4 + j][i], p.limit), uv = fminf(p.limit, fmaxf(-p.limit, acc[f][gi * 8 + j][i]));
                                    hv[f][j][i] = tf_bf16(tf_to_bf16(__fmul_rn(__fmul_rn(gv, tf_logistic_fast(gv)), uv)));
                                }
                            }
                        }
#pragma unroll
                        for (int b = 0; b < 2; ++b) {
                            float m = 0.f;
#pragma unroll
                            for (int j = 2 * b; j < 2 * b + 2; ++j)
#pragma unroll
                                for (int i = 0; i < 4; ++i) m = fmaxf(m, fabsf(hv[f][j][i]));
                            m = fmaxf(m, __shfl_xor(m, 16));
                            amax[f][b] = fmaxf(m, __shfl_xor(m, 32));       // over the 32 columns of weight tiles 2 b, 2 b + 1
                        }
                    }
                    if constexpr (WORDS) {               // one scale a row and 128 columns: both column halves (waves wn = 0, 1)
#pragma unroll
                        for (int f = 0; f < FR; ++f) if (g == 0) s_max[wn][wbase + 16 * f + r16] = fmaxf(amax[f][0], amax[f][1]);
                        tf_lds_barrier();
#pragma unroll
                        for (int f = 0; f < FR; ++f) {
                            const int row = wbase + 16 * f + r16;
                            amax[f][0] = amax[f][1] = fmaxf(s_max[0][row], s_max[1][row]);
                        }
                    }
#pragma unroll
                    for (int f = 0; f < FR; ++f)
#pragma unroll
                        for (int b = 0; b < 2; ++b) {
                            exponent[f][b] = tf_block_exponent(FP8B ? fmaxf(amax[f][b], 1e-4f) : amax[f][b]);     // the shared expert's quantizer floors amax
                            const float inv = tf_block_inverse(exponent[f][b]);
#pragma unroll
                            for (int j = 2 * b; j < 2 * b + 2; ++j)
                                codes[f][j] = tf_pack_e4m3(__fmul_rn(hv[f][j][0], inv), __fmul_rn(hv[f][j][1], inv), __fmul_rn(hv[f][j][2], inv), __fmul_rn(hv[f][j][3], inv));
                        }
                    if (gi == 0) tf_wait_vm<0>();
#pragma unroll
                    for (int f = 0; f < FR; ++f) {
                        const int row = wbase + 16 * f + r16;
                        if (row < rows) {
                            const size_t phys = (size_t)first_tile * 128 + row;
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                const int col = cg * 128 + wn * 64 + j * 16 + 4 * g;
                                *reinterpret_cast<uint32_t*>(p.h_codes + phys * p.inter + col) = codes[f][j];
                                if (p.h_bf16 != nullptr)
                                    *reinterpret_cast<u2v*>(p.h_bf16 + phys * p.inter + col) = u2v{tf_pack_bf16(hv[f][j][0], hv[f][j][1]), tf_pack_bf16(hv[f][j][2], hv[f][j][3])};
                                if constexpr (FP8B) {
                                    if (p.tap != nullptr) {
                                        *reinterpret_cast<u2v*>(p.tap + phys * 2 * p.inter + col) = tap_gate[f][j];
                                        *reinterpret_cast<u2v*>(p.tap + phys * 2 * p.inter + p.inter + col) = tap_up[f][j];
                                    }
                                }
                            }
                            if (g == 0) {
                                if constexpr (WORDS) { if (wn == 0) p.h_scales[phys * (p.inter / 128) + cg] = (uint8_t)exponent[f][0]; }
                                else {
                                    p.h_scales[phys * (p.inter / 32) + cg * 4 + wn * 2] = (uint8_t)exponent[f][0];
                                    p.h_scales[phys * (p.inter / 32) + cg * 4 + wn * 2 + 1] = (uint8_t)exponent[f][1];
                                }
                            }
                        }
                    }
                } else {
                    // output columns 256 cg + 128 wn + 16 t + 4 g + i of the row's route, scaled by its routing weight
                    u2v packed[FRA][8];
                    size_t out_at[FRA];
#pragma unroll
                    for (int f = 0; f < FR; ++f) {
                        const int row = min(wbase + 16 * f + r16, BM - 1);
                        if constexpr (FP8B) {          // dense product: rows in place, no routing weight
                            out_at[f] = ((size_t)first_tile * 128 + row) * p.hidden + cg * 256 + wn * 128 + 4 * g;
#pragma unroll
                            for (int t = 0; t < 8; ++t)
                                packed[f][t] = u2v{tf_pack_bf16(acc[f][t][0], acc[f][t][1]), tf_pack_bf16(acc[f][t][2], acc[f][t][3])};
                        } else {
                            const float share = s_wgt[slot][row];
                            out_at[f] = (size_t)s_src[slot][row] * p.hidden + cg * 256 + wn * 128 + 4 * g;
#pragma unroll
                            for (int t = 0; t < 8; ++t)
                                packed[f][t] = u2v{tf_pack_bf16(__fmul_rn(acc[f][gi * 8 + t][0], share), __fmul_rn(acc[f][gi * 8 + t][1], share)),
                                                   tf_pack_bf16(__fmul_rn(acc[f][gi * 8 + t][2], share), __fmul_rn(acc[f][gi * 8 + t][3], share))};
                        }
                    }
                    if (gi == 0) tf_wait_vm<0>();
#pragma unroll
                    for (int f = 0; f < FR; ++f)
                        if (wbase + 16 * f + r16 < rows) {
#pragma unroll
                            for (int t = 0; t < 8; ++t) *reinterpret_cast<u2v*>(p.out + out_at[f] + 16 * t) = packed[f][t];
                        }
                }
            }
            if constexpr (FR == 0) tf_wait_vm<0>();
        };
        if (nf > NF / 2) run_task(std::integral_constant<int, NF>{});
        else if (nf > 0) run_task(std::integral_constant<int, NF / 2>{});
        else run_task(std::integral_constant<int, 0>{});
        cur = nxt;
        nxt = after;
        now = then;
        const int done = slot;
        slot = slot_next; slot_next = slot_after; slot_after = done;
    }
    if (!late) __builtin_amdgcn_s_barrier();
}

// Shapes the streamed grouped GEMM takes: contraction lengths that are multiples of 512, at most 512 experts (one thread an
// expert in the unit prefix), whole column groups.
inline bool tf_grouped_shape_ok(const GemmArgs& a, bool fc1) {
    return a.k >= 512 && a.k % 512 == 0 && (a.act_block == 32 || a.act_block == 128) && a.experts <= 512 &&
           (fc1 ? (a.inter >= 256 && a.inter % 256 == 0) : (a.hidden >= 512 && a.hidden % 512 == 0));
}
// The FP8 shared expert's first projection (MODE TF_GEMM_FC1_SHARED) and the dense product (TF_GEMM_DENSE) on the same ring:
// whole column groups, contraction lengths that are multiples of 512, weight scale blocks of 32, 64 or 128 rows and columns.
inline bool tf_grouped_dense_shape_ok(const GemmArgs& a, bool fc1) {
    return a.k >= 512 && a.k % 512 == 0 && (a.act_block == 32 || a.act_block == 128) && (a.bn == 32 || a.bn == 64 || a.bn == 128) &&
           (a.bk == 32 || a.bk == 64 || a.bk == 128) && a.k <= 8192 && a.dense_rows >= 1 &&
           (unsigned long long)((a.dense_rows + 127) / 128) * 128ull * (unsigned long long)a.k <= 0xffffffffull &&
           (fc1 ? (a.inter >= 128 && a.inter % 128 == 0) : (a.hidden >= 256 && a.hidden % 256 == 0));
}
template <int MODE>
inline int tf_launch_grouped_dense(const GemmArgs& a, int cus, hipStream_t s) {
    static_assert(MODE == TF_GEMM_FC1_SHARED || MODE == TF_GEMM_DENSE, "dense rows");
    if (!tf_grouped_dense_shape_ok(a, MODE == TF_GEMM_FC1_SHARED)) return -4;
    const int grid = tf_gemm_grid(cus);
    if (a.act_block == 128) tf_grouped_gemm<MODE, 128, true><<<grid, 512, 0, s>>>(a);
    else tf_grouped_gemm<MODE, 128, false><<<grid, 512, 0, s>>>(a);
    return (int)hipGetLastError();
}
// `routes`: rows x top-k of the launch; experts with about two plan tiles or more on average run 256-row units.
template <int MODE>
inline int tf_launch_grouped(const GemmArgs& a, long long routes, int cus, hipStream_t s) {
    if (!tf_grouped_shape_ok(a, MODE == TF_GEMM_FC1_ROUTED)) return -4;
    // a lane's byte offset into the token codes is 32 bits: physical rows x contraction length must stay below 2^32
    if ((unsigned long long)a.max_tiles * TF_GEMM_TILE_M * (unsigned long long)a.k > 0xffffffffull) return -4;
    const int grid = tf_gemm_grid(cus);
    const bool big = routes >= 192ll * a.experts && a.max_tiles / 2 + a.experts <= TF_GROUPED_MAX_UNITS, words = a.act_block == 128;
    if (big) {
        if (words) tf_grouped_gemm<MODE, 256, true><<<grid, 512, 0, s>>>(a);
        else tf_grouped_gemm<MODE, 256, false><<<grid, 512, 0, s>>>(a);
    } else {
        if (words) tf_grouped_gemm<MODE, 128, true><<<grid, 512, 0, s>>>(a);
        else tf_grouped_gemm<MODE, 128, false><<<grid, 512, 0, s>>>(a);
    }
    return (int)hipGetLastError();
}
