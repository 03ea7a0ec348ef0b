// Load-time expert preparation: byte permutations into the gfx950 streaming layouts, scale codes, nibble permutation.
// Reference semantics: src/expert_packing.rs:137-259 (what runs when), kernels/core.cu:802-818 (its NVIDIA layouts, whose
// role these take), kernels/expert_scale_codes.cuh, kernels/moe_nibble_layout_probe.cu.
#pragma once
#include "common.cuh"

// FP4 words [n][k/2 bytes] -> [n/16][k/128][lane 64][16 B]: lane 16 g + r of tile (nt, ks) holds row 16 nt + r, K32 block
// 4 ks + g.  One thread per 16-byte chunk.  `group` is accepted for call compatibility and must equal n.
extern "C" __global__ void ca_expert_compact_words(const u4v* source, u4v* out, int n, int k, int group) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x, chunks = k / 32;
    if (i >= n * chunks) return;
    const int r = i / chunks, ch = i % chunks;
    out[((size_t)(r / 16) * (k / 128) + ch / 4) * 64 + (ch % 4) * 16 + r % 16] = source[i];
    (void)group;
}
extern "C" __global__ void ca_expert_expand_words(const u4v* source, u4v* out, int n, int k) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x, chunks = k / 32;
    if (i >= n * chunks) return;
    const int r = i / chunks, ch = i % chunks;
    out[i] = source[((size_t)(r / 16) * (k / 128) + ch / 4) * 64 + (ch % 4) * 16 + r % 16];
}
// UE8M0 [n][k/32] -> [n/16][k/512][lane 64][4 B]: byte q of lane 16 g + r = scale of row 16 nt + r, K32 block 4 (4 kq + q) + g.
extern "C" __global__ void ca_expert_compact_scales(const uint8_t* source, uint8_t* out, int n, int k, int group) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x, columns = k / 32;
    if (i >= n * columns) return;
    const int r = i / columns, b = i % columns, ks = b / 4, g = b % 4;
    out[(((size_t)(r / 16) * (k / 512) + ks / 4) * 64 + g * 16 + r % 16) * 4 + ks % 4] = source[i];
    (void)group;
}
extern "C" __global__ void ca_expert_expand_scales(const uint8_t* source, uint8_t* out, int n, int k) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x, columns = k / 32;
    if (i >= n * columns) return;
    const int r = i / columns, b = i % columns, ks = b / 4, g = b % 4;
    out[i] = source[(((size_t)(r / 16) * (k / 512) + ks / 4) * 64 + g * 16 + r % 16) * 4 + ks % 4];
}
// E4M3 bytes [n][k] -> [n/16][k/128][half 2][lane 64][16 B] (shared-expert weights).
extern "C" __global__ void ca_dense_compact_fp8(const u4v* source, u4v* out, int n, int k, int inverse) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x, chunks = k / 16;
    if (i >= n * chunks) return;
    const int r = i / chunks, ch = i % chunks, ks = ch / 8, half = (ch % 8) / 4, g = ch % 4;
    const size_t at = (((size_t)(r / 16) * (k / 128) + ks) * 2 + half) * 64 + g * 16 + r % 16;
    if (inverse) out[i] = source[at]; else out[at] = source[i];
}
// Reversible nibble interleave inside each 32-bit word: [e0..e7] -> [e0,e4,e1,e5,e2,e6,e3,e7] (the format of
// kernels/moe_nibble_layout_probe.cu:9-12).  Forward: the low half's four nibbles spread to the even nibble positions, the
// high half's to the odd ones (two shift-and-mask steps a half); inverse: the even and the odd nibbles squeezed back.
__device__ __forceinline__ uint32_t tf_spread_nibbles(uint32_t h) {          // 0x0000dcba -> 0x0d0c0b0a
    h = (h | (h << 8)) & 0x00ff00ffu;
    return (h | (h << 4)) & 0x0f0f0f0fu;
}
__device__ __forceinline__ uint32_t tf_squeeze_nibbles(uint32_t v) {         // 0x0d0c0b0a -> 0x0000dcba
    v = (v | (v >> 4)) & 0x00ff00ffu;
    return (v | (v >> 8)) & 0x0000ffffu;
}
extern "C" __global__ void ca_moe_nibble_permute_words(uint32_t* words, unsigned long long count, int inverse) {
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < count;
         i += (unsigned long long)gridDim.x * blockDim.x) {
        const uint32_t x = words[i];
        words[i] = inverse ? tf_squeeze_nibbles(x & 0x0f0f0f0fu) | (tf_squeeze_nibbles((x >> 4) & 0x0f0f0f0fu) << 16)
                           : tf_spread_nibbles(x & 0xffffu) | (tf_spread_nibbles(x >> 16) << 4);
    }
}

// One-bit scale code (format: kernels/expert_scale_codes.cuh:29-36, word offsets src/config.rs:1365-1375).  Input: the
// scale bytes of one matrix per workgroup, as units of 128 row words of `width` bytes ([128-row tile][4-column slice][row]
// [width]).  Output per matrix: the base word b * 0x01010101 (b = the commonest byte, or the byte below it when that one is
// more common than the byte above); per unit 16 code words (bit 4 (r % 8) + j of word r / 8: byte j of row r is b + 1) and
// 4 flag words (bit r % 32 of word r / 32: row r holds a byte outside {b, b + 1} and stays raw).
// One workgroup of (up to) four waves a matrix.  The byte counts are taken a wave of bytes at a time by matching: the lanes that
// hold the same byte as the first lane still open are counted with one ballot and closed together (scale bytes take a
// handful of values, so a wave's 64 bytes close in two or three rounds); the 256 counts are then ranked by all threads
// at once (largest count, lowest byte on a tie, as one packed key).  A wave then codes a unit at a time, 64 rows a pass: a
// row's four bits meet the seven other rows of its code word through three lane exchanges, and a pass's raw rows are one
// ballot, which is the flag word pair.
__device__ __forceinline__ uint32_t tf_unit_row_word(const uint8_t* unit, int row, int width) {
    uint32_t w = 0;
    for (int j = 0; j < width; ++j) w |= (uint32_t)unit[row * width + j] << (8 * j);
    return w;
}
// bit j: byte j of `word` equals `above` (= b + 1); `raw`: some byte of the row's `width` is neither b nor b + 1
__device__ __forceinline__ uint32_t tf_row_bits(uint32_t word, int width, uint32_t b, bool& raw) {
    uint32_t bits = 0;
    raw = false;
    for (int j = 0; j < width; ++j) {
        const uint32_t v = (word >> (8 * j)) & 255u;
        bits |= (uint32_t)(v == b + 1) << j;
        raw = raw || (v != b && v != b + 1);
    }
    return bits;
}
extern "C" __global__ void __launch_bounds__(256) ca_expert_scale_code1(const uint8_t* scales, uint32_t* code, uint32_t* flags, uint32_t* bases,
                                                                        int n, int columns) {
    __shared__ uint32_t s_count[4][256];          // a table a wave
    __shared__ unsigned long long s_best[4];
    __shared__ uint32_t s_total[256];
    // any block of one to four whole waves (the reference launches 256 threads)
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, threads = (int)blockDim.x, waves = threads >> 6;
    const int matrix = blockIdx.x, tiles = (n + 127) / 128, slices = (columns + 3) / 4;
    const uint8_t* bytes = scales + (size_t)matrix * n * columns;
    const int total = n * columns;
    for (int i = lane; i < 256; i += 64) s_count[wave][i] = 0;
    __builtin_amdgcn_wave_barrier();
    for (int first = wave * 64; first < total; first += waves * 64) {
        const int at = first + lane;
        const int value = at < total ? bytes[at] : -1;
        unsigned long long open = __ballot(value >= 0);
        while (open) {
            const int leader = __ffsll((long long)open) - 1;
            const int which = __shfl(value, leader);
            const unsigned long long same = __ballot(value == which);
            if (lane == leader) s_count[wave][which] += (uint32_t)__popcll(same);
            open &= ~same;
        }
    }
    __syncthreads();
    // a thread ranks bytes t, t + threads, ..: key = count << 8 | (255 - byte) in 64 bits (a matrix may hold 2^24 scale bytes and
    // more), so the largest key is the largest count and, on a tie, the lowest byte
    unsigned long long key = 0;
    for (int v = t; v < 256; v += threads) {
        uint32_t mine = 0;
        for (int w = 0; w < waves; ++w) mine += s_count[w][v];
        s_total[v] = mine;
        const unsigned long long candidate = ((unsigned long long)mine << 8) | (unsigned long long)(255 - v);
        key = candidate > key ? candidate : key;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = ((unsigned long long)(uint32_t)__shfl_xor((int)(key >> 32), o) << 32) | (uint32_t)__shfl_xor((int)(uint32_t)key, o);
        key = other > key ? other : key;
    }
    if (lane == 0) s_best[wave] = key;
    __syncthreads();
    for (int w = 0; w < waves; ++w) key = s_best[w] > key ? s_best[w] : key;
    const int commonest = 255 - (int)(key & 255u);
    const bool below = commonest > 0 && (commonest == 255 || s_total[commonest - 1] > s_total[commonest + 1]);
    const uint32_t b = (uint32_t)(below ? commonest - 1 : commonest);
    if (t == 0) bases[matrix] = b * 0x01010101u;
    const int units = tiles * slices;
    uint32_t* unit_code = code + (size_t)matrix * units * 16;
    uint32_t* unit_flags = flags + (size_t)matrix * units * 4;
    for (int unit = wave; unit < units; unit += waves) {
        const int tile = unit / slices, slice = unit - tile * slices;
        const int rows = min(128, n - tile * 128), width = min(4, columns - slice * 4);
        const uint8_t* u = bytes + (size_t)tile * 128 * columns + (size_t)slice * rows * 4;
        for (int pass = 0; pass < 2; ++pass) {
            const int r = pass * 64 + lane;
            bool raw = false;
            uint32_t bits = 0;
            if (r < rows) bits = tf_row_bits(tf_unit_row_word(u, r, width), width, b, raw);
            const unsigned long long raw_rows = __ballot(raw);
            uint32_t word = raw ? 0u : bits << (4 * (lane & 7));
            word |= (uint32_t)__shfl_xor((int)word, 1);
            word |= (uint32_t)__shfl_xor((int)word, 2);
            word |= (uint32_t)__shfl_xor((int)word, 4);
            if ((lane & 7) == 0) unit_code[(size_t)unit * 16 + pass * 8 + (lane >> 3)] = word;
            if (lane < 2) unit_flags[(size_t)unit * 4 + pass * 2 + lane] = (uint32_t)(raw_rows >> (32 * lane));
        }
    }
}
// The decode the kernels apply, checked against every row word: word = raw row ? the row's bytes : ((four bits * 0x00204081)
// & 0x01010101) + base, masked to the width.  Error bit 1: a coded row decodes wrong; bit 2: a raw row lies wholly on
// {b, b + 1} (the coder never leaves such a row raw).  A wave checks 64 rows of a unit (grid.x * blockDim.x >= units * 128,
// grid.y = matrices) and reports once, from its ballots.
extern "C" __global__ void __launch_bounds__(256) ca_expert_scale_code1_check(const uint8_t* scales, const uint32_t* code, const uint32_t* flags,
                                                                              const uint32_t* bases, uint32_t* error, int n, int columns) {
    const int lane = threadIdx.x & 63, matrix = blockIdx.y, tiles = (n + 127) / 128, slices = (columns + 3) / 4;
    const size_t units = (size_t)tiles * slices;
    const size_t half_unit = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;          // 64 rows
    if (half_unit >= units * 2) return;
    const int unit = (int)(half_unit >> 1), r = (int)(half_unit & 1) * 64 + lane, tile = unit / slices, slice = unit - tile * slices;
    const int rows = min(128, n - tile * 128), width = min(4, columns - slice * 4);
    const uint32_t base = bases[matrix], b = base & 255u;
    bool wrong = false, idle_raw = false;
    if (r < rows) {
        const uint8_t* u = scales + (size_t)matrix * n * columns + (size_t)tile * 128 * columns + (size_t)slice * rows * 4;
        const uint32_t held = tf_unit_row_word(u, r, width);
        const uint32_t mask = width == 4 ? 0xffffffffu : (1u << (8 * width)) - 1u;
        const size_t at = (size_t)matrix * units + unit;
        const bool is_raw = (flags[at * 4 + (r >> 5)] >> (r & 31)) & 1u;
        const uint32_t four = (code[at * 16 + (r >> 3)] >> (4 * (r & 7))) & 15u;
        bool off_pair;
        (void)tf_row_bits(held, width, b, off_pair);
        wrong = !is_raw && ((((four * 0x00204081u) & 0x01010101u) + base) & mask) != held;
        idle_raw = is_raw && !off_pair;
    }
    const uint32_t found = (__ballot(wrong) ? 1u : 0u) | (__ballot(idle_raw) ? 2u : 0u);
    if (found && lane == 0) atomicOr(error, found);
}
// Raw rows of a coded layer (set flag bits), for the load report: a wave adds its words' bit counts and reports once.
extern "C" __global__ void __launch_bounds__(256) ca_expert_scale_code1_census(const uint32_t* flags, unsigned long long* counts, size_t words) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    int bits = i < words ? __popc(flags[i]) : 0;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) bits += __shfl_xor(bits, o);
    if (bits && (threadIdx.x & 63) == 0) atomicAdd(counts, (unsigned long long)bits);
}
// Four-bit row deltas of row-major scale matrices [n][columns]: header byte 4, per-row base at 16 + row, then nibble pairs
// (a - lo) | (b - lo) << 4, rows of a 128-row tile interleaved two bytes at a time.  Fails closed (error bit 1) when a
// byte exceeds 247 or a row spans more than 15; bit 2: a pair did not decode back.  grid (ceil(n / 4), matrices), block 256.
extern "C" __global__ void ca_expert_scale_codes4(const uint8_t* source, uint8_t* output, uint32_t* error, int matrices,
                                                  int n, int columns) {
    const int matrix = blockIdx.y, row = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x % 64;
    if (matrix >= matrices || row >= n) return;
    const size_t stride = (size_t)n * columns;
    const uint8_t* s = source + matrix * stride + (size_t)row * columns;
    int lo = 255, hi = 0;
    for (int k = lane; k < columns; k += 64) { const int x = s[k]; lo = min(lo, x); hi = max(hi, x); }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { lo = min(lo, __shfl_xor(lo, o)); hi = max(hi, __shfl_xor(hi, o)); }
    if (hi > 247 || hi - lo > 15) { if (lane == 0) atomicOr(error, 1u); return; }
    uint8_t* out = output + matrix * stride;
    const int tile = row / 128, nr = min(128, n - tile * 128), r = row % 128;
    if (lane == 0) { out[16 + row] = (uint8_t)lo; if (row == 0) out[0] = 4; }
    for (int pair = lane; pair < columns / 2; pair += 64) {
        const int a = s[pair * 2], b = s[pair * 2 + 1];
        const uint8_t packed = (uint8_t)((a - lo) | ((b - lo) << 4));
        if (lo + (packed & 15) != a || lo + (packed >> 4) != b) atomicOr(error, 2u);
        out[16 + n + (size_t)tile * 128 * (columns / 2) + (size_t)(pair / 2) * nr * 2 + r * 2 + pair % 2] = packed;
    }
}

// The number-format conversions alone (parity tests): E4M3 code and BF16 bits of every input.
extern "C" __global__ void __launch_bounds__(256) ca_convert_formats(const float* __restrict__ in, uint8_t* __restrict__ e4m3,
                                                                     uint16_t* __restrict__ bf16, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const float v = in[i];
        e4m3[i] = (uint8_t)tf_to_e4m3(v);
        bf16[i] = tf_to_bf16(v);
        if ((i & 3) == 0 && i + 3 < n) {          // the four-value packer too: it must agree with the single conversions
            const uint32_t w = tf_pack_e4m3(v, in[i + 1], in[i + 2], in[i + 3]);
            if ((w & 0xffu) != tf_to_e4m3(v) || ((w >> 8) & 0xffu) != tf_to_e4m3(in[i + 1]) || ((w >> 16) & 0xffu) != tf_to_e4m3(in[i + 2]) ||
                (w >> 24) != tf_to_e4m3(in[i + 3]))
                bf16[i] = 0xdead;                 // no BF16 value of a test input: the test fails on it
        }
    }
}

