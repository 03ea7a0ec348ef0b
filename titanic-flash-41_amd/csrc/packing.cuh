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
// Reversible nibble interleave inside each 32-bit word: [e0..e7] -> [e0,e4,e1,e5,e2,e6,e3,e7].
extern "C" __global__ void ca_moe_nibble_permute_words(uint32_t* words, unsigned long long count, int inverse) {
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < count;
         i += (unsigned long long)gridDim.x * blockDim.x) {
        const uint32_t x = words[i];
        uint32_t y = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int source = (j & 1) * 4 + (j >> 1);
            if (inverse) y |= ((x >> (j * 4)) & 15u) << (source * 4);
            else y |= ((x >> (source * 4)) & 15u) << (j * 4);
        }
        words[i] = y;
    }
}

// One-bit scale code.  Input: prepared scale bytes of one matrix per block, as units of 128 row words of `width` bytes
// ([128-row tile][4-column slice][row][width]).  Output per matrix: base word b * 0x01010101 (b = the commonest byte, or
// the one below it when that is more common than the one above); per unit 16 code words (bit 4 (r % 8) + j of word
// r / 8 = byte j of row r minus b) and 4 flag words (bit r % 32 of word r / 32: row r holds a byte outside {b, b + 1}).
__device__ __forceinline__ int sc1_tiles(int n) { return (n + 127) / 128; }
__device__ __forceinline__ int sc1_slices(int columns) { return (columns + 3) / 4; }
extern "C" __global__ void ca_expert_scale_code1(const uint8_t* scales, uint32_t* code, uint32_t* flags, uint32_t* bases,
                                                 int n, int columns) {
    __shared__ unsigned hist[256];
    __shared__ int chosen;
    const int matrix = blockIdx.x, tiles = sc1_tiles(n), slices = sc1_slices(columns);
    const uint8_t* s = scales + (size_t)matrix * n * columns;
    for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n * columns; i += blockDim.x) atomicAdd(&hist[s[i]], 1u);
    __syncthreads();
    if (threadIdx.x == 0) {
        int c = 0;
        for (int v = 1; v < 256; v++) if (hist[v] > hist[c]) c = v;
        const int b = (c > 0 && (c == 255 || hist[c - 1] > hist[c + 1])) ? c - 1 : c;
        chosen = b;
        bases[matrix] = (uint32_t)b * 0x01010101u;
    }
    __syncthreads();
    const unsigned b = (unsigned)chosen;
    const size_t units = (size_t)tiles * slices;
    uint32_t* c = code + (size_t)matrix * units * 16;
    uint32_t* f = flags + (size_t)matrix * units * 4;
    for (size_t g = threadIdx.x; g < units * 4; g += blockDim.x) {
        const int unit = (int)(g / 4), group = (int)(g % 4), tile = unit / slices, slice = unit % slices;
        const int nr = min(128, n - tile * 128), width = min(4, columns - slice * 4);
        const uint8_t* u = s + (size_t)tile * 128 * columns + (size_t)slice * nr * 4;
        uint32_t words[4] = {0, 0, 0, 0}, flag = 0;
        for (int i = 0; i < 32; i++) {
            const int r = group * 32 + i;
            if (r >= nr) continue;
            unsigned nibble = 0;
            bool raw = false;
            for (int j = 0; j < width; j++) {
                const unsigned v = u[r * width + j];
                if (v == b) continue;
                if (v == b + 1) { nibble |= 1u << j; continue; }
                raw = true;
            }
            if (raw) { flag |= 1u << i; continue; }
            words[i / 8] |= nibble << (4 * (i % 8));
        }
        for (int w = 0; w < 4; w++) c[(size_t)unit * 16 + group * 4 + w] = words[w];
        f[(size_t)unit * 4 + group] = flag;
    }
}
// Decode check: word = flagged ? raw : ((nibble * 0x00204081) & 0x01010101) + base, masked to the width.  Error bit 1: a
// coded row decodes wrong; bit 2: a flagged row is fully on {b, b + 1}.
extern "C" __global__ void ca_expert_scale_code1_check(const uint8_t* scales, const uint32_t* code, const uint32_t* flags,
                                                       const uint32_t* bases, uint32_t* error, int n, int columns) {
    const int matrix = blockIdx.y, tiles = sc1_tiles(n), slices = sc1_slices(columns);
    const size_t units = (size_t)tiles * slices;
    const size_t row_id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (row_id >= units * 128) return;
    const int unit = (int)(row_id / 128), r = (int)(row_id % 128), tile = unit / slices, slice = unit % slices;
    const int nr = min(128, n - tile * 128), width = min(4, columns - slice * 4);
    if (r >= nr) return;
    const uint8_t* u = scales + (size_t)matrix * n * columns + (size_t)tile * 128 * columns + (size_t)slice * nr * 4 + (size_t)r * width;
    uint32_t raw = 0;
    for (int j = 0; j < width; j++) raw |= (uint32_t)u[j] << (8 * j);
    const uint32_t mask = width == 4 ? 0xffffffffu : (1u << (8 * width)) - 1u;
    const uint32_t flag = (flags[((size_t)matrix * units + unit) * 4 + r / 32] >> (r % 32)) & 1u;
    const uint32_t word = code[((size_t)matrix * units + unit) * 16 + r / 8];
    const uint32_t nibble = (word >> (4 * (r % 8))) & 15u;
    const uint32_t decoded = (((nibble * 0x00204081u) & 0x01010101u) + bases[matrix]) & mask;
    if (!flag && decoded != raw) atomicOr(error, 1u);
    if (flag) {
        const uint32_t b = bases[matrix] & 255u;
        bool on = true;
        for (int j = 0; j < width; j++) { const uint32_t v = (raw >> (8 * j)) & 255u; on = on && (v == b || v == b + 1); }
        if (on) atomicOr(error, 2u);
    }
}
extern "C" __global__ void ca_expert_scale_code1_census(const uint32_t* flags, unsigned long long* counts, size_t words) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= words) return;
    const unsigned bits = __popc(flags[i]);
    if (bits) atomicAdd(counts, (unsigned long long)bits);
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

