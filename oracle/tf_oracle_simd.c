/*
 * Vectorised build of the CPU oracle's three projection loops.  TEST INFRASTRUCTURE ONLY: the CPU baseline the benchmark
 * reports beside the GPU figure (and a cross-check of the scalar loops); nothing in the shipped library links or calls it.
 *
 * Same arithmetic as orc_expert_fc1 / orc_expert_fc2 / orc_fp8_linear in tf_oracle.c (same operands, same formats, FP32
 * accumulation, the same SwiGLU and BF16 roundings), restated for AVX2 + FMA: a K32 block of weights is decoded to FP32
 * once (E2M1 through a byte shuffle, E4M3 by bit arithmetic), the activation row is decoded and multiplied by its
 * power-of-two block scales once (exact), and a block's 32 products are summed in eight lanes instead of one chain.  The
 * summation order is therefore not the scalar oracle's: results agree to FP32 rounding of the partial sums (the tests
 * hold them to one BF16 step), not bit for bit.  OpenMP over weight rows, as in the scalar loops.
 */
#include "tf_oracle.h"
#include <immintrin.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

#define SIMD __attribute__((target("avx2,fma")))

int32_t orc_simd_available(void) {
    __builtin_cpu_init();
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
}

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
/* orc_ue8m0_to_f32, here so that it inlines into the block loops */
static inline float ue8m0(uint8_t v) { return v == 0 ? u2f(0x00400000u) : v == 255 ? u2f(0x7fc00000u) : u2f((uint32_t)v << 23); }

/* The activation row as FP32 with its block scales applied: a[i] = dq(code) * 2^(e - 127); routed rows: a scale byte 0 marks
 * a zero block (as w4a8_dot).  Power-of-two factors: exact while the result is a normal number. */
static void decode_row(const uint8_t* q, const uint8_t* s, int32_t act_block, int32_t k, int zero_marks_zero_block, float* out) {
    for (int32_t i = 0; i < k; ++i) {
        const uint8_t e = s[i / act_block];
        const float scale = (zero_marks_zero_block && !e) ? 0.f : ue8m0(e);
        out[i] = orc_e4m3_to_f32(q[i]) * scale;
    }
}

SIMD static inline float hsum8(__m256 v) {
    __m128 s = _mm_add_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    s = _mm_add_ps(s, _mm_movehl_ps(s, s));
    s = _mm_add_ss(s, _mm_shuffle_ps(s, s, 1));
    return _mm_cvtss_f32(s);
}

/* sum_k a[k] * dq4(w[k]) * 2^(scale[k / 32] - 127) over one FP4 weight row (low nibble = even k). */
SIMD static float dot_fp4(const float* a, const uint8_t* wrow, const uint8_t* srow, int32_t k) {
    /* twice the E2M1 value as a signed byte: 0 .5 1 1.5 2 3 4 6 -> 0 1 2 3 4 6 8 12 */
    const __m128i table = _mm_setr_epi8(0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12);
    const __m128i low = _mm_set1_epi8(0x0f);
    __m256 total = _mm256_setzero_ps();
    for (int32_t b = 0; b < k / 32; ++b) {
        const __m128i bytes = _mm_loadu_si128((const __m128i*)(wrow + b * 16));
        const __m128i even = _mm_shuffle_epi8(table, _mm_and_si128(bytes, low));
        const __m128i odd = _mm_shuffle_epi8(table, _mm_and_si128(_mm_srli_epi16(bytes, 4), low));
        const __m128i first = _mm_unpacklo_epi8(even, odd), second = _mm_unpackhi_epi8(even, odd);     /* k 0..15, 16..31 */
        const float* x = a + b * 32;
        __m256 sum = _mm256_mul_ps(_mm256_loadu_ps(x), _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(first)));
        sum = _mm256_fmadd_ps(_mm256_loadu_ps(x + 8), _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(_mm_srli_si128(first, 8))), sum);
        sum = _mm256_fmadd_ps(_mm256_loadu_ps(x + 16), _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(second)), sum);
        sum = _mm256_fmadd_ps(_mm256_loadu_ps(x + 24), _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(_mm_srli_si128(second, 8))), sum);
        total = _mm256_fmadd_ps(sum, _mm256_set1_ps(0.5f * ue8m0(srow[b])), total);
    }
    return hsum8(total);
}

/* Eight E4M3 codes -> FP32: normal codes by moving the fields (exponent bias 7 -> 127), subnormal codes as mantissa * 2^-9,
 * 0x7f / 0xff -> NaN. */
SIMD static inline __m256 decode_e4m3x8(const uint8_t* p) {
    const __m256i c = _mm256_cvtepu8_epi32(_mm_loadl_epi64((const __m128i*)p));
    const __m256i mag = _mm256_and_si256(c, _mm256_set1_epi32(0x7f));
    const __m256i normal = _mm256_add_epi32(_mm256_slli_epi32(mag, 20), _mm256_set1_epi32(120 << 23));
    const __m256 sub = _mm256_mul_ps(_mm256_cvtepi32_ps(mag), _mm256_set1_ps(0.001953125f));
    __m256 v = _mm256_blendv_ps(sub, _mm256_castsi256_ps(normal), _mm256_castsi256_ps(_mm256_cmpgt_epi32(mag, _mm256_set1_epi32(7))));
    v = _mm256_blendv_ps(v, _mm256_castsi256_ps(_mm256_set1_epi32(0x7fc00000)), _mm256_castsi256_ps(_mm256_cmpeq_epi32(mag, _mm256_set1_epi32(0x7f))));
    return _mm256_or_ps(v, _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_and_si256(c, _mm256_set1_epi32(0x80)), 24)));
}

/* FC1 + SwiGLU: the same outputs as orc_expert_fc1. */
SIMD void orc_simd_expert_fc1(const orc_config* c, const uint8_t* xq, const uint8_t* xs, const uint8_t* w13, const uint8_t* s13,
                              const int32_t* ids, int32_t rows, uint16_t* h, float* proj) {
    const int32_t H = c->hidden, I = c->inter, K = c->topk;
    float* p = (float*)malloc(sizeof(float) * 2 * (size_t)I);
    float* a = (float*)malloc(sizeof(float) * (size_t)H);
    int32_t decoded = -1;
    for (int32_t t = 0; t < rows * K; ++t) {
        const int32_t e = ids[t], r = t / K;
        if (e < 0 || e >= c->experts) {
            memset(h + (size_t)t * I, 0, sizeof(uint16_t) * (size_t)I);
            if (proj) memset(proj + (size_t)t * 2 * I, 0, sizeof(float) * 2 * (size_t)I);
            continue;
        }
        if (decoded != r) { decode_row(xq + (size_t)r * H, xs + (size_t)r * (H / c->act_block), c->act_block, H, 1, a); decoded = r; }
        const uint8_t* w = w13 + (size_t)e * 2 * I * (H / 2);
        const uint8_t* s = s13 + (size_t)e * 2 * I * (H / 32);
#pragma omp parallel for schedule(static)
        for (int32_t n = 0; n < 2 * I; ++n) p[n] = dot_fp4(a, w + (size_t)n * (H / 2), s + (size_t)n * (H / 32), H);
        for (int32_t i = 0; i < I; ++i) {
            const float g = fminf(p[I + i], c->swiglu_limit);
            const float u = fminf(c->swiglu_limit, fmaxf(-c->swiglu_limit, p[i]));
            h[(size_t)t * I + i] = orc_f32_to_bf16((g * orc_logistic(g)) * u);
        }
        if (proj) memcpy(proj + (size_t)t * 2 * I, p, sizeof(float) * 2 * (size_t)I);
    }
    free(a);
    free(p);
}

/* FC2: the same outputs as orc_expert_fc2. */
SIMD void orc_simd_expert_fc2(const orc_config* c, const uint8_t* hq, const uint8_t* hs, const uint8_t* w2, const uint8_t* s2,
                              const int32_t* ids, const float* weights, int32_t rows, uint16_t* route_out) {
    const int32_t H = c->hidden, I = c->inter, K = c->topk;
    float* a = (float*)malloc(sizeof(float) * (size_t)I);
    for (int32_t t = 0; t < rows * K; ++t) {
        const int32_t e = ids[t];
        if (e < 0 || e >= c->experts) { memset(route_out + (size_t)t * H, 0, sizeof(uint16_t) * (size_t)H); continue; }
        decode_row(hq + (size_t)t * I, hs + (size_t)t * (I / c->act_block), c->act_block, I, 1, a);
        const uint8_t* w = w2 + (size_t)e * H * (I / 2);
        const uint8_t* s = s2 + (size_t)e * H * (I / 32);
#pragma omp parallel for schedule(static)
        for (int32_t col = 0; col < H; ++col)
            route_out[(size_t)t * H + col] = orc_f32_to_bf16(dot_fp4(a, w + (size_t)col * (I / 2), s + (size_t)col * (I / 32), I) * weights[t]);
    }
    free(a);
}

/* Block-scaled FP8 x FP8 dense product: the same outputs as orc_fp8_linear.  A weight row is decoded once and multiplied
 * with every activation row. */
SIMD void orc_simd_fp8_linear(const uint8_t* aq, const uint8_t* as, int32_t act_block, const uint8_t* wq, const uint8_t* ws, int32_t bn,
                              int32_t bk, int32_t rows, int32_t n, int32_t k, uint16_t* out) {
    float* a = (float*)malloc(sizeof(float) * (size_t)rows * k);
    for (int32_t r = 0; r < rows; ++r) decode_row(aq + (size_t)r * k, as + (size_t)r * (k / act_block), act_block, k, 0, a + (size_t)r * k);
#pragma omp parallel
    {
        float* wf = (float*)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(static)
        for (int32_t j = 0; j < n; ++j) {
            const uint8_t* wrow = wq + (size_t)j * k;
            const uint8_t* srow = ws + (size_t)(j / bn) * (k / bk);
            for (int32_t i = 0; i < k; i += 8) _mm256_storeu_ps(wf + i, decode_e4m3x8(wrow + i));
            for (int32_t r = 0; r < rows; ++r) {
                const float* x = a + (size_t)r * k;
                __m256 total = _mm256_setzero_ps();
                for (int32_t b = 0; b < k / 32; ++b) {
                    __m256 sum = _mm256_mul_ps(_mm256_loadu_ps(x + b * 32), _mm256_loadu_ps(wf + b * 32));
                    sum = _mm256_fmadd_ps(_mm256_loadu_ps(x + b * 32 + 8), _mm256_loadu_ps(wf + b * 32 + 8), sum);
                    sum = _mm256_fmadd_ps(_mm256_loadu_ps(x + b * 32 + 16), _mm256_loadu_ps(wf + b * 32 + 16), sum);
                    sum = _mm256_fmadd_ps(_mm256_loadu_ps(x + b * 32 + 24), _mm256_loadu_ps(wf + b * 32 + 24), sum);
                    total = _mm256_fmadd_ps(sum, _mm256_set1_ps(ue8m0(srow[(b * 32) / bk])), total);
                }
                out[(size_t)r * n + j] = orc_f32_to_bf16(hsum8(total));
            }
        }
        free(wf);
    }
    free(a);
}
