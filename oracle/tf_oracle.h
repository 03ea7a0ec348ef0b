/*
 * CPU oracle for the Titanic Flash MoE FFN layer.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a scalar C restatement of the reference's arithmetic for the layer (router top-k, plan /
 * permutation, MXFP8 activation quantizers, MXFP4 routed experts, SwiGLU + FP8 requant, FP8 shared
 * expert, ordered route sum and shared addition, load-time expert layouts and scale codes).  It is the
 * checker the parity tests compare the HIP path against and the "port" CPU baseline the benchmark
 * times.  Nothing in the shipped library links, loads or calls it.
 *
 * Every function cites the reference lines it follows (paths relative to the reference checkout).
 * Where the reference's arithmetic is not source-visible (the routed FC1/FC2 GEMMs and the shared
 * dense GEMMs are third-party binaries there) the header of that function says "parity unpinned":
 * the accumulation order is this oracle's own and results are compared by tolerance only.
 */
#ifndef TF_ORACLE_H
#define TF_ORACLE_H
#include <stdint.h>
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    int32_t hidden;        /* H */
    int32_t experts;       /* E */
    int32_t topk;          /* K */
    int32_t inter;         /* routed expert intermediate I */
    int32_t shared_inter;  /* shared expert intermediate Is */
    int32_t scoring;       /* 0 = sigmoid, 1 = sqrt(softplus) */
    float route_scale;     /* routed_scaling_factor: 1.5 in the reference, 1.0 in the benchmark configs */
    int32_t act_block;     /* activation quantisation block along K: 32 (reference) or 128 */
    int32_t shared_bn;     /* shared-expert weight scale block, rows */
    int32_t shared_bk;     /* shared-expert weight scale block, columns */
    int64_t alt_token;     /* token id that selects bias_alt (129264 in the reference), -1: none */
    float swiglu_limit;    /* 10 */
} orc_config;

void orc_set_threads(int32_t n);

/* ---- number formats ------------------------------------------------------------------------- */
float orc_bf16_to_f32(uint16_t v);
uint16_t orc_f32_to_bf16(float v);
float orc_e4m3_to_f32(uint8_t v);
uint8_t orc_f32_to_e4m3(float v);
float orc_e2m1_to_f32(uint8_t nibble);
uint8_t orc_f32_to_e2m1(float v);
float orc_ue8m0_to_f32(uint8_t v);
float orc_exp(float x);
float orc_log1p_pos(float e);
float orc_logistic(float x);

/* ---- synthetic-weight quantizers (OCP MX) ---------------------------------------------------- */
void orc_quantize_mxfp4(const float* w, int64_t rows, int64_t cols, uint8_t* packed, uint8_t* scales);
void orc_quantize_fp8_blocks(const float* w, int64_t rows, int64_t cols, int32_t bn, int32_t bk,
                             uint8_t* codes, uint8_t* scales);

/* ---- router ------------------------------------------------------------------------------- */
void orc_router_logits(const uint16_t* x, const uint16_t* w, float* logits, int32_t rows, int32_t hidden,
                       int32_t experts);
void orc_route_topk(const orc_config* c, const float* logits, const float* bias, const float* bias_alt,
                    const int64_t* tokens, int32_t live, const int32_t* padding, int32_t* ids, float* weights,
                    int32_t rows);
void orc_route_padding_rows(int32_t* ids, float* weights, const int32_t* source, int32_t rows, int32_t topk);
void orc_route_census(const int32_t* ids, int32_t live, int32_t rows, int32_t topk, int32_t experts,
                      uint32_t* counts);

/* ---- plan / permutation --------------------------------------------------------------------- */
void orc_plan(const int32_t* ids, const float* weights, int32_t rows, int32_t topk, int32_t experts,
              int32_t groups, int32_t tile_m, int32_t* expert_tile_base, int32_t* task_expert,
              int32_t* task_valid_rows, int32_t* token_map, float* token_weights);

/* ---- activation quantizer (MXFP8, power-of-two block scales) -------------------------------- */
void orc_quantize_rows(const uint16_t* x, int32_t rows, int32_t cols, int32_t block, float min_amax,
                       uint8_t* codes, uint8_t* scales);

/* ---- shared expert ------------------------------------------------------------------------- */
void orc_codec_encode(const uint8_t* routed, const uint8_t* routed_scales, const uint8_t* shared, uint8_t* packed,
                      int32_t rows, int32_t k);
void orc_codec_decode(const uint8_t* packed, uint8_t* shared, uint8_t* row_scales, uint8_t* mma_scales, int32_t rows,
                      int32_t k);
void orc_codec_pack_bf16(const uint16_t* input, uint8_t* packed, int32_t rows, int32_t k);
int32_t orc_codec_local_live(int32_t global, int32_t rows, int32_t rank);
void orc_shared_swiglu(const uint16_t* in, uint16_t* act, int32_t rows, int32_t inter, float limit);
void orc_shared_swiglu_quant(const uint16_t* in, uint16_t* act, uint8_t* codes, uint8_t* scales, int32_t rows,
                             int32_t inter, int32_t block, float limit);
void orc_fp8_linear(const uint8_t* aq, const uint8_t* as, int32_t act_block, const uint8_t* wq, const uint8_t* ws,
                    int32_t bn, int32_t bk, int32_t rows, int32_t n, int32_t k, uint16_t* out);

/* ---- routed experts ------------------------------------------------------------------------ */
void orc_expert_fc1(const orc_config* c, const uint8_t* xq, const uint8_t* xs, const uint8_t* w13,
                    const uint8_t* s13, const int32_t* ids, int32_t rows, uint16_t* h, float* proj);
void orc_expert_fc2(const orc_config* c, const uint8_t* hq, const uint8_t* hs, const uint8_t* w2, const uint8_t* s2,
                    const int32_t* ids, const float* weights, int32_t rows, uint16_t* route_out);

/* vectorised (AVX2 + FMA, OpenMP) forms of the three loops above for the CPU baseline: same outputs up to the summation order
 * inside a 32-wide block (tf_oracle_simd.c).  Call only where orc_simd_available() returns non-zero. */
int32_t orc_simd_available(void);
void orc_simd_expert_fc1(const orc_config* c, const uint8_t* xq, const uint8_t* xs, const uint8_t* w13,
                         const uint8_t* s13, const int32_t* ids, int32_t rows, uint16_t* h, float* proj);
void orc_simd_expert_fc2(const orc_config* c, const uint8_t* hq, const uint8_t* hs, const uint8_t* w2, const uint8_t* s2,
                         const int32_t* ids, const float* weights, int32_t rows, uint16_t* route_out);
void orc_simd_fp8_linear(const uint8_t* aq, const uint8_t* as, int32_t act_block, const uint8_t* wq, const uint8_t* ws,
                         int32_t bn, int32_t bk, int32_t rows, int32_t n, int32_t k, uint16_t* out);

/* ---- combine -------------------------------------------------------------------------------- */
void orc_topk_sum(const uint16_t* routes, uint16_t* routed, int32_t rows, int32_t topk, int32_t hidden,
                  int32_t live);
void orc_ffn_add(const uint16_t* a, const uint16_t* b, uint16_t* out, int64_t n);
void orc_ffn_sum_shared(const uint16_t* routes, const uint16_t* shared, uint16_t* routed, uint16_t* out,
                        int32_t rows, int32_t topk, int32_t hidden, int32_t live);
/* the decoder's FFN boundary either side of the layer: RMS norm with a BF16 boundary; BF16 residual addition */
void orc_rmsnorm(const uint16_t* x, const uint16_t* weight, uint16_t* out, int32_t rows, int32_t cols, float eps);
/* the reference's boundary operators: runtime/kernels/mhc-norm-quant-v1/mhc-norm-quant.py, mhc-post-tiles-v1/mhc-post-tiles.py */
void orc_hc_combine_norm_quant(const uint16_t* x, const float* pre, const uint16_t* weight, uint16_t* y, uint8_t* q,
                               uint8_t* sr, uint8_t* sm, int32_t rows, int32_t cols, int32_t streams, int32_t block,
                               float eps);
void orc_hc_post(const uint16_t* a, const uint16_t* residual, const float* post, const float* comb, uint16_t* y,
                 int32_t rows, int32_t cols, int32_t streams);
void orc_residual_add(const uint16_t* a, const uint16_t* b, uint16_t* out, int64_t n);

/* ---- whole layer --------------------------------------------------------------------------- */
typedef struct {
    const uint16_t* x;          /* [rows][H] bf16 */
    const int64_t* tokens;      /* [rows] */
    int32_t rows, live;
    const int32_t* padding;     /* [rows] or NULL */
    const uint16_t* gate_w;     /* [E][H] bf16 */
    const float* bias;          /* [E] */
    const float* bias_alt;      /* [E] */
    const uint8_t* w13;         /* [E][2][I][H/2]  (up rows, then gate rows) */
    const uint8_t* s13;         /* [E][2][I][H/32] */
    const uint8_t* w2;          /* [E][H][I/2] */
    const uint8_t* s2;          /* [E][H][I/32] */
    const uint8_t* sh_w13;      /* [2Is][H] e4m3 (gate rows, then up rows) */
    const uint8_t* sh_s13;      /* [2Is/bn][H/bk] */
    const uint8_t* sh_w2;       /* [H][Is] e4m3 */
    const uint8_t* sh_s2;       /* [H/bn][Is/bk] */
} orc_layer_in;
typedef struct {               /* every tap may be NULL */
    float* logits;              /* [rows][E] */
    int32_t* ids;               /* [rows][K] */
    float* weights;             /* [rows][K] */
    uint8_t* xq_routed; uint8_t* xs_routed;   /* [rows][H], [rows][H/block] */
    uint8_t* xq_shared; uint8_t* xs_shared;
    uint16_t* h;                /* [rows][K][I] bf16 */
    uint8_t* hq; uint8_t* hs;   /* [rows][K][I], [rows][K][I/block] */
    uint16_t* route_out;        /* [rows][K][H] */
    uint16_t* routed;           /* [rows][H] */
    uint16_t* shared_up;        /* [rows][2Is] */
    uint16_t* shared_act;       /* [rows][Is] */
    uint8_t* shared_aq; uint8_t* shared_as;
    uint16_t* shared_down;      /* [rows][H] */
    uint16_t* out;              /* [rows][H] */
} orc_layer_out;
void orc_layer(const orc_config* c, const orc_layer_in* in, const orc_layer_out* out);

/* ---- load-time expert layouts and codes --------------------------------------------------- */
void orc_stream_words(const uint8_t* src, uint8_t* dst, int32_t n, int32_t k, int32_t inverse);
void orc_stream_scales(const uint8_t* src, uint8_t* dst, int32_t n, int32_t k, int32_t inverse);
void orc_stream_fp8(const uint8_t* src, uint8_t* dst, int32_t n, int32_t k, int32_t inverse);
void orc_nibble_permute(uint32_t* words, uint64_t count, int32_t inverse);
void orc_scale_code1_layout(int64_t experts, int64_t hidden, int64_t inter, int64_t out[6]);
void orc_scale_code1(const uint8_t* scales, uint32_t* code, uint32_t* flags, uint32_t* bases, int32_t matrices,
                     int32_t n, int32_t columns);
uint32_t orc_scale_code1_check(const uint8_t* scales, const uint32_t* code, const uint32_t* flags,
                               const uint32_t* bases, int32_t matrices, int32_t n, int32_t columns,
                               uint64_t* raw_rows);
uint32_t orc_scale_codes4(const uint8_t* source, uint8_t* output, int32_t matrices, int32_t n, int32_t columns);
void orc_scale_codes4_decode(const uint8_t* coded, uint8_t* scales, int32_t matrices, int32_t n, int32_t columns);

#ifdef __cplusplus
}
#endif
#endif
