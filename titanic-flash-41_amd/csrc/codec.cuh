// Row codec of the sequence-parallel prefill transport: the wire row "dual_quant_rows_v1".
//
// One row of k values travels as   [k E4M3 codes of the routed quantizer][k / 32 UE8M0 scale bytes][k / 32 correction words]
// (k * 37 / 32 bytes: 5,920 for k = 5,120).  The routed experts read codes and scales as they are.  The shared expert's
// quantizer differs only in flooring a block's amax at 1e-4, i.e. its scale byte is max(scale, 105); for blocks below
// that floor its codes are the routed codes rescaled by 2^(scale - 105) and rounded again, except where the double
// rounding lands one code off: bit i of a block's correction word marks value i as such, and the decoder steps the code
// one towards the magnitude of the rescaled value.  Both quantizers are reproduced exactly.
//
// Reference: runtime/kernels/moe-input-codec-coalesced-v1/moe-dual-quant-codec-fast.cu (encode :25-46, decode_shared :48-79,
// local_live :96-98, fused_pack :113-137).  The reference runs one 32-lane warp per block of 32 values; here a lane holds
// eight values, four lanes a block, and every lane writes its own byte of the correction word.
#pragma once
#include "frontend.cuh"

__device__ __forceinline__ float tf_e4m3_value(uint32_t code) {
    const uint32_t e = (code >> 3) & 15u, m = code & 7u;
    float r;
    if (e == 15u && m == 7u) r = __uint_as_float(0x7fc00000u);
    else if (e == 0u) r = (float)m * 0.001953125f;                           // m * 2^-9
    else r = __uint_as_float(((e + 120u) << 23) | (m << 20));
    return (code & 0x80u) ? -r : r;
}
// The shared quantizer's code of a value the routed quantizer coded as `code` under scale byte `scale` < 105, before the
// correction; `scaled` receives the rescaled value (moe-dual-quant-codec-fast.cu:17-23).
__device__ __forceinline__ uint32_t tf_codec_base(uint32_t code, uint32_t scale, float& scaled) {
    const uint32_t shared_scale = scale > 105u ? scale : 105u;                // ceil_pow2(1e-4 / 448)
    scaled = __fmul_rn(tf_e4m3_value(code), __uint_as_float((scale - shared_scale + 127u) << 23));
    return tf_to_e4m3(scaled);
}
__device__ __forceinline__ uint32_t tf_codec_row_stride(int k) { return (uint32_t)k + (uint32_t)(k >> 5) * 5u; }

// Correction byte of a lane's eight values: bit i set where the rescaled routed code differs from the shared code.
__device__ __forceinline__ uint32_t tf_codec_correction(uint32_t q_lo, uint32_t q_hi, uint32_t s_lo, uint32_t s_hi, uint32_t scale) {
    uint32_t bits = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t q = ((i < 4 ? q_lo : q_hi) >> (8 * (i & 3))) & 0xffu, want = ((i < 4 ? s_lo : s_hi) >> (8 * (i & 3))) & 0xffu;
        float scaled;
        bits |= (uint32_t)(tf_codec_base(q, scale, scaled) != want) << i;
    }
    return bits;
}
__device__ __forceinline__ void tf_codec_store(uint8_t* packed, long long item, int k, uint32_t q_lo, uint32_t q_hi, uint32_t scale,
                                               uint32_t correction) {
    const int groups = k >> 5, per_row = k >> 3;
    const long long row = item / per_row;
    const int piece = (int)(item - row * per_row), col = piece >> 2, part = piece & 3;
    uint8_t* out = packed + row * tf_codec_row_stride(k);
    reinterpret_cast<uint32_t*>(out + col * 32 + part * 8)[0] = q_lo;         // rows are 4-byte aligned (k % 128 == 0)
    reinterpret_cast<uint32_t*>(out + col * 32 + part * 8)[1] = q_hi;
    if (part == 0) out[k + col] = (uint8_t)scale;
    out[k + groups + col * 4 + part] = (uint8_t)correction;
}

// routed [rows][k] codes, routed_scales [rows][k / 32], shared [rows][k] codes -> packed rows.
extern "C" __global__ void __launch_bounds__(256) ca_codec_encode(const uint8_t* __restrict__ routed, const uint8_t* __restrict__ routed_scales,
                                                                  const uint8_t* __restrict__ shared, uint8_t* __restrict__ packed,
                                                                  long long rows, int32_t k) {
    const long long items = rows * (k >> 3);
    for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < items; q += (long long)gridDim.x * blockDim.x) {
        const u2v code = reinterpret_cast<const u2v*>(routed)[q];
        const uint32_t scale = routed_scales[q >> 2];
        uint32_t correction = 0;
        if (scale < 105u) {
            const u2v want = reinterpret_cast<const u2v*>(shared)[q];
            correction = tf_codec_correction(code[0], code[1], want[0], want[1], scale);
        }
        tf_codec_store(packed, q, k, code[0], code[1], scale, correction);
    }
}

// packed rows -> the shared quantizer's codes [rows][k] and scale bytes: row-major [rows][k / 32] and, when `mma_scales` is
// given, also at the reference's matrix-instruction offsets (:69-75; rows % 128 == 0), which a caller that feeds the
// reference's dense kernels expects.
extern "C" __global__ void __launch_bounds__(256) ca_codec_decode(const uint8_t* __restrict__ packed, uint8_t* __restrict__ shared,
                                                                  uint8_t* __restrict__ row_scales, uint8_t* __restrict__ mma_scales,
                                                                  long long rows, int32_t k) {
    const int groups = k >> 5, per_row = k >> 3;
    const long long items = rows * per_row;
    for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < items; q += (long long)gridDim.x * blockDim.x) {
        const long long row = q / per_row;
        const int piece = (int)(q - row * per_row), col = piece >> 2, part = piece & 3;
        const uint8_t* in = packed + row * tf_codec_row_stride(k);
        uint32_t lo = reinterpret_cast<const uint32_t*>(in + col * 32 + part * 8)[0];
        uint32_t hi = reinterpret_cast<const uint32_t*>(in + col * 32 + part * 8)[1];
        const uint32_t scale = in[k + col];
        if (scale < 105u) {
            const uint32_t correction = in[k + groups + col * 4 + part];
            uint32_t out_lo = 0, out_hi = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t code = ((i < 4 ? lo : hi) >> (8 * (i & 3))) & 0xffu;
                float scaled;
                uint32_t base = tf_codec_base(code, scale, scaled);
                if ((correction >> i) & 1u) base = (base + (fabsf(scaled) > fabsf(tf_e4m3_value(base)) ? 1u : 0xffu)) & 0xffu;
                if (i < 4) out_lo |= base << (8 * i); else out_hi |= base << (8 * (i - 4));
            }
            lo = out_lo; hi = out_hi;
        }
        reinterpret_cast<u2v*>(shared)[q] = u2v{lo, hi};
        if (part == 0) {
            const uint8_t shared_scale = (uint8_t)(scale > 105u ? scale : 105u);
            row_scales[row * groups + col] = shared_scale;
            if (mma_scales != nullptr) {
                const long long offset = (row % 32) * 16 + ((row / 32) % 4) * 4 + (row / 128) * (long long)(((groups + 3) / 4) * 512) +
                                         (col % 4) + (long long)(col / 4) * 512;
                mma_scales[offset] = shared_scale;
            }
        }
    }
}

// BF16 rows [rows][k] -> packed rows: both quantizers (32-wide blocks) and the encoder in one pass.
extern "C" __global__ void __launch_bounds__(256) ca_codec_pack_bf16(const uint16_t* __restrict__ input, uint8_t* __restrict__ packed,
                                                                     long long rows, int32_t k) {
    const long long items = rows * (k >> 3), padded = (items + 63) & ~63ll;       // whole blocks (four lanes) stay in one wave
    for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < padded; q += (long long)gridDim.x * blockDim.x) {
        const bool on = q < items;
        float v[8];
        if (on) {
            const u4v w = reinterpret_cast<const u4v*>(input)[q];
#pragma unroll
            for (int i = 0; i < 4; ++i) { v[2 * i] = tf_bf16_lo(w[i]); v[2 * i + 1] = tf_bf16_hi(w[i]); }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = 0.f;
        }
        const float amax = tf_group_amax(v, 4);
        if (!on) continue;
        const Quant8 routed = tf_quant8(v, amax, 0.f);
        uint32_t correction = 0;
        if (routed.exponent < 105u) {
            const Quant8 shared = tf_quant8(v, amax, 1e-4f);
            correction = tf_codec_correction(routed.lo, routed.hi, shared.lo, shared.hi, routed.exponent);
        }
        tf_codec_store(packed, q, k, routed.lo, routed.hi, routed.exponent, correction);
    }
}

// packed rows -> the routed experts' operands as the expert kernels read them: codes [rows][k], scales [rows][k / 32].
extern "C" __global__ void __launch_bounds__(256) ca_codec_unpack_routed(const uint8_t* __restrict__ packed, uint8_t* __restrict__ codes,
                                                                         uint8_t* __restrict__ scales, long long rows, int32_t k) {
    const int per_row = k >> 3;
    const long long items = rows * per_row;
    for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < items; q += (long long)gridDim.x * blockDim.x) {
        const long long row = q / per_row;
        const int piece = (int)(q - row * per_row), col = piece >> 2, part = piece & 3;
        const uint8_t* in = packed + row * tf_codec_row_stride(k);
        const uint32_t lo = reinterpret_cast<const uint32_t*>(in + col * 32 + part * 8)[0];
        const uint32_t hi = reinterpret_cast<const uint32_t*>(in + col * 32 + part * 8)[1];
        reinterpret_cast<u2v*>(codes)[q] = u2v{lo, hi};
        if (part == 0) scales[row * (k >> 5) + col] = in[k + col];
    }
}

// A rank's live rows of a row-sharded batch: min(rows, max(0, global - rank * rows)) (:96-98).
extern "C" __global__ void ca_codec_local_live(const int32_t* global, int32_t* local, int32_t rows, int32_t rank) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *local = min(rows, max(0, *global - rank * rows));
}
