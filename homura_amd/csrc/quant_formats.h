// One weight of a GGUF block, dequantised with the reference's arithmetic step by step (one rounding
// per f32 operation, no contraction), so the bits equal what its CPU code produces.
// Block layouts: Q8_0 34 B = f16 d | 32 int8; Q4_0 18 B = f16 d | 16 bytes of two nibbles (element j
// and j + 16); Q4_K 144 B = f16 d | f16 dmin | 12 bytes of 6-bit scales and mins | 128 bytes of
// nibbles; Q6_K 210 B = 128 bytes low nibbles | 64 bytes of 2-bit highs | 16 int8 scales | f16 d.
#pragma once

#include <cstdint>

#include "hm_common.h"

namespace homura {

enum QuantFormat : int { QF_Q8_0 = 0, QF_Q4_0 = 1, QF_Q4_K = 2, QF_Q6_K = 3 };

template <int QF>
struct QuantFormatTraits;
template <>
struct QuantFormatTraits<QF_Q8_0> {
    static constexpr int BYTES = 34, ELEMS = 32;
};
template <>
struct QuantFormatTraits<QF_Q4_0> {
    static constexpr int BYTES = 18, ELEMS = 32;
};
template <>
struct QuantFormatTraits<QF_Q4_K> {
    static constexpr int BYTES = 144, ELEMS = 256;
};
template <>
struct QuantFormatTraits<QF_Q6_K> {
    static constexpr int BYTES = 210, ELEMS = 256;
};

__device__ __forceinline__ float f16_at(const uint8_t *p) { return f16_bits_to_f32((uint16_t)(p[0] | (p[1] << 8))); }

// element j of the block at blk
template <int QF>
__device__ __forceinline__ float dequant_element(const uint8_t *__restrict__ blk, int j) {
    if (QF == QF_Q8_0) {  // reference src/gguf.rs:825-829
        return __fmul_rn((float)(int8_t)blk[2 + j], f16_at(blk));
    } else if (QF == QF_Q4_0) {
        const uint8_t byte = blk[2 + (j & 15)];
        return __fmul_rn((float)((j < 16 ? (byte & 0x0F) : (byte >> 4)) - 8), f16_at(blk));
    } else if (QF == QF_Q4_K) {  // w = q * (d * sc) - dmin * mn (src/gguf.rs:835-875)
        const float d = f16_at(blk), dmin = f16_at(blk + 2);
        const uint8_t *raw = blk + 4;
        const int sb = j >> 5, l = j & 31;
        int sc, mn;
        if (sb < 4) {
            sc = raw[sb] & 63;
            mn = raw[sb + 4] & 63;
        } else {
            sc = (raw[sb + 4] & 15) | ((raw[sb - 4] >> 6) << 4);
            mn = (raw[sb + 4] >> 4) | ((raw[sb] >> 6) << 4);
        }
        const uint8_t byte = blk[16 + (sb >> 1) * 32 + l];
        const int q = (sb & 1) ? (byte >> 4) : (byte & 15);
        return __fsub_rn(__fmul_rn((float)q, __fmul_rn(d, (float)sc)), __fmul_rn(dmin, (float)mn));
    } else {  // Q6_K: w = (d * sc) * q (src/gguf.rs:880-917)
        const float d = f16_at(blk + 208);
        const int h = j >> 7, g = (j & 127) >> 5, l = j & 31;
        const uint8_t lb = blk[64 * h + 32 * (g & 1) + l];
        const int lo = g >= 2 ? (lb >> 4) : (lb & 15);
        const int hi = (blk[128 + 32 * h + l] >> (2 * g)) & 3;
        const int q = (int)(int8_t)(lo | (hi << 4)) - 32;
        const int sc = (int)(int8_t)blk[192 + 8 * h + 2 * g + (l >> 4)];
        return __fmul_rn(__fmul_rn(d, (float)sc), (float)q);
    }
}

// Four consecutive values of a 256-wide block held by one wavefront (four per lane) through the Q8_K
// quantiser (reference quantize_row_q8_k, src/graph_builder/emit_quant.rs:422-466): q = clamp(roundeven(x *
// (127 / amax)), +-127), scale d = amax / 127. Returns the four int8 values packed low to high.
__device__ __forceinline__ uint32_t q8k_quantize4(f32x4 v, float &d, float r_out[4]) {
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    amax = wave_max(amax);
    const float iscale = amax == 0.f ? 0.f : __fdiv_rn(127.0f, amax);
    d = __fdiv_rn(amax, 127.0f);
    uint32_t packed = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float r = rintf(__fmul_rn(v[k], iscale));
        r = fmaxf(fminf(r, 127.0f), -127.0f);
        r_out[k] = r;
        packed |= ((uint32_t)(int)r & 0xFFu) << (8 * k);
    }
    return packed;
}
__device__ __forceinline__ uint32_t q8k_quantize4(f32x4 v, float &d) {
    float r[4];
    return q8k_quantize4(v, d, r);
}

}  // namespace homura
