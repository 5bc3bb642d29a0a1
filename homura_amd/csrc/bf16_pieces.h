// f32 values as sums of bf16 pieces, in the operand form of the bf16 MFMA instructions.
#pragma once
#include "hm_common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// x = p[0] + p[1] + ... : each piece is the bf16 rounding (nearest-even, the hardware conversion) of
// what the earlier ones left over; the subtraction is exact. Three pieces reproduce every finite f32
// whose last bit is above the bf16 underflow range. Straight-line code: an infinity or NaN turns the
// later pieces into NaN, like the product with it would be anyway.
template <int NP>
__device__ __forceinline__ void split_pieces(float x, uint32_t (&p)[NP]) {
    float r = x;
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const __bf16 b = (__bf16)r;
        p[i] = (uint32_t)__builtin_bit_cast(uint16_t, b);
        r = r - (float)b;
    }
}

// Two neighbours at once: the packed hardware conversion yields the MFMA operand word (x0 low, x1 high)
template <int NP>
__device__ __forceinline__ void split_pair(float x0, float x1, uint32_t (&w)[NP]) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const f32x2_t r = {x0, x1};
        w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(r, bf16x2_t));
        if (i + 1 < NP) {
            x0 = x0 - __uint_as_float(w[i] << 16);
            x1 = x1 - __uint_as_float(w[i] & 0xFFFF0000u);
        }
    }
}

// 8 floats -> NP MFMA operands
template <int NP>
__device__ __forceinline__ void split8(const float *f, bf16x8 (&out)[NP]) {
    u32x4 w[NP];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint32_t pw[NP];
        split_pair<NP>(f[2 * j], f[2 * j + 1], pw);
#pragma unroll
        for (int p = 0; p < NP; p++) w[p][j] = pw[p];
    }
#pragma unroll
    for (int p = 0; p < NP; p++) out[p] = __builtin_bit_cast(bf16x8, w[p]);
}
