// Device helpers of the K8 form of Q4_K / Q6_K matrices (kquant_planes8.h): a lane holds one 16-weight sub-block
// - its 16 signed bytes, its scale and minimum factor, and the f16 d | dmin of its 256-wide super-block, which
// is exactly one DPP row of 16 lanes. The activations go through the reference's Q8_K quantisation
// (src/graph_builder/emit_quant.rs:422-466: amax over the block, d = amax / 127, q = roundeven(x * 127 / amax)
// clamped to +-127), the products are integer dot products, and a block contributes
// (d * act_d) * float(sum sc * isum) - (dmin * act_d) * float(sum mn * bsum) with both sums exact in i32
// (emit_quant.rs:165-816). Internal; shared by the whole-step decode kernel and the per-projection GEMV.
#pragma once

#include "hm_common.h"

__device__ __forceinline__ int dpp_row_isum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, false);
    v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, false);
    return v;
}
__device__ __forceinline__ float dpp_row_fmax(float v) {
    v = fmaxf(v, dpp_move<0xB1, 0xF>(v, 0.f));
    v = fmaxf(v, dpp_move<0x4E, 0xF>(v, 0.f));
    v = fmaxf(v, dpp_move<0x141, 0xF>(v, 0.f));
    v = fmaxf(v, dpp_move<0x140, 0xF>(v, 0.f));
    return v;
}

// The Q8_K form of a lane's 16 activations of a block whose largest magnitude is amax: four words of four
// bytes, their sum, and the block's act_d.
struct Q8kLane {
    uint32_t q[4];
    int bsum;
    float act_d;
};
__device__ __forceinline__ Q8kLane q8k_lane(const float (&x)[16], float amax) {
    Q8kLane r;
    r.act_d = amax / 127.0f;
    const float iscale = amax == 0.0f ? 0.0f : 127.0f / amax;
    r.bsum = 0;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        int qi[4];
#pragma unroll
        for (int e = 0; e < 4; e++)  // round half to even, clamp to +-127 (one median instruction)
            qi[e] = (int)__builtin_amdgcn_fmed3f(rintf(__fmul_rn(x[4 * w + e], iscale)), -127.0f, 127.0f);
        // the low bytes of the four integers side by side
        const uint32_t lo = __builtin_amdgcn_perm((uint32_t)qi[1], (uint32_t)qi[0], 0x0c0c0400u);
        const uint32_t hi = __builtin_amdgcn_perm((uint32_t)qi[3], (uint32_t)qi[2], 0x0c0c0400u);
        r.q[w] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        r.bsum = __builtin_amdgcn_sdot4((int)r.q[w], 0x01010101, r.bsum, false);
    }
    return r;
}
__device__ __forceinline__ float abs_max16(const float (&x)[16]) {
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < 16; j++) m = fmaxf(m, fabsf(x[j]));
    return m;
}
// One block's share of a row from the lane's sub-block: every lane of the block's DPP row gets it.
__device__ __forceinline__ float k8_block(const u32x4 w, uint32_t sub, uint32_t dd, const Q8kLane &a) {
    int isum = __builtin_amdgcn_sdot4((int)w.x, (int)a.q[0], 0, false);
    isum = __builtin_amdgcn_sdot4((int)w.y, (int)a.q[1], isum, false);
    isum = __builtin_amdgcn_sdot4((int)w.z, (int)a.q[2], isum, false);
    isum = __builtin_amdgcn_sdot4((int)w.w, (int)a.q[3], isum, false);
    const int sc = (int)(int8_t)(sub & 0xFFu), mn = (int)((sub >> 8) & 0xFFu);
    const int s_tot = dpp_row_isum(sc * isum), m_tot = dpp_row_isum(mn * a.bsum);
    const float d = f16_bits_to_f32((uint16_t)(dd & 0xFFFFu)), dmin = f16_bits_to_f32((uint16_t)(dd >> 16));
    const float scale_part = __fmul_rn(__fmul_rn(d, a.act_d), (float)s_tot);
    const float min_part = __fmul_rn(__fmul_rn(dmin, a.act_d), (float)m_tot);
    return __fsub_rn(scale_part, min_part);
}

