// Internal definitions shared by the HIP sources of libhomura_amd.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>

#include "../../include/homura_amd.h"

struct hm_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    int num_cus = 256;
    // Workspace for kernels that need partial results (split-K / split-KV); allocated once.
    void *workspace = nullptr;
    size_t workspace_bytes = 0;
    // 4-byte counters used by "last workgroup finishes" reductions; always left at zero.
    unsigned int *counters = nullptr;
    size_t num_counters = 0;
    // Device address, on this context's device, of the fixed array behind hm_gqa_decode_attn_noalloc.
    void *attn_fixed_scratch = nullptr;
    std::string last_error;
    char device_name[128] = {0};
};

int hm_set_error(hm_ctx *ctx, int code, const char *fmt, ...);

#define HM_CHECK_CTX(ctx)                 \
    do {                                  \
        if (!(ctx)) return HM_ERR_INVALID; \
    } while (0)

#define HM_HIP(ctx, expr)                                                                    \
    do {                                                                                     \
        hipError_t _e = (expr);                                                              \
        if (_e != hipSuccess)                                                                \
            return hm_set_error((ctx), HM_ERR_HIP, "%s failed: %s (%s:%d)", #expr,           \
                                hipGetErrorString(_e), __FILE__, __LINE__);                  \
    } while (0)

#define HM_REQUIRE(ctx, cond, ...)                                   \
    do {                                                             \
        if (!(cond)) return hm_set_error((ctx), HM_ERR_INVALID, __VA_ARGS__); \
    } while (0)

// Checked after every launch: an invalid launch configuration surfaces here, not later.
#define HM_LAUNCH_CHECK(ctx) HM_HIP((ctx), hipGetLastError())

constexpr int WAVE = 64;

// Device-resident cursor of a decode loop. Kernels of the decode plan read the position from
// here instead of from launch arguments, so one captured HIP graph serves every token.
struct DecodeState {
    int pos;       // rows already in the KV cache = position of the token being processed
    int token;     // last greedy pick (input of the next step once the forced ids run out)
    int step;      // steps taken since the state was armed
    int n_forced;  // steps [0, n_forced) take their input id from the forced list
};

// ── device helpers ───────────────────────────────────────────────────────────

__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) {
    return __uint_as_float(packed & 0xFFFF0000u);
}

// Round-to-nearest-even f32 -> bf16 (NaN kept quiet).
__device__ __forceinline__ uint16_t f32_to_bf16_rne_dev(float v) {
    uint32_t u = __float_as_uint(v);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu)) return (uint16_t)((u >> 16) | 0x40u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

// IEEE half bits -> f32; exact for every pattern including subnormals (hardware cvt).
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    _Float16 f;
    __builtin_memcpy(&f, &h, 2);
    return (float)f;
}

// Wavefront reductions on the DPP path (no LDS round trips): four steps inside each row of 16
// lanes (quad swaps, half-row and row mirrors), then lane 15 / lane 31 broadcasts carry the row
// totals upward so that lane 63 holds the result, which is read back as a scalar. Fixed order,
// so the result is deterministic; every lane receives the total.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float v, float fill) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), CTRL, ROW_MASK,
                                                      0xF, false));
}

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<0xB1, 0xF>(v, 0.f);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E, 0xF>(v, 0.f);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141, 0xF>(v, 0.f);  // row_half_mirror
    v += dpp_move<0x140, 0xF>(v, 0.f);  // row_mirror: every lane of a row holds the row total
    v += dpp_move<0x142, 0xA>(v, 0.f);  // row_bcast15 into rows 1 and 3
    v += dpp_move<0x143, 0xC>(v, 0.f);  // row_bcast31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ float wave_max(float v) {
    const float ninf = -__builtin_huge_valf();
    v = fmaxf(v, dpp_move<0xB1, 0xF>(v, ninf));
    v = fmaxf(v, dpp_move<0x4E, 0xF>(v, ninf));
    v = fmaxf(v, dpp_move<0x141, 0xF>(v, ninf));
    v = fmaxf(v, dpp_move<0x140, 0xF>(v, ninf));
    v = fmaxf(v, dpp_move<0x142, 0xA>(v, ninf));
    v = fmaxf(v, dpp_move<0x143, 0xC>(v, ninf));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// 16-byte global load as four dwords.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4 ld128(const void *p) { return *reinterpret_cast<const u32x4 *>(p); }
// Streaming variant for data that is read exactly once (weights).
__device__ __forceinline__ u32x4 ld128_stream(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}
