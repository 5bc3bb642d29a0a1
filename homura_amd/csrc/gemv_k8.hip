// Q4_K / Q6_K decode product over the K8 form of the matrices (kquant_planes8.h): one activation row against
// the rows of a byte plane [N][K] with per-row scale records, the reference's integer arithmetic
// (src/graph_builder/emit_quant.rs:165-816, src/hf/emitter_quant.rs:675-702) with nothing staged in LDS.
//
// A lane's unit is one 16-weight sub-block (16 bytes of the plane, its (sc, mn) pair and the (d, dmin) of its
// super-block); the 16 lanes of a DPP row hold one 256-wide super-block, a wavefront's chunk is four of them.
// WPS wavefronts (1, 2 or 4: as many as a row has chunks, so that none idles while holding registers) share a
// set of R rows and take the rows' chunks in turn, NC each; a workgroup works on 4 / WPS sets. Every load is requested
// before anything waits, the activation pieces first. The activation row is prepared on the pieces in
// registers - SiLU pair or residual add, RMSNorm (the wavefronts' chunks cover the row exactly once, so their
// sums of squares add up to the row's), then the Q8_K quantisation of emit_quant.rs:422-466, whose block is
// the DPP row - so neither a launch of its own nor a pass through memory is needed for it, and mixed Q4_K /
// Q6_K groups (q|k in one type, v in the other) multiply in one launch: the K8 form is the same for both.
// The integer sums of a block are exact; blocks and wavefronts are added in f32, in a fixed order.
#include "gemv_k8.h"

#include "k8_device.h"
#include "kquant_planes8.h"

namespace {

using homura::QuantFuse;

constexpr int GTHREADS = 256;
constexpr int GWAVES = GTHREADS / WAVE;

typedef const u32x4 __attribute__((address_space(1))) *global_u32x4_ptr;
typedef const uint32_t __attribute__((address_space(1))) *global_u32_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;

// MODE 0: plain row. 1: a second operand (x2 or res_in). 2: RMSNorm, with or without res_in.
template <int R, int NC, int MODE, int WPS>
__global__ __launch_bounds__(GTHREADS) void gemv_k8_kernel(const float *__restrict__ x, const uint8_t *__restrict__ plane,
                                                           const uint8_t *__restrict__ records, float *__restrict__ out, int K,
                                                           int N, const QuantFuse fuse_arg) {
    const QuantFuse fuse = MODE == 0 ? QuantFuse() : fuse_arg;
    const float *res_out_add = fuse_arg.res_out_add;
    __shared__ float part[GWAVES][R];
    __shared__ float red[GWAVES];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    constexpr int SETS = GWAVES / WPS;
    const int set = wave / WPS, wis = wave % WPS;  // the wavefront's row set and its place among the set's wavefronts
    const int row0 = (blockIdx.x * SETS + set) * R;
    const size_t rs = (size_t)K / 8 + (size_t)K / 64;  // bytes of a row's record
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    constexpr int NS = MODE >= 1 ? NC : 1, NN = MODE == 2 ? NC : 1;
    f32x4 xr[NC][4], ar[NS][4], nr[NN][4];
    u32x4 qw[NC][R];
    uint32_t sub[NC][R], dd[NC][R];
    const float *second = fuse.x2 ? fuse.x2 : fuse.res_in;
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int k = ((c * WPS + wis) * WAVE + lane) * 16;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            xr[c][j] = k < K ? *reinterpret_cast<const f32x4 *>(x + k + 4 * j) : zero4;
            if constexpr (MODE >= 1) ar[c][j] = (second && k < K) ? *reinterpret_cast<const f32x4 *>(second + k + 4 * j) : zero4;
            if constexpr (MODE == 2) nr[c][j] = (fuse.norm_w && k < K) ? *reinterpret_cast<const f32x4 *>(fuse.norm_w + k + 4 * j) : zero4;
        }
    }
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int k = ((c * WPS + wis) * WAVE + lane) * 16;
        const int kc = k < K ? k : 0;  // blocks past the row end re-read its first one against activations of zero
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = min(row0 + r, N - 1);  // rows past the end re-read the last one
            const uint8_t *rec = records + (size_t)row * rs;
            qw[c][r] = __builtin_nontemporal_load((global_u32x4_ptr)(plane + (size_t)row * K + kc));
            sub[c][r] = __builtin_nontemporal_load((global_u16_ptr)(rec + (kc / 16) * 2));
            dd[c][r] = __builtin_nontemporal_load((global_u32_ptr)(rec + K / 8 + (kc / 256) * 4));
        }
    }
    // every request above goes out before any arithmetic below (left alone, the compiler requests three rows,
    // waits for the activations and deals the other rows' requests out between the products)
    __builtin_amdgcn_sched_barrier(0);
    // the light ops of the quantised plan in front of this product (reference src/hf/emitter_quant.rs:713-791,
    // :985-1103), arithmetic as in the stand-alone kernels
    if constexpr (MODE >= 1) {
        if (fuse.x2) {
#pragma unroll
            for (int c = 0; c < NC; c++)
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int e = 0; e < 4; e++) xr[c][j][e] = (xr[c][j][e] / (1.0f + expf(-xr[c][j][e]))) * ar[c][j][e];
        } else if (fuse.res_in) {
#pragma unroll
            for (int c = 0; c < NC; c++) {
                const int k = ((c * WPS + wis) * WAVE + lane) * 16;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    xr[c][j] += ar[c][j];
                    if (fuse.resid_out && blockIdx.x == 0 && set == 0 && k < K) *reinterpret_cast<f32x4 *>(fuse.resid_out + k + 4 * j) = xr[c][j];
                }
            }
        }
    }
    if constexpr (MODE == 2) {
        if (fuse.norm_w) {
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < NC; c++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    ss += (xr[c][j][0] * xr[c][j][0] + xr[c][j][1] * xr[c][j][1]) + (xr[c][j][2] * xr[c][j][2] + xr[c][j][3] * xr[c][j][3]);
            ss = wave_sum(ss);
            if (lane == 0) red[wave] = ss;
            __syncthreads();
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < WPS; w++) tot += red[set * WPS + w];
            const float inv = 1.0f / sqrtf(tot / (float)K + fuse.eps);
#pragma unroll
            for (int c = 0; c < NC; c++)
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int e = 0; e < 4; e++) xr[c][j][e] = (xr[c][j][e] * inv) * nr[c][j][e];
        }
    }
    float a[R];
#pragma unroll
    for (int r = 0; r < R; r++) a[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; c++) {
        float xv[16];
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) xv[4 * j + e] = xr[c][j][e];
        const Q8kLane act = q8k_lane(xv, dpp_row_fmax(abs_max16(xv)));
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float p = k8_block(qw[c][r], sub[c][r], dd[c][r], act);  // the same value in the block's 16 lanes
            a[r] += (lane & 15) == 0 ? p : 0.f;
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) a[r] = wave_sum(a[r]);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; r++) part[wave][r] = a[r];
    }
    __syncthreads();
    const int t = threadIdx.x;
    auto row_total = [&](int ts, int tr) {
        float v = part[ts * WPS][tr];
#pragma unroll
        for (int w = 1; w < WPS; w++) v += part[ts * WPS + w][tr];
        return v;
    };
    if (fuse_arg.silu_pairs) {
        // rows come in (gate_i, up_i) pairs (reference src/hf/emitter_quant.rs:1077-1103: silu(gate) * up)
        if (t < SETS * (R / 2)) {
            const int ts = t / (R / 2), tp = t % (R / 2), row = (blockIdx.x * SETS + ts) * R + 2 * tp;
            if (row + 1 < N) {
                const float gte = row_total(ts, 2 * tp), up = row_total(ts, 2 * tp + 1);
                out[row / 2] = (gte / (1.0f + expf(-gte))) * up;
            }
        }
    } else if (t < SETS * R) {
        const int ts = t / R, tr = t % R, row = (blockIdx.x * SETS + ts) * R + tr;
        if (row < N) {
            float v = row_total(ts, tr);
            if (res_out_add) v = v + res_out_add[row];
            out[row] = v;
        }
    }
}

template <int R, int NC, int MODE, int WPS>
void launch(hm_ctx *ctx, const float *x, const uint8_t *plane, const uint8_t *records, float *out, int K, int N,
            const QuantFuse &fuse) {
    constexpr int ROWS = R * (GWAVES / WPS);
    hipLaunchKernelGGL((gemv_k8_kernel<R, NC, MODE, WPS>), dim3((N + ROWS - 1) / ROWS), dim3(GTHREADS), 0, ctx->stream, x, plane,
                       records, out, K, N, fuse);
}

}  // namespace

int homura::gemv_k8_fused(hm_ctx *ctx, const float *d_x, const uint8_t *d_plane, const uint8_t *d_records, float *d_out, int K,
                          int N, const QuantFuse &fuse) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x && d_plane && d_records && d_out, "gemv_k8: NULL pointer");
    HM_REQUIRE(ctx, K > 0 && K % 256 == 0 && K <= 16384 && N > 0, "gemv_k8: K=%d must be a multiple of 256 up to 16384, N=%d positive", K, N);
    HM_REQUIRE(ctx, !(fuse.x2 && fuse.res_in) && !(fuse.x2 && fuse.norm_w), "gemv_k8: the SiLU pair excludes a residual input and a norm");
    HM_REQUIRE(ctx, !fuse.norm_w || K <= 8192, "gemv_k8: the fused RMSNorm holds rows up to 8192 wide (K=%d)", K);
    HM_REQUIRE(ctx, !fuse.cand_v, "gemv_k8: no argmax candidates here");
    HM_REQUIRE(ctx, !fuse.silu_pairs || (N % 2 == 0 && !fuse.res_out_add), "gemv_k8: the paired epilogue needs an even N and no residual");
    HM_REQUIRE(ctx, ((uintptr_t)d_x % 16) == 0 && ((uintptr_t)d_plane % 16) == 0 && ((uintptr_t)d_records % 4) == 0 &&
                        ((uintptr_t)fuse.x2 % 16) == 0 && ((uintptr_t)fuse.res_in % 16) == 0 && ((uintptr_t)fuse.resid_out % 16) == 0 &&
                        ((uintptr_t)fuse.norm_w % 16) == 0, "gemv_k8: operands must be 16-byte aligned");
    const int wps = K <= WAVE * 16 ? 1 : (K <= 2 * WAVE * 16 ? 2 : 4);
    const int nc = (K + wps * WAVE * 16 - 1) / (wps * WAVE * 16);
    const int mode = fuse.norm_w ? 2 : ((fuse.x2 || fuse.res_in) ? 1 : 0);
    // Rows a set: every set reads the activation pieces itself (4 to 12 bytes per k against 1.14 R of weights), so
    // the more rows the better while there are workgroups enough to fill the chip
    const int big = N >= 2048 ? 8 : 4;  // (16 rows a set measured no faster at 17920 rows)
#define HM_K8(RR, CC, MM, WW)                                                          \
    do {                                                                               \
        launch<RR, CC, MM, WW>(ctx, d_x, d_plane, d_records, d_out, K, N, fuse);       \
        HM_LAUNCH_CHECK(ctx);                                                          \
        return HM_OK;                                                                  \
    } while (0)
#define HM_K8_R(MM, WW)                          \
    do {                                         \
        if (big == 8) HM_K8(8, 1, MM, WW);       \
        HM_K8(4, 1, MM, WW);                     \
    } while (0)
#define HM_K8_W(MM)                              \
    do {                                         \
        if (wps == 1) HM_K8_R(MM, 1);            \
        if (wps == 2) HM_K8_R(MM, 2);            \
        HM_K8_R(MM, 4);                          \
    } while (0)
    if (mode == 0) {
        if (nc == 1) HM_K8_W(0);
        if (nc == 2) { if (big >= 8) HM_K8(8, 2, 0, 4); HM_K8(4, 2, 0, 4); }
        if (nc == 3) HM_K8(4, 3, 0, 4);
        HM_K8(4, 4, 0, 4);
    } else if (mode == 1) {
        if (nc == 1) HM_K8_W(1);
        if (nc == 2) HM_K8(4, 2, 1, 4);
        if (nc == 3) HM_K8(4, 3, 1, 4);
        HM_K8(4, 4, 1, 4);
    } else {
        if (nc == 1) HM_K8_W(2);
        HM_K8(4, 2, 2, 4);
    }
#undef HM_K8_W
#undef HM_K8_R
#undef HM_K8
}

extern "C" {

size_t hm_k8_bytes(int N, int K) {
    if (N <= 0 || K <= 0 || K % 256 != 0) return 0;
    return k8_plane_bytes(N, K) + k8_record_bytes(N, K);
}

int hm_pack_k8(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int rows, uint8_t *d_k8, int N, int K, int row0) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_blocks && d_k8, "hm_pack_k8: NULL pointer");
    HM_REQUIRE(ctx, hm_dtype == HM_DTYPE_Q4_K || hm_dtype == HM_DTYPE_Q6_K, "hm_pack_k8: dtype %d is not Q4_K or Q6_K", hm_dtype);
    HM_REQUIRE(ctx, N > 0 && K > 0 && K % 256 == 0 && rows > 0 && row0 >= 0 && row0 + rows <= N,
               "hm_pack_k8: rows [%d, %d) of %d, K=%d (a multiple of 256)", row0, row0 + rows, N, K);
    return pack_k8_rows(ctx, hm_dtype, d_blocks, rows, K, d_k8, d_k8 + k8_plane_bytes(N, K), row0);
}

int hm_gemv_k8(hm_ctx *ctx, const float *d_x, const uint8_t *d_k8, float *d_out, int M, int K, int N) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x && d_k8 && d_out, "hm_gemv_k8: NULL pointer");
    HM_REQUIRE(ctx, M >= 1 && M <= 8 && N > 0 && K > 0 && K % 256 == 0, "hm_gemv_k8: M=%d outside 1..8 or bad shape K=%d N=%d", M, K, N);
    for (int m = 0; m < M; m++) {
        const int rc = homura::gemv_k8_fused(ctx, d_x + (size_t)m * K, d_k8, d_k8 + k8_plane_bytes(N, K), d_out + (size_t)m * N, K, N,
                                             homura::QuantFuse());
        if (rc != HM_OK) return rc;
    }
    return HM_OK;
}

}  // extern "C"
