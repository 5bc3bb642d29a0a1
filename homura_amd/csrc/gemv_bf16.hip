// Weight-streaming matmul for batch-1 decode: f32 activations x bf16 weights, f32 accumulate.
//
// Two weight layouts are served:
//   [N][K] ("stream layout", K contiguous): one wavefront owns whole output rows, every lane
//       streams 16-byte pieces of the row, partial dot products are folded with a wavefront
//       butterfly. No cross-workgroup reduction, fixed summation order.
//   [K][N] (the layout the reference hands its kernels): lanes own adjacent output columns,
//       K is split across the waves of a workgroup (LDS) and across workgroups (workspace +
//       last-arriver fold in fixed order).
// These are HBM-bandwidth kernels: algorithmic traffic is K*N*2 bytes of weights per call.
#include "gemv_bf16.h"

// ─────────────────────────── [N][K] stream layout ───────────────────────────

namespace {

constexpr int GEMV_THREADS = 256;
constexpr int GEMV_WAVES = GEMV_THREADS / WAVE;

// Stage the activation vector(s) in LDS, optionally applying
//   residual add:  r = x + res          (reference src/hf/emitter.rs:787)
//   RMSNorm:       (r * rsqrt(mean(r^2) + eps)) * w   (src/graph_builder/emit_linalg.rs:7-26)
// Every workgroup performs the same arithmetic in the same order, so all of them see
// bit-identical activations.
template <int MT>
__device__ __forceinline__ void stage_activations(float *xs, const float *__restrict__ x,
                                                  const float *__restrict__ res,
                                                  const float *__restrict__ norm_w, float eps,
                                                  int K, float *__restrict__ resid_out,
                                                  bool write_resid) {
    __shared__ float red[GEMV_WAVES];
    const int tid = threadIdx.x;
    constexpr int XMAX = 16;  // K <= 4096 keeps a thread's elements in registers
    if (K <= XMAX * GEMV_THREADS) {
        for (int m = 0; m < MT; m++) {
            // every global load of the prologue is issued before anything waits on one
            float xv[XMAX], rv[XMAX], wv[XMAX];
#pragma unroll
            for (int j = 0; j < XMAX; j++) {
                const int k = tid + j * GEMV_THREADS;
                const bool ok = k < K;
                xv[j] = ok ? x[(size_t)m * K + k] : 0.f;
                rv[j] = (ok && res) ? res[(size_t)m * K + k] : 0.f;
                wv[j] = (ok && norm_w) ? norm_w[k] : 0.f;
            }
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < XMAX; j++) {
                if (res) xv[j] = xv[j] + rv[j];
                ss += xv[j] * xv[j];
            }
            float inv = 1.f;
            if (norm_w) {
                ss = wave_sum(ss);
                if (m > 0) __syncthreads();
                if ((tid & (WAVE - 1)) == 0) red[tid / WAVE] = ss;
                __syncthreads();
                float tot = 0.f;
#pragma unroll
                for (int w = 0; w < GEMV_WAVES; w++) tot += red[w];
                inv = 1.0f / sqrtf(tot / (float)K + eps);
            }
#pragma unroll
            for (int j = 0; j < XMAX; j++) {
                const int k = tid + j * GEMV_THREADS;
                if (k < K) {
                    if (write_resid && resid_out) resid_out[(size_t)m * K + k] = xv[j];
                    xs[m * K + k] = norm_w ? (xv[j] * inv) * wv[j] : xv[j];
                }
            }
        }
        __syncthreads();
        return;
    }
    for (int m = 0; m < MT; m++) {
        float ss = 0.f;
        for (int k = tid; k < K; k += GEMV_THREADS) {
            float v = x[(size_t)m * K + k];
            if (res) v = v + res[(size_t)m * K + k];
            xs[m * K + k] = v;
            ss += v * v;
        }
        if (norm_w) {
            ss = wave_sum(ss);
            __syncthreads();
            if ((tid & (WAVE - 1)) == 0) red[tid / WAVE] = ss;
            __syncthreads();
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < GEMV_WAVES; w++) tot += red[w];
            float inv = 1.0f / sqrtf(tot / (float)K + eps);
            for (int k = tid; k < K; k += GEMV_THREADS) {
                float v = xs[m * K + k];
                if (write_resid && resid_out) resid_out[(size_t)m * K + k] = v;
                xs[m * K + k] = (v * inv) * norm_w[k];
            }
        } else if (write_resid && resid_out) {
            for (int k = tid; k < K; k += GEMV_THREADS) resid_out[(size_t)m * K + k] = xs[m * K + k];
        }
    }
    __syncthreads();
}

__device__ __forceinline__ float dot8(const u32x4 w, const float *xv, float acc) {
    acc = fmaf(bf16_lo(w.x), xv[0], acc);
    acc = fmaf(bf16_hi(w.x), xv[1], acc);
    acc = fmaf(bf16_lo(w.y), xv[2], acc);
    acc = fmaf(bf16_hi(w.y), xv[3], acc);
    acc = fmaf(bf16_lo(w.z), xv[4], acc);
    acc = fmaf(bf16_hi(w.z), xv[5], acc);
    acc = fmaf(bf16_lo(w.w), xv[6], acc);
    acc = fmaf(bf16_hi(w.w), xv[7], acc);
    return acc;
}

__device__ __forceinline__ float dot4_f32(const u32x4 w, const float *xv, float acc) {
    acc = fmaf(__uint_as_float(w.x), xv[0], acc);
    acc = fmaf(__uint_as_float(w.y), xv[1], acc);
    acc = fmaf(__uint_as_float(w.z), xv[2], acc);
    acc = fmaf(__uint_as_float(w.w), xv[3], acc);
    return acc;
}

// R rows per wavefront per step, MT activation rows. WF32: weights are f32 (4 per 16-byte
// load) instead of bf16 (8 per load); same contraction (reference make_mixed_matmul_region with
// an f32 right-hand side, src/graph_builder/emit_linalg.rs:2224-2307).
template <int R, int MT, int EPI, bool WF32>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_bf16_nk_kernel(GemvArgs a) {
    constexpr int EPL = WF32 ? 4 : 8;  // elements per lane per load
    constexpr int ESZ = WF32 ? 4 : 2;
    extern __shared__ float xs[];  // [MT][K]
    const int K = a.K, N = a.N;
    stage_activations<MT>(xs, a.x, a.prologue_residual, a.norm_w, a.eps, K, a.resid_out,
                          blockIdx.x == 0);

    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int groups = (N + R - 1) / R;
    const int nchunks = (K + WAVE * EPL - 1) / (WAVE * EPL);
    const int gstride = gridDim.x * GEMV_WAVES;

    float best_v = -INFINITY;
    int best_i = -1;

    for (int g = blockIdx.x * GEMV_WAVES + wave; g < groups; g += gstride) {
        const int row0 = g * R;
        float acc[R][MT];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int m = 0; m < MT; m++) acc[r][m] = 0.f;

        const char *wrow[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            int row = row0 + r < N ? row0 + r : N - 1;  // clamp: tail rows re-read a valid row
            wrow[r] = reinterpret_cast<const char *>(a.w) + (size_t)row * K * ESZ;
        }

#pragma unroll 2
        for (int c = 0; c < nchunks; c++) {
            const int k = (c * WAVE + lane) * EPL;
            if (k < K) {
                u32x4 wv[R];
#pragma unroll
                for (int r = 0; r < R; r++) wv[r] = ld128_stream(wrow[r] + (size_t)k * ESZ);
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    float xv[8];
                    const f32x4 x0 = *reinterpret_cast<const f32x4 *>(xs + m * K + k);
                    xv[0] = x0.x; xv[1] = x0.y; xv[2] = x0.z; xv[3] = x0.w;
                    if (!WF32) {
                        const f32x4 x1 = *reinterpret_cast<const f32x4 *>(xs + m * K + k + 4);
                        xv[4] = x1.x; xv[5] = x1.y; xv[6] = x1.z; xv[7] = x1.w;
                    }
#pragma unroll
                    for (int r = 0; r < R; r++)
                        acc[r][m] = WF32 ? dot4_f32(wv[r], xv, acc[r][m]) : dot8(wv[r], xv, acc[r][m]);
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int m = 0; m < MT; m++) acc[r][m] = wave_sum(acc[r][m]);

        if (EPI == GEMV_EPI_SILU_MUL_PAIRS) {
            // rows come in (gate_i, up_i) pairs; output index = row / 2
            // (reference src/hf/emitter.rs:794-799: silu(gate) * up).
#pragma unroll
            for (int r = 0; r < R; r += 2) {
                const int row = row0 + r;
                if (lane == r && row < N) {
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        float gte = acc[r][m], up = acc[r + 1][m];
                        float s = gte / (1.0f + expf(-gte));
                        a.out[(size_t)m * (N / 2) + row / 2] = s * up;
                    }
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int row = row0 + r;
                if (lane == r && row < N) {
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        float v = acc[r][m];
                        if (a.bias) v = v + a.bias[row];
                        if (EPI == GEMV_EPI_RESIDUAL) v = a.epilogue_residual[(size_t)m * N + row] + v;
                        a.out[(size_t)m * N + row] = v;
                    }
                }
            }
            if (EPI == GEMV_EPI_ARGMAX) {
                // running (max, last index) over this wavefront's rows (ascending); m == 0 only.
                // Of equal maxima the later row wins (Rust Iterator::max_by, reference
                // src/generate.rs:735-742). NaN logits are not ordered here.
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const int row = row0 + r;
                    const float v = acc[r][0];
                    if (row < N && (best_i < 0 || v >= best_v)) {
                        best_v = v;
                        best_i = row;
                    }
                }
            }
        }
    }

    if (EPI == GEMV_EPI_ARGMAX) {
        // all lanes of a wavefront hold the same (best_v, best_i); fold the waves of the
        // workgroup through LDS and emit one candidate per workgroup.
        __shared__ float wv[GEMV_WAVES];
        __shared__ int wi[GEMV_WAVES];
        if (lane == 0) {
            wv[wave] = best_v;
            wi[wave] = best_i;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            float bv = -INFINITY;
            int bi = -1;
            for (int w = 0; w < GEMV_WAVES; w++) {
                if (wi[w] < 0) continue;
                if (bi < 0 || wv[w] > bv || (wv[w] == bv && wi[w] > bi)) {
                    bv = wv[w];
                    bi = wi[w];
                }
            }
            a.argmax_val[blockIdx.x] = bv;
            a.argmax_idx[blockIdx.x] = bi;
        }
    }
}

// Latency-ordered variant for one activation row and a matrix small enough that every
// wavefront owns exactly one group of R rows: the wavefront's whole weight slice (R rows x NC
// chunks of 512 k) is requested first, the activation prologue (residual add, RMSNorm) runs
// while those loads are in flight, and only then does anything wait. One HBM round trip per
// kernel instead of two.
template <int R, int NC>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_bf16_nk_oneshot_kernel(GemvArgs a, int epi) {
    extern __shared__ float xs[];  // [K]
    __shared__ float red[GEMV_WAVES];
    const int K = a.K, N = a.N;
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid / WAVE;
    const int row0 = (blockIdx.x * GEMV_WAVES + wave) * R;
    constexpr int NX = 2 * NC;  // K <= 512 * NC: a thread stages at most NX activation elements

    // Loads return to a wavefront in issue order, so the (small, needed-first) activation loads
    // go out before the weight stream and can be consumed while the weights are still in flight.
    float xv[NX], rv[NX], nw[NX];
#pragma unroll
    for (int j = 0; j < NX; j++) {
        const int k = tid + j * GEMV_THREADS;
        const bool ok = k < K;
        xv[j] = ok ? a.x[k] : 0.f;
        rv[j] = (ok && a.prologue_residual) ? a.prologue_residual[k] : 0.f;
        nw[j] = (ok && a.norm_w) ? a.norm_w[k] : 0.f;
    }
    u32x4 wv[NC][R];
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int k = (c * WAVE + lane) * 8;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = row0 + r < N ? row0 + r : N - 1;  // clamp: stays inside the matrix
            wv[c][r] = k < K ? ld128_stream(static_cast<const uint16_t *>(a.w) + (size_t)row * K + k)
                             : u32x4{0u, 0u, 0u, 0u};
        }
    }

    // residual add (reference src/hf/emitter.rs:787) and RMSNorm
    // (src/graph_builder/emit_linalg.rs:7-26); identical arithmetic in every workgroup
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NX; j++) {
        if (a.prologue_residual) xv[j] = xv[j] + rv[j];
        ss += xv[j] * xv[j];
    }
    float inv = 1.f;
    if (a.norm_w) {
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < GEMV_WAVES; w++) tot += red[w];
        inv = 1.0f / sqrtf(tot / (float)K + a.eps);
    }
#pragma unroll
    for (int j = 0; j < NX; j++) {
        const int k = tid + j * GEMV_THREADS;
        if (k < K) {
            if (blockIdx.x == 0 && a.resid_out) a.resid_out[k] = xv[j];
            xs[k] = a.norm_w ? (xv[j] * inv) * nw[j] : xv[j];
        }
    }
    __syncthreads();

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int k = (c * WAVE + lane) * 8;
        if (k < K) {
            float xv[8];
            const f32x4 x0 = *reinterpret_cast<const f32x4 *>(xs + k);
            const f32x4 x1 = *reinterpret_cast<const f32x4 *>(xs + k + 4);
            xv[0] = x0.x; xv[1] = x0.y; xv[2] = x0.z; xv[3] = x0.w;
            xv[4] = x1.x; xv[5] = x1.y; xv[6] = x1.z; xv[7] = x1.w;
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] = dot8(wv[c][r], xv, acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = wave_sum(acc[r]);

    if (epi == GEMV_EPI_SILU_MUL_PAIRS) {
        if constexpr (R % 2 == 0) {
#pragma unroll
            for (int r = 0; r < R; r += 2) {
                const int row = row0 + r;
                if (lane == r && row < N) {
                    const float gte = acc[r], up = acc[r + 1];
                    a.out[row / 2] = (gte / (1.0f + expf(-gte))) * up;
                }
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = row0 + r;
            if (lane == r && row < N) {
                float v = acc[r];
                if (a.bias) v = v + a.bias[row];
                if (epi == GEMV_EPI_RESIDUAL) v = a.epilogue_residual[row] + v;
                a.out[row] = v;
            }
        }
    }
}

template <int R, int NC>
int launch_oneshot(hm_ctx *ctx, const GemvArgs &a, int epi) {
    const int groups = (a.N + R - 1) / R;
    const int grid = (groups + GEMV_WAVES - 1) / GEMV_WAVES;
    hipLaunchKernelGGL((gemv_bf16_nk_oneshot_kernel<R, NC>), dim3(grid), dim3(GEMV_THREADS),
                       (size_t)a.K * 4, ctx->stream, a, epi);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

// Pick rows-per-wavefront so that the launch is about one workgroup per CU (each wavefront
// then has its whole slice in flight at once), within 16 outstanding 16-byte loads per lane.
// Returns false when the shape does not fit the one-shot kernel.
bool try_oneshot(hm_ctx *ctx, const GemvArgs &a, int epi, int *rc) {
    const int nc_exact = (a.K + 511) / 512;
    if (nc_exact > 8 || epi == GEMV_EPI_ARGMAX || a.w_f32) return false;
    static const int max_loads = [] {  // outstanding 16-byte loads per lane; HOMURA_GEMV_LOADS overrides
        const char *e = getenv("HOMURA_GEMV_LOADS");
        const int v = e ? atoi(e) : 4;
        return v < 2 ? 2 : (v > 16 ? 16 : v);
    }();
    const int nc = (nc_exact + 1) / 2 * 2;  // instantiated for 2, 4, 6, 8 chunks
    const int cand[5] = {8, 6, 4, 2, 1};
    int r_pick = 0;
    for (int i = 0; i < 5; i++) {
        const int r = cand[i];
        if (r * nc > max_loads && r > (epi == GEMV_EPI_SILU_MUL_PAIRS ? 2 : 1)) continue;
        if (epi == GEMV_EPI_SILU_MUL_PAIRS && (r % 2)) continue;
        const int wgs = ((a.N + r - 1) / r + GEMV_WAVES - 1) / GEMV_WAVES;
        if (wgs >= ctx->num_cus) {
            r_pick = r;
            break;
        }
        if (!r_pick || r < r_pick) r_pick = r;  // too few rows for a full chip: smallest R
    }
    if (!r_pick) return false;
    // a matrix this large is better served by the persistent kernel (more waves per CU)
    const int wgs = ((a.N + r_pick - 1) / r_pick + GEMV_WAVES - 1) / GEMV_WAVES;
    if (wgs > 4 * ctx->num_cus) return false;
#define HM_ONESHOT(RR, CC) \
    if (r_pick == RR && nc == CC) { *rc = launch_oneshot<RR, CC>(ctx, a, epi); return true; }
    HM_ONESHOT(1, 2) HM_ONESHOT(1, 4) HM_ONESHOT(1, 6) HM_ONESHOT(1, 8)
    HM_ONESHOT(2, 2) HM_ONESHOT(2, 4) HM_ONESHOT(2, 6) HM_ONESHOT(2, 8)
    HM_ONESHOT(4, 2) HM_ONESHOT(4, 4) HM_ONESHOT(6, 2) HM_ONESHOT(8, 2)
#undef HM_ONESHOT
    return false;
}

// Rows cut across the wavefronts of a workgroup. With whole rows per wavefront a matrix of a few thousand rows
// gives a few hundred wavefronts, each walking its rows with a handful of loads in flight (the down projection
// of a 1.5B model, 8960 -> 1536: 22 us); and a matrix that one wave of loads covers still leaves every
// wavefront's requests queued behind one another. Here a workgroup owns R rows and its four wavefronts take K
// in interleaved 512-wide chunks, NC a wavefront, everything requested at once (the activation pieces first:
// loads return in issue order); the four partial sums of a row meet in LDS and are added in wavefront order.
// PRO: residual add and RMSNorm of the activation row (reference src/hf/emitter.rs:787,
// src/graph_builder/emit_linalg.rs:7-26) on the pieces in registers - the wavefronts' chunks cover the row
// exactly once, so their sums of squares add up to the row's. Nothing is staged in LDS.
template <int R, int NC, bool PRO>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_bf16_nk_splitk_kernel(GemvArgs a, int epi) {
    __shared__ float part[GEMV_WAVES][R];
    __shared__ float red[GEMV_WAVES];
    const int K = a.K, N = a.N;
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int row0 = blockIdx.x * R;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    f32x4 x0[NC], x1[NC], p0[PRO ? NC : 1], p1[PRO ? NC : 1], n0[PRO ? NC : 1], n1[PRO ? NC : 1];
    u32x4 wv[NC][R];
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int k = ((c * GEMV_WAVES + wave) * WAVE + lane) * 8;
        const bool ok = k < K;
        x0[c] = ok ? *reinterpret_cast<const f32x4 *>(a.x + k) : zero;
        x1[c] = ok ? *reinterpret_cast<const f32x4 *>(a.x + k + 4) : zero;
        if constexpr (PRO) {
            p0[c] = (ok && a.prologue_residual) ? *reinterpret_cast<const f32x4 *>(a.prologue_residual + k) : zero;
            p1[c] = (ok && a.prologue_residual) ? *reinterpret_cast<const f32x4 *>(a.prologue_residual + k + 4) : zero;
            n0[c] = (ok && a.norm_w) ? *reinterpret_cast<const f32x4 *>(a.norm_w + k) : zero;
            n1[c] = (ok && a.norm_w) ? *reinterpret_cast<const f32x4 *>(a.norm_w + k + 4) : zero;
        }
    }
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int k = ((c * GEMV_WAVES + wave) * WAVE + lane) * 8;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = row0 + r < N ? row0 + r : N - 1;  // clamp: stays inside the matrix
            wv[c][r] = k < K ? ld128_stream(static_cast<const uint16_t *>(a.w) + (size_t)row * K + k)
                             : u32x4{0u, 0u, 0u, 0u};
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // every request above goes out before any arithmetic below
    if constexpr (PRO) {
        float ss = 0.f;
#pragma unroll
        for (int c = 0; c < NC; c++) {
            if (a.prologue_residual) {
                x0[c] = x0[c] + p0[c];
                x1[c] = x1[c] + p1[c];
            }
            ss += x0[c].x * x0[c].x + x0[c].y * x0[c].y + x0[c].z * x0[c].z + x0[c].w * x0[c].w;
            ss += x1[c].x * x1[c].x + x1[c].y * x1[c].y + x1[c].z * x1[c].z + x1[c].w * x1[c].w;
            const int k = ((c * GEMV_WAVES + wave) * WAVE + lane) * 8;
            if (blockIdx.x == 0 && a.resid_out && k < K) {
                *reinterpret_cast<f32x4 *>(a.resid_out + k) = x0[c];
                *reinterpret_cast<f32x4 *>(a.resid_out + k + 4) = x1[c];
            }
        }
        if (a.norm_w) {
            ss = wave_sum(ss);
            if (lane == 0) red[wave] = ss;
            __syncthreads();
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < GEMV_WAVES; w++) tot += red[w];
            const float inv = 1.0f / sqrtf(tot / (float)K + a.eps);
#pragma unroll
            for (int c = 0; c < NC; c++) {
                x0[c] = (x0[c] * inv) * n0[c];
                x1[c] = (x1[c] * inv) * n1[c];
            }
        }
    }
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const float xv[8] = {x0[c].x, x0[c].y, x0[c].z, x0[c].w, x1[c].x, x1[c].y, x1[c].z, x1[c].w};
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = dot8(wv[c][r], xv, acc[r]);
    }
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; r++) part[wave][r] = acc[r];
    }
    __syncthreads();
    const int t = threadIdx.x;
    auto row_sum = [&](int r) {
        float v = part[0][r];
#pragma unroll
        for (int w = 1; w < GEMV_WAVES; w++) v += part[w][r];
        return v;
    };
    if (epi == GEMV_EPI_SILU_MUL_PAIRS) {
        // rows come in (gate_i, up_i) pairs; output index = row / 2 (reference src/hf/emitter.rs:794-799)
        if (R % 2 == 0 && t < R / 2 && row0 + 2 * t < N) {
            const float gte = row_sum(2 * t), up = row_sum(2 * t + 1);
            a.out[(row0 + 2 * t) / 2] = (gte / (1.0f + expf(-gte))) * up;
        }
    } else if (t < R && row0 + t < N) {
        float v = row_sum(t);
        const int row = row0 + t;
        if (a.bias) v = v + a.bias[row];
        if (epi == GEMV_EPI_RESIDUAL) v = a.epilogue_residual[row] + v;
        a.out[row] = v;
    }
}

template <int R, int NC>
int launch_splitk(hm_ctx *ctx, const GemvArgs &a, int epi, bool pro) {
    const int grid = (a.N + R - 1) / R;
    if (pro) {
        if constexpr (NC <= 4)
            hipLaunchKernelGGL((gemv_bf16_nk_splitk_kernel<R, NC, true>), dim3(grid), dim3(GEMV_THREADS), 0, ctx->stream, a, epi);
    } else {
        hipLaunchKernelGGL((gemv_bf16_nk_splitk_kernel<R, NC, false>), dim3(grid), dim3(GEMV_THREADS), 0, ctx->stream, a, epi);
    }
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

// One activation row, bf16 weights, rows of 512 .. 16384 elements (with a prologue: up to 8192), fewer than
// 65536 of them (the LM heads keep the persistent kernel and its candidates).
bool try_splitk(hm_ctx *ctx, const GemvArgs &a, int epi, int *rc) {
    static const bool enabled = [] {  // HOMURA_GEMV_SPLITK=0: rows are never cut (for comparisons)
        const char *e = getenv("HOMURA_GEMV_SPLITK");
        return !e || atoi(e) != 0;
    }();
    if (!enabled || a.w_f32 || epi == GEMV_EPI_ARGMAX) return false;
    const bool pro = a.norm_w || a.prologue_residual || a.resid_out;
    const int per_wg = WAVE * 8 * GEMV_WAVES;  // k covered by one chunk of each wavefront
    const int nc = (a.K + per_wg - 1) / per_wg;
    if (a.K < 512 || nc > (pro ? 4 : 8) || a.N >= 65536) return false;
    // Rows a workgroup, the best of 1 .. 16 measured over 25 shapes. Every workgroup reads the activation
    // pieces itself (4 bytes per k, 12 with residual and norm weights, against 2 R of weights), so a prologue
    // wants more rows; few short rows want one.
    const size_t bytes = (size_t)2 * a.K * a.N;
    int r;
    if (pro) r = (a.K >= 4096 && a.N >= 8192) ? 8 : 4;
    else r = (a.K >= 4096 && a.N >= 2048) ? 4 : ((a.N <= 1536 && bytes < ((size_t)17 << 19)) ? 1 : 2);
    if (epi == GEMV_EPI_SILU_MUL_PAIRS && r == 1) r = 2;
#define HM_SPLITK(RR, CC) \
    if (r == RR && nc == CC) { *rc = launch_splitk<RR, CC>(ctx, a, epi, pro); return true; }
    HM_SPLITK(1, 1) HM_SPLITK(1, 2) HM_SPLITK(1, 3) HM_SPLITK(1, 4) HM_SPLITK(1, 5) HM_SPLITK(1, 6) HM_SPLITK(1, 7) HM_SPLITK(1, 8)
    HM_SPLITK(2, 1) HM_SPLITK(2, 2) HM_SPLITK(2, 3) HM_SPLITK(2, 4) HM_SPLITK(2, 5) HM_SPLITK(2, 6) HM_SPLITK(2, 7) HM_SPLITK(2, 8)
    HM_SPLITK(4, 1) HM_SPLITK(4, 2) HM_SPLITK(4, 3) HM_SPLITK(4, 4) HM_SPLITK(4, 5) HM_SPLITK(4, 6) HM_SPLITK(4, 7) HM_SPLITK(4, 8)
    HM_SPLITK(8, 1) HM_SPLITK(8, 2) HM_SPLITK(8, 3) HM_SPLITK(8, 4)
#undef HM_SPLITK
    return false;
}

template <int R, int MT, bool WF32>
int launch_nk_t(hm_ctx *ctx, const GemvArgs &a, int epi, int grid, size_t lds) {
    dim3 g(grid), b(GEMV_THREADS);
    switch (epi) {
    case GEMV_EPI_NONE:
        hipLaunchKernelGGL((gemv_bf16_nk_kernel<R, MT, GEMV_EPI_NONE, WF32>), g, b, lds, ctx->stream, a);
        break;
    case GEMV_EPI_RESIDUAL:
        hipLaunchKernelGGL((gemv_bf16_nk_kernel<R, MT, GEMV_EPI_RESIDUAL, WF32>), g, b, lds, ctx->stream, a);
        break;
    case GEMV_EPI_SILU_MUL_PAIRS:
        hipLaunchKernelGGL((gemv_bf16_nk_kernel<R, MT, GEMV_EPI_SILU_MUL_PAIRS, WF32>), g, b, lds, ctx->stream, a);
        break;
    case GEMV_EPI_ARGMAX:
        hipLaunchKernelGGL((gemv_bf16_nk_kernel<R, MT, GEMV_EPI_ARGMAX, WF32>), g, b, lds, ctx->stream, a);
        break;
    default:
        return hm_set_error(ctx, HM_ERR_INVALID, "gemv: unknown epilogue %d", epi);
    }
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

template <int R, int MT>
int launch_nk(hm_ctx *ctx, const GemvArgs &a, int epi, int grid, size_t lds) {
    return a.w_f32 ? launch_nk_t<R, MT, true>(ctx, a, epi, grid, lds)
                   : launch_nk_t<R, MT, false>(ctx, a, epi, grid, lds);
}

}  // namespace

int gemv_bf16_nk_grid(const hm_ctx *ctx, int N, int R) {
    const int groups = (N + R - 1) / R;
    int wgs = (groups + GEMV_WAVES - 1) / GEMV_WAVES;
    const int cap = ctx->num_cus * 8;  // 8 workgroups (32 waves) per CU keep the loads deep
    return wgs < cap ? wgs : cap;
}

int gemv_bf16_nk_launch(hm_ctx *ctx, GemvArgs a, int M, int epi) {
    HM_REQUIRE(ctx, a.K > 0 && a.N > 0 && a.K % 8 == 0, "gemv_bf16_nk: K=%d must be a positive multiple of 8", a.K);
    HM_REQUIRE(ctx, a.x && a.w && a.out, "gemv_bf16_nk: NULL pointer");
    HM_REQUIRE(ctx, M >= 1 && M <= 8, "gemv_bf16_nk: M=%d outside 1..8", M);
    HM_REQUIRE(ctx, (size_t)a.K * 4 <= 64 * 1024, "gemv_bf16_nk: K=%d too large for the LDS stage", a.K);
    HM_REQUIRE(ctx, ((uintptr_t)a.w % 16) == 0 && ((uintptr_t)a.x % 16) == 0, "gemv_bf16_nk: pointers must be 16-byte aligned");
    if (epi == GEMV_EPI_SILU_MUL_PAIRS) HM_REQUIRE(ctx, a.N % 2 == 0 && !a.bias, "gemv: paired epilogue needs even N and no bias");
    if (epi == GEMV_EPI_ARGMAX) HM_REQUIRE(ctx, M == 1 && a.argmax_val && a.argmax_idx && !a.bias, "gemv: argmax epilogue needs M == 1, candidate buffers and no bias");
    const int out_n = epi == GEMV_EPI_SILU_MUL_PAIRS ? a.N / 2 : a.N;
    int m0 = 0;
    while (m0 < M) {
        GemvArgs b = a;
        b.x = a.x + (size_t)m0 * a.K;
        if (a.prologue_residual) b.prologue_residual = a.prologue_residual + (size_t)m0 * a.K;
        if (a.resid_out) b.resid_out = a.resid_out + (size_t)m0 * a.K;
        if (a.epilogue_residual) b.epilogue_residual = a.epilogue_residual + (size_t)m0 * a.N;
        b.out = a.out + (size_t)m0 * out_n;
        int rc;
        if (M - m0 >= 4 && (size_t)4 * a.K * 4 <= 64 * 1024) {
            const int grid = gemv_bf16_nk_grid(ctx, a.N, 2);
            rc = launch_nk<2, 4>(ctx, b, epi, grid, (size_t)4 * a.K * 4);
            m0 += 4;
        } else {
            if (!try_splitk(ctx, b, epi, &rc) && !try_oneshot(ctx, b, epi, &rc)) {
                int grid = gemv_bf16_nk_grid(ctx, a.N, 4);
                if (epi == GEMV_EPI_ARGMAX && grid > a.argmax_cap) grid = a.argmax_cap;
                rc = launch_nk<4, 1>(ctx, b, epi, grid, (size_t)a.K * 4);
            }
            m0 += 1;
        }
        if (rc != HM_OK) return rc;
    }
    return HM_OK;
}

// ─────────────────────────── [K][N] reference layout ───────────────────────────

namespace {

constexpr int KN_COLS_PER_LANE = 4;                    // 8-byte loads
constexpr int KN_STRIP = WAVE * KN_COLS_PER_LANE;      // 256 columns per workgroup

// grid = (strips, ksplit). Each wave of the workgroup walks rows k = kbeg + wave, +4, ...
// of the workgroup's K slice; partials are folded over the 4 waves in LDS and written to the
// workspace; a second small kernel folds the ksplit partials in ascending order
// (deterministic, and no device-scope fence is needed: the kernel boundary orders the writes).
__global__ __launch_bounds__(GEMV_THREADS) void gemv_bf16_kn_kernel(
    const float *__restrict__ x, const uint16_t *__restrict__ w, float *__restrict__ out,
    float *__restrict__ partial, int K, int N, int kslice) {
    __shared__ float red[GEMV_WAVES][KN_STRIP];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int strip = blockIdx.x, ks = blockIdx.y, ksplit = gridDim.y;
    const int col = strip * KN_STRIP + lane * KN_COLS_PER_LANE;
    const int kbeg = ks * kslice;
    const int kend = min(K, kbeg + kslice);

    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (col < N) {
#pragma unroll 8
        for (int k = kbeg + wave; k < kend; k += GEMV_WAVES) {
            const u32x2 wv = __builtin_nontemporal_load(
                reinterpret_cast<const u32x2 *>(w + (size_t)k * N + col));
            const float xk = x[k];
            acc[0] = fmaf(bf16_lo(wv.x), xk, acc[0]);
            acc[1] = fmaf(bf16_hi(wv.x), xk, acc[1]);
            acc[2] = fmaf(bf16_lo(wv.y), xk, acc[2]);
            acc[3] = fmaf(bf16_hi(wv.y), xk, acc[3]);
        }
    }
#pragma unroll
    for (int j = 0; j < 4; j++) red[wave][lane * 4 + j] = acc[j];
    __syncthreads();
    const int t = threadIdx.x;  // 256 threads <-> 256 columns
    const int c = strip * KN_STRIP + t;
    const float s = (red[0][t] + red[1][t]) + (red[2][t] + red[3][t]);
    if (c < N) (ksplit == 1 ? out : partial + (size_t)ks * N)[c] = s;
}

__global__ __launch_bounds__(256) void gemv_bf16_kn_fold_kernel(const float *__restrict__ partial,
                                                                float *__restrict__ out, int N,
                                                                int ksplit) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= N) return;
    float tot = 0.f;
#pragma unroll 8
    for (int j = 0; j < ksplit; j++) tot += partial[(size_t)j * N + c];
    out[c] = tot;
}

// Output row n lands at dst row n * row_mult + row_off (1, 0 = plain transpose; 2, 0 / 2, 1
// interleave two matrices row by row).
__global__ __launch_bounds__(256) void pack_kn_to_nk_kernel(const uint16_t *__restrict__ src,
                                                            uint16_t *__restrict__ dst, int K,
                                                            int N, int row_mult, int row_off) {
    __shared__ uint16_t tile[64][66];
    const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        int k = k0 + i, n = n0 + tx;
        tile[i][tx] = (k < K && n < N) ? src[(size_t)k * N + n] : (uint16_t)0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        int n = n0 + i, k = k0 + tx;
        if (n < N && k < K) dst[((size_t)n * row_mult + row_off) * K + k] = tile[tx][i];
    }
}

// f32 [K][N] -> [N][K] (LM head of the quantised plan)
__global__ __launch_bounds__(256) void pack_f32_kn_to_nk_kernel(const float *__restrict__ src,
                                                                float *__restrict__ dst, int K, int N) {
    __shared__ float tile[64][65];
    const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        int k = k0 + i, n = n0 + tx;
        tile[i][tx] = (k < K && n < N) ? src[(size_t)k * N + n] : 0.f;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        int n = n0 + i, k = k0 + tx;
        if (n < N && k < K) dst[(size_t)n * K + k] = tile[tx][i];
    }
}

}  // namespace

int pack_f32_kn_to_nk(hm_ctx *ctx, const float *d_w_kn, float *d_dst, int K, int N) {
    HM_REQUIRE(ctx, d_w_kn && d_dst && K > 0 && N > 0, "pack_f32_kn_to_nk: bad arguments");
    dim3 grid((N + 63) / 64, (K + 63) / 64);
    hipLaunchKernelGGL(pack_f32_kn_to_nk_kernel, grid, dim3(256), 0, ctx->stream, d_w_kn, d_dst, K, N);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int pack_bf16_kn_to_nk_strided(hm_ctx *ctx, const uint16_t *d_w_kn, uint16_t *d_dst, int K, int N,
                               int row_mult, int row_off) {
    HM_REQUIRE(ctx, d_w_kn && d_dst && K > 0 && N > 0 && row_mult >= 1 && row_off >= 0 && row_off < row_mult,
               "pack_bf16_kn_to_nk: bad arguments");
    dim3 grid((N + 63) / 64, (K + 63) / 64);
    hipLaunchKernelGGL(pack_kn_to_nk_kernel, grid, dim3(256), 0, ctx->stream, d_w_kn, d_dst, K, N,
                       row_mult, row_off);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

extern "C" {

int hm_gemv_bf16_nk(hm_ctx *ctx, const float *d_x, const uint16_t *d_w_nk, float *d_out, int M,
                    int K, int N) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x && d_w_nk && d_out, "hm_gemv_bf16_nk: NULL pointer");
    GemvArgs a{};
    a.x = d_x;
    a.w = d_w_nk;
    a.out = d_out;
    a.K = K;
    a.N = N;
    return gemv_bf16_nk_launch(ctx, a, M, GEMV_EPI_NONE);
}

int hm_gemv_bf16(hm_ctx *ctx, const float *d_x, const uint16_t *d_w_kn, float *d_out, int M, int K,
                 int N) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x && d_w_kn && d_out, "hm_gemv_bf16: NULL pointer");
    HM_REQUIRE(ctx, M >= 1 && M <= 8, "hm_gemv_bf16: M=%d outside 1..8", M);
    HM_REQUIRE(ctx, K > 0 && N > 0 && N % 4 == 0, "hm_gemv_bf16: need K > 0 and N %% 4 == 0 (K=%d N=%d)", K, N);
    HM_REQUIRE(ctx, ((uintptr_t)d_w_kn % 8) == 0, "hm_gemv_bf16: weight pointer must be 8-byte aligned");
    const int strips = (N + KN_STRIP - 1) / KN_STRIP;
    // enough workgroups for ~2 per CU, but at least 16 K rows per workgroup
    int ksplit = (2 * ctx->num_cus + strips - 1) / strips;
    int max_split = (K + 15) / 16;
    if (ksplit > max_split) ksplit = max_split;
    if (ksplit < 1) ksplit = 1;
    while ((size_t)ksplit * N * sizeof(float) > ctx->workspace_bytes && ksplit > 1) ksplit--;
    int kslice = (K + ksplit - 1) / ksplit;
    kslice = (kslice + GEMV_WAVES - 1) / GEMV_WAVES * GEMV_WAVES;
    ksplit = (K + kslice - 1) / kslice;
    for (int m = 0; m < M; m++) {
        hipLaunchKernelGGL(gemv_bf16_kn_kernel, dim3(strips, ksplit), dim3(GEMV_THREADS), 0,
                           ctx->stream, d_x + (size_t)m * K, d_w_kn, d_out + (size_t)m * N,
                           (float *)ctx->workspace, K, N, kslice);
        HM_LAUNCH_CHECK(ctx);
        if (ksplit > 1) {
            hipLaunchKernelGGL(gemv_bf16_kn_fold_kernel, dim3((N + 255) / 256), dim3(256), 0, ctx->stream,
                               (const float *)ctx->workspace, d_out + (size_t)m * N, N, ksplit);
            HM_LAUNCH_CHECK(ctx);
        }
    }
    return HM_OK;
}

int hm_pack_bf16_kn_to_nk(hm_ctx *ctx, const uint16_t *d_w_kn, uint16_t *d_w_nk, int K, int N) {
    HM_CHECK_CTX(ctx);
    return pack_bf16_kn_to_nk_strided(ctx, d_w_kn, d_w_nk, K, N, 1, 0);
}

}  // extern "C"
