// The small f32 ops around the heavy kernels of the decode step: RMSNorm, QK-norm + RoPE,
// SiLU*up, residual add, embedding gather, greedy argmax. All are latency-trivial next to the
// weight streams; they exist as separate entry points because the reference's quantised plan
// runs them as separate kernels (src/hf/emitter_quant.rs:713-1134).
#include "light_ops.h"
#include "../../include/homura_amd_bench.h"

namespace {

// One workgroup per row: optional residual add (reference Residual+Norm kernel,
// src/hf/emitter_quant.rs:985-1071), then RMSNorm (src/graph_builder/emit_linalg.rs:7-26).
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float *__restrict__ x,
                                                      const float *__restrict__ res,
                                                      const float *__restrict__ w,
                                                      float *__restrict__ out,
                                                      float *__restrict__ resid_out, int dim,
                                                      float eps) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * dim;
    float ss = 0.f;
    for (int i = threadIdx.x; i < dim; i += 256) {
        float v = x[base + i];
        if (res) v = v + res[base + i];
        if (resid_out) resid_out[base + i] = v;
        ss += v * v;
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv = 1.0f / sqrtf(tot / (float)dim + eps);
    for (int i = threadIdx.x; i < dim; i += 256) {
        float v = x[base + i];
        if (res) v = v + res[base + i];
        out[base + i] = (v * inv) * w[i];
    }
}

// One wavefront per (token, head) row of q or k: optional per-head RMSNorm, then
// x*cos + rotate_half(x)*sin (reference src/hf/emitter.rs:629-644,
// src/graph_builder/emit_linalg.rs:315-342). Lane i owns elements i and i + hd/2, which is
// exactly one rotation pair. Optionally also rounds k and v rows into the bf16 KV cache
// (KvCache::append_key/append_value, src/runtime.rs:521-568).
__global__ __launch_bounds__(256) void qknorm_rope_kernel(QkRopeArgs a) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int q_rows = a.S * a.H, k_rows = a.S * a.kvh;
    const int total = q_rows + k_rows + (a.v ? k_rows : 0);
    if (row >= total) return;
    const int hd = a.hd, half = hd / 2;
    const int pos = a.state ? a.state->pos : a.pos;
    const size_t trow = a.state ? (size_t)pos : 0;  // first table row to use

    if (row >= q_rows + k_rows) {
        // v row: cache append only
        const int r = row - q_rows - k_rows;
        const int s = r / a.kvh, h = r % a.kvh;
        const float *src = a.v + (size_t)r * hd;
        uint16_t *dst = a.vcache + ((size_t)h * a.max_len + pos + s) * hd;
        for (int i = lane; i < hd; i += 64) dst[i] = f32_to_bf16_rne_dev(src[i]);
        return;
    }

    const bool is_q = row < q_rows;
    const int r = is_q ? row : row - q_rows;
    const int heads = is_q ? a.H : a.kvh;
    const int s = r / heads, h = r % heads;
    float *x = (is_q ? a.q : a.k) + (size_t)r * hd;
    const float *nw = is_q ? a.qw : a.kw;
    const float *c = a.cos + (trow + s) * hd;
    const float *sn = a.sin + (trow + s) * hd;

    float lo[2], hi[2];  // hd <= 256
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int i = lane + 64 * j;
        lo[j] = i < half ? x[i] : 0.f;
        hi[j] = i < half ? x[i + half] : 0.f;
        ss += lo[j] * lo[j] + hi[j] * hi[j];
    }
    if (nw) {
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)hd + a.eps);
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int i = lane + 64 * j;
            if (i < half) {
                lo[j] = (lo[j] * inv) * nw[i];
                hi[j] = (hi[j] * inv) * nw[i + half];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int i = lane + 64 * j;
        if (i < half) {
            const float o_lo = lo[j] * c[i] + (-hi[j]) * sn[i];
            const float o_hi = hi[j] * c[i + half] + lo[j] * sn[i + half];
            x[i] = o_lo;
            x[i + half] = o_hi;
            if (!is_q && a.kcache) {
                uint16_t *dst = a.kcache + ((size_t)h * a.max_len + pos + s) * hd;
                dst[i] = f32_to_bf16_rne_dev(o_lo);
                dst[i + half] = f32_to_bf16_rne_dev(o_hi);
            }
        }
    }
}

__global__ void silu_mul_kernel(const float *__restrict__ g, const float *__restrict__ u,
                                float *__restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float gv = g[i];
        out[i] = (gv / (1.0f + expf(-gv))) * u[i];
    }
}

__global__ void add_kernel(const float *__restrict__ a, const float *__restrict__ b,
                           float *__restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}

// ids may come as int64 from the host (reference input_ids, src/hf/emitter.rs:101-105) or as
// the int32 the device argmax produced.
__global__ void embed_kernel(const int64_t *__restrict__ ids64, const int32_t *__restrict__ ids32,
                             const float *__restrict__ table, float *__restrict__ out, int hidden,
                             int vocab) {
    const int i = blockIdx.x;
    long long id = ids64 ? (long long)ids64[i] : (long long)ids32[i];
    if (id < 0 || id >= vocab) id = 0;  // host validates; never index outside the table
    const float *src = table + (size_t)id * hidden;
    for (int k = threadIdx.x; k < hidden; k += blockDim.x) out[(size_t)i * hidden + k] = src[k];
}

// Greedy pick with the reference's tie rule (Rust Iterator::max_by keeps the LAST of equal
// maxima; a NaN compares Equal and therefore displaces the running maximum,
// src/generate.rs:735-742). Sequentially that means: the answer is the last-max of the
// elements after the last NaN, or the NaN's own index if it is the final element.
// Stage 1: per segment, (index of last NaN, last-max of what follows it).
struct ArgSeg {
    float val;
    int idx;      // -1: nothing follows the last NaN inside this segment
    int nan_idx;  // -1: no NaN in this segment
};

__device__ __forceinline__ void arg_merge(float &bv, int &bi, float v, int i) {
    if (i >= 0 && (bi < 0 || v > bv || (v == bv && i > bi))) {
        bv = v;
        bi = i;
    }
}

__global__ __launch_bounds__(256) void argmax_stage1(const float *__restrict__ v, int n,
                                                     int seg_len, ArgSeg *__restrict__ segs) {
    __shared__ int s_nan[4];
    __shared__ float s_v[4];
    __shared__ int s_i[4];
    const int beg = blockIdx.x * seg_len, end = min(n, beg + seg_len);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int nan_idx = -1;
    for (int i = beg + threadIdx.x; i < end; i += 256)
        if (v[i] != v[i]) nan_idx = i;  // ascending per thread => keeps its last
    for (int off = 32; off >= 1; off >>= 1) nan_idx = max(nan_idx, __shfl_xor(nan_idx, off, 64));
    if (lane == 0) s_nan[wave] = nan_idx;
    __syncthreads();
    nan_idx = max(max(s_nan[0], s_nan[1]), max(s_nan[2], s_nan[3]));
    float bv = -INFINITY;
    int bi = -1;
    for (int i = max(beg, nan_idx + 1) + threadIdx.x; i < end; i += 256) arg_merge(bv, bi, v[i], i);
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        arg_merge(bv, bi, ov, oi);
    }
    if (lane == 0) {
        s_v[wave] = bv;
        s_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        bv = -INFINITY;
        bi = -1;
        for (int w = 0; w < 4; w++) arg_merge(bv, bi, s_v[w], s_i[w]);
        segs[blockIdx.x] = ArgSeg{bv, bi, nan_idx};
    }
}

// Stage 2 (one thread; at most a few hundred segments): walk segments from the end.
__global__ void argmax_stage2(const ArgSeg *__restrict__ segs, int nseg, int32_t *__restrict__ out) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    float bv = -INFINITY;
    int bi = -1;
    int result = -1;
    for (int s = nseg - 1; s >= 0; s--) {
        arg_merge(bv, bi, segs[s].val, segs[s].idx);
        if (segs[s].nan_idx >= 0) {
            result = bi >= 0 ? bi : segs[s].nan_idx;
            break;
        }
    }
    if (result < 0) result = bi < 0 ? 0 : bi;
    *out = result;
}

// Fold of the per-workgroup candidates produced by the LM-head GEMV's argmax epilogue.
__global__ __launch_bounds__(256) void argmax_candidates_kernel(const float *__restrict__ vals,
                                                                const int *__restrict__ idxs, int n,
                                                                int32_t *__restrict__ out) {
    __shared__ float s_v[4];
    __shared__ int s_i[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float bv = -INFINITY;
    int bi = -1;
    for (int i = threadIdx.x; i < n; i += 256) arg_merge(bv, bi, vals[i], idxs[i]);
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        arg_merge(bv, bi, ov, oi);
    }
    if (lane == 0) {
        s_v[wave] = bv;
        s_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        bv = -INFINITY;
        bi = -1;
        for (int w = 0; w < 4; w++) arg_merge(bv, bi, s_v[w], s_i[w]);
        *out = bi < 0 ? 0 : bi;
    }
}

__global__ void embed_step_kernel(const DecodeState *__restrict__ state,
                                  const int32_t *__restrict__ forced,
                                  const float *__restrict__ table, float *__restrict__ out,
                                  int hidden, int vocab) {
    const int step = state->step, n_forced = state->n_forced, token = state->token;  // one round trip
    int id = step < n_forced ? forced[step] : token;
    if (id < 0 || id >= vocab) id = 0;
    const float *src = table + (size_t)id * hidden;
    if ((hidden & 3) == 0 && ((uintptr_t)table & 15) == 0 && ((uintptr_t)out & 15) == 0) {
        // 16 bytes per thread: a row of 1024 is one load per thread, not four in a row
        for (int k = threadIdx.x * 4; k < hidden; k += blockDim.x * 4)
            *reinterpret_cast<f32x4 *>(out + k) = *reinterpret_cast<const f32x4 *>(src + k);
    } else {
        for (int k = threadIdx.x; k < hidden; k += blockDim.x) out[k] = src[k];
    }
}

__global__ __launch_bounds__(256) void finish_step_kernel(DecodeState *__restrict__ state,
                                                          const float *__restrict__ vals,
                                                          const int *__restrict__ idxs, int n,
                                                          int32_t *__restrict__ out_tokens,
                                                          int out_cap) {
    __shared__ float s_v[4];
    __shared__ int s_i[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // the cursor is requested together with the candidates (volatile: the loads stay up here), not after the fold
    const volatile DecodeState *cursor = state;
    int step = 0, pos = 0;
    if (threadIdx.x == 0) {
        step = cursor->step;
        pos = cursor->pos;
    }
    float bv = -INFINITY;
    int bi = -1;
    // the first 4096 candidates in one round trip (all loads issued before the first merge), the rest in a loop
    constexpr int FU = 16;
    float cv[FU];
    int ci[FU];
#pragma unroll
    for (int u = 0; u < FU; u++) {
        const int i = threadIdx.x + u * 256;
        cv[u] = i < n ? vals[i] : -INFINITY;
        ci[u] = i < n ? idxs[i] : -1;
    }
#pragma unroll
    for (int u = 0; u < FU; u++) arg_merge(bv, bi, cv[u], ci[u]);
    for (int i = threadIdx.x + FU * 256; i < n; i += 256) arg_merge(bv, bi, vals[i], idxs[i]);
    // wave fold on the DPP path: the maximum, then the highest index that holds it (indices are below 2^24,
    // exact as floats; -1 marks a lane without a candidate)
    const float m = wave_max(bi >= 0 ? bv : -INFINITY);
    const float sel = wave_max(bi >= 0 && bv == m ? (float)bi : -1.f);
    if (lane == 0) {
        s_v[wave] = m;
        s_i[wave] = (int)sel;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        bv = -INFINITY;
        bi = -1;
        for (int w = 0; w < 4; w++) arg_merge(bv, bi, s_v[w], s_i[w]);
        const int tok = bi < 0 ? 0 : bi;
        if (step < out_cap) out_tokens[step] = tok;
        state->token = tok;
        state->step = step + 1;
        state->pos = pos + 1;
    }
}

}  // namespace

int embed_step_launch(hm_ctx *ctx, const DecodeState *state, const int32_t *d_forced,
                      const float *d_table, float *d_out, int vocab, int hidden) {
    HM_REQUIRE(ctx, state && d_forced && d_table && d_out, "embed_step: NULL pointer");
    hipLaunchKernelGGL(embed_step_kernel, dim3(1), dim3(256), 0, ctx->stream, state, d_forced,
                       d_table, d_out, hidden, vocab);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int finish_step_launch(hm_ctx *ctx, DecodeState *state, const float *d_vals, const int *d_idxs,
                       int n, int32_t *d_out_tokens, int out_cap) {
    HM_REQUIRE(ctx, state && d_vals && d_idxs && d_out_tokens && n > 0, "finish_step: bad arguments");
    hipLaunchKernelGGL(finish_step_kernel, dim3(1), dim3(256), 0, ctx->stream, state, d_vals, d_idxs,
                       n, d_out_tokens, out_cap);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int qknorm_rope_launch(hm_ctx *ctx, const QkRopeArgs &a) {
    HM_REQUIRE(ctx, a.q && a.k && a.cos && a.sin, "qknorm_rope: NULL pointer");
    HM_REQUIRE(ctx, a.S > 0 && a.H > 0 && a.kvh > 0, "qknorm_rope: bad shape");
    HM_REQUIRE(ctx, a.hd >= 2 && a.hd <= 256 && a.hd % 2 == 0, "qknorm_rope: head_dim %d not supported", a.hd);
    HM_REQUIRE(ctx, (a.qw == nullptr) == (a.kw == nullptr), "qknorm_rope: q and k norm weights must come together");
    if (a.kcache || a.vcache || a.v) {
        HM_REQUIRE(ctx, a.kcache && a.vcache && a.v, "qknorm_rope: cache append needs kcache, vcache and v");
        if (!a.state && a.pos + a.S > a.max_len)
            return hm_set_error(ctx, HM_ERR_STATE, "KV cache full (%d + %d > %d)", a.pos, a.S, a.max_len);
    }
    const int rows = a.S * (a.H + a.kvh) + (a.v ? a.S * a.kvh : 0);
    hipLaunchKernelGGL(qknorm_rope_kernel, dim3((rows + 3) / 4), dim3(256), 0, ctx->stream, a);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int rmsnorm_launch(hm_ctx *ctx, const float *d_x, const float *d_res, const float *d_w, float *d_out,
                   float *d_resid_out, int rows, int dim, float eps) {
    HM_REQUIRE(ctx, d_x && d_w && d_out, "rmsnorm: NULL pointer");
    HM_REQUIRE(ctx, rows >= 0 && dim > 0, "rmsnorm: bad shape");
    HM_REQUIRE(ctx, d_out != d_x && d_out != d_res, "rmsnorm: output must not alias an input");
    if (rows == 0) return HM_OK;
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(rows), dim3(256), 0, ctx->stream, d_x, d_res, d_w, d_out,
                       d_resid_out, dim, eps);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int embed_launch(hm_ctx *ctx, const int64_t *d_ids64, const int32_t *d_ids32, const float *d_table,
                 float *d_out, int n_ids, int vocab, int hidden) {
    HM_REQUIRE(ctx, (d_ids64 || d_ids32) && d_table && d_out, "embed: NULL pointer");
    HM_REQUIRE(ctx, n_ids > 0 && vocab > 0 && hidden > 0, "embed: bad shape");
    hipLaunchKernelGGL(embed_kernel, dim3(n_ids), dim3(256), 0, ctx->stream, d_ids64, d_ids32,
                       d_table, d_out, hidden, vocab);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int argmax_candidates_launch(hm_ctx *ctx, const float *d_vals, const int *d_idxs, int n,
                             int32_t *d_out) {
    HM_REQUIRE(ctx, d_vals && d_idxs && d_out && n > 0, "argmax_candidates: bad arguments");
    hipLaunchKernelGGL(argmax_candidates_kernel, dim3(1), dim3(256), 0, ctx->stream, d_vals, d_idxs,
                       n, d_out);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

// A kernel that does nothing, and one that waits for a 4-byte load that depends on its predecessor's store:
// the two floors of a step built from dependent launches.
__global__ void floor_empty_kernel() {}
__global__ void floor_chain_kernel(const int *__restrict__ in, int *__restrict__ out) {
    if (threadIdx.x == 0) *out = *in + 1;
}

// Fills the LDS of the CU it runs on with a word and stays for a moment, so that the grid spreads over all CUs.
__global__ __launch_bounds__(256) void fill_lds_kernel(uint32_t word, int words) {
    extern __shared__ uint32_t lds_words[];
    for (int i = threadIdx.x; i < words; i += 256) lds_words[i] = word;
    __syncthreads();
    uint32_t x = lds_words[(threadIdx.x * 61) % words];
    for (int i = 0; i < 200; i++) x = x * 1664525u + 1013904223u;  // a few microseconds of residence
    if (x == 0x12345678u && words < 0) lds_words[0] = x;            // keeps the loop
}

extern "C" {

int hm_test_fill_lds(hm_ctx *ctx, uint32_t word) {
    HM_CHECK_CTX(ctx);
    hipDeviceProp_t prop;
    HM_HIP(ctx, hipGetDeviceProperties(&prop, ctx->device));
    size_t bytes = prop.maxSharedMemoryPerMultiProcessor;  // the whole LDS of a CU: one workgroup a CU at a time
    if (bytes == 0 || bytes > (size_t)160 << 10) bytes = (size_t)64 << 10;
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(fill_lds_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) {
        (void)hipGetLastError();
        bytes = (size_t)64 << 10;
    }
    hipLaunchKernelGGL(fill_lds_kernel, dim3(8 * ctx->num_cus), dim3(256), bytes, ctx->stream, word, (int)(bytes / 4));
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int hm_bench_launch_floor(hm_ctx *ctx, int n_kernels, int chained, int replays, float *us_per_replay) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, n_kernels > 0 && n_kernels <= 4096 && replays > 0 && us_per_replay, "hm_bench_launch_floor: bad arguments");
    int *cells = nullptr;
    HM_HIP(ctx, hipMalloc(&cells, 2 * sizeof(int)));
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = HM_OK;
    auto step = [&](hipError_t e) {
        if (rc == HM_OK && e != hipSuccess) rc = hm_set_error(ctx, HM_ERR_HIP, "launch floor: %s", hipGetErrorString(e));
    };
    floor_chain_kernel<<<1, 64, 0, ctx->stream>>>(cells, cells + 1);  // first use outside the capture; cells need no start value
    step(hipGetLastError());
    step(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
    if (rc == HM_OK) {
        for (int i = 0; i < n_kernels; i++) {
            if (chained)
                floor_chain_kernel<<<1, 64, 0, ctx->stream>>>(cells + (i & 1), cells + ((i + 1) & 1));
            else
                floor_empty_kernel<<<1, 64, 0, ctx->stream>>>();
        }
        step(hipStreamEndCapture(ctx->stream, &graph));
    }
    if (rc == HM_OK) step(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    if (rc == HM_OK) step(hipEventCreate(&e0));
    if (rc == HM_OK) step(hipEventCreate(&e1));
    if (rc == HM_OK) {
        for (int i = 0; i < 3; i++) step(hipGraphLaunch(exec, ctx->stream));
        step(hipEventRecord(e0, ctx->stream));
        for (int i = 0; i < replays; i++) step(hipGraphLaunch(exec, ctx->stream));
        step(hipEventRecord(e1, ctx->stream));
        step(hipEventSynchronize(e1));
        float ms = 0.f;
        step(hipEventElapsedTime(&ms, e0, e1));
        *us_per_replay = ms * 1000.0f / (float)replays;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(cells);
    return rc;
}

int hm_rmsnorm(hm_ctx *ctx, const float *d_x, const float *d_w, float *d_out, int rows, int dim,
               float eps) {
    HM_CHECK_CTX(ctx);
    return rmsnorm_launch(ctx, d_x, nullptr, d_w, d_out, nullptr, rows, dim, eps);
}

int hm_qknorm_rope(hm_ctx *ctx, float *d_q, float *d_k, const float *d_qw, const float *d_kw,
                   const float *d_cos, const float *d_sin, int S, int H, int kvh, int hd,
                   float eps) {
    HM_CHECK_CTX(ctx);
    QkRopeArgs a;
    a.q = d_q;
    a.k = d_k;
    a.qw = d_qw;
    a.kw = d_kw;
    a.cos = d_cos;
    a.sin = d_sin;
    a.S = S;
    a.H = H;
    a.kvh = kvh;
    a.hd = hd;
    a.eps = eps;
    return qknorm_rope_launch(ctx, a);
}

int hm_silu_mul(hm_ctx *ctx, const float *d_gate, const float *d_up, float *d_out, size_t n) {
    HM_CHECK_CTX(ctx);
    if (n == 0) return HM_OK;
    HM_REQUIRE(ctx, d_gate && d_up && d_out, "hm_silu_mul: NULL pointer");
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream,
                       d_gate, d_up, d_out, n);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int hm_add(hm_ctx *ctx, const float *d_a, const float *d_b, float *d_out, size_t n) {
    HM_CHECK_CTX(ctx);
    if (n == 0) return HM_OK;
    HM_REQUIRE(ctx, d_a && d_b && d_out, "hm_add: NULL pointer");
    hipLaunchKernelGGL(add_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream, d_a,
                       d_b, d_out, n);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int hm_embed(hm_ctx *ctx, const int64_t *d_ids, const float *d_table, float *d_out, int n_ids,
             int vocab, int hidden) {
    HM_CHECK_CTX(ctx);
    if (n_ids == 0) return HM_OK;
    return embed_launch(ctx, d_ids, nullptr, d_table, d_out, n_ids, vocab, hidden);
}

int hm_argmax(hm_ctx *ctx, const float *d_values, int n, int32_t *d_index_out) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_values && d_index_out && n > 0, "hm_argmax: bad arguments");
    const int seg_len = 2048;
    const int nseg = (n + seg_len - 1) / seg_len;
    HM_REQUIRE(ctx, (size_t)nseg * sizeof(ArgSeg) <= ctx->workspace_bytes, "hm_argmax: n=%d too large", n);
    ArgSeg *segs = (ArgSeg *)ctx->workspace;
    hipLaunchKernelGGL(argmax_stage1, dim3(nseg), dim3(256), 0, ctx->stream, d_values, n, seg_len,
                       segs);
    HM_LAUNCH_CHECK(ctx);
    hipLaunchKernelGGL(argmax_stage2, dim3(1), dim3(64), 0, ctx->stream, segs, nseg, d_index_out);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // extern "C"
