// GQA decode attention over the HBM-resident bf16 KV cache, plus the cache append.
//
// One query row per sequence. The KV range is split across workgroups (flash-decode):
// grid = (splits, kv_heads, batch). A workgroup serves all G = H/kvh query heads that share
// its KV head (the reference's `h floordiv g` map, src/graph_builder/emit_linalg.rs:123-127),
// so each K/V row is read from HBM once. Rows are streamed with 16-byte loads: HD/8 lanes
// cover a row, 64/(HD/8) rows per wavefront instruction. Scores live in LDS; softmax is f32.
// Partial (o, max, sum) triples go to the workspace and the last workgroup to arrive for a
// (batch, kv head) folds them in split order, so the result does not depend on timing.
// Algorithmic HBM traffic: 2 * kv_len * HD * 2 bytes per (batch, kv head).
#include "attention.h"

namespace {

constexpr int ATT_THREADS = 256;
constexpr int ATT_WAVES = ATT_THREADS / WAVE;

__device__ __forceinline__ void unpack8(const u32x4 w, float *f) {
    f[0] = bf16_lo(w.x); f[1] = bf16_hi(w.x);
    f[2] = bf16_lo(w.y); f[3] = bf16_hi(w.y);
    f[4] = bf16_lo(w.z); f[5] = bf16_hi(w.z);
    f[6] = bf16_lo(w.w); f[7] = bf16_hi(w.w);
}

template <int HD, int G>
__global__ __launch_bounds__(ATT_THREADS) void gqa_decode_attn_kernel(
    const float *__restrict__ q, const uint16_t *__restrict__ kcache,
    const uint16_t *__restrict__ vcache, float *__restrict__ out, float *__restrict__ part_o,
    float *__restrict__ part_ml, unsigned int *__restrict__ counters, int kvh, int max_len,
    int kv_len_arg, int chunk, float scale, const DecodeState *__restrict__ state) {
    constexpr int LPR = HD / 8;    // lanes per row
    constexpr int RPI = WAVE / LPR;  // rows per wavefront instruction
    extern __shared__ float sm[];
    float *sc = sm;                          // [G][chunk] scores, then probabilities
    float *red = sm + (size_t)G * chunk;     // [ATT_WAVES][G][HD]
    __shared__ float s_m[G], s_l[G];
    __shared__ bool is_last;

    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int sub = lane / LPR, dl = lane % LPR;
    const int kv_len = state ? state->pos + 1 : kv_len_arg;
    const int split = blockIdx.x, kvhd = blockIdx.y, b = blockIdx.z;
    const int nsplit = (kv_len + chunk - 1) / chunk;  // live splits; the grid may be larger
    if (split >= nsplit) return;
    const int H = kvh * G;
    const int n0 = split * chunk;
    const int cnt = min(kv_len, n0 + chunk) - n0;
    const size_t head_base = ((size_t)b * kvh + kvhd) * max_len * HD;
    const uint16_t *kbase = kcache + head_base + (size_t)n0 * HD + dl * 8;
    const uint16_t *vbase = vcache + head_base + (size_t)n0 * HD + dl * 8;

    float qv[G][8];
#pragma unroll
    for (int gi = 0; gi < G; gi++) {
        const float *qp = q + ((size_t)b * H + kvhd * G + gi) * HD + dl * 8;
        const f32x4 a = *reinterpret_cast<const f32x4 *>(qp);
        const f32x4 c = *reinterpret_cast<const f32x4 *>(qp + 4);
        qv[gi][0] = a.x; qv[gi][1] = a.y; qv[gi][2] = a.z; qv[gi][3] = a.w;
        qv[gi][4] = c.x; qv[gi][5] = c.y; qv[gi][6] = c.z; qv[gi][7] = c.w;
    }

    // ── scores = (Q.K^T) * scale ──
    constexpr int U = 4;
    const int ngroups = (cnt + RPI - 1) / RPI;
    for (int rg0 = wave; rg0 < ngroups; rg0 += ATT_WAVES * U) {
        u32x4 kv[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int row = (rg0 + u * ATT_WAVES) * RPI + sub;
            kv[u] = row < cnt ? ld128_stream(kbase + (size_t)row * HD) : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int row = (rg0 + u * ATT_WAVES) * RPI + sub;
            float kf[8];
            unpack8(kv[u], kf);
#pragma unroll
            for (int gi = 0; gi < G; gi++) {
                float p = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) p = fmaf(kf[e], qv[gi][e], p);
#pragma unroll
                for (int off = LPR / 2; off >= 1; off >>= 1) p += __shfl_xor(p, off, WAVE);
                if (dl == 0 && row < cnt) sc[gi * chunk + row] = p * scale;
            }
        }
    }
    __syncthreads();

    // ── softmax statistics per head: max, exp, sum (reference emit_softmax order,
    //    src/graph_builder/emit_linalg.rs:509-528) ──
    for (int gi = wave; gi < G; gi += ATT_WAVES) {
        float m = -INFINITY;
        for (int n = lane; n < cnt; n += WAVE) m = fmaxf(m, sc[gi * chunk + n]);
        m = wave_max(m);
        float l = 0.f;
        for (int n = lane; n < cnt; n += WAVE) {
            const float e = expf(sc[gi * chunk + n] - m);
            sc[gi * chunk + n] = e;
            l += e;
        }
        l = wave_sum(l);
        if (lane == 0) {
            s_m[gi] = m;
            s_l[gi] = l;
        }
    }
    __syncthreads();

    // ── o = P.V ──
    float acc[G][8];
#pragma unroll
    for (int gi = 0; gi < G; gi++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[gi][e] = 0.f;

    for (int rg0 = wave; rg0 < ngroups; rg0 += ATT_WAVES * U) {
        u32x4 vv[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int row = (rg0 + u * ATT_WAVES) * RPI + sub;
            vv[u] = row < cnt ? ld128_stream(vbase + (size_t)row * HD) : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int row = (rg0 + u * ATT_WAVES) * RPI + sub;
            float vf[8];
            unpack8(vv[u], vf);
#pragma unroll
            for (int gi = 0; gi < G; gi++) {
                const float p = row < cnt ? sc[gi * chunk + row] : 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) acc[gi][e] = fmaf(p, vf[e], acc[gi][e]);
            }
        }
    }
    // fold the RPI row-subgroups of the wavefront, then the waves of the workgroup
#pragma unroll
    for (int gi = 0; gi < G; gi++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float v = acc[gi][e];
#pragma unroll
            for (int off = LPR; off < WAVE; off <<= 1) v += __shfl_xor(v, off, WAVE);
            acc[gi][e] = v;
        }
    if (sub == 0) {
#pragma unroll
        for (int gi = 0; gi < G; gi++)
#pragma unroll
            for (int e = 0; e < 8; e++) red[((size_t)wave * G + gi) * HD + dl * 8 + e] = acc[gi][e];
    }
    __syncthreads();

    const size_t pair = (size_t)b * kvh + kvhd;
    float *po = part_o + (pair * nsplit + split) * G * HD;
    float *pml = part_ml + (pair * nsplit + split) * G * 2;
    for (int i = tid; i < G * HD; i += ATT_THREADS) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < ATT_WAVES; w++) v += red[(size_t)w * G * HD + i];
        if (nsplit == 1) {
            const int gi = i / HD, d = i % HD;
            out[((size_t)b * H + kvhd * G + gi) * HD + d] = v / s_l[gi];
        } else {
            po[i] = v;
        }
    }
    if (nsplit == 1) return;
    if (tid < G) {
        pml[tid * 2] = s_m[tid];
        pml[tid * 2 + 1] = s_l[tid];
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned int prev = atomicAdd(&counters[pair], 1u);
        is_last = prev == (unsigned int)(nsplit - 1);
    }
    __syncthreads();
    if (!is_last) return;
    __threadfence();
    const float *ao = part_o + pair * nsplit * G * HD;
    const float *aml = part_ml + pair * nsplit * G * 2;
    for (int i = tid; i < G * HD; i += ATT_THREADS) {
        const int gi = i / HD, d = i % HD;
        float M = -INFINITY;
        for (int s = 0; s < nsplit; s++) M = fmaxf(M, aml[((size_t)s * G + gi) * 2]);
        float L = 0.f, O = 0.f;
        for (int s = 0; s < nsplit; s++) {
            const float wgt = expf(aml[((size_t)s * G + gi) * 2] - M);
            L = fmaf(wgt, aml[((size_t)s * G + gi) * 2 + 1], L);
            O = fmaf(wgt, ao[((size_t)s * G + gi) * HD + d], O);
        }
        out[((size_t)b * H + kvhd * G + gi) * HD + d] = O / L;
    }
    if (tid == 0) counters[pair] = 0u;
}

// KvCache::append_key / append_value (reference src/runtime.rs:521-568) with the cache in
// bf16: rows [B][kvh][n_new][hd] f32 -> cache[b][h][pos + t][:] (round to nearest even).
__global__ void kv_append_kernel(uint16_t *__restrict__ kc, uint16_t *__restrict__ vc,
                                 const float *__restrict__ k, const float *__restrict__ v,
                                 int kvh, int hd, int max_len, int pos, int n_new, size_t total) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int d = (int)(i % hd);
    size_t r = i / hd;
    const int t = (int)(r % n_new);
    r /= n_new;  // r = b * kvh + h
    const size_t dst = (r * max_len + pos + t) * hd + d;
    kc[dst] = f32_to_bf16_rne_dev(k[i]);
    vc[dst] = f32_to_bf16_rne_dev(v[i]);
}

template <int HD, int G>
int launch_attn(hm_ctx *ctx, const AttnArgs &a, int nsplit, int chunk) {
    const size_t lds = ((size_t)G * chunk + (size_t)ATT_WAVES * G * HD) * sizeof(float);
    const size_t pairs = (size_t)a.B * a.kvh;
    float *part_o = (float *)ctx->workspace;
    float *part_ml = part_o + pairs * nsplit * G * HD;
    hipLaunchKernelGGL((gqa_decode_attn_kernel<HD, G>), dim3(nsplit, a.kvh, a.B), dim3(ATT_THREADS),
                       lds, ctx->stream, a.q, a.kcache, a.vcache, a.out, part_o, part_ml,
                       ctx->counters, a.kvh, a.max_len, a.kv_len, chunk, a.scale, a.state);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

template <int HD>
int dispatch_g(hm_ctx *ctx, const AttnArgs &a, int g, int nsplit, int chunk) {
    switch (g) {
    case 1: return launch_attn<HD, 1>(ctx, a, nsplit, chunk);
    case 2: return launch_attn<HD, 2>(ctx, a, nsplit, chunk);
    case 3: return launch_attn<HD, 3>(ctx, a, nsplit, chunk);
    case 4: return launch_attn<HD, 4>(ctx, a, nsplit, chunk);
    case 5: return launch_attn<HD, 5>(ctx, a, nsplit, chunk);
    case 6: return launch_attn<HD, 6>(ctx, a, nsplit, chunk);
    case 7: return launch_attn<HD, 7>(ctx, a, nsplit, chunk);
    case 8: return launch_attn<HD, 8>(ctx, a, nsplit, chunk);
    default:
        return hm_set_error(ctx, HM_ERR_INVALID, "gqa_decode_attn: GQA group %d not in 1..8", g);
    }
}

}  // namespace

int gqa_decode_attn_launch(hm_ctx *ctx, const AttnArgs &a) {
    HM_REQUIRE(ctx, a.q && a.kcache && a.vcache && a.out, "gqa_decode_attn: NULL pointer");
    HM_REQUIRE(ctx, a.B > 0 && a.H > 0 && a.kvh > 0 && a.H % a.kvh == 0, "gqa_decode_attn: bad head counts H=%d kvh=%d", a.H, a.kvh);
    HM_REQUIRE(ctx, a.hd == 128 || a.hd == 64, "gqa_decode_attn: head_dim %d not supported (64, 128)", a.hd);
    if (!a.state) HM_REQUIRE(ctx, a.kv_len >= 1 && a.kv_len <= a.max_len, "gqa_decode_attn: kv_len=%d outside 1..max_len=%d", a.kv_len, a.max_len);
    HM_REQUIRE(ctx, ((uintptr_t)a.q % 16) == 0 && ((uintptr_t)a.kcache % 16) == 0 && ((uintptr_t)a.vcache % 16) == 0, "gqa_decode_attn: pointers must be 16-byte aligned");
    const int g = a.H / a.kvh;
    const size_t pairs = (size_t)a.B * a.kvh;
    HM_REQUIRE(ctx, pairs <= ctx->num_counters, "gqa_decode_attn: B*kvh=%zu too large", pairs);
    // Aim at ~2 workgroups per CU; a workgroup takes at least 32 rows and at most 1024.
    const int rows_step = 32;
    const int span = a.state ? a.max_len : a.kv_len;  // rows the grid has to be able to cover
    int chunk = a.fixed_chunk;
    if (chunk <= 0) {
        int want = (int)((2 * (size_t)ctx->num_cus + pairs - 1) / pairs);
        chunk = (span + want - 1) / want;
        chunk = (chunk + rows_step - 1) / rows_step * rows_step;
        if (chunk < rows_step) chunk = rows_step;
        if (chunk > 1024) chunk = 1024;
    }
    HM_REQUIRE(ctx, chunk % 16 == 0 && chunk <= 1024, "gqa_decode_attn: bad chunk %d", chunk);
    int nsplit = (span + chunk - 1) / chunk;
    const size_t ws_need = pairs * nsplit * g * (a.hd + 2) * sizeof(float);
    HM_REQUIRE(ctx, ws_need <= ctx->workspace_bytes, "gqa_decode_attn: workspace too small (%zu bytes needed)", ws_need);
    if (a.hd == 128) return dispatch_g<128>(ctx, a, g, nsplit, chunk);
    return dispatch_g<64>(ctx, a, g, nsplit, chunk);
}

extern "C" {

int hm_gqa_decode_attn(hm_ctx *ctx, const float *d_q, const uint16_t *d_kcache,
                       const uint16_t *d_vcache, float *d_out, int B, int H, int kvh, int hd,
                       int max_len, int kv_len, float scale) {
    HM_CHECK_CTX(ctx);
    AttnArgs a;
    a.q = d_q;
    a.kcache = d_kcache;
    a.vcache = d_vcache;
    a.out = d_out;
    a.B = B;
    a.H = H;
    a.kvh = kvh;
    a.hd = hd;
    a.max_len = max_len;
    a.kv_len = kv_len;
    a.scale = scale;
    return gqa_decode_attn_launch(ctx, a);
}

int hm_kv_append(hm_ctx *ctx, uint16_t *d_kcache, uint16_t *d_vcache, const float *d_k,
                 const float *d_v, int B, int kvh, int hd, int max_len, int pos, int n_new) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_kcache && d_vcache && d_k && d_v, "hm_kv_append: NULL pointer");
    HM_REQUIRE(ctx, B > 0 && kvh > 0 && hd > 0 && n_new >= 0 && pos >= 0, "hm_kv_append: bad shape");
    if (pos + n_new > max_len)
        return hm_set_error(ctx, HM_ERR_STATE, "KV cache full (%d + %d > %d)", pos, n_new, max_len);
    if (n_new == 0) return HM_OK;
    const size_t total = (size_t)B * kvh * n_new * hd;
    hipLaunchKernelGGL(kv_append_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       ctx->stream, d_kcache, d_vcache, d_k, d_v, kvh, hd, max_len, pos, n_new,
                       total);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // extern "C"
