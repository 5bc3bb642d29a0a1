// GQA decode attention over the HBM-resident bf16 KV cache, plus the cache append.
//
// One query row per sequence. The KV range is split across workgroups (flash-decode):
// grid = (splits, kv_heads, batch). A workgroup serves all G = H/kvh query heads that share
// its KV head (the reference's `h floordiv g` map, src/graph_builder/emit_linalg.rs:123-127),
// so each K/V row is read from HBM once. Rows are streamed with 16-byte loads: HD/8 lanes
// cover a row, 64/(HD/8) rows per wavefront instruction. Scores live in LDS; softmax is f32.
// Partial (o, max, sum) triples go to the workspace and a second, tiny kernel folds them per
// (batch, kv head) in split order, so the result does not depend on timing.
// Algorithmic HBM traffic: 2 * kv_len * HD * 2 bytes per (batch, kv head).
#include "attention.h"
#include "bf16_pieces.h"

namespace {

constexpr int ATT_THREADS = 256;
constexpr int ATT_WAVES = ATT_THREADS / WAVE;

__device__ __forceinline__ void unpack8(const u32x4 w, float *f) {
    f[0] = bf16_lo(w.x); f[1] = bf16_hi(w.x);
    f[2] = bf16_lo(w.y); f[3] = bf16_hi(w.y);
    f[4] = bf16_lo(w.z); f[5] = bf16_hi(w.z);
    f[6] = bf16_lo(w.w); f[7] = bf16_hi(w.w);
}

constexpr int NRG_MAX = 8;  // row groups per wavefront held in registers (K and V each)

// Optional prologue fused into the attention kernel (decode plan, batch 1): the raw q|k|v row
// produced by the QKV projection goes through the per-head QK-norm and RoPE of the reference's
// QKV kernel (src/hf/emitter.rs:629-644) here, and the workgroup that owns the last live split
// rounds the new K/V row to bf16, appends it to the cache (KvCache::append_key/append_value,
// src/runtime.rs:521-568) and uses the rounded values itself.
struct AttnFuse {
    const float *qkv_raw;   // [H*hd | kvh*hd | kvh*hd] f32
    const float *qw, *kw;   // [hd] or nullptr
    const float *cos_tab;   // [max_pos][hd]
    const float *sin_tab;
    float eps;
};

// Sum over the LPR (8 or 16) adjacent lanes that share a cache row, on the DPP path; every lane of
// the group receives the total.
template <int LPR>
__device__ __forceinline__ float row_group_sum(float v) {
    static_assert(LPR == 8 || LPR == 16, "a cache row spans 8 or 16 lanes");
    v += dpp_move<0xB1, 0xF>(v, 0.f);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E, 0xF>(v, 0.f);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141, 0xF>(v, 0.f);  // row_half_mirror
    if (LPR == 16) v += dpp_move<0x140, 0xF>(v, 0.f);  // row_mirror
    return v;
}

template <int HD, int G>
__global__ __launch_bounds__(ATT_THREADS) void gqa_decode_attn_kernel(
    const float *__restrict__ q, uint16_t *__restrict__ kcache, uint16_t *__restrict__ vcache,
    float *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml, int kvh,
    int max_len, int kv_len_arg, int chunk, float scale, const DecodeState *__restrict__ state,
    int lds_front, AttnFuse fuse, int g_total) {
    constexpr int LPR = HD / 8;      // lanes per row
    constexpr int RPI = WAVE / LPR;  // rows per wavefront instruction
    extern __shared__ float sm[];
    float *sc = sm;               // [G][chunk] scores, then probabilities; later the fold's (m,l)
    float *red = sm + lds_front;  // [ATT_WAVES * RPI][G][HD]
    __shared__ float qs[G][HD];
    __shared__ float knew[HD], vnew[HD];
    __shared__ float s_m[G], s_l[G];

    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int sub = lane / LPR, dl = lane % LPR;
    // A workgroup serves G of the g_total query heads that share a KV head (all of them when g_total <= G):
    // blockIdx.y = kv head * groups + group. Heads past g_total in the last group multiply zeros and write nothing.
    const int ngroups = (g_total + G - 1) / G;
    const int split = blockIdx.x, kvhd = blockIdx.y / ngroups, hg = blockIdx.y % ngroups, b = blockIdx.z;
    const int g0 = hg * G, g_here = min(G, g_total - g0);
    const int H = kvh * g_total;
    const int n0 = split * chunk;
    const size_t head_base = ((size_t)b * kvh + kvhd) * max_len * HD;
    const uint16_t *kbase = kcache + head_base + (size_t)n0 * HD + dl * 8;
    const uint16_t *vbase = vcache + head_base + (size_t)n0 * HD + dl * 8;
    const int nrg = chunk / (ATT_WAVES * RPI);  // row groups per wavefront (<= NRG_MAX)

    // The live length first (one scalar load): splits past it leave without touching memory.
    const int kv_len = state ? state->pos + 1 : kv_len_arg;
    const int nsplit = (kv_len + chunk - 1) / chunk;  // live splits; the grid may be larger
    if (split >= nsplit) return;
    const int cnt = min(kv_len, n0 + chunk) - n0;

    // ── every live K and V row of the chunk is requested before anything waits ──
    u32x4 kreg[NRG_MAX], vreg[NRG_MAX];
#pragma unroll
    for (int i = 0; i < NRG_MAX; i++) {
        const int row = (i * ATT_WAVES + wave) * RPI + sub;
        const bool ok = i < nrg && row < cnt;
        kreg[i] = ok ? ld128_stream(kbase + (size_t)row * HD) : u32x4{0u, 0u, 0u, 0u};
        vreg[i] = ok ? ld128_stream(vbase + (size_t)row * HD) : u32x4{0u, 0u, 0u, 0u};
    }
    const bool fused = fuse.qkv_raw != nullptr;
    const int pos = kv_len - 1;
    const bool owner = fused && split == nsplit - 1;  // this chunk holds the new row
    const int new_row = pos - n0;

    // ── queries (and, for the owner, the new K/V row) into LDS ──
    if (fused) {
        // A wavefront prepares rows t = wave, wave + 4, ... of (G query heads, new K row, new V row). Every load
        // of all its rows goes out before the first is used: with more than four rows (G > 2) a loop over the rows
        // would pay one trip to memory per turn.
        const float *c = fuse.cos_tab + (size_t)pos * HD;
        const float *sn = fuse.sin_tab + (size_t)pos * HD;
        constexpr int HALF = HD / 2, TMAX = (G + 2 + ATT_WAVES - 1) / ATT_WAVES;
        const bool on = lane < HALF;
        float rlo[TMAX], rhi[TMAX];
#pragma unroll
        for (int j = 0; j < TMAX; j++) {
            const int t = wave + j * ATT_WAVES;
            const float *src = nullptr;
            if (t < g_here) src = fuse.qkv_raw + (size_t)(kvhd * g_total + g0 + t) * HD;
            else if (owner && t == G) src = fuse.qkv_raw + (size_t)H * HD + (size_t)kvhd * HD;
            else if (owner && t == G + 1) src = fuse.qkv_raw + (size_t)(H + kvh) * HD + (size_t)kvhd * HD;
            rlo[j] = (src && on) ? src[lane] : 0.f;
            rhi[j] = (src && on) ? src[lane + HALF] : 0.f;
        }
        const float c_lo = on ? c[lane] : 0.f, c_hi = on ? c[lane + HALF] : 0.f;
        const float s_lo = on ? sn[lane] : 0.f, s_hi = on ? sn[lane + HALF] : 0.f;
        const float qw_lo = (on && fuse.qw) ? fuse.qw[lane] : 1.f, qw_hi = (on && fuse.qw) ? fuse.qw[lane + HALF] : 1.f;
        const float kw_lo = (on && fuse.kw) ? fuse.kw[lane] : 1.f, kw_hi = (on && fuse.kw) ? fuse.kw[lane + HALF] : 1.f;
        // one row: optional RMSNorm over hd, then x*cos + rotate_half(x)*sin; lane i < hd/2 owns the rotation pair
        // (i, i + hd/2)
        auto norm_rope = [&](float lo, float hi, bool norm, float w_lo, float w_hi, float &o_lo, float &o_hi) {
            if (norm) {
                const float ss = wave_sum(lo * lo + hi * hi);
                const float inv = 1.0f / sqrtf(ss / (float)HD + fuse.eps);
                lo = (lo * inv) * w_lo;
                hi = (hi * inv) * w_hi;
            }
            o_lo = lo * c_lo + (-hi) * s_lo;
            o_hi = hi * c_hi + lo * s_hi;
        };
#pragma unroll
        for (int j = 0; j < TMAX; j++) {
            const int t = wave + j * ATT_WAVES;
            if (t < G) {
                float lo, hi;
                norm_rope(rlo[j], rhi[j], fuse.qw != nullptr, qw_lo, qw_hi, lo, hi);
                if (on) {
                    qs[t][lane] = lo;
                    qs[t][lane + HALF] = hi;
                }
            } else if (owner && t == G) {
                float lo, hi;
                norm_rope(rlo[j], rhi[j], fuse.kw != nullptr, kw_lo, kw_hi, lo, hi);
                // round to bf16 exactly once; cache and this kernel use the same rounded values
                if (on) {
                    uint16_t *dst = kcache + head_base + (size_t)pos * HD;
                    const uint16_t r_lo = f32_to_bf16_rne_dev(lo), r_hi = f32_to_bf16_rne_dev(hi);
                    if (hg == 0) {  // every group rounds the row for itself, the first one appends it
                        dst[lane] = r_lo;
                        dst[lane + HALF] = r_hi;
                    }
                    knew[lane] = __uint_as_float((uint32_t)r_lo << 16);
                    knew[lane + HALF] = __uint_as_float((uint32_t)r_hi << 16);
                }
            } else if (owner && t == G + 1) {
                if (on) {
                    uint16_t *dst = vcache + head_base + (size_t)pos * HD;
                    const uint16_t r_lo = f32_to_bf16_rne_dev(rlo[j]), r_hi = f32_to_bf16_rne_dev(rhi[j]);
                    if (hg == 0) {
                        dst[lane] = r_lo;
                        dst[lane + HALF] = r_hi;
                    }
                    vnew[lane] = __uint_as_float((uint32_t)r_lo << 16);
                    vnew[lane + HALF] = __uint_as_float((uint32_t)r_hi << 16);
                }
            }
        }
    } else {
        for (int i = tid; i < G * HD; i += ATT_THREADS)
            qs[i / HD][i % HD] = i < g_here * HD ? q[((size_t)b * H + kvhd * g_total + g0) * HD + i] : 0.f;
    }
    __syncthreads();

    float qv[G][8];
#pragma unroll
    for (int gi = 0; gi < G; gi++)
#pragma unroll
        for (int e = 0; e < 8; e++) qv[gi][e] = qs[gi][dl * 8 + e];

    // ── scores = (Q.K^T) * scale; rows outside the live range (and the not-yet-written new
    //    row) are dropped here ──
#pragma unroll
    for (int i = 0; i < NRG_MAX; i++) {
        if (i < nrg) {
            const int row = (i * ATT_WAVES + wave) * RPI + sub;
            const bool live = row < cnt && !(owner && row == new_row);
            if (!live) vreg[i] = u32x4{0u, 0u, 0u, 0u};  // the new row's slot is not written yet
            float kf[8];
            unpack8(kreg[i], kf);
#pragma unroll
            for (int gi = 0; gi < G; gi++) {
                float p = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) p = fmaf(kf[e], qv[gi][e], p);
                p = row_group_sum<LPR>(p);
                if (dl == 0 && live) sc[gi * chunk + row] = p * scale;
            }
        }
    }
    if (owner && wave == 0) {  // the new row's score from the rounded values in LDS
#pragma unroll
        for (int gi = 0; gi < G; gi++) {
            float p = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) p = fmaf(knew[dl * 8 + e], qv[gi][e], p);
            p = row_group_sum<LPR>(p);
            if (lane == 0) sc[gi * chunk + new_row] = p * scale;
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
#pragma unroll
    for (int i = 0; i < NRG_MAX; i++) {
        if (i < nrg) {
            const int row = (i * ATT_WAVES + wave) * RPI + sub;
            float vf[8];
            unpack8(vreg[i], vf);
#pragma unroll
            for (int gi = 0; gi < G; gi++) {
                const float p = row < cnt ? sc[gi * chunk + row] : 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) acc[gi][e] = fmaf(p, vf[e], acc[gi][e]);
            }
        }
    }
    if (owner && wave == 0 && sub == 0) {
#pragma unroll
        for (int gi = 0; gi < G; gi++) {
            const float p = sc[gi * chunk + new_row];
#pragma unroll
            for (int e = 0; e < 8; e++) acc[gi][e] = fmaf(p, vnew[dl * 8 + e], acc[gi][e]);
        }
    }
    // every row-subgroup of every wavefront leaves its partial in LDS; summed below
#pragma unroll
    for (int gi = 0; gi < G; gi++) {
        float *dst = red + ((size_t)(wave * RPI + sub) * G + gi) * HD + dl * 8;
        *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[gi][0], acc[gi][1], acc[gi][2], acc[gi][3]};
        *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{acc[gi][4], acc[gi][5], acc[gi][6], acc[gi][7]};
    }
    __syncthreads();

    const size_t pair = (size_t)b * kvh + kvhd;
    float *po = part_o + ((pair * nsplit + split) * g_total + g0) * HD;
    float *pml = part_ml + ((pair * nsplit + split) * g_total + g0) * 2;
    for (int i = tid; i < g_here * HD; i += ATT_THREADS) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < ATT_WAVES * RPI; w++) v += red[(size_t)w * G * HD + i];
        if (nsplit == 1) {
            const int gi = i / HD, d = i % HD;
            out[((size_t)b * H + kvhd * g_total + g0 + gi) * HD + d] = v / s_l[gi];
        } else {
            po[i] = v;
        }
    }
    if (nsplit == 1) return;
    if (tid < g_here) {
        pml[tid * 2] = s_m[tid];
        pml[tid * 2 + 1] = s_l[tid];
    }
}

// Long caches (more rows per workgroup than fit in registers at once): the workgroup walks its rows in
// steps of 128, a wavefront owning 32 rows of a step from the scores to P.V with its own softmax reference
// point (nothing inside a step waits for another wavefront; the four wavefronts' results are brought to a
// common maximum once, at the end). Both products run on the matrix cores (v_mfma_f32_16x16x32_bf16):
//  * Q.K^T, contraction over the head dimension: 16 cache rows straight from memory are the A operand (lane
//    r + 16 c holds dims 32 s + 8 c .. + 7 of row r, one 16-byte load), the G query heads, scaled and split
//    into two bf16 pieces (2^-17 of an element left out), are columns of B. Lane h + 16 c receives head h,
//    rows 4 c .. 4 c + 3 of the tile.
//  * P.V, contraction over the 32 rows: contraction slot 4 t + i of lane group c stands for row 16 t + 4 c + i,
//    which is exactly where the scores of the two 16-row tiles t already sit, so the probabilities (two bf16
//    pieces) are the A operand without leaving their lanes. V needs rows along the contraction: lane d + 16 c
//    loads dims 8 d .. 8 d + 7 of its group's eight rows (eight 16-byte loads, 256 contiguous bytes per row and
//    instruction) and transposes the 8 x 8 block in its registers with byte permutes; matrix e of the eight
//    takes dim 8 d + e as column d. The output lane d + 16 c holds heads 4 c .. 4 c + 3 at dim 8 d + e.
// The reference point of a head only moves when a score exceeds it by more than LAZY (the exponentials stay
// below e^LAZY), so the accumulators are rarely rescaled. Partials leave in the same (o, max, sum) form as the
// kernel above, the "max" being the reference point.
constexpr int IT_ROWS = 128;  // rows per step: 32 per wavefront
constexpr float LAZY = 8.0f;

template <int HD, int G>
__global__ __launch_bounds__(ATT_THREADS) void gqa_decode_attn_stream_kernel(
    const float *__restrict__ q, const uint16_t *__restrict__ kcache,
    const uint16_t *__restrict__ vcache, float *__restrict__ out, float *__restrict__ part_o,
    float *__restrict__ part_ml, int kvh, int max_len, int kv_len, int chunk, float scale) {
    constexpr int KS = HD / 32;  // k steps of the score MFMA
    constexpr int DS = HD / 8;   // 8-dim slices of a row
    static_assert(IT_ROWS == 32 * ATT_WAVES, "32 rows per wavefront and step");
    static_assert(G <= 8, "heads 4 c + i of lane group c < 2");
    __shared__ __attribute__((aligned(16))) float red[ATT_WAVES][G][HD];
    __shared__ float qs[G][HD];
    __shared__ float s_m[G], s_l[G];
    __shared__ float s_mw[ATT_WAVES][G], s_lw[ATT_WAVES][G];

    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int l16 = lane & 15, kg = lane >> 4;
    const int split = blockIdx.x, nsplit = gridDim.x, kvhd = blockIdx.y, b = blockIdx.z;
    const int H = kvh * G;
    const int n0 = split * chunk;
    const size_t head_base = ((size_t)b * kvh + kvhd) * max_len * HD;
    const uint16_t *kbase = kcache + head_base + (size_t)n0 * HD + kg * 8;
    const uint16_t *vbase = vcache + head_base + (size_t)n0 * HD + (l16 < DS ? l16 : 0) * 8;
    const int cnt = min(kv_len, n0 + chunk) - n0;  // >= 1: the grid covers kv_len exactly
    const int iters = (cnt + IT_ROWS - 1) / IT_ROWS;

    // Rows past the live range are clamped to the last live row instead of masked: every request issues
    // the same number of loads, so the waits can leave the next step's loads in flight. Their scores become
    // -inf below, hence their probabilities zero, and the clamped V rows are finite.
    // One set of row registers: the next step's K rows are asked for as soon as this step's scores are out of
    // the matrix cores, its V rows as soon as this step's P.V is. (A second set with two steps in flight was
    // slower, alone on a CU or not.)
    u32x4 kr0[2][KS], vr0[8];
    auto request_k = [&](u32x4(&kr)[2][KS], int it) {
        const int base = it * IT_ROWS + 32 * wave;
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const int krow = min(base + 16 * t + l16, cnt - 1);
#pragma unroll
            for (int s = 0; s < KS; s++) kr[t][s] = ld128_stream(kbase + (size_t)krow * HD + 32 * s);
        }
    };
    auto request_v = [&](u32x4(&vr)[8], int it) {
        const int base = it * IT_ROWS + 32 * wave;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int row = min(base + 16 * (j / 4) + 4 * kg + (j % 4), cnt - 1);
            vr[j] = ld128_stream(vbase + (size_t)row * HD);
        }
    };
    // the queries are asked for first: loads return in order, and the operand below is built while the rows arrive
    float qv[(G * HD + ATT_THREADS - 1) / ATT_THREADS];
#pragma unroll
    for (int u = 0; u < (G * HD + ATT_THREADS - 1) / ATT_THREADS; u++) {
        const int i = tid + u * ATT_THREADS;
        qv[u] = i < G * HD ? q[((size_t)b * H + kvhd * G) * HD + i] : 0.f;
    }
    request_k(kr0, 0);
    request_v(vr0, 0);
#pragma unroll
    for (int u = 0; u < (G * HD + ATT_THREADS - 1) / ATT_THREADS; u++) {
        const int i = tid + u * ATT_THREADS;
        if (i < G * HD) qs[i / HD][i % HD] = qv[u];
    }
    __syncthreads();
    // B operand of the scores: column l16 is query head l16 (columns past G are zero), scaled, as two pieces
    bf16x8 qop[KS][2];
#pragma unroll
    for (int s = 0; s < KS; s++) {
        float f[8];
#pragma unroll
        for (int e = 0; e < 8; e++) f[e] = l16 < G ? qs[l16 < G ? l16 : 0][32 * s + 8 * kg + e] * scale : 0.f;
        split8<2>(f, qop[s]);
    }

    f32x4 acc[8];  // matrix e: heads 4 kg .. 4 kg + 3 at dim 8 l16 + e
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    // Softmax state of head l16 over this wavefront's rows so far (the four lanes that share an l16 agree;
    // lanes with l16 >= G carry nothing).
    float m_run = -INFINITY, l_run = 0.f;

    bf16x8 pop[2];  // this step's probabilities as the A operand of P.V, two pieces
    auto scores = [&](u32x4(&kr)[2][KS], int it) {
        f32x4 c[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            c[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const bf16x8 kop = __builtin_bit_cast(bf16x8, kr[t][s]);
                c[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, qop[s][1], c[t], 0, 0, 0);  // the small piece first
                c[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, qop[s][0], c[t], 0, 0, 0);
            }
        }
        const int r0 = it * IT_ROWS + 32 * wave + 4 * kg;
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (r0 + 16 * t + i >= cnt) c[t][i] = -INFINITY;
                mx = fmaxf(mx, c[t][i]);
            }
        // the head's maximum over the 32 rows: eight in this lane, the rest in the lanes 16, 32, 48 on
        mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
        // move the reference point only when it has to move (first live row, or a score LAZY above it)
        const bool move = mx > m_run + LAZY || (m_run == -INFINITY && mx > -INFINITY);
        if (__any(move && l16 < G)) {
            const float m_new = move ? mx : m_run;
            const float f = m_run == -INFINITY ? 0.f : expf(m_run - m_new);  // 1 where the point stays
            l_run *= f;
            m_run = m_new;
            float fh[8];  // factor of head j: held by the lanes with l16 == j
#pragma unroll
            for (int j = 0; j < 8; j++) fh[j] = j < G ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), j)) : 1.f;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float fi = kg == 0 ? fh[i] : fh[4 + i];
#pragma unroll
                for (int e = 0; e < 8; e++) acc[e][i] *= fi;
            }
        }
        const float m_ref = m_run == -INFINITY ? 0.f : m_run;  // no live row yet: everything below becomes 0
        float p[8];
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                p[4 * t + i] = expf(c[t][i] - m_ref);
                psum += p[4 * t + i];
            }
        psum += __shfl_xor(psum, 16, WAVE);
        psum += __shfl_xor(psum, 32, WAVE);
        l_run += psum;
        split8<2>(p, pop);
    };
    auto multiply_v = [&](u32x4(&vr)[8]) {
        // V^T: the 8 (rows) x 8 (dims) block of this lane, transposed in registers
#pragma unroll
        for (int e = 0; e < 8; e++) {
            u32x4 tv;
#pragma unroll
            for (int qd = 0; qd < 4; qd++)
                tv[qd] = __builtin_amdgcn_perm(vr[2 * qd + 1][e / 2], vr[2 * qd][e / 2], (e & 1) ? 0x07060302u : 0x05040100u);
            if (l16 >= DS) tv = u32x4{0u, 0u, 0u, 0u};
            const bf16x8 vop = __builtin_bit_cast(bf16x8, tv);
            acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pop[1], vop, acc[e], 0, 0, 0);
            acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pop[0], vop, acc[e], 0, 0, 0);
        }
    };
    int it = 0;
    for (; it + 1 < iters; it++) {
        scores(kr0, it);
        request_k(kr0, it + 1);
        multiply_v(vr0);
        request_v(vr0, it + 1);
    }
    scores(kr0, it);
    multiply_v(vr0);

    // the four wavefronts' results to a common reference point per head
    if (kg == 0 && l16 < G) {
        s_mw[wave][l16] = m_run;
        s_lw[wave][l16] = l_run;
    }
    __syncthreads();
    if (tid < G) {
        float M = s_mw[0][tid];
        for (int w = 1; w < ATT_WAVES; w++) M = fmaxf(M, s_mw[w][tid]);  // finite: row 0 of the split is live
        float L = 0.f;
        for (int w = 0; w < ATT_WAVES; w++) L = fmaf(s_lw[w][tid], expf(s_mw[w][tid] - M), L);
        s_m[tid] = M;
        s_l[tid] = L;
    }
    if (kg < 2) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int gi = 4 * kg + i;
            if (gi < G && l16 < DS) {
                float M = s_mw[0][gi];
                for (int w = 1; w < ATT_WAVES; w++) M = fmaxf(M, s_mw[w][gi]);
                const float sc_w = expf(s_mw[wave][gi] - M);
                float *dst = &red[wave][gi][8 * l16];
                *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[0][i] * sc_w, acc[1][i] * sc_w, acc[2][i] * sc_w, acc[3][i] * sc_w};
                *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{acc[4][i] * sc_w, acc[5][i] * sc_w, acc[6][i] * sc_w, acc[7][i] * sc_w};
            }
        }
    }
    __syncthreads();

    const size_t pair = (size_t)b * kvh + kvhd;
    float *po = part_o + (pair * nsplit + split) * G * HD;
    float *pml = part_ml + (pair * nsplit + split) * G * 2;
    for (int i = tid; i < G * HD; i += ATT_THREADS) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < ATT_WAVES; w++) v += (&red[w][0][0])[i];
        if (nsplit == 1) {
            const int gi = i / HD, d = i % HD;
            out[((size_t)b * H + kvhd * G + gi) * HD + d] = v / s_l[gi];
        } else {
            po[i] = v;
        }
    }
    if (nsplit > 1 && tid < G) {
        pml[tid * 2] = s_m[tid];
        pml[tid * 2 + 1] = s_l[tid];
    }
}

// Second half of the split attention: one workgroup per (batch, query head) folds that head's partial
// (o, max, sum) triples. A separate launch instead of a "last workgroup to arrive" fold: the kernel boundary
// orders the partial writes, so no device-scope fence (a full L2 write-back + invalidate on this chip) is needed.
// The workgroup is SG groups of HD threads (thread = output element d of group sg). Group sg takes splits sg,
// sg + SG, ... in ascending order against the maximum of its own splits, up to 32 loads a thread in flight; the
// groups' (max, sum, o) then meet in LDS and are merged in group order. One group (grids of at most 32 splits) is the
// plain ascending fold; a grid of hundreds of splits (tens of thousands of cached rows) folded by one group took
// 57 us, longer than the attention itself.
constexpr int FOLD_BATCH = 32;      // splits fetched per batch, all loads of a batch in flight together
constexpr int FOLD_THREADS = 1024;  // of a workgroup with groups

// GROUPS false: one group of HD threads (grids of at most FOLD_BATCH splits: a workgroup of 1024 threads costs about
// 2 us more to start than one of 64 or 128). GROUPS true: FOLD_THREADS / HD groups; with few splits live (a grid
// sized for a long cache with few rows in it yet) one group folds and the others leave at once.
template <int HD, int G, bool GROUPS>
__global__ __launch_bounds__(GROUPS ? FOLD_THREADS : HD) void gqa_decode_fold_kernel(
    float *__restrict__ out, const float *__restrict__ part_o, const float *__restrict__ part_ml,
    int kvh, int kv_len_arg, int chunk, const DecodeState *__restrict__ state) {
    constexpr int SGMAX = GROUPS ? FOLD_THREADS / HD : 1;
    extern __shared__ float s_fold[];  // [SGMAX][HD + 2] group results, then [nsplit][2] (max, sum) of this head
    const int d = GROUPS ? threadIdx.x % HD : threadIdx.x, sg = GROUPS ? threadIdx.x / HD : 0;
    float *s_grp = s_fold, *s_ml = s_fold + SGMAX * (HD + 2);
    const int gi = blockIdx.x % G, kvhd = blockIdx.x / G, b = blockIdx.y;
    const int H = kvh * G;
    const int kv_len = state ? state->pos + 1 : kv_len_arg;
    const int nsplit = (kv_len + chunk - 1) / chunk;
    if (nsplit == 1) return;  // the attention kernel wrote the final result itself
    const int SG = GROUPS && nsplit > FOLD_BATCH / 2 ? SGMAX : 1;
    if (sg >= SG) return;
    const size_t pair = (size_t)b * kvh + kvhd;
    const float *ao = part_o + (pair * nsplit * G + gi) * HD + d;
    const float *aml = part_ml + (pair * nsplit * G + gi) * 2;
    constexpr int FB = FOLD_BATCH;
    float o[FB];
#pragma unroll
    for (int u = 0; u < FB; u++) {
        const int sp = sg + u * SG;
        o[u] = sp < nsplit ? ao[(size_t)sp * G * HD] : 0.f;
    }
    for (int i = threadIdx.x; i < nsplit * 2; i += SG * HD) s_ml[i] = aml[(size_t)(i >> 1) * G * 2 + (i & 1)];
    __syncthreads();
    float M = -INFINITY;
    for (int sp = sg; sp < nsplit; sp += SG) M = fmaxf(M, s_ml[sp * 2]);
    float L = 0.f, O = 0.f;
    for (int u0 = 0; sg + u0 * SG < nsplit; u0 += FB) {
        if (u0 > 0) {
#pragma unroll
            for (int u = 0; u < FB; u++) {
                const int sp = sg + (u0 + u) * SG;
                o[u] = sp < nsplit ? ao[(size_t)sp * G * HD] : 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < FB; u++) {
            const int sp = sg + (u0 + u) * SG;
            if (sp < nsplit) {
                const float wgt = expf(s_ml[sp * 2] - M);
                L = fmaf(wgt, s_ml[sp * 2 + 1], L);
                O = fmaf(wgt, o[u], O);
            }
        }
    }
    float *res = out + ((size_t)b * H + kvhd * G + gi) * HD + d;
    if (SG == 1) {
        *res = O / L;
        return;
    }
    s_grp[sg * (HD + 2) + d] = O;
    if (d == 0) {
        s_grp[sg * (HD + 2) + HD] = M;
        s_grp[sg * (HD + 2) + HD + 1] = L;
    }
    __syncthreads();
    if (sg != 0) return;
    float Mt = -INFINITY;
    for (int g = 0; g < SG; g++) Mt = fmaxf(Mt, s_grp[g * (HD + 2) + HD]);
    float Lt = 0.f, Ot = 0.f;
    for (int g = 0; g < SG; g++) {
        const float mg = s_grp[g * (HD + 2) + HD];
        if (mg == -INFINITY) continue;  // a group without splits
        const float wgt = expf(mg - Mt);
        Lt = fmaf(wgt, s_grp[g * (HD + 2) + HD + 1], Lt);
        Ot = fmaf(wgt, s_grp[g * (HD + 2) + d], Ot);
    }
    *res = Ot / Lt;
}

// nsplit: the grid's split count (what a call can ever have live)
template <int HD, int G>
int launch_fold(hm_ctx *ctx, const AttnArgs &a, const float *part_o, const float *part_ml, int nsplit, int chunk,
                const DecodeState *state) {
    const bool groups = nsplit > FOLD_BATCH;
    const int sg = groups ? FOLD_THREADS / HD : 1;
    const size_t fold_lds = ((size_t)sg * (HD + 2) + (size_t)nsplit * 2) * sizeof(float);
    HM_REQUIRE(ctx, fold_lds <= 64 * 1024, "gqa_decode_attn: too many splits (%d)", nsplit);
    if (groups)
        hipLaunchKernelGGL((gqa_decode_fold_kernel<HD, G, true>), dim3(a.kvh * G, a.B), dim3(FOLD_THREADS), fold_lds,
                           ctx->stream, a.out, part_o, part_ml, a.kvh, a.kv_len, chunk, state);
    else
        hipLaunchKernelGGL((gqa_decode_fold_kernel<HD, G, false>), dim3(a.kvh * G, a.B), dim3(HD), fold_lds, ctx->stream,
                           a.out, part_o, part_ml, a.kvh, a.kv_len, chunk, state);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
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

// G = the query heads that share a KV head. A workgroup of the split kernel serves GB of them: all when there are
// at most four, else two (the kernel's length grows with the heads it serves, and with two KV heads a 1024-row
// cache gives only 32 workgroups of all heads; groups of three or four measured slower than two at G = 6 .. 8,
// single heads slower again).
template <int HD, int G>
int launch_attn(hm_ctx *ctx, const AttnArgs &a, int nsplit, int chunk) {
    constexpr int GB = G <= 4 ? G : 2, NG = (G + GB - 1) / GB;
    // scores [GB][chunk] + partials of every row-subgroup of every wavefront [4 * RPI][GB][HD]
    const size_t front = (size_t)GB * chunk;
    const size_t lds = (front + (size_t)ATT_WAVES * (WAVE / (HD / 8)) * GB * HD) * sizeof(float);
    const size_t pairs = (size_t)a.B * a.kvh;
    float *part_o = a.partials ? a.partials : (float *)ctx->workspace;
    float *part_ml = part_o + pairs * nsplit * G * HD;
    AttnFuse f{a.qkv_raw, a.qw, a.kw, a.cos_tab, a.sin_tab, a.eps};
    if (a.phase != AttnArgs::FOLD_ONLY) {
        static bool lds_limit_raised = false;  // per instantiation; large groups need more than 64 KiB
        if (lds > 64 * 1024 && !lds_limit_raised) {
            HM_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(&gqa_decode_attn_kernel<HD, GB>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
            lds_limit_raised = true;
        }
        HM_REQUIRE(ctx, lds <= 96 * 1024, "gqa_decode_attn: LDS need %zu too large", lds);
        hipLaunchKernelGGL((gqa_decode_attn_kernel<HD, GB>), dim3(nsplit, a.kvh * NG, a.B), dim3(ATT_THREADS),
                           lds, ctx->stream, a.q, const_cast<uint16_t *>(a.kcache),
                           const_cast<uint16_t *>(a.vcache), a.out, part_o, part_ml, a.kvh, a.max_len,
                           a.kv_len, chunk, a.scale, a.state, (int)front, f, G);
        HM_LAUNCH_CHECK(ctx);
    }
    // nsplit is the grid's split count: 1 means no call can ever need a fold
    if (nsplit > 1 && a.phase != AttnArgs::SPLIT_ONLY) {
        const int rc = launch_fold<HD, G>(ctx, a, part_o, part_ml, nsplit, chunk, a.state);
        if (rc != HM_OK) return rc;
    }
    return HM_OK;
}

// Long caches through the stepping kernel; its partials go through the same fold.
template <int HD, int G>
int launch_attn_stream(hm_ctx *ctx, const AttnArgs &a, int nsplit, int chunk) {
    const size_t pairs = (size_t)a.B * a.kvh;
    float *part_o = a.partials ? a.partials : (float *)ctx->workspace;
    float *part_ml = part_o + pairs * nsplit * G * HD;
    HM_REQUIRE(ctx, chunk % IT_ROWS == 0, "gqa_decode_attn: chunk %d must be a multiple of %d", chunk, IT_ROWS);
    hipLaunchKernelGGL((gqa_decode_attn_stream_kernel<HD, G>), dim3(nsplit, a.kvh, a.B),
                       dim3(ATT_THREADS), 0, ctx->stream, a.q, a.kcache, a.vcache, a.out, part_o,
                       part_ml, a.kvh, a.max_len, a.kv_len, chunk, a.scale);
    HM_LAUNCH_CHECK(ctx);
    if (nsplit > 1) {
        const int rc = launch_fold<HD, G>(ctx, a, part_o, part_ml, nsplit, chunk, (const DecodeState *)nullptr);
        if (rc != HM_OK) return rc;
    }
    return HM_OK;
}

template <int HD>
int dispatch_g(hm_ctx *ctx, const AttnArgs &a, int g, int nsplit, int chunk, bool stepping) {
    if (stepping) {
        switch (g) {
        case 1: return launch_attn_stream<HD, 1>(ctx, a, nsplit, chunk);
        case 2: return launch_attn_stream<HD, 2>(ctx, a, nsplit, chunk);
        case 3: return launch_attn_stream<HD, 3>(ctx, a, nsplit, chunk);
        case 4: return launch_attn_stream<HD, 4>(ctx, a, nsplit, chunk);
        case 5: return launch_attn_stream<HD, 5>(ctx, a, nsplit, chunk);
        case 6: return launch_attn_stream<HD, 6>(ctx, a, nsplit, chunk);
        case 7: return launch_attn_stream<HD, 7>(ctx, a, nsplit, chunk);
        case 8: return launch_attn_stream<HD, 8>(ctx, a, nsplit, chunk);
        default: break;
        }
    }
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

// Partial results of hm_gqa_decode_attn_noalloc. In host code this name is only a handle for
// hipGetSymbolAddress; kernels get the address that call returns. Every GPU the library runs on
// holds its own copy until the process ends.
constexpr size_t FIXED_SCRATCH_BYTES = (size_t)4 << 20;
static __device__ __align__(256) unsigned char fixed_scratch[FIXED_SCRATCH_BYTES];

}  // namespace

int gqa_attn_fixed_scratch_setup(hm_ctx *ctx) {
    void *p = nullptr;
    HM_HIP(ctx, hipGetSymbolAddress(&p, HIP_SYMBOL(fixed_scratch)));
    HM_REQUIRE(ctx, p != nullptr, "gqa_decode_attn: the fixed partials array has no device address");
    ctx->attn_fixed_scratch = p;
    return HM_OK;
}

int gqa_decode_attn_launch(hm_ctx *ctx, const AttnArgs &a) {
    HM_REQUIRE(ctx, a.kcache && a.vcache && a.out, "gqa_decode_attn: NULL pointer");
    HM_REQUIRE(ctx, a.B > 0 && a.H > 0 && a.kvh > 0 && a.H % a.kvh == 0, "gqa_decode_attn: bad head counts H=%d kvh=%d", a.H, a.kvh);
    HM_REQUIRE(ctx, a.hd == 128 || a.hd == 64, "gqa_decode_attn: head_dim %d not supported (64, 128)", a.hd);
    if (!a.state) HM_REQUIRE(ctx, a.kv_len >= 1 && a.kv_len <= a.max_len, "gqa_decode_attn: kv_len=%d outside 1..max_len=%d", a.kv_len, a.max_len);
    HM_REQUIRE(ctx, ((uintptr_t)a.kcache % 16) == 0 && ((uintptr_t)a.vcache % 16) == 0, "gqa_decode_attn: caches must be 16-byte aligned");
    const int g = a.H / a.kvh;
    const size_t pairs = (size_t)a.B * a.kvh;
    const size_t ws_have = a.partials ? a.partials_bytes : ctx->workspace_bytes;
    // A workgroup keeps its whole chunk in registers: 32..128 rows. Aim at about one workgroup
    // per CU over the rows that can be live.
    const int rows_step = 32;
    // rows the grid has to be able to cover
    const int span = a.state ? (a.span > 0 && a.span < a.max_len ? a.span : a.max_len) : a.kv_len;
    int chunk = a.fixed_chunk;
    bool stepping = false;
    if (chunk <= 0) {
        int want = (int)(((size_t)ctx->num_cus + pairs - 1) / pairs);
        chunk = (span + want - 1) / want;
        chunk = (chunk + rows_step - 1) / rows_step * rows_step;
        // More rows per workgroup than its registers hold: the stepping kernel (plain calls only; the decode
        // plan's fused prologue lives in the other kernel). One workgroup a CU while that keeps a workgroup's
        // walk at four steps or fewer (fewer partial results, a shorter fold), else two.
        if (chunk > 128 && !a.state && !a.qkv_raw) {
            const int it_rows = IT_ROWS;
            chunk = (chunk + it_rows - 1) / it_rows * it_rows;
            stepping = true;
            if (chunk > 4 * it_rows) {
                want = (int)(((size_t)2 * ctx->num_cus + pairs - 1) / pairs);
                chunk = (span + want - 1) / want;
                chunk = (chunk + it_rows - 1) / it_rows * it_rows;
            }
        }
    }
    if (stepping) {
        HM_REQUIRE(ctx, a.q != nullptr, "gqa_decode_attn: NULL query");
        const int nsplit = (a.kv_len + chunk - 1) / chunk;
        const size_t ws_need = pairs * nsplit * g * (a.hd + 2) * sizeof(float);
        HM_REQUIRE(ctx, ws_need <= ws_have, "gqa_decode_attn: %zu bytes of partial results exceed the %zu available", ws_need, ws_have);
        if (a.hd == 128) return dispatch_g<128>(ctx, a, g, nsplit, chunk, stepping);
        return dispatch_g<64>(ctx, a, g, nsplit, chunk, stepping);
    }
    if (chunk < rows_step) chunk = rows_step;
    if (chunk > 128) chunk = 128;
    HM_REQUIRE(ctx, chunk % rows_step == 0, "gqa_decode_attn: chunk %d must be a multiple of 32", chunk);
    if (a.qkv_raw) {
        HM_REQUIRE(ctx, a.B == 1 && a.state && a.cos_tab && a.sin_tab, "gqa_decode_attn: the fused prologue needs batch 1, a decode cursor and RoPE tables");
        HM_REQUIRE(ctx, (a.qw == nullptr) == (a.kw == nullptr), "gqa_decode_attn: q and k norm weights must come together");
    } else {
        HM_REQUIRE(ctx, a.q != nullptr, "gqa_decode_attn: NULL query");
    }
    int nsplit = (span + chunk - 1) / chunk;
    const size_t ws_need = pairs * nsplit * g * (a.hd + 2) * sizeof(float);
    HM_REQUIRE(ctx, ws_need <= ws_have, "gqa_decode_attn: %zu bytes of partial results exceed the %zu available", ws_need, ws_have);
    if (a.hd == 128) return dispatch_g<128>(ctx, a, g, nsplit, chunk, false);
    return dispatch_g<64>(ctx, a, g, nsplit, chunk, false);
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

int hm_gqa_decode_attn_noalloc(hm_ctx *ctx, const float *d_q, const uint16_t *d_kcache,
                               const uint16_t *d_vcache, float *d_out, int B, int H, int kvh, int hd,
                               int max_len, int kv_len, float scale) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, ctx->attn_fixed_scratch != nullptr, "hm_gqa_decode_attn_noalloc: the fixed partials array was not set up");
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
    a.partials = (float *)ctx->attn_fixed_scratch;
    a.partials_bytes = FIXED_SCRATCH_BYTES;
    return gqa_decode_attn_launch(ctx, a);
}

size_t hm_gqa_decode_attn_noalloc_limit(void) { return FIXED_SCRATCH_BYTES; }

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
