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

// One wavefront: optional RMSNorm over hd, then x*cos + rotate_half(x)*sin; lane i < hd/2 owns
// the rotation pair (i, i + hd/2) and gets its two results back in (o_lo, o_hi).
template <int HD>
__device__ __forceinline__ void norm_rope_row(const float *__restrict__ src,
                                              const float *__restrict__ nw,
                                              const float *__restrict__ c,
                                              const float *__restrict__ sn, float eps, int lane,
                                              float &o_lo, float &o_hi) {
    constexpr int HALF = HD / 2;
    const bool on = lane < HALF;
    float lo = on ? src[lane] : 0.f, hi = on ? src[lane + HALF] : 0.f;
    const float c_lo = on ? c[lane] : 0.f, c_hi = on ? c[lane + HALF] : 0.f;
    const float s_lo = on ? sn[lane] : 0.f, s_hi = on ? sn[lane + HALF] : 0.f;
    const float w_lo = (on && nw) ? nw[lane] : 1.f, w_hi = (on && nw) ? nw[lane + HALF] : 1.f;
    if (nw) {
        const float ss = wave_sum(lo * lo + hi * hi);
        const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
        lo = (lo * inv) * w_lo;
        hi = (hi * inv) * w_hi;
    }
    o_lo = lo * c_lo + (-hi) * s_lo;
    o_hi = hi * c_hi + lo * s_hi;
}

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
    int lds_front, AttnFuse fuse) {
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
    const int split = blockIdx.x, kvhd = blockIdx.y, b = blockIdx.z;
    const int H = kvh * G;
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
        const float *c = fuse.cos_tab + (size_t)pos * HD;
        const float *sn = fuse.sin_tab + (size_t)pos * HD;
        constexpr int HALF = HD / 2;
        for (int t = wave; t < G + 2; t += ATT_WAVES) {
            if (t < G) {
                float lo, hi;
                norm_rope_row<HD>(fuse.qkv_raw + (size_t)(kvhd * G + t) * HD, fuse.qw, c, sn, fuse.eps,
                                  lane, lo, hi);
                if (lane < HALF) {
                    qs[t][lane] = lo;
                    qs[t][lane + HALF] = hi;
                }
            } else if (owner && t == G) {
                float lo, hi;
                norm_rope_row<HD>(fuse.qkv_raw + (size_t)H * HD + (size_t)kvhd * HD, fuse.kw, c, sn,
                                  fuse.eps, lane, lo, hi);
                // round to bf16 exactly once; cache and this kernel use the same rounded values
                if (lane < HALF) {
                    uint16_t *dst = kcache + head_base + (size_t)pos * HD;
                    const uint16_t r_lo = f32_to_bf16_rne_dev(lo), r_hi = f32_to_bf16_rne_dev(hi);
                    dst[lane] = r_lo;
                    dst[lane + HALF] = r_hi;
                    knew[lane] = __uint_as_float((uint32_t)r_lo << 16);
                    knew[lane + HALF] = __uint_as_float((uint32_t)r_hi << 16);
                }
            } else if (owner && t == G + 1) {
                const float *src = fuse.qkv_raw + (size_t)(H + kvh) * HD + (size_t)kvhd * HD;
                uint16_t *dst = vcache + head_base + (size_t)pos * HD;
                for (int i = lane; i < HD; i += WAVE) {
                    const uint16_t r = f32_to_bf16_rne_dev(src[i]);
                    dst[i] = r;
                    vnew[i] = __uint_as_float((uint32_t)r << 16);
                }
            }
        }
    } else {
        for (int i = tid; i < G * HD; i += ATT_THREADS)
            qs[i / HD][i % HD] = q[((size_t)b * H + kvhd * G) * HD + i];
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
    float *po = part_o + (pair * nsplit + split) * G * HD;
    float *pml = part_ml + (pair * nsplit + split) * G * 2;
    for (int i = tid; i < G * HD; i += ATT_THREADS) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < ATT_WAVES * RPI; w++) v += red[(size_t)w * G * HD + i];
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
}

// Long caches (more rows per workgroup than fit in registers at once): the workgroup walks its
// rows in steps of 64. The loads of step i + 1 are in flight while step i is multiplied, the
// softmax reference point is the running maximum (sums and the output accumulators are rescaled
// when it moves), and scores and rescale factors alternate between two LDS slots so a step needs
// two barriers. Q.K^T runs on the matrix cores: v_mfma_f32_16x16x32_bf16 takes 16 cache rows
// straight from memory as its A operand (lane r + 16 c holds dims 32 s + 8 c .. + 7 of row r, one
// 16-byte load) and the G query heads, scaled and split into two bf16 pieces, as columns of B;
// what the pieces leave out is 2^-17 of a query element. P.V stays on the vector ALUs (V would have
// to be transposed for the matrix cores, which costs more than the multiply for so few heads).
// Partials leave in the same (o, max, sum) form as the kernel above.
constexpr int IT_ROWS = 64;  // rows per step: 16 per wavefront for Q.K^T

template <int HD, int G>
__global__ __launch_bounds__(ATT_THREADS) void gqa_decode_attn_stream_kernel(
    const float *__restrict__ q, const uint16_t *__restrict__ kcache,
    const uint16_t *__restrict__ vcache, float *__restrict__ out, float *__restrict__ part_o,
    float *__restrict__ part_ml, int kvh, int max_len, int kv_len, int chunk, float scale,
    int lds_front) {
    constexpr int LPR = HD / 8, RPI = WAVE / LPR;
    constexpr int NRG_V = IT_ROWS / (ATT_WAVES * RPI);      // V row groups per wavefront and step
    constexpr int KS = HD / 32;                             // k steps of the score MFMA
    constexpr int SLOTS = (G + ATT_WAVES - 1) / ATT_WAVES;  // heads whose statistics a wavefront keeps
    static_assert(IT_ROWS == WAVE && IT_ROWS == 16 * ATT_WAVES, "one score per lane; 16 rows per wavefront");
    static_assert(G <= 16, "heads are columns of a 16-wide MFMA tile");
    extern __shared__ __attribute__((aligned(16))) float sm[];
    float *sc = sm;                      // [2][G][IT_ROWS] scores, then probabilities
    float *fac = sm + 2 * G * IT_ROWS;   // [2][G] rescale factor of the step
    float *red = sm + lds_front;         // [ATT_WAVES * RPI][G][HD]
    __shared__ float qs[G][HD];
    __shared__ float s_m[G], s_l[G];

    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int sub = lane / LPR, dl = lane % LPR;  // V: row within a group, 8-dim slice
    const int l16 = lane & 15, kg = lane >> 4;     // K operand: row of the wavefront's 16, 8-dim slice of a k step
    const int split = blockIdx.x, nsplit = gridDim.x, kvhd = blockIdx.y, b = blockIdx.z;
    const int H = kvh * G;
    const int n0 = split * chunk;
    const size_t head_base = ((size_t)b * kvh + kvhd) * max_len * HD;
    const uint16_t *kbase = kcache + head_base + (size_t)n0 * HD + kg * 8;
    const uint16_t *vbase = vcache + head_base + (size_t)n0 * HD + dl * 8;
    const int cnt = min(kv_len, n0 + chunk) - n0;  // >= 1: the grid covers kv_len exactly
    const int iters = (cnt + IT_ROWS - 1) / IT_ROWS;

    // Rows past the live range are clamped to the last live row instead of masked: every request issues
    // the same number of loads, so the waits can leave the next step's loads in flight. Their scores become
    // -inf below, hence their probabilities zero, and the clamped V rows are finite.
    auto request = [&](u32x4(&kr)[KS], u32x4(&vr)[NRG_V], int it) {
        const int krow = min(it * IT_ROWS + 16 * wave + l16, cnt - 1);
#pragma unroll
        for (int s = 0; s < KS; s++) kr[s] = ld128_stream(kbase + (size_t)krow * HD + 32 * s);
#pragma unroll
        for (int i = 0; i < NRG_V; i++) {
            const int row = min(it * IT_ROWS + (i * ATT_WAVES + wave) * RPI + sub, cnt - 1);
            vr[i] = ld128_stream(vbase + (size_t)row * HD);
        }
    };
    // Two steps are in flight from the start (a short walk has its whole range requested at once; the second
    // request of a one-step walk re-reads the first, so the number of loads outstanding is the same for all).
    u32x4 ka[KS], va[NRG_V], kb[KS], vb[NRG_V];
    request(ka, va, 0);
    request(kb, vb, min(1, iters - 1));

    for (int i = tid; i < G * HD; i += ATT_THREADS)
        qs[i / HD][i % HD] = q[((size_t)b * H + kvhd * G) * HD + i];
    __syncthreads();
    // B operand: column l16 is query head l16 (columns past G are zero), scaled, as two pieces
    bf16x8 qop[KS][2];
#pragma unroll
    for (int s = 0; s < KS; s++) {
        float f[8];
#pragma unroll
        for (int e = 0; e < 8; e++) f[e] = l16 < G ? qs[l16 < G ? l16 : 0][32 * s + 8 * kg + e] * scale : 0.f;
        split8<2>(f, qop[s]);
    }

    float acc[G][8];
#pragma unroll
    for (int gi = 0; gi < G; gi++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[gi][e] = 0.f;
    float m_run[SLOTS], l_run[SLOTS];
#pragma unroll
    for (int s = 0; s < SLOTS; s++) {
        m_run[s] = -INFINITY;
        l_run[s] = 0.f;
    }

    auto step = [&](u32x4(&kr)[KS], u32x4(&vr)[NRG_V], int it) {
        float *scp = sc + (it & 1) * G * IT_ROWS;
        float *facp = fac + (it & 1) * G;
        // scores of the wavefront's 16 rows against every head; the small piece first. Lane
        // l16 + 16 c receives head l16, rows 4 c .. 4 c + 3; rows past the live range count as -inf.
        {
            f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const bf16x8 kop = __builtin_bit_cast(bf16x8, kr[s]);
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, qop[s][1], c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, qop[s][0], c, 0, 0, 0);
            }
            const int r0 = 16 * wave + 4 * kg;
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (it * IT_ROWS + r0 + i >= cnt) c[i] = -INFINITY;
            if (l16 < G) *reinterpret_cast<f32x4 *>(scp + l16 * IT_ROWS + r0) = c;
        }
        __syncthreads();
        // one wavefront per head: move the running maximum, turn scores into exp(s - max)
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            const int gi = wave + s * ATT_WAVES;
            if (gi < G) {
                const float x = scp[gi * IT_ROWS + lane];
                const float m_new = fmaxf(m_run[s], wave_max(x));  // finite: row 0 of a step is live
                const float e = expf(x - m_new);
                scp[gi * IT_ROWS + lane] = e;
                const float f = expf(m_run[s] - m_new);
                l_run[s] = fmaf(l_run[s], f, wave_sum(e));
                m_run[s] = m_new;
                if (lane == 0) facp[gi] = f;
            }
        }
        __syncthreads();
        // o = o * factor + P.V
#pragma unroll
        for (int gi = 0; gi < G; gi++) {
            const float f = facp[gi];
            if (f != 1.f) {
#pragma unroll
                for (int e = 0; e < 8; e++) acc[gi][e] *= f;
            }
        }
#pragma unroll
        for (int i = 0; i < NRG_V; i++) {
            const int r = (i * ATT_WAVES + wave) * RPI + sub;
            float vf[8];
            unpack8(vr[i], vf);
#pragma unroll
            for (int gi = 0; gi < G; gi++) {
                const float p = scp[gi * IT_ROWS + r];
#pragma unroll
                for (int e = 0; e < 8; e++) acc[gi][e] = fmaf(p, vf[e], acc[gi][e]);
            }
        }
    };
    // A step's registers are asked for again (two steps on) as soon as it has been multiplied; the last steps,
    // with nothing left to ask for, are written out so that every wait knows how many loads are behind it.
    int it = 0;
    for (; it + 3 < iters; it += 2) {
        step(ka, va, it);
        request(ka, va, it + 2);
        step(kb, vb, it + 1);
        request(kb, vb, it + 3);
    }
    const int left = iters - it;  // 1..3
    step(ka, va, it);
    if (left == 3) request(ka, va, it + 2);
    if (left >= 2) step(kb, vb, it + 1);
    if (left == 3) step(ka, va, it + 2);

#pragma unroll
    for (int s = 0; s < SLOTS; s++) {
        const int gi = wave + s * ATT_WAVES;
        if (gi < G && lane == 0) {
            s_m[gi] = m_run[s];
            s_l[gi] = l_run[s];
        }
    }
#pragma unroll
    for (int gi = 0; gi < G; gi++) {
        float *dst = red + ((size_t)(wave * RPI + sub) * G + gi) * HD + dl * 8;
        *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[gi][0], acc[gi][1], acc[gi][2], acc[gi][3]};
        *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{acc[gi][4], acc[gi][5], acc[gi][6], acc[gi][7]};
    }
    __syncthreads();

    const size_t pair = (size_t)b * kvh + kvhd;
    float *po = part_o + (pair * nsplit + split) * G * HD;
    float *pml = part_ml + (pair * nsplit + split) * G * 2;
    for (int i = tid; i < G * HD; i += ATT_THREADS) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < ATT_WAVES * RPI; w++) v += red[(size_t)w * G * HD + i];
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

// Second half of the split attention: one workgroup of HD threads per (batch, query head)
// folds that head's partial (o, max, sum) triples in ascending split order. A separate launch
// instead of a "last workgroup to arrive" fold: the kernel boundary orders the partial writes,
// so no device-scope fence (a full L2 write-back + invalidate on this chip) is needed.
template <int HD, int G>
__global__ __launch_bounds__(HD) void gqa_decode_fold_kernel(
    float *__restrict__ out, const float *__restrict__ part_o, const float *__restrict__ part_ml,
    int kvh, int kv_len_arg, int chunk, const DecodeState *__restrict__ state) {
    extern __shared__ float s_ml[];  // [nsplit][2] of this head
    const int d = threadIdx.x;
    const int gi = blockIdx.x % G, kvhd = blockIdx.x / G, b = blockIdx.y;
    const int H = kvh * G;
    const int kv_len = state ? state->pos + 1 : kv_len_arg;
    const int nsplit = (kv_len + chunk - 1) / chunk;
    if (nsplit == 1) return;  // the attention kernel wrote the final result itself
    const size_t pair = (size_t)b * kvh + kvhd;
    const float *ao = part_o + (pair * nsplit * G + gi) * HD + d;
    const float *aml = part_ml + (pair * nsplit * G + gi) * 2;
    constexpr int FB = 16;  // splits fetched per batch, all loads of a batch in flight together
    float o[FB];
#pragma unroll
    for (int u = 0; u < FB; u++) o[u] = u < nsplit ? ao[(size_t)u * G * HD] : 0.f;
    for (int i = d; i < nsplit * 2; i += HD) s_ml[i] = aml[(size_t)(i >> 1) * G * 2 + (i & 1)];
    __syncthreads();
    float M = -INFINITY;
    for (int s = 0; s < nsplit; s++) M = fmaxf(M, s_ml[s * 2]);
    float L = 0.f, O = 0.f;
    for (int s0 = 0; s0 < nsplit; s0 += FB) {
        if (s0 > 0) {
#pragma unroll
            for (int u = 0; u < FB; u++) o[u] = s0 + u < nsplit ? ao[(size_t)(s0 + u) * G * HD] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < FB; u++) {
            if (s0 + u < nsplit) {
                const float wgt = expf(s_ml[(s0 + u) * 2] - M);
                L = fmaf(wgt, s_ml[(s0 + u) * 2 + 1], L);
                O = fmaf(wgt, o[u], O);
            }
        }
    }
    out[((size_t)b * H + kvhd * G + gi) * HD + d] = O / L;
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
    // scores [G][chunk] + partials of every row-subgroup of every wavefront [4 * RPI][G][HD]
    const size_t front = (size_t)G * chunk;
    const size_t lds = (front + (size_t)ATT_WAVES * (WAVE / (HD / 8)) * G * HD) * sizeof(float);
    const size_t pairs = (size_t)a.B * a.kvh;
    float *part_o = a.partials ? a.partials : (float *)ctx->workspace;
    float *part_ml = part_o + pairs * nsplit * G * HD;
    AttnFuse f{a.qkv_raw, a.qw, a.kw, a.cos_tab, a.sin_tab, a.eps};
    if (a.phase != AttnArgs::FOLD_ONLY) {
        static bool lds_limit_raised = false;  // per instantiation; large groups need more than 64 KiB
        if (lds > 64 * 1024 && !lds_limit_raised) {
            HM_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(&gqa_decode_attn_kernel<HD, G>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
            lds_limit_raised = true;
        }
        HM_REQUIRE(ctx, lds <= 96 * 1024, "gqa_decode_attn: LDS need %zu too large", lds);
        hipLaunchKernelGGL((gqa_decode_attn_kernel<HD, G>), dim3(nsplit, a.kvh, a.B), dim3(ATT_THREADS),
                           lds, ctx->stream, a.q, const_cast<uint16_t *>(a.kcache),
                           const_cast<uint16_t *>(a.vcache), a.out, part_o, part_ml, a.kvh, a.max_len,
                           a.kv_len, chunk, a.scale, a.state, (int)front, f);
        HM_LAUNCH_CHECK(ctx);
    }
    // nsplit is the grid's split count: 1 means no call can ever need a fold
    if (nsplit > 1 && a.phase != AttnArgs::SPLIT_ONLY) {
        const size_t fold_lds = (size_t)nsplit * 2 * sizeof(float);
        HM_REQUIRE(ctx, fold_lds <= 64 * 1024, "gqa_decode_attn: too many splits (%d)", nsplit);
        hipLaunchKernelGGL((gqa_decode_fold_kernel<HD, G>), dim3(a.kvh * G, a.B), dim3(HD), fold_lds,
                           ctx->stream, a.out, part_o, part_ml, a.kvh, a.kv_len, chunk, a.state);
        HM_LAUNCH_CHECK(ctx);
    }
    return HM_OK;
}

// Long caches through the stepping kernel; its partials go through the same fold.
template <int HD, int G>
int launch_attn_stream(hm_ctx *ctx, const AttnArgs &a, int nsplit, int chunk) {
    constexpr int RPI = WAVE / (HD / 8);
    const size_t front = ((size_t)2 * G * IT_ROWS + 2 * G + 3) / 4 * 4;  // 16-byte rows behind it
    const size_t lds = (front + (size_t)ATT_WAVES * RPI * G * HD) * sizeof(float);
    const size_t pairs = (size_t)a.B * a.kvh;
    float *part_o = a.partials ? a.partials : (float *)ctx->workspace;
    float *part_ml = part_o + pairs * nsplit * G * HD;
    static bool lds_limit_raised = false;  // per instantiation
    if (lds > 64 * 1024 && !lds_limit_raised) {
        HM_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(&gqa_decode_attn_stream_kernel<HD, G>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        lds_limit_raised = true;
    }
    HM_REQUIRE(ctx, lds <= 96 * 1024, "gqa_decode_attn: LDS need %zu too large", lds);
    HM_REQUIRE(ctx, chunk % IT_ROWS == 0, "gqa_decode_attn: chunk %d must be a multiple of %d", chunk, IT_ROWS);
    hipLaunchKernelGGL((gqa_decode_attn_stream_kernel<HD, G>), dim3(nsplit, a.kvh, a.B),
                       dim3(ATT_THREADS), lds, ctx->stream, a.q, a.kcache, a.vcache, a.out, part_o,
                       part_ml, a.kvh, a.max_len, a.kv_len, chunk, a.scale, (int)front);
    HM_LAUNCH_CHECK(ctx);
    if (nsplit > 1) {
        const size_t fold_lds = (size_t)nsplit * 2 * sizeof(float);
        HM_REQUIRE(ctx, fold_lds <= 64 * 1024, "gqa_decode_attn: too many splits (%d)", nsplit);
        hipLaunchKernelGGL((gqa_decode_fold_kernel<HD, G>), dim3(a.kvh * G, a.B), dim3(HD), fold_lds,
                           ctx->stream, a.out, part_o, part_ml, a.kvh, a.kv_len, chunk,
                           (const DecodeState *)nullptr);
        HM_LAUNCH_CHECK(ctx);
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
    const int span = a.state ? a.max_len : a.kv_len;  // rows the grid has to be able to cover
    int chunk = a.fixed_chunk;
    bool stepping = false;
    if (chunk <= 0) {
        int want = (int)(((size_t)ctx->num_cus + pairs - 1) / pairs);
        chunk = (span + want - 1) / want;
        chunk = (chunk + rows_step - 1) / rows_step * rows_step;
        // More rows per workgroup than its registers hold: the stepping kernel, two workgroups per
        // CU (plain calls only; the decode plan's fused prologue lives in the other kernel).
        if (chunk > 128 && !a.state && !a.qkv_raw) {
            stepping = true;
            const int it_rows = IT_ROWS;
            want = (int)(((size_t)2 * ctx->num_cus + pairs - 1) / pairs);
            chunk = (span + want - 1) / want;
            chunk = (chunk + it_rows - 1) / it_rows * it_rows;
        }
    }
    if (stepping) {
        HM_REQUIRE(ctx, a.q != nullptr, "gqa_decode_attn: NULL query");
        const int nsplit = (a.kv_len + chunk - 1) / chunk;
        const size_t ws_need = pairs * nsplit * g * (a.hd + 2) * sizeof(float);
        HM_REQUIRE(ctx, ws_need <= ws_have, "gqa_decode_attn: %zu bytes of partial results exceed the %zu available", ws_need, ws_have);
        if (a.hd == 128) return dispatch_g<128>(ctx, a, g, nsplit, chunk, true);
        return dispatch_g<64>(ctx, a, g, nsplit, chunk, true);
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
