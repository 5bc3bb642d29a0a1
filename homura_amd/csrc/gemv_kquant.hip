// GGUF K-quants (Q4_K, Q6_K): activation quantisation to Q8_K, integer-dot GEMV, and bit-exact
// block dequantisation (reference src/graph_builder/emit_quant.rs:165-816, src/gguf.rs:835-917).
//
// The reference multiplies these weights against an activation quantised to int8 per 256-wide
// block (Q8_K: scale amax/127, round half to even) with integer dot products per sub-block; the
// GPU does the same arithmetic - the integer sums are identical, only the order of the f32 adds
// differs - with v_dot4_i32_i8 doing four multiply-adds per instruction.
//
// Weights stay the raw GGUF super-blocks, rows of K/256 blocks. A workgroup copies a run of rows
// into LDS with aligned 16-byte loads (the next run travels in registers meanwhile). The unit of
// work of a lane is 16 weights: one sub-block half of Q4_K (16 bytes, low or high nibbles) or one
// sub-block of Q6_K. Units are dealt to the lanes round-robin (K/16 per row, so K = 1024 fills the
// wavefront exactly); a lane keeps the 16 int8 activations of each of its units, their sum and
// the block's activation scale in registers for the life of the workgroup and walks the rows.
#include "gemv_kquant.h"
#include "hm_common.h"
#include "quant_formats.h"

namespace {

constexpr int KTHREADS = 256;
constexpr int KWAVES = KTHREADS / WAVE;
constexpr int KMAX_ROWS = KWAVES * 8;
constexpr int KSTAGE_U = 8;                            // 16-byte chunks a thread carries per row step
constexpr int KSTAGE_BYTES = KTHREADS * KSTAGE_U * 16; // most bytes one row step may span
constexpr int KMAXC = 8;                               // unit rounds a lane keeps in registers (K <= 8192)
// Rows of 8193 .. 16384 (the down projection of models with wide MLPs): twice the rounds, a deeper row stage,
// no light ops inside the launch.
constexpr int KMAXC_LONG = 16;
constexpr int KSTAGE_U_LONG = 14;
constexpr int KSTAGE_BYTES_LONG = KTHREADS * KSTAGE_U_LONG * 16;

template <int QT>
struct KTraits;
template <>
struct KTraits<0> {  // Q4_K
    static constexpr int BYTES = 144;
};
template <>
struct KTraits<1> {  // Q6_K
    static constexpr int BYTES = 210;
};

__device__ __forceinline__ uint32_t lds16(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }
__device__ __forceinline__ uint32_t lds32_a2(const uint8_t *p) { return lds16(p) | (lds16(p + 2) << 16); }

// ── Q8_K quantisation of the activation: one wavefront per 256-wide block ──
// (emit_quant.rs:422-466) amax, act_d = amax / 127, iscale = 127 / amax (0 for a zero block),
// q = roundeven(x * iscale) clamped to +-127, bsums = sums of 16 consecutive q.
__global__ __launch_bounds__(WAVE) void quantize_q8_k_kernel(const float *__restrict__ x, int8_t *__restrict__ q8,
                                                             float *__restrict__ act_d, int *__restrict__ bsums) {
    const int lane = threadIdx.x;
    const size_t blk = blockIdx.x;
    const f32x4 v = *reinterpret_cast<const f32x4 *>(x + blk * 256 + lane * 4);
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = wave_max(amax);
    const float iscale = amax == 0.f ? 0.f : __fdiv_rn(127.0f, amax);
    int q[4];
    const float xs[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float r = rintf(__fmul_rn(xs[i], iscale));  // round half to even
        r = fminf(r, 127.0f);
        r = fmaxf(r, -127.0f);
        q[i] = (int)r;
    }
    const uint32_t packed = (uint32_t)(q[0] & 0xFF) | ((uint32_t)(q[1] & 0xFF) << 8) | ((uint32_t)(q[2] & 0xFF) << 16) |
                            ((uint32_t)(q[3] & 0xFF) << 24);
    *reinterpret_cast<uint32_t *>(q8 + blk * 256 + lane * 4) = packed;
    // 16 consecutive values = four adjacent lanes
    int s = q[0] + q[1] + q[2] + q[3];
    s += __builtin_amdgcn_update_dpp(0, s, 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
    s += __builtin_amdgcn_update_dpp(0, s, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
    if ((lane & 3) == 0) bsums[blk * 16 + (lane >> 2)] = s;
    if (lane == 0) act_d[blk] = __fdiv_rn(amax, 127.0f);
}

// What a lane keeps of the activation for one of its 16-weight units.
struct ActUnit {
    uint32_t q[4];  // 16 int8
    int bsum;       // their sum
    float d;        // activation scale of the unit's 256-block
};

__device__ __forceinline__ int dot16(const uint32_t *w, const uint32_t *a) {
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) s = __builtin_amdgcn_sdot4((int)w[i], (int)a[i], s, false);
    return s;
}

// One Q4_K unit: i = unit index inside the super-block (0..15) = 2 * sub-block + half.
// Sub-blocks come in pairs sharing 32 bytes, even = low nibbles, odd = high nibbles; scale and min
// of sub-block sb unpack from the 12 packed bytes as in get_scale_min_k4 (src/gguf.rs:847-862).
__device__ __forceinline__ float q4k_unit(const uint8_t *blk, int i, const ActUnit &a) {
    const int sb = i >> 1, h = i & 1, pair = sb >> 1, odd = sb & 1;
    const uint32_t hdr = *reinterpret_cast<const uint32_t *>(blk);  // d | dmin << 16
    const float d = f16_bits_to_f32((uint16_t)(hdr & 0xFFFFu)), dmin = f16_bits_to_f32((uint16_t)(hdr >> 16));
    const uint8_t *raw = blk + 4;
    int sc, mn;
    if (sb < 4) {
        sc = raw[sb] & 63;
        mn = raw[sb + 4] & 63;
    } else {
        const int hi = raw[sb + 4];
        sc = (hi & 15) | ((raw[sb - 4] >> 6) << 4);
        mn = (hi >> 4) | ((raw[sb] >> 6) << 4);
    }
    const u32x4 w = *reinterpret_cast<const u32x4 *>(blk + 16 + pair * 32 + h * 16);
    const int sh = odd * 4;
    const uint32_t nib[4] = {(w.x >> sh) & 0x0F0F0F0Fu, (w.y >> sh) & 0x0F0F0F0Fu, (w.z >> sh) & 0x0F0F0F0Fu,
                             (w.w >> sh) & 0x0F0F0F0Fu};
    const int isum = dot16(nib, a.q);
    // d*act_d*(sc*isum) - dmin*act_d*(mn*bsum): the unit's share of the block's scale and min parts
    return (d * a.d) * (float)(sc * isum) - (dmin * a.d) * (float)(mn * a.bsum);
}

// One Q6_K unit: i = sub-block (0..15); chunk = i/8, group = (i%8)/2, parity = i%2:
// low nibbles at ql[64 chunk + 32 (group&1) + 16 parity ..] (upper nibble for group >= 2), bit pair
// `group` of qh[32 chunk + 16 parity ..], q = (lo | hi << 4) - 32 (emit_quant.rs:668-760).
// stage = start of the LDS row stage (16-byte aligned), off = byte offset of the block in it (even): the
// 16-byte pieces sit two bytes into a dword for every other block, so each is read as five aligned dwords
// and shifted into place (five LDS reads and four funnel shifts instead of eight 16-bit reads and four merges).
__device__ __forceinline__ float q6k_unit(const uint8_t *stage, int off, int i, const ActUnit &a) {
    const uint8_t *blk = stage + off;
    const int chunk = i >> 3, group = (i & 7) >> 1, parity = i & 1;
    const int qlo = off + chunk * 64 + (group & 1) * 32 + parity * 16, qho = off + 128 + chunk * 32 + parity * 16;
    const uint32_t sh = (uint32_t)(off & 2) * 8;
    const uint32_t *pl = reinterpret_cast<const uint32_t *>(stage + (qlo & ~3));
    const uint32_t *ph = reinterpret_cast<const uint32_t *>(stage + (qho & ~3));
    uint32_t l[5], hg[5];
#pragma unroll
    for (int j = 0; j < 5; j++) {
        l[j] = pl[j];
        hg[j] = ph[j];
    }
    const int lo_sh = group >= 2 ? 4 : 0, hi_sh = group * 2;
    uint32_t v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t lw = __builtin_amdgcn_alignbit(l[j + 1], l[j], sh), hw = __builtin_amdgcn_alignbit(hg[j + 1], hg[j], sh);
        v[j] = ((lw >> lo_sh) & 0x0F0F0F0Fu) | (((hw >> hi_sh) & 0x03030303u) << 4);
    }
    const int isum = dot16(v, a.q) - 32 * a.bsum;
    const int sc = (int)(int8_t)blk[192 + i];
    const float d = f16_bits_to_f32((uint16_t)lds16(blk + 208));
    return (d * a.d) * (float)(sc * isum);
}

struct StepRange {
    size_t abeg;
    int shift, nchunks, r0, nrows;
};
// The aligned 16-byte chunks covering rows [r0, r0+nrows). A chunk that holds at least one byte of
// the buffer lies in that byte's page, so whole aligned chunks at the buffer's ends cannot fault.
__device__ __forceinline__ StepRange step_range(int step, int rows_per_step, int N, size_t rowbytes) {
    StepRange r;
    r.r0 = step * rows_per_step;
    r.nrows = min(rows_per_step, N - r.r0);
    const size_t beg = (size_t)r.r0 * rowbytes, end = beg + (size_t)r.nrows * rowbytes;
    r.abeg = beg & ~(size_t)15;
    r.shift = (int)(beg - r.abeg);
    r.nchunks = (int)((end - r.abeg + 15) / 16);
    return r;
}

// RT rows lr, lr + KWAVES, ... of the staged step for one wavefront. Round t of a lane is unit
// lane + 64 t of the row: block (lane + 64 t) / 16 = lane/16 + 4 t, unit-in-block lane % 16.
template <int QT, int CPL, int RT>
__device__ __forceinline__ void krows_trip(const uint8_t *stage, int shift, size_t rowbytes, int lr, int lane, int nu,
                                           const ActUnit (&act)[CPL], float *out, const float *add) {
    constexpr int BB = KTraits<QT>::BYTES;
    const int boff = (lane >> 4) * BB, ui = lane & 15;
    float a[RT];
#pragma unroll
    for (int j = 0; j < RT; j++) a[j] = 0.f;
#pragma unroll
    for (int t = 0; t < CPL; t++) {
        const bool live = lane + t * WAVE < nu;
#pragma unroll
        for (int j = 0; j < RT; j++) {
            // lanes past the row end read the block of unit 0..15 of the row start: valid memory, dropped below
            const int off = shift + (lr + j * KWAVES) * (int)rowbytes + (live ? boff + t * 4 * BB : 0);
            const float v = QT == 0 ? q4k_unit(stage + off, ui, act[t]) : q6k_unit(stage, off, ui, act[t]);
            a[j] += live ? v : 0.f;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j = 0; j < RT; j++) {
        a[j] = wave_sum(a[j]);
        if (lane == 0) out[lr + j * KWAVES] = add ? a[j] + add[lr + j * KWAVES] : a[j];
    }
}

// The activation row of a fused launch, prepared by the whole workgroup into LDS: light ops (SiLU pair /
// residual add / RMSNorm, arithmetic as in the stand-alone kernels), then the Q8_K quantisation with the
// arithmetic of quantize_q8_k_kernel. Thread t holds elements 4 (t + 256 u) .. +3 of round u, so each
// wavefront owns whole 256-wide blocks: amax is a wave reduction, a sum of 16 a quad reduction.
constexpr int KXU = 4;  // rounds of 1024 elements: K <= 4096
__device__ __forceinline__ void stage_activation(const float *__restrict__ x, const homura::QuantFuse &fuse, int K,
                                                 int8_t *q8, float *act_d, int *bsums, float *red) {
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 xr[KXU], ar[KXU], nr[KXU];
    const float *second = fuse.x2 ? fuse.x2 : fuse.res_in;
#pragma unroll
    for (int u = 0; u < KXU; u++) {
        const int k = (tid + u * KTHREADS) * 4;
        xr[u] = k < K ? *reinterpret_cast<const f32x4 *>(x + k) : zero4;
        ar[u] = second && k < K ? *reinterpret_cast<const f32x4 *>(second + k) : zero4;
        nr[u] = fuse.norm_w && k < K ? *reinterpret_cast<const f32x4 *>(fuse.norm_w + k) : zero4;
    }
    if (fuse.x2) {
#pragma unroll
        for (int u = 0; u < KXU; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) xr[u][e] = (xr[u][e] / (1.0f + expf(-xr[u][e]))) * ar[u][e];
    } else if (fuse.res_in) {
#pragma unroll
        for (int u = 0; u < KXU; u++) {
            xr[u] += ar[u];
            const int k = (tid + u * KTHREADS) * 4;
            if (fuse.resid_out && blockIdx.x == 0 && k < K) *reinterpret_cast<f32x4 *>(fuse.resid_out + k) = xr[u];
        }
    }
    if (fuse.norm_w) {
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < KXU; u++) ss += (xr[u][0] * xr[u][0] + xr[u][1] * xr[u][1]) + (xr[u][2] * xr[u][2] + xr[u][3] * xr[u][3]);
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weight loads stay in flight
        float tot = 0.f;
#pragma unroll
        for (int wv = 0; wv < KWAVES; wv++) tot += red[wv];
        const float inv = 1.0f / sqrtf(tot / (float)K + fuse.eps);
#pragma unroll
        for (int u = 0; u < KXU; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) xr[u][e] = (xr[u][e] * inv) * nr[u][e];
    }
#pragma unroll
    for (int u = 0; u < KXU; u++) {
        const int k = (tid + u * KTHREADS) * 4;  // block k / 256 = wave + 4 u belongs to this wavefront alone
        if (u * KTHREADS * 4 >= K) break;        // uniform
        float amax = fmaxf(fmaxf(fabsf(xr[u][0]), fabsf(xr[u][1])), fmaxf(fabsf(xr[u][2]), fabsf(xr[u][3])));
        amax = wave_max(amax);
        const float iscale = amax == 0.f ? 0.f : __fdiv_rn(127.0f, amax);
        int q[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float r = rintf(__fmul_rn(xr[u][i], iscale));  // round half to even
            r = fminf(r, 127.0f);
            r = fmaxf(r, -127.0f);
            q[i] = (int)r;
        }
        int s = q[0] + q[1] + q[2] + q[3];
        s += __builtin_amdgcn_update_dpp(0, s, 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
        s += __builtin_amdgcn_update_dpp(0, s, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
        if (k < K) {
            *reinterpret_cast<uint32_t *>(q8 + k) = (uint32_t)(q[0] & 0xFF) | ((uint32_t)(q[1] & 0xFF) << 8) |
                                                    ((uint32_t)(q[2] & 0xFF) << 16) | ((uint32_t)(q[3] & 0xFF) << 24);
            if ((lane & 3) == 0) bsums[k >> 4] = s;
            if (lane == 0) act_d[k >> 8] = __fdiv_rn(amax, 127.0f);
        }
    }
}

// QT2 >= 0: a second matrix of the other K-quant type (w2, N2 rows, results to out2) shares the launch and
// the prepared activation row - q|k in Q4_K with v in Q6_K, as Q4_K_M files have them. Its row steps follow
// the first matrix's; a step never straddles the two.
template <int QT, int CPL, bool FUSED, int QT2 = -1, int U_ = KSTAGE_U>
__global__ __launch_bounds__(KTHREADS) void gemv_kquant_kernel(const int8_t *__restrict__ q8,
                                                               const float *__restrict__ act_d,
                                                               const int *__restrict__ bsums,
                                                               const uint8_t *__restrict__ w, float *__restrict__ out,
                                                               int K, int N, int rows_per_step, const float *x_f32_arg,
                                                               const homura::QuantFuse fuse_arg, int act_lds_off,
                                                               const uint8_t *__restrict__ w2 = nullptr,
                                                               float *__restrict__ out2 = nullptr, int N2 = 0) {
    constexpr bool TWO = QT2 >= 0;
    constexpr int BB2 = KTraits<TWO ? QT2 : QT>::BYTES;
    // FUSED = false is the plain product over an activation quantised by its own launch
    const float *x_f32 = FUSED ? x_f32_arg : nullptr;
    const homura::QuantFuse fuse = FUSED ? fuse_arg : homura::QuantFuse();
    constexpr int BB = KTraits<QT>::BYTES;
    constexpr int U = U_;
    extern __shared__ __attribute__((aligned(16))) uint8_t ws[];
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int nb = K / 256, nu = K / 16;
    const size_t rowbytes = (size_t)nb * BB, rowbytes2 = (size_t)nb * BB2;
    const int nsteps1 = (N + rows_per_step - 1) / rows_per_step;
    const int nsteps = nsteps1 + (TWO ? (N2 + rows_per_step - 1) / rows_per_step : 0);
    auto range_of = [&](int st) {
        return TWO && st >= nsteps1 ? step_range(st - nsteps1, rows_per_step, N2, rowbytes2)
                                    : step_range(st, rows_per_step, N, rowbytes);
    };
    auto src_of = [&](int st) { return TWO && st >= nsteps1 ? w2 : w; };

    // the first row step is requested before anything else waits
    u32x4 tmp[U];
    int step = blockIdx.x;
    StepRange cur = range_of(step);
    const uint8_t *src = src_of(step);
    if (x_f32) {  // fused launch: the f32 row is prepared and quantised here, into LDS behind the row stage
        int8_t *lq8 = reinterpret_cast<int8_t *>(ws + act_lds_off);
        float *ld = reinterpret_cast<float *>(lq8 + K);
        int *lbs = reinterpret_cast<int *>(ld + nb);
        float *red = reinterpret_cast<float *>(lbs + nu);
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = tid + u * KTHREADS;
            tmp[u] = i < cur.nchunks ? ld128_stream(src + cur.abeg + (size_t)i * 16) : u32x4{0u, 0u, 0u, 0u};
        }
        stage_activation(x_f32, fuse, K, lq8, ld, lbs, red);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        q8 = lq8;
        act_d = ld;
        bsums = lbs;
    }
    // the lane's share of the quantised activation (small, cached)
    ActUnit act[CPL];
#pragma unroll
    for (int t = 0; t < CPL; t++) {
        const int u = min(lane + t * WAVE, nu - 1);
        const u32x4 q = *reinterpret_cast<const u32x4 *>(q8 + (size_t)u * 16);
        act[t].q[0] = q.x; act[t].q[1] = q.y; act[t].q[2] = q.z; act[t].q[3] = q.w;
        act[t].bsum = bsums[u];
        act[t].d = act_d[u >> 4];
    }
    if (!x_f32) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = tid + u * KTHREADS;
            tmp[u] = i < cur.nchunks ? ld128_stream(src + cur.abeg + (size_t)i * 16) : u32x4{0u, 0u, 0u, 0u};
        }
    }

    for (; step < nsteps; step += gridDim.x) {
        __syncthreads();  // previous step's readers are done with ws
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = tid + u * KTHREADS;
            if (i < cur.nchunks) *reinterpret_cast<u32x4 *>(ws + (size_t)i * 16) = tmp[u];
        }
        __syncthreads();
        const StepRange now = cur;
        const bool second = TWO && step >= nsteps1;
        if (step + (int)gridDim.x < nsteps) {  // the next step's weights travel while this one is multiplied
            cur = range_of(step + gridDim.x);
            src = src_of(step + gridDim.x);
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int i = tid + u * KTHREADS;
                tmp[u] = i < cur.nchunks ? ld128_stream(src + cur.abeg + (size_t)i * 16) : u32x4{0u, 0u, 0u, 0u};
            }
        }
        int lr = wave;
        if (second) {
            constexpr int Q2 = TWO ? QT2 : QT;
            float *o = out2 + now.r0;
            for (; lr + 3 * KWAVES < now.nrows; lr += 4 * KWAVES) krows_trip<Q2, CPL, 4>(ws, now.shift, rowbytes2, lr, lane, nu, act, o, nullptr);
            if (lr + KWAVES < now.nrows) {
                krows_trip<Q2, CPL, 2>(ws, now.shift, rowbytes2, lr, lane, nu, act, o, nullptr);
                lr += 2 * KWAVES;
            }
            if (lr < now.nrows) krows_trip<Q2, CPL, 1>(ws, now.shift, rowbytes2, lr, lane, nu, act, o, nullptr);
            continue;
        }
        float *o = out + now.r0;
        const float *add = fuse.res_out_add ? fuse.res_out_add + now.r0 : nullptr;
        if constexpr (CPL <= KMAXC) {
            for (; lr + 3 * KWAVES < now.nrows; lr += 4 * KWAVES) krows_trip<QT, CPL, 4>(ws, now.shift, rowbytes, lr, lane, nu, act, o, add);
            if (lr + KWAVES < now.nrows) {
                krows_trip<QT, CPL, 2>(ws, now.shift, rowbytes, lr, lane, nu, act, o, add);
                lr += 2 * KWAVES;
            }
            if (lr < now.nrows) krows_trip<QT, CPL, 1>(ws, now.shift, rowbytes, lr, lane, nu, act, o, add);
        } else {  // long rows: the lane's share of the activation takes the registers of the side-by-side chains
            for (; lr < now.nrows; lr += KWAVES) krows_trip<QT, CPL, 1>(ws, now.shift, rowbytes, lr, lane, nu, act, o, add);
        }
    }
}

// ── f32 activations against the dequantised weights ─────────────────────────────────────────────────
//
// What the reference computes when a K-quant tensor feeds an f32 kernel (its loader dequantises the
// embedding / output matrices, src/gguf.rs:589-708, and the LM head multiplies f32 by f32): out[n] =
// sum_k x[k] * w[n][k] with w the dequantised weight. Every w is d * sc * q (Q6_K) or q * (d * sc) - dmin * mn
// (Q4_K) with small integers q, so a 16-weight unit is (d * sc) * (sum_j u_j x_j - off * sum_j x_j)
// [- (dmin * mn) * sum_j x_j] in f32: one byte -> float conversion and one FMA per weight, the sums of x per
// unit computed once. The rows are staged like in the integer kernel; optional RMSNorm of the row on the way
// in (the LM head's final norm), optional best (value, index) per workgroup on the way out.
struct ActF32 {
    float x[16];
    float sx;
};

__device__ __forceinline__ float dot16_f32(const uint32_t *w, const float *x) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        s = fmaf((float)(w[i] & 0xFFu), x[4 * i], s);
        s = fmaf((float)((w[i] >> 8) & 0xFFu), x[4 * i + 1], s);
        s = fmaf((float)((w[i] >> 16) & 0xFFu), x[4 * i + 2], s);
        s = fmaf((float)(w[i] >> 24), x[4 * i + 3], s);
    }
    return s;
}

__device__ __forceinline__ float q4k_unit_f32(const uint8_t *blk, int i, const ActF32 &a) {
    const int sb = i >> 1, h = i & 1, pair = sb >> 1, odd = sb & 1;
    const uint32_t hdr = *reinterpret_cast<const uint32_t *>(blk);  // d | dmin << 16
    const float d = f16_bits_to_f32((uint16_t)(hdr & 0xFFFFu)), dmin = f16_bits_to_f32((uint16_t)(hdr >> 16));
    const uint8_t *raw = blk + 4;
    int sc, mn;
    if (sb < 4) {
        sc = raw[sb] & 63;
        mn = raw[sb + 4] & 63;
    } else {
        const int hi = raw[sb + 4];
        sc = (hi & 15) | ((raw[sb - 4] >> 6) << 4);
        mn = (hi >> 4) | ((raw[sb] >> 6) << 4);
    }
    const u32x4 w = *reinterpret_cast<const u32x4 *>(blk + 16 + pair * 32 + h * 16);
    const int sh = odd * 4;
    const uint32_t nib[4] = {(w.x >> sh) & 0x0F0F0F0Fu, (w.y >> sh) & 0x0F0F0F0Fu, (w.z >> sh) & 0x0F0F0F0Fu,
                             (w.w >> sh) & 0x0F0F0F0Fu};
    return (d * (float)sc) * dot16_f32(nib, a.x) - (dmin * (float)mn) * a.sx;
}

// same reads as q6k_unit: aligned dwords and funnel shifts
__device__ __forceinline__ float q6k_unit_f32(const uint8_t *stage, int off, int i, const ActF32 &a) {
    const uint8_t *blk = stage + off;
    const int chunk = i >> 3, group = (i & 7) >> 1, parity = i & 1;
    const int qlo = off + chunk * 64 + (group & 1) * 32 + parity * 16, qho = off + 128 + chunk * 32 + parity * 16;
    const uint32_t sh = (uint32_t)(off & 2) * 8;
    const uint32_t *pl = reinterpret_cast<const uint32_t *>(stage + (qlo & ~3));
    const uint32_t *ph = reinterpret_cast<const uint32_t *>(stage + (qho & ~3));
    uint32_t l[5], hg[5];
#pragma unroll
    for (int j = 0; j < 5; j++) {
        l[j] = pl[j];
        hg[j] = ph[j];
    }
    const int lo_sh = group >= 2 ? 4 : 0, hi_sh = group * 2;
    uint32_t v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t lw = __builtin_amdgcn_alignbit(l[j + 1], l[j], sh), hw = __builtin_amdgcn_alignbit(hg[j + 1], hg[j], sh);
        v[j] = ((lw >> lo_sh) & 0x0F0F0F0Fu) | (((hw >> hi_sh) & 0x03030303u) << 4);
    }
    const int sc = (int)(int8_t)blk[192 + i];
    const float d = f16_bits_to_f32((uint16_t)lds16(blk + 208));
    return (d * (float)sc) * (dot16_f32(v, a.x) - 32.f * a.sx);
}

template <int QT, int CPL, int RT>
__device__ __forceinline__ void krows_trip_f32(const uint8_t *stage, int shift, size_t rowbytes, int lr, int lane, int nu,
                                               const ActF32 (&act)[CPL], float *out, int row0, float &best_v, int &best_i) {
    constexpr int BB = KTraits<QT>::BYTES;
    const int boff = (lane >> 4) * BB, ui = lane & 15;
    float a[RT];
#pragma unroll
    for (int j = 0; j < RT; j++) a[j] = 0.f;
#pragma unroll
    for (int t = 0; t < CPL; t++) {
        const bool live = lane + t * WAVE < nu;
#pragma unroll
        for (int j = 0; j < RT; j++) {
            const int off = shift + (lr + j * KWAVES) * (int)rowbytes + (live ? boff + t * 4 * BB : 0);
            const float v = QT == 0 ? q4k_unit_f32(stage + off, ui, act[t]) : q6k_unit_f32(stage, off, ui, act[t]);
            a[j] += live ? v : 0.f;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j = 0; j < RT; j++) {
        a[j] = wave_sum(a[j]);
        const int r = lr + j * KWAVES;
        if (lane == 0) out[r] = a[j];
        // of equal maxima the later row wins (Rust Iterator::max_by, reference src/generate.rs:457-468,
        // :735-742); rows reach a wavefront in ascending order
        if (best_i < 0 || a[j] >= best_v) {
            best_v = a[j];
            best_i = row0 + r;
        }
    }
}

template <int QT, int CPL>
__global__ __launch_bounds__(KTHREADS) void gemv_kquant_f32_kernel(const float *__restrict__ x, const float *__restrict__ norm_w,
                                                                   float eps, const uint8_t *__restrict__ w,
                                                                   float *__restrict__ out, int K, int N, int rows_per_step,
                                                                   int x_lds_off, float *__restrict__ cand_v,
                                                                   int *__restrict__ cand_i) {
    constexpr int BB = KTraits<QT>::BYTES;
    constexpr int U = KSTAGE_U;
    extern __shared__ __attribute__((aligned(16))) uint8_t ws[];
    float *xs = reinterpret_cast<float *>(ws + x_lds_off);  // [K] the (normed) row, then 8 floats of scratch
    float *red = xs + K;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int nb = K / 256, nu = K / 16;
    const size_t rowbytes = (size_t)nb * BB;
    const int nsteps = (N + rows_per_step - 1) / rows_per_step;

    // the row first (loads return in issue order), the first step's weights right behind it
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 xr[KXU], nr[KXU];
#pragma unroll
    for (int u = 0; u < KXU; u++) {
        const int k = (tid + u * KTHREADS) * 4;
        xr[u] = k < K ? *reinterpret_cast<const f32x4 *>(x + k) : zero4;
        nr[u] = norm_w && k < K ? *reinterpret_cast<const f32x4 *>(norm_w + k) : zero4;
    }
    u32x4 tmp[U];
    int step = blockIdx.x;
    StepRange cur = step_range(step, rows_per_step, N, rowbytes);
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int i = tid + u * KTHREADS;
        tmp[u] = i < cur.nchunks ? ld128_stream(w + cur.abeg + (size_t)i * 16) : u32x4{0u, 0u, 0u, 0u};
    }
    if (norm_w) {  // emit_rms_norm (src/graph_builder/emit_linalg.rs:7-26): (x * inv) * w
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < KXU; u++) ss += (xr[u][0] * xr[u][0] + xr[u][1] * xr[u][1]) + (xr[u][2] * xr[u][2] + xr[u][3] * xr[u][3]);
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weight loads stay in flight
        float tot = 0.f;
#pragma unroll
        for (int wv = 0; wv < KWAVES; wv++) tot += red[wv];
        const float inv = 1.0f / sqrtf(tot / (float)K + eps);
#pragma unroll
        for (int u = 0; u < KXU; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) xr[u][e] = (xr[u][e] * inv) * nr[u][e];
    }
#pragma unroll
    for (int u = 0; u < KXU; u++) {
        const int k = (tid + u * KTHREADS) * 4;
        if (k < K) *reinterpret_cast<f32x4 *>(xs + k) = xr[u];
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    ActF32 act[CPL];
#pragma unroll
    for (int t = 0; t < CPL; t++) {
        const int u = min(lane + t * WAVE, nu - 1);
        float sx = 0.f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(xs + (size_t)u * 16 + 4 * q);
            act[t].x[4 * q] = v.x; act[t].x[4 * q + 1] = v.y; act[t].x[4 * q + 2] = v.z; act[t].x[4 * q + 3] = v.w;
            sx += (v.x + v.y) + (v.z + v.w);
        }
        act[t].sx = sx;
    }

    float best_v = -INFINITY;
    int best_i = -1;
    for (; step < nsteps; step += gridDim.x) {
        __syncthreads();  // previous step's readers are done with the row stage
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = tid + u * KTHREADS;
            if (i < cur.nchunks) *reinterpret_cast<u32x4 *>(ws + (size_t)i * 16) = tmp[u];
        }
        __syncthreads();
        const StepRange now = cur;
        if (step + (int)gridDim.x < nsteps) {  // the next step's weights travel while this one is multiplied
            cur = step_range(step + gridDim.x, rows_per_step, N, rowbytes);
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int i = tid + u * KTHREADS;
                tmp[u] = i < cur.nchunks ? ld128_stream(w + cur.abeg + (size_t)i * 16) : u32x4{0u, 0u, 0u, 0u};
            }
        }
        float *o = out + now.r0;
        int lr = wave;
        for (; lr + 3 * KWAVES < now.nrows; lr += 4 * KWAVES) krows_trip_f32<QT, CPL, 4>(ws, now.shift, rowbytes, lr, lane, nu, act, o, now.r0, best_v, best_i);
        if (lr + KWAVES < now.nrows) {
            krows_trip_f32<QT, CPL, 2>(ws, now.shift, rowbytes, lr, lane, nu, act, o, now.r0, best_v, best_i);
            lr += 2 * KWAVES;
        }
        if (lr < now.nrows) krows_trip_f32<QT, CPL, 1>(ws, now.shift, rowbytes, lr, lane, nu, act, o, now.r0, best_v, best_i);
    }
    if (cand_v) {  // the workgroup's best row: largest value, highest index among equals; -1 = no row
        __syncthreads();
        int *redi = reinterpret_cast<int *>(red + KWAVES);
        if (lane == 0) {
            red[wave] = best_v;
            redi[wave] = best_i;
        }
        __syncthreads();
        if (tid == 0) {
            float bv = -INFINITY;
            int bi = -1;
            for (int wv = 0; wv < KWAVES; wv++) {
                if (redi[wv] < 0) continue;
                if (bi < 0 || red[wv] > bv || (red[wv] == bv && redi[wv] > bi)) {
                    bv = red[wv];
                    bi = redi[wv];
                }
            }
            cand_v[blockIdx.x] = bv;
            cand_i[blockIdx.x] = bi;
        }
    }
}

// One thread per weight, the reference's arithmetic step by step (no contraction) so the bits match
// the CPU: Q4_K w = q * (d * sc) - dmin * mn; Q6_K w = (d * sc) * q (src/gguf.rs:835-917).
template <int QT>
__global__ __launch_bounds__(256) void dequant_kquant_kernel(const uint8_t *__restrict__ blocks,
                                                             float *__restrict__ out, size_t n_elems) {
    constexpr int QF = QT == 0 ? homura::QF_Q4_K : homura::QF_Q6_K;
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; e < n_elems; e += stride)
        out[e] = homura::dequant_element<QF>(blocks + (e >> 8) * KTraits<QT>::BYTES, (int)(e & 255));
}

int quantize_launch(hm_ctx *ctx, const float *d_x, int8_t *q8, float *act_d, int *bsums, int M, int K) {
    hipLaunchKernelGGL(quantize_q8_k_kernel, dim3((unsigned)((size_t)M * K / 256)), dim3(WAVE), 0, ctx->stream, d_x, q8,
                       act_d, bsums);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

template <int QT>
int gemv_kquant_launch(hm_ctx *ctx, const char *name, const float *d_x, const uint8_t *d_w, float *d_out, int M, int K,
                       int N, bool reuse_activation = false, const homura::QuantFuse *fuse = nullptr) {
    HM_CHECK_CTX(ctx);
    constexpr int BB = KTraits<QT>::BYTES;
    HM_REQUIRE(ctx, d_x && d_w && d_out, "%s: NULL pointer", name);
    HM_REQUIRE(ctx, M >= 1 && M <= 8, "%s: M=%d outside 1..8", name, M);
    HM_REQUIRE(ctx, K > 0 && K % 256 == 0 && N > 0, "%s: K=%d must be a positive multiple of 256, N=%d positive", name, K, N);
    HM_REQUIRE(ctx, K <= KMAXC_LONG * WAVE * 16, "%s: K=%d above %d", name, K, KMAXC_LONG * WAVE * 16);
    HM_REQUIRE(ctx, ((uintptr_t)d_w % 16) == 0 && ((uintptr_t)d_x % 16) == 0, "%s: weight and activation buffers must be 16-byte aligned", name);
    const size_t rowbytes = (size_t)(K / 256) * BB;
    const bool long_rows = K > KMAXC * WAVE * 16 || KWAVES * rowbytes + 32 > (size_t)KSTAGE_BYTES;
    const size_t stage_cap = long_rows ? (size_t)KSTAGE_BYTES_LONG : (size_t)KSTAGE_BYTES;
    HM_REQUIRE(ctx, KWAVES * rowbytes + 32 <= stage_cap, "%s: K=%d too large for the LDS stage", name, K);
    HM_REQUIRE(ctx, !(fuse && long_rows), "%s: the fused form takes rows up to %d", name, KMAXC * WAVE * 16);
    if (fuse) {
        HM_REQUIRE(ctx, M == 1 && K <= KXU * KTHREADS * 4, "%s: the fused form takes one row of at most %d", name, KXU * KTHREADS * 4);
        HM_REQUIRE(ctx, !(fuse->x2 && fuse->res_in), "%s: SiLU pair and residual input exclude each other", name);
        HM_REQUIRE(ctx, ((uintptr_t)fuse->x2 % 16) == 0 && ((uintptr_t)fuse->res_in % 16) == 0 && ((uintptr_t)fuse->resid_out % 16) == 0 &&
                            ((uintptr_t)fuse->norm_w % 16) == 0, "%s: fused operands must be 16-byte aligned", name);
    }
    // the quantised activation lives at the top of the workspace: q8 | act_d | bsums per activation row
    const size_t per_m = ((size_t)K + (size_t)K / 256 * 4 + (size_t)K / 16 * 4 + 255) & ~(size_t)255;
    HM_REQUIRE(ctx, per_m * M <= ctx->workspace_bytes, "%s: workspace too small", name);
    uint8_t *wsp = (uint8_t *)ctx->workspace + ctx->workspace_bytes - per_m * M;

    int rows = (int)(((size_t)40 * 1024) / rowbytes);
    rows = rows / KWAVES * KWAVES;
    if (rows < KWAVES) rows = KWAVES;
    if (rows > KMAX_ROWS) rows = KMAX_ROWS;
    while (rows > KWAVES && (size_t)rows * rowbytes + 32 > stage_cap) rows -= KWAVES;
    while (rows > KWAVES && (N + rows - 1) / rows < 2 * ctx->num_cus) rows -= KWAVES;
    // fused launches keep the quantised row in LDS behind the row stage: q8 | act_d | bsums | 4 floats
    const size_t stage_bytes = ((size_t)rows * rowbytes + 32 + 16 + 15) & ~(size_t)15;
    const size_t lds = fuse ? stage_bytes + (size_t)K + (size_t)(K / 256) * 4 + (size_t)(K / 16) * 4 + 16 : stage_bytes;
    const int nsteps = (N + rows - 1) / rows;
    int wg_per_cu = (int)(120 * 1024 / lds);
    if (wg_per_cu < 1) wg_per_cu = 1;
    if (wg_per_cu > 6) wg_per_cu = 6;
    const int grid = nsteps < ctx->num_cus * wg_per_cu ? nsteps : ctx->num_cus * wg_per_cu;
    const int cpl = (K / 16 + WAVE - 1) / WAVE;
    for (int m = 0; m < M; m++) {
        int8_t *q8 = (int8_t *)(wsp + per_m * m);
        float *act_d = (float *)(q8 + K);
        int *bsums = (int *)(act_d + K / 256);
        if (!reuse_activation && !fuse) {
            int rc = quantize_launch(ctx, d_x + (size_t)m * K, q8, act_d, bsums, 1, K);
            if (rc != HM_OK) return rc;
        }
        float *om = d_out + (size_t)m * N;
        const float *xf = fuse ? d_x : nullptr;
        const homura::QuantFuse fz = fuse ? *fuse : homura::QuantFuse();
#define HM_KQ_CASE(C)                                                                                              \
    do {                                                                                                            \
        if (fuse)                                                                                                   \
            hipLaunchKernelGGL((gemv_kquant_kernel<QT, C, true>), dim3(grid), dim3(KTHREADS), lds, ctx->stream, q8, \
                               act_d, bsums, d_w, om, K, N, rows, xf, fz, (int)stage_bytes);                        \
        else                                                                                                        \
            hipLaunchKernelGGL((gemv_kquant_kernel<QT, C, false>), dim3(grid), dim3(KTHREADS), lds, ctx->stream, q8, \
                               act_d, bsums, d_w, om, K, N, rows, xf, fz, (int)stage_bytes);                        \
    } while (0)
#define HM_KQ_LONG(C)                                                                                                     \
    hipLaunchKernelGGL((gemv_kquant_kernel<QT, C, false, -1, KSTAGE_U_LONG>), dim3(grid), dim3(KTHREADS), lds, ctx->stream, \
                       q8, act_d, bsums, d_w, om, K, N, rows, xf, fz, (int)stage_bytes)
        if (long_rows) {
            if (cpl <= 10) HM_KQ_LONG(10);
            else if (cpl <= 12) HM_KQ_LONG(12);
            else HM_KQ_LONG(16);
        } else
        switch (cpl) {
            case 1: HM_KQ_CASE(1); break;
            case 2: HM_KQ_CASE(2); break;
            case 3: HM_KQ_CASE(3); break;
            case 4: HM_KQ_CASE(4); break;
            case 5: HM_KQ_CASE(5); break;
            case 6: HM_KQ_CASE(6); break;
            case 7: HM_KQ_CASE(7); break;
            default: HM_KQ_CASE(8); break;
        }
#undef HM_KQ_LONG
#undef HM_KQ_CASE
        HM_LAUNCH_CHECK(ctx);
    }
    return HM_OK;
}

// One fused launch over two matrices of different K-quant types that share the activation row: the first
// (type QT, N rows, results to d_out) and the second (the other type, N2 rows, results to d_out2).
template <int QT>
int gemv_kquant_pair_launch(hm_ctx *ctx, const char *name, const float *d_x, const uint8_t *d_w, float *d_out, int N,
                            const uint8_t *d_w2, float *d_out2, int N2, int K, const homura::QuantFuse &fuse) {
    HM_CHECK_CTX(ctx);
    constexpr int QT2 = 1 - QT;
    constexpr int BBMAX = KTraits<1>::BYTES;  // Q6_K rows are the longer ones
    HM_REQUIRE(ctx, d_x && d_w && d_out && d_w2 && d_out2, "%s: NULL pointer", name);
    HM_REQUIRE(ctx, K > 0 && K % 256 == 0 && N > 0 && N2 > 0, "%s: K=%d must be a positive multiple of 256, N=%d and N2=%d positive", name, K, N, N2);
    HM_REQUIRE(ctx, K <= KXU * KTHREADS * 4, "%s: the fused form takes one row of at most %d", name, KXU * KTHREADS * 4);
    HM_REQUIRE(ctx, ((uintptr_t)d_w % 16) == 0 && ((uintptr_t)d_w2 % 16) == 0 && ((uintptr_t)d_x % 16) == 0,
               "%s: weight and activation buffers must be 16-byte aligned", name);
    HM_REQUIRE(ctx, !fuse.x2 && !fuse.res_out_add, "%s: a pair takes the residual and norm prologue only", name);
    HM_REQUIRE(ctx, ((uintptr_t)fuse.res_in % 16) == 0 && ((uintptr_t)fuse.resid_out % 16) == 0 && ((uintptr_t)fuse.norm_w % 16) == 0,
               "%s: fused operands must be 16-byte aligned", name);
    const size_t rowbytes = (size_t)(K / 256) * BBMAX;
    HM_REQUIRE(ctx, KWAVES * rowbytes + 32 <= (size_t)KSTAGE_BYTES, "%s: K=%d too large for the LDS stage", name, K);
    int rows = (int)(((size_t)40 * 1024) / rowbytes);
    rows = rows / KWAVES * KWAVES;
    if (rows < KWAVES) rows = KWAVES;
    if (rows > KMAX_ROWS) rows = KMAX_ROWS;
    while (rows > KWAVES && (size_t)rows * rowbytes + 32 > (size_t)KSTAGE_BYTES) rows -= KWAVES;
    while (rows > KWAVES && (N + N2 + rows - 1) / rows < 2 * ctx->num_cus) rows -= KWAVES;
    const size_t stage_bytes = ((size_t)rows * rowbytes + 32 + 16 + 15) & ~(size_t)15;
    const size_t lds = stage_bytes + (size_t)K + (size_t)(K / 256) * 4 + (size_t)(K / 16) * 4 + 16;
    const int nsteps = (N + rows - 1) / rows + (N2 + rows - 1) / rows;
    int wg_per_cu = (int)(120 * 1024 / lds);
    if (wg_per_cu < 1) wg_per_cu = 1;
    if (wg_per_cu > 6) wg_per_cu = 6;
    const int grid = nsteps < ctx->num_cus * wg_per_cu ? nsteps : ctx->num_cus * wg_per_cu;
    const int cpl = (K / 16 + WAVE - 1) / WAVE;
#define HM_KP_CASE(C)                                                                                                   \
    hipLaunchKernelGGL((gemv_kquant_kernel<QT, C, true, QT2>), dim3(grid), dim3(KTHREADS), lds, ctx->stream,             \
                       (const int8_t *)nullptr, (const float *)nullptr, (const int *)nullptr, d_w, d_out, K, N, rows, d_x, \
                       fuse, (int)stage_bytes, d_w2, d_out2, N2)
    switch (cpl) {
        case 1: HM_KP_CASE(1); break;
        case 2: HM_KP_CASE(2); break;
        case 3: HM_KP_CASE(3); break;
        default: HM_KP_CASE(4); break;
    }
#undef HM_KP_CASE
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

// Rows per step, LDS and grid of the f32-activation kernel (the grid is also the number of argmax
// candidates it leaves, so the plan has to be able to ask for it).
struct F32Shape {
    int rows, grid;
    size_t stage_bytes, lds;
};
template <int QT>
F32Shape f32_shape(const hm_ctx *ctx, int K, int N, int cand_cap) {
    const size_t rowbytes = (size_t)(K / 256) * KTraits<QT>::BYTES;
    int rows = (int)(((size_t)40 * 1024) / rowbytes);
    rows = rows / KWAVES * KWAVES;
    if (rows < KWAVES) rows = KWAVES;
    if (rows > KMAX_ROWS) rows = KMAX_ROWS;
    while (rows > KWAVES && (size_t)rows * rowbytes + 32 > (size_t)KSTAGE_BYTES) rows -= KWAVES;
    while (rows > KWAVES && (N + rows - 1) / rows < 2 * ctx->num_cus) rows -= KWAVES;
    F32Shape sh;
    sh.rows = rows;
    sh.stage_bytes = ((size_t)rows * rowbytes + 32 + 16 + 15) & ~(size_t)15;
    sh.lds = sh.stage_bytes + (size_t)K * 4 + 64;
    const int nsteps = (N + rows - 1) / rows;
    int wg_per_cu = (int)(120 * 1024 / sh.lds);
    if (wg_per_cu < 1) wg_per_cu = 1;
    if (wg_per_cu > 6) wg_per_cu = 6;
    sh.grid = nsteps < ctx->num_cus * wg_per_cu ? nsteps : ctx->num_cus * wg_per_cu;
    if (cand_cap > 0 && sh.grid > cand_cap) sh.grid = cand_cap;
    return sh;
}

template <int QT>
int gemv_kquant_f32_launch(hm_ctx *ctx, const char *name, const float *d_x, const float *d_norm_w, float eps,
                           const uint8_t *d_w, float *d_out, int M, int K, int N, float *cand_v, int *cand_i, int cand_cap,
                           int *grid_out) {
    HM_CHECK_CTX(ctx);
    constexpr int BB = KTraits<QT>::BYTES;
    HM_REQUIRE(ctx, d_x && d_w && d_out, "%s: NULL pointer", name);
    HM_REQUIRE(ctx, M >= 1 && M <= 8, "%s: M=%d outside 1..8", name, M);
    HM_REQUIRE(ctx, K > 0 && K % 256 == 0 && N > 0, "%s: K=%d must be a positive multiple of 256, N=%d positive", name, K, N);
    HM_REQUIRE(ctx, K <= KXU * KTHREADS * 4, "%s: K=%d above %d", name, K, KXU * KTHREADS * 4);
    HM_REQUIRE(ctx, ((uintptr_t)d_w % 16) == 0 && ((uintptr_t)d_x % 16) == 0 && ((uintptr_t)d_norm_w % 16) == 0,
               "%s: weight, activation and norm buffers must be 16-byte aligned", name);
    HM_REQUIRE(ctx, !cand_v || (cand_i && M == 1), "%s: argmax candidates need an index buffer and one row", name);
    const size_t rowbytes = (size_t)(K / 256) * BB;
    HM_REQUIRE(ctx, KWAVES * rowbytes + 32 <= (size_t)KSTAGE_BYTES, "%s: K=%d too large for the LDS stage", name, K);
    const F32Shape sh = f32_shape<QT>(ctx, K, N, cand_v ? cand_cap : 0);
    const int rows = sh.rows, grid = sh.grid;
    const size_t stage_bytes = sh.stage_bytes, lds = sh.lds;
    HM_REQUIRE(ctx, grid >= 1, "%s: no room for argmax candidates", name);
    if (grid_out) *grid_out = grid;
    const int cpl = (K / 16 + WAVE - 1) / WAVE;
    for (int m = 0; m < M; m++) {
        const float *xm = d_x + (size_t)m * K;
        float *om = d_out + (size_t)m * N;
#define HM_KF_CASE(C)                                                                                                   \
    hipLaunchKernelGGL((gemv_kquant_f32_kernel<QT, C>), dim3(grid), dim3(KTHREADS), lds, ctx->stream, xm, d_norm_w, eps, \
                       d_w, om, K, N, rows, (int)stage_bytes, cand_v, cand_i)
        switch (cpl) {
            case 1: HM_KF_CASE(1); break;
            case 2: HM_KF_CASE(2); break;
            case 3: HM_KF_CASE(3); break;
            default: HM_KF_CASE(4); break;
        }
#undef HM_KF_CASE
        HM_LAUNCH_CHECK(ctx);
    }
    return HM_OK;
}

template <int QT>
int dequant_kquant_launch(hm_ctx *ctx, const char *name, const uint8_t *d_blocks, float *d_out, size_t nblocks) {
    HM_CHECK_CTX(ctx);
    if (nblocks == 0) return HM_OK;
    HM_REQUIRE(ctx, d_blocks && d_out, "%s: NULL pointer", name);
    const size_t n = nblocks * 256;
    size_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL((dequant_kquant_kernel<QT>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, d_blocks, d_out, n);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // namespace

int homura::gemv_kquant_fused(hm_ctx *ctx, bool q6, const float *d_x, const uint8_t *d_w, float *d_out, int K, int N,
                              const QuantFuse &fuse) {
    return q6 ? gemv_kquant_launch<1>(ctx, "gemv_kquant[q6_k]", d_x, d_w, d_out, 1, K, N, false, &fuse)
              : gemv_kquant_launch<0>(ctx, "gemv_kquant[q4_k]", d_x, d_w, d_out, 1, K, N, false, &fuse);
}

int homura::gemv_kquant_f32_head(hm_ctx *ctx, bool q6, const float *d_x, const float *d_norm_w, float eps,
                                 const uint8_t *d_w, float *d_out, int K, int N, float *cand_v, int *cand_i, int cand_cap) {
    return q6 ? gemv_kquant_f32_launch<1>(ctx, "gemv_q6_k_f32[head]", d_x, d_norm_w, eps, d_w, d_out, 1, K, N, cand_v, cand_i, cand_cap, nullptr)
              : gemv_kquant_f32_launch<0>(ctx, "gemv_q4_k_f32[head]", d_x, d_norm_w, eps, d_w, d_out, 1, K, N, cand_v, cand_i, cand_cap, nullptr);
}

int homura::gemv_kquant_f32_head_candidates(const hm_ctx *ctx, bool q6, int K, int N, int cand_cap) {
    return q6 ? f32_shape<1>(ctx, K, N, cand_cap).grid : f32_shape<0>(ctx, K, N, cand_cap).grid;
}

int homura::gemv_kquant_fused_pair(hm_ctx *ctx, bool first_q6, const float *d_x, const uint8_t *d_w, float *d_out, int N,
                                   const uint8_t *d_w2, float *d_out2, int N2, int K, const QuantFuse &fuse) {
    return first_q6 ? gemv_kquant_pair_launch<1>(ctx, "gemv_kquant[q6_k+q4_k]", d_x, d_w, d_out, N, d_w2, d_out2, N2, K, fuse)
                    : gemv_kquant_pair_launch<0>(ctx, "gemv_kquant[q4_k+q6_k]", d_x, d_w, d_out, N, d_w2, d_out2, N2, K, fuse);
}

int homura::gemv_kquant(hm_ctx *ctx, bool q6, const float *d_x, const uint8_t *d_w, float *d_out, int K, int N,
                        bool reuse_activation) {
    return q6 ? gemv_kquant_launch<1>(ctx, "gemv_kquant[q6_k]", d_x, d_w, d_out, 1, K, N, reuse_activation)
              : gemv_kquant_launch<0>(ctx, "gemv_kquant[q4_k]", d_x, d_w, d_out, 1, K, N, reuse_activation);
}

extern "C" {

int hm_gemv_q4_k(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M, int K, int N) {
    return gemv_kquant_launch<0>(ctx, "hm_gemv_q4_k", d_x, d_w_blocks, d_out, M, K, N);
}
int hm_gemv_q6_k(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M, int K, int N) {
    return gemv_kquant_launch<1>(ctx, "hm_gemv_q6_k", d_x, d_w_blocks, d_out, M, K, N);
}
int hm_gemv_q4_k_f32(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M, int K, int N) {
    return gemv_kquant_f32_launch<0>(ctx, "hm_gemv_q4_k_f32", d_x, nullptr, 0.f, d_w_blocks, d_out, M, K, N, nullptr, nullptr, 0, nullptr);
}
int hm_gemv_q6_k_f32(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M, int K, int N) {
    return gemv_kquant_f32_launch<1>(ctx, "hm_gemv_q6_k_f32", d_x, nullptr, 0.f, d_w_blocks, d_out, M, K, N, nullptr, nullptr, 0, nullptr);
}
int hm_dequant_q4_k(hm_ctx *ctx, const uint8_t *d_blocks, float *d_out, size_t nblocks) {
    return dequant_kquant_launch<0>(ctx, "hm_dequant_q4_k", d_blocks, d_out, nblocks);
}
int hm_dequant_q6_k(hm_ctx *ctx, const uint8_t *d_blocks, float *d_out, size_t nblocks) {
    return dequant_kquant_launch<1>(ctx, "hm_dequant_q6_k", d_blocks, d_out, nblocks);
}
int hm_quantize_q8_k(hm_ctx *ctx, const float *d_x, int8_t *d_q8, float *d_act_d, int32_t *d_bsums, int M, int K) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x && d_q8 && d_act_d && d_bsums, "hm_quantize_q8_k: NULL pointer");
    HM_REQUIRE(ctx, M >= 1 && K > 0 && K % 256 == 0, "hm_quantize_q8_k: need M >= 1 and K a positive multiple of 256");
    HM_REQUIRE(ctx, ((uintptr_t)d_x % 16) == 0 && ((uintptr_t)d_q8 % 4) == 0, "hm_quantize_q8_k: misaligned buffer");
    return quantize_launch(ctx, d_x, d_q8, d_act_d, d_bsums, M, K);
}

}  // extern "C"
