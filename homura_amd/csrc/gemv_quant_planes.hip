// Q8_0 / Q4_0 dequant-GEMV over weights re-packed once, at upload, into two planes: the quant bytes
// of all blocks, row after row (Q8_0: K bytes a row; Q4_0: K / 2, each block's 16 bytes of nibble
// pairs as they are in the file), then the f16 scales of all blocks, row after row. Same bytes as the
// GGUF blocks (reference src/hf/weights.rs:136-194 keeps them raw; src/graph_builder/emit_quant.rs:17-21
// layout), but every quant word sits at its natural alignment, so a lane loads its words straight
// from global memory into registers: no LDS stage, no two-byte LDS reads, no funnel shifts.
//
// A lane's unit of work is a quarter block (8 weights = 8 quant bytes for Q8_0, one 32-bit word of
// nibble pairs for Q4_0) plus the block's scale; quarter columns are dealt to the lanes round-robin as
// in gemv_quant.hip, and the arithmetic is that kernel's: d * (sum_j q_j x_j - offset * sum_j x_j) with
// the quants used as stored. A wavefront walks the rows in trips of RB rows, the loads of the next
// trip in flight while this one is multiplied.
#include "gemv_quant_planes.h"

#include <algorithm>

#include "hm_common.h"
#include "quant_formats.h"

namespace {

using homura::QuantFuse;

constexpr int PTHREADS = 256;
constexpr int PWAVES = PTHREADS / WAVE;

template <int QT>
struct PlaneTraits;
template <>
struct PlaneTraits<0> {  // Q8_0
    static constexpr int QBYTES = 8;  // quant bytes of a quarter block
    static constexpr int BLOCK = 34;
};
template <>
struct PlaneTraits<1> {  // Q4_0
    static constexpr int QBYTES = 4;
    static constexpr int BLOCK = 18;
};

// The four bytes of w as floats against xv. The empty asm keeps the compiler from folding the mask that
// produced w into one bit-field extract per byte: on a masked dword the four conversions select their
// byte themselves (v_cvt_f32_ubyte0..3), one instruction a weight instead of two.
__device__ __forceinline__ float dot4_bytes(uint32_t w, const float *xv, float s) {
    asm("" : "+v"(w));
    s = fmaf((float)(w & 0xFFu), xv[0], s);
    s = fmaf((float)((w >> 8) & 0xFFu), xv[1], s);
    s = fmaf((float)((w >> 16) & 0xFFu), xv[2], s);
    s = fmaf((float)(w >> 24), xv[3], s);
    return s;
}

// A masked dword of nibbles (each byte 0..15) as four floats, two conversions instead of four: read as
// OCP FP8 E4M3 a byte 0000nnnn is n * 2^-9 whether n falls in the subnormal range (n < 8: 2^-6 * n / 8) or in
// the first binade (n >= 8: 2^-6 * (1 + (n - 8) / 8)), and v_cvt_pk_f32_fp8 converts two bytes at a time,
// exactly. The activations carry the factor 2^9 (exact as well), so the products are those of n.
constexpr float NIBBLE_FP8_UNIT = 512.0f;
__device__ __forceinline__ float dot4_nibbles(uint32_t w, const float *xs512, float s) {
    const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    const auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    s = fmaf(lo[0], xs512[0], s);
    s = fmaf(lo[1], xs512[1], s);
    s = fmaf(hi[0], xs512[2], s);
    s = fmaf(hi[1], xs512[3], s);
    return s;
}

// Activations of quarter column c (block c / 4, quarter c % 4) in the order the quant bytes use them,
// and offset * their sum. Q4_0: the activations come back multiplied by 2^9 for dot4_nibbles.
template <int QT>
__device__ __forceinline__ void load_xv(const float *xs, int c, float *xv, float &sx_off) {
    const int b = c >> 2, q = c & 3;
    const float *p0 = xs + b * 32 + (QT == 0 ? q * 8 : q * 4);
    const float *p1 = QT == 0 ? p0 + 4 : p0 + 16;
    const f32x4 lo = *reinterpret_cast<const f32x4 *>(p0);
    const f32x4 hi = *reinterpret_cast<const f32x4 *>(p1);
    xv[0] = lo.x; xv[1] = lo.y; xv[2] = lo.z; xv[3] = lo.w;
    xv[4] = hi.x; xv[5] = hi.y; xv[6] = hi.z; xv[7] = hi.w;
    float sx = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) sx += xv[j];
    sx_off = sx * (QT == 0 ? 128.f : 8.f);
    if (QT == 1) {
#pragma unroll
        for (int j = 0; j < 8; j++) xv[j] *= NIBBLE_FP8_UNIT;
    }
}

// The quant words of one quarter: Q8_0 two dwords, Q4_0 one.
template <int QT>
struct QWords {
    uint32_t w0, w1;
};

typedef const uint32_t __attribute__((address_space(1))) *global_u32_ptr;
typedef const u32x2 __attribute__((address_space(1))) *global_u32x2_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;
typedef const u32x4 __attribute__((address_space(1))) *global_u32x4_ptr;

template <int QT>
__device__ __forceinline__ QWords<QT> load_quarter(const uint8_t *q) {
    QWords<QT> r;
    if (QT == 0) {
        const u32x2 v = __builtin_nontemporal_load((global_u32x2_ptr)q);
        r.w0 = v.x;
        r.w1 = v.y;
    } else {
        r.w0 = __builtin_nontemporal_load((global_u32_ptr)q);
        r.w1 = 0u;
    }
    return r;
}

template <int QT>
__device__ __forceinline__ float quarter_value(const QWords<QT> &w, uint32_t scale_bits, const float *xv, float sx_off) {
    const float d = f16_bits_to_f32((uint16_t)scale_bits);
    float s;
    if (QT == 0) {
        s = dot4_bytes(w.w1 ^ 0x80808080u, xv + 4, dot4_bytes(w.w0 ^ 0x80808080u, xv, 0.f));  // int8 -> biased unsigned
    } else {
        // byte i of the word: low nibble = weight 4q + i, high nibble = weight 16 + 4q + i
        s = dot4_nibbles((w.w0 >> 4) & 0x0F0F0F0Fu, xv + 4, dot4_nibbles(w.w0 & 0x0F0F0F0Fu, xv, 0.f));
    }
    return d * (s - sx_off);
}

// CPL = quarter columns per lane (ceil(K / 8 / 64)); RB = rows per trip of a wavefront.
template <int QT, int CPL, int RB, bool FUSED>
__global__ __launch_bounds__(PTHREADS) void gemv_planes_kernel(const float *__restrict__ x, const uint8_t *__restrict__ quants,
                                                               const uint16_t *__restrict__ scales, float *__restrict__ out,
                                                               int K, int N, const QuantFuse fuse_arg) {
    const QuantFuse fuse = FUSED ? fuse_arg : QuantFuse();
    constexpr int QB = PlaneTraits<QT>::QBYTES;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    float *xs = reinterpret_cast<float *>(smem);
    float *red = xs + K;  // [PWAVES] sums of squares, later the wavefronts' argmax candidates
    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);  // uniform: row addresses stay in scalar registers
    const int nb = K / 32, nq = K / 8;
    const size_t qrow = (size_t)nq * QB;

    // this wavefront's trips: rows (trip * total waves + global wave) * RB ...
    const int gw = blockIdx.x * PWAVES + wave, nwaves = gridDim.x * PWAVES;
    const int ntrips = (N + RB - 1) / RB;
    QWords<QT> qn[RB][CPL];
    uint32_t sn[RB][CPL];
    uint32_t qoff[CPL], soff[CPL];  // byte offsets of the lane's quarters / element offsets of their scales in a row
    int col[CPL];
    bool live[CPL];
#pragma unroll
    for (int t = 0; t < CPL; t++) {
        live[t] = lane + t * WAVE < nq;
        col[t] = live[t] ? lane + t * WAVE : nq - 1;  // lanes past the row end re-read its last column ...
        qoff[t] = (uint32_t)col[t] * QB;
        soff[t] = (uint32_t)col[t] >> 2;
    }
    auto request = [&](int trip) {
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const int row = min(trip * RB + r, N - 1);  // rows past the end re-read the last one
            const uint8_t *qr = quants + (size_t)row * qrow;
            const uint16_t *sr = scales + (size_t)row * nb;
#pragma unroll
            for (int t = 0; t < CPL; t++) {
                qn[r][t] = load_quarter<QT>(qr + qoff[t]);
                sn[r][t] = __builtin_nontemporal_load((global_u16_ptr)(sr + soff[t]));
            }
        }
    };

    // Loads return in issue order: the (small, cached) activation loads go first, the first trip's
    // weights right behind them, so staging the activations does not wait for HBM.
    constexpr int XU = 4;  // covers K <= 4096 in one round
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 xr[XU], ar[XU], nr[XU];  // activation; second operand (x2 or res_in); norm weight
    const float *second = fuse.x2 ? fuse.x2 : fuse.res_in;
#pragma unroll
    for (int u = 0; u < XU; u++) {
        const int k = (tid + u * PTHREADS) * 4;
        xr[u] = k < K ? *reinterpret_cast<const f32x4 *>(x + k) : zero4;
        ar[u] = second && k < K ? *reinterpret_cast<const f32x4 *>(second + k) : zero4;
        nr[u] = fuse.norm_w && k < K ? *reinterpret_cast<const f32x4 *>(fuse.norm_w + k) : zero4;
    }
    int trip = gw;
    if (trip < ntrips) request(trip);
    // the light ops of the quantised plan that sit in front of this product (reference
    // src/hf/emitter_quant.rs:713-791, :985-1071, :1077-1103); the host allows the norm only for
    // K <= XU * 1024, where the whole row is in xr
    if (fuse.x2) {
#pragma unroll
        for (int u = 0; u < XU; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) xr[u][e] = (xr[u][e] / (1.0f + expf(-xr[u][e]))) * ar[u][e];
    } else if (fuse.res_in) {
#pragma unroll
        for (int u = 0; u < XU; u++) {
            xr[u] += ar[u];
            const int k = (tid + u * PTHREADS) * 4;
            if (fuse.resid_out && blockIdx.x == 0 && k < K) *reinterpret_cast<f32x4 *>(fuse.resid_out + k) = xr[u];
        }
    }
    if (fuse.norm_w) {
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < XU; u++) ss += (xr[u][0] * xr[u][0] + xr[u][1] * xr[u][1]) + (xr[u][2] * xr[u][2] + xr[u][3] * xr[u][3]);
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weight loads stay in flight
        float tot = 0.f;
#pragma unroll
        for (int wv = 0; wv < PWAVES; wv++) tot += red[wv];
        const float inv = 1.0f / sqrtf(tot / (float)K + fuse.eps);
#pragma unroll
        for (int u = 0; u < XU; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) xr[u][e] = (xr[u][e] * inv) * nr[u][e];
    }
#pragma unroll
    for (int u = 0; u < XU; u++) {
        const int k = (tid + u * PTHREADS) * 4;
        if (k < K) *reinterpret_cast<f32x4 *>(xs + k) = xr[u];
    }
    for (int k = (tid + XU * PTHREADS) * 4; k < K; k += PTHREADS * 4) {  // longer rows (no norm here)
        f32x4 v = *reinterpret_cast<const f32x4 *>(x + k);
        if (fuse.x2) {
            const f32x4 o = *reinterpret_cast<const f32x4 *>(fuse.x2 + k);
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = (v[e] / (1.0f + expf(-v[e]))) * o[e];
        } else if (fuse.res_in) {
            v += *reinterpret_cast<const f32x4 *>(fuse.res_in + k);
            if (fuse.resid_out && blockIdx.x == 0) *reinterpret_cast<f32x4 *>(fuse.resid_out + k) = v;
        }
        *reinterpret_cast<f32x4 *>(xs + k) = v;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    float xv[CPL][8], sxo[CPL];
#pragma unroll
    for (int t = 0; t < CPL; t++) {
        load_xv<QT>(xs, col[t], xv[t], sxo[t]);
        if (!live[t]) {  // ... against activations of zero, so they add nothing
#pragma unroll
            for (int j = 0; j < 8; j++) xv[t][j] = 0.f;
            sxo[t] = 0.f;
        }
    }

    float best_v = -INFINITY;
    int best_i = -1;
    for (; trip < ntrips; trip += nwaves) {
        QWords<QT> qc[RB][CPL];
        uint32_t sc[RB][CPL];
#pragma unroll
        for (int r = 0; r < RB; r++)
#pragma unroll
            for (int t = 0; t < CPL; t++) {
                qc[r][t] = qn[r][t];
                sc[r][t] = sn[r][t];
            }
        if (trip + nwaves < ntrips) request(trip + nwaves);  // the next trip travels while this one is multiplied
        float a[RB];
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] = 0.f;
#pragma unroll
        for (int t = 0; t < CPL; t++)
#pragma unroll
            for (int r = 0; r < RB; r++) {
                a[r] += quarter_value<QT>(qc[r][t], sc[r][t], xv[t], sxo[t]);
            }
        // wave sums of the RB rows, the chains stepping side by side
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0xB1, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x4E, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x141, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x140, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x142, 0xA>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x143, 0xC>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const int row = trip * RB + r;
            float v = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(a[r]), 63));
            if (row < N) {
                if (fuse.res_out_add) v = v + fuse.res_out_add[row];
                if (lane == 0) out[row] = v;
                // of equal maxima the later row wins (Rust Iterator::max_by, reference src/generate.rs:735-742)
                if (best_i < 0 || v > best_v || (v == best_v && row > best_i)) {
                    best_v = v;
                    best_i = row;
                }
            }
        }
    }
    if (fuse.cand_v) {  // the workgroup's best row: largest value, highest index among equals; -1 = no row
        __syncthreads();
        float *cv = red;
        int *ci = reinterpret_cast<int *>(red) + PWAVES;
        if (lane == 0) {
            cv[wave] = best_v;
            ci[wave] = best_i;
        }
        __syncthreads();
        if (tid == 0) {
            float bv = -INFINITY;
            int bi = -1;
            for (int wv = 0; wv < PWAVES; wv++) {
                if (ci[wv] < 0) continue;
                if (bi < 0 || cv[wv] > bv || (cv[wv] == bv && ci[wv] > bi)) {
                    bv = cv[wv];
                    bi = ci[wv];
                }
            }
            fuse.cand_v[blockIdx.x] = bv;
            fuse.cand_i[blockIdx.x] = bi;
        }
    }
}

// Rows cut across the wavefronts of a workgroup, for rows longer than gemv_planes_kernel keeps in registers
// (K > 4096: the down projection of models with wide MLPs) and for matrices of few rows. A workgroup owns R
// rows; a lane's unit is 16 bytes of a row's quant plane (Q8_0: half a block, Q4_0: a whole block) and its
// scale, a wavefront's chunk 64 units, the four wavefronts take a row's chunks in turn, NC each. Every load is
// requested before anything waits, the activation pieces first; the light ops in front of the product
// (SiLU pair, residual add) are applied to the pieces in registers; the four partial sums of a row meet in
// LDS and are added in wavefront order. No RMSNorm here (rows that long are normalised by their own launch).
// MODE 0: plain row. 1: a second operand (x2 or res_in). 2: RMSNorm, with or without res_in.
template <int QT, int R, int NC, int MODE, int WPS>
__global__ __launch_bounds__(PTHREADS) void gemv_planes_splitk_kernel(const float *__restrict__ x, const uint8_t *__restrict__ quants,
                                                                      const uint16_t *__restrict__ scales, float *__restrict__ out,
                                                                      int K, int N, const QuantFuse fuse_arg) {
    constexpr bool FUSED = MODE >= 1;
    const QuantFuse fuse = FUSED ? fuse_arg : QuantFuse();
    constexpr int KPL = QT == 0 ? 16 : 32, XV = KPL / 4;  // weights and f32x4 activation pieces of a unit
    __shared__ float part[PWAVES][R];
    __shared__ float red[PWAVES];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    // WPS wavefronts (as many as a row has chunks, so that none idles) share a set of R rows; a workgroup works
    // on PWAVES / WPS sets
    constexpr int SETS = PWAVES / WPS;
    const int set = wave / WPS, wis = wave % WPS;
    const int row0 = (blockIdx.x * SETS + set) * R;
    const size_t qrow = QT == 0 ? (size_t)K : (size_t)K / 2;
    const int nb = K / 32;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 xr[NC][XV], ar[FUSED ? NC : 1][FUSED ? XV : 1], nr[MODE == 2 ? NC : 1][MODE == 2 ? XV : 1];
    u32x4 qw[NC][R];
    uint32_t sc[NC][R];
    const float *second = fuse.x2 ? fuse.x2 : fuse.res_in;
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int k = ((c * WPS + wis) * WAVE + lane) * KPL;
#pragma unroll
        for (int j = 0; j < XV; j++) {
            xr[c][j] = k < K ? *reinterpret_cast<const f32x4 *>(x + k + 4 * j) : zero4;
            if constexpr (FUSED) ar[c][j] = (second && k < K) ? *reinterpret_cast<const f32x4 *>(second + k + 4 * j) : zero4;
            if constexpr (MODE == 2) nr[c][j] = (fuse.norm_w && k < K) ? *reinterpret_cast<const f32x4 *>(fuse.norm_w + k + 4 * j) : zero4;
        }
    }
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const int k = ((c * WPS + wis) * WAVE + lane) * KPL;
        const int kc = k < K ? k : 0;  // units past the row end re-read its first one against activations of zero
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = min(row0 + r, N - 1);  // rows past the end re-read the last one
            qw[c][r] = __builtin_nontemporal_load((global_u32x4_ptr)(quants + (size_t)row * qrow + (QT == 0 ? kc : kc / 2)));
            sc[c][r] = __builtin_nontemporal_load((global_u16_ptr)(scales + (size_t)row * nb + kc / 32));
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // every request above goes out before any arithmetic below
    // the light ops of the quantised plan in front of this product (reference src/hf/emitter_quant.rs:985-1103)
    if constexpr (FUSED) {
        if (fuse.x2) {
#pragma unroll
            for (int c = 0; c < NC; c++)
#pragma unroll
                for (int j = 0; j < XV; j++)
#pragma unroll
                    for (int e = 0; e < 4; e++) xr[c][j][e] = (xr[c][j][e] / (1.0f + expf(-xr[c][j][e]))) * ar[c][j][e];
        } else if (fuse.res_in) {
#pragma unroll
            for (int c = 0; c < NC; c++) {
                const int k = ((c * WPS + wis) * WAVE + lane) * KPL;
#pragma unroll
                for (int j = 0; j < XV; j++) {
                    xr[c][j] += ar[c][j];
                    if (fuse.resid_out && blockIdx.x == 0 && set == 0 && k < K) *reinterpret_cast<f32x4 *>(fuse.resid_out + k + 4 * j) = xr[c][j];
                }
            }
        }
    }
    if constexpr (MODE == 2) {
        // RMSNorm on the pieces: the set's wavefronts cover the row exactly once, their sums of squares meet in LDS
        if (fuse.norm_w) {
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < NC; c++)
#pragma unroll
                for (int j = 0; j < XV; j++)
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
                for (int j = 0; j < XV; j++)
#pragma unroll
                    for (int e = 0; e < 4; e++) xr[c][j][e] = (xr[c][j][e] * inv) * nr[c][j][e];
        }
    }
    float a[R];
#pragma unroll
    for (int r = 0; r < R; r++) a[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; c++) {
        float xv[KPL], sx = 0.f;
#pragma unroll
        for (int j = 0; j < XV; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                xv[4 * j + e] = xr[c][j][e];
                sx += xr[c][j][e];
            }
        const float sx_off = sx * (QT == 0 ? 128.f : 8.f);
        if (QT == 1) {
#pragma unroll
            for (int j = 0; j < KPL; j++) xv[j] *= NIBBLE_FP8_UNIT;
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float d = f16_bits_to_f32((uint16_t)sc[c][r]);
            const uint32_t w[4] = {qw[c][r].x, qw[c][r].y, qw[c][r].z, qw[c][r].w};
            float t = 0.f;
            if (QT == 0) {
#pragma unroll
                for (int i = 0; i < 4; i++) t = dot4_bytes(w[i] ^ 0x80808080u, xv + 4 * i, t);  // int8 -> biased unsigned
            } else {
                // byte i of the block's 16: low nibble = weight i, high nibble = weight 16 + i
#pragma unroll
                for (int i = 0; i < 4; i++) t = dot4_nibbles(w[i] & 0x0F0F0F0Fu, xv + 4 * i, t);
#pragma unroll
                for (int i = 0; i < 4; i++) t = dot4_nibbles((w[i] >> 4) & 0x0F0F0F0Fu, xv + 16 + 4 * i, t);
            }
            a[r] += d * (t - sx_off);
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
    if (t < SETS * R) {
        const int ts = t / R, tr = t % R, row = (blockIdx.x * SETS + ts) * R + tr;
        if (row < N) {
            float v = part[ts * WPS][tr];
#pragma unroll
            for (int w = 1; w < WPS; w++) v += part[ts * WPS + w][tr];
            if (fuse.res_out_add) v = v + fuse.res_out_add[row];
            out[row] = v;
        }
    }
}

// raw GGUF blocks [N][K / 32] -> planes; one thread per quarter block
template <int QT>
__global__ __launch_bounds__(256) void pack_planes_kernel(const uint8_t *__restrict__ blocks, uint8_t *__restrict__ quants,
                                                          uint16_t *__restrict__ scales, size_t n_quarters) {
    constexpr int QB = PlaneTraits<QT>::QBYTES, BB = PlaneTraits<QT>::BLOCK;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_quarters) return;
    const size_t b = i >> 2;
    const int q = (int)(i & 3);
    const uint8_t *blk = blocks + b * BB;
    if (q == 0) scales[b] = (uint16_t)(blk[0] | (blk[1] << 8));
#pragma unroll
    for (int j = 0; j < QB; j++) quants[i * QB + j] = blk[2 + q * QB + j];
}

// Q4_0, tall matrices (the LM-head shape), no fused light ops: a lane's unit is half a block. A trip is two
// rows; their 4 * K / 32 half blocks lie one after the other in the quant plane, so lane l takes halves l,
// l + 64, ... of the trip with one 8-byte and one 2-byte load each: half the load instructions of the
// quarter-block kernel above, one scale conversion per 16 weights instead of 8, and the half's 16 activations
// (times 2^9) stay in registers for every trip. A row's halves are spread over the lanes (and over a lane's
// units), so the two row sums are masked wave sums. Needs K / 32 a multiple of 16 (the trip then is UPL * 64
// halves) and UPL <= 4. (Whole blocks per lane, four rows a trip: 144 registers, three workgroups a CU, slower.)
template <int UPL>
__global__ __launch_bounds__(PTHREADS) void gemv_q4_0_halves_kernel(const float *__restrict__ x, const uint8_t *__restrict__ quants,
                                                                    const uint16_t *__restrict__ scales, float *__restrict__ out,
                                                                    int K, int N) {
    constexpr int RB = 2;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    float *xs = reinterpret_cast<float *>(smem);
    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int nb = K / 32;  // == UPL * 16
    const int gw = blockIdx.x * PWAVES + wave, nwaves = gridDim.x * PWAVES;
    const int ntrips = (N + RB - 1) / RB;
    // this lane's units: row (within the trip), block (within the row) and half (within the block) of unit u
    int urow[UPL], ublk[UPL], uhalf[UPL];
#pragma unroll
    for (int u = 0; u < UPL; u++) {
        const int f = u * WAVE + lane;
        urow[u] = f / (2 * nb);
        ublk[u] = (f % (2 * nb)) >> 1;
        uhalf[u] = f & 1;
    }
    // D trips of a wavefront are in flight at a time (1.7 KB each at K = 1536): with one, the sixteen wavefronts
    // of a CU have 27 KB outstanding (30.8 us at the 1536 -> 151936 shape), with four 29.2 us; six cost a
    // workgroup of occupancy and bring nothing.
    constexpr int D = 4;
    u32x2 qn[D][UPL];
    uint32_t sn[D][UPL];
    auto request = [&](u32x2(&q)[UPL], uint32_t(&sc)[UPL], int trip) {
#pragma unroll
        for (int u = 0; u < UPL; u++) {
            const int row = min(trip * RB + urow[u], N - 1);  // rows past the end re-read the last one
            const size_t blk = (size_t)row * nb + ublk[u];
            q[u] = __builtin_nontemporal_load((global_u32x2_ptr)(quants + blk * 16 + uhalf[u] * 8));
            sc[u] = __builtin_nontemporal_load((global_u16_ptr)(scales + blk));
        }
    };
    // activations first (loads return in issue order), the first trip's weights right behind them
    f32x4 xr[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int k = (tid + u * PTHREADS) * 4;
        xr[u] = k < K ? *reinterpret_cast<const f32x4 *>(x + k) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    int trip = gw;  // the trip in buffer 0; buffer d holds trip + d * nwaves
#pragma unroll
    for (int d = 0; d < D; d++)
        if (trip + d * nwaves < ntrips) request(qn[d], sn[d], trip + d * nwaves);
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int k = (tid + u * PTHREADS) * 4;
        if (k < K) *reinterpret_cast<f32x4 *>(xs + k) = xr[u];
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weight loads stay in flight
    // byte j of a block holds weight j (low nibble) and weight 16 + j (high nibble); this half has bytes 8 h .. 8 h + 7
    float xlo[UPL][8], xhi[UPL][8], sx8[UPL];
#pragma unroll
    for (int u = 0; u < UPL; u++) {
        float sx = 0.f;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const f32x4 a = *reinterpret_cast<const f32x4 *>(xs + ublk[u] * 32 + uhalf[u] * 8 + 4 * j);
            const f32x4 b = *reinterpret_cast<const f32x4 *>(xs + ublk[u] * 32 + 16 + uhalf[u] * 8 + 4 * j);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                sx += a[e] + b[e];
                xlo[u][4 * j + e] = a[e] * NIBBLE_FP8_UNIT;
                xhi[u][4 * j + e] = b[e] * NIBBLE_FP8_UNIT;
            }
        }
        sx8[u] = sx * 8.f;
    }
    auto consume = [&](const u32x2(&qc)[UPL], const uint32_t(&sc)[UPL], int t) {
        float a[RB] = {0.f, 0.f};
#pragma unroll
        for (int u = 0; u < UPL; u++) {
            float s0 = 0.f, s1 = 0.f;  // two chains
#pragma unroll
            for (int j = 0; j < 2; j++) {
                s0 = dot4_nibbles(qc[u][j] & 0x0F0F0F0Fu, &xlo[u][4 * j], s0);
                s1 = dot4_nibbles((qc[u][j] >> 4) & 0x0F0F0F0Fu, &xhi[u][4 * j], s1);
            }
            const float v = f16_bits_to_f32((uint16_t)sc[u]) * ((s0 + s1) - sx8[u]);
#pragma unroll
            for (int r = 0; r < RB; r++) a[r] += urow[u] == r ? v : 0.f;
        }
        // wave sums of the two rows, the chains stepping side by side
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0xB1, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x4E, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x141, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x140, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x142, 0xA>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < RB; r++) a[r] += dpp_move<0x143, 0xC>(a[r], 0.f);
        // lane 63 holds the totals; it stores the rows
#pragma unroll
        for (int r = 0; r < RB; r++)
            if (lane == WAVE - 1 && t * RB + r < N) out[(size_t)t * RB + r] = a[r];
    };
    // steady state: every buffer is multiplied and asked for again, D trips on, with no condition in the way
    // (every wait then knows how many loads are behind the ones it needs)
    while (trip + (2 * D - 1) * nwaves < ntrips) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            consume(qn[d], sn[d], trip + d * nwaves);
            request(qn[d], sn[d], trip + (D + d) * nwaves);
        }
        trip += D * nwaves;
    }
    // what the buffers still hold, each asked for again at once where a trip is left for it (at most D - 1 are)
#pragma unroll
    for (int d = 0; d < D; d++)
        if (trip + d * nwaves < ntrips) {
            consume(qn[d], sn[d], trip + d * nwaves);
            if (trip + (D + d) * nwaves < ntrips) request(qn[d], sn[d], trip + (D + d) * nwaves);
        }
    trip += D * nwaves;
#pragma unroll
    for (int d = 0; d < D; d++)
        if (trip + d * nwaves < ntrips) consume(qn[d], sn[d], trip + d * nwaves);
}

// Q4_0, tall matrices, no fused light ops: a lane's unit is a whole block (one 16-byte and one 2-byte load for
// 32 weights). A trip is two runs of UPL * 64 consecutive blocks = 2 * RB whole rows; a lane takes the same block
// position in both runs, so the block's activations, which stay in LDS (times 2^9, a block's 32 floats 36
// apart so that the sixteen lanes of a 16-byte LDS read hit sixteen different bank groups), are read once
// for two blocks of weights. The registers hold only the trips in flight.
template <int UPL, int RB>
__global__ __launch_bounds__(PTHREADS) void gemv_q4_0_blocks_kernel(const float *__restrict__ x, const uint8_t *__restrict__ quants,
                                                                    const uint16_t *__restrict__ scales, float *__restrict__ out,
                                                                    int K, int N) {
    constexpr int XPAD = 36, TR = 2 * RB;  // rows of a trip
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    float *xs = reinterpret_cast<float *>(smem);  // [nb][XPAD]: 32 activations * 2^9, then 8 * their sum
    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int nb = K / 32;  // == UPL * 64 / RB
    const int gw = blockIdx.x * PWAVES + wave, nwaves = gridDim.x * PWAVES;
    const int ntrips = (N + TR - 1) / TR;
    int urow[UPL], ublk[UPL];
#pragma unroll
    for (int u = 0; u < UPL; u++) {
        const int f = u * WAVE + lane;
        urow[u] = f / nb;
        ublk[u] = f % nb;
    }
    constexpr int D = 2;  // trips of a wavefront in flight
    u32x4 qn[D][2][UPL];
    uint32_t sn[D][2][UPL];
    auto request = [&](u32x4(&q)[2][UPL], uint32_t(&sc)[2][UPL], int trip) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int u = 0; u < UPL; u++) {
                const int row = min(trip * TR + h * RB + urow[u], N - 1);  // rows past the end re-read the last one
                const size_t blk = (size_t)row * nb + ublk[u];
                q[h][u] = ld128_stream(quants + blk * 16);
                sc[h][u] = __builtin_nontemporal_load((global_u16_ptr)(scales + blk));
            }
    };
    // activations first (loads return in issue order), the first trips' weights right behind them
    f32x4 xr[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int k = (tid + u * PTHREADS) * 4;
        xr[u] = k < K ? *reinterpret_cast<const f32x4 *>(x + k) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    int trip = gw;  // the trip in buffer 0; buffer d holds trip + d * nwaves
#pragma unroll
    for (int d = 0; d < D; d++)
        if (trip + d * nwaves < ntrips) request(qn[d], sn[d], trip + d * nwaves);
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int k = (tid + u * PTHREADS) * 4;
        if (k < K) *reinterpret_cast<f32x4 *>(xs + (k >> 5) * XPAD + (k & 31)) = xr[u] * NIBBLE_FP8_UNIT;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weight loads stay in flight
    for (int b = tid; b < nb; b += PTHREADS) {
        float sx = 0.f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(xs + b * XPAD + 4 * j);
            sx += (v.x + v.y) + (v.z + v.w);
        }
        xs[b * XPAD + 32] = sx * (8.f / NIBBLE_FP8_UNIT);
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    auto consume = [&](const u32x4(&qc)[2][UPL], const uint32_t(&sc)[2][UPL], int t) {
        float a[TR];
#pragma unroll
        for (int r = 0; r < TR; r++) a[r] = 0.f;
#pragma unroll
        for (int u = 0; u < UPL; u++) {
            int xoff = ublk[u] * XPAD;
            asm volatile("" : "+v"(xoff));  // read again in every trip: hoisted out of the loop the activations would fill the registers
            const float *xb = xs + xoff;
            float s[2][2] = {{0.f, 0.f}, {0.f, 0.f}};  // two chains a block
#pragma unroll
            for (int j = 0; j < 4; j++) {  // byte i of word j: low nibble = weight 4 j + i, high nibble = weight 16 + 4 j + i
                const f32x4 lo = *reinterpret_cast<const f32x4 *>(xb + 4 * j);
                const f32x4 hi = *reinterpret_cast<const f32x4 *>(xb + 16 + 4 * j);
                const float xl[4] = {lo.x, lo.y, lo.z, lo.w}, xh[4] = {hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    s[h][0] = dot4_nibbles(qc[h][u][j] & 0x0F0F0F0Fu, xl, s[h][0]);
                    s[h][1] = dot4_nibbles((qc[h][u][j] >> 4) & 0x0F0F0F0Fu, xh, s[h][1]);
                }
            }
            const float sx8 = xb[32];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const float v = f16_bits_to_f32((uint16_t)sc[h][u]) * ((s[h][0] + s[h][1]) - sx8);
#pragma unroll
                for (int r = 0; r < RB; r++) a[h * RB + r] += (RB == 1 || urow[u] == r) ? v : 0.f;
            }
        }
#pragma unroll
        for (int r = 0; r < TR; r++) a[r] += dpp_move<0xB1, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < TR; r++) a[r] += dpp_move<0x4E, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < TR; r++) a[r] += dpp_move<0x141, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < TR; r++) a[r] += dpp_move<0x140, 0xF>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < TR; r++) a[r] += dpp_move<0x142, 0xA>(a[r], 0.f);
#pragma unroll
        for (int r = 0; r < TR; r++) a[r] += dpp_move<0x143, 0xC>(a[r], 0.f);
        // lane 63 holds the totals; it stores the rows
#pragma unroll
        for (int r = 0; r < TR; r++)
            if (lane == WAVE - 1 && t * TR + r < N) out[(size_t)t * TR + r] = a[r];
    };
    // steady state: every buffer is multiplied and asked for again, D trips on, with no condition in the way
    while (trip + (2 * D - 1) * nwaves < ntrips) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            consume(qn[d], sn[d], trip + d * nwaves);
            request(qn[d], sn[d], trip + (D + d) * nwaves);
        }
        trip += D * nwaves;
    }
#pragma unroll
    for (int d = 0; d < D; d++)
        if (trip + d * nwaves < ntrips) {
            consume(qn[d], sn[d], trip + d * nwaves);
            if (trip + (D + d) * nwaves < ntrips) request(qn[d], sn[d], trip + (D + d) * nwaves);
        }
    trip += D * nwaves;
#pragma unroll
    for (int d = 0; d < D; d++)
        if (trip + d * nwaves < ntrips) consume(qn[d], sn[d], trip + d * nwaves);
}

// planes -> raw blocks (the inverse, for checks)
template <int QT>
__global__ __launch_bounds__(256) void unpack_planes_kernel(const uint8_t *__restrict__ quants, const uint16_t *__restrict__ scales,
                                                            uint8_t *__restrict__ blocks, size_t n_quarters) {
    constexpr int QB = PlaneTraits<QT>::QBYTES, BB = PlaneTraits<QT>::BLOCK;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_quarters) return;
    const size_t b = i >> 2;
    const int q = (int)(i & 3);
    uint8_t *blk = blocks + b * BB;
    if (q == 0) {
        blk[0] = (uint8_t)(scales[b] & 0xFF);
        blk[1] = (uint8_t)(scales[b] >> 8);
    }
#pragma unroll
    for (int j = 0; j < QB; j++) blk[2 + q * QB + j] = quants[i * QB + j];
}

// One thread per element, the reference's one multiply (src/gguf.rs:825-829), read from the planes.
template <int QT>
__global__ __launch_bounds__(256) void dequant_planes_kernel(const uint8_t *__restrict__ quants, const uint16_t *__restrict__ scales,
                                                             float *__restrict__ out, size_t n_elems) {
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; e < n_elems; e += stride) {
        const size_t b = e >> 5;
        const int j = (int)(e & 31);
        const float d = f16_bits_to_f32(scales[b]);
        float q;
        if (QT == 0) {
            q = (float)(int8_t)quants[e];
        } else {
            const uint8_t byte = quants[b * 16 + (j & 15)];
            q = (float)((j < 16 ? (byte & 0x0F) : (byte >> 4)) - 8);
        }
        out[e] = __fmul_rn(q, d);
    }
}

// Rows per trip for C quarter columns per lane: two trips live in registers (this one and the next), and
// four workgroups should fit a CU, so the longer the rows the fewer of them; a power of two up to 8.
template <int QT, int C>
struct TripRows {
    static constexpr int CAP = 12 / C;
    static constexpr int MOST = CAP >= 8 ? 8 : (CAP >= 4 ? 4 : (CAP >= 2 ? 2 : 1));
};

constexpr int planes_cpl_instance(int cpl) {  // the kernel instance that serves cpl quarter columns per lane
    return cpl <= 4 ? cpl : (cpl <= 6 ? 6 : 8);
}

struct PlanesShape {
    int rb, grid;
    size_t lds;
};

PlanesShape planes_shape(const hm_ctx *ctx, bool q4, int K, int N) {
    PlanesShape s;
    const int c = planes_cpl_instance((K / 8 + WAVE - 1) / WAVE);
    const int cap = 12 / c;
    const int most = cap >= 8 ? 8 : (cap >= 4 ? 4 : (cap >= 2 ? 2 : 1));
    // long trips where there are rows enough to give every CU two workgroups of them, else single rows
    (void)q4;
    s.rb = (N + most - 1) / most >= 2 * PWAVES * ctx->num_cus ? most : 1;
    const int ntrips = (N + s.rb - 1) / s.rb;
    const int want = (ntrips + PWAVES - 1) / PWAVES;
    const int persistent = 4 * ctx->num_cus;  // four workgroups a CU: measured better than two with trips twice as long
    s.grid = want < persistent ? want : persistent;
    if (s.grid < 1) s.grid = 1;
    s.lds = (size_t)K * 4 + 2 * PWAVES * 4 + 16;
    return s;
}

template <int QT>
int planes_launch(hm_ctx *ctx, const char *name, const float *d_x, const uint8_t *d_planes, float *d_out, int M, int K, int N,
                  const QuantFuse &fuse) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x && d_planes && d_out, "%s: NULL pointer", name);
    HM_REQUIRE(ctx, M >= 1 && M <= 8, "%s: M=%d outside 1..8", name, M);
    HM_REQUIRE(ctx, K > 0 && K % 32 == 0 && K <= 16384 && N > 0, "%s: K=%d must be a multiple of 32 up to 16384, N=%d positive", name, K, N);
    HM_REQUIRE(ctx, ((uintptr_t)d_planes % 16) == 0 && ((uintptr_t)d_x % 16) == 0, "%s: weight and activation buffers must be 16-byte aligned", name);
    HM_REQUIRE(ctx, !(fuse.x2 && fuse.res_in), "%s: SiLU pair and residual input exclude each other", name);
    HM_REQUIRE(ctx, !fuse.norm_w || K <= 4096, "%s: the fused RMSNorm holds rows up to 4096 wide (K=%d)", name, K);
    HM_REQUIRE(ctx, ((uintptr_t)fuse.x2 % 16) == 0 && ((uintptr_t)fuse.res_in % 16) == 0 && ((uintptr_t)fuse.resid_out % 16) == 0 &&
                        ((uintptr_t)fuse.norm_w % 16) == 0, "%s: fused operands must be 16-byte aligned", name);
    HM_REQUIRE(ctx, M == 1 || (!fuse.x2 && !fuse.res_in && !fuse.norm_w && !fuse.res_out_add), "%s: fused light ops need M == 1", name);
    HM_REQUIRE(ctx, !fuse.cand_v || fuse.cand_i, "%s: argmax candidates need an index buffer", name);
    const bool q4 = QT == 1;
    const uint8_t *quants = d_planes;
    const uint16_t *scales = reinterpret_cast<const uint16_t *>(d_planes + homura::quant_planes_scale_offset(q4, N, K));
    const int cpl = (K / 8 + WAVE - 1) / WAVE;
    const bool fused = fuse.x2 || fuse.res_in || fuse.norm_w || fuse.res_out_add || fuse.cand_v;
    // rows longer than the kernels below hold: cut across the wavefronts of a workgroup
    static const bool force_cut = [] {
        const char *e = getenv("HOMURA_PLANES_SPLITK");
        return e && atoi(e) != 0;
    }();
    // ... and Q8_0 matrices of fewer than 32768 rows at any width (2048 -> 5632: 4.6 us against 5.3; Q4_0 rows up to
    // 4096 and the LM heads measured no faster that way), with an RMSNorm riding in up to 16 M weights (beyond,
    // the trips of gemv_planes_kernel, which prepares the row once per workgroup, are faster)
    if ((K > 4096 || force_cut || (!q4 && N < 32768)) && !(fuse.norm_w && (K > 4096 || q4 || (size_t)N * K > ((size_t)16 << 20))) && !fuse.cand_v) {
        const int mode = fuse.norm_w ? 2 : ((fuse.x2 || fuse.res_in) ? 1 : 0);
        const int chunk_k = WAVE * (q4 ? 32 : 16);
        const int wps = K <= chunk_k ? 1 : (K <= 2 * chunk_k ? 2 : 4);
        const int nc = (K + wps * chunk_k - 1) / (wps * chunk_k);
        for (int m = 0; m < M; m++) {
            const float *xm = d_x + (size_t)m * K;
            float *om = d_out + (size_t)m * N;
#define HM_CUT(RR, CC, WW)                                                                                                  \
    do {                                                                                                                    \
        const int rows_wg = RR * (PWAVES / WW), grid = (N + rows_wg - 1) / rows_wg;                                         \
        if (mode == 2) {                                                                                                    \
            if constexpr (CC == 1 && QT == 0)                                                                               \
                hipLaunchKernelGGL((gemv_planes_splitk_kernel<QT, RR, CC, 2, WW>), dim3(grid), dim3(PTHREADS), 0, ctx->stream, \
                                   xm, quants, scales, om, K, N, fuse);                                                     \
        } else if (fused)                                                                                                   \
            hipLaunchKernelGGL((gemv_planes_splitk_kernel<QT, RR, CC, 1, WW>), dim3(grid), dim3(PTHREADS), 0, ctx->stream,  \
                               xm, quants, scales, om, K, N, fuse);                                                         \
        else                                                                                                                \
            hipLaunchKernelGGL((gemv_planes_splitk_kernel<QT, RR, CC, 0, WW>), dim3(grid), dim3(PTHREADS), 0, ctx->stream,  \
                               xm, quants, scales, om, K, N, fuse);                                                         \
    } while (0)
            if (wps <= 2) {
                // rows a set: as many as leave a thousand workgroups or so (every set re-reads the activation pieces)
                const int sets = PWAVES / wps;
                int r = N / (16 * sets) >= 1024 ? 16 : (N / (8 * sets) >= 512 ? 8 : 4);
                if (fused && r > 8) r = 8;
                if (wps == 1) {
                    if (r == 16) HM_CUT(16, 1, 1); else if (r == 8) HM_CUT(8, 1, 1); else HM_CUT(4, 1, 1);
                } else {
                    if (r == 16) HM_CUT(16, 1, 2); else if (r == 8) HM_CUT(8, 1, 2); else HM_CUT(4, 1, 2);
                }
            } else if (!q4) {
                if (nc == 1) HM_CUT(8, 1, 4);
                else if (nc == 2) HM_CUT(8, 2, 4);
                else if (nc == 3) { if (fused) HM_CUT(4, 3, 4); else HM_CUT(8, 3, 4); }
                else HM_CUT(4, 4, 4);
            } else {
                if (nc == 1) { if (fused) HM_CUT(8, 1, 4); else HM_CUT(16, 1, 4); }
                else { if (fused) HM_CUT(4, 2, 4); else HM_CUT(8, 2, 4); }
            }
#undef HM_CUT
            HM_LAUNCH_CHECK(ctx);
        }
        return HM_OK;
    }
    HM_REQUIRE(ctx, K <= 4096, "%s: K=%d above 4096 with a fused RMSNorm or argmax candidates", name, K);
    const PlanesShape sh = planes_shape(ctx, q4, K, N);
    // Q4_0 at the LM-head shape: the half-block-per-lane kernel
    const int nblk = K / 32;
    // Q4_0, tall matrices with rows of 2048, 3072 or 4096: the whole-block-per-lane kernel (35.6 us against 39.5 of
    // the half-block kernel at 2048 -> 151936; 25 against 31 us and 30 against 44 us of the quarter-block kernel at
    // 3072 and 4096 -> 65536); narrower rows are no faster that way (29-30 us at 1536 -> 151936 either way)
    if (q4 && !fused && N >= 8 * PWAVES * ctx->num_cus && (nblk == 64 || nblk == 96 || nblk == 128)) {
        const int rb = nblk == 96 ? 2 : 1;
        const int ntrips = (N + 2 * rb - 1) / (2 * rb);
        const int want = (ntrips + PWAVES - 1) / PWAVES;
        const int grid = std::min(want, 8 * ctx->num_cus);
        const size_t lds = (size_t)nblk * 36 * 4 + 16;
        for (int m = 0; m < M; m++) {
            const float *xm = d_x + (size_t)m * K;
            float *om = d_out + (size_t)m * N;
            if (nblk == 64)
                hipLaunchKernelGGL((gemv_q4_0_blocks_kernel<1, 1>), dim3(grid), dim3(PTHREADS), lds, ctx->stream, xm, quants, scales, om, K, N);
            else if (nblk == 96)
                hipLaunchKernelGGL((gemv_q4_0_blocks_kernel<3, 2>), dim3(grid), dim3(PTHREADS), lds, ctx->stream, xm, quants, scales, om, K, N);
            else
                hipLaunchKernelGGL((gemv_q4_0_blocks_kernel<2, 1>), dim3(grid), dim3(PTHREADS), lds, ctx->stream, xm, quants, scales, om, K, N);
            HM_LAUNCH_CHECK(ctx);
        }
        return HM_OK;
    }
    if (q4 && !fused && nblk % 16 == 0 && nblk / 16 <= 4 && N >= 8 * PWAVES * ctx->num_cus) {
        const int ntrips = (N + 1) / 2;
        const int want = (ntrips + PWAVES - 1) / PWAVES;
        const int grid = std::min(want, 4 * ctx->num_cus);  // four workgroups a CU (five fit: slower)
        const size_t lds = (size_t)K * 4 + 16;
        for (int m = 0; m < M; m++) {
            const float *xm = d_x + (size_t)m * K;
            float *om = d_out + (size_t)m * N;
            switch (nblk / 16) {
            case 1: hipLaunchKernelGGL((gemv_q4_0_halves_kernel<1>), dim3(grid), dim3(PTHREADS), lds, ctx->stream, xm, quants, scales, om, K, N); break;
            case 2: hipLaunchKernelGGL((gemv_q4_0_halves_kernel<2>), dim3(grid), dim3(PTHREADS), lds, ctx->stream, xm, quants, scales, om, K, N); break;
            case 3: hipLaunchKernelGGL((gemv_q4_0_halves_kernel<3>), dim3(grid), dim3(PTHREADS), lds, ctx->stream, xm, quants, scales, om, K, N); break;
            default: hipLaunchKernelGGL((gemv_q4_0_halves_kernel<4>), dim3(grid), dim3(PTHREADS), lds, ctx->stream, xm, quants, scales, om, K, N); break;
            }
            HM_LAUNCH_CHECK(ctx);
        }
        return HM_OK;
    }
    for (int m = 0; m < M; m++) {
        const float *xm = d_x + (size_t)m * K;
        float *om = d_out + (size_t)m * N;
#define HM_PL(C, R)                                                                                                        \
    do {                                                                                                                   \
        if (fused)                                                                                                         \
            hipLaunchKernelGGL((gemv_planes_kernel<QT, C, R, true>), dim3(sh.grid), dim3(PTHREADS), sh.lds, ctx->stream, xm, \
                               quants, scales, om, K, N, fuse);                                                            \
        else                                                                                                               \
            hipLaunchKernelGGL((gemv_planes_kernel<QT, C, R, false>), dim3(sh.grid), dim3(PTHREADS), sh.lds, ctx->stream, xm, \
                               quants, scales, om, K, N, fuse);                                                            \
    } while (0)
#define HM_PL_RB(C)                                      \
    do {                                                 \
        if (sh.rb == 1)                                  \
            HM_PL(C, 1);                                 \
        else                                             \
            HM_PL(C, (TripRows<QT, C>::MOST));           \
    } while (0)
        switch (planes_cpl_instance(cpl)) {
        case 1: HM_PL_RB(1); break;
        case 2: HM_PL_RB(2); break;
        case 3: HM_PL_RB(3); break;
        case 4: HM_PL_RB(4); break;
        case 6: HM_PL_RB(6); break;
        default: HM_PL_RB(8); break;
        }
#undef HM_PL_RB
#undef HM_PL
        HM_LAUNCH_CHECK(ctx);
    }
    return HM_OK;
}

template <int QT>
int pack_launch(hm_ctx *ctx, const char *name, const uint8_t *d_blocks, uint8_t *d_planes, int N, int K, bool unpack) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_blocks && d_planes, "%s: NULL pointer", name);
    HM_REQUIRE(ctx, N > 0 && K > 0 && K % 32 == 0, "%s: K=%d must be a positive multiple of 32, N=%d positive", name, K, N);
    HM_REQUIRE(ctx, ((uintptr_t)d_planes % 16) == 0, "%s: the planes must be 16-byte aligned", name);
    const size_t nq = (size_t)N * (K / 8);
    uint16_t *scales = reinterpret_cast<uint16_t *>(d_planes + homura::quant_planes_scale_offset(QT == 1, N, K));
    const unsigned grid = (unsigned)((nq + 255) / 256);
    if (unpack)
        hipLaunchKernelGGL((unpack_planes_kernel<QT>), dim3(grid), dim3(256), 0, ctx->stream, d_planes, scales,
                           const_cast<uint8_t *>(d_blocks), nq);
    else
        hipLaunchKernelGGL((pack_planes_kernel<QT>), dim3(grid), dim3(256), 0, ctx->stream, d_blocks, d_planes, scales, nq);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // namespace

size_t homura::quant_planes_scale_offset(bool q4, int N, int K) {
    const size_t qbytes = (size_t)N * (q4 ? K / 2 : K);
    return (qbytes + 255) & ~(size_t)255;
}

size_t homura::quant_planes_bytes(bool q4, int N, int K) {
    return quant_planes_scale_offset(q4, N, K) + (size_t)N * (K / 32) * 2;
}

int homura::gemv_planes_workgroups(const hm_ctx *ctx, bool q4, int K, int N) { return planes_shape(ctx, q4, K, N).grid; }

int homura::gemv_planes_fused(hm_ctx *ctx, bool q4, const float *d_x, const uint8_t *d_planes, float *d_out, int K, int N,
                              const QuantFuse &fuse) {
    return q4 ? planes_launch<1>(ctx, "gemv_planes[q4_0]", d_x, d_planes, d_out, 1, K, N, fuse)
              : planes_launch<0>(ctx, "gemv_planes[q8_0]", d_x, d_planes, d_out, 1, K, N, fuse);
}

int homura::pack_quant_planes(hm_ctx *ctx, bool q4, const uint8_t *d_blocks, uint8_t *d_planes, int N, int K) {
    return q4 ? pack_launch<1>(ctx, "pack_quant_planes[q4_0]", d_blocks, d_planes, N, K, false)
              : pack_launch<0>(ctx, "pack_quant_planes[q8_0]", d_blocks, d_planes, N, K, false);
}

extern "C" {

size_t hm_quant_planes_bytes(int hm_dtype, int N, int K) {
    if (hm_dtype == HM_DTYPE_Q6_K) return N > 0 && K > 0 && K % 256 == 0 ? homura::q6k_planes_bytes(N, K) : 0;
    if ((hm_dtype != HM_DTYPE_Q8_0 && hm_dtype != HM_DTYPE_Q4_0) || N <= 0 || K <= 0 || K % 32 != 0) return 0;
    return homura::quant_planes_bytes(hm_dtype == HM_DTYPE_Q4_0, N, K);
}

int hm_pack_quant_planes(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, uint8_t *d_planes, int N, int K) {
    HM_CHECK_CTX(ctx);
    if (hm_dtype == HM_DTYPE_Q6_K) return homura::pack_q6k_planes(ctx, d_blocks, d_planes, N, K, false);
    HM_REQUIRE(ctx, hm_dtype == HM_DTYPE_Q8_0 || hm_dtype == HM_DTYPE_Q4_0, "hm_pack_quant_planes: dtype %d is not Q8_0, Q4_0 or Q6_K", hm_dtype);
    return homura::pack_quant_planes(ctx, hm_dtype == HM_DTYPE_Q4_0, d_blocks, d_planes, N, K);
}

int hm_unpack_quant_planes(hm_ctx *ctx, int hm_dtype, const uint8_t *d_planes, uint8_t *d_blocks, int N, int K) {
    HM_CHECK_CTX(ctx);
    if (hm_dtype == HM_DTYPE_Q6_K) return homura::pack_q6k_planes(ctx, d_blocks, const_cast<uint8_t *>(d_planes), N, K, true);
    HM_REQUIRE(ctx, hm_dtype == HM_DTYPE_Q8_0 || hm_dtype == HM_DTYPE_Q4_0, "hm_unpack_quant_planes: dtype %d is not Q8_0, Q4_0 or Q6_K", hm_dtype);
    return hm_dtype == HM_DTYPE_Q4_0 ? pack_launch<1>(ctx, "hm_unpack_quant_planes", d_blocks, const_cast<uint8_t *>(d_planes), N, K, true)
                                     : pack_launch<0>(ctx, "hm_unpack_quant_planes", d_blocks, const_cast<uint8_t *>(d_planes), N, K, true);
}

int hm_gemv_q8_0_planes(hm_ctx *ctx, const float *d_x, const uint8_t *d_planes, float *d_out, int M, int K, int N) {
    return planes_launch<0>(ctx, "hm_gemv_q8_0_planes", d_x, d_planes, d_out, M, K, N, QuantFuse());
}

int hm_gemv_q4_0_planes(hm_ctx *ctx, const float *d_x, const uint8_t *d_planes, float *d_out, int M, int K, int N) {
    return planes_launch<1>(ctx, "hm_gemv_q4_0_planes", d_x, d_planes, d_out, M, K, N, QuantFuse());
}

int hm_gemv_q6_k_f32_planes(hm_ctx *ctx, const float *d_x, const uint8_t *d_planes, float *d_out, int M, int K, int N) {
    return homura::gemv_q6k_planes_f32(ctx, "hm_gemv_q6_k_f32_planes", d_x, nullptr, 0.f, d_planes, d_out, M, K, N, nullptr, nullptr, 0);
}

int hm_dequant_quant_planes(hm_ctx *ctx, int hm_dtype, const uint8_t *d_planes, float *d_out, int N, int K) {
    HM_CHECK_CTX(ctx);
    if (hm_dtype == HM_DTYPE_Q6_K) return homura::dequant_q6k_planes(ctx, d_planes, d_out, N, K);
    HM_REQUIRE(ctx, hm_dtype == HM_DTYPE_Q8_0 || hm_dtype == HM_DTYPE_Q4_0, "hm_dequant_quant_planes: dtype %d is not Q8_0, Q4_0 or Q6_K", hm_dtype);
    HM_REQUIRE(ctx, d_planes && d_out && N > 0 && K > 0 && K % 32 == 0, "hm_dequant_quant_planes: bad arguments");
    const bool q4 = hm_dtype == HM_DTYPE_Q4_0;
    const size_t n = (size_t)N * K;
    size_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    const uint16_t *scales = reinterpret_cast<const uint16_t *>(d_planes + homura::quant_planes_scale_offset(q4, N, K));
    if (q4)
        hipLaunchKernelGGL((dequant_planes_kernel<1>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, d_planes, scales, d_out, n);
    else
        hipLaunchKernelGGL((dequant_planes_kernel<0>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, d_planes, scales, d_out, n);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // extern "C"
