// One decode token of a bf16 model in one launch: embedding row, then every decoder layer
// (RMSNorm -> Q|K|V -> QK-norm, RoPE, cache append -> GQA attention -> O -> residual -> RMSNorm ->
// gate|up -> SiLU*up -> down -> residual; reference src/hf/emitter.rs:549-822), leaving the last
// hidden state for the LM head launch.
//
// The reference dispatches three kernels per layer and the plan's kernel-per-projection path issues
// six; each dependent launch costs 1.6 us on this chip even when empty, and that, not bandwidth,
// bounds a 0.6 B model. Here NWG workgroups (one per CU) stay resident for the whole step:
//
//  * Every workgroup owns a fixed slice of every matrix. Its four compute wavefronts keep that
//    slice in registers and reload each phase's registers with the NEXT layer's slice as soon as the
//    phase is done, so weights and cache rows stream from HBM a full layer ahead of their use and
//    no phase waits for HBM.
//  * Phases hand their small results (4-24 KB per layer) to each other through an exchange area in
//    device memory: every value travels as an 8-byte {f32, tag} pair written with a device-scope
//    store and polled with device-scope loads, tag = 1 + number of layers run since the area was
//    zeroed. A reader accepts a pair only with the tag of the layer it is in, so no fence, counter or
//    cache invalidation is needed and a stale pair can never be mistaken for a fresh one.
//  * The four communication wavefronts of a workgroup do all the polling and publishing (loads return
//    to a wavefront in issue order, so a poll issued behind a weight prefetch would wait for HBM), stage
//    the phase input in LDS, and meet the compute wavefronts at two workgroup barriers per phase.
//  * The workgroups of a KV head (one die when there are as many KV heads as dies) form a group, and the
//    groups split the layer like tensor-parallel ranks: Q|K|V and gate|up by rows (a group computes its
//    own heads' rows and a contiguous share of the SiLU*up values), O and down by K (a group multiplies
//    the K slice it produced itself for every output row). What a group's phases hand to each other
//    stays in the group; only the partial hidden increments cross groups, and they are added up on the
//    way into the next phase.
//
// Six exchanges per layer: hidden -> (Q|K|V rows) -> (attention partials per cache split) ->
// (folded heads) -> (partial O rows, summed over the groups) -> (SiLU*up) -> (partial down rows, summed).
// The arithmetic is that of gemv_bf16.hip and attention.hip: Q|K|V and gate|up rows bit for bit, O and
// down rows as sums of per-group partial dot products, attention with the cache split into
// NWG / kv_heads pieces instead of 64-row chunks.
//
// Every wait is a bounded spin: on a timeout the workgroup records a status word, stops waiting,
// and still walks through the remaining barriers, so the grid always drains.
#include "decode_fused.h"
#include "k8_device.h"

#include <cstdlib>
#include <type_traits>

namespace {

constexpr int FT = 512;     // threads per workgroup: wavefronts 0-3 compute, 4-7 communicate
constexpr int NCW = 4;      // compute wavefronts
constexpr int CT = 256;     // communicating threads
constexpr int SPIN_MAX = 1 << 20;
constexpr int MAX_LAYERS = 64;

template <int HIDDEN_, int H_, int KVH_, int HD_, int INTER_, int NWG_, int NR_ = 4, int XR_ = 0>
struct Geo {
    static constexpr int HIDDEN = HIDDEN_, H = H_, KVH = KVH_, HD = HD_, INTER = INTER_, NWG = NWG_;
    static constexpr int G = H / KVH, QD = H * HD, KVD = KVH * HD, NQKV = QD + 2 * KVD;
    static constexpr int CH = HIDDEN / 512, CO = QD / 512, CD = INTER / 512;  // 512-wide chunks of a row
    static constexpr int RQ = NQKV / NWG, RQW = RQ / NCW;      // Q|K|V rows per workgroup / wavefront
    static constexpr int SPH = NWG / KVH;                      // workgroups (= cache splits) per KV head
    // O and down: the workgroups of a KV head multiply a K slice (the head group's own attention outputs,
    // its own SiLU*up values) for every output row, RPG rows a workgroup; the KVH partial vectors are
    // added up on the way into the next phase.
    static constexpr int RPG = HIDDEN / SPH, RPW = RPG / NCW;  // partial rows per workgroup / wavefront
    static constexpr int KSO = G * HD, KSD = INTER / KVH;      // K slice of the O / down projection
    // A workgroup's partial rows are two runs of RPG / 2 rows, 256 rows apart: hidden elements k and k + 256
    // share a 16-byte exchange unit (hidden_slot), which one workgroup then writes whole.
    static constexpr int RUN = RPG / 2, WPP = 256 / RUN;
    __device__ static int partial_row(int split, int i) { return (split % WPP) * RUN + i % RUN + 256 * (2 * (split / WPP) + i / RUN); }
    static constexpr int RG = 2 * INTER / NWG, RGW = RG / NCW; // gate|up rows (interleaved pairs)
    static constexpr int APW = INTER / NWG;                    // SiLU*up values per workgroup
    static constexpr int NR = NR_;                             // row rounds a wavefront keeps in registers
    static constexpr int LPR = HD / 8, RPI = WAVE / LPR;       // lanes per cache row, rows per load
    static constexpr int XR = XR_;                             // further rounds, streamed inside the attention phase
    static constexpr int MAX_KV = SPH * (NR + XR) * NCW * RPI;
    static constexpr int FPW = QD / NWG;                       // folded attention outputs per workgroup
    static constexpr int PART = G * HD + 2 * G;                // one split's partial: o[G][HD], (m, l)[G]
    static constexpr int NJ = HIDDEN / CT;                     // hidden elements per communicating thread
    static constexpr int NXCD = 8, NPX = NWG / NXCD;           // accelerator dies (one L2 each), workgroups per die
    static constexpr int GROWS = (G + 2) * HD;                 // q|k|v rows of one KV head
    // A KV head's workgroups are wg % KVH == head; with workgroups dealt round-robin to the dies they all
    // share one L2 when KVH is a multiple of the die count.
    static constexpr bool GROUP_ON_XCD = KVH % NXCD == 0;
    // Exchange area of one layer parity, in 8-byte slots: the partial hidden increments of every KV-head
    // group (down rows XH, O rows XO: KVH vectors each), per die one relay copy of their sums, and per KV
    // head the raw q|k|v rows (LQ), the attention partials of its splits (LP), its folded attention
    // outputs (LA) and its SiLU*up values (LC).
    static constexpr int XH = 0, XO = KVH * HIDDEN, GLOB_SLOTS = 2 * KVH * HIDDEN;
    static constexpr int RELAY0 = GLOB_SLOTS, RELAY_SLOTS = 2 * HIDDEN;
    static constexpr int LQ0 = RELAY0 + NXCD * RELAY_SLOTS, LP0 = LQ0 + KVH * GROWS, LA0 = LP0 + KVH * SPH * PART;
    static constexpr int LC0 = LA0 + KVH * KSO;
    // K8 format, when a group's K slice of down does not start and end on 256-wide blocks: per workgroup the
    // largest |SiLU*up| among its values in the block that the slice shares with the group before (first slot)
    // and with the group after (second slot)
    static constexpr int LM0 = LC0 + KVH * KSD;
    static constexpr int PAR_SLOTS = (LM0 + 2 * NWG + 31) / 32 * 32;
    static constexpr int CHK0 = 2 * PAR_SLOTS;                 // placement check: one slot per workgroup
    static constexpr int CAND0 = CHK0 + NWG;                   // LM head: one {value, index} unit per workgroup
    static constexpr int ALL_SLOTS = CAND0 + 2 * NWG;
    static constexpr int HR = 8;                               // LM-head rows a wavefront multiplies per batch
    static constexpr int PUB0 = (PART > RQ ? PART : RQ) > RG ? (PART > RQ ? PART : RQ) : RG;
    static constexpr int PUB = PUB0 > RPG ? PUB0 : RPG;
    static_assert(HIDDEN % 512 == 0 && QD % 512 == 0 && INTER % 512 == 0, "rows are cut into 512-wide chunks");
    static_assert(NQKV % (NWG * NCW) == 0 && HIDDEN % (SPH * NCW) == 0 && (2 * INTER) % (NWG * NCW) == 0,
                  "every wavefront owns whole rows");
    static_assert(KSO % 128 == 0 && KSD % 128 == 0 && INTER % KVH == 0, "K slices are cut into 128-wide parts");
    static_assert(RUN % RPW == 0 && 256 % RUN == 0 && SPH % WPP == 0, "a wavefront's partial rows lie in one run");
    static_assert(RGW % 2 == 0, "a wavefront owns whole gate|up pairs");
    static_assert(NWG % KVH == 0 && SPH <= WAVE, "one fold lane per cache split");
    static_assert(HD == 64 || HD == 128, "head_dim 64 or 128");
    static_assert(QD % NWG == 0 && FPW % 2 == 0 && HD % FPW == 0, "a workgroup folds a run inside one head");
    static_assert(RQ <= CT && RPG <= CT && APW <= CT, "one publishing thread per value");
    static_assert(KSO / 2 <= CT && KSD / 2 <= CT, "one staging thread per 16-byte unit of a K slice");
    static_assert(GROWS % SPH == 0 && GROWS / SPH == RQ && HD % RQW == 0, "a wavefront's q|k|v rows lie in one of q, k, v");
    static_assert(NWG % NXCD == 0 && (HIDDEN / 2) % NPX == 0 && HIDDEN / 2 / NPX <= WAVE,
                  "one wavefront relays a die's share of a vector");
    static_assert(NWG % 2 == 0 && NWG / 2 <= 2 * WAVE, "two placement-check units per lane");
    static_assert(NWG % WAVE == 0 && NWG / WAVE <= 8, "workgroup 0 gathers the LM-head candidates with one wavefront");
    // row of the stacked q|k|v matrix for local row lr of KV head kh
    __device__ static int qkv_row(int kh, int lr) {
        return lr < G * HD ? kh * G * HD + lr : (lr < (G + 1) * HD ? QD + kh * HD + (lr - G * HD) : QD + KVD + kh * HD + (lr - (G + 1) * HD));
    }
};

template <class GE>
struct Lds {
    float hx[GE::HIDDEN];                 // hidden state entering the phase's RMSNorm
    float nw[GE::HIDDEN];                 // that norm's weights
    float attn[GE::KSO];                  // folded attention output of this workgroup's KV head
    float act[GE::KSD];                   // SiLU(gate) * up of this workgroup's KV-head group
    float rowbuf[GE::G + 2][GE::HD];      // raw q heads, k, v of this workgroup's KV head
    float qs[GE::G][GE::HD];              // after QK-norm and RoPE
    float knew[GE::HD], vnew[GE::HD];     // the new cache row, as rounded to bf16
    float part[NCW * GE::RPI][GE::G][GE::HD];
    float wstat[NCW][GE::G][2];
    float pub[GE::PUB];                   // results of the phase, read by the publishing threads
    float red[4];
    float nbmax[2];                       // K8: the neighbouring groups' maxima of the two shared blocks
    float head_v[NCW + 4];                // LM head: every wavefront's best row
    int head_i[NCW + 4];
    float bias[GE::RQ];
    FusedLayerPtrs lp[MAX_LAYERS];        // the layer table (compute wavefronts must not wait on global loads)
};

// Pointers that reach the kernel through the layer table are generic; loads through them would be flat
// loads, which count against the LDS counter too. These helpers pin them to global memory.
typedef const u32x4 __attribute__((address_space(1))) *global_u32x4_ptr;
typedef const float __attribute__((address_space(1))) *global_f32_ptr;
__device__ __forceinline__ u32x4 ld128_global_stream(const void *p) {
    return __builtin_nontemporal_load((global_u32x4_ptr)p);
}
__device__ __forceinline__ float ldf_global(const float *p) { return *(global_f32_ptr)p; }

__device__ __forceinline__ void wg_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Exchange primitives. Every poll is a device-scope load: it never reads the CU's L1, and it sees what its
// die's L2 holds. "Far" stores cross dies: device scope, written through to memory. "Near" stores are
// plain stores, which stop in the die's L2 (0.27 us from store to a poll on the same die, against 0.6 us
// through memory); they are only used between workgroups that the placement check found on one die, and
// never on memory that far stores touch. (Non-temporal loads also skip the L1 most of the time, but a
// line they left there can be served again later: a poll built on them can spin on a stale copy.)
__device__ __forceinline__ void st_slot(unsigned char *area, int slot, float v, uint32_t tag, bool near) {
    unsigned char *p = area + (size_t)slot * 8;
    const uint64_t w = ((uint64_t)tag << 32) | __float_as_uint(v);
    // compiler-issued stores: a store written in inline asm is invisible to the hazard recognizer (a store
    // of more than 8 bytes must not be followed at once by a write to its data registers)
    if (near)
        __hip_atomic_store(reinterpret_cast<uint64_t *>(p), w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
    else
        __hip_atomic_store(reinterpret_cast<uint64_t *>(p), w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("" ::: "memory");
}

struct PollState {
    uint32_t *ctl;
    bool failed;
    uint32_t where;  // what is being waited for: phase | layer << 4 | workgroup << 12, stored on a timeout
    int spin_max;    // polls before a wait gives up
};

// 16-byte loads of `NU` units {v0, tag, v1, tag}, all issued before one wait, repeated until every
// wanted unit carries `tag` in both halves. Units with on[u] false are not waited for.
template <int NU>
__device__ __forceinline__ void poll_units(PollState &ps, const unsigned char *area, const int (&unit)[NU],
                                           const bool (&on)[NU], uint32_t tag, u32x4 (&w)[NU]) {
    bool any = false;
#pragma unroll
    for (int u = 0; u < NU; u++) {
        w[u] = u32x4{0u, 0u, 0u, 0u};
        any = any || on[u];
    }
    if (ps.failed || !any) return;
    int spins = 0;
    while (true) {
#pragma unroll
        for (int u = 0; u < NU; u++) {
            const unsigned char *p = area + (size_t)(on[u] ? unit[u] : 0) * 16;
            asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(w[u]) : "v"(p) : "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int u = 0; u < NU; u++) asm volatile("" : "+v"(w[u]));
        bool ok = true;
#pragma unroll
        for (int u = 0; u < NU; u++) ok = ok && (!on[u] || (w[u].y == tag && w[u].w == tag));
        if (ok) return;
        if (++spins > ps.spin_max) {
            atomicCAS(ps.ctl + 1, 0u, 0x80000000u | ps.where);  // the first timeout is the one reported
            ps.failed = true;
            return;
        }
        if ((spins & 1023) == 0 &&
            __hip_atomic_load(ps.ctl + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {
            ps.failed = true;
            return;
        }
    }
}

__device__ __forceinline__ float dot8f(const u32x4 w, const float *xv, float acc) {
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

__device__ __forceinline__ void unpack8f(const u32x4 w, float *f) {
    f[0] = bf16_lo(w.x); f[1] = bf16_hi(w.x);
    f[2] = bf16_lo(w.y); f[3] = bf16_hi(w.y);
    f[4] = bf16_lo(w.z); f[5] = bf16_hi(w.z);
    f[6] = bf16_lo(w.w); f[7] = bf16_hi(w.w);
}

__device__ __forceinline__ void lds_x8(const float *v, int k, float *xv) {
    const f32x4 a = *reinterpret_cast<const f32x4 *>(v + k);
    const f32x4 b = *reinterpret_cast<const f32x4 *>(v + k + 4);
    xv[0] = a.x; xv[1] = a.y; xv[2] = a.z; xv[3] = a.w;
    xv[4] = b.x; xv[5] = b.y; xv[6] = b.z; xv[7] = b.w;
}

// Vectors that the compute wavefronts read out of LDS (the staged hidden state and its norm weights, the folded
// attention outputs, the SiLU*up values) are stored permuted, by weight format: a lane reads GRP consecutive
// elements (8 with bf16 weights, 16 with the byte formats) as 16-byte pieces, and piece j of every group lies
// in quarter j of the vector, so that the lanes of one read touch consecutive addresses (no bank conflicts;
// stored in index order a read strides by 32 or 64 bytes a lane). Q4_0 reads two runs of 8 a lane and keeps
// the index order.
template <int WF>
struct XLay {
    static constexpr int GRP = (WF == FUSED_WF_Q8_0 || WF == FUSED_WF_K8) ? 16 : (WF == FUSED_WF_BF16 ? 8 : 0);
    __device__ __forceinline__ static int pos(int k, int n) {
        if (GRP == 0) return k;
        return ((k % GRP) / 4) * (n / (GRP / 4)) + (k / GRP) * 4 + (k % 4);
    }
};
// elements k .. k + 7 (k a multiple of 8) of a vector of n elements stored as XLay<WF> lays it out
template <int WF>
__device__ __forceinline__ void lds_v8(const float *v, int n, int k, float *xv) {
    const f32x4 a = *reinterpret_cast<const f32x4 *>(v + XLay<WF>::pos(k, n));
    const f32x4 b = *reinterpret_cast<const f32x4 *>(v + XLay<WF>::pos(k + 4, n));
    xv[0] = a.x; xv[1] = a.y; xv[2] = a.z; xv[3] = a.w;
    xv[4] = b.x; xv[5] = b.y; xv[6] = b.z; xv[7] = b.w;
}

template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
    v += dpp_move<0xB1, 0xF>(v, 0.f);
    v += dpp_move<0x4E, 0xF>(v, 0.f);
    v += dpp_move<0x141, 0xF>(v, 0.f);
    if (LPR == 16) v += dpp_move<0x140, 0xF>(v, 0.f);
    return v;
}

// One wavefront: optional RMSNorm over hd, then x*cos + rotate_half(x)*sin (the arithmetic of
// attention.hip's fused prologue; reference src/hf/emitter.rs:629-644). Lane i < hd/2 owns the pair
// (i, i + hd/2); the lane's table entries and norm weights are handed in (loaded before the wait for
// the row, so no global load sits between the row's arrival and the result).
struct RopeLane {
    float c_lo, c_hi, s_lo, s_hi;
};
template <int HD>
__device__ __forceinline__ void norm_rope(const float *src, bool normed, float w_lo, float w_hi, const RopeLane &t,
                                          float eps, int lane, float &o_lo, float &o_hi) {
    constexpr int HALF = HD / 2;
    const bool on = lane < HALF;
    float lo = on ? src[lane] : 0.f, hi = on ? src[lane + HALF] : 0.f;
    if (normed) {
        const float ss = wave_sum(lo * lo + hi * hi);
        const float inv = __builtin_amdgcn_rsqf(ss / (float)HD + eps);
        lo = (lo * inv) * w_lo;
        hi = (hi * inv) * w_hi;
    }
    o_lo = lo * t.c_lo + (-hi) * t.s_lo;
    o_hi = hi * t.c_hi + lo * t.s_hi;
}

// Dot products of R rows x C chunks kept as R * C independent chains (one wavefront per SIMD: the
// chains are what hides the latency of a dependent multiply-add), the k loop outermost.
template <int R, int C>
__device__ __forceinline__ void dots_from(const u32x4 (&w)[R][C], const float (&xv)[C][8], float (&acc)[R][C]) {
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int c = 0; c < C; c++) acc[r][c] = 0.f;
#pragma unroll
    for (int e = 0; e < 4; e++) {
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int c = 0; c < C; c++) {
                const uint32_t d = e == 0 ? w[r][c].x : (e == 1 ? w[r][c].y : (e == 2 ? w[r][c].z : w[r][c].w));
                acc[r][c] = fmaf(bf16_lo(d), xv[c][2 * e], acc[r][c]);
            }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int c = 0; c < C; c++) {
                const uint32_t d = e == 0 ? w[r][c].x : (e == 1 ? w[r][c].y : (e == 2 ? w[r][c].z : w[r][c].w));
                acc[r][c] = fmaf(bf16_hi(d), xv[c][2 * e + 1], acc[r][c]);
            }
    }
}

// rows against (h * inv) * norm_w read from LDS (RMSNorm: reference src/graph_builder/emit_linalg.rs:7-26)
template <int R, int C>
__device__ __forceinline__ void normed_dots(const u32x4 (&w)[R][C], const float *hx, const float *nw, float inv,
                                            int lane, float (&acc)[R][C]) {
    float xv[C][8];
#pragma unroll
    for (int c = 0; c < C; c++) {
        float hv[8], wv[8];
        lds_v8<FUSED_WF_BF16>(hx, C * 512, (c * WAVE + lane) * 8, hv);
        lds_v8<FUSED_WF_BF16>(nw, C * 512, (c * WAVE + lane) * 8, wv);
#pragma unroll
        for (int e = 0; e < 8; e++) xv[c][e] = (hv[e] * inv) * wv[e];
    }
    dots_from<R, C>(w, xv, acc);
}

template <int R, int C>
__device__ __forceinline__ void plain_dots(const u32x4 (&w)[R][C], const float *x, int lane, float (&acc)[R][C]) {
    float xv[C][8];
#pragma unroll
    for (int c = 0; c < C; c++) lds_v8<FUSED_WF_BF16>(x, C * 512, (c * WAVE + lane) * 8, xv[c]);
    dots_from<R, C>(w, xv, acc);
}

template <int C>
__device__ __forceinline__ float chunk_total(const float (&a)[C]) {
    float t = a[0];
#pragma unroll
    for (int c = 1; c < C; c++) t += a[c];
    return t;
}

// wave_sum / wave_max of N values with the N chains stepping side by side; every lane gets the totals
template <int N>
__device__ __forceinline__ void wave_sum_n(float (&v)[N]) {
#pragma unroll
    for (int i = 0; i < N; i++) v[i] += dpp_move<0xB1, 0xF>(v[i], 0.f);
#pragma unroll
    for (int i = 0; i < N; i++) v[i] += dpp_move<0x4E, 0xF>(v[i], 0.f);
#pragma unroll
    for (int i = 0; i < N; i++) v[i] += dpp_move<0x141, 0xF>(v[i], 0.f);
#pragma unroll
    for (int i = 0; i < N; i++) v[i] += dpp_move<0x140, 0xF>(v[i], 0.f);
#pragma unroll
    for (int i = 0; i < N; i++) v[i] += dpp_move<0x142, 0xA>(v[i], 0.f);
#pragma unroll
    for (int i = 0; i < N; i++) v[i] += dpp_move<0x143, 0xC>(v[i], 0.f);
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v[i]), 63));
}

template <int N>
__device__ __forceinline__ void wave_max_n(float (&v)[N]) {
    const float ninf = -__builtin_huge_valf();
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = fmaxf(v[i], dpp_move<0xB1, 0xF>(v[i], ninf));
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = fmaxf(v[i], dpp_move<0x4E, 0xF>(v[i], ninf));
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = fmaxf(v[i], dpp_move<0x141, 0xF>(v[i], ninf));
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = fmaxf(v[i], dpp_move<0x140, 0xF>(v[i], ninf));
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = fmaxf(v[i], dpp_move<0x142, 0xA>(v[i], ninf));
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = fmaxf(v[i], dpp_move<0x143, 0xC>(v[i], ninf));
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v[i]), 63));
}

// ── the rows of one matrix that a compute wavefront keeps in registers, by weight format ──
//
// bf16 (stream layout [N][K]): a lane holds 8 consecutive weights of each 512-wide chunk of a row, and the
// products are those of gemv_bf16.hip bit for bit. Q8_0 / Q4_0 (planes, gemv_quant_planes.hip: quant
// bytes [N][K] or [N][K / 2], f16 scales [N][K / 32]): a lane holds half a block, 16 weights, of each
// 1024-wide chunk plus the block's scale, and a row is sum over half blocks of d * (sum_j q_j x_j -
// offset * sum_j x_j) with the quants used as stored, as in gemv_quant.hip.
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;
typedef const u32x2 __attribute__((address_space(1))) *global_u32x2_ptr;

template <int WF, int R, int K>
struct Rows;

template <int R, int K>
struct Rows<FUSED_WF_BF16, R, K> {
    static constexpr int C = K / 512;
    static_assert(K % 512 == 0, "bf16 rows are cut into 512-wide chunks");
    u32x4 w[R][C];
    template <class RowOf>
    __device__ __forceinline__ void load(const void *quants, const uint16_t *, RowOf row_of, int r0, int r1, int lane) {
        const uint16_t *base = reinterpret_cast<const uint16_t *>(quants);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int c = 0; c < C; c++)
                if (r >= r0 && r < r1) w[r][c] = ld128_global_stream(base + (size_t)row_of(r) * K + (c * WAVE + lane) * 8);
    }
    __device__ __forceinline__ void dots_normed(const float *hx, const float *nw, float inv, int lane, float (&v)[R]) const {
        float acc[R][C];
        normed_dots<R, C>(w, hx, nw, inv, lane, acc);
#pragma unroll
        for (int r = 0; r < R; r++) v[r] = chunk_total<C>(acc[r]);
    }
    __device__ __forceinline__ void dots_plain(const float *x, int lane, float (&v)[R]) const {
        float acc[R][C];
        plain_dots<R, C>(w, x, lane, acc);
#pragma unroll
        for (int r = 0; r < R; r++) v[r] = chunk_total<C>(acc[r]);
    }
};

// The four bytes of w as floats against xv (the empty asm keeps the compiler from folding the mask that made
// w into one bit-field extract per byte: the conversions select their byte themselves).
__device__ __forceinline__ float dot4_bytes(uint32_t w, const float *xv, float s) {
    asm("" : "+v"(w));
    s = fmaf((float)(w & 0xFFu), xv[0], s);
    s = fmaf((float)((w >> 8) & 0xFFu), xv[1], s);
    s = fmaf((float)((w >> 16) & 0xFFu), xv[2], s);
    s = fmaf((float)(w >> 24), xv[3], s);
    return s;
}

// sum_j q_j x_j of half a block with the quants used as stored (Q8_0: biased to unsigned); xv holds the half's
// 16 activations in the order its quant bytes use them (Rows::x_index)
template <bool Q4>
__device__ __forceinline__ float half_block_dot(const uint32_t *qw, const float *xv) {
    float sum;
    if constexpr (Q4) {
        const uint32_t w0 = qw[0], w1 = qw[1];
        sum = dot4_bytes(w1 & 0x0F0F0F0Fu, xv + 4, dot4_bytes(w0 & 0x0F0F0F0Fu, xv, 0.f));
        sum = dot4_bytes((w1 >> 4) & 0x0F0F0F0Fu, xv + 12, dot4_bytes((w0 >> 4) & 0x0F0F0F0Fu, xv + 8, sum));
    } else {
        sum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) sum = dot4_bytes(qw[e] ^ 0x80808080u, xv + 4 * e, sum);  // int8 -> biased unsigned
    }
    return sum;
}

template <int WF, int R, int K>
struct Rows {
    static constexpr bool Q4 = WF == FUSED_WF_Q4_0;
    static constexpr int C = K / 1024;
    static_assert(K % 1024 == 0, "quantised rows are cut into 1024-wide chunks (16 weights a lane)");
    uint32_t q[R][C][Q4 ? 2 : 4];  // the lane's half block: 8 bytes of nibble pairs or 16 int8
    uint32_t d[R][C];              // f16 bits of its block's scale
    template <class RowOf>
    __device__ __forceinline__ void load(const void *quants, const uint16_t *scales, RowOf row_of, int r0, int r1, int lane) {
        const unsigned char *base = reinterpret_cast<const unsigned char *>(quants);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int c = 0; c < C; c++)
                if (r >= r0 && r < r1) {
                    const size_t row = (size_t)row_of(r);
                    const int hb = c * WAVE + lane;  // half block of the row
                    if constexpr (Q4) {
                        const u32x2 t = __builtin_nontemporal_load((global_u32x2_ptr)(base + row * (K / 2) + (size_t)hb * 8));
                        q[r][c][0] = t.x;
                        q[r][c][1] = t.y;
                    } else {
                        const u32x4 t = ld128_global_stream(base + row * K + (size_t)hb * 16);
                        q[r][c][0] = t.x;
                        q[r][c][1] = t.y;
                        q[r][c][2] = t.z;
                        q[r][c][3] = t.w;
                    }
                    d[r][c] = __builtin_nontemporal_load((global_u16_ptr)(scales + row * (K / 32) + (hb >> 1)));
                }
    }
    // the lane's 16 activations of chunk c in the order its quant bytes use them: Q8_0 16 in a row; Q4_0 the
    // low nibbles' eight (8 h + j of the block), then the high nibbles' (16 + 8 h + j)
    __device__ __forceinline__ static int x_index(int c, int lane, int part) {
        const int hb = c * WAVE + lane;
        return Q4 ? (hb >> 1) * 32 + (hb & 1) * 8 + part * 16 : hb * 16 + part * 8;
    }
    __device__ __forceinline__ void finish(const float (&xv)[C][16], float (&v)[R]) const {
        float off[C];
#pragma unroll
        for (int c = 0; c < C; c++) {
            float sx = 0.f;
#pragma unroll
            for (int j = 0; j < 16; j++) sx += xv[c][j];
            off[c] = sx * (Q4 ? 8.f : 128.f);
        }
#pragma unroll
        for (int r = 0; r < R; r++) v[r] = 0.f;
#pragma unroll
        for (int c = 0; c < C; c++)
#pragma unroll
            for (int r = 0; r < R; r++) {
                v[r] += f16_bits_to_f32((uint16_t)d[r][c]) * (half_block_dot<Q4>(q[r][c], xv[c]) - off[c]);
            }
    }
    __device__ __forceinline__ void dots_normed(const float *hx, const float *nw, float inv, int lane, float (&v)[R]) const {
        float xv[C][16];
#pragma unroll
        for (int c = 0; c < C; c++)
#pragma unroll
            for (int part = 0; part < 2; part++) {
                float hv[8], wv[8];
                lds_v8<WF>(hx, K, x_index(c, lane, part), hv);
                lds_v8<WF>(nw, K, x_index(c, lane, part), wv);
#pragma unroll
                for (int e = 0; e < 8; e++) xv[c][part * 8 + e] = (hv[e] * inv) * wv[e];
            }
        finish(xv, v);
    }
    __device__ __forceinline__ void dots_plain(const float *x, int lane, float (&v)[R]) const {
        float xv[C][16];
#pragma unroll
        for (int c = 0; c < C; c++)
#pragma unroll
            for (int part = 0; part < 2; part++) lds_v8<WF>(x, K, x_index(c, lane, part), xv[c] + part * 8);
        finish(xv, v);
    }
};

// ── rows of one matrix restricted to a K slice, as a compute wavefront keeps them for the O and down phases ──
//
// R rows x KS columns [k0, k0 + KS) of an [N][KTOT] matrix. bf16: a register holds four rows of one 128-wide
// part of the slice (lane = 16 * row + position, 8 weights a lane), so a row's sum is the sum of its parts'
// registers followed by a reduction inside a DPP row of 16 lanes. Q8_0 / Q4_0 planes: a lane holds half a
// block (16 weights), a register set eight rows of one part, and a row's sum ends inside 8 lanes. dots()
// leaves in v[q], in every lane of row q * ROWS_PER_SET + lane / LANES_PER_ROW, that row's sum.
template <int WF, int R, int KS, int KTOT>
struct SliceRows;

template <int R, int KS, int KTOT>
struct SliceRows<FUSED_WF_BF16, R, KS, KTOT> {
    static constexpr int P = KS / 128, LANES_PER_ROW = 16, ROWS_PER_SET = 4, Q = R / ROWS_PER_SET;
    static_assert(KS % 128 == 0 && R % ROWS_PER_SET == 0 && Q >= 1, "four rows and a 128-wide part per register");
    u32x4 w[Q][P];
    __device__ __forceinline__ void load(const void *quants, const uint16_t *, int row0, int k0, int lane) {
        const uint16_t *base = reinterpret_cast<const uint16_t *>(quants);
#pragma unroll
        for (int q = 0; q < Q; q++)
#pragma unroll
            for (int p = 0; p < P; p++)
                w[q][p] = ld128_global_stream(base + (size_t)(row0 + q * ROWS_PER_SET + lane / LANES_PER_ROW) * KTOT + k0 + p * 128 +
                                              (lane % LANES_PER_ROW) * 8);
    }
    __device__ __forceinline__ void dots(const float *x, int lane, float (&v)[Q]) const {
        float xv[P][8], acc[Q][P];
#pragma unroll
        for (int p = 0; p < P; p++) lds_v8<FUSED_WF_BF16>(x, KS, p * 128 + (lane % LANES_PER_ROW) * 8, xv[p]);
        dots_from<Q, P>(w, xv, acc);
#pragma unroll
        for (int q = 0; q < Q; q++) v[q] = chunk_total<P>(acc[q]);
#pragma unroll
        for (int q = 0; q < Q; q++) v[q] += dpp_move<0xB1, 0xF>(v[q], 0.f);
#pragma unroll
        for (int q = 0; q < Q; q++) v[q] += dpp_move<0x4E, 0xF>(v[q], 0.f);
#pragma unroll
        for (int q = 0; q < Q; q++) v[q] += dpp_move<0x141, 0xF>(v[q], 0.f);
#pragma unroll
        for (int q = 0; q < Q; q++) v[q] += dpp_move<0x140, 0xF>(v[q], 0.f);
    }
};

template <int WF, int R, int KS, int KTOT>
struct SliceRows {
    static constexpr bool Q4 = WF == FUSED_WF_Q4_0;
    static constexpr int P = KS / 128, LANES_PER_ROW = 8, ROWS_PER_SET = 8, Q = R / ROWS_PER_SET;
    static_assert(KS % 128 == 0 && R % ROWS_PER_SET == 0 && Q >= 1 && KTOT % 32 == 0, "eight rows and a 128-wide part per register set");
    uint32_t q[Q][P][Q4 ? 2 : 4];  // the lane's half block: 8 bytes of nibble pairs or 16 int8
    uint32_t d[Q][P];              // f16 bits of its block's scale
    __device__ __forceinline__ void load(const void *quants, const uint16_t *scales, int row0, int k0, int lane) {
        const unsigned char *base = reinterpret_cast<const unsigned char *>(quants);
#pragma unroll
        for (int s = 0; s < Q; s++)
#pragma unroll
            for (int p = 0; p < P; p++) {
                const size_t row = (size_t)(row0 + s * ROWS_PER_SET + lane / LANES_PER_ROW);
                const int hb = (k0 + p * 128) / 16 + lane % LANES_PER_ROW;  // half block of the row
                if constexpr (Q4) {
                    const u32x2 t = __builtin_nontemporal_load((global_u32x2_ptr)(base + row * (KTOT / 2) + (size_t)hb * 8));
                    q[s][p][0] = t.x;
                    q[s][p][1] = t.y;
                } else {
                    const u32x4 t = ld128_global_stream(base + row * KTOT + (size_t)hb * 16);
                    q[s][p][0] = t.x;
                    q[s][p][1] = t.y;
                    q[s][p][2] = t.z;
                    q[s][p][3] = t.w;
                }
                d[s][p] = __builtin_nontemporal_load((global_u16_ptr)(scales + row * (KTOT / 32) + (hb >> 1)));
            }
    }
    __device__ __forceinline__ void dots(const float *x, int lane, float (&v)[Q]) const {
        float xv[P][16], off[P];
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int hb = p * 8 + lane % LANES_PER_ROW;  // half block inside the slice (slices start on a block)
#pragma unroll
            for (int part = 0; part < 2; part++)
                lds_v8<WF>(x, KS, Q4 ? (hb >> 1) * 32 + (hb & 1) * 8 + part * 16 : hb * 16 + part * 8, xv[p] + part * 8);
            float sx = 0.f;
#pragma unroll
            for (int j = 0; j < 16; j++) sx += xv[p][j];
            off[p] = sx * (Q4 ? 8.f : 128.f);
        }
#pragma unroll
        for (int s = 0; s < Q; s++) v[s] = 0.f;
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int s = 0; s < Q; s++) v[s] += f16_bits_to_f32((uint16_t)d[s][p]) * (half_block_dot<Q4>(q[s][p], xv[p]) - off[p]);
#pragma unroll
        for (int s = 0; s < Q; s++) v[s] += dpp_move<0xB1, 0xF>(v[s], 0.f);
#pragma unroll
        for (int s = 0; s < Q; s++) v[s] += dpp_move<0x4E, 0xF>(v[s], 0.f);
#pragma unroll
        for (int s = 0; s < Q; s++) v[s] += dpp_move<0x141, 0xF>(v[s], 0.f);
    }
};


// ── K8: Q4_K / Q6_K matrices as byte planes (kquant_planes8.h) ──
//
// A lane holds one 16-weight sub-block of each 1024-wide chunk of a row: its 16 signed bytes, its scale and
// minimum factor, and the f16 d | dmin of its 256-wide super-block, which is exactly one DPP row of 16 lanes.
// The activations go through the reference's Q8_K quantisation (src/graph_builder/emit_quant.rs:422-466:
// amax over the block, d = amax / 127, q = roundeven(x * 127 / amax) clamped to +-127) in every wavefront, the
// products are integer dot products, and a block contributes (d * act_d) * float(sum sc * isum) -
// (dmin * act_d) * float(sum mn * bsum) with both sums exact in i32 (emit_quant.rs:165-816); blocks are added
// in ascending order, as the reference adds them.
typedef const uint32_t __attribute__((address_space(1))) *global_u32_ptr;

template <int R, int K>
struct Rows<FUSED_WF_K8, R, K> {
    static constexpr int C = K / 1024;
    static constexpr int RS = K / 8 + K / 64;  // bytes of a row's scale record: (sc, mn) per 16 weights, then (d, dmin) per 256
    static_assert(K % 1024 == 0, "K8 rows are cut into 1024-wide chunks (16 weights a lane)");
    u32x4 q[R][C];
    uint32_t sub[R][C], dd[R][C];
    template <class RowOf>
    __device__ __forceinline__ void load(const void *quants, const uint16_t *scales, RowOf row_of, int r0, int r1, int lane) {
        const unsigned char *base = reinterpret_cast<const unsigned char *>(quants);
        const unsigned char *rec = reinterpret_cast<const unsigned char *>(scales);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int c = 0; c < C; c++)
                if (r >= r0 && r < r1) {
                    const size_t row = (size_t)row_of(r);
                    const int s16 = c * WAVE + lane;  // sub-block of the row
                    q[r][c] = ld128_global_stream(base + row * K + (size_t)s16 * 16);
                    sub[r][c] = __builtin_nontemporal_load((global_u16_ptr)(rec + row * RS + (size_t)s16 * 2));
                    dd[r][c] = __builtin_nontemporal_load((global_u32_ptr)(rec + row * RS + K / 8 + (size_t)(s16 / 16) * 4));
                }
    }
    // v[r]: the row's value in lane 0, zero in the others (the caller's sum over the wavefront keeps it exact)
    __device__ __forceinline__ void finish(const float (&xv)[C][16], int lane, float (&v)[R]) const {
        Q8kLane a[C];
#pragma unroll
        for (int c = 0; c < C; c++) a[c] = q8k_lane(xv[c], dpp_row_fmax(abs_max16(xv[c])));
#pragma unroll
        for (int r = 0; r < R; r++) {
            float acc = 0.f;
#pragma unroll
            for (int c = 0; c < C; c++) {
                const float p = k8_block(q[r][c], sub[r][c], dd[r][c], a[c]);
#pragma unroll
                for (int b = 0; b < 4; b++)  // the chunk's four blocks, ascending
                    acc = __fadd_rn(acc, __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), 16 * b)));
            }
            v[r] = lane == 0 ? acc : 0.f;
        }
    }
    __device__ __forceinline__ void dots_normed(const float *hx, const float *nw, float inv, int lane, float (&v)[R]) const {
        float xv[C][16];
#pragma unroll
        for (int c = 0; c < C; c++)
#pragma unroll
            for (int part = 0; part < 2; part++) {
                float hv[8], wv[8];
                lds_v8<FUSED_WF_K8>(hx, K, (c * WAVE + lane) * 16 + part * 8, hv);
                lds_v8<FUSED_WF_K8>(nw, K, (c * WAVE + lane) * 16 + part * 8, wv);
#pragma unroll
                for (int e = 0; e < 8; e++) xv[c][part * 8 + e] = (hv[e] * inv) * wv[e];
            }
        finish(xv, lane, v);
    }
    __device__ __forceinline__ void dots_plain(const float *x, int lane, float (&v)[R]) const {
        float xv[C][16];
#pragma unroll
        for (int c = 0; c < C; c++)
#pragma unroll
            for (int part = 0; part < 2; part++) lds_v8<FUSED_WF_K8>(x, K, (c * WAVE + lane) * 16 + part * 8, xv[c] + part * 8);
        finish(xv, lane, v);
    }
};

// R rows x the K slice [k0, k0 + KS) of a K8 matrix with KTOT columns. A register set holds four rows of one
// 256-wide block that the slice touches (lane = 16 * row + sub-block of the block); lanes whose sub-block lies
// outside the slice carry zeros. A block that the slice shares with a neighbouring slice takes its Q8_K
// maximum from both sides: `shared_max[0]` is the other side's maximum of the block the slice starts in,
// `shared_max[1]` that of the block it ends in.
template <int R, int KS, int KTOT>
struct SliceRows<FUSED_WF_K8, R, KS, KTOT> {
    static constexpr int LANES_PER_ROW = 16, ROWS_PER_SET = 4, Q = R / ROWS_PER_SET;
    static constexpr int P = (KS + 255) / 256;  // blocks a slice touches (slices start on a block or end on one)
    static constexpr int RS = KTOT / 8 + KTOT / 64;
    static_assert(R % ROWS_PER_SET == 0 && Q >= 1 && KTOT % 256 == 0 && KS % 16 == 0, "four rows and one block per register set");
    static_assert(KS % 256 == 0 || (KS % 128 == 0 && P == KS / 256 + 1), "slices are whole blocks, or whole blocks and a half");
    u32x4 q[Q][P];
    uint32_t sub[Q][P], dd[Q][P];
    // global column of the lane's sub-block in part p, and whether it lies inside the slice
    __device__ __forceinline__ static int col(int k0, int p, int lane) { return (k0 / 256 + p) * 256 + (lane % LANES_PER_ROW) * 16; }
    __device__ __forceinline__ static bool inside(int k0, int p, int lane) {
        const int k = col(k0, p, lane);
        return k >= k0 && k < k0 + KS;
    }
    __device__ __forceinline__ void load(const void *quants, const uint16_t *scales, int row0, int k0, int lane, int s0 = 0, int s1 = Q) {
        const unsigned char *base = reinterpret_cast<const unsigned char *>(quants);
        const unsigned char *rec = reinterpret_cast<const unsigned char *>(scales);
#pragma unroll
        for (int s = 0; s < Q; s++)
#pragma unroll
            for (int p = 0; p < P; p++) {
                if (s < s0 || s >= s1) continue;
                const size_t row = (size_t)(row0 + s * ROWS_PER_SET + lane / LANES_PER_ROW);
                const bool in = inside(k0, p, lane);
                const int k = in ? col(k0, p, lane) : k0;  // lanes outside re-read the slice's first sub-block
                q[s][p] = ld128_global_stream(base + row * KTOT + k);
                sub[s][p] = __builtin_nontemporal_load((global_u16_ptr)(rec + row * RS + (size_t)(k / 16) * 2));
                dd[s][p] = __builtin_nontemporal_load((global_u32_ptr)(rec + row * RS + KTOT / 8 + (size_t)(k0 / 256 + p) * 4));
                if (!in) q[s][p] = u32x4{0u, 0u, 0u, 0u};
            }
    }
    __device__ __forceinline__ void dots(const float *x, int lane, int k0, const float *shared_max, float (&v)[Q]) const {
        Q8kLane a[P];
#pragma unroll
        for (int p = 0; p < P; p++) {
            float xv[16];
            const bool in = inside(k0, p, lane);
            const int local = in ? col(k0, p, lane) - k0 : 0;
            lds_v8<FUSED_WF_K8>(x, KS, local, xv);
            lds_v8<FUSED_WF_K8>(x, KS, local + 8, xv + 8);
#pragma unroll
            for (int j = 0; j < 16; j++) xv[j] = in ? xv[j] : 0.f;
            float amax = dpp_row_fmax(abs_max16(xv));
            const int b_lo = (k0 / 256 + p) * 256;  // the block's first column
            if (b_lo < k0) amax = fmaxf(amax, shared_max[0]);
            if (b_lo + 256 > k0 + KS) amax = fmaxf(amax, shared_max[1]);
            a[p] = q8k_lane(xv, amax);
        }
#pragma unroll
        for (int s = 0; s < Q; s++) {
            float acc = 0.f;
#pragma unroll
            for (int p = 0; p < P; p++) acc = __fadd_rn(acc, k8_block(q[s][p], sub[s][p], dd[s][p], a[p]));
            v[s] = acc;
        }
    }
};

// The attention split of a workgroup for a cache of kv_len rows (the new row included).
template <class GE>
struct Split {
    int kh, split, nsl, n0, cnt, cached;
    bool owner;
    __device__ Split(int wg, int pos) {
        const int kv_len = pos + 1;
        const int chunk = (kv_len + GE::SPH - 1) / GE::SPH;
        nsl = (kv_len + chunk - 1) / chunk;
        kh = wg % GE::KVH;
        split = wg / GE::KVH;
        n0 = split * chunk;
        cnt = min(kv_len, n0 + chunk) - n0;
        if (cnt < 0) cnt = 0;
        owner = split == nsl - 1;  // holds row `pos`, which is not in the cache yet
        cached = min(cnt, pos - n0);
        if (cached < 0) cached = 0;
    }
};

// LM head (reference src/hf/emitter.rs:828-862) and the wavefront's best row. The workgroup owns a contiguous
// run of the vocabulary; all eight wavefronts (the communicating ones have nothing else left to do) take
// batches of HR rows in turn, the next batch's rows in flight while this one is multiplied. EARLY: the
// caller has not yet passed the barrier behind which the last hidden state is staged, and the first batch is
// requested before it. Ends behind the barrier after which head_v / head_i hold every wavefront's best row.
constexpr int HEAD_WORKERS = NCW + 4;
template <class GE, int WF, bool EARLY>
__device__ __forceinline__ void head_rows(const FusedDecodeArgs &a, Lds<GE> &sm, const int wg, const int worker, const int lane) {
    constexpr int HR = GE::HR, HC = GE::HIDDEN / 512;
    const int per_wg = (a.vocab + GE::NWG - 1) / GE::NWG;
    const int row0 = wg * per_wg, row1 = min(a.vocab, row0 + per_wg);
    const int nbatch = (max(row1 - row0, 0) + HEAD_WORKERS * HR - 1) / (HEAD_WORKERS * HR);  // batches of this wavefront
    u32x4 wn[HR][HC];
    auto request = [&](int b) {
#pragma unroll
        for (int r = 0; r < HR; r++) {
            const int row = min(row0 + (b * HEAD_WORKERS + worker) * HR + r, a.vocab - 1);  // rows past the end re-read the last one
#pragma unroll
            for (int c = 0; c < HC; c++) wn[r][c] = ld128_global_stream(a.head_w + (size_t)row * GE::HIDDEN + (c * WAVE + lane) * 8);
        }
    };
    if (nbatch > 0) request(0);
    if (EARLY) wg_barrier();
    const float tot = ((sm.red[0] + sm.red[1]) + sm.red[2]) + sm.red[3];
    const float inv = __builtin_amdgcn_rsqf(tot / (float)GE::HIDDEN + a.eps);
    float xv[HC][8];
#pragma unroll
    for (int c = 0; c < HC; c++) {
        float hv[8], wv[8];
        lds_v8<WF>(sm.hx, GE::HIDDEN, (c * WAVE + lane) * 8, hv);
        lds_v8<WF>(sm.nw, GE::HIDDEN, (c * WAVE + lane) * 8, wv);
#pragma unroll
        for (int e = 0; e < 8; e++) xv[c][e] = (hv[e] * inv) * wv[e];
    }
    float best_v = -INFINITY;
    int best_i = -1;
    for (int b = 0; b < nbatch; b++) {
        u32x4 wc[HR][HC];
#pragma unroll
        for (int r = 0; r < HR; r++)
#pragma unroll
            for (int c = 0; c < HC; c++) wc[r][c] = wn[r][c];
        if (b + 1 < nbatch) request(b + 1);
        float acc[HR][HC], v[HR];
        dots_from<HR, HC>(wc, xv, acc);
#pragma unroll
        for (int r = 0; r < HR; r++) v[r] = chunk_total<HC>(acc[r]);
        wave_sum_n<HR>(v);
        const int first = row0 + (b * HEAD_WORKERS + worker) * HR;
        float mine = 0.f;
#pragma unroll
        for (int r = 0; r < HR; r++) {
            mine = lane == r ? v[r] : mine;
            // of equal maxima the later row wins (Rust Iterator::max_by, reference src/generate.rs:735-742)
            if (first + r < row1 && (best_i < 0 || v[r] >= best_v)) {
                best_v = v[r];
                best_i = first + r;
            }
        }
        if (lane < HR && first + lane < row1) a.logits[first + lane] = mine;
    }
    if (lane == 0) {
        sm.head_v[worker] = best_v;
        sm.head_i[worker] = best_i;
    }
    wg_barrier();
}

// Registers of one compute wavefront that hold its slice of a layer.
template <class GE, int WF>
struct Slice {
    Rows<WF, GE::RQW, GE::HIDDEN> wq;
    u32x4 kr[GE::NR], vr[GE::NR];
    SliceRows<WF, GE::RPW, GE::KSO, GE::QD> wo;
    Rows<WF, GE::RGW, GE::HIDDEN> wg;
    SliceRows<WF, GE::RPW, GE::KSD, GE::INTER> wd;
};

template <class GE, int WF>
__device__ __forceinline__ void compute_role(const FusedDecodeArgs &a, Lds<GE> &sm, const int wg, const int cw,
                                             const int lane, const int pos) {
    const Split<GE> sp(wg, pos);
    constexpr int LPR = GE::LPR, RPI = GE::RPI, G = GE::G, HD = GE::HD, NR = GE::NR;
    const int sub = lane / LPR, dl = lane % LPR;
    const int L = a.n_layers;
    Slice<GE, WF> s;

    // Requests are spread over the step in small batches (rows [r0, r1) of a slice at a time): a batch that
    // overfills the CU's memory pipeline blocks the wavefront that issues it, and a burst from all
    // CUs at once delays the polls of the communication wavefronts behind it.
    auto load_wq = [&](const FusedLayerPtrs &lp, int r0, int r1) {
        s.wq.load(lp.wqkv, lp.sqkv, [&](int r) { return GE::qkv_row(sp.kh, sp.split * GE::RQ + cw * GE::RQW + r); }, r0, r1, lane);
    };
    constexpr bool RECOMPUTE = GE::XR > 0 || (WF == FUSED_WF_K8 && NR > 4);
    // Element offset of this lane's part of round `round` of the split. With streamed rounds (XR > 0) the
    // lane's row is made opaque at every use: the offsets of all rounds, kept across the layer loop as loop
    // invariants, would take the registers the slices need (and a spilled one comes back behind every
    // outstanding weight request).
    auto kv_off = [&](int round) -> size_t {
        int r0 = cw * RPI + sub;
        if constexpr (RECOMPUTE) asm volatile("" : "+v"(r0));
        const int rl = round * NCW * RPI + r0;
        const int row = rl < sp.cached ? sp.n0 + rl : 0;  // rows outside the split re-read a valid row
        if constexpr (GE::XR > 0) return (size_t)(((uint32_t)sp.kh * (uint32_t)a.max_len + (uint32_t)row) * HD + dl * 8);  // < 2^32: checked by the host
        else return ((size_t)sp.kh * a.max_len + row) * HD + dl * 8;
    };
    auto load_kv = [&](const FusedLayerPtrs &lp, int i0, int i1) {
#pragma unroll
        for (int i = 0; i < NR; i++) {
            if (i < i0 || i >= i1) continue;
            const size_t off = kv_off(i);
            s.kr[i] = ld128_global_stream(lp.kcache + off);
            s.vr[i] = ld128_global_stream(lp.vcache + off);
        }
    };
    // (the lane index is made opaque for the same reason as in kv_off: per-lane row offsets are recomputed, not held)
    auto opaque_lane = [&]() {
        int ln = lane;
        if constexpr (RECOMPUTE) asm volatile("" : "+v"(ln));
        return ln;
    };
    auto load_wo = [&](const FusedLayerPtrs &lp) {
        s.wo.load(lp.wo, lp.so, GE::partial_row(sp.split, cw * GE::RPW), sp.kh * GE::KSO, opaque_lane());
    };
    // bf16 keeps gate and up rows interleaved (g0, u0, g1, u1, ...); the quantised formats keep the run as
    // uploaded, all gate rows and then all up rows, so local row r = 2 p + (0 gate | 1 up) of pair p.
    // Pairs are dealt by KV-head group first (wgp), so a group's SiLU*up values are one K slice of down.
    const int wgp = sp.kh * GE::SPH + sp.split;
    auto load_wg = [&](const FusedLayerPtrs &lp, int r0, int r1) {
        s.wg.load(lp.wgu, lp.sgu, [&](int r) {
            const int lr = cw * GE::RGW + r;
            return WF == FUSED_WF_BF16 ? wgp * GE::RG + lr : (lr & 1) * GE::INTER + wgp * GE::APW + (lr >> 1);
        }, r0, r1, lane);
    };
    auto load_wd = [&](const FusedLayerPtrs &lp) {
        s.wd.load(lp.wd, lp.sd, GE::partial_row(sp.split, cw * GE::RPW), sp.kh * GE::KSD, opaque_lane());
    };

    // What a phase start asks for drains while the phase computes and, after that, in front of the polls of the
    // exchange behind it, so the requests of a layer are shared out by what each phase can hide (Qwen3-0.6B, bf16,
    // KB a workgroup): Q|K|V 24 (half the gate|up rows), attention 32 (next Q|K|V rows), O 32 (down rows, first
    // cache rows), gate|up 32 (next O rows, the other cache rows), down 24 (half of the next gate|up rows). With
    // the down rows beside the gate|up rows at the start of the Q|K|V phase (40 KB there, 8 with the O phase) and
    // two thirds of the gate|up rows with the down phase a layer took 11.93 us instead of 11.52.
    // (The K-quant form asks for half the bytes and was 2-3 % faster with the earlier lots: it keeps them.)
    constexpr bool K8_LOTS = WF == FUSED_WF_K8;
    constexpr int KV_CUT = NR / 2, WG_CUT = K8_LOTS ? 2 * GE::RGW / 3 : GE::RGW / 2;
    // With eight row rounds in registers a layer's slices and the next layer's cache rows do not all fit at once
    // (a spilled value would come back through the memory pipeline, behind every outstanding weight request): those
    // instances request the second half of the cache rows and a quarter of the Q|K|V rows one phase later, when the
    // registers they land in have just been read for the last time. (All Q|K|V rows at the start of the attention
    // phase spill 20 to 192 bytes a lane in three of the eight instances; none of them there, as it was first
    // built, costs 0.489 -> 0.507 ms a token at 4000 rows. Six rounds fit without any of this: 0.447 -> 0.421 ms
    // at 2100 rows.)
    constexpr bool LATE = NR > 6;
    constexpr int WQ_EARLY = LATE ? 3 * GE::RQW / 4 : GE::RQW;  // Q|K|V rows of the next layer asked for at the start of the attention phase
    // Their cache rows go out in four lots so that no phase start asks for much more than the CU keeps in flight
    // (a wavefront that asks for more waits, with its phase's arithmetic behind it): the first rounds at the end of
    // the attention phase, the rest of the first half with the O phase, the second half with gate|up and down.
    constexpr int LATE_KV_P2 = LATE ? KV_CUT / 2 : 0, LATE_KV_P4 = LATE ? (NR - KV_CUT) / 2 : 0;
    {
        // the first layer's slice, in the order the loop re-requests it (the rest follows inside the loop)
        const FusedLayerPtrs lp = sm.lp[0];
        load_wq(lp, 0, GE::RQW);
        load_kv(lp, 0, NR);
        load_wo(lp);
        load_wg(lp, 0, WG_CUT);
    }

    for (int l = 0; l < L; l++) {
        // The slice of the next layer replaces each phase's registers once the phase is over. After the
        // last layer the first layer's slice is requested again and never used: the requests keep the
        // number of loads in flight the same in every iteration, which the wait counts rely on.
        const FusedLayerPtrs nx = sm.lp[l + 1 < L ? l + 1 : 0];
        const bool has_bias = sm.lp[l].qkv_bias != nullptr;

        // ── Q|K|V rows (RMSNorm applied on the way in; reference src/hf/emitter.rs:560-619) ──
        wg_barrier();
        // Requests go out at the start of a phase, never right before the communicating wavefronts poll:
        // the CU's vector memory pipeline returns data in order, so a poll issued behind a weight request
        // waits for HBM. Here: the second half of this layer's gate|up rows (registers last read one layer ago).
        if (K8_LOTS && !LATE) load_wd(sm.lp[l]);
        load_wg(sm.lp[l], WG_CUT, GE::RGW);
        {
            const float tot = ((sm.red[0] + sm.red[1]) + sm.red[2]) + sm.red[3];
            const float inv = __builtin_amdgcn_rsqf(tot / (float)GE::HIDDEN + a.eps);
            float v[GE::RQW];
            s.wq.dots_normed(sm.hx, sm.nw, inv, lane, v);
            wave_sum_n<GE::RQW>(v);
            if (has_bias) {
#pragma unroll
                for (int r = 0; r < GE::RQW; r++) v[r] = v[r] + sm.bias[cw * GE::RQW + r];
            }
            float mine = 0.f;
#pragma unroll
            for (int r = 0; r < GE::RQW; r++) mine = lane == r ? v[r] : mine;
            if (lane < GE::RQW) sm.pub[cw * GE::RQW + lane] = mine;
        }
        wg_barrier();

        // ── attention over this workgroup's split of the cache (reference src/hf/emitter.rs:709-731).
        //    Every wavefront leaves the (max, sum, P.V) of its own rows in LDS; the publishing threads
        //    merge the four. ──
        wg_barrier();
        load_wq(nx, 0, WQ_EARLY);
        if (sp.split < sp.nsl) {
            float qv[G][8];
#pragma unroll
            for (int g = 0; g < G; g++) lds_x8(sm.qs[g], dl * 8, qv[g]);
            const bool with_new = sp.owner && cw == 0;  // the new row rides with wavefront 0 of the last split
            // The rounds held in registers are taken PR at a time, at most four (the float forms of more would not
            // fit beside the weight slices, and a spilled register is reloaded through the same in-order memory
            // pipeline the weight requests wait in): one pass up to four rounds, two of three or of four beyond;
            // passes after the first rescale what the earlier ones left. A pass costs its reductions and
            // exponentials whatever its width: eight rounds as four passes of two took 0.519 ms a token at 4000 rows,
            // as two of four 0.507. Streamed sets (below) stay two rounds wide, the ring holds three of them. The
            // new row rides with the last pass.
            constexpr int PR = NR == 6 ? 3 : (NR == 8 ? 4 : NR), NPASS = NR / PR;  // rounds a pass over the held rows
            constexpr int PX = 2;                                                  // rounds a streamed set
            static_assert(NR % PR == 0, "row rounds are taken in equal passes");
            float m[G], lsum[G], acc[G][8];
            // One pass: rounds i0 .. i0 + PW - 1 of the split, their rows handed over by kk(i) / vv(i).
            auto attn_pass = [&](auto first_tag, auto width_tag, auto kk, auto vv, const int i0, const bool last) __attribute__((always_inline)) {
                constexpr bool FIRST = decltype(first_tag)::value;
                constexpr int PW = decltype(width_tag)::value;  // rounds of this pass
                // slot PW is the new row (last pass only; elsewhere it is dead and multiplies zeros)
                float kf[PW + 1][8];
#pragma unroll
                for (int i = 0; i < PW; i++) unpack8f(kk(i), kf[i]);
                if (last) lds_x8(sm.knew, dl * 8, kf[PW]);
                else {
#pragma unroll
                    for (int e = 0; e < 8; e++) kf[PW][e] = 0.f;
                }
                float sc[G][PW + 1];
#pragma unroll
                for (int g = 0; g < G; g++)
#pragma unroll
                    for (int i = 0; i <= PW; i++) sc[g][i] = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++)
#pragma unroll
                    for (int g = 0; g < G; g++)
#pragma unroll
                        for (int i = 0; i <= PW; i++) sc[g][i] = fmaf(kf[i][e], qv[g][e], sc[g][i]);
                // sums over the lanes of a row, all (head, row) chains side by side
#pragma unroll
                for (int g = 0; g < G; g++)
#pragma unroll
                    for (int i = 0; i <= PW; i++) sc[g][i] += dpp_move<0xB1, 0xF>(sc[g][i], 0.f);
#pragma unroll
                for (int g = 0; g < G; g++)
#pragma unroll
                    for (int i = 0; i <= PW; i++) sc[g][i] += dpp_move<0x4E, 0xF>(sc[g][i], 0.f);
#pragma unroll
                for (int g = 0; g < G; g++)
#pragma unroll
                    for (int i = 0; i <= PW; i++) sc[g][i] += dpp_move<0x141, 0xF>(sc[g][i], 0.f);
                if (LPR == 16) {
#pragma unroll
                    for (int g = 0; g < G; g++)
#pragma unroll
                        for (int i = 0; i <= PW; i++) sc[g][i] += dpp_move<0x140, 0xF>(sc[g][i], 0.f);
                }
                bool live[PW + 1];
#pragma unroll
                for (int i = 0; i < PW; i++) live[i] = ((i0 + i) * NCW + cw) * RPI + sub < sp.cached;
                live[PW] = last && with_new;
                float mp[G];
#pragma unroll
                for (int g = 0; g < G; g++) {
                    mp[g] = -INFINITY;
#pragma unroll
                    for (int i = 0; i <= PW; i++) {
                        sc[g][i] = live[i] ? sc[g][i] * a.scale : -INFINITY;
                        mp[g] = fmaxf(mp[g], sc[g][i]);
                    }
                }
                wave_max_n<G>(mp);
                // softmax terms against the wavefront's own maximum (max, exp, sum:
                // reference emit_softmax, src/graph_builder/emit_linalg.rs:509-528)
                float alpha[G];
#pragma unroll
                for (int g = 0; g < G; g++) {
                    if (FIRST) {
                        m[g] = mp[g];
                        alpha[g] = 0.f;
                        lsum[g] = 0.f;
                    } else {
                        const float mn = fmaxf(m[g], mp[g]);
                        alpha[g] = m[g] == -INFINITY ? 0.f : __expf(m[g] - mn);  // nothing live so far: nothing to keep
                        m[g] = mn;
                        lsum[g] *= alpha[g];
                    }
                }
                float pr[G][PW + 1];
#pragma unroll
                for (int g = 0; g < G; g++) {
#pragma unroll
                    for (int i = 0; i <= PW; i++) {
                        pr[g][i] = live[i] ? __expf(sc[g][i] - m[g]) : 0.f;
                        // a cache row is counted by the first of its lanes, the new row by lane 0
                        if (i < PW ? dl == 0 : lane == 0) lsum[g] += pr[g][i];
                    }
                }
                if (last) {
                    wave_sum_n<G>(lsum);
                    if (lane < G) {
                        float mm = 0.f, ll = 0.f;
#pragma unroll
                        for (int g = 0; g < G; g++) {
                            mm = lane == g ? m[g] : mm;
                            ll = lane == g ? lsum[g] : ll;
                        }
                        sm.wstat[cw][lane][0] = mm;
                        sm.wstat[cw][lane][1] = ll;
                    }
                }
                float vf[PW + 1][8];
#pragma unroll
                for (int i = 0; i < PW; i++) unpack8f(vv(i), vf[i]);
                if (last) lds_x8(sm.vnew, dl * 8, vf[PW]);
                else {
#pragma unroll
                    for (int e = 0; e < 8; e++) vf[PW][e] = 0.f;
                }
#pragma unroll
                for (int g = 0; g < G; g++)
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[g][e] = FIRST ? 0.f : acc[g][e] * alpha[g];
#pragma unroll
                for (int i = 0; i <= PW; i++) {
#pragma unroll
                    for (int g = 0; g < G; g++) {
                        const float p = (i < PW || sub == 0) ? pr[g][i] : 0.f;  // the new row: one row group only
#pragma unroll
                        for (int e = 0; e < 8; e++) acc[g][e] = fmaf(p, vf[i][e], acc[g][e]);
                    }
                }
            };
            // Rounds past the held ones (XR > 0: caches longer than the registers hold) are streamed inside
            // the phase through a ring of XD sets of PX rounds: one is multiplied while XD - 1 are in flight
            // (they take the registers of the held rounds, which are dead by then). A request past the split's
            // last round reads a valid row that nobody uses (kv_off), so the requests need no conditions.
            constexpr int XD = 3;
            int npx = 0;
            if constexpr (GE::XR > 0) {
                const int over = sp.cached - NR * NCW * RPI;
                npx = over > 0 ? (over + PX * NCW * RPI - 1) / (PX * NCW * RPI) : 0;
            }
            u32x4 kx[XD][PX], vx[XD][PX];
            auto load_x = [&](u32x4 (&kxs)[PX], u32x4 (&vxs)[PX], const int r0) __attribute__((always_inline)) {
                const uint16_t *kc = sm.lp[l].kcache, *vc = sm.lp[l].vcache;
#pragma unroll
                for (int i = 0; i < PX; i++) {
                    const size_t off = kv_off(r0 + i);
                    kxs[i] = ld128_global_stream(kc + off);
                    vxs[i] = ld128_global_stream(vc + off);
                }
            };
#pragma unroll
            for (int ps = 0; ps < NPASS; ps++) {
                const int i0 = ps * PR;
                auto kk = [&](int i) { return s.kr[i0 + i]; };
                auto vv = [&](int i) { return s.vr[i0 + i]; };
                const bool last = ps == NPASS - 1 && npx == 0;
                // the first streamed sets go out ahead of the last held pass, into registers of earlier rounds
                if constexpr (GE::XR > 0) {
                    if (ps == NPASS - 1 && npx > 0) {
#pragma unroll
                        for (int j = 0; j < XD - 1; j++) load_x(kx[j], vx[j], NR + j * PX);
                    }
                }
                if (ps == 0) attn_pass(std::true_type{}, std::integral_constant<int, PR>{}, kk, vv, i0, last);
                else attn_pass(std::false_type{}, std::integral_constant<int, PR>{}, kk, vv, i0, last);
            }
            if constexpr (GE::XR > 0) {
                // set x + j sits in ring slot j; the request that refills the slot freed last goes out first
                auto ring_step = [&](auto self, auto jc, const int x) __attribute__((always_inline)) -> void {
                    constexpr int j = decltype(jc)::value;
                    load_x(kx[(j + XD - 1) % XD], vx[(j + XD - 1) % XD], NR + (x + j + XD - 1) * PX);
                    attn_pass(std::false_type{}, std::integral_constant<int, PX>{}, [&](int i) { return kx[j][i]; }, [&](int i) { return vx[j][i]; },
                              NR + (x + j) * PX, x + j == npx - 1);
                    if constexpr (j + 1 < XD) {
                        if (x + j + 1 < npx) self(self, std::integral_constant<int, j + 1>{}, x);
                    }
                };
                for (int x = 0; x < npx; x += XD) ring_step(ring_step, std::integral_constant<int, 0>{}, x);
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                float *dst = &sm.part[cw * RPI + sub][g][dl * 8];
                *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[g][0], acc[g][1], acc[g][2], acc[g][3]};
                *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{acc[g][4], acc[g][5], acc[g][6], acc[g][7]};
            }
        }
        load_wq(nx, WQ_EARLY, GE::RQW);  // behind the arithmetic that needed the registers
        if (LATE) load_kv(nx, 0, LATE_KV_P2);
        wg_barrier();

        // ── O projection rows (reference src/hf/emitter.rs:738-745) ──
        wg_barrier();
        load_kv(nx, LATE_KV_P2, KV_CUT);
        if (!K8_LOTS || LATE) load_wd(sm.lp[l]);
        {
            using S = decltype(s.wo);
            float v[S::Q];
            if constexpr (WF == FUSED_WF_K8) s.wo.dots(sm.attn, lane, sp.kh * GE::KSO, sm.nbmax, v);  // whole blocks: nbmax is not read
            else s.wo.dots(sm.attn, lane, v);
            if (lane % S::LANES_PER_ROW == 0) {
#pragma unroll
                for (int q = 0; q < S::Q; q++) sm.pub[cw * GE::RPW + q * S::ROWS_PER_SET + lane / S::LANES_PER_ROW] = v[q];
            }
        }
        wg_barrier();

        // ── gate|up rows, SiLU(gate) * up (reference src/hf/emitter.rs:787-799) ──
        wg_barrier();
        if (!LATE) load_kv(nx, KV_CUT, NR);
        if (LATE) load_kv(nx, KV_CUT, KV_CUT + LATE_KV_P4);
        load_wo(nx);
        {
            const float tot = ((sm.red[0] + sm.red[1]) + sm.red[2]) + sm.red[3];
            const float inv = __builtin_amdgcn_rsqf(tot / (float)GE::HIDDEN + a.eps);
            float v[GE::RGW];
            s.wg.dots_normed(sm.hx, sm.nw, inv, lane, v);
            wave_sum_n<GE::RGW>(v);
            float gte = 0.f, up = 0.f;
#pragma unroll
            for (int r = 0; r < GE::RGW; r += 2) {
                gte = lane == r / 2 ? v[r] : gte;
                up = lane == r / 2 ? v[r + 1] : up;
            }
            if (lane < GE::RGW / 2) sm.pub[cw * (GE::RGW / 2) + lane] = (gte * __builtin_amdgcn_rcpf(1.0f + __expf(-gte))) * up;
        }
        wg_barrier();

        // ── down rows (reference src/hf/emitter.rs:801-804; the residual is added by the readers) ──
        wg_barrier();
        load_wg(nx, 0, WG_CUT);
        if (LATE) load_kv(nx, KV_CUT + LATE_KV_P4, NR);
        {
            using S = decltype(s.wd);
            float v[S::Q];
            if constexpr (WF == FUSED_WF_K8) s.wd.dots(sm.act, lane, sp.kh * GE::KSD, sm.nbmax, v);
            else s.wd.dots(sm.act, lane, v);
            if (lane % S::LANES_PER_ROW == 0) {
#pragma unroll
                for (int q = 0; q < S::Q; q++) sm.pub[cw * GE::RPW + q * S::ROWS_PER_SET + lane / S::LANES_PER_ROW] = v[q];
            }
        }
        wg_barrier();
    }

    if (a.head_w) head_rows<GE, WF, true>(a, sm, wg, cw, lane);
}

// Slot of hidden element k in the XH / XO areas: the communicating thread c = k % 256 owns elements
// k = c + 256 j (the partition of the RMSNorm's sum of squares in gemv_bf16.hip), so its elements
// 2u and 2u + 1 share 16-byte unit u * 256 + c.
__device__ __forceinline__ int hidden_slot(int k) {
    const int j = k / CT, c = k % CT;
    return 2 * ((j / 2) * CT + c) + (j & 1);
}

__device__ __forceinline__ unsigned xcc_id() { return __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 0xF; }

template <class GE, int WF>
__device__ __forceinline__ void comm_role(const FusedDecodeArgs &a, Lds<GE> &sm, const int wg, const int cwv,
                                          const int lane, const int pos, const uint32_t launches) {
    constexpr int G = GE::G, HD = GE::HD, NJ = GE::NJ;
    const Split<GE> sp(wg, pos);
    const int ct = cwv * WAVE + lane;
    const int L = a.n_layers;
    const uint32_t base = launches * (uint32_t)L;
    PollState ps{a.ctl, false, 0u, a.spin_limit > 0 ? a.spin_limit : SPIN_MAX};
    const size_t par_bytes = (size_t)GE::PAR_SLOTS * 8;
    unsigned long long *trace = (a.trace && ct == 0) ? a.trace + (size_t)wg * (L * FUSED_TRACE_PER_LAYER + 2) : nullptr;
    auto mark = [&]() {
        if (trace) *trace++ = wall_clock64();
    };

    // the token of this step (reference embed kernel, src/hf/emitter.rs:506-537)
    const int step = a.state->step, n_forced = a.state->n_forced;
    int id = step < n_forced ? a.forced[step] : a.state->token;
    if (id < 0 || id >= a.vocab) {  // decoding goes on with id 0; the host reports it
        if (wg == 0 && ct == 0) atomicOr(a.ctl + 3, FUSED_WARN_TOKEN_RANGE);
        id = 0;
    }
    float h[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) h[j] = a.embed[(size_t)id * GE::HIDDEN + ct + CT * j];

    // this position's RoPE table entries (the same for every layer)
    RopeLane rope{0.f, 0.f, 0.f, 0.f};
    if (lane < HD / 2) {
        const float *c = a.cos_tab + (size_t)pos * HD, *sn = a.sin_tab + (size_t)pos * HD;
        rope = RopeLane{c[lane], c[lane + HD / 2], sn[lane], sn[lane + HD / 2]};
    }

    // ── placement check: workgroups are dealt to the dies round-robin, starting wherever the previous
    //    launch stopped, so wg % 8 names a die up to a rotation. Every workgroup reports the die it runs
    //    on, every communicating wavefront reads all reports and reaches the same verdict: die-local
    //    traffic is used only if all workgroups with the same wg % 8 sit on one die. ──
    const int xcd = wg % GE::NXCD, rank = wg / GE::NXCD;
    bool die_ok;
    {
        unsigned char *chk = a.xch + (size_t)GE::CHK0 * 8;
        if (ct == 0) st_slot(chk, wg, (float)xcc_id(), launches + 1u, false);
        int unit[2] = {lane, lane + WAVE};
        bool on[2] = {lane < GE::NWG / 2, lane + WAVE < GE::NWG / 2};
        u32x4 w[2];
        poll_units<2>(ps, chk, unit, on, launches + 1u, w);
        float ref[GE::NXCD];  // the dies of workgroups 0..7
#pragma unroll
        for (int j = 0; j < GE::NXCD; j++)
            ref[j] = __shfl(__uint_as_float((j & 1) ? w[0].z : w[0].x), j / 2);
        bool mine = true;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int j0 = (2 * unit[u]) % GE::NXCD;  // even, so the unit's two reports are j0 and j0 + 1
            float r0 = 0.f, r1 = 0.f;
#pragma unroll
            for (int j = 0; j < GE::NXCD; j += 2) {
                r0 = j == j0 ? ref[j] : r0;
                r1 = j == j0 ? ref[j + 1] : r1;
            }
            if (on[u]) mine = mine && __uint_as_float(w[u].x) == r0 && __uint_as_float(w[u].z) == r1;
        }
        die_ok = __all(mine) && !__any(ps.failed) && !a.far_only;
        if (!die_ok && wg == 0 && ct == 0) atomicAdd(a.ctl + 2, 1u);  // steps that ran without die-local traffic
    }
    const bool near_g = die_ok && GE::GROUP_ON_XCD;  // a KV head's workgroups talk through their die's L2

    // The hidden increments reach the exchange area as KVH partial vectors (one per KV-head group, each a K
    // slice of the O or down projection). They are fetched from memory once per die: one wavefront of each
    // of the die's workgroups waits for its share of the units of all KVH vectors, adds them in group order
    // and writes the sums to the die's relay area, which all of the die's workgroups then read through
    // the L2. Without die-local placement the relay's stores go through to memory.
    auto relay_sum = [&](unsigned char *par, int off, uint32_t tag) -> const unsigned char * {
        unsigned char *rel = par + (size_t)(GE::RELAY0 + xcd * GE::RELAY_SLOTS + (off == GE::XH ? 0 : GE::HIDDEN)) * 8;
        {
            // All four wavefronts poll for the same share, a quarter of a round trip apart (whichever sees it
            // complete first publishes the sums; the others publish the same values again): a share is noticed sooner.
            if (cwv == 1) __builtin_amdgcn_s_sleep(4);
            if (cwv == 2) __builtin_amdgcn_s_sleep(8);
            if (cwv == 3) __builtin_amdgcn_s_sleep(12);
            constexpr int per = GE::HIDDEN / 2 / GE::NPX;
            int unit[GE::KVH];
            bool on[GE::KVH];
            u32x4 w[GE::KVH];
#pragma unroll
            for (int d = 0; d < GE::KVH; d++) {
                unit[d] = (off + d * GE::HIDDEN) / 2 + rank * per + lane;
                on[d] = lane < per;
            }
            poll_units<GE::KVH>(ps, par, unit, on, tag, w);
            if (lane < per) {
                float v0 = __uint_as_float(w[0].x), v1 = __uint_as_float(w[0].z);
#pragma unroll
                for (int d = 1; d < GE::KVH; d++) {
                    v0 += __uint_as_float(w[d].x);
                    v1 += __uint_as_float(w[d].z);
                }
                st_slot(rel, 2 * (rank * per + lane), v0, tag, die_ok);
                st_slot(rel, 2 * (rank * per + lane) + 1, v1, tag, die_ok);
            }
        }
        return rel;
    };
    // hidden <- hidden + (the sum of the partial vectors at slot offset `off`), then stage hidden, the norm
    // weights and this wavefront's share of the sum of squares
    auto stage_hidden = [&](unsigned char *par, int off, uint32_t tag, bool add, const float (&nwv)[NJ]) {
        if (add) {
            const unsigned char *src = relay_sum(par, off, tag);
            int unit[NJ / 2];
            bool on[NJ / 2];
            u32x4 w[NJ / 2];
#pragma unroll
            for (int u = 0; u < NJ / 2; u++) {
                unit[u] = u * CT + ct;
                on[u] = true;
            }
            poll_units<NJ / 2>(ps, src, unit, on, tag, w);
#pragma unroll
            for (int u = 0; u < NJ / 2; u++) {
                h[2 * u] = h[2 * u] + __uint_as_float(w[u].x);
                h[2 * u + 1] = h[2 * u + 1] + __uint_as_float(w[u].z);
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; j++) ss += h[j] * h[j];
        ss = wave_sum(ss);
        if (lane == 0) sm.red[cwv] = ss;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            sm.hx[XLay<WF>::pos(ct + CT * j, GE::HIDDEN)] = h[j];
            sm.nw[XLay<WF>::pos(ct + CT * j, GE::HIDDEN)] = nwv[j];
        }
    };
    // copy a vector of this KV head's group (n_units 16-byte units in plain slot order) into LDS
    auto stage_group = [&](const unsigned char *src, int n_units, uint32_t tag, float *dst) {
        int unit[1] = {ct};
        bool on[1] = {ct < n_units};
        u32x4 w[1];
        poll_units<1>(ps, src, unit, on, tag, w);
        if (on[0]) {
            dst[XLay<WF>::pos(2 * ct, 2 * n_units)] = __uint_as_float(w[0].x);
            dst[XLay<WF>::pos(2 * ct + 1, 2 * n_units)] = __uint_as_float(w[0].z);
        }
    };

    // The small per-layer parameters (norm weights, bias) are requested one layer before their use, right
    // after the barrier that ends the use of the previous layer's: a load that misses the die's L2 would
    // otherwise sit in front of the polls of the exchange that follows it (loads return in issue order).
    float nw_in[NJ], nw_post[NJ], bias_v = 0.f;
    float qn_lo = 1.f, qn_hi = 1.f, kn_lo = 1.f, kn_hi = 1.f;
    auto load_in_ln = [&](const FusedLayerPtrs &p) {
#pragma unroll
        for (int j = 0; j < NJ; j++) nw_in[j] = ldf_global(p.in_ln + ct + CT * j);
        if (p.qkv_bias && ct < GE::RQ) bias_v = ldf_global(p.qkv_bias + GE::qkv_row(sp.kh, sp.split * GE::RQ + ct));
    };
    auto load_post_ln = [&](const FusedLayerPtrs &p) {
#pragma unroll
        for (int j = 0; j < NJ; j++) nw_post[j] = ldf_global(p.post_ln + ct + CT * j);
    };
    auto load_qk_norm = [&](const FusedLayerPtrs &p) {
        if (p.q_norm != nullptr && lane < HD / 2) {
            qn_lo = ldf_global(p.q_norm + lane);
            qn_hi = ldf_global(p.q_norm + lane + HD / 2);
            kn_lo = ldf_global(p.k_norm + lane);
            kn_hi = ldf_global(p.k_norm + lane + HD / 2);
        }
    };
    load_in_ln(sm.lp[0]);
    load_post_ln(sm.lp[0]);
    load_qk_norm(sm.lp[0]);
    float nw_head[NJ];  // the final norm's weights, for the LM head
#pragma unroll
    for (int j = 0; j < NJ; j++) nw_head[j] = a.head_w ? ldf_global(a.head_norm + ct + CT * j) : 0.f;

    for (int l = 0; l < L; l++) {
        const FusedLayerPtrs cur = sm.lp[l];
        const FusedLayerPtrs nxt = sm.lp[l + 1 < L ? l + 1 : l];
        const bool qk_normed = cur.q_norm != nullptr;
        const uint32_t gl = base + (uint32_t)l;  // layers run since the exchange area was zeroed
        const uint32_t tag = gl + 1u;
        unsigned char *xc = a.xch + (size_t)(gl & 1u) * par_bytes;
        unsigned char *xprev = a.xch + (size_t)((gl & 1u) ^ 1u) * par_bytes;
        unsigned char *lq = xc + (size_t)(GE::LQ0 + sp.kh * GE::GROWS) * 8;             // this KV head's raw rows
        unsigned char *lp = xc + (size_t)(GE::LP0 + sp.kh * GE::SPH * GE::PART) * 8;    // its splits' partials,
        unsigned char *la = xc + (size_t)(GE::LA0 + sp.kh * GE::KSO) * 8;               // its folded attention outputs
        unsigned char *lc = xc + (size_t)(GE::LC0 + sp.kh * GE::KSD) * 8;               // and its group's SiLU*up values

        // ── into the Q|K|V phase: hidden += down rows of the previous layer ──
        ps.where = 1u | (uint32_t)l << 4 | (uint32_t)wg << 12;
        stage_hidden(xprev, GE::XH, tag - 1u, l > 0, nw_in);
        if (cur.qkv_bias && ct < GE::RQ) sm.bias[ct] = bias_v;
        wg_barrier();
        load_in_ln(nxt);
        mark();
        wg_barrier();
        mark();
        // (a.withhold_wg: a test's way to make every wait for this workgroup's rows run into its bound)
        if (ct < GE::RQ && !(l == 0 && wg == a.withhold_wg)) st_slot(lq, sp.split * GE::RQ + ct, sm.pub[ct], tag, near_g);

        // ── into attention: this KV head's raw q rows (and k, v for the split that holds the new row),
        //    QK-norm + RoPE, cache append (reference src/hf/emitter.rs:629-649, src/runtime.rs:521-568) ──
        ps.where = 2u | (uint32_t)l << 4 | (uint32_t)wg << 12;
        if (sp.split < sp.nsl) {
            for (int t = cwv; t < G + 2; t += 4) {
                if (t >= G && !sp.owner) continue;
                int unit[1] = {t * HD / 2 + lane};
                bool on[1] = {lane < HD / 2};
                u32x4 w[1];
                poll_units<1>(ps, lq, unit, on, tag, w);
                if (on[0]) {
                    sm.rowbuf[t][2 * lane] = __uint_as_float(w[0].x);
                    sm.rowbuf[t][2 * lane + 1] = __uint_as_float(w[0].z);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                constexpr int HALF = HD / 2;
                const size_t row_off = ((size_t)sp.kh * a.max_len + pos) * HD;
                if (t < G) {
                    float lo, hi;
                    norm_rope<HD>(sm.rowbuf[t], qk_normed, qn_lo, qn_hi, rope, a.eps, lane, lo, hi);
                    if (lane < HALF) {
                        sm.qs[t][lane] = lo;
                        sm.qs[t][lane + HALF] = hi;
                    }
                } else if (t == G) {
                    float lo, hi;
                    norm_rope<HD>(sm.rowbuf[t], qk_normed, kn_lo, kn_hi, rope, a.eps, lane, lo, hi);
                    if (lane < HALF) {  // rounded to bf16 once; cache and this step use the same values
                        uint16_t *dst = cur.kcache + row_off;
                        const uint16_t r_lo = f32_to_bf16_rne_dev(lo), r_hi = f32_to_bf16_rne_dev(hi);
                        dst[lane] = r_lo;
                        dst[lane + HALF] = r_hi;
                        sm.knew[lane] = __uint_as_float((uint32_t)r_lo << 16);
                        sm.knew[lane + HALF] = __uint_as_float((uint32_t)r_hi << 16);
                    }
                } else {
                    uint16_t *dst = cur.vcache + row_off;
                    for (int i = lane; i < HD; i += WAVE) {
                        const uint16_t r = f32_to_bf16_rne_dev(sm.rowbuf[t][i]);
                        dst[i] = r;
                        sm.vnew[i] = __uint_as_float((uint32_t)r << 16);
                    }
                }
            }
        }
        wg_barrier();
        load_qk_norm(nxt);
        mark();
        wg_barrier();
        mark();
        if (sp.split < sp.nsl) {
            // merge the compute wavefronts' partials (one output per thread) and publish the split's
            // (o, max, sum): o = sum_w exp(m_w - M) * (sum over w's row groups), in wavefront order. The
            // threads of a head's first two outputs also publish the head's (max, sum): same weights.
            for (int i = ct; i < G * HD; i += CT) {
                const int g = i / HD, d = i % HD;
                float mw[NCW], f[NCW], M = -INFINITY;
#pragma unroll
                for (int w = 0; w < NCW; w++) {
                    mw[w] = sm.wstat[w][g][0];
                    M = fmaxf(M, mw[w]);
                }
                float v = 0.f;
#pragma unroll
                for (int w = 0; w < NCW; w++) {
                    f[w] = mw[w] == -INFINITY ? 0.f : __expf(mw[w] - M);
                    float t = 0.f;
#pragma unroll
                    for (int sb = 0; sb < GE::RPI; sb++) t += sm.part[w * GE::RPI + sb][g][d];
                    v += f[w] * t;
                }
                st_slot(lp, sp.split * GE::PART + i, v, tag, near_g);
                if (d < 2) {
                    float st = M;
                    if (d == 1) {
                        st = 0.f;
#pragma unroll
                        for (int w = 0; w < NCW; w++) st += f[w] * sm.wstat[w][g][1];
                    }
                    st_slot(lp, sp.split * GE::PART + G * HD + 2 * g + d, st, tag, near_g);
                }
            }
        }

        // ── fold the splits of this KV head for FPW of its outputs (one wavefront) ──
        ps.where = 3u | (uint32_t)l << 4 | (uint32_t)wg << 12;
        constexpr bool FOLD_HALVES = GE::SPH <= 32 && (GE::FPW / 2) % 2 == 0;
        if (cwv == 0 && FOLD_HALVES) {
            // lanes 0-31 fold the first half of the workgroup's outputs over the (at most 32) splits, lanes 32-63
            // the second half: half the loads and half the sums a lane, and a sum ends inside 32 lanes
            constexpr int HU = GE::FPW / 4;  // 16-byte units of outputs per lane
            const int o0 = sp.split * GE::FPW;
            const int t = o0 / HD, d0 = o0 % HD;
            const int half = lane >> 5, sl = lane & 31;
            const int pbase = sl * GE::PART;
            int unit[HU + 1];
            bool on[HU + 1];
            u32x4 w[HU + 1];
#pragma unroll
            for (int u = 0; u < HU; u++) {
                unit[u] = (pbase + t * HD + d0) / 2 + half * HU + u;
                on[u] = sl < sp.nsl;
            }
            unit[HU] = (pbase + G * HD + 2 * t) / 2;
            on[HU] = sl < sp.nsl;
            poll_units<HU + 1>(ps, lp, unit, on, tag, w);
            const float m_s = on[HU] ? __uint_as_float(w[HU].x) : -INFINITY;
            const float l_s = on[HU] ? __uint_as_float(w[HU].z) : 0.f;
            const float m = wave_max(m_s);  // both halves hold the same maxima
            const float f = on[HU] ? __expf(m_s - m) : 0.f;
            float red[2 * HU + 1];  // the sum of the splits' sums, then this half's weighted outputs
            red[0] = f * l_s;
#pragma unroll
            for (int u = 0; u < HU; u++) {
                red[1 + 2 * u] = f * __uint_as_float(w[u].x);
                red[2 + 2 * u] = f * __uint_as_float(w[u].z);
            }
#pragma unroll
            for (int i = 0; i < 2 * HU + 1; i++) red[i] += dpp_move<0xB1, 0xF>(red[i], 0.f);
#pragma unroll
            for (int i = 0; i < 2 * HU + 1; i++) red[i] += dpp_move<0x4E, 0xF>(red[i], 0.f);
#pragma unroll
            for (int i = 0; i < 2 * HU + 1; i++) red[i] += dpp_move<0x141, 0xF>(red[i], 0.f);
#pragma unroll
            for (int i = 0; i < 2 * HU + 1; i++) red[i] += dpp_move<0x140, 0xF>(red[i], 0.f);
#pragma unroll
            for (int i = 0; i < 2 * HU + 1; i++) red[i] += dpp_move<0x142, 0xA>(red[i], 0.f);  // lanes 31 and 63: the halves' totals
            const int e = lane % (2 * HU);  // lane l < FPW publishes output l: half l / (2 HU), element l % (2 HU)
            float num = 0.f, den = 0.f;
#pragma unroll
            for (int hh = 0; hh < 2; hh++) {
                const float d0v = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(red[0]), 31 + 32 * hh));
#pragma unroll
                for (int k = 0; k < 2 * HU; k++) {
                    const float nv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(red[1 + k]), 31 + 32 * hh));
                    if (lane / (2 * HU) == hh && e == k) {
                        num = nv;
                        den = d0v;
                    }
                }
            }
            if (lane < GE::FPW) st_slot(la, o0 + lane, num * __builtin_amdgcn_rcpf(den), tag, near_g);
        } else if (cwv == 0) {
            constexpr int FU = GE::FPW / 2;
            const int o0 = sp.split * GE::FPW;  // first output, counted inside the KV head's G * HD
            const int t = o0 / HD, d0 = o0 % HD;
            const int pbase = lane * GE::PART;
            int unit[FU + 1];
            bool on[FU + 1];
            u32x4 w[FU + 1];
#pragma unroll
            for (int u = 0; u < FU; u++) {
                unit[u] = (pbase + t * HD + d0) / 2 + u;
                on[u] = lane < sp.nsl;
            }
            unit[FU] = (pbase + G * HD + 2 * t) / 2;
            on[FU] = lane < sp.nsl;
            poll_units<FU + 1>(ps, lp, unit, on, tag, w);
            const float m_s = on[FU] ? __uint_as_float(w[FU].x) : -INFINITY;
            const float l_s = on[FU] ? __uint_as_float(w[FU].z) : 0.f;
            const float m = wave_max(m_s);
            const float f = on[FU] ? __expf(m_s - m) : 0.f;
            float red[2 * FU + 1];  // the sum of the splits' sums, then the FPW weighted outputs
            red[0] = f * l_s;
#pragma unroll
            for (int u = 0; u < FU; u++) {
                red[1 + 2 * u] = f * __uint_as_float(w[u].x);
                red[2 + 2 * u] = f * __uint_as_float(w[u].z);
            }
            wave_sum_n<2 * FU + 1>(red);
            float mine = 0.f;
#pragma unroll
            for (int e = 0; e < GE::FPW; e++) mine = lane == e ? red[1 + e] : mine;
            if (lane < GE::FPW) st_slot(la, o0 + lane, mine * __builtin_amdgcn_rcpf(red[0]), tag, near_g);
        }
        mark();

        // ── into the O phase ──
        ps.where = 4u | (uint32_t)l << 4 | (uint32_t)wg << 12;
        stage_group(la, GE::KSO / 2, tag, sm.attn);
        wg_barrier();
        mark();
        wg_barrier();
        mark();
        if (ct < GE::RPG) st_slot(xc, GE::XO + sp.kh * GE::HIDDEN + hidden_slot(GE::partial_row(sp.split, ct)), sm.pub[ct], tag, false);

        // ── into the gate|up phase: hidden += O rows (reference src/hf/emitter.rs:787) ──
        ps.where = 5u | (uint32_t)l << 4 | (uint32_t)wg << 12;
        stage_hidden(xc, GE::XO, tag, true, nw_post);
        wg_barrier();
        load_post_ln(nxt);
        mark();
        wg_barrier();
        mark();
        if (ct < GE::APW) st_slot(lc, sp.split * GE::APW + ct, sm.pub[ct], tag, near_g);
        // K8 with K slices of down that share a 256-wide block with the neighbouring group: the Q8_K scale of such
        // a block needs the largest magnitude on both sides. Every workgroup writes the maxima of its own values
        // in the block its group's slice starts in and in the block it ends in through to memory ...
        constexpr bool SHARED_BLOCKS = WF == FUSED_WF_K8 && GE::KSD % 256 != 0;
        unsigned char *lm = xc + (size_t)GE::LM0 * 8;
        if (SHARED_BLOCKS && cwv == 1) {  // (wavefront 0 is busy publishing the values themselves)
            static_assert(GE::APW <= WAVE, "one wavefront holds a workgroup's SiLU*up values");
            const int k0 = sp.kh * GE::KSD, k = k0 + sp.split * GE::APW + lane;  // column of this lane's value
            const float mag = lane < GE::APW ? fabsf(sm.pub[lane]) : 0.f;
            const bool first = lane < GE::APW && k / 256 * 256 < k0, last = lane < GE::APW && k / 256 * 256 + 256 > k0 + GE::KSD;
            const float m_first = wave_max(first ? mag : 0.f), m_last = wave_max(last ? mag : 0.f);
            if (lane == 0) {
                st_slot(lm, 2 * wg, m_first, tag, false);
                st_slot(lm, 2 * wg + 1, m_last, tag, false);
            }
        }

        // ── into the down phase ──
        ps.where = 6u | (uint32_t)l << 4 | (uint32_t)wg << 12;
        stage_group(lc, GE::KSD / 2, tag, sm.act);
        // (behind the staging, not beside it: a CU returns its loads in issue order, and a poll of this CU's L2
        // issued behind a poll that goes to memory would wait for it)
        if (SHARED_BLOCKS && cwv == 0) {
            // ... and reads the group before's maxima of its last block (lanes 0-31) and the group after's of its
            // first block (lanes 32-63): the workgroups of KV head kh are wg = kh + KVH * split
            static_assert(GE::SPH <= 32, "a neighbouring group's workgroups fit half a wavefront");
            const int k0 = sp.kh * GE::KSD;
            const bool after = lane >= 32;
            const int nb = sp.kh + (after ? 1 : -1), i = lane & 31;
            const bool want = i < GE::SPH && (after ? (k0 + GE::KSD) % 256 != 0 && nb < GE::KVH : k0 % 256 != 0 && nb >= 0);
            int unit[1] = {want ? nb + GE::KVH * i : 0};
            bool on[1] = {want};
            u32x4 w[1];
            poll_units<1>(ps, lm, unit, on, tag, w);
            const float m = want ? __uint_as_float(after ? w[0].x : w[0].z) : 0.f;
            const float m_before = wave_max(after ? 0.f : m), m_after = wave_max(after ? m : 0.f);
            if (lane == 0) {
                sm.nbmax[0] = m_before;
                sm.nbmax[1] = m_after;
            }
        }
        wg_barrier();
        mark();
        wg_barrier();
        mark();
        if (ct < GE::RPG) st_slot(xc, GE::XH + sp.kh * GE::HIDDEN + hidden_slot(GE::partial_row(sp.split, ct)), sm.pub[ct], tag, false);
    }

    if (a.head_w) {
        // ── into the LM head: hidden += down rows of the last layer, under the final RMSNorm ──
        const uint32_t gl = base + (uint32_t)(L - 1);
        unsigned char *xl = a.xch + (size_t)(gl & 1u) * par_bytes;
        ps.where = 7u | (uint32_t)(L - 1) << 4 | (uint32_t)wg << 12;
        stage_hidden(xl, GE::XH, gl + 1u, true, nw_head);
        if (wg == 0) {
#pragma unroll
            for (int j = 0; j < NJ; j++) a.hidden_out[ct + CT * j] = h[j];
        }
        wg_barrier();
        head_rows<GE, WF, false>(a, sm, wg, NCW + cwv, lane);
        // this workgroup's best row, then (workgroup 0) the best of all and the end of the step
        // (greedy pick of reference src/generate.rs:735-742 taken on the device)
        unsigned char *cand = a.xch + (size_t)GE::CAND0 * 8;
        const uint32_t ctag = launches + 1u;
        if (cwv == 0) {
            float bv = -INFINITY;
            int bi = -1;
            if (lane < HEAD_WORKERS) {
                bv = sm.head_v[lane];
                bi = sm.head_i[lane];
            }
            const float m = wave_max(bi >= 0 ? bv : -INFINITY);
            const float sel = wave_max(bi >= 0 && bv == m ? (float)bi : -1.f);  // indices are below 2^24: exact as floats
            if (lane == 0) {
                st_slot(cand, 2 * wg, m, ctag, false);
                st_slot(cand, 2 * wg + 1, __int_as_float((int)sel), ctag, false);
            }
            if (wg == 0) {
                constexpr int NU = GE::NWG / WAVE;
                int unit[NU];
                bool on[NU];
                u32x4 w[NU];
#pragma unroll
                for (int u = 0; u < NU; u++) {
                    unit[u] = u * WAVE + lane;
                    on[u] = true;
                }
                poll_units<NU>(ps, cand, unit, on, ctag, w);
                float gv = -INFINITY;
                int gi = -1;
#pragma unroll
                for (int u = 0; u < NU; u++) {
                    const float v = __uint_as_float(w[u].x);
                    const int i = (int)w[u].z;
                    if (i >= 0 && (gi < 0 || v > gv || (v == gv && i > gi))) {
                        gv = v;
                        gi = i;
                    }
                }
                const float gm = wave_max(gi >= 0 ? gv : -INFINITY);
                const float gs = wave_max(gi >= 0 && gv == gm ? (float)gi : -1.f);
                if (lane == 0 && gs < 0.f) atomicOr(a.ctl + 3, FUSED_WARN_NO_FINITE_LOGIT);
                const bool gave_up = ps.failed || __hip_atomic_load(a.ctl + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
                if (lane == 0 && a.advance && !gave_up) {
                    const int tok = gs < 0.f ? 0 : (int)gs;
                    if (step < a.out_cap) a.out_tokens[step] = tok;
                    a.state_rw->token = tok;
                    a.state_rw->step = step + 1;
                    a.state_rw->pos = pos + 1;
                }
                // every workgroup read the launch count before its first exchange
                if (lane == 0) __hip_atomic_store(a.ctl, launches + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    } else if (wg == 0) {
        // hidden += down rows of the last layer (the groups' partial vectors, added in group order as the
        // relays do): the LM head's input
        const uint32_t gl = base + (uint32_t)(L - 1);
        const unsigned char *xl = a.xch + (size_t)(gl & 1u) * par_bytes;
        float inc[NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++) inc[j] = 0.f;
        for (int d = 0; d < GE::KVH; d++) {
            int unit[NJ / 2];
            bool on[NJ / 2];
            u32x4 w[NJ / 2];
#pragma unroll
            for (int u = 0; u < NJ / 2; u++) {
                unit[u] = (GE::XH + d * GE::HIDDEN) / 2 + u * CT + ct;
                on[u] = true;
            }
            poll_units<NJ / 2>(ps, xl, unit, on, gl + 1u, w);
#pragma unroll
            for (int u = 0; u < NJ / 2; u++) {
                inc[2 * u] = d == 0 ? __uint_as_float(w[u].x) : inc[2 * u] + __uint_as_float(w[u].x);
                inc[2 * u + 1] = d == 0 ? __uint_as_float(w[u].z) : inc[2 * u + 1] + __uint_as_float(w[u].z);
            }
        }
#pragma unroll
        for (int j = 0; j < NJ; j++) a.hidden_out[ct + CT * j] = h[j] + inc[j];
        // Every workgroup read the launch count before its first exchange, and this point is only reached
        // after all of them have published their last rows.
        if (ct == 0) __hip_atomic_store(a.ctl, launches + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    mark();
    if (trace) *trace++ = die_ok ? 1ull : 0ull;
}

template <class GE, int WF>
__global__ __launch_bounds__(FT) void decode_fused_kernel(FusedDecodeArgs a) {
    __shared__ Lds<GE> sm;
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int wg = blockIdx.x;
    const int pos = a.state->pos;
    // The attention phase keeps a split's rows in registers: more live rows than MAX_KV are not served. The
    // host takes the other path through the layers from there on; should a launch get here all the same,
    // every workgroup leaves at once (they all read the same position) and the status word says why.
    if (pos + 1 > GE::MAX_KV || pos + 1 > a.max_len) {
        if (wg == 0 && threadIdx.x == 0) atomicCAS(a.ctl + 1, 0u, 0x80000000u | 0xFu);
        return;
    }
    {
        static_assert(sizeof(FusedLayerPtrs) % 8 == 0, "the table is copied in 8-byte words");
        const uint64_t *src = reinterpret_cast<const uint64_t *>(a.layers);
        uint64_t *dst = reinterpret_cast<uint64_t *>(sm.lp);
        const int words = a.n_layers * (int)(sizeof(FusedLayerPtrs) / 8);
        for (int i = threadIdx.x; i < words; i += FT) dst[i] = src[i];
        // Only the workgroup that holds the new cache row stages it; the others multiply these by a weight of
        // zero, so they must not hold whatever an earlier kernel left in LDS (0 * NaN is NaN).
        for (int i = threadIdx.x; i < GE::HD; i += FT) {
            sm.knew[i] = 0.f;
            sm.vnew[i] = 0.f;
        }
        __syncthreads();
    }
    if (wave < NCW) {
        compute_role<GE, WF>(a, sm, wg, wave, lane, pos);
    } else {
        const uint32_t launches = __hip_atomic_load(a.ctl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        comm_role<GE, WF>(a, sm, wg, wave - NCW, lane, pos, launches);
    }
}

// Kernel instances: Qwen3-0.6B in the three weight formats, a small shape of the same family for tests
// (bf16), and a small shape whose widths are multiples of 1024 for the quantised formats.
using GeoQwen3_0p6b = Geo<1024, 16, 8, 128, 3072, 256>;
using GeoSmall = Geo<512, 4, 2, 128, 1024, 64>;
using GeoSmallQ = Geo<1024, 8, 4, 128, 1024, 64>;
// The same shapes with three row rounds: caches up to 1536 live rows, with an attention phase a fifth shorter.
using GeoQwen3_0p6bShort = Geo<1024, 16, 8, 128, 3072, 256, 3>;
using GeoSmallShort = Geo<512, 4, 2, 128, 1024, 64, 3>;
using GeoSmallQShort = Geo<1024, 8, 4, 128, 1024, 64, 3>;
// Six row rounds (3072 live rows): three attention passes instead of the four of the eight-round instances, and a
// quarter fewer cache rows to ask for (Qwen3-0.6B, bf16: 0.453 against 0.468 ms a token at 2100 rows).
using GeoQwen3_0p6bMid = Geo<1024, 16, 8, 128, 3072, 256, 6>;
using GeoSmallMid = Geo<512, 4, 2, 128, 1024, 64, 6>;
using GeoSmallQMid = Geo<1024, 8, 4, 128, 1024, 64, 6>;
// The same shapes with eight row rounds: twice the live cache rows (4096) for 32 more registers a lane and an
// attention phase twice as long; taken only by steps that the four-round instances do not serve.
using GeoQwen3_0p6bLong = Geo<1024, 16, 8, 128, 3072, 256, 8>;
using GeoSmallLong = Geo<512, 4, 2, 128, 1024, 64, 8>;
using GeoSmallQLong = Geo<1024, 8, 4, 128, 1024, 64, 8>;
// Eight row rounds held and up to 56 more streamed inside the attention phase: 32768 live rows. Every further
// 1000 rows cost the Qwen3-0.6B shape about 26 us a token; below 4096 rows these instances are 1-2 % slower than
// the ones above (per-lane offsets are recomputed in every layer instead of held), so they come last.
using GeoQwen3_0p6bStream = Geo<1024, 16, 8, 128, 3072, 256, 8, 56>;
using GeoSmallStream = Geo<512, 4, 2, 128, 1024, 64, 8, 56>;
using GeoSmallQStream = Geo<1024, 8, 4, 128, 1024, 64, 8, 56>;

template <class GE>
bool shape_is(const FusedShape &s) {
    return s.hidden == GE::HIDDEN && s.heads == GE::H && s.kv_heads == GE::KVH && s.head_dim == GE::HD &&
           s.inter == GE::INTER;
}

struct Instance {
    bool (*matches)(const FusedShape &);
    int wf, max_kv, nwg;
    size_t xch_bytes;
    const void *kernel;
};

template <class GE, int WF>
Instance instance() {
    return Instance{&shape_is<GE>, WF, GE::MAX_KV, GE::NWG, (size_t)GE::ALL_SLOTS * 8,
                    reinterpret_cast<const void *>(&decode_fused_kernel<GE, WF>)};
}

// The first instance of the shape and format that holds `live_rows` cache rows (the short ones come first); with
// live_rows = 0, the one that holds the most.
const Instance *find_instance(const FusedShape &s, int live_rows = 1) {
    static const Instance table[] = {
        instance<GeoQwen3_0p6bShort, FUSED_WF_K8>(), instance<GeoSmallQShort, FUSED_WF_K8>(),
        instance<GeoQwen3_0p6b, FUSED_WF_K8>(), instance<GeoSmallQ, FUSED_WF_K8>(),
        instance<GeoQwen3_0p6bMid, FUSED_WF_K8>(), instance<GeoSmallQMid, FUSED_WF_K8>(),
        instance<GeoQwen3_0p6bLong, FUSED_WF_K8>(), instance<GeoSmallQLong, FUSED_WF_K8>(),
        instance<GeoQwen3_0p6bStream, FUSED_WF_K8>(), instance<GeoSmallQStream, FUSED_WF_K8>(),
        instance<GeoQwen3_0p6bShort, FUSED_WF_BF16>(), instance<GeoQwen3_0p6bShort, FUSED_WF_Q8_0>(), instance<GeoQwen3_0p6bShort, FUSED_WF_Q4_0>(),
        instance<GeoSmallShort, FUSED_WF_BF16>(),      instance<GeoSmallQShort, FUSED_WF_Q8_0>(),     instance<GeoSmallQShort, FUSED_WF_Q4_0>(),
        instance<GeoQwen3_0p6b, FUSED_WF_BF16>(), instance<GeoQwen3_0p6b, FUSED_WF_Q8_0>(), instance<GeoQwen3_0p6b, FUSED_WF_Q4_0>(),
        instance<GeoSmall, FUSED_WF_BF16>(),      instance<GeoSmallQ, FUSED_WF_Q8_0>(),     instance<GeoSmallQ, FUSED_WF_Q4_0>(),
        instance<GeoQwen3_0p6bMid, FUSED_WF_BF16>(), instance<GeoQwen3_0p6bMid, FUSED_WF_Q8_0>(), instance<GeoQwen3_0p6bMid, FUSED_WF_Q4_0>(),
        instance<GeoSmallMid, FUSED_WF_BF16>(),      instance<GeoSmallQMid, FUSED_WF_Q8_0>(),     instance<GeoSmallQMid, FUSED_WF_Q4_0>(),
        instance<GeoQwen3_0p6bLong, FUSED_WF_BF16>(), instance<GeoQwen3_0p6bLong, FUSED_WF_Q8_0>(), instance<GeoQwen3_0p6bLong, FUSED_WF_Q4_0>(),
        instance<GeoSmallLong, FUSED_WF_BF16>(),      instance<GeoSmallQLong, FUSED_WF_Q8_0>(),     instance<GeoSmallQLong, FUSED_WF_Q4_0>(),
        instance<GeoQwen3_0p6bStream, FUSED_WF_BF16>(), instance<GeoQwen3_0p6bStream, FUSED_WF_Q8_0>(), instance<GeoQwen3_0p6bStream, FUSED_WF_Q4_0>(),
        instance<GeoSmallStream, FUSED_WF_BF16>(),      instance<GeoSmallQStream, FUSED_WF_Q8_0>(),     instance<GeoSmallQStream, FUSED_WF_Q4_0>(),
    };
    const Instance *most = nullptr;
    for (const Instance &i : table) {
        if (i.wf != s.wf || !i.matches(s)) continue;
        if (live_rows > 0 && i.max_kv >= live_rows) return &i;
        if (!most || i.max_kv > most->max_kv) most = &i;
    }
    return live_rows > 0 ? nullptr : most;
}

}  // namespace

int decode_fused_max_kv(const FusedShape &s) {
    const Instance *i = find_instance(s, 0);
    return i ? i->max_kv : 0;
}

int decode_fused_tier(const FusedShape &s, int live_rows) {
    const Instance *i = find_instance(s, live_rows);
    return i ? i->max_kv : 0;
}

size_t decode_fused_xch_bytes(const FusedShape &s) {
    const Instance *i = find_instance(s);
    return i ? i->xch_bytes : 0;
}

bool decode_fused_supported(const hm_ctx *ctx, const FusedShape &s, int n_layers, int max_seq_len, const char **why) {
    static const char *none = "";
    const char *dummy;
    if (!why) why = &dummy;
    *why = none;
    if (n_layers < 1 || n_layers > MAX_LAYERS) {
        *why = "layer count outside 1..64";
        return false;
    }
    const Instance *i = find_instance(s);
    if (!i) {
        *why = "no kernel instance for this shape and weight format";
        return false;
    }
    // any cache length: what is limited is the number of live rows (decode_fused_max_kv); the instances that
    // stream cache rows address a layer's cache with 32-bit element offsets
    if ((uint64_t)s.kv_heads * (uint64_t)(max_seq_len < 0 ? 0 : max_seq_len) * s.head_dim >= (1ull << 32)) {
        *why = "a layer's KV cache holds 2^32 elements or more";
        return false;
    }
    if (ctx->num_cus < i->nwg) {
        *why = "fewer compute units than resident workgroups";
        return false;
    }
    // every instance a step of this shape and format may take must fit a compute unit
    for (int rows = 1; rows > 0;) {
        const Instance *j = find_instance(s, rows);
        if (!j) break;
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, j->kernel, FT, 0) != hipSuccess || per_cu < 1) {
            (void)hipGetLastError();
            *why = "the kernel does not fit a compute unit";
            return false;
        }
        rows = j->max_kv + 1;
    }
    return true;
}

int decode_fused_launch(hm_ctx *ctx, const FusedShape &s, const FusedDecodeArgs &a, int live_rows) {
    HM_REQUIRE(ctx, a.layers && a.embed && a.state && a.forced && a.hidden_out && a.cos_tab && a.sin_tab && a.xch && a.ctl,
               "decode_fused: NULL pointer");
    const Instance *i = find_instance(s, live_rows < 1 ? 1 : live_rows);
    if (!i) return hm_set_error(ctx, HM_ERR_INVALID, "decode_fused: no kernel instance for this shape, weight format and %d live cache rows", live_rows);
    HM_REQUIRE(ctx, !a.head_w || (a.head_norm && a.logits && a.state_rw && a.out_tokens && i->wf == FUSED_WF_BF16),
               "decode_fused: the LM head needs its norm weights, a logits row, the cursor and the token list (bf16 instances only)");
    HM_REQUIRE(ctx, a.n_layers >= 1 && a.n_layers <= MAX_LAYERS && a.max_len >= 1,
               "decode_fused: %d layers / %d cache rows not served for this shape", a.n_layers, a.max_len);
    FusedDecodeArgs args = a;
    void *params[] = {&args};
    // HOMURA_WHOLE_STEP_COOP=1: a cooperative launch, which the runtime refuses when the grid cannot be resident
    // as a whole (it does not reserve the compute units against other streams either)
    static const bool coop = [] {
        const char *e = std::getenv("HOMURA_WHOLE_STEP_COOP");
        return e && std::atoi(e) != 0;
    }();
    if (coop)
        HM_HIP(ctx, hipLaunchCooperativeKernel(i->kernel, dim3(i->nwg), dim3(FT), params, 0, ctx->stream));
    else
        HM_HIP(ctx, hipLaunchKernel(i->kernel, dim3(i->nwg), dim3(FT), params, 0, ctx->stream));
    return HM_OK;
}

int decode_fused_check(hm_ctx *ctx, const uint32_t *d_ctl, bool *gave_up) {
    uint32_t h[16] = {0};
    if (gave_up) *gave_up = false;
    int rc = hm_download(ctx, h, d_ctl, sizeof(h));
    if (rc != HM_OK) return rc;
    return decode_fused_check_words(ctx, h, gave_up);
}

int decode_fused_check_words(hm_ctx *ctx, const uint32_t *h, bool *gave_up) {
    if (gave_up) *gave_up = false;
    if (h[1] != 0 && (h[1] & 15u) == 15u)
        return hm_set_error(ctx, HM_ERR_HIP, "decode_fused: launched with more live cache rows than the kernel serves (launch %u)", h[0]);
    if (h[1] != 0) {
        if (gave_up) *gave_up = true;
        return hm_set_error(ctx, HM_ERR_HIP,
                            "decode_fused: workgroup %u stopped waiting in phase %u of layer %u (launch %u): the grid's "
                            "workgroups were not all resident at once, or another whole-step model ran on this GPU",
                            (h[1] >> 12) & 0xFFFFu, h[1] & 15u, (h[1] >> 4) & 255u, h[0]);
    }
    if (h[3] & FUSED_WARN_TOKEN_RANGE)
        return hm_set_error(ctx, HM_ERR_HIP, "decode_fused: a fed-back token id lay outside the vocabulary (decoded as id 0; launch %u)", h[0]);
    if (h[3] & FUSED_WARN_NO_FINITE_LOGIT)
        return hm_set_error(ctx, HM_ERR_HIP, "decode_fused: a step's logits held no finite value (token 0 taken; launch %u)", h[0]);
    return HM_OK;
}
