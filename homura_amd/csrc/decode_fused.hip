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
//
// Six exchanges per layer: hidden -> (Q|K|V rows) -> (attention partials per cache split) ->
// (folded heads) -> (O rows) -> (SiLU*up) -> (down rows). The arithmetic and its order are those of
// gemv_bf16.hip and attention.hip (the GEMV phases bit for bit; attention splits the cache into
// NWG / kv_heads pieces instead of 64-row chunks).
//
// Every wait is a bounded spin: on a timeout the workgroup records a status word, stops waiting,
// and still walks through the remaining barriers, so the grid always drains.
#include "decode_fused.h"

#include <type_traits>

namespace {

constexpr int FT = 512;     // threads per workgroup: wavefronts 0-3 compute, 4-7 communicate
constexpr int NCW = 4;      // compute wavefronts
constexpr int CT = 256;     // communicating threads
constexpr int SPIN_MAX = 1 << 20;
constexpr int MAX_LAYERS = 64;

template <int HIDDEN_, int H_, int KVH_, int HD_, int INTER_, int NWG_>
struct Geo {
    static constexpr int HIDDEN = HIDDEN_, H = H_, KVH = KVH_, HD = HD_, INTER = INTER_, NWG = NWG_;
    static constexpr int G = H / KVH, QD = H * HD, KVD = KVH * HD, NQKV = QD + 2 * KVD;
    static constexpr int CH = HIDDEN / 512, CO = QD / 512, CD = INTER / 512;  // 512-wide chunks of a row
    static constexpr int RQ = NQKV / NWG, RQW = RQ / NCW;      // Q|K|V rows per workgroup / wavefront
    static constexpr int RO = HIDDEN / NWG, ROW = RO / NCW;    // O and down rows
    static constexpr int RG = 2 * INTER / NWG, RGW = RG / NCW; // gate|up rows (interleaved pairs)
    static constexpr int APW = INTER / NWG;                    // SiLU*up values per workgroup
    static constexpr int SPH = NWG / KVH;                      // cache splits per KV head
    static constexpr int NR = 4;                               // row rounds a wavefront keeps in registers
    static constexpr int LPR = HD / 8, RPI = WAVE / LPR;       // lanes per cache row, rows per load
    static constexpr int MAX_KV = SPH * NR * NCW * RPI;
    static constexpr int FPW = QD / NWG;                       // folded attention outputs per workgroup
    static constexpr int PART = G * HD + 2 * G;                // one split's partial: o[G][HD], (m, l)[G]
    static constexpr int NJ = HIDDEN / CT;                     // hidden elements per communicating thread
    // exchange area of one layer parity, in 8-byte slots
    static constexpr int XH = 0, XO = HIDDEN, XQ = 2 * HIDDEN, XA = XQ + NQKV, XC = XA + QD, XP = XC + INTER;
    static constexpr int PAR_SLOTS = (XP + KVH * SPH * PART + 31) / 32 * 32;
    static constexpr int PUB = (PART > RQ ? PART : RQ) > RG ? (PART > RQ ? PART : RQ) : RG;
    static_assert(HIDDEN % 512 == 0 && QD % 512 == 0 && INTER % 512 == 0, "rows are cut into 512-wide chunks");
    static_assert(NQKV % (NWG * NCW) == 0 && HIDDEN % (NWG * NCW) == 0 && (2 * INTER) % (NWG * NCW) == 0,
                  "every wavefront owns whole rows");
    static_assert(RGW % 2 == 0, "a wavefront owns whole gate|up pairs");
    static_assert(NWG % KVH == 0 && SPH <= WAVE, "one fold lane per cache split");
    static_assert(HD == 64 || HD == 128, "head_dim 64 or 128");
    static_assert(QD % NWG == 0 && FPW % 2 == 0 && HD % FPW == 0, "a workgroup folds a run inside one head");
    static_assert(RQ <= CT && RO <= CT && APW <= CT, "one publishing thread per value");
};

template <class GE>
struct Lds {
    float hx[GE::HIDDEN];                 // hidden state entering the phase's RMSNorm
    float nw[GE::HIDDEN];                 // that norm's weights
    float attn[GE::QD];                   // folded attention output
    float act[GE::INTER];                 // SiLU(gate) * up
    float rowbuf[GE::G + 2][GE::HD];      // raw q heads, k, v of this workgroup's KV head
    float qs[GE::G][GE::HD];              // after QK-norm and RoPE
    float knew[GE::HD], vnew[GE::HD];     // the new cache row, as rounded to bf16
    float part[NCW * GE::RPI][GE::G][GE::HD];
    float wstat[NCW][GE::G][2];
    float pub[GE::PUB];                   // results of the phase, read by the publishing threads
    float red[4];
    float bias[GE::RQ];
    int arrive;
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

__device__ __forceinline__ void st_slot(unsigned char *area, int slot, float v, uint32_t tag) {
    __hip_atomic_store(reinterpret_cast<uint64_t *>(area) + slot, ((uint64_t)tag << 32) | __float_as_uint(v),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct PollState {
    uint32_t *ctl;
    bool failed;
};

// Device-scope 16-byte loads of `NU` units {v0, tag, v1, tag}, all issued before one wait, repeated
// until every wanted unit carries `tag` in both halves. Units with on[u] false are not waited for.
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
        if (++spins > SPIN_MAX) {
            __hip_atomic_store(ps.ctl + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
// (i, i + hd/2).
template <int HD>
__device__ __forceinline__ void norm_rope(const float *src, const float *__restrict__ nwp,
                                          const float *__restrict__ c, const float *__restrict__ sn, float eps,
                                          int lane, float &o_lo, float &o_hi) {
    constexpr int HALF = HD / 2;
    const bool on = lane < HALF;
    float lo = on ? src[lane] : 0.f, hi = on ? src[lane + HALF] : 0.f;
    const float c_lo = on ? c[lane] : 0.f, c_hi = on ? c[lane + HALF] : 0.f;
    const float s_lo = on ? sn[lane] : 0.f, s_hi = on ? sn[lane + HALF] : 0.f;
    const float w_lo = (on && nwp) ? ldf_global(nwp + lane) : 1.f, w_hi = (on && nwp) ? ldf_global(nwp + lane + HALF) : 1.f;
    if (nwp) {
        const float ss = wave_sum(lo * lo + hi * hi);
        const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
        lo = (lo * inv) * w_lo;
        hi = (hi * inv) * w_hi;
    }
    o_lo = lo * c_lo + (-hi) * s_lo;
    o_hi = hi * c_hi + lo * s_hi;
}

// The attention split of a workgroup for a cache of kv_len rows (the new row included).
template <class GE>
struct Split {
    int kh, split, nsl, n0, cnt, cached;
    bool owner;
    __device__ Split(int wg, int pos) {
        const int kv_len = pos + 1;
        const int chunk = (kv_len + GE::SPH - 1) / GE::SPH;
        nsl = (kv_len + chunk - 1) / chunk;
        kh = wg / GE::SPH;
        split = wg % GE::SPH;
        n0 = split * chunk;
        cnt = min(kv_len, n0 + chunk) - n0;
        if (cnt < 0) cnt = 0;
        owner = split == nsl - 1;  // holds row `pos`, which is not in the cache yet
        cached = min(cnt, pos - n0);
        if (cached < 0) cached = 0;
    }
};

// Registers of one compute wavefront that hold its slice of a layer.
template <class GE>
struct Slice {
    u32x4 wq[GE::RQW][GE::CH];
    u32x4 kr[GE::NR], vr[GE::NR];
    u32x4 wo[GE::ROW][GE::CO];
    u32x4 wg[GE::RGW][GE::CH];
    u32x4 wd[GE::ROW][GE::CD];
};

template <class GE>
__device__ __forceinline__ void compute_role(const FusedDecodeArgs &a, Lds<GE> &sm, const int wg, const int cw,
                                             const int lane, const int pos) {
    const Split<GE> sp(wg, pos);
    constexpr int LPR = GE::LPR, RPI = GE::RPI, G = GE::G, HD = GE::HD, NR = GE::NR;
    const int sub = lane / LPR, dl = lane % LPR;
    const int L = a.n_layers;
    Slice<GE> s;

    auto load_wq = [&](const FusedLayerPtrs &lp) {
#pragma unroll
        for (int r = 0; r < GE::RQW; r++)
#pragma unroll
            for (int c = 0; c < GE::CH; c++)
                s.wq[r][c] = ld128_global_stream(lp.wqkv + (size_t)(wg * GE::RQ + cw * GE::RQW + r) * GE::HIDDEN + (c * WAVE + lane) * 8);
    };
    auto load_kv = [&](const FusedLayerPtrs &lp) {
#pragma unroll
        for (int i = 0; i < NR; i++) {
            const int rl = (i * NCW + cw) * RPI + sub;
            const int row = rl < sp.cached ? sp.n0 + rl : 0;  // rows outside the split re-read a valid row
            const size_t off = ((size_t)sp.kh * a.max_len + row) * HD + dl * 8;
            s.kr[i] = ld128_global_stream(lp.kcache + off);
            s.vr[i] = ld128_global_stream(lp.vcache + off);
        }
    };
    auto load_wo = [&](const FusedLayerPtrs &lp) {
#pragma unroll
        for (int r = 0; r < GE::ROW; r++)
#pragma unroll
            for (int c = 0; c < GE::CO; c++)
                s.wo[r][c] = ld128_global_stream(lp.wo + (size_t)(wg * GE::RO + cw * GE::ROW + r) * GE::QD + (c * WAVE + lane) * 8);
    };
    auto load_wg = [&](const FusedLayerPtrs &lp) {
#pragma unroll
        for (int r = 0; r < GE::RGW; r++)
#pragma unroll
            for (int c = 0; c < GE::CH; c++)
                s.wg[r][c] = ld128_global_stream(lp.wgu + (size_t)(wg * GE::RG + cw * GE::RGW + r) * GE::HIDDEN + (c * WAVE + lane) * 8);
    };
    auto load_wd = [&](const FusedLayerPtrs &lp) {
#pragma unroll
        for (int r = 0; r < GE::ROW; r++)
#pragma unroll
            for (int c = 0; c < GE::CD; c++)
                s.wd[r][c] = ld128_global_stream(lp.wd + (size_t)(wg * GE::RO + cw * GE::ROW + r) * GE::INTER + (c * WAVE + lane) * 8);
    };

    {
        const FusedLayerPtrs lp = sm.lp[0];
        load_wq(lp);
        load_kv(lp);
        load_wo(lp);
        load_wg(lp);
        load_wd(lp);
    }

    for (int l = 0; l < L; l++) {
        // The slice of the next layer replaces each phase's registers as soon as the phase is over. After
        // the last layer the first layer's slice is requested again and never used: the request keeps the
        // number of loads in flight the same in every iteration, which the wait counts rely on.
        const FusedLayerPtrs nx = sm.lp[l + 1 < L ? l + 1 : 0];
        const bool has_bias = sm.lp[l].qkv_bias != nullptr;

        // ── Q|K|V rows (RMSNorm applied on the way in; reference src/hf/emitter.rs:560-619) ──
        wg_barrier();
        {
            const float tot = ((sm.red[0] + sm.red[1]) + sm.red[2]) + sm.red[3];
            const float inv = 1.0f / sqrtf(tot / (float)GE::HIDDEN + a.eps);
            float acc[GE::RQW];
#pragma unroll
            for (int r = 0; r < GE::RQW; r++) acc[r] = 0.f;
#pragma unroll
            for (int c = 0; c < GE::CH; c++) {
                const int k = (c * WAVE + lane) * 8;
                float hv[8], wv[8], xv[8];
                lds_x8(sm.hx, k, hv);
                lds_x8(sm.nw, k, wv);
#pragma unroll
                for (int e = 0; e < 8; e++) xv[e] = (hv[e] * inv) * wv[e];
#pragma unroll
                for (int r = 0; r < GE::RQW; r++) acc[r] = dot8f(s.wq[r][c], xv, acc[r]);
            }
#pragma unroll
            for (int r = 0; r < GE::RQW; r++) {
                float v = wave_sum(acc[r]);
                if (has_bias) v = v + sm.bias[cw * GE::RQW + r];
                if (lane == 0) sm.pub[cw * GE::RQW + r] = v;
            }
            load_wq(nx);
        }
        wg_barrier();

        // ── attention over this workgroup's split of the cache (reference src/hf/emitter.rs:709-731) ──
        wg_barrier();
        if (sp.split < sp.nsl) {
            float qv[G][8];
#pragma unroll
            for (int g = 0; g < G; g++) lds_x8(sm.qs[g], dl * 8, qv[g]);
            float sc[G][NR];
            bool live[NR];
#pragma unroll
            for (int i = 0; i < NR; i++) {
                const int rl = (i * NCW + cw) * RPI + sub;
                live[i] = rl < sp.cached;
                float kf[8];
                unpack8f(s.kr[i], kf);
#pragma unroll
                for (int g = 0; g < G; g++) {
                    float p = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; e++) p = fmaf(kf[e], qv[g][e], p);
                    p = row_sum<LPR>(p);
                    sc[g][i] = live[i] ? p * a.scale : -INFINITY;
                }
            }
            const bool with_new = sp.owner && cw == 0;  // the new row rides with wavefront 0 of the last split
            float sc_new[G];
#pragma unroll
            for (int g = 0; g < G; g++) {
                float kn[8];
                lds_x8(sm.knew, dl * 8, kn);
                float p = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) p = fmaf(kn[e], qv[g][e], p);
                p = row_sum<LPR>(p);
                sc_new[g] = with_new ? p * a.scale : -INFINITY;
            }
            float acc[G][8];
#pragma unroll
            for (int g = 0; g < G; g++) {
                float m = sc_new[g];
#pragma unroll
                for (int i = 0; i < NR; i++) m = fmaxf(m, sc[g][i]);
                m = wave_max(m);
                // softmax terms against the wavefront's own maximum (max, exp, sum:
                // reference emit_softmax, src/graph_builder/emit_linalg.rs:509-528)
                float lsum = 0.f;
                float pr[NR];
#pragma unroll
                for (int i = 0; i < NR; i++) {
                    pr[i] = live[i] ? expf(sc[g][i] - m) : 0.f;
                    if (dl == 0) lsum += pr[i];
                }
                const float pn = with_new ? expf(sc_new[g] - m) : 0.f;
                if (lane == 0) lsum += pn;
                lsum = wave_sum(lsum);
                if (lane == 0) {
                    sm.wstat[cw][g][0] = m;
                    sm.wstat[cw][g][1] = lsum;
                }
#pragma unroll
                for (int e = 0; e < 8; e++) acc[g][e] = 0.f;
#pragma unroll
                for (int i = 0; i < NR; i++) {
                    float vf[8];
                    unpack8f(s.vr[i], vf);
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[g][e] = fmaf(pr[i], vf[e], acc[g][e]);
                }
                if (with_new && sub == 0) {
                    float vn[8];
                    lds_x8(sm.vnew, dl * 8, vn);
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[g][e] = fmaf(pn, vn[e], acc[g][e]);
                }
                float *dst = &sm.part[cw * RPI + sub][g][dl * 8];
                *reinterpret_cast<f32x4 *>(dst) = f32x4{acc[g][0], acc[g][1], acc[g][2], acc[g][3]};
                *reinterpret_cast<f32x4 *>(dst + 4) = f32x4{acc[g][4], acc[g][5], acc[g][6], acc[g][7]};
            }
            // the last of the four wavefronts to get here merges their partials (LDS operations of a CU
            // execute in order: a later arrival sees what the earlier ones wrote before they counted in)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            int arrived = 0;
            if (lane == 0) arrived = atomicAdd(&sm.arrive, 1);
            arrived = __builtin_amdgcn_readfirstlane(arrived);
            if (arrived == NCW - 1) {
                if (lane == 0) sm.arrive = 0;
                float f[G][NCW], mx[G], ls[G];
#pragma unroll
                for (int g = 0; g < G; g++) {
                    float m = -INFINITY;
#pragma unroll
                    for (int w = 0; w < NCW; w++) m = fmaxf(m, sm.wstat[w][g][0]);
                    float lt = 0.f;
#pragma unroll
                    for (int w = 0; w < NCW; w++) {
                        const float mw = sm.wstat[w][g][0];
                        f[g][w] = mw == -INFINITY ? 0.f : expf(mw - m);
                        lt += f[g][w] * sm.wstat[w][g][1];
                    }
                    mx[g] = m;
                    ls[g] = lt;
                }
                constexpr int QUADS = G * HD / 4;
#pragma unroll
                for (int q0 = 0; q0 < QUADS; q0 += WAVE) {
                    const int q = q0 + lane;
                    if (q < QUADS) {
                        const int g = q / (HD / 4), d = (q % (HD / 4)) * 4;
                        f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int w = 0; w < NCW; w++) {
                            f32x4 t = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                            for (int sb = 0; sb < RPI; sb++) t += *reinterpret_cast<const f32x4 *>(&sm.part[w * RPI + sb][g][d]);
                            float fw = 0.f;
#pragma unroll
                            for (int gg = 0; gg < G; gg++) fw = gg == g ? f[gg][w] : fw;
                            o += fw * t;
                        }
                        *reinterpret_cast<f32x4 *>(&sm.pub[g * HD + d]) = o;
                    }
                }
#pragma unroll
                for (int g = 0; g < G; g++)
                    if (lane == g) {
                        sm.pub[G * HD + 2 * g] = mx[g];
                        sm.pub[G * HD + 2 * g + 1] = ls[g];
                    }
            }
        }
        load_kv(nx);
        wg_barrier();

        // ── O projection rows (reference src/hf/emitter.rs:738-745) ──
        wg_barrier();
        {
            float acc[GE::ROW];
#pragma unroll
            for (int r = 0; r < GE::ROW; r++) acc[r] = 0.f;
#pragma unroll
            for (int c = 0; c < GE::CO; c++) {
                float xv[8];
                lds_x8(sm.attn, (c * WAVE + lane) * 8, xv);
#pragma unroll
                for (int r = 0; r < GE::ROW; r++) acc[r] = dot8f(s.wo[r][c], xv, acc[r]);
            }
#pragma unroll
            for (int r = 0; r < GE::ROW; r++) {
                const float v = wave_sum(acc[r]);
                if (lane == 0) sm.pub[cw * GE::ROW + r] = v;
            }
            load_wo(nx);
        }
        wg_barrier();

        // ── gate|up rows, SiLU(gate) * up (reference src/hf/emitter.rs:787-799) ──
        wg_barrier();
        {
            const float tot = ((sm.red[0] + sm.red[1]) + sm.red[2]) + sm.red[3];
            const float inv = 1.0f / sqrtf(tot / (float)GE::HIDDEN + a.eps);
            float acc[GE::RGW];
#pragma unroll
            for (int r = 0; r < GE::RGW; r++) acc[r] = 0.f;
#pragma unroll
            for (int c = 0; c < GE::CH; c++) {
                const int k = (c * WAVE + lane) * 8;
                float hv[8], wv[8], xv[8];
                lds_x8(sm.hx, k, hv);
                lds_x8(sm.nw, k, wv);
#pragma unroll
                for (int e = 0; e < 8; e++) xv[e] = (hv[e] * inv) * wv[e];
#pragma unroll
                for (int r = 0; r < GE::RGW; r++) acc[r] = dot8f(s.wg[r][c], xv, acc[r]);
            }
#pragma unroll
            for (int r = 0; r < GE::RGW; r += 2) {
                const float gte = wave_sum(acc[r]), up = wave_sum(acc[r + 1]);
                if (lane == 0) sm.pub[cw * (GE::RGW / 2) + r / 2] = (gte / (1.0f + expf(-gte))) * up;
            }
            load_wg(nx);
        }
        wg_barrier();

        // ── down rows (reference src/hf/emitter.rs:801-804; the residual is added by the readers) ──
        wg_barrier();
        {
            float acc[GE::ROW];
#pragma unroll
            for (int r = 0; r < GE::ROW; r++) acc[r] = 0.f;
#pragma unroll
            for (int c = 0; c < GE::CD; c++) {
                float xv[8];
                lds_x8(sm.act, (c * WAVE + lane) * 8, xv);
#pragma unroll
                for (int r = 0; r < GE::ROW; r++) acc[r] = dot8f(s.wd[r][c], xv, acc[r]);
            }
#pragma unroll
            for (int r = 0; r < GE::ROW; r++) {
                const float v = wave_sum(acc[r]);
                if (lane == 0) sm.pub[cw * GE::ROW + r] = v;
            }
            load_wd(nx);
        }
        wg_barrier();
    }
}

// Slot of hidden element k in the XH / XO areas: the communicating thread c = k % 256 owns elements
// k = c + 256 j (the partition of the RMSNorm's sum of squares in gemv_bf16.hip), so its elements
// 2u and 2u + 1 share 16-byte unit u * 256 + c.
__device__ __forceinline__ int hidden_slot(int k) {
    const int j = k / CT, c = k % CT;
    return 2 * ((j / 2) * CT + c) + (j & 1);
}

template <class GE>
__device__ __forceinline__ void comm_role(const FusedDecodeArgs &a, Lds<GE> &sm, const int wg, const int cwv,
                                          const int lane, const int pos, const uint32_t base) {
    constexpr int G = GE::G, HD = GE::HD, NJ = GE::NJ;
    const Split<GE> sp(wg, pos);
    const int ct = cwv * WAVE + lane;
    const int L = a.n_layers;
    PollState ps{a.ctl, false};
    const size_t par_bytes = (size_t)GE::PAR_SLOTS * 8;

    // the token of this step (reference embed kernel, src/hf/emitter.rs:506-537)
    const int step = a.state->step, n_forced = a.state->n_forced;
    int id = step < n_forced ? a.forced[step] : a.state->token;
    if (id < 0 || id >= a.vocab) id = 0;
    float h[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) h[j] = a.embed[(size_t)id * GE::HIDDEN + ct + CT * j];

    // hidden <- hidden + (the vector published in `area` at slot offset `off`), then stage hidden, the
    // norm weights and this wavefront's share of the sum of squares
    auto stage_hidden = [&](const unsigned char *area, int off, uint32_t tag, bool add, const float *norm_w) {
        float nwv[NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++) nwv[j] = ldf_global(norm_w + ct + CT * j);
        if (add) {
            int unit[NJ / 2];
            bool on[NJ / 2];
            u32x4 w[NJ / 2];
#pragma unroll
            for (int u = 0; u < NJ / 2; u++) {
                unit[u] = off / 2 + u * CT + ct;
                on[u] = true;
            }
            poll_units<NJ / 2>(ps, area, unit, on, tag, w);
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
            sm.hx[ct + CT * j] = h[j];
            sm.nw[ct + CT * j] = nwv[j];
        }
    };
    // copy a published vector of n values (plain slot order) into LDS
    auto stage_vector = [&](const unsigned char *area, int off, uint32_t tag, float *dst, auto nu_tag) {
        constexpr int NU = decltype(nu_tag)::value;
        int unit[NU];
        bool on[NU];
        u32x4 w[NU];
#pragma unroll
        for (int u = 0; u < NU; u++) {
            unit[u] = off / 2 + u * CT + ct;
            on[u] = true;
        }
        poll_units<NU>(ps, area, unit, on, tag, w);
#pragma unroll
        for (int u = 0; u < NU; u++) {
            dst[2 * (u * CT + ct)] = __uint_as_float(w[u].x);
            dst[2 * (u * CT + ct) + 1] = __uint_as_float(w[u].z);
        }
    };

    for (int l = 0; l < L; l++) {
        const FusedLayerPtrs cur = sm.lp[l];
        const uint32_t gl = base + (uint32_t)l;  // layers run since the exchange area was zeroed
        const uint32_t tag = gl + 1u;
        unsigned char *xc = a.xch + (size_t)(gl & 1u) * par_bytes;
        const unsigned char *xprev = a.xch + (size_t)((gl & 1u) ^ 1u) * par_bytes;

        // ── into the Q|K|V phase: hidden += down rows of the previous layer ──
        stage_hidden(xprev, GE::XH, tag - 1u, l > 0, cur.in_ln);
        if (cur.qkv_bias && ct < GE::RQ) sm.bias[ct] = ldf_global(cur.qkv_bias + wg * GE::RQ + ct);
        wg_barrier();
        wg_barrier();
        if (ct < GE::RQ) st_slot(xc, GE::XQ + wg * GE::RQ + ct, sm.pub[ct], tag);

        // ── into attention: this KV head's raw q rows (and k, v for the split that holds the new row),
        //    QK-norm + RoPE, cache append (reference src/hf/emitter.rs:629-649, src/runtime.rs:521-568) ──
        if (sp.split < sp.nsl) {
            const float *c = a.cos_tab + (size_t)pos * HD;
            const float *sn = a.sin_tab + (size_t)pos * HD;
            for (int t = cwv; t < G + 2; t += 4) {
                if (t >= G && !sp.owner) continue;
                const int first = t < G ? (sp.kh * G + t) * HD : (t == G ? GE::QD : GE::QD + GE::KVD) + sp.kh * HD;
                int unit[1] = {(GE::XQ + first) / 2 + lane};
                bool on[1] = {lane < HD / 2};
                u32x4 w[1];
                poll_units<1>(ps, xc, unit, on, tag, w);
                if (on[0]) {
                    sm.rowbuf[t][2 * lane] = __uint_as_float(w[0].x);
                    sm.rowbuf[t][2 * lane + 1] = __uint_as_float(w[0].z);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                constexpr int HALF = HD / 2;
                const size_t row_off = ((size_t)sp.kh * a.max_len + pos) * HD;
                if (t < G) {
                    float lo, hi;
                    norm_rope<HD>(sm.rowbuf[t], cur.q_norm, c, sn, a.eps, lane, lo, hi);
                    if (lane < HALF) {
                        sm.qs[t][lane] = lo;
                        sm.qs[t][lane + HALF] = hi;
                    }
                } else if (t == G) {
                    float lo, hi;
                    norm_rope<HD>(sm.rowbuf[t], cur.k_norm, c, sn, a.eps, lane, lo, hi);
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
        wg_barrier();
        if (sp.split < sp.nsl)
            for (int i = ct; i < GE::PART; i += CT)
                st_slot(xc, GE::XP + (sp.kh * GE::SPH + sp.split) * GE::PART + i, sm.pub[i], tag);

        // ── fold the splits of one head for this workgroup's FPW outputs (one wavefront) ──
        if (cwv == 0) {
            constexpr int FU = GE::FPW / 2;
            const int hh = (wg * GE::FPW) / HD, d0 = (wg * GE::FPW) % HD;
            const int kh2 = hh / G, gg = hh % G;
            const int pbase = GE::XP + (kh2 * GE::SPH + lane) * GE::PART;
            int unit[FU + 1];
            bool on[FU + 1];
            u32x4 w[FU + 1];
#pragma unroll
            for (int u = 0; u < FU; u++) {
                unit[u] = (pbase + gg * HD + d0) / 2 + u;
                on[u] = lane < sp.nsl;
            }
            unit[FU] = (pbase + G * HD + 2 * gg) / 2;
            on[FU] = lane < sp.nsl;
            poll_units<FU + 1>(ps, xc, unit, on, tag, w);
            const float m_s = on[FU] ? __uint_as_float(w[FU].x) : -INFINITY;
            const float l_s = on[FU] ? __uint_as_float(w[FU].z) : 0.f;
            const float m = wave_max(m_s);
            const float f = on[FU] ? expf(m_s - m) : 0.f;
            const float lt = wave_sum(f * l_s);
            float mine = 0.f;
#pragma unroll
            for (int u = 0; u < FU; u++) {
                const float o0 = wave_sum(f * __uint_as_float(w[u].x)) / lt;
                const float o1 = wave_sum(f * __uint_as_float(w[u].z)) / lt;
                if (lane == 2 * u) mine = o0;
                if (lane == 2 * u + 1) mine = o1;
            }
            if (lane < GE::FPW) st_slot(xc, GE::XA + wg * GE::FPW + lane, mine, tag);
        }

        // ── into the O phase ──
        stage_vector(xc, GE::XA, tag, sm.attn, std::integral_constant<int, GE::QD / 2 / CT>());
        wg_barrier();
        wg_barrier();
        if (ct < GE::RO) st_slot(xc, GE::XO + hidden_slot(wg * GE::RO + ct), sm.pub[ct], tag);

        // ── into the gate|up phase: hidden += O rows (reference src/hf/emitter.rs:787) ──
        stage_hidden(xc, GE::XO, tag, true, cur.post_ln);
        wg_barrier();
        wg_barrier();
        if (ct < GE::APW) st_slot(xc, GE::XC + wg * GE::APW + ct, sm.pub[ct], tag);

        // ── into the down phase ──
        stage_vector(xc, GE::XC, tag, sm.act, std::integral_constant<int, GE::INTER / 2 / CT>());
        wg_barrier();
        wg_barrier();
        if (ct < GE::RO) st_slot(xc, GE::XH + hidden_slot(wg * GE::RO + ct), sm.pub[ct], tag);
    }

    // hidden += down rows of the last layer: the LM head's input
    if (wg == 0) {
        const uint32_t gl = base + (uint32_t)(L - 1);
        const unsigned char *xl = a.xch + (size_t)(gl & 1u) * par_bytes;
        int unit[NJ / 2];
        bool on[NJ / 2];
        u32x4 w[NJ / 2];
#pragma unroll
        for (int u = 0; u < NJ / 2; u++) {
            unit[u] = GE::XH / 2 + u * CT + ct;
            on[u] = true;
        }
        poll_units<NJ / 2>(ps, xl, unit, on, gl + 1u, w);
#pragma unroll
        for (int u = 0; u < NJ / 2; u++) {
            a.hidden_out[ct + CT * (2 * u)] = h[2 * u] + __uint_as_float(w[u].x);
            a.hidden_out[ct + CT * (2 * u + 1)] = h[2 * u + 1] + __uint_as_float(w[u].z);
        }
        // Every workgroup read the launch count before its first exchange, and this point is only reached
        // after all of them have published their last rows.
        if (ct == 0)
            __hip_atomic_store(a.ctl, base / (uint32_t)L + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <class GE>
__global__ __launch_bounds__(FT) void decode_fused_kernel(FusedDecodeArgs a) {
    __shared__ Lds<GE> sm;
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int wg = blockIdx.x;
    const int pos = a.state->pos;
    {
        static_assert(sizeof(FusedLayerPtrs) % 8 == 0, "the table is copied in 8-byte words");
        const uint64_t *src = reinterpret_cast<const uint64_t *>(a.layers);
        uint64_t *dst = reinterpret_cast<uint64_t *>(sm.lp);
        const int words = a.n_layers * (int)(sizeof(FusedLayerPtrs) / 8);
        for (int i = threadIdx.x; i < words; i += FT) dst[i] = src[i];
        if (threadIdx.x == 0) sm.arrive = 0;
        __syncthreads();
    }
    if (wave < NCW) {
        compute_role<GE>(a, sm, wg, wave, lane, pos);
    } else {
        const uint32_t launches = __hip_atomic_load(a.ctl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        comm_role<GE>(a, sm, wg, wave - NCW, lane, pos, launches * (uint32_t)a.n_layers);
    }
}

// Qwen3-0.6B and a small shape of the same family for tests
using GeoQwen3_0p6b = Geo<1024, 16, 8, 128, 3072, 256>;
using GeoSmall = Geo<512, 4, 2, 128, 1024, 64>;

template <class GE>
bool shape_is(const FusedShape &s) {
    return s.hidden == GE::HIDDEN && s.heads == GE::H && s.kv_heads == GE::KVH && s.head_dim == GE::HD &&
           s.inter == GE::INTER;
}

template <class GE>
bool fits_device(const hm_ctx *ctx, const char **why) {
    if (ctx->num_cus < GE::NWG) {
        *why = "fewer compute units than resident workgroups";
        return false;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, decode_fused_kernel<GE>, FT, 0) != hipSuccess || per_cu < 1) {
        (void)hipGetLastError();
        *why = "the kernel does not fit a compute unit";
        return false;
    }
    return true;
}

}  // namespace

int decode_fused_max_kv(const FusedShape &s) {
    if (shape_is<GeoQwen3_0p6b>(s)) return GeoQwen3_0p6b::MAX_KV;
    if (shape_is<GeoSmall>(s)) return GeoSmall::MAX_KV;
    return 0;
}

size_t decode_fused_xch_bytes(const FusedShape &s) {
    if (shape_is<GeoQwen3_0p6b>(s)) return (size_t)GeoQwen3_0p6b::PAR_SLOTS * 8 * 2;
    if (shape_is<GeoSmall>(s)) return (size_t)GeoSmall::PAR_SLOTS * 8 * 2;
    return 0;
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
    const int max_kv = decode_fused_max_kv(s);
    if (!max_kv) {
        *why = "no kernel instance for this shape";
        return false;
    }
    if (max_seq_len > max_kv) {
        *why = "cache longer than the attention phase keeps in registers";
        return false;
    }
    if (shape_is<GeoQwen3_0p6b>(s)) return fits_device<GeoQwen3_0p6b>(ctx, why);
    return fits_device<GeoSmall>(ctx, why);
}

int decode_fused_launch(hm_ctx *ctx, const FusedShape &s, const FusedDecodeArgs &a) {
    HM_REQUIRE(ctx, a.layers && a.embed && a.state && a.forced && a.hidden_out && a.cos_tab && a.sin_tab && a.xch && a.ctl,
               "decode_fused: NULL pointer");
    HM_REQUIRE(ctx, a.n_layers >= 1 && a.n_layers <= MAX_LAYERS && a.max_len >= 1 && a.max_len <= decode_fused_max_kv(s),
               "decode_fused: %d layers / %d cache rows not served for this shape", a.n_layers, a.max_len);
    if (shape_is<GeoQwen3_0p6b>(s))
        hipLaunchKernelGGL(decode_fused_kernel<GeoQwen3_0p6b>, dim3(GeoQwen3_0p6b::NWG), dim3(FT), 0, ctx->stream, a);
    else if (shape_is<GeoSmall>(s))
        hipLaunchKernelGGL(decode_fused_kernel<GeoSmall>, dim3(GeoSmall::NWG), dim3(FT), 0, ctx->stream, a);
    else
        return hm_set_error(ctx, HM_ERR_INVALID, "decode_fused: no kernel instance for this shape");
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int decode_fused_check(hm_ctx *ctx, const uint32_t *d_ctl) {
    uint32_t h[2] = {0, 0};
    int rc = hm_download(ctx, h, d_ctl, sizeof(h));
    if (rc != HM_OK) return rc;
    if (h[1] != 0)
        return hm_set_error(ctx, HM_ERR_HIP, "decode_fused: an exchange timed out (status %u after %u launches)", h[1], h[0]);
    return HM_OK;
}
