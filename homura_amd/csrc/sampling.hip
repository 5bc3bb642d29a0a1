// Token sampling (reference sample_token, src/generate.rs:698-801, and its xorshift64 Rng, :609-642).
//
// Two implementations behind one configuration struct:
//  * hm_sample_token_host: the reference's procedure statement by statement on a host logits row
//    (libm expf, sequential f32 sums, full sort). Any top_k.
//  * hm_sample_token: the same procedure on a logits row that stays in HBM, for 1 <= top_k <= 1024.
//    One workgroup of 1024 threads: penalties + temperature + max, exponentials + sum, a radix select
//    (12 + 10 + 10 bits) of the top_k-th largest exponential, the candidates gathered and sorted in LDS (probability
//    descending, index ascending among equals), then one thread runs the reference's sequential top_p
//    and draw loops over at most 1024 candidates. The vocabulary-wide sum is a tree sum here, so a
//    probability may differ from the host's in the last bit; the picked token differs only when the
//    draw sits on a cumulative boundary to within that bit.
// The draw itself (Rng::next_f32) is taken on the host and passed in, so both consume the same stream.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

#include "hm_common.h"

namespace {

constexpr int SAMPLE_THREADS = 1024;
constexpr int SAMPLE_MAX_K = 1024;

struct SampleArgs {
    const float *logits;
    float *work;          // [vocab] scratch: adjusted logits, then exponentials
    const int *counts;    // [vocab] occurrences among the generated tokens, or nullptr
    int vocab;
    hm_sampling_config cfg;
    float draw;           // Rng::next_f32 of this step
    int32_t *out;         // the picked token
    int *counts_update;   // if set: counts_update[token]++ after the pick (the token joins generated_ids)
    int32_t *list;        // if set: list[list_pos] = token
    int list_pos;
    // Device-resident loop: the step that was just taken is cursor->step - 1; its draw is draws[that], the pick
    // goes to list[that] and replaces the step's own greedy pick as the next input (cursor->token), and the
    // first step whose pick is `eos` is noted in stop[0] (-1 until then).
    DecodeState *cursor;
    const float *draws;
    int eos;
    int *stop;
};

// What a sampler kernel needs to know about its step, read once at its start: the loads are two dependent trips
// to memory (the cursor, then the draw it points at) that would otherwise sit at the very end of a kernel that
// runs as a single workgroup.
struct StepInfo {
    int idx;     // the step that was just taken (cursor->step - 1), or -1 without a cursor
    float draw;  // Rng::next_f32 of this step
    int stop;    // *stop (-1: no end-of-sequence pick so far), 0 without a stop cell
};
__device__ __forceinline__ StepInfo load_step(const SampleArgs &a) {
    StepInfo s;
    s.idx = a.cursor ? a.cursor->step - 1 : -1;
    s.draw = (a.cursor && a.draws) ? a.draws[s.idx] : a.draw;  // (a greedy pick with penalties has no draws)
    s.stop = a.stop ? *a.stop : 0;
    return s;
}

// Where the pick goes when the cursor says which step this is.
__device__ __forceinline__ void deliver_pick(const SampleArgs &a, const StepInfo &st, int pick) {
    *a.out = pick;
    if (a.counts_update) a.counts_update[pick] += 1;
    if (a.cursor) {
        if (a.list) a.list[st.idx] = pick;
        a.cursor->token = pick;
        if (a.stop && pick == a.eos && st.stop < 0) *a.stop = st.idx;
    } else if (a.list) {
        a.list[a.list_pos] = pick;
    }
}

__device__ __forceinline__ float penalised(float l, int c, const hm_sampling_config &cfg) {
    if (c > 0) {
        if (cfg.repetition_penalty != 1.0f)
            for (int k = 0; k < c; k++) l = l > 0.0f ? l / cfg.repetition_penalty : l * cfg.repetition_penalty;
        if (cfg.frequency_penalty != 0.0f || cfg.presence_penalty != 0.0f) {
            l -= cfg.frequency_penalty * (float)c;
            l -= cfg.presence_penalty;
        }
    }
    return l;
}

// a > b in the candidate order: larger probability first, smaller index first among equals
__device__ __forceinline__ bool cand_before(float pa, int ia, float pb, int ib) {
    return pa > pb || (pa == pb && ia < ib);
}

// One pass of the workgroup over [0, n): thread t visits t, t + 1024, ... in ascending order, eight elements'
// loads in flight before the first is used (a plain strided loop waits for every load in turn, and with one
// workgroup on the whole chip the passes are pure latency).
template <class Load, class Use>
__device__ __forceinline__ void sweep(int n, int tid, Load load, Use use) {
    constexpr int UN = 8;
    for (int base = tid; base < n; base += UN * SAMPLE_THREADS) {
        decltype(load(0)) v[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int i = base + u * SAMPLE_THREADS;
            if (i < n) v[u] = load(i);
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int i = base + u * SAMPLE_THREADS;
            if (i < n) use(i, v[u]);
        }
    }
}

struct LogitAndCount {
    float l;
    int c;
};

// Shared memory of the selection below.
struct SelectShared {
    float red_f[SAMPLE_THREADS / WAVE];
    int red_i[SAMPLE_THREADS / WAVE];
    unsigned hist[4096];
    unsigned sel_prefix, sel_need;
    float cand_p[SAMPLE_MAX_K];
    int cand_i[SAMPLE_MAX_K];
    unsigned n_cand, eq_taken, n_eq;
    int eq_idx[SAMPLE_MAX_K];
};

// The second half of the procedure over n items: key_at(j) is item j's 32-bit key (larger key = larger
// exponential; items with equal keys must appear in ascending token order), idx_at(j) its token,
// weight_of(key) its exponential; `sum` is the sum of all n_all exponentials of the vocabulary. Selects the
// top_k items, normalises, applies min_p, sorts and runs the reference's sequential top_p and draw loops.
template <class KeyAt, class IdxAt, class WeightOf>
__device__ __forceinline__ void select_sort_draw(SelectShared &sh, const SampleArgs &a, const StepInfo &st, int n, int n_all,
                                                 float sum, KeyAt key_at, IdxAt idx_at, WeightOf weight_of) {
    float (&red_f)[SAMPLE_THREADS / WAVE] = sh.red_f;
    int (&red_i)[SAMPLE_THREADS / WAVE] = sh.red_i;
    unsigned (&hist)[4096] = sh.hist;
    unsigned &sel_prefix = sh.sel_prefix, &sel_need = sh.sel_need;
    float (&cand_p)[SAMPLE_MAX_K] = sh.cand_p;
    int (&cand_i)[SAMPLE_MAX_K] = sh.cand_i;
    unsigned &n_cand = sh.n_cand, &eq_taken = sh.eq_taken, &n_eq = sh.n_eq;
    int (&eq_idx)[SAMPLE_MAX_K] = sh.eq_idx;
    (void)red_f;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const hm_sampling_config cfg = a.cfg;
    // ── radix select: key of the K-th largest item (keys order like the exponentials). 12 + 10 + 10 bits: the first pass sees every element, and 4096 bins keep neighbouring
    //    lanes off each other's LDS word; later passes only count the elements inside the chosen bin. ──
    const unsigned K = (unsigned)min(cfg.top_k, n_all);
    if (tid == 0) {
        sel_prefix = 0;
        sel_need = K;
    }
    for (int pass = 0; pass < 3; pass++) {
        const int shift = pass == 0 ? 20 : pass == 1 ? 10 : 0;
        const int bits = pass == 0 ? 12 : 10;
        const int bpt = (1 << bits) / SAMPLE_THREADS;  // bins per thread: 4, 1, 1
        for (int b = tid; b < (1 << bits); b += SAMPLE_THREADS) hist[b] = 0;
        __syncthreads();
        const unsigned prefix = sel_prefix, need = sel_need;
        const unsigned mask = pass == 0 ? 0u : 0xFFFFFFFFu << (shift + bits);
        sweep(n, tid, key_at, [&](int, unsigned u) {
            if ((u & mask) == prefix) atomicAdd(&hist[(u >> shift) & ((1u << bits) - 1u)], 1u);
        });
        __syncthreads();
        // the bin that holds the need-th largest of the counted elements: thread t owns bins [t*bpt, (t+1)*bpt)
        unsigned mine = 0;
        for (int j = 0; j < bpt; j++) mine += hist[tid * bpt + j];
        unsigned incl = mine;  // inclusive prefix sum over threads, low bins first
        for (int off = 1; off < WAVE; off <<= 1) {
            const unsigned up = __shfl_up(incl, off, WAVE);
            if (lane >= off) incl += up;
        }
        if (lane == WAVE - 1) red_i[wave] = (int)incl;
        __syncthreads();
        unsigned before = 0, total = 0;
        for (int w = 0; w < SAMPLE_THREADS / WAVE; w++) {
            if (w < wave) before += (unsigned)red_i[w];
            total += (unsigned)red_i[w];
        }
        const unsigned below_or_mine = before + incl;      // elements in bins up to and including mine
        const unsigned above = total - below_or_mine;      // elements in higher bins
        if (above < need && need <= above + mine) {        // exactly one thread
            unsigned acc = above;
            for (int j = bpt - 1; j >= 0; j--) {
                const unsigned h = hist[tid * bpt + j];
                if (acc + h >= need) {
                    sel_prefix = prefix | ((unsigned)(tid * bpt + j) << shift);
                    sel_need = need - acc;  // how many elements of this bin are still wanted
                    break;
                }
                acc += h;
            }
        }
        __syncthreads();
    }
    const unsigned T = sel_prefix;
    const unsigned need_eq = sel_need;
    if (tid == 0) {
        n_cand = 0;
        eq_taken = 0;
        n_eq = 0;
    }
    __syncthreads();
    // everything above the K-th value; then the wanted number of elements equal to it, lowest indices first
    sweep(n, tid, key_at, [&](int i, unsigned u) {
        if (u > T) {
            const unsigned at = atomicAdd(&n_cand, 1u);
            cand_p[at] = weight_of(u);
            cand_i[at] = idx_at(i);
        } else if (u == T) {
            const unsigned at = atomicAdd(&n_eq, 1u);
            if (at < (unsigned)SAMPLE_MAX_K) eq_idx[at] = idx_at(i);
        }
    });
    __syncthreads();
    // Few elements equal the K-th value (nearly always exactly one): they were noted on the way, and each takes
    // its rank among them by index. Otherwise (a flat tail, underflowed exponentials) one ordered walk.
    const bool eq_listed = n_eq <= (unsigned)SAMPLE_MAX_K;
    if (eq_listed && tid < (int)n_eq) {
        const int mine = eq_idx[tid];
        unsigned rank = 0;
        for (unsigned j = 0; j < n_eq; j++) rank += eq_idx[j] < mine ? 1u : 0u;
        if (rank < need_eq) {
            const unsigned at = atomicAdd(&n_cand, 1u);
            cand_p[at] = weight_of(T);
            cand_i[at] = mine;
        }
    }
    for (int base = 0; base < n; base += SAMPLE_THREADS) {  // index order: one block-wide ordered take per 1024
        if (eq_listed || eq_taken >= need_eq) break;
        const int i = base + tid;
        const bool eq = i < n && key_at(i) == T;
        const unsigned long long m = __ballot(eq);
        if (lane == 0) red_i[wave] = __popcll(m);
        __syncthreads();
        unsigned before = eq_taken;
        for (int w = 0; w < wave; w++) before += red_i[w];
        const unsigned rank = before + __popcll(m & ((1ull << lane) - 1ull));
        if (eq && rank < need_eq) {
            const unsigned at = atomicAdd(&n_cand, 1u);
            cand_p[at] = weight_of(T);
            cand_i[at] = idx_at(i);
        }
        __syncthreads();
        if (tid == 0) {
            unsigned tot = 0;
            for (int w = 0; w < SAMPLE_THREADS / WAVE; w++) tot += red_i[w];
            eq_taken += tot;
        }
        __syncthreads();
    }
    __syncthreads();
    const int nc = (int)n_cand;  // == K
    // normalise, min_p (the maximum probability is exp(0) / sum), pad to the sort size
    const float max_prob = 1.0f / sum;
    const float threshold = cfg.min_p * max_prob;
    int sort_n = 2;  // the power of two that holds the candidates: 64 for the default top_k of 50, not 1024
    while (sort_n < nc) sort_n <<= 1;
    if (tid < sort_n) {
        if (tid < nc) {
            float p = cand_p[tid] / sum;
            if (cfg.min_p > 0.0f && p < threshold) p = 0.0f;
            cand_p[tid] = p;
        } else {
            cand_p[tid] = -1.0f;  // sorts behind every real candidate
            cand_i[tid] = 0x7FFFFFFF;
        }
    }
    __syncthreads();
    // bitonic sort of sort_n (probability descending, index ascending among equals)
    for (int k = 2; k <= sort_n; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            const int partner = tid ^ j;
            if (partner > tid && tid < sort_n) {
                const float pa = cand_p[tid], pb = cand_p[partner];
                const int ia = cand_i[tid], ib = cand_i[partner];
                const bool up = (tid & k) == 0;  // this pair ends in candidate order
                if (cand_before(pb, ib, pa, ia) == up) {
                    cand_p[tid] = pb;
                    cand_i[tid] = ib;
                    cand_p[partner] = pa;
                    cand_i[partner] = ia;
                }
            }
            __syncthreads();
        }
    // the reference's sequential loops (src/generate.rs:771-800). Up to a wavefront's worth of candidates (the
    // default top_k of 50) sit in the registers of wavefront 0 and the loops read them lane by lane: the same
    // additions in the same order, without an LDS round trip per step.
    if (nc <= WAVE) {
        if (wave != 0) return;
        const float p = lane < nc ? cand_p[lane] : 0.0f;
        const int ci = lane < nc ? cand_i[lane] : 0;
        auto p_at = [&](int i) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), i)); };
        float cumulative = 0.0f;
        int cutoff = nc;
        for (int i = 0; i < nc; i++) {
            cumulative += p_at(i);
            if (cumulative >= cfg.top_p) {
                cutoff = i + 1;
                break;
            }
        }
        float total = 0.0f;
        for (int i = 0; i < cutoff; i++) total += p_at(i);
        const float r = st.draw * total;
        float accum = 0.0f;
        int at = cutoff > 0 ? cutoff - 1 : -1;
        for (int i = 0; i < cutoff; i++) {
            accum += p_at(i);
            if (accum >= r) {
                at = i;
                break;
            }
        }
        const int pick = at >= 0 ? __builtin_amdgcn_readlane(ci, at) : 0;
        if (lane == 0) deliver_pick(a, st, pick);
        return;
    }
    if (tid == 0) {
        float cumulative = 0.0f;
        int cutoff = nc;
        for (int i = 0; i < nc; i++) {
            cumulative += cand_p[i];
            if (cumulative >= cfg.top_p) {
                cutoff = i + 1;
                break;
            }
        }
        float total = 0.0f;
        for (int i = 0; i < cutoff; i++) total += cand_p[i];
        const float r = st.draw * total;
        float accum = 0.0f;
        int pick = cutoff > 0 ? cand_i[cutoff - 1] : 0;
        for (int i = 0; i < cutoff; i++) {
            accum += cand_p[i];
            if (accum >= r) {
                pick = cand_i[i];
                break;
            }
        }
        deliver_pick(a, st, pick);
    }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_token_kernel(SampleArgs a) {
    __shared__ SelectShared sh;
    float (&red_f)[SAMPLE_THREADS / WAVE] = sh.red_f;
    int (&red_i)[SAMPLE_THREADS / WAVE] = sh.red_i;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int n = a.vocab;
    const hm_sampling_config cfg = a.cfg;
    const StepInfo st = load_step(a);

    // ── pass 1: penalties, then either the greedy pick or temperature + maximum ──
    const bool greedy = cfg.temperature <= 0.0f;
    const float inv_temp = greedy ? 1.0f : 1.0f / cfg.temperature;
    float mx = -INFINITY;
    int best = -1;  // greedy: last index of the maximum (Rust max_by keeps the last of equal maxima)
    sweep(n, tid, [&](int i) { return LogitAndCount{a.logits[i], a.counts ? a.counts[i] : 0}; },
          [&](int i, const LogitAndCount &lc) {
              float l = penalised(lc.l, lc.c, cfg);
              if (greedy) {
                  if (best < 0 || l >= mx) {
                      mx = l;
                      best = i;
                  }
              } else {
                  l *= inv_temp;
                  a.work[i] = l;
                  mx = fmaxf(mx, l);
              }
          });
    if (greedy) {
        for (int off = 32; off >= 1; off >>= 1) {
            const float om = __shfl_xor(mx, off, WAVE);
            const int ob = __shfl_xor(best, off, WAVE);
            if (ob >= 0 && (best < 0 || om > mx || (om == mx && ob > best))) {
                mx = om;
                best = ob;
            }
        }
        if (lane == 0) {
            red_f[wave] = mx;
            red_i[wave] = best;
        }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < SAMPLE_THREADS / WAVE; w++)
                if (red_i[w] >= 0 && (best < 0 || red_f[w] > mx || (red_f[w] == mx && red_i[w] > best))) {
                    mx = red_f[w];
                    best = red_i[w];
                }
            deliver_pick(a, st, best < 0 ? 0 : best);
        }
        return;
    }
    mx = wave_max(mx);
    if (lane == 0) red_f[wave] = mx;
    __syncthreads();
    mx = red_f[0];
    for (int w = 1; w < SAMPLE_THREADS / WAVE; w++) mx = fmaxf(mx, red_f[w]);
    __syncthreads();

    // ── pass 2: exponentials and their sum ──
    float sum = 0.f;
    sweep(n, tid, [&](int i) { return a.work[i]; }, [&](int i, float l) {
        const float e = expf(l - mx);
        a.work[i] = e;
        sum += e;
    });
    sum = wave_sum(sum);
    if (lane == 0) red_f[wave] = sum;
    __syncthreads();
    sum = 0.f;
    for (int w = 0; w < SAMPLE_THREADS / WAVE; w++) sum += red_f[w];
    __syncthreads();
    // exponentials are >= 0, so their bit patterns order like their values
    select_sort_draw(sh, a, st, n, n, sum, [&](int i) { return __float_as_uint(a.work[i]); }, [&](int i) { return i; },
                     [&](unsigned key) { return __uint_as_float(key); });
}

// ── Small top_k (<= 64) over a large vocabulary: two launches instead of one workgroup's eight passes ──
// Front: a workgroup per 1024 tokens applies penalties and temperature, takes its maximum and the sum of
// exponentials relative to it, and keeps the 64 of its tokens that come first by (logit descending, token
// ascending), in token order: the vocabulary's top_k are among them. Back: one workgroup combines the maxima and sums (sum over the
// vocabulary = sum_b sum_b * exp(max_b - max), equal to the single pass's up to rounding) and runs the shared
// selection over the kept tokens; it selects by logit, which orders tokens like their exponentials except
// where two different logits round to one exponential.
constexpr int FRONT_KEEP = 64;

// larger float <-> larger key (-inf the smallest key of all finite and infinite values)
__device__ __forceinline__ unsigned order_key(float x) {
    const unsigned u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(unsigned k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
}

struct FrontOut {
    unsigned *key;  // [blocks][FRONT_KEEP]
    int *idx;       // [blocks][FRONT_KEEP]
    float *stat;    // [blocks][2]: maximum, sum of exponentials relative to it
};
__host__ __device__ inline FrontOut front_out(float *work, int blocks) {
    FrontOut f;
    f.key = reinterpret_cast<unsigned *>(work);
    f.idx = reinterpret_cast<int *>(work) + (size_t)blocks * FRONT_KEEP;
    f.stat = work + (size_t)blocks * FRONT_KEEP * 2;
    return f;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_front_kernel(SampleArgs a) {
    __shared__ unsigned hist[4096];
    __shared__ float red[SAMPLE_THREADS / WAVE], red_s[SAMPLE_THREADS / WAVE];
    __shared__ int red_i[SAMPLE_THREADS / WAVE];
    __shared__ unsigned sel_prefix, sel_need;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int i = blockIdx.x * SAMPLE_THREADS + tid;
    const bool on = i < a.vocab;
    const float inv_temp = 1.0f / a.cfg.temperature;
    const float x = on ? penalised(a.logits[i], a.counts ? a.counts[i] : 0, a.cfg) * inv_temp : -INFINITY;
    float m = wave_max(x);
    if (lane == 0) red[wave] = m;
    if (tid == 0) {
        sel_prefix = 0;
        sel_need = FRONT_KEEP;
    }
    __syncthreads();
    m = red[0];
    for (int w = 1; w < SAMPLE_THREADS / WAVE; w++) m = fmaxf(m, red[w]);
    const float e = (on && x > -INFINITY) ? expf(x - m) : 0.f;
    const float ws = wave_sum(e);
    if (lane == 0) red_s[wave] = ws;
    // The 64 tokens that come first by (logit descending, token ascending), kept in token order: the key of the
    // 64th by a radix select over the 1024 keys (12 + 10 + 10 bits, one element per thread), then everything
    // above it and the lowest-numbered of the tokens equal to it. Tokens past the vocabulary carry the key of
    // -inf and come last among equals.
    const unsigned key = order_key(x);
    for (int pass = 0; pass < 3; pass++) {
        const int shift = pass == 0 ? 20 : pass == 1 ? 10 : 0;
        const int bits = pass == 0 ? 12 : 10;
        const int bpt = (1 << bits) / SAMPLE_THREADS;  // bins per thread: 4, 1, 1
        for (int b = tid; b < (1 << bits); b += SAMPLE_THREADS) hist[b] = 0;
        __syncthreads();
        const unsigned prefix = sel_prefix, need = sel_need;
        const unsigned mask = pass == 0 ? 0u : 0xFFFFFFFFu << (shift + bits);
        if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & ((1u << bits) - 1u)], 1u);
        __syncthreads();
        unsigned mine = 0;
        for (int j = 0; j < bpt; j++) mine += hist[tid * bpt + j];
        unsigned incl = mine;  // inclusive prefix sum over threads, low bins first
        for (int off = 1; off < WAVE; off <<= 1) {
            const unsigned up = __shfl_up(incl, off, WAVE);
            if (lane >= off) incl += up;
        }
        if (lane == WAVE - 1) red_i[wave] = (int)incl;
        __syncthreads();
        unsigned before = 0, total = 0;
        for (int w = 0; w < SAMPLE_THREADS / WAVE; w++) {
            if (w < wave) before += (unsigned)red_i[w];
            total += (unsigned)red_i[w];
        }
        const unsigned above = total - (before + incl);  // elements in higher bins
        if (above < need && need <= above + mine) {      // exactly one thread
            unsigned acc = above;
            for (int j = bpt - 1; j >= 0; j--) {
                const unsigned h = hist[tid * bpt + j];
                if (acc + h >= need) {
                    sel_prefix = prefix | ((unsigned)(tid * bpt + j) << shift);
                    sel_need = need - acc;
                    break;
                }
                acc += h;
            }
        }
        __syncthreads();
    }
    const unsigned T = sel_prefix, need_eq = sel_need;
    // rank of this thread among the threads whose key equals T (thread order = token order)
    const bool eq = key == T;
    const unsigned long long em = __ballot(eq);
    if (lane == 0) red_i[wave] = __popcll(em);
    __syncthreads();
    unsigned eq_rank = __popcll(em & ((1ull << lane) - 1ull));
    for (int w = 0; w < wave; w++) eq_rank += (unsigned)red_i[w];
    __syncthreads();
    const bool keep = key > T || (eq && eq_rank < need_eq);
    const unsigned long long km = __ballot(keep);
    if (lane == 0) red_i[wave] = __popcll(km);
    __syncthreads();
    unsigned pos = __popcll(km & ((1ull << lane) - 1ull));
    for (int w = 0; w < wave; w++) pos += (unsigned)red_i[w];
    const FrontOut f = front_out(a.work, gridDim.x);
    if (keep) {  // exactly FRONT_KEEP threads
        f.key[(size_t)blockIdx.x * FRONT_KEEP + pos] = key;
        f.idx[(size_t)blockIdx.x * FRONT_KEEP + pos] = on ? i : 0x7FFFFFFF;
    }
    if (tid == 0) {
        float sum = 0.f;
        for (int w = 0; w < SAMPLE_THREADS / WAVE; w++) sum += red_s[w];
        f.stat[blockIdx.x * 2] = m;
        f.stat[blockIdx.x * 2 + 1] = sum;
    }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_back_kernel(SampleArgs a, int blocks) {
    __shared__ SelectShared sh;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const StepInfo st = load_step(a);
    const FrontOut f = front_out(a.work, blocks);
    // This kernel is one workgroup, and every dependent trip to memory costs it a couple of microseconds: the kept
    // tokens (up to PRE per thread) are asked for before anything waits on the blocks' statistics.
    constexpr int PRE = 16;
    const int n_kept = blocks * FRONT_KEEP;
    const bool preloaded = n_kept <= PRE * SAMPLE_THREADS;
    unsigned pk[PRE];
    int pi[PRE];
    if (preloaded) {
#pragma unroll
        for (int u = 0; u < PRE; u++) {
            const int j = tid + u * SAMPLE_THREADS;
            pk[u] = j < n_kept ? f.key[j] : 0u;
            pi[u] = j < n_kept ? f.idx[j] : 0;
        }
    }
    float m = -INFINITY;
    for (int b = tid; b < blocks; b += SAMPLE_THREADS) m = fmaxf(m, f.stat[b * 2]);
    m = wave_max(m);
    if (lane == 0) sh.red_f[wave] = m;
    __syncthreads();
    m = sh.red_f[0];
    for (int w = 1; w < SAMPLE_THREADS / WAVE; w++) m = fmaxf(m, sh.red_f[w]);
    __syncthreads();
    float sum = 0.f;
    for (int b = tid; b < blocks; b += SAMPLE_THREADS) {
        const float bm = f.stat[b * 2];
        if (bm > -INFINITY) sum += f.stat[b * 2 + 1] * expf(bm - m);
    }
    sum = wave_sum(sum);
    if (lane == 0) sh.red_f[wave] = sum;
    __syncthreads();
    sum = 0.f;
    for (int w = 0; w < SAMPLE_THREADS / WAVE; w++) sum += sh.red_f[w];
    __syncthreads();
    auto weight = [&](unsigned key) {
        const float x = key_value(key);
        return x > -INFINITY ? expf(x - m) : 0.f;
    };
    // The K-th largest of the blocks' maxima is a floor for the K-th largest logit of the vocabulary (K tokens reach
    // it), so only kept tokens at or above it can be among the top K: usually a hundred or so of the blocks * 64.
    // With at most 1024 of them the selection is done by rank: every survivor counts the survivors ahead of it in
    // (logit descending, token ascending), the first K take their rank as their place, and after normalisation and
    // min_p the same count over (probability descending, token ascending) gives the order the reference's
    // sequential loops walk. A flat distribution (more survivors) takes the general selection over the full list.
    // a survivor as one 64-bit number that orders like (logit descending, token ascending): key, then the
    // token counted down from the largest
    __shared__ unsigned bkey[SAMPLE_THREADS], tau, fcount;
    __shared__ unsigned long long fcomp[SAMPLE_MAX_K];
    const unsigned K = (unsigned)min(a.cfg.top_k, a.vocab);
    if (preloaded && blocks <= SAMPLE_THREADS && (unsigned)blocks >= K && K >= 1 && K <= (unsigned)WAVE) {
        bkey[tid] = tid < blocks ? order_key(f.stat[tid * 2]) : 0u;
        if (tid == 0) fcount = 0;
        __syncthreads();
        if (tid < blocks) {
            const unsigned mine = bkey[tid];
            unsigned rank = 0;
#pragma unroll 16
            for (int c = 0; c < blocks; c++) {  // (unrolled: sixteen LDS reads in flight, not one)
                const unsigned o = bkey[c];
                rank += ((o > mine) | ((o == mine) & (c < tid))) ? 1u : 0u;
            }
            if (rank == K - 1) tau = mine;
        }
        __syncthreads();
        const unsigned floor_key = tau;
#pragma unroll
        for (int u = 0; u < PRE; u++) {
            const int j = tid + u * SAMPLE_THREADS;
            if (j < n_kept && pk[u] >= floor_key) {
                const unsigned at = atomicAdd(&fcount, 1u);
                if (at < (unsigned)SAMPLE_MAX_K) fcomp[at] = ((unsigned long long)pk[u] << 32) | (unsigned)(0x7FFFFFFF - pi[u]);
            }
        }
        __syncthreads();
        const int nf = (int)fcount;
        if (nf <= SAMPLE_MAX_K) {
            float (&cand_p)[SAMPLE_MAX_K] = sh.cand_p;
            int (&cand_i)[SAMPLE_MAX_K] = sh.cand_i;
            if (tid < nf) {
                const unsigned long long mine = fcomp[tid];
                const int mi = 0x7FFFFFFF - (int)(unsigned)(mine & 0xFFFFFFFFull);
                unsigned rank = 0;
#pragma unroll 16
                for (int c = 0; c < nf; c++) rank += fcomp[c] > mine ? 1u : 0u;  // (straight-line: sixteen LDS reads in flight)
                if (rank < K) {  // normalise, min_p (the maximum probability is exp(0) / sum)
                    float p = weight((unsigned)(mine >> 32)) / sum;
                    if (a.cfg.min_p > 0.0f && p < a.cfg.min_p * (1.0f / sum)) p = 0.0f;
                    cand_p[rank] = p;
                    cand_i[rank] = mi;
                }
            }
            __syncthreads();
            if (wave != 0) return;
            // K <= 64 candidates, one per lane: place by (probability descending, token ascending), then the
            // reference's sequential loops (src/generate.rs:771-800) over the lanes
            const int nc = (int)K;
            const float p0 = lane < nc ? cand_p[lane] : -1.0f;
            const int i0 = lane < nc ? cand_i[lane] : 0x7FFFFFFF;
            // (lanes past nc hold (-1, largest token): behind every candidate. Constant lane numbers: the
            // loops below are straight-line code.)
            int place = 0;
#pragma unroll
            for (int c = 0; c < WAVE; c++) {
                const float pc = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p0), c));
                const int ic = __builtin_amdgcn_readlane(i0, c);
                place += cand_before(pc, ic, p0, i0) ? 1 : 0;
            }
            // lane l wants the candidate whose place is l: scatter through LDS (wavefront 0 only; no other
            // wavefront touches cand_p / cand_i any more)
            cand_p[SAMPLE_MAX_K / 2 + place] = p0;  // (the candidates' places are 0 .. nc - 1; every other lane writes slot nc)
            cand_i[SAMPLE_MAX_K / 2 + place] = i0;
            __builtin_amdgcn_wave_barrier();  // (LDS operations of a wavefront execute in order)
            const float p = lane < nc ? cand_p[SAMPLE_MAX_K / 2 + lane] : 0.0f;
            const int ci = cand_i[SAMPLE_MAX_K / 2 + lane];
            // The reference's three loops add the same probabilities in the same order from zero: cumulative until
            // top_p is reached, the total of the kept candidates (= that cumulative sum), and the running sum
            // the draw is compared with. One chain of additions gives all three; lane i keeps the sum after
            // candidate i. (Lanes past nc add 0.)
            float chain = 0.0f, upto = 0.0f;
#pragma unroll
            for (int i = 0; i < WAVE; i++) {
                chain += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), i));
                upto = lane == i ? chain : upto;
            }
            const unsigned long long live = nc >= WAVE ? ~0ull : ((1ull << nc) - 1ull);
            const unsigned long long reached = __ballot(upto >= a.cfg.top_p) & live;
            const int cutoff = reached ? __ffsll((long long)reached) : nc;  // index of the first + 1
            const float total = cutoff > 0 ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(upto), cutoff - 1)) : 0.0f;
            const float r = st.draw * total;
            const unsigned long long kept = cutoff >= WAVE ? ~0ull : ((1ull << cutoff) - 1ull);
            const unsigned long long hit = __ballot(upto >= r) & kept;
            const int at = hit ? __ffsll((long long)hit) - 1 : cutoff - 1;
            const int pick = at >= 0 ? __builtin_amdgcn_readlane(ci, at) : 0;
            if (lane == 0) deliver_pick(a, st, pick);
            return;
        }
    }
    // padding entries (tokens past the vocabulary) carry the key of -inf and the largest token number: they sort
    // behind every real token and are never among the vocabulary's top_k
    select_sort_draw(sh, a, st, n_kept, a.vocab, sum, [&](int j) { return f.key[j]; }, [&](int j) { return f.idx[j]; }, weight);
}

__global__ void count_tokens_kernel(const uint32_t *__restrict__ ids, int n_ids, int *__restrict__ counts, int vocab) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_ids && ids[i] < (uint32_t)vocab) atomicAdd(&counts[ids[i]], 1);
}

__global__ void zero_ints_kernel(int *__restrict__ p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

}  // namespace

namespace homura {

int sample_check_config(hm_ctx *ctx, const hm_sampling_config *cfg, bool device) {
    HM_REQUIRE(ctx, cfg != nullptr, "sampling: NULL configuration");
    HM_REQUIRE(ctx, cfg->top_k >= 0 && cfg->top_p > 0.0f && cfg->min_p >= 0.0f && cfg->repetition_penalty > 0.0f,
               "sampling: need top_k >= 0, top_p > 0, min_p >= 0, repetition_penalty > 0");
    if (device && cfg->temperature > 0.0f)
        HM_REQUIRE(ctx, cfg->top_k >= 1 && cfg->top_k <= SAMPLE_MAX_K,
                   "sampling on the device needs 1 <= top_k <= %d (got %d); use the host sampler", SAMPLE_MAX_K, cfg->top_k);
    return HM_OK;
}

// One workgroup for everything, or the front / back pair when top_k is small and the vocabulary large (the pair
// keeps its 130 words per 1024 tokens in `work`, which has a word per token).
static int sample_enqueue(hm_ctx *ctx, const SampleArgs &a) {
    const bool pair = a.cfg.temperature > 0.0f && a.cfg.top_k >= 1 && a.cfg.top_k <= FRONT_KEEP && a.vocab >= 4096;
    if (pair) {
        const int blocks = (a.vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
        hipLaunchKernelGGL(sample_front_kernel, dim3(blocks), dim3(SAMPLE_THREADS), 0, ctx->stream, a);
        HM_LAUNCH_CHECK(ctx);
        hipLaunchKernelGGL(sample_back_kernel, dim3(1), dim3(SAMPLE_THREADS), 0, ctx->stream, a, blocks);
    } else {
        hipLaunchKernelGGL(sample_token_kernel, dim3(1), dim3(SAMPLE_THREADS), 0, ctx->stream, a);
    }
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

// counts: device [vocab] occurrences (or nullptr); work: device [vocab] floats
int sample_token_launch(hm_ctx *ctx, const float *d_logits, float *d_work, const int *d_counts, int vocab,
                        const hm_sampling_config &cfg, float draw, int32_t *d_out, int *d_counts_update, int32_t *d_list,
                        int list_pos) {
    SampleArgs a;
    a.logits = d_logits;
    a.work = d_work;
    a.counts = d_counts;
    a.vocab = vocab;
    a.cfg = cfg;
    a.draw = draw;
    a.out = d_out;
    a.counts_update = d_counts_update;
    a.list = d_list;
    a.list_pos = list_pos;
    a.cursor = nullptr;
    a.draws = nullptr;
    a.eos = -1;
    a.stop = nullptr;
    return sample_enqueue(ctx, a);
}

// The sampler behind a decode step whose cursor has already moved on: no argument depends on the step, so the
// host can enqueue step after step without reading anything back.
int sample_step_launch(hm_ctx *ctx, const float *d_logits, float *d_work, int *d_counts, int vocab,
                       const hm_sampling_config &cfg, DecodeState *d_cursor, const float *d_draws, int32_t *d_list,
                       int eos, int *d_stop, int32_t *d_out) {
    SampleArgs a;
    a.logits = d_logits;
    a.work = d_work;
    a.counts = d_counts;
    a.vocab = vocab;
    a.cfg = cfg;
    a.draw = 0.0f;
    a.out = d_out;
    a.counts_update = d_counts;
    a.list = d_list;
    a.list_pos = 0;
    a.cursor = d_cursor;
    a.draws = d_draws;
    a.eos = eos;
    a.stop = d_stop;
    return sample_enqueue(ctx, a);
}

int zero_ints_launch(hm_ctx *ctx, int *d, size_t n) {
    if (n == 0) return HM_OK;
    hipLaunchKernelGGL(zero_ints_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream, d, n);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // namespace homura

extern "C" {

uint64_t hm_rng_seed(uint64_t seed) { return seed | 1u; }

float hm_rng_next_f32(uint64_t *state) {
    uint64_t s = *state;
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    *state = s;
    return (float)(s >> 40) / (float)(1ull << 24);
}

int hm_sample_token_host(const float *h_logits, int vocab, const hm_sampling_config *cfg, const uint32_t *h_generated,
                         int n_generated, uint64_t *rng_state, int32_t *token_out) {
    if (!h_logits || vocab <= 0 || !cfg || !rng_state || !token_out || n_generated < 0 || (n_generated && !h_generated))
        return HM_ERR_INVALID;
    std::vector<float> logits(h_logits, h_logits + vocab);
    if (cfg->repetition_penalty != 1.0f)
        for (int g = 0; g < n_generated; g++) {
            const uint32_t idx = h_generated[g];
            if (idx < (uint32_t)vocab) {
                if (logits[idx] > 0.0f)
                    logits[idx] /= cfg->repetition_penalty;
                else
                    logits[idx] *= cfg->repetition_penalty;
            }
        }
    if (cfg->frequency_penalty != 0.0f || cfg->presence_penalty != 0.0f) {
        std::vector<int> counts(vocab, 0);
        for (int g = 0; g < n_generated; g++)
            if (h_generated[g] < (uint32_t)vocab) counts[h_generated[g]]++;
        for (int i = 0; i < vocab; i++)
            if (counts[i]) {
                logits[i] -= cfg->frequency_penalty * (float)counts[i];
                logits[i] -= cfg->presence_penalty;
            }
    }
    if (cfg->temperature <= 0.0f) {  // greedy: the last of equal maxima (Rust max_by)
        int best = 0;
        for (int i = 1; i < vocab; i++)
            if (!(logits[best] > logits[i])) best = i;
        *token_out = best;
        return HM_OK;
    }
    const float inv_temp = 1.0f / cfg->temperature;
    float max_logit = -INFINITY;
    for (float &l : logits) {
        l *= inv_temp;
        max_logit = std::fmax(max_logit, l);
    }
    struct Cand {
        int idx;
        float p;
    };
    std::vector<Cand> c(vocab);
    float sum = 0.0f;
    for (int i = 0; i < vocab; i++) {
        c[i] = Cand{i, std::exp(logits[i] - max_logit)};
        sum += c[i].p;
    }
    for (Cand &x : c) x.p /= sum;
    if (cfg->min_p > 0.0f) {
        float max_prob = 0.0f;
        for (const Cand &x : c) max_prob = std::fmax(max_prob, x.p);
        const float threshold = cfg->min_p * max_prob;
        for (Cand &x : c)
            if (x.p < threshold) x.p = 0.0f;
    }
    // probability descending; the reference's sort_unstable_by leaves equal probabilities in an
    // unspecified order, here they keep index order
    std::sort(c.begin(), c.end(), [](const Cand &x, const Cand &y) { return x.p > y.p || (x.p == y.p && x.idx < y.idx); });
    size_t len = c.size();
    if (cfg->top_k > 0 && (size_t)cfg->top_k < len) len = (size_t)cfg->top_k;
    float cumulative = 0.0f;
    size_t cutoff = len;
    for (size_t i = 0; i < len; i++) {
        cumulative += c[i].p;
        if (cumulative >= cfg->top_p) {
            cutoff = i + 1;
            break;
        }
    }
    float total = 0.0f;
    for (size_t i = 0; i < cutoff; i++) total += c[i].p;
    const float r = hm_rng_next_f32(rng_state) * total;
    float accum = 0.0f;
    int pick = cutoff > 0 ? c[cutoff - 1].idx : 0;
    for (size_t i = 0; i < cutoff; i++) {
        accum += c[i].p;
        if (accum >= r) {
            pick = c[i].idx;
            break;
        }
    }
    *token_out = pick;
    return HM_OK;
}

int hm_sample_token(hm_ctx *ctx, const float *d_logits, int vocab, const hm_sampling_config *cfg,
                    const uint32_t *h_generated, int n_generated, uint64_t *rng_state, int32_t *token_out) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_logits && vocab > 0 && rng_state && token_out && n_generated >= 0 && (!n_generated || h_generated),
               "hm_sample_token: bad arguments");
    int rc = homura::sample_check_config(ctx, cfg, true);
    if (rc != HM_OK) return rc;
    // workspace: work [vocab] f32 | counts [vocab] i32 | token i32 | generated ids
    const size_t need = (size_t)vocab * 8 + 256 + (size_t)n_generated * 4;
    HM_REQUIRE(ctx, need <= ctx->workspace_bytes, "hm_sample_token: vocabulary / history too large for the workspace");
    float *work = (float *)ctx->workspace;
    int *counts = (int *)(work + vocab);
    int32_t *d_tok = (int32_t *)(counts + vocab);
    uint32_t *d_gen = (uint32_t *)((char *)d_tok + 256);
    const bool need_counts = n_generated > 0 && (cfg->repetition_penalty != 1.0f || cfg->frequency_penalty != 0.0f ||
                                                 cfg->presence_penalty != 0.0f);
    if (need_counts) {
        if ((rc = homura::zero_ints_launch(ctx, counts, (size_t)vocab)) != HM_OK) return rc;
        if ((rc = hm_upload(ctx, d_gen, h_generated, (size_t)n_generated * 4)) != HM_OK) return rc;
        hipLaunchKernelGGL(count_tokens_kernel, dim3((unsigned)((n_generated + 255) / 256)), dim3(256), 0, ctx->stream,
                           d_gen, n_generated, counts, vocab);
        HM_LAUNCH_CHECK(ctx);
    }
    const float draw = cfg->temperature > 0.0f ? hm_rng_next_f32(rng_state) : 0.0f;  // greedy leaves the stream alone
    rc = homura::sample_token_launch(ctx, d_logits, work, need_counts ? counts : nullptr, vocab, *cfg, draw, d_tok, nullptr,
                                     nullptr, 0);
    if (rc != HM_OK) return rc;
    return hm_download(ctx, token_out, d_tok, 4);
}

}  // extern "C"
