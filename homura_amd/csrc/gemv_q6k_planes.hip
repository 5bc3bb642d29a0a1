// Q6_K output matrix re-packed once, at upload, into four planes, and the f32 product over them (the LM head of
// a GGUF model whose output matrix is Q6_K: f32 row x dequantised weights, reference src/hf/emitter_quant.rs
// LM head and src/gguf.rs:880-917 for the block arithmetic).
//
// A 210-byte Q6_K block interleaves four 16-weight groups in every byte run: byte l of the low-nibble run
// carries weight l (low nibble) and weight l + 64 (high nibble), byte l + 32 weights l + 32 and l + 96, and
// byte l of the 2-bit run the top bits of all four. A "unit" is what shares bytes: 64 weights = groups g, g + 2,
// g + 4, g + 6 of one 128-weight half (l in 0..15 or 16..31), i.e. 32 bytes of nibbles, 16 bytes of top bits and
// four int8 scales. The planes hold, for all units of all rows in order,
//   nibbles  [units][32]   bytes ql[64 h + 16 p + j] (j = 0..15), then ql[64 h + 32 + 16 p + j]
//   top bits [units][16]   bytes qh[32 h + 16 p + j]
//   scales   [units][4]    sc[8 h + p], sc[8 h + p + 2], sc[8 h + p + 4], sc[8 h + p + 6]
//   d        [blocks]      f16
// for unit u = 2 h + p of a block: the same bytes as the block, every run at its natural alignment, so a lane
// loads its unit with three 16-byte loads, one dword and one half word straight into registers (the raw
// blocks start at multiples of 210 bytes and need an LDS stage and funnel shifts).
//
// A lane keeps the 64 activations of its unit position in registers for the whole launch; a trip of a
// wavefront is 64 consecutive units (= 64 / NU rows, NU = K / 64 units a row), and a row's sum is a segmented
// DPP reduction over its NU lanes.
#include "gemv_quant_planes.h"

#include "hm_common.h"

namespace {

constexpr int QTHREADS = 256;
constexpr int QWAVES = QTHREADS / WAVE;
constexpr int Q6K_BLOCK = 210;

typedef const uint32_t __attribute__((address_space(1))) *global_u32_ptr;
typedef const uint16_t __attribute__((address_space(1))) *global_u16_ptr;

struct Q6kPlanes {
    size_t top_off, scale_off, d_off, bytes;
};

Q6kPlanes q6k_planes_layout(int N, int K) {
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t units = (size_t)N * (K / 64);
    Q6kPlanes p;
    p.top_off = up(units * 32);
    p.scale_off = up(p.top_off + units * 16);
    p.d_off = up(p.scale_off + units * 4);
    p.bytes = p.d_off + (size_t)N * (K / 256) * 2;
    return p;
}

// The four bytes of w as floats against xv (the empty asm keeps the compiler from folding the masks that made
// w into one bit-field extract per byte: the conversions select their byte themselves).
__device__ __forceinline__ float dot4_bytes(uint32_t w, const float *xv, float s) {
    asm("" : "+v"(w));
    s = fmaf((float)(w & 0xFFu), xv[0], s);
    s = fmaf((float)((w >> 8) & 0xFFu), xv[1], s);
    s = fmaf((float)((w >> 16) & 0xFFu), xv[2], s);
    s = fmaf((float)(w >> 24), xv[3], s);
    return s;
}

// Sum over the NU lanes of a row's segment; the segment's last lane holds the total.
template <int NU>
__device__ __forceinline__ float segment_sum(float v) {
    if (NU >= 2) v += dpp_move<0xB1, 0xF>(v, 0.f);
    if (NU >= 4) v += dpp_move<0x4E, 0xF>(v, 0.f);
    if (NU >= 8) v += dpp_move<0x141, 0xF>(v, 0.f);
    if (NU >= 16) v += dpp_move<0x140, 0xF>(v, 0.f);
    if (NU >= 32) v += dpp_move<0x142, 0xA>(v, 0.f);
    if (NU >= 64) v += dpp_move<0x143, 0xC>(v, 0.f);
    return v;
}

struct UnitRegs {
    u32x4 a, b, h;  // nibbles of groups 0|2, of groups 1|3, top bits
    uint32_t sc;    // four int8 scales
    uint32_t d;     // f16 bits of the block's scale
};

// NU = units per row (K / 64): 4, 8, 16, 32 or 64.
template <int NU>
__global__ __launch_bounds__(QTHREADS) void gemv_q6k_units_kernel(const float *__restrict__ x, const float *__restrict__ norm_w,
                                                                  float eps, const uint8_t *__restrict__ nib,
                                                                  const uint8_t *__restrict__ top, const uint32_t *__restrict__ scales,
                                                                  const uint16_t *__restrict__ ds, float *__restrict__ out, int N,
                                                                  float *__restrict__ cand_v, int *__restrict__ cand_i) {
    constexpr int K = NU * 64, RB = WAVE / NU;
    __shared__ __attribute__((aligned(16))) float xs[K];
    __shared__ float red[2 * QWAVES];
    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int gw = blockIdx.x * QWAVES + wave, nwaves = gridDim.x * QWAVES;
    const int ntrips = (N + RB - 1) / RB;
    const size_t last_unit = (size_t)N * NU - 1;

    constexpr int D = 3;  // trips of a wavefront in flight (3.4 KB each)
    UnitRegs un[D];
    auto request = [&](UnitRegs &r, int trip) {
        size_t ui = (size_t)trip * WAVE + lane;
        ui = ui < last_unit ? ui : last_unit;  // units past the end re-read the last one
        r.a = ld128_stream(nib + ui * 32);
        r.b = ld128_stream(nib + ui * 32 + 16);
        r.h = ld128_stream(top + ui * 16);
        r.sc = __builtin_nontemporal_load((global_u32_ptr)(scales + ui));
        r.d = __builtin_nontemporal_load((global_u16_ptr)(ds + (ui >> 2)));
    };

    // activations first (loads return in issue order), the first trips' weights right behind them
    constexpr int XU = (K / 4 + QTHREADS - 1) / QTHREADS;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 xr[XU], nr[XU];
#pragma unroll
    for (int u = 0; u < XU; u++) {
        const int k = (tid + u * QTHREADS) * 4;
        xr[u] = k < K ? *reinterpret_cast<const f32x4 *>(x + k) : zero4;
        nr[u] = norm_w && k < K ? *reinterpret_cast<const f32x4 *>(norm_w + k) : zero4;
    }
    int trip = gw;  // the trip in buffer 0; buffer d holds trip + d * nwaves
#pragma unroll
    for (int d = 0; d < D; d++)
        if (trip + d * nwaves < ntrips) request(un[d], trip + d * nwaves);
    if (norm_w) {  // emit_rms_norm (src/graph_builder/emit_linalg.rs:7-26): (x * inv) * w
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < XU; u++) ss += (xr[u][0] * xr[u][0] + xr[u][1] * xr[u][1]) + (xr[u][2] * xr[u][2] + xr[u][3] * xr[u][3]);
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weight loads stay in flight
        float tot = 0.f;
#pragma unroll
        for (int wv = 0; wv < QWAVES; wv++) tot += red[wv];
        const float inv = 1.0f / sqrtf(tot / (float)K + eps);
#pragma unroll
        for (int u = 0; u < XU; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) xr[u][e] = (xr[u][e] * inv) * nr[u][e];
    }
#pragma unroll
    for (int u = 0; u < XU; u++) {
        const int k = (tid + u * QTHREADS) * 4;
        if (k < K) *reinterpret_cast<f32x4 *>(xs + k) = xr[u];
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // unit position ur of the row: block ur / 4, half (ur / 2) % 2, l range ur % 2; group g covers weights
    // 256 blk + 128 h + 32 g + 16 p + j
    const int ur = lane % NU;
    const int xbase = (ur >> 2) * 256 + ((ur >> 1) & 1) * 128 + (ur & 1) * 16;
    float xv[4][16], sx32[4];
#pragma unroll
    for (int g = 0; g < 4; g++) {
        float sx = 0.f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(xs + xbase + 32 * g + 4 * q);
            xv[g][4 * q] = v.x; xv[g][4 * q + 1] = v.y; xv[g][4 * q + 2] = v.z; xv[g][4 * q + 3] = v.w;
            sx += (v.x + v.y) + (v.z + v.w);
        }
        sx32[g] = 32.f * sx;
    }

    float best_v = -INFINITY;
    int best_i = -1;
    const bool writer = (lane % NU) == NU - 1;
    auto consume = [&](const UnitRegs &r, int t) {
        float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t a = r.a[i], b = r.b[i], h = r.h[i];
            s[0] = dot4_bytes((a & 0x0F0F0F0Fu) | ((h << 4) & 0x30303030u), &xv[0][4 * i], s[0]);
            s[1] = dot4_bytes((b & 0x0F0F0F0Fu) | ((h << 2) & 0x30303030u), &xv[1][4 * i], s[1]);
            s[2] = dot4_bytes(((a >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u), &xv[2][4 * i], s[2]);
            s[3] = dot4_bytes(((b >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u), &xv[3][4 * i], s[3]);
        }
        const float d = f16_bits_to_f32((uint16_t)r.d);
        float v = 0.f;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int sc = (int)(int8_t)(r.sc >> (8 * g));
            v += (d * (float)sc) * (s[g] - sx32[g]);
        }
        v = segment_sum<NU>(v);
        const int row = t * RB + lane / NU;
        if (writer && row < N) {
            out[row] = v;
            // of equal maxima the later row wins (Rust Iterator::max_by, reference src/generate.rs:735-742);
            // rows reach a lane in ascending order
            if (best_i < 0 || v >= best_v) {
                best_v = v;
                best_i = row;
            }
        }
    };
    // steady state: every buffer is multiplied and asked for again, D trips on, with no condition in the way
    while (trip + (2 * D - 1) * nwaves < ntrips) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            consume(un[d], trip + d * nwaves);
            request(un[d], trip + (D + d) * nwaves);
        }
        trip += D * nwaves;
    }
    // what the buffers still hold, each asked for again at once where a trip is left for it (at most D - 1 are)
#pragma unroll
    for (int d = 0; d < D; d++)
        if (trip + d * nwaves < ntrips) {
            consume(un[d], trip + d * nwaves);
            if (trip + (D + d) * nwaves < ntrips) request(un[d], trip + (D + d) * nwaves);
        }
    trip += D * nwaves;
#pragma unroll
    for (int d = 0; d < D; d++)
        if (trip + d * nwaves < ntrips) consume(un[d], trip + d * nwaves);

    if (cand_v) {  // the workgroup's best row: largest value, highest index among equals; -1 = no row
#pragma unroll
        for (int m = 1; m < WAVE; m <<= 1) {
            const float ov = __shfl_xor(best_v, m);
            const int oi = __shfl_xor(best_i, m);
            if (oi >= 0 && (best_i < 0 || ov > best_v || (ov == best_v && oi > best_i))) {
                best_v = ov;
                best_i = oi;
            }
        }
        __syncthreads();
        int *redi = reinterpret_cast<int *>(red) + QWAVES;
        if (lane == 0) {
            red[wave] = best_v;
            redi[wave] = best_i;
        }
        __syncthreads();
        if (tid == 0) {
            float bv = -INFINITY;
            int bi = -1;
            for (int wv = 0; wv < QWAVES; wv++) {
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

// raw blocks [N][K / 256] <-> planes; one thread per unit
template <bool UNPACK>
__global__ __launch_bounds__(256) void q6k_pack_kernel(uint8_t *__restrict__ blocks, uint8_t *__restrict__ nib, uint8_t *__restrict__ top,
                                                       uint8_t *__restrict__ scales, uint16_t *__restrict__ ds, size_t n_units) {
    const size_t ui = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (ui >= n_units) return;
    uint8_t *blk = blocks + (ui >> 2) * Q6K_BLOCK;
    const int h = (int)(ui >> 1) & 1, p = (int)ui & 1;
    uint8_t *ql = blk + 64 * h + 16 * p, *qh = blk + 128 + 32 * h + 16 * p, *sc = blk + 192 + 8 * h + p;
    uint8_t *un = nib + ui * 32, *ut = top + ui * 16, *us = scales + ui * 4;
#pragma unroll
    for (int j = 0; j < 16; j++) {
        if (UNPACK) {
            ql[j] = un[j];
            ql[32 + j] = un[16 + j];
            qh[j] = ut[j];
        } else {
            un[j] = ql[j];
            un[16 + j] = ql[32 + j];
            ut[j] = qh[j];
        }
    }
#pragma unroll
    for (int g = 0; g < 4; g++) {
        if (UNPACK)
            sc[2 * g] = us[g];
        else
            us[g] = sc[2 * g];
    }
    if ((ui & 3) == 0) {
        if (UNPACK) {
            blk[208] = (uint8_t)(ds[ui >> 2] & 0xFF);
            blk[209] = (uint8_t)(ds[ui >> 2] >> 8);
        } else {
            ds[ui >> 2] = (uint16_t)(blk[208] | (blk[209] << 8));
        }
    }
}

// One thread per element, the reference's arithmetic step by step: w = (d * sc) * q (src/gguf.rs:880-917),
// read from the planes.
__global__ __launch_bounds__(256) void q6k_dequant_planes_kernel(const uint8_t *__restrict__ nib, const uint8_t *__restrict__ top,
                                                                 const uint8_t *__restrict__ scales, const uint16_t *__restrict__ ds,
                                                                 float *__restrict__ out, size_t n_elems) {
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; e < n_elems; e += stride) {
        const size_t blk = e >> 8;
        const int j = (int)(e & 255);
        const int h = j >> 7, g = (j & 127) >> 5, l = j & 31, p = l >> 4, jj = l & 15;
        const size_t ui = blk * 4 + 2 * h + p;
        const uint8_t lb = nib[ui * 32 + 16 * (g & 1) + jj];
        const int lo = g >= 2 ? (lb >> 4) : (lb & 15);
        const int hi = (top[ui * 16 + jj] >> (2 * g)) & 3;
        const int q = (lo | (hi << 4)) - 32;
        const int sc = (int)(int8_t)scales[ui * 4 + g];
        out[e] = __fmul_rn(__fmul_rn(f16_bits_to_f32(ds[blk]), (float)sc), (float)q);
    }
}

int q6k_grid(const hm_ctx *ctx, int K, int N, int cand_cap) {
    const int rb = WAVE / (K / 64);
    const int ntrips = (N + rb - 1) / rb;
    const int want = (ntrips + QWAVES - 1) / QWAVES;
    int grid = std::min(want, 4 * ctx->num_cus);
    if (cand_cap > 0 && grid > cand_cap) grid = cand_cap;
    return grid < 1 ? 1 : grid;
}

}  // namespace

bool homura::q6k_planes_shape_ok(int N, int K) {
    return N > 0 && (K == 256 || K == 512 || K == 1024 || K == 2048 || K == 4096);
}

size_t homura::q6k_planes_bytes(int N, int K) { return q6k_planes_layout(N, K).bytes; }

int homura::q6k_planes_workgroups(const hm_ctx *ctx, int K, int N, int cand_cap) { return q6k_grid(ctx, K, N, cand_cap); }

int homura::pack_q6k_planes(hm_ctx *ctx, const uint8_t *d_blocks, uint8_t *d_planes, int N, int K, bool unpack) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_blocks && d_planes, "q6_k planes: NULL pointer");
    HM_REQUIRE(ctx, N > 0 && K > 0 && K % 256 == 0, "q6_k planes: K=%d must be a positive multiple of 256, N=%d positive", K, N);
    HM_REQUIRE(ctx, ((uintptr_t)d_planes % 16) == 0, "q6_k planes: the planes must be 16-byte aligned");
    const Q6kPlanes p = q6k_planes_layout(N, K);
    const size_t units = (size_t)N * (K / 64);
    const unsigned grid = (unsigned)((units + 255) / 256);
    uint8_t *blocks = const_cast<uint8_t *>(d_blocks);
    if (unpack)
        hipLaunchKernelGGL((q6k_pack_kernel<true>), dim3(grid), dim3(256), 0, ctx->stream, blocks, d_planes, d_planes + p.top_off,
                           d_planes + p.scale_off, reinterpret_cast<uint16_t *>(d_planes + p.d_off), units);
    else
        hipLaunchKernelGGL((q6k_pack_kernel<false>), dim3(grid), dim3(256), 0, ctx->stream, blocks, d_planes, d_planes + p.top_off,
                           d_planes + p.scale_off, reinterpret_cast<uint16_t *>(d_planes + p.d_off), units);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int homura::dequant_q6k_planes(hm_ctx *ctx, const uint8_t *d_planes, float *d_out, int N, int K) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_planes && d_out && N > 0 && K > 0 && K % 256 == 0, "q6_k planes: bad arguments");
    const Q6kPlanes p = q6k_planes_layout(N, K);
    const size_t n = (size_t)N * K;
    size_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(q6k_dequant_planes_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, d_planes, d_planes + p.top_off,
                       d_planes + p.scale_off, reinterpret_cast<const uint16_t *>(d_planes + p.d_off), d_out, n);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int homura::gemv_q6k_planes_f32(hm_ctx *ctx, const char *name, const float *d_x, const float *d_norm_w, float eps,
                                const uint8_t *d_planes, float *d_out, int M, int K, int N, float *cand_v, int *cand_i, int cand_cap) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x && d_planes && d_out, "%s: NULL pointer", name);
    HM_REQUIRE(ctx, M >= 1 && M <= 8, "%s: M=%d outside 1..8", name, M);
    HM_REQUIRE(ctx, q6k_planes_shape_ok(N, K), "%s: K=%d must be 256, 512, 1024, 2048 or 4096, N=%d positive", name, K, N);
    HM_REQUIRE(ctx, ((uintptr_t)d_planes % 16) == 0 && ((uintptr_t)d_x % 16) == 0 && ((uintptr_t)d_norm_w % 16) == 0,
               "%s: weight, activation and norm buffers must be 16-byte aligned", name);
    HM_REQUIRE(ctx, !cand_v || (cand_i && M == 1), "%s: argmax candidates need an index buffer and M == 1", name);
    const Q6kPlanes p = q6k_planes_layout(N, K);
    const int grid = q6k_grid(ctx, K, N, cand_v ? cand_cap : 0);
    const uint8_t *top = d_planes + p.top_off;
    const uint32_t *sc = reinterpret_cast<const uint32_t *>(d_planes + p.scale_off);
    const uint16_t *ds = reinterpret_cast<const uint16_t *>(d_planes + p.d_off);
    for (int m = 0; m < M; m++) {
        const float *xm = d_x + (size_t)m * K;
        float *om = d_out + (size_t)m * N;
#define HM_Q6(NU)                                                                                                            \
    hipLaunchKernelGGL((gemv_q6k_units_kernel<NU>), dim3(grid), dim3(QTHREADS), 0, ctx->stream, xm, d_norm_w, eps, d_planes, top, \
                       sc, ds, om, N, cand_v, cand_i)
        switch (K / 64) {
        case 4: HM_Q6(4); break;
        case 8: HM_Q6(8); break;
        case 16: HM_Q6(16); break;
        case 32: HM_Q6(32); break;
        default: HM_Q6(64); break;
        }
#undef HM_Q6
        HM_LAUNCH_CHECK(ctx);
    }
    return HM_OK;
}
