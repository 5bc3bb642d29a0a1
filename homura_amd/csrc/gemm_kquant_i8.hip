// Q8_K rows x K-quant matrix on the int8 matrix cores (see gemm_kquant_i8.h for the formats).
//
// Workgroup tile 128 (rows of A) x 128 (rows of the weight matrix), eight wavefronts of 64 x 32 = 2 x 1
// `v_mfma_i32_32x32x32_i8` tiles, two per SIMD, so that one wavefront's matrix instructions run under the
// other's block arithmetic. A stage is 64 bytes of k for the four operand tiles (the
// activations and the three digit planes, 8 KiB each), moved global -> LDS directly
// (global_load_lds_dwordx4, rows XOR-swizzled on the global side as in gemm_pieces_mfma.hip); four stages
// rotate through LDS, one barrier per stage. Four stages are one 256-wide block: its three integer sums are
// exact, and its value joins the f32 sums with the arithmetic of the decode kernels (gemv_kquant.hip).
// The scales of the workgroup's rows and of its slice of K wait in LDS from the start.
#include "gemm_kquant_i8.h"

#include <algorithm>

#include "quant_formats.h"

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TM = 128, TN = 128;
constexpr int ROW_BYTES = 64;                   // bytes (= values) of k per stage and row
constexpr int TILE = TM * ROW_BYTES;            // 8 KiB: one operand tile of a stage
constexpr int T = 4;                            // tiles per stage: activations, hi, lo, mn
constexpr int STAGE = T * TILE;                 // 32 KiB
constexpr int NB = 4;                           // stages in LDS
constexpr int THREADS = 512;
constexpr int MAXB = 16;                        // 256-wide blocks of a K slice whose scales fit in LDS
constexpr int SC_A = MAXB * TM * 4, SC_W = MAXB * TN * 8;
constexpr int LDS_BYTES = NB * STAGE + SC_A + SC_W;  // 155648
constexpr int DMA_PER_STAGE = T;                // instructions a wavefront issues per stage

struct I8Dims {
    int M, N, K, ldc;
    int blocks_per_split;
};

__device__ __forceinline__ int lds_off(int r, int chunk) { return r * ROW_BYTES + ((chunk ^ ((r >> 2) & 3)) << 4); }

__device__ __forceinline__ void dma16(const int8_t *src, char *dst) {
    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)src,
                                     (void __attribute__((address_space(3))) *)dst, 16, 0, 0);
}

// The compiler does not see when an asm load's registers are written: every use of them is behind one of
// the waits below that names them ("+v"), and they are not touched in between.
__device__ __forceinline__ i32x4 lds_read16(uint32_t addr) {
    i32x4 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}

extern __shared__ __attribute__((aligned(16))) char i8_lds[];

__global__ __launch_bounds__(THREADS) void gemm_q8k_kquant_kernel(const int8_t *__restrict__ A,
                                                                  const float *__restrict__ Asc,
                                                                  const int8_t *__restrict__ P,
                                                                  const float *__restrict__ Wsc, float *__restrict__ C,
                                                                  const I8Dims g) {
    const int M = g.M, N = g.N, K = g.K, KB = K / 256;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 2, wn = wave & 3;  // rows wm * 64 .. + 63, columns wn * 32 .. + 31 of the tile
    const int l32 = lane & 31, lh = lane >> 5;

    const int mb = (M + TM - 1) / TM, total = gridDim.x;
    int lin = blockIdx.x;
    if ((total & 7) == 0) lin = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);  // neighbours share a die's L2
    const int m0 = (lin % mb) * TM, n0 = (lin / mb) * TN;

    const int b_first = blockIdx.y * g.blocks_per_split;
    const int nblk = min(g.blocks_per_split, KB - b_first);
    C += (size_t)blockIdx.y * M * g.ldc;

    // scales of this tile's rows for the slice's blocks: asc[blk][128], wsc[blk][128][2]
    float *asc = reinterpret_cast<float *>(i8_lds + NB * STAGE);
    float *wsc = reinterpret_cast<float *>(i8_lds + NB * STAGE + SC_A);
    for (int idx = tid; idx < nblk * TM; idx += THREADS) {
        const int blk = idx / TM, r = idx % TM;
        asc[idx] = Asc[(size_t)min(m0 + r, M - 1) * KB + b_first + blk];
        const float2 dd = *reinterpret_cast<const float2 *>(Wsc + ((size_t)min(n0 + r, N - 1) * KB + b_first + blk) * 2);
        wsc[idx * 2] = dd.x;
        wsc[idx * 2 + 1] = dd.y;
    }
    __syncthreads();  // (every load above has returned: the wait counts below see the tile loads only)

    // Wavefront w fills rows 16 w .. 16 w + 15 of every tile of a stage, one instruction per tile.
    const int8_t *a_src, *p_src;
    {
        const int r = wave * 16 + (lane >> 2), s = lane & 3;
        const int c = s ^ ((r >> 2) & 3);
        a_src = A + (size_t)min(m0 + r, M - 1) * K + c * 16;
        p_src = P + (size_t)min(n0 + r, N - 1) * K + c * 16;
    }
    const size_t plane = (size_t)N * K;
    const int wave_dst = __builtin_amdgcn_readfirstlane(wave * 16 * ROW_BYTES);
    const int k_end = (b_first + nblk) * 256;
    int k_req = b_first * 256;
    // a stage past the end re-reads the last one (nobody multiplies it): the wait counts stay exact
    auto request = [&](int buf) {
        char *base = i8_lds + buf * STAGE + wave_dst;
        const int k = min(k_req, k_end - ROW_BYTES);
        dma16(a_src + k, base);
#pragma unroll
        for (int p = 0; p < 3; p++) dma16(p_src + p * plane + k, base + (1 + p) * TILE);
        k_req += ROW_BYTES;
    };
#pragma unroll
    for (int d = 0; d < NB; d++) request(d);

    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)i8_lds;
    // operand addresses inside a stage: k step ks takes 16-byte chunks 2 ks (lanes 0-31) and 2 ks + 1
    uint32_t a_off[2][2], b_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
#pragma unroll
        for (int i = 0; i < 2; i++) a_off[ks][i] = lds0 + lds_off(wm * 64 + i * 32 + l32, ks * 2 + lh);
        b_off[ks] = lds0 + TILE + lds_off(wn * 32 + l32, ks * 2 + lh);
    }
    // operand registers of a whole stage, two sets: the next stage's reads are in flight during the MFMAs
    i32x4 fa[2][2][2], fb[2][3][2];
    auto read_stage = [&](int set, int buf) {
        const uint32_t off = (uint32_t)(buf * STAGE);
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
#pragma unroll
            for (int i = 0; i < 2; i++) fa[set][ks][i] = lds_read16(a_off[ks][i] + off);
#pragma unroll
            for (int p = 0; p < 3; p++) fb[set][p][ks] = lds_read16(b_off[ks] + off + p * TILE);
        }
    };
    // Wait for every LDS read issued so far (operand set SET among them) and for all tile loads except
    // those of the youngest NB - 2 stages, then meet the other wavefronts.
#define HM_I8_WAIT(CNT, SET)                                                                                          \
    asm volatile("s_waitcnt vmcnt(" #CNT ") lgkmcnt(0)\n\ts_barrier"                                                   \
                 : "+v"(fa[SET][0][0]), "+v"(fa[SET][0][1]), "+v"(fa[SET][1][0]), "+v"(fa[SET][1][1]),                \
                   "+v"(fb[SET][0][0]), "+v"(fb[SET][0][1]), "+v"(fb[SET][1][0]), "+v"(fb[SET][1][1]),                \
                   "+v"(fb[SET][2][0]), "+v"(fb[SET][2][1])                                                           \
                 :                                                                                                    \
                 : "memory")
    static_assert((NB - 2) * DMA_PER_STAGE == 8, "wait count");

    i32x16 acc_i[3][2];   // the block's integer sums per plane
    f32x16 acc[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0.f;

    auto multiply = [&](int set, bool first) {
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int p = 0; p < 3; p++)
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    i32x16 c = acc_i[p][i];
                    if (first && ks == 0) {
#pragma unroll
                        for (int v = 0; v < 16; v++) c[v] = 0;
                    }
                    acc_i[p][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][ks][i], fb[set][p][ks], c, 0, 0, 0);
                }
    };

    int buf = 0;  // stage s sits in buffer s % NB
    auto stage = [&](int set, bool first) {
        if (set == 0) HM_I8_WAIT(8, 0); else HM_I8_WAIT(8, 1);
        const int nbuf = buf + 1 == NB ? 0 : buf + 1;
        request(buf);
        read_stage(set ^ 1, nbuf);
        multiply(set, first);
        __builtin_amdgcn_sched_barrier(0);
        buf = nbuf;
    };

    // stage 0 has landed for everyone (NB - 1 stages may be in flight)
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NB - 1) * DMA_PER_STAGE) : "memory");
    read_stage(0, 0);
    for (int blk = 0; blk < nblk; blk++) {
        stage(0, true);
        stage(1, false);
        stage(0, false);
        stage(1, false);
        // the block's value: (d a) float(128 S_hi + S_lo) - (dmin a) float(S_mn), each operation rounded once
        const float *ab = asc + blk * TM + wm * 64 + lh * 4;
        const float *wb = wsc + (blk * TN + wn * 32 + l32) * 2;
        const float d = wb[0], dmin = wb[1];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int gq = 0; gq < 4; gq++) {
                const f32x4 a4 = *reinterpret_cast<const f32x4 *>(ab + i * 32 + gq * 8);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int v = gq * 4 + e;
                    const float fs = (float)(acc_i[0][i][v] * 128 + acc_i[1][i][v]);
                    const float fm = (float)acc_i[2][i][v];
                    const float part = __fsub_rn(__fmul_rn(__fmul_rn(d, a4[e]), fs), __fmul_rn(__fmul_rn(dmin, a4[e]), fm));
                    acc[i][v] = __fadd_rn(acc[i][v], part);
                }
            }
    }
    // drain what is in flight (tile loads of the stages past the end, the operand reads that target set 0)
    HM_I8_WAIT(0, 0);
#undef HM_I8_WAIT

    // accumulator element v of lane l sits at row (v / 4) * 8 + (l / 32) * 4 + v % 4, column l % 32
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int row = m0 + wm * 64 + i * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
            const int col = n0 + wn * 32 + l32;
            if (row < M && col < N) __builtin_nontemporal_store(acc[i][v], C + (size_t)row * g.ldc + col);
        }
}

// get_scale_min_k4 (reference src/gguf.rs:847-862)
__device__ __forceinline__ void q4k_scale_min(const uint8_t *raw, int j, int &sc, int &mn) {
    if (j < 4) {
        sc = raw[j] & 0x3F;
        mn = raw[4 + j] & 0x3F;
    } else {
        sc = (raw[4 + j] & 0x0F) | ((raw[j - 4] >> 6) << 4);
        mn = (raw[4 + j] >> 4) | ((raw[j] >> 6) << 4);
    }
}

// one thread per (row, 16 weights): the digits of sc * q and the minimum factor, 16 bytes per plane
__global__ __launch_bounds__(256) void kq_i8_pack_kernel(const uint8_t *__restrict__ blocks, int q6, int rows, int K,
                                                         int8_t *__restrict__ planes, float *__restrict__ scales,
                                                         int N_total, int row_mult, int row_off) {
    const int per_row = K / 16;
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (size_t)rows * per_row) return;
    const int r = (int)(id / per_row), s = (int)(id % per_row), b = s / 16, t = s % 16;
    const uint8_t *blk = blocks + ((size_t)r * (K / 256) + b) * (q6 ? 210 : 144);
    const size_t orow = (size_t)r * row_mult + row_off;
    int q[16], sc, mn;
    if (q6) {
        // reference dequant_q6_k (src/gguf.rs:886-917): weight w = 128 chunk + 32 grp + l
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int w = t * 16 + e, chunk = w / 128, rr = w % 128, l = rr % 32, grp = rr / 32;
            const uint8_t ql = blk[chunk * 64 + (grp & 1) * 32 + l];
            const int lo = grp >= 2 ? (ql >> 4) : (ql & 0x0F);
            const int hi = (blk[128 + chunk * 32 + l] >> (2 * grp)) & 3;
            q[e] = (lo | (hi << 4)) - 32;
        }
        sc = (int8_t)blk[192 + t];
        mn = 0;
    } else {
        // reference dequant_q4_k (src/gguf.rs:835-882): pairs of 32-wide sub-blocks share 32 bytes, even = low nibbles
        const uint8_t *qs = blk + 16;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int w = t * 16 + e, pair = w / 64, within = w % 64;
            const uint8_t byte = qs[pair * 32 + within % 32];
            q[e] = within < 32 ? (byte & 0x0F) : (byte >> 4);
        }
        q4k_scale_min(blk + 4, t / 2, sc, mn);
    }
    uint32_t hi4[4], lo4[4], mn4[4];
#pragma unroll
    for (int w4 = 0; w4 < 4; w4++) {
        hi4[w4] = lo4[w4] = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int wv = sc * q[w4 * 4 + e];
            const int lo = ((wv + 64) & 127) - 64;
            const int hi = (wv - lo) / 128;
            hi4[w4] |= (uint32_t)(hi & 0xFF) << (8 * e);
            lo4[w4] |= (uint32_t)(lo & 0xFF) << (8 * e);
        }
        mn4[w4] = (uint32_t)mn * 0x01010101u;
    }
    const size_t plane = (size_t)N_total * K;
    int8_t *o = planes + orow * K + (size_t)s * 16;
    *reinterpret_cast<u32x4 *>(o) = u32x4{hi4[0], hi4[1], hi4[2], hi4[3]};
    *reinterpret_cast<u32x4 *>(o + plane) = u32x4{lo4[0], lo4[1], lo4[2], lo4[3]};
    *reinterpret_cast<u32x4 *>(o + 2 * plane) = u32x4{mn4[0], mn4[1], mn4[2], mn4[3]};
    if (t == 0) {
        float *dd = scales + (orow * (K / 256) + b) * 2;
        if (q6) {
            dd[0] = f16_bits_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
            dd[1] = 0.f;
        } else {
            dd[0] = f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
            dd[1] = f16_bits_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
        }
    }
}

// a wavefront per 256-wide block, four consecutive values per lane (reference quantize_row_q8_k,
// src/graph_builder/emit_quant.rs:422-466)
__global__ __launch_bounds__(256) void quantize_q8k_rows_kernel(const float *__restrict__ x, int8_t *__restrict__ q,
                                                                float *__restrict__ scale, size_t n) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= n) return;
    const f32x4 v = *reinterpret_cast<const f32x4 *>(x + i);
    float d;
    const uint32_t packed = homura::q8k_quantize4(v, d);
    *reinterpret_cast<uint32_t *>(q + i) = packed;
    if ((threadIdx.x & 63) == 0) scale[i / 256] = d;
}

}  // namespace

namespace homura {

int kq_i8_pack(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int rows, int K, int8_t *d_planes, float *d_scales,
               int N_total, int row_mult, int row_off) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, hm_dtype == HM_DTYPE_Q4_K || hm_dtype == HM_DTYPE_Q6_K, "kq_i8_pack: dtype %d is not a K-quant", hm_dtype);
    HM_REQUIRE(ctx, d_blocks && d_planes && d_scales && rows > 0 && K > 0 && K % 256 == 0 && row_mult >= 1 && row_off >= 0 &&
                        row_off < row_mult && (size_t)(rows - 1) * row_mult + row_off < (size_t)N_total,
               "kq_i8_pack: bad arguments (rows=%d K=%d N=%d)", rows, K, N_total);
    HM_REQUIRE(ctx, ((uintptr_t)d_planes % 16) == 0 && ((uintptr_t)d_scales % 8) == 0, "kq_i8_pack: misaligned output");
    const size_t total = (size_t)rows * (K / 16);
    hipLaunchKernelGGL(kq_i8_pack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, d_blocks,
                       hm_dtype == HM_DTYPE_Q6_K ? 1 : 0, rows, K, d_planes, d_scales, N_total, row_mult, row_off);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int quantize_q8k_rows_launch(hm_ctx *ctx, const float *d_x, int8_t *d_q, float *d_scale, size_t rows, int dim) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x && d_q && d_scale && rows > 0 && dim > 0 && dim % 256 == 0, "quantize_q8k_rows: bad arguments (dim=%d)", dim);
    HM_REQUIRE(ctx, ((uintptr_t)d_x % 16) == 0 && ((uintptr_t)d_q % 4) == 0, "quantize_q8k_rows: misaligned buffer");
    const size_t n = rows * dim;
    HM_REQUIRE(ctx, (n / 4 + 255) / 256 <= 0x7fffffffULL, "quantize_q8k_rows: too many elements");
    hipLaunchKernelGGL(quantize_q8k_rows_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, ctx->stream, d_x, d_q,
                       d_scale, n);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int gemm_q8k_kquant_nk(hm_ctx *ctx, const int8_t *d_aq, const float *d_ascale, const int8_t *d_planes,
                       const float *d_scales, float *d_c, int M, int K, int N, int max_parts, int *parts, int ldc) {
    const char *who = "gemm_q8k_kquant_nk";
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_aq && d_ascale && d_planes && d_scales && d_c, "%s: NULL pointer", who);
    HM_REQUIRE(ctx, M > 0 && N > 0 && K > 0 && K % 256 == 0, "%s: need M, N > 0 and K %% 256 == 0 (M=%d K=%d N=%d)", who, M, K, N);
    HM_REQUIRE(ctx, ((uintptr_t)d_aq % 16) == 0 && ((uintptr_t)d_planes % 16) == 0 && ((uintptr_t)d_scales % 8) == 0,
               "%s: operands must be 16-byte aligned", who);
    const long long tiles = (long long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    HM_REQUIRE(ctx, tiles <= 0x7fffffffLL, "%s: too many tiles", who);
    I8Dims g;
    g.M = M;
    g.N = N;
    g.K = K;
    g.ldc = ldc > 0 ? ldc : N;
    HM_REQUIRE(ctx, g.ldc >= N, "%s: ldc %d below N %d", who, g.ldc, N);
    // K slices of whole blocks while they still add whole waves of workgroups to a grid smaller than the chip;
    // a slice's scales must fit their LDS tables
    const int KB = K / 256;
    int want = (int)std::max<long long>(1, ctx->num_cus / tiles);
    want = std::min(std::min(want, std::max(1, max_parts)), KB);
    if (!parts) want = 1;
    g.blocks_per_split = (KB + want - 1) / want;
    HM_REQUIRE(ctx, g.blocks_per_split <= MAXB, "%s: K = %d needs %d K slices (%d allowed)", who, K, (KB + MAXB - 1) / MAXB,
               parts ? max_parts : 1);
    const int slices = (KB + g.blocks_per_split - 1) / g.blocks_per_split;
    if (parts) *parts = slices;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q8k_kquant_kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    HM_REQUIRE(ctx, attr == hipSuccess, "%s: cannot reserve %d bytes of LDS: %s", who, LDS_BYTES, hipGetErrorString(attr));
    hipLaunchKernelGGL(gemm_q8k_kquant_kernel, dim3((unsigned)tiles, (unsigned)slices), dim3(THREADS), LDS_BYTES, ctx->stream,
                       d_aq, d_ascale, d_planes, d_scales, d_c, g);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // namespace homura
