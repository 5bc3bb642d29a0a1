// MFMA GEMM for operands carried as bf16 pieces (see prefill.h): C[M][N] f32 = (sum of A's pieces) x
// (sum of B's pieces)^T, A [M][AP Kb], B [N][BP Kb] (piece p in columns [p Kb, (p+1) Kb)).
//
// The plain kernel of gemm_bf16_mfma.hip runs one pass over K per product of pieces and loads a B tile
// again for every A piece. It is bound by what a CU can pull into LDS (about half of its 64 B/clk;
// the MFMAs of a tile take 40 % of the time the loads do), so this kernel loads every tile once: a
// stage holds the tiles of all pieces for 32 values of k, and every product that matters is taken from
// them: the AP products with a single B (bf16 weights), or the six products (a, b), a + b <= 2, of
// two three-piece operands (f32 x f32 up to 2^-24). Per product that is a third less (AP = 3, BP = 1)
// or half (AP = BP = 3) of the bytes, and the operand reads out of LDS shrink the same way.
//
// Workgroup tile 128 x 128, eight wavefronts as two k groups of 2 x 2 (group g takes k step g of the
// two in a stage), `mfma_f32_32x32x16_bf16`, tiles go global -> LDS directly (global_load_lds_dwordx4:
// lane l's 16 bytes land at base + 16 l, so an instruction fills sixteen 64-byte rows; the lane that
// fills slot s of row r fetches chunk s ^ ((r >> 2) & 3), which makes the operand reads conflict
// free). NB stages rotate through LDS (128 to 144 KiB), one barrier per stage. M, N ragged as in the
// other kernel; K slices (grid.y) write partial sums the consumer adds in index order.
//
// SC (block-scaled B): B holds the integers of a Q8_0 / Q4_0 matrix as bf16 (exact) and every 32-wide block
// of a row has an f32 scale, scales[k / 32][n] (row stride npad, a multiple of 128). A stage is exactly one
// block: its AP products are summed on their own and join the result times the block's scale, d * sum(x q),
// the decode kernels' form of the reference's sum(x (d q)) (src/hf/emitter_quant.rs:675-702). The 128 scales
// of a stage travel with its tiles (64 bytes per wavefront).
#include <algorithm>
#include <type_traits>

#include "gemm_bf16_mfma.h"
#include "hm_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TM = 128, TN = 128, TK = 32;
constexpr int ROW_BYTES = TK * 2;               // 64
constexpr int PIECE_TILE = TM * ROW_BYTES;      // 8 KiB: one piece of one operand for one stage
constexpr int THREADS = 512;

struct PieceDims {
    int M, N, Kb, lda, ldb, ldc;
    int stages_per_split;  // stages of 32 k per grid.y slice
    const float *scales;   // SC: [Kb / 32][npad]
    int npad;
};

__device__ __forceinline__ int lds_off(int r, int chunk) { return r * ROW_BYTES + ((chunk ^ ((r >> 2) & 3)) << 4); }

__device__ __forceinline__ void dma16(const uint16_t *src, char *dst) {
    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)src,
                                     (void __attribute__((address_space(3))) *)dst, 16, 0, 0);
}

// The compiler does not see when an asm load's registers are written: every use of them is behind one of
// the waits below that names them ("+v"), and they are not touched in between.
__device__ __forceinline__ bf16x8 lds_read16(uint32_t addr) {
    bf16x8 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
__device__ __forceinline__ float lds_read4(uint32_t addr) {
    float v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}

extern __shared__ __attribute__((aligned(16))) char stage_lds[];

template <int AP, int BP, bool SC = false>
struct Shape {
    static constexpr int TILES = AP + BP;                   // operand tiles per stage
    static constexpr int T = TILES + (SC ? 1 : 0);          // loads per wavefront and stage
    static constexpr int STAGE = TILES * PIECE_TILE + (SC ? TN * 4 : 0);  // bytes
    static constexpr int NB = TILES * PIECE_TILE <= 32 * 1024 ? 4 : 3;    // stages in LDS
    static constexpr int LDS = NB * STAGE > 64 * 1024 ? NB * STAGE : 64 * 1024;  // the final exchange wants 64 KiB
};

template <int AP, int BP, bool SC = false>
__global__ __launch_bounds__(THREADS) void gemm_pieces_kernel(const uint16_t *__restrict__ A,
                                                              const uint16_t *__restrict__ B, float *__restrict__ C,
                                                              const PieceDims g) {
    using S = Shape<AP, BP, SC>;
    constexpr int T = S::T, NB = S::NB, STAGE = S::STAGE;
    static_assert(!SC || BP == 1, "block scales go with a single B operand");
    const int M = g.M, N = g.N;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kgrp = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    // XCD-aware tile order, as in the other kernel
    const int mb = (M + TM - 1) / TM, total = gridDim.x;
    int lin = blockIdx.x;
    if ((total & 7) == 0) lin = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
    const int m0 = (lin % mb) * TM, n0 = (lin / mb) * TN;

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    const int s_first = blockIdx.y * g.stages_per_split;
    const int ns = min(g.stages_per_split, g.Kb / TK - s_first);
    C += (size_t)blockIdx.y * M * g.ldc;

    // Wavefront w fills rows 16 w .. 16 w + 15 of every tile of a stage, one instruction per tile.
    const uint16_t *a_src, *b_src;
    {
        const int r = wave * 16 + (lane >> 2), s = lane & 3;
        const int c = s ^ ((r >> 2) & 3);
        a_src = A + (size_t)min(m0 + r, M - 1) * g.lda + c * 8;
        b_src = B + (size_t)min(n0 + r, N - 1) * g.ldb + c * 8;
    }
    const int wave_dst = __builtin_amdgcn_readfirstlane(wave * 1024);
    const int wave_dst64 = __builtin_amdgcn_readfirstlane(wave * 64);
    const float *s_src = SC ? g.scales + n0 + wave * 16 + (lane & 3) * 4 : nullptr;  // (n0 + 127 < npad)
    int k_req = s_first * TK;  // k of the next stage to request
    // a stage past the end re-reads the last one (nobody multiplies it): the wait counts stay exact
    auto request = [&](int buf) {
        char *base = stage_lds + buf * STAGE + wave_dst;
        const int k = min(k_req, g.Kb - TK);
#pragma unroll
        for (int p = 0; p < AP; p++) dma16(a_src + p * g.Kb + k, base + p * PIECE_TILE);
#pragma unroll
        for (int p = 0; p < BP; p++) dma16(b_src + p * g.Kb + k, base + (AP + p) * PIECE_TILE);
        if (SC && lane < 4)  // this wavefront's 16 of the stage's 128 block scales
            dma16(reinterpret_cast<const uint16_t *>(s_src + (size_t)(k / TK) * g.npad),
                  stage_lds + buf * STAGE + S::TILES * PIECE_TILE + wave_dst64);
        k_req += TK;
    };
#pragma unroll
    for (int d = 0; d < NB; d++) request(d);

    // this lane's operand addresses inside a stage: piece tiles are PIECE_TILE apart
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)stage_lds;
    const int chunk = kgrp * 2 + lh;  // k step kgrp of the stage, 8 k per half-wavefront
    uint32_t a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        a_off[i] = lds0 + lds_off(wm * 64 + i * 32 + l32, chunk);
        b_off[i] = lds0 + AP * PIECE_TILE + lds_off(wn * 64 + i * 32 + l32, chunk);
    }
    // operand registers, two sets: the reads of the next stage are in flight during the MFMAs
    bf16x8 fa[2][AP][2], fb[2][BP][2];
    float fs[2][2];  // SC: the block scales of this lane's two columns
    const uint32_t s_off = lds0 + S::TILES * PIECE_TILE + (wn * 64 + l32) * 4;
    auto read_stage = [&](int set, int buf) {
        const uint32_t off = (uint32_t)(buf * STAGE);
        if (SC) {
#pragma unroll
            for (int j = 0; j < 2; j++) fs[set][j] = lds_read4(s_off + off + j * 128);
        }
#pragma unroll
        for (int p = 0; p < AP; p++)
#pragma unroll
            for (int i = 0; i < 2; i++) fa[set][p][i] = lds_read16(a_off[i] + off + p * PIECE_TILE);
#pragma unroll
        for (int p = 0; p < BP; p++)
#pragma unroll
            for (int i = 0; i < 2; i++) fb[set][p][i] = lds_read16(b_off[i] + off + p * PIECE_TILE);
    };
    // Wait for every LDS read issued so far (the operand set `set` among them; the statement names its
    // registers so that nothing touches them before the data is there) and for all loads except the
    // youngest (NB - 2) T (DRAIN: for all of them), then meet the other wavefronts.
#define HM_PIECES_WAIT(CNT, SET)                                                                                    \
    do {                                                                                                            \
        if constexpr (SC)                                                                                           \
            asm volatile("s_waitcnt vmcnt(" #CNT ") lgkmcnt(0)\n\ts_barrier"                                        \
                         : "+v"(fa[SET][0][0]), "+v"(fa[SET][0][1]), "+v"(fa[SET][1][0]), "+v"(fa[SET][1][1]),      \
                           "+v"(fa[SET][2][0]), "+v"(fa[SET][2][1]), "+v"(fb[SET][0][0]), "+v"(fb[SET][0][1]),      \
                           "+v"(fs[SET][0]), "+v"(fs[SET][1])                                                       \
                         :                                                                                          \
                         : "memory");                                                                               \
        else if constexpr (AP == 3 && BP == 3)                                                                      \
            asm volatile("s_waitcnt vmcnt(" #CNT ") lgkmcnt(0)\n\ts_barrier"                                        \
                         : "+v"(fa[SET][0][0]), "+v"(fa[SET][0][1]), "+v"(fa[SET][1][0]), "+v"(fa[SET][1][1]),      \
                           "+v"(fa[SET][2][0]), "+v"(fa[SET][2][1]), "+v"(fb[SET][0][0]), "+v"(fb[SET][0][1]),      \
                           "+v"(fb[SET][1][0]), "+v"(fb[SET][1][1]), "+v"(fb[SET][2][0]), "+v"(fb[SET][2][1])       \
                         :                                                                                          \
                         : "memory");                                                                               \
        else if constexpr (AP == 3)                                                                                 \
            asm volatile("s_waitcnt vmcnt(" #CNT ") lgkmcnt(0)\n\ts_barrier"                                        \
                         : "+v"(fa[SET][0][0]), "+v"(fa[SET][0][1]), "+v"(fa[SET][1][0]), "+v"(fa[SET][1][1]),      \
                           "+v"(fa[SET][2][0]), "+v"(fa[SET][2][1]), "+v"(fb[SET][0][0]), "+v"(fb[SET][0][1])       \
                         :                                                                                          \
                         : "memory");                                                                               \
        else                                                                                                        \
            asm volatile("s_waitcnt vmcnt(" #CNT ") lgkmcnt(0)\n\ts_barrier"                                        \
                         : "+v"(fa[SET][0][0]), "+v"(fa[SET][0][1]), "+v"(fa[SET][1][0]), "+v"(fa[SET][1][1]),      \
                           "+v"(fb[SET][0][0]), "+v"(fb[SET][0][1])                                                 \
                         :                                                                                          \
                         : "memory");                                                                               \
    } while (0)
    // (NB - 2) T: 3 x 1 pieces 8, 2 x 1 pieces 6, 3 x 3 pieces 6
    static_assert(!SC || (AP == 3 && (NB - 2) * T == 10), "wait count");
    static_assert(SC || (AP == 3 && BP == 1 && (NB - 2) * T == 8) || (AP != 3 || BP != 1), "wait count");
    static_assert(SC || ((AP == 2 || BP == 3) && (NB - 2) * T == 6) || (AP == 3 && BP == 1), "wait count");
    auto wait_and_meet = [&](int set) {
        if (set == 0) {
            if constexpr (SC) HM_PIECES_WAIT(10, 0); else if constexpr (AP == 3 && BP == 1) HM_PIECES_WAIT(8, 0); else HM_PIECES_WAIT(6, 0);
        } else {
            if constexpr (SC) HM_PIECES_WAIT(10, 1); else if constexpr (AP == 3 && BP == 1) HM_PIECES_WAIT(8, 1); else HM_PIECES_WAIT(6, 1);
        }
    };
    // the products of one stage: smallest pieces first
    auto multiply = [&](int set) {
        if constexpr (SC) {
            // the block's sum on its own (smallest pieces first), then times the block's scale
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    f32x16 t;
#pragma unroll
                    for (int v = 0; v < 16; v++) t[v] = 0.f;
#pragma unroll
                    for (int pa = AP - 1; pa >= 0; pa--)
                        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][pa][i], fb[set][0][j], t, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[i][j][v] = fmaf(t[v], fs[set][j], acc[i][j][v]);
                }
            return;
        }
#pragma unroll
        for (int order = AP + BP - 2; order >= 0; order--)
#pragma unroll
            for (int pa = AP - 1; pa >= 0; pa--) {
                const int pb = order - pa;
                if (pb < 0 || pb >= BP || (BP > 1 && order > 2)) continue;
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][pa][i], fb[set][pb][j], acc[i][j], 0, 0, 0);
            }
    };

    // stage 0 has landed for everyone (NB - 1 stages of T loads may be in flight)
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NB - 1) * T) : "memory");
    read_stage(0, 0);
    int buf = 0;  // stage s sits in buffer s % NB
    // One stage: its operands (set `set`) were requested from LDS during the previous stage. After the
    // barrier everyone holds this stage's operands in registers and the next stage has landed for
    // everyone, so this stage's buffer takes stage s + NB and the next stage's operands are read while
    // this stage's MFMAs run.
    auto stage = [&](int set, bool live) {
        wait_and_meet(set);
        const int nbuf = buf + 1 == NB ? 0 : buf + 1;
        request(buf);
        read_stage(set ^ 1, nbuf);
        if (live) multiply(set);
        __builtin_amdgcn_sched_barrier(0);
        buf = nbuf;
    };
    for (int s = 0; s < ns; s += 2) {
        stage(0, true);
        stage(1, s + 1 < ns);  // workgroup-uniform; a dead stage keeps the rhythm of loads and barriers
    }

    // drain what is in flight before the buffers are reused: loads into LDS, and the operand reads of
    // the stage after the last, which target set 0 (the wait names it, so its registers stay untouched
    // until the data has arrived). Then the second k group hands its sums over through LDS (64 KiB = 4
    // wavefronts x 64 x 64 floats, lane-major).
    HM_PIECES_WAIT(0, 0);
#undef HM_PIECES_WAIT
    float *xch = reinterpret_cast<float *>(stage_lds) + (size_t)(wave & 3) * 64 * 64 + lane;
    if (kgrp == 1) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) xch[((i * 2 + j) * 16 + v) * 64] = acc[i][j][v];
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (kgrp == 1) return;

    // accumulator element v of lane l sits at row (v/4)*8 + (l/32)*4 + v%4, column l%32
    const bool interior = m0 + TM <= M && n0 + TN <= N;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = m0 + wm * 64 + i * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
                const int col = n0 + wn * 64 + j * 32 + l32;
                const float sum = acc[i][j][v] + xch[((i * 2 + j) * 16 + v) * 64];
                if (interior)
                    __builtin_nontemporal_store(sum, C + (size_t)row * g.ldc + col);
                else if (row < M && col < N)
                    __builtin_nontemporal_store(sum, C + (size_t)row * g.ldc + col);
            }
}

template <int AP, int BP, bool SC = false>
int launch(hm_ctx *ctx, const char *who, const uint16_t *a, const uint16_t *b, float *c, const PieceDims &g,
           unsigned tiles, unsigned slices) {
    using S = Shape<AP, BP, SC>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_pieces_kernel<AP, BP, SC>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, S::LDS);
    HM_REQUIRE(ctx, attr == hipSuccess, "%s: cannot reserve %d bytes of LDS: %s", who, S::LDS, hipGetErrorString(attr));
    hipLaunchKernelGGL((gemm_pieces_kernel<AP, BP, SC>), dim3(tiles, slices), dim3(THREADS), S::LDS, ctx->stream, a, b, c, g);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // namespace

int homura::gemm_pieces_scaled_nk(hm_ctx *ctx, const uint16_t *d_a_split, const uint16_t *d_b_ints, const float *d_scales,
                                  int npad, float *d_c, int M, int K, int N, int max_parts, int *parts, int ldc) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_scales && npad >= (N + TN - 1) / TN * TN && npad % 4 == 0 && ((uintptr_t)d_scales % 16) == 0,
               "gemm_pieces_scaled_nk: the scales need a row stride of whole tiles (N=%d, stride %d)", N, npad);
    return gemm_pieces_any(ctx, d_a_split, 3, d_b_ints, 1, d_scales, npad, d_c, M, K, N, max_parts, parts, ldc);
}

int homura::gemm_pieces_nk(hm_ctx *ctx, const uint16_t *d_a_split, int a_pieces, const uint16_t *d_b_split, int b_pieces,
                           float *d_c, int M, int K, int N, int max_parts, int *parts, int ldc) {
    return gemm_pieces_any(ctx, d_a_split, a_pieces, d_b_split, b_pieces, nullptr, 0, d_c, M, K, N, max_parts, parts, ldc);
}

int homura::gemm_pieces_any(hm_ctx *ctx, const uint16_t *d_a_split, int a_pieces, const uint16_t *d_b_split, int b_pieces,
                            const float *d_scales, int npad, float *d_c, int M, int K, int N, int max_parts, int *parts,
                            int ldc) {
    const char *who = d_scales ? "gemm_pieces_scaled_nk" : "gemm_pieces_nk";
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_a_split && d_b_split && d_c, "%s: NULL pointer", who);
    HM_REQUIRE(ctx, M > 0 && N > 0 && K > 0 && K % TK == 0, "%s: need M, N > 0 and K %% 32 == 0 (M=%d K=%d N=%d)", who, M, K, N);
    HM_REQUIRE(ctx, (b_pieces == 1 && (a_pieces == 2 || a_pieces == 3)) || (b_pieces == 3 && a_pieces == 3),
               "%s: %d x %d pieces (2 x 1, 3 x 1 or 3 x 3)", who, a_pieces, b_pieces);
    HM_REQUIRE(ctx, ((uintptr_t)d_a_split % 16) == 0 && ((uintptr_t)d_b_split % 16) == 0, "%s: operands must be 16-byte aligned", who);
    const long long tiles = (long long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    HM_REQUIRE(ctx, tiles <= 0x7fffffffLL, "%s: too many tiles", who);
    PieceDims g;
    g.M = M;
    g.N = N;
    g.Kb = K;
    g.lda = a_pieces * K;
    g.ldb = b_pieces * K;
    g.ldc = ldc > 0 ? ldc : N;
    g.scales = d_scales;
    g.npad = npad;
    HM_REQUIRE(ctx, g.ldc >= N, "%s: ldc %d below N %d", who, g.ldc, N);
    // K slices while they still add whole waves of workgroups to a grid smaller than the chip, at least
    // eight stages (256 k) per slice
    const int ns_total = K / TK;
    int want = (int)std::max<long long>(1, ctx->num_cus / tiles);
    want = std::min(std::min(want, std::max(1, max_parts)), std::max(1, ns_total / 8));
    if (!parts) want = 1;
    g.stages_per_split = ((ns_total + want - 1) / want + 1) / 2 * 2;  // even: stages run in pairs
    const int slices = (ns_total + g.stages_per_split - 1) / g.stages_per_split;
    if (parts) *parts = slices;
    if (d_scales) return launch<3, 1, true>(ctx, who, d_a_split, d_b_split, d_c, g, (unsigned)tiles, (unsigned)slices);
    if (b_pieces == 3) return launch<3, 3>(ctx, who, d_a_split, d_b_split, d_c, g, (unsigned)tiles, (unsigned)slices);
    if (a_pieces == 3) return launch<3, 1>(ctx, who, d_a_split, d_b_split, d_c, g, (unsigned)tiles, (unsigned)slices);
    return launch<2, 1>(ctx, who, d_a_split, d_b_split, d_c, g, (unsigned)tiles, (unsigned)slices);
}
