// Prefill-chunk GEMM on the CDNA4 matrix cores: C[M][N] f32 = A[M][K] bf16 x B bf16, with B either
// [K][N] (the reference's weight layout, src/hf/weights.rs:225-261) or [N][K] (the K-contiguous
// stream layout the decode GEMVs use).
//
// The only MFMA kernel of the path (everything at batch 1 is HBM-bound). Workgroup tile 128x128,
// four wavefronts 2x2, each owning 64x64 = 2x2 accumulator tiles of v_mfma_f32_32x32x16_bf16.
// K advances 64 at a time. The next K tile travels global -> registers while the current one is
// multiplied out of LDS; two LDS buffers, one barrier per tile.
//
// LDS holds both operands K-contiguous: row r (an m of A or an n of B) is 128 bytes = eight 16-byte
// chunks of 8 k; chunk c of row r lives at slot c ^ (r & 7) ^ ((r >> 3) & 7). The MFMA operand read
// (32 consecutive rows, one chunk each, 16 bytes per lane) then touches every bank once per 8 lanes,
// and the transposing writes of a [K][N] tile (rows 8 apart per instruction) spread as well.
// A [K][N] tile is transposed in registers: a thread loads a 4(k) x 8(n) block as four 16-byte rows,
// regroups it with byte permutes into eight 8-byte columns and writes those.
//
// Workgroups that share a B column block (the M/128 row blocks) get consecutive ids on one XCD, so
// B is fetched from HBM once and served to the others from that XCD's L2.
#include "hm_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int TM = 128, TN = 128, TK = 64;
constexpr int ROW_BYTES = TK * 2;           // 128
constexpr int TILE_BYTES = TM * ROW_BYTES;  // 16 KiB per operand per buffer

__device__ __forceinline__ int lds_off(int r, int chunk) {
    return r * ROW_BYTES + ((chunk ^ (r & 7) ^ ((r >> 3) & 7)) << 4);
}

// Orders LDS traffic only: global loads stay in flight across it (a full __syncthreads() would
// also drain them).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Registers holding one K tile in flight: A always four 16-byte chunks; B four chunks as well
// (rows of a [N][K] tile, or the 4 x 8 block of a [K][N] tile).
struct TileRegs {
    u32x4 a[4], b[4];
};

// Requests one K tile. No branches: a chunk beyond K reads the last valid chunk of its row (and is
// replaced by zeros when it is written to LDS), so the loop body stays one basic block and the
// compiler can count exactly which loads a later LDS write has to wait for.
template <bool B_NK>
__device__ __forceinline__ void load_tile(TileRegs &t, const uint16_t *__restrict__ A,
                                          const uint16_t *__restrict__ B, int m0, int n0, int k0, int K,
                                          int N, int tid) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int id = tid + j * 256, r = id >> 3, c = id & 7;
        const int kc = min(k0 + c * 8, K - 8);
        t.a[j] = ld128(A + (size_t)(m0 + r) * K + kc);
        if (B_NK) t.b[j] = ld128(B + (size_t)(n0 + r) * K + kc);
    }
    if (!B_NK) {
        const int ng = tid & 15, kg = tid >> 4;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int kc = min(k0 + kg * 4 + r, K - 1);
            t.b[r] = ld128(B + (size_t)kc * N + n0 + ng * 8);
        }
    }
}

// Quarter `part` (0..3) of the LDS writes of one tile; the four quarters are placed between the
// MFMA groups of the tile being multiplied so they issue in the matrix pipe's shadow.
template <bool B_NK>
__device__ __forceinline__ void store_tile_part(const TileRegs &t, char *__restrict__ as,
                                                char *__restrict__ bs, int tid, int part, int k0, int K) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    {
        const int id = tid + part * 256, r = id >> 3, c = id & 7;
        const bool ok = k0 + c * 8 < K;
        *reinterpret_cast<u32x4 *>(as + lds_off(r, c)) = ok ? t.a[part] : zero;
        if (B_NK) *reinterpret_cast<u32x4 *>(bs + lds_off(r, c)) = ok ? t.b[part] : zero;
    }
    if (!B_NK) {
        const int ng = tid & 15, kg = tid >> 4;
        const int kb = k0 + kg * 4;  // K is a multiple of 32: the four rows are in or out together
        const bool ok = kb < K;
#pragma unroll
        for (int i = part * 2; i < part * 2 + 2; i++) {
            // column n = ng*8 + i of the block: k+0..k+3 packed low to high
            const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
            u32x2 col;
            col.x = ok ? __builtin_amdgcn_perm(t.b[1][i >> 1], t.b[0][i >> 1], sel) : 0u;
            col.y = ok ? __builtin_amdgcn_perm(t.b[3][i >> 1], t.b[2][i >> 1], sel) : 0u;
            const int n = ng * 8 + i;
            *reinterpret_cast<u32x2 *>(bs + lds_off(n, kg >> 1) + (kg & 1) * 8) = col;
        }
    }
}

template <bool B_NK>
__global__ __launch_bounds__(256) void gemm_bf16_mfma_kernel(const uint16_t *__restrict__ A,
                                                             const uint16_t *__restrict__ B,
                                                             float *__restrict__ C, int M, int K, int N) {
    __shared__ __attribute__((aligned(16))) char lds[2][2][TILE_BYTES];  // [buffer][A|B]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    // XCD-aware tile order: ids are dealt round-robin to the 8 XCDs, so XCD x runs ids x, x+8, ...;
    // give each XCD a contiguous range of the (n block major, m block minor) order.
    const int mb = M / TM, total = gridDim.x;
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

    // DEPTH tiles in flight in registers: tile j is requested DEPTH iterations before its LDS
    // writes, which sit between the MFMA groups of tile j-1. The iteration count is rounded up to
    // a multiple of DEPTH (the extra tiles are zeros) so the register ring is indexed statically.
    constexpr int DEPTH = 4;
    const int nk = (K + TK - 1) / TK;
    const int nkp = (nk + DEPTH - 1) / DEPTH * DEPTH;
    TileRegs t[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) load_tile<B_NK>(t[d], A, B, m0, n0, d * TK, K, N, tid);
#pragma unroll
    for (int part = 0; part < 4; part++) store_tile_part<B_NK>(t[0], lds[0][0], lds[0][1], tid, part, 0, K);
    lds_barrier();

    // operand registers, two stages: the reads of step ks+1 are in flight during the MFMAs of ks
    bf16x8 af[2][2], bfr[2][2];
    const int arow = wm * 64 + l32, brow = wn * 64 + l32;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        af[0][i] = *reinterpret_cast<const bf16x8 *>(lds[0][0] + lds_off(arow + i * 32, lh));
        bfr[0][i] = *reinterpret_cast<const bf16x8 *>(lds[0][1] + lds_off(brow + i * 32, lh));
    }

    for (int kt0 = 0; kt0 < nkp; kt0 += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; u++) {
            const int cur = u & 1;  // DEPTH is even: tile kt0+u sits in buffer u & 1
            // tile kt0+u left its registers during the previous iteration: refill them
            load_tile<B_NK>(t[u], A, B, m0, n0, (kt0 + u + DEPTH) * TK, K, N, tid);
#pragma unroll
            for (int ks = 0; ks < TK / 16; ks++) {
                const int st = ks & 1, nx = st ^ 1;
                if (ks < TK / 16 - 1) {
                    const int chunk = (ks + 1) * 2 + lh;
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        af[nx][i] = *reinterpret_cast<const bf16x8 *>(lds[cur][0] + lds_off(arow + i * 32, chunk));
                        bfr[nx][i] = *reinterpret_cast<const bf16x8 *>(lds[cur][1] + lds_off(brow + i * 32, chunk));
                    }
                } else {
                    // every wave has written its share of the next tile and read the last operands
                    // of this one: switch buffers, and fetch the next tile's first operands under
                    // the last MFMA group of this tile
                    lds_barrier();
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        af[nx][i] = *reinterpret_cast<const bf16x8 *>(lds[cur ^ 1][0] + lds_off(arow + i * 32, lh));
                        bfr[nx][i] = *reinterpret_cast<const bf16x8 *>(lds[cur ^ 1][1] + lds_off(brow + i * 32, lh));
                    }
                }
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] =
                            __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[st][i], bfr[st][j], acc[i][j], 0, 0, 0);
                const int k_next = (kt0 + u + 1) * TK;
                char *an = lds[cur ^ 1][0], *bn = lds[cur ^ 1][1];
                if (ks == 0) store_tile_part<B_NK>(t[(u + 1) % DEPTH], an, bn, tid, 0, k_next, K);
                if (ks == 1) store_tile_part<B_NK>(t[(u + 1) % DEPTH], an, bn, tid, 1, k_next, K);
                if (ks == 2) {
                    store_tile_part<B_NK>(t[(u + 1) % DEPTH], an, bn, tid, 2, k_next, K);
                    store_tile_part<B_NK>(t[(u + 1) % DEPTH], an, bn, tid, 3, k_next, K);
                }
            }
        }
    }

    // accumulator element v of lane l sits at row (v/4)*8 + (l/32)*4 + v%4, column l%32
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = m0 + wm * 64 + i * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
                const int col = n0 + wn * 64 + j * 32 + l32;
                __builtin_nontemporal_store(acc[i][j][v], C + (size_t)row * N + col);
            }
}

int gemm_launch(hm_ctx *ctx, const char *who, const uint16_t *a, const uint16_t *b, float *c, int M, int K,
                int N, bool b_nk) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, a && b && c, "%s: NULL pointer", who);
    HM_REQUIRE(ctx, M > 0 && N > 0 && K > 0 && M % TM == 0 && N % TN == 0 && K % 32 == 0,
               "%s: need M %% 128 == 0, N %% 128 == 0, K %% 32 == 0 (M=%d K=%d N=%d)", who, M, K, N);
    HM_REQUIRE(ctx, ((uintptr_t)a % 16) == 0 && ((uintptr_t)b % 16) == 0, "%s: operands must be 16-byte aligned",
               who);
    HM_REQUIRE(ctx, (long long)(M / TM) * (N / TN) <= 0x7fffffffLL, "%s: too many tiles", who);
    const dim3 grid((M / TM) * (N / TN));
    if (b_nk)
        hipLaunchKernelGGL(gemm_bf16_mfma_kernel<true>, grid, dim3(256), 0, ctx->stream, a, b, c, M, K, N);
    else
        hipLaunchKernelGGL(gemm_bf16_mfma_kernel<false>, grid, dim3(256), 0, ctx->stream, a, b, c, M, K, N);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // namespace

extern "C" int hm_gemm_bf16(hm_ctx *ctx, const uint16_t *d_a_mk, const uint16_t *d_b_kn, float *d_c,
                            int M, int K, int N) {
    return gemm_launch(ctx, "hm_gemm_bf16", d_a_mk, d_b_kn, d_c, M, K, N, false);
}

extern "C" int hm_gemm_bf16_nk(hm_ctx *ctx, const uint16_t *d_a_mk, const uint16_t *d_b_nk, float *d_c,
                               int M, int K, int N) {
    return gemm_launch(ctx, "hm_gemm_bf16_nk", d_a_mk, d_b_nk, d_c, M, K, N, true);
}
