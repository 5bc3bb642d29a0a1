// Prefill-chunk GEMM on the CDNA4 matrix cores: C[M][N] f32 = A[M][K] bf16 x B bf16, with B either
// [K][N] (the reference's weight layout, src/hf/weights.rs:225-261) or [N][K] (the K-contiguous
// stream layout the decode GEMVs use).
//
// The only MFMA kernel of the path (everything at batch 1 is HBM-bound). Workgroup tile 128x128,
// eight wavefronts: two groups of 2x2, each wavefront owning 64x64 = 2x2 accumulator tiles of
// v_mfma_f32_32x32x16_bf16 over half of the k steps. K advances 64 at a time. Four K tiles travel
// global -> registers while the current one is multiplied out of LDS; two LDS buffers, one
// barrier per tile.
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
//
// M and N need not be multiples of the tile: rows past the end re-read the last row and their
// results are not stored. Operands carried as several bf16 pieces (the prompt pass of f32
// activations) go through gemm_pieces_mfma.hip.
//
// Split-K: grid.y workgroups share an output tile, each multiplies a contiguous range of K tiles and
// writes its own partial C (partial s at C + s M N); the consumer adds the partials in index order,
// so the sum does not depend on timing. For products whose M x N alone gives too few tiles to fill
// the chip (the O and down projections of a prompt chunk).
#include "gemm_bf16_mfma.h"

#include <algorithm>

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

constexpr int GEMM_THREADS = 512;
constexpr int GEMM_DEPTH = 4;  // K tiles in flight in registers

// Registers holding a thread's share of one K tile in flight (four 16-byte chunks):
//   B [N][K]: v[0..1] two chunks of A, v[2..3] two chunks of B;
//   B [K][N]: threads 0..255 carry a 4(k) x 8(n) block of B as four rows, threads 256..511 four
//             chunks of A.
struct TileRegs {
    u32x4 v[4];
};

// M, N: logical sizes; K: length of the k loop; lda: row stride of A; Kb: k extent of B (k wraps at Kb)
// kt_per_split: K tiles per grid.y slice (a multiple of the register ring depth)
// ldb, ldc: row strides of B ([N][K] layout) and C
struct GemmDims {
    int M, N, K, lda, Kb, kt_per_split;
    int ldb, ldc;
};

// k index of B for loop index kc: the loop covers at most three copies of B's k range
__device__ __forceinline__ int wrap_k(int kc, int Kb) {
    kc = kc >= Kb ? kc - Kb : kc;
    return kc >= Kb ? kc - Kb : kc;
}

// Requests one K tile. No branches on k: a chunk beyond K reads the last valid chunk of its row
// (and is replaced by zeros when it is written to LDS), so the loop body stays one basic block and
// the compiler can count exactly which loads a later LDS write has to wait for.
// ALIGNED (the k loop length and B's k extent are multiples of the 64-wide tile): the k offsets are
// the same for every thread, so they stay in scalar registers and a load costs one address add.
template <bool B_NK, bool ALIGNED>
__device__ __forceinline__ void load_tile(TileRegs &t, const uint16_t *__restrict__ A,
                                          const uint16_t *__restrict__ B, int m0, int n0, int k0, int kb,
                                          const GemmDims &g, int tid) {
    const int K = g.K;
    if (ALIGNED) {
        // tiles past the end re-read the last one of A and whatever tile of B comes next (both are
        // replaced by zeros at the LDS write)
        const int ka = min(k0, K - TK);
        if (B_NK) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int id = tid + j * GEMM_THREADS, r = id >> 3, c = id & 7;
                t.v[j] = ld128(A + ((size_t)min(m0 + r, g.M - 1) * g.lda + c * 8) + ka);
                t.v[2 + j] = ld128(B + ((size_t)min(n0 + r, g.N - 1) * g.Kb + c * 8) + kb);
            }
        } else if (tid < 256) {
            const int ng = tid & 15, kg = tid >> 4;
            const int nc = min(n0 + ng * 8, g.N - 8);
#pragma unroll
            for (int r = 0; r < 4; r++) t.v[r] = ld128(B + ((size_t)(kg * 4 + r) * g.N + nc) + (size_t)kb * g.N);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int id = (tid - 256) + j * 256, r = id >> 3, c = id & 7;
                t.v[j] = ld128(A + ((size_t)min(m0 + r, g.M - 1) * g.lda + c * 8) + ka);
            }
        }
        return;
    }
    if (B_NK) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int id = tid + j * GEMM_THREADS, r = id >> 3, c = id & 7;
            const int kc = min(k0 + c * 8, K - 8);
            const int kb = wrap_k(kc, g.Kb);
            t.v[j] = ld128(A + (size_t)min(m0 + r, g.M - 1) * g.lda + kc);
            t.v[2 + j] = ld128(B + (size_t)min(n0 + r, g.N - 1) * g.Kb + kb);
        }
    } else if (tid < 256) {  // wavefront-uniform
        const int ng = tid & 15, kg = tid >> 4;
        const int nc = min(n0 + ng * 8, g.N - 8);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int kc = min(k0 + kg * 4 + r, K - 1);
            const int kb = wrap_k(kc, g.Kb);
            t.v[r] = ld128(B + (size_t)kb * g.N + nc);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int id = (tid - 256) + j * 256, r = id >> 3, c = id & 7;
            const int kc = min(k0 + c * 8, K - 8);
            t.v[j] = ld128(A + (size_t)min(m0 + r, g.M - 1) * g.lda + kc);
        }
    }
}

// Half `part` (0, 1) of a thread's LDS writes of one tile; the halves sit next to the two MFMA
// groups a wavefront runs per tile.
template <bool B_NK, bool ALIGNED>
__device__ __forceinline__ void store_tile_part(const TileRegs &t, char *__restrict__ as,
                                                char *__restrict__ bs, int tid, int part, int k0, int K) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    if (B_NK) {
        const int id = tid + part * GEMM_THREADS, r = id >> 3, c = id & 7;
        const bool ok = ALIGNED ? k0 < K : k0 + c * 8 < K;
        *reinterpret_cast<u32x4 *>(as + lds_off(r, c)) = ok ? t.v[part] : zero;
        *reinterpret_cast<u32x4 *>(bs + lds_off(r, c)) = ok ? t.v[2 + part] : zero;
    } else if (tid < 256) {
        const int ng = tid & 15, kg = tid >> 4;
        const bool ok = ALIGNED ? k0 < K : k0 + kg * 4 < K;  // K is a multiple of 32: the four rows are in or out together
#pragma unroll
        for (int i = part * 4; i < part * 4 + 4; i++) {
            // column n = ng*8 + i of the block: k+0..k+3 packed low to high
            const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
            u32x2 col;
            col.x = ok ? __builtin_amdgcn_perm(t.v[1][i >> 1], t.v[0][i >> 1], sel) : 0u;
            col.y = ok ? __builtin_amdgcn_perm(t.v[3][i >> 1], t.v[2][i >> 1], sel) : 0u;
            const int n = ng * 8 + i;
            *reinterpret_cast<u32x2 *>(bs + lds_off(n, kg >> 1) + (kg & 1) * 8) = col;
        }
    } else {
#pragma unroll
        for (int j = part * 2; j < part * 2 + 2; j++) {
            const int id = (tid - 256) + j * 256, r = id >> 3, c = id & 7;
            *reinterpret_cast<u32x4 *>(as + lds_off(r, c)) = (ALIGNED ? k0 < K : k0 + c * 8 < K) ? t.v[j] : zero;
        }
    }
}

// Eight wavefronts, two per SIMD: one wavefront alone cannot issue the LDS reads and writes, the
// global loads and the MFMAs of a tile fast enough to keep the matrix pipe busy. Wavefronts 0-3
// multiply k steps 0 and 1 of every K tile, wavefronts 4-7 steps 2 and 3, each group with its own
// 2x2 arrangement of 64x64 accumulators; the two groups' sums meet in LDS at the end.
template <bool B_NK, bool ALIGNED>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_bf16_mfma_kernel(const uint16_t *__restrict__ A,
                                                                      const uint16_t *__restrict__ B,
                                                                      float *__restrict__ C, const GemmDims g) {
    const int M = g.M, K = g.K, N = g.N;
    __shared__ __attribute__((aligned(16))) char lds[2][2][TILE_BYTES];  // [buffer][A|B]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kgrp = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

    // XCD-aware tile order: ids are dealt round-robin to the 8 XCDs, so XCD x runs ids x, x+8, ...;
    // give each XCD a contiguous range of the (n block major, m block minor) order.
    const int mb = (M + TM - 1) / TM, total = gridDim.x;  // tiles; gridDim.y = K slices
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
    // writes, which sit next to the MFMA groups of tile j-1. The iteration count is rounded up to
    // a multiple of DEPTH (the extra tiles are zeros) so the register ring is indexed statically.
    constexpr int DEPTH = GEMM_DEPTH;
    // this workgroup's K tiles: [kt_first, kt_first + nk). A slice that is not the last one has a
    // multiple of DEPTH tiles, so only the last one pads (with k >= K, i.e. zeros).
    const int kt_first = blockIdx.y * g.kt_per_split;
    const int nk = min(g.kt_per_split, (K + TK - 1) / TK - kt_first);
    const int nkp = (nk + DEPTH - 1) / DEPTH * DEPTH;
    const int kbase = kt_first * TK;
    C += (size_t)blockIdx.y * M * g.ldc;
    TileRegs t[DEPTH];
    // B's k offset of the next tile to request: runs along with the loop and wraps at Kb (ALIGNED only)
    int kb_run = kbase % g.Kb;
    auto request = [&](TileRegs &dst, int k0) {
        load_tile<B_NK, ALIGNED>(dst, A, B, m0, n0, k0, kb_run, g, tid);
        kb_run += TK;
        kb_run = kb_run >= g.Kb ? kb_run - g.Kb : kb_run;
    };
#pragma unroll
    for (int d = 0; d < DEPTH; d++) request(t[d], kbase + d * TK);
#pragma unroll
    for (int part = 0; part < 2; part++) store_tile_part<B_NK, ALIGNED>(t[0], lds[0][0], lds[0][1], tid, part, kbase, K);
    lds_barrier();

    // operand registers, two stages: the reads of the next step are in flight during the MFMAs
    bf16x8 af[2][2], bfr[2][2];
    const int arow = wm * 64 + l32, brow = wn * 64 + l32;
    const int chunk0 = kgrp * 4 + lh, chunk1 = chunk0 + 2;  // this group's two k steps of a tile
#pragma unroll
    for (int i = 0; i < 2; i++) {
        af[0][i] = *reinterpret_cast<const bf16x8 *>(lds[0][0] + lds_off(arow + i * 32, chunk0));
        bfr[0][i] = *reinterpret_cast<const bf16x8 *>(lds[0][1] + lds_off(brow + i * 32, chunk0));
    }

    for (int kt0 = 0; kt0 < nkp; kt0 += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; u++) {
            const int cur = u & 1;  // DEPTH is even: tile kt0+u sits in buffer u & 1
            // tile kt0+u left its registers during the previous iteration: refill them
            request(t[u], kbase + (kt0 + u + DEPTH) * TK);
            const int k_next = kbase + (kt0 + u + 1) * TK;
            char *an = lds[cur ^ 1][0], *bn = lds[cur ^ 1][1];

            // first step: its operands are in stage 0; fetch the second step's meanwhile
#pragma unroll
            for (int i = 0; i < 2; i++) {
                af[1][i] = *reinterpret_cast<const bf16x8 *>(lds[cur][0] + lds_off(arow + i * 32, chunk1));
                bfr[1][i] = *reinterpret_cast<const bf16x8 *>(lds[cur][1] + lds_off(brow + i * 32, chunk1));
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[0][i], bfr[0][j], acc[i][j], 0, 0, 0);
            store_tile_part<B_NK, ALIGNED>(t[(u + 1) % DEPTH], an, bn, tid, 0, k_next, K);
            store_tile_part<B_NK, ALIGNED>(t[(u + 1) % DEPTH], an, bn, tid, 1, k_next, K);
            // every wavefront has written its share of the next tile and read the last operands of
            // this one: switch buffers, and fetch the next tile's first operands under the second
            // MFMA group of this tile
            lds_barrier();
#pragma unroll
            for (int i = 0; i < 2; i++) {
                af[0][i] = *reinterpret_cast<const bf16x8 *>(an + lds_off(arow + i * 32, chunk0));
                bfr[0][i] = *reinterpret_cast<const bf16x8 *>(bn + lds_off(brow + i * 32, chunk0));
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[1][i], bfr[1][j], acc[i][j], 0, 0, 0);
        }
    }

    // the second group hands its sums over through LDS (64 KiB = 4 wavefronts x 64 x 64 floats,
    // lane-major so consecutive lanes touch consecutive words)
    lds_barrier();  // nobody reads operands any more
    float *xch = reinterpret_cast<float *>(&lds[0][0][0]) + (size_t)(wave & 3) * 64 * 64 + lane;
    if (kgrp == 1) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) xch[((i * 2 + j) * 16 + v) * 64] = acc[i][j][v];
    }
    lds_barrier();
    if (kgrp == 1) return;

    // accumulator element v of lane l sits at row (v/4)*8 + (l/32)*4 + v%4, column l%32
    const bool interior = m0 + TM <= M && n0 + TN <= N;  // workgroup-uniform: edge tiles check every element
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

// ---- [N][K] operand, K tiles aligned: global -> LDS loads without the trip through registers ----
//
// global_load_lds_dwordx4 writes lane l's 16 bytes to LDS at (wave-uniform base) + 16 l, so one
// instruction fills eight 128-byte rows. The slot swizzle moves to the global side: the lane that
// fills slot s of row r fetches chunk s ^ (r & 7) ^ ((r >> 3) & 7) of that row. The tiles in flight
// live in LDS (DMA_BUFS buffers of 32 KiB), the registers of the ring above are free, and the LDS
// write instructions are gone.
constexpr int DMA_BUFS = 4;  // the vmcnt values in the kernel count DMA_BUFS - 1 tiles of four loads in flight
static_assert(DMA_BUFS == 4, "adjust the wait counts of gemm_nk_dma_kernel");
constexpr int DMA_LDS_BYTES = DMA_BUFS * 2 * TILE_BYTES;  // 128 of the CU's 160 KiB

extern __shared__ __attribute__((aligned(16))) char dma_lds[];

__device__ __forceinline__ void dma16(const uint16_t *src, char *dst) {
    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)src,
                                     (void __attribute__((address_space(3))) *)dst, 16, 0, 0);
}

// The operand reads and their waits are written out: the compiler's own wait insertion stalls on
// all outstanding LDS reads at the top of the loop, these wait only for the ones about to be used.
// (LDS operations of a wavefront return in order.)
template <int IMM>
__device__ __forceinline__ bf16x8 lds_read16_imm(uint32_t addr) {
    bf16x8 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(IMM) : "memory");
    return v;
}

__global__ __launch_bounds__(GEMM_THREADS) void gemm_nk_dma_kernel(const uint16_t *__restrict__ A,
                                                                   const uint16_t *__restrict__ B,
                                                                   float *__restrict__ C, const GemmDims g) {
    const int M = g.M, K = g.K, N = g.N;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kgrp = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;

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

    const int kt_first = blockIdx.y * g.kt_per_split;
    const int nk = min(g.kt_per_split, K / TK - kt_first);
    C += (size_t)blockIdx.y * M * g.ldc;

    // this thread's two rows of A and of B: instruction j of wavefront w fills rows 8 (2 w + j) .. + 7
    const uint16_t *a_src[2], *b_src[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int r = (wave * 2 + j) * 8 + (lane >> 3), s = lane & 7;
        const int c = s ^ (r & 7) ^ ((r >> 3) & 7);
        a_src[j] = A + (size_t)min(m0 + r, M - 1) * g.lda + c * 8;
        b_src[j] = B + (size_t)min(n0 + r, N - 1) * g.ldb + c * 8;
    }
    // where this wavefront's first instruction lands inside an operand tile (scalar: it goes to M0)
    const int wave_dst = __builtin_amdgcn_readfirstlane(wave * 2048);
    // k offset of the next tile to request (scalar; the loop is short enough for its bookkeeping to
    // show in the run time). A tile past the end re-reads the last one (nobody multiplies it), so every
    // iteration issues the same four loads and the wait counts below are exact.
    int koff = kt_first * TK;
    auto request = [&](int buf) {
        char *base = dma_lds + buf * (2 * TILE_BYTES) + wave_dst;
        const int k = min(koff, K - TK);
#pragma unroll
        for (int j = 0; j < 2; j++) {
            dma16(a_src[j] + k, base + j * 1024);
            dma16(b_src[j] + k, base + TILE_BYTES + j * 1024);
        }
        koff += TK;
    };
#pragma unroll
    for (int d = 0; d < DMA_BUFS; d++) request(d);

    const int arow = wm * 64 + l32, brow = wn * 64 + l32;
    const int chunk0 = kgrp * 4 + lh, chunk1 = chunk0 + 2;  // this group's two k steps of a tile
    // LDS addresses of this lane's operands in buffer 0, [k step][i]. Buffers 1..3 are 32 KiB apart;
    // the immediate offset of an LDS instruction has 16 bits, so buffers 2 and 3 get addresses of
    // their own (64 KiB on) and the odd buffers the immediate 32 KiB.
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)dma_lds;
    uint32_t a_lo[2][2], b_lo[2][2], a_hi[2][2], b_hi[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        a_lo[0][i] = lds0 + lds_off(arow + i * 32, chunk0);
        a_lo[1][i] = lds0 + lds_off(arow + i * 32, chunk1);
        b_lo[0][i] = lds0 + TILE_BYTES + lds_off(brow + i * 32, chunk0);
        b_lo[1][i] = lds0 + TILE_BYTES + lds_off(brow + i * 32, chunk1);
#pragma unroll
        for (int st = 0; st < 2; st++) {
            a_hi[st][i] = a_lo[st][i] + 4 * TILE_BYTES;
            b_hi[st][i] = b_lo[st][i] + 4 * TILE_BYTES;
        }
    }
    // operand registers, two stages: the reads of the next step are in flight during the MFMAs
    bf16x8 af[2][2], bfr[2][2];
    // stage `st` <- k step `st` of buffer `buf` (a compile-time constant in the main loop)
    auto read_step = [&](int buf, int st) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t pa = buf < 2 ? a_lo[st][i] : a_hi[st][i], pb = buf < 2 ? b_lo[st][i] : b_hi[st][i];
            if (buf & 1) {
                af[st][i] = lds_read16_imm<2 * TILE_BYTES>(pa);
                bfr[st][i] = lds_read16_imm<2 * TILE_BYTES>(pb);
            } else {
                af[st][i] = lds_read16_imm<0>(pa);
                bfr[st][i] = lds_read16_imm<0>(pb);
            }
        }
    };
    // tiles 1..3 (four loads each) may still be in flight; tile 0 has landed for everyone
    asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");
    read_step(0, 0);

    // one K tile out of buffer `buf`
    auto tile = [&](int buf) {
        read_step(buf, 1);
        // the four reads above may be in flight; the four before them (stage 0) have arrived
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(af[0][0]), "+v"(af[0][1]), "+v"(bfr[0][0]), "+v"(bfr[0][1]));
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[0][i], bfr[0][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);  // these MFMAs go out before the wait: it hides behind them
        // every wavefront has read its last operands of this tile, and the next tile has landed for
        // everyone (the two after it may be in flight): this tile's buffer takes tile kt + 4
        asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier"
                     : "+v"(af[1][0]), "+v"(af[1][1]), "+v"(bfr[1][0]), "+v"(bfr[1][1])
                     :
                     : "memory");
        request(buf);
        read_step((buf + 1) % DMA_BUFS, 0);
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[1][i], bfr[1][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    // whole rounds of four tiles: every buffer index is a constant, the body is one basic block
    int kt = 0;
    for (; kt + DMA_BUFS <= nk; kt += DMA_BUFS) {
#pragma unroll
        for (int u = 0; u < DMA_BUFS; u++) tile(u);
    }
    // the last zero to three tiles (buffers 0, 1, 2 in turn)
    for (int u = 0; kt < nk; kt++, u++) {
        if (u == 0)
            tile(0);
        else if (u == 1)
            tile(1);
        else
            tile(2);
    }

    // drain what is in flight before the buffers are reused for the exchange: the loads into LDS, and
    // the operand reads of the tile after the last (stage 0; the wait names its registers so that they
    // stay untouched until the data has arrived)
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier"
                 : "+v"(af[0][0]), "+v"(af[0][1]), "+v"(bfr[0][0]), "+v"(bfr[0][1])
                 :
                 : "memory");
    float *xch = reinterpret_cast<float *>(dma_lds) + (size_t)(wave & 3) * 64 * 64 + lane;
    if (kgrp == 1) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) xch[((i * 2 + j) * 16 + v) * 64] = acc[i][j][v];
    }
    lds_barrier();
    if (kgrp == 1) return;

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

// a_pieces > 1: A is a split matrix [M][a_pieces * K] and the k loop runs over all its pieces against the same B
// (B's k index wraps at K), so C is the sum of the pieces' products.
int gemm_launch(hm_ctx *ctx, const char *who, const uint16_t *a, const uint16_t *b, float *c, int M, int K,
                int N, bool b_nk, int ksplit = 1, int *ksplit_used = nullptr, int ldc = 0, int a_pieces = 1) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, a && b && c, "%s: NULL pointer", who);
    HM_REQUIRE(ctx, M > 0 && N > 0 && K > 0 && K % 32 == 0, "%s: need M, N > 0 and K %% 32 == 0 (M=%d K=%d N=%d)", who,
               M, K, N);
    HM_REQUIRE(ctx, b_nk || N % 8 == 0, "%s: a [K][N] operand needs N %% 8 == 0 (N=%d)", who, N);
    HM_REQUIRE(ctx, ((uintptr_t)a % 16) == 0 && ((uintptr_t)b % 16) == 0, "%s: operands must be 16-byte aligned",
               who);
    const long long tiles = (long long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    HM_REQUIRE(ctx, tiles <= 0x7fffffffLL, "%s: too many tiles", who);
    GemmDims g;
    g.M = M;
    g.N = N;
    g.Kb = K;
    g.K = a_pieces * K;
    g.lda = a_pieces * K;
    g.ldb = K;
    g.ldc = ldc > 0 ? ldc : N;
    HM_REQUIRE(ctx, g.ldc >= N, "%s: ldc %d below N %d", who, g.ldc, N);
    const int nk_total = (g.K + TK - 1) / TK;
    if (ksplit < 1) ksplit = 1;
    g.kt_per_split = ((nk_total + ksplit - 1) / ksplit + GEMM_DEPTH - 1) / GEMM_DEPTH * GEMM_DEPTH;
    const int slices = (nk_total + g.kt_per_split - 1) / g.kt_per_split;
    if (ksplit_used) *ksplit_used = slices;
    const dim3 grid((unsigned)tiles, (unsigned)slices);
    const bool aligned = g.K % TK == 0 && g.Kb % TK == 0;
    if (b_nk && aligned) {
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_nk_dma_kernel),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, DMA_LDS_BYTES);
        HM_REQUIRE(ctx, attr == hipSuccess, "%s: cannot reserve %d bytes of LDS: %s", who, DMA_LDS_BYTES,
                   hipGetErrorString(attr));
        hipLaunchKernelGGL(gemm_nk_dma_kernel, grid, dim3(GEMM_THREADS), DMA_LDS_BYTES, ctx->stream, a, b, c, g);
    } else if (b_nk)
        hipLaunchKernelGGL((gemm_bf16_mfma_kernel<true, false>), grid, dim3(GEMM_THREADS), 0, ctx->stream, a, b, c, g);
    else if (aligned)
        hipLaunchKernelGGL((gemm_bf16_mfma_kernel<false, true>), grid, dim3(GEMM_THREADS), 0, ctx->stream, a, b, c, g);
    else
        hipLaunchKernelGGL((gemm_bf16_mfma_kernel<false, false>), grid, dim3(GEMM_THREADS), 0, ctx->stream, a, b, c, g);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // namespace

int homura::gemm_split_nk(hm_ctx *ctx, const uint16_t *d_a_split, int pieces, const uint16_t *d_b_nk, float *d_c,
                          int M, int K, int N, int max_parts, int *parts) {
    HM_REQUIRE(ctx, pieces >= 1 && pieces <= 3, "gemm_split_nk: %d pieces (1..3)", pieces);
    if (pieces >= 2)  // every tile once, all piece products per stage
        return gemm_pieces_nk(ctx, d_a_split, pieces, d_b_nk, 1, d_c, M, K, N, max_parts, parts);
    // K slices while they still add whole waves of workgroups to a grid smaller than the chip (the
    // slices cost a write and a read of C each), at least 4 K tiles per slice
    const long long tiles = (long long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    const int nk_total = (K + TK - 1) / TK;
    int want = (int)std::max<long long>(1, ctx->num_cus / tiles);
    want = std::min(std::min(want, max_parts), std::max(1, nk_total / GEMM_DEPTH));
    if (!parts) want = 1;
    return gemm_launch(ctx, "gemm_split_nk", d_a_split, d_b_nk, d_c, M, K, N, true, want, parts);
}

int homura::gemm_split_split_nk(hm_ctx *ctx, const uint16_t *d_a_split, const uint16_t *d_b_split, float *d_c, int M,
                                int K, int N, int max_parts, int *parts, int ldc) {
    return gemm_pieces_nk(ctx, d_a_split, 3, d_b_split, 3, d_c, M, K, N, max_parts, parts, ldc);
}

int homura::gemm_split_kn(hm_ctx *ctx, const uint16_t *d_a_split, int pieces, const uint16_t *d_b_kn, float *d_c, int M,
                          int K, int N) {
    HM_REQUIRE(ctx, pieces >= 1 && pieces <= 3, "gemm_split_kn: %d pieces (1..3)", pieces);
    return gemm_launch(ctx, "gemm_split_kn", d_a_split, d_b_kn, d_c, M, K, N, false, 1, nullptr, 0, pieces);
}

extern "C" int hm_gemm_bf16(hm_ctx *ctx, const uint16_t *d_a_mk, const uint16_t *d_b_kn, float *d_c,
                            int M, int K, int N) {
    return gemm_launch(ctx, "hm_gemm_bf16", d_a_mk, d_b_kn, d_c, M, K, N, false);
}

extern "C" int hm_gemm_bf16_nk(hm_ctx *ctx, const uint16_t *d_a_mk, const uint16_t *d_b_nk, float *d_c,
                               int M, int K, int N) {
    return gemm_launch(ctx, "hm_gemm_bf16_nk", d_a_mk, d_b_nk, d_c, M, K, N, true);
}
