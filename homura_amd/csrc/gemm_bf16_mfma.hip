// Prefill-chunk GEMM on the CDNA4 matrix cores: C[M][N] f32 = A[M][K] bf16 x B[K][N] bf16.
//
// The only MFMA kernel of the path (everything at batch 1 is HBM-bound). Workgroup tile
// 128x128, four wavefronts in a 2x2 arrangement, each owning 64x64 = 2x2 accumulator tiles of
// v_mfma_f32_32x32x16_bf16. K advances 32 at a time through LDS; B arrives [K][N] (the
// reference's weight layout) and is transposed on its way into LDS so that both operands are
// read as 8 consecutive k (16 bytes) per lane.
#include "hm_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TM = 128, TN = 128, TK = 32;
constexpr int LDK = TK + 8;  // padded k extent of an LDS row (bf16 elements)

__global__ __launch_bounds__(256) void gemm_bf16_mfma_kernel(const uint16_t *__restrict__ A,
                                                             const uint16_t *__restrict__ B,
                                                             float *__restrict__ C, int M, int K,
                                                             int N) {
    __shared__ __attribute__((aligned(16))) uint16_t As[TM][LDK];
    __shared__ __attribute__((aligned(16))) uint16_t Bt[TN][LDK];  // [n][k]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    const int l32 = lane & 31, lh = lane >> 5;

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    for (int k0 = 0; k0 < K; k0 += TK) {
        // A tile: 128 rows x 32 k = 512 chunks of 8 bf16; two per thread
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + c * 256;
            const int r = chunk >> 2, kc = (chunk & 3) * 8;
            const u32x4 v = ld128(A + (size_t)(m0 + r) * K + k0 + kc);
            *reinterpret_cast<u32x4 *>(&As[r][kc]) = v;
        }
        // B tile: 32 k rows x 128 n = 512 chunks of 8 n; transposed into Bt[n][k]
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + c * 256;
            const int kr = chunk >> 4, nc = (chunk & 15) * 8;
            const u32x4 v = ld128(B + (size_t)(k0 + kr) * N + n0 + nc);
            Bt[nc + 0][kr] = (uint16_t)(v.x & 0xFFFF);
            Bt[nc + 1][kr] = (uint16_t)(v.x >> 16);
            Bt[nc + 2][kr] = (uint16_t)(v.y & 0xFFFF);
            Bt[nc + 3][kr] = (uint16_t)(v.y >> 16);
            Bt[nc + 4][kr] = (uint16_t)(v.z & 0xFFFF);
            Bt[nc + 5][kr] = (uint16_t)(v.z >> 16);
            Bt[nc + 6][kr] = (uint16_t)(v.w & 0xFFFF);
            Bt[nc + 7][kr] = (uint16_t)(v.w >> 16);
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < TK; ks += 16) {
            bf16x8 af[2], bfr[2];
#pragma unroll
            for (int i = 0; i < 2; i++)
                af[i] = *reinterpret_cast<const bf16x8 *>(&As[wm * 64 + i * 32 + l32][ks + lh * 8]);
#pragma unroll
            for (int j = 0; j < 2; j++)
                bfr[j] = *reinterpret_cast<const bf16x8 *>(&Bt[wn * 64 + j * 32 + l32][ks + lh * 8]);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
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
                C[(size_t)row * N + col] = acc[i][j][v];
            }
}

}  // namespace

extern "C" int hm_gemm_bf16(hm_ctx *ctx, const uint16_t *d_a_mk, const uint16_t *d_b_kn, float *d_c,
                            int M, int K, int N) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_a_mk && d_b_kn && d_c, "hm_gemm_bf16: NULL pointer");
    HM_REQUIRE(ctx, M > 0 && N > 0 && K > 0 && M % TM == 0 && N % TN == 0 && K % TK == 0,
               "hm_gemm_bf16: need M %% 128 == 0, N %% 128 == 0, K %% 32 == 0 (M=%d K=%d N=%d)", M, K, N);
    HM_REQUIRE(ctx, ((uintptr_t)d_a_mk % 16) == 0 && ((uintptr_t)d_b_kn % 16) == 0,
               "hm_gemm_bf16: operands must be 16-byte aligned");
    hipLaunchKernelGGL(gemm_bf16_mfma_kernel, dim3(N / TN, M / TM), dim3(256), 0, ctx->stream, d_a_mk,
                       d_b_kn, d_c, M, K, N);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}
