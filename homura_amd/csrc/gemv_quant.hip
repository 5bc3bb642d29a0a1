// GGUF block-quantised weights: dequant-GEMV (Q8_0, Q4_0) and bit-exact block dequantisation.
//
// Weights stay in HBM as the raw GGUF block bytes, rows of K/32 blocks. A workgroup takes a
// contiguous run of rows, which is a contiguous byte range of the weight buffer, and copies
// it into LDS with aligned 16-byte loads (blocks are 34 or 18 bytes, so block starts are only
// 2-byte aligned; the copy is aligned on the buffer, not on the blocks). Each lane then owns
// one block column: it keeps the 32 activations of that column in registers and walks the
// rows, unpacking scale and quants from LDS. HBM traffic is exactly the block bytes.
#include "hm_common.h"

namespace {

constexpr int QTHREADS = 256;
constexpr int QWAVES = QTHREADS / WAVE;
constexpr int MAX_ROWS_PER_WAVE = 8;

template <int QT>
struct BlockTraits;
template <>
struct BlockTraits<0> {  // Q8_0: f16 d + 32 x int8 (reference src/gguf.rs:817-831)
    static constexpr int BYTES = 34;
};
template <>
struct BlockTraits<1> {  // Q4_0: f16 d + 16 bytes of nibble pairs (ggml block_q4_0)
    static constexpr int BYTES = 18;
};

__device__ __forceinline__ uint32_t lds_u16(const uint8_t *p) {
    return *reinterpret_cast<const uint16_t *>(p);
}

// sum_j q_j * x_j for one block, q taken as stored (unsigned byte / nibble); the caller
// removes the offset (128 or 8) with the precomputed sum of the activations.
template <int QT>
__device__ __forceinline__ float block_dot_unsigned(const uint8_t *blk, const float *xv) {
    float s = 0.f;
    if (QT == 0) {
#pragma unroll
        for (int j = 0; j < 16; j++) {
            uint32_t v = lds_u16(blk + 2 + 2 * j) ^ 0x8080u;  // int8 -> biased unsigned
            s = fmaf((float)(v & 0xFFu), xv[2 * j], s);
            s = fmaf((float)(v >> 8), xv[2 * j + 1], s);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            uint32_t v = lds_u16(blk + 2 + 2 * j);  // bytes 2j, 2j+1
            s = fmaf((float)(v & 0xFu), xv[2 * j], s);
            s = fmaf((float)((v >> 4) & 0xFu), xv[2 * j + 16], s);
            s = fmaf((float)((v >> 8) & 0xFu), xv[2 * j + 1], s);
            s = fmaf((float)(v >> 12), xv[2 * j + 17], s);
        }
    }
    return s;
}

template <int QT>
__global__ __launch_bounds__(QTHREADS) void gemv_quant_kernel(
    const float *__restrict__ x, const uint8_t *__restrict__ w, float *__restrict__ out, int K,
    int N, int rows_per_step, size_t total_bytes) {
    constexpr int BB = BlockTraits<QT>::BYTES;
    constexpr float OFFSET = QT == 0 ? 128.f : 8.f;
    constexpr int U = 8;  // 16-byte weight loads a thread keeps in flight while staging
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    float *xs = reinterpret_cast<float *>(smem);
    uint8_t *ws = smem + (size_t)K * 4;

    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int nb = K / 32;
    const size_t rowbytes = (size_t)nb * BB;
    const int nsteps = (N + rows_per_step - 1) / rows_per_step;

    // activations once per workgroup; the workgroup then walks row steps blockIdx, +grid, ...
    for (int k = tid; k < K; k += QTHREADS) xs[k] = x[k];

    for (int step = blockIdx.x; step < nsteps; step += gridDim.x) {
        const int r0 = step * rows_per_step;
        const int nrows = min(rows_per_step, N - r0);
        const size_t beg = (size_t)r0 * rowbytes;
        const size_t end = beg + (size_t)nrows * rowbytes;
        const size_t abeg = beg & ~(size_t)15;
        const int shift = (int)(beg - abeg);
        const int nchunks = (int)((end - abeg + 15) / 16);

        __syncthreads();  // previous step's readers are done with ws (and xs is complete)
        for (int i0 = tid; i0 < nchunks; i0 += QTHREADS * U) {
            u32x4 tmp[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int i = i0 + u * QTHREADS;
                const size_t off = abeg + (size_t)i * 16;
                tmp[u] = (i < nchunks && off + 16 <= total_bytes) ? ld128_stream(w + off)
                                                                  : u32x4{0u, 0u, 0u, 0u};
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int i = i0 + u * QTHREADS;
                if (i < nchunks) {
                    const size_t off = abeg + (size_t)i * 16;
                    if (off + 16 <= total_bytes) {
                        *reinterpret_cast<u32x4 *>(ws + (size_t)i * 16) = tmp[u];
                    } else {  // last, partial chunk of the buffer: stay inside it
                        for (int b = 0; b < 16; b++)
                            ws[(size_t)i * 16 + b] = off + b < total_bytes ? w[off + b] : 0;
                    }
                }
            }
        }
        __syncthreads();

        float acc[MAX_ROWS_PER_WAVE];
#pragma unroll
        for (int i = 0; i < MAX_ROWS_PER_WAVE; i++) acc[i] = 0.f;
        for (int bc = lane; bc < nb; bc += WAVE) {
            float xv[32];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const f32x4 t = *reinterpret_cast<const f32x4 *>(xs + bc * 32 + j * 4);
                xv[4 * j] = t.x; xv[4 * j + 1] = t.y; xv[4 * j + 2] = t.z; xv[4 * j + 3] = t.w;
            }
            float sx = 0.f;
#pragma unroll
            for (int j = 0; j < 32; j++) sx += xv[j];
#pragma unroll
            for (int i = 0; i < MAX_ROWS_PER_WAVE; i++) {
                const int lr = wave + QWAVES * i;
                if (lr < nrows) {
                    const uint8_t *blk = ws + shift + ((size_t)lr * nb + bc) * BB;
                    const float d = f16_bits_to_f32((uint16_t)lds_u16(blk));
                    const float s = block_dot_unsigned<QT>(blk, xv);
                    acc[i] = fmaf(d, s - OFFSET * sx, acc[i]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MAX_ROWS_PER_WAVE; i++) {
            const int lr = wave + QWAVES * i;
            const float v = wave_sum(acc[i]);
            if (lane == 0 && lr < nrows) out[r0 + lr] = v;
        }
    }
}

// One thread per element; a single f32 multiply per element so the result is the same bits
// the CPU produces (reference src/gguf.rs:825-829).
template <int QT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t *__restrict__ blocks,
                                                      float *__restrict__ out, size_t n_elems) {
    constexpr int BB = BlockTraits<QT>::BYTES;
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; e < n_elems; e += stride) {
        const size_t b = e >> 5;
        const int j = (int)(e & 31);
        const uint8_t *blk = blocks + b * BB;
        const float d = f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        float q;
        if (QT == 0) {
            q = (float)(int8_t)blk[2 + j];
        } else {
            const uint8_t byte = blk[2 + (j & 15)];
            q = (float)((j < 16 ? (byte & 0x0F) : (byte >> 4)) - 8);
        }
        out[e] = q * d;
    }
}

template <int QT>
int gemv_quant_launch(hm_ctx *ctx, const char *name, const float *d_x, const uint8_t *d_w,
                      float *d_out, int M, int K, int N) {
    HM_CHECK_CTX(ctx);
    constexpr int BB = BlockTraits<QT>::BYTES;
    HM_REQUIRE(ctx, d_x && d_w && d_out, "%s: NULL pointer", name);
    HM_REQUIRE(ctx, M >= 1 && M <= 8, "%s: M=%d outside 1..8", name, M);
    HM_REQUIRE(ctx, K > 0 && K % 32 == 0 && N > 0, "%s: K=%d must be a positive multiple of 32, N=%d positive", name, K, N);
    HM_REQUIRE(ctx, ((uintptr_t)d_w % 16) == 0 && ((uintptr_t)d_x % 4) == 0, "%s: weight buffer must be 16-byte aligned", name);
    const size_t rowbytes = (size_t)(K / 32) * BB;
    const size_t x_bytes = (size_t)K * 4;
    const size_t lds_budget = 48 * 1024;
    HM_REQUIRE(ctx, x_bytes + QWAVES * rowbytes + 32 <= 64 * 1024, "%s: K=%d too large for the LDS stage", name, K);
    // rows staged per step: as many as fit the LDS budget (at most 8 per wavefront), but few
    // enough that every CU gets a workgroup
    int rows = (int)((lds_budget - x_bytes) / rowbytes);
    rows = rows / QWAVES * QWAVES;
    if (rows < QWAVES) rows = QWAVES;
    if (rows > QWAVES * MAX_ROWS_PER_WAVE) rows = QWAVES * MAX_ROWS_PER_WAVE;
    while (rows > QWAVES && (N + rows - 1) / rows < 2 * ctx->num_cus) rows -= QWAVES;
    const size_t lds = x_bytes + (size_t)rows * rowbytes + 32;
    const int nsteps = (N + rows - 1) / rows;
    // persistent workgroups: a few per CU, each stages the activations once
    int wg_per_cu = (int)(120 * 1024 / lds);
    if (wg_per_cu < 1) wg_per_cu = 1;
    if (wg_per_cu > 6) wg_per_cu = 6;
    const int grid = nsteps < ctx->num_cus * wg_per_cu ? nsteps : ctx->num_cus * wg_per_cu;
    const size_t total = (size_t)N * rowbytes;
    for (int m = 0; m < M; m++) {
        hipLaunchKernelGGL((gemv_quant_kernel<QT>), dim3(grid), dim3(QTHREADS), lds, ctx->stream,
                           d_x + (size_t)m * K, d_w, d_out + (size_t)m * N, K, N, rows, total);
        HM_LAUNCH_CHECK(ctx);
    }
    return HM_OK;
}

template <int QT>
int dequant_launch(hm_ctx *ctx, const char *name, const uint8_t *d_blocks, float *d_out,
                   size_t nblocks) {
    HM_CHECK_CTX(ctx);
    if (nblocks == 0) return HM_OK;
    HM_REQUIRE(ctx, d_blocks && d_out, "%s: NULL pointer", name);
    const size_t n = nblocks * 32;
    size_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL((dequant_kernel<QT>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       d_blocks, d_out, n);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

}  // namespace

extern "C" {

int hm_gemv_q8_0(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M,
                 int K, int N) {
    return gemv_quant_launch<0>(ctx, "hm_gemv_q8_0", d_x, d_w_blocks, d_out, M, K, N);
}

int hm_gemv_q4_0(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M,
                 int K, int N) {
    return gemv_quant_launch<1>(ctx, "hm_gemv_q4_0", d_x, d_w_blocks, d_out, M, K, N);
}

int hm_dequant_q8_0(hm_ctx *ctx, const uint8_t *d_blocks, float *d_out, size_t nblocks) {
    return dequant_launch<0>(ctx, "hm_dequant_q8_0", d_blocks, d_out, nblocks);
}

int hm_dequant_q4_0(hm_ctx *ctx, const uint8_t *d_blocks, float *d_out, size_t nblocks) {
    return dequant_launch<1>(ctx, "hm_dequant_q4_0", d_blocks, d_out, nblocks);
}

}  // extern "C"
