// GGUF block-quantised weights: dequant-GEMV (Q8_0, Q4_0) and bit-exact block dequantisation.
//
// Weights stay in HBM as the raw GGUF block bytes, rows of K/32 blocks. A workgroup takes a
// contiguous run of rows, which is a contiguous byte range of the weight buffer, and copies
// it into LDS with aligned 16-byte loads (blocks are 34 or 18 bytes, so block starts are only
// 2-byte aligned; the copy is aligned on the buffer, not on the blocks). HBM traffic is exactly
// the block bytes.
//
// The unit of work of a lane is a quarter block: 8 weights = 8 quant bytes (Q8_0) or one 32-bit
// word of nibble pairs (Q4_0), plus the block's scale. Quarter columns are dealt to the lanes
// round-robin (K/8 of them, so K = 1536 fills three full rounds where whole blocks would leave a
// quarter of the wavefront idle); a lane keeps the 8 activations of each of its columns, and
// their sum, in registers for the life of the workgroup and walks the staged rows. Quants are
// used as stored (biased unsigned): sum_j q_j x_j - offset * sum_j x_j, four byte->float
// conversions per 32-bit word with no shifts for the byte lanes.
#include "gemv_quant.h"
#include "gemv_quant_planes.h"

#include "hm_common.h"
#include "quant_formats.h"

namespace {

constexpr int QTHREADS = 256;
constexpr int QWAVES = QTHREADS / WAVE;
constexpr int MAX_ROWS_PER_WAVE = 8;
constexpr int MAXC = 8;  // most quarter columns a lane keeps in registers (K <= 4096); more are re-read

template <int QT>
struct BlockTraits;
template <>
struct BlockTraits<0> {  // Q8_0: f16 d + 32 x int8 (reference src/gguf.rs:817-831)
    static constexpr int BYTES = 34;
    static constexpr int QUARTER = 8;  // quant bytes of 8 weights
};
template <>
struct BlockTraits<1> {  // Q4_0: f16 d + 16 bytes of nibble pairs (ggml block_q4_0)
    static constexpr int BYTES = 18;
    static constexpr int QUARTER = 4;
};

__device__ __forceinline__ uint32_t lds_u16(const uint8_t *p) {
    return *reinterpret_cast<const uint16_t *>(p);
}
// 32-bit word at a 2-byte aligned LDS address
__device__ __forceinline__ uint32_t lds_u32_a2(const uint8_t *p) { return lds_u16(p) | (lds_u16(p + 2) << 16); }

__device__ __forceinline__ float dot4_bytes(uint32_t w, const float *xv, float s) {
    s = fmaf((float)(w & 0xFFu), xv[0], s);
    s = fmaf((float)((w >> 8) & 0xFFu), xv[1], s);
    s = fmaf((float)((w >> 16) & 0xFFu), xv[2], s);
    s = fmaf((float)(w >> 24), xv[3], s);
    return s;
}

// Activations of quarter column c (block c/4, quarter c%4) in the order the quant bytes use them.
template <int QT>
__device__ __forceinline__ void load_xv(const float *xs, int c, float *xv, float &sx_off) {
    const int b = c >> 2, q = c & 3;
    const float *p0 = xs + b * 32 + (QT == 0 ? q * 8 : q * 4);
    const float *p1 = QT == 0 ? p0 + 4 : p0 + 16;
    const f32x4 lo = *reinterpret_cast<const f32x4 *>(p0);
    const f32x4 hi = *reinterpret_cast<const f32x4 *>(p1);
    xv[0] = lo.x; xv[1] = lo.y; xv[2] = lo.z; xv[3] = lo.w;
    xv[4] = hi.x; xv[5] = hi.y; xv[6] = hi.z; xv[7] = hi.w;
    float sx = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) sx += xv[j];
    sx_off = sx * (QT == 0 ? 128.f : 8.f);
}

// d * (sum_j q_j x_j - offset * sum_j x_j) for one quarter block: `dp` points at the block's scale,
// `qp` at the quarter's quant bytes (both in LDS, 2-byte aligned).
template <int QT>
__device__ __forceinline__ float quarter_dot(const uint8_t *dp, const uint8_t *qp, const float *xv, float sx_off) {
    const float d = f16_bits_to_f32((uint16_t)lds_u16(dp));
    float s;
    if (QT == 0) {
        const uint32_t w0 = lds_u32_a2(qp) ^ 0x80808080u;  // int8 -> biased unsigned
        const uint32_t w1 = lds_u32_a2(qp + 4) ^ 0x80808080u;
        s = dot4_bytes(w1, xv + 4, dot4_bytes(w0, xv, 0.f));
    } else {
        // byte i of the word: low nibble = weight 4q+i, high nibble = weight 16+4q+i
        const uint32_t w = lds_u32_a2(qp);
        s = dot4_bytes((w >> 4) & 0x0F0F0F0Fu, xv + 4, dot4_bytes(w & 0x0F0F0F0Fu, xv, 0.f));
    }
    return d * (s - sx_off);
}

// The same with the block given as a byte offset `boff` (even) into the 16-byte aligned LDS stage: the quant
// bytes of a quarter are read as aligned dwords around them and moved into place with a funnel shift (blocks
// are 34 or 18 bytes, so the words sit two bytes into a dword for every other block) - for Q8_0 three LDS
// reads per quarter instead of five 16-bit ones.
template <int QT>
__device__ __forceinline__ float quarter_dot_at(const uint8_t *stage, int boff, int q, const float *xv, float sx_off) {
    const int qo = boff + 2 + q * BlockTraits<QT>::QUARTER;  // first quant byte of the quarter
    // Q4_0 has one word per quarter: two 16-bit reads were measured faster there than a dword pair and a shift
    if (QT == 1) return quarter_dot<1>(stage + boff, stage + qo, xv, sx_off);
    const float d = f16_bits_to_f32((uint16_t)lds_u16(stage + boff));
    const uint32_t sh = (uint32_t)(qo & 2) * 8;
    const uint32_t *p = reinterpret_cast<const uint32_t *>(stage + (qo & ~3));
    float s;
    if (QT == 0) {
        const uint32_t a0 = p[0], a1 = p[1], a2 = p[2];
        const uint32_t w0 = __builtin_amdgcn_alignbit(a1, a0, sh) ^ 0x80808080u;  // int8 -> biased unsigned
        const uint32_t w1 = __builtin_amdgcn_alignbit(a2, a1, sh) ^ 0x80808080u;
        s = dot4_bytes(w1, xv + 4, dot4_bytes(w0, xv, 0.f));
    } else {
        const uint32_t a0 = p[0], a1 = p[1];
        const uint32_t w = __builtin_amdgcn_alignbit(a1, a0, sh);
        s = dot4_bytes((w >> 4) & 0x0F0F0F0Fu, xv + 4, dot4_bytes(w & 0x0F0F0F0Fu, xv, 0.f));
    }
    return d * (s - sx_off);
}

constexpr int STAGE_U = 8;                       // 16-byte chunks a thread carries per row step
constexpr int STAGE_BYTES = QTHREADS * STAGE_U * 16;  // most bytes one row step may span

// The aligned 16-byte chunks covering rows [r0, r0+nrows): chunk i of the step starts at abeg + 16 i.
// A chunk that holds at least one byte of the buffer lies in that byte's page, so reading whole
// aligned chunks at both ends of the buffer cannot fault.
struct StepRange {
    size_t abeg;
    int shift, nchunks, r0, nrows;
};
__device__ __forceinline__ StepRange step_range(int step, int rows_per_step, int N, size_t rowbytes) {
    StepRange r;
    r.r0 = step * rows_per_step;
    r.nrows = min(rows_per_step, N - r.r0);
    const size_t beg = (size_t)r.r0 * rowbytes, end = beg + (size_t)r.nrows * rowbytes;
    r.abeg = beg & ~(size_t)15;
    r.shift = (int)(beg - r.abeg);
    r.nchunks = (int)((end - r.abeg + 15) / 16);
    return r;
}

// RT rows lr, lr+QWAVES, ... of the staged step for one wavefront, activations in registers.
// Round t of a lane is quarter column lane + 64 t: 16 blocks further along the row, a constant
// offset from the lane's first column. Lanes past the row end read whatever follows in LDS (the
// allocation carries slack for it) and their value is dropped by a select.
// AL: Q8_0 quant words through aligned dword reads (quarter_dot_at); measured faster in the model's fused
// launches, not in the plain product, which keeps the 16-bit reads.
template <int QT, int NXV, int RT, bool AL>
__device__ __forceinline__ void rows_trip(const uint8_t *stage, int shift, size_t rowbytes, int lr, int lane, int nq,
                                          const float (&xv)[NXV][8], const float (&sxo)[NXV], float *out,
                                          const float *add, int row0, float &best_v, int &best_i) {
    constexpr int BB = BlockTraits<QT>::BYTES;
    const int doff = (lane >> 2) * BB;
    int row[RT];  // byte offset of the row in the stage
    float a[RT];
#pragma unroll
    for (int j = 0; j < RT; j++) {
        row[j] = shift + (lr + j * QWAVES) * (int)rowbytes;
        a[j] = 0.f;
    }
#pragma unroll
    for (int t = 0; t < NXV; t++) {
        const bool live = lane + t * WAVE < nq;
#pragma unroll
        for (int j = 0; j < RT; j++) {
            const int boff = row[j] + doff + t * 16 * BB;
            const float v = AL ? quarter_dot_at<QT>(stage, boff, lane & 3, xv[t], sxo[t])
                               : quarter_dot<QT>(stage + boff, stage + boff + 2 + (lane & 3) * BlockTraits<QT>::QUARTER, xv[t], sxo[t]);
            a[j] += live ? v : 0.f;
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the LDS reads of later rounds from piling up in registers
    }
#pragma unroll
    for (int j = 0; j < RT; j++) {
        a[j] = wave_sum(a[j]);
        const float v = add ? a[j] + add[lr + j * QWAVES] : a[j];
        if (lane == 0) out[lr + j * QWAVES] = v;
        // of equal maxima the later row wins (Rust Iterator::max_by, reference src/generate.rs:735-742)
        if (best_i < 0 || v >= best_v) {
            best_v = v;
            best_i = row0 + lr + j * QWAVES;
        }
    }
}

// CPL = quarter columns per lane held in registers (ceil(K/8/64)); 0 = re-read them from LDS.
template <int QT, int CPL, bool FUSED>
__global__ __launch_bounds__(QTHREADS) void gemv_quant_kernel(
    const float *__restrict__ x, const uint8_t *__restrict__ w, float *__restrict__ out, int K,
    int N, int rows_per_step, const homura::QuantFuse fuse_arg) {
    // FUSED = false is the plain product: every pointer of the fusion record reads as null at compile time
    const homura::QuantFuse fuse = FUSED ? fuse_arg : homura::QuantFuse();
    constexpr int BB = BlockTraits<QT>::BYTES;
    constexpr int U = STAGE_U;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    float *xs = reinterpret_cast<float *>(smem);
    uint8_t *ws = smem + (size_t)K * 4;

    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int nb = K / 32, nq = K / 8;
    constexpr bool resident = CPL > 0;
    constexpr int NXV = resident ? CPL : 1;
    const size_t rowbytes = (size_t)nb * BB;
    const int nsteps = (N + rows_per_step - 1) / rows_per_step;

    // Loads return in issue order: the (small, cached) activation loads go first, the first step's
    // weights right behind them, so staging the activations does not wait for HBM.
    constexpr int XU = 4;  // covers K <= 4096 in one round
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 xr[XU], ar[XU], nr[XU];  // activation; second operand (x2 or res_in); norm weight
    const float *second = fuse.x2 ? fuse.x2 : fuse.res_in;
#pragma unroll
    for (int u = 0; u < XU; u++) {
        const int k = (tid + u * QTHREADS) * 4;
        xr[u] = k < K ? *reinterpret_cast<const f32x4 *>(x + k) : zero4;
        ar[u] = second && k < K ? *reinterpret_cast<const f32x4 *>(second + k) : zero4;
        nr[u] = fuse.norm_w && k < K ? *reinterpret_cast<const f32x4 *>(fuse.norm_w + k) : zero4;
    }
    u32x4 tmp[U];
    int step = blockIdx.x;
    StepRange cur = step_range(step, rows_per_step, N, rowbytes);
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int i = tid + u * QTHREADS;
        tmp[u] = i < cur.nchunks ? ld128_stream(w + cur.abeg + (size_t)i * 16) : u32x4{0u, 0u, 0u, 0u};
    }
    // the light ops of the quantised plan that sit in front of this product (the host allows the
    // norm only for K <= XU * 1024, where the whole row is in xr)
    if (fuse.x2) {
#pragma unroll
        for (int u = 0; u < XU; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) xr[u][e] = (xr[u][e] / (1.0f + expf(-xr[u][e]))) * ar[u][e];
    } else if (fuse.res_in) {
#pragma unroll
        for (int u = 0; u < XU; u++) {
            xr[u] += ar[u];
            const int k = (tid + u * QTHREADS) * 4;
            if (fuse.resid_out && blockIdx.x == 0 && k < K) *reinterpret_cast<f32x4 *>(fuse.resid_out + k) = xr[u];
        }
    }
    if (fuse.norm_w) {
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < XU; u++) ss += (xr[u][0] * xr[u][0] + xr[u][1] * xr[u][1]) + (xr[u][2] * xr[u][2] + xr[u][3] * xr[u][3]);
        ss = wave_sum(ss);
        float *red = reinterpret_cast<float *>(ws);  // the weight stage is not in use yet
        if (lane == 0) red[wave] = ss;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weight loads stay in flight
        float tot = 0.f;
#pragma unroll
        for (int wv = 0; wv < QWAVES; wv++) tot += red[wv];
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // red is read before ws is written
        const float inv = 1.0f / sqrtf(tot / (float)K + fuse.eps);
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
    for (int k = (tid + XU * QTHREADS) * 4; k < K; k += QTHREADS * 4) {  // longer rows (no norm here)
        f32x4 v = *reinterpret_cast<const f32x4 *>(x + k);
        if (fuse.x2) {
            const f32x4 o = *reinterpret_cast<const f32x4 *>(fuse.x2 + k);
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = (v[e] / (1.0f + expf(-v[e]))) * o[e];
        } else if (fuse.res_in) {
            v += *reinterpret_cast<const f32x4 *>(fuse.res_in + k);
            if (fuse.resid_out && blockIdx.x == 0) *reinterpret_cast<f32x4 *>(fuse.resid_out + k) = v;
        }
        *reinterpret_cast<f32x4 *>(xs + k) = v;
    }
    __syncthreads();
    float xv[NXV][8], sxo[NXV];
    if (resident) {
#pragma unroll
        for (int t = 0; t < NXV; t++) {
            const int c = min(lane + t * WAVE, nq - 1);  // lanes past the row end hold unused values
            load_xv<QT>(xs, c, xv[t], sxo[t]);
        }
    }

    float best_v = -INFINITY;
    int best_i = -1;
    for (; step < nsteps; step += gridDim.x) {
        __syncthreads();  // previous step's readers are done with ws
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = tid + u * QTHREADS;
            if (i < cur.nchunks) *reinterpret_cast<u32x4 *>(ws + (size_t)i * 16) = tmp[u];
        }
        __syncthreads();
        const StepRange now = cur;
        // the next step's weights travel while this one is multiplied
        if (step + (int)gridDim.x < nsteps) {
            cur = step_range(step + gridDim.x, rows_per_step, N, rowbytes);
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int i = tid + u * QTHREADS;
                tmp[u] = i < cur.nchunks ? ld128_stream(w + cur.abeg + (size_t)i * 16) : u32x4{0u, 0u, 0u, 0u};
            }
        }

        const uint8_t *base = ws + now.shift;
        const float *add = fuse.res_out_add ? fuse.res_out_add + now.r0 : nullptr;
        if (resident) {
            // up to four rows per trip: independent chains for the LDS reads and the reductions
            int lr = wave;
            for (; lr + 3 * QWAVES < now.nrows; lr += 4 * QWAVES)
                rows_trip<QT, NXV, 4, FUSED>(ws, now.shift, rowbytes, lr, lane, nq, xv, sxo, out + now.r0, add, now.r0, best_v, best_i);
            if (lr + QWAVES < now.nrows) {
                rows_trip<QT, NXV, 2, FUSED>(ws, now.shift, rowbytes, lr, lane, nq, xv, sxo, out + now.r0, add, now.r0, best_v, best_i);
                lr += 2 * QWAVES;
            }
            if (lr < now.nrows) rows_trip<QT, NXV, 1, FUSED>(ws, now.shift, rowbytes, lr, lane, nq, xv, sxo, out + now.r0, add, now.r0, best_v, best_i);
        } else {  // long rows: the activations of a column are re-read from LDS
            float acc[MAX_ROWS_PER_WAVE];
#pragma unroll
            for (int i = 0; i < MAX_ROWS_PER_WAVE; i++) acc[i] = 0.f;
            for (int c = lane; c < nq; c += WAVE) {
                float xc[8], so;
                load_xv<QT>(xs, c, xc, so);
#pragma unroll
                for (int i = 0; i < MAX_ROWS_PER_WAVE; i++) {
                    const int lr = wave + QWAVES * i;
                    if (lr < now.nrows)
                        {
                        const uint8_t *blk = base + (size_t)lr * rowbytes + (c >> 2) * BB;
                        acc[i] += quarter_dot<QT>(blk, blk + 2 + (c & 3) * BlockTraits<QT>::QUARTER, xc, so);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < MAX_ROWS_PER_WAVE; i++) {
                const int lr = wave + QWAVES * i;
                const float dot = wave_sum(acc[i]);
                if (lr < now.nrows) {
                    const float v = add ? dot + add[lr] : dot;
                    if (lane == 0) out[now.r0 + lr] = v;
                    if (best_i < 0 || v >= best_v) {
                        best_v = v;
                        best_i = now.r0 + lr;
                    }
                }
            }
        }
    }
    if (fuse.cand_v) {  // the workgroup's best row: largest value, highest index among equals; -1 = no row
        __syncthreads();
        float *cv = reinterpret_cast<float *>(ws);
        int *ci = reinterpret_cast<int *>(ws) + QWAVES;
        if (lane == 0) {
            cv[wave] = best_v;
            ci[wave] = best_i;
        }
        __syncthreads();
        if (tid == 0) {
            float bv = -INFINITY;
            int bi = -1;
            for (int wv = 0; wv < QWAVES; wv++) {
                if (ci[wv] < 0) continue;
                if (bi < 0 || cv[wv] > bv || (cv[wv] == bv && ci[wv] > bi)) {
                    bv = cv[wv];
                    bi = ci[wv];
                }
            }
            fuse.cand_v[blockIdx.x] = bv;
            fuse.cand_i[blockIdx.x] = bi;
        }
    }
}

// One thread per element; a single f32 multiply per element so the result is the same bits
// the CPU produces (reference src/gguf.rs:825-829).
template <int QT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t *__restrict__ blocks,
                                                      float *__restrict__ out, size_t n_elems) {
    constexpr int QF = QT == 0 ? homura::QF_Q8_0 : homura::QF_Q4_0;
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; e < n_elems; e += stride)
        out[e] = homura::dequant_element<QF>(blocks + (e >> 5) * BlockTraits<QT>::BYTES, (int)(e & 31));
}

// Rows staged per step, LDS and grid of gemv_quant_kernel for a shape.
struct QuantShape {
    int rows, grid;
    size_t lds;
};
template <int QT>
QuantShape quant_shape(const hm_ctx *ctx, int K, int N) {
    constexpr int BB = BlockTraits<QT>::BYTES;
    const size_t rowbytes = (size_t)(K / 32) * BB, x_bytes = (size_t)K * 4, lds_budget = 48 * 1024;
    // rows staged per step: as many as fit the LDS budget (at most 8 per wavefront), but few
    // enough that every CU gets a workgroup
    int rows = (int)((lds_budget - x_bytes) / rowbytes);
    rows = rows / QWAVES * QWAVES;
    if (rows < QWAVES) rows = QWAVES;
    if (rows > QWAVES * MAX_ROWS_PER_WAVE) rows = QWAVES * MAX_ROWS_PER_WAVE;
    while (rows > QWAVES && (size_t)rows * rowbytes + 32 > (size_t)STAGE_BYTES) rows -= QWAVES;
    while (rows > QWAVES && (N + rows - 1) / rows < 2 * ctx->num_cus) rows -= QWAVES;
    QuantShape sh;
    sh.rows = rows;
    sh.lds = x_bytes + (size_t)rows * rowbytes + 32 + 16 * BB;  // slack: see rows_trip
    const int nsteps = (N + rows - 1) / rows;
    // persistent workgroups: a few per CU, each stages the activations once
    int wg_per_cu = (int)(120 * 1024 / sh.lds);
    if (wg_per_cu < 1) wg_per_cu = 1;
    if (wg_per_cu > 6) wg_per_cu = 6;
    sh.grid = nsteps < ctx->num_cus * wg_per_cu ? nsteps : ctx->num_cus * wg_per_cu;
    return sh;
}

template <int QT>
int gemv_quant_launch(hm_ctx *ctx, const char *name, const float *d_x, const uint8_t *d_w,
                      float *d_out, int M, int K, int N, const homura::QuantFuse &fuse = homura::QuantFuse()) {
    HM_CHECK_CTX(ctx);
    constexpr int BB = BlockTraits<QT>::BYTES;
    HM_REQUIRE(ctx, d_x && d_w && d_out, "%s: NULL pointer", name);
    HM_REQUIRE(ctx, M >= 1 && M <= 8, "%s: M=%d outside 1..8", name, M);
    HM_REQUIRE(ctx, K > 0 && K % 32 == 0 && N > 0, "%s: K=%d must be a positive multiple of 32, N=%d positive", name, K, N);
    HM_REQUIRE(ctx, ((uintptr_t)d_w % 16) == 0 && ((uintptr_t)d_x % 16) == 0, "%s: weight and activation buffers must be 16-byte aligned", name);
    HM_REQUIRE(ctx, !(fuse.x2 && fuse.res_in), "%s: SiLU pair and residual input exclude each other", name);
    HM_REQUIRE(ctx, !fuse.norm_w || K <= 4096, "%s: the fused RMSNorm holds rows up to 4096 wide (K=%d)", name, K);
    HM_REQUIRE(ctx, ((uintptr_t)fuse.x2 % 16) == 0 && ((uintptr_t)fuse.res_in % 16) == 0 && ((uintptr_t)fuse.resid_out % 16) == 0 &&
                        ((uintptr_t)fuse.norm_w % 16) == 0, "%s: fused operands must be 16-byte aligned", name);
    HM_REQUIRE(ctx, M == 1 || (!fuse.x2 && !fuse.res_in && !fuse.norm_w && !fuse.res_out_add), "%s: fused light ops need M == 1", name);
    const size_t rowbytes = (size_t)(K / 32) * BB;
    const size_t x_bytes = (size_t)K * 4;
    if (!(x_bytes + QWAVES * rowbytes + 32 <= 64 * 1024 && QWAVES * rowbytes + 32 <= (size_t)STAGE_BYTES)) {
        // Rows too long for the LDS stage (above about 7700 for Q8_0, 14500 for Q4_0): the blocks are re-packed
        // into planes in the workspace and multiplied by the cut-row kernel, two launches a call. (A caller that
        // keeps its weights on the device packs them once and calls the planes entry points.)
        const size_t need = homura::quant_planes_bytes(QT == 1, N, K);
        HM_REQUIRE(ctx, K <= 16384 && need <= ctx->workspace_bytes && !fuse.norm_w && !fuse.cand_v,
                   "%s: K=%d too large for the LDS stage (and %zu bytes of planes do not fit the workspace, or a norm / "
                   "argmax rides along)", name, K, need);
        uint8_t *planes = static_cast<uint8_t *>(ctx->workspace);
        int rc = homura::pack_quant_planes(ctx, QT == 1, d_w, planes, N, K);
        for (int m = 0; m < M && rc == HM_OK; m++)
            rc = homura::gemv_planes_fused(ctx, QT == 1, d_x + (size_t)m * K, planes, d_out + (size_t)m * N, K, N, fuse);
        return rc;
    }
    const QuantShape sh = quant_shape<QT>(ctx, K, N);
    const int rows = sh.rows, grid = sh.grid;
    const size_t lds = sh.lds;
    HM_REQUIRE(ctx, !fuse.cand_v || fuse.cand_i, "%s: argmax candidates need an index buffer", name);
    const int cpl = (K / 8 + WAVE - 1) / WAVE;
    const bool fused = fuse.x2 || fuse.res_in || fuse.norm_w || fuse.res_out_add || fuse.cand_v;
    for (int m = 0; m < M; m++) {
        const float *xm = d_x + (size_t)m * K;
        float *om = d_out + (size_t)m * N;
#define HM_QUANT_CASE(C)                                                                                  \
    do {                                                                                                  \
        if (fused)                                                                                        \
            hipLaunchKernelGGL((gemv_quant_kernel<QT, C, true>), dim3(grid), dim3(QTHREADS), lds, ctx->stream, xm, \
                               d_w, om, K, N, rows, fuse);                                                \
        else                                                                                              \
            hipLaunchKernelGGL((gemv_quant_kernel<QT, C, false>), dim3(grid), dim3(QTHREADS), lds, ctx->stream, xm, \
                               d_w, om, K, N, rows, fuse);                                                \
    } while (0)
        switch (cpl <= MAXC ? cpl : 0) {
            case 1: HM_QUANT_CASE(1); break;
            case 2: HM_QUANT_CASE(2); break;
            case 3: HM_QUANT_CASE(3); break;
            case 4: HM_QUANT_CASE(4); break;
            case 5: HM_QUANT_CASE(5); break;
            case 6: HM_QUANT_CASE(6); break;
            case 7: HM_QUANT_CASE(7); break;
            case 8: HM_QUANT_CASE(8); break;
            default: HM_QUANT_CASE(0); break;
        }
#undef HM_QUANT_CASE
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

int homura::gemv_quant_workgroups(const hm_ctx *ctx, bool q4, int K, int N) {
    return q4 ? quant_shape<1>(ctx, K, N).grid : quant_shape<0>(ctx, K, N).grid;
}

int homura::gemv_quant_fused(hm_ctx *ctx, bool q4, const float *d_x, const uint8_t *d_w, float *d_out, int K, int N,
                             const QuantFuse &fuse) {
    return q4 ? gemv_quant_launch<1>(ctx, "gemv_quant[q4_0]", d_x, d_w, d_out, 1, K, N, fuse)
              : gemv_quant_launch<0>(ctx, "gemv_quant[q8_0]", d_x, d_w, d_out, 1, K, N, fuse);
}

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
