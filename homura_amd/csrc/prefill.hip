// Multi-token (prefill) kernels: row-wise ops that hand f32 activations to the MFMA GEMM as split
// bf16 matrices, the tail of the QKV kernel for a block of positions, and a causal GQA attention
// on the matrix cores.
//
// Attention works on the transposed problem so that softmax statistics stay inside a lane:
//   S^T[key][q] = K[key][:] . Q[q][:]      (A operand = K rows from LDS, B operand = Q in registers)
//   O^T[d][q]   = V^T[d][:] . P^T[:][q]    (A operand = V^T from LDS, B operand = P in registers)
// With v_mfma_f32_16x16x32_bf16 a lane owns one query column of the result tile (lane % 16) and four of
// its 16 rows, so the running maximum and the rescaling factor of a query are per-lane scalars; the four
// lanes of a query exchange one maximum per key tile. The probabilities leave the S^T accumulators and
// enter the second product without touching LDS (the contraction slots of the second product are numbered
// the way the scores arrive; see the kernel).
// Queries and probabilities are f32 carried as two or three bf16 pieces each (see prefill.h); K and
// V are the cache's own bf16 rows.
#include "prefill.h"
#include "bf16_pieces.h"

#include <algorithm>
#include <cstdlib>

#include "gemm_bf16_mfma.h"
#include "gemm_kquant_i8.h"
#include "quant_formats.h"

namespace {

using namespace homura;

typedef float f32x16 __attribute__((ext_vector_type(16)));

// element c of a split row: piece p goes to column p * dim + c
__device__ __forceinline__ void split_store(uint16_t *__restrict__ row, int dim, int c, float x, int pieces) {
    uint32_t p[3];
    split_pieces<3>(x, p);
    row[c] = (uint16_t)p[0];
    if (pieces > 1) row[dim + c] = (uint16_t)p[1];
    if (pieces > 2) row[2 * dim + c] = (uint16_t)p[2];
}

__global__ void split_rows_kernel(const float *__restrict__ x, uint16_t *__restrict__ out, int dim, size_t n,
                                  int pieces) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t row = i / dim;
    split_store(out + row * pieces * dim, dim, (int)(i % dim), x[i], pieces);
}

// A GEMM result that was cut along K: the slices added in index order
// Sum of the K slices of a projection result, in slice order. Every slice is requested before the first is used:
// a loop of loads waits for each in turn, eight trips to memory at eight slices.
constexpr int MAX_SUM_PARTS = 8;
template <int MAXP, class V>
__device__ __forceinline__ V sum_parts_upto(const float *__restrict__ p, size_t i, int parts, size_t stride) {
    V t[MAXP];
#pragma unroll
    for (int s = 0; s < MAXP; s++) t[s] = *reinterpret_cast<const V *>(p + i + (size_t)(s < parts ? s : 0) * stride);
    V v = t[0];
#pragma unroll
    for (int s = 1; s < MAXP; s++)
        if (s < parts) v += t[s];
    return v;
}
template <class V>
__device__ __forceinline__ V sum_parts_as(const float *__restrict__ p, size_t i, int parts, size_t stride) {
    if (parts == 1) return *reinterpret_cast<const V *>(p + i);
    if (parts <= 2) return sum_parts_upto<2, V>(p, i, parts, stride);
    if (parts <= 4) return sum_parts_upto<4, V>(p, i, parts, stride);
    return sum_parts_upto<MAX_SUM_PARTS, V>(p, i, parts, stride);
}
__device__ __forceinline__ float sum_parts(const float *__restrict__ p, size_t i, int parts, size_t stride) {
    return sum_parts_as<float>(p, i, parts, stride);
}
__device__ __forceinline__ f32x4 sum_parts4(const float *__restrict__ p, size_t i, int parts, size_t stride) {
    return sum_parts_as<f32x4>(p, i, parts, stride);
}

// elements c .. c+3 of a split row
__device__ __forceinline__ void split_store4(uint16_t *__restrict__ row, int dim, int c, f32x4 x, int pieces) {
    uint32_t lo[3], hi[3];
    split_pair<3>(x[0], x[1], lo);
    split_pair<3>(x[2], x[3], hi);
    for (int k = 0; k < pieces; k++) {
        u32x2 w;
        w.x = lo[k];
        w.y = hi[k];
        *reinterpret_cast<u32x2 *>(row + (size_t)k * dim + c) = w;
    }
}

// The activation a K-quant product sees (reference emit_quant.rs:422-466): every 256-wide block is
// quantised to Q8_K, q = clamp(roundeven(x * (127 / amax)), +-127) with scale amax / 127; the integer
// dot products of the decode kernels equal a plain dot product with scale * q. A wavefront holds one
// block, four consecutive values per lane.
__device__ __forceinline__ f32x4 q8k_round_trip(f32x4 v) {
    float d, r[4];
    (void)q8k_quantize4(v, d, r);
    f32x4 y;
#pragma unroll
    for (int k = 0; k < 4; k++) y[k] = __fmul_rn(d, r[k]);
    return y;
}

// rows of f32 -> split rows, four consecutive elements per thread (dim % 4 == 0; % 256 with q8k)
__global__ void split_rows4_kernel(const float *__restrict__ x, uint16_t *__restrict__ out, int dim, size_t n, int pieces,
                                   int q8k) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= n) return;
    f32x4 v = *reinterpret_cast<const f32x4 *>(x + i);
    if (q8k) v = q8k_round_trip(v);
    const size_t row = i / dim;
    split_store4(out + row * pieces * dim, dim, (int)(i % dim), v, pieces);
}

// A quantised weight matrix, raw blocks [N][K / block], as a split matrix of its f32 values: row n goes
// to row n * row_mult + row_off of out ([.][3 K]). Eight consecutive weights per thread.
template <int QF>
__global__ __launch_bounds__(256) void dequant_split_kernel(const uint8_t *__restrict__ blocks,
                                                            uint16_t *__restrict__ out, int K, size_t n8, int row_mult,
                                                            int row_off) {
    constexpr int BB = QuantFormatTraits<QF>::BYTES, BE = QuantFormatTraits<QF>::ELEMS;
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n8) return;
    const size_t e = t * 8, row = e / K;
    const int c = (int)(e % K);
    const uint8_t *blk = blocks + (e / BE) * BB;  // rows are whole blocks: K % BE == 0
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; j++) f[j] = dequant_element<QF>(blk, (int)(e % BE) + j);
    bf16x8 pc[3];
    split8<3>(f, pc);
    uint16_t *o = out + (row * row_mult + row_off) * 3 * (size_t)K + c;
#pragma unroll
    for (int p = 0; p < 3; p++) *reinterpret_cast<bf16x8 *>(o + (size_t)p * K) = pc[p];
}

// A Q8_0 / Q4_0 matrix as its integers (bf16, exact) and its block scales: row n goes to row n * row_mult +
// row_off of ints ([.][K]) and to that column of scales ([K / 32][npad] f32). Eight consecutive weights per
// thread. The weight is scale * integer (reference src/gguf.rs:825-833; Q4_0: nibble - 8).
template <int QF>
__global__ __launch_bounds__(256) void quant_ints_kernel(const uint8_t *__restrict__ blocks, uint16_t *__restrict__ ints,
                                                         float *__restrict__ scales, int K, size_t n8, int npad,
                                                         int row_mult, int row_off) {
    constexpr int BB = QuantFormatTraits<QF>::BYTES;
    static_assert(QF == QF_Q8_0 || QF == QF_Q4_0, "32-wide blocks with one scale");
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n8) return;
    const size_t e = t * 8, row = e / K, orow = row * row_mult + row_off;
    const int c = (int)(e % K), j0 = c % 32;
    const uint8_t *blk = blocks + (e / 32) * BB;
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        if (QF == QF_Q8_0) {
            f[j] = (float)(int8_t)blk[2 + j0 + j];
        } else {
            const uint8_t byte = blk[2 + (j0 + j) % 16];
            f[j] = (float)((j0 + j < 16 ? (byte & 0x0F) : (byte >> 4)) - 8);
        }
    }
    bf16x8 pc[1];
    split8<1>(f, pc);  // integers of at most 8 bits: the bf16 is exact
    *reinterpret_cast<bf16x8 *>(ints + orow * (size_t)K + c) = pc[0];
    if (j0 == 0) scales[(size_t)(c / 32) * npad + orow] = f16_at(blk);
}

// One workgroup per row, four consecutive elements per thread and step (dim % 4 == 0); the arithmetic
// of the decode path's RMSNorm kernel (reference src/graph_builder/emit_linalg.rs:7-26; Residual+Norm,
// src/hf/emitter.rs:787-790).
__global__ __launch_bounds__(256) void rmsnorm_split_kernel(const float *__restrict__ x, const float *__restrict__ res,
                                                            int res_parts, size_t res_stride,
                                                            const float *__restrict__ w, uint16_t *__restrict__ out,
                                                            float *__restrict__ resid_out, int dim, float eps,
                                                            int pieces, int q8k, float *__restrict__ pre_q8k,
                                                            int8_t *__restrict__ q8, float *__restrict__ q8_scale) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * dim;
    constexpr int KEEP = 2;  // rows up to 2048 wide stay in registers between the two passes
    f32x4 keep[KEEP];
    float ss = 0.f;
    int at = 0;
    for (int i = threadIdx.x * 4; i < dim; i += 1024, at++) {
        f32x4 v = *reinterpret_cast<const f32x4 *>(x + base + i);
        if (res) v += sum_parts4(res, base + i, res_parts, res_stride);
        if (resid_out) *reinterpret_cast<f32x4 *>(resid_out + base + i) = v;
        if (at < KEEP) keep[at] = v;
        ss += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv = 1.0f / sqrtf(tot / (float)dim + eps);
    uint16_t *o = out + (size_t)blockIdx.x * pieces * dim;
    at = 0;
    for (int i = threadIdx.x * 4; i < dim; i += 1024, at++) {
        f32x4 v;
        if (at < KEEP) {
            v = keep[at];
        } else {
            v = *reinterpret_cast<const f32x4 *>(x + base + i);
            if (res) v += sum_parts4(res, base + i, res_parts, res_stride);
        }
        const f32x4 wv = *reinterpret_cast<const f32x4 *>(w + i);
        f32x4 y;
#pragma unroll
        for (int k = 0; k < 4; k++) y[k] = (v[k] * inv) * wv[k];
        if (pre_q8k) *reinterpret_cast<f32x4 *>(pre_q8k + base + i) = y;
        if (q8) {  // the Q8_K row itself, for the integer matrix cores (dim % 256 == 0: a wavefront's 256 values are one block)
            float d;
            *reinterpret_cast<uint32_t *>(q8 + base + i) = q8k_quantize4(y, d);
            if ((threadIdx.x & 63) == 0) q8_scale[(base + i) / 256] = d;
            continue;
        }
        if (q8k) y = q8k_round_trip(y);
        split_store4(o, dim, i, y, pieces);
    }
}

// silu(gate) * up (reference src/graph_builder/emit_arithmetic.rs:101-107, src/hf/emitter.rs:797-799);
// four outputs per thread (inter % 4 == 0)
__global__ void silu_mul_split_kernel(const float *__restrict__ gu, int parts, size_t stride, uint16_t *__restrict__ out,
                                      int inter, size_t n, int pieces, int q8k, float *__restrict__ pre_q8k,
                                      int8_t *__restrict__ q8, float *__restrict__ q8_scale) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= n) return;
    const size_t row = i / inter;
    const f32x4 a = sum_parts4(gu, 2 * i, parts, stride), b = sum_parts4(gu, 2 * i + 4, parts, stride);
    const float g[4] = {a[0], a[2], b[0], b[2]}, u[4] = {a[1], a[3], b[1], b[3]};
    f32x4 y;
#pragma unroll
    for (int k = 0; k < 4; k++) y[k] = (g[k] / (1.0f + expf(-g[k]))) * u[k];
    if (pre_q8k) *reinterpret_cast<f32x4 *>(pre_q8k + i) = y;
    if (q8) {
        float d;
        *reinterpret_cast<uint32_t *>(q8 + i) = q8k_quantize4(y, d);
        if ((threadIdx.x & 63) == 0) q8_scale[i / 256] = d;
        return;
    }
    if (q8k) y = q8k_round_trip(y);
    split_store4(out + row * pieces * inter, inter, (int)(i % inter), y, pieces);
}

// One wavefront per (position, head) row of q, k or v.
__global__ __launch_bounds__(256) void qkv_post_kernel(QkvPostArgs a) {
    const int lane = threadIdx.x & 63;
    const int per_pos = a.H + 2 * a.kvh;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= a.S * per_pos) return;
    const int s = r / per_pos, j = r % per_pos;
    const int hd = a.hd, half = hd / 2;
    const int pos = a.past + s;
    float *x = a.qkv + (size_t)s * per_pos * hd + (size_t)j * hd;
    const float *b = a.bias ? a.bias + (size_t)j * hd : nullptr;
    // element i of the row: the K slices of the projection added up, then the bias
    auto elem = [&](int i) {
        const float v = sum_parts(x, (size_t)i, a.parts, a.part_stride);
        return b ? v + b[i] : v;
    };

    if (j >= a.H + a.kvh) {  // a v row: bias, then the cache append
        uint16_t *dst = a.vcache + ((size_t)(j - a.H - a.kvh) * a.max_len + pos) * hd;
        for (int i = lane; i < hd; i += 64) dst[i] = f32_to_bf16_rne_dev(elem(i));
        return;
    }
    const bool is_q = j < a.H;
    const float *nw = is_q ? a.qw : a.kw;
    const float *c = a.cos_tab + (size_t)pos * hd;
    const float *sn = a.sin_tab + (size_t)pos * hd;
    float lo[2], hi[2];  // hd <= 256
    float ss = 0.f;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int i = lane + 64 * t;
        lo[t] = i < half ? elem(i) : 0.f;
        hi[t] = i < half ? elem(i + half) : 0.f;
        ss += lo[t] * lo[t] + hi[t] * hi[t];
    }
    if (nw) {
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)hd + a.eps);
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const int i = lane + 64 * t;
            if (i < half) {
                lo[t] = (lo[t] * inv) * nw[i];
                hi[t] = (hi[t] * inv) * nw[i + half];
            }
        }
    }
    uint16_t *kdst = is_q ? nullptr : a.kcache + ((size_t)(j - a.H) * a.max_len + pos) * hd;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int i = lane + 64 * t;
        if (i < half) {
            const float o_lo = lo[t] * c[i] + (-hi[t]) * sn[i];
            const float o_hi = hi[t] * c[i + half] + lo[t] * sn[i + half];
            if (is_q) {
                x[i] = o_lo;
                x[i + half] = o_hi;
            } else {
                kdst[i] = f32_to_bf16_rne_dev(o_lo);
                kdst[i + half] = f32_to_bf16_rne_dev(o_hi);
            }
        }
    }
}

// ── causal attention ─────────────────────────────────────────────────────────

// K / V tile in LDS: row = key, HD * 2 bytes, 16-byte chunk c of row r at slot c ^ (swizzle of r): conflict-free
// for the operand reads (16 consecutive rows, one chunk)
template <int HD>
__device__ __forceinline__ int k_off(int key, int chunk) {
    if (HD == 128) return key * 256 + ((chunk ^ (key & 15)) << 4);
    return key * 128 + ((chunk ^ (key & 7) ^ ((key >> 3) & 7)) << 4);
}

// V tile: the transposing reads of a group of 16 lanes take 32 contiguous bytes (two chunks) from each of four
// neighbouring rows, and a pass of the LDS serves two such groups: the swizzle moves chunk PAIRS, by the row's
// low three bits, so that eight neighbouring rows land on eight different bank groups.
template <int HD>
__device__ __forceinline__ int v_off(int key, int chunk) {
    if (HD == 128) return key * 256 + (((((chunk >> 1) ^ (key & 7)) << 1) | (chunk & 1)) << 4);
    return k_off<HD>(key, chunk);
}

extern __shared__ __attribute__((aligned(16))) char at_lds[];

// 16 query rows per wavefront (v_mfma_f32_16x16x32_bf16) and eight wavefronts a workgroup: 8 / KS blocks of 16
// rows times KS key groups (with KS > 1 the wavefronts of a row block take every KS-th key tile each and their
// partial softmax sums meet in LDS at the end; KS = 1: 128 rows per workgroup, the fewest tile loads; KS = 2, 4:
// 64, 32 rows, for prompts whose rows x heads alone leave most of the chip idle). A wavefront needs ~150
// registers, so two or three share a SIMD and one's matrix instructions run under the others' softmax arithmetic.
// K and V tiles (32 keys) go global -> LDS directly (global_load_lds_dwordx4, no staging registers, no LDS
// write instructions), row-major and XOR-swizzled on the global side; two sets of KS tile pairs alternate, the
// next round's tiles arrive while this round is multiplied.
//   S^T block: A = 16 keys x 32 dims from the K tile, B = the queries' pieces; lane q + 16 c receives keys
//   4 c .. 4 c + 3 of the block for query q.
//   O^T block: A = 16 dims x 32 keys, B = the probabilities' pieces. Contraction slot 8 c + i (i < 4) stands
//   for key 4 c + i of the tile, slot 8 c + 4 + i for key 16 + 4 c + i: exactly the eight scores lane q + 16 c
//   holds from the tile's two key blocks, so the probabilities never leave their lanes. V^T comes out of the
//   row-major V tile through the transposing LDS read (ds_read_b64_tr_b16: lane l of a group of 16 receives
//   element l % 4 of the 8 bytes that lanes l / 4, 4 + l / 4, 8 + l / 4, 12 + l / 4 point at): lane i points at
//   dims 16 db + 4 (i % 4) .. + 3 of key 4 c + i / 4, and receives dim 16 db + i of keys 4 c .. 4 c + 3.
constexpr int A8_THREADS = 512;
constexpr int A8_WAVES = A8_THREADS / 64;
constexpr int A8_KEYS = 32;  // keys per tile

typedef short s16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void dma16_lds(const uint16_t *src, char *dst) {
    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)src,
                                     (void __attribute__((address_space(3))) *)dst, 16, 0, 0);
}

// max / sum over the four lanes l16 + 16 c of a wavefront, every lane receives it: the row swaps of gfx950
// (odd rows of one operand against even rows of the other, then the upper half against the lower) instead of
// two trips through the LDS crossbar
__device__ __forceinline__ float quad_rows_max(float x) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    const float m = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(m), __float_as_uint(m), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_rows_sum(float x) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    const float m = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(m), __float_as_uint(m), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

template <int HD, int NP, int KS>
__global__ __launch_bounds__(A8_THREADS) void prefill_attn16_kernel(PrefillAttnArgs a) {
    constexpr int CH = HD / 8;                         // 16-byte chunks per row
    constexpr int KSTEPS = HD / 32;                    // k steps of K . Q
    constexpr int DB = HD / 16;                        // 16-row blocks of O^T
    constexpr int QW = A8_WAVES / KS;                  // 16-row query blocks per workgroup
    constexpr int AT_QROWS = 16 * QW;
    constexpr int TILE = A8_KEYS * HD * 2;             // bytes of a K or V tile
    constexpr int SET = KS * 2 * TILE;                 // the KS tile pairs of a round
    constexpr int ROWS_PER_DMA = 1024 / (HD * 2);      // rows one wavefront-wide 16-byte-per-lane load fills
    constexpr int DMA_WAVES = A8_KEYS / ROWS_PER_DMA;  // wavefronts that fill a tile (8 or 4)
    static_assert(DMA_WAVES <= A8_WAVES, "head_dim 64 or 128");

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l16 = lane & 15, c4 = lane >> 4;
    const int qw = wave % QW, kh = wave / QW;  // row block and key group of this wavefront
    // Workgroups are dealt to the eight dies round-robin by their linear index. With a multiple of eight heads
    // every die gets H / 8 neighbouring heads and all their row blocks, so the K and V rows of a KV head are
    // fetched into one die's L2 (or as few as the head grouping allows) instead of all eight.
    int hx = blockIdx.y, bx = blockIdx.x;
    if (a.H % 8 == 0) {
        const int lin = blockIdx.y * gridDim.x + blockIdx.x, per = a.H / 8;
        hx = (lin & 7) * per + (lin >> 3) % per;
        bx = (lin >> 3) / per;
    }
    const int h = hx, kvhd = h / (a.H / a.kvh);
    const int q0 = bx * AT_QROWS;
    const int kv_total = a.past + a.S;
    const uint16_t *kc = a.kcache + (size_t)kvhd * a.max_len * HD;
    const uint16_t *vc = a.vcache + (size_t)kvhd * a.max_len * HD;

    const int wg_end = a.past + min(a.S, q0 + AT_QROWS);
    const int wave_end = q0 + qw * 16 < a.S ? a.past + min(a.S, q0 + qw * 16 + 16) : 0;
    const int ntiles = (wg_end + A8_KEYS - 1) / A8_KEYS;
    const int nrounds_all = (ntiles + KS - 1) / KS;
    // the rounds of this workgroup: all of them, or its share when the keys are cut over gridDim.z workgroups
    const int per_z = (nrounds_all + (int)gridDim.z - 1) / (int)gridDim.z;
    const int r_begin = (int)blockIdx.z * per_z, nrounds = min(nrounds_all, r_begin + per_z);
    const int wave_first = a.past + min(q0 + qw * 16, a.S - 1);

    // This lane's part of a tile load: row dma_row of the tile, the chunk that belongs in slot dma_slot.
    const int dma_row = wave * ROWS_PER_DMA + lane / CH, dma_slot = lane % CH;
    const int dma_chunk = (k_off<HD>(dma_row, dma_slot) - dma_row * HD * 2) >> 4;  // the swizzles are involutions
    const int dma_chunk_v = (v_off<HD>(dma_row, dma_slot) - dma_row * HD * 2) >> 4;
    const int wave_dst = __builtin_amdgcn_readfirstlane(wave * 1024);
    auto request_round = [&](int r) {
        if (wave >= DMA_WAVES) return;
        char *base = at_lds + (r & 1) * SET + wave_dst;
#pragma unroll
        for (int u = 0; u < KS; u++) {
            const int row = min((r * KS + u) * A8_KEYS + dma_row, kv_total - 1);
            dma16_lds(kc + (size_t)row * HD + dma_chunk * 8, base + u * 2 * TILE);
            dma16_lds(vc + (size_t)row * HD + dma_chunk_v * 8, base + u * 2 * TILE + TILE);
        }
    };
    // this lane's query (rows past the end repeat the last one and are not stored): dims 32 ks + 8 c4 .. + 7.
    // Asked for ahead of the first tiles (loads return in order): it is split into pieces while they arrive.
    const int qrow = q0 + qw * 16 + l16;
    const int qc = min(qrow, a.S - 1);
    const int qabs = a.past + qc;
    bf16x8 qp_[KSTEPS][NP];
    {
        const float qscale = a.scale * 1.44269504088896340736f;  // scores in units of ln 2: the softmax uses exp2
        const float *qp = a.q + (size_t)qc * a.ldq + (size_t)h * HD + c4 * 8;
        f32x4 x0[KSTEPS], x1[KSTEPS];
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            x0[ks] = *reinterpret_cast<const f32x4 *>(qp + 32 * ks);
            x1[ks] = *reinterpret_cast<const f32x4 *>(qp + 32 * ks + 4);
        }
        if (r_begin < nrounds) request_round(r_begin);  // (a tile load must not outlive the workgroup)
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            float f[8];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                f[i] = x0[ks][i] * qscale;
                f[4 + i] = x1[ks][i] * qscale;
            }
            split8<NP>(f, qp_[ks]);
        }
    }

    f32x4 acc_o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++) acc_o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    // transposing V reads: lane i of a group points at dims 4 (i % 4) .. + 3 of a 16-dim block, key 4 c4 + i / 4
    const int v_key = 4 * c4 + (l16 >> 2), v_sub = l16 & 3;

    for (int r = r_begin; r < nrounds; r++) {
        // this round's tiles have landed for this wavefront (nothing else is in flight), then for everybody,
        // and everybody is done with the other set
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (r + 1 < nrounds) request_round(r + 1);
        const int t = r * KS + kh;               // this wavefront's tile of the round
        if (t * A8_KEYS >= wave_end) continue;  // wavefront-uniform: nothing visible to these 16 rows
        const char *k_lds = at_lds + (r & 1) * SET + kh * 2 * TILE, *v_lds = k_lds + TILE;

        f32x4 s[2];  // key blocks of 16
        s[0] = s[1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            bf16x8 kf[2];
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
                kf[kb] = *reinterpret_cast<const bf16x8 *>(k_lds + k_off<HD>(16 * kb + l16, 4 * ks + c4));
#pragma unroll
            for (int p = NP - 1; p >= 0; p--)
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
                    s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kb], qp_[ks][p], s[kb], 0, 0, 0);
        }
        // value i of block kb belongs to key 16 kb + 4 c4 + i; only tiles that reach past the first row of
        // this wavefront need the causal mask
        if (t * A8_KEYS + A8_KEYS - 1 > wave_first) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int key = t * A8_KEYS + 16 * kb + 4 * c4 + i;
                    s[kb][i] = key > qabs ? -INFINITY : s[kb][i];
                }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int i = 0; i < 4; i++) mx = fmaxf(mx, s[kb][i]);
        mx = quad_rows_max(mx);
        // The reference point of the exponentials only has to be near the maximum, not on it (softmax is
        // shift-invariant and l, O are f32): it moves when the maximum has grown by more than 2^8, so after the
        // first tiles the rescaling of O is skipped for the whole wavefront. The four lanes of a query decide
        // alike. A row that has not seen a visible key yet (possible in key groups other than the first, whose
        // tiles may lie wholly in a row's future) gets a finite floor as its reference point, so that every
        // exponential below is 0 and not exp2(inf - inf).
        const float m_new = fmaxf(mx > m_run + 8.0f ? mx : m_run, -1e30f);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        float f[8], psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                f[4 * kb + i] = __builtin_amdgcn_exp2f(s[kb][i] - m_new);
                psum += f[4 * kb + i];
            }
        l_run = l_run * alpha + psum;  // this lane's quarter of the keys; the quarters meet at the end
        m_run = m_new;
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int db = 0; db < DB; db++) acc_o[db] *= alpha;
        }
        bf16x8 pp[NP];
        split8<NP>(f, pp);
#pragma unroll
        for (int db = 0; db < DB; db++) {
            const int chunk = 2 * db + (v_sub >> 1), within = (v_sub & 1) * 8;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (s16x4 __attribute__((address_space(3))) *)(v_lds + v_off<HD>(v_key, chunk) + within));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (s16x4 __attribute__((address_space(3))) *)(v_lds + v_off<HD>(16 + v_key, chunk) + within));
            struct Pair { s16x4 lo, hi; } pr{lo, hi};
            const bf16x8 vf = __builtin_bit_cast(bf16x8, pr);
#pragma unroll
            for (int p = NP - 1; p >= 0; p--)
                acc_o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pp[p], acc_o[db], 0, 0, 0);
        }
    }

    if (KS > 1) {
        // The key groups of a row block meet: groups 1 .. KS-1 leave (O, m, l) in LDS, lane-major, and group 0
        // adds them in group order, rescaled to the larger reference point (a group that saw no visible key has
        // m = -inf and weighs nothing; group 0 always sees key 0).
        constexpr int PER_LANE = DB * 4 + 2;
        float *xch = reinterpret_cast<float *>(at_lds);
        __syncthreads();  // nobody reads tiles any more (and no tile load is in flight: the last round requested none)
        if (kh > 0) {
            float *mine = xch + (size_t)((kh - 1) * QW + qw) * PER_LANE * 64 + lane;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int v = 0; v < 4; v++) mine[(db * 4 + v) * 64] = acc_o[db][v];
            mine[(DB * 4) * 64] = m_run;
            mine[(DB * 4 + 1) * 64] = l_run;
        }
        __syncthreads();
        if (kh > 0) return;
#pragma unroll
        for (int g = 1; g < KS; g++) {
            const float *other = xch + (size_t)((g - 1) * QW + qw) * PER_LANE * 64 + lane;
            const float m_o = other[(DB * 4) * 64], l_o = other[(DB * 4 + 1) * 64];
            const float m_new = fmaxf(fmaxf(m_run, m_o), -1e30f);  // (with the keys cut over workgroups group 0 may have seen none either)
            const float w_me = __builtin_amdgcn_exp2f(m_run - m_new), w_o = __builtin_amdgcn_exp2f(m_o - m_new);
            l_run = l_run * w_me + l_o * w_o;
            m_run = m_new;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int v = 0; v < 4; v++) acc_o[db][v] = acc_o[db][v] * w_me + other[(db * 4 + v) * 64] * w_o;
        }
    }
    const float l_tot = quad_rows_sum(l_run);
    if (qrow >= a.S) return;
    const int qd = a.H * HD;
    if (a.part_o) {  // this workgroup's share of the keys: (O, max, sum) as they are
        float *po = a.part_o + ((size_t)blockIdx.z * a.S + qrow) * qd + h * HD + 4 * c4;
#pragma unroll
        for (int db = 0; db < DB; db++) *reinterpret_cast<f32x4 *>(po + 16 * db) = acc_o[db];
        if (c4 == 0) {
            float *pm = a.part_ml + (((size_t)blockIdx.z * a.S + qrow) * a.H + h) * 2;
            pm[0] = m_run;
            pm[1] = l_tot;
        }
        return;
    }
    const float inv = 1.0f / l_tot;
    // value v of block db is d = 16 db + 4 c4 + v
#pragma unroll
    for (int db = 0; db < DB; db++) {
        const int d0 = h * HD + 16 * db + 4 * c4;
        f32x4 o = acc_o[db] * inv;
        if (a.out_f32) *reinterpret_cast<f32x4 *>(a.out_f32 + (size_t)qrow * qd + d0) = o;
        if (a.out_split) {
            uint32_t lo[NP], hi[NP];
            split_pair<NP>(o[0], o[1], lo);
            split_pair<NP>(o[2], o[3], hi);
            uint16_t *o16 = a.out_split + (size_t)qrow * NP * qd + d0;
#pragma unroll
            for (int p = 0; p < NP; p++) {
                u32x2 w;
                w.x = lo[p];
                w.y = hi[p];
                *reinterpret_cast<u32x2 *>(o16 + (size_t)p * qd) = w;
            }
        }
    }
}

// Joins the shares of prefill_attn16_kernel when the keys were cut over nz workgroups: four neighbouring outputs of
// one (query row, head) per thread, the shares in index order against the largest reference point (scores are in
// units of ln 2; a share that saw no visible key has max = -inf or the floor -1e30 and sum 0; share 0 sees key 0).
template <int NP>
__global__ __launch_bounds__(256) void prefill_attn_join_kernel(const float *__restrict__ part_o, const float *__restrict__ part_ml,
                                                                int nz, int S, int H, int hd, float *__restrict__ out_f32,
                                                                uint16_t *__restrict__ out_split) {
    const size_t qd = (size_t)H * hd, e = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (e >= (size_t)S * qd) return;
    const size_t qrow = e / qd;
    const int col = (int)(e % qd), h = col / hd;
    float m = -INFINITY;
    for (int z = 0; z < nz; z++) m = fmaxf(m, part_ml[(((size_t)z * S + qrow) * H + h) * 2]);
    float l = 0.f;
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
    for (int z = 0; z < nz; z++) {
        const float *pm = part_ml + (((size_t)z * S + qrow) * H + h) * 2;
        const float w = __builtin_amdgcn_exp2f(pm[0] - m);
        l = fmaf(w, pm[1], l);
        const f32x4 oz = *reinterpret_cast<const f32x4 *>(part_o + ((size_t)z * S + qrow) * qd + col);
#pragma unroll
        for (int k = 0; k < 4; k++) o[k] = fmaf(w, oz[k], o[k]);
    }
    const float inv = 1.0f / l;
    o = o * inv;
    if (out_f32) *reinterpret_cast<f32x4 *>(out_f32 + qrow * qd + col) = o;
    if (out_split) {
        uint32_t lo[NP], hi[NP];
        split_pair<NP>(o[0], o[1], lo);
        split_pair<NP>(o[2], o[3], hi);
        uint16_t *o16 = out_split + qrow * NP * qd + col;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            u32x2 w;
            w.x = lo[p];
            w.y = hi[p];
            *reinterpret_cast<u32x2 *>(o16 + (size_t)p * qd) = w;
        }
    }
}

}  // namespace

namespace homura {

int rmsnorm_split_launch(hm_ctx *ctx, const float *d_x, const float *d_res, int res_parts, const float *d_w,
                         uint16_t *d_out_split, int pieces, float *d_resid_out, int rows, int dim, float eps, bool q8k,
                         float *d_pre_q8k, int8_t *d_q8, float *d_q8_scale) {
    HM_REQUIRE(ctx, !q8k || dim % 256 == 0, "rmsnorm_split: Q8_K activations need dim %% 256 == 0 (dim=%d)", dim);
    HM_REQUIRE(ctx, d_x && d_w && (d_out_split || d_q8), "rmsnorm_split: NULL pointer");
    HM_REQUIRE(ctx, !d_q8 || (q8k && d_q8_scale && ((uintptr_t)d_q8 % 4) == 0), "rmsnorm_split: Q8_K rows need q8k, a scale buffer and 4-byte alignment");
    HM_REQUIRE(ctx, rows > 0 && dim > 0 && dim % 4 == 0 && pieces >= 1 && pieces <= 3 && res_parts >= 1 && res_parts <= MAX_SUM_PARTS,
               "rmsnorm_split: bad shape (dim %% 4 == 0 needed)");
    HM_REQUIRE(ctx, ((uintptr_t)d_x % 16) == 0 && ((uintptr_t)d_w % 16) == 0 && ((uintptr_t)d_out_split % 8) == 0 &&
                        ((uintptr_t)d_res % 16) == 0 && ((uintptr_t)d_resid_out % 16) == 0, "rmsnorm_split: misaligned buffer");
    hipLaunchKernelGGL(rmsnorm_split_kernel, dim3(rows), dim3(256), 0, ctx->stream, d_x, d_res, res_parts,
                       (size_t)rows * dim, d_w, d_out_split, d_resid_out, dim, eps, pieces, q8k ? 1 : 0, d_pre_q8k, d_q8,
                       d_q8_scale);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int silu_mul_split_launch(hm_ctx *ctx, const float *d_gu, int parts, uint16_t *d_out_split, int pieces, int rows,
                          int inter, bool q8k, float *d_pre_q8k, int8_t *d_q8, float *d_q8_scale) {
    HM_REQUIRE(ctx, !q8k || inter % 256 == 0, "silu_mul_split: Q8_K activations need a width %% 256 == 0 (%d)", inter);
    HM_REQUIRE(ctx, d_gu && (d_out_split || d_q8), "silu_mul_split: NULL pointer");
    HM_REQUIRE(ctx, !d_q8 || (q8k && d_q8_scale && ((uintptr_t)d_q8 % 4) == 0), "silu_mul_split: Q8_K rows need q8k, a scale buffer and 4-byte alignment");
    HM_REQUIRE(ctx, rows > 0 && inter > 0 && inter % 4 == 0 && pieces >= 1 && pieces <= 3 && parts >= 1 && parts <= MAX_SUM_PARTS,
               "silu_mul_split: bad shape (intermediate size %% 4 == 0 needed)");
    HM_REQUIRE(ctx, ((uintptr_t)d_gu % 16) == 0 && ((uintptr_t)d_out_split % 8) == 0, "silu_mul_split: misaligned buffer");
    const size_t n = (size_t)rows * inter;
    hipLaunchKernelGGL(silu_mul_split_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, ctx->stream, d_gu, parts,
                       2 * n, d_out_split, inter, n, pieces, q8k ? 1 : 0, d_pre_q8k, d_q8, d_q8_scale);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int split_rows_launch(hm_ctx *ctx, const float *d_x, uint16_t *d_out_split, int pieces, size_t rows, int dim, bool q8k) {
    HM_REQUIRE(ctx, d_x && d_out_split, "split_rows: NULL pointer");
    HM_REQUIRE(ctx, rows > 0 && dim > 0 && dim % 4 == 0 && pieces >= 1 && pieces <= 3, "split_rows: bad shape (dim %% 4 == 0 needed)");
    HM_REQUIRE(ctx, !q8k || dim % 256 == 0, "split_rows: Q8_K activations need dim %% 256 == 0 (dim=%d)", dim);
    HM_REQUIRE(ctx, ((uintptr_t)d_x % 16) == 0 && ((uintptr_t)d_out_split % 8) == 0, "split_rows: misaligned buffer");
    const size_t n = rows * dim;
    HM_REQUIRE(ctx, (n / 4 + 255) / 256 <= 0x7fffffffULL, "split_rows: too many elements");
    hipLaunchKernelGGL(split_rows4_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, ctx->stream, d_x, d_out_split,
                       dim, n, pieces, q8k ? 1 : 0);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int dequant_split_launch(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int N, int K, uint16_t *d_out_split,
                         int row_mult, int row_off) {
    HM_REQUIRE(ctx, d_blocks && d_out_split, "dequant_split: NULL pointer");
    const bool kq = hm_dtype == HM_DTYPE_Q4_K || hm_dtype == HM_DTYPE_Q6_K;
    HM_REQUIRE(ctx, N > 0 && K > 0 && K % (kq ? 256 : 32) == 0 && row_mult >= 1 && row_off >= 0 && row_off < row_mult,
               "dequant_split: bad shape (N=%d K=%d)", N, K);
    HM_REQUIRE(ctx, ((uintptr_t)d_out_split % 16) == 0, "dequant_split: misaligned output");
    const size_t n8 = (size_t)N * K / 8;
    const dim3 grid((unsigned)((n8 + 255) / 256));
    HM_REQUIRE(ctx, (n8 + 255) / 256 <= 0x7fffffffULL, "dequant_split: matrix too large");
    switch (hm_dtype) {
    case HM_DTYPE_Q8_0:
        hipLaunchKernelGGL((dequant_split_kernel<QF_Q8_0>), grid, dim3(256), 0, ctx->stream, d_blocks, d_out_split, K, n8, row_mult, row_off);
        break;
    case HM_DTYPE_Q4_0:
        hipLaunchKernelGGL((dequant_split_kernel<QF_Q4_0>), grid, dim3(256), 0, ctx->stream, d_blocks, d_out_split, K, n8, row_mult, row_off);
        break;
    case HM_DTYPE_Q4_K:
        hipLaunchKernelGGL((dequant_split_kernel<QF_Q4_K>), grid, dim3(256), 0, ctx->stream, d_blocks, d_out_split, K, n8, row_mult, row_off);
        break;
    case HM_DTYPE_Q6_K:
        hipLaunchKernelGGL((dequant_split_kernel<QF_Q6_K>), grid, dim3(256), 0, ctx->stream, d_blocks, d_out_split, K, n8, row_mult, row_off);
        break;
    default:
        return hm_set_error(ctx, HM_ERR_INVALID, "dequant_split: dtype %d is not a block format", hm_dtype);
    }
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int quant_ints_launch(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int N, int K, uint16_t *d_ints, float *d_scales,
                      int npad, int row_mult, int row_off) {
    HM_REQUIRE(ctx, d_blocks && d_ints && d_scales, "quant_ints: NULL pointer");
    HM_REQUIRE(ctx, hm_dtype == HM_DTYPE_Q8_0 || hm_dtype == HM_DTYPE_Q4_0, "quant_ints: dtype %d is not Q8_0 / Q4_0", hm_dtype);
    HM_REQUIRE(ctx, N > 0 && K > 0 && K % 32 == 0 && row_mult >= 1 && row_off >= 0 && row_off < row_mult &&
                        (size_t)(N - 1) * row_mult + row_off < (size_t)npad,
               "quant_ints: bad shape (N=%d K=%d stride %d)", N, K, npad);
    HM_REQUIRE(ctx, ((uintptr_t)d_ints % 16) == 0, "quant_ints: misaligned output");
    const size_t n8 = (size_t)N * K / 8;
    HM_REQUIRE(ctx, (n8 + 255) / 256 <= 0x7fffffffULL, "quant_ints: matrix too large");
    const dim3 grid((unsigned)((n8 + 255) / 256));
    if (hm_dtype == HM_DTYPE_Q8_0)
        hipLaunchKernelGGL((quant_ints_kernel<QF_Q8_0>), grid, dim3(256), 0, ctx->stream, d_blocks, d_ints, d_scales, K, n8, npad, row_mult, row_off);
    else
        hipLaunchKernelGGL((quant_ints_kernel<QF_Q4_0>), grid, dim3(256), 0, ctx->stream, d_blocks, d_ints, d_scales, K, n8, npad, row_mult, row_off);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int qkv_post_launch(hm_ctx *ctx, const QkvPostArgs &a) {
    HM_REQUIRE(ctx, a.qkv && a.cos_tab && a.sin_tab && a.kcache && a.vcache, "qkv_post: NULL pointer");
    HM_REQUIRE(ctx, a.S > 0 && a.H > 0 && a.kvh > 0 && a.past >= 0 && a.parts >= 1 && a.parts <= MAX_SUM_PARTS, "qkv_post: bad shape");
    HM_REQUIRE(ctx, a.hd >= 2 && a.hd <= 256 && a.hd % 2 == 0, "qkv_post: head_dim %d not supported", a.hd);
    HM_REQUIRE(ctx, (a.qw == nullptr) == (a.kw == nullptr), "qkv_post: q and k norm weights must come together");
    if (a.past + a.S > a.max_len)
        return hm_set_error(ctx, HM_ERR_STATE, "KV cache full (%d + %d > %d)", a.past, a.S, a.max_len);
    const long long rows = (long long)a.S * (a.H + 2 * a.kvh);
    hipLaunchKernelGGL(qkv_post_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, ctx->stream, a);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int prefill_attn_launch(hm_ctx *ctx, const PrefillAttnArgs &a) {
    HM_REQUIRE(ctx, a.q && a.kcache && a.vcache && (a.out_f32 || a.out_split), "prefill_attn: NULL pointer");
    HM_REQUIRE(ctx, a.S > 0 && a.H > 0 && a.kvh > 0 && a.H % a.kvh == 0 && a.past >= 0, "prefill_attn: bad shape");
    HM_REQUIRE(ctx, a.hd == 64 || a.hd == 128, "prefill_attn: head_dim %d not supported (64 or 128)", a.hd);
    HM_REQUIRE(ctx, a.past + a.S <= a.max_len, "prefill_attn: %d + %d rows exceed the cache (%d)", a.past, a.S, a.max_len);
    HM_REQUIRE(ctx, a.ldq >= a.H * a.hd && a.ldq % 4 == 0 && ((uintptr_t)a.q % 16) == 0, "prefill_attn: q rows must be 16-byte aligned");
    HM_REQUIRE(ctx, ((uintptr_t)a.kcache % 16) == 0 && ((uintptr_t)a.vcache % 16) == 0, "prefill_attn: caches must be 16-byte aligned");
    HM_REQUIRE(ctx, (!a.out_f32 || ((uintptr_t)a.out_f32 % 16) == 0) && (!a.out_split || ((uintptr_t)a.out_split % 8) == 0),
               "prefill_attn: misaligned output");
    HM_REQUIRE(ctx, a.pieces == 2 || a.pieces == 3, "prefill_attn: %d pieces (2 or 3)", a.pieces);
    // the fewest key groups that still give every CU a workgroup (more groups mean more tile loads)
    int ks = 4;
    for (int cand = 1; cand < 4; cand *= 2)
        if ((long long)((a.S + 128 / cand - 1) / (128 / cand)) * a.H >= ctx->num_cus) {
            ks = cand;
            break;
        }
    if (const char *e = getenv("HOMURA_PREFILL_KEY_GROUPS")) {
        const int v = atoi(e);
        if (v == 1 || v == 2 || v == 4) ks = v;
    }
    const int qrows = 128 / ks;
    dim3 grid((unsigned)((a.S + qrows - 1) / qrows), (unsigned)a.H);
    // Few query rows in front of a long cache (a chat turn behind a long conversation) leave most CUs without a
    // workgroup while each workgroup walks every key: the keys are then cut over nz workgroups, eight rounds of
    // tiles each at least, which leave their (O, max, sum) in the workspace for a second kernel to join.
    PrefillAttnArgs b = a;
    int nz = 1;
    {
        const long long wgs = (long long)grid.x * grid.y;
        const int rounds = ((a.past + a.S + A8_KEYS - 1) / A8_KEYS + ks - 1) / ks;
        nz = (int)std::min<long long>(std::min<long long>(32, ctx->num_cus / std::max<long long>(1, wgs)), rounds / 8);
        const size_t per_z = (size_t)a.S * a.H * (a.hd + 2) * sizeof(float);
        // (callers that carve scratch of their own from the workspace leave its first 16 MiB to the kernels)
        const size_t room = std::min<size_t>(ctx->workspace_bytes, (size_t)16 << 20);
        if (nz >= 2 && per_z * nz > room) nz = (int)(room / per_z);
        if (nz < 2) nz = 1;
        if (nz > 1) {
            b.part_o = (float *)ctx->workspace;
            b.part_ml = b.part_o + (size_t)nz * a.S * a.H * a.hd;
            grid.z = (unsigned)nz;
        }
    }
    // two sets of ks pairs of 32-key tiles; the final exchange of the key groups wants
    // (ks - 1) * (128 / ks / 16) sets of (hd / 4 + 2) * 256 bytes
    const size_t lds = std::max<size_t>((size_t)2 * ks * 2 * A8_KEYS * a.hd * 2, (size_t)(ks - 1) * (8 / ks) * (a.hd / 4 + 2) * 256);
    auto launch = [&](auto kernel) -> int {
        if (lds > 64 * 1024) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            HM_REQUIRE(ctx, e == hipSuccess, "prefill_attn: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        }
        hipLaunchKernelGGL(kernel, grid, dim3(A8_THREADS), lds, ctx->stream, b);
        return HM_OK;
    };
    int rc = HM_OK;
#define HM_AT_CASE(HDV, NPV)                                                             \
    if (a.hd == HDV && a.pieces == NPV) {                                                \
        if (ks == 1) rc = launch(prefill_attn16_kernel<HDV, NPV, 1>);                    \
        else if (ks == 2) rc = launch(prefill_attn16_kernel<HDV, NPV, 2>);               \
        else rc = launch(prefill_attn16_kernel<HDV, NPV, 4>);                            \
    }
    HM_AT_CASE(128, 3)
    HM_AT_CASE(128, 2)
    HM_AT_CASE(64, 3)
    HM_AT_CASE(64, 2)
#undef HM_AT_CASE
    if (rc != HM_OK) return rc;
    HM_LAUNCH_CHECK(ctx);
    if (nz > 1) {
        const size_t n4 = (size_t)a.S * a.H * a.hd / 4;
        const dim3 jg((unsigned)((n4 + 255) / 256));
        if (a.pieces == 3)
            hipLaunchKernelGGL(prefill_attn_join_kernel<3>, jg, dim3(256), 0, ctx->stream, b.part_o, b.part_ml, nz, a.S, a.H, a.hd,
                               a.out_f32, a.out_split);
        else
            hipLaunchKernelGGL(prefill_attn_join_kernel<2>, jg, dim3(256), 0, ctx->stream, b.part_o, b.part_ml, nz, a.S, a.H, a.hd,
                               a.out_f32, a.out_split);
        HM_LAUNCH_CHECK(ctx);
    }
    return HM_OK;
}

}  // namespace homura

extern "C" int hm_gemm_f32_bf16_nk(hm_ctx *ctx, const float *d_x_mk, const uint16_t *d_w_nk, float *d_out, int M, int K,
                                   int N) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x_mk && d_w_nk && d_out, "hm_gemm_f32_bf16_nk: NULL pointer");
    HM_REQUIRE(ctx, M > 0 && N > 0 && K > 0 && K % 32 == 0, "hm_gemm_f32_bf16_nk: need M, N > 0 and K %% 32 == 0");
    const size_t n = (size_t)M * K;
    HM_REQUIRE(ctx, n * 6 <= ctx->workspace_bytes, "hm_gemm_f32_bf16_nk: M * K = %zu activations exceed the workspace", n);
    uint16_t *split = (uint16_t *)ctx->workspace;
    const int rc = homura::split_rows_launch(ctx, d_x_mk, split, 3, (size_t)M, K);
    if (rc != HM_OK) return rc;
    return homura::gemm_split_nk(ctx, split, 3, d_w_nk, d_out, M, K, N);
}

extern "C" int hm_gemm_f32_quant_nk(hm_ctx *ctx, const float *d_x_mk, const uint8_t *d_w_blocks, int dtype, float *d_out,
                                    int M, int K, int N) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_x_mk && d_w_blocks && d_out, "hm_gemm_f32_quant_nk: NULL pointer");
    const bool kq = dtype == HM_DTYPE_Q4_K || dtype == HM_DTYPE_Q6_K;
    HM_REQUIRE(ctx, kq || dtype == HM_DTYPE_Q8_0 || dtype == HM_DTYPE_Q4_0, "hm_gemm_f32_quant_nk: dtype %d is not a block format", dtype);
    HM_REQUIRE(ctx, M > 0 && N > 0 && K > 0 && K % (kq ? 256 : 64) == 0,
               "hm_gemm_f32_quant_nk: need M, N > 0 and K %% %d == 0 (K=%d)", kq ? 256 : 64, K);
    if (kq && K / 256 <= 16) {  // (wider rows would need K slices: they keep the bf16 pieces below)
        // K-quants: Q8_K rows x the matrix's int8 digit planes on the integer matrix cores. Workspace: the
        // quantised rows and their scales, then the planes and block scales of as many weight rows as fit.
        const size_t q_bytes = ((size_t)M * K + 255) / 256 * 256, s_bytes = ((size_t)M * (K / 256) * 4 + 255) / 256 * 256;
        const size_t per_row = (size_t)3 * K + (size_t)(K / 256) * 8;
        HM_REQUIRE(ctx, q_bytes + s_bytes + 128 * per_row + 256 <= ctx->workspace_bytes,
                   "hm_gemm_f32_quant_nk: M * K = %zu activations exceed the workspace", (size_t)M * K);
        int8_t *aq = (int8_t *)ctx->workspace;
        float *asc = (float *)((char *)ctx->workspace + q_bytes);
        char *wbase = (char *)ctx->workspace + q_bytes + s_bytes;
        const int slab = (int)std::min<size_t>((size_t)N, (ctx->workspace_bytes - q_bytes - s_bytes - 256) / per_row / 128 * 128);
        int rc = homura::quantize_q8k_rows_launch(ctx, d_x_mk, aq, asc, (size_t)M, K);
        const size_t row_bytes = (size_t)K / 256 * (dtype == HM_DTYPE_Q4_K ? 144 : 210);
        for (int n0 = 0; n0 < N && rc == HM_OK; n0 += slab) {
            const int rows = std::min(slab, N - n0);
            int8_t *planes = (int8_t *)wbase;
            float *wsc = (float *)(wbase + ((size_t)3 * rows * K + 255) / 256 * 256);
            rc = homura::kq_i8_pack(ctx, dtype, d_w_blocks + (size_t)n0 * row_bytes, rows, K, planes, wsc, rows, 1, 0);
            if (rc == HM_OK) rc = homura::gemm_q8k_kquant_nk(ctx, aq, asc, planes, wsc, d_out + n0, M, K, rows, 1, nullptr, N);
        }
        return rc;
    }
    if (!kq) {
        // Q8_0 / Q4_0: three-piece rows x the matrix's integers, every 32-wide block's sum times its scale.
        // Workspace: the split activations, then the integers (bf16) and scales of as many weight rows as fit.
        const size_t a_bytes = ((size_t)M * K * 6 + 255) / 256 * 256;
        const size_t per_row = (size_t)K * 2 + (size_t)(K / 32) * 4;
        HM_REQUIRE(ctx, a_bytes + 128 * per_row + 256 <= ctx->workspace_bytes,
                   "hm_gemm_f32_quant_nk: M * K = %zu activations exceed the workspace", (size_t)M * K);
        uint16_t *a_split = (uint16_t *)ctx->workspace;
        char *wbase = (char *)ctx->workspace + a_bytes;
        const int slab = (int)std::min<size_t>((size_t)(N + 127) / 128 * 128, (ctx->workspace_bytes - a_bytes - 256) / per_row / 128 * 128);
        int rc = homura::split_rows_launch(ctx, d_x_mk, a_split, 3, (size_t)M, K, false);
        const size_t row_bytes = (size_t)K / 32 * (dtype == HM_DTYPE_Q8_0 ? 34 : 18);
        for (int n0 = 0; n0 < N && rc == HM_OK; n0 += slab) {
            const int rows = std::min(slab, N - n0), npad = (rows + 127) / 128 * 128;
            uint16_t *ints = (uint16_t *)wbase;
            float *wsc = (float *)(wbase + ((size_t)rows * K * 2 + 255) / 256 * 256);
            rc = homura::quant_ints_launch(ctx, dtype, d_w_blocks + (size_t)n0 * row_bytes, rows, K, ints, wsc, npad);
            if (rc == HM_OK) rc = homura::gemm_pieces_scaled_nk(ctx, a_split, ints, wsc, npad, d_out + n0, M, K, rows, 1, nullptr, N);
        }
        return rc;
    }
    // (K-quant rows wider than the int8 path takes)
    // workspace: the split activations, then as many split weight rows as fit (a multiple of the tile)
    const size_t a_bytes = ((size_t)M * K * 6 + 255) / 256 * 256;
    HM_REQUIRE(ctx, a_bytes + (size_t)128 * K * 6 <= ctx->workspace_bytes,
               "hm_gemm_f32_quant_nk: M * K = %zu activations exceed the workspace", (size_t)M * K);
    uint16_t *a_split = (uint16_t *)ctx->workspace;
    uint16_t *w_split = (uint16_t *)((char *)ctx->workspace + a_bytes);
    const int slab = (int)std::min<size_t>((size_t)N, (ctx->workspace_bytes - a_bytes) / ((size_t)K * 6) / 128 * 128);
    int rc = homura::split_rows_launch(ctx, d_x_mk, a_split, 3, (size_t)M, K, kq);
    const size_t block_bytes = dtype == HM_DTYPE_Q8_0 ? 34 : dtype == HM_DTYPE_Q4_0 ? 18 : dtype == HM_DTYPE_Q4_K ? 144 : 210;
    const size_t row_bytes = (size_t)K / (kq ? 256 : 32) * block_bytes;
    for (int n0 = 0; n0 < N && rc == HM_OK; n0 += slab) {
        const int rows = std::min(slab, N - n0);
        rc = homura::dequant_split_launch(ctx, dtype, d_w_blocks + (size_t)n0 * row_bytes, rows, K, w_split);
        if (rc == HM_OK) rc = homura::gemm_split_split_nk(ctx, a_split, w_split, d_out + n0, M, K, rows, 1, nullptr, N);
    }
    return rc;
}

extern "C" int hm_gqa_prefill_attn(hm_ctx *ctx, const float *d_q, const uint16_t *d_kcache, const uint16_t *d_vcache,
                                   float *d_out, int S, int H, int kvh, int hd, int max_len, int past, float scale) {
    HM_CHECK_CTX(ctx);
    homura::PrefillAttnArgs a;
    a.q = d_q;
    a.ldq = H * hd;
    a.kcache = d_kcache;
    a.vcache = d_vcache;
    a.out_f32 = d_out;
    a.S = S;
    a.H = H;
    a.kvh = kvh;
    a.hd = hd;
    a.max_len = max_len;
    a.past = past;
    a.scale = scale;
    return homura::prefill_attn_launch(ctx, a);
}
