// The reference's own kernel ABI on top of the GPU kernels: symbols
// `_mlir__mlir_ciface_k{idx}(void **args)` that take memref descriptors, exactly what
// CompiledGraph::load_from_handle resolves with dlsym and run_with_output_bufs calls
// (reference src/runtime.rs:779-824, :930-1037; descriptor layout :654-698).
//
// With Buffers that hold device memory, the reference's ExecutionPlan can dlopen this library
// in place of its compiled CPU kernels. hm_ciface_bind_transformer() records which fused kernel
// each index stands for, in the order emit_transformer_plan numbers them (src/hf/emitter.rs:
// 902-1014): k0 Embed; per layer k(3l+1) QKV(+QK-norm)+RoPE, k(3l+2) Attn, k(3l+3) MLP; then
// LMHead. Arguments follow each emitter's input order, outputs after inputs.
//
// hm_ciface_bind_transformer_quant() does the same for the quantised plan (src/hf/emitter_quant.rs:
// 1170-1440): k0 Embed; per layer thirteen kernels, RMSNorm, QuantMM Q, K, V, PostQKV, AttnBody,
// QuantMM O, Residual+Norm, QuantMM Gate, Up, SiLU*Up, QuantMM Down, ResAdd; then the f32 LMHead.
//
// This is the compatibility path: weights are consumed in the reference's layouts ([K,N] bf16 / f32,
// raw GGUF blocks), the KV views are the reference's f32 cache (copied to a bf16 scratch cache per
// call), and every reference kernel becomes one or several launches. The model-level API is the
// fast path.
//
// A call may carry any number of tokens (the reference's prefill hands the whole prompt to the same
// kernels, src/hf/model.rs:321-336): matrix products of fewer than 16 rows go through the GEMVs in blocks of
// up to eight rows, longer ones through the matrix-core GEMMs (f32 rows as three bf16 pieces; Q8_0 / Q4_0
// matrices dequantised to pieces first), attention with more than one query row through the causal prompt kernel, which applies the mask of
// build_causal_mask (src/hf/precompute.rs:134-161) by position instead of reading the mask operand.
//
// The ABI returns void. A failing call prints a line, fills every output operand with NaN (all-ones
// bytes), and leaves its code in a sticky status word that hm_ciface_last_status() reads and
// hm_ciface_clear_status() resets.
#include <cmath>
#include <cstdio>
#include <vector>

#include "../gemm_bf16_mfma.h"
#include "../hm_common.h"
#include "../prefill.h"

namespace {

enum class Kind { Embed, Qkv, Attn, Mlp, LmHead,                                              // bf16 plan
                  RmsNorm, QuantMM, PostQkv, AttnBody, ResidualNorm, SiluMul, ResAdd, LmHeadF32 };  // quantised plan

struct KernelInfo {
    Kind kind;
    int K = 0, N = 0, dtype = 0;  // QuantMM: the matrix
    KernelInfo(Kind k) : kind(k) {}
    KernelInfo(int k_dim, int n_dim, int dt) : kind(Kind::QuantMM), K(k_dim), N(n_dim), dtype(dt) {}
};

struct Bound {
    hm_ctx *ctx = nullptr;
    hm_transformer_config cfg{};
    bool qk_norm = false;
    int kv_heads = 0, head_dim = 0, q_dim = 0, kv_dim = 0;
    std::vector<KernelInfo> kinds;
} g_bound;

// One rank-N memref argument: args[i] points at a pointer to the descriptor bytes.
struct MemRef {
    char *data = nullptr;
    const int64_t *sizes = nullptr, *strides = nullptr;
    template <class T>
    T *as() const { return reinterpret_cast<T *>(data); }
};
MemRef memref(void **args, int i, int rank) {
    char *desc = *reinterpret_cast<char **>(args[i]);
    MemRef m;
    int64_t offset;
    std::memcpy(&m.data, desc + 8, 8);  // aligned pointer
    std::memcpy(&offset, desc + 16, 8);
    (void)offset;  // always 0 (reference src/runtime.rs:689)
    m.sizes = reinterpret_cast<const int64_t *>(desc + 24);
    m.strides = m.sizes + rank;
    return m;
}

int g_status = HM_OK;       // first failure since the last hm_ciface_clear_status
int g_status_kernel = -1;

// The reference's kernels return void: a failure is recorded on the context and reported here.
void report(int idx, int rc) {
    if (rc == HM_OK) return;
    if (g_status == HM_OK) {
        g_status = rc;
        g_status_kernel = idx;
    }
    std::fprintf(stderr, "homura_amd: _mlir__mlir_ciface_k%d failed (%d): %s\n", idx, rc,
                 g_bound.ctx ? hm_last_error(g_bound.ctx) : "no transformer bound");
}

#define TRY(expr)                 \
    do {                          \
        int _rc = (expr);         \
        if (_rc != HM_OK) return _rc; \
    } while (0)

// Scratch carved from the context workspace, 256-byte aligned pieces. The kernels called from here
// keep their own partials (split-K sums, attention splits, argmax segments: a few MiB at most at
// the sizes accepted here) at the start of the workspace, so the first KERNEL_RESERVE bytes are
// left to them.
constexpr size_t KERNEL_RESERVE = (size_t)16 << 20;
struct Scratch {
    char *p;
    size_t left;
    explicit Scratch(hm_ctx *ctx)
        : p((char *)ctx->workspace + KERNEL_RESERVE),
          left(ctx->workspace_bytes > KERNEL_RESERVE ? ctx->workspace_bytes - KERNEL_RESERVE : 0) {}
    template <class T>
    T *take(size_t n) {
        const size_t bytes = (n * sizeof(T) + 255) & ~(size_t)255;
        if (bytes > left) return nullptr;
        T *r = reinterpret_cast<T *>(p);
        p += bytes;
        left -= bytes;
        return r;
    }
};

__global__ void kv_view_to_bf16_kernel(const float *__restrict__ src, int64_t head_stride, int64_t row_stride,
                                       uint16_t *__restrict__ dst, int rows, int hd, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int d = (int)(i % hd);
    const size_t r = i / hd;
    const int row = (int)(r % rows);
    const size_t head = r / rows;
    dst[i] = f32_to_bf16_rne_dev(src[head * head_stride + (size_t)row * row_stride + d]);
}

__global__ void add_bias_rows_kernel(float *__restrict__ x, const float *__restrict__ bias, int n, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) x[i] = x[i] + bias[i % n];
}

// [S][heads][hd] -> [heads][S][hd] (the BSHD -> BHSD transposes of src/hf/emitter.rs:648-649)
__global__ void bshd_to_bhsd_kernel(const float *__restrict__ src, float *__restrict__ dst, int S, int heads, int hd,
                                    size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int d = (int)(i % hd);
    const size_t r = i / hd;
    const int h = (int)(r % heads);
    const size_t sq = r / heads;
    dst[((size_t)h * S + sq) * hd + d] = src[i];
}

int seq_ok(hm_ctx *ctx, int64_t seq, const char *what) {
    if (seq >= 1 && seq <= (1 << 20)) return HM_OK;
    return hm_set_error(ctx, HM_ERR_INVALID, "%s: %lld tokens in one call", what, (long long)seq);
}

int add_bias_rows(hm_ctx *ctx, float *x, const float *bias, int rows, int n) {
    const size_t total = (size_t)rows * n;
    hipLaunchKernelGGL(add_bias_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, x, bias, n, total);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int bshd_to_bhsd(hm_ctx *ctx, const float *src, float *dst, int S, int heads, int hd) {
    const size_t total = (size_t)S * heads * hd;
    hipLaunchKernelGGL(bshd_to_bhsd_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, src, dst, S, heads,
                       hd, total);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

// Calls of at least this many tokens take their matrix products to the matrix cores.
constexpr int GEMM_MIN_ROWS = 16;

// out [S][N] = x [S][K] times a [K,N] bf16 matrix. A few rows: the batch-1 kernel, up to eight rows a launch.
// A prompt (the reference's prefill hands all its tokens to the same kernels, src/hf/model.rs:321-336): the
// f32 rows as three bf16 pieces each (all 24 significant bits) against the matrix on the matrix cores.
int rows_matmul_bf16(hm_ctx *ctx, Scratch &s, const float *x, const uint16_t *w, float *out, int S, int K, int N) {
    if (S >= GEMM_MIN_ROWS && K % 32 == 0 && N % 8 == 0 && ((uintptr_t)w % 16) == 0) {
        Scratch local = s;  // the pieces are dead once the product is enqueued: later calls may reuse the space
        uint16_t *split = local.take<uint16_t>((size_t)S * 3 * K);
        if (split) {
            TRY(homura::split_rows_launch(ctx, x, split, 3, (size_t)S, K));
            return homura::gemm_split_kn(ctx, split, 3, w, out, S, K, N);
        }
    }
    for (int r = 0; r < S; r += 8)
        TRY(hm_gemv_bf16(ctx, x + (size_t)r * K, w, out + (size_t)r * N, S - r < 8 ? S - r : 8, K, N));
    return HM_OK;
}

// emit_embed_kernel (src/hf/emitter.rs:506-537): ids [1,S] i64, table [V,H] f32 -> [1,S,H]
int run_embed(void **a) {
    const Bound &b = g_bound;
    const MemRef ids = memref(a, 0, 2), table = memref(a, 1, 2), out = memref(a, 2, 3);
    return hm_embed(b.ctx, ids.as<int64_t>(), table.as<float>(), out.as<float>(), (int)ids.sizes[1],
                    b.cfg.vocab_size, b.cfg.hidden_size);
}

// emit_qkv_kernel (src/hf/emitter.rs:549-673): h, ln_w, q_w, [q_b], k_w, [k_b], v_w, [v_b], cos, sin,
// [q_norm_w, k_norm_w] -> q [1,S,H,hd], k [1,kvh,S,hd], v [1,kvh,S,hd]
int run_qkv(void **a) {
    const Bound &b = g_bound;
    hm_ctx *ctx = b.ctx;
    const int hidden = b.cfg.hidden_size, bias = b.cfg.attention_bias ? 1 : 0;
    int i = 0;
    const MemRef h = memref(a, i++, 3), ln = memref(a, i++, 1), qw = memref(a, i++, 2);
    const float *qb = bias ? memref(a, i++, 1).as<float>() : nullptr;
    const MemRef kw = memref(a, i++, 2);
    const float *kb = bias ? memref(a, i++, 1).as<float>() : nullptr;
    const MemRef vw = memref(a, i++, 2);
    const float *vb = bias ? memref(a, i++, 1).as<float>() : nullptr;
    const MemRef cosv = memref(a, i++, 2), sinv = memref(a, i++, 2);
    const float *qn = nullptr, *kn = nullptr;
    if (b.qk_norm) {
        qn = memref(a, i++, 1).as<float>();
        kn = memref(a, i++, 1).as<float>();
    }
    const MemRef q = memref(a, i++, 4), k = memref(a, i++, 4), v = memref(a, i++, 4);
    const int S = (int)h.sizes[1], H = b.cfg.num_attention_heads;
    TRY(seq_ok(ctx, h.sizes[1], "QKV kernel"));
    Scratch s(ctx);
    float *normed = s.take<float>((size_t)S * hidden);
    // more than one token: k and v are projected as [S][kvh][hd] rows and transposed into the outputs
    float *krows = S > 1 ? s.take<float>((size_t)S * b.kv_dim) : k.as<float>();
    float *vrows = S > 1 ? s.take<float>((size_t)S * b.kv_dim) : v.as<float>();
    if (!normed || !krows || !vrows) return hm_set_error(ctx, HM_ERR_OOM, "QKV kernel: workspace too small for %d tokens", S);
    TRY(hm_rmsnorm(ctx, h.as<float>(), ln.as<float>(), normed, S, hidden, (float)b.cfg.rms_norm_eps));
    TRY(rows_matmul_bf16(ctx, s, normed, qw.as<uint16_t>(), q.as<float>(), S, hidden, b.q_dim));
    TRY(rows_matmul_bf16(ctx, s, normed, kw.as<uint16_t>(), krows, S, hidden, b.kv_dim));
    TRY(rows_matmul_bf16(ctx, s, normed, vw.as<uint16_t>(), vrows, S, hidden, b.kv_dim));
    if (bias) {
        TRY(add_bias_rows(ctx, q.as<float>(), qb, S, b.q_dim));
        TRY(add_bias_rows(ctx, krows, kb, S, b.kv_dim));
        TRY(add_bias_rows(ctx, vrows, vb, S, b.kv_dim));
    }
    TRY(hm_qknorm_rope(ctx, q.as<float>(), krows, qn, kn, cosv.as<float>(), sinv.as<float>(), S, H, b.kv_heads, b.head_dim,
                       (float)b.cfg.rms_norm_eps));
    if (S == 1) return HM_OK;  // with one token the BSHD rows and the BHSD outputs coincide
    TRY(bshd_to_bhsd(ctx, krows, k.as<float>(), S, b.kv_heads, b.head_dim));
    return bshd_to_bhsd(ctx, vrows, v.as<float>(), S, b.kv_heads, b.head_dim);
}

// emit_attention_kernel (src/hf/emitter.rs:683-758): q [1,S,H,hd], k/v views [1,kvh,T,hd] f32 with the
// cache's max-length strides (src/runtime.rs:610-615), mask [1,1,S,T], o_w [q_dim,hidden] -> [1,S,hidden]
int attention_over_views(const MemRef &q, const MemRef &k, const MemRef &v, float *out, Scratch &s, const char *who);

int run_attn(void **a) {
    const Bound &b = g_bound;
    hm_ctx *ctx = b.ctx;
    const MemRef q = memref(a, 0, 4), k = memref(a, 1, 4), v = memref(a, 2, 4), ow = memref(a, 4, 2),
                 out = memref(a, 5, 3);
    TRY(seq_ok(ctx, q.sizes[1], "Attn kernel"));
    const int S = (int)q.sizes[1];
    Scratch s(ctx);
    float *flat = s.take<float>((size_t)S * b.q_dim);
    if (!flat) return hm_set_error(ctx, HM_ERR_OOM, "Attn kernel: workspace too small for %d tokens", S);
    TRY(attention_over_views(q, k, v, flat, s, "Attn kernel"));
    return rows_matmul_bf16(ctx, s, flat, ow.as<uint16_t>(), out.as<float>(), S, b.q_dim, b.cfg.hidden_size);
}

// emit_mlp_kernel (src/hf/emitter.rs:767-822): h, attn_out, ln_w, gate_w, up_w, down_w -> [1,S,hidden]
int run_mlp(void **a) {
    const Bound &b = g_bound;
    hm_ctx *ctx = b.ctx;
    const int hidden = b.cfg.hidden_size, inter = b.cfg.intermediate_size;
    const MemRef h = memref(a, 0, 3), attn = memref(a, 1, 3), ln = memref(a, 2, 1), gw = memref(a, 3, 2),
                 uw = memref(a, 4, 2), dw = memref(a, 5, 2), out = memref(a, 6, 3);
    TRY(seq_ok(ctx, h.sizes[1], "MLP kernel"));
    const size_t S = (size_t)h.sizes[1];
    Scratch s(ctx);
    float *resid = s.take<float>(S * hidden), *normed = s.take<float>(S * hidden), *gate = s.take<float>(S * inter),
          *up = s.take<float>(S * inter), *down = s.take<float>(S * hidden);
    if (!resid || !normed || !gate || !up || !down)
        return hm_set_error(ctx, HM_ERR_OOM, "MLP kernel: workspace too small for %d tokens", (int)S);
    TRY(hm_add(ctx, h.as<float>(), attn.as<float>(), resid, S * hidden));
    TRY(hm_rmsnorm(ctx, resid, ln.as<float>(), normed, (int)S, hidden, (float)b.cfg.rms_norm_eps));
    TRY(rows_matmul_bf16(ctx, s, normed, gw.as<uint16_t>(), gate, (int)S, hidden, inter));
    TRY(rows_matmul_bf16(ctx, s, normed, uw.as<uint16_t>(), up, (int)S, hidden, inter));
    TRY(hm_silu_mul(ctx, gate, up, gate, S * inter));
    TRY(rows_matmul_bf16(ctx, s, gate, dw.as<uint16_t>(), down, (int)S, inter, hidden));
    return hm_add(ctx, resid, down, out.as<float>(), S * hidden);
}

// emit_lm_head_kernel (src/hf/emitter.rs:828-862): h, norm_w, lm_head_w [hidden,vocab] -> [1,S,vocab]
int run_lm_head(void **a) {
    const Bound &b = g_bound;
    hm_ctx *ctx = b.ctx;
    const MemRef h = memref(a, 0, 3), nw = memref(a, 1, 1), lw = memref(a, 2, 2), out = memref(a, 3, 3);
    TRY(seq_ok(ctx, h.sizes[1], "LMHead kernel"));
    const int S = (int)h.sizes[1];
    Scratch s(ctx);
    float *normed = s.take<float>((size_t)S * b.cfg.hidden_size);
    if (!normed) return hm_set_error(ctx, HM_ERR_OOM, "LMHead kernel: workspace too small for %d tokens", S);
    TRY(hm_rmsnorm(ctx, h.as<float>(), nw.as<float>(), normed, S, b.cfg.hidden_size, (float)b.cfg.rms_norm_eps));
    return rows_matmul_bf16(ctx, s, normed, lw.as<uint16_t>(), out.as<float>(), S, b.cfg.hidden_size, b.cfg.vocab_size);
}

// ── the quantised plan's kernels (src/hf/emitter_quant.rs) ───────────────────

// out[n] = sum_k x[k] W[k][n], f32, k ascending: the LM head of the quantised plan keeps its weights
// in f32 [hidden, vocab] (src/hf/emitter_quant.rs:1399-1440). One column per thread, coalesced rows.
__global__ __launch_bounds__(256) void gemv_f32_kn_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                          float *__restrict__ out, int K, int N) {
    extern __shared__ float xs[];
    for (int k = threadIdx.x; k < K; k += blockDim.x) xs[k] = x[k];
    __syncthreads();
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    float acc = 0.f;
    for (int k = 0; k < K; k++) acc += xs[k] * w[(size_t)k * N + n];
    out[n] = acc;
}

// emit_rms_norm_kernel (src/hf/emitter_quant.rs:713-791): h [1,S,hidden], w [hidden] -> [1,S,hidden]
int run_rms_norm(void **a) {
    const Bound &b = g_bound;
    const MemRef h = memref(a, 0, 3), w = memref(a, 1, 1), out = memref(a, 2, 3);
    TRY(seq_ok(b.ctx, h.sizes[1], "RMSNorm kernel"));
    return hm_rmsnorm(b.ctx, h.as<float>(), w.as<float>(), out.as<float>(), (int)h.sizes[1], b.cfg.hidden_size,
                      (float)b.cfg.rms_norm_eps);
}

// emit_quant_matmul_kernel (src/hf/emitter_quant.rs:675-702): x [1,S,K], raw blocks (flat bytes) -> [1,S,N]
int run_quant_mm(void **a, const KernelInfo &ki) {
    const Bound &b = g_bound;
    const MemRef x = memref(a, 0, 3), w = memref(a, 1, 1), out = memref(a, 2, 3);
    TRY(seq_ok(b.ctx, x.sizes[1], "QuantMM kernel"));
    const int S = (int)x.sizes[1];
    const bool kq = ki.dtype == HM_DTYPE_Q4_K || ki.dtype == HM_DTYPE_Q6_K;
    // A prompt goes to the matrix cores (hm_gemm_f32_quant_nk: Q8_K rows x int8 digit planes for the K-quants,
    // whose kernel quantises its activations, src/graph_builder/emit_quant.rs:422-466; three-piece rows x block
    // integers with block scales for Q8_0 / Q4_0), when the rows fit the workspace beside a slab of the matrix.
    if (S >= GEMM_MIN_ROWS && ki.K % 64 == 0 && (!kq || ki.K % 256 == 0) &&
        ((size_t)S + 160) * ki.K * 8 <= b.ctx->workspace_bytes)
        return hm_gemm_f32_quant_nk(b.ctx, x.as<float>(), w.as<uint8_t>(), ki.dtype, out.as<float>(), S, ki.K, ki.N);
    for (int r = 0; r < S; r += 8) {
        const float *xr = x.as<float>() + (size_t)r * ki.K;
        float *outr = out.as<float>() + (size_t)r * ki.N;
        const int m = S - r < 8 ? S - r : 8;
        switch (ki.dtype) {
        case HM_DTYPE_Q8_0: TRY(hm_gemv_q8_0(b.ctx, xr, w.as<uint8_t>(), outr, m, ki.K, ki.N)); break;
        case HM_DTYPE_Q4_0: TRY(hm_gemv_q4_0(b.ctx, xr, w.as<uint8_t>(), outr, m, ki.K, ki.N)); break;
        case HM_DTYPE_Q4_K: TRY(hm_gemv_q4_k(b.ctx, xr, w.as<uint8_t>(), outr, m, ki.K, ki.N)); break;
        case HM_DTYPE_Q6_K: TRY(hm_gemv_q6_k(b.ctx, xr, w.as<uint8_t>(), outr, m, ki.K, ki.N)); break;
        default: return hm_set_error(b.ctx, HM_ERR_INVALID, "QuantMM kernel: dtype %d", ki.dtype);
        }
    }
    return HM_OK;
}

// emit_post_qkv_kernel (src/hf/emitter_quant.rs:802-912): q_raw [1,S,q_dim], k_raw, v_raw [1,S,kv_dim],
// [q_b, k_b, v_b], cos, sin, [q_norm_w, k_norm_w] -> q [1,S,H,hd], k [1,kvh,S,hd], v [1,kvh,S,hd]
int run_post_qkv(void **a) {
    const Bound &b = g_bound;
    hm_ctx *ctx = b.ctx;
    const bool bias = b.cfg.attention_bias != 0;
    int i = 0;
    const MemRef qr = memref(a, i++, 3), kr = memref(a, i++, 3), vr = memref(a, i++, 3);
    const float *qb = nullptr, *kb = nullptr, *vb = nullptr;
    if (bias) {
        qb = memref(a, i++, 1).as<float>();
        kb = memref(a, i++, 1).as<float>();
        vb = memref(a, i++, 1).as<float>();
    }
    const MemRef cosv = memref(a, i++, 2), sinv = memref(a, i++, 2);
    const float *qn = nullptr, *kn = nullptr;
    if (b.qk_norm) {
        qn = memref(a, i++, 1).as<float>();
        kn = memref(a, i++, 1).as<float>();
    }
    const MemRef q = memref(a, i++, 4), k = memref(a, i++, 4), v = memref(a, i++, 4);
    TRY(seq_ok(ctx, qr.sizes[1], "PostQKV kernel"));
    const int S = (int)qr.sizes[1];
    Scratch s(ctx);
    // q [1,S,H,hd] is the raw row layout; k and v leave as [1,kvh,S,hd], so with more than one token they
    // are finished as rows in scratch and transposed on the way out
    float *krows = S > 1 ? s.take<float>((size_t)S * b.kv_dim) : k.as<float>();
    float *vrows = S > 1 ? s.take<float>((size_t)S * b.kv_dim) : v.as<float>();
    if (!krows || !vrows) return hm_set_error(ctx, HM_ERR_OOM, "PostQKV kernel: workspace too small for %d tokens", S);
    TRY(hm_copy(ctx, q.data, qr.data, (size_t)S * b.q_dim * 4));
    TRY(hm_copy(ctx, krows, kr.data, (size_t)S * b.kv_dim * 4));
    TRY(hm_copy(ctx, vrows, vr.data, (size_t)S * b.kv_dim * 4));
    if (bias) {
        TRY(add_bias_rows(ctx, q.as<float>(), qb, S, b.q_dim));
        TRY(add_bias_rows(ctx, krows, kb, S, b.kv_dim));
        TRY(add_bias_rows(ctx, vrows, vb, S, b.kv_dim));
    }
    TRY(hm_qknorm_rope(ctx, q.as<float>(), krows, qn, kn, cosv.as<float>(), sinv.as<float>(), S, b.cfg.num_attention_heads,
                       b.kv_heads, b.head_dim, (float)b.cfg.rms_norm_eps));
    if (S == 1) return HM_OK;
    TRY(bshd_to_bhsd(ctx, krows, k.as<float>(), S, b.kv_heads, b.head_dim));
    return bshd_to_bhsd(ctx, vrows, v.as<float>(), S, b.kv_heads, b.head_dim);
}

// The attention part shared by emit_attention_kernel and emit_attention_body_kernel: q [1,S,H,hd] over the
// f32 K/V views [1,kvh,T,hd], whose last S rows are the new tokens' -> out [S][q_dim] (device pointer).
// One query row attends to all T rows (the decode mask is all zero, src/hf/precompute.rs:49-64); S rows
// attend causally, row i to keys 0 .. T - S + i.
int attention_over_views(const MemRef &q, const MemRef &k, const MemRef &v, float *out, Scratch &s, const char *who) {
    const Bound &b = g_bound;
    hm_ctx *ctx = b.ctx;
    const int S = (int)q.sizes[1], T = (int)k.sizes[2], kvh = b.kv_heads, hd = b.head_dim;
    if (T < S || k.strides[3] != 1 || v.strides[3] != 1 || v.sizes[2] != k.sizes[2])
        return hm_set_error(ctx, HM_ERR_INVALID, "%s: K/V views must hold the %d new rows and have unit inner stride", who, S);
    // the attention kernel's split partials must fit the part of the workspace left to the kernels
    if ((size_t)b.cfg.num_attention_heads * ((T + 31) / 32) * (hd + 2) * 4 > KERNEL_RESERVE)
        return hm_set_error(ctx, HM_ERR_INVALID, "%s: %d cache rows are more than this entry point takes", who, T);
    const size_t n = (size_t)kvh * T * hd;
    uint16_t *kc = s.take<uint16_t>(n), *vc = s.take<uint16_t>(n);
    if (!kc || !vc) return hm_set_error(ctx, HM_ERR_OOM, "%s: workspace too small for %d rows", who, T);
    const unsigned blocks = (unsigned)((n + 255) / 256);
    hipLaunchKernelGGL(kv_view_to_bf16_kernel, dim3(blocks), dim3(256), 0, ctx->stream, k.as<float>(), k.strides[1],
                       k.strides[2], kc, T, hd, n);
    hipLaunchKernelGGL(kv_view_to_bf16_kernel, dim3(blocks), dim3(256), 0, ctx->stream, v.as<float>(), v.strides[1],
                       v.strides[2], vc, T, hd, n);
    HM_LAUNCH_CHECK(ctx);
    const float scale = (float)(1.0 / std::sqrt((double)hd));
    if (S == 1) return hm_gqa_decode_attn(ctx, q.as<float>(), kc, vc, out, 1, b.cfg.num_attention_heads, kvh, hd, T, T, scale);
    return hm_gqa_prefill_attn(ctx, q.as<float>(), kc, vc, out, S, b.cfg.num_attention_heads, kvh, hd, T, T - S, scale);
}

// emit_attention_body_kernel (src/hf/emitter_quant.rs:922-975): q, K view, V view, mask -> [1,S,q_dim]
int run_attn_body(void **a) {
    const Bound &b = g_bound;
    const MemRef q = memref(a, 0, 4), k = memref(a, 1, 4), v = memref(a, 2, 4), out = memref(a, 4, 3);
    TRY(seq_ok(b.ctx, q.sizes[1], "AttnBody kernel"));
    Scratch s(b.ctx);
    return attention_over_views(q, k, v, out.as<float>(), s, "AttnBody kernel");
}

// emit_residual_norm_kernel (src/hf/emitter_quant.rs:985-1064): h, attn_out, ln_w -> residual, normed
int run_residual_norm(void **a) {
    const Bound &b = g_bound;
    const MemRef h = memref(a, 0, 3), attn = memref(a, 1, 3), w = memref(a, 2, 1), resid = memref(a, 3, 3),
                 normed = memref(a, 4, 3);
    TRY(seq_ok(b.ctx, h.sizes[1], "Residual+Norm kernel"));
    const int S = (int)h.sizes[1];
    TRY(hm_add(b.ctx, h.as<float>(), attn.as<float>(), resid.as<float>(), (size_t)S * b.cfg.hidden_size));
    return hm_rmsnorm(b.ctx, resid.as<float>(), w.as<float>(), normed.as<float>(), S, b.cfg.hidden_size,
                      (float)b.cfg.rms_norm_eps);
}

// emit_silu_mul_kernel (src/hf/emitter_quant.rs:1074-1100): gate, up [1,S,inter] -> [1,S,inter]
int run_silu_mul(void **a) {
    const Bound &b = g_bound;
    const MemRef g = memref(a, 0, 3), u = memref(a, 1, 3), out = memref(a, 2, 3);
    TRY(seq_ok(b.ctx, g.sizes[1], "SiLU*Up kernel"));
    return hm_silu_mul(b.ctx, g.as<float>(), u.as<float>(), out.as<float>(), (size_t)g.sizes[1] * b.cfg.intermediate_size);
}

// emit_residual_add_kernel (src/hf/emitter_quant.rs:1110-1134): residual, down_out -> hidden_out
int run_res_add(void **a) {
    const Bound &b = g_bound;
    const MemRef r = memref(a, 0, 3), d = memref(a, 1, 3), out = memref(a, 2, 3);
    TRY(seq_ok(b.ctx, r.sizes[1], "ResAdd kernel"));
    return hm_add(b.ctx, r.as<float>(), d.as<float>(), out.as<float>(), (size_t)r.sizes[1] * b.cfg.hidden_size);
}

// LM head of the quantised plan (src/hf/emitter_quant.rs:1399-1440): h, norm_w, lm_head_w f32 [hidden,vocab]
int run_lm_head_f32(void **a) {
    const Bound &b = g_bound;
    hm_ctx *ctx = b.ctx;
    const MemRef h = memref(a, 0, 3), nw = memref(a, 1, 1), lw = memref(a, 2, 2), out = memref(a, 3, 3);
    TRY(seq_ok(ctx, h.sizes[1], "LMHead kernel"));
    const int S = (int)h.sizes[1];
    const int hidden = b.cfg.hidden_size, vocab = b.cfg.vocab_size;
    Scratch s(ctx);
    float *normed = s.take<float>((size_t)S * hidden);
    if (!normed) return hm_set_error(ctx, HM_ERR_OOM, "LMHead kernel: workspace too small for %d tokens", S);
    HM_REQUIRE(ctx, (size_t)hidden * 4 <= 64 * 1024, "LMHead kernel: hidden size %d above 16384", hidden);
    TRY(hm_rmsnorm(ctx, h.as<float>(), nw.as<float>(), normed, S, hidden, (float)b.cfg.rms_norm_eps));
    for (int r = 0; r < S; r++) {
        hipLaunchKernelGGL(gemv_f32_kn_kernel, dim3((unsigned)((vocab + 255) / 256)), dim3(256), (size_t)hidden * 4, ctx->stream,
                           normed + (size_t)r * hidden, lw.as<float>(), out.as<float>() + (size_t)r * vocab, hidden, vocab);
        HM_LAUNCH_CHECK(ctx);
    }
    return HM_OK;
}

// The operands a kernel writes: (first output operand, count, rank) by kind, in each emitter's order.
void outputs_of(const KernelInfo &ki, int *first, int *count, int *rank) {
    const Bound &b = g_bound;
    const int bias = b.cfg.attention_bias ? 1 : 0, qkn = b.qk_norm ? 2 : 0;
    *count = 1;
    *rank = 3;
    switch (ki.kind) {
    case Kind::Embed: *first = 2; break;
    case Kind::Qkv: *first = 7 + 3 * bias + qkn; *count = 3; *rank = 4; break;
    case Kind::Attn: *first = 5; break;
    case Kind::Mlp: *first = 6; break;
    case Kind::LmHead: case Kind::LmHeadF32: *first = 3; break;
    case Kind::RmsNorm: case Kind::QuantMM: case Kind::SiluMul: case Kind::ResAdd: *first = 2; break;
    case Kind::PostQkv: *first = 5 + 3 * bias + qkn; *count = 3; *rank = 4; break;
    case Kind::AttnBody: *first = 4; break;
    case Kind::ResidualNorm: *first = 3; *count = 2; break;
    }
}

// After a failure no caller may mistake stale bytes for results: every output operand becomes NaN.
void poison_outputs(const KernelInfo &ki, void **args) {
    hm_ctx *ctx = g_bound.ctx;
    int first, count, rank;
    outputs_of(ki, &first, &count, &rank);
    for (int j = 0; j < count; j++) {
        const MemRef m = memref(args, first + j, rank);
        if (!m.data || rank < 1) continue;
        size_t n = 1;
        bool dense = true;  // row-major without gaps: one fill covers the operand
        for (int d = rank - 1; d >= 0; d--) {
            const size_t sz = (size_t)(m.sizes[d] > 0 ? m.sizes[d] : 0);
            if (sz > 1 && m.strides[d] != (int64_t)n) dense = false;
            n *= sz;
        }
        if (n == 0 || n >= ((size_t)1 << 34)) continue;
        if (dense) {
            (void)hipMemsetAsync(m.data, 0xFF, n * 4, ctx->stream);
            continue;
        }
        // A strided view (say, rows of one head inside a longer cache): fill run by run along the innermost
        // dimension, and only where that dimension is contiguous, so that no byte outside the operand changes.
        const size_t inner = (size_t)m.sizes[rank - 1];
        if (m.strides[rank - 1] != 1 || n / inner > ((size_t)1 << 20)) continue;
        std::vector<int64_t> idx((size_t)rank, 0);
        for (size_t run = 0; run < n / inner; run++) {
            int64_t off = 0;
            for (int d = 0; d < rank - 1; d++) off += idx[(size_t)d] * m.strides[d];
            (void)hipMemsetAsync(m.data + off * 4, 0xFF, inner * 4, ctx->stream);
            for (int d = rank - 2; d >= 0; d--) {
                if (++idx[(size_t)d] < m.sizes[d]) break;
                idx[(size_t)d] = 0;
            }
        }
    }
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipGetLastError();
}

void dispatch(int idx, void **args) {
    if (!g_bound.ctx || idx >= (int)g_bound.kinds.size()) {
        report(idx, HM_ERR_STATE);
        return;
    }
    int rc = HM_ERR_INVALID;
    const KernelInfo &ki = g_bound.kinds[idx];
    switch (ki.kind) {
    case Kind::Embed: rc = run_embed(args); break;
    case Kind::Qkv: rc = run_qkv(args); break;
    case Kind::Attn: rc = run_attn(args); break;
    case Kind::Mlp: rc = run_mlp(args); break;
    case Kind::LmHead: rc = run_lm_head(args); break;
    case Kind::RmsNorm: rc = run_rms_norm(args); break;
    case Kind::QuantMM: rc = run_quant_mm(args, ki); break;
    case Kind::PostQkv: rc = run_post_qkv(args); break;
    case Kind::AttnBody: rc = run_attn_body(args); break;
    case Kind::ResidualNorm: rc = run_residual_norm(args); break;
    case Kind::SiluMul: rc = run_silu_mul(args); break;
    case Kind::ResAdd: rc = run_res_add(args); break;
    case Kind::LmHeadF32: rc = run_lm_head_f32(args); break;
    }
    if (rc != HM_OK) poison_outputs(ki, args);
    report(idx, rc);
}

int bind_common(hm_ctx *ctx, const hm_transformer_config *cfg, int has_qk_norm, int kernels, Bound *out) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, cfg, "hm_ciface_bind_transformer: NULL config");
    const int kvh = cfg->num_key_value_heads ? cfg->num_key_value_heads : cfg->num_attention_heads;
    HM_REQUIRE(ctx, cfg->hidden_size > 0 && cfg->num_attention_heads > 0 && cfg->num_hidden_layers > 0 &&
                        cfg->num_attention_heads % kvh == 0,
               "hm_ciface_bind_transformer: bad config");
    HM_REQUIRE(ctx, kernels <= HM_CIFACE_MAX_KERNELS, "hm_ciface_bind_transformer: %d kernels, at most %d symbols are exported",
               kernels, HM_CIFACE_MAX_KERNELS);
    Bound b;
    b.ctx = ctx;
    b.cfg = *cfg;
    b.qk_norm = has_qk_norm != 0;
    b.kv_heads = kvh;
    b.head_dim = cfg->head_dim ? cfg->head_dim : cfg->hidden_size / cfg->num_attention_heads;
    b.q_dim = cfg->num_attention_heads * b.head_dim;
    b.kv_dim = kvh * b.head_dim;
    if (b.cfg.rms_norm_eps <= 0) b.cfg.rms_norm_eps = 1e-6;
    *out = std::move(b);
    return HM_OK;
}

}  // namespace

extern "C" {

int hm_ciface_bind_transformer_quant(hm_ctx *ctx, const hm_transformer_config *cfg, const int *proj_dtypes,
                                     int has_qk_norm) {
    Bound b;
    const int rc = bind_common(ctx, cfg, has_qk_norm, cfg ? 13 * cfg->num_hidden_layers + 2 : 0, &b);
    if (rc != HM_OK) return rc;
    HM_REQUIRE(ctx, proj_dtypes, "hm_ciface_bind_transformer_quant: NULL projection types");
    const int hidden = cfg->hidden_size, inter = cfg->intermediate_size;
    const int kdim[7] = {hidden, hidden, hidden, b.q_dim, hidden, hidden, inter};
    const int ndim[7] = {b.q_dim, b.kv_dim, b.kv_dim, hidden, inter, inter, hidden};
    b.kinds.push_back(Kind::Embed);
    for (int l = 0; l < cfg->num_hidden_layers; l++) {
        const int *t = proj_dtypes + 7 * l;
        for (int j = 0; j < 7; j++) {
            const bool kq = t[j] == HM_DTYPE_Q4_K || t[j] == HM_DTYPE_Q6_K;
            HM_REQUIRE(ctx, kq || t[j] == HM_DTYPE_Q8_0 || t[j] == HM_DTYPE_Q4_0,
                       "hm_ciface_bind_transformer_quant: layer %d projection %d: dtype %d is not a block format", l, j, t[j]);
            HM_REQUIRE(ctx, kdim[j] % (kq ? 256 : 32) == 0, "hm_ciface_bind_transformer_quant: layer %d projection %d: K=%d", l, j,
                       kdim[j]);
        }
        auto mm = [&](int j) { return KernelInfo(kdim[j], ndim[j], t[j]); };
        b.kinds.push_back(Kind::RmsNorm);
        b.kinds.push_back(mm(0));
        b.kinds.push_back(mm(1));
        b.kinds.push_back(mm(2));
        b.kinds.push_back(Kind::PostQkv);
        b.kinds.push_back(Kind::AttnBody);
        b.kinds.push_back(mm(3));
        b.kinds.push_back(Kind::ResidualNorm);
        b.kinds.push_back(mm(4));
        b.kinds.push_back(mm(5));
        b.kinds.push_back(Kind::SiluMul);
        b.kinds.push_back(mm(6));
        b.kinds.push_back(Kind::ResAdd);
    }
    b.kinds.push_back(Kind::LmHeadF32);
    g_bound = std::move(b);
    return HM_OK;
}

int hm_ciface_bind_transformer(hm_ctx *ctx, const hm_transformer_config *cfg, int has_qk_norm) {
    Bound b;
    const int rc = bind_common(ctx, cfg, has_qk_norm, cfg ? 3 * cfg->num_hidden_layers + 2 : 0, &b);
    if (rc != HM_OK) return rc;
    b.kinds.push_back(Kind::Embed);
    for (int l = 0; l < cfg->num_hidden_layers; l++) {
        b.kinds.push_back(Kind::Qkv);
        b.kinds.push_back(Kind::Attn);
        b.kinds.push_back(Kind::Mlp);
    }
    b.kinds.push_back(Kind::LmHead);
    g_bound = std::move(b);
    return HM_OK;
}

int hm_ciface_num_kernels(void) { return (int)g_bound.kinds.size(); }

void hm_ciface_unbind(void) { g_bound = Bound(); }

int hm_ciface_last_status(int *kernel_index) {
    if (kernel_index) *kernel_index = g_status_kernel;
    return g_status;
}

void hm_ciface_clear_status(void) {
    g_status = HM_OK;
    g_status_kernel = -1;
}

// HM_CIFACE_MAX_KERNELS exported symbols _mlir__mlir_ciface_k0 ... _mlir__mlir_ciface_k1023
#define HM_K(i) \
    __attribute__((visibility("default"))) void _mlir__mlir_ciface_k##i(void **args) { dispatch(i, args); }
#define HM_K10(p) HM_K(p##0) HM_K(p##1) HM_K(p##2) HM_K(p##3) HM_K(p##4) HM_K(p##5) HM_K(p##6) HM_K(p##7) HM_K(p##8) HM_K(p##9)
#define HM_K100(p) HM_K10(p##0) HM_K10(p##1) HM_K10(p##2) HM_K10(p##3) HM_K10(p##4) HM_K10(p##5) HM_K10(p##6) HM_K10(p##7) HM_K10(p##8) HM_K10(p##9)
HM_K(0) HM_K(1) HM_K(2) HM_K(3) HM_K(4) HM_K(5) HM_K(6) HM_K(7) HM_K(8) HM_K(9)
HM_K10(1) HM_K10(2) HM_K10(3) HM_K10(4) HM_K10(5) HM_K10(6) HM_K10(7) HM_K10(8) HM_K10(9)
HM_K100(1) HM_K100(2) HM_K100(3) HM_K100(4) HM_K100(5) HM_K100(6) HM_K100(7) HM_K100(8) HM_K100(9)
HM_K10(100) HM_K10(101)
HM_K(1020) HM_K(1021) HM_K(1022) HM_K(1023)
#undef HM_K100
#undef HM_K10
#undef HM_K

}  // extern "C"
