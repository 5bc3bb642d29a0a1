/*
 * homura_amd — MI355X (gfx950) kernels for Homura's batch-1 decode hot path.
 *
 * This header is the drop-in boundary. In the reference every heavy op is a symbol
 * `_mlir__mlir_ciface_k{idx}(void** args)` in a dlopen'ed CPU kernel library, called by
 * `CompiledGraph::run_with_output_bufs` (reference src/runtime.rs:930-1037) with memref
 * descriptors built by `build_memref_descriptor` (src/runtime.rs:664-698). Here the same
 * ops are plain C entry points over HBM-resident buffers: pointers named `d_*` are device
 * pointers obtained from hm_alloc(); everything else is host memory. Each entry point cites
 * the reference kernel it stands in for.
 *
 * Conventions
 *  - every function returns HM_OK (0) or a negative HM_ERR_*; hm_last_error() gives the text.
 *    (The reference's kernels return void and panic in Rust; a GPU call can fail, so the
 *    boundary carries a status.)
 *  - one hm_ctx = one GPU + one HIP stream; all kernels are enqueued on that stream and are
 *    asynchronous; hm_download() and hm_sync() are the blocking calls. One host thread per
 *    context at a time (the reference serialises runs under a Mutex, src/hf/model.rs:205).
 *  - activations, norms, logits are f32; bf16 values travel as uint16_t (top half of an f32,
 *    reference src/hf/safetensors.rs:105-115); quantised weights are raw GGUF block bytes.
 */
#ifndef HOMURA_AMD_H
#define HOMURA_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* every declaration below is exported from libhomura_amd.so */
#pragma GCC visibility push(default)

#define HM_OK 0
#define HM_ERR_INVALID (-1) /* bad argument / shape the kernels do not support */
#define HM_ERR_HIP (-2)     /* a HIP runtime call failed */
#define HM_ERR_OOM (-3)     /* device allocation failed */
#define HM_ERR_STATE (-4)   /* call made in the wrong state (e.g. KV cache full) */

typedef struct hm_ctx hm_ctx;

/* ── context, memory, stream (replaces the reference's Vec<u8>-backed Buffer,
 *    src/runtime.rs:35-299, for device residency) ───────────────────────────── */
hm_ctx *hm_init(int device);       /* NULL on failure: see hm_last_error(NULL) */
void hm_destroy(hm_ctx *ctx);
const char *hm_last_error(hm_ctx *ctx); /* ctx may be NULL for hm_init failures */
int hm_alloc(hm_ctx *ctx, size_t bytes, void **d_out);
int hm_free(hm_ctx *ctx, void *d_ptr);
int hm_upload(hm_ctx *ctx, void *d_dst, const void *h_src, size_t bytes);
int hm_download(hm_ctx *ctx, void *h_dst, const void *d_src, size_t bytes);
int hm_copy(hm_ctx *ctx, void *d_dst, const void *d_src, size_t bytes);
int hm_fill_zero(hm_ctx *ctx, void *d_dst, size_t bytes);
int hm_sync(hm_ctx *ctx);
void *hm_stream(hm_ctx *ctx); /* the context's hipStream_t */
int hm_device_name(hm_ctx *ctx, char *buf, size_t buflen);

/* HIP-event timing on the context stream (the GPU-side analogue of the reference's
 * HOMURA_PROFILE Instant timers, src/runtime.rs:1676-1681). */
int hm_event_create(hm_ctx *ctx, void **ev_out);
int hm_event_destroy(hm_ctx *ctx, void *ev);
int hm_event_record(hm_ctx *ctx, void *ev);
int hm_event_elapsed_ms(hm_ctx *ctx, void *ev_start, void *ev_stop, float *ms_out);

/* Stream capture for launch-bound loops: every kernel-level entry point called between
 * hm_graph_begin and hm_graph_end is recorded instead of run (no hm_alloc / hm_free / hm_upload /
 * hm_download / hm_sync in between); hm_graph_launch replays the recording `reps` times.
 * No counterpart in the reference (its kernels are plain host function calls). */
int hm_graph_begin(hm_ctx *ctx);
int hm_graph_end(hm_ctx *ctx, void **graph_out);
int hm_graph_launch(hm_ctx *ctx, void *graph, int reps);
int hm_graph_destroy(hm_ctx *ctx, void *graph);

/* ── heavy ops ─────────────────────────────────────────────────────────────── */

/* bf16-weight matmul, reference GraphBuilder::emit_matmul 3D x 2D arm with the mixed
 * f32 x bf16 region (src/graph_builder/emit_linalg.rs:1328-1339, :1928-2008, :2224-2307):
 * out[m,n] = sum_k x[m,k] * f32(W[k,n]); x f32 [M,K], W bf16 [K,N] row-major (the layout
 * the reference hands its kernels, src/hf/weights.rs:225-261), out f32 [M,N].
 * M <= 8, N % 4 == 0. */
int hm_gemv_bf16(hm_ctx *ctx, const float *d_x, const uint16_t *d_w_kn, float *d_out, int M,
                 int K, int N);

/* One-time re-pack of a [K,N] bf16 weight into the K-contiguous [N,K] stream layout
 * (which is also HuggingFace's native [out,in] layout, i.e. the reference's load-time
 * transpose_2d of src/hf/weights.rs:225-261 undone). */
int hm_pack_bf16_kn_to_nk(hm_ctx *ctx, const uint16_t *d_w_kn, uint16_t *d_w_nk, int K, int N);

/* Same contraction as hm_gemv_bf16 on the [N,K] stream layout. M <= 8, K % 8 == 0. */
int hm_gemv_bf16_nk(hm_ctx *ctx, const float *d_x, const uint16_t *d_w_nk, float *d_out, int M,
                    int K, int N);

/* Q8_0 dequant-matmul, reference emit_dequant_matmul_q8_0
 * (src/graph_builder/emit_quant.rs:30-142): weight = raw GGUF blocks [N][K/32] x 34 bytes
 * (LE f16 d + 32 int8), out[m,n] = sum_k x[m,k] * (q * d). M <= 8, K % 32 == 0, K <= 16384. Rows above
 * about 7700 (Q4_0: 14500) do not fit the kernel's LDS stage: such a call re-packs the blocks into planes in the
 * context's workspace first (the planes must fit it: 64 MiB) and multiplies those - a caller that owns its
 * device copies packs once (hm_pack_quant_planes) and calls hm_gemv_q8_0_planes. */
int hm_gemv_q8_0(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M,
                 int K, int N);

/* Q4_0 dequant-matmul. The reference parses the type (src/gguf.rs:28,116,141) but has no
 * kernel for it (src/gguf.rs:94-108); blocks are ggml block_q4_0: [N][K/32] x 18 bytes
 * (LE f16 d + 16 bytes, byte j = element j low nibble, element j+16 high nibble),
 * w = (q - 8) * d. M <= 8, K % 32 == 0. */
int hm_gemv_q4_0(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M,
                 int K, int N);

/* The same two products over weights re-packed once into "planes": the quant bytes of all blocks row after
 * row (Q8_0: K bytes a row; Q4_0: K / 2, each block's 16 bytes as in the file), then, from the next
 * multiple of 256 bytes, the f16 scales of all blocks row after row. The bytes are those of the GGUF blocks
 * (src/graph_builder/emit_quant.rs:17-21 layout) in another order: quant words sit at their natural
 * alignment and are loaded straight into registers. hm_quant_planes_bytes gives the size of the planes
 * of an [N][K] matrix (0 for a type other than HM_DTYPE_Q8_0 / Q4_0 / Q6_K or a bad shape), hm_pack_quant_planes
 * fills them from raw blocks [N][K/32] in one launch, hm_unpack_quant_planes is its inverse.
 * Results equal hm_gemv_q8_0 / hm_gemv_q4_0 up to the order of the f32 additions. M <= 8, K % 32 == 0,
 * K <= 16384 (rows above 4096 are cut across the wavefronts of a workgroup). hm_dequant_quant_planes writes the N * K dequantised weights, bit-exact with the CPU. */
size_t hm_quant_planes_bytes(int hm_dtype, int N, int K);
int hm_pack_quant_planes(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, uint8_t *d_planes, int N, int K);
int hm_unpack_quant_planes(hm_ctx *ctx, int hm_dtype, const uint8_t *d_planes, uint8_t *d_blocks, int N, int K);
int hm_gemv_q8_0_planes(hm_ctx *ctx, const float *d_x, const uint8_t *d_planes, float *d_out, int M, int K, int N);
int hm_gemv_q4_0_planes(hm_ctx *ctx, const float *d_x, const uint8_t *d_planes, float *d_out, int M, int K, int N);
int hm_dequant_quant_planes(hm_ctx *ctx, int hm_dtype, const uint8_t *d_planes, float *d_out, int N, int K);

/* Q6_K planes (the same four functions with HM_DTYPE_Q6_K; K % 256 == 0). A 210-byte block (src/gguf.rs:880-917)
 * interleaves four 16-weight groups in every byte run; the unit that shares bytes is 64 weights (groups g, g + 2,
 * g + 4, g + 6 of one 128-weight half, l in 0..15 or 16..31). The planes hold, for all units of all rows in
 * order: [units][32] low nibbles (ql[64h + 16p + j], then ql[64h + 32 + 16p + j], j = 0..15), from the next
 * multiple of 256 bytes [units][16] top bits (qh[32h + 16p + j]), then [units][4] int8 scales (sc[8h + p + 2g]),
 * then [blocks] f16 d; unit 2h + p of a block. hm_gemv_q6_k_f32_planes is hm_gemv_q6_k_f32 over them
 * (f32 row x dequantised weights, the product of a Q6_K LM head; results equal up to the order of the f32
 * additions) for K = 256, 512, 1024, 2048 or 4096 and M <= 8. */
int hm_gemv_q6_k_f32_planes(hm_ctx *ctx, const float *d_x, const uint8_t *d_planes, float *d_out, int M, int K, int N);

/* Block dequantisation to f32, reference dequant_q8_0 (src/gguf.rs:817-831): one f32
 * multiply per element, bit-exact with the CPU. hm_dequant_q4_0 is its Q4_0 analogue. */
int hm_dequant_q8_0(hm_ctx *ctx, const uint8_t *d_blocks, float *d_out, size_t nblocks);
int hm_dequant_q4_0(hm_ctx *ctx, const uint8_t *d_blocks, float *d_out, size_t nblocks);

/* K-quants, reference emit_dequant_matmul_q4_k / _q6_k (src/graph_builder/emit_quant.rs:165-816):
 * the f32 activation is quantised to Q8_K per 256-wide block (scale amax/127, round half to even),
 * then integer dot products per sub-block against the raw GGUF super-blocks [N][K/256] x 144 B
 * (Q4_K) or 210 B (Q6_K). K % 256 == 0, K <= 16384, M <= 8. The integer sums are the reference's; the
 * f32 adds over units and blocks come in a different order. */
int hm_gemv_q4_k(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M, int K, int N);
int hm_gemv_q6_k(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M, int K, int N);
/* The same product over the "K8" form of a Q4_K / Q6_K matrix, for a caller that keeps its weights on the device:
 * every weight as one signed byte in a plane [N][K] (Q4_K: the nibble; Q6_K: the 6-bit value - 32), then, from byte
 * N * K on, a record of K / 8 + K / 64 bytes per row: (scale, minimum factor) per 16 weights, then the f16 (d, dmin)
 * per 256 - the same integers as the blocks at 1.14 bytes a weight, both types alike, so matrices of either type can be
 * stacked by rows and multiplied in one call. hm_k8_bytes gives the size (0 for a bad shape), hm_pack_k8 fills rows
 * [row0, row0 + rows) of a K8 matrix of N rows from `rows` rows of raw blocks of one type. hm_gemv_k8: the
 * activation row is quantised to Q8_K inside the launch (no pass through memory), integer sums as the reference's
 * (emit_quant.rs:165-816, :422-466). K % 256 == 0, K <= 16384, M <= 8. This is what the model's decode reads. */
size_t hm_k8_bytes(int N, int K);
int hm_pack_k8(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int rows, uint8_t *d_k8, int N, int K, int row0);
int hm_gemv_k8(hm_ctx *ctx, const float *d_x, const uint8_t *d_k8, float *d_out, int M, int K, int N);
/* The f32 product with the dequantised weights: out[m][n] = sum_k x[m][k] * w[n][k], w = dequant_q4_k /
 * dequant_q6_k of the blocks (src/gguf.rs:835-917). This is what the reference computes where a K-quant
 * tensor feeds an f32 kernel: its loader dequantises the embedding and output matrices
 * (GgufFile::load_transformer_weights, src/gguf.rs:589-708) and the LM head multiplies f32 by f32
 * (emit_lm_head_kernel, src/hf/emitter.rs:828-862). The blocks are read as they are (144 / 210 bytes per
 * 256 weights instead of 1024) and every weight enters as the exact dequantised value. K % 256 == 0,
 * K <= 4096, M <= 8. */
int hm_gemv_q4_k_f32(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M, int K, int N);
int hm_gemv_q6_k_f32(hm_ctx *ctx, const float *d_x, const uint8_t *d_w_blocks, float *d_out, int M, int K, int N);
/* The Q8_K activation quantisation on its own (emit_quant.rs:422-466): d_q8 int8 [M][K], d_act_d f32
 * [M][K/256], d_bsums int32 [M][K/16] (sums of 16 consecutive q). Bit-exact with the CPU. */
int hm_quantize_q8_k(hm_ctx *ctx, const float *d_x, int8_t *d_q8, float *d_act_d, int32_t *d_bsums, int M, int K);
/* dequant_q4_k / dequant_q6_k (src/gguf.rs:835-917), 256 weights per block, bit-exact with the CPU. */
int hm_dequant_q4_k(hm_ctx *ctx, const uint8_t *d_blocks, float *d_out, size_t nblocks);
int hm_dequant_q6_k(hm_ctx *ctx, const uint8_t *d_blocks, float *d_out, size_t nblocks);

/* Prefill-chunk GEMM on the matrix cores: the reference runs the same emit_matmul with
 * seq > 1 (docs/kv-cache.md:31-37); here A bf16 [M,K], B bf16 [K,N] (reference layout),
 * C f32 [M,N], f32 accumulate. K % 32 == 0, N % 8 == 0; any M (tiles are 128 x 128, partial
 * tiles at the edges cost a whole one). */
int hm_gemm_bf16(hm_ctx *ctx, const uint16_t *d_a_mk, const uint16_t *d_b_kn, float *d_c, int M,
                 int K, int N);
/* Same product with B in the stream layout [N,K] (what hm_pack_bf16_kn_to_nk writes and the
 * decode GEMVs read), so prefill and decode share one copy of a weight. K % 32 == 0, any M and N. */
int hm_gemm_bf16_nk(hm_ctx *ctx, const uint16_t *d_a_mk, const uint16_t *d_b_nk, float *d_c, int M,
                    int K, int N);

/* The reference's mixed matmul at seq > 1 (make_mixed_matmul_region,
 * src/graph_builder/emit_linalg.rs:2224-2307): x f32 [M,K] times W bf16 in the stream layout [N,K],
 * out f32 [M,N]. Each activation enters the bf16 MFMA as three bf16 numbers (its bf16 rounding, the
 * rounding of what is left, and again), which together hold all 24 significant bits, so the
 * products are those of the f32 value. K % 32 == 0; M * K * 6 bytes must fit in the context
 * workspace (64 MiB). */
int hm_gemm_f32_bf16_nk(hm_ctx *ctx, const float *d_x_mk, const uint16_t *d_w_nk, float *d_out, int M, int K,
                        int N);

/* The reference's quantised matmul at seq > 1 (emit_quant_matmul_kernel,
 * src/hf/emitter_quant.rs:675-702; src/graph_builder/emit_quant.rs): x f32 [M,K] times a block-
 * quantised W (raw GGUF blocks [N][K / block], dtype HM_DTYPE_Q8_0 / Q4_0 / Q4_K / Q6_K), out f32
 * [M,N], on the matrix cores. The weights are dequantised to f32 with the reference's arithmetic and,
 * like the activations, carried as three bf16 pieces; the six piece products that matter are
 * accumulated in f32, so the result is the f32 product up to rounding. For the K-quants every
 * activation row first goes through the Q8_K quantisation the reference applies (per 256-wide block:
 * scale amax / 127, round half to even, clamp +-127), and the product is taken with scale * q, which
 * is what its integer dot products add up to. K % 64 == 0 (K % 256 for the K-quants); the split
 * activations (M * K * 6 bytes) and at least 128 split weight rows must fit in the context
 * workspace. */
int hm_gemm_f32_quant_nk(hm_ctx *ctx, const float *d_x_mk, const uint8_t *d_w_blocks, int dtype, float *d_out,
                         int M, int K, int N);

/* ── KV cache + attention ──────────────────────────────────────────────────── */

/* KvCache::append_key / append_value (src/runtime.rs:521-568) on an HBM cache
 * [B][kvh][max_len][hd] bf16: rows d_k/d_v f32 [B][kvh][n_new][hd] (BHSD, as the
 * reference's QKV kernel emits them) are rounded to bf16 (nearest-even) and written at
 * row `pos`. Fails with HM_ERR_STATE when pos + n_new > max_len (the reference panics
 * "KV cache full"). */
int hm_kv_append(hm_ctx *ctx, uint16_t *d_kcache, uint16_t *d_vcache, const float *d_k,
                 const float *d_v, int B, int kvh, int hd, int max_len, int pos, int n_new);

/* Decode attention, the attention part of reference emit_attention_kernel
 * (src/hf/emitter.rs:709-737; emit_gqa_qk_transpose / emit_softmax / emit_gqa_av,
 * src/graph_builder/emit_linalg.rs:93-245, :509-528): one query row per sequence,
 * q f32 [B][H][hd]; K,V bf16 caches [B][kvh][max_len][hd] of which rows [0,kv_len) are
 * attended (the all-zero decode mask of src/hf/precompute.rs:49-64); kv head = h / (H/kvh);
 * scores * scale, softmax in f32, out f32 [B][H*hd]. hd == 128 or 64. The cache rows are split over
 * workgroups and a second launch folds the partial sums in row order; with more than 128 rows per
 * workgroup (long caches, many sequences) the workgroups walk their rows in steps and take both products
 * on the matrix cores, q and the probabilities as two bf16 pieces each (2^-17 of an element left out). */
int hm_gqa_decode_attn(hm_ctx *ctx, const float *d_q, const uint16_t *d_kcache,
                       const uint16_t *d_vcache, float *d_out, int B, int H, int kvh, int hd,
                       int max_len, int kv_len, float scale);

/* hm_gqa_decode_attn for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it). It has no counterpart in the reference. Same
 * arguments, kernels and results; the splits' partial sums go to a fixed array inside the library
 * (hm_gqa_decode_attn_noalloc_limit() bytes, 4 MiB, held by each GPU the library runs on until the
 * process ends) whose device address hm_init resolves once per context. The call allocates nothing
 * and fails with HM_ERR_INVALID when B * kv_heads * splits * (H / kv_heads) * (hd + 2) * 4 bytes exceed
 * the limit. Nothing in the array has to start at zero (every partial is written before it is read),
 * but all calls on one GPU share it: calls that overlap on one GPU (two streams, two contexts) race. */
int hm_gqa_decode_attn_noalloc(hm_ctx *ctx, const float *d_q, const uint16_t *d_kcache,
                               const uint16_t *d_vcache, float *d_out, int B, int H, int kvh, int hd,
                               int max_len, int kv_len, float scale);
size_t hm_gqa_decode_attn_noalloc_limit(void);

/* Causal attention of S new query rows at positions past .. past + S - 1 over cache rows
 * [0, past + S), batch 1: the attention part of emit_attention_kernel (src/hf/emitter.rs:709-737)
 * under the mask of build_causal_mask (src/hf/precompute.rs:134-161: key j is visible to query i
 * when j <= past + i). q f32 [S][H][hd], already normed and rotated; the S new K/V rows must be in
 * the caches [kvh][max_len][hd] bf16 already (hm_kv_append); out f32 [S][H*hd]. hd = 64 or 128.
 * QK^T and PV run on the matrix cores with q and the probabilities carried as three bf16 numbers
 * each (all 24 significant bits). */
int hm_gqa_prefill_attn(hm_ctx *ctx, const float *d_q, const uint16_t *d_kcache, const uint16_t *d_vcache,
                        float *d_out, int S, int H, int kvh, int hd, int max_len, int past, float scale);

/* ── light ops ─────────────────────────────────────────────────────────────── */

/* emit_rms_norm (src/graph_builder/emit_linalg.rs:7-26): out = (x * rsqrt(mean(x^2)+eps)) * w
 * per row; x,out f32 [rows][dim], w f32 [dim]. */
int hm_rmsnorm(hm_ctx *ctx, const float *d_x, const float *d_w, float *d_out, int rows, int dim,
               float eps);

/* The per-head QK-norm + emit_rope_half tail of emit_qkv_kernel (src/hf/emitter.rs:629-644,
 * src/graph_builder/emit_linalg.rs:315-342), in place: q f32 [S][H][hd], k f32 [S][kvh][hd];
 * d_qw/d_kw f32 [hd] or NULL (no QK-norm); cos/sin f32 [S][hd] (rows already sliced for the
 * positions, src/hf/precompute.rs:73-101). */
int hm_qknorm_rope(hm_ctx *ctx, float *d_q, float *d_k, const float *d_qw, const float *d_kw,
                   const float *d_cos, const float *d_sin, int S, int H, int kvh, int hd,
                   float eps);

/* silu(gate) * up (src/graph_builder/emit_arithmetic.rs:101-107, src/hf/emitter.rs:797-799). */
int hm_silu_mul(hm_ctx *ctx, const float *d_gate, const float *d_up, float *d_out, size_t n);
/* residual add (src/hf/emitter.rs:787, :804). */
int hm_add(hm_ctx *ctx, const float *d_a, const float *d_b, float *d_out, size_t n);
/* emit_embed_kernel (src/hf/emitter.rs:506-537): out[i,:] = table[ids[i],:]. */
int hm_embed(hm_ctx *ctx, const int64_t *d_ids, const float *d_table, float *d_out, int n_ids,
             int vocab, int hidden);
/* greedy pick of src/generate.rs:457-468 / :735-742: index of the maximum; of equal maxima
 * the LAST (Rust Iterator::max_by). Writes one int32 to d_index_out. */
int hm_argmax(hm_ctx *ctx, const float *d_values, int n, int32_t *d_index_out);

/* ── sampling ─────────────────────────────────────────────────────────────────── */

/* SamplingConfig (src/generate.rs:646-686) without the stop strings and the seed; the reference's
 * defaults are temperature 0.7, top_k 50, top_p 0.9, min_p 0, repetition_penalty 1.1, others 0. */
typedef struct hm_sampling_config {
    float temperature; /* <= 0: greedy */
    int top_k;         /* 0: no cut */
    float top_p;
    float min_p;
    float repetition_penalty;
    float frequency_penalty;
    float presence_penalty;
} hm_sampling_config;

/* Rng (src/generate.rs:609-642): xorshift64 with shifts 13, 7, 17; the state is seed | 1; next_f32 is
 * the top 24 bits over 2^24. Host functions, no context needed. */
uint64_t hm_rng_seed(uint64_t seed);
float hm_rng_next_f32(uint64_t *state);

/* sample_token (src/generate.rs:698-801) on a host logits row, statement by statement: repetition penalty
 * once per occurrence in generated_ids, frequency / presence penalties, greedy when temperature <= 0
 * (last of equal maxima, the stream is not advanced), temperature, softmax with sequential f32 sums,
 * min_p, sort by probability (equal probabilities keep index order; the reference's unstable sort leaves
 * that open), top_k, top_p, one draw. No GPU involved. */
int hm_sample_token_host(const float *h_logits, int vocab, const hm_sampling_config *cfg,
                         const uint32_t *h_generated, int n_generated, uint64_t *rng_state, int32_t *token_out);
/* The same procedure on a logits row in HBM (the row never crosses PCIe; 4 bytes come back). Needs
 * 1 <= top_k <= 1024 when temperature > 0. The vocabulary-wide sum of exponentials is a tree sum, so
 * the pick can differ from the host's only when the draw sits on a cumulative boundary to within the
 * last bit of a probability. */
int hm_sample_token(hm_ctx *ctx, const float *d_logits, int vocab, const hm_sampling_config *cfg,
                    const uint32_t *h_generated, int n_generated, uint64_t *rng_state, int32_t *token_out);

/* ── host-side mirror of Model / ExecutionPlan / KvCache, C view ─────────────
 * The C++ classes in homura_amd/csrc/host/ keep the reference's names (HfModel,
 * ExecutionPlan, KernelStep, KvCache, Buffer); these functions are their C handles. */

typedef struct hm_model hm_model;

/* reference TransformerConfig (src/hf/config.rs:11-73) */
typedef struct {
    int hidden_size;
    int intermediate_size;
    int num_attention_heads;
    int num_hidden_layers;
    int num_key_value_heads; /* 0 => num_attention_heads */
    int vocab_size;
    int head_dim;            /* 0 => hidden_size / num_attention_heads */
    int max_position_embeddings;
    int tie_word_embeddings;
    double rms_norm_eps;
    double rope_theta;
    int attention_bias;      /* Q/K/V projections carry a bias (Qwen2-style); the reference reads this
                                off the checkpoint (src/hf/weights.rs:64-69) */
    int eos_token_id;        /* -1 => none (the reference's Option<u32>, src/hf/config.rs:32-35; GGUF: */
    int bos_token_id;        /*  tokenizer.ggml.eos_token_id / bos_token_id, src/gguf.rs:559-565) */
} hm_transformer_config;

#define HM_DTYPE_F32 0
#define HM_DTYPE_BF16 1
#define HM_DTYPE_Q8_0 2
#define HM_DTYPE_Q4_0 3
#define HM_DTYPE_I64 4
#define HM_DTYPE_Q4_K 5
#define HM_DTYPE_Q6_K 6

/* HfModel::load_with_dtype / load_gguf stand-in (src/hf/model.rs:46-145) for weights that
 * are already in host memory: create, hand over every weight slot in
 * TransformerWeights::to_slot_buffers order (src/hf/weights.rs:63-116, :136-183), finalize.
 * `weight_dtype` is the dtype of the seven projections (BF16, Q8_0 or Q4_0). */
hm_model *hm_model_create(hm_ctx *ctx, const hm_transformer_config *cfg, int weight_dtype,
                          int has_qk_norm);
/* A quantised model whose projections do not all share one type (Q4_K_M files keep some in Q6_K):
 * proj_dtypes holds 7 HM_DTYPE_* codes per layer in the order q, k, v, o, gate, up, down. The
 * reference carries the type per weight buffer (Buffer dtype, src/hf/weights.rs:136-183). */
hm_model *hm_model_create_mixed(hm_ctx *ctx, const hm_transformer_config *cfg, const int *proj_dtypes,
                                int has_qk_norm);
void hm_model_destroy(hm_model *m);
int hm_model_num_weight_slots(hm_model *m);
/* name is copied into buf; dtype/rows/cols describe the host buffer expected for the slot */
int hm_model_weight_slot_info(hm_model *m, int slot, char *name_buf, size_t buflen, int *dtype,
                              int64_t *dim0, int64_t *dim1, size_t *bytes);
int hm_model_set_weight(hm_model *m, int slot, const void *h_data, size_t bytes);
/* ensure_compiled (src/hf/model.rs:148-160): builds the ExecutionPlan, RoPE tables, packs. */
int hm_model_finalize(hm_model *m, int max_seq_len);

/* ExecutionPlan::init_kv_cache (src/runtime.rs:1898-1938): h_kv = 2*layers host buffers
 * (K,V alternating) of f32 [1][kvh][seq_len][hd]; rounds to bf16 into the HBM cache. */
int hm_model_init_kv_cache(hm_model *m, const float *const *h_kv, int seq_len);
int hm_model_reset_kv_cache(hm_model *m);  /* src/runtime.rs:1941-1945 */
int hm_model_kv_cache_len(hm_model *m);    /* src/runtime.rs:1948-1950 */

/* Replay every decode step from one captured HIP graph (on != 0) or launch kernel by kernel. A step of
 * one or two launches (the whole-step kernel) is launched directly either way: that is quicker than replaying
 * a graph of one node. No counterpart in the reference (its plan is a host loop over dlsym'ed functions). */
int hm_model_set_graph(hm_model *m, int on);

/* One launch for a whole decode step's embedding row and decoder layers (on != 0) instead of one
 * launch per projection; the reference dispatches 1 + 3 * layers + 1 kernels per step
 * (src/hf/emitter.rs:1016-1021). Served for bf16, all-Q8_0, all-Q4_0 and Q4_K / Q6_K (in any mix per
 * projection) models whose shape has a kernel instance (hm_model_whole_step_available); on by default then, and for bf16 models the same launch runs the
 * LM head and the greedy pick. The cache may be of any length: a step takes the instance of the kernel that
 * holds its live rows (1536, 2048, 3072, 4096 or 32768 of them; the smaller the faster; the last streams the rows beyond
 * 4096 inside its attention phase), beyond 32768 the per-projection path, chosen step by step. Results agree with the per-projection
 * path to f32 summation order.
 *
 * The launch needs all its workgroups (one per compute unit) resident at once, since they wait for one
 * another: one whole-step model per GPU at a time, and nothing else that holds compute units while it
 * steps. Every wait is bounded. When one runs into its bound (the grid was not resident as a whole), the
 * launch ends normally without moving the cursor, and the call that finds the status - hm_model_run_kv,
 * hm_model_generate_greedy, hm_model_generate, hm_model_bench_decode - clears the exchange state, takes
 * the cache back to where it found it, and runs its steps again with one launch per projection, as do the
 * calls after it; it returns what that second run returns. hm_model_whole_step_status then keeps returning
 * the error the launch left behind (phase, layer and workgroup of the first wait that gave up) until
 * hm_model_reset_kv_cache or hm_model_set_whole_step(m, 1) re-arms the launch. It also reports, once, a
 * fed-back token id outside the vocabulary or a step whose logits held no finite value (both decoded as
 * token 0). */
int hm_model_set_whole_step(hm_model *m, int on);
int hm_model_whole_step(hm_model *m);
int hm_model_whole_step_available(hm_model *m);
int hm_model_whole_step_status(hm_model *m);
/* Test support, no counterpart in the reference: the next whole-step launches give up a wait after
 * `spin_limit` polls (instead of 2^20), and workgroup `workgroup` withholds its first publish, so that every
 * workgroup runs into that bound and the launch ends normally with its status set. Cleared by the recovery
 * described above. */
int hm_model_whole_step_inject_timeout(hm_model *m, int workgroup, int spin_limit);

/* HfModel::run_kv (src/hf/model.rs:198-218) -> ExecutionPlan::run_kv
 * (src/runtime.rs:1580-1892): n_ids new tokens on top of the cache; h_logits receives
 * [n_ids][vocab] f32 (may be NULL to skip the download). Advances the cache by n_ids. */
int hm_model_run_kv(hm_model *m, const int64_t *h_ids, int n_ids, float *h_logits);

/* The multi-token pass that hm_model_run_kv and hm_model_generate_greedy take for inputs of at
 * least `prefill_min` tokens (reference HfGenerationContext::prefill, src/hf/model.rs:321-336: the
 * whole prompt in one run_kv): projections as GEMMs on the matrix cores, causal attention over
 * cache + chunk, chunks of 512 rows. head_dim 64 or 128; h_logits [n_ids][vocab] or NULL (then the
 * LM head is skipped). bf16 models need widths that are multiples of 32. Block-quantised models
 * (the products of hm_gemm_f32_quant_nk) need multiples of 64, and q|k|v as well as gate|up must each
 * be of one kind, Q8_0 / Q4_0 or K-quants, because the members of a group share an activation
 * matrix; other models keep stepping token by token. hm_model_set_prefill_min: 0 = always token by
 * token (default 8). hm_model_set_prefill_pieces (bf16 models): bf16 numbers per f32 activation on the
 * matrix cores, 3 (default, every bit of the f32) or 2 (16 bits, a third less MFMA work; K/V rows
 * then round to a neighbouring bf16 now and then). */
int hm_model_prefill(hm_model *m, const int64_t *h_ids, int n_ids, float *h_logits);
int hm_model_set_prefill_min(hm_model *m, int n_tokens);
int hm_model_set_prefill_pieces(hm_model *m, int pieces);
/* Block-quantised models: HBM the prompt pass may keep for the dequantised projections (three bf16
 * pieces = 6 bytes per weight; default 32 GiB). If all projections fit, and an eighth of the device
 * stays free, each is dequantised on first use and kept; otherwise, or with 0, every chunk
 * dequantises them again into one scratch matrix. No counterpart in the reference (its CPU kernels
 * dequantise in registers). */
int hm_model_set_prefill_weight_cache(hm_model *m, size_t bytes);

/* The greedy loop of generate_streaming_core (src/generate.rs:187-270) with pure argmax:
 * the prompt is consumed as incremental prefill through run_kv, then n_new tokens are
 * produced with the argmax taken on the device and fed straight back, no per-token host
 * round trip. h_tokens_out receives n_new ids. */
int hm_model_generate_greedy(hm_model *m, const int64_t *h_prompt, int n_prompt, int n_new,
                             int32_t *h_tokens_out);

/* The generation loop of generate_streaming_core (src/generate.rs:100-315) with the reference's sampler:
 * the prompt goes through run_kv (the prompt pass for longer prompts), the first token is sampled from
 * the last prompt position, then one decode step + one sample per token, each new token joining
 * generated_ids for the penalties. Stops before max_new_tokens at eos_token_id (not stored; pass -1 for
 * none) or when the KV cache is full. Logits stay in HBM and the pick is made there when
 * 1 <= top_k <= 1024 or temperature <= 0; otherwise each logits row is sampled on the host.
 * h_tokens_out holds max_new_tokens ids; *n_tokens_out receives how many were produced. */
int hm_model_generate(hm_model *m, const int64_t *h_prompt, int n_prompt, int max_new_tokens,
                      const hm_sampling_config *cfg, uint64_t seed, int eos_token_id, int32_t *h_tokens_out,
                      int *n_tokens_out);

/* Number of HIP kernel launches one decode step issues. */
int hm_model_launches_per_step(hm_model *m);

/* Same as hm_model_set_weight for every slot except matrices: a bf16 projection or an LM head
 * arrives [N][K] (one output row after the other, K contiguous) - the layout of HF safetensors
 * ([out, in]) and of GGUF tensors, and the layout kept in HBM, so nothing is transposed. The
 * reference transposes these on the host (transpose_2d, src/hf/weights.rs:225-261). */
int hm_model_set_weight_nk(hm_model *m, int slot, const void *h_data, size_t bytes);
/* Block-quantised models, before hm_model_finalize: the LM head as the raw blocks of the output matrix
 * (Q4_K / Q6_K: [vocab][hidden / 256] x 144 / 210 bytes; Q8_0 / Q4_0: [vocab][hidden / 32] x 34 / 18 bytes),
 * in place of the f32 lm_head.weight slot (which
 * need not be set then). The reference's quantised plan keeps an f32 head over the matrix its loader
 * dequantises (src/gguf.rs:696-700, emit_lm_head_kernel src/hf/emitter.rs:828-862); here the same product
 * is taken with every weight dequantised in registers, so a token reads 125 or 87 MB of head instead of
 * 622 MB at the Qwen3-0.6B width. hidden_size a multiple of the block length and <= 4096.
 * hm_model_load_gguf does this by itself when the file's output matrix (or, for tied models, its
 * embedding) has one of these types. No counterpart call in the reference. */
int hm_model_set_lm_head_blocks(hm_model *m, int dtype, const void *h_blocks, size_t bytes);
/* The configuration a model was created or loaded with. */
int hm_model_config(hm_model *m, hm_transformer_config *out, int *has_qk_norm, int *weight_dtype);

/* ── checkpoint containers (reference src/gguf.rs, src/hf/safetensors.rs, src/hf/config.rs) ──
 * Host-side readers over a memory mapping; none of them needs a GPU. Open functions return NULL
 * and write a message into err (if given). */
typedef struct hm_gguf hm_gguf;
/* GgufFile::load (src/gguf.rs:345-451): GGUF v2/v3 header, metadata, tensor infos. */
hm_gguf *hm_gguf_open(const char *path, char *err, size_t errlen);
void hm_gguf_close(hm_gguf *g);
int hm_gguf_version(const hm_gguf *g);
int hm_gguf_num_tensors(const hm_gguf *g);
size_t hm_gguf_data_offset(const hm_gguf *g); /* start of the aligned tensor data region */
/* dims come outermost first (the file stores them innermost first, src/gguf.rs:416-422);
 * ggml_type is the GGML code (0 F32, 1 F16, 2 Q4_0, 8 Q8_0, 12 Q4_K, 14 Q6_K, 30 BF16, ...). */
int hm_gguf_tensor_info(const hm_gguf *g, int index, char *name_buf, size_t buflen, int *n_dims,
                        uint64_t dims[8], int *ggml_type, uint64_t *offset, size_t *nbytes);
int hm_gguf_find_tensor(const hm_gguf *g, const char *name); /* index, -1 when absent */
const void *hm_gguf_tensor_data(const hm_gguf *g, int index); /* raw bytes in the mapping */
/* GgufFile::load_f32_buffer (src/gguf.rs:727-776): the tensor as f32 in host memory, dequantised
 * when it is F16, BF16, Q8_0, Q4_0, Q4_K or Q6_K. out holds n_elements floats; HM_ERR_INVALID for
 * a wrong count or a type without a conversion (message in err). Host only, no GPU involved. */
int hm_gguf_tensor_f32(const hm_gguf *g, int index, float *out, size_t n_elements, char *err, size_t errlen);
/* GgufValue::as_str / as_u64 / as_f32 (src/gguf.rs:200-233); HM_ERR_INVALID when the key is
 * absent or of another kind. hm_gguf_meta_str returns the string length. */
int hm_gguf_meta_str(const hm_gguf *g, const char *key, char *buf, size_t buflen);
int hm_gguf_meta_u64(const hm_gguf *g, const char *key, uint64_t *out);
int hm_gguf_meta_f32(const hm_gguf *g, const char *key, float *out);
int64_t hm_gguf_meta_array_len(const hm_gguf *g, const char *key); /* -1 when not an array */
/* GgufFile::transformer_config (src/gguf.rs:508-582). */
int hm_gguf_transformer_config(const hm_gguf *g, hm_transformer_config *out, int *has_qk_norm, char *err,
                               size_t errlen);

typedef struct hm_safetensors hm_safetensors;
/* the container part of load_safetensors_impl (src/hf/safetensors.rs:38-99) */
hm_safetensors *hm_safetensors_open(const char *path, char *err, size_t errlen);
void hm_safetensors_close(hm_safetensors *s);
int hm_safetensors_num_tensors(const hm_safetensors *s);
int hm_safetensors_tensor_info(const hm_safetensors *s, int index, char *name_buf, size_t buflen,
                               char dtype_buf[8], int *n_dims, uint64_t dims[8], size_t *nbytes);
const void *hm_safetensors_tensor_data(const hm_safetensors *s, int index);
/* TransformerConfig::load on the text of a config.json, with its defaults (src/hf/config.rs:11-54). */
int hm_config_from_json(const char *json_text, hm_transformer_config *out, char *err, size_t errlen);

/* HfModel::load for a GGUF file (src/gguf.rs:589-708, src/hf/model.rs) and for a directory with
 * config.json + model.safetensors (or model.safetensors.index.json and its shards)
 * (src/hf/model.rs:75-146, src/hf/weights.rs:267-417): parse, convert, upload, finalize.
 * max_seq_len <= 0 picks min(max_position_embeddings, 4096). NULL on failure: hm_last_error(ctx).
 * The projections of a GGUF file must be all float (F32 / F16 / BF16) or all block-quantised, each
 * tensor Q8_0, Q4_0, Q4_K or Q6_K (the Q4_K_M mixes included). */
hm_model *hm_model_load_gguf(hm_ctx *ctx, const char *path, int max_seq_len);
hm_model *hm_model_load_hf_dir(hm_ctx *ctx, const char *dir, int max_seq_len);

/* ── the reference's kernel ABI, literally ─────────────────────────────────
 * The library also exports HM_CIFACE_MAX_KERNELS symbols
 *     void _mlir__mlir_ciface_k0(void **args) ... void _mlir__mlir_ciface_k1023(void **args)
 * with the signature and argument convention of the reference's compiled kernels: args[i]
 * points at a pointer to a rank-N memref descriptor {allocated, aligned, offset, sizes[N],
 * strides[N]} (src/runtime.rs:654-698, :930-1037), inputs first, outputs after; `aligned` holds
 * a device pointer. CompiledGraph::load_from_handle (src/runtime.rs:803-824) resolves them with
 * dlsym exactly as it resolves its own. hm_ciface_bind_transformer tells the library which
 * fused kernel each index is, in emit_transformer_plan's numbering (src/hf/emitter.rs:902-1014):
 * k0 Embed, k(3l+1) QKV(+QK-norm)+RoPE, k(3l+2) Attn, k(3l+3) MLP for layer l, then LMHead;
 * bf16 weights [K,N], f32 K/V views with the cache's strides; a call carries any number of tokens
 * (the reference's prefill feeds whole prompts to the same kernels, src/hf/model.rs:321-336): with more
 * than one query row attention is causal by position (build_causal_mask, src/hf/precompute.rs:134-161;
 * the mask operand itself is not read), the last S rows of the K/V views being the new tokens'.
 * hm_ciface_bind_transformer_quant does the same for emit_transformer_plan_quant's numbering
 * (src/hf/emitter_quant.rs:1170-1440): k0 Embed; for layer l the thirteen kernels k(13l+1) ..
 * k(13l+13) = RMSNorm, QuantMM Q, K, V, PostQKV, AttnBody, QuantMM O, Residual+Norm, QuantMM Gate, Up,
 * SiLU*Up, QuantMM Down, ResAdd; then the LMHead with f32 weights [hidden, vocab]. proj_dtypes: 7
 * HM_DTYPE_* block formats per layer (q k v o gate up down); the weights are the raw GGUF blocks.
 * A failure cannot be returned (the ABI is void): it is recorded for hm_last_error and printed to
 * stderr, every output operand of the failing call is filled with NaN, and the first failure's code stays
 * in a status word until it is cleared: hm_ciface_last_status returns it (HM_OK when every call since the
 * last clear went through) and stores the failing kernel's index in *kernel_index (may be NULL).
 * One binding per process at a time. */
#define HM_CIFACE_MAX_KERNELS 1024
int hm_ciface_bind_transformer(hm_ctx *ctx, const hm_transformer_config *cfg, int has_qk_norm);
int hm_ciface_bind_transformer_quant(hm_ctx *ctx, const hm_transformer_config *cfg, const int *proj_dtypes,
                                     int has_qk_norm);
int hm_ciface_num_kernels(void);
void hm_ciface_unbind(void);
int hm_ciface_last_status(int *kernel_index);
void hm_ciface_clear_status(void);

uint16_t hm_f32_to_bf16_rne(float v);
uint16_t hm_f32_to_f16_rne(float v);

const char *hm_version(void);

/* ── tokenizer (reference src/tokenizer.rs) ───────────────────────────────────
 * The reference's own byte-level BPE over vocab.json + merges.txt (GPT-2 files): Tokenizer::from_files
 * (src/tokenizer.rs:44-82), encode (:119-144), decode (:147-159). Host code, no GPU.
 * hm_tokenizer_open_json stands in for HfTokenizer::from_file (src/hf/tokenizer.rs:10-14), which hands a
 * tokenizer.json to the `tokenizers` crate (0.21.4 in the reference's Cargo.lock): it reads the files of
 * the byte-level BPE family (Qwen2/3, Llama-3: BPE model, Split on their pattern + ByteLevel, added
 * tokens, ByteLevel or TemplateProcessing post-processor) and of the SentencePiece-style BPE family
 * (Llama-2, TinyLlama, Mistral: BPE with unk_token, fuse_unk and byte_fallback, normaliser Prepend U+2581 +
 * Replace " " by U+2581, no pre-tokeniser, decoder Replace / ByteFallback / Fuse / Strip), and refuses
 * everything else with a message.
 * A file that asks for NFC normalisation is accepted and hm_tokenizer_wants_nfc says so: the caller
 * normalises the text, this library does not.
 * hm_tokenizer_open* return NULL and write a message into err. encode / decode return the full
 * count of ids / bytes (negative: an HM_ERR_* code) and write at most `capacity` of them; call again
 * with a larger buffer when the count exceeds it. The decoded text is UTF-8 without a terminator.
 * encode_ex / decode_ex: HfTokenizer::encode (add_special_tokens = 0) and encode_with_special (1)
 * (src/hf/tokenizer.rs:17-23, :41-47: added tokens written in the text are recognised either way, the flag
 * puts the post-processor's template around the ids); decode (skip_special_tokens = 1) and decode_raw (0)
 * (:25-38). hm_tokenizer_token_to_id: id of a vocabulary entry or added token, -1 when there is none.
 * hm_tokenizer_pieces: the end offsets (bytes) of the pieces the pre-tokeniser pattern
 * (src/tokenizer.rs:71-74) cuts the text into. */
typedef struct hm_tokenizer hm_tokenizer;
hm_tokenizer *hm_tokenizer_open(const char *vocab_json_path, const char *merges_txt_path, char *err, size_t errlen);
hm_tokenizer *hm_tokenizer_open_json(const char *tokenizer_json_path, char *err, size_t errlen);
void hm_tokenizer_close(hm_tokenizer *t);
int hm_tokenizer_wants_nfc(const hm_tokenizer *t);
long long hm_tokenizer_token_to_id(const hm_tokenizer *t, const char *token_utf8);
long long hm_tokenizer_encode_ex(const hm_tokenizer *t, const char *text, size_t text_len, int add_special_tokens,
                                 uint32_t *ids_out, size_t capacity);
long long hm_tokenizer_decode_ex(const hm_tokenizer *t, const uint32_t *ids, size_t n_ids, int skip_special_tokens,
                                 char *text_out, size_t capacity);
int hm_tokenizer_vocab_size(const hm_tokenizer *t);
long long hm_tokenizer_encode(const hm_tokenizer *t, const char *text, size_t text_len, uint32_t *ids_out,
                              size_t capacity);
long long hm_tokenizer_decode(const hm_tokenizer *t, const uint32_t *ids, size_t n_ids, char *text_out,
                              size_t capacity);
long long hm_tokenizer_pieces(const char *text, size_t text_len, size_t *ends_out, size_t capacity);

#pragma GCC visibility pop

#ifdef __cplusplus
}
#endif
#endif /* HOMURA_AMD_H */
