/* Measurement and test-support entry points of libhomura_amd.so. They are not part of the drop-in
 * boundary (include/homura_amd.h): nothing here has a counterpart in the reference's FFI. */
#ifndef HOMURA_AMD_BENCH_H
#define HOMURA_AMD_BENCH_H

#include "homura_amd.h"

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

/* Timed decode for benchmarking: runs `n_steps` decode steps starting from token `first_id`
 * (greedy feedback on device), returns total milliseconds measured with HIP events on the
 * context stream. */
int hm_model_bench_decode(hm_model *m, int64_t first_id, int n_steps, float *ms_out,
                          int32_t *h_tokens_out);

/* Per-kernel profile of one decode step (HOMURA_PROFILE analogue, reference
 * src/runtime.rs:1849-1873): HIP events around every device launch; one record per device
 * kernel name. Fills up to `cap` records; returns the number written. */
typedef struct {
    char label[32]; /* "gemv_bf16[qkv]", "gqa_decode_attn", "gemv_bf16[lm_head+argmax]", ... */
    float ms;       /* summed over the launches */
    int launches;
    double bytes;   /* algorithmic bytes moved by these launches */
} hm_kernel_profile;
int hm_model_profile_step(hm_model *m, int64_t token_id, hm_kernel_profile *out, int cap);
/* Roofline timing: per device kernel name, all of the step's launches of that kernel (one per
 * layer, different weights each) back to back, `rounds` times, between two HIP events.
 * Disturbs activations and the current cache row: call after the decode. */
int hm_model_time_kernels(hm_model *m, int rounds, hm_kernel_profile *out, int cap);

/* ── deterministic synthetic data (host side, no GPU needed) ─────────────────
 * Counter-based generator shared by tests and benchmarks: sample i of stream `seed` uses
 * outputs 3i..3i+2 of the splitmix64 sequence seeded with `seed`; a normal variate is the
 * centred sum of the twelve 16-bit fields of those outputs (Irwin-Hall, unit variance),
 * computed in integers so that every platform produces the same bits. */
void hm_synth_normal_f32(uint64_t seed, uint64_t first, size_t n, float scale, float *out);
void hm_synth_normal_bf16(uint64_t seed, uint64_t first, size_t n, float scale, uint16_t *out);
void hm_synth_token_ids(uint64_t seed, size_t n, int vocab, int64_t *out);
/* n_blocks Q8_0 blocks: q uniform in [-127,127], d = f16(|N(0,1)| * d_scale) */
void hm_synth_q8_0(uint64_t seed, size_t n_blocks, float d_scale, uint8_t *out);
/* n_blocks Q4_0 blocks: nibbles uniform in [0,15], d = f16(|N(0,1)| * d_scale) */
void hm_synth_q4_0(uint64_t seed, size_t n_blocks, float d_scale, uint8_t *out);

/* Floor of a step made of dependent launches: a HIP graph of `n_kernels` one-wavefront kernels that do
 * nothing (chained = 0) or that each read 4 bytes their predecessor wrote and write 4 bytes (chained = 1),
 * replayed `replays` times between two events; microseconds per replay. */
int hm_bench_launch_floor(hm_ctx *ctx, int n_kernels, int chained, int replays, float *us_per_replay);

/* Test support: writes `word` over the whole LDS of every CU (a grid of workgroups that each take a CU's LDS).
 * LDS keeps its contents from one kernel to the next, and from one process to the next: a kernel that reads
 * LDS it did not write works or fails by what ran before it. Filled with 0xFFFFFFFF (a NaN), any such read
 * that reaches a result shows. Device allocations can be pre-filled the same way with the environment
 * variable HOMURA_ALLOC_FILL=<byte>, read when the first buffer is allocated. */
int hm_test_fill_lds(hm_ctx *ctx, uint32_t word);

/* Phase trace of the latest whole-step decode launch: device-clock ticks (100 MHz) taken by workgroup
 * 0 at 11 points per layer (both workgroup barriers of the Q|K|V, attention, O, gate|up and down
 * phases; the end of the fold follows attention's second barrier) and one at the end of the kernel, then
 * a word that is 1 when the step found its workgroups dealt round-robin to the dies and used die-local
 * exchanges. The first call switches recording on and stores 0 in *n_out; later calls copy
 * layers * 11 + 2 entries of the step that ran last (workgroup 0's), or, when cap has room for 256
 * times as many, one such row per workgroup (256 rows; those of workgroups the grid lacks stay 0). */
int hm_model_whole_step_trace(hm_model *m, unsigned long long *h_out, int cap, int *n_out);

/* Test support for block-quantised models with K-quant projections: keep the f32 activation rows that the
 * prompt pass hands to the Q8_K quantiser (reference emit_quant.rs:422-466) for the next `rows` cache
 * positions (0 = stop, free the buffer), and copy them to the host afterwards. Per layer: [rows][hidden]
 * (input of q|k|v), [rows][heads * head_dim] (o), [rows][hidden] (gate|up), [rows][intermediate] (down);
 * rows of groups whose matrices are not K-quants stay zero. A checker can then quantise the very values
 * the GPU quantised, so that a rounding decision taken differently on the two sides is counted instead of
 * being seen as an error. */
int hm_model_prefill_capture_q8k_inputs(hm_model *m, int rows);
int hm_model_prefill_captured_q8k_inputs(hm_model *m, float *h_out, size_t n_floats);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif
