#!/usr/bin/env python3
"""Decode benchmark: tokens/s of batch-1 greedy decode on the Qwen3-0.6B-shaped model
(benchmark configuration 2: 28 layers, hidden 1024, 16/8 heads, head_dim 128, SwiGLU 3072,
vocab 151936, tied bf16 LM head; KV cache pre-filled to 1024 rows; synthetic seeded weights).

A "step" is one decode token: embed -> 28 x (QKV+QK-norm+RoPE+append, attention+O, MLP) -> LM head
-> greedy pick, all on the GPU, the pick fed back on the device. A step of many launches is replayed from one
HIP graph; the whole-step kernel makes a step one launch, and the library then launches it directly.

    python bench.py --gpus 1 --steps 64 --warmup 8

Prints one JSON line. `roofline` describes the device kernel with the largest share of a step
(timed with HIP events on the launch stream; `traffic` comes from the committed rocprofv3 --pmc table
under profiles/, flagged `traffic_stale` when the kernel sources have changed since);
`cpu_baseline` is the CPU oracle (a port of the reference's CPU kernels) timed on this host.
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
PREFILL = 1024

# Kernels that share one device function; the roofline line describes the family with the
# largest share of a step, averaged over its launches.
KERNEL_FAMILY = {
    "gemv_bf16[qkv]": "gemv_bf16_nk_oneshot_kernel",
    "gemv_bf16[o]": "gemv_bf16_nk_oneshot_kernel",
    "gemv_bf16[gate_up+silu]": "gemv_bf16_nk_oneshot_kernel",
    "gemv_bf16[down+residual]": "gemv_bf16_nk_oneshot_kernel",
    "gemv_bf16[lm_head+argmax]": "gemv_bf16_nk_kernel",
    "qknorm_rope_append+gqa_attn": "gqa_decode_attn_kernel",
    "gqa_attn_fold": "gqa_decode_fold_kernel",
}

TRAFFIC_TABLE = ROOT / "profiles" / "hbm_traffic_decode_and_kernel_cases_pmc.md"


def kernel_sources_hash() -> str:
    """sha256/16 over the kernel sources (names and contents), the stamp the traffic table carries."""
    import hashlib
    h = hashlib.sha256()
    csrc = ROOT / "homura_amd" / "csrc"
    for f in sorted(list(csrc.glob("*.hip")) + list(csrc.glob("*.h")), key=lambda p: str(p)):
        h.update(f.name.encode())
        h.update(f.read_bytes())
    return h.hexdigest()[:16]


def measured_traffic():
    """HBM bytes per launch by bench.py kernel label, from the committed rocprofv3 --pmc summary
    (FETCH_SIZE and WRITE_SIZE scaled by a copy kernel of known size; the counter runs are separate from
    this program). Returns (table, stale): stale when the kernel sources changed since the table was made."""
    table, stamp = {}, None
    if not TRAFFIC_TABLE.exists():
        return table, True
    for line in TRAFFIC_TABLE.read_text().splitlines():
        if line.startswith("kernel sources sha256/16:"):
            stamp = line.split(":", 1)[1].strip()
        cells = [c.strip() for c in line.split("|")]
        if len(cells) > 9 and cells[2].startswith("`") and cells[8].isdigit():
            table[cells[2].strip("`")] = int(cells[8])
    return table, stamp != kernel_sources_hash()


def algorithmic_bytes_per_token(cfg, kv_rows: float) -> float:
    """Weights streamed once + KV rows read + the logits written (bytes)."""
    hd = cfg.get_head_dim()
    qd, kvd = cfg.num_attention_heads * hd, cfg.kv_heads() * hd
    per_layer = cfg.hidden_size * (qd + 2 * kvd) + qd * cfg.hidden_size + 3 * cfg.hidden_size * cfg.intermediate_size
    weights = 2.0 * (cfg.num_hidden_layers * per_layer + cfg.hidden_size * cfg.vocab_size)
    kv = cfg.num_hidden_layers * 2.0 * cfg.kv_heads() * kv_rows * hd * 2
    return weights + kv + cfg.vocab_size * 4.0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--no-graph", action="store_true",
                    help="launch kernel by kernel instead of graph replay (decode steps and stand-alone kernels)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=96, help="tokens of the CPU-baseline sample")
    ap.add_argument("--kernel-rounds", type=int, default=20)
    ap.add_argument("--kernel-reps", type=int, default=10, help="graph replays per stand-alone kernel measurement")
    ap.add_argument("--kernel-max-launches", type=int, default=0,
                    help="cap on kernel launches per stand-alone measurement graph (0 = the whole weight ring)")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prompt-pass measurement")
    ap.add_argument("--no-quantised", action="store_true", help="skip the decode measurements with quantised projections")
    ap.add_argument("--no-other-shapes", action="store_true", help="skip the decode measurements at the other listed models' shapes")
    ap.add_argument("--no-long-cache", action="store_true", help="skip the decode measurements on caches of 4000 to 32000 rows")
    ap.add_argument("--no-kernel-configs", action="store_true",
                    help="skip the stand-alone kernel measurements (benchmark configurations 1, 3, 4, 5)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); "
              "the decode path is not sharded", file=sys.stderr)
        return 2
    if args.steps < 1 or args.warmup < 0 or PREFILL + args.steps + args.warmup + 2 > 2048:
        print("bench.py: need steps >= 1 and prefill(1024) + warmup + steps <= 2046", file=sys.stderr)
        return 2

    import homura_amd
    from homura_amd import synth, synth_model

    cfg = synth_model.QWEN3_0P6B
    seed = synth.SEED_CFG2
    t_setup = time.perf_counter()
    weights = synth_model.synth_weights(cfg, seed)
    kv = synth_model.synth_kv(cfg, seed + 0x100, PREFILL)
    prompt = synth.token_ids(seed + 0x200, 32, cfg.vocab_size)

    with homura_amd.Context(0) as ctx:
        model = synth_model.build_model(ctx, cfg, weights, 2048)
        model.init_kv_cache(kv, PREFILL)
        model.set_graph(not args.no_graph)
        # untimed: the first tokens of the same greedy run that the CPU baseline leg makes below, kept to be
        # compared with its tokens (the cache is set up again afterwards)
        gpu_check_tokens = None
        if not args.no_cpu_baseline:
            model.generate_greedy(prompt[:1], 4)  # the baseline leg's warm-up, which moves its cache on
            gpu_check_tokens = [int(t) for t in model.generate_greedy(prompt[1:2], min(16, args.cpu_tokens))]
            model.init_kv_cache(kv, PREFILL)
        setup_s = time.perf_counter() - t_setup

        if args.warmup:
            model.bench_decode(int(prompt[0]), args.warmup)
        pos0 = model.kv_cache_len()
        ctx.sync()
        t0 = time.perf_counter()
        event_ms, _tokens = model.bench_decode(int(prompt[1]), args.steps)
        ctx.sync()
        wall_s = time.perf_counter() - t0
        pos1 = model.kv_cache_len()
        assert pos1 - pos0 == args.steps

        tok_s = args.steps / wall_s
        ms_per_step = wall_s * 1e3 / args.steps
        mean_rows = (pos0 + pos1 + 1) / 2.0
        bytes_tok = algorithmic_bytes_per_token(cfg, mean_rows)
        step_gbs = bytes_tok / (wall_s / args.steps) / 1e9

        # per-kernel timing on the launch stream (HIP events), kernels issued layer after layer
        recs = model.time_kernels(args.kernel_rounds)
        kernels = []
        for r in recs:
            us = r["ms"] * 1e3 / r["launches"]
            per_launch_bytes = r["bytes"] / r["launches"]
            kernels.append({
                "kernel": r["label"],
                "launches_per_step": r["launches"] // args.kernel_rounds,
                "avg_us": round(us, 3),
                "bytes_per_launch": int(per_launch_bytes),
                "GBps": round(per_launch_bytes / (us * 1e-6) / 1e9, 1),
                "step_share_us": round(us * (r["launches"] // args.kernel_rounds), 2),
            })
        PMC_TRAFFIC_BYTES, traffic_stale = measured_traffic()
        fams = {}
        for k in kernels:
            f = fams.setdefault(KERNEL_FAMILY.get(k["kernel"], k["kernel"]),
                                {"us": 0.0, "bytes": 0.0, "launches": 0, "traffic": 0.0, "members": []})
            f["us"] += k["step_share_us"]
            f["bytes"] += k["bytes_per_launch"] * k["launches_per_step"]
            f["launches"] += k["launches_per_step"]
            t = PMC_TRAFFIC_BYTES.get(k["kernel"])
            f["traffic"] = None if (t is None or f["traffic"] is None) else f["traffic"] + t * k["launches_per_step"]
            f["members"].append(k["kernel"])
        dom_name, dom = max(fams.items(), key=lambda kv: kv[1]["us"])
        dom_gbs = dom["bytes"] / (dom["us"] * 1e-6) / 1e9
        roofline = {
            "bound": "hbm", "kernel": dom_name, "launches": dom["members"],
            "achieved": round(dom_gbs, 1), "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(dom_gbs / HBM_PEAK_GBS, 4),
            "avg_launch_us": round(dom["us"] / dom["launches"], 3),
            "bytes_per_launch": int(dom["bytes"] / dom["launches"]),
            "launches_per_step": dom["launches"], "step_share_us": round(dom["us"], 1),
            "traffic": None if dom["traffic"] is None else int(dom["traffic"] / dom["launches"]),
            "traffic_stale": traffic_stale,
            "whole_step": {"bytes_per_token": int(bytes_tok), "achieved": round(step_gbs, 1),
                           "frac": round(step_gbs / HBM_PEAK_GBS, 4)},
        }
        # The reference's own loop shape (HfGenerationContext::decode_step, src/hf/model.rs:340-371):
        # one run_kv per token, the 608 KB logits row copied to the host, argmax on the host.
        # Reported beside `value`, never as it.
        import numpy as np
        host_steps = min(16, 2044 - model.kv_cache_len())
        tok = int(prompt[2])
        for _ in range(2):  # untimed: the first call after the per-kernel timing above sets the step up again
            row = model.run_kv([tok], want_logits=True).reshape(-1)
            tok = int(len(row) - 1 - np.argmax(row[::-1]))
        ctx.sync()
        t0 = time.perf_counter()
        for _ in range(host_steps):
            logits = model.run_kv([tok], want_logits=True)
            row = logits.reshape(-1)
            tok = int(len(row) - 1 - np.argmax(row[::-1]))  # last index among equal maxima
        host_loop_s = time.perf_counter() - t0
        pcie_inclusive = {"value": round(host_steps / host_loop_s, 2), "unit": "tok/s", "steps": host_steps,
                          "what": "run_kv per token with the logits row downloaded and argmax on the host"}
        # Sampled decoding through hm_model_generate (reference generate_streaming_core with its default
        # SamplingConfig, src/generate.rs:646-686): the sampler kernel runs behind every step on the GPU and
        # the host reads tokens back once per 16 steps.
        sampled = None
        room = 2046 - model.kv_cache_len()
        if room >= 72:
            from homura_amd.runtime import SamplingConfig
            scfg = SamplingConfig(0.7, 50, 0.9, 0.0, 1.1, 0.0, 0.0)
            model.generate([tok], 8, scfg, seed=1)
            ctx.sync()
            t0 = time.perf_counter()
            got = model.generate([tok], 64, scfg, seed=2)
            dt = time.perf_counter() - t0
            sampled = {"value": round(len(got) / dt, 2), "unit": "tok/s", "steps": int(len(got)),
                       "what": "hm_model_generate, temperature 0.7, top_k 50, top_p 0.9, repetition penalty 1.1; "
                               "wall clock around the call"}
        # What a step of one launch per projection could reach at best: the per-projection plan's 171 launches
        # as empty kernels in one graph, and the same with a 4-byte dependency from each to the next.
        launch_floor = {"kernels": 171, "unit": "us per replay",
                        "empty": round(ctx.launch_floor(171, False), 1),
                        "chained_4_byte_load": round(ctx.launch_floor(171, True), 1)}
        # The prompt side of the same model: 512 tokens on an empty cache through the prefill pass
        # (projections on the matrix cores), against the same tokens one decode step at a time.
        prefill = None
        if not args.no_prefill:
            ptoks = synth.token_ids(seed + 0x300, 512, cfg.vocab_size)
            prefill = {"tokens": 512, "unit": "tok/s"}
            for pieces in (3, 2):
                model.set_prefill_pieces(pieces)
                model.reset_kv_cache()
                model.prefill(ptoks, want_logits=False)   # warm-up (allocates the chunk's scratch)
                best = None
                for _ in range(5):
                    model.reset_kv_cache()
                    ctx.sync()
                    t0 = time.perf_counter()
                    model.prefill(ptoks, want_logits=False)
                    dt = time.perf_counter() - t0
                    best = dt if best is None or dt < best else best
                prefill[f"bf16x{pieces}"] = {"value": round(512 / best, 1), "ms": round(best * 1e3, 3)}
            model.set_prefill_pieces(3)
            prefill["what"] = ("HfModel.prefill of 512 prompt tokens, empty cache, no LM head; bf16x3 = every f32 "
                               "activation as three bf16 pieces (default, exact), bf16x2 = two pieces")
        launches = model.launches_per_step()
        device = ctx.device_name()
        model.close()
        # The same decode with GGUF-quantised projections (untied f32 LM head, as the reference's quantised
        # plan keeps it): Q8_0, Q4_0 and a Q4_K_M-style mix of Q4_K and Q6_K. Reported beside `value`.
        quantised = None
        if not args.no_quantised:
            import dataclasses
            from homura_amd.runtime import DTYPE_Q4_0, DTYPE_Q8_0
            qcfg = dataclasses.replace(cfg, tie_word_embeddings=False)
            quantised = {"unit": "tok/s", "steps": args.steps,
                         "what": "same shape, cache and step count; raw GGUF blocks dequantised in registers "
                                 "(K-quants: Q8_K activations, integer dots), f32 LM head; "
                                 "*_head: the head as Q8_0 / Q6_K blocks multiplied in f32"}
            kmix = synth_model.q4_k_m_mix(qcfg)
            from homura_amd.runtime import DTYPE_Q6_K, HfModel
            nw = qcfg.vocab_size * qcfg.hidden_size
            for name, wdt, mix, head in (("q8_0", DTYPE_Q8_0, None, None), ("q4_0", DTYPE_Q4_0, None, None),
                                         ("q4_k_m_mix", None, kmix, None),
                                         # as the files come: the output matrix in blocks too, read as it is
                                         ("q8_0_q8_0_head", DTYPE_Q8_0, None, (DTYPE_Q8_0, lambda: synth.q8_0_blocks(seed + 9, nw // 32, 0.01))),
                                         ("q4_k_m_mix_q6_k_head", None, kmix, (DTYPE_Q6_K, lambda: synth.q6_k_blocks(seed + 9, nw // 256)))):
                qw = synth_model.synth_weights(qcfg, seed + 7, wdt if mix is None else DTYPE_Q8_0, has_qk_norm=True,
                                               proj_dtypes=mix)
                if head is not None:
                    qm = HfModel(ctx, qcfg, wdt if mix is None else DTYPE_Q8_0, True, proj_dtypes=mix)
                    for i, (_n, arr) in enumerate(qw[:-1]):
                        qm.set_weight(i, arr)
                    qm.set_lm_head_blocks(head[0], head[1]())
                    qm.finalize(2048)
                else:
                    qm = synth_model.build_model(ctx, qcfg, qw, 2048, wdt if mix is None else DTYPE_Q8_0, has_qk_norm=True,
                                                 proj_dtypes=mix)
                qm.init_kv_cache(kv, PREFILL)
                qm.set_graph(not args.no_graph)
                qm.bench_decode(int(prompt[0]), max(args.warmup, 2))
                q_ms, _ = qm.bench_decode(int(prompt[1]), args.steps)
                quantised[name] = {"value": round(args.steps * 1e3 / q_ms, 1), "ms_per_step": round(q_ms / args.steps, 4),
                                   "kernel_launches_per_step": qm.launches_per_step()}
                if not args.no_prefill:
                    # the prompt pass of the quantised plan: 512 tokens on an empty cache, no LM head
                    ptoks = synth.token_ids(seed + 0x300, 512, cfg.vocab_size)
                    qm.reset_kv_cache()
                    qm.prefill(ptoks, want_logits=False)
                    best = None
                    for _ in range(3):
                        qm.reset_kv_cache()
                        ctx.sync()
                        t0 = time.perf_counter()
                        qm.prefill(ptoks, want_logits=False)
                        dt = time.perf_counter() - t0
                        best = dt if best is None or dt < best else best
                    quantised[name]["prefill_512"] = {"value": round(512 / best, 1), "unit": "tok/s", "ms": round(best * 1e3, 3)}
                qm.close()
                del qw
        # The other models the reference lists with decode figures, at their full depth and vocabulary: no
        # whole-step instance, one launch per projection replayed from a graph. Reported beside `value`.
        other_shapes = None
        if not args.no_other_shapes:
            import dataclasses
            from homura_amd.runtime import DTYPE_Q8_0 as _Q8
            other_shapes = {"unit": "tok/s", "steps": args.steps,
                            "what": "greedy decode from a 1024-row cache, one launch per projection (graph replay); "
                                    "bf16 weights, and a Q4_K_M-style mix of Q4_K / Q6_K with an f32 LM head; "
                                    "reference_cpu_tok_s: the reference's README figure (bf16, Ryzen 9 7900X3D)"}
            for name, ref_tok_s in (("qwen2.5-0.5b", 36), ("tinyllama-1.1b", 20), ("qwen2.5-1.5b", 13), ("smollm2-1.7b", 11)):
                ocfg = synth_model.listed_shape(name)
                entry = {"reference_cpu_tok_s": ref_tok_s}
                for fmt in ("bf16", "q4_k_m_mix"):
                    if fmt != "bf16" and ocfg.hidden_size % 256 != 0:
                        continue   # K-quant blocks are 256 wide
                    fcfg = ocfg if fmt == "bf16" else dataclasses.replace(ocfg, tie_word_embeddings=False)
                    mix = None if fmt == "bf16" else synth_model.q4_k_m_mix(fcfg)
                    wdt = 1 if fmt == "bf16" else _Q8
                    ow = synth_model.synth_weights(fcfg, seed + 21, wdt, has_qk_norm=False, proj_dtypes=mix)
                    omdl = synth_model.build_model(ctx, fcfg, ow, 2048, wdt, has_qk_norm=False, proj_dtypes=mix)
                    del ow
                    omdl.init_kv_cache(synth_model.synth_kv(fcfg, seed + 22, PREFILL), PREFILL)
                    omdl.set_graph(not args.no_graph)
                    omdl.bench_decode(int(prompt[0]) % fcfg.vocab_size, max(args.warmup, 2))
                    o_ms, _ = omdl.bench_decode(int(prompt[1]) % fcfg.vocab_size, args.steps)
                    entry[fmt] = {"value": round(args.steps * 1e3 / o_ms, 1), "ms_per_step": round(o_ms / args.steps, 4),
                                  "kernel_launches_per_step": omdl.launches_per_step()}
                    omdl.close()
                other_shapes[name] = entry
        # The benchmarked model on longer caches: the whole-step launch keeps what fits in its wavefronts'
        # registers and streams the further rows through its attention phase (instances for up to 1536, 2048, 3072,
        # 4096 and 32768 live rows). Reported beside `value`.
        long_cache = None
        if not args.no_long_cache:
            import dataclasses
            import numpy as np
            lcfg = dataclasses.replace(cfg, max_position_embeddings=32768)
            lm = synth_model.build_model(ctx, lcfg, weights, 32768)
            lm.set_graph(not args.no_graph)
            long_cache = {"unit": "ms per token", "steps": 32,
                          "what": "the benchmarked model (bf16, greedy, one launch per token) from caches of that many "
                                  "rows: the 1024 synthetic rows repeated; turn_of_32_tokens_ms: 32 tokens behind "
                                  "that cache in one prompt pass"}
            for rows in (4000, 16300, 32000):
                lkv = []
                for a in kv:
                    big = np.empty((1, a.shape[1], rows, a.shape[3]), dtype=np.float32)
                    for r0 in range(0, rows, PREFILL):
                        n = min(PREFILL, rows - r0)
                        big[:, :, r0:r0 + n] = a[:, :, :n]
                    lkv.append(big)
                lm.init_kv_cache(lkv, rows)
                lm.bench_decode(int(prompt[0]), 8)
                l_ms, _ = lm.bench_decode(int(prompt[1]), 32)
                long_cache[str(rows)] = {"ms_per_step": round(l_ms / 32, 4), "value": round(32e3 / l_ms, 1),
                                         "whole_step": bool(lm.whole_step()), "kernel_launches_per_step": lm.launches_per_step()}
                # a chat turn behind that cache: 32 tokens consumed in one prompt pass (wall clock around run_kv)
                turn = synth.token_ids(seed + 0x300, 32, cfg.vocab_size)
                best = None
                for _ in range(3):
                    lm.init_kv_cache(lkv, rows)
                    ctx.sync()
                    t0 = time.perf_counter()
                    lm.run_kv(turn, want_logits=False)
                    ctx.sync()
                    dt = time.perf_counter() - t0
                    best = dt if best is None or dt < best else best
                long_cache[str(rows)]["turn_of_32_tokens_ms"] = round(best * 1e3, 3)
                del lkv
            lm.close()
        kernel_configs = None
        if not args.no_kernel_configs:
            from homura_amd import kernel_bench
            kernel_bench.REPS = args.kernel_reps
            kernel_bench.MAX_LAUNCHES = args.kernel_max_launches
            kernel_bench.USE_GRAPH = not args.no_graph
            kernel_configs = kernel_bench.run_all(ctx)

    cpu_baseline = None
    if not args.no_cpu_baseline:
        sys.path.insert(0, str(ROOT / "tests"))
        import model_fixture as mf  # the CPU oracle: checker / baseline only
        import pyoracle
        pyoracle.use_isa(pyoracle.best_isa())  # the AVX-512 build of the same source where the host has it
        om = mf.build_oracle_model(cfg, weights, 2048)
        mf.oracle_init_kv(om, kv)
        om.generate_greedy(prompt[:1], 4)  # warm-up
        t0 = time.perf_counter()
        cpu_tokens, _margins = om.generate_greedy(prompt[1:2], args.cpu_tokens)
        cpu_s = time.perf_counter() - t0
        n_chk = len(gpu_check_tokens)
        same = 0
        while same < n_chk and int(cpu_tokens[same]) == gpu_check_tokens[same]:
            same += 1
        cpu_baseline = {
            "value": round(args.cpu_tokens / cpu_s, 2), "unit": "tok/s",
            "cores": pyoracle.num_threads(), "kind": "port",
            "sample": f"{args.cpu_tokens} greedy tokens of the same model from the same 1024-row cache "
                      f"(C oracle built for {pyoracle.isa()}, OpenMP, f32 KV values rounded to bf16)",
            "gpu_tokens_identical": f"{same} of the first {n_chk} tokens of that run, taken on the GPU before the timed region",
        }

    out = {
        "metric": "decode tok/s Qwen3-0.6B-shape bf16 bs=1",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 weights / f32 accumulate", "data": "synthetic",
        "config": {"workload": "Qwen3-0.6B-shape decode: 28 layers, hidden 1024, 16q/8kv heads x 128, "
                               "SwiGLU 3072, vocab 151936 tied head, KV cache 1024+ rows, batch 1, greedy",
                   "kv_rows_start": pos0, "graph_replay": (not args.no_graph) and launches > 2,
                   "kernel_launches_per_step": launches},
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "pcie_inclusive": pcie_inclusive,
        "sampled_decode": sampled,
        "launch_floor": launch_floor,
        "prefill": prefill,
        "quantised_decode": quantised,
        "other_shapes": other_shapes,
        "long_cache": long_cache,
        "event_ms_per_step": round(event_ms / args.steps, 4),
        "kernels": kernels,
        "kernel_configs": kernel_configs,
        "device": device,
        "setup_s": round(setup_s, 1),
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
