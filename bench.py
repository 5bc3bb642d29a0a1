#!/usr/bin/env python3
"""Decode benchmark: tokens/s of batch-1 greedy decode on the Qwen3-0.6B-shaped model
(BASELINE configuration 2: 28 layers, hidden 1024, 16/8 heads, head_dim 128, SwiGLU 3072,
vocab 151936, tied bf16 LM head; KV cache pre-filled to 1024 rows; synthetic seeded weights).

A "step" is one decode token: embed -> 28 x (QKV+QK-norm+RoPE+append, attention+O, MLP) -> LM head
-> greedy pick, all on the GPU, replayed from one HIP graph, the pick fed back on the device.

    python bench.py --gpus 1 --steps 64 --warmup 8

Prints one JSON line. `roofline` describes the device kernel with the largest share of a step
(its per-layer launches are timed back to back with HIP events on the launch stream);
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
    ap.add_argument("--no-graph", action="store_true", help="launch kernel by kernel instead of graph replay")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=96, help="tokens of the CPU-baseline sample")
    ap.add_argument("--kernel-rounds", type=int, default=20)
    ap.add_argument("--kernel-reps", type=int, default=10, help="graph replays per stand-alone kernel measurement")
    ap.add_argument("--no-kernel-configs", action="store_true",
                    help="skip the stand-alone kernel measurements (BASELINE configurations 1, 3, 4, 5)")
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
        dom = max(kernels, key=lambda k: k["step_share_us"])
        roofline = {
            "bound": "hbm", "kernel": dom["kernel"], "achieved": dom["GBps"], "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(dom["GBps"] / HBM_PEAK_GBS, 4),
            "avg_launch_us": dom["avg_us"], "bytes_per_launch": dom["bytes_per_launch"],
            "traffic": None,
            "whole_step": {"bytes_per_token": int(bytes_tok), "achieved": round(step_gbs, 1),
                           "frac": round(step_gbs / HBM_PEAK_GBS, 4)},
        }
        launches = model.launches_per_step()
        device = ctx.device_name()
        model.close()
        kernel_configs = None
        if not args.no_kernel_configs:
            from homura_amd import kernel_bench
            kernel_bench.REPS = args.kernel_reps
            kernel_configs = kernel_bench.run_all(ctx)

    cpu_baseline = None
    if not args.no_cpu_baseline:
        sys.path.insert(0, str(ROOT / "tests"))
        import model_fixture as mf  # the CPU oracle: checker / baseline only
        import pyoracle
        om = mf.build_oracle_model(cfg, weights, 2048)
        mf.oracle_init_kv(om, kv)
        om.generate_greedy(prompt[:1], 4)  # warm-up
        t0 = time.perf_counter()
        om.generate_greedy(prompt[1:2], args.cpu_tokens)
        cpu_s = time.perf_counter() - t0
        cpu_baseline = {
            "value": round(args.cpu_tokens / cpu_s, 2), "unit": "tok/s",
            "cores": pyoracle.num_threads(), "kind": "port",
            "sample": f"{args.cpu_tokens} greedy tokens of the same model from the same 1024-row cache "
                      f"(C oracle, OpenMP, f32 KV values rounded to bf16)",
        }

    out = {
        "metric": "decode tok/s Qwen3-0.6B-shape bf16 bs=1",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 weights / f32 accumulate", "data": "synthetic",
        "config": {"workload": "Qwen3-0.6B-shape decode: 28 layers, hidden 1024, 16q/8kv heads x 128, "
                               "SwiGLU 3072, vocab 151936 tied head, KV cache 1024+ rows, batch 1, greedy",
                   "kv_rows_start": pos0, "graph_replay": not args.no_graph,
                   "kernel_launches_per_step": launches},
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
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
