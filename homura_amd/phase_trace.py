"""Phase trace of the whole-step decode launch at the Qwen3-0.6B shape (1024 cached rows).

`python -m homura_amd.phase_trace [--weights bf16|q8_0|q4_0|q4_k_m] [--out FILE.md] [--dump FILE.npy]` runs a few decode steps with
`hm_model_whole_step_trace` recording, and prints, as Markdown, what a layer spends between each pair of
the kernel's 11 per-layer marks (both barriers of the Q|K|V, attention, O, gate|up and down phases, and the end
of the fold): mean and spread over workgroups and over layers 1..L-2 (the first and last layer carry the
start and the LM head's prefetch).
"""
from __future__ import annotations

import argparse

import numpy as np

import dataclasses

from . import synth, synth_model
from .runtime import DTYPE_Q4_0, DTYPE_Q8_0, Context

# what lies between mark i and mark i + 1 (the last entry: from mark 10 to mark 0 of the next layer)
INTERVALS = [
    ("Q|K|V rows (between the phase's barriers)", "compute"),
    ("rows published, raw q rows arrive, QK-norm + RoPE, cache append", "exchange (die)"),
    ("attention over the workgroup's cache split", "compute"),
    ("merge of four wavefronts, publish, fold over the splits", "exchange (die) + fold"),
    ("folded attention arrives", "exchange (die)"),
    ("O rows of the K slice", "compute"),
    ("partial O rows summed by the relays, hidden staged", "exchange (memory + die)"),
    ("gate|up rows, SiLU*up", "compute"),
    ("SiLU*up of the group arrives", "exchange (die)"),
    ("down rows of the K slice", "compute"),
    ("partial down rows summed by the relays, hidden staged (next layer)", "exchange (memory + die)"),
]


def collect(steps: int = 4, weights: str = "bf16"):
    """One launch's marks in microseconds: [workgroup][layer][11], its total, and whether it ran die-local."""
    with Context(0) as ctx:
        if weights == "bf16":
            cfg = synth_model.QWEN3_0P6B
            gm = synth_model.build_model(ctx, cfg, synth_model.synth_weights(cfg, 0xC0FFEE02), 1200)
        else:  # block-quantised projections, untied f32 LM head (a launch of its own behind the layers)
            cfg = dataclasses.replace(synth_model.QWEN3_0P6B, tie_word_embeddings=False)
            mix = synth_model.q4_k_m_mix(cfg) if weights == "q4_k_m" else None
            wdt = DTYPE_Q4_0 if weights == "q4_0" else DTYPE_Q8_0
            qw = synth_model.synth_weights(cfg, 7, wdt, has_qk_norm=True, proj_dtypes=mix)
            gm = synth_model.build_model(ctx, cfg, qw, 1200, wdt, has_qk_norm=True, proj_dtypes=mix)
        gm.init_kv_cache(synth_model.synth_kv(cfg, 11, 1024), 1024)
        ids = synth.token_ids(8, 4, cfg.vocab_size)
        gm.generate_greedy(ids, 8)
        gm.whole_step_trace()  # switches recording on
        gm.generate_greedy(ids[:1], steps)
        L = cfg.num_hidden_layers
        per_wg = L * 11 + 2
        t = gm.whole_step_trace(True).astype(np.int64).reshape(256, per_wg)
        gm.whole_step_status()
        gm.close()
    marks = t[:, :L * 11].reshape(256, L, 11) / 100.0
    total = (t[:, -2].max() - t[:, 0].min()) / 100.0
    return marks, total, bool(t[:, -1].min())


def summary(marks: np.ndarray, total: float, die_local: bool, weights: str = "bf16") -> str:
    L = marks.shape[1]
    names = INTERVALS
    # interval i of layer l, per workgroup: mark i+1 - mark i (the last one reaches into the next layer)
    nxt = np.concatenate([marks[:, :, 1:], np.concatenate([marks[:, 1:, :1], marks[:, -1:, :1]], axis=1)], axis=2)
    d = (nxt - marks)[:, 1:L - 1, :]                 # [wg][layer][11]
    per_layer = marks[:, 2:L, 0].mean(axis=0) - marks[:, 1:L - 1, 0].mean(axis=0)
    out = []
    out.append(f"decode_fused_kernel, Qwen3-0.6B shape, {weights} projections, 1024 cached rows; die-local exchanges: {die_local}")
    out.append(f"launch, first mark to last: {total:.1f} us; one layer (layers 1..{L - 2}): mean {per_layer.mean():.2f} us, "
               f"min {per_layer.min():.2f}, max {per_layer.max():.2f}")
    out.append("")
    out.append("| # | between mark i and i+1 | kind | mean us | std over workgroups | std over layers | slowest workgroup (mean) |")
    out.append("|---|---|---|---|---|---|---|")
    kinds: dict[str, float] = {}
    for i, (what, kind) in enumerate(names):
        x = d[:, :, i]
        out.append(f"| {i} | {what} | {kind} | {x.mean():.2f} | {x.mean(axis=1).std():.3f} | {x.mean(axis=0).std():.3f} | {x.mean(axis=1).max():.2f} |")
        kinds[kind.split(" ")[0]] = kinds.get(kind.split(" ")[0], 0.0) + float(x.mean())
    out.append("")
    out.append("per layer: " + ", ".join(f"{k} {v:.2f} us" for k, v in kinds.items()))
    spread = (marks.max(axis=0) - marks.min(axis=0))[1:L - 1]
    out.append("spread of one mark over the workgroups (latest - earliest, mean over layers): " +
               " ".join(f"{spread[:, i].mean():.2f}" for i in range(11)))
    return "\n".join(out)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out")
    ap.add_argument("--dump")
    ap.add_argument("--steps", type=int, default=4)
    ap.add_argument("--weights", choices=["bf16", "q8_0", "q4_0", "q4_k_m"], default="bf16")
    args = ap.parse_args()
    marks, total, die_local = collect(args.steps, args.weights)
    text = summary(marks, total, die_local, args.weights)
    print(text, flush=True)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text + "\n")
    if args.dump:
        np.save(args.dump, marks)


if __name__ == "__main__":
    main()
