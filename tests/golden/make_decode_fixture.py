"""Writes tests/golden/qwen3_0p6b_decode.json: the CPU oracle's greedy tokens (and top-1/top-2
logit margins) for the Qwen3-0.6B-shape decode configuration with seeded synthetic weights.

Run from the repository root:  python tests/golden/make_decode_fixture.py
Needs ~4 GB of host memory and about a minute of CPU; no GPU and no reference checkout.
"""
import json
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

from homura_amd import synth, synth_model  # noqa: E402
import model_fixture  # noqa: E402

PREFILL, N_PROMPT, N_NEW, MAX_SEQ = 1024, 32, 64, 1152


def main():
    cfg = synth_model.QWEN3_0P6B
    seed = synth.SEED_CFG2
    t0 = time.time()
    weights = synth_model.synth_weights(cfg, seed)
    kv = synth_model.synth_kv(cfg, seed + 0x100, PREFILL)
    prompt = synth.token_ids(seed + 0x200, N_PROMPT, cfg.vocab_size)
    print(f"synthesised in {time.time() - t0:.1f}s", flush=True)
    om = model_fixture.build_oracle_model(cfg, weights, MAX_SEQ)
    model_fixture.oracle_init_kv(om, kv)
    t0 = time.time()
    toks, margins = om.generate_greedy(prompt, N_NEW)
    dt = time.time() - t0
    print(f"oracle: {N_PROMPT + N_NEW - 1} steps in {dt:.1f}s; min margin {margins.min():.4e}", flush=True)
    out = {
        "config": "Qwen3-0.6B shape, synthetic weights",
        "seed": seed, "prefill_len": PREFILL, "n_prompt": N_PROMPT, "n_new": N_NEW,
        "max_seq_len": MAX_SEQ,
        "prompt": [int(t) for t in prompt],
        "tokens": [int(t) for t in toks],
        "margins": [float(m) for m in margins],
        "min_margin": float(margins.min()),
        "weights_checksum": int(sum(int(np.asarray(a).view(np.uint8).astype(np.uint64).sum()) for _, a in weights[:20]) % (1 << 61)),
    }
    (Path(__file__).parent / "qwen3_0p6b_decode.json").write_text(json.dumps(out, indent=1))
    print("wrote qwen3_0p6b_decode.json")


if __name__ == "__main__":
    main()
