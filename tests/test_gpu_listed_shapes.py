"""The widths of the other models the reference lists with decode figures (Qwen2.5-0.5B, TinyLlama-1.1B,
Qwen2.5-1.5B, SmolLM2-1.7B; reference README "Performance", src/hf/config.rs:79-123), two layers deep and with
a small vocabulary, against the CPU oracle: decode steps from a cache (one launch per projection: the
cut-row GEMVs, rows of 4864 .. 8960, GQA groups of 1 .. 8, head_dim 64 and 128) and a prompt consumed in one
pass. Decode logits within 1e-2 max relative error, |gpu - ref| / max(|ref|, 1e-2 * max|ref|), prompt-pass logits
within 2e-3 of the logit scale; K-quant mixes
quantise activations to Q8_K integers, which now and then round differently on the two sides, and are held
to the quantisation noise instead (some positions within 1e-3, none off by more than 5 % of the logit scale)."""
import dataclasses

import numpy as np
import pytest

import model_fixture as mf
from homura_amd import synth, synth_model
from homura_amd.runtime import DTYPE_BF16, DTYPE_Q4_0, DTYPE_Q8_0

pytestmark = pytest.mark.gpu

FORMATS = {"bf16": DTYPE_BF16, "q8_0": DTYPE_Q8_0, "q4_0": DTYPE_Q4_0, "q4_k_m": DTYPE_Q8_0}


def say(msg):
    print(msg, flush=True)


@pytest.mark.parametrize("shape,fmt", [("qwen2.5-0.5b", "bf16"), ("qwen2.5-0.5b", "q8_0"),
                                       ("tinyllama-1.1b", "bf16"), ("tinyllama-1.1b", "q4_0"), ("tinyllama-1.1b", "q4_k_m"),
                                       ("qwen2.5-1.5b", "bf16"), ("qwen2.5-1.5b", "q8_0"), ("qwen2.5-1.5b", "q4_0"),
                                       ("qwen2.5-1.5b", "q4_k_m"),
                                       ("smollm2-1.7b", "bf16"), ("smollm2-1.7b", "q8_0"), ("smollm2-1.7b", "q4_k_m")])
def test_listed_shape_against_oracle(ctx, shape, fmt):
    cfg = synth_model.listed_shape(shape, layers=2, vocab=1500)
    if fmt != "bf16":
        cfg = dataclasses.replace(cfg, tie_word_embeddings=False)   # the quantised plan keeps an f32 LM head
    wdt = FORMATS[fmt]
    mix = synth_model.q4_k_m_mix(cfg) if fmt == "q4_k_m" else None
    say(f"{shape} {fmt}: synthesising weights")
    weights = synth_model.synth_weights(cfg, 4242, wdt, has_qk_norm=False, proj_dtypes=mix)
    gm = synth_model.build_model(ctx, cfg, weights, 160, wdt, has_qk_norm=False, proj_dtypes=mix)
    om = mf.build_oracle_model(cfg, weights, 160, wdt, has_qk_norm=False, proj_dtypes=mix)
    assert not gm.whole_step()          # no whole-step instance for these widths
    kv = synth_model.synth_kv(cfg, 17, 70)
    ids = synth.token_ids(18, 30, cfg.vocab_size)

    def check(got, want, what, prompt=False):
        errs = np.array([mf.rel_err(got[i], want[i]) for i in range(len(want))])
        scale = np.array([np.abs(got[i] - want[i]).max() / np.abs(want[i]).max() for i in range(len(want))])
        say(f"{shape} {fmt} {what}: rel err max {errs.max():.2e} median {np.median(errs):.2e}, of the logit scale {scale.max():.2e}")
        if fmt == "q4_k_m":
            assert np.sum(errs < (1e-2 if prompt else 1e-3)) >= min(2, len(errs) - 1) and scale.max() < 5e-2, what
        elif prompt:
            # the prompt pass rounds K, V and the attention weights to bf16 for the matrix cores: held, like the
            # prompt-pass tests of the served shape, to 2e-3 of the logit scale
            assert scale.max() < 2e-3, what
        else:
            assert errs.max() < 1e-2, what

    # decode: five steps from a 70-row cache
    gm.set_prefill_min(0)
    gm.init_kv_cache(kv, 70)
    mf.oracle_init_kv(om, kv)
    got = gm.run_kv(ids[:5])
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(5)])
    check(got, want, "decode steps")
    assert gm.kv_cache_len() == 75
    # the same steps replayed from a recorded graph
    gm.set_graph(True)
    gm.init_kv_cache(kv, 70)
    again = gm.run_kv(ids[:5])
    assert np.array_equal(again, got)
    gm.set_graph(False)
    # a 30-token prompt behind the cache in one pass, then two decode steps on top of it
    gm.set_prefill_min(16)
    gm.init_kv_cache(kv, 70)
    mf.oracle_init_kv(om, kv)
    got = gm.run_kv(ids)
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(30)])
    check(got[-6:], want[-6:], "prompt pass", prompt=True)
    got2 = gm.run_kv(ids[:2])
    want2 = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(2)])
    check(got2, want2, "steps behind the prompt", prompt=True)
    gm.close()


@pytest.mark.parametrize("shape,fmt", [("qwen2.5-0.5b", "bf16"), ("tinyllama-1.1b", "bf16"), ("qwen2.5-1.5b", "bf16"),
                                       ("smollm2-1.7b", "bf16"), ("qwen2.5-1.5b", "q8_0"), ("tinyllama-1.1b", "q4_0")])
def test_listed_shape_on_longer_caches(ctx, shape, fmt):
    """One launch per projection on caches of thousands of rows: the attention grid of the recorded step covers
    the live rows rounded up to a power of two (2048 at least) and is recorded anew when they outgrow it; beyond
    2048 rows a split takes 128 rows instead of 64 and the fold of the splits' partial results is shared out
    over groups of threads. Decode steps across both borders (2048, 4096 live rows), eager and replayed from a
    graph, against the oracle."""
    cfg = dataclasses.replace(synth_model.listed_shape(shape, layers=2, vocab=1500), max_position_embeddings=16384)
    if fmt != "bf16":
        cfg = dataclasses.replace(cfg, tie_word_embeddings=False)   # the quantised plan keeps an f32 LM head
    wdt = FORMATS[fmt]
    weights = synth_model.synth_weights(cfg, 4343, wdt, has_qk_norm=False)
    L = 9000
    gm = synth_model.build_model(ctx, cfg, weights, L, wdt, has_qk_norm=False)
    om = mf.build_oracle_model(cfg, weights, L, wdt, has_qk_norm=False)
    assert not gm.whole_step()
    gm.set_prefill_min(0)
    ids = synth.token_ids(19, 12, cfg.vocab_size)
    for rows in (2040, 4090, 8900):
        kv = synth_model.synth_kv(cfg, 20 + rows, rows)
        results = []
        for graph in (False, True):
            gm.set_graph(graph)
            gm.init_kv_cache(kv, rows)
            results.append(gm.run_kv(ids))
            assert gm.kv_cache_len() == rows + len(ids)
        mf.oracle_init_kv(om, kv)
        want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(len(ids))])
        errs = [mf.rel_err(results[0][i], want[i]) for i in range(len(ids))]
        scale = max(np.abs(results[0][i] - want[i]).max() / np.abs(want[i]).max() for i in range(len(ids)))
        say(f"{shape} {fmt} from {rows} rows: rel err max {max(errs):.2e}, of the logit scale {scale:.2e}")
        # The Q4_0 TinyLlama of this test sits at 1e-4 of the logit scale on long caches (1e-6 at 70 rows, and
        # 3e-6 for the others here), whichever Q4_0 kernels multiply (planes, cut rows, raw blocks) and however the
        # attention grid is cut: its scores are large, and a softmax over thousands of rows turns their rounding
        # into output error. A wrong split, span or fold gives errors of order 1.
        assert max(errs) < (1e-2 if fmt == "bf16" else 3e-2) and scale < 1e-3
        assert np.array_equal(results[0], results[1])
    gm.set_graph(False)
    gm.close()
