"""The reference's sampler (src/generate.rs:698-801) on logits that stay in HBM, against the oracle: the
same token for the same xorshift64 stream. The device sums the exponentials as a tree and uses its own
expf, so a probability can differ from the oracle's in the last bits; draws that the oracle reports within
1e-4 (relative) of a cumulative boundary are not compared."""
import numpy as np
import pytest

import model_fixture as mf
import pyoracle
from pyoracle import OrcSamplingConfig as Cfg
from homura_amd import HomuraError, runtime, synth, synth_model

pytestmark = pytest.mark.gpu
EDGE = 1e-4


def on_edge(margins, cfg, edge=EDGE):
    """margins = (draw vs cumulative boundary, top_p vs cumulative value), both relative. With top_p >= 1 the
    cut can only drop a tail whose mass is a rounding error of the total, which moves the draw by as much:
    covered by the draw margin."""
    return margins[0] < edge or (cfg.top_p < 1.0 and margins[1] < edge)


def say(msg):
    print(f"[sampling] {msg}", flush=True)


def lib_cfg(c):
    return runtime.SamplingConfig(c.temperature, c.top_k, c.top_p, c.min_p, c.repetition_penalty, c.frequency_penalty,
                                  c.presence_penalty)


CONFIGS = {
    "reference defaults": Cfg(),
    "greedy with penalties": Cfg(temperature=0.0, repetition_penalty=1.3, frequency_penalty=0.4, presence_penalty=0.2),
    "top_k 1": Cfg(temperature=1.5, top_k=1, top_p=1.0, repetition_penalty=1.0),
    "top_k 1024, top_p 1": Cfg(temperature=1.2, top_k=1024, top_p=1.0, repetition_penalty=1.0),
    "min_p and penalties": Cfg(temperature=0.6, top_k=300, top_p=0.97, min_p=0.02, repetition_penalty=1.2,
                               frequency_penalty=0.3, presence_penalty=0.1),
}


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("vocab", [151936, 1000, 50])
def test_device_sampler_against_oracle(ctx, name, vocab):
    cfg = CONFIGS[name]
    gen = np.random.default_rng(vocab + len(name))
    compared = skipped = 0
    for trial in range(12):
        logits = (gen.standard_normal(vocab) * 2.5).astype(np.float32)
        if trial % 3 == 0:                       # equal logits: equal probabilities must order by index
            logits[gen.integers(0, vocab, 4)] = np.float32(logits.max())
        generated = gen.integers(0, vocab, size=[0, 5, 40][trial % 3]).tolist()
        if generated:
            generated += generated[:2]           # repeats: the repetition penalty compounds
        d = ctx.to_device(logits)
        seed = 900 + trial
        a, b = pyoracle.Rng(seed), runtime.Rng(seed)
        for _ in range(3):
            want, margins = pyoracle.sample_token(logits, cfg, generated, a, want_margins=True)
            got = ctx.sample_token(d, vocab, lib_cfg(cfg), generated, b)
            assert a.state.value == b.state.value
            if on_edge(margins, cfg):
                skipped += 1
                continue
            assert got == want, (name, vocab, trial)
            compared += 1
        d.free()
    say(f"{name}, vocab {vocab}: {compared} draws identical, {skipped} on a boundary")
    assert compared >= 24


@pytest.mark.parametrize("vocab,top_k", [(5000, 64), (4096, 33), (151936, 7)])
def test_two_launch_sampler_with_ties_and_masked_logits(ctx, vocab, top_k):
    """The front / back pair (top_k <= 64, vocabulary >= 4096) where its selection is hardest: logits on a
    coarse grid, so that the top_k-th value is shared by many tokens spread over the front workgroups (the
    lowest token numbers must win, as in the oracle's stable order), a run of -inf logits, a last block that
    is not full, top_k at the limit, and a plateau of equal maxima wider than the back launch's short list."""
    gen = np.random.default_rng(vocab * 131 + top_k)
    cfg = Cfg(temperature=0.9, top_k=top_k, top_p=0.98, min_p=0.0, repetition_penalty=1.0)
    compared = skipped = 0
    for trial in range(8):
        logits = (np.round(gen.standard_normal(vocab) * 4.0) * 0.5).astype(np.float32)   # steps of 0.5: heavy ties
        logits[gen.integers(0, vocab, vocab // 10)] = -np.inf
        if trial % 2:
            logits[-3:] = logits.max()            # ties at the very end of the partial block
        if trial in (2, 5):
            # a plateau: a third of the vocabulary shares the maximum, so more tokens reach the back launch's
            # floor than its short list holds and the selection walks the full list in token order
            logits[gen.integers(0, vocab, vocab // 3)] = logits.max()
        d = ctx.to_device(logits)
        a, b = pyoracle.Rng(50 + trial), runtime.Rng(50 + trial)
        for _ in range(4):
            want, margins = pyoracle.sample_token(logits, cfg, [], a, want_margins=True)
            got = ctx.sample_token(d, vocab, lib_cfg(cfg), [], b)
            if on_edge(margins, cfg):
                skipped += 1
                continue
            assert got == want, (vocab, top_k, trial)
            compared += 1
        d.free()
    say(f"ties, vocab {vocab}, top_k {top_k}: {compared} draws identical, {skipped} on a boundary")
    assert compared >= 16


def test_device_sampler_reference_cases_and_errors(ctx):
    # sample_token_greedy and min_p_filters_low_prob (src/generate.rs:891-900, :990-1008)
    d = ctx.to_device(np.array([0.0, 1.0, 0.5, 0.2], np.float32))
    assert ctx.sample_token(d, 4, runtime.SamplingConfig(temperature=0.0), [], runtime.Rng(1)) == 1
    d2 = ctx.to_device(np.array([10.0, 0.0, 0.0, 0.0], np.float32))
    cfg = runtime.SamplingConfig(temperature=1.0, min_p=0.5, top_k=4, top_p=1.0, repetition_penalty=1.0)
    rng = runtime.Rng(42)
    assert [ctx.sample_token(d2, 4, cfg, [], rng) for _ in range(10)] == [0] * 10
    # last of equal maxima
    d3 = ctx.to_device(np.array([1.0, 3.0, 3.0, 2.0], np.float32))
    assert ctx.sample_token(d3, 4, runtime.SamplingConfig(temperature=0.0, repetition_penalty=1.0), [], runtime.Rng(1)) == 2
    with pytest.raises(HomuraError, match="top_k"):
        ctx.sample_token(d, 4, runtime.SamplingConfig(top_k=0), [], runtime.Rng(1))
    with pytest.raises(HomuraError, match="top_k"):
        ctx.sample_token(d, 4, runtime.SamplingConfig(top_k=5000), [], runtime.Rng(1))


MODEL_CONFIGS = {
    "reference defaults": Cfg(),
    # min_p removes the long tail, where cumulative boundaries are closer together than the logits agree
    "min_p and penalties": Cfg(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, repetition_penalty=1.2,
                               frequency_penalty=0.3, presence_penalty=0.1),
    "host path: no top_k": Cfg(temperature=0.9, top_k=0, top_p=0.9, min_p=0.6, repetition_penalty=1.15),
}


@pytest.mark.parametrize("name", list(MODEL_CONFIGS))
def test_model_generate_against_oracle_loop(ctx, name):
    """hm_model_generate against the reference's loop written with the oracle's pieces
    (generate_streaming_core, src/generate.rs:100-315): prompt through run_kv, first token from the last
    prompt position, then decode step + sample_token with the growing generated_ids, stop at EOS."""
    cfg = MODEL_CONFIGS[name]
    mcfg = synth_model.TINY
    weights = synth_model.synth_weights(mcfg, 321)
    gm = synth_model.build_model(ctx, mcfg, weights, 160)
    om = mf.build_oracle_model(mcfg, weights, 160)
    prompt = synth.token_ids(12, 20, mcfg.vocab_size)
    agree = 0
    for seed in (1, 2, 3):
        gm.reset_kv_cache()
        om.kv.reset(0)
        rng = pyoracle.Rng(seed)
        om.run_kv(prompt[:-1])
        cur, want, edge_at = int(prompt[-1]), [], None
        for step in range(40):
            logits = om.run_kv([cur])[0]
            tok, margins = pyoracle.sample_token(logits, cfg, want, rng, want_margins=True)
            if edge_at is None and on_edge(margins, cfg, 3 * EDGE):   # GPU logits differ by ~3e-5 of their scale: keep clear of boundaries
                edge_at = step
            want.append(tok)
            cur = tok
        got = gm.generate(prompt, 40, lib_cfg(cfg), seed=seed)
        upto = 40 if edge_at is None else edge_at
        assert list(got[:upto]) == want[:upto], (name, seed, upto)
        assert len(got) == 40 and gm.kv_cache_len() == 19 + 40
        agree += upto
        # EOS: declare the 6th generated token the end-of-sequence id
        if upto > 6 and want[5] not in want[:5]:
            gm.reset_kv_cache()
            got_eos = gm.generate(prompt, 40, lib_cfg(cfg), seed=seed, eos_token_id=want[5])
            assert list(got_eos) == want[:5]
            # the cache ends behind the step that produced the end token, although more steps were enqueued
            assert gm.kv_cache_len() == 19 + 6
    say(f"{name}: {agree} of 120 generated tokens compared, all identical")
    assert agree >= 30
    gm.close()


@pytest.mark.parametrize("model", ["tiny", "whole_step"])
def test_generate_stops_on_device_and_resumes(ctx, model):
    """The device-resident loop enqueues steps in chunks and reads the tokens back once per chunk: an
    end-of-sequence token in the middle of a chunk must cut the output there, take the cache back to the row of
    the step that produced it, and a continuation from that token must land where the uninterrupted run went
    (the rows of the dropped steps are written again). Greedy, and sampled with a fixed seed, against the
    same model's uninterrupted run; the greedy run also against hm_model_generate_greedy."""
    mcfg = synth_model.TINY if model == "tiny" else synth_model.SMALL_WS
    weights = synth_model.synth_weights(mcfg, 99)
    gm = synth_model.build_model(ctx, mcfg, weights, 256)
    prompt = synth.token_ids(5, 11, mcfg.vocab_size)
    greedy = runtime.SamplingConfig(0.0, 0, 1.0, 0.0, 1.0, 0.0, 0.0)
    whole = gm.generate(prompt, 45, greedy)
    assert len(whole) == 45 and gm.kv_cache_len() == 10 + 45
    gm.reset_kv_cache()
    assert list(gm.generate_greedy(prompt, 45)) == list(whole)

    def stop_index(seq):
        """last position that holds an id for the first time, away from the chunk borders when there is one"""
        firsts = [i for i in range(len(seq)) if seq[i] not in seq[:i]]
        inner = [i for i in firsts if 17 <= i <= 29]   # steps behind it in the same chunk of 16 have been enqueued
        return (inner or firsts)[-1]

    notes = []
    # greedy (the step's own pick), greedy with a repetition penalty (the sampler kernel behind every step, and a
    # varied sequence), sampled (draws made up front, one per step): the uninterrupted run is the yardstick
    for name, cfg, seed in (("greedy", greedy, 0),
                            ("penalised greedy", runtime.SamplingConfig(0.0, 0, 1.0, 0.0, 1.5, 0.2, 0.1), 0),
                            ("sampled", runtime.SamplingConfig(0.8, 40, 0.95, 0.0, 1.1, 0.0, 0.0), 7)):
        gm.reset_kv_cache()
        full = gm.generate(prompt, 45, cfg, seed=seed)
        assert len(full) == 45
        j = stop_index(list(full))
        gm.reset_kv_cache()
        cut = gm.generate(prompt, 45, cfg, seed=seed, eos_token_id=int(full[j]))
        assert list(cut) == list(full[:j]) and gm.kv_cache_len() == 10 + j + 1, name
        if name == "greedy" and j < 44:
            rest = gm.generate([int(full[j])], 45 - j - 1, cfg)
            assert list(rest) == list(full[j + 1:])
        notes.append(f"{name}: stop at step {j} ({len(set(full.tolist()))} distinct ids)")
    say(f"{model}: " + "; ".join(notes))
    gm.close()


def test_chat_turn_feeds_only_the_new_tokens(ctx):
    """The incremental prefill of chat mode (docs/chat.md:34-45): after a turn the cache holds the prompt and
    all generated tokens but the last; the next turn feeds the conversation's ids from there on and must land
    where a fresh pass over the whole conversation lands."""
    mcfg = synth_model.TINY
    weights = synth_model.synth_weights(mcfg, 77)
    gm = synth_model.build_model(ctx, mcfg, weights, 256)
    greedy = runtime.SamplingConfig(0.0, 0, 1.0, 0.0, 1.0, 0.0, 0.0)
    turn1 = synth.token_ids(31, 37, mcfg.vocab_size)
    answer1 = gm.generate(turn1, 9, greedy)
    in_cache = gm.kv_cache_len()
    assert len(answer1) == 9 and in_cache == len(turn1) + len(answer1) - 1
    user2 = synth.token_ids(32, 14, mcfg.vocab_size)
    whole = np.concatenate([turn1, answer1.astype(np.int64), user2])
    step = gm.run_kv(whole[in_cache:])[-1]
    assert gm.kv_cache_len() == len(whole)
    gm.reset_kv_cache()
    fresh = gm.run_kv(whole)[-1]
    assert mf.rel_err(step, fresh) < 1e-2
    top2 = np.sort(fresh)[-2:]
    if top2[1] - top2[0] > 4 * np.abs(step - fresh).max():  # the greedy pick is compared when it is not a near tie
        assert int(np.argmax(step)) == int(np.argmax(fresh))
    say(f"chat turn: {len(whole) - in_cache} new ids on {in_cache} cached, max logit difference "
        f"{np.abs(step - fresh).max():.2e} (scale {np.abs(fresh).max():.2f})")
    gm.close()
