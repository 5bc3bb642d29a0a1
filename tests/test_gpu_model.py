"""Whole-decode-step parity through the C boundary: the GPU ExecutionPlan against the CPU oracle's
restatement of the reference's step list, on identical seeded weights, KV cache and prompt.
Logits within 1e-2 max relative error, |gpu - ref| / max(|ref|, 1e-2 * max|ref|) (see
model_fixture.rel_err for why the floor is 1% here); greedy tokens identical."""
import json
from pathlib import Path

import numpy as np
import pytest

import model_fixture as mf
from homura_amd import HomuraError, synth, synth_model
from homura_amd.runtime import DTYPE_BF16, HfModel

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).parent / "golden"


def say(msg):
    print(msg, flush=True)


@pytest.fixture(scope="module")
def tiny(ctx):
    cfg = synth_model.TINY
    weights = synth_model.synth_weights(cfg, 4242)
    gm = synth_model.build_model(ctx, cfg, weights, 160)
    om = mf.build_oracle_model(cfg, weights, 160)
    yield cfg, weights, gm, om
    gm.close()


def test_tiny_logits_and_tokens(tiny):
    cfg, _w, gm, om = tiny
    kv = synth_model.synth_kv(cfg, 7, 50)
    gm.init_kv_cache(kv, 50)
    mf.oracle_init_kv(om, kv)
    assert gm.kv_cache_len() == 50
    ids = synth.token_ids(8, 5, cfg.vocab_size)
    # multi-token run_kv = incremental prefill on top of the cache (reference src/hf/model.rs:321-336)
    got = gm.run_kv(ids)
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(5)])
    assert gm.kv_cache_len() == 55 and om.kv.current_len() == 55
    for i in range(5):
        assert mf.rel_err(got[i], want[i]) < 1e-2, f"position {i}"
    want_t, margins = om.generate_greedy(ids, 40)
    got_t = gm.generate_greedy(ids, 40)
    say(f"tiny: min margin {margins.min():.3e}")
    assert np.array_equal(got_t, want_t)
    assert gm.kv_cache_len() == 55 + 5 + 39


def test_tiny_empty_cache_and_reset(tiny):
    cfg, _w, gm, om = tiny
    gm.reset_kv_cache()
    om.kv.reset(0)
    assert gm.kv_cache_len() == 0
    ids = synth.token_ids(9, 3, cfg.vocab_size)
    got = gm.run_kv(ids)       # a prefill from nothing, token by token
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(3)])
    assert mf.rel_err(got, want) < 1e-2
    # same prompt after a reset gives the same bits (no state leaks between sequences)
    gm.reset_kv_cache()
    again = gm.run_kv(ids)
    assert np.array_equal(got, again)


def test_tiny_graph_replay_matches_eager(ctx, tiny):
    cfg, weights, gm, _om = tiny
    kv = synth_model.synth_kv(cfg, 17, 30)
    ids = synth.token_ids(18, 4, cfg.vocab_size)
    gm.init_kv_cache(kv, 30)
    eager_tokens = gm.generate_greedy(ids, 24)
    eager_logits = gm.run_kv(ids[:1])
    gm.set_graph(True)
    try:
        for rep in range(3):  # replays interleaved with eager work and syncs in between
            gm.init_kv_cache(kv, 30)
            assert np.array_equal(gm.generate_greedy(ids, 24), eager_tokens), f"replay round {rep}"
            assert np.array_equal(gm.run_kv(ids[:1]), eager_logits)
    finally:
        gm.set_graph(False)


def test_kv_overflow_and_bad_input(ctx, tiny):
    cfg, weights, gm, _om = tiny
    kv = synth_model.synth_kv(cfg, 7, 158)
    gm.init_kv_cache(kv, 158)
    gm.run_kv([1, 2])
    with pytest.raises(HomuraError) as e:   # the reference panics "KV cache full"
        gm.run_kv([3])
    assert e.value.code == -4 and "KV cache full" in str(e.value)
    assert gm.kv_cache_len() == 160
    gm.reset_kv_cache()
    with pytest.raises(HomuraError):
        gm.run_kv([cfg.vocab_size])          # id outside the vocabulary
    with pytest.raises(HomuraError):
        gm.generate_greedy([1], 200)         # would overflow the cache
    # weights: wrong byte size and missing slot (reference: size-mismatch panic, "missing weight")
    m2 = HfModel(ctx, cfg, DTYPE_BF16, True)
    with pytest.raises(HomuraError):
        m2.set_weight(0, np.zeros(7, np.float32))
    m2.set_weight(0, weights[0][1])
    with pytest.raises(HomuraError) as e2:
        m2.finalize(64)
    assert "missing weight" in str(e2.value)
    m2.close()


def test_weight_slot_listing_matches_reference_order(tiny):
    cfg, weights, gm, _om = tiny
    names = [s[0] for s in gm.weight_slots()]
    assert names == [n for n, _ in weights]
    assert names[0] == "model.embed_tokens.weight" and names[-1] == "lm_head.weight"
    per_layer = ["input_layernorm", "q_proj", "k_proj", "v_proj", "q_norm", "k_norm", "o_proj",
                 "post_attention_layernorm", "gate_proj", "up_proj", "down_proj"]
    assert [n.split(".")[-2] for n in names[1:12]] == per_layer


def test_qwen3_0p6b_decode_token_identical(ctx):
    """benchmark configuration 2: 28-layer Qwen3-0.6B shape, cache pre-filled to 1024 rows,
    32 prompt ids, 64 greedy tokens: GPU tokens == oracle tokens == committed fixture."""
    fx = json.loads((GOLDEN / "qwen3_0p6b_decode.json").read_text())
    cfg = synth_model.QWEN3_0P6B
    say("synthesising weights")
    weights = synth_model.synth_weights(cfg, fx["seed"])
    kv = synth_model.synth_kv(cfg, fx["seed"] + 0x100, fx["prefill_len"])
    prompt = synth.token_ids(fx["seed"] + 0x200, fx["n_prompt"], cfg.vocab_size)
    assert [int(t) for t in prompt] == fx["prompt"]
    say("building GPU model")
    gm = synth_model.build_model(ctx, cfg, weights, fx["max_seq_len"])
    gm.init_kv_cache(kv, fx["prefill_len"])
    om = mf.build_oracle_model(cfg, weights, fx["max_seq_len"])
    mf.oracle_init_kv(om, kv)
    say("first-step logits")
    got_logits = gm.run_kv(prompt[:1])
    want_logits = om.run_kv(prompt[:1])
    err = mf.rel_err(got_logits, want_logits)
    absd = float(np.abs(got_logits - want_logits).max())
    say(f"logits: rel err {err:.3e}, max abs diff {absd:.3e}, min fixture margin {fx['min_margin']:.3e}")
    assert err < 1e-2
    say("greedy decode on both sides")
    gm.set_prefill_min(0)   # the prompt token by token through the batch-1 path, as the fixture defines it
    got = gm.generate_greedy(prompt[1:], fx["n_new"])
    want, margins = om.generate_greedy(prompt[1:], fx["n_new"])
    assert np.array_equal(want, np.array(fx["tokens"], np.int32)), "oracle drifted from its committed fixture"
    assert np.array_equal(got, want), f"first mismatch at {int(np.argmax(got != want))}"
    gm.set_graph(True)
    gm.init_kv_cache(kv, fx["prefill_len"])
    assert np.array_equal(gm.generate_greedy(prompt, fx["n_new"]), want), "graph replay differs"
    say("prompt through the prefill pass (matrix cores), then decode")
    gm.set_prefill_min(8)
    gm.init_kv_cache(kv, fx["prefill_len"])
    assert np.array_equal(gm.generate_greedy(prompt, fx["n_new"]), want), "prefill + decode differs"
    gm.close()


@pytest.mark.parametrize("wdt,name", [(2, "q8_0"), (3, "q4_0")])
def test_quantised_plan_against_oracle(ctx, wdt, name):
    """GGUF-quantised projections (reference emit_transformer_plan_quant): raw blocks uploaded as
    they are, dequantised in registers; f32 LM head. Llama-style config: no QK-norm, untied head."""
    cfg = synth_model.TINY_LLAMA
    weights = synth_model.synth_weights(cfg, 31, wdt, has_qk_norm=False)
    gm = synth_model.build_model(ctx, cfg, weights, 96, wdt, has_qk_norm=False)
    om = mf.build_oracle_model(cfg, weights, 96, wdt, has_qk_norm=False)
    kv = synth_model.synth_kv(cfg, 3, 37)
    gm.init_kv_cache(kv, 37)
    mf.oracle_init_kv(om, kv)
    ids = synth.token_ids(4, 6, cfg.vocab_size)
    got = gm.run_kv(ids)
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(6)])
    for i in range(6):
        assert mf.rel_err(got[i], want[i]) < 1e-2, f"{name} position {i}"
    want_t, margins = om.generate_greedy(ids[:2], 24)
    got_t = gm.generate_greedy(ids[:2], 24)
    say(f"{name}: min margin {margins.min():.3e}")
    assert np.array_equal(got_t, want_t)
    gm.set_graph(True)
    gm.init_kv_cache(kv, 37)
    gm.run_kv(ids)
    assert np.array_equal(gm.generate_greedy(ids[:2], 24), want_t)
    names = [s[0] for s in gm.weight_slots()]
    assert names == [n for n, _ in weights]
    gm.close()


@pytest.mark.parametrize("name", ["q8_0", "q4_0", "q4_k_m_mix"])
def test_qwen3_0p6b_shape_quantised_decode_against_oracle(ctx, name):
    """The quantised decode plans at the shape bench.py times them on (Qwen3-0.6B widths, 28 layers, untied
    f32 LM head, cache pre-filled to 1024 rows): first-step logits and 16 greedy tokens against the oracle.
    Q8_0 / Q4_0 have no step function besides the bf16 cache rounding: tokens identical. The Q4_K_M-style
    mix quantises its activations to Q8_K on both sides independently; tokens are compared while the
    oracle's lead of the best logit exceeds what rounding decisions taken differently move two logits by at
    this width (measured worst row 2e-4 of the logit scale; allowed 1e-3 each)."""
    import dataclasses
    from homura_amd.runtime import DTYPE_Q4_0, DTYPE_Q8_0
    cfg = dataclasses.replace(synth_model.QWEN3_0P6B, tie_word_embeddings=False)
    mix = synth_model.q4_k_m_mix(cfg) if name == "q4_k_m_mix" else None
    wdt = {"q8_0": DTYPE_Q8_0, "q4_0": DTYPE_Q4_0, "q4_k_m_mix": DTYPE_Q8_0}[name]
    say(f"{name}: synthesising weights")
    weights = synth_model.synth_weights(cfg, synth.SEED_CFG2 + 7, wdt, has_qk_norm=True, proj_dtypes=mix)
    kv = synth_model.synth_kv(cfg, synth.SEED_CFG2 + 0x100, 1024)
    gm = synth_model.build_model(ctx, cfg, weights, 1200, wdt, has_qk_norm=True, proj_dtypes=mix)
    om = mf.build_oracle_model(cfg, weights, 1200, wdt, has_qk_norm=True, proj_dtypes=mix)
    gm.init_kv_cache(kv, 1024)
    mf.oracle_init_kv(om, kv)
    gm.set_graph(True)
    gm.set_prefill_min(0)
    ids = synth.token_ids(synth.SEED_CFG2 + 0x200, 3, cfg.vocab_size)
    got = gm.run_kv(ids[:1])
    want = om.run_kv(ids[:1])
    err = mf.rel_err(got, want)
    say(f"{name}: first-step logits rel err {err:.2e}")
    assert err < 1e-2
    want_t, margins = om.generate_greedy(ids[1:], 16)
    got_t = gm.generate_greedy(ids[1:], 16)
    scale = float(np.abs(want).max())
    thr = 2 * 1e-3 * scale if mix is not None else 0.0
    close = np.nonzero(margins < thr)[0]
    n_cmp = int(close[0]) if close.size else len(want_t)
    say(f"{name}: min margin {margins.min():.3e} (logit scale {scale:.3e}), {n_cmp} of 16 tokens compared")
    assert n_cmp >= 8
    assert np.array_equal(got_t[:n_cmp], want_t[:n_cmp])
    gm.close()


@pytest.mark.parametrize("kind", ["q6_k", "q8_0"])
def test_qwen3_0p6b_shape_lm_head_from_blocks_against_oracle(ctx, kind):
    """The configurations bench.py times with the output matrix read from its blocks (re-packed into planes at
    finalize): the Q4_K_M-style mix with a Q6_K head and the Q8_0 plan with a Q8_0 head, at Qwen3-0.6B widths
    with a 1024-row cache. The oracle multiplies the dequantised matrix in its f32 slot: first-step logits,
    and greedy tokens while the oracle's margin exceeds what differently taken Q8_K rounding decisions move
    two logits by (mix only)."""
    import dataclasses
    import pyoracle
    from homura_amd.runtime import DTYPE_Q8_0
    cfg = dataclasses.replace(synth_model.QWEN3_0P6B, tie_word_embeddings=False)
    mix = synth_model.q4_k_m_mix(cfg) if kind == "q6_k" else None
    say(f"head from {kind} blocks: synthesising weights")
    weights = synth_model.synth_weights(cfg, synth.SEED_CFG2 + 9, DTYPE_Q8_0, has_qk_norm=True, proj_dtypes=mix)
    assert weights[-1][0] == "lm_head.weight"
    if kind == "q6_k":
        raw, code = synth.q6_k_blocks(93, cfg.vocab_size * cfg.hidden_size // 256), 6
        dense = pyoracle.dequant_q6_k(raw)
    else:
        raw, code = synth.q8_0_blocks(93, cfg.vocab_size * cfg.hidden_size // 32, 0.01), 2
        dense = pyoracle.dequant_q8_0(raw)
    weights[-1] = ("lm_head.weight", np.ascontiguousarray(dense.reshape(cfg.vocab_size, cfg.hidden_size).T))
    om = mf.build_oracle_model(cfg, weights, 1200, DTYPE_Q8_0, has_qk_norm=True, proj_dtypes=mix)
    gm = HfModel(ctx, cfg, weight_dtype=DTYPE_Q8_0, has_qk_norm=True, proj_dtypes=mix)
    for i, (_name, arr) in enumerate(weights[:-1]):
        gm.set_weight(i, arr)
    gm.set_lm_head_blocks(code, raw)
    gm.finalize(1200)
    kv = synth_model.synth_kv(cfg, synth.SEED_CFG2 + 0x101, 1024)
    gm.init_kv_cache(kv, 1024)
    mf.oracle_init_kv(om, kv)
    gm.set_graph(True)
    gm.set_prefill_min(0)
    ids = synth.token_ids(synth.SEED_CFG2 + 0x201, 3, cfg.vocab_size)
    got, want = gm.run_kv(ids[:1]), om.run_kv(ids[:1])
    err = mf.rel_err(got, want)
    say(f"head from {kind} blocks: first-step logits rel err {err:.2e}")
    assert err < 1e-2
    want_t, margins = om.generate_greedy(ids[1:], 12)
    got_t = gm.generate_greedy(ids[1:], 12)
    scale = float(np.abs(want).max())
    thr = 2 * 1e-3 * scale if mix is not None else 0.0
    close = np.nonzero(margins < thr)[0]
    n_cmp = int(close[0]) if close.size else len(want_t)
    say(f"head from {kind} blocks: min margin {margins.min():.3e} (logit scale {scale:.3e}), {n_cmp} of 12 tokens compared")
    assert n_cmp >= 6
    assert np.array_equal(got_t[:n_cmp], want_t[:n_cmp])
    gm.close()


@pytest.mark.parametrize("wdt,name", [(1, "bf16"), (2, "q8_0")])
def test_qkv_bias_model_against_oracle(ctx, wdt, name):
    """Qwen2-style checkpoint: Q/K/V biases (slots q,[qb],k,[kb],v,[vb] of the reference's
    to_slot_buffers), no QK-norm, GQA group of 7, head_dim 64."""
    cfg = synth_model.TINY_QWEN2
    weights = synth_model.synth_weights(cfg, 77, wdt, has_qk_norm=False)
    assert any(n.endswith("q_proj.bias") for n, _ in weights)
    gm = synth_model.build_model(ctx, cfg, weights, 96, wdt, has_qk_norm=False)
    om = mf.build_oracle_model(cfg, weights, 96, wdt, has_qk_norm=False)
    assert [s[0] for s in gm.weight_slots()] == [n for n, _ in weights]
    kv = synth_model.synth_kv(cfg, 8, 21)
    gm.init_kv_cache(kv, 21)
    mf.oracle_init_kv(om, kv)
    ids = synth.token_ids(6, 5, cfg.vocab_size)
    got = gm.run_kv(ids)
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(5)])
    for i in range(5):
        assert mf.rel_err(got[i], want[i]) < 1e-2, f"{name} position {i}"
    want_t, margins = om.generate_greedy(ids[:2], 24)
    say(f"bias model {name}: min margin {margins.min():.3e}")
    assert np.array_equal(gm.generate_greedy(ids[:2], 24), want_t)
    gm.set_graph(True)
    gm.init_kv_cache(kv, 21)
    gm.run_kv(ids)
    assert np.array_equal(gm.generate_greedy(ids[:2], 24), want_t)
    gm.close()


@pytest.mark.parametrize("which", ["q4_k", "q6_k", "q4_k_m_mix", "q8_0_q6_k_mix"])
def test_kquant_plan_against_oracle(ctx, which):
    """K-quant projections, one type throughout or mixed per matrix as Q4_K_M files are (attn_v and
    ffn_down of some layers in Q6_K): same-type neighbours share a launch, the others get their own,
    and the activation is rounded to Q8_K once per group."""
    cfg = synth_model.TINY_K
    L = cfg.num_hidden_layers
    mix = {"q4_k": [5] * 7 * L, "q6_k": [6] * 7 * L, "q4_k_m_mix": synth_model.q4_k_m_mix(cfg),
           # q alone, k|v stacked, gate and up apart: every way a group can split
           "q8_0_q6_k_mix": [2, 6, 6, 2, 6, 5, 2] + [6, 2, 6, 5, 5, 5, 6] * (L - 1)}[which]
    weights = synth_model.synth_weights(cfg, 57, has_qk_norm=False, proj_dtypes=mix)
    gm = synth_model.build_model(ctx, cfg, weights, 96, has_qk_norm=False, proj_dtypes=mix)
    om = mf.build_oracle_model(cfg, weights, 96, has_qk_norm=False, proj_dtypes=mix)
    assert [s[0] for s in gm.weight_slots()] == [n for n, _ in weights]
    kv = synth_model.synth_kv(cfg, 3, 29)
    gm.init_kv_cache(kv, 29)
    mf.oracle_init_kv(om, kv)
    ids = synth.token_ids(4, 5, cfg.vocab_size)
    got = gm.run_kv(ids)
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(5)])
    # A step through Q8_K activations is a discontinuous function of its input: where an activation lies within
    # f32 summation noise of a rounding boundary the two sides round it to different integers, the layers behind
    # differ in many more, and the logits end up apart by the quantisation noise (1-4 % of their scale) instead
    # of 1e-6. Most positions are not hit; none may be further off than that noise.
    errs = np.array([mf.rel_err(got[i], want[i]) for i in range(5)])
    scale = np.array([np.abs(got[i] - want[i]).max() / np.abs(want[i]).max() for i in range(5)])
    say(f"{which}: rel err " + " ".join(f"{e:.1e}" for e in errs) + f"; of the logit scale at most {scale.max():.1e}")
    assert np.sum(errs < 1e-3) >= 3 and scale.max() < 5e-2, which
    want_t, margins = om.generate_greedy(ids[:2], 24)
    got_t = gm.generate_greedy(ids[:2], 24)
    # tokens are compared while the oracle's margin is clear of that noise
    close = np.nonzero(margins < 5e-3 * float(np.abs(want).max()))[0]   # (a flipped step moved the logits by 8e-4 of it here)
    n_cmp = int(close[0]) if close.size else len(want_t)
    say(f"{which}: min margin {margins.min():.3e}, {n_cmp} of {len(want_t)} tokens compared")
    assert np.array_equal(got_t[:n_cmp], want_t[:n_cmp])
    gm.set_graph(True)
    gm.init_kv_cache(kv, 29)
    gm.run_kv(ids)
    assert np.array_equal(gm.generate_greedy(ids[:2], 24), got_t)   # the recorded graph replays the eager steps
    gm.close()


def test_mixed_model_rejects_bad_dtype_lists(ctx):
    cfg = synth_model.TINY_K
    with pytest.raises(ValueError):
        HfModel(ctx, cfg, proj_dtypes=[5] * 7)                       # 7 per layer needed
    with pytest.raises(HomuraError):
        HfModel(ctx, cfg, proj_dtypes=[1] * 7 * cfg.num_hidden_layers)  # bf16 is not a block type
    with pytest.raises(HomuraError):                                 # hidden 256*k needed for K-quants
        HfModel(ctx, synth_model.TINY_LLAMA, proj_dtypes=[2, 2, 2, 2, 2, 2, 5] * 2)  # inter 704 % 256 != 0


@pytest.mark.parametrize("kind", ["q6_k", "q4_k", "q8_0", "q4_0"])
def test_lm_head_from_kquant_blocks(ctx, kind):
    """The LM head of a block-quantised plan given as the raw blocks of the output matrix: the same f32
    product as with the dequantised matrix in the f32 slot (the oracle, and a second model, get
    oracle.dequant of the blocks), for single steps, the greedy loop, graph replay and the prompt pass."""
    import pyoracle
    cfg = synth_model.TINY_K
    L = cfg.num_hidden_layers
    mix = synth_model.q4_k_m_mix(cfg)
    weights = synth_model.synth_weights(cfg, 91, has_qk_norm=False, proj_dtypes=mix)
    assert weights[-1][0] == "lm_head.weight"
    code = {"q8_0": 2, "q4_0": 3, "q4_k": 5, "q6_k": 6}[kind]
    if kind in ("q6_k", "q4_k"):
        raw = (synth.q6_k_blocks if kind == "q6_k" else synth.q4_k_blocks)(92, cfg.vocab_size * cfg.hidden_size // 256)
    else:
        raw = (synth.q8_0_blocks if kind == "q8_0" else synth.q4_0_blocks)(92, cfg.vocab_size * cfg.hidden_size // 32, 0.01)
    dequant = {"q8_0": pyoracle.dequant_q8_0, "q4_0": pyoracle.dequant_q4_0, "q4_k": pyoracle.dequant_q4_k,
               "q6_k": pyoracle.dequant_q6_k}[kind]
    dense = dequant(raw).reshape(cfg.vocab_size, cfg.hidden_size)
    weights[-1] = ("lm_head.weight", np.ascontiguousarray(dense.T))   # the slot takes [hidden][vocab]
    dense_model = synth_model.build_model(ctx, cfg, weights, 160, has_qk_norm=False, proj_dtypes=mix)
    om = mf.build_oracle_model(cfg, weights, 160, has_qk_norm=False, proj_dtypes=mix)

    gm = HfModel(ctx, cfg, has_qk_norm=False, proj_dtypes=mix)
    for i, (name, arr) in enumerate(weights[:-1]):
        gm.set_weight(i, arr)
    with pytest.raises(HomuraError):
        gm.set_lm_head_blocks(code, raw[:-1])       # wrong size
    with pytest.raises(HomuraError):
        gm.set_lm_head_blocks(1, raw)               # bf16 is not a block type
    gm.set_lm_head_blocks(code, raw)
    gm.finalize(160)

    kv = synth_model.synth_kv(cfg, 3, 29)
    ids = synth.token_ids(4, 5, cfg.vocab_size)
    for m in (gm, dense_model):
        m.set_prefill_min(0)
        m.init_kv_cache(kv, 29)
    mf.oracle_init_kv(om, kv)
    got, dense_got = gm.run_kv(ids), dense_model.run_kv(ids)
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(5)])
    scale = np.abs(want).max()
    for i in range(5):
        assert mf.rel_err(got[i], want[i]) < 1e-2, f"position {i}"
    assert np.abs(got - dense_got).max() < 2e-5 * scale   # two f32 summation orders over the same terms
    want_t, margins = om.generate_greedy(ids[:2], 24)
    say(f"LM head from {kind} blocks: min margin {margins.min():.3e}, blocks vs dense {np.abs(got - dense_got).max() / scale:.1e}")
    assert np.array_equal(gm.generate_greedy(ids[:2], 24), want_t)
    gm.set_graph(True)
    gm.init_kv_cache(kv, 29)
    gm.run_kv(ids)
    assert np.array_equal(gm.generate_greedy(ids[:2], 24), want_t)
    # prompt pass: logits of every row through the piece GEMM over the dequantised blocks
    long_ids = synth.token_ids(8, 40, cfg.vocab_size)
    for m in (gm, dense_model):
        m.set_prefill_min(8)
        m.reset_kv_cache()
    a, b = gm.run_kv(long_ids), dense_model.run_kv(long_ids)
    assert np.abs(a - b).max() < 2e-5 * np.abs(b).max()
    gm.close()
    dense_model.close()

    # equal maxima: the winning row's blocks copied to two more rows; the last of the three must win
    # (Rust Iterator::max_by, src/generate.rs:735-742), through the candidates of every workgroup
    rowbytes = raw.size // cfg.vocab_size
    rows = raw.reshape(cfg.vocab_size, rowbytes).copy()
    t = int(want_t[0])
    twins = sorted({t, (t + 17) % cfg.vocab_size, (t + 401) % cfg.vocab_size})
    for r in twins:
        rows[r] = rows[t]
    gm2 = HfModel(ctx, cfg, has_qk_norm=False, proj_dtypes=mix)
    for i, (name, arr) in enumerate(weights[:-1]):
        gm2.set_weight(i, arr)
    gm2.set_lm_head_blocks(code, rows.reshape(-1))
    gm2.finalize(160)
    gm2.init_kv_cache(kv, 29)
    gm2.run_kv(ids)
    assert int(gm2.generate_greedy(ids[:2], 1)[0]) == twins[-1]
    gm2.close()
