"""The whole-step decode launch (one resident kernel for the embedding row and every layer, phases
exchanging tagged values through device memory) against the CPU oracle and against the plan's
one-launch-per-projection path, through the C boundary. Logits within 1e-2 max relative error,
|gpu - ref| / max(|ref|, 1e-2 * max|ref|); greedy tokens identical."""
import dataclasses

import numpy as np
import pytest

import model_fixture as mf
from homura_amd import HomuraError, synth, synth_model

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)


@pytest.fixture(scope="module")
def small(ctx):
    cfg = synth_model.SMALL_WS
    weights = synth_model.synth_weights(cfg, 5151)
    gm = synth_model.build_model(ctx, cfg, weights, 2048)
    om = mf.build_oracle_model(cfg, weights, 2048)
    yield cfg, weights, gm, om
    gm.close()


def test_small_shape_is_served_and_on_by_default(small):
    _cfg, _w, gm, _om = small
    assert gm.whole_step_available() and gm.whole_step()
    assert gm.launches_per_step() == 1   # embedding row, layers, LM head and greedy pick in one launch


@pytest.mark.parametrize("cache_rows", [0, 2, 31, 50, 333])
def test_logits_and_tokens_against_oracle(small, cache_rows):
    """Caches that leave most attention splits empty (0, 2 rows), that straddle a split boundary while
    tokens are appended (31 -> 36), and ordinary ones. (With so few rows one cache row that lands on the
    other side of a bf16 rounding boundary moves the logits by 1e-4..4e-4 of their scale; both GPU paths
    show it against the oracle, e.g. from a one-row cache, and the 1% floor of rel_err absorbs it here.)"""
    cfg, _w, gm, om = small
    kv = synth_model.synth_kv(cfg, 7 + cache_rows, max(cache_rows, 1))
    gm.set_whole_step(True)
    gm.init_kv_cache(kv, cache_rows)
    mf.oracle_init_kv(om, kv)
    om.kv.reset(cache_rows)
    ids = synth.token_ids(8 + cache_rows, 5, cfg.vocab_size)
    gm.set_prefill_min(0)
    got = gm.run_kv(ids)
    gm.whole_step_status()
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(5)])
    for i in range(5):
        assert mf.rel_err(got[i], want[i]) < 1e-2, f"cache {cache_rows}, position {i}"
    want_t, margins = om.generate_greedy(ids[:2], 24)
    got_t = gm.generate_greedy(ids[:2], 24)
    say(f"cache {cache_rows}: min margin {margins.min():.3e}")
    assert np.array_equal(got_t, want_t)
    assert gm.kv_cache_len() == cache_rows + 5 + 2 + 23


def test_whole_step_against_per_projection_path(small):
    """Same arithmetic as the per-projection kernels up to the order of f32 sums in attention."""
    cfg, _w, gm, _om = small
    kv = synth_model.synth_kv(cfg, 21, 200)
    ids = synth.token_ids(22, 6, cfg.vocab_size)
    gm.set_prefill_min(0)
    gm.set_whole_step(False)
    gm.init_kv_cache(kv, 200)
    ref = gm.run_kv(ids)
    ref_t = gm.generate_greedy(ids[:1], 30)
    gm.set_whole_step(True)
    gm.init_kv_cache(kv, 200)
    got = gm.run_kv(ids)
    got_t = gm.generate_greedy(ids[:1], 30)
    gm.whole_step_status()
    assert mf.rel_err(got, ref) < 1e-3
    assert np.array_equal(got_t, ref_t)


def test_graph_replay_and_cache_rebuild(small):
    """Replays interleaved with eager work; re-creating the KV cache (other max length would move its
    addresses) refreshes the device layer table."""
    cfg, _w, gm, _om = small
    kv = synth_model.synth_kv(cfg, 17, 30)
    ids = synth.token_ids(18, 4, cfg.vocab_size)
    gm.set_whole_step(True)
    gm.set_prefill_min(0)
    gm.init_kv_cache(kv, 30)
    eager_tokens = gm.generate_greedy(ids, 24)
    gm.init_kv_cache(kv, 30)
    eager_logits = gm.run_kv(ids[:1])
    gm.set_graph(True)
    try:
        for rep in range(3):
            gm.init_kv_cache(kv, 30)
            assert np.array_equal(gm.generate_greedy(ids, 24), eager_tokens), f"replay round {rep}"
            gm.init_kv_cache(kv, 30)
            assert np.array_equal(gm.run_kv(ids[:1]), eager_logits)
    finally:
        gm.set_graph(False)
    gm.whole_step_status()


def test_long_cache_up_to_the_served_maximum(small):
    """2048 rows is what the attention phase of this instance keeps in registers (32 splits x 64 rows)."""
    cfg, _w, gm, om = small
    rows = 2040
    kv = synth_model.synth_kv(cfg, 99, rows)
    gm.set_whole_step(True)
    gm.set_prefill_min(0)
    gm.init_kv_cache(kv, rows)
    mf.oracle_init_kv(om, kv)
    ids = synth.token_ids(98, 8, cfg.vocab_size)
    got = gm.run_kv(ids)
    gm.whole_step_status()
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(8)])
    assert gm.kv_cache_len() == 2048
    for i in range(8):
        assert mf.rel_err(got[i], want[i]) < 1e-2, f"position {i}"
    with pytest.raises(HomuraError) as e:
        gm.run_kv(ids[:1])
    assert "KV cache full" in str(e.value)


@pytest.mark.parametrize("name,qk_norm,bias", [("q8_0", True, False), ("q4_0", True, False), ("q8_0", False, True)])
def test_quantised_whole_step_against_oracle_and_per_projection_path(ctx, name, qk_norm, bias):
    """Q8_0 / Q4_0 projections (re-packed into planes at finalize) through the whole-step launch: logits
    against the oracle's quantised plan, and logits and greedy tokens against the plan's own
    one-launch-per-projection path, from a cache that crosses an attention split boundary."""
    from homura_amd.runtime import DTYPE_Q4_0, DTYPE_Q8_0
    wdt = DTYPE_Q8_0 if name == "q8_0" else DTYPE_Q4_0
    cfg = dataclasses.replace(synth_model.SMALL_WS_Q, attention_bias=bias)
    weights = synth_model.synth_weights(cfg, 909, wdt, has_qk_norm=qk_norm)
    gm = synth_model.build_model(ctx, cfg, weights, 1024, wdt, has_qk_norm=qk_norm)
    om = mf.build_oracle_model(cfg, weights, 1024, wdt, has_qk_norm=qk_norm)
    assert gm.whole_step_available() and gm.whole_step()
    kv = synth_model.synth_kv(cfg, 31, 61)
    ids = synth.token_ids(32, 7, cfg.vocab_size)
    gm.set_prefill_min(0)
    gm.init_kv_cache(kv, 61)
    mf.oracle_init_kv(om, kv)
    got = gm.run_kv(ids)
    got_t = gm.generate_greedy(ids[:1], 30)
    gm.whole_step_status()
    assert gm.launches_per_step() == 3
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(7)])
    for i in range(7):
        err = mf.rel_err(got[i], want[i])
        say(f"{name} qk_norm={qk_norm} bias={bias}: position {i} rel err {err:.2e}")
        assert err < 1e-2
    gm.set_whole_step(False)
    gm.init_kv_cache(kv, 61)
    ref = gm.run_kv(ids)
    ref_t = gm.generate_greedy(ids[:1], 30)
    assert gm.launches_per_step() > 3
    # the two paths add the same products in different orders; where that puts a new K or V element on the
    # other side of a bf16 rounding boundary the rows that follow differ by up to a few 1e-3 in a model this small
    assert mf.rel_err(got, ref) < 1e-2
    assert np.array_equal(got_t, ref_t)
    gm.set_whole_step(True)
    gm.set_graph(True)
    gm.init_kv_cache(kv, 61)
    gm.run_kv(ids)
    assert np.array_equal(gm.generate_greedy(ids[:1], 30), got_t)
    gm.close()


def test_bias_and_no_qk_norm_variant(ctx):
    """Q/K/V biases ride in the Q|K|V phase; without QK-norm the rows go straight to RoPE."""
    cfg = dataclasses.replace(synth_model.SMALL_WS, attention_bias=True)
    weights = synth_model.synth_weights(cfg, 77, has_qk_norm=False)
    assert any(n.endswith("q_proj.bias") for n, _ in weights)
    gm = synth_model.build_model(ctx, cfg, weights, 128, has_qk_norm=False)
    om = mf.build_oracle_model(cfg, weights, 128, has_qk_norm=False)
    assert gm.whole_step()
    kv = synth_model.synth_kv(cfg, 8, 21)
    gm.init_kv_cache(kv, 21)
    mf.oracle_init_kv(om, kv)
    ids = synth.token_ids(6, 5, cfg.vocab_size)
    gm.set_prefill_min(0)
    got = gm.run_kv(ids)
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(5)])
    for i in range(5):
        assert mf.rel_err(got[i], want[i]) < 1e-2, f"position {i}"
    want_t, _ = om.generate_greedy(ids[:2], 20)
    assert np.array_equal(gm.generate_greedy(ids[:2], 20), want_t)
    gm.whole_step_status()
    gm.close()


def test_qwen3_0p6b_shape_against_per_projection_path(ctx):
    """The benchmark shape: same tokens and close logits from both ways through the layers (the 64-token
    oracle identity of this shape runs in test_gpu_model.py with the whole-step launch on)."""
    cfg = synth_model.QWEN3_0P6B
    weights = synth_model.synth_weights(cfg, 0xC0FFEE02)
    gm = synth_model.build_model(ctx, cfg, weights, 1120)
    assert gm.whole_step_available() and gm.whole_step()
    kv = synth_model.synth_kv(cfg, 5, 1024)
    ids = synth.token_ids(6, 3, cfg.vocab_size)
    gm.set_prefill_min(0)
    gm.set_graph(True)
    gm.init_kv_cache(kv, 1024)
    got = gm.run_kv(ids)
    got_t = gm.generate_greedy(ids[:1], 32)
    gm.whole_step_status()
    trace = gm.whole_step_trace()      # switches recording on
    assert len(trace) == 0
    gm.generate_greedy(ids[:1], 2)
    trace = gm.whole_step_trace().astype(np.int64)
    assert len(trace) == cfg.num_hidden_layers * 11 + 2
    assert np.all(np.diff(trace[:-1]) >= 0) and trace[-1] in (0, 1)
    say(f"whole-step kernel {(trace[-2] - trace[0]) / 100.0:.1f} us from first to last mark, die-local exchanges: {trace[-1]}")
    gm.set_whole_step(False)
    gm.init_kv_cache(kv, 1024)
    ref = gm.run_kv(ids)
    ref_t = gm.generate_greedy(ids[:1], 32)
    assert mf.rel_err(got, ref) < 1e-3
    assert np.array_equal(got_t, ref_t)
    gm.close()


@pytest.mark.parametrize("shape", ["small", "qwen3_0p6b"])
def test_exchanges_through_memory_when_placement_is_not_die_local(ctx, monkeypatch, shape):
    """The path a step takes when the kernel does not find its workgroups dealt to the dies round-robin (no
    die-local stores, the relays publish their sums through memory), forced from the host: same logits and
    tokens as with die-local exchanges, and the trace's last word says which path ran."""
    cfg = synth_model.SMALL_WS if shape == "small" else synth_model.QWEN3_0P6B
    rows = 150 if shape == "small" else 700
    weights = synth_model.synth_weights(cfg, 777)
    kv = synth_model.synth_kv(cfg, 8, rows)
    ids = synth.token_ids(9, 4, cfg.vocab_size)
    out = {}
    for far in ("1", "0"):
        monkeypatch.setenv("HOMURA_WHOLE_STEP_FAR", far)
        gm = synth_model.build_model(ctx, cfg, weights, rows + 64)
        assert gm.whole_step_available() and gm.whole_step()
        gm.set_prefill_min(0)
        gm.init_kv_cache(kv, rows)
        gm.whole_step_trace()          # switches recording on
        logits = gm.run_kv(ids)
        tokens = gm.generate_greedy(ids[:1], 24)
        gm.whole_step_status()
        trace = gm.whole_step_trace()
        out[far] = (logits, tokens, int(trace[-1]))
        gm.close()
    assert out["1"][2] == 0
    say(f"{shape}: die-local exchanges in the unforced run: {out['0'][2]}")
    assert mf.rel_err(out["1"][0], out["0"][0]) < 1e-5   # the same sums in the same order
    assert np.array_equal(out["1"][1], out["0"][1])


def test_unserved_shapes_keep_the_per_projection_path(ctx):
    cfg = synth_model.TINY
    weights = synth_model.synth_weights(cfg, 4242)
    gm = synth_model.build_model(ctx, cfg, weights, 64)
    assert not gm.whole_step_available() and not gm.whole_step()
    with pytest.raises(HomuraError):
        gm.set_whole_step(True)
    gm.whole_step_status()
    gm.close()


@pytest.fixture(scope="module")
def long_small(ctx):
    cfg = dataclasses.replace(synth_model.SMALL_WS, max_position_embeddings=32768)
    weights = synth_model.synth_weights(cfg, 4141)
    L = 32768
    gm = synth_model.build_model(ctx, cfg, weights, L)
    plain = synth_model.build_model(ctx, cfg, weights, L)
    plain.set_whole_step(False)
    om = mf.build_oracle_model(cfg, weights, L)
    yield cfg, gm, plain, om
    gm.close()
    plain.close()


@pytest.mark.parametrize("rows", [4094, 4600, 5000, 6200, 9000, 12287, 20000, 32754])
def test_rows_streamed_inside_the_attention_phase(long_small, rows):
    """More than 4096 live rows: a split's rows beyond the eight rounds held in registers are loaded inside
    the attention phase, two rounds at a time through a ring of three register sets. The lengths give a split one
    streamed row (4097 live rows: 129 a split), a partly filled round, an odd and an even number of
    passes, a split boundary that moves while tokens are appended, and the last round the instance
    serves (32768 rows). Logits against the oracle, tokens against the per-projection path."""
    cfg, gm, plain, om = long_small
    kv = synth_model.synth_kv(cfg, 900 + rows, rows)
    n = 10
    ids = synth.token_ids(901 + rows, n, cfg.vocab_size)
    for m in (gm, plain):
        m.set_prefill_min(0)
        m.init_kv_cache(kv, rows)
    gm.set_whole_step(True)
    mf.oracle_init_kv(om, kv)
    say(f"streamed rounds: {rows} cached rows")
    got = gm.run_kv(ids)
    gm.whole_step_status()
    assert gm.whole_step() and gm.launches_per_step() == 1
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(n)])
    for i in range(n):
        assert mf.rel_err(got[i], want[i]) < 1e-2, f"position {rows + i}"
    ref = plain.run_kv(ids)
    assert mf.rel_err(got, ref) < 1e-2
    a, b = gm.generate_greedy(ids[:1], 4), plain.generate_greedy(ids[:1], 4)   # 32754: up to the last row of the cache
    assert np.array_equal(a, b)
    gm.whole_step_status()
    assert gm.kv_cache_len() == rows + n + 4


def test_cache_longer_than_the_kernel_serves_changes_over_and_back(ctx):
    """The whole-step launch holds a split's cache rows in registers: an instance with three row rounds serves
    1536 live rows of this shape, one with four 2048, one with six 3072, one with eight 4096 and, streaming further
    rounds inside its attention phase, 32768. A model with a longer cache starts on the first, takes the next from the step
    whose live rows exceed it, one launch per projection beyond 32768, and comes back after a cache reset; the
    steps on either side of each change give the oracle's logits and the per-projection path's tokens."""
    cfg = dataclasses.replace(synth_model.SMALL_WS, max_position_embeddings=65536)
    weights = synth_model.synth_weights(cfg, 31)
    L = 32900
    gm = synth_model.build_model(ctx, cfg, weights, L)
    plain = synth_model.build_model(ctx, cfg, weights, L)
    plain.set_whole_step(False)
    om = mf.build_oracle_model(cfg, weights, L)
    assert gm.whole_step_available() and gm.whole_step() and gm.launches_per_step() == 1
    ids = synth.token_ids(33, 14, cfg.vocab_size)
    for rows, still_whole in ((1528, True), (2040, True), (3064, True), (4088, True), (32760, False)):
        kv = synth_model.synth_kv(cfg, 32 + rows, rows)
        for m in (gm, plain):
            m.set_prefill_min(0)
            m.init_kv_cache(kv, rows)
        mf.oracle_init_kv(om, kv)
        got = gm.run_kv(ids)                      # 14 positions across the border
        gm.whole_step_status()
        want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(14)])
        for i in range(14):
            assert mf.rel_err(got[i], want[i]) < 1e-2, f"position {rows + i}"
        assert gm.kv_cache_len() == rows + 14 and gm.whole_step() == still_whole
        assert (gm.launches_per_step() == 1) == still_whole
        plain.run_kv(ids)
        a, b = gm.generate_greedy(ids[:1], 12), plain.generate_greedy(ids[:1], 12)
        assert np.array_equal(a, b)
        # a device-resident run across the same border
        for m in (gm, plain):
            m.init_kv_cache(synth_model.synth_kv(cfg, 34, rows - 10), rows - 10)
        a, b = gm.generate_greedy(ids[:1], 2), plain.generate_greedy(ids[:1], 2)   # the path is chosen step by step
        assert np.array_equal(a, b) and gm.whole_step()
        a, b = gm.generate_greedy(ids[:3], 40), plain.generate_greedy(ids[:3], 40)
        gm.whole_step_status()
        assert np.array_equal(a, b) and gm.whole_step() == still_whole
    gm.reset_kv_cache()
    gm.run_kv(ids[:2])
    assert gm.whole_step()
    gm.close()
    plain.close()


def test_a_wait_that_gives_up_is_reported_and_the_call_runs_again_per_projection(small):
    """Forced from the host: a small spin bound and one workgroup that withholds its first publish, so every
    workgroup gives up its wait and the launch ends normally with the status word set. The call that meets
    the status clears the exchange state, takes the cache back and runs its steps again with one launch per
    projection; the status stays readable until the launch is re-armed."""
    cfg, _w, gm, _om = small
    kv = synth_model.synth_kv(cfg, 41, 100)
    ids = synth.token_ids(42, 4, cfg.vocab_size)
    gm.set_prefill_min(0)
    gm.set_whole_step(True)
    try:
        gm.init_kv_cache(kv, 100)
        healthy = gm.run_kv(ids)
        gm.whole_step_status()
        assert gm.whole_step()
        gm.set_whole_step(False)
        gm.init_kv_cache(kv, 100)
        per_projection = gm.run_kv(ids)
        per_projection_tokens = gm.generate_greedy(ids[:1], 6)
        gm.set_whole_step(True)

        gm.init_kv_cache(kv, 100)
        gm.whole_step_inject_timeout(workgroup=5, spin_limit=3000)
        got = gm.run_kv(ids)
        assert gm.kv_cache_len() == 104          # the failed launch moved nothing; the second run appended 4 rows
        assert not gm.whole_step()               # one launch per projection from here on
        assert np.array_equal(got, per_projection)
        with pytest.raises(HomuraError) as e:
            gm.whole_step_status()
        msg = str(e.value)
        say(msg)
        assert "stopped waiting in phase 2 of layer 0" in msg and "workgroup" in msg
        # later calls stay on the per-projection path, and the status stays readable
        assert np.array_equal(gm.generate_greedy(ids[:1], 6), per_projection_tokens)
        assert not gm.whole_step()
        with pytest.raises(HomuraError):
            gm.whole_step_status()
        # a new conversation re-arms the launch, and it works as before
        gm.reset_kv_cache()
        gm.whole_step_status()
        gm.init_kv_cache(kv, 100)
        again = gm.run_kv(ids)
        gm.whole_step_status()
        assert gm.whole_step()
        assert np.array_equal(again, healthy)
        # the device-resident greedy loop recovers the same way
        gm.set_whole_step(False)
        gm.init_kv_cache(kv, 100)
        want_tokens = gm.generate_greedy(ids, 6)
        gm.set_whole_step(True)
        gm.init_kv_cache(kv, 100)
        gm.whole_step_inject_timeout(workgroup=0, spin_limit=3000)
        assert np.array_equal(gm.generate_greedy(ids, 6), want_tokens)
        assert not gm.whole_step()
    finally:
        gm.reset_kv_cache()
        gm.set_whole_step(True)



def test_kquant_mix_whole_step_against_oracle_and_per_projection_path(ctx):
    """Q4_K / Q6_K projections (a Q4_K_M-style mix, re-packed into byte planes at finalize) through the
    whole-step launch: the same Q8_K activation quantisation and integer dot products as the per-projection
    kernels and the oracle (reference src/graph_builder/emit_quant.rs:165-816). Where the two GPU paths or the
    oracle round an activation to different Q8_K integers the logits move by ~1e-3 of their scale; tokens are
    compared where the oracle's margin is clear."""
    from homura_amd.runtime import DTYPE_Q8_0
    cfg = synth_model.SMALL_WS_Q
    mix = synth_model.q4_k_m_mix(cfg)
    weights = synth_model.synth_weights(cfg, 911, DTYPE_Q8_0, has_qk_norm=True, proj_dtypes=mix)
    gm = synth_model.build_model(ctx, cfg, weights, 1024, DTYPE_Q8_0, has_qk_norm=True, proj_dtypes=mix)
    om = mf.build_oracle_model(cfg, weights, 1024, DTYPE_Q8_0, has_qk_norm=True, proj_dtypes=mix)
    assert gm.whole_step_available() and gm.whole_step()
    kv = synth_model.synth_kv(cfg, 31, 61)
    ids = synth.token_ids(32, 7, cfg.vocab_size)
    gm.set_prefill_min(0)
    gm.init_kv_cache(kv, 61)
    mf.oracle_init_kv(om, kv)
    got = gm.run_kv(ids)
    got_t = gm.generate_greedy(ids[:1], 20)
    gm.whole_step_status()
    assert gm.launches_per_step() == 3
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(7)])
    for i in range(7):
        err = mf.rel_err(got[i], want[i])
        say(f"k-quant mix: position {i} rel err {err:.2e}")
        assert err < 1e-2
    gm.set_whole_step(False)
    gm.init_kv_cache(kv, 61)
    ref = gm.run_kv(ids)
    ref_t = gm.generate_greedy(ids[:1], 20)
    assert gm.launches_per_step() > 3
    assert mf.rel_err(got, ref) < 1e-2
    same = int(np.sum(got_t == ref_t))
    say(f"k-quant mix: {same} of {len(ref_t)} greedy tokens equal on the two GPU paths")
    assert np.array_equal(got_t[:4], ref_t[:4])
    gm.close()


@pytest.mark.parametrize("name", ["q8_0", "q4_0", "q4_k_m"])
def test_quantised_whole_step_on_long_caches(ctx, name):
    """The quantised instances of every cache tier of the small shape (16 splits a KV head: 768, 1024, 2048 live
    rows held in registers, up to 16384 with streamed rounds): logits against the oracle on both sides of each
    change of tier. The K-quant mix quantises activations to Q8_K integers, which makes a step a discontinuous
    function of its input: at about one position in eight some activation lies within f32 summation noise of a
    rounding boundary, the implementations round it to different integers, the layers behind it then differ in
    many more, and the logits end up apart by the Q8_K quantisation noise itself (1-3 % of their scale) instead of
    1e-6. Both GPU paths show such positions against the oracle and against each other, more of them the longer
    the cache (the attention sums are the noisier input). The mix is therefore held to: some positions equal
    to the oracle's within 1e-3 and none further than 5 % of the logit scale, against the oracle and against
    the per-projection path (rows left out of the attention sum, or a wrong tier, move every position)."""
    from homura_amd.runtime import DTYPE_Q4_0, DTYPE_Q8_0
    wdt = DTYPE_Q4_0 if name == "q4_0" else DTYPE_Q8_0
    cfg = dataclasses.replace(synth_model.SMALL_WS_Q, max_position_embeddings=8192)
    mix = synth_model.q4_k_m_mix(cfg) if name == "q4_k_m" else None
    weights = synth_model.synth_weights(cfg, 913, wdt, has_qk_norm=True, proj_dtypes=mix)
    L = 6100
    gm = synth_model.build_model(ctx, cfg, weights, L, wdt, has_qk_norm=True, proj_dtypes=mix)
    om = mf.build_oracle_model(cfg, weights, L, wdt, has_qk_norm=True, proj_dtypes=mix)
    assert gm.whole_step_available() and gm.whole_step()
    gm.set_prefill_min(0)
    ids = synth.token_ids(35, 8, cfg.vocab_size)
    for rows in (764, 1020, 2044, 3001, 6080):
        kv = synth_model.synth_kv(cfg, 36 + rows, rows)
        gm.init_kv_cache(kv, rows)
        mf.oracle_init_kv(om, kv)
        say(f"{name}: {rows} cached rows")
        got = gm.run_kv(ids)
        gm.whole_step_status()
        assert gm.whole_step() and gm.launches_per_step() == 3
        want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(8)])
        errs = np.array([mf.rel_err(got[i], want[i]) for i in range(8)])
        scale = np.array([np.abs(got[i] - want[i]).max() / np.abs(want[i]).max() for i in range(8)])
        say(f"{name}: {rows} cached rows: rel err " + " ".join(f"{e:.1e}" for e in errs))
        gm.set_whole_step(False)
        gm.init_kv_cache(kv, rows)
        ref = gm.run_kv(ids)
        assert gm.launches_per_step() > 3
        gm.set_whole_step(True)
        if name == "q4_k_m":
            assert np.sum(errs < 1e-3) >= 2 and scale.max() < 5e-2, f"{name}: {rows} cached rows"
            assert max(np.abs(got[i] - ref[i]).max() / np.abs(ref[i]).max() for i in range(8)) < 5e-2
        else:
            assert errs.max() < 1e-2, f"{name}: {rows} cached rows"
            assert mf.rel_err(got, ref) < 1e-2
    gm.close()
