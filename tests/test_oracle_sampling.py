"""CPU checks that pin the oracle's restatement of the reference's sampler (src/generate.rs:609-801):
the xorshift64 stream against Python integers, the reference's own sampling tests, closed-form cases and
an independent numpy restatement."""
import numpy as np
import pytest

import model_fixture  # noqa: F401  (puts oracle/ on the path)
import pyoracle
from pyoracle import OrcSamplingConfig as Cfg


def xorshift_f32(seed, n):
    s, out, mask = seed | 1, [], (1 << 64) - 1
    for _ in range(n):
        s ^= (s << 13) & mask
        s ^= s >> 7
        s ^= (s << 17) & mask
        out.append(np.float32(s >> 40) / np.float32(1 << 24))
    return out


@pytest.mark.parametrize("seed", [0, 1, 42, 2**63 + 12345, 2**64 - 1])
def test_rng_stream_matches_integer_arithmetic(seed):
    r = pyoracle.Rng(seed)
    got = [r.next_f32() for _ in range(12)]
    assert got == [float(v) for v in xorshift_f32(seed, 12)]
    assert all(0.0 <= v < 1.0 for v in got)
    # reference rng_is_deterministic (src/generate.rs:882-889)
    r1, r2 = pyoracle.Rng(42), pyoracle.Rng(42)
    assert [r1.next_f32() for _ in range(10)] == [r2.next_f32() for _ in range(10)]
    # seed | 1: an even seed and the next odd one give the same stream
    assert [pyoracle.Rng(42).next_f32()] == [pyoracle.Rng(43).next_f32()]


def test_reference_sampling_tests():
    # sample_token_greedy (src/generate.rs:891-900)
    assert pyoracle.sample_token([0.0, 1.0, 0.5, 0.2], Cfg(temperature=0.0), [], pyoracle.Rng(1)) == 1
    # min_p_filters_low_prob (src/generate.rs:990-1008)
    cfg = Cfg(temperature=1.0, min_p=0.5, top_k=0, top_p=1.0, repetition_penalty=1.0)
    rng = pyoracle.Rng(42)
    assert [pyoracle.sample_token([10.0, 0.0, 0.0, 0.0], cfg, [], rng) for _ in range(10)] == [0] * 10


def test_greedy_keeps_the_last_of_equal_maxima_and_does_not_touch_the_rng():
    rng = pyoracle.Rng(7)
    before = rng.state.value
    assert pyoracle.sample_token([1.0, 3.0, 3.0, 2.0], Cfg(temperature=0.0, repetition_penalty=1.0), [], rng) == 2
    assert rng.state.value == before


def test_top_k_one_is_the_argmax_whatever_the_draw():
    logits = np.random.default_rng(3).standard_normal(500).astype(np.float32)
    cfg = Cfg(temperature=1.3, top_k=1, top_p=1.0, repetition_penalty=1.0)
    rng = pyoracle.Rng(9)
    assert {pyoracle.sample_token(logits, cfg, [], rng) for _ in range(20)} == {int(np.argmax(logits))}


def test_repetition_penalty_applies_once_per_occurrence():
    """The reference walks generated_ids, so a token generated twice is divided twice (src/generate.rs:707-718)."""
    logits = np.array([4.0, 3.0, -1.0], np.float32)
    g = Cfg(temperature=0.0, repetition_penalty=1.2)
    assert pyoracle.sample_token(logits, g, [0], pyoracle.Rng(1)) == 0          # 4/1.2 = 3.33 > 3
    assert pyoracle.sample_token(logits, g, [0, 0], pyoracle.Rng(1)) == 1       # 4/1.44 = 2.78 < 3
    # negative logits are multiplied: -1 -> -1.2, still the smallest; ids outside the vocabulary are ignored
    assert pyoracle.sample_token(logits, g, [2, 99], pyoracle.Rng(1)) == 0
    # frequency and presence penalties: 4 - 0.6*2 - 0.5 = 2.3 < 3
    fp = Cfg(temperature=0.0, repetition_penalty=1.0, frequency_penalty=0.6, presence_penalty=0.5)
    assert pyoracle.sample_token(logits, fp, [0, 0], pyoracle.Rng(1)) == 1
    assert pyoracle.sample_token(logits, fp, [0], pyoracle.Rng(1)) == 1         # 4 - 0.6 - 0.5 = 2.9 < 3
    assert pyoracle.sample_token(logits, Cfg(temperature=0.0, repetition_penalty=1.0, presence_penalty=0.5),
                                 [0], pyoracle.Rng(1)) == 0                     # 3.5 > 3


def test_draw_frequencies_follow_the_softmax():
    logits = np.array([2.0, 1.0, 0.5, 0.0, -1.0, -3.0], np.float32)
    cfg = Cfg(temperature=0.8, top_k=0, top_p=1.0, repetition_penalty=1.0)
    p = np.exp(logits.astype(np.float64) / 0.8)
    p /= p.sum()
    rng = pyoracle.Rng(2024)
    n = 20000
    counts = np.bincount([pyoracle.sample_token(logits, cfg, [], rng) for _ in range(n)], minlength=6)
    sigma = np.sqrt(n * p * (1 - p))
    assert np.all(np.abs(counts - n * p) < 4.5 * sigma), (counts, n * p)
    # top_p = 0.75 keeps the smallest prefix whose mass reaches 0.75; top_k = 2 keeps two
    cut = int(np.searchsorted(np.cumsum(p), 0.75)) + 1
    rng = pyoracle.Rng(5)
    seen = {pyoracle.sample_token(logits, Cfg(temperature=0.8, top_k=0, top_p=0.75, repetition_penalty=1.0), [], rng)
            for _ in range(3000)}
    assert seen == set(range(cut))
    seen = {pyoracle.sample_token(logits, Cfg(temperature=0.8, top_k=2, top_p=1.0, repetition_penalty=1.0), [], rng)
            for _ in range(2000)}
    assert seen == {0, 1}


def numpy_sample(logits, cfg, generated, u):
    """The same procedure written with numpy float32 arrays (cumsum is a sequential f32 sum)."""
    l = np.array(logits, np.float32)
    for t in generated:
        if cfg.repetition_penalty != 1.0:
            l[t] = l[t] / np.float32(cfg.repetition_penalty) if l[t] > 0 else l[t] * np.float32(cfg.repetition_penalty)
    if cfg.frequency_penalty != 0.0 or cfg.presence_penalty != 0.0:
        cnt = np.bincount(np.array(generated, np.int64), minlength=l.size)
        seen = cnt > 0
        l[seen] = l[seen] - np.float32(cfg.frequency_penalty) * cnt[seen].astype(np.float32)
        l[seen] = l[seen] - np.float32(cfg.presence_penalty)
    l = l * (np.float32(1.0) / np.float32(cfg.temperature))
    p = np.exp(l - l.max()).astype(np.float32)
    p = p / np.cumsum(p, dtype=np.float32)[-1]
    if cfg.min_p > 0:
        p[p < np.float32(cfg.min_p) * p.max()] = 0
    order = np.lexsort((np.arange(p.size), -p))
    if 0 < cfg.top_k < p.size:
        order = order[:cfg.top_k]
    cum = np.cumsum(p[order], dtype=np.float32)
    hit = np.nonzero(cum >= np.float32(cfg.top_p))[0]
    cutoff = int(hit[0]) + 1 if hit.size else order.size
    cum = cum[:cutoff]
    r = np.float32(u) * cum[-1]
    hit = np.nonzero(cum >= r)[0]
    return int(order[hit[0]] if hit.size else order[cutoff - 1])


@pytest.mark.parametrize("cfg", [Cfg(), Cfg(temperature=1.0, top_k=0, top_p=0.95, repetition_penalty=1.0),
                                 Cfg(temperature=0.5, top_k=200, top_p=1.0, min_p=0.05, repetition_penalty=1.3,
                                     frequency_penalty=0.2, presence_penalty=0.1)])
def test_against_a_numpy_restatement_on_random_logits(cfg):
    gen = np.random.default_rng(11)
    checked = 0
    for trial in range(60):
        logits = (gen.standard_normal(1500) * 2.5).astype(np.float32)
        generated = gen.integers(0, 1500, size=trial % 7).tolist()
        rng = pyoracle.Rng(1000 + trial)
        for _ in range(trial % 5):
            rng.next_f32()
        state = rng.state.value
        tok, (m_draw, m_top_p) = pyoracle.sample_token(logits, cfg, generated, rng, want_margins=True)
        u = pyoracle.Rng.__new__(pyoracle.Rng)
        u.state = type(rng.state)(state)
        draw = u.next_f32()
        if min(m_draw, m_top_p) < 1e-5:
            continue        # numpy's exp may differ from libm's in the last bit: skip draws that sit on a boundary
        assert tok == numpy_sample(logits, cfg, generated, draw), trial
        checked += 1
    assert checked > 50


# ── the library's host-side sampler (no GPU involved): exact agreement with the oracle ──

def _lib_cfg(c):
    from homura_amd.runtime import SamplingConfig
    return SamplingConfig(c.temperature, c.top_k, c.top_p, c.min_p, c.repetition_penalty, c.frequency_penalty,
                          c.presence_penalty)


@pytest.mark.parametrize("cfg", [Cfg(), Cfg(temperature=0.0), Cfg(temperature=1.0, top_k=0, top_p=0.95, repetition_penalty=1.0),
                                 Cfg(temperature=0.5, top_k=200, top_p=1.0, min_p=0.05, repetition_penalty=1.3,
                                     frequency_penalty=0.2, presence_penalty=0.1),
                                 Cfg(temperature=2.0, top_k=5000, top_p=0.5)])
def test_library_host_sampler_equals_the_oracle(cfg):
    from homura_amd import runtime
    gen = np.random.default_rng(5)
    for trial in range(40):
        n = [7, 300, 4000][trial % 3]
        logits = (gen.standard_normal(n) * 3).astype(np.float32)
        if trial % 4 == 0:
            logits[gen.integers(0, n, 3)] = logits.max()        # equal maxima / equal probabilities
        generated = gen.integers(0, n + 2, size=trial % 9).tolist()   # some ids outside the vocabulary
        seed = 77 + trial
        a, b = pyoracle.Rng(seed), runtime.Rng(seed)
        for _ in range(3):          # consecutive draws from one stream
            want = pyoracle.sample_token(logits, cfg, generated, a)
            got = runtime.sample_token_host(logits, _lib_cfg(cfg), generated, b)
            assert got == want and a.state.value == b.state.value, (trial, n)


def test_library_rng_equals_the_oracle():
    from homura_amd import runtime
    for seed in (0, 42, 2**64 - 1):
        a, b = pyoracle.Rng(seed), runtime.Rng(seed)
        assert [a.next_f32() for _ in range(8)] == [b.next_f32() for _ in range(8)]
