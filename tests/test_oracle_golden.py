"""Pins the CPU oracle: every function is checked against the reference's own known-answer
vectors (tests/golden/reference_vectors.json) and, where those leave room, against facts the
mathematics fixes (closed forms, numpy float16, fp64 brute force, invariants). CPU only."""
import math

import numpy as np
import pytest


def rel_err(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    floor = 1e-6 * max(1e-30, np.abs(b).max())
    return np.max(np.abs(a - b) / np.maximum(np.abs(b), floor))


# ── scalar conversions ────────────────────────────────────────────────────────

def test_f16_exhaustive_against_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.f16_to_f32_array(bits)
    # bit patterns must agree everywhere, NaN payloads included
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_f16_reference_constants(oracle, golden):
    for bits, val in golden["f16_constants"]["bits_to_value"].items():
        assert oracle.f16_to_f32(int(bits)) == val


def test_bf16_reference_constants(oracle, golden):
    lib = oracle.load()
    for bits, val in golden["bf16_conversion_basic"]["bits_to_value"].items():
        assert lib.orc_bf16_to_f32(int(bits)) == val
    # truncation is the top half of the f32 pattern (reference src/hf/weights.rs:206-214)
    x = np.float32(1.0 + 2 ** -9)
    assert lib.orc_f32_to_bf16_trunc(x) == (x.view(np.uint32) >> 16)


def test_bf16_rne_matches_textbook(oracle):
    lib = oracle.load()
    rng = np.random.default_rng(0)
    xs = rng.standard_normal(20000).astype(np.float32)
    xs[:4] = [1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, -0.0, 3.0e38]  # exact ties, sign, near-overflow
    for x in xs:
        got = lib.orc_f32_to_bf16_rne(x)
        lo = np.uint32(x.view(np.uint32) & 0xFFFF0000).view(np.float32)
        hi = np.uint32((x.view(np.uint32) & 0xFFFF0000) + 0x10000).view(np.float32)
        gotf = np.uint32(got << 16).view(np.float32)
        # nearest of the two neighbours; on a tie the even mantissa
        dl, dh = abs(float(x) - float(lo)), abs(float(hi) - float(x))
        if dl < dh:
            assert gotf == lo
        elif dh < dl:
            assert gotf == hi
        else:
            assert (got & 1) == 0 and gotf in (lo, hi)


# ── block formats ─────────────────────────────────────────────────────────────

def test_block_sizes(golden):
    assert golden["block_sizes"]["q8_0"] == {"block_elems": 32, "block_bytes": 34}
    assert golden["block_sizes"]["q4_0"]["block_bytes"] == 18


def q8_blocks(d_bits, quants):
    """Build raw Q8_0 bytes: quants [nblocks][32] int8, d_bits [nblocks] uint16."""
    nb = len(d_bits)
    out = np.zeros((nb, 34), np.uint8)
    out[:, 0] = np.asarray(d_bits) & 0xFF
    out[:, 1] = np.asarray(d_bits) >> 8
    out[:, 2:] = np.asarray(quants, np.int8).view(np.uint8).reshape(nb, 32)
    return out.reshape(-1)


def test_q8_0_reference_kat(oracle, golden):
    g = golden["emit_q8_0_correctness"]
    K, N = g["K"], g["N"]
    blocks = q8_blocks([g["scale_bits"]] * N, np.tile(np.arange(1, 33), (N, 1)))
    x = np.full((1, K), g["activation"], np.float32)
    out = oracle.gemv_q8_0(x, blocks, 1, K, N)
    assert np.all(np.abs(out - g["expected_each"]) < g["tolerance"])
    assert np.all(out == 528.0)  # exactly representable, so the oracle must hit it exactly


def numpy_dequant_q8_0(raw):
    blk = raw.reshape(-1, 34)
    d = blk[:, :2].copy().view(np.float16).astype(np.float32)  # [nb,1]
    q = blk[:, 2:].view(np.int8).astype(np.float32)
    return (q * d).reshape(-1)


def numpy_dequant_q4_0(raw):
    """Independent decode of ggml block_q4_0: low nibbles are elements 0..15, high 16..31."""
    blk = raw.reshape(-1, 18)
    d = blk[:, :2].copy().view(np.float16).astype(np.float32)
    qs = blk[:, 2:]
    lo = (qs & 0x0F).astype(np.int32) - 8
    hi = (qs >> 4).astype(np.int32) - 8
    q = np.concatenate([lo, hi], axis=1).astype(np.float32)
    return (q * d).reshape(-1)


def test_dequant_q8_0_bit_exact_vs_numpy(oracle):
    from homura_amd import synth
    raw = synth.q8_0_blocks(11, 4096)
    raw[:2] = [0x01, 0x00]  # a subnormal f16 scale in block 0
    assert np.array_equal(oracle.dequant_q8_0(raw).view(np.uint32),
                          numpy_dequant_q8_0(raw).view(np.uint32))


def test_dequant_q4_0_bit_exact_vs_numpy(oracle):
    from homura_amd import synth
    raw = synth.q4_0_blocks(12, 4096)
    assert np.array_equal(oracle.dequant_q4_0(raw).view(np.uint32),
                          numpy_dequant_q4_0(raw).view(np.uint32))


def test_q4_0_hand_block(oracle):
    # d = 0.5, byte j = (j) | ((15-j) << 4): element j = j-8, element j+16 = 7-j
    raw = np.zeros(18, np.uint8)
    raw[0], raw[1] = 0x00, 0x38
    for j in range(16):
        raw[2 + j] = j | ((15 - j) << 4)
    got = oracle.dequant_q4_0(raw)
    want = np.array([(j - 8) * 0.5 for j in range(16)] + [(7 - j) * 0.5 for j in range(16)], np.float32)
    assert np.array_equal(got, want)
    x = np.arange(32, dtype=np.float32)[None, :]
    assert oracle.gemv_q4_0(x, raw, 1, 32, 1)[0, 0] == float(np.dot(want.astype(np.float64), x[0]))


@pytest.mark.parametrize("kind", ["q8_0", "q4_0"])
def test_quant_gemv_vs_fp64(oracle, kind):
    from homura_amd import synth
    K, N = 256, 96
    nb = N * K // 32
    raw = synth.q8_0_blocks(21, nb) if kind == "q8_0" else synth.q4_0_blocks(22, nb)
    w = (numpy_dequant_q8_0(raw) if kind == "q8_0" else numpy_dequant_q4_0(raw)).reshape(N, K)
    x = synth.normal_f32(23, 2 * K).reshape(2, K)
    fn = oracle.gemv_q8_0 if kind == "q8_0" else oracle.gemv_q4_0
    got = fn(x, raw, 2, K, N)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    assert rel_err(got, want) < 1e-4


# ── matmul ────────────────────────────────────────────────────────────────────

def to_bf16_bits_exact(a):
    a = np.asarray(a, np.float32)
    bits = (a.view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal((bits.astype(np.uint32) << 16).view(np.float32), a), "not bf16-representable"
    return bits


def test_matmul_reference_vectors(oracle, golden):
    for name in ("matmul_2d_known_values", "matmul_2d_static"):
        g = golden[name]
        a, b = np.array(g["a"], np.float32), np.array(g["b"], np.float32)
        M, K = a.shape
        N = b.shape[1]
        want = np.array(g["expected"], np.float32)
        assert np.allclose(oracle.matmul_f32_f32(a, b, M, K, N), want, atol=1e-4)
        # the same integers are exact in bf16, so the mixed-precision path must agree too
        assert np.allclose(oracle.matmul_f32_bf16(a, to_bf16_bits_exact(b), M, K, N), want, atol=1e-4)
        assert np.allclose(oracle.matmul_bf16_bf16(to_bf16_bits_exact(a), to_bf16_bits_exact(b), M, K, N),
                           want, atol=1e-4)


def test_matmul_bf16_vs_fp64_and_transposition(oracle):
    from homura_amd import synth
    M, K, N = 3, 200, 136
    x = synth.normal_f32(31, M * K).reshape(M, K)
    wb = synth.normal_bf16(32, K * N, 0.02).reshape(K, N)
    w = synth.bf16_to_f32(wb)
    got = oracle.matmul_f32_bf16(x, wb, M, K, N)
    want = x.astype(np.float64) @ w.astype(np.float64)
    assert rel_err(got, want) < 1e-4
    # a transposed operand or a swapped M/N would not survive a non-square, non-symmetric case
    assert rel_err(got, (w.astype(np.float64).T @ x.astype(np.float64).T).T) < 1e-4


# ── light ops ─────────────────────────────────────────────────────────────────

def test_rms_norm_reference_vector(oracle, golden):
    g = golden["rms_norm_basic"]
    x = np.array([g["input"]], np.float32)
    w = np.array(g["weight"], np.float32)
    want = x / math.sqrt(g["mean_square"] + g["eps"])
    for variant in ("f32", "f64acc", "f64mean"):
        assert np.allclose(oracle.rms_norm(x, w, g["eps"], variant), want, atol=g["tolerance"])


def test_rms_norm_weight_and_eps(oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 64)).astype(np.float32)
    w = rng.standard_normal(64).astype(np.float32)
    eps = 1e-2  # large enough that dropping it would show
    want = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + eps) * w
    for variant in ("f32", "f64acc", "f64mean"):
        assert rel_err(oracle.rms_norm(x, w, eps, variant), want) < 1e-5


def test_silu_reference_vector(oracle, golden):
    g = golden["silu_basic"]
    x = np.array(g["input"], np.float32)
    want = np.array([v / (1.0 + math.exp(-v)) for v in g["input"]])
    got = oracle.silu_mul(x, np.ones_like(x))
    assert np.allclose(got, want, atol=g["tolerance"])
    up = np.array([2.0, -3.0, 0.5, 4.0], np.float32)
    assert np.allclose(oracle.silu_mul(x, up), want * up, atol=1e-5)


def test_softmax_reference_vectors(oracle, golden):
    g = golden["softmax_static"]
    for f64 in (False, True):
        got = oracle.softmax(np.array([g["input"]], np.float32), f64)[0]
        assert np.allclose(got, g["expected"], atol=g["tolerance"])
        assert abs(got.sum() - 1.0) < g["sum_tolerance"]
        sigma = 1.0 / (1.0 + math.e)
        cols = oracle.softmax(np.array(golden["softmax_2d_axis0"]["columns"], np.float32), f64)
        assert np.allclose(cols, [[sigma, 1 - sigma]] * 2, atol=1e-5)
    # shift invariance and -inf entries (the causal mask) give exact zeros
    x = np.array([[0.3, -np.inf, 1.2, -np.inf]], np.float32)
    p = oracle.softmax(x)
    assert p[0, 1] == 0.0 and p[0, 3] == 0.0 and abs(p.sum() - 1) < 1e-6


def test_rope_tables_reference_vector(oracle, golden):
    g = golden["rope_basic_values"]
    cos, sin = oracle.rope_tables(g["head_dim"], g["max_seq_len"], g["theta"])
    c, s = cos.reshape(-1), sin.reshape(-1)
    for i, v in g["cos"].items():
        assert abs(c[int(i)] - v) < g["tolerance"]
    for i, v in g["sin"].items():
        assert abs(s[int(i)] - v) < g["tolerance"]
    for a, b in g["duplicated_pairs"]:
        assert c[a] == c[b] and s[a] == s[b]
    # theta 1e6, head_dim 128 spot value: angle = pos / theta^(2i/hd)
    cos2, sin2 = oracle.rope_tables(128, 1100, 1e6)
    pos, i = 1077, 37
    ang = pos / (1e6 ** (2 * i / 128))
    assert abs(cos2[pos, i] - math.cos(ang)) < 1e-6 and abs(sin2[pos, 64 + i] - math.sin(ang)) < 1e-6


def test_causal_mask_reference_vectors(oracle, golden):
    g = golden["causal_mask_prefill"]
    m = oracle.causal_mask(g["seq"], g["past"]).reshape(-1)
    assert all(np.isneginf(m[i]) for i in g["neg_inf_at"]) and all(m[i] == 0.0 for i in g["zero_at"])
    d = golden["causal_mask_decode"]
    assert np.all(oracle.causal_mask(d["seq"], d["past"]) == 0.0)
    # incremental multi-token append: row i may see columns <= i + past
    m2 = oracle.causal_mask(2, 3)
    assert np.array_equal(np.isneginf(m2), [[False] * 4 + [True], [False] * 5])


def test_rope_half_closed_form(oracle):
    """rotate_half convention: pairs are (i, i + hd/2), NOT interleaved (2i, 2i+1)."""
    hd, S, heads = 8, 3, 2
    cos, sin = oracle.rope_tables(hd, 16, 10000.0)
    rng = np.random.default_rng(2)
    x = rng.standard_normal((S, heads, hd)).astype(np.float32)
    pos = [0, 5, 9]
    got = oracle.rope_half(x, cos[pos], sin[pos])
    half = hd // 2
    for s, p in enumerate(pos):
        for h in range(heads):
            for i in range(half):
                ang = p / (10000.0 ** (2 * i / hd))
                a, b = float(x[s, h, i]), float(x[s, h, i + half])
                assert abs(got[s, h, i] - (a * math.cos(ang) - b * math.sin(ang))) < 1e-5
                assert abs(got[s, h, i + half] - (b * math.cos(ang) + a * math.sin(ang))) < 1e-5
    assert np.array_equal(got[0], x[0])  # position 0 is the identity
    # each (i, i+half) pair keeps its norm
    n0 = x[..., :half] ** 2 + x[..., half:] ** 2
    n1 = got[..., :half] ** 2 + got[..., half:] ** 2
    assert np.allclose(n0, n1, rtol=1e-5)


def test_embedding_reference_vector(oracle, golden):
    g = golden["embedding_basic"]
    got = oracle.embed(np.array(g["ids"]), np.array(g["table"], np.float32))
    assert np.array_equal(got, np.array(g["expected"], np.float32))


def test_argmax_reference_vector_and_ties(oracle, golden):
    g = golden["sample_token_greedy"]
    assert oracle.argmax_last(np.array(g["logits"], np.float32)) == g["expected"]
    # Rust's Iterator::max_by returns the LAST maximum
    assert oracle.argmax_last(np.array([3.0, 1.0, 3.0, 2.0, 3.0, 0.0], np.float32)) == 4
    assert oracle.argmax_last(np.array([-np.inf, -np.inf], np.float32)) == 1
    # NaN compares Equal and so displaces the running maximum
    assert oracle.argmax_last(np.array([1.0, np.nan, 0.5], np.float32)) == 2
    assert oracle.argmax_last(np.array([1.0, 2.0, np.nan], np.float32)) == 2


# ── attention ─────────────────────────────────────────────────────────────────

def test_gqa_head_order_matches_repeat_kv(oracle, golden):
    """repeat_kv lays heads out h0,h0,h1,h1; the floordiv map must pick the same KV head."""
    g = golden["repeat_kv_repeats_2"]
    x = np.array(g["input"], np.float32).reshape(g["input_shape"])  # [1, seq=2, kvh=2, hd=3]
    rep = np.array(g["expected"], np.float32).reshape(1, 2, 4, 3)    # [1, seq, H=4, hd]
    S, kvh, hd, H = 2, 2, 3, 4
    v_bhsd = np.ascontiguousarray(x[0].transpose(1, 0, 2))           # [kvh][seq][hd]
    k_bhsd = np.zeros_like(v_bhsd)                                   # equal scores -> mean over rows
    q = np.ones((1, H, hd), np.float32)
    out = oracle.gqa_attention(q, k_bhsd, v_bhsd, np.zeros((1, S), np.float32)).reshape(H, hd)
    want = rep[0].mean(axis=0)  # mean over seq of the repeated layout, per query head
    assert np.allclose(out, want, atol=1e-6)


def test_attention_special_cases_and_fp64(oracle):
    rng = np.random.default_rng(3)
    S, H, kvh, hd, total, max_len = 1, 6, 2, 16, 37, 64
    q = rng.standard_normal((S, H, hd)).astype(np.float32)
    k = rng.standard_normal((kvh, max_len, hd)).astype(np.float32)
    v = rng.standard_normal((kvh, max_len, hd)).astype(np.float32)
    mask = np.zeros((S, total), np.float32)
    got = oracle.gqa_attention(q, k, v, mask).reshape(H, hd)
    g = H // kvh
    for h in range(H):
        s = (k[h // g, :total].astype(np.float64) @ q[0, h].astype(np.float64)) / math.sqrt(hd)
        p = np.exp(s - s.max())
        p /= p.sum()
        want = p @ v[h // g, :total].astype(np.float64)
        assert np.allclose(got[h], want, atol=1e-5)
    # one overwhelming score selects that V row
    k2 = np.zeros_like(k)
    k2[:, 11, :] = 50.0 * np.sign(q[0, 0])  # aligned with head 0's query
    out = oracle.gqa_attention(q[:, :1].repeat(H, 1), k2, v, mask).reshape(H, hd)
    assert np.allclose(out[0], v[0, 11], atol=1e-4)
    # rows beyond `total` must not be read as attended
    k3, v3 = k.copy(), v.copy()
    k3[:, total:] = 1e6
    v3[:, total:] = 1e6
    assert np.array_equal(oracle.gqa_attention(q, k3, v3, mask), oracle.gqa_attention(q, k, v, mask))
    # multi-token causal: first of 2 new rows must not see the last column
    q2 = rng.standard_normal((2, H, hd)).astype(np.float32)
    m2 = oracle.causal_mask(2, total - 2)
    full = oracle.gqa_attention(q2, k, v, m2)
    first_only = oracle.gqa_attention(q2[:1], k, v, np.zeros((1, total - 1), np.float32))
    assert np.allclose(full[0], first_only[0], atol=1e-6)


# ── KV cache ──────────────────────────────────────────────────────────────────

def test_kv_cache_reference_arrays(oracle, golden):
    g = golden["kv_cache_append_and_view"]
    c = oracle.KvCache(g["layers"], g["heads"], g["max_len"], g["head_dim"])
    shape = (1, g["heads"], 1, g["head_dim"])
    for k, v in ((g["k0"], g["v0"]), (g["k1"], g["v1"])):
        assert c.append_key(0, np.array(k, np.float32).reshape(shape)) == 0
        assert c.append_value(0, np.array(v, np.float32).reshape(shape)) == 0
        c.advance_by(1)
    kv, vv = c.view(0)
    assert kv.shape == (1, 2, 2, 3)
    assert np.array_equal(kv.reshape(-1), np.array(g["view_k_after_2"], np.float32))
    assert np.array_equal(vv.reshape(-1), np.array(g["view_v_after_2"], np.float32))


def test_kv_cache_multi_token_and_overflow(oracle, golden):
    g = golden["kv_cache_multi_token_append"]
    c = oracle.KvCache(g["layers"], g["heads"], g["max_len"], g["head_dim"])
    c.append_key(0, np.array(g["k3"], np.float32).reshape(1, 2, 3, 3))
    c.append_value(0, np.array(g["v3"], np.float32).reshape(1, 2, 3, 3))
    c.advance_by(3)
    assert c.current_len() == 3
    c.append_key(0, np.array(g["k1"], np.float32).reshape(1, 2, 1, 3))
    c.append_value(0, np.array(g["v1"], np.float32).reshape(1, 2, 1, 3))
    c.advance_by(1)
    kv, _ = c.view(0)
    assert np.array_equal(kv.reshape(-1), np.array(g["view_k_after_4"], np.float32))
    # the reference panics "KV cache full"; the oracle reports it
    assert c.append_key(0, np.zeros((1, 2, 5, 3), np.float32)) != 0
    c.reset(0)
    assert c.current_len() == 0


def test_config_vectors(golden):
    from homura_amd import TransformerConfig
    g = golden["qwen3_config"]
    cfg = TransformerConfig(hidden_size=g["hidden_size"], intermediate_size=g["intermediate_size"],
                            num_attention_heads=g["num_attention_heads"],
                            num_hidden_layers=g["num_hidden_layers"], vocab_size=g["vocab_size"],
                            num_key_value_heads=g["num_key_value_heads"], head_dim=g["head_dim"])
    assert (cfg.kv_heads(), cfg.get_head_dim(), cfg.gqa_repeat()) == (8, 128, 2)
    assert cfg.num_attention_heads * cfg.get_head_dim() == g["expect_q_dim"]
    assert cfg.rms_norm_eps == 1e-6 and cfg.max_position_embeddings == 2048  # reference defaults
    g2 = golden["qwen2_config"]
    cfg2 = TransformerConfig(hidden_size=896, intermediate_size=4864, num_attention_heads=14,
                             num_hidden_layers=24, vocab_size=151936, num_key_value_heads=2)
    assert (cfg2.kv_heads(), cfg2.get_head_dim(), cfg2.gqa_repeat()) == (2, 64, 7)
    assert g2["expect_gqa_repeat"] == 7
