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


# ── K-quants: Q4_K, Q6_K (reference src/gguf.rs:835-917, src/graph_builder/emit_quant.rs:165-816) ──

def _np_dequant_q4_k(raw):
    """Independent decode of ggml block_q4_K written from the format description: 8 sub-blocks of
    32; sub-block j of a super-block takes the low (j even) or high (j odd) nibbles of the 32 bytes
    at qs[32*(j//2)]; 6-bit scale/min j come from the 12 packed bytes."""
    blocks = raw.reshape(-1, 144)
    out = np.empty((len(blocks), 256), np.float64)
    for b, blk in enumerate(blocks):
        d, dmin = (float(x) for x in blk[0:4].view(np.float16))
        p = blk[4:16].astype(int)
        for j in range(8):
            if j < 4:
                sc, mn = p[j] & 63, p[j + 4] & 63
            else:
                sc = (p[j + 4] & 15) | ((p[j - 4] >> 6) << 4)
                mn = (p[j + 4] >> 4) | ((p[j] >> 6) << 4)
            q = blk[16 + 32 * (j // 2): 16 + 32 * (j // 2) + 32].astype(int)
            nib = (q >> 4) if j % 2 else (q & 15)
            out[b, 32 * j: 32 * j + 32] = d * sc * nib - dmin * mn
    return out.reshape(-1)


def _np_dequant_q6_k(raw):
    """Independent decode of ggml block_q6_K: element e of a super-block lives in half h = e // 128,
    quarter g = (e % 128) // 32, position l = e % 32: low nibble from ql[64 h + 32 (g % 2) + l]
    (upper nibble when g >= 2), bit pair g of qh[32 h + l], scale sc[8 h + 2 g + l // 16]."""
    blocks = raw.reshape(-1, 210)
    out = np.empty((len(blocks), 256), np.float64)
    for b, blk in enumerate(blocks):
        d = float(blk[208:210].view(np.float16)[0])
        ql, qh, sc = blk[0:128].astype(int), blk[128:192].astype(int), blk[192:208].view(np.int8).astype(int)
        for e in range(256):
            h, g, l = e // 128, (e % 128) // 32, e % 32
            lo = ql[64 * h + 32 * (g % 2) + l]
            lo = (lo >> 4) if g >= 2 else (lo & 15)
            hi = (qh[32 * h + l] >> (2 * g)) & 3
            out[b, e] = d * sc[8 * h + 2 * g + l // 16] * ((lo | (hi << 4)) - 32)
    return out.reshape(-1)


def _q4k_kat_block():
    """The block of the reference's emit_q4_k_correctness (src/graph_builder/emit_quant.rs:1018-1078):
    d = 1.0, dmin = 0, scales_raw[0..3] = 1, every nibble 1."""
    blk = np.zeros(144, np.uint8)
    blk[0:2] = (0x00, 0x3C)
    blk[4:8] = 1
    blk[16:144] = 0x11
    return blk


def test_q4_k_reference_kat(oracle):
    w = np.tile(_q4k_kat_block(), 4)
    out = oracle.gemv_q4_k(np.ones(256, np.float32), w, 1, 256, 4)
    assert np.allclose(out, 128.0, atol=1e-3)          # reference asserts |out - 128| < 1
    deq = oracle.dequant_q4_k(w)[:256]
    assert np.array_equal(deq[:128], np.ones(128, np.float32)) and not deq[128:].any()


def test_q6_k_reference_kat(oracle):
    """emit_q6_k_correctness (src/graph_builder/emit_quant.rs:1286-1360): d = 1, sc = 1, low nibbles 1,
    high bits 0 -> every weight -31, 256 * -31 = -7936."""
    blk = np.zeros(210, np.uint8)
    blk[208:210] = (0x00, 0x3C)
    blk[192:208] = 1
    blk[0:128] = 0x11
    w = np.tile(blk, 4)
    out = oracle.gemv_q6_k(np.ones(256, np.float32), w, 1, 256, 4)
    assert np.allclose(out, -7936.0, atol=1e-2)
    assert np.array_equal(oracle.dequant_q6_k(w), np.full(1024, -31.0, np.float32))


def test_q4_k_reference_realistic_case(oracle):
    """emit_q4_k_correctness_realistic (src/graph_builder/emit_quant.rs:1105-1224): d = 0.5,
    dmin = 0.25, sc = 5/10/15/20, mn = 2/4/6/8, patterned nibbles, activation all ones; the kernel
    must equal the row sum of the dequantised weights (the reference allows 1 % or 0.1)."""
    rows = []
    for b in range(2):
        blk = np.zeros(144, np.uint8)
        blk[0:4] = (0x00, 0x38, 0x00, 0x34)
        blk[4:12] = (5, 10, 15, 20, 2, 4, 6, 8)
        qi = np.arange(128)
        blk[16:144] = ((qi * 3 + b * 7) % 16) | (((qi * 5 + b * 11) % 16) << 4)
        rows.append(blk)
    w = np.concatenate(rows)
    out = oracle.gemv_q4_k(np.ones(256, np.float32), w, 1, 256, 2)[0]
    ref = _np_dequant_q4_k(w).reshape(2, 256).sum(1)
    assert np.all(np.abs(out - ref) < np.maximum(0.01 * np.abs(ref), 0.1))
    # with an activation of ones the Q8_K quantisation is exact (every q8 = 127): equality to rounding
    assert np.allclose(out, ref, rtol=1e-6)


def test_kquant_dequant_against_independent_decode(oracle):
    from homura_amd import synth
    w4 = synth.q4_k_blocks(11, 37)
    assert np.allclose(oracle.dequant_q4_k(w4), _np_dequant_q4_k(w4), rtol=1e-6, atol=1e-9)
    w6 = synth.q6_k_blocks(12, 29)
    assert np.allclose(oracle.dequant_q6_k(w6), _np_dequant_q6_k(w6), rtol=1e-6, atol=1e-9)


def test_q8_k_activation_quantisation(oracle):
    """amax/127 scale, round half to even, clamp, sums of 16 (emit_quant.rs:422-466)."""
    x = np.zeros(256, np.float32)
    q, d, bs = oracle.quantize_q8_k(x)
    assert d == 0.0 and not q.any() and not bs.any()          # iscale = 0 for an all-zero block
    x[0] = 127.0                                               # iscale = 1: values map to themselves
    x[1:6] = (0.5, 1.5, 2.5, -0.5, -3.5)
    x[16:20] = (100.0, -127.0, 126.49, 3.0)
    q, d, bs = oracle.quantize_q8_k(x)
    assert d == 1.0
    assert q[:6].tolist() == [127, 0, 2, 2, 0, -4]             # ties go to the even neighbour
    assert q[16:20].tolist() == [100, -127, 126, 3]
    assert bs[0] == int(q[:16].astype(int).sum()) and bs[1] == 102 and not bs[2:].any()
    rng = np.random.default_rng(5)
    x = rng.standard_normal(256).astype(np.float32)
    q, d, bs = oracle.quantize_q8_k(x)
    assert np.abs(q).max() == 127 and np.abs(q.astype(np.float64) * d - x).max() <= d / 2 + 1e-7
    assert np.array_equal(bs, q.astype(np.int32).reshape(16, 16).sum(1))


@pytest.mark.parametrize("kind", ["q4_k", "q6_k"])
def test_kquant_gemv_against_dequantised_product(oracle, kind):
    """What the reference's real-weight tests check (emit_quant.rs:1363-1500): the integer-dot kernel
    agrees with dequantise-then-multiply up to the Q8_K rounding of the activation. A wrong sub-block
    order, nibble half or scale index would be off by O(1), not by a fraction of a percent."""
    from homura_amd import synth
    K, N = 512, 24
    w = (synth.q4_k_blocks if kind == "q4_k" else synth.q6_k_blocks)(21, N * K // 256)
    x = np.random.default_rng(3).standard_normal((2, K)).astype(np.float32)
    got = (oracle.gemv_q4_k if kind == "q4_k" else oracle.gemv_q6_k)(x, w, 2, K, N)
    deq = (_np_dequant_q4_k if kind == "q4_k" else _np_dequant_q6_k)(w).reshape(N, K)
    want = x.astype(np.float64) @ deq.T
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < 1e-2, err
    # and exactly: the same integers through numpy int64 arithmetic and one float per block
    xq = [[oracle.quantize_q8_k(x[m, kb * 256:(kb + 1) * 256]) for kb in range(K // 256)] for m in range(2)]
    xdq = np.array([np.concatenate([q.astype(np.float64) * d for q, d, _ in row]) for row in xq])
    exact = xdq @ deq.T
    assert np.abs(got - exact).max() / np.abs(exact).max() < 1e-5
