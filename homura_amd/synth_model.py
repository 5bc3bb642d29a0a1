"""Random-init decoder models of a given shape (seeded, reproducible) for tests and benchmarks.

Weights come out in the order and layouts of the reference's TransformerWeights::to_slot_buffers
(reference src/hf/weights.rs:63-116): f32 embedding table [vocab, hidden], f32 norm vectors,
bf16 projections transposed to [in, out], tied LM head = transposed embedding in bf16.
"""
from __future__ import annotations

import numpy as np

from . import synth
from .runtime import (DTYPE_BF16, DTYPE_Q4_0, DTYPE_Q4_K, DTYPE_Q6_K, DTYPE_Q8_0, Context, HfModel,
                      TransformerConfig)

# Qwen3-0.6B shape (reference src/hf/config.rs:125-150): the decode benchmark configuration
QWEN3_0P6B = TransformerConfig(
    hidden_size=1024, intermediate_size=3072, num_attention_heads=16, num_hidden_layers=28,
    vocab_size=151936, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6,
    max_position_embeddings=2048, tie_word_embeddings=True)

# a few-megabyte model with the same structure (GQA 2:1, QK-norm, tied head) for quick checks
TINY = TransformerConfig(
    hidden_size=256, intermediate_size=512, num_attention_heads=4, num_hidden_layers=3,
    vocab_size=1000, num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-6, rope_theta=1e6,
    max_position_embeddings=512, tie_word_embeddings=True)

# the small shape the whole-step decode launch has an instance for (same structure as Qwen3-0.6B)
SMALL_WS = TransformerConfig(
    hidden_size=512, intermediate_size=1024, num_attention_heads=4, num_hidden_layers=3,
    vocab_size=1000, num_key_value_heads=2, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6,
    max_position_embeddings=2048, tie_word_embeddings=True)

# the small shape the whole-step decode launch serves in Q8_0 / Q4_0 (widths that are multiples of 1024)
SMALL_WS_Q = TransformerConfig(
    hidden_size=1024, intermediate_size=1024, num_attention_heads=8, num_hidden_layers=3,
    vocab_size=1000, num_key_value_heads=4, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6,
    max_position_embeddings=1024, tie_word_embeddings=False)

# Qwen2.5-like: Q/K/V biases, no QK-norm, GQA 7:1 as in Qwen2.5-0.5B (14 q heads, 2 kv heads)
TINY_QWEN2 = TransformerConfig(
    hidden_size=448, intermediate_size=608, num_attention_heads=7, num_hidden_layers=2,
    vocab_size=512, num_key_value_heads=1, head_dim=64, rms_norm_eps=1e-6, rope_theta=1e6,
    max_position_embeddings=512, tie_word_embeddings=True, attention_bias=True)

# TinyLlama-like proportions (MHA:GQA 4:1, no QK-norm, untied head) for the quantised plan
TINY_LLAMA = TransformerConfig(
    hidden_size=256, intermediate_size=704, num_attention_heads=8, num_hidden_layers=2,
    vocab_size=640, num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-5, rope_theta=1e4,
    max_position_embeddings=512, tie_word_embeddings=False)


# The widths of the other models the reference lists with decode figures (README "Performance"): these run
# one launch per projection. `layers` cuts the depth for tests; vocabularies as the checkpoints have them.
def listed_shape(name: str, layers: int | None = None, vocab: int | None = None) -> TransformerConfig:
    shapes = {
        "qwen2.5-0.5b": dict(hidden_size=896, intermediate_size=4864, num_attention_heads=14, num_hidden_layers=24,
                             vocab_size=151936, num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-6, rope_theta=1e6,
                             tie_word_embeddings=True, attention_bias=True),
        "tinyllama-1.1b": dict(hidden_size=2048, intermediate_size=5632, num_attention_heads=32, num_hidden_layers=22,
                               vocab_size=32000, num_key_value_heads=4, head_dim=64, rms_norm_eps=1e-5, rope_theta=1e4,
                               tie_word_embeddings=False),
        "qwen2.5-1.5b": dict(hidden_size=1536, intermediate_size=8960, num_attention_heads=12, num_hidden_layers=28,
                             vocab_size=151936, num_key_value_heads=2, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6,
                             tie_word_embeddings=True, attention_bias=True),
        "smollm2-1.7b": dict(hidden_size=2048, intermediate_size=8192, num_attention_heads=32, num_hidden_layers=24,
                             vocab_size=49152, num_key_value_heads=32, head_dim=64, rms_norm_eps=1e-5, rope_theta=1.3e5,
                             tie_word_embeddings=True),
    }
    d = dict(shapes[name], max_position_embeddings=2048)
    if layers is not None:
        d["num_hidden_layers"] = layers
    if vocab is not None:
        d["vocab_size"] = vocab
    return TransformerConfig(**d)


# K-quant proportions (every projection input a multiple of 256) for Q4_K / Q6_K files
TINY_K = TransformerConfig(
    hidden_size=512, intermediate_size=768, num_attention_heads=8, num_hidden_layers=2,
    vocab_size=640, num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-5, rope_theta=1e4,
    max_position_embeddings=512, tie_word_embeddings=False)


def q4_k_m_mix(cfg: TransformerConfig):
    """Per-projection types in the manner of llama.cpp's Q4_K_M files: Q4_K throughout, attn_v and
    ffn_down in Q6_K for part of the layers (here: the even ones). 7 per layer: q k v o gate up down."""
    out = []
    for l in range(cfg.num_hidden_layers):
        hi = DTYPE_Q6_K if l % 2 == 0 else DTYPE_Q4_K
        out += [DTYPE_Q4_K, DTYPE_Q4_K, hi, DTYPE_Q4_K, DTYPE_Q4_K, DTYPE_Q4_K, hi]
    return out


def synth_weights(cfg: TransformerConfig, seed: int, weight_dtype: int = DTYPE_BF16,
                  has_qk_norm: bool = True, proj_dtypes=None):
    """[(name, array)] in slot order. Projections: bf16 bits [K, N], or raw GGUF blocks
    [N][K/block] for Q8_0 / Q4_0 / Q4_K / Q6_K (then the LM head is f32 [hidden, vocab], as in the
    reference's quantised plan, src/hf/weights.rs:174-180). proj_dtypes: 7 types per layer
    (q k v o gate up down) instead of one weight_dtype."""
    hidden, inter, vocab = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    hd = cfg.get_head_dim()
    qd, kvd = cfg.num_attention_heads * hd, cfg.kv_heads() * hd
    cursor = [0]

    def normal_bits(n, scale):
        a = synth.normal_bf16(seed, n, scale, first=cursor[0])
        cursor[0] += n
        return a

    def norm_vec(n):
        a = synth.normal_f32(seed ^ 0x5EED, n, 0.1, first=cursor[0])
        cursor[0] += n
        return (1.0 + a).astype(np.float32)

    def bias_vec(n):
        a = synth.normal_f32(seed ^ 0xB1A5, n, 0.5, first=cursor[0])
        cursor[0] += n
        return a.astype(np.float32)

    qseed = [seed * 7919 + 1]

    pidx = [0]

    def proj(K, N):
        dt = weight_dtype
        if proj_dtypes is not None:
            dt = proj_dtypes[pidx[0]]
            pidx[0] += 1
        if dt == DTYPE_BF16:
            return normal_bits(K * N, 0.02).reshape(K, N)
        qseed[0] += 1
        if dt == DTYPE_Q4_K:    # w = d*sc*q - dmin*m with sc, m < 64 and q < 16
            return synth.q4_k_blocks(qseed[0], N * (K // 256), 0.02 / 260.0)
        if dt == DTYPE_Q6_K:    # w = d*sc*q with |sc| < 128 and |q| <= 32
            return synth.q6_k_blocks(qseed[0], N * (K // 256), 0.02 / 1400.0)
        nb = N * (K // 32)
        if dt == DTYPE_Q8_0:   # w = q * d with q in [-127,127]: d ~ 0.02 / 73
            return synth.q8_0_blocks(qseed[0], nb, 0.02 / 73.0 * 1.25)
        return synth.q4_0_blocks(qseed[0], nb, 0.02 / 4.6 * 1.25)

    out = []
    embed_bits = normal_bits(vocab * hidden, 0.02).reshape(vocab, hidden)
    out.append(("model.embed_tokens.weight", synth.bf16_to_f32(embed_bits)))
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        out.append((p + "input_layernorm.weight", norm_vec(hidden)))
        out.append((p + "self_attn.q_proj.weight", proj(hidden, qd)))
        if cfg.attention_bias:
            out.append((p + "self_attn.q_proj.bias", bias_vec(qd)))
        out.append((p + "self_attn.k_proj.weight", proj(hidden, kvd)))
        if cfg.attention_bias:
            out.append((p + "self_attn.k_proj.bias", bias_vec(kvd)))
        out.append((p + "self_attn.v_proj.weight", proj(hidden, kvd)))
        if cfg.attention_bias:
            out.append((p + "self_attn.v_proj.bias", bias_vec(kvd)))
        if has_qk_norm:
            out.append((p + "self_attn.q_norm.weight", norm_vec(hd)))
            out.append((p + "self_attn.k_norm.weight", norm_vec(hd)))
        out.append((p + "self_attn.o_proj.weight", proj(qd, hidden)))
        out.append((p + "post_attention_layernorm.weight", norm_vec(hidden)))
        out.append((p + "mlp.gate_proj.weight", proj(hidden, inter)))
        out.append((p + "mlp.up_proj.weight", proj(hidden, inter)))
        out.append((p + "mlp.down_proj.weight", proj(inter, hidden)))
    out.append(("model.norm.weight", norm_vec(hidden)))
    if cfg.tie_word_embeddings:
        head_bits = np.ascontiguousarray(embed_bits.T)          # [hidden, vocab]
    else:
        head_bits = normal_bits(hidden * vocab, 0.02).reshape(hidden, vocab)
    if weight_dtype == DTYPE_BF16 and proj_dtypes is None:
        out.append(("lm_head.weight", head_bits))
    else:
        out.append(("lm_head.weight", synth.bf16_to_f32(head_bits)))
    return out


def synth_kv(cfg: TransformerConfig, seed: int, seq_len: int):
    """2*layers arrays (K, V alternating) of f32 [1, kv_heads, seq_len, head_dim] holding
    bf16-representable N(0,1) values: a cache "as if" seq_len tokens had been processed."""
    n = cfg.kv_heads() * seq_len * cfg.get_head_dim()
    out = []
    for i in range(2 * cfg.num_hidden_layers):
        bits = synth.normal_bf16(seed, n, 1.0, first=i * n)
        out.append(synth.bf16_to_f32(bits).reshape(1, cfg.kv_heads(), seq_len, cfg.get_head_dim()))
    return out


def build_model(ctx: Context, cfg: TransformerConfig, weights, max_seq_len: int,
                weight_dtype: int = DTYPE_BF16, has_qk_norm: bool = True, proj_dtypes=None) -> HfModel:
    m = HfModel(ctx, cfg, weight_dtype, has_qk_norm, proj_dtypes=proj_dtypes)
    slots = m.weight_slots()
    if len(slots) != len(weights):
        raise ValueError(f"model lists {len(slots)} weight slots, got {len(weights)} arrays")
    for i, ((name, arr), (sname, _dt, _d0, _d1, nbytes)) in enumerate(zip(weights, slots)):
        if name != sname or arr.nbytes != nbytes:
            raise ValueError(f"slot {i}: have {name} ({arr.nbytes} B), model expects {sname} ({nbytes} B)")
        m.set_weight(i, arr)
    m.finalize(max_seq_len)
    return m
