"""Whole models loaded from checkpoint files (GGUF; config.json + safetensors, single and sharded)
straight into HBM and checked against the oracle fed with the same arrays
(reference HfModel::load, src/hf/model.rs:75-146; GgufFile::load_transformer_weights,
src/gguf.rs:589-708)."""
from __future__ import annotations

import json

import numpy as np
import pytest

import ckpt_writers as cw
import model_fixture as mf
import pyoracle
from homura_amd import HfModel, checkpoints as ck, synth, synth_model
from homura_amd.runtime import DTYPE_BF16, DTYPE_Q4_0, DTYPE_Q4_K, DTYPE_Q6_K, DTYPE_Q8_0, HomuraError

pytestmark = pytest.mark.gpu

GGUF_NAMES = {
    "input_layernorm.weight": "attn_norm.weight", "self_attn.q_proj.weight": "attn_q.weight",
    "self_attn.q_proj.bias": "attn_q.bias", "self_attn.k_proj.weight": "attn_k.weight",
    "self_attn.k_proj.bias": "attn_k.bias", "self_attn.v_proj.weight": "attn_v.weight",
    "self_attn.v_proj.bias": "attn_v.bias", "self_attn.q_norm.weight": "attn_q_norm.weight",
    "self_attn.k_norm.weight": "attn_k_norm.weight", "self_attn.o_proj.weight": "attn_output.weight",
    "post_attention_layernorm.weight": "ffn_norm.weight", "mlp.gate_proj.weight": "ffn_gate.weight",
    "mlp.up_proj.weight": "ffn_up.weight", "mlp.down_proj.weight": "ffn_down.weight"}


def say(msg):
    print(f"[checkpoints] {msg}", flush=True)


def gguf_name(hf: str) -> str:
    if hf == "model.embed_tokens.weight":
        return "token_embd.weight"
    if hf == "model.norm.weight":
        return "output_norm.weight"
    if hf == "lm_head.weight":
        return "output.weight"
    _m, _l, layer, rest = hf.split(".", 3)
    return f"blk.{layer}.{GGUF_NAMES[rest]}"


def gguf_metadata(cfg, arch):
    md = [("general.architecture", cw.STRING, arch), ("general.name", cw.STRING, "synthetic"),
          (f"{arch}.embedding_length", cw.U32, cfg.hidden_size),
          (f"{arch}.feed_forward_length", cw.U32, cfg.intermediate_size),
          (f"{arch}.attention.head_count", cw.U32, cfg.num_attention_heads),
          (f"{arch}.attention.head_count_kv", cw.U32, cfg.kv_heads()),
          (f"{arch}.block_count", cw.U32, cfg.num_hidden_layers),
          (f"{arch}.attention.layer_norm_rms_epsilon", cw.F32, cfg.rms_norm_eps),
          (f"{arch}.rope.freq_base", cw.F32, cfg.rope_theta),
          (f"{arch}.context_length", cw.U32, cfg.max_position_embeddings),
          (f"{arch}.attention.key_length", cw.U32, cfg.get_head_dim()),
          ("tokenizer.ggml.tokens", cw.ARRAY, (cw.STRING, [f"t{i}" for i in range(cfg.vocab_size)]))]
    return md


def check_against_oracle(gm, om, cfg, tag):
    kv = synth_model.synth_kv(cfg, 8, 19)
    gm.init_kv_cache(kv, 19)
    mf.oracle_init_kv(om, kv)
    ids = synth.token_ids(2, 4, cfg.vocab_size)
    got = gm.run_kv(ids)
    want = np.concatenate([om.run_kv(ids[i:i + 1]) for i in range(4)])
    for i in range(4):
        assert mf.rel_err(got[i], want[i]) < 1e-2, f"{tag} position {i}"
    want_t, margins = om.generate_greedy(ids[:2], 16)
    say(f"{tag}: min margin {margins.min():.3e}")
    assert np.array_equal(gm.generate_greedy(ids[:2], 16), want_t)


@pytest.mark.parametrize("wdt,code,name", [(DTYPE_Q8_0, ck.GGML_Q8_0, "q8_0"), (DTYPE_Q4_0, ck.GGML_Q4_0, "q4_0")])
def test_load_quantised_gguf(ctx, tmp_path, wdt, code, name):
    """Llama-style file: raw quantised projections, f32 norms, a Q8_0 token embedding (dequantised on
    load, src/gguf.rs:759-764) and an untied f32 output matrix."""
    cfg = synth_model.TINY_LLAMA
    weights = synth_model.synth_weights(cfg, 41, wdt, has_qk_norm=False)
    emb_blocks = synth.q8_0_blocks(977, cfg.vocab_size * cfg.hidden_size // 32, 0.02 / 73.0)
    emb = pyoracle.dequant_q8_0(emb_blocks)
    weights = [(n, emb.reshape(cfg.vocab_size, cfg.hidden_size) if n == "model.embed_tokens.weight" else a)
               for n, a in weights]
    tensors = []
    for n, a in weights:
        if n == "model.embed_tokens.weight":
            tensors.append((gguf_name(n), a.shape, ck.GGML_Q8_0, emb_blocks.tobytes()))
        elif n.endswith("_proj.weight"):
            K = {"q": cfg.hidden_size, "k": cfg.hidden_size, "v": cfg.hidden_size, "o": cfg.num_attention_heads * cfg.get_head_dim(),
                 "gate": cfg.hidden_size, "up": cfg.hidden_size, "down": cfg.intermediate_size}[n.split(".")[-2].split("_")[0]]
            N = a.size // (K // 32) // (34 if wdt == DTYPE_Q8_0 else 18)
            tensors.append((gguf_name(n), (N, K), code, a.tobytes()))
        elif n == "lm_head.weight":                      # f32 [hidden, vocab] -> file keeps [vocab, hidden]
            tensors.append((gguf_name(n), (cfg.vocab_size, cfg.hidden_size), ck.GGML_F32, np.ascontiguousarray(a.T).tobytes()))
        else:
            tensors.append((gguf_name(n), a.shape, ck.GGML_F32, a.tobytes()))
    path = tmp_path / f"tiny-{name}.gguf"
    path.write_bytes(cw.gguf_bytes(gguf_metadata(cfg, "llama"), tensors))
    gm = HfModel.load_gguf(ctx, path, 96)
    assert gm.weight_dtype == wdt and gm.has_qk_norm is False and gm.config.tie_word_embeddings is False
    assert gm.config.vocab_size == cfg.vocab_size and gm.config.kv_heads() == cfg.kv_heads()
    om = mf.build_oracle_model(cfg, weights, 96, wdt, has_qk_norm=False)
    check_against_oracle(gm, om, cfg, f"gguf {name}")
    gm.close()


def test_load_q4_k_m_style_gguf(ctx, tmp_path):
    """A file quantised the way llama.cpp's Q4_K_M recipe does it: projections in Q4_K with attn_v and
    ffn_down of some layers in Q6_K, the token embedding in Q4_K and the output matrix in Q6_K (both
    dequantised on load, src/gguf.rs:759-764), f32 norms."""
    cfg = synth_model.TINY_K
    mix = synth_model.q4_k_m_mix(cfg)
    weights = synth_model.synth_weights(cfg, 43, has_qk_norm=False, proj_dtypes=mix)
    V, Hd = cfg.vocab_size, cfg.hidden_size
    emb_blocks = synth.q4_k_blocks(811, V * Hd // 256, 0.02 / 260.0)
    head_blocks = synth.q6_k_blocks(812, V * Hd // 256, 0.02 / 1400.0)
    emb = pyoracle.dequant_q4_k(emb_blocks).reshape(V, Hd)
    head = np.ascontiguousarray(pyoracle.dequant_q6_k(head_blocks).reshape(V, Hd).T)   # slot layout [hidden, vocab]
    weights = [(n, emb if n == "model.embed_tokens.weight" else head if n == "lm_head.weight" else a)
               for n, a in weights]
    code = {DTYPE_Q4_K: ck.GGML_Q4_K, DTYPE_Q6_K: ck.GGML_Q6_K}
    bb = {DTYPE_Q4_K: 144, DTYPE_Q6_K: 210}
    tensors, pi = [], 0
    for n, a in weights:
        if n == "model.embed_tokens.weight":
            tensors.append((gguf_name(n), (V, Hd), ck.GGML_Q4_K, emb_blocks.tobytes()))
        elif n == "lm_head.weight":
            tensors.append((gguf_name(n), (V, Hd), ck.GGML_Q6_K, head_blocks.tobytes()))
        elif n.endswith("_proj.weight"):
            K = {"q": Hd, "k": Hd, "v": Hd, "o": cfg.num_attention_heads * cfg.get_head_dim(), "gate": Hd, "up": Hd,
                 "down": cfg.intermediate_size}[n.split(".")[-2].split("_")[0]]
            dt = mix[pi]
            pi += 1
            tensors.append((gguf_name(n), (a.size // (K // 256) // bb[dt], K), code[dt], a.tobytes()))
        else:
            tensors.append((gguf_name(n), a.shape, ck.GGML_F32, a.tobytes()))
    path = tmp_path / "tiny-q4_k_m.gguf"
    path.write_bytes(cw.gguf_bytes(gguf_metadata(cfg, "llama"), tensors))
    gm = HfModel.load_gguf(ctx, path, 96)
    assert gm.weight_dtype == DTYPE_Q4_K and gm.has_qk_norm is False and gm.config.tie_word_embeddings is False
    slot_types = [s[1] for s in gm.weight_slots() if s[0].endswith("_proj.weight")]
    assert slot_types == mix
    om = mf.build_oracle_model(cfg, weights, 96, has_qk_norm=False, proj_dtypes=mix)
    check_against_oracle(gm, om, cfg, "gguf q4_k_m")
    gm.close()


def test_load_bf16_gguf_tied_qknorm(ctx, tmp_path):
    """Qwen3-style file with unquantised projections: BF16 tensors as they are, the F32 ones cut to
    their top 16 bits (reference f32_buf_to_bf16), tied head, QK-norm."""
    cfg = synth_model.TINY
    weights = synth_model.synth_weights(cfg, 52)
    tensors = []
    for i, (n, a) in enumerate(weights):
        if n == "lm_head.weight":
            continue                                     # tied: no output.weight in the file
        if n.endswith("_proj.weight"):                   # bf16 bits [K, N] -> file keeps [N, K]
            t = np.ascontiguousarray(a.T)
            if i % 2:                                    # every other projection as F32 with junk low bits
                f = (t.astype(np.uint32) << 16) | 0x1234
                tensors.append((gguf_name(n), t.shape, ck.GGML_F32, f.astype(np.uint32).tobytes()))
            else:
                tensors.append((gguf_name(n), t.shape, ck.GGML_BF16, t.tobytes()))
        elif n == "model.embed_tokens.weight":
            tensors.append((gguf_name(n), a.shape, ck.GGML_BF16, cw.f32_to_bf16_trunc(a).tobytes()))
        else:
            tensors.append((gguf_name(n), a.shape, ck.GGML_F32, a.tobytes()))
    path = tmp_path / "tiny-bf16.gguf"
    path.write_bytes(cw.gguf_bytes(gguf_metadata(cfg, "qwen3"), tensors))
    gm = HfModel.load_gguf(ctx, path, 96)
    assert gm.weight_dtype == DTYPE_BF16 and gm.has_qk_norm is True and gm.config.tie_word_embeddings is True
    check_against_oracle(gm, mf.build_oracle_model(cfg, weights, 96), cfg, "gguf bf16")
    gm.close()


def hf_tensors(cfg, weights):
    """HF names and orientation: linear weights [out, in] in BF16, the embedding in BF16, norms and
    biases in F32."""
    out = {}
    for n, a in weights:
        if n == "lm_head.weight" and cfg.tie_word_embeddings:
            continue
        if n.endswith("_proj.weight") or n == "lm_head.weight":
            t = np.ascontiguousarray(a.T)
            out[n] = ("BF16", t.shape, t.tobytes())
        elif n == "model.embed_tokens.weight":
            out[n] = ("BF16", a.shape, cw.f32_to_bf16_trunc(a).tobytes())
        else:
            out[n] = ("F32", a.shape, a.tobytes())
    return out


def write_config(cfg, d):
    c = {"architectures": ["Qwen2ForCausalLM"], "hidden_size": cfg.hidden_size,
         "intermediate_size": cfg.intermediate_size, "num_attention_heads": cfg.num_attention_heads,
         "num_hidden_layers": cfg.num_hidden_layers, "num_key_value_heads": cfg.kv_heads(),
         "vocab_size": cfg.vocab_size, "rms_norm_eps": cfg.rms_norm_eps, "rope_theta": cfg.rope_theta,
         "max_position_embeddings": cfg.max_position_embeddings,
         "tie_word_embeddings": cfg.tie_word_embeddings, "head_dim": cfg.get_head_dim(), "torch_dtype": "bfloat16"}
    (d / "config.json").write_text(json.dumps(c, indent=2))


@pytest.mark.parametrize("sharded", [False, True])
def test_load_hf_directory(ctx, tmp_path, sharded):
    """config.json + model.safetensors, or an index and two shards (src/hf/model.rs:86-123); a
    Qwen2-style checkpoint with Q/K/V biases and a tied head."""
    cfg = synth_model.TINY_QWEN2
    weights = synth_model.synth_weights(cfg, 63, has_qk_norm=False)
    tensors = hf_tensors(cfg, weights)
    write_config(cfg, tmp_path)
    if sharded:
        names = list(tensors)
        parts = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
        for fname, keys in parts.items():
            (tmp_path / fname).write_bytes(cw.safetensors_bytes({k: tensors[k] for k in keys}, {"format": "pt"}))
        index = {"metadata": {"total_size": 0}, "weight_map": {k: f for f, keys in parts.items() for k in keys}}
        (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    else:
        (tmp_path / "model.safetensors").write_bytes(cw.safetensors_bytes(tensors, {"format": "pt"}))
    gm = HfModel.load_hf_dir(ctx, tmp_path, 96)
    assert gm.config.attention_bias is True and gm.has_qk_norm is False and gm.weight_dtype == DTYPE_BF16
    om = mf.build_oracle_model(cfg, weights, 96, has_qk_norm=False)
    check_against_oracle(gm, om, cfg, "safetensors sharded" if sharded else "safetensors")
    gm.close()


def test_loader_errors_are_reported(ctx, tmp_path):
    cfg = synth_model.TINY_LLAMA
    with pytest.raises(HomuraError, match="No such file"):
        HfModel.load_gguf(ctx, tmp_path / "absent.gguf")
    # a Q5_K projection: understood by the parser, refused by the loader with the reason
    t = [("blk.0.attn_q.weight", (256, 256), ck.GGML_Q5_K, bytes(256 * 176))]
    p = tmp_path / "q5k.gguf"
    p.write_bytes(cw.gguf_bytes(gguf_metadata(cfg, "llama"), t))
    with pytest.raises(HomuraError, match="blk.0.attn_q.weight is Q5_K"):
        HfModel.load_gguf(ctx, p)
    # float and block-quantised projections in one file
    t = [(f"blk.{l}.{n}.weight", (32, 32), ck.GGML_Q8_0 if n == "attn_k" else ck.GGML_F32, bytes(32 * (34 if n == "attn_k" else 128)))
         for l in range(cfg.num_hidden_layers) for n in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")]
    p = tmp_path / "halfquant.gguf"
    p.write_bytes(cw.gguf_bytes(gguf_metadata(cfg, "llama"), t))
    with pytest.raises(HomuraError, match="some projections are block-quantised and some are float"):
        HfModel.load_gguf(ctx, p)
    p = tmp_path / "empty.gguf"
    p.write_bytes(cw.gguf_bytes(gguf_metadata(cfg, "llama"), []))
    with pytest.raises(HomuraError, match="missing GGUF tensor: blk.0.attn_q.weight"):
        HfModel.load_gguf(ctx, p)
    with pytest.raises(HomuraError, match="config.json"):
        HfModel.load_hf_dir(ctx, tmp_path / "nowhere")
    d = tmp_path / "noweights"
    d.mkdir()
    write_config(cfg, d)
    with pytest.raises(HomuraError, match="no model.safetensors or index found"):
        HfModel.load_hf_dir(ctx, d)
    (d / "model.safetensors").write_bytes(cw.safetensors_bytes({"x": ("F32", (1,), bytes(4))}))
    with pytest.raises(HomuraError, match="missing weight: model.embed_tokens.weight"):
        HfModel.load_hf_dir(ctx, d)
