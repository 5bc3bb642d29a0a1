"""Host-side checkpoint readers against the reference's own parser fixtures: the byte sequences
its tests assemble (reference src/gguf.rs:1055-1191, src/hf/safetensors.rs:194-342,
src/hf/config.rs:76-170) are rebuilt here and must parse to the values those tests assert."""
from __future__ import annotations

import struct

import numpy as np
import pytest

import ckpt_writers as cw
from homura_amd import checkpoints as ck


def write(tmp_path, name, data: bytes):
    p = tmp_path / name
    p.write_bytes(data)
    return p


# ── GGUF: the reference's fixtures ───────────────────────────────────────────

def test_parse_minimal_gguf(tmp_path):
    """reference parse_minimal_gguf (src/gguf.rs:1099-1127)"""
    data = cw.gguf_bytes([("general.architecture", cw.STRING, "test")],
                         [("weight", (2, 3), ck.GGML_F32, np.arange(6, dtype=np.float32).tobytes())])
    with ck.GgufFile(write(tmp_path, "minimal.gguf", data)) as g:
        assert g.version == 3
        assert g.meta_str("general.architecture") == "test"
        (name, shape, ty, off, nbytes), = g.tensors()
        assert (name, shape, ty, off, nbytes) == ("weight", (2, 3), ck.GGML_F32, 0, 24)   # dims reversed
        raw = g.tensor_bytes("weight").view(np.float32)
        assert raw[0] == 0.0 and raw[-1] == 5.0 and len(raw) == 6
        assert g.data_offset % 32 == 0


def test_parse_with_q8_0_tensor(tmp_path):
    """reference parse_with_q8_0_tensor (src/gguf.rs:1129-1172)"""
    data = cw.gguf_bytes([], [("blk.0.attn_q.weight", (64, 32), ck.GGML_Q8_0, b"\xAB" * (64 * 34))])
    with ck.GgufFile(write(tmp_path, "q8.gguf", data)) as g:
        (name, shape, ty, _off, nbytes), = g.tensors()
        assert (name, shape, ty, nbytes) == ("blk.0.attn_q.weight", (64, 32), ck.GGML_Q8_0, 2176)
        raw = g.tensor_bytes(name)
        assert len(raw) == 2176 and (raw == 0xAB).all()


def test_ggml_type_byte_sizes_and_alignment(tmp_path):
    """reference ggml_type_byte_sizes and align_up_works (src/gguf.rs:1174-1191)"""
    tensors = [("a", (32,), ck.GGML_Q8_0, bytes(34)), ("b", (256,), ck.GGML_Q4_K, bytes(144)),
               ("c", (256,), ck.GGML_Q6_K, bytes(210)), ("d", (32,), ck.GGML_Q4_0, bytes(18)),
               ("e", (3,), ck.GGML_BF16, bytes(6))]
    with ck.GgufFile(write(tmp_path, "sizes.gguf", cw.gguf_bytes([], tensors))) as g:
        got = {n: (nb, off) for n, _s, _t, off, nb in g.tensors()}
        assert [got[k][0] for k in "abcde"] == [34, 144, 210, 18, 6]
        assert [got[k][1] for k in "abcde"] == [0, 64, 224, 448, 480]     # each rounded up to 32
    # general.alignment overrides the default of 32
    data = cw.gguf_bytes([("general.alignment", cw.U32, 64)], [("w", (4,), ck.GGML_F32, bytes(16))], alignment=64)
    with ck.GgufFile(write(tmp_path, "align64.gguf", data)) as g:
        assert g.data_offset % 64 == 0
        assert g.tensor_bytes("w").nbytes == 16


def test_gguf_v2_counts_are_32_bit(tmp_path):
    data = cw.gguf_bytes([("general.architecture", cw.STRING, "llama")],
                         [("w", (2, 2), ck.GGML_F32, np.ones(4, np.float32).tobytes())], version=2)
    with ck.GgufFile(write(tmp_path, "v2.gguf", data)) as g:
        assert g.version == 2 and len(g.tensors()) == 1
        assert (g.tensor_bytes("w").view(np.float32) == 1).all()


def test_gguf_metadata_kinds(tmp_path):
    md = [("u8", cw.U8, 200), ("i8", cw.I8, -5), ("u16", cw.U16, 60000), ("i16", cw.I16, -300),
          ("u32", cw.U32, 4000000000), ("i32", cw.I32, 7), ("f32", cw.F32, 0.5), ("b", cw.BOOL, 1),
          ("s", cw.STRING, "héllo"), ("u64", cw.U64, 1 << 40), ("i64", cw.I64, 9), ("f64", cw.F64, 1e-6),
          ("toks", cw.ARRAY, (cw.STRING, ["a", "bb", "ccc"])),
          ("nested", cw.ARRAY, (cw.ARRAY, [(cw.U32, [1, 2]), (cw.U32, [3])]))]
    with ck.GgufFile(write(tmp_path, "meta.gguf", cw.gguf_bytes(md, []))) as g:
        # the reference's lenient accessors (src/gguf.rs:200-233): u64 from U32/I32/I64/U64 only
        assert g.meta_u64("u32") == 4000000000 and g.meta_u64("i32") == 7
        assert g.meta_u64("u64") == 1 << 40 and g.meta_u64("i64") == 9
        assert g.meta_u64("u8") is None and g.meta_u64("f32") is None and g.meta_u64("absent") is None
        assert g.meta_f32("f32") == 0.5 and abs(g.meta_f32("f64") - 1e-6) < 1e-12
        assert g.meta_f32("u32") is None
        assert g.meta_str("s") == "héllo" and g.meta_str("u8") is None
        assert g.meta_array_len("toks") == 3 and g.meta_array_len("nested") == 2 and g.meta_array_len("s") is None


def _arch_md(arch="qwen3", **over):
    md = {f"{arch}.embedding_length": 1024, f"{arch}.feed_forward_length": 3072,
          f"{arch}.attention.head_count": 16, f"{arch}.block_count": 28,
          f"{arch}.attention.head_count_kv": 8, f"{arch}.vocab_size": 151936,
          f"{arch}.attention.layer_norm_rms_epsilon": 1e-6, f"{arch}.rope.freq_base": 1e6,
          f"{arch}.context_length": 40960, f"{arch}.attention.key_length": 128}
    md.update(over)
    out = [("general.architecture", cw.STRING, arch)]
    for k, v in md.items():
        if v is None:
            continue
        out.append((k, cw.F32 if isinstance(v, float) else cw.U32, v))
    return out


def test_gguf_transformer_config(tmp_path):
    """reference GgufFile::transformer_config (src/gguf.rs:508-582)"""
    tensors = [("blk.0.attn_q_norm.weight", (128,), ck.GGML_F32, bytes(512))]
    with ck.GgufFile(write(tmp_path, "cfg.gguf", cw.gguf_bytes(_arch_md(), tensors))) as g:
        cfg, qkn = g.transformer_config()
        assert (cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads, cfg.num_hidden_layers) == (1024, 3072, 16, 28)
        assert cfg.kv_heads() == 8 and cfg.vocab_size == 151936 and cfg.get_head_dim() == 128
        assert cfg.rope_theta == 1e6 and abs(cfg.rms_norm_eps - 1e-6) < 1e-12 and cfg.max_position_embeddings == 40960
        assert cfg.tie_word_embeddings is True        # no output.weight tensor
        assert qkn is True and cfg.attention_bias is False
        assert cfg.eos_token_id is None and cfg.bos_token_id is None
    # defaults and fallbacks: no kv heads, no eps/theta/context, vocab from the tokenizer, untied, biased
    md = _arch_md("llama", **{"llama.attention.head_count_kv": None, "llama.vocab_size": None,
                              "llama.attention.layer_norm_rms_epsilon": None, "llama.rope.freq_base": None,
                              "llama.context_length": None, "llama.attention.key_length": None})
    md.append(("tokenizer.ggml.tokens", cw.ARRAY, (cw.STRING, [str(i) for i in range(77)])))
    md.append(("tokenizer.ggml.eos_token_id", cw.U32, 2))          # src/gguf.rs:559-565
    md.append(("tokenizer.ggml.bos_token_id", cw.U32, 1))
    tensors = [("output.weight", (4, 4), ck.GGML_F32, bytes(64)), ("blk.0.attn_q.bias", (4,), ck.GGML_F32, bytes(16))]
    with ck.GgufFile(write(tmp_path, "cfg2.gguf", cw.gguf_bytes(md, tensors))) as g:
        cfg, qkn = g.transformer_config()
        assert cfg.kv_heads() == 16 and cfg.vocab_size == 77 and cfg.get_head_dim() == 64
        assert cfg.rope_theta == 10000.0 and cfg.rms_norm_eps == 1e-6 and cfg.max_position_embeddings == 2048
        assert cfg.tie_word_embeddings is False and qkn is False and cfg.attention_bias is True
        assert cfg.eos_token_id == 2 and cfg.bos_token_id == 1
    md = [m for m in _arch_md() if m[0] != "qwen3.embedding_length"]
    with ck.GgufFile(write(tmp_path, "cfg3.gguf", cw.gguf_bytes(md, []))) as g:
        with pytest.raises(ValueError, match="missing or invalid metadata: qwen3.embedding_length"):
            g.transformer_config()
    with ck.GgufFile(write(tmp_path, "cfg4.gguf", cw.gguf_bytes([], []))) as g:
        with pytest.raises(ValueError, match="missing general.architecture"):
            g.transformer_config()


def test_gguf_malformed_files(tmp_path):
    good = cw.gguf_bytes([("general.architecture", cw.STRING, "x")], [("w", (8,), ck.GGML_F32, bytes(32))])
    cases = {
        "small": (good[:12], "too small"),
        "magic": (b"GGUX" + good[4:], r"invalid GGUF magic: 0x58554747 \(expected 0x46554747\)"),
        "version": (good[:4] + struct.pack("<I", 4) + good[8:], r"unsupported GGUF version: 4 \(expected 2 or 3\)"),
        "cut_meta": (good[:40], "unexpected end|runs past"),
        "cut_data": (good[:-8], "runs past the end of the file"),
    }
    bad_type = bytearray(good)
    pos = good.index(b"w", 60) + 1 + 4 + 8       # name, n_dims, one dim -> the type code
    bad_type[pos:pos + 4] = struct.pack("<I", 5)  # 4 and 5 are retired GGML codes
    cases["type"] = (bytes(bad_type), "unknown GGML type code 5 for tensor 'w'")
    huge_string = good[:24] + struct.pack("<Q", 1 << 60) + good[32:]
    cases["string"] = (huge_string, "runs past the end of the file")
    for name, (data, pattern) in cases.items():
        with pytest.raises(ValueError, match=pattern):
            ck.GgufFile(write(tmp_path, name + ".gguf", data))
    with pytest.raises(ValueError, match="No such file"):
        ck.GgufFile(tmp_path / "absent.gguf")
    # a block type whose element count is not a whole number of blocks
    with pytest.raises(ValueError, match="not a multiple"):
        ck.GgufFile(write(tmp_path, "blk.gguf", cw.gguf_bytes([], [("w", (33,), ck.GGML_Q8_0, bytes(34))])))


# ── safetensors: the reference's fixtures ────────────────────────────────────

def test_load_safetensors_file(tmp_path):
    """reference load_safetensors_file (src/hf/safetensors.rs:242-269): the literal header string"""
    header = b'{"x":{"dtype":"F32","shape":[2],"data_offsets":[0,8]}}'
    data = struct.pack("<Q", len(header)) + header + np.array([1.0, 2.0], np.float32).tobytes()
    with ck.SafeTensorsFile(write(tmp_path, "test.safetensors", data)) as s:
        t = s.tensors()
        assert list(t) == ["x"] and t["x"][:3] == ("F32", (2,), 8)
        assert s.tensor_bytes("x").view(np.float32).tolist() == [1.0, 2.0]


def test_load_safetensors_bf16(tmp_path):
    """reference load_safetensors_bf16 (src/hf/safetensors.rs:312-342)"""
    header = b'{"w":{"dtype":"BF16","shape":[3],"data_offsets":[0,6]}}'
    vals = np.array([1.0, -0.5, 2.0], np.float32)
    data = struct.pack("<Q", len(header)) + header + cw.f32_to_bf16_trunc(vals).tobytes()
    with ck.SafeTensorsFile(write(tmp_path, "bf16.safetensors", data)) as s:
        assert s.tensors()["w"][:3] == ("BF16", (3,), 6)
        bits = s.tensor_bytes("w").view(np.uint16).astype(np.uint32) << 16
        assert bits.view(np.float32).tolist() == [1.0, -0.5, 2.0]     # bf16 = top half of the f32


def test_safetensors_metadata_and_errors(tmp_path):
    data = cw.safetensors_bytes({"a": ("I64", (2,), bytes(16)), "b.c": ("F16", (2, 2), bytes(8))},
                                metadata={"format": "pt"})
    with ck.SafeTensorsFile(write(tmp_path, "m.safetensors", data)) as s:
        assert set(s.tensors()) == {"a", "b.c"}                       # __metadata__ is skipped
    with pytest.raises(ValueError, match=r"too small \(< 8 bytes\)"):
        ck.SafeTensorsFile(write(tmp_path, "s.safetensors", b"abc"))
    with pytest.raises(ValueError, match="header length 1000 exceeds file size 18"):
        ck.SafeTensorsFile(write(tmp_path, "h.safetensors", struct.pack("<Q", 1000) + b"0123456789"))
    bad = b'{"x":{"dtype":"F32","shape":[2],"data_offsets":[0,80]}}'
    with pytest.raises(ValueError, match="runs past the end"):
        ck.SafeTensorsFile(write(tmp_path, "o.safetensors", struct.pack("<Q", len(bad)) + bad + bytes(8)))
    with pytest.raises(ValueError, match="JSON"):
        ck.SafeTensorsFile(write(tmp_path, "j.safetensors", struct.pack("<Q", 5) + b"{oops"))
    deep = b'{"x":{"dtype":"F32","shape":[1,1,1,1,1,1,1,1,2],"data_offsets":[0,8]}}'   # nine dimensions
    with pytest.raises(ValueError, match="9 dimensions"):
        ck.SafeTensorsFile(write(tmp_path, "d.safetensors", struct.pack("<Q", len(deep)) + deep + bytes(8)))


# ── config.json: the reference's fixtures ────────────────────────────────────

def test_parse_qwen2_config():
    """reference parse_qwen2_config (src/hf/config.rs:80-104)"""
    cfg = ck.config_from_json('''{
            "architectures": ["Qwen2ForCausalLM"],
            "hidden_size": 896,
            "intermediate_size": 4864,
            "num_attention_heads": 14,
            "num_hidden_layers": 24,
            "num_key_value_heads": 2,
            "vocab_size": 151936,
            "rms_norm_eps": 1e-6,
            "rope_theta": 1000000.0,
            "max_position_embeddings": 32768,
            "tie_word_embeddings": true,
            "eos_token_id": 151643,
            "bos_token_id": 151643
        }''')
    assert cfg.hidden_size == 896 and cfg.num_attention_heads == 14
    assert cfg.kv_heads() == 2 and cfg.get_head_dim() == 64 and cfg.gqa_repeat() == 7
    assert cfg.tie_word_embeddings is True and cfg.rope_theta == 1e6 and cfg.max_position_embeddings == 32768
    assert cfg.eos_token_id == 151643 and cfg.bos_token_id == 151643


def test_parse_llama_config_no_kv_heads():
    """reference parse_llama_config_no_kv_heads (src/hf/config.rs:106-124)"""
    cfg = ck.config_from_json('''{
            "hidden_size": 4096,
            "intermediate_size": 11008,
            "num_attention_heads": 32,
            "num_hidden_layers": 32,
            "vocab_size": 32000,
            "rope_theta": 10000.0
        }''')
    assert cfg.kv_heads() == 32 and cfg.gqa_repeat() == 1
    assert cfg.tie_word_embeddings is False and cfg.rope_theta == 10000.0
    assert cfg.rms_norm_eps == 1e-6 and cfg.max_position_embeddings == 2048        # serde defaults


def test_config_errors_and_head_dim():
    with pytest.raises(ValueError, match="missing field `vocab_size`"):
        ck.config_from_json('{"hidden_size": 8, "intermediate_size": 8, "num_attention_heads": 2, "num_hidden_layers": 1}')
    with pytest.raises(ValueError, match="JSON"):
        ck.config_from_json('{"hidden_size": 8,')
    cfg = ck.config_from_json('{"hidden_size": 1024, "intermediate_size": 3072, "num_attention_heads": 16, '
                              '"num_hidden_layers": 28, "vocab_size": 151936, "head_dim": 128, '
                              '"nested": {"a": [1, 2.5e3, -3, null, false], "s": "q\\"\\u00e9\\n"}}')
    assert cfg.get_head_dim() == 128


def test_gguf_tensor_f32_dequantises_like_the_oracle(tmp_path):
    """reference load_f32_buffer (src/gguf.rs:727-776): F32 as stored, F16/BF16 widened, Q8_0/Q4_0/Q4_K/
    Q6_K dequantised. The host conversion must give the oracle's floats bit for bit (the oracle's
    decodes are pinned by the reference's known-answer tests and independent numpy decodes)."""
    import pyoracle
    from homura_amd import synth
    rng = np.random.default_rng(5)
    f32 = rng.standard_normal(64).astype(np.float32)
    f16 = rng.standard_normal(64).astype(np.float16)
    b16 = synth.normal_bf16(9, 64, 1.0)
    q8, q4 = synth.q8_0_blocks(1, 6), synth.q4_0_blocks(2, 6)
    q4k, q6k = synth.q4_k_blocks(3, 5), synth.q6_k_blocks(4, 5)
    tensors = [("f32", (4, 16), ck.GGML_F32, f32.tobytes()), ("f16", (64,), ck.GGML_F16, f16.tobytes()),
               ("bf16", (64,), ck.GGML_BF16, b16.tobytes()), ("q8_0", (6, 32), ck.GGML_Q8_0, q8.tobytes()),
               ("q4_0", (3, 64), ck.GGML_Q4_0, q4.tobytes()), ("q4_k", (5, 256), ck.GGML_Q4_K, q4k.tobytes()),
               ("q6_k", (5, 256), ck.GGML_Q6_K, q6k.tobytes()), ("q5_k", (256,), ck.GGML_Q5_K, bytes(176))]
    want = {"f32": f32.reshape(4, 16), "f16": f16.astype(np.float32), "bf16": synth.bf16_to_f32(b16),
            "q8_0": pyoracle.dequant_q8_0(q8).reshape(6, 32), "q4_0": pyoracle.dequant_q4_0(q4).reshape(3, 64),
            "q4_k": pyoracle.dequant_q4_k(q4k).reshape(5, 256), "q6_k": pyoracle.dequant_q6_k(q6k).reshape(5, 256)}
    with ck.GgufFile(write(tmp_path, "kinds.gguf", cw.gguf_bytes([], tensors))) as g:
        for name, w in want.items():
            got = g.tensor_f32(name)
            assert got.shape == w.shape and np.array_equal(got.view(np.uint32), w.view(np.uint32)), name
        with pytest.raises(ValueError, match="q5_k"):
            g.tensor_f32("q5_k")
        with pytest.raises(KeyError):
            g.tensor_f32("absent")
