"""Read-only views of checkpoint containers through the library's host-side parsers
(reference src/gguf.rs, src/hf/safetensors.rs, src/hf/config.rs). No GPU needed."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _ffi
from .runtime import TransformerConfig

GGML_F32, GGML_F16, GGML_Q4_0, GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_BF16 = 0, 1, 2, 8, 12, 13, 14, 30


def _config_from_c(c) -> TransformerConfig:
    return TransformerConfig(
        hidden_size=c.hidden_size, intermediate_size=c.intermediate_size,
        num_attention_heads=c.num_attention_heads, num_hidden_layers=c.num_hidden_layers,
        vocab_size=c.vocab_size, num_key_value_heads=c.num_key_value_heads or None,
        rms_norm_eps=c.rms_norm_eps, rope_theta=c.rope_theta,
        max_position_embeddings=c.max_position_embeddings,
        tie_word_embeddings=bool(c.tie_word_embeddings), head_dim=c.head_dim or None,
        attention_bias=bool(c.attention_bias),
        eos_token_id=None if c.eos_token_id < 0 else c.eos_token_id,
        bos_token_id=None if c.bos_token_id < 0 else c.bos_token_id)


class GgufFile:
    """reference GgufFile (src/gguf.rs:333-470)."""

    def __init__(self, path):
        self.lib = _ffi.load()
        err = C.create_string_buffer(512)
        self.h = self.lib.hm_gguf_open(str(path).encode(), err, 512)
        if not self.h:
            raise ValueError(err.value.decode())

    def close(self):
        if self.h:
            self.lib.hm_gguf_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def version(self) -> int:
        return self.lib.hm_gguf_version(self.h)

    @property
    def data_offset(self) -> int:
        return self.lib.hm_gguf_data_offset(self.h)

    def tensors(self):
        """[(name, shape, ggml_type, offset, nbytes)] in file order."""
        out = []
        for i in range(self.lib.hm_gguf_num_tensors(self.h)):
            name = C.create_string_buffer(256)
            nd, ty, off, nb = C.c_int(), C.c_int(), C.c_uint64(), C.c_size_t()
            dims = (C.c_uint64 * 8)()
            assert self.lib.hm_gguf_tensor_info(self.h, i, name, 256, C.byref(nd), dims, C.byref(ty),
                                                C.byref(off), C.byref(nb)) == 0
            out.append((name.value.decode(), tuple(dims[:nd.value]), ty.value, off.value, nb.value))
        return out

    def tensor_bytes(self, name: str) -> np.ndarray:
        i = self.lib.hm_gguf_find_tensor(self.h, name.encode())
        if i < 0:
            raise KeyError(name)
        nbytes = self.tensors()[i][4]
        ptr = self.lib.hm_gguf_tensor_data(self.h, i)
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_uint8)), shape=(nbytes,)).copy()

    def tensor_f32(self, name: str) -> np.ndarray:
        """reference load_f32_buffer (src/gguf.rs:727-776): the tensor as f32, dequantised on the host."""
        i = self.lib.hm_gguf_find_tensor(self.h, name.encode())
        if i < 0:
            raise KeyError(name)
        shape = self.tensors()[i][1]
        out = np.empty(shape, np.float32)
        err = C.create_string_buffer(256)
        if self.lib.hm_gguf_tensor_f32(self.h, i, out.ctypes.data, out.size, err, 256) != 0:
            raise ValueError(err.value.decode())
        return out

    def meta_str(self, key: str):
        buf = C.create_string_buffer(4096)
        n = self.lib.hm_gguf_meta_str(self.h, key.encode(), buf, 4096)
        return None if n < 0 else buf.value.decode()

    def meta_u64(self, key: str):
        v = C.c_uint64()
        return v.value if self.lib.hm_gguf_meta_u64(self.h, key.encode(), C.byref(v)) == 0 else None

    def meta_f32(self, key: str):
        v = C.c_float()
        return v.value if self.lib.hm_gguf_meta_f32(self.h, key.encode(), C.byref(v)) == 0 else None

    def meta_array_len(self, key: str):
        n = self.lib.hm_gguf_meta_array_len(self.h, key.encode())
        return None if n < 0 else n

    def transformer_config(self):
        """(TransformerConfig, has_qk_norm) - reference GgufFile::transformer_config."""
        c, qkn = _ffi.HmTransformerConfig(), C.c_int()
        err = C.create_string_buffer(512)
        if self.lib.hm_gguf_transformer_config(self.h, C.byref(c), C.byref(qkn), err, 512) != 0:
            raise ValueError(err.value.decode())
        return _config_from_c(c), bool(qkn.value)


class SafeTensorsFile:
    """The container part of the reference's load_safetensors (src/hf/safetensors.rs:38-99)."""

    def __init__(self, path):
        self.lib = _ffi.load()
        err = C.create_string_buffer(512)
        self.h = self.lib.hm_safetensors_open(str(path).encode(), err, 512)
        if not self.h:
            raise ValueError(err.value.decode())

    def close(self):
        if self.h:
            self.lib.hm_safetensors_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def tensors(self):
        """{name: (dtype, shape, nbytes, index)}"""
        out = {}
        for i in range(self.lib.hm_safetensors_num_tensors(self.h)):
            name, dt = C.create_string_buffer(256), C.create_string_buffer(8)
            nd, nb = C.c_int(), C.c_size_t()
            dims = (C.c_uint64 * 8)()
            assert self.lib.hm_safetensors_tensor_info(self.h, i, name, 256, dt, C.byref(nd), dims, C.byref(nb)) == 0
            out[name.value.decode()] = (dt.value.decode(), tuple(dims[:nd.value]), nb.value, i)
        return out

    def tensor_bytes(self, name: str) -> np.ndarray:
        _dt, _shape, nbytes, i = self.tensors()[name]
        ptr = self.lib.hm_safetensors_tensor_data(self.h, i)
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_uint8)), shape=(nbytes,)).copy()


def config_from_json(text: str) -> TransformerConfig:
    """reference TransformerConfig::load on the text of a config.json (src/hf/config.rs:49-54)."""
    lib = _ffi.load()
    c = _ffi.HmTransformerConfig()
    err = C.create_string_buffer(512)
    if lib.hm_config_from_json(text.encode(), C.byref(c), err, 512) != 0:
        raise ValueError(err.value.decode())
    return _config_from_c(c)
