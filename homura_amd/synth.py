"""Deterministic synthetic tensors (numpy views of the library's host-side generator).

Same bits on every platform: the generator is integer arithmetic (see csrc/synth.cpp).
Seeds used by the benchmark configurations live here so tests and bench agree.
"""
from __future__ import annotations

import numpy as np

from . import _ffi

SEED_CFG1 = 0xC0FFEE01  # single bf16 GEMV 896 x 4864
SEED_CFG2 = 0xC0FFEE02  # Qwen3-0.6B-shape decode
SEED_CFG3 = 0xC0FFEE03  # Q8_0 GEMV 2048 -> 5632
SEED_CFG4 = 0xC0FFEE04  # Q4_0 GEMV 1536 -> 151936
SEED_CFG5 = 0xC0FFEE05  # prefill GEMM + long-context attention


def _ptr(a: np.ndarray):
    return a.ctypes.data


def normal_f32(seed: int, n: int, scale: float = 1.0, first: int = 0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    _ffi.load().hm_synth_normal_f32(seed, first, n, scale, _ptr(out))
    return out


def normal_bf16(seed: int, n: int, scale: float = 1.0, first: int = 0) -> np.ndarray:
    """bf16 bit patterns (uint16) of round-to-nearest-even(N(0,1) * scale)."""
    out = np.empty(n, dtype=np.uint16)
    _ffi.load().hm_synth_normal_bf16(seed, first, n, scale, _ptr(out))
    return out


def token_ids(seed: int, n: int, vocab: int) -> np.ndarray:
    out = np.empty(n, dtype=np.int64)
    _ffi.load().hm_synth_token_ids(seed, n, vocab, _ptr(out))
    return out


def q8_0_blocks(seed: int, n_blocks: int, d_scale: float = 0.01) -> np.ndarray:
    out = np.empty(n_blocks * 34, dtype=np.uint8)
    _ffi.load().hm_synth_q8_0(seed, n_blocks, d_scale, _ptr(out))
    return out


def q4_0_blocks(seed: int, n_blocks: int, d_scale: float = 0.01) -> np.ndarray:
    out = np.empty(n_blocks * 18, dtype=np.uint8)
    _ffi.load().hm_synth_q4_0(seed, n_blocks, d_scale, _ptr(out))
    return out


def _f16_scales(rng, n, scale):
    return np.abs(rng.standard_normal(n) * scale).astype(np.float16).view(np.uint16)


def q4_k_blocks(seed: int, n_blocks: int, d_scale: float = 0.001) -> np.ndarray:
    """Random Q4_K super-blocks (144 B: f16 d, f16 dmin, 12 bytes of 6-bit scales/mins, 128 bytes of
    nibbles; ggml block_q4_K as the reference reads it, src/gguf.rs:835-882)."""
    rng = np.random.default_rng(seed)
    out = rng.integers(0, 256, size=(n_blocks, 144), dtype=np.uint8)
    out[:, 0:2] = _f16_scales(rng, n_blocks, d_scale).view(np.uint8).reshape(n_blocks, 2)
    out[:, 2:4] = _f16_scales(rng, n_blocks, d_scale).view(np.uint8).reshape(n_blocks, 2)
    return out.reshape(-1)


def q6_k_blocks(seed: int, n_blocks: int, d_scale: float = 0.0005) -> np.ndarray:
    """Random Q6_K super-blocks (210 B: 128 bytes low nibbles, 64 bytes high bit pairs, 16 int8
    scales, f16 d; src/gguf.rs:886-917)."""
    rng = np.random.default_rng(seed)
    out = rng.integers(0, 256, size=(n_blocks, 210), dtype=np.uint8)
    out[:, 208:210] = _f16_scales(rng, n_blocks, d_scale).view(np.uint8).reshape(n_blocks, 2)
    return out.reshape(-1)


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_rne(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)
