"""Python handles over the C boundary: Context / DeviceBuffer for the kernel-level entry
points, HfModel for the C++ host classes that mirror the reference's
HfModel -> ExecutionPlan -> KvCache stack (reference src/hf/model.rs, src/runtime.rs).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _ffi

DTYPE_F32, DTYPE_BF16, DTYPE_Q8_0, DTYPE_Q4_0, DTYPE_I64, DTYPE_Q4_K, DTYPE_Q6_K = 0, 1, 2, 3, 4, 5, 6


class HomuraError(RuntimeError):
    """A C entry point returned a negative status; `.code` carries it."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[{code}] {message}")
        self.code = code


class DeviceBuffer:
    """An HBM allocation owned by a Context (freed explicitly or with the context)."""

    def __init__(self, ctx: "Context", ptr: int, nbytes: int):
        self.ctx, self.ptr, self.nbytes = ctx, ptr, nbytes

    def upload(self, arr: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(arr)
        if a.nbytes > self.nbytes:
            raise ValueError(f"upload of {a.nbytes} bytes into a buffer of {self.nbytes}")
        self.ctx._check(self.ctx.lib.hm_upload(self.ctx.h, self.ptr, a.ctypes.data, a.nbytes))
        return self

    def download(self, dtype, shape=None) -> np.ndarray:
        dtype = np.dtype(dtype)
        n = self.nbytes // dtype.itemsize if shape is None else int(np.prod(shape))
        out = np.empty(n, dtype=dtype)
        if out.nbytes > self.nbytes:
            raise ValueError("download larger than the buffer")
        self.ctx._check(self.ctx.lib.hm_download(self.ctx.h, out.ctypes.data, self.ptr, out.nbytes))
        return out if shape is None else out.reshape(shape)

    def free(self):
        if self.ptr:
            self.ctx._check(self.ctx.lib.hm_free(self.ctx.h, self.ptr))
            self.ptr = 0


class Context:
    """One GPU + one HIP stream (hm_ctx)."""

    def __init__(self, device: int = 0):
        self.lib = _ffi.load()
        self.h = self.lib.hm_init(device)
        if not self.h:
            raise HomuraError(-2, (self.lib.hm_last_error(None) or b"hm_init failed").decode())
        self._bufs: list[DeviceBuffer] = []

    def _check(self, rc: int):
        if rc != 0:
            raise HomuraError(rc, (self.lib.hm_last_error(self.h) or b"").decode())

    def close(self):
        if self.h:
            self.lib.hm_destroy(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        for b in self._bufs:
            if b.ptr:
                try:
                    b.free()
                except HomuraError:
                    pass
        self.close()

    # memory
    def alloc(self, nbytes: int) -> DeviceBuffer:
        p = C.c_void_p()
        self._check(self.lib.hm_alloc(self.h, nbytes, C.byref(p)))
        b = DeviceBuffer(self, p.value, max(nbytes, 1))
        self._bufs.append(b)
        return b

    def to_device(self, arr: np.ndarray) -> DeviceBuffer:
        a = np.ascontiguousarray(arr)
        return self.alloc(a.nbytes).upload(a)

    def empty(self, n: int, dtype=np.float32) -> DeviceBuffer:
        return self.alloc(int(n) * np.dtype(dtype).itemsize)

    def sync(self):
        self._check(self.lib.hm_sync(self.h))

    def fill_lds(self, word: int = 0xFFFFFFFF):
        """Test support: overwrite the LDS of every CU with `word` (default: a NaN pattern)."""
        self._check(self.lib.hm_test_fill_lds(self.h, word))

    def launch_floor(self, n_kernels: int, chained: bool, replays: int = 20) -> float:
        """Microseconds per replay of a graph of n_kernels dependent one-wavefront kernels (empty, or each
        reading 4 bytes its predecessor wrote)."""
        us = C.c_float()
        self._check(self.lib.hm_bench_launch_floor(self.h, n_kernels, int(chained), replays, C.byref(us)))
        return us.value

    def device_name(self) -> str:
        buf = C.create_string_buffer(128)
        self._check(self.lib.hm_device_name(self.h, buf, 128))
        return buf.value.decode()

    # timing on the context stream
    def time_ms(self, fn, iters: int = 1, warmup: int = 0) -> float:
        """Average milliseconds per call of `fn` measured with HIP events on the stream."""
        e0, e1 = C.c_void_p(), C.c_void_p()
        self._check(self.lib.hm_event_create(self.h, C.byref(e0)))
        self._check(self.lib.hm_event_create(self.h, C.byref(e1)))
        try:
            for _ in range(warmup):
                fn()
            self._check(self.lib.hm_event_record(self.h, e0))
            for _ in range(iters):
                fn()
            self._check(self.lib.hm_event_record(self.h, e1))
            ms = C.c_float()
            self._check(self.lib.hm_event_elapsed_ms(self.h, e0, e1, C.byref(ms)))
            return ms.value / iters
        finally:
            self.lib.hm_event_destroy(self.h, e0)
            self.lib.hm_event_destroy(self.h, e1)

    def time_graph_ms(self, record, reps: int = 20, warmup: int = 2) -> float:
        """Capture the kernel launches `record()` makes into a HIP graph, replay it `reps`
        times between two events and return the average milliseconds per replay."""
        g = C.c_void_p()
        self._check(self.lib.hm_graph_begin(self.h))
        try:
            record()
        finally:
            self._check(self.lib.hm_graph_end(self.h, C.byref(g)))
        try:
            return self.time_ms(lambda: self._check(self.lib.hm_graph_launch(self.h, g, 1)), reps, warmup)
        finally:
            self._check(self.lib.hm_graph_destroy(self.h, g))

    # kernel-level entry points (thin: pointer plumbing only)
    def gemv_bf16(self, x, w_kn, out, M, K, N):
        self._check(self.lib.hm_gemv_bf16(self.h, x.ptr, w_kn.ptr, out.ptr, M, K, N))

    def pack_bf16_kn_to_nk(self, w_kn, w_nk, K, N):
        self._check(self.lib.hm_pack_bf16_kn_to_nk(self.h, w_kn.ptr, w_nk.ptr, K, N))

    def gemv_bf16_nk(self, x, w_nk, out, M, K, N):
        self._check(self.lib.hm_gemv_bf16_nk(self.h, x.ptr, w_nk.ptr, out.ptr, M, K, N))

    def gemv_q8_0(self, x, w, out, M, K, N):
        self._check(self.lib.hm_gemv_q8_0(self.h, x.ptr, w.ptr, out.ptr, M, K, N))

    def gemv_q4_0(self, x, w, out, M, K, N):
        self._check(self.lib.hm_gemv_q4_0(self.h, x.ptr, w.ptr, out.ptr, M, K, N))

    def pack_quant_planes(self, dtype, blocks, N, K):
        """Raw Q8_0 / Q4_0 blocks [N][K/32] (device buffer) -> a new device buffer holding their planes."""
        planes = self.alloc(self.lib.hm_quant_planes_bytes(dtype, N, K))
        self._check(self.lib.hm_pack_quant_planes(self.h, dtype, blocks.ptr, planes.ptr, N, K))
        return planes

    def unpack_quant_planes(self, dtype, planes, blocks_out, N, K):
        self._check(self.lib.hm_unpack_quant_planes(self.h, dtype, planes.ptr, blocks_out.ptr, N, K))

    def gemv_q8_0_planes(self, x, planes, out, M, K, N):
        self._check(self.lib.hm_gemv_q8_0_planes(self.h, x.ptr, planes.ptr, out.ptr, M, K, N))

    def gemv_q4_0_planes(self, x, planes, out, M, K, N):
        self._check(self.lib.hm_gemv_q4_0_planes(self.h, x.ptr, planes.ptr, out.ptr, M, K, N))

    def gemv_q6_k_f32_planes(self, x, planes, out, M, K, N):
        self._check(self.lib.hm_gemv_q6_k_f32_planes(self.h, x.ptr, planes.ptr, out.ptr, M, K, N))

    def dequant_quant_planes(self, dtype, planes, out, N, K):
        self._check(self.lib.hm_dequant_quant_planes(self.h, dtype, planes.ptr, out.ptr, N, K))

    def gemv_q4_k(self, x, w, out, M, K, N):
        self._check(self.lib.hm_gemv_q4_k(self.h, x.ptr, w.ptr, out.ptr, M, K, N))

    def gemv_q6_k(self, x, w, out, M, K, N):
        self._check(self.lib.hm_gemv_q6_k(self.h, x.ptr, w.ptr, out.ptr, M, K, N))

    def pack_k8(self, dtype, blocks, N, K):
        """Raw Q4_K / Q6_K blocks [N][K/256] (device buffer) -> a new device buffer holding their K8 form."""
        k8 = self.alloc(self.lib.hm_k8_bytes(N, K))
        self._check(self.lib.hm_pack_k8(self.h, dtype, blocks.ptr, N, k8.ptr, N, K, 0))
        return k8

    def gemv_k8(self, x, k8, out, M, K, N):
        self._check(self.lib.hm_gemv_k8(self.h, x.ptr, k8.ptr, out.ptr, M, K, N))

    def gemv_q4_k_f32(self, x, w, out, M, K, N):
        self._check(self.lib.hm_gemv_q4_k_f32(self.h, x.ptr, w.ptr, out.ptr, M, K, N))

    def gemv_q6_k_f32(self, x, w, out, M, K, N):
        self._check(self.lib.hm_gemv_q6_k_f32(self.h, x.ptr, w.ptr, out.ptr, M, K, N))

    def quantize_q8_k(self, x, q8, act_d, bsums, M, K):
        self._check(self.lib.hm_quantize_q8_k(self.h, x.ptr, q8.ptr, act_d.ptr, bsums.ptr, M, K))

    def dequant_q4_k(self, blocks, out, nblocks):
        self._check(self.lib.hm_dequant_q4_k(self.h, blocks.ptr, out.ptr, nblocks))

    def dequant_q6_k(self, blocks, out, nblocks):
        self._check(self.lib.hm_dequant_q6_k(self.h, blocks.ptr, out.ptr, nblocks))

    def dequant_q8_0(self, blocks, out, nblocks):
        self._check(self.lib.hm_dequant_q8_0(self.h, blocks.ptr, out.ptr, nblocks))

    def dequant_q4_0(self, blocks, out, nblocks):
        self._check(self.lib.hm_dequant_q4_0(self.h, blocks.ptr, out.ptr, nblocks))

    def gemm_bf16(self, a, b, c, M, K, N):
        self._check(self.lib.hm_gemm_bf16(self.h, a.ptr, b.ptr, c.ptr, M, K, N))

    def gemm_bf16_nk(self, a, b_nk, c, M, K, N):
        self._check(self.lib.hm_gemm_bf16_nk(self.h, a.ptr, b_nk.ptr, c.ptr, M, K, N))

    def gemm_f32_bf16_nk(self, x, w_nk, out, M, K, N):
        self._check(self.lib.hm_gemm_f32_bf16_nk(self.h, x.ptr, w_nk.ptr, out.ptr, M, K, N))

    def gemm_f32_quant_nk(self, x, w_blocks, dtype, out, M, K, N):
        """Prompt-pass product with a block-quantised weight matrix (dtype: DTYPE_Q8_0 / Q4_0 / Q4_K / Q6_K)."""
        self._check(self.lib.hm_gemm_f32_quant_nk(self.h, x.ptr, w_blocks.ptr, dtype, out.ptr, M, K, N))

    def gqa_prefill_attn(self, q, kc, vc, out, S, H, kvh, hd, max_len, past, scale):
        self._check(self.lib.hm_gqa_prefill_attn(self.h, q.ptr, kc.ptr, vc.ptr, out.ptr, S, H, kvh, hd,
                                                 max_len, past, scale))

    def sample_token(self, d_logits, vocab, cfg: "SamplingConfig", generated, rng: "Rng") -> int:
        """reference sample_token on a logits row in HBM (top_k in 1..1024 when temperature > 0)."""
        gen = np.ascontiguousarray(generated, np.uint32).reshape(-1)
        c, tok = cfg.to_c(), C.c_int32()
        self._check(self.lib.hm_sample_token(self.h, d_logits.ptr, vocab, C.byref(c), gen.ctypes.data if gen.size else None,
                                             gen.size, C.byref(rng.state), C.byref(tok)))
        return tok.value

    def kv_append(self, kc, vc, k, v, B, kvh, hd, max_len, pos, n_new):
        self._check(self.lib.hm_kv_append(self.h, kc.ptr, vc.ptr, k.ptr, v.ptr, B, kvh, hd,
                                          max_len, pos, n_new))

    def gqa_decode_attn(self, q, kc, vc, out, B, H, kvh, hd, max_len, kv_len, scale):
        self._check(self.lib.hm_gqa_decode_attn(self.h, q.ptr, kc.ptr, vc.ptr, out.ptr, B, H, kvh,
                                                hd, max_len, kv_len, scale))

    def gqa_decode_attn_noalloc(self, q, kc, vc, out, B, H, kvh, hd, max_len, kv_len, scale):
        """hm_gqa_decode_attn with the partial sums in the library's fixed array (allocates nothing)."""
        self._check(self.lib.hm_gqa_decode_attn_noalloc(self.h, q.ptr, kc.ptr, vc.ptr, out.ptr, B, H,
                                                        kvh, hd, max_len, kv_len, scale))

    def rmsnorm(self, x, w, out, rows, dim, eps):
        self._check(self.lib.hm_rmsnorm(self.h, x.ptr, w.ptr, out.ptr, rows, dim, eps))

    def qknorm_rope(self, q, k, qw, kw, cos, sin, S, H, kvh, hd, eps):
        self._check(self.lib.hm_qknorm_rope(self.h, q.ptr, k.ptr, qw.ptr if qw else None,
                                            kw.ptr if kw else None, cos.ptr, sin.ptr, S, H, kvh,
                                            hd, eps))

    def silu_mul(self, g, u, out, n):
        self._check(self.lib.hm_silu_mul(self.h, g.ptr, u.ptr, out.ptr, n))

    def add(self, a, b, out, n):
        self._check(self.lib.hm_add(self.h, a.ptr, b.ptr, out.ptr, n))

    def embed(self, ids, table, out, n_ids, vocab, hidden):
        self._check(self.lib.hm_embed(self.h, ids.ptr, table.ptr, out.ptr, n_ids, vocab, hidden))

    def argmax(self, values, n, out):
        self._check(self.lib.hm_argmax(self.h, values.ptr, n, out.ptr))


@dataclass
class SamplingConfig:
    """reference SamplingConfig (src/generate.rs:646-686) with its defaults; temperature <= 0 is greedy."""
    temperature: float = 0.7
    top_k: int = 50
    top_p: float = 0.9
    min_p: float = 0.0
    repetition_penalty: float = 1.1
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0

    def to_c(self) -> _ffi.HmSamplingConfig:
        return _ffi.HmSamplingConfig(self.temperature, self.top_k, self.top_p, self.min_p, self.repetition_penalty,
                                     self.frequency_penalty, self.presence_penalty)


class Rng:
    """reference Rng (src/generate.rs:609-642): the state lives here, the arithmetic in the library."""

    def __init__(self, seed: int):
        self.state = C.c_uint64(_ffi.load().hm_rng_seed(seed))

    def next_f32(self) -> float:
        return float(_ffi.load().hm_rng_next_f32(C.byref(self.state)))


def sample_token_host(logits, cfg: SamplingConfig, generated, rng: Rng) -> int:
    """reference sample_token (src/generate.rs:698-801) on a host logits row."""
    row = np.ascontiguousarray(logits, np.float32).reshape(-1)
    gen = np.ascontiguousarray(generated, np.uint32).reshape(-1)
    c, tok = cfg.to_c(), C.c_int32()
    rc = _ffi.load().hm_sample_token_host(row.ctypes.data, row.size, C.byref(c), gen.ctypes.data if gen.size else None,
                                          gen.size, C.byref(rng.state), C.byref(tok))
    if rc != 0:
        raise HomuraError(rc, "hm_sample_token_host: bad arguments")
    return tok.value


@dataclass
class TransformerConfig:
    """Field-for-field the reference's TransformerConfig (src/hf/config.rs:11-73)."""
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_hidden_layers: int
    vocab_size: int
    num_key_value_heads: int | None = None
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10_000.0
    max_position_embeddings: int = 2048
    tie_word_embeddings: bool = False
    head_dim: int | None = None
    attention_bias: bool = False   # q/k/v_proj.bias present (reference src/hf/weights.rs:64-69)
    eos_token_id: int | None = None
    bos_token_id: int | None = None

    def kv_heads(self) -> int:
        return self.num_key_value_heads or self.num_attention_heads

    def get_head_dim(self) -> int:
        return self.head_dim or self.hidden_size // self.num_attention_heads

    def gqa_repeat(self) -> int:
        return self.num_attention_heads // self.kv_heads()

    def to_c(self) -> _ffi.HmTransformerConfig:
        return _ffi.HmTransformerConfig(
            self.hidden_size, self.intermediate_size, self.num_attention_heads,
            self.num_hidden_layers, self.num_key_value_heads or 0, self.vocab_size,
            self.head_dim or 0, self.max_position_embeddings, int(self.tie_word_embeddings),
            self.rms_norm_eps, self.rope_theta, int(self.attention_bias),
            -1 if self.eos_token_id is None else self.eos_token_id,
            -1 if self.bos_token_id is None else self.bos_token_id)


class HfModel:
    """Handle on the C++ HfModel (reference src/hf/model.rs:17-268): weights are handed over
    in TransformerWeights::to_slot_buffers order, then run_kv / generate run on the GPU."""

    def __init__(self, ctx: Context, config: TransformerConfig, weight_dtype: int = DTYPE_BF16,
                 has_qk_norm: bool = False, proj_dtypes=None):
        """proj_dtypes: optional 7 DTYPE_* codes per layer (q, k, v, o, gate, up, down) for a quantised
        model whose projections differ in type (then weight_dtype is ignored)."""
        self.ctx, self.config, self.lib = ctx, config, ctx.lib
        cfg = config.to_c()
        if proj_dtypes is not None:
            flat = [int(t) for t in proj_dtypes]
            if len(flat) != 7 * config.num_hidden_layers:
                raise ValueError(f"need {7 * config.num_hidden_layers} projection dtypes, got {len(flat)}")
            arr = (C.c_int * len(flat))(*flat)
            self.h = self.lib.hm_model_create_mixed(ctx.h, C.byref(cfg), arr, int(has_qk_norm))
        else:
            self.h = self.lib.hm_model_create(ctx.h, C.byref(cfg), weight_dtype, int(has_qk_norm))
        if not self.h:
            raise HomuraError(-1, (self.lib.hm_last_error(ctx.h) or b"").decode())

    @classmethod
    def _from_handle(cls, ctx: Context, handle) -> "HfModel":
        if not handle:
            raise HomuraError(-1, (ctx.lib.hm_last_error(ctx.h) or b"").decode())
        self = cls.__new__(cls)
        self.ctx, self.lib, self.h = ctx, ctx.lib, handle
        c, qkn, wdt = _ffi.HmTransformerConfig(), C.c_int(), C.c_int()
        self._check(self.lib.hm_model_config(handle, C.byref(c), C.byref(qkn), C.byref(wdt)))
        self.config = TransformerConfig(
            hidden_size=c.hidden_size, intermediate_size=c.intermediate_size,
            num_attention_heads=c.num_attention_heads, num_hidden_layers=c.num_hidden_layers,
            vocab_size=c.vocab_size, num_key_value_heads=c.num_key_value_heads or None,
            rms_norm_eps=c.rms_norm_eps, rope_theta=c.rope_theta,
            max_position_embeddings=c.max_position_embeddings,
            tie_word_embeddings=bool(c.tie_word_embeddings), head_dim=c.head_dim or None,
            attention_bias=bool(c.attention_bias),
            eos_token_id=None if c.eos_token_id < 0 else c.eos_token_id,
            bos_token_id=None if c.bos_token_id < 0 else c.bos_token_id)
        self.has_qk_norm, self.weight_dtype = bool(qkn.value), wdt.value
        return self

    @classmethod
    def load_gguf(cls, ctx: Context, path, max_seq_len: int = 0) -> "HfModel":
        """reference HfModel::load on a GGUF file (src/gguf.rs:589-708): parse, upload, finalize."""
        return cls._from_handle(ctx, ctx.lib.hm_model_load_gguf(ctx.h, str(path).encode(), max_seq_len))

    @classmethod
    def load_hf_dir(cls, ctx: Context, model_dir, max_seq_len: int = 0) -> "HfModel":
        """reference HfModel::load (src/hf/model.rs:75-146): config.json + safetensors."""
        return cls._from_handle(ctx, ctx.lib.hm_model_load_hf_dir(ctx.h, str(model_dir).encode(), max_seq_len))

    def _check(self, rc: int):
        if rc < 0:
            raise HomuraError(rc, (self.lib.hm_last_error(self.ctx.h) or b"").decode())
        return rc

    def close(self):
        if self.h:
            self.lib.hm_model_destroy(self.h)
            self.h = None

    def weight_slots(self):
        """[(name, dtype, dim0, dim1, nbytes)] in upload order."""
        out = []
        n = self._check(self.lib.hm_model_num_weight_slots(self.h))
        for i in range(n):
            name = C.create_string_buffer(96)
            dt, d0, d1, nb = C.c_int(), C.c_int64(), C.c_int64(), C.c_size_t()
            self._check(self.lib.hm_model_weight_slot_info(self.h, i, name, 96, C.byref(dt),
                                                           C.byref(d0), C.byref(d1), C.byref(nb)))
            out.append((name.value.decode(), dt.value, d0.value, d1.value, nb.value))
        return out

    def set_weight(self, slot: int, arr: np.ndarray):
        a = np.ascontiguousarray(arr)
        self._check(self.lib.hm_model_set_weight(self.h, slot, a.ctypes.data, a.nbytes))

    def set_weight_nk(self, slot: int, arr: np.ndarray):
        """Like set_weight, but a matrix slot arrives [N, K] (HF [out, in] / GGUF orientation)."""
        arr = np.ascontiguousarray(arr)
        self._check(self.lib.hm_model_set_weight_nk(self.h, slot, arr.ctypes.data_as(C.c_void_p), arr.nbytes))

    def set_lm_head_blocks(self, dtype: int, blocks: np.ndarray):
        """Block-quantised plans: the LM head as raw Q4_K / Q6_K blocks [vocab][hidden / 256] instead of the
        f32 lm_head.weight slot (hm_model_set_lm_head_blocks)."""
        a = np.ascontiguousarray(blocks, np.uint8).reshape(-1)
        self._check(self.lib.hm_model_set_lm_head_blocks(self.h, int(dtype), a.ctypes.data, a.nbytes))

    def finalize(self, max_seq_len: int):
        self._check(self.lib.hm_model_finalize(self.h, max_seq_len))

    def init_kv_cache(self, kv_buffers: list[np.ndarray], seq_len: int):
        """kv_buffers: key and value of every layer in turn, each at least kv_heads * seq_len * head_dim floats
        ([1, kv_heads, seq_len, head_dim]); the C side reads exactly that many from every pointer."""
        c = self.config
        want = c.kv_heads() * seq_len * c.get_head_dim()
        if len(kv_buffers) != 2 * c.num_hidden_layers:
            raise ValueError(f"init_kv_cache: {len(kv_buffers)} buffers for {c.num_hidden_layers} layers (2 per layer needed)")
        for i, b in enumerate(kv_buffers):
            if np.asarray(b).size < want:
                raise ValueError(f"init_kv_cache: buffer {i} holds {np.asarray(b).size} values, {want} needed")
        arrs = [np.ascontiguousarray(b, dtype=np.float32) for b in kv_buffers]
        ptrs = (_ffi.c_f32_p * len(arrs))(*[a.ctypes.data_as(_ffi.c_f32_p) for a in arrs])
        self._check(self.lib.hm_model_init_kv_cache(self.h, ptrs, seq_len))

    def set_graph(self, on: bool):
        """Replay each decode step from a captured HIP graph instead of launching kernel by kernel."""
        self._check(self.lib.hm_model_set_graph(self.h, int(on)))

    def set_whole_step(self, on: bool):
        """One launch for the embedding row and all layers of a decode step (bf16 models of a served
        shape) instead of one launch per projection."""
        self._check(self.lib.hm_model_set_whole_step(self.h, int(on)))

    def whole_step(self) -> bool:
        return bool(self._check(self.lib.hm_model_whole_step(self.h)))

    def whole_step_available(self) -> bool:
        return bool(self._check(self.lib.hm_model_whole_step_available(self.h)))

    def whole_step_status(self):
        """Raises if a whole-step launch left an error behind (an exchange that timed out)."""
        self._check(self.lib.hm_model_whole_step_status(self.h))

    def whole_step_inject_timeout(self, workgroup: int, spin_limit: int):
        """Test support: the next whole-step launches give up a wait after `spin_limit` polls and workgroup
        `workgroup` withholds its first publish, so the launch ends normally with its status set."""
        self._check(self.lib.hm_model_whole_step_inject_timeout(self.h, workgroup, spin_limit))

    def whole_step_trace(self, all_workgroups: bool = False) -> np.ndarray:
        """Device-clock ticks (100 MHz) of the latest whole-step launch: 11 per layer (both barriers of the
        Q|K|V, attention, O, gate|up and down phases; the fold's end comes after attention's) and a final
        one. The first call only switches recording on and returns an empty array. With all_workgroups
        the rows of all 256 workgroup slots come back (rows of workgroups the grid does not have stay 0)."""
        cap = (64 * 11 + 2) * (256 if all_workgroups else 1)
        out = np.zeros(cap, dtype=np.uint64)
        n = C.c_int(0)
        self._check(self.lib.hm_model_whole_step_trace(self.h, out.ctypes.data, cap, C.byref(n)))
        return out[:n.value]

    def prefill_capture_q8k_inputs(self, rows: int):
        """Test support: keep the rows the prompt pass hands to the Q8_K quantiser for the next `rows`
        cache positions (0 = stop)."""
        self._check(self.lib.hm_model_prefill_capture_q8k_inputs(self.h, rows))
        self._capture_rows = rows

    def prefill_captured_q8k_inputs(self) -> np.ndarray:
        """Those rows: per layer [rows][hidden], [rows][q_dim], [rows][hidden], [rows][inter], flat f32."""
        c = self.config
        n = c.num_hidden_layers * self._capture_rows * (
            2 * c.hidden_size + c.num_attention_heads * c.get_head_dim() + c.intermediate_size)
        out = np.zeros(n, np.float32)
        self._check(self.lib.hm_model_prefill_captured_q8k_inputs(self.h, out.ctypes.data, n))
        return out

    def reset_kv_cache(self):
        self._check(self.lib.hm_model_reset_kv_cache(self.h))

    def kv_cache_len(self) -> int:
        return self._check(self.lib.hm_model_kv_cache_len(self.h))

    def run_kv(self, input_ids, want_logits: bool = True):
        ids = np.ascontiguousarray(input_ids, dtype=np.int64).reshape(-1)
        logits = np.empty((len(ids), self.config.vocab_size), dtype=np.float32) if want_logits else None
        self._check(self.lib.hm_model_run_kv(
            self.h, ids.ctypes.data_as(C.POINTER(C.c_int64)), len(ids),
            logits.ctypes.data_as(_ffi.c_f32_p) if want_logits else None))
        return logits

    def prefill(self, input_ids, want_logits: bool = True):
        """The multi-token pass (reference HfGenerationContext::prefill, src/hf/model.rs:321-336)."""
        ids = np.ascontiguousarray(input_ids, dtype=np.int64).reshape(-1)
        logits = np.empty((len(ids), self.config.vocab_size), dtype=np.float32) if want_logits else None
        self._check(self.lib.hm_model_prefill(
            self.h, ids.ctypes.data_as(C.POINTER(C.c_int64)), len(ids),
            logits.ctypes.data_as(_ffi.c_f32_p) if want_logits else None))
        return logits

    def set_prefill_min(self, n_tokens: int):
        """Inputs of at least n_tokens take the prefill pass in run_kv / generate_greedy (0 = never)."""
        self._check(self.lib.hm_model_set_prefill_min(self.h, n_tokens))

    def generate(self, prompt_ids, max_new_tokens: int, cfg: "SamplingConfig", seed: int = 0, eos_token_id: int = -1):
        """reference generate_streaming_core (src/generate.rs:100-315): sampled generation; returns the new ids."""
        ids = np.ascontiguousarray(prompt_ids, dtype=np.int64).reshape(-1)
        out = np.empty(max_new_tokens, dtype=np.int32)
        c, n = cfg.to_c(), C.c_int()
        self._check(self.lib.hm_model_generate(
            self.h, ids.ctypes.data_as(C.POINTER(C.c_int64)), len(ids), max_new_tokens, C.byref(c), seed, eos_token_id,
            out.ctypes.data_as(C.POINTER(C.c_int32)), C.byref(n)))
        return out[:n.value].copy()

    def set_prefill_weight_cache(self, nbytes: int):
        """Block-quantised models: HBM the prompt pass may keep for dequantised projections (0 = none)."""
        self._check(self.lib.hm_model_set_prefill_weight_cache(self.h, nbytes))

    def set_prefill_pieces(self, pieces: int):
        """bf16 numbers per f32 activation in the prefill pass: 3 (default, exact) or 2."""
        self._check(self.lib.hm_model_set_prefill_pieces(self.h, pieces))

    def generate_greedy(self, prompt_ids, n_new: int) -> np.ndarray:
        ids = np.ascontiguousarray(prompt_ids, dtype=np.int64).reshape(-1)
        out = np.empty(n_new, dtype=np.int32)
        self._check(self.lib.hm_model_generate_greedy(
            self.h, ids.ctypes.data_as(C.POINTER(C.c_int64)), len(ids), n_new,
            out.ctypes.data_as(C.POINTER(C.c_int32))))
        return out

    def bench_decode(self, first_id: int, n_steps: int):
        ms = C.c_float()
        toks = np.empty(n_steps, dtype=np.int32)
        self._check(self.lib.hm_model_bench_decode(self.h, first_id, n_steps, C.byref(ms),
                                                   toks.ctypes.data_as(C.POINTER(C.c_int32))))
        return ms.value, toks

    @staticmethod
    def _records(recs, n):
        return [dict(label=recs[i].label.decode(), ms=recs[i].ms, launches=recs[i].launches,
                     bytes=recs[i].bytes) for i in range(n)]

    def profile_step(self, token_id: int):
        """One real decode step with HIP events around every device launch."""
        recs = (_ffi.HmKernelProfile * 32)()
        n = self._check(self.lib.hm_model_profile_step(self.h, token_id, recs, 32))
        return self._records(recs, n)

    def time_kernels(self, rounds: int):
        """Per device kernel: its per-layer launches back to back, `rounds` times (see header)."""
        recs = (_ffi.HmKernelProfile * 32)()
        n = self._check(self.lib.hm_model_time_kernels(self.h, rounds, recs, 32))
        return self._records(recs, n)

    def launches_per_step(self) -> int:
        return self._check(self.lib.hm_model_launches_per_step(self.h))
