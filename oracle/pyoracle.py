"""ctypes binding of oracle/liboracle.so — the CPU restatement of the reference's decode path.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the CPU-baseline leg of
the benchmark. The product package (homura_amd/) must never import this module.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "liboracle.so"

W_BF16, W_Q8_0, W_Q4_0, W_Q4_K, W_Q6_K = 1, 2, 3, 4, 5

_P = C.c_void_p
_I = C.c_int
_F = C.c_float


class OrcSamplingConfig(C.Structure):
    """reference SamplingConfig (src/generate.rs:646-686) without the strings; defaults as there."""
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_int), ("top_p", C.c_float), ("min_p", C.c_float),
                ("repetition_penalty", C.c_float), ("frequency_penalty", C.c_float), ("presence_penalty", C.c_float)]

    def __init__(self, temperature=0.7, top_k=50, top_p=0.9, min_p=0.0, repetition_penalty=1.1,
                 frequency_penalty=0.0, presence_penalty=0.0):
        super().__init__(temperature, top_k, top_p, min_p, repetition_penalty, frequency_penalty, presence_penalty)


class OrcConfig(C.Structure):
    _fields_ = [("hidden", _I), ("inter", _I), ("heads", _I), ("kv_heads", _I),
                ("head_dim", _I), ("layers", _I), ("vocab", _I), ("eps", _F),
                ("weight_kind", _I), ("has_qk_norm", _I)]


def build():
    """Compile the oracle with gcc (a few seconds): the x86-64-v3 build the tests use and the AVX-512 one."""
    subprocess.run(["make", "-s", "-C", str(HERE), "all"], check=True)


_lib = None
_isa = "x86-64-v3"


def best_isa() -> str:
    """'x86-64-v4' where this host lists the AVX-512 sets that level needs, else 'x86-64-v3'."""
    try:
        flags = next(l for l in open("/proc/cpuinfo") if l.startswith("flags")).split()
    except (OSError, StopIteration):
        return "x86-64-v3"
    need = {"avx512f", "avx512bw", "avx512cd", "avx512dq", "avx512vl"}
    return "x86-64-v4" if need <= set(flags) else "x86-64-v3"


def use_isa(isa: str):
    """Pick the build before the first load(): the timed CPU baseline asks for best_isa(), everything else
    keeps the default."""
    global _isa
    if _lib is not None and isa != _isa:
        raise RuntimeError("the oracle library is already loaded")
    if isa not in ("x86-64-v3", "x86-64-v4"):
        raise ValueError(isa)
    _isa = isa


def isa() -> str:
    return _isa


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    path = LIB_PATH if _isa == "x86-64-v3" else HERE / "liboracle_v4.so"
    if not path.exists():
        build()
    lib = C.CDLL(str(path))
    sig = {
        "orc_f16_to_f32": (_F, [C.c_uint16]),
        "orc_f16_to_f32_array": (None, [_P, C.c_size_t, _P]),
        "orc_bf16_to_f32": (_F, [C.c_uint16]),
        "orc_f32_to_bf16_trunc": (C.c_uint16, [_F]),
        "orc_f32_to_bf16_rne": (C.c_uint16, [_F]),
        "orc_dequant_q8_0": (None, [_P, C.c_size_t, _P]),
        "orc_dequant_q4_k": (None, [_P, C.c_size_t, _P]),
        "orc_dequant_q6_k": (None, [_P, C.c_size_t, _P]),
        "orc_quantize_q8_k": (None, [_P, _P, _P, _P]),
        "orc_gemv_q4_k": (None, [_P, _P, _P, _I, _I, _I]),
        "orc_gemv_q6_k": (None, [_P, _P, _P, _I, _I, _I]),
        "orc_dequant_q4_0": (None, [_P, C.c_size_t, _P]),
        "orc_matmul_f32_bf16": (None, [_P, _P, _P, _I, _I, _I]),
        "orc_matmul_f32_f32": (None, [_P, _P, _P, _I, _I, _I]),
        "orc_matmul_bf16_bf16": (None, [_P, _P, _P, _I, _I, _I]),
        "orc_gemv_q8_0": (None, [_P, _P, _P, _I, _I, _I]),
        "orc_gemv_q4_0": (None, [_P, _P, _P, _I, _I, _I]),
        "orc_rms_norm": (None, [_P, _P, _P, _I, _I, _F]),
        "orc_rms_norm_f64acc": (None, [_P, _P, _P, _I, _I, _F]),
        "orc_rms_norm_f64mean": (None, [_P, _P, _P, _I, _I, _F]),
        "orc_silu_mul": (None, [_P, _P, _P, C.c_size_t]),
        "orc_add": (None, [_P, _P, _P, C.c_size_t]),
        "orc_softmax": (None, [_P, _P, _I, _I]),
        "orc_softmax_f64acc": (None, [_P, _P, _I, _I]),
        "orc_rope_tables": (None, [_I, _I, C.c_double, _P, _P]),
        "orc_causal_mask": (None, [_I, _I, _P]),
        "orc_rope_half": (None, [_P, _P, _P, _I, _I, _I]),
        "orc_embed": (None, [_P, _I, _P, _I, _P]),
        "orc_argmax_last": (_I, [_P, _I]),
        "orc_gqa_attention": (None, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, C.c_long, _I, _P]),
        "orc_kv_new": (_P, [_I, _I, _I, _I, _I]),
        "orc_kv_free": (None, [_P]),
        "orc_kv_append_key": (_I, [_P, _I, _P, _I]),
        "orc_kv_append_value": (_I, [_P, _I, _P, _I]),
        "orc_kv_advance_by": (None, [_P, _I]),
        "orc_kv_reset": (None, [_P, _I]),
        "orc_kv_current_len": (_I, [_P]),
        "orc_kv_view_len": (_I, [_P]),
        "orc_kv_head_stride": (C.c_long, [_P]),
        "orc_kv_key_ptr": (_P, [_P, _I]),
        "orc_kv_value_ptr": (_P, [_P, _I]),
        "orc_kv_view_copy": (None, [_P, _I, _P, _P]),
        "orc_kv_init_from": (_I, [_P, _I, _P, _P, _I]),
        "orc_model_new": (_P, [C.POINTER(OrcConfig)]),
        "orc_model_set_global": (None, [_P, _P, _P, _P, _P, _P, _I]),
        "orc_model_set_layer": (None, [_P, _I] + [_P] * 11),
        "orc_model_set_layer_bias": (None, [_P, _I, _P, _P, _P]),
        "orc_model_set_layer_kinds": (None, [_P, _I, C.POINTER(_I)]),
        "orc_model_attach_kv": (None, [_P, _P]),
        "orc_model_free": (None, [_P]),
        "orc_model_run_kv": (_I, [_P, _P, _I, _P]),
        "orc_model_set_q8k_inputs": (None, [_P, _P, _I, _I]),
        "orc_model_capture_q8k_inputs": (None, [_P, _P, _I, _I]),
        "orc_model_q8k_input_stats": (None, [_P, C.POINTER(C.c_longlong), C.POINTER(C.c_longlong), C.POINTER(C.c_float)]),
        "orc_generate_greedy": (_I, [_P, _P, _I, _I, _P, _P]),
        "orc_num_threads": (_I, []),
        "orc_rng_seed": (C.c_uint64, [C.c_uint64]),
        "orc_rng_next_f32": (C.c_float, [C.POINTER(C.c_uint64)]),
        "orc_sample_token": (_I, [_P, _I, C.POINTER(OrcSamplingConfig), _P, _I, C.POINTER(C.c_uint64), _P]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def _p(a):
    return a.ctypes.data if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


# ── numpy-level wrappers ──────────────────────────────────────────────────────

def f16_to_f32(bits: int) -> float:
    return load().orc_f16_to_f32(bits)


def f16_to_f32_array(bits: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(bits, np.uint16)
    out = np.empty(bits.size, np.float32)
    load().orc_f16_to_f32_array(_p(bits), bits.size, _p(out))
    return out


def dequant_q8_0(blocks: np.ndarray) -> np.ndarray:
    nb = blocks.size // 34
    out = np.empty(nb * 32, np.float32)
    load().orc_dequant_q8_0(_p(blocks), nb, _p(out))
    return out


def dequant_q4_k(blocks: np.ndarray) -> np.ndarray:
    nb = blocks.size // 144
    out = np.empty(nb * 256, np.float32)
    load().orc_dequant_q4_k(_p(blocks), nb, _p(out))
    return out


def dequant_q6_k(blocks: np.ndarray) -> np.ndarray:
    nb = blocks.size // 210
    out = np.empty(nb * 256, np.float32)
    load().orc_dequant_q6_k(_p(blocks), nb, _p(out))
    return out


def quantize_q8_k(x: np.ndarray):
    """(q int8[256], act_d, bsums int32[16]) of one 256-wide block."""
    x = np.ascontiguousarray(x, np.float32)
    q, d, bs = np.empty(256, np.int8), np.empty(1, np.float32), np.empty(16, np.int32)
    load().orc_quantize_q8_k(_p(x), _p(q), _p(d), _p(bs))
    return q, float(d[0]), bs


def _gemv_k(fn, x, w, M, K, N):
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.uint8)
    out = np.empty((M, N), np.float32)
    fn(_p(x), _p(w), _p(out), M, K, N)
    return out


def gemv_q4_k(x, w, M, K, N):
    return _gemv_k(load().orc_gemv_q4_k, x, w, M, K, N)


def gemv_q6_k(x, w, M, K, N):
    return _gemv_k(load().orc_gemv_q6_k, x, w, M, K, N)


def dequant_q4_0(blocks: np.ndarray) -> np.ndarray:
    nb = blocks.size // 18
    out = np.empty(nb * 32, np.float32)
    load().orc_dequant_q4_0(_p(blocks), nb, _p(out))
    return out


def matmul_f32_bf16(x, w_kn_bits, M, K, N):
    x = _f32(x)
    out = np.empty((M, N), np.float32)
    load().orc_matmul_f32_bf16(_p(x), _p(w_kn_bits), _p(out), M, K, N)
    return out


def matmul_f32_f32(x, w_kn, M, K, N):
    x, w_kn = _f32(x), _f32(w_kn)
    out = np.empty((M, N), np.float32)
    load().orc_matmul_f32_f32(_p(x), _p(w_kn), _p(out), M, K, N)
    return out


def matmul_bf16_bf16(a_bits, b_bits, M, K, N):
    out = np.empty((M, N), np.float32)
    load().orc_matmul_bf16_bf16(_p(a_bits), _p(b_bits), _p(out), M, K, N)
    return out


def gemv_q8_0(x, blocks, M, K, N):
    x = _f32(x)
    out = np.empty((M, N), np.float32)
    load().orc_gemv_q8_0(_p(x), _p(blocks), _p(out), M, K, N)
    return out


def gemv_q4_0(x, blocks, M, K, N):
    x = _f32(x)
    out = np.empty((M, N), np.float32)
    load().orc_gemv_q4_0(_p(x), _p(blocks), _p(out), M, K, N)
    return out


def rms_norm(x, w, eps, variant="f32"):
    x, w = _f32(x), _f32(w)
    rows, dim = x.reshape(-1, x.shape[-1]).shape
    out = np.empty_like(x)
    fn = {"f32": "orc_rms_norm", "f64acc": "orc_rms_norm_f64acc", "f64mean": "orc_rms_norm_f64mean"}[variant]
    getattr(load(), fn)(_p(x), _p(w), _p(out), rows, dim, eps)
    return out


def silu_mul(g, u):
    g, u = _f32(g), _f32(u)
    out = np.empty_like(g)
    load().orc_silu_mul(_p(g), _p(u), _p(out), g.size)
    return out


def softmax(x, f64acc=False):
    x = _f32(x)
    rows, n = x.reshape(-1, x.shape[-1]).shape
    out = np.empty_like(x)
    (load().orc_softmax_f64acc if f64acc else load().orc_softmax)(_p(x), _p(out), rows, n)
    return out


def rope_tables(head_dim, max_pos, theta):
    cos = np.empty((max_pos, head_dim), np.float32)
    sin = np.empty((max_pos, head_dim), np.float32)
    load().orc_rope_tables(head_dim, max_pos, theta, _p(cos), _p(sin))
    return cos, sin


def causal_mask(seq, past):
    m = np.empty((seq, seq + past), np.float32)
    load().orc_causal_mask(seq, past, _p(m))
    return m


def rope_half(x, cos, sin):
    """x [S][heads][hd]; cos/sin [S][hd]. Returns a rotated copy."""
    x = _f32(x).copy()
    S, heads, hd = x.shape
    cos, sin = _f32(cos), _f32(sin)
    load().orc_rope_half(_p(x), _p(cos), _p(sin), S, heads, hd)
    return x


def embed(ids, table):
    ids = np.ascontiguousarray(ids, np.int64)
    table = _f32(table)
    out = np.empty((ids.size, table.shape[1]), np.float32)
    load().orc_embed(_p(ids), ids.size, _p(table), table.shape[1], _p(out))
    return out


class Rng:
    """The reference's seedable xorshift64 (src/generate.rs:609-642)."""

    def __init__(self, seed: int):
        self.state = C.c_uint64(load().orc_rng_seed(seed))

    def next_f32(self) -> float:
        return float(load().orc_rng_next_f32(C.byref(self.state)))


def sample_token(logits, cfg: "OrcSamplingConfig", generated, rng: Rng, want_margins=False):
    """reference sample_token (src/generate.rs:698-801). Returns the token, or (token, (draw margin,
    top_p margin)) with want_margins."""
    logits = _f32(logits).reshape(-1)
    gen = np.ascontiguousarray(generated, np.uint32).reshape(-1)
    m = np.empty(2, np.float32)
    tok = load().orc_sample_token(_p(logits), logits.size, C.byref(cfg), _p(gen) if gen.size else None, gen.size,
                                  C.byref(rng.state), _p(m) if want_margins else None)
    return (tok, (float(m[0]), float(m[1]))) if want_margins else tok


def argmax_last(v):
    v = _f32(v)
    return load().orc_argmax_last(_p(v), v.size)


def gqa_attention(q, k, v, mask, head_stride=None, f64_softmax=False):
    """q [S][H][hd]; k, v [kvh][rows][hd] f32 of which the first `total` = mask.shape[1] rows
    are attended; returns [S][H*hd]."""
    q, k, v, mask = _f32(q), _f32(k), _f32(v), _f32(mask)
    S, H, hd = q.shape
    kvh = k.shape[0]
    total = mask.shape[1]
    if head_stride is None:
        head_stride = k.shape[1] * hd
    out = np.empty((S, H * hd), np.float32)
    scratch = np.empty(H * S * total, np.float32)
    load().orc_gqa_attention(_p(q), _p(k), _p(v), _p(mask), _p(out), S, H, kvh, hd, total,
                             head_stride, int(f64_softmax), _p(scratch))
    return out


class KvCache:
    """The reference's KvCache (src/runtime.rs:355-650) as restated by the oracle."""

    def __init__(self, layers, heads, max_len, hd, round_bf16=False):
        self.lib = load()
        self.layers, self.heads, self.max_len, self.hd = layers, heads, max_len, hd
        self.h = self.lib.orc_kv_new(layers, heads, max_len, hd, int(round_bf16))

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.orc_kv_free(self.h)
            self.h = None

    def append_key(self, layer, new_k):
        a = _f32(new_k)
        return self.lib.orc_kv_append_key(self.h, layer, _p(a), a.shape[-2])

    def append_value(self, layer, new_v):
        a = _f32(new_v)
        return self.lib.orc_kv_append_value(self.h, layer, _p(a), a.shape[-2])

    def advance_by(self, n):
        self.lib.orc_kv_advance_by(self.h, n)

    def reset(self, n=0):
        self.lib.orc_kv_reset(self.h, n)

    def current_len(self):
        return self.lib.orc_kv_current_len(self.h)

    def view(self, layer):
        n = self.current_len()
        k = np.empty((1, self.heads, n, self.hd), np.float32)
        v = np.empty((1, self.heads, n, self.hd), np.float32)
        self.lib.orc_kv_view_copy(self.h, layer, _p(k), _p(v))
        return k, v

    def init_from(self, layer, k, v, seq_len):
        k, v = _f32(k), _f32(v)
        return self.lib.orc_kv_init_from(self.h, layer, _p(k), _p(v), seq_len)


class Model:
    """Whole-model oracle: weights in TransformerWeights::to_slot_buffers order."""

    def __init__(self, hidden, inter, heads, kv_heads, head_dim, layers, vocab, eps,
                 weight_kind=W_BF16, has_qk_norm=True, rope_theta=1e6, max_pos=2048,
                 max_seq_len=2048, round_kv_bf16=True):
        self.lib = load()
        self.cfg = OrcConfig(hidden, inter, heads, kv_heads, head_dim, layers, vocab, eps,
                             weight_kind, int(has_qk_norm))
        self.h = self.lib.orc_model_new(C.byref(self.cfg))
        self.vocab = vocab
        self._keep = []  # numpy arrays the C side points into
        self.cos, self.sin = rope_tables(head_dim, max_pos, rope_theta)
        self.max_pos = max_pos
        self.kv = KvCache(layers, kv_heads, max_seq_len, head_dim, round_bf16=round_kv_bf16)
        self.lib.orc_model_attach_kv(self.h, self.kv.h)

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.orc_model_free(self.h)
            self.h = None

    def _hold(self, a):
        if a is None:
            return None
        a = np.ascontiguousarray(a)
        self._keep.append(a)
        return a.ctypes.data

    def set_global(self, embed, final_norm, lm_head):
        self.lib.orc_model_set_global(self.h, self._hold(_f32(embed)), self._hold(_f32(final_norm)),
                                      self._hold(lm_head), _p(self.cos), _p(self.sin), self.max_pos)

    def set_layer(self, l, input_ln, q, k, v, q_norm, k_norm, o, post_ln, gate, up, down):
        args = [self._hold(_f32(input_ln)), self._hold(q), self._hold(k), self._hold(v),
                self._hold(_f32(q_norm)) if q_norm is not None else None,
                self._hold(_f32(k_norm)) if k_norm is not None else None,
                self._hold(o), self._hold(_f32(post_ln)), self._hold(gate), self._hold(up),
                self._hold(down)]
        self.lib.orc_model_set_layer(self.h, l, *args)

    def set_layer_bias(self, l, q_bias, k_bias, v_bias):
        self.lib.orc_model_set_layer_bias(self.h, l, self._hold(_f32(q_bias)), self._hold(_f32(k_bias)),
                                          self._hold(_f32(v_bias)))

    def set_layer_kinds(self, l, kinds):
        """W_* of q, k, v, o, gate, up, down for a layer whose projections differ in block type."""
        assert len(kinds) == 7
        self.lib.orc_model_set_layer_kinds(self.h, l, (C.c_int * 7)(*[int(k) for k in kinds]))

    def q8k_inputs_size(self, rows):
        """Floats of the activation rows that the K-quant products of `rows` cache positions quantise
        (per layer: q|k|v input, o input, gate|up input, down input)."""
        c = self.cfg
        return c.layers * rows * (2 * c.hidden + c.heads * c.head_dim + c.inter)

    def set_q8k_inputs(self, rows_f32, rows, base_pos):
        """K-quant products of cache positions [base_pos, base_pos + rows) quantise these rows instead of
        the model's own (None switches it off). See orc_model_set_q8k_inputs."""
        if rows_f32 is None:
            self.lib.orc_model_set_q8k_inputs(self.h, None, 0, 0)
            return
        a = np.ascontiguousarray(rows_f32, np.float32).reshape(-1)
        assert a.size == self.q8k_inputs_size(rows)
        self._q8k_rows = a
        self.lib.orc_model_set_q8k_inputs(self.h, _p(a), rows, base_pos)

    def capture_q8k_inputs(self, rows, base_pos):
        """The model's own rows of those positions are written to the returned array as it runs."""
        a = np.zeros(self.q8k_inputs_size(rows), np.float32)
        self._q8k_rows = a
        self.lib.orc_model_capture_q8k_inputs(self.h, _p(a), rows, base_pos)
        return a

    def q8k_input_stats(self):
        """(blocks quantised from handed-in rows, values the model's own rows would have rounded
        differently, largest |own - given| / amax of a block)"""
        b, f, d = C.c_longlong(0), C.c_longlong(0), C.c_float(0)
        self.lib.orc_model_q8k_input_stats(self.h, C.byref(b), C.byref(f), C.byref(d))
        return b.value, f.value, d.value

    def run_kv(self, ids):
        ids = np.ascontiguousarray(ids, np.int64).reshape(-1)
        logits = np.empty((ids.size, self.vocab), np.float32)
        rc = self.lib.orc_model_run_kv(self.h, _p(ids), ids.size, _p(logits))
        if rc != 0:
            raise RuntimeError("KV cache full")
        return logits

    def generate_greedy(self, prompt, n_new):
        prompt = np.ascontiguousarray(prompt, np.int64).reshape(-1)
        toks = np.empty(n_new, np.int32)
        margins = np.empty(n_new, np.float32)
        rc = self.lib.orc_generate_greedy(self.h, _p(prompt), prompt.size, n_new, _p(toks),
                                          _p(margins))
        if rc != n_new:
            raise RuntimeError(f"oracle generate returned {rc}")
        return toks, margins


def num_threads() -> int:
    return load().orc_num_threads()
