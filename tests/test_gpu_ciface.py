"""The reference's own kernel ABI (`_mlir__mlir_ciface_k{idx}(void **args)` with memref
descriptors, reference src/runtime.rs:654-698, :930-1037) driven the way ExecutionPlan::run_kv
drives it (src/runtime.rs:1580-1892): kernels in plan order, K/V appended into an f32 cache
[1, kvh, max, hd] and handed on as strided views (src/runtime.rs:521-625)."""
from __future__ import annotations

import ctypes as C

import numpy as np
import pytest

import model_fixture as mf
from homura_amd import _ffi, synth, synth_model

pytestmark = pytest.mark.gpu


def say(msg):
    print(f"[ciface] {msg}", flush=True)


class Desc:
    """A rank-N memref descriptor plus the pointer-to-pointer the ABI wants."""

    def __init__(self, ptr: int, shape, strides=None):
        n = len(shape)
        if strides is None:
            strides, acc = [0] * n, 1
            for i in reversed(range(n)):
                strides[i] = acc
                acc *= shape[i]
        self.raw = (C.c_int64 * (3 + 2 * n))(ptr, ptr, 0, *shape, *strides)
        self.p = C.c_void_p(C.addressof(self.raw))

    def arg(self):
        return C.cast(C.pointer(self.p), C.c_void_p)


def call(lib, idx, descs):
    args = (C.c_void_p * len(descs))(*[d.arg() for d in descs])
    fn = getattr(lib, f"_mlir__mlir_ciface_k{idx}")
    fn.restype, fn.argtypes = None, [C.c_void_p]
    fn(C.cast(args, C.c_void_p))


# Tokens per call: the reference's prefill hands the whole prompt to the kernels (src/hf/model.rs:321-336),
# its decode one token; eleven rows take the matrix products through more than one block of eight rows, and
# sixty-four through the matrix-core GEMMs.
CHUNKS = [5, 1, 11, 64]


def check_rows(which, got, want, tol=1e-2):
    """Logits of one call against the oracle's batched run_kv over the same tokens. Calls of 16 tokens or more
    run on the matrix cores like the prompt pass and are held to the prompt-pass tests' bound: 2e-3 of the
    logit scale (K/V elements that land on the other side of a bf16 rounding boundary move small logits by
    ~1e-4 of the scale, which the element-wise metric of the shorter calls counts as 1e-2)."""
    for r in range(len(want)):
        if len(want) >= 16:
            err = float(np.abs(np.asarray(got[r], np.float64) - want[r]).max() / np.abs(want[r]).max())
            say(f"{which}: row {r} of {len(want)} logits err / logit scale {err:.2e}")
            assert err < 2e-3
        else:
            err = mf.rel_err(got[r], want[r])
            say(f"{which}: row {r} of {len(want)} logits rel err {err:.2e}")
            assert err < tol
        assert int(len(got[r]) - 1 - np.argmax(got[r][::-1])) == int(len(want[r]) - 1 - np.argmax(want[r][::-1]))


@pytest.mark.parametrize("which", ["qwen3_qknorm", "qwen2_bias"])
def test_plan_through_memref_entry_points(ctx, which):
    qkn = which == "qwen3_qknorm"
    cfg = synth_model.TINY if qkn else synth_model.TINY_QWEN2
    weights = synth_model.synth_weights(cfg, 314, has_qk_norm=qkn)
    W = dict(weights)
    L, hidden, inter, vocab = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    H, kvh, hd = cfg.num_attention_heads, cfg.kv_heads(), cfg.get_head_dim()
    max_len, past, chunks = 128, 9, CHUNKS
    SM = max(chunks)
    om = mf.build_oracle_model(cfg, weights, max_len, has_qk_norm=qkn)
    kv = synth_model.synth_kv(cfg, 12, past)
    mf.oracle_init_kv(om, kv)

    lib = C.CDLL(str(_ffi.LIB_PATH))
    ccfg = cfg.to_c()
    ctx._check(ctx.lib.hm_ciface_bind_transformer(ctx.h, C.byref(ccfg), int(qkn)))
    assert ctx.lib.hm_ciface_num_kernels() == 3 * L + 2

    dev = {n: ctx.to_device(a) for n, a in weights}     # the reference's slot buffers, as they are
    cos, sin = om.cos, om.sin                            # [max_pos, hd] tables (precompute_rope_cos_sin)
    cache = []
    for l in range(2 * L):                               # f32 caches [1, kvh, max_len, hd]
        full = np.zeros((kvh, max_len, hd), np.float32)
        full[:, :past] = kv[l][0]
        cache.append(ctx.to_device(full))
    d_h = [ctx.empty(SM * hidden), ctx.empty(SM * hidden)]
    d_q, d_k, d_v = ctx.empty(SM * H * hd), ctx.empty(SM * kvh * hd), ctx.empty(SM * kvh * hd)
    d_attn, d_logits = ctx.empty(SM * hidden), ctx.empty(SM * vocab)
    d_mask = ctx.empty(SM * max_len)
    ids = synth.token_ids(21, sum(chunks), vocab)
    cur, t0 = past, 0
    ctx.lib.hm_ciface_clear_status()
    for S in chunks:
        say(f"{which}: {S} token(s) at position {cur}")
        d_ids = ctx.to_device(ids[t0:t0 + S].astype(np.int64))
        d_cos, d_sin = ctx.to_device(cos[cur:cur + S]), ctx.to_device(sin[cur:cur + S])
        call(lib, 0, [Desc(d_ids.ptr, [1, S]), Desc(dev["model.embed_tokens.weight"].ptr, [vocab, hidden]),
                      Desc(d_h[0].ptr, [1, S, hidden])])
        for l in range(L):
            p = f"model.layers.{l}."
            qkv_in = [Desc(d_h[0].ptr, [1, S, hidden]), Desc(dev[p + "input_layernorm.weight"].ptr, [hidden]),
                      Desc(dev[p + "self_attn.q_proj.weight"].ptr, [hidden, H * hd])]
            if cfg.attention_bias:
                qkv_in.append(Desc(dev[p + "self_attn.q_proj.bias"].ptr, [H * hd]))
            qkv_in.append(Desc(dev[p + "self_attn.k_proj.weight"].ptr, [hidden, kvh * hd]))
            if cfg.attention_bias:
                qkv_in.append(Desc(dev[p + "self_attn.k_proj.bias"].ptr, [kvh * hd]))
            qkv_in.append(Desc(dev[p + "self_attn.v_proj.weight"].ptr, [hidden, kvh * hd]))
            if cfg.attention_bias:
                qkv_in.append(Desc(dev[p + "self_attn.v_proj.bias"].ptr, [kvh * hd]))
            qkv_in += [Desc(d_cos.ptr, [S, hd]), Desc(d_sin.ptr, [S, hd])]
            if qkn:
                qkv_in += [Desc(dev[p + "self_attn.q_norm.weight"].ptr, [hd]),
                           Desc(dev[p + "self_attn.k_norm.weight"].ptr, [hd])]
            outs = [Desc(d_q.ptr, [1, S, H, hd]), Desc(d_k.ptr, [1, kvh, S, hd]), Desc(d_v.ptr, [1, kvh, S, hd])]
            call(lib, 3 * l + 1, qkv_in + outs)
            # NativeOp::Concat on the cache: S rows per kv head from row `cur`
            for which_kv, src in ((0, d_k), (1, d_v)):
                c = cache[2 * l + which_kv]
                for h in range(kvh):
                    ctx._check(ctx.lib.hm_copy(ctx.h, c.ptr + ((h * max_len + cur) * hd) * 4,
                                               src.ptr + h * S * hd * 4, S * hd * 4))
            view = lambda c: Desc(c.ptr, [1, kvh, cur + S, hd], [kvh * max_len * hd, max_len * hd, hd, 1])
            call(lib, 3 * l + 2, [Desc(d_q.ptr, [1, S, H, hd]), view(cache[2 * l]), view(cache[2 * l + 1]),
                                  Desc(d_mask.ptr, [1, 1, S, cur + S]),
                                  Desc(dev[p + "self_attn.o_proj.weight"].ptr, [H * hd, hidden]),
                                  Desc(d_attn.ptr, [1, S, hidden])])
            call(lib, 3 * l + 3, [Desc(d_h[0].ptr, [1, S, hidden]), Desc(d_attn.ptr, [1, S, hidden]),
                                  Desc(dev[p + "post_attention_layernorm.weight"].ptr, [hidden]),
                                  Desc(dev[p + "mlp.gate_proj.weight"].ptr, [hidden, inter]),
                                  Desc(dev[p + "mlp.up_proj.weight"].ptr, [hidden, inter]),
                                  Desc(dev[p + "mlp.down_proj.weight"].ptr, [inter, hidden]),
                                  Desc(d_h[1].ptr, [1, S, hidden])])
            d_h.reverse()
        call(lib, 3 * L + 1, [Desc(d_h[0].ptr, [1, S, hidden]), Desc(dev["model.norm.weight"].ptr, [hidden]),
                              Desc(dev["lm_head.weight"].ptr, [hidden, vocab]), Desc(d_logits.ptr, [1, S, vocab])])
        check_rows(which, d_logits.download(np.float32)[:S * vocab].reshape(S, vocab), om.run_kv(ids[t0:t0 + S]))
        cur += S
        t0 += S
    assert ctx.lib.hm_ciface_last_status(None) == 0
    ctx.lib.hm_ciface_unbind()


@pytest.mark.parametrize("which", ["q8_0", "q4_k_m_mix", "q4_0_bias"])
def test_quantised_plan_through_memref_entry_points(ctx, which):
    """emit_transformer_plan_quant's kernels (reference src/hf/emitter_quant.rs:1170-1440) in plan
    order: k0 Embed, thirteen kernels per layer, the f32 LMHead."""
    import dataclasses
    if which == "q8_0":
        cfg, mix = synth_model.TINY_LLAMA, [2] * 7 * synth_model.TINY_LLAMA.num_hidden_layers
    elif which == "q4_0_bias":
        cfg = dataclasses.replace(synth_model.TINY_LLAMA, attention_bias=True)
        mix = [3] * 7 * cfg.num_hidden_layers
    else:
        cfg, mix = synth_model.TINY_K, synth_model.q4_k_m_mix(synth_model.TINY_K)
    weights = synth_model.synth_weights(cfg, 271, has_qk_norm=False, proj_dtypes=mix)
    L, hidden, inter, vocab = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    H, kvh, hd = cfg.num_attention_heads, cfg.kv_heads(), cfg.get_head_dim()
    qd, kvd = H * hd, kvh * hd
    max_len, past, chunks = 128, 9, CHUNKS
    SM = max(chunks)
    om = mf.build_oracle_model(cfg, weights, max_len, has_qk_norm=False, proj_dtypes=mix)
    kv = synth_model.synth_kv(cfg, 12, past)
    mf.oracle_init_kv(om, kv)

    lib = C.CDLL(str(_ffi.LIB_PATH))
    ccfg = cfg.to_c()
    arr = (C.c_int * len(mix))(*mix)
    ctx._check(ctx.lib.hm_ciface_bind_transformer_quant(ctx.h, C.byref(ccfg), arr, 0))
    assert ctx.lib.hm_ciface_num_kernels() == 13 * L + 2

    dev = {n: ctx.to_device(a) for n, a in weights}     # the reference's slot buffers, as they are
    cos, sin = om.cos, om.sin
    cache = []
    for l in range(2 * L):                               # f32 caches [1, kvh, max_len, hd]
        full = np.zeros((kvh, max_len, hd), np.float32)
        full[:, :past] = kv[l][0]
        cache.append(ctx.to_device(full))
    f = lambda n: ctx.empty(SM * n)
    d_h = [f(hidden), f(hidden)]
    d_normed, d_qr, d_kr, d_vr = f(hidden), f(qd), f(kvd), f(kvd)
    d_q, d_k, d_v, d_body, d_attn = f(qd), f(kvd), f(kvd), f(qd), f(hidden)
    d_resid, d_pnorm, d_gate, d_up, d_silu, d_down = f(hidden), f(hidden), f(inter), f(inter), f(inter), f(hidden)
    d_logits, d_mask = f(vocab), f(max_len)
    ids = synth.token_ids(21, sum(chunks), vocab)
    cur, t0 = past, 0
    ctx.lib.hm_ciface_clear_status()
    # K-quant products quantise their activation to Q8_K, a step function: the oracle is handed the rows the
    # GPU's QuantMM calls were given (they pass through this driver anyway), so both sides round the same
    # values and a decision that 1e-6 of summation noise would flip cannot pose as an error; the oracle
    # counts such flips and reports how far its own rows are from the GPU's (tests/test_oracle_model.py
    # pins the device).
    kquant = any(t in (5, 6) for t in mix)
    n_rows = sum(chunks)
    gdim = (hidden, qd, hidden, inter)
    per_layer = n_rows * sum(gdim)
    handed = np.zeros(L * per_layer, np.float32)
    flips = blocks = 0
    maxdiff = 0.0

    def hand_in(l, group, buf, S):
        off = l * per_layer + n_rows * sum(gdim[:group]) + t0 * gdim[group]
        handed[off:off + S * gdim[group]] = buf.download(np.float32)[:S * gdim[group]]

    for S in chunks:
        row = lambda buf, n: Desc(buf.ptr, [1, S, n])
        say(f"quant {which}: {S} token(s) at position {cur}")
        d_ids = ctx.to_device(ids[t0:t0 + S].astype(np.int64))
        d_cos, d_sin = ctx.to_device(cos[cur:cur + S]), ctx.to_device(sin[cur:cur + S])
        call(lib, 0, [Desc(d_ids.ptr, [1, S]), Desc(dev["model.embed_tokens.weight"].ptr, [vocab, hidden]), row(d_h[0], hidden)])
        for l in range(L):
            p, k0 = f"model.layers.{l}.", 13 * l + 1
            w = lambda name: Desc(dev[p + name].ptr, [dev[p + name].nbytes])      # flat bytes
            vec = lambda name, n: Desc(dev[p + name].ptr, [n])
            call(lib, k0 + 0, [row(d_h[0], hidden), vec("input_layernorm.weight", hidden), row(d_normed, hidden)])
            hand_in(l, 0, d_normed, S)
            call(lib, k0 + 1, [row(d_normed, hidden), w("self_attn.q_proj.weight"), row(d_qr, qd)])
            call(lib, k0 + 2, [row(d_normed, hidden), w("self_attn.k_proj.weight"), row(d_kr, kvd)])
            call(lib, k0 + 3, [row(d_normed, hidden), w("self_attn.v_proj.weight"), row(d_vr, kvd)])
            post = [row(d_qr, qd), row(d_kr, kvd), row(d_vr, kvd)]
            if cfg.attention_bias:
                post += [vec("self_attn.q_proj.bias", qd), vec("self_attn.k_proj.bias", kvd), vec("self_attn.v_proj.bias", kvd)]
            post += [Desc(d_cos.ptr, [S, hd]), Desc(d_sin.ptr, [S, hd])]
            post += [Desc(d_q.ptr, [1, S, H, hd]), Desc(d_k.ptr, [1, kvh, S, hd]), Desc(d_v.ptr, [1, kvh, S, hd])]
            call(lib, k0 + 4, post)
            for which_kv, src in ((0, d_k), (1, d_v)):   # NativeOp::Concat on the cache
                c = cache[2 * l + which_kv]
                for h in range(kvh):
                    ctx._check(ctx.lib.hm_copy(ctx.h, c.ptr + ((h * max_len + cur) * hd) * 4, src.ptr + h * S * hd * 4, S * hd * 4))
            view = lambda c: Desc(c.ptr, [1, kvh, cur + S, hd], [kvh * max_len * hd, max_len * hd, hd, 1])
            call(lib, k0 + 5, [Desc(d_q.ptr, [1, S, H, hd]), view(cache[2 * l]), view(cache[2 * l + 1]),
                               Desc(d_mask.ptr, [1, 1, S, cur + S]), row(d_body, qd)])
            hand_in(l, 1, d_body, S)
            call(lib, k0 + 6, [row(d_body, qd), w("self_attn.o_proj.weight"), row(d_attn, hidden)])
            call(lib, k0 + 7, [row(d_h[0], hidden), row(d_attn, hidden), vec("post_attention_layernorm.weight", hidden),
                               row(d_resid, hidden), row(d_pnorm, hidden)])
            hand_in(l, 2, d_pnorm, S)
            call(lib, k0 + 8, [row(d_pnorm, hidden), w("mlp.gate_proj.weight"), row(d_gate, inter)])
            call(lib, k0 + 9, [row(d_pnorm, hidden), w("mlp.up_proj.weight"), row(d_up, inter)])
            call(lib, k0 + 10, [row(d_gate, inter), row(d_up, inter), row(d_silu, inter)])
            hand_in(l, 3, d_silu, S)
            call(lib, k0 + 11, [row(d_silu, inter), w("mlp.down_proj.weight"), row(d_down, hidden)])
            call(lib, k0 + 12, [row(d_resid, hidden), row(d_down, hidden), row(d_h[1], hidden)])
            d_h.reverse()
        call(lib, 13 * L + 1, [row(d_h[0], hidden), Desc(dev["model.norm.weight"].ptr, [hidden]),
                               Desc(dev["lm_head.weight"].ptr, [hidden, vocab]), row(d_logits, vocab)])
        if kquant:
            om.set_q8k_inputs(handed, n_rows, past)
        check_rows(f"quant {which}", d_logits.download(np.float32)[:S * vocab].reshape(S, vocab), om.run_kv(ids[t0:t0 + S]),
                   1e-4 if kquant else 1e-2)
        if kquant:
            b_, f_, d_ = om.q8k_input_stats()
            blocks, flips, maxdiff = blocks + b_, flips + f_, max(maxdiff, d_)
        cur += S
        t0 += S
    if kquant:
        say(f"quant {which}: {flips} rounding decisions differ in {blocks} blocks of 256; largest activation distance {maxdiff:.2e}")
        assert blocks > 0 and flips <= max(3, 5 * blocks * 256 // 10000) and maxdiff < 1e-3
    assert ctx.lib.hm_ciface_last_status(None) == 0
    ctx.lib.hm_ciface_unbind()


def test_failing_call_poisons_its_outputs_and_sets_the_status(ctx, capfd):
    """A call that cannot run (here: K/V views shorter than the query rows they must contain) prints a line,
    leaves NaN in every output operand and its code in the sticky status word."""
    cfg = synth_model.TINY
    H, kvh, hd, hidden = cfg.num_attention_heads, cfg.kv_heads(), cfg.get_head_dim(), cfg.hidden_size
    lib = C.CDLL(str(_ffi.LIB_PATH))
    ccfg = cfg.to_c()
    ctx._check(ctx.lib.hm_ciface_bind_transformer(ctx.h, C.byref(ccfg), 1))
    ctx.lib.hm_ciface_clear_status()
    S, T = 4, 2
    d_q, d_kv = ctx.to_device(np.zeros(S * H * hd, np.float32)), ctx.to_device(np.zeros(kvh * 8 * hd, np.float32))
    d_mask, d_ow = ctx.empty(S * T), ctx.to_device(np.zeros(H * hd * hidden, np.uint16))
    d_out = ctx.to_device(np.ones(S * hidden, np.float32))
    view = Desc(d_kv.ptr, [1, kvh, T, hd], [kvh * 8 * hd, 8 * hd, hd, 1])
    call(lib, 2, [Desc(d_q.ptr, [1, S, H, hd]), view, view, Desc(d_mask.ptr, [1, 1, S, T]),
                  Desc(d_ow.ptr, [H * hd, hidden]), Desc(d_out.ptr, [1, S, hidden])])
    assert "K/V views must hold" in capfd.readouterr().err
    assert np.isnan(d_out.download(np.float32)).all()
    idx = C.c_int(-1)
    assert ctx.lib.hm_ciface_last_status(C.byref(idx)) == -1 and idx.value == 2   # HM_ERR_INVALID from kernel 2
    ctx.lib.hm_ciface_clear_status()
    assert ctx.lib.hm_ciface_last_status(None) == 0
    ctx.lib.hm_ciface_unbind()


def test_unbound_call_is_reported_not_fatal(ctx, capfd):
    """No binding: the entry point records an error and returns (the ABI has no status)."""
    ctx.lib.hm_ciface_unbind()
    lib = C.CDLL(str(_ffi.LIB_PATH))
    d = ctx.empty(4)
    call(lib, 5, [Desc(d.ptr, [4])])
    assert "no transformer bound" in capfd.readouterr().err
