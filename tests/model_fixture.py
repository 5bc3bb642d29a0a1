"""Shared by the model-level tests, the smoke check and the benchmark's CPU-baseline leg:
builds the CPU oracle's model from the same synthetic weights the GPU model gets."""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

from homura_amd import synth, synth_model  # noqa: E402
from homura_amd.runtime import DTYPE_BF16, DTYPE_Q4_0, DTYPE_Q4_K, DTYPE_Q6_K, DTYPE_Q8_0  # noqa: E402


def build_oracle_model(cfg, weights, max_seq_len, weight_dtype=DTYPE_BF16, has_qk_norm=True, proj_dtypes=None):
    import pyoracle
    kinds = {DTYPE_BF16: pyoracle.W_BF16, DTYPE_Q8_0: pyoracle.W_Q8_0, DTYPE_Q4_0: pyoracle.W_Q4_0,
             DTYPE_Q4_K: pyoracle.W_Q4_K, DTYPE_Q6_K: pyoracle.W_Q6_K}
    kind = kinds[proj_dtypes[0] if proj_dtypes is not None else weight_dtype]
    m = pyoracle.Model(cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads, cfg.kv_heads(),
                       cfg.get_head_dim(), cfg.num_hidden_layers, cfg.vocab_size, cfg.rms_norm_eps,
                       weight_kind=kind, has_qk_norm=has_qk_norm, rope_theta=cfg.rope_theta,
                       max_pos=cfg.max_position_embeddings, max_seq_len=max_seq_len, round_kv_bf16=True)
    w = dict(weights)
    m.set_global(w["model.embed_tokens.weight"], w["model.norm.weight"], w["lm_head.weight"])
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        m.set_layer(l, w[p + "input_layernorm.weight"], w[p + "self_attn.q_proj.weight"],
                    w[p + "self_attn.k_proj.weight"], w[p + "self_attn.v_proj.weight"],
                    w.get(p + "self_attn.q_norm.weight"), w.get(p + "self_attn.k_norm.weight"),
                    w[p + "self_attn.o_proj.weight"], w[p + "post_attention_layernorm.weight"],
                    w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                    w[p + "mlp.down_proj.weight"])
        if proj_dtypes is not None:
            m.set_layer_kinds(l, [kinds[t] for t in proj_dtypes[7 * l:7 * l + 7]])
        if cfg.attention_bias:
            m.set_layer_bias(l, w[p + "self_attn.q_proj.bias"], w[p + "self_attn.k_proj.bias"],
                             w[p + "self_attn.v_proj.bias"])
    return m


def oracle_init_kv(omodel, kv):
    for l in range(len(kv) // 2):
        assert omodel.kv.init_from(l, kv[2 * l], kv[2 * l + 1], kv[0].shape[2]) == 0


def rel_err(a, b, floor_frac=1e-2):
    """max |a-b| / max(|b|, floor_frac * max|b|).

    Whole-step logits pass through the bf16 rounding of every appended K/V row; where the GPU's
    and the oracle's f32 sums (different order) straddle a rounding boundary the stored row
    differs by one bf16 ulp, which moves logits by ~1e-4 of their scale. Elements smaller than
    1% of the largest logit are therefore measured against that 1% floor."""
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    floor = floor_frac * max(np.abs(b).max(), 1e-30)
    return float(np.max(np.abs(a - b) / np.maximum(np.abs(b), floor)))


def smoke_decode():
    """One small decode through the HIP path on GPU 0 (a shape the whole-step kernel serves, on LDS that has
    been overwritten with NaNs first), checked against the oracle."""
    import homura_amd
    cfg = synth_model.SMALL_WS
    weights = synth_model.synth_weights(cfg, 1234)
    kv = synth_model.synth_kv(cfg, 99, 40)
    prompt = synth.token_ids(5, 4, cfg.vocab_size)
    with homura_amd.Context(0) as ctx:
        print("smoke: device", ctx.device_name(), flush=True)
        ctx.fill_lds()
        gm = synth_model.build_model(ctx, cfg, weights, 128)
        assert gm.whole_step(), "smoke: the whole-step kernel does not serve the smoke shape"
        gm.init_kv_cache(kv, 40)
        om = build_oracle_model(cfg, weights, 128)
        oracle_init_kv(om, kv)
        want_logits = om.run_kv(prompt[:1])
        got_logits = gm.run_kv(prompt[:1])
        err = rel_err(got_logits, want_logits)
        assert err < 1e-2, f"smoke: logits differ from the oracle (rel err {err})"
        want, margins = om.generate_greedy(prompt[1:], 8)
        got = gm.generate_greedy(prompt[1:], 8)
        assert np.array_equal(got, want), f"smoke: tokens {got} != oracle {want}"
        gm.close()
    print(f"smoke: ok (logit rel err {err:.2e}, 8 greedy tokens identical, min margin {margins.min():.3e})",
          flush=True)
