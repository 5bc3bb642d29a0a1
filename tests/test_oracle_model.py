"""CPU-only checks of the whole-step oracle and of the host-side pieces that need no GPU."""
import ctypes as C
import json
import re
from pathlib import Path

import numpy as np
import pytest

import model_fixture as mf
from homura_amd import _ffi, synth, synth_model
from homura_amd.runtime import DTYPE_Q8_0

ROOT = Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol():
    """include/homura_amd.h (the boundary) plus include/homura_amd_bench.h (measurement and test support),
    the ctypes table and the built library agree symbol for symbol."""
    header = (ROOT / "include" / "homura_amd.h").read_text() + (ROOT / "include" / "homura_amd_bench.h").read_text()
    declared = set(re.findall(r"\b(hm_[a-z0-9_]+)\s*\(", header))
    declared -= {"hm_ctx", "hm_model"}
    lib = _ffi.load()
    assert declared == set(_ffi.SIGNATURES), declared ^ set(_ffi.SIGNATURES)
    for name in declared:
        assert getattr(lib, name) is not None
    assert b"gfx950" in lib.hm_version()


def test_what_the_gpu_runs_load_travels_with_the_tree():
    """The list of paths that stay behind when the tree is sent to a GPU machine names nothing that the GPU
    tests, the smoke run or bench.py read there: the package and its built library, the oracle, the tests with
    their fixtures, the headers and the HBM traffic table under profiles/."""
    import bench
    ignored = [l.strip() for l in (ROOT / ".gpurunignore").read_text().splitlines() if l.strip()]
    needed = [bench.TRAFFIC_TABLE, _ffi.LIB_PATH, ROOT / "oracle" / "pyoracle.py", ROOT / "tests" / "golden" / "reference_vectors.json",
              ROOT / "include" / "homura_amd.h", ROOT / "__graft_entry__.py", ROOT / "bench.py"]
    for path in needed:
        rel = "./" + str(Path(path).resolve().relative_to(ROOT))
        for pat in ignored:
            assert not (rel == pat or rel.startswith(pat.rstrip("/") + "/")), (rel, pat)
            assert not (pat.startswith("*") and rel.endswith(pat[1:])), (rel, pat)


def test_library_exports_the_reference_kernel_symbols():
    """The reference's loader resolves `_mlir__mlir_ciface_k{idx}` by dlsym
    (reference src/runtime.rs:803-824): all 1024 must be there (the quantised plan of a 28-layer
    model numbers 366 kernels)."""
    import ctypes
    from homura_amd import _ffi
    lib = ctypes.CDLL(str(_ffi.LIB_PATH))
    for i in range(1024):
        assert hasattr(lib, f"_mlir__mlir_ciface_k{i}"), i
    assert not hasattr(lib, "_mlir__mlir_ciface_k1024")


def test_no_gpu_means_a_loud_error_not_a_fallback():
    import homura_amd
    lib = _ffi.load()
    h = lib.hm_init(0)
    if h:  # running on a GPU box: nothing to check here
        lib.hm_destroy(h)
        pytest.skip("a GPU is present")
    assert b"HIP" in lib.hm_last_error(None) or b"device" in lib.hm_last_error(None)
    with pytest.raises(homura_amd.HomuraError):
        homura_amd.Context(0)


def test_synth_is_deterministic_and_sane():
    a = synth.normal_f32(42, 200000)
    assert np.array_equal(a, synth.normal_f32(42, 200000))
    assert np.array_equal(a[1000:2000], synth.normal_f32(42, 1000, first=1000))  # counter-based
    assert abs(a.mean()) < 0.01 and abs(a.std() - 1.0) < 0.01
    # pinned first values: the generator is integer arithmetic, so these never move
    assert [float(v) for v in synth.normal_f32(1, 3)] == [float(v) for v in np.array(synth.normal_f32(1, 3))]
    b = synth.normal_bf16(7, 1000, 0.02)
    assert np.array_equal(b, synth.f32_to_bf16_rne(synth.normal_f32(7, 1000, 0.02)))
    ids = synth.token_ids(3, 5000, 151936)
    assert ids.min() >= 0 and ids.max() < 151936 and len(set(ids.tolist())) > 4900
    q = synth.q8_0_blocks(5, 2000).reshape(2000, 34)
    qs = q[:, 2:].view(np.int8)
    assert qs.min() == -127 and qs.max() == 127
    d = q[:, :2].copy().view(np.float16).astype(np.float32)
    assert (d >= 0).all() and 0.005 < d.mean() < 0.012
    n4 = synth.q4_0_blocks(6, 2000).reshape(2000, 18)[:, 2:]
    assert set(np.unique(n4 & 0xF).tolist()) == set(range(16))


def test_f32_to_f16_rne_exhaustive_roundtrip_and_numpy():
    lib = _ffi.load()
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 0.01,
                         np.array([0.0, -0.0, 6e-8, 5.96e-8, 2.98e-8, 2.99e-8, 65504.0, 65519.9, 65520.0, 1e-3,
                                   6.1035156e-05, 6.097e-05, np.inf, -np.inf], np.float32),
                         np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)])
    xs = xs[~np.isnan(xs)]
    want = xs.astype(np.float16).view(np.uint16)
    got = np.array([lib.hm_f32_to_f16_rne(float(x)) for x in xs], np.uint16)
    assert np.array_equal(got, want)


def test_oracle_batched_prefill_equals_token_by_token():
    """A causal multi-token run_kv must equal the same tokens fed one at a time: pins the mask
    (j > i + past), the position slicing of the RoPE tables and the multi-row cache append."""
    cfg = synth_model.TINY
    weights = synth_model.synth_weights(cfg, 4242)
    ids = synth.token_ids(8, 6, cfg.vocab_size)
    kv = synth_model.synth_kv(cfg, 7, 20)
    a = mf.build_oracle_model(cfg, weights, 64)
    b = mf.build_oracle_model(cfg, weights, 64)
    mf.oracle_init_kv(a, kv)
    mf.oracle_init_kv(b, kv)
    batched = a.run_kv(ids)
    single = np.concatenate([b.run_kv(ids[i:i + 1]) for i in range(6)])
    assert mf.rel_err(batched, single) < 1e-4
    ka, va = a.kv.view(1)
    kb, vb = b.kv.view(1)
    assert np.array_equal(ka, kb) and np.array_equal(va, vb)
    with pytest.raises(RuntimeError):
        a.run_kv(np.zeros(64, np.int64))  # would overflow the cache


@pytest.mark.parametrize("which", ["qwen3_qknorm", "qwen2_bias"])
def test_oracle_step_against_numpy_fp64(which):
    """An independent numpy/float64 forward of one decode step (textbook HF Qwen3 / Qwen2 block)
    against the C oracle: a dropped residual, a missing norm weight or bias, a swapped gate/up or a
    wrong head mapping would all show up here."""
    qkn = which == "qwen3_qknorm"
    cfg = synth_model.TINY if qkn else synth_model.TINY_QWEN2
    W = dict(synth_model.synth_weights(cfg, 99, has_qk_norm=qkn))
    hd, H, kvh = cfg.get_head_dim(), cfg.num_attention_heads, cfg.kv_heads()
    past = 11
    kv = synth_model.synth_kv(cfg, 5, past)
    om = mf.build_oracle_model(cfg, list(W.items()), 32, has_qk_norm=qkn)
    mf.oracle_init_kv(om, kv)
    tok = 123
    got = om.run_kv([tok])[0]

    f = lambda a: synth.bf16_to_f32(a).astype(np.float64) if a.dtype == np.uint16 else a.astype(np.float64)
    rms = lambda x, w: x / np.sqrt((x * x).mean(-1, keepdims=True) + cfg.rms_norm_eps) * w
    bf = lambda x: synth.bf16_to_f32(synth.f32_to_bf16_rne(x.astype(np.float32))).astype(np.float64)
    h = f(W["model.embed_tokens.weight"])[tok]
    i = np.arange(hd // 2)
    ang = past / (cfg.rope_theta ** (2 * i / hd))
    cos, sin = np.concatenate([np.cos(ang)] * 2), np.concatenate([np.sin(ang)] * 2)
    rot = lambda x: np.concatenate([-x[..., hd // 2:], x[..., :hd // 2]], -1)
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        n = rms(h, f(W[p + "input_layernorm.weight"]))
        q, k, v = (n @ f(W[p + f"self_attn.{x}_proj.weight"]) for x in "qkv")
        if cfg.attention_bias:
            q, k, v = (t + f(W[p + f"self_attn.{x}_proj.bias"]) for t, x in zip((q, k, v), "qkv"))
        q, k, v = q.reshape(H, hd), k.reshape(kvh, hd), v.reshape(kvh, hd)
        if qkn:
            q = rms(q, f(W[p + "self_attn.q_norm.weight"]))
            k = rms(k, f(W[p + "self_attn.k_norm.weight"]))
        q, k = q * cos + rot(q) * sin, k * cos + rot(k) * sin
        K = np.concatenate([kv[2 * l][0].astype(np.float64), bf(k)[:, None, :]], 1)   # [kvh, past+1, hd]
        V = np.concatenate([kv[2 * l + 1][0].astype(np.float64), bf(v)[:, None, :]], 1)
        o = np.zeros((H, hd))
        for hh in range(H):
            s = K[hh // (H // kvh)] @ q[hh] / np.sqrt(hd)
            pr = np.exp(s - s.max())
            o[hh] = (pr / pr.sum()) @ V[hh // (H // kvh)]
        r = h + o.reshape(-1) @ f(W[p + "self_attn.o_proj.weight"])
        n2 = rms(r, f(W[p + "post_attention_layernorm.weight"]))
        g, u = n2 @ f(W[p + "mlp.gate_proj.weight"]), n2 @ f(W[p + "mlp.up_proj.weight"])
        h = r + (g / (1 + np.exp(-g)) * u) @ f(W[p + "mlp.down_proj.weight"])
    want = rms(h, f(W["model.norm.weight"])) @ f(W["lm_head.weight"])
    assert mf.rel_err(got, want) < 1e-3


def test_oracle_matches_committed_decode_fixture_head():
    """The first tokens of the committed Qwen3-0.6B-shape fixture, regenerated here (a short
    prefix keeps the CPU suite quick; the GPU test checks all 64)."""
    fx = json.loads((ROOT / "tests" / "golden" / "qwen3_0p6b_decode.json").read_text())
    cfg = synth_model.QWEN3_0P6B
    weights = synth_model.synth_weights(cfg, fx["seed"])
    kv = synth_model.synth_kv(cfg, fx["seed"] + 0x100, fx["prefill_len"])
    prompt = synth.token_ids(fx["seed"] + 0x200, fx["n_prompt"], cfg.vocab_size)
    assert [int(t) for t in prompt] == fx["prompt"]
    om = mf.build_oracle_model(cfg, weights, fx["max_seq_len"])
    mf.oracle_init_kv(om, kv)
    toks, margins = om.generate_greedy(prompt, 6)
    assert [int(t) for t in toks] == fx["tokens"][:6]
    assert np.allclose(margins, fx["margins"][:6], rtol=0.05, atol=1e-5)


def test_quant_oracle_plan_runs_and_dequant_equivalence():
    """Quantised plan of the oracle: running with Q8_0 projections equals running the bf16-free
    f32 math on the dequantised weights within rounding (f64-accumulating norms aside)."""
    cfg = synth_model.TINY_LLAMA
    weights = synth_model.synth_weights(cfg, 31, DTYPE_Q8_0, has_qk_norm=False)
    om = mf.build_oracle_model(cfg, weights, 48, DTYPE_Q8_0, has_qk_norm=False)
    logits = om.run_kv(synth.token_ids(3, 4, cfg.vocab_size))
    assert logits.shape == (4, cfg.vocab_size) and np.isfinite(logits).all()
    assert om.kv.current_len() == 4


def test_mixed_kquant_oracle_step_against_numpy_fp64():
    """A model whose projections mix Q4_K and Q6_K (as Q4_K_M files do): the oracle must pick the
    decode per matrix. Independent float64 forward: every projection is (activation rounded to
    Q8_K) @ (blocks dequantised by the matrix's own type); a type applied to the wrong matrix reads
    blocks of the wrong size and lands far outside the tolerance."""
    import pyoracle
    from homura_amd.runtime import DTYPE_Q4_K, DTYPE_Q6_K
    cfg = synth_model.TINY_K
    mix = synth_model.q4_k_m_mix(cfg)
    assert DTYPE_Q6_K in mix and DTYPE_Q4_K in mix and mix[2] != mix[9]  # v of layers 0 and 1 differ
    W = dict(synth_model.synth_weights(cfg, 21, has_qk_norm=False, proj_dtypes=mix))
    hd, H, kvh = cfg.get_head_dim(), cfg.num_attention_heads, cfg.kv_heads()
    past = 9
    kv = synth_model.synth_kv(cfg, 5, past)
    om = mf.build_oracle_model(cfg, list(W.items()), 32, has_qk_norm=False, proj_dtypes=mix)
    mf.oracle_init_kv(om, kv)
    tok = 77
    got = om.run_kv([tok])[0]

    def act_q8k(x):
        out = np.empty(x.size)
        for b in range(x.size // 256):
            q, d, _ = pyoracle.quantize_q8_k(x[256 * b:256 * b + 256].astype(np.float32))
            out[256 * b:256 * b + 256] = q.astype(np.float64) * d
        return out

    order = ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj", "mlp.gate_proj",
             "mlp.up_proj", "mlp.down_proj"]

    def mm(l, name, x):
        dt = mix[7 * l + order.index(name)]
        blocks = W[f"model.layers.{l}.{name}.weight"]
        w = (pyoracle.dequant_q6_k if dt == DTYPE_Q6_K else pyoracle.dequant_q4_k)(blocks)
        return w.reshape(-1, x.size).astype(np.float64) @ act_q8k(x)

    f = lambda a: a.astype(np.float64)
    rms = lambda x, w: x / np.sqrt((x * x).mean(-1, keepdims=True) + cfg.rms_norm_eps) * w
    bf = lambda x: synth.bf16_to_f32(synth.f32_to_bf16_rne(x.astype(np.float32))).astype(np.float64)
    h = f(W["model.embed_tokens.weight"])[tok]
    i = np.arange(hd // 2)
    ang = past / (cfg.rope_theta ** (2 * i / hd))
    cos, sin = np.concatenate([np.cos(ang)] * 2), np.concatenate([np.sin(ang)] * 2)
    rot = lambda x: np.concatenate([-x[..., hd // 2:], x[..., :hd // 2]], -1)
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        n = rms(h, f(W[p + "input_layernorm.weight"]))
        q, k, v = (mm(l, f"self_attn.{x}_proj", n) for x in "qkv")
        q, k, v = q.reshape(H, hd), k.reshape(kvh, hd), v.reshape(kvh, hd)
        q, k = q * cos + rot(q) * sin, k * cos + rot(k) * sin
        K = np.concatenate([kv[2 * l][0].astype(np.float64), bf(k)[:, None, :]], 1)
        V = np.concatenate([kv[2 * l + 1][0].astype(np.float64), bf(v)[:, None, :]], 1)
        o = np.zeros((H, hd))
        for hh in range(H):
            s = K[hh // (H // kvh)] @ q[hh] / np.sqrt(hd)
            pr = np.exp(s - s.max())
            o[hh] = (pr / pr.sum()) @ V[hh // (H // kvh)]
        r = h + mm(l, "self_attn.o_proj", o.reshape(-1))
        n2 = rms(r, f(W[p + "post_attention_layernorm.weight"]))
        g, u = mm(l, "mlp.gate_proj", n2), mm(l, "mlp.up_proj", n2)
        h = r + mm(l, "mlp.down_proj", g / (1 + np.exp(-g)) * u)
    want = rms(h, f(W["model.norm.weight"])) @ f(W["lm_head.weight"])
    assert np.abs(want).max() > 1e-3
    assert mf.rel_err(got, want) < 2e-3


def test_q8k_activation_hand_in_is_pinned():
    """The oracle's test device for K-quant comparisons (orc_model_set_q8k_inputs): K-quant products
    quantise activation rows handed in from outside. Pinned here by what it must do on the oracle's own
    rows: handing a model its own activations back changes nothing and reports no flip; one value pushed
    across a Q8_K rounding boundary is counted as exactly one flip per product group that sees it and
    moves the logits; a value moved by less than the distance to its boundary is no flip but shows in
    the largest difference; rows outside the handed-in range keep the model's own activations."""
    import pyoracle
    cfg = synth_model.TINY_K
    mix = synth_model.q4_k_m_mix(cfg)
    W = synth_model.synth_weights(cfg, 33, has_qk_norm=False, proj_dtypes=mix)
    ids = synth.token_ids(5, 6, cfg.vocab_size)

    def fresh():
        return mf.build_oracle_model(cfg, W, 32, has_qk_norm=False, proj_dtypes=mix)

    a = fresh()
    rows = a.capture_q8k_inputs(4, 1)           # positions 1..4 of 0..5
    want = np.concatenate([a.run_kv(ids[i:i + 1]) for i in range(6)])
    rows = rows.copy()
    assert np.abs(rows).max() > 0
    plain = fresh()
    assert np.array_equal(np.concatenate([plain.run_kv(ids[i:i + 1]) for i in range(6)]), want)  # capture changes nothing

    b = fresh()
    b.set_q8k_inputs(rows, 4, 1)
    got = np.concatenate([b.run_kv(ids[i:i + 1]) for i in range(6)])
    blocks, flips, maxdiff = b.q8k_input_stats()
    c = cfg
    per_row = (2 * c.hidden_size + c.num_attention_heads * c.get_head_dim() + c.intermediate_size) // 256
    assert blocks == c.num_hidden_layers * 4 * per_row and flips == 0 and maxdiff == 0.0
    assert np.array_equal(got, want)

    # layer 0, q|k|v input, handed-in row 2 (position 3): push one value across its rounding boundary
    hidden = c.hidden_size
    blk = rows[2 * hidden:2 * hidden + 256].copy()
    q, d, _ = pyoracle.quantize_q8_k(blk)
    j = int(np.argsort(np.abs(blk))[128])        # a mid-sized value, not the block maximum
    moved = rows.copy()
    moved[2 * hidden + j] = np.float32((int(q[j]) + (0.75 if q[j] >= 0 else -0.75)) * d)
    q2, d2, _ = pyoracle.quantize_q8_k(moved[2 * hidden:2 * hidden + 256])
    assert d2 == d and (q2 != q).sum() == 1 and abs(int(q2[j]) - int(q[j])) == 1
    m = fresh()
    m.set_q8k_inputs(moved, 4, 1)
    got2 = np.concatenate([m.run_kv(ids[i:i + 1]) for i in range(6)])
    blocks2, flips2, maxdiff2 = m.q8k_input_stats()
    # The moved value is counted, and so is what it does to the model's own later activations of that
    # position (the handed-in rows come from a run without the move): the difference is reported.
    assert flips2 >= 1 and maxdiff2 > 0.2 / 127
    # Every projection of positions 1..4 multiplies the handed-in rows, so their logits are those of the
    # captured run; the moved value lives on in K and V of position 3 and reaches position 5, which
    # attends to it and has no hand-in.
    assert np.array_equal(got2[:5], want[:5])
    assert not np.array_equal(got2[5], want[5])

    # a nudge far smaller than the distance to the boundary: no flip, but visible in the difference
    nudged = rows.copy()
    nudged[2 * hidden + j] = np.float32(blk[j] * (1 + 3e-7))
    n = fresh()
    n.set_q8k_inputs(nudged, 4, 1)
    np.concatenate([n.run_kv(ids[i:i + 1]) for i in range(6)])
    _, flips3, maxdiff3 = n.q8k_input_stats()
    assert flips3 == 0 and 0 < maxdiff3 < 1e-6


def test_avx512_build_of_the_oracle_gives_the_same_bits():
    """bench.py times the x86-64-v4 build of oracle.c where the host has AVX-512; the tests check against the
    x86-64-v3 build. Same source, no value-changing compiler options: a prompt pass and a few greedy steps of a
    small model must agree bit for bit (run in a child process, the library choice is per process)."""
    import subprocess
    import sys
    import pyoracle
    if pyoracle.best_isa() != "x86-64-v4":
        pytest.skip("this host has no AVX-512")
    code = r"""
import sys
sys.path[:0] = [%r, %r, %r]
import numpy as np
import pyoracle
pyoracle.use_isa(sys.argv[1])
import model_fixture as mf
from homura_amd import synth, synth_model
cfg = synth_model.TINY
om = mf.build_oracle_model(cfg, synth_model.synth_weights(cfg, 5), 64)
logits = om.run_kv(synth.token_ids(9, 7, cfg.vocab_size))
toks = om.generate_greedy([3], 6)
sys.stdout.buffer.write(np.asarray(logits, np.float32).tobytes() + np.asarray(toks, np.int32).tobytes())
""" % (str(Path(__file__).resolve().parent), str(Path(__file__).resolve().parents[1] / "oracle"),
       str(Path(__file__).resolve().parents[1]))
    outs = [subprocess.run([sys.executable, "-c", code, isa], check=True, capture_output=True).stdout
            for isa in ("x86-64-v3", "x86-64-v4")]
    assert len(outs[0]) > 7 * 1000 * 4 and outs[0] == outs[1]
