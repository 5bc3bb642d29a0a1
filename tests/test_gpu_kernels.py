"""GPU parity of every kernel-level entry point of the C boundary against the CPU oracle, on the
same seeded inputs. Bit-exact for byte/integer work (dequantisation, KV append, argmax,
embedding); max relative error <= 1e-2 for matmul/attention outputs, where
    rel = |gpu - ref| / max(|ref|, 1e-3 * max|ref|)
(the floor keeps outputs that happen to land near zero from dividing by nothing)."""
import math

import numpy as np
import pytest

from homura_amd import HomuraError, synth

pytestmark = pytest.mark.gpu

TOL = 1e-2


def rel_err(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    floor = 1e-3 * max(np.abs(b).max(), 1e-30)
    return float(np.max(np.abs(a - b) / np.maximum(np.abs(b), floor)))


def say(msg):
    print(msg, flush=True)


# ── bf16 GEMV (reference emit_matmul with bf16 weights) ───────────────────────

@pytest.mark.parametrize("M,K,N", [(1, 896, 4864),   # benchmark configuration 1
                                   (1, 1024, 4096), (1, 3072, 1024), (1, 2048, 1024),
                                   (3, 896, 4864), (5, 1024, 1024), (8, 256, 136),
                                   (1, 40, 12), (2, 8, 8)])
def test_gemv_bf16_both_layouts(ctx, oracle, M, K, N):
    say(f"gemv_bf16 M={M} K={K} N={N}")
    x = synth.normal_f32(synth.SEED_CFG1, M * K).reshape(M, K)
    w = synth.normal_bf16(synth.SEED_CFG1 + 1, K * N, 0.02).reshape(K, N)
    want = oracle.matmul_f32_bf16(x, w, M, K, N)
    dx, dw, dout = ctx.to_device(x), ctx.to_device(w), ctx.empty(M * N)
    ctx.gemv_bf16(dx, dw, dout, M, K, N)
    got = dout.download(np.float32, (M, N))
    assert rel_err(got, want) < TOL
    # a second call must see clean split-K counters
    ctx.gemv_bf16(dx, dw, dout, M, K, N)
    assert np.array_equal(dout.download(np.float32, (M, N)), got)
    if K % 8 == 0:
        dnk, dout2 = ctx.empty(K * N, np.uint16), ctx.empty(M * N)
        ctx.pack_bf16_kn_to_nk(dw, dnk, K, N)
        assert np.array_equal(dnk.download(np.uint16, (N, K)), w.T)  # pure data movement: exact
        ctx.gemv_bf16_nk(dx, dnk, dout2, M, K, N)
        assert rel_err(dout2.download(np.float32, (M, N)), want) < TOL
        dnk.free(); dout2.free()
    for b in (dx, dw, dout):
        b.free()


def test_gemv_bf16_reference_vectors(ctx, golden):
    """The reference's exact matmul vectors (integers are bf16-representable)."""
    g = golden["matmul_2d_known_values"]
    a = np.zeros((2, 8), np.float32)
    b = np.zeros((8, 8), np.float32)
    a[:, :2] = g["a"]
    b[:2, :2] = g["b"]
    bits = (b.view(np.uint32) >> 16).astype(np.uint16)
    dx, dw, dout = ctx.to_device(a), ctx.to_device(bits), ctx.empty(16)
    ctx.gemv_bf16(dx, dw, dout, 2, 8, 8)
    got = dout.download(np.float32, (2, 8))
    assert np.array_equal(got[:, :2], np.array(g["expected"], np.float32))
    assert np.all(got[:, 2:] == 0)


# ── Q8_0 / Q4_0 ───────────────────────────────────────────────────────────────

def test_dequant_bit_exact(ctx, oracle):
    nb = 8192 + 3
    for kind, bb, gen, dq, orc in (("q8_0", 34, synth.q8_0_blocks, ctx.dequant_q8_0, oracle.dequant_q8_0),
                                   ("q4_0", 18, synth.q4_0_blocks, ctx.dequant_q4_0, oracle.dequant_q4_0)):
        say(f"dequant {kind}")
        raw = gen(77, nb)
        blk = raw.reshape(nb, bb)
        # scales that exercise f16 subnormals, zero, max, inf and NaN
        for i, bits in enumerate([0x0001, 0x03FF, 0x0000, 0x8000, 0x7BFF, 0x7C00, 0xFC00, 0x7E00, 0x0400]):
            blk[i, 0], blk[i, 1] = bits & 0xFF, bits >> 8
        want = orc(raw)
        d_in, d_out = ctx.to_device(raw), ctx.empty(nb * 32)
        dq(d_in, d_out, nb)
        got = d_out.download(np.float32)
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
        d_in.free(); d_out.free()


def test_q8_0_reference_kat(ctx, golden):
    g = golden["emit_q8_0_correctness"]
    N, K = g["N"], g["K"]
    raw = np.zeros((N, 34), np.uint8)
    raw[:, 0], raw[:, 1] = g["scale_bits"] & 0xFF, g["scale_bits"] >> 8
    raw[:, 2:] = np.arange(1, 33, dtype=np.uint8)
    dx, dw, dout = ctx.to_device(np.ones(K, np.float32)), ctx.to_device(raw), ctx.empty(N)
    ctx.gemv_q8_0(dx, dw, dout, 1, K, N)
    assert np.all(dout.download(np.float32) == g["expected_each"])


@pytest.mark.parametrize("kind,M,K,N", [("q8_0", 1, 2048, 5632),    # benchmark configuration 3
                                        ("q4_0", 1, 1536, 151936),  # benchmark configuration 4
                                        ("q8_0", 1, 2048, 2048), ("q8_0", 1, 5632, 2048),
                                        ("q8_0", 2, 4096, 77), ("q8_0", 1, 32, 5), ("q8_0", 1, 96, 1),
                                        ("q4_0", 3, 2048, 260), ("q4_0", 1, 32, 7), ("q4_0", 1, 8960, 64),
                                        # large Q4_0 products: short and long rows, N not a multiple
                                        # of the rows staged per step, two rows of x
                                        ("q4_0", 1, 256, 233100), ("q4_0", 1, 1792, 33333),
                                        ("q4_0", 2, 2048, 29201), ("q4_0", 1, 4096, 14601),
                                        ("q4_0", 1, 7168, 8400),
                                        # rows too long for the LDS stage: re-packed into planes in the workspace
                                        ("q8_0", 1, 8960, 1536), ("q8_0", 2, 8192, 300), ("q4_0", 1, 16384, 130)])
def test_quant_gemv(ctx, oracle, kind, M, K, N):
    say(f"gemv_{kind} M={M} K={K} N={N}")
    nb = N * (K // 32)
    seed = synth.SEED_CFG3 if kind == "q8_0" else synth.SEED_CFG4
    raw = (synth.q8_0_blocks if kind == "q8_0" else synth.q4_0_blocks)(seed, nb, 0.01)
    x = synth.normal_f32(seed + 1, M * K).reshape(M, K)
    want = (oracle.gemv_q8_0 if kind == "q8_0" else oracle.gemv_q4_0)(x, raw, M, K, N)
    dx, dw, dout = ctx.to_device(x), ctx.to_device(raw), ctx.empty(M * N)
    (ctx.gemv_q8_0 if kind == "q8_0" else ctx.gemv_q4_0)(dx, dw, dout, M, K, N)
    got = dout.download(np.float32, (M, N))
    assert rel_err(got, want) < TOL
    # both sides add exact products in f32, in different orders
    assert np.abs(got - want).max() < 1e-4 * np.sqrt(np.mean(want.astype(np.float64) ** 2))
    for b in (dx, dw, dout):
        b.free()


# ── Q8_0 / Q4_0 re-packed into planes ─────────────────────────────────────────

@pytest.mark.parametrize("kind", ["q8_0", "q4_0"])
def test_quant_planes_hold_the_blocks_bit_for_bit(ctx, oracle, kind):
    """The re-packed form is the same bytes in another order: packing and unpacking returns the blocks,
    the planes are where the declaration says (quants row after row, scales from the next multiple of 256
    bytes), and dequantising from the planes gives the oracle's bits, special scales included."""
    from homura_amd.runtime import DTYPE_Q4_0, DTYPE_Q8_0
    dt, bb, qpb = (DTYPE_Q8_0, 34, 32) if kind == "q8_0" else (DTYPE_Q4_0, 18, 16)
    N, K = 203, 96
    nb = N * (K // 32)
    raw = (synth.q8_0_blocks if kind == "q8_0" else synth.q4_0_blocks)(91, nb)
    blk = raw.reshape(nb, bb)
    for i, bits in enumerate([0x0001, 0x03FF, 0x0000, 0x8000, 0x7BFF, 0x7C00, 0xFC00, 0x7E00, 0x0400]):
        blk[i, 0], blk[i, 1] = bits & 0xFF, bits >> 8
    d_raw = ctx.to_device(raw)
    planes = ctx.pack_quant_planes(dt, d_raw, N, K)
    size = ctx.lib.hm_quant_planes_bytes(dt, N, K)
    qbytes = nb * qpb
    soff = (qbytes + 255) // 256 * 256
    assert size == soff + nb * 2
    host = planes.download(np.uint8)[:size]
    assert np.array_equal(host[:qbytes].reshape(nb, qpb), blk[:, 2:])
    assert np.array_equal(host[soff:soff + 2 * nb].reshape(nb, 2), blk[:, :2])
    back = ctx.empty(raw.size, np.uint8)
    ctx.unpack_quant_planes(dt, planes, back, N, K)
    assert np.array_equal(back.download(np.uint8), raw.reshape(-1))
    want = (oracle.dequant_q8_0 if kind == "q8_0" else oracle.dequant_q4_0)(raw)
    d_out = ctx.empty(N * K)
    ctx.dequant_quant_planes(dt, planes, d_out, N, K)
    got = d_out.download(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    for b in (d_raw, planes, back, d_out):
        b.free()


@pytest.mark.parametrize("kind,M,K,N", [("q8_0", 1, 2048, 5632),    # benchmark configuration 3
                                        ("q4_0", 1, 1536, 151936),  # benchmark configuration 4
                                        ("q8_0", 1, 1024, 151936),  # an LM head read from Q8_0 blocks
                                        ("q8_0", 1, 2048, 2048), ("q8_0", 1, 3072, 1024), ("q8_0", 2, 4096, 77),
                                        ("q8_0", 1, 32, 5), ("q8_0", 1, 96, 1), ("q8_0", 1, 1024, 6144),
                                        ("q4_0", 3, 2048, 260), ("q4_0", 1, 32, 7), ("q4_0", 1, 3072, 1024),
                                        ("q4_0", 1, 256, 233100), ("q4_0", 1, 1792, 33333),
                                        ("q4_0", 2, 2048, 29201), ("q4_0", 1, 4096, 14601), ("q4_0", 1, 2528, 4099),
                                        ("q4_0", 1, 3072, 9001), ("q4_0", 1, 2048, 8193),
                                        # rows cut across a workgroup's wavefronts (K > 4096): the down projections of
                                        # Qwen2.5-1.5B, TinyLlama, SmolLM2, Llama-2-7B; ragged ends; the widest served
                                        ("q8_0", 1, 8960, 1536), ("q4_0", 1, 8960, 1536), ("q8_0", 1, 5632, 2048),
                                        ("q4_0", 1, 5632, 2048), ("q8_0", 2, 8192, 2047), ("q4_0", 1, 8192, 2049),
                                        ("q8_0", 1, 11008, 515), ("q4_0", 3, 11008, 77), ("q8_0", 1, 4128, 9),
                                        ("q4_0", 1, 4128, 3), ("q8_0", 1, 16384, 130), ("q4_0", 1, 16384, 130),
                                        ("q8_0", 1, 12320, 21), ("q4_0", 1, 8224, 17)])
def test_quant_planes_gemv(ctx, oracle, kind, M, K, N):
    """The dequant-GEMV over the re-packed weights against the oracle on the raw blocks."""
    from homura_amd.runtime import DTYPE_Q4_0, DTYPE_Q8_0
    say(f"gemv_{kind}_planes M={M} K={K} N={N}")
    nb = N * (K // 32)
    seed = synth.SEED_CFG3 if kind == "q8_0" else synth.SEED_CFG4
    raw = (synth.q8_0_blocks if kind == "q8_0" else synth.q4_0_blocks)(seed, nb, 0.01)
    x = synth.normal_f32(seed + 1, M * K).reshape(M, K)
    want = (oracle.gemv_q8_0 if kind == "q8_0" else oracle.gemv_q4_0)(x, raw, M, K, N)
    dx, dw, dout = ctx.to_device(x), ctx.to_device(raw), ctx.empty(M * N)
    planes = ctx.pack_quant_planes(DTYPE_Q8_0 if kind == "q8_0" else DTYPE_Q4_0, dw, N, K)
    (ctx.gemv_q8_0_planes if kind == "q8_0" else ctx.gemv_q4_0_planes)(dx, planes, dout, M, K, N)
    got = dout.download(np.float32, (M, N))
    assert rel_err(got, want) < TOL
    # both sides add exact products in f32, in different orders
    assert np.abs(got - want).max() < 1e-4 * np.sqrt(np.mean(want.astype(np.float64) ** 2))
    for b in (dx, dw, dout, planes):
        b.free()


def test_quant_planes_reference_kat_and_limits(ctx, golden):
    from homura_amd.runtime import DTYPE_Q8_0
    g = golden["emit_q8_0_correctness"]     # reference src/graph_builder/emit_quant.rs:893-958: every output 528
    N, K = g["N"], g["K"]
    raw = np.zeros((N, 34), np.uint8)
    raw[:, 0], raw[:, 1] = g["scale_bits"] & 0xFF, g["scale_bits"] >> 8
    raw[:, 2:] = np.arange(1, 33, dtype=np.uint8)
    dx, dw, dout = ctx.to_device(np.ones(K, np.float32)), ctx.to_device(raw), ctx.empty(N)
    planes = ctx.pack_quant_planes(DTYPE_Q8_0, dw, N, K)
    ctx.gemv_q8_0_planes(dx, planes, dout, 1, K, N)
    assert np.all(dout.download(np.float32) == g["expected_each"])
    assert ctx.lib.hm_quant_planes_bytes(1, 8, 32) == 0 and ctx.lib.hm_quant_planes_bytes(DTYPE_Q8_0, 8, 48) == 0
    with pytest.raises(HomuraError, match="up to 16384"):
        ctx.gemv_q8_0_planes(dx, planes, dout, 1, 16416, 1)


def test_q6_k_planes_hold_the_blocks_bit_for_bit(ctx, oracle):
    """Q6_K re-packed into four planes: every byte of a block sits where the declaration says (a numpy
    restatement of the unit order), unpacking returns the blocks, and dequantising from the planes gives the
    oracle's bits, special block scales included."""
    from homura_amd.runtime import DTYPE_Q6_K
    N, K = 37, 768
    nb = N * (K // 256)
    raw = synth.q6_k_blocks(93, nb)
    blk = raw.reshape(nb, 210)
    for i, bits in enumerate([0x0001, 0x03FF, 0x0000, 0x8000, 0x7BFF, 0x7C00, 0xFC00, 0x7E00, 0x0400]):
        blk[i, 208], blk[i, 209] = bits & 0xFF, bits >> 8
    d_raw = ctx.to_device(raw)
    planes = ctx.pack_quant_planes(DTYPE_Q6_K, d_raw, N, K)
    size = ctx.lib.hm_quant_planes_bytes(DTYPE_Q6_K, N, K)
    units = nb * 4
    up = lambda v: (v + 255) // 256 * 256
    top_off = up(units * 32)
    sc_off = up(top_off + units * 16)
    d_off = up(sc_off + units * 4)
    assert size == d_off + nb * 2
    host = planes.download(np.uint8)[:size]
    nib = host[:units * 32].reshape(nb, 2, 2, 2, 16)          # block, h, p, run, j
    ql = blk[:, :128].reshape(nb, 2, 2, 2, 16)                 # block, h, run (l / 32), p, j
    assert np.array_equal(nib, ql.transpose(0, 1, 3, 2, 4))
    top = host[top_off:top_off + units * 16].reshape(nb, 2, 2, 16)
    assert np.array_equal(top, blk[:, 128:192].reshape(nb, 2, 2, 16))
    sc = host[sc_off:sc_off + units * 4].reshape(nb, 2, 2, 4)  # block, h, p, g
    assert np.array_equal(sc, blk[:, 192:208].reshape(nb, 2, 4, 2).transpose(0, 1, 3, 2))
    assert np.array_equal(host[d_off:d_off + 2 * nb].reshape(nb, 2), blk[:, 208:])
    back = ctx.empty(raw.size, np.uint8)
    ctx.unpack_quant_planes(DTYPE_Q6_K, planes, back, N, K)
    assert np.array_equal(back.download(np.uint8), raw.reshape(-1))
    want = oracle.dequant_q6_k(raw)
    d_out = ctx.empty(N * K)
    ctx.dequant_quant_planes(DTYPE_Q6_K, planes, d_out, N, K)
    got = d_out.download(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert ctx.lib.hm_quant_planes_bytes(DTYPE_Q6_K, 8, 128) == 0
    for b in (d_raw, planes, back, d_out):
        b.free()


@pytest.mark.parametrize("M,K,N", [(1, 1024, 151936),   # LM head of the Qwen3-0.6B shape
                                   (1, 1024, 3073), (2, 256, 7), (3, 2048, 515), (1, 4096, 130), (1, 512, 1001),
                                   (1, 2048, 1), (1, 1024, 2)])
def test_q6_k_planes_f32_product(ctx, oracle, M, K, N):
    """f32 row times the dequantised Q6_K weights, read from the planes: the checker multiplies the oracle's
    dequantised matrix (bit-exact with the reference's dequant_q6_k) in float64; widths the unit kernel has
    no instance for are refused."""
    from homura_amd.runtime import DTYPE_Q6_K
    say(f"gemv_q6_k_f32_planes M={M} K={K} N={N}")
    raw = synth.q6_k_blocks(15, N * K // 256)
    x = synth.normal_f32(16, M * K, 1.0).reshape(M, K)
    w = oracle.dequant_q6_k(raw).reshape(N, K)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    dx, dw, dout = ctx.to_device(x), ctx.to_device(raw), ctx.empty(M * N)
    planes = ctx.pack_quant_planes(DTYPE_Q6_K, dw, N, K)
    ctx.gemv_q6_k_f32_planes(dx, planes, dout, M, K, N)
    got = dout.download(np.float32, (M, N))
    err = np.abs(got - want).max() / np.sqrt(np.mean(want ** 2))
    say(f"  max error / rms {err:.2e}")
    assert err < 2e-6 * max(1.0, np.sqrt(K / 1024))   # f32 sums of exact terms
    with pytest.raises(HomuraError, match="must be 256, 512, 1024, 2048 or 4096"):
        ctx.gemv_q6_k_f32_planes(dx, planes, dout, 1, 768, 1)
    for b in (dx, dw, dout, planes):
        b.free()


# ── K-quants ──────────────────────────────────────────────────────────────────

@pytest.mark.parametrize("kind", ["q4_k", "q6_k"])
def test_kquant_dequant_bit_exact(ctx, oracle, kind):
    say(f"dequant {kind}")
    nblocks = 1031
    raw = (synth.q4_k_blocks if kind == "q4_k" else synth.q6_k_blocks)(77, nblocks)
    want = (oracle.dequant_q4_k if kind == "q4_k" else oracle.dequant_q6_k)(raw)
    dw, dout = ctx.to_device(raw), ctx.empty(nblocks * 256)
    (ctx.dequant_q4_k if kind == "q4_k" else ctx.dequant_q6_k)(dw, dout, nblocks)
    got = dout.download(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    dw.free(); dout.free()


def test_quantize_q8_k_bit_exact(ctx, oracle):
    say("quantize_q8_k")
    M, K = 3, 1024
    x = synth.normal_f32(31, M * K, 1.0).reshape(M, K)
    x[0, 256:512] = 0.0                        # an all-zero block
    x[1, :8] = (0.5, 1.5, 2.5, -0.5, -2.5, 127.0, -127.0, 63.5)
    x[1, 8:256] = 0.0                          # amax 127 -> iscale 1: ties visible
    dx = ctx.to_device(x)
    dq, dd, db = ctx.alloc(M * K), ctx.empty(M * K // 256), ctx.alloc(M * K // 16 * 4)
    ctx.quantize_q8_k(dx, dq, dd, db, M, K)
    q, d, bs = dq.download(np.int8), dd.download(np.float32), db.download(np.int32)
    for m in range(M):
        for kb in range(K // 256):
            wq, wd, wbs = oracle.quantize_q8_k(x[m, kb * 256:(kb + 1) * 256])
            i = m * K // 256 + kb
            assert np.array_equal(q[i * 256:(i + 1) * 256], wq) and np.float32(wd) == d[i]
            assert np.array_equal(bs[i * 16:(i + 1) * 16], wbs)
    assert q[K:K + 8].tolist() == [0, 2, 2, 0, -2, 127, -127, 64]


@pytest.mark.parametrize("kind", ["q4_k", "q6_k"])
@pytest.mark.parametrize("M,K,N", [(1, 1024, 3072), (1, 3072, 1024), (1, 1024, 151936), (2, 256, 7), (1, 2048, 515),
                                   (1, 8192, 64),
                                   # rows above 8192: twice the rounds a lane, a deeper row stage (Qwen2.5-1.5B's and
                                   # Llama-2-7B's down projections, the widest row served)
                                   (1, 8960, 1536), (2, 11008, 130), (1, 16384, 33), (1, 8448, 5)])
def test_gemv_kquant(ctx, oracle, kind, M, K, N):
    say(f"gemv_{kind} M={M} K={K} N={N}")
    raw = (synth.q4_k_blocks if kind == "q4_k" else synth.q6_k_blocks)(5, N * K // 256)
    x = synth.normal_f32(6, M * K, 1.0).reshape(M, K)
    want = (oracle.gemv_q4_k if kind == "q4_k" else oracle.gemv_q6_k)(x, raw, M, K, N)
    dx, dw, dout = ctx.to_device(x), ctx.to_device(raw), ctx.empty(M * N)
    (ctx.gemv_q4_k if kind == "q4_k" else ctx.gemv_q6_k)(dx, dw, dout, M, K, N)
    got = dout.download(np.float32, (M, N))
    err = rel_err(got, want)
    say(f"  rel err {err:.2e}")
    # same integer sums; only the order of the f32 adds differs (35-64 block sums a row above 8192)
    assert err < (1e-4 if K <= 8192 else 3e-4)
    for b in (dx, dw, dout):
        b.free()


@pytest.mark.parametrize("kind", ["q4_k", "q6_k", "mixed"])
@pytest.mark.parametrize("M,K,N", [(1, 1024, 3072), (1, 1536, 2048), (1, 2048, 515), (2, 256, 7), (1, 3072, 1024),
                                   (1, 4096, 130), (1, 5632, 2048), (1, 8960, 1536), (1, 16384, 33), (1, 768, 9)])
def test_gemv_k8(ctx, oracle, kind, M, K, N):
    """The K-quant product over the K8 form (rows cut across a workgroup's wavefronts, the activation row quantised
    to Q8_K on the pieces in registers) against the oracle's product on the raw blocks: same integer sums, the f32
    adds in another order. "mixed": the upper rows Q4_K, the lower ones Q6_K, stacked in one K8 matrix and
    multiplied in one launch."""
    from homura_amd.runtime import DTYPE_Q4_K, DTYPE_Q6_K
    say(f"gemv_k8 {kind} M={M} K={K} N={N}")
    x = synth.normal_f32(16, M * K, 1.0).reshape(M, K)
    n4 = N if kind == "q4_k" else (0 if kind == "q6_k" else N // 2)
    n6 = N - n4
    dx, dout = ctx.to_device(x), ctx.empty(M * N)
    k8 = ctx.alloc(ctx.lib.hm_k8_bytes(N, K))
    want = np.zeros((M, N), np.float32)
    held = []
    if n4:
        raw = synth.q4_k_blocks(15, n4 * K // 256)
        want[:, :n4] = oracle.gemv_q4_k(x, raw, M, K, n4)
        d = ctx.to_device(raw)
        held.append(d)
        ctx._check(ctx.lib.hm_pack_k8(ctx.h, DTYPE_Q4_K, d.ptr, n4, k8.ptr, N, K, 0))
    if n6:
        raw = synth.q6_k_blocks(17, n6 * K // 256)
        want[:, n4:] = oracle.gemv_q6_k(x, raw, M, K, n6)
        d = ctx.to_device(raw)
        held.append(d)
        ctx._check(ctx.lib.hm_pack_k8(ctx.h, DTYPE_Q6_K, d.ptr, n6, k8.ptr, N, K, n4))
    ctx.gemv_k8(dx, k8, dout, M, K, N)
    got = dout.download(np.float32, (M, N))
    err = rel_err(got, want)
    say(f"  rel err {err:.2e}")
    assert err < (1e-4 if K <= 8192 else 3e-4)
    with pytest.raises(HomuraError):
        ctx.gemv_k8(dx, k8, dout, 1, 128, N)     # K not a multiple of 256
    for b in held + [dx, dout, k8]:
        b.free()


# ── prefill GEMM (MFMA) ───────────────────────────────────────────────────────

@pytest.mark.parametrize("layout", ["kn", "nk"])
@pytest.mark.parametrize("M,K,N", [(512, 2048, 8192),  # benchmark configuration 5a
                                   (128, 32, 128), (256, 96, 384), (384, 64, 1152), (128, 160, 1024)])
def test_gemm_bf16_mfma(ctx, oracle, M, K, N, layout):
    say(f"gemm_bf16 M={M} K={K} N={N} B layout {layout}")
    a = synth.normal_bf16(synth.SEED_CFG5, M * K, 1.0).reshape(M, K)
    b = synth.normal_bf16(synth.SEED_CFG5 + 1, K * N, 0.02).reshape(K, N)
    want = oracle.matmul_bf16_bf16(a, b, M, K, N)
    da, dc = ctx.to_device(a), ctx.empty(M * N)
    if layout == "kn":
        db = ctx.to_device(b)
        ctx.gemm_bf16(da, db, dc, M, K, N)
    else:
        db = ctx.to_device(np.ascontiguousarray(b.T))
        ctx.gemm_bf16_nk(da, db, dc, M, K, N)
    got = dc.download(np.float32, (M, N))
    assert rel_err(got, want) < TOL
    for buf in (da, db, dc):
        buf.free()


def test_gemm_identity_exact(ctx):
    """A = I (bf16) picks rows of B exactly: catches a wrong fragment layout or transposition."""
    M = K = 128
    N = 256
    a = np.zeros((M, K), np.float32)
    a[np.arange(M), (np.arange(M) * 37) % K] = 1.0  # a permutation matrix
    b = synth.normal_bf16(5, K * N, 1.0).reshape(K, N)
    da, db, dc = ctx.to_device((a.view(np.uint32) >> 16).astype(np.uint16)), ctx.to_device(b), ctx.empty(M * N)
    ctx.gemm_bf16(da, db, dc, M, K, N)
    got = dc.download(np.float32, (M, N))
    assert np.array_equal(got, synth.bf16_to_f32(b)[(np.arange(M) * 37) % K])


@pytest.mark.parametrize("layout", ["kn", "nk"])
@pytest.mark.parametrize("M,K,N", [(1, 64, 8), (37, 96, 200), (130, 160, 264), (512, 1024, 4096 + 64)])
def test_gemm_bf16_ragged_edges(ctx, oracle, M, K, N, layout):
    """M and N that are not multiples of the 128 x 128 tile: edge tiles re-read the last row and
    must neither store outside C nor disturb the rows inside."""
    say(f"gemm_bf16 ragged M={M} K={K} N={N} B layout {layout}")
    a = synth.normal_bf16(11, M * K, 1.0).reshape(M, K)
    b = synth.normal_bf16(12, K * N, 0.02).reshape(K, N)
    want = oracle.matmul_bf16_bf16(a, b, M, K, N)
    guard = 4096
    host_c = np.full(M * N + guard, -77.0, np.float32)
    da, dc = ctx.to_device(a), ctx.to_device(host_c)
    if layout == "kn":
        db = ctx.to_device(b)
        ctx.gemm_bf16(da, db, dc, M, K, N)
    else:
        db = ctx.to_device(np.ascontiguousarray(b.T))
        ctx.gemm_bf16_nk(da, db, dc, M, K, N)
    got = dc.download(np.float32, (M * N + guard,))
    assert np.all(got[M * N:] == -77.0), "wrote past the end of C"
    assert rel_err(got[:M * N], want) < TOL
    for buf in (da, db, dc):
        buf.free()


@pytest.mark.parametrize("kind", ["q4_k", "q6_k"])
@pytest.mark.parametrize("M,K,N", [(1, 1024, 151936),   # LM head of the Qwen3-0.6B shape
                                   (1, 1024, 3072), (2, 256, 7), (3, 2048, 515), (1, 4096, 130), (1, 3072, 1024)])
def test_gemv_kquant_f32_activation(ctx, oracle, kind, M, K, N):
    """f32 row times the dequantised weights: the checker multiplies the oracle's dequantised matrix
    (bit-exact with the reference's dequant_q4_k / dequant_q6_k) in float64."""
    say(f"gemv_{kind}_f32 M={M} K={K} N={N}")
    raw = (synth.q4_k_blocks if kind == "q4_k" else synth.q6_k_blocks)(15, N * K // 256)
    x = synth.normal_f32(16, M * K, 1.0).reshape(M, K)
    w = (oracle.dequant_q4_k if kind == "q4_k" else oracle.dequant_q6_k)(raw).reshape(N, K)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    dx, dw, dout = ctx.to_device(x), ctx.to_device(raw), ctx.empty(M * N)
    (ctx.gemv_q4_k_f32 if kind == "q4_k" else ctx.gemv_q6_k_f32)(dx, dw, dout, M, K, N)
    got = dout.download(np.float32, (M, N))
    err = np.abs(got - want).max() / np.sqrt(np.mean(want ** 2))
    say(f"  max error / rms {err:.2e}")
    assert err < 2e-6 * max(1.0, np.sqrt(K / 1024))   # f32 sums of exact terms
    for b in (dx, dw, dout):
        b.free()


@pytest.mark.parametrize("kind", ["q8_0", "q4_0", "q4_k", "q6_k"])
@pytest.mark.parametrize("M,K,N", [(200, 1024, 1000), (5, 256, 130), (64, 2048, 6000), (512, 512, 256), (3, 4352, 200)])
def test_gemm_f32_quantised_weights(ctx, oracle, kind, M, K, N):
    """The quantised matmul at seq > 1 on the matrix cores against the oracle's row-by-row product (the
    decode formula: f32 activations for Q8_0 / Q4_0, Q8_K activations and integer sums for the
    K-quants). Both sides add the same products in f32, in different orders. N = 6000 at K = 2048 does
    not fit the workspace in one piece and goes through in slabs. K-quants up to 4096 wide multiply on the
    integer matrix cores with the decode kernels' block arithmetic (the oracle's, up to how the host compiler
    contracts it); K = 4352 takes the bf16 pieces."""
    say(f"gemm_f32_quant_nk {kind} M={M} K={K} N={N}")
    import homura_amd
    make = {"q8_0": synth.q8_0_blocks, "q4_0": synth.q4_0_blocks, "q4_k": synth.q4_k_blocks, "q6_k": synth.q6_k_blocks}[kind]
    per = 32 if kind in ("q8_0", "q4_0") else 256
    raw = make(41, N * K // per, 0.01) if per == 32 else make(41, N * K // per)
    x = synth.normal_f32(42, M * K, 1.0).reshape(M, K)
    want = getattr(oracle, "gemv_" + kind)(x, raw, M, K, N)
    # float64 truth: dequantised weights times the activation the format multiplies with
    w64 = getattr(oracle, "dequant_" + kind)(raw).reshape(N, K).astype(np.float64)
    x64 = x.astype(np.float64)
    if per == 256:
        for m in range(M):
            for kb in range(K // 256):
                q, d, _ = oracle.quantize_q8_k(x[m, kb * 256:(kb + 1) * 256])
                x64[m, kb * 256:(kb + 1) * 256] = np.float64(d) * q.astype(np.float64)
    truth = x64 @ w64.T
    dtype = {"q8_0": homura_amd.DTYPE_Q8_0, "q4_0": homura_amd.DTYPE_Q4_0, "q4_k": homura_amd.DTYPE_Q4_K,
             "q6_k": homura_amd.DTYPE_Q6_K}[kind]
    dx, dw, dout = ctx.to_device(x), ctx.to_device(raw), ctx.empty(M * N)
    ctx.gemm_f32_quant_nk(dx, dw, dtype, dout, M, K, N)
    got = dout.download(np.float32, (M, N))
    # error in units of a typical output, sqrt(K) rms(x) rms(w): f32 accumulation of six products per 32 k
    # leaves 1e-6 .. 7e-6; a dropped first-order piece product would leave 1e-3, a second-order one 3e-5
    unit = np.sqrt(K) * np.sqrt(np.mean(x64 ** 2)) * np.sqrt(np.mean(w64 ** 2))
    e_gpu, e_orc = np.abs(got - truth).max() / unit, np.abs(want - truth).max() / unit
    say(f"  error / typical output: gpu {e_gpu:.2e}, oracle {e_orc:.2e}; rel_err vs oracle {rel_err(got, want):.2e}")
    assert e_gpu < 1.2e-5
    assert rel_err(got, want) < (1e-4 if per == 256 and K <= 4096 else 2e-3)
    for b in (dx, dw, dout):
        b.free()


@pytest.mark.parametrize("M,K,N", [(512, 1024, 4096), (1, 1024, 1024), (77, 448, 576), (300, 3072, 1024)])
def test_gemm_f32_activations_bf16_weights(ctx, oracle, M, K, N):
    """The reference's mixed matmul at seq > 1: f32 activations, bf16 weights. The activation goes
    through the bf16 matrix cores as three bf16 numbers that add up to the f32 exactly. Measured
    against the float64 product with this file's rel_err (floor 1e-3 of the largest output): the f32
    oracle sits between 1e-4 and 1e-3 on the outputs closest to zero and the GPU must be in the same
    range (below 3x the oracle's own error); one bf16 rounding of the activations lands near 1."""
    say(f"gemm_f32_bf16_nk M={M} K={K} N={N}")
    x = synth.normal_f32(21, M * K).reshape(M, K)
    w = synth.normal_bf16(22, K * N, 0.02).reshape(K, N)
    want = oracle.matmul_f32_bf16(x, w, M, K, N)
    truth = x.astype(np.float64) @ synth.bf16_to_f32(w).astype(np.float64)
    dx, dw, dc = ctx.to_device(x), ctx.to_device(np.ascontiguousarray(w.T)), ctx.empty(M * N)
    ctx.gemm_f32_bf16_nk(dx, dw, dc, M, K, N)
    got = dc.download(np.float32, (M, N))
    coarse = synth.bf16_to_f32(synth.f32_to_bf16_rne(x)).astype(np.float64) @ synth.bf16_to_f32(w).astype(np.float64)
    e_gpu, e_orc, e_bf16 = rel_err(got, truth), rel_err(want, truth), rel_err(coarse, truth)
    say(f"  vs float64: gpu {e_gpu:.2e}, f32 oracle {e_orc:.2e}, activations rounded to bf16 {e_bf16:.2e}")
    assert e_gpu < 3 * e_orc and e_gpu < e_bf16 / 100
    assert rel_err(got, want) < 2e-3
    for buf in (dx, dw, dc):
        buf.free()


# ── KV cache append + decode attention ────────────────────────────────────────

def test_kv_append_reference_arrays(ctx, golden):
    g = golden["kv_cache_multi_token_append"]
    heads, max_len, hd = g["heads"], g["max_len"], g["head_dim"]
    kc, vc = ctx.empty(heads * max_len * hd, np.uint16), ctx.empty(heads * max_len * hd, np.uint16)
    ctx._check(ctx.lib.hm_fill_zero(ctx.h, kc.ptr, kc.nbytes))
    ctx._check(ctx.lib.hm_fill_zero(ctx.h, vc.ptr, vc.nbytes))
    k3, v3 = ctx.to_device(np.array(g["k3"], np.float32)), ctx.to_device(np.array(g["v3"], np.float32))
    ctx.kv_append(kc, vc, k3, v3, 1, heads, hd, max_len, 0, 3)
    k1, v1 = ctx.to_device(np.array(g["k1"], np.float32)), ctx.to_device(np.array(g["v1"], np.float32))
    ctx.kv_append(kc, vc, k1, v1, 1, heads, hd, max_len, 3, 1)
    cache = synth.bf16_to_f32(kc.download(np.uint16)).reshape(heads, max_len, hd)
    assert np.array_equal(cache[:, :4].reshape(-1), np.array(g["view_k_after_4"], np.float32))
    assert np.all(cache[:, 4:] == 0)
    # the reference panics "KV cache full"; here it is an error status and nothing is written
    with pytest.raises(HomuraError) as e:
        ctx.kv_append(kc, vc, k3, v3, 1, heads, hd, max_len, 6, 3)
    assert e.value.code == -4 and "KV cache full" in str(e.value)


def test_kv_append_rounds_to_nearest_even(ctx, oracle):
    lib = oracle.load()
    x = synth.normal_f32(9, 2 * 4 * 128)
    x[:3] = [1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, -1.0 - 2 ** -8]  # exact ties
    kc, vc = ctx.empty(2 * 8 * 128, np.uint16), ctx.empty(2 * 8 * 128, np.uint16)
    dk = ctx.to_device(x)
    ctx.kv_append(kc, vc, dk, dk, 1, 2, 128, 8, 2, 4)
    got = kc.download(np.uint16).reshape(2, 8, 128)[:, 2:6].reshape(-1)
    want = np.array([lib.orc_f32_to_bf16_rne(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(vc.download(np.uint16).reshape(2, 8, 128)[:, 2:6].reshape(-1), want)


@pytest.mark.parametrize("B,H,kvh,hd,max_len,kv_len", [
    (8, 12, 2, 128, 4096, 4096),   # benchmark configuration 5b
    (1, 16, 8, 128, 2048, 1025),   # Qwen3-0.6B decode shape
    (1, 16, 8, 128, 1152, 1),      # first token
    (2, 14, 2, 64, 300, 33),       # Qwen2.5-0.5B heads (g = 7), ragged length
    (1, 4, 4, 128, 64, 64),        # MHA (g = 1), single split
    (3, 32, 4, 64, 512, 511),      # g = 8
    (8, 12, 2, 128, 4096, 3001),   # long cache, ragged: workgroups walk their rows in steps
    (8, 8, 4, 64, 1500, 1399),     # same with 64-wide heads (g = 2)
    (16, 32, 4, 128, 700, 650),    # same with g = 8
    (2, 2, 1, 128, 16384, 16384),  # few (sequence, kv head) pairs, many steps per workgroup
    (40, 4, 4, 64, 600, 577),      # same with g = 1 (MHA)
    (24, 20, 4, 128, 1100, 1031)]) # same with g = 5
def test_gqa_decode_attn(ctx, oracle, B, H, kvh, hd, max_len, kv_len):
    say(f"gqa_decode_attn B={B} H={H} kvh={kvh} hd={hd} max_len={max_len} kv_len={kv_len}")
    q = synth.normal_f32(synth.SEED_CFG5 + 2, B * H * hd).reshape(B, H, hd)
    kb = synth.normal_bf16(synth.SEED_CFG5 + 3, B * kvh * max_len * hd).reshape(B, kvh, max_len, hd)
    vb = synth.normal_bf16(synth.SEED_CFG5 + 4, B * kvh * max_len * hd).reshape(B, kvh, max_len, hd)
    scale = 1.0 / math.sqrt(hd)
    dq, dk, dv, dout = ctx.to_device(q), ctx.to_device(kb), ctx.to_device(vb), ctx.empty(B * H * hd)
    ctx.gqa_decode_attn(dq, dk, dv, dout, B, H, kvh, hd, max_len, kv_len, scale)
    got = dout.download(np.float32, (B, H * hd))
    mask = np.zeros((1, kv_len), np.float32)  # decode: every cached row is attended
    for b in range(B):
        want = oracle.gqa_attention(q[b:b + 1], synth.bf16_to_f32(kb[b]), synth.bf16_to_f32(vb[b]), mask)
        assert rel_err(got[b], want) < TOL, f"sequence {b}"
    # repeat: the split counters must have been left clean
    ctx.gqa_decode_attn(dq, dk, dv, dout, B, H, kvh, hd, max_len, kv_len, scale)
    assert np.array_equal(dout.download(np.float32, (B, H * hd)), got)
    for buf in (dq, dk, dv, dout):
        buf.free()


@pytest.mark.parametrize("rising", [True, False])
def test_long_cache_attention_with_scores_that_keep_moving_the_maximum(ctx, oracle, rising):
    """The stepping kernel moves a wavefront's softmax reference point only when a score exceeds it by a
    margin, and rescales its sums and accumulators then. Random keys never do that after the first step; here
    the scores climb (or fall) by tens over every workgroup's rows, several margins from one step to the next, so the rescaling, the
    exponentials far below the reference point and the merge of wavefronts with very different reference
    points all carry weight in the result."""
    B, H, kvh, hd, L = 8, 12, 2, 128, 4096   # 16 (sequence, kv head) pairs x 4096 rows: 256 rows a workgroup, two steps
    q = synth.normal_f32(71, B * H * hd).reshape(B, H, hd)
    kf = synth.bf16_to_f32(synth.normal_bf16(72, B * kvh * L * hd)).reshape(B, kvh, L, hd) * 0.05
    ramp = (np.arange(L) % 256).astype(np.float32) / 256.0   # a sawtooth: the climb repeats inside every workgroup's rows
    if not rising:
        ramp = 1.0 - ramp
    for b in range(B):
        for k in range(kvh):
            direction = q[b, k * (H // kvh)] / np.linalg.norm(q[b, k * (H // kvh)])   # the first head of the group
            kf[b, k] += np.outer(ramp * 60.0, direction)
    kb = synth.f32_to_bf16_rne(kf.reshape(-1)).reshape(B, kvh, L, hd)
    vb = synth.normal_bf16(73, B * kvh * L * hd).reshape(B, kvh, L, hd)
    scale = 1.0 / math.sqrt(hd)
    dq, dk, dv, dout = ctx.to_device(q), ctx.to_device(kb), ctx.to_device(vb), ctx.empty(B * H * hd)
    ctx.gqa_decode_attn(dq, dk, dv, dout, B, H, kvh, hd, L, L, scale)
    got = dout.download(np.float32, (B, H * hd))
    mask = np.zeros((1, L), np.float32)
    spread = 0.0
    for b in range(B):
        want = oracle.gqa_attention(q[b:b + 1], synth.bf16_to_f32(kb[b]), synth.bf16_to_f32(vb[b]), mask)
        assert rel_err(got[b], want) < TOL, f"sequence {b}"
        s = (synth.bf16_to_f32(kb[b, 0]) @ q[b, 0]) * scale
        spread = max(spread, float(s.max() - s.min()))
    say(f"long-cache attention, scores {'rising' if rising else 'falling'} over a range of {spread:.0f}: within tolerance")
    assert spread > 30
    for buf in (dq, dk, dv, dout):
        buf.free()


def test_attention_uniform_keys_give_mean_of_values(ctx):
    B, H, kvh, hd, L = 1, 4, 2, 128, 200
    q = synth.normal_f32(1, H * hd)
    k = np.zeros((kvh, L, hd), np.uint16)
    vb = synth.normal_bf16(2, kvh * L * hd).reshape(kvh, L, hd)
    dq, dk, dv, dout = ctx.to_device(q), ctx.to_device(k), ctx.to_device(vb), ctx.empty(H * hd)
    ctx.gqa_decode_attn(dq, dk, dv, dout, B, H, kvh, hd, L, L, 0.1)
    got = dout.download(np.float32, (H, hd))
    mean = synth.bf16_to_f32(vb).astype(np.float64).mean(axis=1)
    for h in range(H):
        assert np.allclose(got[h], mean[h // 2], atol=1e-5)  # heads h0,h0,h1,h1 (floordiv map)


@pytest.mark.parametrize("S,H,kvh,hd,max_len,past", [
    (512, 16, 8, 128, 2048, 0),     # Qwen3-0.6B prompt chunk on an empty cache
    (200, 16, 8, 128, 2048, 1024),  # incremental prefill on top of 1024 cached rows, ragged S
    (1, 4, 2, 128, 64, 0),          # a single row
    (37, 14, 2, 64, 300, 33),       # g = 7, head_dim 64, nothing aligned
    (129, 4, 4, 64, 512, 64),       # MHA, one row into the second query block
    (64, 12, 2, 128, 256, 191),     # g = 6, the last key tile is a single key short of full
    (8, 16, 8, 128, 9000, 8000),    # a chat turn behind a long conversation: the keys are cut over several workgroups
    (40, 14, 2, 64, 5000, 4531),    # the same with g = 7, head_dim 64, nothing aligned
    (48, 16, 8, 128, 16400, 16000),
    (3, 4, 2, 128, 3000, 2900)])
@pytest.mark.parametrize("key_groups", [0, 1, 2, 4])
def test_gqa_prefill_attn(ctx, oracle, monkeypatch, S, H, kvh, hd, max_len, past, key_groups):
    """key_groups: how many wavefronts of a workgroup share a block of 32 query rows, each taking every
    n-th key tile (0 = the launch's own choice by grid size; the others force a variant)."""
    say(f"gqa_prefill_attn S={S} H={H} kvh={kvh} hd={hd} max_len={max_len} past={past} key groups {key_groups}")
    if key_groups:
        monkeypatch.setenv("HOMURA_PREFILL_KEY_GROUPS", str(key_groups))
    else:
        monkeypatch.delenv("HOMURA_PREFILL_KEY_GROUPS", raising=False)
    total = past + S
    q = synth.normal_f32(31, S * H * hd).reshape(S, H, hd)
    kb = synth.normal_bf16(32, kvh * max_len * hd).reshape(kvh, max_len, hd)
    vb = synth.normal_bf16(33, kvh * max_len * hd).reshape(kvh, max_len, hd)
    # rows past the live range must never be looked at: poison them
    kb[:, total:] = 0x7FC0
    vb[:, total:] = 0x7FC0
    scale = 1.0 / math.sqrt(hd)
    dq, dk, dv, dout = ctx.to_device(q), ctx.to_device(kb), ctx.to_device(vb), ctx.empty(S * H * hd)
    ctx.gqa_prefill_attn(dq, dk, dv, dout, S, H, kvh, hd, max_len, past, scale)
    got = dout.download(np.float32, (S, H * hd))
    assert np.isfinite(got).all()
    kf, vf = synth.bf16_to_f32(kb[:, :total]), synth.bf16_to_f32(vb[:, :total])
    want = oracle.gqa_attention(q, kf, vf, oracle.causal_mask(S, past))
    err = rel_err(got, want)
    say(f"  rel err {err:.2e}")
    assert err < 5e-3   # f32 rounding noise on the outputs nearest zero is ~1e-3 in this metric
    # the last row attends to everything: it must agree with the decode kernel on the same cache
    d1 = ctx.empty(H * hd)
    dq1 = ctx.to_device(q[S - 1])
    ctx.gqa_decode_attn(dq1, dk, dv, d1, 1, H, kvh, hd, max_len, total, scale)
    assert rel_err(got[S - 1], d1.download(np.float32, (H * hd,))) < 5e-3
    for buf in (dq, dk, dv, dout, d1, dq1):
        buf.free()


@pytest.mark.parametrize("key_groups", [1, 2, 4])
def test_prefill_attn_first_row_copies_its_value_row(ctx, monkeypatch, key_groups):
    """Position 0 on an empty cache sees one key: the output is exactly that V row for every head of
    the group, whatever q is (softmax of a single score is 1)."""
    monkeypatch.setenv("HOMURA_PREFILL_KEY_GROUPS", str(key_groups))
    S, H, kvh, hd, L = 40, 4, 2, 128, 64
    q = synth.normal_f32(41, S * H * hd)
    kb = synth.normal_bf16(42, kvh * L * hd).reshape(kvh, L, hd)
    vb = synth.normal_bf16(43, kvh * L * hd).reshape(kvh, L, hd)
    dq, dk, dv, dout = ctx.to_device(q), ctx.to_device(kb), ctx.to_device(vb), ctx.empty(S * H * hd)
    ctx.gqa_prefill_attn(dq, dk, dv, dout, S, H, kvh, hd, L, 0, 0.1)
    got = dout.download(np.float32, (S, H, hd))
    v0 = synth.bf16_to_f32(vb)[:, 0]
    for h in range(H):
        assert np.array_equal(got[0, h], v0[h // 2])


# ── light ops ─────────────────────────────────────────────────────────────────

def test_rmsnorm(ctx, oracle, golden):
    g = golden["rms_norm_basic"]
    dx, dw, dout = ctx.to_device(np.array(g["input"], np.float32)), ctx.to_device(np.array(g["weight"], np.float32)), ctx.empty(4)
    ctx.rmsnorm(dx, dw, dout, 1, 4, g["eps"])
    want = np.array(g["input"]) / math.sqrt(g["mean_square"] + g["eps"])
    assert np.allclose(dout.download(np.float32), want, atol=g["tolerance"])
    x = synth.normal_f32(3, 5 * 1024).reshape(5, 1024)
    w = synth.normal_f32(4, 1024)
    dx, dw, dout = ctx.to_device(x), ctx.to_device(w), ctx.empty(5 * 1024)
    ctx.rmsnorm(dx, dw, dout, 5, 1024, 1e-6)
    assert rel_err(dout.download(np.float32, (5, 1024)), oracle.rms_norm(x, w, 1e-6)) < 1e-4


@pytest.mark.parametrize("S,H,kvh,hd,qk_norm", [(1, 16, 8, 128, True), (3, 14, 2, 64, False), (2, 4, 4, 128, True)])
def test_qknorm_rope(ctx, oracle, S, H, kvh, hd, qk_norm):
    q = synth.normal_f32(5, S * H * hd).reshape(S, H, hd)
    k = synth.normal_f32(6, S * kvh * hd).reshape(S, kvh, hd)
    qw, kw = synth.normal_f32(7, hd), synth.normal_f32(8, hd)
    cos, sin = oracle.rope_tables(hd, 2048, 1e6)
    pos = [1029 + i for i in range(S)]
    wq = oracle.rms_norm(q, qw, 1e-6) if qk_norm else q
    wk = oracle.rms_norm(k, kw, 1e-6) if qk_norm else k
    wq, wk = oracle.rope_half(wq, cos[pos], sin[pos]), oracle.rope_half(wk, cos[pos], sin[pos])
    dq, dk = ctx.to_device(q), ctx.to_device(k)
    dqw, dkw = (ctx.to_device(qw), ctx.to_device(kw)) if qk_norm else (None, None)
    dc, ds = ctx.to_device(cos[pos]), ctx.to_device(sin[pos])
    ctx.qknorm_rope(dq, dk, dqw, dkw, dc, ds, S, H, kvh, hd, 1e-6)
    assert rel_err(dq.download(np.float32, q.shape), wq) < 1e-4
    assert rel_err(dk.download(np.float32, k.shape), wk) < 1e-4


def test_silu_add_embed(ctx, oracle, golden):
    g = synth.normal_f32(10, 3072) * 3
    u = synth.normal_f32(11, 3072)
    dg, du, dout = ctx.to_device(g), ctx.to_device(u), ctx.empty(3072)
    ctx.silu_mul(dg, du, dout, 3072)
    assert rel_err(dout.download(np.float32), oracle.silu_mul(g, u)) < 1e-5
    ctx.add(dg, du, dout, 3072)
    assert np.array_equal(dout.download(np.float32), g + u)  # one f32 add: exact
    e = golden["embedding_basic"]
    table = np.array(e["table"], np.float32)
    ids = np.array(e["ids"], np.int64)
    dt, di, do = ctx.to_device(table), ctx.to_device(ids), ctx.empty(4 * 3)
    ctx.embed(di, dt, do, 4, 4, 3)
    assert np.array_equal(do.download(np.float32, (4, 3)), np.array(e["expected"], np.float32))


def test_argmax_tie_rule(ctx, oracle, golden):
    cases = [np.array(golden["sample_token_greedy"]["logits"], np.float32),
             np.array([3.0, 1.0, 3.0, 2.0, 3.0, 0.0], np.float32),
             np.array([-np.inf, -np.inf], np.float32),
             np.array([1.0, np.nan, 0.5], np.float32),
             np.array([1.0, 2.0, np.nan], np.float32)]
    big = synth.normal_f32(12, 151936)
    top = float(big.max()) + 1.0
    big[[7, 70000, 151000]] = top            # three equal maxima: the last one wins
    cases.append(big)
    big2 = big.copy()
    big2[100000] = np.nan                     # a NaN discards everything before it
    cases.append(big2)
    dout = ctx.empty(1, np.int32)
    for c in cases:
        dv = ctx.to_device(c)
        ctx.argmax(dv, c.size, dout)
        assert int(dout.download(np.int32)[0]) == oracle.argmax_last(c)
        dv.free()
    assert oracle.argmax_last(big) == 151000 and oracle.argmax_last(big2) == 151000


# ── error behaviour ───────────────────────────────────────────────────────────

def test_bad_arguments_are_errors_not_faults(ctx):
    d = ctx.empty(64)
    with pytest.raises(HomuraError) as e:
        ctx.gemv_q8_0(d, d, d, 1, 48, 4)          # K not a multiple of 32
    assert e.value.code == -1
    with pytest.raises(HomuraError):
        ctx.gemv_bf16(d, d, d, 9, 8, 8)           # M out of range
    with pytest.raises(HomuraError):
        ctx.gemm_bf16(d, d, d, 128, 40, 128)      # K not a multiple of 32
    with pytest.raises(HomuraError):
        ctx.gemm_bf16(d, d, d, 128, 32, 100)      # [K,N] operand with N not a multiple of 8
    with pytest.raises(HomuraError):
        ctx.gqa_prefill_attn(d, d, d, d, 4, 4, 2, 128, 16, 14, 1.0)   # past + S > max_len
    with pytest.raises(HomuraError):
        ctx.gqa_prefill_attn(d, d, d, d, 4, 4, 2, 96, 16, 0, 1.0)     # head_dim 96
    with pytest.raises(HomuraError):
        ctx.gemv_q4_k(d, d, d, 1, 128, 4)         # K not a multiple of 256
    with pytest.raises(HomuraError):
        ctx.gqa_decode_attn(d, d, d, d, 1, 6, 4, 128, 16, 4, 1.0)  # heads not divisible
    with pytest.raises(HomuraError):
        ctx.gqa_decode_attn(d, d, d, d, 1, 4, 4, 128, 16, 17, 1.0)  # kv_len > max_len
    ctx.sync()
