"""Roofline timing of the kernel-level entry points at the benchmark shapes (configurations
1, 3, 4, 5a, 5b). Every kernel is launched over a ring of weight copies larger than the last-
level caches (Infinity Cache 256 MiB), all launches recorded into one HIP graph and replayed
between two HIP events on the launch stream, so the numbers are cold-cache per-launch times;
configurations 1 and 3 also carry `hot_us`, the same launch repeated on one weight buffer.
"""
from __future__ import annotations

import math

import numpy as np

from . import synth
from .runtime import Context

RING_BYTES = 400 << 20
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def _ring(ctx: Context, host: np.ndarray):
    """Device copies of `host`, enough of them to exceed RING_BYTES."""
    n = max(2, math.ceil(RING_BYTES / host.nbytes))
    first = ctx.to_device(host)
    copies = [first]
    for _ in range(n - 1):
        b = ctx.alloc(host.nbytes)
        ctx._check(ctx.lib.hm_copy(ctx.h, b.ptr, first.ptr, host.nbytes))
        copies.append(b)
    ctx.sync()
    return copies


REPS = 10  # graph replays per measurement (bench.py lowers it under a profiler)
MAX_LAUNCHES = 0  # > 0: at most this many kernel launches per measurement (counter runs keep them short)
USE_GRAPH = True  # False: launch kernel by kernel (for runs under a profiler; host launch gaps enter the time)


def _time(ctx: Context, launches, reps=None):
    reps = reps or REPS
    if MAX_LAUNCHES > 0:
        launches = launches[:MAX_LAUNCHES]
    def record():
        for fn in launches:
            fn()
    if USE_GRAPH:
        ms = ctx.time_graph_ms(record, reps=reps, warmup=4)
    else:
        ms = ctx.time_ms(record, reps, 1)
    return ms * 1e3 / len(launches)  # microseconds per launch


def _hot(ctx: Context, fn, launches=32):
    """The same launch over and over on one set of buffers: weights that fit the caches stay in them
    (the per-die L2s hold 32 MiB together, the Infinity Cache 256 MiB)."""
    return _time(ctx, [fn] * launches)


def _entry(name, us, nbytes=None, flops=None, note=None, hot_us=None):
    e = {"config": name, "avg_us": round(us, 3)}
    if hot_us is not None:
        e["hot_us"] = round(hot_us, 3)
    if nbytes is not None:
        gbs = nbytes / (us * 1e-6) / 1e9
        e.update({"bytes_per_launch": int(nbytes), "GBps": round(gbs, 1),
                  "hbm_frac": round(gbs / HBM_PEAK_GBS, 4)})
    if flops is not None:
        tf = flops / (us * 1e-6) / 1e12
        e.update({"flop_per_launch": int(flops), "TFLOPs": round(tf, 1),
                  "mfma_frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4)})
    if note:
        e["note"] = note
    return e


def run_copy_calibration(ctx: Context):
    """A plain transposing copy of known size (reads 32 MiB, writes 32 MiB of bf16): the yardstick
    the FETCH_SIZE / WRITE_SIZE hardware counters of the other kernels are scaled by."""
    K = N = 4096
    src = ctx.to_device(synth.normal_bf16(1, K * N))
    dst = ctx.empty(K * N, np.uint16)
    us = _time(ctx, [lambda: ctx.pack_bf16_kn_to_nk(src, dst, K, N)] * 4)
    src.free()
    dst.free()
    return _entry("calibration pack_kn_to_nk 4096x4096 bf16 (read 32 MiB + write 32 MiB)", us, 2 * K * N * 2)


def run_quant_cases(ctx: Context):
    """Configurations 3 and 4, each on the raw GGUF blocks (what a drop-in caller hands over) and on the
    same weights re-packed into planes at upload (what the model keeps)."""
    from .runtime import DTYPE_Q4_0, DTYPE_Q8_0
    out = []
    for name, dt, bb, blocks, seed, K, N, raw_fn, planes_fn in (
            ("cfg3 gemv_q8_0 2048->5632", DTYPE_Q8_0, 34, synth.q8_0_blocks, synth.SEED_CFG3, 2048, 5632, ctx.gemv_q8_0, ctx.gemv_q8_0_planes),
            ("cfg4 gemv_q4_0 1536->151936", DTYPE_Q4_0, 18, synth.q4_0_blocks, synth.SEED_CFG4, 1536, 151936, ctx.gemv_q4_0, ctx.gemv_q4_0_planes)):
        x = ctx.to_device(synth.normal_f32(seed + 1, K))
        ring = _ring(ctx, blocks(seed, N * K // 32))
        o = ctx.empty(N)
        nbytes = N * (K // 32) * bb + K * 4 + N * 4
        us = _time(ctx, [lambda b=b: raw_fn(x, b, o, 1, K, N) for b in ring])
        hot = _hot(ctx, lambda: raw_fn(x, ring[0], o, 1, K, N)) if nbytes < (64 << 20) else None
        out.append(_entry(name, us, nbytes, note="raw GGUF blocks", hot_us=hot))
        planes = [ctx.pack_quant_planes(dt, b, N, K) for b in ring]
        for b in ring:
            b.free()
        us = _time(ctx, [lambda p=p: planes_fn(x, p, o, 1, K, N) for p in planes])
        hot = _hot(ctx, lambda: planes_fn(x, planes[0], o, 1, K, N)) if nbytes < (64 << 20) else None
        out.append(_entry(name.replace(" gemv", " planes gemv"), us, nbytes, note="the same blocks re-packed into planes at upload",
                          hot_us=hot))
        for b in planes + [x, o]:
            b.free()
    out += run_q6_k_head_case(ctx)
    return out


def run_q6_k_head_case(ctx: Context):
    """The f32 product of a Q6_K output matrix at the Qwen3-0.6B shape (the LM head of a Q4_K_M file),
    on the raw blocks and on the planes the model keeps."""
    from .runtime import DTYPE_Q6_K
    K, N = 1024, 151936
    x = ctx.to_device(synth.normal_f32(31, K))
    ring = _ring(ctx, synth.q6_k_blocks(30, N * K // 256))
    o = ctx.empty(N)
    nbytes = N * (K // 256) * 210 + K * 4 + N * 4
    name = "LM head gemv_q6_k_f32 1024->151936"
    us = _time(ctx, [lambda b=b: ctx.gemv_q6_k_f32(x, b, o, 1, K, N) for b in ring])
    out = [_entry(name, us, nbytes, note="raw GGUF blocks")]
    planes = [ctx.pack_quant_planes(DTYPE_Q6_K, b, N, K) for b in ring]
    for b in ring:
        b.free()
    us = _time(ctx, [lambda p=p: ctx.gemv_q6_k_f32_planes(x, p, o, 1, K, N) for p in planes])
    out.append(_entry(name.replace(" gemv", " planes gemv"), us, nbytes, note="the same blocks re-packed into planes at upload"))
    for b in planes + [x, o]:
        b.free()
    return out


def run_all(ctx: Context):
    out = [run_copy_calibration(ctx)]
    # configuration 1: single bf16 GEMV x[1,896] x W[896,4864]
    K, N = 896, 4864
    x = ctx.to_device(synth.normal_f32(synth.SEED_CFG1, K))
    w = synth.normal_bf16(synth.SEED_CFG1 + 1, K * N, 0.02)
    ring = _ring(ctx, w)
    o = ctx.empty(N)
    nbytes = K * N * 2 + K * 4 + N * 4
    us = _time(ctx, [lambda b=b: ctx.gemv_bf16(x, b, o, 1, K, N) for b in ring])
    out.append(_entry("cfg1 gemv_bf16 [K,N] 896x4864", us, nbytes, note="reference weight layout",
                      hot_us=_hot(ctx, lambda: ctx.gemv_bf16(x, ring[0], o, 1, K, N))))
    us = _time(ctx, [lambda b=b: ctx.gemv_bf16_nk(x, b, o, 1, K, N) for b in ring])
    out.append(_entry("cfg1 gemv_bf16_nk [N,K] 4864x896", us, nbytes, note="stream layout",
                      hot_us=_hot(ctx, lambda: ctx.gemv_bf16_nk(x, ring[0], o, 1, K, N))))
    for b in ring:
        b.free()

    out += run_quant_cases(ctx)

    # configuration 5a: prefill-chunk GEMM 512 x 2048 x 8192 on the matrix cores
    M, K, N = 512, 2048, 8192
    a = ctx.to_device(synth.normal_bf16(synth.SEED_CFG5, M * K, 1.0))
    ring = _ring(ctx, synth.normal_bf16(synth.SEED_CFG5 + 1, K * N, 0.02))
    c = ctx.empty(M * N)
    us = _time(ctx, [lambda b=b: ctx.gemm_bf16(a, b, c, M, K, N) for b in ring])
    out.append(_entry("cfg5a gemm_bf16 512x2048x8192", us, M * K * 2 + K * N * 2 + M * N * 4, 2.0 * M * K * N,
                      note="B [K,N], reference weight layout"))
    us = _time(ctx, [lambda b=b: ctx.gemm_bf16_nk(a, b, c, M, K, N) for b in ring])
    out.append(_entry("cfg5a gemm_bf16_nk 512x2048x8192", us, M * K * 2 + K * N * 2 + M * N * 4, 2.0 * M * K * N,
                      note="B [N,K], stream layout (same bytes; values differ from the [K,N] case)"))
    for b in ring:
        b.free()

    # configuration 5b: GQA decode attention, 8 sequences, 12/2 heads, hd 128, KV length 4096
    B, H, kvh, hd, L = 8, 12, 2, 128, 4096
    q = ctx.to_device(synth.normal_f32(synth.SEED_CFG5 + 2, B * H * hd))
    kring = _ring(ctx, synth.normal_bf16(synth.SEED_CFG5 + 3, B * kvh * L * hd))
    vring = _ring(ctx, synth.normal_bf16(synth.SEED_CFG5 + 4, B * kvh * L * hd))
    o = ctx.empty(B * H * hd)
    scale = 1.0 / math.sqrt(hd)
    us = _time(ctx, [lambda k=k, v=v: ctx.gqa_decode_attn(q, k, v, o, B, H, kvh, hd, L, L, scale)
                     for k, v in zip(kring, vring)])
    out.append(_entry("cfg5b gqa_decode_attn 8x(12q/2kv)x128, kv 4096", us,
                      2 * B * kvh * L * hd * 2 + 2 * B * H * hd * 4))
    for b in kring + vring:
        b.free()

    # K-quant GEMVs at the projection shapes of a 0.6B model (Q8_K activation quantisation included)
    for kind, bb, blocks, fn in (("q4_k", 144, synth.q4_k_blocks, ctx.gemv_q4_k), ("q6_k", 210, synth.q6_k_blocks, ctx.gemv_q6_k)):
        for K, N in ((1024, 6144), (3072, 1024)):
            x = ctx.to_device(synth.normal_f32(7, K))
            ring = _ring(ctx, blocks(11, N * K // 256))
            o = ctx.empty(N)
            us = _time(ctx, [lambda b=b: fn(x, b, o, 1, K, N) for b in ring])
            out.append(_entry(f"gemv_{kind} {K}->{N}", us, N * (K // 256) * bb + K * 4 + N * 4,
                              note="two launches: activation to Q8_K, then the integer-dot GEMV"))
            for b in ring:
                b.free()
            x.free()
            o.free()

    # prefill: f32 activations x bf16 weights (three bf16 pieces per activation) at config 5a's shape
    M, K, N = 512, 2048, 8192
    a = ctx.to_device(synth.normal_f32(synth.SEED_CFG5, M * K))
    ring = _ring(ctx, synth.normal_bf16(synth.SEED_CFG5 + 1, K * N, 0.02))
    c = ctx.empty(M * N)
    us = _time(ctx, [lambda b=b: ctx.gemm_f32_bf16_nk(a, b, c, M, K, N) for b in ring])
    out.append(_entry("gemm_f32_bf16_nk 512x2048x8192", us, M * K * 4 + K * N * 2 + M * N * 4, 3 * 2.0 * M * K * N,
                      note="flop = the three bf16 passes the matrix cores run; includes the kernel that splits A"))
    for b in ring + [a, c]:
        b.free()

    # prefill attention: 512 new rows on 1024 cached ones, Qwen3-0.6B heads
    S, H, kvh, hd, L, past = 512, 16, 8, 128, 2048, 1024
    q = ctx.to_device(synth.normal_f32(5, S * H * hd))
    kc = ctx.to_device(synth.normal_bf16(6, kvh * L * hd))
    vc = ctx.to_device(synth.normal_bf16(7, kvh * L * hd))
    o = ctx.empty(S * H * hd)
    us = _time(ctx, [lambda: ctx.gqa_prefill_attn(q, kc, vc, o, S, H, kvh, hd, L, past, 1.0 / math.sqrt(hd))] * 8)
    visible = S * past + S * (S + 1) // 2                      # (query, key) pairs under the causal mask
    out.append(_entry(f"gqa_prefill_attn {S} rows on {past} cached, 16q/8kv x 128", us,
                      flops=3 * 2 * 2.0 * H * hd * visible,
                      note="flop = QK^T and PV over the visible pairs, three bf16 passes each"))
    for b in (q, kc, vc, o):
        b.free()
    return out
