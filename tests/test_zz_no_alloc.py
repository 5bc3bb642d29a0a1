"""The entry point that allocates nothing: hm_gqa_decode_attn_noalloc keeps the splits' partial sums
in a fixed array inside the library. Same kernels and split as hm_gqa_decode_attn, so the outputs
must be identical bit for bit, also when a smaller call follows a larger one on the same array."""
import math

import numpy as np
import pytest

from homura_amd import HomuraError, synth

pytestmark = pytest.mark.gpu


def run_pair(ctx, B, H, kvh, hd, max_len, kv_len, seed):
    print(f"noalloc attention B={B} H={H} kvh={kvh} hd={hd} max_len={max_len} kv_len={kv_len}", flush=True)
    q = synth.normal_f32(seed, B * H * hd)
    kb = synth.normal_bf16(seed + 1, B * kvh * max_len * hd)
    vb = synth.normal_bf16(seed + 2, B * kvh * max_len * hd)
    scale = 1.0 / math.sqrt(hd)
    dq, dk, dv = ctx.to_device(q), ctx.to_device(kb), ctx.to_device(vb)
    want_buf, got_buf = ctx.empty(B * H * hd), ctx.empty(B * H * hd)
    ctx.gqa_decode_attn(dq, dk, dv, want_buf, B, H, kvh, hd, max_len, kv_len, scale)
    ctx.gqa_decode_attn_noalloc(dq, dk, dv, got_buf, B, H, kvh, hd, max_len, kv_len, scale)
    want, got = want_buf.download(np.float32), got_buf.download(np.float32)
    for buf in (dq, dk, dv, want_buf, got_buf):
        buf.free()
    assert np.isfinite(want).all()
    assert np.array_equal(got, want)


def test_two_calls_in_a_row_the_second_smaller(ctx):
    run_pair(ctx, 8, 12, 2, 128, 4096, 4096, 700)   # long cache: stepping kernel, 32 splits per pair
    run_pair(ctx, 1, 16, 8, 128, 2048, 1025, 710)   # smaller: whole-chunk kernel, fewer partials
    run_pair(ctx, 2, 14, 2, 64, 300, 33, 720)       # ragged, head_dim 64
    run_pair(ctx, 1, 4, 4, 128, 64, 64, 730)        # a single split: no partials at all


def test_sizes_beyond_the_fixed_array_are_refused(ctx):
    limit = ctx.lib.hm_gqa_decode_attn_noalloc_limit()
    assert limit == 4 << 20
    B, H, kvh, hd, max_len = 256, 32, 8, 128, 64  # 2048 (sequence, kv head) pairs x 4 heads x 130 floats > 4 MiB
    dq = ctx.empty(B * H * hd)
    dk = ctx.empty(B * kvh * max_len * hd, np.uint16)
    dout = ctx.empty(B * H * hd)
    with pytest.raises(HomuraError, match="exceed"):
        ctx.gqa_decode_attn_noalloc(dq, dk, dk, dout, B, H, kvh, hd, max_len, max_len, 0.1)
    for buf in (dq, dk, dout):
        buf.free()
