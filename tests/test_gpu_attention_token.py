"""The decode attention layer of a token wave in two dispatches (attention_decode_token_ms +
attention_decode_token_finish_ms) on the GPU against the CPU checker, through the C ABI.
The first dispatch norms and rotates the token's query heads inside the split-K walk over
the cached keys; the second merges the split records, folds in the token's own key and
value, applies the gate and appends the key and value rows.  Outputs are held to the path's
tolerance (max-abs 2e-2, mean-abs 2e-3); the appended V row and every untouched cache row
are exact; the appended K row is the rope operator's (one bf16 step where the device's
cosine differs from libm's; deep in a context also what one fp32 step of the rotation
frequency moves the angle)."""
import numpy as np
import pytest

import oracle_lib as ol
from gpu_util import check_bf16, gpu, run

pytestmark = pytest.mark.gpu
o = ol.oracle


def _weights():
    q_w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(0x5157, 256))
    k_w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(0x4B57, 256))
    return q_w, k_w


def flags(interleave=0, compact=0, rotate=0):
    return 2 * interleave + 4 * compact + 8 * rotate


def token_batch(contexts, cap, forms, seed, replays=0, projection_stride=9216,
                query_stride=4096, stripes=None, pool_stripes=None, against_rope=False,
                parts_hint=None):
    """forms: list of (part, flags).  Returns the outputs per form."""
    B, dev, queue, lib = gpu()
    rows = len(contexts)
    q_w, k_w = _weights()
    stripe = 2 * cap * 256
    k_pool, stride = dev.create_pool(stripe * 2, pool_stripes or rows)
    v_pool, _ = dev.create_pool(stripe * 2, pool_stripes or rows)
    stripes = stripes or list(range(rows))[::-1]          # row != stripe
    proj = np.zeros((rows, projection_stride), np.uint16)
    want = np.zeros((rows, 4096), np.uint16)
    table = np.zeros(64, np.uint32)
    caches = []
    for r, ctx in enumerate(contexts):
        lane_seed = seed ^ (r * 0x9E3779B97F4A7C15 & 0xFFFFFFFFFFFFFFFF)
        proj[r, :9216] = ol.gaussian_bf16(lane_seed + 1, 9216)
        proj[r, 9216:] = 0x7FC0                # NaN in the padding of a wider stride
        k = np.zeros((2, cap, 256), np.uint16); v = np.zeros_like(k)
        k[:, :ctx] = ol.gaussian_bf16(lane_seed + 3, 2 * ctx * 256).reshape(2, ctx, 256) if ctx else 0
        v[:, :ctx] = ol.gaussian_bf16(lane_seed + 4, 2 * ctx * 256).reshape(2, ctx, 256) if ctx else 0
        # rows past the context hold NaN: they must never be read into the result
        k[:, ctx:] = 0x7FC0
        v[:, ctx:] = 0x7FC0
        k_pool.write(k, stripes[r] * stride)
        v_pool.write(v, stripes[r] * stride)
        q = np.zeros(4096, np.uint16); gate = np.zeros(4096, np.uint16)
        kk, vv = k.reshape(-1).copy(), v.reshape(-1).copy()
        o.tto_attn_qk_rope(np.ascontiguousarray(proj[r, :9216]), q_w, k_w, ctx, cap, q, gate, kk, vv)
        o.tto_attention_decode_split(q, gate, kk, vv, ctx, cap, 256, None, want[r], 8)
        caches.append((k, v, kk.reshape(2, cap, 256), vv.reshape(2, cap, 256)))
        table[r * 4] = stripes[r] * (stride // 2)
        table[r * 4 + 1] = ctx
    b_tab = dev.buffer_from(table)
    b_proj = dev.buffer_from(proj.reshape(-1))
    b_qw, b_kw = dev.buffer_from(q_w), dev.buffer_from(k_w)
    outs = {}
    for part, flag in forms:
        splits = (cap + part - 1) // part
        # records start as NaN: a record no workgroup wrote must never reach the result
        b_rec = dev.buffer_from(np.full(rows * 16 * splits * 258, np.nan, np.float32))
        for r, (k, v, _, _) in enumerate(caches):   # caches back to their state before the token
            k_pool.write(k, stripes[r] * stride)
            v_pool.write(v, stripes[r] * stride)
        b_o = dev.create_buffer(rows * query_stride * 2)
        bind = {0: b_proj, 1: b_qw, 2: b_kw, 3: k_pool, 4: v_pool, 5: b_tab, 6: b_rec, 7: b_o}
        hint = parts_hint if parts_hint is not None else -(-max(contexts) // part)
        const = {8: cap, 9: projection_stride, 10: query_stride, 11: part, 12: splits, 13: flag,
                 14: hint}

        def rec(cb, bind=bind, const=const, splits=splits):
            cb.encode(lib.pipeline("attention_decode_token_ms"), bind, const, (splits, 2, rows), (256,))
            cb.barrier()
            cb.encode(lib.pipeline("attention_decode_token_finish_ms"), bind, const, (16, rows), (256,))
        run(rec)
        got = b_o.read(np.uint16).reshape(rows, query_stride)[:, :4096]
        what = f"part {part} flags {flag}"
        for r, ctx in enumerate(contexts):
            check_bf16(got[r], want[r], f"{what} lane {r} ctx {ctx} (stripe {stripes[r]})")
            gk = k_pool.read(np.uint16, 2 * cap * 256, stripes[r] * stride).reshape(2, cap, 256)
            gv = v_pool.read(np.uint16, 2 * cap * 256, stripes[r] * stride).reshape(2, cap, 256)
            k0, v0, k1, v1 = caches[r]
            assert np.array_equal(gv, v1), f"{what} lane {r}: V cache"          # exact
            keep = np.ones(cap, bool); keep[ctx] = False
            assert np.array_equal(gk[:, keep], k0[:, keep]), f"{what} lane {r}: K rows moved"
            new, ref = ol.bf16_to_f32(gk[:, ctx].reshape(-1)), ol.bf16_to_f32(k1[:, ctx].reshape(-1))
            # one bf16 step of the result, plus what one fp32 step of the device's powf
            # against libm's moves the rotation angle at this position
            bar = 2.0 ** -7 * np.maximum(np.abs(ref), 1e-3) + ctx * 2.4e-7 * np.abs(ref).max()
            err = np.abs(new - ref)
            assert np.all(err <= bar), \
                f"{what} lane {r}: appended K row off by {err.max():.3e} (bar {bar.min():.3e})"
        outs[(part, flag)] = got.copy()
        if against_rope:
            # the appended key rows are the rope operator's own, bit for bit
            mine = [k_pool.read(np.uint16, 2 * cap * 256, stripes[r] * stride).reshape(2, cap, 256)
                    [:, ctx].copy() for r, ctx in enumerate(contexts)]
            for r, (k, v, _, _) in enumerate(caches):
                k_pool.write(k, stripes[r] * stride)
                v_pool.write(v, stripes[r] * stride)
            b_q, b_g = dev.create_buffer(rows * 8192), dev.create_buffer(rows * 8192)
            run(lambda cb: cb.encode(lib.pipeline("attn_qk_rope_ms"),
                                     {0: b_proj, 1: b_qw, 2: b_kw, 3: b_q, 4: b_g, 5: k_pool, 6: v_pool,
                                      8: b_tab}, {7: cap, 9: projection_stride, 10: 4096},
                                     (18, rows), (256,)))
            for r, ctx in enumerate(contexts):
                roped = k_pool.read(np.uint16, 2 * cap * 256, stripes[r] * stride).reshape(2, cap, 256)
                assert np.array_equal(roped[:, ctx], mine[r]), \
                    f"{what} lane {r}: appended K row differs from attn_qk_rope_ms"
        if replays:
            cb = queue.create_command_buffer()
            cb.begin_compute_pass(); rec(cb); cb.end_compute_pass()
            cb.compile()
            for replay in range(replays):
                b_o.write(np.zeros(rows * query_stride, np.uint16))
                cb.commit().wait()
                again = b_o.read(np.uint16).reshape(rows, query_stride)[:, :4096]
                assert np.array_equal(again, got), f"{what} replay {replay}"
    return outs


@pytest.mark.parametrize("part,flag", [(2048, 0), (256, 0), (256, flags(rotate=1)), (64, flags(compact=1)),
                                       (32, flags(interleave=1)), (128, flags(compact=1, rotate=3))])
def test_token_small_ragged_lanes(part, flag):
    """Seven ragged lanes incl. an empty cache and contexts around the 32-key block and the
    256-key partition."""
    print(f"[case] token layer, 7 ragged lanes, part {part} flags {flag}", flush=True)
    token_batch([2000, 1499, 700, 100, 255, 256, 0], 2048, [(part, flag)], 0x1A7E, replays=2)


@pytest.mark.parametrize("ctx", [0, 1, 31, 32, 33, 63, 64, 65, 300, 1000])
def test_token_single_lane_context_edges(ctx):
    print(f"[case] token layer, one lane, context {ctx}", flush=True)
    token_batch([ctx], 1100, [(1120, 0), (32, flags(rotate=1)), (96, flags(interleave=1, compact=1))],
                0x2B00 + ctx)


def test_token_wide_strides():
    print("[case] token layer, slab strides wider than the rows", flush=True)
    token_batch([500, 37], 512, [(128, 0)], 0x3C01, projection_stride=9216 + 64, query_stride=4096 + 256)


def test_token_appended_rows_are_the_rope_operators():
    print("[case] token layer, appended key rows against attn_qk_rope_ms", flush=True)
    token_batch([777, 5, 0], 1024, [(256, 0)], 0x4D11, against_rope=True)


def test_token_sixteen_lanes():
    print("[case] token layer, 16 lanes", flush=True)
    contexts = [37 * (i + 1) + (i % 3) * 200 for i in range(16)]
    token_batch(contexts, 1024, [(256, flags(compact=1, rotate=1)), (1024, 0)], 0x1616, replays=1)


@pytest.mark.parametrize("hint", [0, 1, 3, 40, 200])
def test_token_finish_hint_is_only_a_hint(hint):
    """The finishing dispatch sizes its first batch of record requests by the caller's hint;
    whatever the hint (none, too small, too large), every record is merged: 1..157 records
    per head here, past the largest batch of 128."""
    print(f"[case] token layer, finish hint {hint}", flush=True)
    token_batch([5000, 31, 2100, 0], 5024, [(32, flags(rotate=1))], 0x7117, parts_hint=hint)
