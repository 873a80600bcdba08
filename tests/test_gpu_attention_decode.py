"""Full-attention decode on the GPU against the CPU checker, through the C ABI.
Tolerance of the path: max-abs <= 2e-2, mean-abs <= 2e-3 on bf16 outputs; slot
indexing (which cache rows are written, raw V and gate copies) is exact."""
import os

import numpy as np
import pytest

import oracle_lib as ol
from golden import cases
from gpu_util import check_bf16, gpu, run

pytestmark = pytest.mark.gpu
o = ol.oracle


def _weights():
    q_w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(0x5157, 256))
    k_w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(0x4B57, 256))
    return q_w, k_w


def test_qk_rope_chain_matches_reference_vectors():
    """Five chained positions on the reference's own fixture inputs (capacity 512)."""
    print("[case] qk_rope chain, seed 0xA77E1755, capacity 512", flush=True)
    B, dev, queue, lib = gpu()
    G = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz"))
    proj, q_w, k_w = cases.attention_chain_inputs(ol.banded_bf16)
    cap, n = cases.ATTN_CAPACITY, cases.ATTN_CHAIN_POSITIONS
    b_proj = [dev.buffer_from(proj[p]) for p in range(n)]
    b_qw, b_kw = dev.buffer_from(q_w), dev.buffer_from(k_w)
    b_q, b_g = dev.create_buffer(8192), dev.create_buffer(8192)
    b_k, b_v = dev.create_buffer(2 * cap * 512), dev.create_buffer(2 * cap * 512)
    rope = lib.pipeline("attn_qk_rope")

    def rec(cb):
        for p in range(n):
            cb.encode(rope, {0: b_proj[p], 1: b_qw, 2: b_kw, 3: b_q, 4: b_g, 5: b_k, 6: b_v},
                      {7: p, 8: cap}, (18,), (256,))
            cb.barrier()
    run(rec)
    keys = b_k.read(np.uint16).reshape(2, cap, 256)
    vals = b_v.read(np.uint16).reshape(2, cap, 256)
    assert np.array_equal(b_g.read(np.uint16), G["chain_gate"])          # raw copy: exact
    assert np.array_equal(vals[:, :n], G["chain_values"])                # raw copy: exact
    assert not keys[:, n:].any() and not vals[:, n:].any()               # slot indexing: exact
    # banded fixture values reach 2^8, so compare relative to magnitude
    for got, want, what in ((b_q.read(np.uint16), G["chain_q"], "q"),
                            (keys[:, :n], G["chain_keys"], "k rows")):
        g, w = ol.bf16_to_f32(got.reshape(-1)), ol.bf16_to_f32(want.reshape(-1))
        rel = np.abs(g - w) / np.maximum(np.abs(w), 1e-3)
        print(f"[parity] rope {what}: exact {np.mean(got.reshape(-1) == want.reshape(-1)):.4f} "
              f"max-rel {rel.max():.3e}", flush=True)
        assert rel.max() <= 2 ** -7     # at most one bf16 ulp
        assert np.mean(got.reshape(-1) == want.reshape(-1)) > 0.99


def _fill_cache_by_rope(seed, rows, cap):
    """K rows normed+roped at their own positions, V raw, through the block rope
    operator on the GPU and the checker on the CPU; returns both caches."""
    B, dev, queue, lib = gpu()
    q_w, k_w = _weights()
    proj = ol.gaussian_bf16(seed, rows * 9216)
    keys = np.zeros(2 * cap * 256, np.uint16)
    values = np.zeros_like(keys)
    query = np.zeros(rows * 4096, np.uint16)
    gate = np.zeros_like(query)
    att = np.zeros_like(query)
    sel = np.zeros(1, np.uint32)
    o.tto_attention_prefill(proj, q_w, k_w, rows, 0, cap, query, gate, keys, values, sel, 0, att, 8)
    b_proj = dev.buffer_from(proj)
    b_qw, b_kw = dev.buffer_from(q_w), dev.buffer_from(k_w)
    b_q, b_g = dev.create_buffer(rows * 8192), dev.create_buffer(rows * 8192)
    b_k, b_v = dev.create_buffer(2 * cap * 512), dev.create_buffer(2 * cap * 512)
    run(lambda cb: cb.encode(lib.pipeline("attn_qk_rope_blk"),
                             {0: b_proj, 1: b_qw, 2: b_kw, 3: b_q, 4: b_g, 5: b_k, 6: b_v},
                             {7: 0, 8: cap}, (18, rows), (256,)))
    return dict(proj=proj, q_w=q_w, k_w=k_w, keys=keys, values=values, query=query, gate=gate,
                b_q=b_q, b_g=b_g, b_k=b_k, b_v=b_v, b_qw=b_qw, b_kw=b_kw)


def test_config1_single_decode_step_4096():
    """Batch 1, 16 q / 2 kv heads, 4096 keys, position 4095: qk-RMSNorm, rotary on
    64 dims at theta 1e7, softmax(qK^T/16)V * sigmoid(gate)."""
    print("[case] config 1: decode, context 4095, capacity 4096", flush=True)
    B, dev, queue, lib = gpu()
    cap, ctx = 4096, 4095
    c = _fill_cache_by_rope(0xC0F1, cap, cap)
    gk = c["b_k"].read(np.uint16)
    gv = c["b_v"].read(np.uint16)
    assert np.array_equal(gv, c["values"])                                # raw V: exact
    check_bf16(gk, c["keys"], "config1 K cache", max_abs=4e-2, mean_abs=1e-4)
    assert np.mean(gk == c["keys"]) > 0.995
    # the decode token itself: last row's projection through the one-token operator
    q_w, k_w = c["q_w"], c["k_w"]
    proj_last = c["proj"][ctx * 9216:(ctx + 1) * 9216]
    q = np.zeros(4096, np.uint16); gate = np.zeros(4096, np.uint16)
    keys, values = c["keys"].copy(), c["values"].copy()
    o.tto_attn_qk_rope(proj_last, q_w, k_w, ctx, cap, q, gate, keys, values)
    want_tiled = np.zeros(4096, np.uint16); want_split = np.zeros(4096, np.uint16)
    o.tto_attention_decode(q, gate, keys, values, ctx, cap, want_tiled, 8)
    o.tto_attention_decode_split(q, gate, keys, values, ctx, cap, 256, None, want_split, 8)

    b_p = dev.buffer_from(proj_last)
    b_q, b_g, b_o = dev.create_buffer(8192), dev.create_buffer(8192), dev.create_buffer(8192)
    nparts = (ctx + 256) // 256
    b_part = dev.create_buffer(16 * nparts * 258 * 4)
    b_wts = dev.create_buffer(16 * nparts * 258 * 4)
    outs = {}

    def rec(cb):
        cb.encode(lib.pipeline("attn_qk_rope"),
                  {0: b_p, 1: c["b_qw"], 2: c["b_kw"], 3: b_q, 4: b_g, 5: c["b_k"], 6: c["b_v"]},
                  {7: ctx, 8: cap}, (18,), (256,))
        cb.barrier()
        cb.encode(lib.pipeline("attention_decode"),
                  {0: b_q, 1: b_g, 2: c["b_k"], 3: c["b_v"], 5: b_o}, {4: ctx, 6: cap},
                  (16,), (256,))
    run(rec)
    outs["single"] = b_o.read(np.uint16)
    check_bf16(b_q.read(np.uint16), q, "config1 q")
    assert np.array_equal(b_g.read(np.uint16), gate)

    def rec_fused(cb):
        cb.encode(lib.pipeline("attention_decode_scores_values_gqa8"),
                  {0: b_q, 1: c["b_k"], 2: c["b_v"], 6: b_part},
                  {3: ctx, 4: cap, 5: 256, 7: nparts}, (2, nparts), (256, 4))
        cb.barrier()
        cb.encode(lib.pipeline("attention_decode_combine"), {0: b_part, 1: b_g, 3: b_o},
                  {2: nparts}, (16,), (256,))
    b_o.write(np.zeros(4096, np.uint16))
    run(rec_fused)
    outs["fused split"] = b_o.read(np.uint16)

    def rec_two_stage(cb):
        cb.encode(lib.pipeline("attention_decode_scores_gqa4"), {0: b_q, 1: c["b_k"], 5: b_wts},
                  {2: ctx, 3: cap, 4: 256, 6: nparts}, (4, nparts), (256, 4))
        cb.barrier()
        cb.encode(lib.pipeline("attention_decode_values_gqa8"), {0: b_wts, 1: c["b_v"], 5: b_part},
                  {2: ctx, 3: cap, 4: 256, 6: nparts}, (2, nparts), (32, 4, 8))
        cb.barrier()
        cb.encode(lib.pipeline("attention_decode_combine"), {0: b_part, 1: b_g, 3: b_o},
                  {2: nparts}, (16,), (256,))
    b_o.write(np.zeros(4096, np.uint16))
    run(rec_two_stage)
    outs["two-stage split"] = b_o.read(np.uint16)
    check_bf16(outs["single"], want_tiled, "config1 attention_decode vs tiled checker")
    check_bf16(outs["fused split"], want_split, "config1 scores_values_gqa8+combine")
    check_bf16(outs["two-stage split"], want_split, "config1 scores+values+combine")


@pytest.mark.parametrize("ctx", [0, 1, 30, 31, 32, 33, 63, 64, 127, 255, 256, 257, 300, 511, 512,
                                 1000])
def test_decode_context_edges(ctx):
    print(f"[case] decode edge context {ctx}, capacity 1100", flush=True)
    B, dev, queue, lib = gpu()
    cap = 1100
    q = ol.gaussian_bf16(100 + ctx, 4096); gate = ol.gaussian_bf16(200 + ctx, 4096)
    keys = ol.gaussian_bf16(300 + ctx, 2 * cap * 256)
    values = ol.gaussian_bf16(400 + ctx, 2 * cap * 256)
    # rows past the context hold NaN: they must never be read into the result
    keys.reshape(2, cap, 256)[:, ctx + 1:] = 0x7FC0
    values.reshape(2, cap, 256)[:, ctx + 1:] = 0x7FC0
    want = np.zeros(4096, np.uint16)
    o.tto_attention_decode_split(q, gate, keys, values, ctx, cap, 256, None, want, 4)
    b_q, b_g = dev.buffer_from(q), dev.buffer_from(gate)
    b_k, b_v = dev.buffer_from(keys), dev.buffer_from(values)
    b_o = dev.create_buffer(8192)
    run(lambda cb: cb.encode(lib.pipeline("attention_decode"),
                             {0: b_q, 1: b_g, 2: b_k, 3: b_v, 5: b_o}, {4: ctx, 6: cap},
                             (16,), (256,)))
    check_bf16(b_o.read(np.uint16), want, f"attention_decode ctx {ctx}")
    for part in (256, 64):
        nparts = (ctx + part) // part
        b_part = dev.create_buffer(16 * nparts * 258 * 4)
        b_o2 = dev.create_buffer(8192)

        def rec(cb):
            cb.encode(lib.pipeline("attention_decode_scores_values_gqa8"),
                      {0: b_q, 1: b_k, 2: b_v, 6: b_part}, {3: ctx, 4: cap, 5: part, 7: nparts},
                      (2, nparts), (256, 4))
            cb.barrier()
            cb.encode(lib.pipeline("attention_decode_combine"), {0: b_part, 1: b_g, 3: b_o2},
                      {2: nparts}, (16,), (256,))
        run(rec)
        check_bf16(b_o2.read(np.uint16), want, f"split part {part} ctx {ctx}")


def _lane_batch(contexts, cap, part, seed, replays=0, interleave=False, compact=False,
                stripes=None, pool_stripes=None, sharpen=0, rotate=0):
    """Lane-batched decode over a striped pool with a state table, long rows
    through attention_decode_split_ms and short rows through attention_decode_ms.
    interleave: a lane's workgroups take its 32-key blocks in turn (bit 1 of c9).
    rotate: a workgroup starts (split + 5 kv head + 11 row) * rotate blocks into its range
    and wraps (bits 3-7 of c9); the same keys per record in another order.
    compact: the workgroups whose splits hold keys lead the dispatch order (bit 2 of c9);
    the records, and so the output bits, are those of the plain order.
    stripes / pool_stripes: which stripe of a pool of `pool_stripes` each lane lives on
    (default: the lanes in reverse order on a pool of their number).
    sharpen: the queries are scaled by 2^sharpen (scores in the hundreds: a one-hot softmax);
    negative: zero queries (a flat softmax).
    replays > 0: the recording is also compiled into a HIP graph and replayed that
    many times with the outputs and records cleared in between; every replay must
    reproduce the eager bits."""
    B, dev, queue, lib = gpu()
    rows = len(contexts)
    stripe = 2 * cap * 256          # elements per lane cache
    k_pool, stride = dev.create_pool(stripe * 2, pool_stripes or rows)
    v_pool, _ = dev.create_pool(stripe * 2, pool_stripes or rows)
    assert stride == stripe * 2
    q = np.zeros((rows, 4096), np.uint16); gate = np.zeros_like(q)
    want = np.zeros_like(q)
    # lanes are placed on stripes in reverse order so row != stripe
    stripes = stripes or list(range(rows))[::-1]
    table = np.zeros(64, np.uint32)
    for r, ctx in enumerate(contexts):
        lane_seed = seed ^ (r * 0x9E3779B97F4A7C15 & 0xFFFFFFFFFFFFFFFF)
        q[r] = ol.gaussian_bf16(lane_seed + 1, 4096)
        if sharpen > 0:
            q[r] = np.where(q[r] & 0x7F80, q[r] + np.uint16(sharpen << 7), q[r])   # exponent + sharpen
        elif sharpen < 0:
            q[r] = 0                                    # every score zero: the mean of the values
        gate[r] = ol.gaussian_bf16(lane_seed + 2, 4096)
        n = ctx + 1
        k = np.zeros((2, cap, 256), np.uint16); v = np.zeros_like(k)
        k[:, :n] = ol.gaussian_bf16(lane_seed + 3, 2 * n * 256).reshape(2, n, 256)
        v[:, :n] = ol.gaussian_bf16(lane_seed + 4, 2 * n * 256).reshape(2, n, 256)
        o.tto_attention_decode_split(q[r], gate[r], k.reshape(-1), v.reshape(-1), ctx, cap, 256,
                                     None, want[r], 8)
        k_pool.write(k, stripes[r] * stride)
        v_pool.write(v, stripes[r] * stride)
        table[r * 4] = stripes[r] * (stride // 2)
        table[r * 4 + 1] = ctx
    short = [r for r, c in enumerate(contexts) if c + 1 <= 256]
    bucket = np.zeros(16, np.uint32)
    bucket[:len(short)] = short
    b_tab = dev.buffer_from(np.concatenate([table, bucket]))
    b_q, b_g = dev.buffer_from(q), dev.buffer_from(gate)
    b_o = dev.create_buffer(rows * 8192)
    max_splits = (cap + part - 1) // part
    b_part = dev.create_buffer(rows * 16 * max_splits * 258 * 4)

    def rec(cb):
        cb.encode(lib.pipeline("attention_decode_split_ms"),
                  {0: b_q, 1: k_pool, 2: v_pool, 3: b_tab, 4: b_part},
                  {5: cap, 6: 4096, 7: part, 8: max_splits,
                   9: 1 + 2 * int(interleave) + 4 * int(compact) + 8 * int(rotate)},
                  (max_splits, 2, rows), (256,))
        cb.barrier()
        cb.encode(lib.pipeline("attention_decode_combine_ms"),
                  {0: b_part, 1: b_g, 2: b_tab, 3: b_o},
                  {4: part, 5: max_splits, 6: 4096, 7: 1, 8: cap}, (16, rows), (256,))
        if short:
            cb.encode(lib.pipeline("attention_decode_ms"),
                      {0: b_q, 1: b_g, 2: k_pool, 3: v_pool, 4: b_tab, 5: b_o,
                       7: (b_tab, 256)}, {6: cap, 8: 4096}, (16, len(short)), (256,))
    run(rec)
    got = b_o.read(np.uint16).reshape(rows, 4096)
    for r, ctx in enumerate(contexts):
        check_bf16(got[r], want[r], f"lane {r} ctx {ctx} (stripe {stripes[r]}, part {part})")
    if replays:
        cb = queue.create_command_buffer()
        cb.begin_compute_pass(); rec(cb); cb.end_compute_pass()
        cb.compile()
        for replay in range(replays):
            b_o.write(np.zeros(rows * 4096, np.uint16))
            b_part.write(np.full(rows * 16 * max_splits * 258, np.nan, np.float32))
            cb.commit().wait()
            assert np.array_equal(b_o.read(np.uint16).reshape(rows, 4096), got), f"replay {replay}"
    return got


def test_lane_batch_small_ragged():
    print("[case] lane batch ragged small", flush=True)
    _lane_batch([2000, 1499, 700, 100, 255, 256, 0], 2048, 128, 0xBEEF)


@pytest.mark.parametrize("contexts,cap,part", [
    ([2000, 1499, 700, 100, 255, 256, 0, 287, 288, 319], 2048, 128),   # blocks not a multiple of the splits
    ([5000, 4999, 31], 5120, 1024),                                    # a partial last block, one split short
    ([99999], 100000, 800),                                            # the single deep lane of config 3
], ids=["ragged-128", "partial-1024", "lane100k-800"])
def test_lane_batch_interleaved_blocks(contexts, cap, part):
    """The same rows with a lane's workgroups taking its blocks of 32 keys in turn: the
    records cover interleaved key sets, the combined output is held to the same bar."""
    print(f"[case] lane batch interleaved {contexts} part {part}", flush=True)
    _lane_batch(contexts, cap, part, 0x1E7E, replays=2, interleave=True)


@pytest.mark.parametrize("contexts,cap,part,interleave", [
    ([2000, 1499, 700, 100, 255, 256, 0, 287, 288, 319], 2048, 128, False),  # short rows between long ones
    ([300, 5000, 4999, 31, 2047], 8192, 1024, False),          # capacity well past every context
    ([99999], 100000, 800, True),                               # the single deep lane, blocks in turn
    ([32767, 29999, 24575, 8191], 32768, 768, False),           # config 3's ragged lanes, 252 live of 344
    ([1000] * 16, 1024, 128, False),                            # every row of a full wave
], ids=["ragged-128", "roomy-1024", "lane100k-800", "config3-ragged-768", "sixteen-lanes"])
def test_lane_batch_compact_dispatch_order(contexts, cap, part, interleave):
    """The workgroups that hold keys placed first in the dispatch order: same records as
    the order by grid position, so the output must equal that order's bit for bit, and
    the oracle's within the bar."""
    print(f"[case] lane batch compact {contexts} part {part}", flush=True)
    outputs = [_lane_batch(contexts, cap, part, 0xC0AC, replays=2 if compact else 0,
                           interleave=interleave, compact=compact) for compact in (False, True)]
    assert np.array_equal(outputs[0], outputs[1])


def test_compact_walk_compiled_once_replayed_while_contexts_grow():
    """One compiled split + combine, replayed after the state table has moved on: the rows'
    split counts change under the same grid (a row crosses a split boundary, a short row
    becomes a split-path row, a row's split count shrinks to zero when its lane is reset), and
    the workgroup placement has to follow from the table alone."""
    print("[case] compact walk, one graph, moving contexts", flush=True)
    B, dev, queue, lib = gpu()
    cap, part, rows = 2048, 128, 4
    stripe = 2 * cap * 256
    k_pool, stride = dev.create_pool(stripe * 2, rows)
    v_pool, _ = dev.create_pool(stripe * 2, rows)
    q = np.stack([ol.gaussian_bf16(0x6A01 + r, 4096) for r in range(rows)])
    gate = np.stack([ol.gaussian_bf16(0x6B01 + r, 4096) for r in range(rows)])
    keys = [ol.gaussian_bf16(0x6C01 + r, stripe).reshape(2, cap, 256) for r in range(rows)]
    values = [ol.gaussian_bf16(0x6D01 + r, stripe).reshape(2, cap, 256) for r in range(rows)]
    for r in range(rows):
        k_pool.write(keys[r], r * stride)
        v_pool.write(values[r], r * stride)
    b_q, b_g = dev.buffer_from(q), dev.buffer_from(gate)
    b_o = dev.create_buffer(rows * 8192)
    max_splits = cap // part
    b_part = dev.create_buffer(rows * 16 * max_splits * 258 * 4)
    b_tab = dev.create_buffer(256)
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    cb.encode(lib.pipeline("attention_decode_split_ms"),
              {0: b_q, 1: k_pool, 2: v_pool, 3: b_tab, 4: b_part},
              {5: cap, 6: 4096, 7: part, 8: max_splits, 9: 4}, (max_splits, 2, rows), (256,))
    cb.barrier()
    cb.encode(lib.pipeline("attention_decode_combine_ms"),
              {0: b_part, 1: b_g, 2: b_tab, 3: b_o}, {4: part, 5: max_splits, 6: 4096, 7: 0, 8: cap},
              (16, rows), (256,))
    cb.end_compute_pass()
    cb.compile()
    for contexts in ([255, 126, 2047, 600], [256, 127, 2047, 601], [257, 128, 0, 602],
                     [383, 1000, 1, 639], [384, 1001, 2, 640]):
        table = np.zeros(64, np.uint32)
        for r, ctx in enumerate(contexts):
            table[r * 4] = r * (stride // 2)
            table[r * 4 + 1] = ctx
        b_tab.write(table)
        b_o.write(np.zeros(rows * 4096, np.uint16))
        b_part.write(np.full(rows * 16 * max_splits * 258, np.nan, np.float32))
        cb.commit().wait()
        got = b_o.read(np.uint16).reshape(rows, 4096)
        for r, ctx in enumerate(contexts):
            want = np.zeros(4096, np.uint16)
            o.tto_attention_decode_split(q[r], gate[r], keys[r].reshape(-1), values[r].reshape(-1),
                                         ctx, cap, 256, None, want, 4)
            check_bf16(got[r], want, f"contexts {contexts} lane {r}")


@pytest.mark.parametrize("compact", [False, True], ids=["grid-order", "keyed-first"])
def test_table_rows_past_the_capacity_are_left_alone(compact):
    """A state-table row whose context is not a cache position (the capacity itself, or far
    past it) must neither be read nor written for: its output keeps what it held, the rows
    around it come out as always."""
    print(f"[case] lane batch with table rows past the capacity, compact={compact}", flush=True)
    B, dev, queue, lib = gpu()
    cap, part, rows = 1024, 128, 4
    stripe = 2 * cap * 256
    k_pool, stride = dev.create_pool(stripe * 2, rows)
    v_pool, _ = dev.create_pool(stripe * 2, rows)
    contexts = [700, cap, 300, cap + 4000]          # rows 1 and 3 are not cache positions
    q = np.stack([ol.gaussian_bf16(0x7A01 + r, 4096) for r in range(rows)])
    gate = np.stack([ol.gaussian_bf16(0x7B01 + r, 4096) for r in range(rows)])
    keys = [ol.gaussian_bf16(0x7C01 + r, stripe) for r in range(rows)]
    values = [ol.gaussian_bf16(0x7D01 + r, stripe) for r in range(rows)]
    table = np.zeros(64, np.uint32)
    for r in range(rows):
        k_pool.write(keys[r], r * stride)
        v_pool.write(values[r], r * stride)
        table[r * 4] = r * (stride // 2)
        table[r * 4 + 1] = contexts[r]
    b_tab, b_q, b_g = dev.buffer_from(table), dev.buffer_from(q), dev.buffer_from(gate)
    sentinel = np.full(rows * 4096, 0x4321, np.uint16)
    b_o = dev.buffer_from(sentinel)
    max_splits = cap // part
    b_part = dev.buffer_from(np.full(rows * 16 * max_splits * 258, np.nan, np.float32))

    def rec(cb):
        cb.encode(lib.pipeline("attention_decode_split_ms"),
                  {0: b_q, 1: k_pool, 2: v_pool, 3: b_tab, 4: b_part},
                  {5: cap, 6: 4096, 7: part, 8: max_splits, 9: 4 * int(compact)},
                  (max_splits, 2, rows), (256,))
        cb.barrier()
        cb.encode(lib.pipeline("attention_decode_combine_ms"),
                  {0: b_part, 1: b_g, 2: b_tab, 3: b_o}, {4: part, 5: max_splits, 6: 4096, 7: 0, 8: cap},
                  (16, rows), (256,))
    run(rec)
    got = b_o.read(np.uint16).reshape(rows, 4096)
    records = b_part.read(np.float32).reshape(rows, -1)
    for r, ctx in enumerate(contexts):
        if ctx >= cap:
            assert np.isnan(records[r]).all(), f"row {r}: records written for a context past the capacity"
            if ctx >= max_splits * part:
                assert (got[r] == 0x4321).all(), f"row {r}: output written"
            continue
        want = np.zeros(4096, np.uint16)
        o.tto_attention_decode_split(q[r], gate[r], keys[r], values[r], ctx, cap, 256, None, want, 4)
        check_bf16(got[r], want, f"lane {r} ctx {ctx} beside rows past the capacity")


def test_qk_rope_of_a_token_wave_on_striped_pools():
    """attn_qk_rope_ms: every row of a wave normed, rotated at its own position and appended
    to its own lane's stripe; a row whose context is not a cache position is skipped whole."""
    print("[case] attn_qk_rope_ms, 5 rows on reversed stripes, one row past the capacity", flush=True)
    B, dev, queue, lib = gpu()
    cap, rows = 512, 5
    contexts = [0, 511, 17, cap, 300]               # row 3 is not a cache position
    stripes = [4, 3, 2, 1, 0]
    q_w, k_w = _weights()
    stripe = 2 * cap * 256
    k_pool, stride = dev.create_pool(stripe * 2, rows)
    v_pool, _ = dev.create_pool(stripe * 2, rows)
    old_k = np.full(rows * (stride // 2), 0x1111, np.uint16)
    old_v = np.full(rows * (stride // 2), 0x2222, np.uint16)
    k_pool.write(old_k); v_pool.write(old_v)
    proj = np.stack([ol.gaussian_bf16(0x8A01 + r, 9216) for r in range(rows)])
    table = np.zeros(64, np.uint32)
    for r in range(rows):
        table[r * 4] = stripes[r] * (stride // 2)
        table[r * 4 + 1] = contexts[r]
    b_proj, b_tab = dev.buffer_from(proj), dev.buffer_from(table)
    b_qw, b_kw = dev.buffer_from(q_w), dev.buffer_from(k_w)
    b_q = dev.buffer_from(np.full(rows * 4096, 0x3333, np.uint16))
    b_g = dev.buffer_from(np.full(rows * 4096, 0x4444, np.uint16))

    def rec(cb):
        cb.encode(lib.pipeline("attn_qk_rope_ms"),
                  {0: b_proj, 1: b_qw, 2: b_kw, 3: b_q, 4: b_g, 5: k_pool, 6: v_pool, 8: b_tab},
                  {7: cap, 9: 9216, 10: 4096}, (18, rows), (256,))
    run(rec)
    got_q = b_q.read(np.uint16).reshape(rows, 4096)
    got_g = b_g.read(np.uint16).reshape(rows, 4096)
    got_k = k_pool.read(np.uint16).reshape(rows, stride // 2)
    got_v = v_pool.read(np.uint16).reshape(rows, stride // 2)
    want_k = old_k.reshape(rows, -1).copy(); want_v = old_v.reshape(rows, -1).copy()
    for r, ctx in enumerate(contexts):
        if ctx >= cap:
            assert (got_q[r] == 0x3333).all() and (got_g[r] == 0x4444).all()
            continue
        q = np.zeros(4096, np.uint16); gate = np.zeros(4096, np.uint16)
        lane_k = want_k[stripes[r], :stripe].copy(); lane_v = want_v[stripes[r], :stripe].copy()
        o.tto_attn_qk_rope(proj[r], q_w, k_w, ctx, cap, q, gate, lane_k, lane_v)
        want_k[stripes[r], :stripe] = lane_k; want_v[stripes[r], :stripe] = lane_v
        assert np.array_equal(got_g[r], gate)                              # raw copy: exact
        check_bf16(got_q[r], q, f"row {r} q at position {ctx}", ulps=1)
        assert np.mean(got_q[r] == q) > 0.99
    assert np.array_equal(got_v, want_v)                                   # raw copies, slots: exact
    # K: the appended rows within a bf16 step, every other element of every stripe untouched
    changed = got_k != want_k
    rope_rows = np.zeros_like(changed)
    for r, ctx in enumerate(contexts):
        if ctx < cap:
            for head in range(2):
                rope_rows[stripes[r], (head * cap + ctx) * 256:(head * cap + ctx + 1) * 256] = True
    assert not (changed & ~rope_rows).any()
    check_bf16(got_k[rope_rows], want_k[rope_rows], "appended K rows", ulps=1)


def test_qk_norm_over_every_bf16_value_bit_for_bit():
    """The qk norm of attn_qk_rope_ms on all 65536 bf16 bit patterns (non-finite ones replaced
    by zero; ordered by magnitude, so a head of 256 holds neighbouring binades) at position 0,
    where the rotation is the identity: the square sums, the inverse, both roundings and the
    flushes of the reference's model, bit for bit."""
    print("[case] attn_qk_rope_ms over every bf16 value", flush=True)
    B, dev, queue, lib = gpu()
    cap, rows = 32, 16
    patterns = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    patterns[(patterns & 0x7F80) == 0x7F80] = 0
    x = patterns[np.argsort(patterns & 0x7FFF, kind="stable")].reshape(rows, 16, 256)
    q_w, k_w = _weights()
    proj = np.zeros((rows, 9216), np.uint16)
    proj.reshape(rows, -1)[:, :8192].reshape(rows, 16, 2, 256)[:, :, 0, :] = x     # q halves
    proj[:, 8192:8704] = x[:, 5:7, :].reshape(rows, 512)                            # two k heads
    stripe = 2 * cap * 256
    k_pool, stride = dev.create_pool(stripe * 2, rows)
    v_pool, _ = dev.create_pool(stripe * 2, rows)
    table = np.zeros(64, np.uint32)
    for r in range(rows):
        table[r * 4] = r * (stride // 2)
    b_proj, b_tab = dev.buffer_from(proj), dev.buffer_from(table)
    b_qw, b_kw = dev.buffer_from(q_w), dev.buffer_from(k_w)
    b_q, b_g = dev.create_buffer(rows * 8192), dev.create_buffer(rows * 8192)
    run(lambda cb: cb.encode(lib.pipeline("attn_qk_rope_ms"),
                             {0: b_proj, 1: b_qw, 2: b_kw, 3: b_q, 4: b_g, 5: k_pool, 6: v_pool,
                              8: b_tab}, {7: cap, 9: 9216, 10: 4096}, (18, rows), (256,)))
    got_q = b_q.read(np.uint16).reshape(rows, 4096)
    got_k = k_pool.read(np.uint16).reshape(rows, stride // 2)
    for r in range(rows):
        q = np.zeros(4096, np.uint16); gate = np.zeros(4096, np.uint16)
        keys = np.zeros(stripe, np.uint16); values = np.zeros(stripe, np.uint16)
        o.tto_attn_qk_rope(proj[r], q_w, k_w, 0, cap, q, gate, keys, values)
        differ = np.flatnonzero(got_q[r] != q)
        assert differ.size == 0, (f"row {r}: {differ.size} q values differ, first: input "
                                  f"{x[r].reshape(-1)[differ[0]]:#06x} got "
                                  f"{got_q[r][differ[0]]:#06x} want {q[differ[0]]:#06x}")
        assert np.array_equal(got_k[r, :stripe], keys), f"row {r}: K rows"


@pytest.mark.parametrize("position", [100000, 65535, 262143])
def test_qk_rope_far_positions(position):
    """The rotation at the deep end of config 3 and beyond: angles up to 2.6e5 rad, where the
    sine and cosine stand or fall with the argument reduction.  Against the golden q of the
    reference's model at position 100000, and the checker within a bf16 step elsewhere."""
    print(f"[case] attn_qk_rope at position {position}", flush=True)
    B, dev, queue, lib = gpu()
    proj, q_w, k_w = cases.attention_chain_inputs(ol.banded_bf16)
    cap = position + 1
    b_p, b_qw, b_kw = dev.buffer_from(proj[0]), dev.buffer_from(q_w), dev.buffer_from(k_w)
    b_q, b_g = dev.create_buffer(8192), dev.create_buffer(8192)
    b_k, b_v = dev.create_buffer(2 * cap * 512), dev.create_buffer(2 * cap * 512)
    run(lambda cb: cb.encode(lib.pipeline("attn_qk_rope"),
                             {0: b_p, 1: b_qw, 2: b_kw, 3: b_q, 4: b_g, 5: b_k, 6: b_v},
                             {7: position, 8: cap}, (18,), (256,)))
    q = np.zeros(4096, np.uint16); gate = np.zeros(4096, np.uint16)
    keys = np.zeros(2 * cap * 256, np.uint16); values = np.zeros_like(keys)
    o.tto_attn_qk_rope(proj[0], q_w, k_w, position, cap, q, gate, keys, values)
    if position == 100000:
        G = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz"))
        assert np.array_equal(q, G["rope_far_q"])
    got_q = b_q.read(np.uint16)
    got_k = b_k.read(np.uint16).reshape(2, cap, 256)[:, position]
    for what, got, want in (("q", got_q, q), ("k row", got_k.reshape(-1),
                                              keys.reshape(2, cap, 256)[:, position].reshape(-1))):
        g = ol.bf16_to_f32(got).reshape(-1, 256)
        w = ol.bf16_to_f32(want).reshape(-1, 256)
        # a rotated value may be the small difference of two large products: the step that
        # counts is the one of the pair's size (the rotation keeps the pair's norm)
        size = np.abs(w).copy()
        pair = np.maximum(size[:, :32], size[:, 32:64])
        size[:, :32] = pair; size[:, 32:64] = pair
        rel = np.abs(g - w) / np.maximum(size, 1e-3)
        print(f"[parity] far rope {what}: exact {np.mean(got == want):.4f} max-rel {rel.max():.3e}",
              flush=True)
        assert rel.max() <= 2 ** -7          # at most one bf16 step of the pair's size
        assert np.mean(got == want) > 0.99
    assert np.array_equal(b_g.read(np.uint16), gate)


def test_lane_on_the_last_stripe_a_32_bit_offset_can_name():
    """State-table offsets are 32-bit element counts (decode_step.cpp:476): a pool of 127
    stripes of a 65536-key cache (8.5 GB) puts the last stripe 4.23e9 elements in, the first
    one at zero.  Every address past the table entry has to be 64-bit arithmetic."""
    print("[case] lane batch on stripes 126 and 0 of 127 x 65536 keys", flush=True)
    cap, pool_stripes = 65536, 127
    assert (pool_stripes - 1) * 2 * cap * 256 > 0.98 * 2 ** 32      # the last stripe's offset
    assert (pool_stripes + 1) * 2 * cap * 512 > 2 * 0xFFFFFFFF      # one stripe more is refused
    _lane_batch([65535, 40000], cap, 1024, 0x32B1, replays=1, compact=True, stripes=[126, 0],
                pool_stripes=pool_stripes)
    # order by grid position, blocks in turn, and a short row through attention_decode_ms
    _lane_batch([100, 5000], cap, 512, 0x32B2, interleave=True, stripes=[126, 125],
                pool_stripes=pool_stripes)
    # the appending side: the rope of a token wave writes its K / V rows there
    B, dev, queue, lib = gpu()
    stripe = 2 * cap * 256
    k_pool, stride = dev.create_pool(stripe * 2, pool_stripes)
    v_pool, _ = dev.create_pool(stripe * 2, pool_stripes)
    q_w, k_w = _weights()
    proj = np.stack([ol.gaussian_bf16(0x32C1 + r, 9216) for r in range(2)])
    positions, stripes = [65535, 7], [126, 0]
    table = np.zeros(64, np.uint32)
    for r in range(2):
        table[r * 4] = stripes[r] * (stride // 2)
        table[r * 4 + 1] = positions[r]
    b_proj, b_tab = dev.buffer_from(proj), dev.buffer_from(table)
    b_qw, b_kw = dev.buffer_from(q_w), dev.buffer_from(k_w)
    b_q, b_g = dev.create_buffer(2 * 8192), dev.create_buffer(2 * 8192)
    run(lambda cb: cb.encode(lib.pipeline("attn_qk_rope_ms"),
                             {0: b_proj, 1: b_qw, 2: b_kw, 3: b_q, 4: b_g, 5: k_pool, 6: v_pool,
                              8: b_tab}, {7: cap, 9: 9216, 10: 4096}, (18, 2), (256,)))
    for r in range(2):
        q = np.zeros(4096, np.uint16); gate = np.zeros(4096, np.uint16)
        keys = np.zeros(stripe, np.uint16); values = np.zeros(stripe, np.uint16)
        o.tto_attn_qk_rope(proj[r], q_w, k_w, positions[r], cap, q, gate, keys, values)
        got_v = v_pool.read(np.uint16, stripe, stripes[r] * stride)
        got_k = k_pool.read(np.uint16, stripe, stripes[r] * stride)
        assert np.array_equal(got_v, values), f"row {r}: V rows of stripe {stripes[r]}"
        assert np.array_equal(got_k != 0, keys != 0), f"row {r}: which K elements were written"
        check_bf16(got_k, keys, f"row {r} K row on stripe {stripes[r]}", ulps=1)


def test_lane_at_the_longest_context_of_the_model():
    """One lane at 262144 visible keys (the model's context length): 128 splits of 2048 keys
    as the host picks them, blocks in turn, the 128-record combine."""
    print("[case] lane batch, 1 lane at 262144 keys", flush=True)
    from tatara_amd import stack as S
    assert S.choose_split_keys([262144]) == 2048
    _lane_batch([262143], 262144, 2048, 0x40000, interleave=True)


def test_lane_batch_drawn_shapes():
    """Two dozen waves drawn from a fixed seed: 1 to 16 lanes, contexts anywhere in the cache
    (empty and full ones among them), split sizes from one block up, every combination of the
    dispatch order and the block order; half of them also compiled and replayed."""
    import random
    rng = random.Random(0xD1CE)
    for case in range(24):
        rows = rng.choice([1, 2, 3, 4, 5, 8, 11, 16])
        cap = rng.choice([512, 1024, 2048, 4096])
        part = 32 * rng.randint(1, 16)
        contexts = [rng.choice([0, cap - 1, rng.randrange(cap), rng.randrange(cap)]) for _ in range(rows)]
        interleave, compact = rng.random() < 0.5, rng.random() < 0.5
        rotate = 0 if interleave else (0, 1, 1, 3, 31)[case % 5]
        print(f"[case] drawn wave {case}: contexts {contexts} cap {cap} part {part} "
              f"interleave {interleave} compact {compact} rotate {rotate}", flush=True)
        _lane_batch(contexts, cap, part, 0xD1CE00 + case, replays=case % 2, interleave=interleave,
                    compact=compact, rotate=rotate)


def test_lane_batch_with_scores_in_the_hundreds():
    """Queries 32 times as large: scores of several hundred either way, a softmax that is one-hot
    to working precision, records whose maxima differ by hundreds between splits."""
    print("[case] lane batch, queries x 32", flush=True)
    _lane_batch([5000, 4999, 31, 2047, 300], 8192, 512, 0x5A4B, replays=1, compact=True, sharpen=5)
    _lane_batch([40000], 40960, 320, 0x5A4C, interleave=True, sharpen=5)


def test_lane_batch_with_zero_queries():
    """Every score zero: the output is the plain mean of the visible values times the gate,
    each split's record a sum of `part` values with weight one."""
    print("[case] lane batch, zero queries", flush=True)
    _lane_batch([5000, 0, 255, 256, 8191], 8192, 1024, 0x5A4D, compact=True, sharpen=-1)


def test_four_deep_lanes_with_the_split_the_host_picks():
    """Four lanes around 100k keys: the host's rule goes well past 1024 keys a workgroup here
    (2656: 25 to 38 workgroups per lane and head, 256 in all), ranges in a grid that covers
    the capacity."""
    from tatara_amd import stack as S
    contexts = [99999, 65535, 99999, 70000]
    part = S.choose_split_keys([c + 1 for c in contexts])
    print(f"[case] lane batch, 4 deep lanes, {part} keys per workgroup", flush=True)
    assert part > 1024 and S.split_workgroups([c + 1 for c in contexts], part) <= 256
    _lane_batch(contexts, 100000, part, 0xDEE9, replays=1, compact=True)


def test_config3_four_ragged_lanes_at_depth():
    """Config 3: lanes at (32768, 30000, 24576, 8192) visible keys in a
    capacity-32768 pool."""
    print("[case] config 3: 4 ragged lanes 32768/30000/24576/8192", flush=True)
    _lane_batch([32767, 29999, 24575, 8191], 32768, 512, 0xC0F3)


def test_headline_shape_four_lanes_32768_split_1024_graph_replay():
    """The benchmark's own configuration: 4 lanes x 32768 visible keys, 1024 keys per
    split (32 records per head: the all-loads-up-front combine), eager and as a
    compiled walk."""
    print("[case] headline shape: 4 x 32768, split 1024, graph replay", flush=True)
    _lane_batch([32767] * 4, 32768, 1024, 0xBE7C, replays=3)


@pytest.mark.parametrize("cap", [33024, 131136])
def test_rotated_walk_at_capacities_that_alias(cap):
    """The benchmark's lanes in caches whose capacity used to put the ranges of the 256
    workgroups on the same memory channels: the host walks such ranges from a rotated starting
    block (and, the grid being larger than the chip, with the workgroups that hold keys
    first).  Same bar as every other order, eager and replayed."""
    print(f"[case] 4 x 32768 in capacity {cap}, rotated ranges, keyed first", flush=True)
    _lane_batch([32767] * 4, cap, 1024, 0xA11A5 + cap, replays=2, compact=True, rotate=1)


def test_rotated_ranges_with_partial_and_single_blocks():
    """Rotation where it has little room: ranges of one block (nothing to rotate), a last range
    with a partial block, a last range of a single partial block, contexts of 0 and 31."""
    print("[case] rotated ranges, partial and single blocks", flush=True)
    _lane_batch([2000, 1499, 700, 100, 255, 256, 0, 31, 32, 319], 2048, 32, 0x2071, rotate=1)
    _lane_batch([5000, 4999, 31, 1024, 1025], 5120, 1024, 0x2072, replays=1, rotate=1)
    _lane_batch([5000, 4127, 4128, 63], 5120, 96, 0x2073, compact=True, rotate=7)


def test_lane_batch_record_counts_straddle_32():
    """Rows with 64, 33, 32, 31 and 1 records per head in one dispatch: both combine
    paths (up to 32 records with every load up front, more than 32 staged) side by side."""
    print("[case] lane batch, records per head 64/33/32/31/1", flush=True)
    _lane_batch([8191, 4096, 4095, 3967, 100], 8192, 128, 0x5732, replays=2)


def test_config3_single_lane_100k():
    print("[case] config 3: 1 lane, 100000 visible keys, capacity 100096", flush=True)
    _lane_batch([99999], 100096, 512, 0xC0F4)


def test_binding_validation_precedes_dispatch():
    """Typed errors are returned before anything is launched
    (commands.mm:607-648 behaviour)."""
    B, dev, queue, lib = gpu()
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    small = dev.create_buffer(64)
    cb.set_pipeline(lib.pipeline("attention_decode"))
    with pytest.raises(B.BackendError) as e:
        cb.set_buffer(small, 64, 0)
    assert e.value.status == 10          # InvalidBufferOffset
    with pytest.raises(B.BackendError) as e:
        cb.set_buffer(small, 0, 31)
    assert e.value.status == 9           # InvalidBufferIndex
    with pytest.raises(B.BackendError) as e:
        cb.dispatch((16, 0, 1), (256,))
    assert e.value.status == 15          # InvalidDispatchExtent
    # context == capacity is one past the cache
    big = dev.create_buffer(2 * 8 * 512)
    q = dev.create_buffer(8192)
    for i, b in {0: q, 1: q, 2: big, 3: big, 5: q}.items():
        cb.set_buffer(b, 0, i)
    cb.set_bytes(8, 4); cb.set_bytes(8, 6)
    with pytest.raises(B.BackendError) as e:
        cb.dispatch((16,), (256,))
    assert e.value.status == 16          # ContextOutOfRange
    # a cache smaller than capacity says is refused, not read out of bounds
    cb.set_bytes(3, 4); cb.set_bytes(4096, 6)
    with pytest.raises(B.BackendError) as e:
        cb.dispatch((16,), (256,))
    assert e.value.status == 10
    assert cb.command_count == 0


def test_compiled_walk_replays_equal_eager():
    """A recording compiled into a HIP graph, replayed several times with eager
    work and synchronisation in between, gives the eager result every time."""
    print("[case] graph replay vs eager", flush=True)
    B, dev, queue, lib = gpu()
    cap, ctx, part = 4096, 3000, 256
    q = ol.gaussian_bf16(71, 4096); gate = ol.gaussian_bf16(72, 4096)
    keys = ol.gaussian_bf16(73, 2 * cap * 256); values = ol.gaussian_bf16(74, 2 * cap * 256)
    b_q, b_g = dev.buffer_from(q), dev.buffer_from(gate)
    b_k, b_v = dev.buffer_from(keys), dev.buffer_from(values)
    nparts = (ctx + part) // part
    b_part = dev.create_buffer(16 * nparts * 258 * 4)
    b_o = dev.create_buffer(8192)

    def rec(cb):
        cb.encode(lib.pipeline("attention_decode_scores_values_gqa8"),
                  {0: b_q, 1: b_k, 2: b_v, 6: b_part}, {3: ctx, 4: cap, 5: part, 7: nparts},
                  (2, nparts), (256, 4))
        cb.barrier()
        cb.encode(lib.pipeline("attention_decode_combine"), {0: b_part, 1: b_g, 3: b_o},
                  {2: nparts}, (16,), (256,))
    run(rec)
    eager = b_o.read(np.uint16)
    cb = queue.create_command_buffer()
    cb.begin_compute_pass(); rec(cb); cb.end_compute_pass()
    cb.compile()
    for replay in range(4):
        b_o.write(np.zeros(4096, np.uint16))
        b_part.write(np.zeros(16 * nparts * 258, np.float32))
        cb.commit().wait()
        assert np.array_equal(b_o.read(np.uint16), eager), f"replay {replay}"
        run(rec)   # eager work between replays
        assert np.array_equal(b_o.read(np.uint16), eager)
