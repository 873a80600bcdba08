"""Block-prefill full attention on the GPU against the CPU checker (exact
partial/combine semantics, row r sees keys [0, context + r]).  Tolerance of the
path: max-abs <= 2e-2, mean-abs <= 2e-3; cache rows written by the rope stage are
compared at the decode tests' bar."""
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


def _prefill_case(rows, base, cap, seed, select=None, control=False, proj=None, weights=None,
                  splits=None, replays=0):
    """Runs rope + flash prefill on the GPU for `rows` new tokens after `base`
    cached ones and compares the selected rows with the checker.  splits: through
    attention_flash_split_blk with that many workgroups sharing each position tile's key walk,
    and held to the one-workgroup operator's result as well."""
    B, dev, queue, lib = gpu()
    q_w, k_w = _weights() if weights is None else weights
    if proj is None:
        proj = ol.gaussian_bf16(seed, rows * 9216)
    keys = np.zeros(2 * cap * 256, np.uint16); values = np.zeros_like(keys)
    if base:
        keys.reshape(2, cap, 256)[:, :base] = ol.gaussian_bf16(seed + 1, 2 * base * 256).reshape(
            2, base, 256)
        values.reshape(2, cap, 256)[:, :base] = ol.gaussian_bf16(seed + 2, 2 * base * 256).reshape(
            2, base, 256)
    b_k, b_v = dev.buffer_from(keys), dev.buffer_from(values)
    sel = np.arange(rows, dtype=np.uint32) if select is None else np.asarray(select, np.uint32)
    query = np.zeros(rows * 4096, np.uint16); gate = np.zeros_like(query)
    want = np.zeros_like(query)
    o.tto_attention_prefill(proj, q_w, k_w, rows, base, cap, query, gate, keys, values, sel,
                            len(sel), want, 8)
    b_p = dev.buffer_from(proj)
    b_qw, b_kw = dev.buffer_from(q_w), dev.buffer_from(k_w)
    b_q, b_g, b_o = (dev.create_buffer(rows * 8192) for _ in range(3))
    tiles = (rows + 15) // 16
    if splits:
        # scratch starts as 0xFF bytes: the operator clears its arrival counts itself
        need = B.flash_prefill_scratch_bytes(rows, splits)
        b_s = dev.buffer_from(np.full(max(need, 256), 0xFF, np.uint8))

    def flash(cb, out):
        if splits:
            cb.encode(lib.pipeline("attention_flash_split_blk"),
                      {0: b_q, 1: b_k, 2: b_v, 3: b_g, 4: out, 9: b_s},
                      {5: base + rows, 6: cap, 7: rows, 8: base, 10: splits}, (16, tiles), (256,))
        else:
            # the reference's two names of the streaming path resolve to the one kernel
            cb.encode(lib.pipeline("attention_streaming_blk" if base % 2 else "attention_flash_v2_blk"),
                      {0: b_q, 1: b_k, 2: b_v, 3: b_g, 4: out},
                      {5: base + rows, 6: cap, 7: rows, 8: base}, (16, tiles), (256,))

    def rec(cb):
        cb.encode(lib.pipeline("attn_qk_rope_blk"),
                  {0: b_p, 1: b_qw, 2: b_kw, 3: b_q, 4: b_g, 5: b_k, 6: b_v}, {7: base, 8: cap},
                  (18, rows), (256,))
        cb.barrier()
        flash(cb, b_o)
    ms = run(rec)
    got = b_o.read(np.uint16).reshape(rows, 4096)
    w = want.reshape(rows, 4096)
    what = f"flash prefill rows {rows} base {base}" + (f" splits {splits}" if splits else "")
    check_bf16(got[sel], w[sel], what)
    if splits:
        # against one workgroup per position tile: each share rounds its probabilities to bf16
        # against its own reference, so the two differ like either does from the checker
        # (c10 = 1; attention_flash_v2_blk shares walks by itself through its queue's workspace)
        b_o1 = dev.create_buffer(rows * 8192)
        run(lambda cb: cb.encode(lib.pipeline("attention_flash_split_blk"),
                                 {0: b_q, 1: b_k, 2: b_v, 3: b_g, 4: b_o1},
                                 {5: base + rows, 6: cap, 7: rows, 8: base, 10: 1}, (16, tiles), (256,)))
        check_bf16(got, b_o1.read(np.uint16).reshape(rows, 4096), what + " vs one workgroup a tile",
                   max_abs=8e-3, mean_abs=2e-4, ulps=2)
    if replays:
        # a compiled command buffer replayed: every replay clears and counts again
        cb = queue.create_command_buffer()
        cb.begin_compute_pass(); flash(cb, b_o); cb.end_compute_pass()
        cb.compile()
        for replay in range(replays):
            b_o.write(np.zeros(rows * 4096, np.uint16))
            cb.commit().wait()
            again = b_o.read(np.uint16).reshape(rows, 4096)
            check_bf16(again, got, what + f" replay {replay}", max_abs=8e-3, mean_abs=1e-5, ulps=1)
    # cache: raw V exact, roped K at the decode bar, rows beyond untouched
    gk = b_k.read(np.uint16).reshape(2, cap, 256)
    gv = b_v.read(np.uint16).reshape(2, cap, 256)
    assert np.array_equal(gv, values.reshape(2, cap, 256))
    check_bf16(gk, keys, "prefill K cache", max_abs=4e-2, mean_abs=1e-4)
    check_bf16(b_q.read(np.uint16), query, "prefill roped Q", max_abs=4e-2, mean_abs=1e-4)
    assert np.array_equal(b_g.read(np.uint16), gate)
    if control:
        parts = (base + rows + 255) // 256
        b_part = dev.create_buffer(16 * rows * parts * 258 * 4)
        b_o2 = dev.create_buffer(rows * 8192)

        def rec2(cb):
            cb.encode(lib.pipeline("attention_partial_blk"), {0: b_q, 1: b_k, 2: b_v, 6: b_part},
                      {3: base, 4: cap, 5: 256, 7: parts, 8: rows}, (16, parts, rows), (256,))
            cb.barrier()
            cb.encode(lib.pipeline("attention_combine_blk"), {0: b_part, 1: b_g, 3: b_o2},
                      {2: parts, 4: rows}, (16, rows), (256,))
        run(rec2)
        got2 = b_o2.read(np.uint16).reshape(rows, 4096)
        check_bf16(got2[sel], w[sel], f"partial/combine control rows {rows} base {base}")
        # fast vs control, the reference's own band (normalised error <= 0.02,
        # attention_fixture_probe.cpp:1241-1269)
        a, c = ol.bf16_to_f32(got.reshape(-1)), ol.bf16_to_f32(got2.reshape(-1))
        assert np.abs(a - c).max() / max(np.abs(c).max(), 1e-6) <= 0.02
    return ms, dict(b_q=b_q, b_g=b_g, b_k=b_k, b_v=b_v, got=got, cap=cap, base=base)


def test_block_13_rows_at_context_300():
    """The reference probe's block: 13 rows at context 300 -> 313 visible, capacity 512."""
    print("[case] prefill 13 rows at context 300", flush=True)
    _prefill_case(13, 300, 512, 0xB10C, control=True)


@pytest.mark.parametrize("rows,base", [(1, 0), (16, 0), (17, 0), (48, 0), (100, 1000), (256, 31),
                                       (300, 33)])
def test_block_shapes(rows, base):
    print(f"[case] prefill rows {rows} base {base}", flush=True)
    _prefill_case(rows, base, 2048, 0x5EED + rows, control=rows <= 48)


def test_block_at_the_deep_end_of_a_100k_cache():
    """13 rows appended at positions 99987 .. 99999: the block rope's angles at the far end
    (argument reduction), 32-bit offsets into a 102 MB cache, and a flash pass over 100k keys."""
    print("[case] prefill 13 rows at context 99987, capacity 100000", flush=True)
    _prefill_case(13, 99987, 100000, 0xFA12, control=False)


def test_prefill_row_equals_decode_step_on_gpu():
    """Row r of a block at context c is the decode operator at context c + r over
    the same cache (prefill_attention.metal:117-119)."""
    print("[case] prefill rows vs decode operator", flush=True)
    B, dev, queue, lib = gpu()
    rows, base, cap = 40, 500, 1024
    _, c = _prefill_case(rows, base, cap, 0xD3C0)
    for r in (0, 15, 16, 39):
        b_o = dev.create_buffer(8192)
        run(lambda cb: cb.encode(lib.pipeline("attention_decode"),
                                 {0: (c["b_q"], r * 8192), 1: (c["b_g"], r * 8192), 2: c["b_k"],
                                  3: c["b_v"], 5: b_o}, {4: base + r, 6: cap}, (16,), (256,)))
        check_bf16(b_o.read(np.uint16), c["got"][r], f"decode vs prefill row {r}",
                   max_abs=8e-3, mean_abs=2e-4)


def test_scores_far_above_the_first_tile_take_the_exact_loop():
    """The flash kernel fixes each row's softmax reference at its first key tile
    and falls back to an exact online-softmax loop when a later score exceeds it
    by more than 2^100.  Norm weights of 3 and late keys that repeat the last
    row's query direction give scores near 150 log2 units above the early ones,
    so the last position tiles finish in that loop."""
    print("[case] prefill with scores that force the exact softmax loop", flush=True)
    rows = 96
    proj = ol.gaussian_bf16(0xE8AC, rows * 9216).reshape(rows, 9216)
    for r in range(64, rows):
        proj[r, 8192:8448] = proj[rows - 1, 0:256]          # kv head 0 key := head 0 query of the last row
        proj[r, 8448:8704] = proj[rows - 1, 4096:4352]      # kv head 1 key := head 8 query of the last row
    w = np.full(256, 0x4040, np.uint16)                     # 3.0
    _prefill_case(rows, 0, 128, 0xE8AD, proj=np.ascontiguousarray(proj).reshape(-1), weights=(w, w),
                  control=True)


@pytest.mark.parametrize("rows,base,splits", [(64, 1000, 2), (64, 1000, 8), (37, 700, 4), (13, 300, 8),
                                              (1, 0, 8), (1, 4000, 3), (300, 33, 2), (100, 5000, 8),
                                              (40, 95, 5)])
def test_key_walk_shared_between_workgroups(rows, base, splits):
    """attention_flash_split_blk: up to eight workgroups share a position tile's key walk and the
    last to finish adds the others' results to its own.  Walks too short for the count asked
    are shared by fewer (13 rows at 300: two of eight; the first tiles of a block at context
    0 or 33: one), rows that are not whole tiles, one row."""
    print(f"[case] shared key walk rows {rows} base {base} splits {splits}", flush=True)
    _prefill_case(rows, base, 8192, 0x5A1E + rows + splits, splits=splits, replays=2)


def test_shared_walk_with_a_share_in_the_exact_loop():
    """The upper share of the last position tiles meets scores 150 log2 units above its first
    tile's and finishes in the exact loop; its reference then lies far above the lower share's,
    whose result the merge scales to nothing."""
    print("[case] shared key walk, one share in the exact softmax loop", flush=True)
    rows = 320
    proj = ol.gaussian_bf16(0xE8B0, rows * 9216).reshape(rows, 9216)
    for r in range(288, rows):
        proj[r, 8192:8448] = proj[rows - 1, 0:256]
        proj[r, 8448:8704] = proj[rows - 1, 4096:4352]
    w = np.full(256, 0x4040, np.uint16)                     # 3.0
    _prefill_case(rows, 0, 512, 0xE8B1, proj=np.ascontiguousarray(proj).reshape(-1), weights=(w, w),
                  splits=2, select=list(range(0, 320, 7)) + list(range(280, 320)))


def test_shared_walk_of_a_2048_row_block_deep_in_a_cache():
    """The shape the operator is for: a 2048-row block behind 6144 cached tokens, as many shares
    as fill the device (two on 256 compute units); sampled rows against the checker, every row
    against the one-workgroup operator."""
    B, dev, queue, lib = gpu()
    splits = B.flash_prefill_splits(2048, 8192, dev.compute_units)
    print(f"[case] shared key walk, 2048 rows at context 6144, splits {splits}", flush=True)
    rows = [0, 1, 31, 32, 33, 1000, 1023, 1024, 2016, 2047] + list(range(300, 2048, 97))
    ms, _ = _prefill_case(2048, 6144, 8192, 0x2048, select=sorted(set(rows)), splits=max(splits, 2))
    print(f"[time] rope + flash, 2048 rows at 6144: {ms:.3f} ms", flush=True)


def test_shared_walk_on_drawn_shapes_against_one_workgroup_a_tile():
    """Twenty drawn blocks (1-700 rows behind 0-9000 cached tokens, 2-8 sharers asked for, random
    bf16 operands straight into the flash operators): the shared walk - with the caller's scratch
    and count, and as attention_flash_v2_blk plans it in its queue's workspace - against the
    unshared one on the same buffers, and no row left unwritten."""
    B, dev, queue, lib = gpu()
    rng = np.random.default_rng(0x5A4E)
    cap = 9728
    keys = dev.buffer_from(ol.gaussian_bf16(0x5A4F, 2 * cap * 256))
    values = dev.buffer_from(ol.gaussian_bf16(0x5A50, 2 * cap * 256))
    for case in range(20):
        rows = int(rng.integers(1, 701))
        base = int(rng.integers(0, 9001)) if case % 4 else 0
        splits = int(rng.integers(2, 9))
        print(f"[case] drawn block {case}: rows {rows} base {base} splits {splits}", flush=True)
        q = dev.buffer_from(ol.gaussian_bf16(0x6000 + case, rows * 4096, 0.0, 0.25))
        gate = dev.buffer_from(ol.gaussian_bf16(0x7000 + case, rows * 4096))
        outs = [dev.buffer_from(np.full(rows * 4096, 0x7FC0, np.uint16)) for _ in range(3)]
        scratch = dev.buffer_from(np.full(max(B.flash_prefill_scratch_bytes(rows, splits), 256), 0xA5, np.uint8))
        const = {5: base + rows, 6: cap, 7: rows, 8: base}
        grid = (16, (rows + 15) // 16)

        def rec(cb):
            cb.encode(lib.pipeline("attention_flash_split_blk"), {0: q, 1: keys, 2: values, 3: gate, 4: outs[0]},
                      {**const, 10: 1}, grid, (256,))
            cb.encode(lib.pipeline("attention_flash_split_blk"),
                      {0: q, 1: keys, 2: values, 3: gate, 4: outs[1], 9: scratch}, {**const, 10: splits},
                      grid, (256,))
            cb.encode(lib.pipeline("attention_flash_v2_blk"), {0: q, 1: keys, 2: values, 3: gate, 4: outs[2]},
                      const, grid, (256,))
        run(rec)
        one, shared, planned = (o_.read(np.uint16) for o_ in outs)
        check_bf16(shared, one, f"drawn block {case}", max_abs=8e-3, mean_abs=2e-4, ulps=2)
        check_bf16(planned, one, f"drawn block {case}, planned by the operator", max_abs=8e-3,
                   mean_abs=2e-4, ulps=2)


def test_config4_prefill_16384_rows():
    """Config 4: 16384 new tokens into an empty capacity-16384 cache.  The checker
    computes a strided subset of query rows (every 257th plus the first and last
    16: a stride coprime with the kernel's 32-row tile, so every row of a tile is
    compared somewhere at depth); the K/V cache written by the rope stage is compared in
    full."""
    print("[case] config 4: prefill 16384 rows", flush=True)
    rows = 16384
    sel = sorted(set(list(range(16)) + list(range(0, rows, 257)) + list(range(rows - 16, rows))))
    assert {r % 32 for r in sel} == set(range(32))
    ms, _ = _prefill_case(rows, 0, rows, 0xC0F4, select=sel)
    print(f"[time] rope + flash prefill 16384 rows (first run): {ms:.3f} ms", flush=True)
