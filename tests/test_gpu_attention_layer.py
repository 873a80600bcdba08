"""The whole decode attention layer in one dispatch (attention_decode_layer_ms) on the GPU
against the CPU checker, through the C ABI: qk-norm and rotation of the new token, K / V
append, split-K attention with the keys of all lanes dealt evenly to the workgroups, and
the gated combine - finished by a second dispatch or inside the first by the last
workgroup of each (row, kv head) stream.  Both forms must give the same bits; outputs are
held to the path's tolerance (max-abs 2e-2, mean-abs 2e-3), the appended V row and every
untouched cache row are exact, the appended K row is the rope operator's (one bf16 step
where the device's cosine differs from libm's; deep in a context also what one fp32 step of
the rotation frequency moves the angle)."""
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


def _layer_batch(contexts, cap, groups_list, seed, replays=0, projection_stride=9216,
                 query_stride=4096, stripes=None, pool_stripes=None):
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
    for groups in groups_list:
        b_scratch = dev.create_buffer(256 + 131072 + (groups + 2 * rows - 1) * 8 * 258 * 4)
        for mode in (0, 1):
            for r, (k, v, _, _) in enumerate(caches):   # caches back to their state before the token
                k_pool.write(k, stripes[r] * stride)
                v_pool.write(v, stripes[r] * stride)
            b_o = dev.create_buffer(rows * query_stride * 2)
            bind = {0: b_proj, 1: b_qw, 2: b_kw, 3: k_pool, 4: v_pool, 5: b_tab, 6: b_scratch, 7: b_o}
            const = {8: cap, 9: projection_stride, 10: query_stride}

            def rec(cb, mode=mode, bind=bind, const=const, groups=groups):
                cb.encode(lib.pipeline("attention_decode_layer_ms"), bind, {**const, 11: mode},
                          (groups, rows), (256,))
                if mode == 0:
                    cb.barrier()
                    cb.encode(lib.pipeline("attention_decode_layer_finish_ms"), bind,
                              {**const, 11: groups}, (16, rows), (64,))
            run(rec)
            got = b_o.read(np.uint16).reshape(rows, query_stride)[:, :4096]
            what = f"groups {groups} mode {mode}"
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
            assert not b_scratch.read(np.uint32, 64).any(), f"{what}: tickets not left at zero"
            outs[(groups, mode)] = got.copy()
            if mode == 1 and replays:
                cb = queue.create_command_buffer()
                cb.begin_compute_pass(); rec(cb); cb.end_compute_pass()
                cb.compile()
                for replay in range(replays):
                    b_o.write(np.zeros(rows * query_stride, np.uint16))
                    cb.commit().wait()
                    again = b_o.read(np.uint16).reshape(rows, query_stride)[:, :4096]
                    assert np.array_equal(again, got), f"{what} replay {replay}"
        assert np.array_equal(outs[(groups, 0)], outs[(groups, 1)]), \
            f"groups {groups}: finishing inside the dispatch differs from the second dispatch"
    return outs


@pytest.mark.parametrize("groups", [1, 7, 64, 256, 512])
def test_layer_small_ragged_lanes(groups):
    """Seven ragged lanes incl. an empty cache and contexts around the 32-key unit and the
    256-key partition; 1 workgroup walks every stream, 512 leave some workgroups idle."""
    print(f"[case] decode layer, 7 ragged lanes, {groups} workgroups", flush=True)
    _layer_batch([2000, 1499, 700, 100, 255, 256, 0], 2048, [groups], 0x1A7E, replays=2)


@pytest.mark.parametrize("ctx", [0, 1, 31, 32, 33, 63, 64, 65, 300, 1000])
def test_layer_single_lane_context_edges(ctx):
    print(f"[case] decode layer, one lane, context {ctx}", flush=True)
    _layer_batch([ctx], 1100, [3, 32], 0x2B00 + ctx)


@pytest.mark.parametrize("groups", [10, 11, 40, 300])
def test_layer_tiny_streams_between_deep_ones(groups):
    """Lanes of 3, 0 and 40 cached keys beside lanes of thousands: every stream that holds
    keys keeps a workgroup of its own however small its share (10 workgroups for 10
    streams), and more workgroups than a short stream has 32-key units leave some idle."""
    print(f"[case] decode layer, tiny streams between deep ones, {groups} workgroups", flush=True)
    _layer_batch([5000, 3, 0, 4000, 40], 5120, [groups], 0x5E03, replays=1)


def test_layer_wide_strides():
    print("[case] decode layer, slab strides wider than the rows", flush=True)
    _layer_batch([500, 37], 512, [16], 0x3C01, projection_stride=9216 + 64, query_stride=4096 + 256)


def test_layer_headline_shape_four_lanes_32768():
    """The benchmark's configuration: 4 lanes x 32768 visible keys (32767 cached + the
    new token), 256 and 512 workgroups, eager and as a compiled walk."""
    print("[case] decode layer headline shape: 4 x 32768", flush=True)
    _layer_batch([32767] * 4, 32768, [256, 512], 0xBE7D, replays=3)


def test_layer_config3_ragged_lanes_at_depth():
    print("[case] decode layer config 3: lanes 32768/30000/24576/8192", flush=True)
    _layer_batch([32767, 29999, 24575, 8191], 32768, [256], 0xC0F5, replays=1)


def test_layer_config3_single_lane_100k():
    print("[case] decode layer config 3: 1 lane, 100000 visible keys", flush=True)
    _layer_batch([99999], 100096, [256, 512], 0xC0F6, replays=1)


def test_layer_sixteen_lanes():
    print("[case] decode layer, 16 lanes (32 streams)", flush=True)
    _layer_batch([100 + 61 * i for i in range(16)], 1280, [256], 0x4D02, replays=1)


def test_layer_lane_on_the_last_stripe_a_32_bit_offset_can_name():
    """A pool of 127 stripes of a 65536-key cache puts the last stripe 4.23e9 elements in:
    state-table offsets are 32-bit element counts, every address beyond them 64-bit."""
    print("[case] layer batch on stripes 126 and 0 of 127 x 65536 keys", flush=True)
    _layer_batch([65534, 3000], 65536, [64], 0x32D1, stripes=[126, 0], pool_stripes=127)


def test_layer_drawn_shapes():
    """A dozen waves drawn from a fixed seed through both forms of the whole-layer dispatch:
    1 to 16 lanes, contexts anywhere short of the last position, 1 to 400 workgroups - fewer
    than streams, more than units, and everything between."""
    import random
    rng = random.Random(0x1A7E)
    for case in range(12):
        rows = rng.choice([1, 2, 3, 4, 7, 16])
        cap = rng.choice([512, 1024, 2048])
        contexts = [rng.choice([0, cap - 2, rng.randrange(cap - 1), rng.randrange(cap - 1)])
                    for _ in range(rows)]
        groups = [rng.choice([1, 2, 3, 5, 8, 17, 32, 33, 64, 100, 256, 400]) for _ in range(2)]
        print(f"[case] drawn layer wave {case}: contexts {contexts} cap {cap} groups {groups}", flush=True)
        _layer_batch(contexts, cap, groups, 0x1A7E00 + case, replays=case % 2)


def test_layer_validation():
    B, dev, queue, lib = gpu()
    rows, cap, groups = 2, 512, 8
    ok = dev.create_buffer(rows * 9216 * 2)
    w = dev.create_buffer(512)
    pool = dev.create_buffer(2 * cap * 512 * rows)
    tab = dev.create_buffer(256)
    out = dev.create_buffer(rows * 8192)
    need = 256 + 131072 + (groups + 2 * rows - 1) * 8 * 258 * 4
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    bind = {0: ok, 1: w, 2: w, 3: pool, 4: pool, 5: tab, 7: out}
    const = {8: cap, 9: 9216, 10: 4096, 11: 1}
    with pytest.raises(B.BackendError) as e:      # scratch one byte short
        cb.encode(lib.pipeline("attention_decode_layer_ms"), {**bind, 6: dev.create_buffer(need - 1)},
                  const, (groups, rows), (256,))
    assert e.value.status == 10
    with pytest.raises(B.BackendError) as e:      # more rows than a state table carries
        cb.encode(lib.pipeline("attention_decode_layer_ms"), {**bind, 6: dev.create_buffer(need)},
                  const, (groups, 17), (256,))
    assert e.value.status == 15
    with pytest.raises(B.BackendError) as e:      # the finish dispatch needs the same scratch
        cb.encode(lib.pipeline("attention_decode_layer_finish_ms"),
                  {**bind, 6: dev.create_buffer(need - 1)}, {**const, 11: groups}, (16, rows), (64,))
    assert e.value.status == 10
    assert cb.command_count == 0
