"""The entry point that allocates nothing (tt_attention_decode_lanes_static): the lane-batched
split-K decode attention with its split records in the library's fixed device scratch,
called through the C ABI and compared bit for bit with the recorded dispatches of
attention_decode_split_ms + attention_decode_combine_ms on the same operands (whose records
live in a caller-bound buffer), and with the CPU checker at the path's output tolerance.
Two calls in a row, the second with a smaller input, so records left by the first call in
the shared scratch must not reach the second call's result."""
import numpy as np
import pytest

import oracle_lib as ol
from gpu_util import check_bf16, gpu, run

pytestmark = pytest.mark.gpu
o = ol.oracle
SCRATCH_BYTES = 8 << 20


def _case(contexts, cap, part, seed):
    B, dev, queue, lib = gpu()
    rows = len(contexts)
    stripe = 2 * cap * 256
    k_pool, stride = dev.create_pool(stripe * 2, rows)
    v_pool, _ = dev.create_pool(stripe * 2, rows)
    q = np.zeros((rows, 4096), np.uint16); gate = np.zeros_like(q); want = np.zeros_like(q)
    table = np.zeros(64, np.uint32)
    for r, ctx in enumerate(contexts):
        q[r] = ol.gaussian_bf16(seed + 10 * r + 1, 4096)
        gate[r] = ol.gaussian_bf16(seed + 10 * r + 2, 4096)
        n = ctx + 1
        k = np.zeros((2, cap, 256), np.uint16); v = np.zeros_like(k)
        k[:, :n] = ol.gaussian_bf16(seed + 10 * r + 3, 2 * n * 256).reshape(2, n, 256)
        v[:, :n] = ol.gaussian_bf16(seed + 10 * r + 4, 2 * n * 256).reshape(2, n, 256)
        o.tto_attention_decode_split(q[r], gate[r], k.reshape(-1), v.reshape(-1), ctx, cap, 256,
                                     None, want[r], 8)
        k_pool.write(k, r * stride)
        v_pool.write(v, r * stride)
        table[r * 4] = r * (stride // 2)
        table[r * 4 + 1] = ctx
    b_tab = dev.buffer_from(table)
    b_q, b_g = dev.buffer_from(q), dev.buffer_from(gate)
    splits = (cap + part - 1) // part
    # the existing entry points: recorded dispatches with a caller-bound record buffer
    b_part = dev.create_buffer(rows * 16 * splits * 258 * 4)
    b_ref = dev.create_buffer(rows * 8192)

    def rec(cb):
        cb.encode(lib.pipeline("attention_decode_split_ms"),
                  {0: b_q, 1: k_pool, 2: v_pool, 3: b_tab, 4: b_part},
                  {5: cap, 6: 4096, 7: part, 8: splits, 9: 8}, (splits, 2, rows), (256,))   # rotated ranges, as the entry point walks them
        cb.barrier()
        cb.encode(lib.pipeline("attention_decode_combine_ms"),
                  {0: b_part, 1: b_g, 2: b_tab, 3: b_ref},
                  {4: part, 5: splits, 6: 4096, 7: 0, 8: cap}, (16, rows), (256,))
    run(rec)
    reference = b_ref.read(np.uint16).reshape(rows, 4096)
    b_out = dev.create_buffer(rows * 8192)
    return dict(rows=rows, cap=cap, part=part, contexts=contexts, want=want, reference=reference,
                operands=(b_q, b_g, k_pool, v_pool, b_tab, b_out), out=b_out)


def _call_and_check(queue, case, what):
    case["out"].write(np.zeros(case["rows"] * 4096, np.uint16))
    queue.attention_decode_lanes_static(*case["operands"], case["rows"], case["cap"], 4096,
                                        case["part"])
    queue.synchronize()
    got = case["out"].read(np.uint16).reshape(case["rows"], 4096)
    assert np.array_equal(got, case["reference"]), f"{what}: differs from the recorded dispatches"
    for r, ctx in enumerate(case["contexts"]):
        check_bf16(got[r], case["want"][r], f"{what} lane {r} ctx {ctx}")


def test_static_scratch_entry_point_two_calls_in_a_row():
    print("[case] no-alloc entry: 3 lanes cap 4096 part 128, then 2 lanes cap 1024 part 64",
          flush=True)
    B, dev, queue, lib = gpu()
    large = _case([4095, 2500, 100], 4096, 128, 0x2A01)
    small = _case([700, 0], 1024, 64, 0x2A02)
    _call_and_check(queue, large, "first call")
    _call_and_check(queue, small, "second call (smaller)")
    _call_and_check(queue, large, "third call (large again)")
    # a grid larger than the chip (128 splits x 2 x 3 workgroups, most of them without keys):
    # the entry point then places the workgroups that hold keys first; same records, same bits
    print("[case] no-alloc entry: 3 lanes cap 4096 part 32", flush=True)
    fine = _case([4095, 2500, 100], 4096, 32, 0x2A04)
    _call_and_check(queue, fine, "fourth call (grid larger than the chip)")


def test_static_scratch_entry_point_rejects_what_it_cannot_hold():
    print("[case] no-alloc entry: limits and operand checks", flush=True)
    B, dev, queue, lib = gpu()
    case = _case([300], 512, 64, 0x2A03)
    ops = case["operands"]
    # 16 rows x 16 heads x 1024 splits x 1032 B is far beyond the fixed scratch
    with pytest.raises(B.BackendError) as e:
        queue.attention_decode_lanes_static(*ops, 1, 1 << 20, 4096, 32)
    assert e.value.status in (10, 40)        # cache extent is checked before the scratch limit
    big_cap = 65536
    k_pool, _ = dev.create_pool(2 * big_cap * 512, 1)
    need = 16 * (big_cap // 32) * 258 * 4
    assert need > SCRATCH_BYTES
    with pytest.raises(B.BackendError) as e:
        queue.attention_decode_lanes_static(ops[0], ops[1], k_pool, k_pool, ops[4], ops[5], 1,
                                            big_cap, 4096, 32)
    assert e.value.status == 40              # StaticScratchExceeded
    with pytest.raises(B.BackendError) as e:
        queue.attention_decode_lanes_static(*ops, 1, 512, 4096, 48)
    assert e.value.status == 15              # split_keys not a multiple of 32
    with pytest.raises(B.BackendError) as e:
        queue.attention_decode_lanes_static(*ops, 2, 512, 4096, 64)
    assert e.value.status == 10              # slabs hold one row only
    with pytest.raises(B.BackendError) as e:
        queue.attention_decode_lanes_static(*ops, 17, 512, 4096, 64)
    assert e.value.status == 15
    # nothing above launched anything: the valid call still gives the reference bits
    _call_and_check(queue, case, "after rejected calls")


def test_static_scratch_row_outside_its_cache_is_left_alone():
    """A table row whose context is not a position of the cache (here: equal to the capacity,
    and the all-ones word) has no records of the call; its output row must stay untouched,
    whatever an earlier, larger call left in the shared scratch."""
    print("[case] no-alloc entry: a row outside its cache after a larger call", flush=True)
    B, dev, queue, lib = gpu()
    large = _case([4095, 2500, 100], 4096, 128, 0x2A05)
    _call_and_check(queue, large, "larger call first")
    small = _case([500, 300], 1000, 96, 0x2A06)      # capacity not a multiple of the split
    b_q, b_g, k_pool, v_pool, b_tab, b_out = small["operands"]
    for bad in (1000, 0xFFFFFFFF):
        table = b_tab.read(np.uint32)
        table[1 * 4 + 1] = bad
        b_bad = dev.buffer_from(table)
        sentinel = np.full(2 * 4096, 0x1234, np.uint16)
        b_out.write(sentinel)
        queue.attention_decode_lanes_static(b_q, b_g, k_pool, v_pool, b_bad, b_out, 2, 1000, 4096, 96)
        queue.synchronize()
        got = b_out.read(np.uint16).reshape(2, 4096)
        assert np.array_equal(got[0], small["reference"][0]), f"context {bad}: the good row changed"
        assert np.array_equal(got[1], sentinel[:4096]), f"context {bad}: the refused row was written"
