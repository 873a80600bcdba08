"""Resource and blit behaviour of the backend on the GPU: zero-filled
allocations, windows, staging views, device-to-device copies and fills."""
import numpy as np
import pytest

from gpu_util import gpu

pytestmark = pytest.mark.gpu


def test_allocations_are_zero_filled_and_windows_alias():
    B, dev, queue, lib = gpu()
    buf = dev.create_buffer(4096 + 100)
    assert not buf.read(np.uint8).any()
    data = np.arange(4196, dtype=np.uint32).astype(np.uint8)
    buf.write(data)
    window = buf.window(256, 1024)
    assert np.array_equal(window.read(np.uint8), data[256:1280])
    window.write(np.full(1024, 7, np.uint8))
    assert np.array_equal(buf.read(np.uint8)[256:1280], np.full(1024, 7, np.uint8))
    assert np.array_equal(buf.read(np.uint8)[:256], data[:256])


@pytest.mark.parametrize("src_off,dst_off,length", [
    (0, 0, 1 << 20), (16, 48, 4096 + 5), (3, 16, 1000), (16, 7, 33), (0, 0, 1), (32, 64, 15)])
def test_blit_copy_and_fill(src_off, dst_off, length):
    """Copies with 16-byte aligned and unaligned ends and ragged tails; bytes
    outside the destination range stay untouched."""
    B, dev, queue, lib = gpu()
    rng = np.random.default_rng(length)
    total = (1 << 20) + 256
    a = rng.integers(0, 256, total, dtype=np.uint8)
    b = rng.integers(0, 256, total, dtype=np.uint8)
    src, dst = dev.buffer_from(a), dev.buffer_from(b)
    cb = queue.create_command_buffer()
    cb.copy_buffer(src, src_off, dst, dst_off, length)
    cb.commit().wait()
    want = b.copy()
    want[dst_off:dst_off + length] = a[src_off:src_off + length]
    assert np.array_equal(dst.read(np.uint8), want)
    cb = queue.create_command_buffer()
    cb.fill_buffer(dst, dst_off, length, 0xA5)
    cb.commit().wait()
    want[dst_off:dst_off + length] = 0xA5
    assert np.array_equal(dst.read(np.uint8), want)


def test_staging_view_round_trip():
    B, dev, queue, lib = gpu()
    buf = dev.create_buffer(1 << 16)
    view = buf.contents(np.uint16)
    view[:] = np.arange(1 << 15, dtype=np.uint16)
    buf.did_modify()
    assert np.array_equal(buf.read(np.uint16), np.arange(1 << 15, dtype=np.uint16))
    buf.write(np.full(1 << 15, 9, np.uint16))
    buf.synchronize()
    assert (buf.contents(np.uint16) == 9).all()


def test_recording_keeps_its_buffers_alive():
    """A recording names buffers by device address; it holds a reference on each, so a
    caller that destroys its handles between encode and commit (or before a later replay
    of a compiled recording) does not leave the GPU working on freed memory."""
    B, dev, queue, lib = gpu()
    L = B.lib()
    n = 1 << 16
    data = np.arange(n, dtype=np.uint32)
    src, mid = dev.buffer_from(data), dev.create_buffer(n * 4)
    dst = dev.create_buffer(n * 4)
    cb = queue.create_command_buffer()
    cb.copy_buffer(src, 0, mid, 0, n * 4)
    cb.copy_buffer(mid, 0, dst, 0, n * 4)
    cb._refs.clear()                       # drop the Python wrapper's own references ...
    for doomed in (src, mid):              # ... and the caller's handles
        L.tt_buffer_destroy(doomed.handle)
        doomed.handle = None
    # other allocations may now land where freed memory would have been
    noise = [dev.buffer_from(np.full(n, 0xDEAD, np.uint32)) for _ in range(4)]
    cb.compile()
    for _ in range(2):
        dst.write(np.zeros(n, np.uint32))
        cb.commit().wait()
        assert np.array_equal(dst.read(np.uint32), data)
    del noise


def test_events_order_command_buffers_of_two_queues():
    """encode_signal_event / encode_wait_for_event: a chain of copies alternating between two
    queues, each step waiting for the value the step before it signals; without the waits the
    two streams would run the copies in any order."""
    B, dev, queue, lib = gpu()
    other = dev.create_queue()
    event = dev.create_event()
    n = 1 << 22
    data = np.arange(n, dtype=np.uint32)
    stages = [dev.buffer_from(data)] + [dev.create_buffer(n * 4) for _ in range(6)]
    buffers = []
    for step in range(6):
        cb = (queue if step % 2 == 0 else other).create_command_buffer()
        if step > 0:
            cb.wait_for_event(event, step)
        cb.copy_buffer(stages[step], 0, stages[step + 1], 0, n * 4)
        cb.signal_event(event, step + 1)
        assert cb.command_count == (3 if step > 0 else 2)
        buffers.append(cb.commit())            # committed in dependency order
    for cb in buffers:
        cb.wait()
    assert np.array_equal(stages[6].read(np.uint32), data)
    # a wait is satisfied by a signal of a larger value
    cb = other.create_command_buffer()
    cb.wait_for_event(event, 3)
    cb.fill_buffer(stages[1], 0, 16, 0xAB)
    cb.commit().wait()
    assert (stages[1].read(np.uint8)[:16] == 0xAB).all()


def test_event_keeps_serving_old_values():
    """Many signalled values: the library keeps a bounded number of them, and a wait for one
    it has let go of is served by a newer signal."""
    B, dev, queue, lib = gpu()
    other = dev.create_queue()
    event = dev.create_event()
    buf = dev.create_buffer(4096)
    for value in range(1, 101):
        cb = queue.create_command_buffer()
        cb.fill_buffer(buf, 0, 4096, value)
        cb.signal_event(event, value)
        cb.commit()
    cb = other.create_command_buffer()
    cb.wait_for_event(event, 1)
    copied = dev.create_buffer(4096)
    cb.copy_buffer(buf, 0, copied, 0, 4096)
    cb.commit().wait()
    queue.synchronize()
    seen = copied.read(np.uint8)
    assert (seen == seen[0]).all() and 1 <= int(seen[0]) <= 100


def test_event_encoding_errors():
    B, dev, queue, lib = gpu()
    event = dev.create_event()
    cb = queue.create_command_buffer()
    with pytest.raises(B.BackendError) as e:
        cb.signal_event(event, 0)
    assert e.value.status == 4                 # InvalidEventValue
    with pytest.raises(B.BackendError) as e:
        cb.wait_for_event(None, 1)
    assert e.value.status == 3                 # InvalidEvent
    cb.begin_compute_pass()
    with pytest.raises(B.BackendError) as e:   # between passes only
        cb.signal_event(event, 1)
    assert e.value.status == 2
    cb.end_compute_pass()
    assert cb.command_count == 0
    # a wait whose signal has not been committed cannot be submitted
    cb.wait_for_event(event, 7)
    with pytest.raises(RuntimeError):          # the submission is reported as failed
        cb.commit().wait()
    # event commands keep a recording out of a graph
    cb2 = queue.create_command_buffer()
    cb2.signal_event(event, 7)
    with pytest.raises(B.BackendError) as e:
        cb2.compile()
    assert e.value.status == 19
    cb2.commit().wait()
    cb.commit().wait()                         # now the value has been signalled
