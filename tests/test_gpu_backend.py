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
