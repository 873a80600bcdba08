"""ctypes binding of the C ABI in include/tatara_hip.h.

Names follow the reference backend (MetalDevice -> Device, create_shared_buffer
-> Device.create_buffer, set_buffer / set_bytes / dispatch_threadgroups ->
CommandBuffer.set_buffer / set_bytes / dispatch, commit / wait_until_completed
-> CommandBuffer.commit / wait).  Errors are the C ABI's status codes raised as
BackendError; nothing here computes anything."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# TATARA_HIP_LIBRARY selects another build of the same C ABI (e.g. a debug build).
LIBRARY_PATH = os.environ.get("TATARA_HIP_LIBRARY") or os.path.join(_HERE, "lib",
                                                                    "libtatara_hip.so")

EXPORTED_SYMBOLS = [
    "tt_abi_version", "tt_status_name", "tt_device_create", "tt_device_destroy",
    "tt_device_name", "tt_device_compute_units", "tt_queue_create", "tt_queue_destroy",
    "tt_queue_native_stream", "tt_buffer_create", "tt_pool_create", "tt_buffer_window",
    "tt_buffer_wrap", "tt_buffer_destroy", "tt_buffer_size", "tt_buffer_contents",
    "tt_buffer_device_pointer", "tt_buffer_did_modify", "tt_buffer_synchronize",
    "tt_buffer_write", "tt_buffer_read", "tt_library_create", "tt_library_destroy",
    "tt_library_function_count", "tt_library_function_name", "tt_pipeline_create",
    "tt_pipeline_destroy", "tt_pipeline_name", "tt_command_buffer_create",
    "tt_command_buffer_destroy", "tt_pass_begin", "tt_pass_end", "tt_pass_set_pipeline",
    "tt_pass_set_buffer", "tt_pass_set_bytes", "tt_pass_dispatch", "tt_pass_barrier",
    "tt_blit_copy", "tt_blit_fill", "tt_command_count", "tt_commit", "tt_wait",
    "tt_command_buffer_reset", "tt_command_buffer_compile", "tt_command_buffer_set_profiling",
    "tt_command_name", "tt_command_gpu_ms", "tt_attention_decode_lanes_static",
    "tt_event_create", "tt_event_destroy", "tt_encode_signal_event", "tt_encode_wait_for_event",
    "tt_split_workgroups", "tt_choose_split_keys",
    "tt_flash_prefill_splits", "tt_flash_prefill_scratch_bytes",
]


class ExecutionResult(C.Structure):
    _fields_ = [("status", C.c_int32), ("completed", C.c_int32), ("failure", C.c_int32),
                ("has_native_error_code", C.c_int32), ("native_error_code", C.c_int64),
                ("gpu_ms", C.c_double), ("diagnostic_length", C.c_uint64),
                ("diagnostic", C.c_char * 512)]


class BackendError(RuntimeError):
    def __init__(self, status, where):
        self.status = int(status)
        name = lib().tt_status_name(self.status).decode()
        super().__init__(f"{where}: {name} ({self.status})")


_lib = None


def lib():
    """Loads libtatara_hip.so; raises (never falls back) when it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBRARY_PATH):
        raise ImportError(
            f"{LIBRARY_PATH} is not built; run `make -C tatara_amd/csrc` "
            "(there is no CPU fallback for this backend)")
    L = C.CDLL(LIBRARY_PATH)
    vp, u64, u32, i32 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_int32
    pvp = C.POINTER(C.c_void_p)
    sig = {
        "tt_abi_version": (u32, []),
        "tt_status_name": (C.c_char_p, [i32]),
        "tt_device_create": (i32, [pvp]), "tt_device_destroy": (None, [vp]),
        "tt_device_name": (C.c_char_p, [vp]), "tt_device_compute_units": (u32, [vp]),
        "tt_queue_create": (i32, [vp, pvp]), "tt_queue_destroy": (None, [vp]),
        "tt_queue_native_stream": (vp, [vp]),
        "tt_buffer_create": (i32, [vp, u64, pvp]),
        "tt_pool_create": (i32, [vp, u64, u32, pvp, C.POINTER(u64)]),
        "tt_buffer_window": (i32, [vp, u64, u64, pvp]),
        "tt_buffer_wrap": (i32, [vp, vp, u64, pvp]),
        "tt_buffer_destroy": (None, [vp]), "tt_buffer_size": (u64, [vp]),
        "tt_buffer_contents": (vp, [vp]), "tt_buffer_device_pointer": (vp, [vp]),
        "tt_buffer_did_modify": (i32, [vp, u64, u64]),
        "tt_buffer_synchronize": (i32, [vp, u64, u64]),
        "tt_buffer_write": (i32, [vp, u64, vp, u64]),
        "tt_buffer_read": (i32, [vp, u64, vp, u64]),
        "tt_library_create": (i32, [vp, pvp]), "tt_library_destroy": (None, [vp]),
        "tt_library_function_count": (u32, [vp]),
        "tt_library_function_name": (C.c_char_p, [vp, u32]),
        "tt_pipeline_create": (i32, [vp, C.c_char_p, pvp]),
        "tt_pipeline_destroy": (None, [vp]), "tt_pipeline_name": (C.c_char_p, [vp]),
        "tt_command_buffer_create": (i32, [vp, pvp]),
        "tt_command_buffer_destroy": (None, [vp]),
        "tt_pass_begin": (i32, [vp]), "tt_pass_end": (i32, [vp]),
        "tt_pass_set_pipeline": (i32, [vp, vp]),
        "tt_pass_set_buffer": (i32, [vp, vp, u64, u32]),
        "tt_pass_set_bytes": (i32, [vp, vp, u32, u32]),
        "tt_pass_dispatch": (i32, [vp, u64, u64, u64, u64, u64, u64]),
        "tt_pass_barrier": (i32, [vp]),
        "tt_blit_copy": (i32, [vp, vp, u64, vp, u64, u64]),
        "tt_blit_fill": (i32, [vp, vp, u64, u64, C.c_uint8]),
        "tt_command_count": (u32, [vp]),
        "tt_commit": (i32, [vp]), "tt_wait": (i32, [vp, C.POINTER(ExecutionResult)]),
        "tt_command_buffer_reset": (i32, [vp]),
        "tt_command_buffer_compile": (i32, [vp]),
        "tt_command_buffer_set_profiling": (i32, [vp, i32]),
        "tt_command_name": (C.c_char_p, [vp, u32]),
        "tt_command_gpu_ms": (i32, [vp, u32, C.POINTER(C.c_double)]),
        "tt_attention_decode_lanes_static": (i32, [vp] + [vp, u64] * 6 + [u32] * 4),
        "tt_split_workgroups": (u32, [C.POINTER(u32), u32, u32]),
        "tt_choose_split_keys": (u32, [C.POINTER(u32), u32, u32]),
        "tt_flash_prefill_splits": (u32, [u32, u32, u32]),
        "tt_flash_prefill_scratch_bytes": (u64, [u32, u32]),
        "tt_event_create": (i32, [vp, pvp]), "tt_event_destroy": (None, [vp]),
        "tt_encode_signal_event": (i32, [vp, vp, u64]),
        "tt_encode_wait_for_event": (i32, [vp, vp, u64]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def _check(status, where):
    if status != 0:
        raise BackendError(status, where)

def _release(owner, destroy_name):
    """Finalizer body shared by the handle classes.  During interpreter shutdown the
    module's globals are already cleared; a handle that outlives them is left to the
    process exit (the library frees device memory with the HIP context)."""
    handle = getattr(owner, "handle", None)
    if not handle:
        return
    owner.handle = None
    if _lib is None:
        return
    getattr(_lib, destroy_name)(handle)



class Device:
    def __init__(self):
        h = C.c_void_p()
        _check(lib().tt_device_create(C.byref(h)), "create_system_device")
        self.handle = h
        self.name = lib().tt_device_name(h).decode()
        self.compute_units = lib().tt_device_compute_units(h)

    def create_queue(self):
        return CommandQueue(self)

    def create_buffer(self, size_bytes):
        h = C.c_void_p()
        _check(lib().tt_buffer_create(self.handle, int(size_bytes), C.byref(h)),
               "create_shared_buffer")
        return Buffer(h, self)

    def create_pool(self, stripe_bytes, stripe_count):
        h, stride = C.c_void_p(), C.c_uint64()
        _check(lib().tt_pool_create(self.handle, int(stripe_bytes), int(stripe_count), C.byref(h),
                                    C.byref(stride)), "create_striped_pool_buffer")
        return Buffer(h, self), stride.value

    def wrap(self, device_pointer, size_bytes, keepalive=None):
        h = C.c_void_p()
        _check(lib().tt_buffer_wrap(self.handle, C.c_void_p(int(device_pointer)), int(size_bytes),
                                    C.byref(h)), "buffer_wrap")
        buf = Buffer(h, self)
        buf._keepalive = keepalive
        return buf

    def buffer_from(self, array):
        """New HBM buffer holding a copy of a numpy array."""
        a = np.ascontiguousarray(array)
        buf = self.create_buffer(max(a.nbytes, 1))
        if a.nbytes:
            buf.write(a)
        return buf

    def create_library(self):
        return Library(self)

    def create_event(self):
        return Event(self)


class Event:
    """create_event: a counter that command buffers of any queue signal and wait for."""

    def __init__(self, device):
        h = C.c_void_p()
        _check(lib().tt_event_create(device.handle, C.byref(h)), "create_event")
        self.handle, self.device = h, device

    def __del__(self, _release=_release):
        _release(self, "tt_event_destroy")


class CommandQueue:
    def __init__(self, device):
        h = C.c_void_p()
        _check(lib().tt_queue_create(device.handle, C.byref(h)), "create_command_queue")
        self.handle, self.device = h, device

    @property
    def native_stream(self):
        return lib().tt_queue_native_stream(self.handle)

    def create_command_buffer(self):
        return CommandBuffer(self)

    def attention_decode_lanes_static(self, q, gate, keys_pool, values_pool, state_table, out,
                                      rows, capacity, query_stride, split_keys):
        """tt_attention_decode_lanes_static: the lane-batched split-K decode launched directly
        on this queue with its split records in the library's fixed device scratch (no
        allocation).  Operands are Buffers or (Buffer, byte offset) pairs; only enqueues."""
        args = []
        for operand in (q, gate, keys_pool, values_pool, state_table, out):
            buffer, offset = operand if isinstance(operand, tuple) else (operand, 0)
            args += [C.c_void_p(buffer.device_pointer + offset),
                     C.c_uint64(buffer.size_bytes - offset)]
        _check(lib().tt_attention_decode_lanes_static(self.handle, *args, rows, capacity,
                                                      query_stride, split_keys),
               "attention_decode_lanes_static")

    def synchronize(self):
        """Blocks until everything enqueued on the queue's stream has completed (an empty
        recording committed and waited on the same in-order stream)."""
        cb = self.create_command_buffer()
        cb.commit().wait()

    def __del__(self, _release=_release):
        _release(self, "tt_queue_destroy")


class Buffer:
    def __init__(self, handle, device):
        self.handle, self.device = handle, device
        self._keepalive = None

    @property
    def size_bytes(self):
        return lib().tt_buffer_size(self.handle)

    @property
    def device_pointer(self):
        return lib().tt_buffer_device_pointer(self.handle)

    def window(self, offset, length):
        h = C.c_void_p()
        _check(lib().tt_buffer_window(self.handle, int(offset), int(length), C.byref(h)),
               "create_buffer_window")
        w = Buffer(h, self.device)
        w._keepalive = self
        return w

    def contents(self, dtype=np.uint8):
        """numpy view of the pinned host staging copy (publish with did_modify,
        refresh with synchronize)."""
        p = lib().tt_buffer_contents(self.handle)
        if not p:
            raise BackendError(8, "contents")
        n = self.size_bytes
        raw = (C.c_uint8 * n).from_address(p)
        return np.frombuffer(raw, dtype=np.uint8).view(dtype)

    def did_modify(self, offset=0, length=None):
        length = self.size_bytes - offset if length is None else length
        _check(lib().tt_buffer_did_modify(self.handle, offset, length), "did_modify_range")

    def synchronize(self, offset=0, length=None):
        length = self.size_bytes - offset if length is None else length
        _check(lib().tt_buffer_synchronize(self.handle, offset, length), "synchronize")

    def write(self, array, offset=0):
        a = np.ascontiguousarray(array)
        _check(lib().tt_buffer_write(self.handle, int(offset), a.ctypes.data_as(C.c_void_p),
                                     a.nbytes), "buffer_write")

    def read(self, dtype, count=None, offset=0):
        dt = np.dtype(dtype)
        if count is None:
            count = (self.size_bytes - offset) // dt.itemsize
        out = np.empty(count, dt)
        _check(lib().tt_buffer_read(self.handle, int(offset), out.ctypes.data_as(C.c_void_p),
                                    out.nbytes), "buffer_read")
        return out

    def __del__(self, _release=_release):
        _release(self, "tt_buffer_destroy")


class Library:
    def __init__(self, device):
        h = C.c_void_p()
        _check(lib().tt_library_create(device.handle, C.byref(h)), "create_library")
        self.handle, self.device = h, device
        self._cache = {}

    def function_names(self):
        n = lib().tt_library_function_count(self.handle)
        return [lib().tt_library_function_name(self.handle, i).decode() for i in range(n)]

    def pipeline(self, name):
        if name not in self._cache:
            h = C.c_void_p()
            _check(lib().tt_pipeline_create(self.handle, name.encode(), C.byref(h)),
                   f"create_compute_pipeline({name})")
            self._cache[name] = Pipeline(h, name)
        return self._cache[name]

    def __del__(self, _release=_release):
        self._cache.clear()
        _release(self, "tt_library_destroy")


class Pipeline:
    def __init__(self, handle, name):
        self.handle, self.name = handle, name

    def __del__(self, _release=_release):
        _release(self, "tt_pipeline_destroy")


class CommandBuffer:
    """A recording of compute-pass and blit commands; commit() submits it to the
    queue's HIP stream, wait() blocks and reports device time."""

    def __init__(self, queue):
        h = C.c_void_p()
        _check(lib().tt_command_buffer_create(queue.handle, C.byref(h)), "create_command_buffer")
        self.handle, self.queue = h, queue
        self._refs = []

    def begin_compute_pass(self):
        _check(lib().tt_pass_begin(self.handle), "begin_compute_pass")
        return self

    def end_compute_pass(self):
        _check(lib().tt_pass_end(self.handle), "end_compute_pass")
        return self

    def set_pipeline(self, pipeline):
        _check(lib().tt_pass_set_pipeline(self.handle, pipeline.handle), "set_compute_pipeline")
        self._refs.append(pipeline)

    def set_buffer(self, buffer, offset, index):
        _check(lib().tt_pass_set_buffer(self.handle, buffer.handle, int(offset), int(index)),
               f"set_buffer[{index}]")
        self._refs.append(buffer)

    def set_bytes(self, value, index):
        if isinstance(value, (int, np.integer)):
            value = np.uint32(value).tobytes()
        value = bytes(value)
        _check(lib().tt_pass_set_bytes(self.handle, value, len(value), int(index)),
               f"set_bytes[{index}]")

    def dispatch(self, groups, threads):
        g = tuple(groups) + (1,) * (3 - len(groups))
        t = tuple(threads) + (1,) * (3 - len(threads))
        _check(lib().tt_pass_dispatch(self.handle, *[int(x) for x in g], *[int(x) for x in t]),
               "dispatch_threadgroups")

    def barrier(self):
        _check(lib().tt_pass_barrier(self.handle), "memory_barrier")

    def encode(self, pipeline, buffers, constants, groups, threads):
        """set_pipeline + bindings + dispatch; buffers {index: Buffer | (Buffer, offset)},
        constants {index: uint32}."""
        self.set_pipeline(pipeline)
        for index, b in buffers.items():
            if isinstance(b, tuple):
                self.set_buffer(b[0], b[1], index)
            else:
                self.set_buffer(b, 0, index)
        for index, c in constants.items():
            self.set_bytes(c, index)
        self.dispatch(groups, threads)

    def copy_buffer(self, source, source_offset, destination, destination_offset, length):
        _check(lib().tt_blit_copy(self.handle, source.handle, source_offset, destination.handle,
                                  destination_offset, length), "copy_buffer")
        self._refs += [source, destination]

    def signal_event(self, event, value):
        """encode_signal_event: `value` is reached once everything recorded so far completes."""
        handle = event.handle if event is not None else None
        _check(lib().tt_encode_signal_event(self.handle, handle, value), "encode_signal_event")
        self._refs.append(event)

    def wait_for_event(self, event, value):
        """encode_wait_for_event: what is recorded after this waits for the event to reach
        `value`; the signal must be committed before this command buffer is."""
        handle = event.handle if event is not None else None
        _check(lib().tt_encode_wait_for_event(self.handle, handle, value), "encode_wait_for_event")
        self._refs.append(event)

    def fill_buffer(self, destination, offset, length, value):
        _check(lib().tt_blit_fill(self.handle, destination.handle, offset, length, value),
               "fill_buffer")
        self._refs.append(destination)

    @property
    def command_count(self):
        return lib().tt_command_count(self.handle)

    def commit(self):
        _check(lib().tt_commit(self.handle), "commit")
        return self

    def wait(self):
        r = ExecutionResult()
        _check(lib().tt_wait(self.handle, C.byref(r)), "wait_until_completed")
        if not r.completed:
            raise RuntimeError("command buffer failed: class %d native %d: %s" % (
                r.failure, r.native_error_code, r.diagnostic.decode(errors="replace")))
        return r.gpu_ms

    def reset(self):
        _check(lib().tt_command_buffer_reset(self.handle), "reset")
        self._refs.clear()

    def compile(self):
        """Turns the recording into a HIP graph; later commits replay it."""
        _check(lib().tt_command_buffer_compile(self.handle), "compile")
        return self

    def set_profiling(self, enabled=True):
        _check(lib().tt_command_buffer_set_profiling(self.handle, 1 if enabled else 0),
               "set_profiling")

    def command_times(self):
        """[(kernel name, device ms)] of the last eager commit made with profiling on."""
        out = []
        for i in range(self.command_count):
            ms = C.c_double()
            _check(lib().tt_command_gpu_ms(self.handle, i, C.byref(ms)), "command_gpu_ms")
            out.append((lib().tt_command_name(self.handle, i).decode(), ms.value))
        return out

    def __del__(self, _release=_release):
        _release(self, "tt_command_buffer_destroy")


def _u32_array(values):
    values = [int(v) for v in values]
    return (C.c_uint32 * max(len(values), 1))(*values), len(values)


def split_workgroups(visible_keys, split_keys):
    """Workgroups of one attention layer's split-K grid that hold keys (tt_split_workgroups)."""
    array, count = _u32_array(visible_keys)
    return int(lib().tt_split_workgroups(array, count, int(split_keys)))


def choose_split_keys(visible_keys, compute_units=256):
    """Keys per split-K workgroup for a token wave (tt_choose_split_keys)."""
    array, count = _u32_array(visible_keys)
    return int(lib().tt_choose_split_keys(array, count, int(compute_units)))


def flash_prefill_splits(rows, visible_keys, compute_units=256):
    """Workgroups that share a position tile's key walk in attention_flash_split_blk so that a
    block of `rows` rows, whose last row sees `visible_keys` keys, fills the device
    (tt_flash_prefill_splits)."""
    return int(lib().tt_flash_prefill_splits(int(rows), int(visible_keys), int(compute_units)))


def flash_prefill_scratch_bytes(rows, splits):
    """Bytes the scratch binding of attention_flash_split_blk must hold (0 for one split)."""
    return int(lib().tt_flash_prefill_scratch_bytes(int(rows), int(splits)))
