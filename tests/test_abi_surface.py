"""The C-ABI shared object loads and exports every symbol include/tatara_hip.h
declares (no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

from tatara_amd import backend as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tatara_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tt_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 40
    L = ctypes.CDLL(B.LIBRARY_PATH)
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    # the Python binding covers the same set
    assert sorted(B.EXPORTED_SYMBOLS) == names


def test_version_and_status_names():
    L = B.lib()
    assert L.tt_abi_version() == 1
    # MetalCommandError numbering (commands.h:232-262)
    assert L.tt_status_name(0) == b"None"
    assert L.tt_status_name(10) == b"InvalidBufferOffset"
    assert L.tt_status_name(16) == b"ContextOutOfRange"
    assert L.tt_status_name(17) == b"StateSlotMismatch"
    assert L.tt_status_name(28) == b"InvalidStreamGroup"


def test_null_handles_are_typed_errors_not_crashes():
    """Host-side validation precedes every native call: null handles return the
    reference's typed errors (metal_*_contract_test.cpp pattern)."""
    L = B.lib()
    null = ctypes.c_void_p(0)
    out = ctypes.c_void_p()
    assert L.tt_queue_create(null, ctypes.byref(out)) == 101          # InvalidDevice
    assert L.tt_buffer_create(null, 16, ctypes.byref(out)) == 101
    assert L.tt_library_create(null, ctypes.byref(out)) == 201
    assert L.tt_pipeline_create(null, b"attention_decode", ctypes.byref(out)) == 202
    assert L.tt_command_buffer_create(null, ctypes.byref(out)) == 1   # InvalidCommandQueue
    assert L.tt_pass_begin(null) == 2                                  # InvalidCommandBuffer
    assert L.tt_pass_set_pipeline(null, null) == 5                     # InvalidComputePass
    assert L.tt_pass_dispatch(null, 1, 1, 1, 1, 1, 1) == 5
    assert L.tt_commit(null) == 2
    r = B.ExecutionResult()
    assert L.tt_wait(null, ctypes.byref(r)) == 18                      # InvalidPendingExecution
    assert L.tt_buffer_size(null) == 0 and not L.tt_buffer_contents(null)
