"""ctypes access to the CPU checker (oracle/liboracle.so) and, where it was
built, to the unmodified reference scalar model (oracle/_ref/libtatara_ref.so).

Test infrastructure only: nothing under tatara_amd/ imports this module."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
u32, u64, f32, f64 = C.c_uint32, C.c_uint64, C.c_float, C.c_double


def _nullable(ptr_type):
    class _N:
        @classmethod
        def from_param(cls, obj):
            if obj is None:
                return C.c_void_p(0)
            return ptr_type.from_param(obj)
    return _N


_u16n, _f32n, _u32n = _nullable(_u16p), _nullable(_f32p), _nullable(_u32p)


def _load_oracle():
    path = os.path.join(ORACLE_DIR, "liboracle.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "all"])
    lib = C.CDLL(path)
    sig = {
        "tto_bf16_from_f32": (C.c_uint16, [f32]),
        "tto_f32_from_bf16": (f32, [C.c_uint16]),
        "tto_flush_bf16": (C.c_uint16, [C.c_uint16]),
        "tto_flush_f32": (f32, [f32]),
        "tto_bf16_mul": (C.c_uint16, [C.c_uint16, C.c_uint16]),
        "tto_tree_adjacent32": (f32, [_f32p]),
        "tto_tree_halving256": (f32, [_f32p]),
        "tto_fill_banded_bf16": (None, [u64, _u16p, u64]),
        "tto_fill_banded_f32": (None, [u64, _f32p, u64]),
        "tto_fill_gaussian_bf16": (None, [u64, f64, f64, _u16p, u64]),
        "tto_fill_gaussian_f32": (None, [u64, f64, f64, _f32p, u64]),
        "tto_fill_uniform_f32": (None, [u64, f64, f64, _f32p, u64]),
        "tto_attn_qk_rope": (None, [_u16p, _u16p, _u16p, u32, u32, _u16p, _u16p, _u16p, _u16p]),
        "tto_attention_decode": (None, [_u16p, _u16p, _u16p, _u16p, u32, u32, _u16p, u32]),
        "tto_attention_scores_record": (None, [_u16p, _u16p, u32, u32, u32, u32, u32, _f32p]),
        "tto_attention_values_record": (None, [_f32p, _u16p, u32, u32, u32, u32, u32, _f32p]),
        "tto_attention_combine": (None, [_f32p, _u16p, u32, C.c_int, _u16p]),
        "tto_attention_decode_split": (None, [_u16p, _u16p, _u16p, _u16p, u32, u32, u32, _f32n,
                                              _u16p, u32]),
        "tto_attention_prefill": (None, [_u16p, _u16p, _u16p, u32, u32, u32, _u16p, _u16p, _u16p,
                                         _u16p, _u32n, u32, _u16p, u32]),
        "tto_attention_prefill_rows": (None, [_u16p, _u16p, _u16p, _u16p, u32, u32, _u32p, u32,
                                              _u16p, u32]),
        "tto_gdn_prepare": (None, [_u16p] * 7),
        "tto_gdn_gates": (None, [_u16p, _u16p, _u16p, _f32p, _f32p]),
        "tto_gdn_recurrence": (None, [_u16p, _u16p, _f32p, _f32p, _f32p, u32, u32, _u16p, _f32p,
                                      u32]),
        "tto_gdn_gate_norm": (None, [_u16p, _u16p, _u16p, u32, _u16p]),
        "tto_gdn_decode_step": (None, [_u16p] * 6 + [_f32p, _u16p, _f32p, _u16p, u32]),
        "tto_gdn_prefill": (None, [_u16p, u32, _u16p, _u16p, _u16p, _u16p, _u16p, _f32p, _u16p,
                                   _f32p, _u16p, _u16n, _u16n, _u16n, u32]),
        "tto_gdn_scan": (None, [_u16p, _u16p, _f32p, _f32p, u32, _f32p, _u16p, _f32p, u32]),
        "tto_gdn_conv_tape": (None, [_u16p, u32, _u16p, _u16p, u32]),
        "tto_gdn_scan_tape": (None, [_u16p, _u16p, _f32p, _f32p, u32, _f32p, _u16p, _f32p, _f32p,
                                     u32, u32]),
        "tto_gdn_tape_replay": (None, [_f32p, _f32p, _f32p, u32, u32, u32]),
        "tto_q4_dot": (f32, [_u16p, _u32p, _u16p, _u16p, u32]),
        "tto_q4_project": (None, [_u16p, u64, u32, _u32p, _u16p, _u16p, u32, u32, _u16p, u64, u32]),
        "tto_rms_only": (None, [_u16p, _u16p, u32, u32, _u16p]),
        "tto_dense_bf16": (None, [_u16p, _u16p, u32, u32, u32, _u16p, u32]),
        "tto_add_bf16": (None, [_u16p, _u16p, C.c_uint64, _u16p]),
        "tto_gdn_sequential_f64": (None, [_f64p] * 5 + [u32, u32, u32, _f64p, _f64p]),
        "tto_gdn_chunked_f64": (None, [_f64p] * 5 + [u32, u32, u32, u32, _f64p, _f64p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def _load_ref():
    path = os.path.join(ORACLE_DIR, "_ref", "libtatara_ref.so")
    if not os.path.exists(path):
        if os.path.exists("/root/reference/tests/native/kernel_reference.cpp"):
            subprocess.call(["make", "-C", ORACLE_DIR, "ref"])
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path)
    sig = {
        "ref_bf16_from_f32": (C.c_uint16, [f32]),
        "ref_f32_from_bf16": (f32, [C.c_uint16]),
        "ref_flush_bf16": (C.c_uint16, [C.c_uint16]),
        "ref_bf16_mul": (C.c_uint16, [C.c_uint16, C.c_uint16]),
        "ref_fill_banded_bf16": (None, [u64, _u16p, u64]),
        "ref_tree_sum": (f32, [_f32p, u32, u32]),
        "ref_rms_only": (None, [_u16p, _u16p, u32, u32, u32, _u16p]),
        "ref_residual_sums": (None, [_u16p, _u16p, u64, _u16p]),
        "ref_q4_dot": (f32, [_u16p, _u32p, _u16p, _u16p, u32]),
        "ref_attn_qk_rope": (None, [_u16p, _u16p, _u16p, u32, u32, _u16p, _u16p, _u16p, _u16p]),
        "ref_attention_decode": (None, [_u16p, _u16p, _u16p, _u16p, u32, u32, _u16p]),
        "ref_attention_decode_split": (None, [_u16p, _u16p, _u16p, _u16p, u32, u32, u32, _f32n,
                                              _u16p]),
        "ref_gdn_prepare": (None, [_u16p] * 7),
        "ref_gdn_gates": (None, [_u16p, _u16p, _u16p, _f32p, _f32p]),
        "ref_gdn_recurrence": (None, [_u16p, _u16p, _f32p, _f32p, _f32p, u32, u32, _u16p, _f32p]),
        "ref_gdn_gate_norm": (None, [_u16p, _u16p, _u16p, u32, _u16p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


oracle = _load_oracle()
ref = _load_ref()


def bf16_to_f32(a):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    return (a.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(a):
    """Round-to-nearest-even narrowing, NaN/inf truncated (numpy restatement of
    the oracle's conversion, used only to prepare inputs)."""
    b = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    special = (b & 0x7F800000) == 0x7F800000
    r = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(special, (b >> 16).astype(np.uint16), r)


def banded_bf16(seed, n):
    out = np.empty(n, np.uint16)
    oracle.tto_fill_banded_bf16(seed, out, n)
    return out


def gaussian_bf16(seed, n, mean=0.0, sigma=1.0):
    out = np.empty(n, np.uint16)
    oracle.tto_fill_gaussian_bf16(seed, mean, sigma, out, n)
    return out


def gaussian_f32(seed, n, mean=0.0, sigma=1.0):
    out = np.empty(n, np.float32)
    oracle.tto_fill_gaussian_f32(seed, mean, sigma, out, n)
    return out


def uniform_f32(seed, n, low, high):
    out = np.empty(n, np.float32)
    oracle.tto_fill_uniform_f32(seed, low, high, out, n)
    return out
