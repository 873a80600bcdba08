#!/usr/bin/env python3
"""Benchmark of the attention-family hot path on one MI355X.

A step is one decode token wave of 4 lanes at 32768 visible keys through one
hybrid period of the layer stack, G,G,G,A (three Gated DeltaNet layers, one
full-attention layer), with the lane-batched operators:
    GDN:       gdn_decode_fused_ms (prepare + recurrence + gate-norm in one dispatch)
    attention: attn_qk_rope_ms -> attention_decode_split_ms -> attention_decode_combine_ms
Projections (the reference's Q4 GEMVs) are not on the path: their outputs are
resident random bf16 slabs.  KV caches, GDN state and all scratch are in HBM
before the timed region; two copies of the attention layer's KV pools (537 MB in
total) alternate from step to step so the 256 MB last-level cache cannot serve
the stream.  The step is compiled into a HIP graph and replayed.

`detail.prefill_16k` adds the block-prefill side of the metric: 16384 new tokens of
one lane through a full-attention layer (causal flash attention on MFMA) and a
Gated DeltaNet layer (chunk-64 recurrence on MFMA), tok/s and fraction of MFMA peak.

`detail.q4_projections` adds the affine 4-bit projections either side of the family
(attention / GDN in-projection, output projection) for the same 4-lane wave and the same
16384-row block, device microseconds per dispatch (tatara_amd.q4_sweep).

Prints ONE JSON line: `value` = microseconds per layer over the period,
`roofline` for the dominant kernel (the split-K flash-decode), `cpu_baseline` =
the CPU checker timed on this box's host cores on the same period."""
import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LANES = 4
VISIBLE = 32768
CAPACITY = 32768
DEFAULT_SPLIT_KEYS = 1024       # keys per split-K workgroup
HBM_PEAK_GBS = 8000.0
CALIBRATION_COPY_BYTES = 256 << 20
# HBM traffic of one launch of the split-K kernel at this workload, from two
# rocprofv3 counter runs (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each
# scaled by what the same counter read for a plain 256 MiB copy of known size.
FLASH_FETCH_KIB, FETCH_SCALE = 131297.0, 262144.0 / 131083.3
FLASH_WRITE_KIB, WRITE_SCALE = 2112.0, 262144.0 / 262144.0
ATTN_BYTES_PER_KEY = 2048       # K and V rows of both kv heads, bf16
GDN_BYTES_PER_LANE_LAYER = 4194304 + 2 * 49152 + 65536 + 24704 + 4 * 8192


def build_workload(B, dev, lib, torch, PART):
    """Allocates and fills every buffer of the period; returns the two step
    recorders (even/odd KV copy) and bookkeeping."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x7A7A)
    keep = []

    def rand_bf16(n, sigma=1.0):
        t = (torch.randn(n, generator=gen, device="cuda", dtype=torch.float32) * sigma).to(
            torch.bfloat16)
        keep.append(t)
        return dev.wrap(t.data_ptr(), t.numel() * 2, keepalive=t)

    def rand_f32(n, sigma):
        t = torch.randn(n, generator=gen, device="cuda", dtype=torch.float32) * sigma
        keep.append(t)
        return dev.wrap(t.data_ptr(), t.numel() * 4, keepalive=t)

    def from_np(a):
        return dev.buffer_from(a)

    rows = LANES
    context = VISIBLE - 1
    stripe_elems = 2 * CAPACITY * 256
    max_splits = (CAPACITY + PART - 1) // PART
    # attention layer: two alternating KV copies, 4 stripes each
    kv = [(rand_bf16(rows * stripe_elems), rand_bf16(rows * stripe_elems)) for _ in range(2)]
    attn_table = np.zeros(64, np.uint32)
    for r in range(rows):
        attn_table[r * 4] = r * stripe_elems
        attn_table[r * 4 + 1] = context
    b_attn_table = from_np(attn_table)
    attn_proj = rand_bf16(rows * 9216)
    q_w = from_np(np.full(256, 0x3F80, np.uint16))
    k_w = from_np(np.full(256, 0x3F80, np.uint16))
    b_q, b_gate, b_att = (dev.create_buffer(rows * 8192) for _ in range(3))
    b_part = dev.create_buffer(rows * 16 * max_splits * 258 * 4)

    # three GDN layers, each with its own pooled state and weights
    conv_elems, rec_elems = 3 * 8192, 32 * 128 * 128
    gdn_layers = []
    for _ in range(3):
        conv_pool = rand_bf16(2 * rows * conv_elems, 0.5)
        rec_pool = rand_f32(2 * rows * rec_elems, 0.02)
        table = np.zeros(64, np.uint32)
        for r in range(rows):
            table[r * 4 + 0] = (2 * r) * conv_elems
            table[r * 4 + 1] = (2 * r + 1) * conv_elems
            table[r * 4 + 2] = (2 * r) * rec_elems
            table[r * 4 + 3] = (2 * r + 1) * rec_elems
        rng = np.random.default_rng(len(gdn_layers) + 1)
        a_log = (rng.uniform(-4.0, -2.5, 32).astype(np.float32).view(np.uint32) >> 16).astype(
            np.uint16)
        dt_bias = (rng.normal(0, 0.3, 32).astype(np.float32).view(np.uint32) >> 16).astype(
            np.uint16)
        gdn_layers.append(dict(conv=conv_pool, rec=rec_pool, table=from_np(table),
                               proj=rand_bf16(rows * 12352, 0.5), conv_w=rand_bf16(4 * 8192, 0.5),
                               a_log=from_np(a_log), dt_bias=from_np(dt_bias),
                               norm_w=from_np(np.full(128, 0x3F80, np.uint16))))
    g_out = dev.create_buffer(rows * 8192)

    P = lib.pipeline

    def record(cb, copy):
        for layer in gdn_layers:
            cb.encode(P("gdn_decode_fused_ms"),
                      {0: layer["proj"], 1: layer["conv"], 2: layer["conv_w"], 3: layer["a_log"],
                       4: layer["dt_bias"], 5: layer["rec"], 6: layer["norm_w"], 7: g_out,
                       8: layer["table"]}, {9: 12352, 10: 4096}, (32, rows), (512,))
            cb.barrier()
        keys, values = kv[copy]
        cb.encode(P("attn_qk_rope_ms"),
                  {0: attn_proj, 1: q_w, 2: k_w, 3: b_q, 4: b_gate, 5: keys, 6: values,
                   8: b_attn_table}, {7: CAPACITY, 9: 9216, 10: 4096}, (18, rows), (256,))
        cb.barrier()
        cb.encode(P("attention_decode_split_ms"),
                  {0: b_q, 1: keys, 2: values, 3: b_attn_table, 4: b_part},
                  {5: CAPACITY, 6: 4096, 7: PART, 8: max_splits, 9: 0}, (max_splits, 2, rows),
                  (256,))
        cb.barrier()
        cb.encode(P("attention_decode_combine_ms"),
                  {0: b_part, 1: b_gate, 2: b_attn_table, 3: b_att},
                  {4: PART, 5: max_splits, 6: 4096, 7: 0}, (16, rows), (256,))

    def record_split_only(cb, copy):
        keys, values = kv[copy]
        cb.encode(P("attention_decode_split_ms"),
                  {0: b_q, 1: keys, 2: values, 3: b_attn_table, 4: b_part},
                  {5: CAPACITY, 6: 4096, 7: PART, 8: max_splits, 9: 0}, (max_splits, 2, rows),
                  (256,))

    return record, record_split_only, keep


def build_period(dev, lib, torch, variant, cus, part=DEFAULT_SPLIT_KEYS):
    """Recorder of one decode period for the timing variants: `three` = rope, split and
    combine dispatches; `layer0` / `layer1` = the whole-layer dispatch finished by a second
    dispatch / inside the first; `gdn_only`, `attn_three`, `attn_layer0`, `attn_layer1` =
    parts of the period."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x7A7A)

    def rand_bf16(n, sigma=1.0):
        t = (torch.randn(n, generator=gen, device="cuda", dtype=torch.float32) * sigma).to(
            torch.bfloat16)
        return dev.wrap(t.data_ptr(), t.numel() * 2, keepalive=t)

    def rand_f32(n, sigma):
        t = torch.randn(n, generator=gen, device="cuda", dtype=torch.float32) * sigma
        return dev.wrap(t.data_ptr(), t.numel() * 4, keepalive=t)

    rows, context = LANES, VISIBLE - 1
    stripe_elems = 2 * CAPACITY * 256
    max_splits = (CAPACITY + part - 1) // part
    kv = [(rand_bf16(rows * stripe_elems), rand_bf16(rows * stripe_elems)) for _ in range(2)]
    attn_table = np.zeros(64, np.uint32)
    for r in range(rows):
        attn_table[r * 4] = r * stripe_elems
        attn_table[r * 4 + 1] = context
    b_attn_table = dev.buffer_from(attn_table)
    attn_proj = rand_bf16(rows * 9216)
    q_w = dev.buffer_from(np.full(256, 0x3F80, np.uint16))
    b_q, b_gate, b_att = (dev.create_buffer(rows * 8192) for _ in range(3))
    b_part = dev.create_buffer(rows * 16 * max_splits * 258 * 4)
    groups = cus
    b_scratch = dev.create_buffer(256 + 131072 + (groups + 2 * rows - 1) * 8 * 258 * 4)
    conv_elems, rec_elems = 3 * 8192, 32 * 128 * 128
    gdn_layers = []
    for i in range(3):
        table = np.zeros(64, np.uint32)
        for r in range(rows):
            table[r * 4 + 0] = (2 * r) * conv_elems
            table[r * 4 + 1] = (2 * r + 1) * conv_elems
            table[r * 4 + 2] = (2 * r) * rec_elems
            table[r * 4 + 3] = (2 * r + 1) * rec_elems
        rng = np.random.default_rng(i + 1)
        a_log = (rng.uniform(-4.0, -2.5, 32).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        dt_bias = (rng.normal(0, 0.3, 32).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        gdn_layers.append(dict(conv=rand_bf16(2 * rows * conv_elems, 0.5),
                               rec=rand_f32(2 * rows * rec_elems, 0.02), table=dev.buffer_from(table),
                               proj=rand_bf16(rows * 12352, 0.5), conv_w=rand_bf16(4 * 8192, 0.5),
                               a_log=dev.buffer_from(a_log), dt_bias=dev.buffer_from(dt_bias),
                               norm_w=dev.buffer_from(np.full(128, 0x3F80, np.uint16))))
    g_out = dev.create_buffer(rows * 8192)
    P = lib.pipeline

    def record(cb, copy):
        if not variant.startswith("attn_"):
            for layer in gdn_layers:
                cb.encode(P("gdn_decode_fused_ms"),
                          {0: layer["proj"], 1: layer["conv"], 2: layer["conv_w"], 3: layer["a_log"],
                           4: layer["dt_bias"], 5: layer["rec"], 6: layer["norm_w"], 7: g_out,
                           8: layer["table"]}, {9: 12352, 10: 4096}, (32, rows), (512,))
        if variant == "gdn_only":
            return
        keys, values = kv[copy]
        if variant.endswith("three"):
            cb.encode(P("attn_qk_rope_ms"),
                      {0: attn_proj, 1: q_w, 2: q_w, 3: b_q, 4: b_gate, 5: keys, 6: values,
                       8: b_attn_table}, {7: CAPACITY, 9: 9216, 10: 4096}, (18, rows), (256,))
            cb.encode(P("attention_decode_split_ms"),
                      {0: b_q, 1: keys, 2: values, 3: b_attn_table, 4: b_part},
                      {5: CAPACITY, 6: 4096, 7: part, 8: max_splits, 9: 0}, (max_splits, 2, rows), (256,))
            cb.encode(P("attention_decode_combine_ms"),
                      {0: b_part, 1: b_gate, 2: b_attn_table, 3: b_att},
                      {4: part, 5: max_splits, 6: 4096, 7: 0}, (16, rows), (256,))
            return
        mode = 1 if variant.endswith("1") else 0
        bind = {0: attn_proj, 1: q_w, 2: q_w, 3: keys, 4: values, 5: b_attn_table, 6: b_scratch, 7: b_att}
        const = {8: CAPACITY, 9: 9216, 10: 4096}
        cb.encode(P("attention_decode_layer_ms"), bind, {**const, 11: mode}, (groups, rows), (256,))
        if mode == 0:
            cb.encode(P("attention_decode_layer_finish_ms"), bind, {**const, 11: groups}, (16, rows), (64,))

    return record


def prefill_figures(B, dev, queue, lib, torch, rows=16384, repeats=3):
    """Block prefill of `rows` new tokens into an empty cache, one lane, resident
    random inputs: the causal flash attention kernel (rope stage timed beside it) and
    the chunk-64 Gated DeltaNet recurrence (conv, gates and gate-norm beside it).
    Per-command device time, best of `repeats`."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0xF1A5)
    keep = []

    def rb(n, sigma=1.0):
        t = (torch.randn(n, generator=gen, device="cuda") * sigma).to(torch.bfloat16)
        keep.append(t)
        return dev.wrap(t.data_ptr(), n * 2, keepalive=t)

    P = lib.pipeline
    mk = dev.create_buffer
    # attention layer
    a_proj = rb(rows * 9216)
    ones = dev.buffer_from(np.full(256, 0x3F80, np.uint16))
    q, gate, out = mk(rows * 8192), mk(rows * 8192), mk(rows * 8192)
    keys, values = mk(2 * rows * 256 * 2), mk(2 * rows * 256 * 2)
    # GDN layer
    g_proj = rb(rows * 12352, 0.5)
    conv_w = rb(4 * 8192, 0.5)
    rng = np.random.default_rng(3)
    a_log = dev.buffer_from((rng.uniform(-4.0, -2.5, 32).astype(np.float32).view(np.uint32) >> 16)
                            .astype(np.uint16))
    dt_bias = dev.buffer_from(np.zeros(32, np.uint16))
    norm_w = dev.buffer_from(np.full(128, 0x3F80, np.uint16))
    conv_in, conv_out = mk(3 * 8192 * 2), mk(3 * 8192 * 2)
    rec = mk(32 * 128 * 128 * 4)
    qk, v, z, y, gated = (mk(rows * 8192) for _ in range(5))
    decay, beta = mk(rows * 128), mk(rows * 128)
    chunk = mk(((min(rows, 2048) + 63) // 64) * 32 * 115712)
    best = {}
    for _ in range(repeats):
        cb = queue.create_command_buffer()
        cb.set_profiling(True)
        cb.begin_compute_pass()
        cb.encode(P("attn_qk_rope_blk"), {0: a_proj, 1: ones, 2: ones, 3: q, 4: gate, 5: keys, 6: values},
                  {7: 0, 8: rows}, (18, rows), (256,))
        cb.barrier()
        cb.encode(P("attention_flash_v2_blk"), {0: q, 1: keys, 2: values, 3: gate, 4: out},
                  {5: rows, 6: rows, 7: rows, 8: 0}, (16, (rows + 15) // 16), (256,))
        cb.encode(P("gdn_conv_blk"), {0: g_proj, 1: conv_in, 2: conv_w, 3: qk, 4: v, 5: z, 6: conv_out},
                  {7: rows}, (96, rows), (128,))
        cb.encode(P("gdn_gates_blk"), {0: g_proj, 1: a_log, 2: dt_bias, 3: decay, 4: beta}, {5: rows},
                  (1, (rows + 3) // 4, 1), (32, 4, 1))
        cb.barrier()
        cb.encode(P("gdn_chunk_recurrence_blk"),
                  {0: qk, 1: v, 2: decay, 3: beta, 4: chunk, 5: rec, 6: y, 7: rec}, {8: rows},
                  (8, 32), (256,))
        cb.barrier()
        cb.encode(P("gdn_gate_norm_blk"), {0: y, 1: z, 2: norm_w, 3: gated}, {}, (32, rows), (128,))
        cb.end_compute_pass()
        cb.commit().wait()
        for name, ms in cb.command_times():
            best[name] = min(best.get(name, ms), ms)
    flash_ms = best["attention_flash_v2_blk"]
    flops = 16 * 4 * 256 * rows * (rows + 1) / 2
    attn_ms = flash_ms + best["attn_qk_rope_blk"]
    gdn_ms = sum(best[k] for k in ("gdn_conv_blk", "gdn_gates_blk", "gdn_chunk_recurrence_blk",
                                   "gdn_gate_norm_blk"))
    return {"rows": rows,
            "attention_layer_ms": round(attn_ms, 3),
            "attention_layer_tok_per_s": round(rows / (attn_ms * 1e-3)),
            "flash_kernel_ms": round(flash_ms, 3),
            "flash_kernel_tflops": round(flops / (flash_ms * 1e-3) / 1e12, 1),
            "flash_kernel_frac_of_bf16_mfma_peak": round(flops / (flash_ms * 1e-3) / 2.5e15, 4),
            "roofline": {"bound": "mfma", "kernel": "attention_flash_v2_blk "
                                                    "(attention_flash_prefill_kernel)",
                         "achieved": round(flops / (flash_ms * 1e-3) / 1e12, 1), "peak": 2500.0,
                         "unit": "TFLOP/s",
                         "frac": round(flops / (flash_ms * 1e-3) / 2.5e15, 4),
                         "algorithmic_flops": flops},
            "gdn_layer_ms": round(gdn_ms, 3),
            "gdn_layer_tok_per_s": round(rows / (gdn_ms * 1e-3)),
            "kernel_ms": {k: round(v, 3) for k, v in best.items()}}


def cpu_baseline(threads):
    """The CPU checker (reference arithmetic restated, oracle/liboracle.so) on one
    G,G,G,A period at the same shapes: 4 lanes x 32768 keys of attention decode and
    3 x 4 lanes of GDN decode.  Baseline only; never part of the product path."""
    path = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(path):
        return None
    L = C.CDLL(path)
    u16 = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
    f32 = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
    L.tto_attention_decode_split.argtypes = [u16, u16, u16, u16, C.c_uint32, C.c_uint32,
                                             C.c_uint32, C.c_void_p, u16, C.c_uint32]
    L.tto_attention_decode_split.restype = None
    L.tto_gdn_decode_step.argtypes = [u16] * 6 + [f32, u16, f32, u16, C.c_uint32]
    L.tto_gdn_decode_step.restype = None
    rng = np.random.default_rng(7)

    def bf16(n, sigma=1.0):
        x = rng.standard_normal(n, dtype=np.float32) * np.float32(sigma)
        return (x.view(np.uint32) >> 16).astype(np.uint16)   # truncation is fine for random data

    keys = bf16(2 * CAPACITY * 256)
    values = bf16(2 * CAPACITY * 256)
    q, gate = bf16(4096), bf16(4096)
    out = np.zeros(4096, np.uint16)
    proj, cs, cw = bf16(12352, 0.5), bf16(3 * 8192, 0.5), bf16(4 * 8192, 0.5)
    a_log = np.full(32, 0xC040, np.uint16)   # -3.0
    dtb = np.zeros(32, np.uint16)
    nw = np.full(128, 0x3F80, np.uint16)
    st = (rng.standard_normal(32 * 128 * 128, dtype=np.float32) * 0.02)
    ncs = np.zeros(3 * 8192, np.uint16)
    so = np.zeros_like(st)
    gated = np.zeros(4096, np.uint16)
    t0 = time.perf_counter()
    for _ in range(LANES):   # lanes are independent; same-shape data per lane
        L.tto_attention_decode_split(q, gate, keys, values, VISIBLE - 1, CAPACITY, 256, None, out,
                                     threads)
    t_attn = time.perf_counter() - t0
    t0 = time.perf_counter()
    for _ in range(3 * LANES):
        L.tto_gdn_decode_step(proj, cs, cw, a_log, dtb, nw, st, ncs, so, gated, threads)
    t_gdn = time.perf_counter() - t0
    return {"value": round((t_attn + t_gdn) * 1e6 / 4.0, 1), "unit": "us/layer",
            "cores": threads, "kind": "port",
            "sample": "one full G,G,G,A period, 4 lanes x 32768 keys (attention layer "
                      f"{t_attn * 1e6:.0f} us, GDN layer {t_gdn * 1e6 / 3:.0f} us)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-prefill", action="store_true",
                    help="skip the 16384-row block prefill figures in detail.prefill_16k")
    ap.add_argument("--split-keys", type=int, default=DEFAULT_SPLIT_KEYS,
                    help="keys per split-K workgroup (multiple of 32)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 256 MiB device-to-device copies first, so a "
                         "counter run has a kernel of known traffic to scale its readings by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU leg (lanes and heads "
              "would shard without exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from tatara_amd import backend as B
    if not torch.cuda.is_available():
        print("no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    dev = B.Device()
    queue = dev.create_queue()
    lib = dev.create_library()
    PART = args.split_keys
    if args.calibrate_copy:
        src = dev.create_buffer(CALIBRATION_COPY_BYTES)
        dst = dev.create_buffer(CALIBRATION_COPY_BYTES)
        for _ in range(3):
            cb = queue.create_command_buffer()
            cb.copy_buffer(src, 0, dst, 0, CALIBRATION_COPY_BYTES)
            cb.commit().wait()
    record, record_split_only, keep = build_workload(B, dev, lib, torch, PART)

    steps = []
    for copy in range(2):
        cb = queue.create_command_buffer()
        cb.begin_compute_pass()
        record(cb, copy)
        cb.end_compute_pass()
        cb.compile()
        steps.append(cb)

    for k in range(args.warmup):
        steps[k & 1].commit()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        steps[k & 1].commit()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    # per-kernel device time: eager commits with an event after every command
    prof = []
    for copy in range(2):
        cb = queue.create_command_buffer()
        cb.begin_compute_pass()
        record(cb, copy)
        cb.end_compute_pass()
        cb.set_profiling(True)
        prof.append(cb)
    per_kernel = {}
    reps = 30
    for k in range(reps):
        cb = prof[k & 1]
        cb.commit().wait()
        for name, ms in cb.command_times():
            per_kernel.setdefault(name, []).append(ms)
    # one list entry per launch: average launch duration of each kernel
    kernel_us = {name: round(statistics.mean(v) * 1e3, 2) for name, v in per_kernel.items()}
    # the dominant kernel alone, back to back between one pair of events on its
    # stream, alternating the two KV copies: average launch duration
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    launches = 40
    for k in range(launches):
        record_split_only(cb, k & 1)
    cb.end_compute_pass()
    cb.commit().wait()
    split_us = round(statistics.mean(cb.commit().wait() for _ in range(3)) * 1e3 / launches, 2)
    algo_bytes = LANES * VISIBLE * ATTN_BYTES_PER_KEY
    achieved = algo_bytes / (split_us * 1e-6) / 1e9
    attn_layer_us = sum(kernel_us[k] for k in ("attn_qk_rope_ms", "attention_decode_split_ms",
                                               "attention_decode_combine_ms"))
    gdn_layer_us = kernel_us["gdn_decode_fused_ms"]
    gdn_gbs = LANES * GDN_BYTES_PER_LANE_LAYER / (gdn_layer_us * 1e-6) / 1e9

    line = {
        "metric": "decode attn+GDN us/layer @32k ctx x4 lanes",
        "value": round(ms_per_step * 1e3 / 4.0, 3),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "decode wave, 4 lanes x 32768 visible keys, one G,G,G,A period "
                               "(3 GDN layers + 1 full-attention layer), HIP-graph replay",
                   "lanes": LANES, "visible_keys": VISIBLE, "capacity": CAPACITY,
                   "split_keys": PART, "device": dev.name},
        "roofline": {"bound": "hbm", "kernel": "attention_decode_split_ms (flash_decode_kernel)",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": (round((FLASH_FETCH_KIB * FETCH_SCALE +
                                        FLASH_WRITE_KIB * WRITE_SCALE) * 1024)
                                 if PART == DEFAULT_SPLIT_KEYS else None),
                     "algorithmic_bytes": algo_bytes, "avg_launch_us": split_us},
        "detail": {"attention_layer_us": round(attn_layer_us, 2),
                   "gdn_layer_us": round(gdn_layer_us, 2),
                   "gdn_layer_gbs": round(gdn_gbs, 1),
                   "kernel_avg_us": kernel_us},
    }
    if not args.no_prefill:
        line["detail"]["prefill_16k"] = prefill_figures(B, dev, queue, lib, torch)
    if not args.no_prefill:
        from tatara_amd import q4_sweep
        line["detail"]["q4_projections"] = (
            [q4_sweep.measure(dev, queue, lib, name, LANES, False, 3, matrix_unit=True)
             for name in q4_sweep.FAMILIES] +
            [q4_sweep.measure(dev, queue, lib, name, 16384, True, 2) for name in q4_sweep.FAMILIES])
    if not args.no_cpu_baseline:
        threads = min(16, os.cpu_count() or 1)
        line["cpu_baseline"] = cpu_baseline(threads)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
