#!/usr/bin/env python3
"""Benchmark of the attention-family hot path on one MI355X.

A step is one decode token wave of 4 lanes at 32768 visible keys through the attention
family of the whole 40-layer hybrid stack, G,G,G,A x 10 (30 Gated DeltaNet layers, 10
full-attention layers), with the lane-batched operators:
    GDN:       gdn_decode_fused_ms (prepare + recurrence + gate-norm in one dispatch)
    attention: attention_decode_token_ms -> attention_decode_token_finish_ms (qk-norm and
               rotation inside the split-K walk; the token's own key and value folded in and
               appended by the finishing dispatch: what the host runtime records), or with
               --attention three the reference's own sequence attn_qk_rope_ms ->
               attention_decode_split_ms -> attention_decode_combine_ms
Projections (the reference's Q4 GEMVs) are not on the path: their outputs are resident
random bf16 slabs.  Every layer has its own KV pools, recurrent state and inputs, all in
HBM before the timed region (2.7 GB of keys and values: the 256 MB last-level cache cannot
serve the stream).  The wave is compiled into one HIP graph and replayed, one launch per
token as a serving loop would issue it.  `value` = microseconds per layer = step / 40.

`roofline` is for the dominant kernel, the key walk of the attention layer
(flash_decode_kernel): algorithmic bytes (2048 B per visible key and lane) over its
launch duration, measured with HIP events on the queue's stream around a graph that holds
that kernel once per attention layer (10 launches on 10 different KV sets per replay; median
and p10 / p90 over the replays).  `detail.config3` repeats the figure for the ragged lanes and
the single deep lane, next to the duration of all dispatches of the layer.

`detail.prefill_16k` adds the block-prefill side of the metric: 16384 new tokens of one lane
through a full-attention layer (causal flash attention on MFMA) and a Gated DeltaNet layer
(chunk-64 recurrence on MFMA), tok/s and fraction of MFMA peak, with the CPU checker timed on
a strided subset of the rows beside it.

`cpu_baseline` = the CPU checker (the reference's scalar arithmetic restated) timed on this
box's host cores on one G,G,G,A period of the same wave, one thread and all threads.

Prints ONE JSON line."""
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

from tatara_amd import stack as stack_rules   # noqa: E402  (the host's split-K planning rule)

LANES = 4
VISIBLE = 32768
CAPACITY = 32768
LAYERS = 40
PERIOD = 4                      # G,G,G,A
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0   # dense bf16
CALIBRATION_COPY_BYTES = 256 << 20
# HBM traffic of one launch of the key-walk kernel at 4 lanes x 32768 keys, from two rocprofv3
# counter runs (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each scaled by what the same
# counter read for a plain 256 MiB copy of known size; see the file named here.
TRAFFIC_SOURCE = "profiles/flash_decode_4x32768_hbm_counters.md"
TRAFFIC_BYTES = {"three": round((131289.6 * 262144.0 / 131083.3 + 2151.0) * 1024),    # 271,060,546
                 "token": round((131303.6 * 262144.0 / 131083.3 + 2146.9) * 1024)}    # 271,085,019
ATTN_BYTES_PER_KEY = 2048       # K and V rows of both kv heads, bf16
GDN_BYTES_PER_LANE_LAYER = 4194304 + 2 * 49152 + 65536 + 24704 + 4 * 8192
CONFIG3 = {
    "uniform": ([VISIBLE - 1] * 4, CAPACITY),
    "ragged": ([32767, 29999, 24575, 8191], CAPACITY),
    "lane100k": ([99999], 100096),
}
CAPACITY_SWEEP = (33024, 100096, 131072, 131136, 262144)


class Wave:
    """Buffers and recorders of the attention family of one token wave."""

    def __init__(self, dev, lib, torch, attention, split_keys, attention_layers, gdn_layers,
                 contexts, capacity, seed=0x7A7A):
        self.dev, self.lib, self.attention = dev, lib, attention
        self.forced_split = split_keys
        self.contexts, self.capacity = list(contexts), capacity
        self.rows = len(contexts)
        self.groups = dev.compute_units
        gen = torch.Generator(device="cuda")
        gen.manual_seed(seed)

        def rand_bf16(n, sigma=1.0):
            t = (torch.randn(n, generator=gen, device="cuda", dtype=torch.float32) * sigma).to(
                torch.bfloat16)
            return dev.wrap(t.data_ptr(), t.numel() * 2, keepalive=t)

        def rand_f32(n, sigma):
            t = torch.randn(n, generator=gen, device="cuda", dtype=torch.float32) * sigma
            return dev.wrap(t.data_ptr(), t.numel() * 4, keepalive=t)

        rows = self.rows
        stripe = 2 * capacity * 256
        ones = dev.buffer_from(np.full(256, 0x3F80, np.uint16))
        self.set_contexts(contexts)
        self.attn = []
        for _ in range(attention_layers):
            self.attn.append(dict(keys=rand_bf16(rows * stripe), values=rand_bf16(rows * stripe),
                                  proj=rand_bf16(rows * 9216), q_w=ones, k_w=ones))
        self.b_q, self.b_gate, self.b_out = (dev.create_buffer(rows * 8192) for _ in range(3))
        # records down to the finest split the rule picks (128 keys)
        self.b_part = dev.create_buffer(rows * 16 * ((capacity + 127) // 128) * 258 * 4)
        conv_elems, rec_elems = 3 * 8192, 32 * 128 * 128
        table = np.zeros(64, np.uint32)
        for r in range(rows):
            table[r * 4 + 0] = (2 * r) * conv_elems
            table[r * 4 + 1] = (2 * r + 1) * conv_elems
            table[r * 4 + 2] = (2 * r) * rec_elems
            table[r * 4 + 3] = (2 * r + 1) * rec_elems
        gdn_table = dev.buffer_from(table)
        self.gdn = []
        for i in range(gdn_layers):
            rng = np.random.default_rng(i + 1)
            a_log = (rng.uniform(-4.0, -2.5, 32).astype(np.float32).view(np.uint32) >> 16).astype(
                np.uint16)
            dt_bias = (rng.normal(0, 0.3, 32).astype(np.float32).view(np.uint32) >> 16).astype(
                np.uint16)
            self.gdn.append(dict(conv=rand_bf16(2 * rows * conv_elems, 0.5),
                                 rec=rand_f32(2 * rows * rec_elems, 0.02), table=gdn_table,
                                 proj=rand_bf16(rows * 12352, 0.5), conv_w=rand_bf16(4 * 8192, 0.5),
                                 a_log=dev.buffer_from(a_log), dt_bias=dev.buffer_from(dt_bias),
                                 norm_w=dev.buffer_from(np.full(128, 0x3F80, np.uint16))))
        self.g_out = dev.create_buffer(rows * 8192)

    def set_contexts(self, contexts):
        """A new state table (same pools): other lane depths over the same caches."""
        assert len(contexts) == self.rows and max(contexts) < self.capacity
        stripe = 2 * self.capacity * 256
        table = np.zeros(64, np.uint32)
        for r, context in enumerate(contexts):
            table[r * 4] = r * stripe
            table[r * 4 + 1] = context
        self.contexts = list(contexts)
        self.attn_table = self.dev.buffer_from(table)
        # The split-K walk as the host runtime plans it for a wave (runtime.cpp
        # choose_split_keys and the operator's c9): keys per workgroup so that the
        # workgroups that hold keys come to about one per compute unit (at least 128 keys, a
        # multiple of 32); waves of one or two lanes deal a lane's 32-key blocks to its
        # workgroups in turn; where the grid is larger than the chip and part of it holds no
        # keys, the workgroups that do are placed first in the dispatch order.
        visible = [c + 1 for c in contexts]
        self.part = self.forced_split or stack_rules.choose_split_keys(visible, self.dev.compute_units)
        self.max_splits = (self.capacity + self.part - 1) // self.part
        self.interleave = 1 if self.rows <= 2 else 0
        # contiguous ranges are walked from a rotated starting block, so that the stride
        # between ranges (the cache capacity) does not decide how the requests of the moment
        # fall on the memory channels
        self.rotate = 0 if self.interleave else 1
        live = stack_rules.split_workgroups(visible, self.part)
        grid = self.max_splits * 2 * self.rows
        self.compact = 1 if grid > live and grid > self.dev.compute_units else 0
        # the token form walks the cached keys only (the token itself is folded in afterwards)
        cached = [max(c, 1) for c in contexts]
        self.token_part = self.forced_split or stack_rules.choose_split_keys(cached, self.dev.compute_units)
        token_splits = (self.capacity + self.token_part - 1) // self.token_part
        grid = token_splits * 2 * self.rows
        self.token_compact = 1 if (grid > stack_rules.split_workgroups(cached, self.token_part)
                                   and grid > self.dev.compute_units) else 0

    def visible_keys(self):
        return sum(c + 1 for c in self.contexts)

    def record_gdn(self, cb, index):
        layer = self.gdn[index]
        cb.encode(self.lib.pipeline("gdn_decode_fused_ms"),
                  {0: layer["proj"], 1: layer["conv"], 2: layer["conv_w"], 3: layer["a_log"],
                   4: layer["dt_bias"], 5: layer["rec"], 6: layer["norm_w"], 7: self.g_out,
                   8: layer["table"]}, {9: 12352, 10: 4096}, (32, self.rows), (512,))

    def record_attention(self, cb, index, walk_only=False):
        """All dispatches of one attention layer; walk_only: the key-walk kernel alone."""
        layer, rows, cap, P = self.attn[index], self.rows, self.capacity, self.lib.pipeline
        if self.attention == "token":
            splits = (cap + self.token_part - 1) // self.token_part
            bind = {0: layer["proj"], 1: layer["q_w"], 2: layer["k_w"], 3: layer["keys"],
                    4: layer["values"], 5: self.attn_table, 6: self.b_part, 7: self.b_out}
            const = {8: cap, 9: 9216, 10: 4096, 11: self.token_part, 12: splits,
                     13: 2 * self.interleave + 4 * self.token_compact + 8 * self.rotate,
                     14: -(-max(self.contexts) // self.token_part)}
            cb.encode(P("attention_decode_token_ms"), bind, const, (splits, 2, rows), (256,))
            if not walk_only:
                cb.barrier()
                cb.encode(P("attention_decode_token_finish_ms"), bind, const, (16, rows), (256,))
            return
        if not walk_only:
            cb.encode(P("attn_qk_rope_ms"),
                      {0: layer["proj"], 1: layer["q_w"], 2: layer["k_w"], 3: self.b_q,
                       4: self.b_gate, 5: layer["keys"], 6: layer["values"], 8: self.attn_table},
                      {7: cap, 9: 9216, 10: 4096}, (18, rows), (256,))
            cb.barrier()
        cb.encode(P("attention_decode_split_ms"),
                  {0: self.b_q, 1: layer["keys"], 2: layer["values"], 3: self.attn_table,
                   4: self.b_part}, {5: cap, 6: 4096, 7: self.part, 8: self.max_splits,
                   9: 2 * self.interleave + 4 * self.compact + 8 * self.rotate},
                  (self.max_splits, 2, rows), (256,))
        if not walk_only:
            cb.barrier()
            cb.encode(P("attention_decode_combine_ms"),
                      {0: self.b_part, 1: self.b_gate, 2: self.attn_table, 3: self.b_out},
                      {4: self.part, 5: self.max_splits, 6: 4096, 7: 0, 8: cap}, (16, rows), (256,))

    def record_wave(self, cb):
        gdn = attn = 0
        for layer in range(len(self.gdn) + len(self.attn)):
            if layer % PERIOD == PERIOD - 1:
                self.record_attention(cb, attn)
                attn += 1
            else:
                self.record_gdn(cb, gdn)
                gdn += 1
            cb.barrier()


def percentiles(samples_us):
    s = sorted(samples_us)
    pick = lambda f: s[min(len(s) - 1, int(round(f * (len(s) - 1))))]
    return {"median_us": round(statistics.median(s), 2), "p10_us": round(pick(0.1), 2),
            "p90_us": round(pick(0.9), 2), "mean_us": round(statistics.mean(s), 2)}


def time_graph(queue, record, launches_per_replay, replays=12, warm=3):
    """Compiles `record` into a graph; device time of each replay (events on the queue's
    stream around the launch) divided by the launches it holds."""
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    record(cb)
    cb.end_compute_pass()
    cb.compile()
    for _ in range(warm):
        cb.commit().wait()
    per_launch = [cb.commit().wait() * 1e3 / launches_per_replay for _ in range(replays)]
    out = percentiles(per_launch)
    out["launches"] = launches_per_replay * replays
    return out


def attention_figures(queue, wave):
    """Key-walk kernel and whole attention layer of `wave` at its current contexts."""
    n = len(wave.attn)
    walk = time_graph(queue, lambda cb: [wave.record_attention(cb, i, walk_only=True)
                                         for i in range(n)], n)
    layer = time_graph(queue, lambda cb: [wave.record_attention(cb, i) for i in range(n)], n)
    algo = wave.visible_keys() * ATTN_BYTES_PER_KEY
    gbs = algo / (walk["median_us"] * 1e-6) / 1e9
    return {"lanes_visible_keys": [c + 1 for c in wave.contexts], "algorithmic_bytes": algo,
            "split_keys": wave.part if wave.attention == "three" else wave.token_part,
            "workgroups_with_keys_first": bool(wave.compact if wave.attention == "three" else wave.token_compact),
            "walk_kernel": walk, "walk_kernel_gbs": round(gbs, 1),
            "walk_kernel_frac": round(gbs / HBM_PEAK_GBS, 4),
            "layer_all_dispatches": layer,
            "layer_frac": round(algo / (layer["median_us"] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}


def prefill_figures(B, dev, queue, lib, torch, rows=16384, repeats=16, warm=6):
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
    # the first passes run at the clock the device idles at; the figures are medians of the
    # passes after them (a block prefill is a long run of such passes)
    times = {}
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
            times.setdefault(name, []).append(ms)
    best = {name: statistics.median(ms[warm:]) for name, ms in times.items()}
    flash_ms = best["attention_flash_v2_blk"]
    flops = 16 * 4 * 256 * rows * (rows + 1) / 2
    attn_ms = flash_ms + best["attn_qk_rope_blk"]
    gdn_ms = sum(best[k] for k in ("gdn_conv_blk", "gdn_gates_blk", "gdn_chunk_recurrence_blk",
                                   "gdn_gate_norm_blk"))
    gdn_flops = 32 * 7 * 128 * 128 * rows      # sequential-equivalent delta rule
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
            "gdn_recurrence_note": "chunk-64 recurrence: bound by the serial chain over 256 chunks "
                                   "and its chunk records, not by MFMA throughput",
            "gdn_recurrence_frac_of_bf16_mfma_peak_sequential_equivalent": round(
                gdn_flops / (best["gdn_chunk_recurrence_blk"] * 1e-3) / 2.5e15, 4),
            "kernel_ms": {k: round(v, 3) for k, v in best.items()}}


CONFIG5_DECODE_CONTEXTS = (1024, 4096, 16384, 32768, 65536, 100000)
CONFIG5_PREFILL_TOKENS = (4096, 32768)
CONFIG5_LANES = (1, 4)
CONFIG5_BLOCK_ROWS = 2048


def dense_block_figures(dev, queue, lib, torch, rows=16384, repeats=15):
    """dense_bf16 (the stub stack's stand-in for the projections) on a block of rows at the
    three projection shapes of the family: device time per dispatch and MFMA rate."""
    out = []
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0xDE75E)
    for in_dim, out_dim in ((2048, 9216), (2048, 12352), (4096, 2048)):
        x = torch.randn(rows * in_dim, generator=gen, device="cuda").to(torch.bfloat16)
        w = (torch.randn(out_dim * in_dim, generator=gen, device="cuda") * in_dim ** -0.5).to(torch.bfloat16)
        y = torch.empty(rows * out_dim, device="cuda", dtype=torch.bfloat16)
        torch.cuda.synchronize()
        b_x, b_w, b_y = (dev.wrap(t.data_ptr(), t.numel() * 2, keepalive=t) for t in (x, w, y))
        figures = time_graph(queue, lambda cb: cb.encode(
            lib.pipeline("dense_bf16"), {0: b_x, 1: b_w, 2: b_y}, {3: rows, 4: in_dim, 5: out_dim},
            ((out_dim + 63) // 64, (rows + 15) // 16), (256,)), 1, replays=repeats, warm=10)
        flops = 2.0 * rows * in_dim * out_dim
        tflops = flops / (figures["median_us"] * 1e-6) / 1e12
        out.append({"operator": "dense_bf16", "rows": rows, "in": in_dim, "out": out_dim,
                    "us": figures["median_us"], "tflops": round(tflops, 1),
                    "frac_of_bf16_mfma_peak": round(tflops / MFMA_PEAK_TFLOPS, 4)})
        del x, w, y
        torch.cuda.empty_cache()
    return out


def block_2048_figures(B, dev, queue, lib, torch, capacity=32768, repeats=12):
    """The causal flash kernel on the reference's block size: 2048 new rows behind 30720, 14336
    and 0 cached tokens of one lane, with one workgroup per 32 rows and kv head (128 workgroups:
    attention_flash_split_blk told to share nothing), with the sharers the library plans for the
    device in the caller's scratch, and as attention_flash_v2_blk, which plans the same in its
    queue's workspace.  Device time per dispatch (the clearing dispatch of a shared walk
    included)."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x2048)
    rows = 2048

    def rb(n):
        t = torch.randn(n, generator=gen, device="cuda").to(torch.bfloat16)
        return dev.wrap(t.data_ptr(), n * 2, keepalive=t)

    keys, values = rb(2 * capacity * 256), rb(2 * capacity * 256)
    q, gate = rb(rows * 4096), rb(rows * 4096)
    out = dev.create_buffer(rows * 8192)
    points = []
    for base in (capacity - rows, 14336, 0):
        sharers = B.flash_prefill_splits(rows, base + rows, dev.compute_units)
        scratch = dev.create_buffer(max(B.flash_prefill_scratch_bytes(rows, sharers), 256))
        flops = 16 * 1024.0 * (rows * base + rows * (rows + 1) / 2)
        point = {"rows": rows, "cached_tokens": base, "sharers": sharers}
        for label, name, bind, const in (
                ("one_workgroup_a_tile", "attention_flash_split_blk", {}, {10: 1}),
                ("attention_flash_split_blk", "attention_flash_split_blk", {9: scratch}, {10: sharers}),
                ("attention_flash_v2_blk", "attention_flash_v2_blk", {}, {})):
            figures = time_graph(queue, lambda cb: cb.encode(
                lib.pipeline(name), {0: q, 1: keys, 2: values, 3: gate, 4: out, **bind},
                {5: base + rows, 6: capacity, 7: rows, 8: base, **const},
                (16, (rows + 15) // 16), (256,)), 1, replays=repeats, warm=6)
            tflops = flops / (figures["median_us"] * 1e-6) / 1e12
            point[label] = {"us": figures["median_us"], "tflops": round(tflops, 1),
                            "frac_of_bf16_mfma_peak": round(tflops / MFMA_PEAK_TFLOPS, 4)}
        points.append(point)
    return points


def config5_decode_point(dev, queue, lib, torch, attention, lanes, visible):
    """One decode token wave of `lanes` lanes at `visible` visible keys through the
    attention family of all 40 layers (own caches and state per layer), compiled into one
    graph and replayed: device time of whole replays, launch gaps and all."""
    capacity = (visible + 1023) // 1024 * 1024
    attention_layers = LAYERS // PERIOD
    wave = Wave(dev, lib, torch, attention, 0, attention_layers, LAYERS - attention_layers,
                [visible - 1] * lanes, capacity)
    step = time_graph(queue, wave.record_wave, 1, replays=10, warm=2)
    us = step["median_us"]
    kv = attention_layers * wave.visible_keys() * ATTN_BYTES_PER_KEY
    gdn = (LAYERS - attention_layers) * lanes * GDN_BYTES_PER_LANE_LAYER
    split = wave.part if attention == "three" else wave.token_part
    del wave
    torch.cuda.empty_cache()
    return {"lanes": lanes, "visible_keys": visible, "capacity": capacity, "split_keys": split,
            "wave_us": us, "wave_p10_us": step["p10_us"], "wave_p90_us": step["p90_us"],
            "us_per_layer": round(us / LAYERS, 3), "tok_per_s": round(lanes / (us * 1e-6)),
            "algorithmic_gbs": round((kv + gdn) / (us * 1e-6) / 1e9, 1)}


class PrefillFamily:
    """The attention family of all 40 layers over blocks of 2048 rows: per Gated DeltaNet layer
    conv, gates, chunk-64 recurrence and gate-norm, per attention layer rope and causal flash
    attention over the lane's cache so far.  Own caches and recurrent state per layer and
    lane; the projections (resident random slabs) are shared by the layers of a kind."""

    def __init__(self, dev, lib, torch, lanes, tokens):
        from tatara_amd import backend as B
        self.B, self.dev, self.lib = B, dev, lib
        self.lanes, self.tokens = lanes, tokens
        gen = torch.Generator(device="cuda")
        gen.manual_seed(0xC5F1 + tokens)
        self.rows_max = min(CONFIG5_BLOCK_ROWS, tokens)
        mk = dev.create_buffer

        def rb(n, sigma=1.0):
            t = (torch.randn(n, generator=gen, device="cuda") * sigma).to(torch.bfloat16)
            return dev.wrap(t.data_ptr(), n * 2, keepalive=t)

        self.ones256 = dev.buffer_from(np.full(256, 0x3F80, np.uint16))
        self.ones128 = dev.buffer_from(np.full(128, 0x3F80, np.uint16))
        self.a_proj, self.g_proj = rb(self.rows_max * 9216), rb(self.rows_max * 12352, 0.5)
        self.conv_w = rb(4 * 8192, 0.5)
        rng = np.random.default_rng(5)
        self.a_log = dev.buffer_from((rng.uniform(-4.0, -2.5, 32).astype(np.float32).view(np.uint32) >> 16)
                                     .astype(np.uint16))
        self.dt_bias = dev.buffer_from(np.zeros(32, np.uint16))
        attention_layers = LAYERS // PERIOD
        self.stripe_bytes = 2 * tokens * 256 * 2
        self.caches = [(mk(lanes * self.stripe_bytes), mk(lanes * self.stripe_bytes))
                       for _ in range(attention_layers)]
        self.conv_bytes, self.rec_bytes = 3 * 8192 * 2, 32 * 128 * 128 * 4
        self.states = [(mk(2 * lanes * self.conv_bytes), mk(2 * lanes * self.rec_bytes))
                       for _ in range(LAYERS - attention_layers)]

    def working_set(self):
        """The block-sized buffers one stream of blocks works in."""
        B, mk, rows_max, units = self.B, self.dev.create_buffer, self.rows_max, self.dev.compute_units
        work = {name: mk(rows_max * 8192) for name in ("q", "gate", "out", "qk", "v", "z", "y")}
        work["decay"], work["beta"] = mk(rows_max * 128), mk(rows_max * 128)
        work["chunk"] = mk(((rows_max + 63) // 64) * 32 * 115712)
        # a 2048-row block is 128 workgroups of the flash kernel: the host shares each position
        # tile's key walk between as many workgroups as fill the device (attention_flash_split_blk)
        work["shared_walk"] = mk(max(
            [B.flash_prefill_scratch_bytes(r, B.flash_prefill_splits(r, self.tokens, units))
             for r in range(32, rows_max + 1, 32)] + [256]))
        return work

    def record_block(self, cb, w, lane, base, rows, swapped):
        B, P, tokens = self.B, self.lib.pipeline, self.tokens
        units = self.dev.compute_units
        attn = gdn = 0
        for layer in range(LAYERS):
            if layer % PERIOD == PERIOD - 1:
                keys = (self.caches[attn][0], lane * self.stripe_bytes)
                values = (self.caches[attn][1], lane * self.stripe_bytes)
                attn += 1
                cb.encode(P("attn_qk_rope_blk"),
                          {0: self.a_proj, 1: self.ones256, 2: self.ones256, 3: w["q"], 4: w["gate"],
                           5: keys, 6: values}, {7: base, 8: tokens}, (18, rows), (256,))
                cb.barrier()
                sharers = B.flash_prefill_splits(rows, base + rows, units)
                if sharers > 1:
                    cb.encode(P("attention_flash_split_blk"),
                              {0: w["q"], 1: keys, 2: values, 3: w["gate"], 4: w["out"], 9: w["shared_walk"]},
                              {5: base + rows, 6: tokens, 7: rows, 8: base, 10: sharers},
                              (16, (rows + 15) // 16), (256,))
                else:
                    cb.encode(P("attention_flash_v2_blk"),
                              {0: w["q"], 1: keys, 2: values, 3: w["gate"], 4: w["out"]},
                              {5: base + rows, 6: tokens, 7: rows, 8: base},
                              (16, (rows + 15) // 16), (256,))
            else:
                conv, rec = self.states[gdn]
                gdn += 1
                plane_in, plane_out = (2 * lane + 1, 2 * lane) if swapped else (2 * lane, 2 * lane + 1)
                cb.encode(P("gdn_conv_blk"),
                          {0: self.g_proj, 1: (conv, plane_in * self.conv_bytes), 2: self.conv_w, 3: w["qk"],
                           4: w["v"], 5: w["z"], 6: (conv, plane_out * self.conv_bytes)}, {7: rows},
                          (96, rows), (128,))
                cb.encode(P("gdn_gates_blk"),
                          {0: self.g_proj, 1: self.a_log, 2: self.dt_bias, 3: w["decay"], 4: w["beta"]},
                          {5: rows}, (1, (rows + 3) // 4, 1), (32, 4, 1))
                cb.barrier()
                cb.encode(P("gdn_chunk_recurrence_blk"),
                          {0: w["qk"], 1: w["v"], 2: w["decay"], 3: w["beta"], 4: w["chunk"],
                           5: (rec, plane_in * self.rec_bytes), 6: w["y"], 7: (rec, plane_out * self.rec_bytes)},
                          {8: rows}, (8, 32), (256,))
                cb.barrier()
                cb.encode(P("gdn_gate_norm_blk"), {0: w["y"], 1: w["z"], 2: self.ones128, 3: w["out"]}, {},
                          (32, rows), (128,))
            cb.barrier()

    def blocks(self):
        return [(base, min(CONFIG5_BLOCK_ROWS, self.tokens - base))
                for base in range(0, self.tokens, CONFIG5_BLOCK_ROWS)]


def config5_prefill_point(dev, queue, lib, torch, lanes, tokens):
    """`tokens` new tokens of each of `lanes` lanes, lane after lane on one queue, through the
    attention family of all 40 layers in blocks of 2048 rows.  Device time of each block's
    command buffer (launch gaps included), summed."""
    family = PrefillFamily(dev, lib, torch, lanes, tokens)
    work = family.working_set()
    total_ms = 0.0
    for lane in range(lanes):
        swapped = False
        for base, rows in family.blocks():
            cb = queue.create_command_buffer()
            cb.begin_compute_pass()
            family.record_block(cb, work, lane, base, rows, swapped)
            cb.end_compute_pass()
            total_ms += cb.commit().wait()
            swapped = not swapped
    total = lanes * tokens
    del family, work
    torch.cuda.empty_cache()
    return {"lanes": lanes, "tokens": tokens, "block_rows": CONFIG5_BLOCK_ROWS,
            "family_ms": round(total_ms, 3), "tok_per_s": round(total / (total_ms * 1e-3)),
            "us_per_layer_token": round(total_ms * 1e3 / (LAYERS * total), 4)}


def config5_figures(dev, queue, lib, torch, attention):
    """The hybrid stack sweep: decode waves at six depths and blocked prefill of two prompt
    lengths, one lane and four, attention family of all 40 layers only (the projections are
    resident inputs, as in the headline)."""
    decode = [config5_decode_point(dev, queue, lib, torch, attention, lanes, visible)
              for lanes in CONFIG5_LANES for visible in CONFIG5_DECODE_CONTEXTS]
    prefill = [config5_prefill_point(dev, queue, lib, torch, lanes, tokens)
               for lanes in CONFIG5_LANES for tokens in CONFIG5_PREFILL_TOKENS]
    return {"layers": LAYERS, "pattern": "G,G,G,A x 10", "attention_form": attention,
            "decode": decode, "prefill": prefill,
            "how": "decode: one HIP-graph replay per token wave, median of 10; prefill: device "
                   "time of every 2048-row block's command buffer, summed, lane after lane"}


def _oracle():
    path = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(path):
        return None
    L = C.CDLL(path)
    u16 = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
    f32 = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
    u32 = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
    c32 = C.c_uint32
    L.tto_attn_qk_rope.argtypes = [u16, u16, u16, c32, c32, u16, u16, u16, u16]
    L.tto_attn_qk_rope.restype = None
    L.tto_attention_decode_split.argtypes = [u16, u16, u16, u16, c32, c32, c32, C.c_void_p, u16, c32]
    L.tto_attention_decode_split.restype = None
    L.tto_gdn_decode_step.argtypes = [u16] * 6 + [f32, u16, f32, u16, c32]
    L.tto_gdn_decode_step.restype = None
    L.tto_attention_prefill.argtypes = [u16, u16, u16, c32, c32, c32, u16, u16, u16, u16, u32, c32,
                                        u16, c32]
    L.tto_attention_prefill.restype = None
    L.tto_gdn_prefill.argtypes = [u16, c32, u16, u16, u16, u16, u16, f32, u16, f32, u16, u16, u16,
                                  u16, c32]
    L.tto_gdn_prefill.restype = None
    return L


def _bf16(rng, n, sigma=1.0):
    x = rng.standard_normal(n, dtype=np.float32) * np.float32(sigma)
    return (x.view(np.uint32) >> 16).astype(np.uint16)      # truncation is fine for random data


def cpu_baseline(all_threads):
    """The CPU checker (reference arithmetic restated, oracle/liboracle.so) on one G,G,G,A
    period of the wave: per lane its own data, rope + append + 32768-key attention, and
    3 x 4 lanes of GDN decode; timed with one thread and with all host threads.  Baseline
    only; never part of the product path."""
    L = _oracle()
    if L is None:
        return None
    rng = np.random.default_rng(7)
    ones = np.full(256, 0x3F80, np.uint16)
    lanes = []
    for _ in range(LANES):
        lanes.append(dict(keys=_bf16(rng, 2 * CAPACITY * 256), values=_bf16(rng, 2 * CAPACITY * 256),
                          proj=_bf16(rng, 9216), gproj=_bf16(rng, 12352, 0.5),
                          cs=_bf16(rng, 3 * 8192, 0.5),
                          st=rng.standard_normal(32 * 128 * 128, dtype=np.float32) * np.float32(0.02)))
    cw = _bf16(rng, 4 * 8192, 0.5)
    a_log = np.full(32, 0xC040, np.uint16)   # -3.0
    dtb = np.zeros(32, np.uint16)
    nw = np.full(128, 0x3F80, np.uint16)
    q = np.zeros(4096, np.uint16); gate = np.zeros(4096, np.uint16); out = np.zeros(4096, np.uint16)
    ncs = np.zeros(3 * 8192, np.uint16); so = np.zeros(32 * 128 * 128, np.float32)
    gated = np.zeros(4096, np.uint16)

    def period(threads):
        t0 = time.perf_counter()
        for lane in lanes:
            L.tto_attn_qk_rope(lane["proj"], ones, ones, VISIBLE - 1, CAPACITY, q, gate,
                               lane["keys"], lane["values"])
            L.tto_attention_decode_split(q, gate, lane["keys"], lane["values"], VISIBLE - 1,
                                         CAPACITY, 256, None, out, threads)
        t_attn = time.perf_counter() - t0
        t0 = time.perf_counter()
        for _ in range(3):
            for lane in lanes:
                L.tto_gdn_decode_step(lane["gproj"], lane["cs"], cw, a_log, dtb, nw, lane["st"],
                                      ncs, so, gated, threads)
        return t_attn, time.perf_counter() - t0

    a1, g1 = period(1)
    an, gn = period(all_threads)
    return {"value": round((an + gn) * 1e6 / 4.0, 1), "unit": "us/layer", "cores": all_threads,
            "kind": "port", "host_cpu_count": os.cpu_count(),
            "single_thread": {"value": round((a1 + g1) * 1e6 / 4.0, 1), "unit": "us/layer", "cores": 1,
                              "attention_layer_us": round(a1 * 1e6), "gdn_layer_us": round(g1 * 1e6 / 3)},
            "sample": "one full G,G,G,A period of the wave, 4 lanes x 32768 keys, distinct data per "
                      f"lane, rope and append included (all threads: attention layer {an * 1e6:.0f} us, "
                      f"GDN layer {gn * 1e6 / 3:.0f} us)"}


def cpu_prefill_baseline(threads, rows=16384):
    """The CPU checker beside the 16384-row block prefill: the attention layer on every 256th
    query row (plus the rope of all rows), extrapolated by causal pair count; the GDN layer on
    the first 2048 rows, extrapolated by rows."""
    L = _oracle()
    if L is None:
        return None
    rng = np.random.default_rng(11)
    ones = np.full(256, 0x3F80, np.uint16)
    proj = _bf16(rng, rows * 9216)
    keys = np.zeros(2 * rows * 256, np.uint16); values = np.zeros_like(keys)
    query = np.zeros(rows * 4096, np.uint16); gate = np.zeros_like(query); att = np.zeros_like(query)
    sel = np.arange(255, rows, 256, dtype=np.uint32)
    t0 = time.perf_counter()
    L.tto_attention_prefill(proj, ones, ones, rows, 0, rows, query, gate, keys, values, sel,
                            len(sel), att, threads)
    t_attn = time.perf_counter() - t0
    sampled_pairs = int(sum(int(r) + 1 for r in sel))
    all_pairs = rows * (rows + 1) // 2
    g_rows = 2048
    gproj = _bf16(rng, g_rows * 12352, 0.5)
    outs = [np.zeros(g_rows * 4096, np.uint16) for _ in range(4)]
    conv = np.zeros(3 * 8192, np.uint16); state = np.zeros(32 * 128 * 128, np.float32)
    t0 = time.perf_counter()
    L.tto_gdn_prefill(gproj, g_rows, _bf16(rng, 3 * 8192, 0.5), _bf16(rng, 4 * 8192, 0.5),
                      np.full(32, 0xC040, np.uint16), np.zeros(32, np.uint16),
                      np.full(128, 0x3F80, np.uint16),
                      rng.standard_normal(32 * 128 * 128, dtype=np.float32) * np.float32(0.02), conv,
                      state, *outs, threads)
    t_gdn = time.perf_counter() - t0
    attn_full = t_attn * all_pairs / sampled_pairs
    gdn_full = t_gdn * rows / g_rows
    return {"kind": "port", "cores": threads, "extrapolated": True,
            "attention_layer_tok_per_s": round(rows / attn_full, 1),
            "gdn_layer_tok_per_s": round(rows / gdn_full, 1),
            "sample": f"attention: {len(sel)} of {rows} query rows (every 256th) = {sampled_pairs} of "
                      f"{all_pairs} causal pairs in {t_attn:.2f} s incl. the rope of all rows; GDN: first "
                      f"{g_rows} of {rows} rows in {t_gdn:.2f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--attention", choices=("three", "token"), default="token",
                    help="token: the walk norms and rotates the query heads itself, a finishing "
                         "dispatch folds in the token's own key and value (what the host runtime "
                         "records: the shorter wave); three: rope, split and combine dispatches, "
                         "the reference's own sequence")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-prefill", action="store_true",
                    help="skip the 16384-row block prefill figures in detail.prefill_16k")
    ap.add_argument("--no-config5", action="store_true",
                    help="skip the stack sweep in detail.config5 (decode waves at 1k ... 100k keys and "
                         "blocked prefill of 4k / 32k tokens, 1 and 4 lanes)")
    ap.add_argument("--no-config3", action="store_true",
                    help="skip the ragged-lane and deep-lane figures in detail.config3")
    ap.add_argument("--split-keys", type=int, default=0,
                    help="keys per split-K workgroup of the key walk (multiple of 32); 0: what "
                         "the host runtime picks for the wave (1024 at 4 x 32768, 800 at 1 x 100000)")
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
    if args.calibrate_copy:
        src = dev.create_buffer(CALIBRATION_COPY_BYTES)
        dst = dev.create_buffer(CALIBRATION_COPY_BYTES)
        for _ in range(3):
            cb = queue.create_command_buffer()
            cb.copy_buffer(src, 0, dst, 0, CALIBRATION_COPY_BYTES)
            cb.commit().wait()
    attention_layers = LAYERS // PERIOD
    wave = Wave(dev, lib, torch, args.attention, args.split_keys, attention_layers,
                LAYERS - attention_layers, CONFIG3["uniform"][0], CAPACITY)

    step = queue.create_command_buffer()
    step.begin_compute_pass()
    wave.record_wave(step)
    step.end_compute_pass()
    step.compile()
    for _ in range(args.warmup):
        step.commit()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step.commit()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    # the same step, device time of single replays (median and tails)
    step_us = percentiles([step.commit().wait() * 1e3 for _ in range(max(20, min(args.steps, 100)))])

    uniform = attention_figures(queue, wave)
    gdn = time_graph(queue, lambda cb: [wave.record_gdn(cb, i) for i in range(len(wave.gdn))],
                     len(wave.gdn))
    gdn_gbs = LANES * GDN_BYTES_PER_LANE_LAYER / (gdn["median_us"] * 1e-6) / 1e9
    walk = uniform["walk_kernel"]
    kernel_name = ("attention_decode_token_ms (flash_decode_kernel, rope form)"
                   if args.attention == "token" else "attention_decode_split_ms (flash_decode_kernel)")
    line = {
        "metric": "decode attn+GDN us/layer @32k ctx x4 lanes",
        "value": round(ms_per_step * 1e3 / LAYERS, 3),
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
        "config": {"workload": "decode token wave, 4 lanes x 32768 visible keys, attention family of "
                               "the 40-layer stack (G,G,G,A x 10: 30 GDN + 10 full-attention layers, "
                               "own KV / state per layer), one HIP-graph replay per wave",
                   "lanes": LANES, "visible_keys": VISIBLE, "capacity": CAPACITY, "layers": LAYERS,
                   "attention_form": args.attention, "workgroups": wave.groups,
                   "split_keys": wave.part if args.attention == "three" else wave.token_part,
                   "device": dev.name},
        "roofline": {"bound": "hbm", "kernel": kernel_name,
                     "achieved": uniform["walk_kernel_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": uniform["walk_kernel_frac"],
                     "traffic": TRAFFIC_BYTES[args.attention],
                     "traffic_source": TRAFFIC_SOURCE,
                     "algorithmic_bytes": uniform["algorithmic_bytes"],
                     "avg_launch_us": walk["mean_us"], "median_launch_us": walk["median_us"],
                     "p10_launch_us": walk["p10_us"], "p90_launch_us": walk["p90_us"],
                     "launches": walk["launches"],
                     "how": "graph of this kernel alone, once per attention layer (10 KV sets), "
                            "HIP events on the queue's stream around each replay"},
        "detail": {"step_device_us": step_us,
                   "attention_layer_us": uniform["layer_all_dispatches"],
                   "attention_layer_frac_of_hbm_peak": uniform["layer_frac"],
                   "gdn_layer_us": gdn, "gdn_layer_gbs": round(gdn_gbs, 1),
                   "gdn_layer_frac_of_hbm_peak": round(gdn_gbs / HBM_PEAK_GBS, 4)},
    }
    if not args.no_config3:
        config3 = {"uniform": uniform}
        wave.set_contexts(CONFIG3["ragged"][0])
        config3["ragged"] = attention_figures(queue, wave)
        del wave, step
        torch.cuda.empty_cache()
        deep = Wave(dev, lib, torch, args.attention, args.split_keys, 4, 0, *CONFIG3["lane100k"])
        config3["lane100k"] = attention_figures(queue, deep)
        del deep
        torch.cuda.empty_cache()
        # the uniform wave again in caches of other capacities: the stride between the ranges
        # of a lane's workgroups, between heads and between lanes is the capacity's, and the
        # walk must not depend on how those strides fall on the memory channels
        config3["uniform_by_capacity"] = []
        for capacity in CAPACITY_SWEEP:
            other = Wave(dev, lib, torch, args.attention, args.split_keys, 4, 0,
                         CONFIG3["uniform"][0], capacity)
            figures = attention_figures(queue, other)
            config3["uniform_by_capacity"].append(
                {"capacity": capacity, "split_keys": figures["split_keys"],
                 "workgroups_with_keys_first": figures["workgroups_with_keys_first"],
                 "walk_kernel": figures["walk_kernel"], "walk_kernel_frac": figures["walk_kernel_frac"],
                 "layer_all_dispatches": figures["layer_all_dispatches"],
                 "layer_frac": figures["layer_frac"]})
            del other
            torch.cuda.empty_cache()
        line["detail"]["config3"] = config3
    else:
        del wave, step
        torch.cuda.empty_cache()
    if not args.no_config5:
        line["detail"]["config5"] = config5_figures(dev, queue, lib, torch, args.attention)
    # host threads of the CPU legs: what this process may run on, bounded by the box's CPU
    # share where the environment states one (OMP_NUM_THREADS)
    threads = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    if os.environ.get("OMP_NUM_THREADS", "").isdigit():
        threads = max(1, min(threads, int(os.environ["OMP_NUM_THREADS"])))
    if not args.no_prefill:
        line["detail"]["prefill_16k"] = prefill_figures(B, dev, queue, lib, torch)
        if not args.no_cpu_baseline:
            line["detail"]["prefill_16k"]["cpu_baseline"] = cpu_prefill_baseline(threads)
        line["detail"]["dense_bf16_block"] = dense_block_figures(dev, queue, lib, torch)
        line["detail"]["prefill_block_2048"] = block_2048_figures(B, dev, queue, lib, torch)
        from tatara_amd import q4_sweep
        line["detail"]["q4_projections"] = (
            [q4_sweep.measure(dev, queue, lib, name, LANES, False, 3, matrix_unit=True)
             for name in q4_sweep.FAMILIES] +
            [q4_sweep.measure(dev, queue, lib, name, 16384, True, 6) for name in q4_sweep.FAMILIES] +
            # the reference's block size: the last, partly filled round of tiles is shared
            [q4_sweep.measure(dev, queue, lib, name, 2048, True, 6) for name in q4_sweep.FAMILIES])
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(threads)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
