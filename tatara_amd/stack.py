"""A stubbed hybrid stack around the attention family, for stacked parity runs and
context sweeps: `layers` layers in the G,G,G,A pattern at hidden 2048, with the
reference's MoE block left out and its projections (hidden -> 12352 / 9216 in,
4096 -> hidden out) either as random bf16 dense matrices or, with quantized weights,
as the reference's affine 4-bit projections (attn_project / gdn_project / gdn_outproj
and their _ms / _blk forms).  Per layer:

    n = rms_only(x, input_norm);  p = dense(n, W_in)
    a = GatedDeltaNet(p) | FullAttention(p);  x = x + dense(a, W_out)

and after the last layer  logits = dense(rms_only(x, final_norm), W_vocab).  The
residual sum of a layer and the norm that follows it (the next layer's input norm or
the final norm) are one dispatch, residual_rms_ms, as in the reference's layer loop
(decode_step.cpp:1298-1308).

The walk mirrors the reference's layer loop (src/runtime/decode_step.cpp:1008-1293
for a token wave over pooled lanes, prefill_step.cpp:1386-2081 for a block of one
lane): lane state lives in per-layer pools addressed through a state offset table,
GDN planes ping-pong, attention caches append at the lane's context.
"""
import numpy as np

from tatara_amd import backend

HIDDEN = 2048
GDN_PROJ = 12352
ATTN_PROJ = 9216
CONV_ELEMS = 3 * 8192
REC_ELEMS = 32 * 128 * 128
CHUNK_RECORD_BYTES = 115712


def layer_kinds(layers):
    """'G' for Gated DeltaNet, 'A' for full attention: every fourth layer attends."""
    return ["A" if (i % 4) == 3 else "G" for i in range(layers)]


def _bf16(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


ATTN_SEGMENTS = (8192, 512, 512)        # query + gate, key, value rows of the in-projection
GDN_SEGMENTS = (8192, 4096, 32, 32)     # qkv, z, b, a rows


def quantize_random(rng, rows, k, sigma):
    """A random affine 4-bit matrix (group 64) whose entries have standard deviation
    about `sigma`: nibbles uniform in 0..15 (standard deviation 4.61 around 7.5), one
    bf16 scale and bias per 64 columns.  Returns (words u32, scales bf16, biases bf16)."""
    words = rng.integers(0, 2 ** 32, rows * k // 8, dtype=np.uint64).astype(np.uint32)
    scale = (sigma / 4.61) * rng.uniform(0.8, 1.2, rows * k // 64).astype(np.float32)
    return words, _bf16(scale), _bf16(-7.5 * scale)


def make_weights(layers, vocab, seed, quantized=False):
    """Host-side weights as uint16 bf16 arrays; scales keep the residual stream O(1).
    With `quantized`, the in- and out-projections are affine 4-bit: w["in_q4"] holds one
    (words, scales, biases) triple per matrix of the projection, w["out_q4"] one triple."""
    rng = np.random.default_rng(seed)

    def normal(n, sigma):
        return _bf16(rng.standard_normal(n, dtype=np.float32) * np.float32(sigma))

    out = {"layers": [], "final_norm": _bf16(1.0 + 0.05 * rng.standard_normal(HIDDEN)),
           "vocab": normal(vocab * HIDDEN, HIDDEN ** -0.5),
           "embed": normal(vocab * HIDDEN, 1.0)}
    for kind in layer_kinds(layers):
        w = {"kind": kind, "input_norm": _bf16(1.0 + 0.05 * rng.standard_normal(HIDDEN)),
             "w_out": normal(HIDDEN * 4096, 0.5 * 4096 ** -0.5)}
        if kind == "G":
            w["w_in"] = normal(GDN_PROJ * HIDDEN, HIDDEN ** -0.5)
            w["conv_w"] = normal(4 * 8192, 0.5)
            w["a_log"] = _bf16(rng.uniform(-4.0, -2.5, 32))
            w["dt_bias"] = normal(32, 0.3)
            w["norm_w"] = _bf16(1.0 + 0.1 * rng.standard_normal(128))
        else:
            w["w_in"] = normal(ATTN_PROJ * HIDDEN, HIDDEN ** -0.5)
            w["q_norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(256))
            w["k_norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(256))
        if quantized:
            segments = GDN_SEGMENTS if kind == "G" else ATTN_SEGMENTS
            w["in_q4"] = [quantize_random(rng, rows, HIDDEN, HIDDEN ** -0.5) for rows in segments]
            w["out_q4"] = quantize_random(rng, HIDDEN, 4096, 0.5 * 4096 ** -0.5)
            del w["w_in"], w["w_out"]
        out["layers"].append(w)
    return out


def split_workgroups(visible_keys, split_keys):
    """Workgroups of one attention layer's split-K grid that hold keys (two kv heads); the
    backend library's rule, which the C++ runtime calls as well."""
    return backend.split_workgroups(list(visible_keys), split_keys)


def choose_split_keys(visible_keys, compute_units=256):
    """Keys per split-K workgroup for a token wave whose lanes see `visible_keys[r]` keys
    each: the finest multiple of 32, at least 128, with which the workgroups that hold
    keys fit the compute units one each.  The backend library's rule (tt_choose_split_keys),
    the same call the C++ runtime makes."""
    return backend.choose_split_keys(list(visible_keys), compute_units)


class StubStack:
    """Device side of the stubbed stack: uploads weights, owns the pooled lane
    state and the scratch, and records token waves and prefill blocks."""

    def __init__(self, dev, lib, weights, lanes, capacity, vocab, block_rows=2048,
                 split_keys=None, attention_form="token", fused_wave_steps=False):
        """attention_form: "token" records a token wave's attention layer as the two-dispatch
        form (attention_decode_token_ms norms and rotates the query heads inside the split-K
        walk, attention_decode_token_finish_ms folds in and appends the token's own key and
        value: the shorter wave at every depth); "three" as rope, split-K and combine
        dispatches (split_keys keys per workgroup), the reference's own sequence.
        fused_wave_steps: decode waves of several lanes over 4-bit weights take the norm in
        the prologue of the input projection and the residual sum in the epilogue of the
        output projection (same bits, one dispatch less per layer; measured slower, because
        every workgroup of the projection norms the rows again)."""
        assert attention_form in ("three", "token")
        self.dev, self.lib = dev, lib
        self.attention_form = attention_form
        self.fused_wave_steps = fused_wave_steps
        self.groups = dev.compute_units
        self.lanes, self.capacity, self.vocab = lanes, capacity, vocab
        self.block_rows = block_rows
        self.split_keys = split_keys or choose_split_keys([capacity] * lanes, dev.compute_units)
        split_keys = self.split_keys
        self.max_splits = (capacity + split_keys - 1) // split_keys
        up = dev.buffer_from
        self.final_norm = up(weights["final_norm"])
        self.w_vocab = up(weights["vocab"])
        self.layers = []
        self.context = [0] * lanes          # cached positions per lane
        self.swapped = [False] * lanes      # GDN ping-pong phase per lane
        stripe = 2 * capacity * 256
        for w in weights["layers"]:
            layer = {"kind": w["kind"], "input_norm": up(w["input_norm"]),
                     "table": dev.create_buffer(256)}
            if "in_q4" in w:
                layer["in_q4"] = [tuple(up(part) for part in matrix) for matrix in w["in_q4"]]
                layer["out_q4"] = tuple(up(part) for part in w["out_q4"])
            else:
                layer["w_in"], layer["w_out"] = up(w["w_in"]), up(w["w_out"])
            if w["kind"] == "G":
                for name in ("conv_w", "a_log", "dt_bias", "norm_w"):
                    layer[name] = up(w[name])
                layer["conv"] = dev.create_buffer(2 * lanes * CONV_ELEMS * 2)
                layer["rec"] = dev.create_buffer(2 * lanes * REC_ELEMS * 4)
            else:
                layer["q_norm"], layer["k_norm"] = up(w["q_norm"]), up(w["k_norm"])
                layer["keys"] = dev.create_buffer(lanes * stripe * 2)
                layer["values"] = dev.create_buffer(lanes * stripe * 2)
            self.layers.append(layer)
        rows = max(lanes, block_rows)
        mk = dev.create_buffer
        self.x = mk(rows * HIDDEN * 2)
        self.normed = mk(rows * HIDDEN * 2)
        self.proj = mk(rows * GDN_PROJ * 2)
        self.mixed = mk(rows * 4096 * 2)
        self.delta = mk(rows * HIDDEN * 2)
        self.qk, self.v, self.z, self.y = (mk(rows * 8192) for _ in range(4))
        self.q, self.gate = mk(rows * 8192), mk(rows * 8192)
        self.decay, self.beta = mk(rows * 128), mk(rows * 128)
        self.partials = mk(lanes * 16 * self.max_splits * 258 * 4)
        self.chunk = mk(((min(block_rows, 2048) + 63) // 64) * 32 * CHUNK_RECORD_BYTES)
        # blocks of few rows share each position tile's key walk between workgroups; the most
        # scratch any block up to block_rows needs is at one workgroup per compute unit
        self.flash_scratch = mk(max(
            [backend.flash_prefill_scratch_bytes(r, backend.flash_prefill_splits(r, 1 << 20, self.groups))
             for r in range(32, max(block_rows, 32) + 1, 32)] + [256]))
        self.logits = mk(rows * vocab * 2)
        self._write_tables()

    # ---- lane bookkeeping (decode_step.cpp:1044-1060) ----
    def _gdn_planes(self, lane):
        a, b = 2 * lane, 2 * lane + 1
        return (b, a) if self.swapped[lane] else (a, b)   # (in, out)

    def _write_tables(self):
        stripe = 2 * self.capacity * 256
        gdn = np.zeros(64, np.uint32)
        att = np.zeros(64, np.uint32)
        for lane in range(self.lanes):
            i, o = self._gdn_planes(lane)
            gdn[4 * lane:4 * lane + 4] = (i * CONV_ELEMS, o * CONV_ELEMS, i * REC_ELEMS, o * REC_ELEMS)
            att[4 * lane] = lane * stripe
            att[4 * lane + 1] = self.context[lane]
        for layer in self.layers:
            layer["table"].write(gdn if layer["kind"] == "G" else att)

    def install_lane_state(self, lane, context, states):
        """Writes a lane's whole state as it would stand after `context` tokens, without
        running them: states[i] holds layer i's arrays - {"conv": [3 x 8192] bf16, "rec":
        [32 x 128 x 128] fp32} for a Gated DeltaNet layer, {"keys", "values"}: [2 x capacity
        x 256] bf16 for an attention layer - the record body of the reference's state record
        (tools/native/decode_harness.cpp:339-460) in host arrays.  GDN planes go to the
        lane's live plane; the tables are rewritten."""
        assert 0 <= context < self.capacity and len(states) == len(self.layers)
        live, _ = self._gdn_planes(lane)
        stripe_bytes = 2 * self.capacity * 256 * 2
        for layer, state in zip(self.layers, states):
            if layer["kind"] == "G":
                layer["conv"].write(np.ascontiguousarray(state["conv"], np.uint16).reshape(-1),
                                    live * CONV_ELEMS * 2)
                layer["rec"].write(np.ascontiguousarray(state["rec"], np.float32).reshape(-1),
                                   live * REC_ELEMS * 4)
            else:
                layer["keys"].write(np.ascontiguousarray(state["keys"], np.uint16).reshape(-1),
                                    lane * stripe_bytes)
                layer["values"].write(np.ascontiguousarray(state["values"], np.uint16).reshape(-1),
                                      lane * stripe_bytes)
        self.context[lane] = context
        self._write_tables()

    # ---- shared steps ----
    def _dense(self, cb, x, w, out, rows, k, n):
        cb.encode(self.lib.pipeline("dense_bf16"), {0: x, 1: w, 2: out}, {3: rows, 4: k, 5: n},
                  ((n + 63) // 64, (rows + 15) // 16), (256,))
        cb.barrier()

    def _fused_wave(self, layer, rows):
        """Decode waves of several lanes over 4-bit weights take the norm in the prologue of
        the input projection and the residual sum in the epilogue of the output projection:
        two dispatches of a layer instead of three outside the attention family."""
        return self.fused_wave_steps and "in_q4" in layer and "out_q4" in layer and rows >= 2

    def _project_in(self, cb, layer, rows, block):
        """normed -> proj: the layer's input projection (a decode wave or a block); with
        _fused_wave x -> proj through the layer's input norm."""
        gated = layer["kind"] == "G"
        width = GDN_PROJ if gated else ATTN_PROJ
        if "in_q4" not in layer:
            self._dense(cb, self.normed, layer["w_in"], self.proj, rows, HIDDEN, width)
            return
        name = "gdn_project" if gated else "attn_project"
        fused = not block and self._fused_wave(layer, rows)
        bindings = {0: self.x if fused else self.normed}
        for index, matrix in enumerate(layer["in_q4"]):
            for part in range(3):
                bindings[1 + 3 * index + part] = matrix[part]
        out = 1 + 3 * len(layer["in_q4"])
        bindings[out] = self.proj
        if block:
            cb.encode(self.lib.pipeline(name + "_blk"), bindings, {out + 1: rows},
                      ((width + 3) // 4,), (128,))
        else:
            # several lanes: the matrix-unit form; one lane: the reference's own order
            suffix = "_rms_mfma_ms" if fused else "_mfma_ms" if rows >= 2 else "_ms"
            if fused:
                bindings[out + 3] = layer["input_norm"]
            cb.encode(self.lib.pipeline(name + suffix), bindings, {out + 1: rows, out + 2: 16},
                      ((width + 3) // 4, 1), (128,))
        cb.barrier()

    def _project_out(self, cb, layer, rows, block):
        """mixed -> delta: the projection back to the hidden width."""
        if "out_q4" not in layer:
            self._dense(cb, self.mixed, layer["w_out"], self.delta, rows, 4096, HIDDEN)
            return
        words, scales, biases = layer["out_q4"]
        bindings = {0: self.mixed, 1: words, 2: scales, 3: biases, 4: self.delta}
        if block:
            cb.encode(self.lib.pipeline("outproj_blk"), bindings, {5: rows, 6: 4096},
                      (HIDDEN // 2,), (64,))
        elif self._fused_wave(layer, rows):
            # x = bf16(x + bf16(projection)) in place
            cb.encode(self.lib.pipeline("gdn_outproj_residual_mfma_ms"),
                      {**bindings, 4: self.x, 8: self.x}, {5: rows, 6: HIDDEN, 7: 16},
                      (HIDDEN // 2, 1), (64,))
        else:
            name = "gdn_outproj_mfma_ms" if rows >= 2 else "gdn_outproj_ms"
            cb.encode(self.lib.pipeline(name), bindings, {5: rows, 6: HIDDEN, 7: 16},
                      (HIDDEN // 2, 1), (64,))
        cb.barrier()

    def _rms(self, cb, x, w, out, rows):
        cb.encode(self.lib.pipeline("rms_only_ms"), {0: x, 1: w, 2: out}, {3: HIDDEN, 4: HIDDEN},
                  (1, rows), (HIDDEN // 4,))
        cb.barrier()

    def _residual_and_norm(self, cb, rows, index):
        """x = bf16(x + delta) in place and normed = the norm layer `index + 1` (or the
        head) starts from."""
        following = (self.layers[index + 1]["input_norm"] if index + 1 < len(self.layers)
                     else self.final_norm)
        cb.encode(self.lib.pipeline("residual_rms_ms"),
                  {0: self.x, 1: self.delta, 2: self.x, 3: following, 4: self.normed},
                  {5: HIDDEN, 6: HIDDEN, 7: HIDDEN}, (1, rows), (HIDDEN // 4,))
        cb.barrier()

    def _head(self, cb, rows):
        """The final norm has been applied by the last layer's residual step."""
        self._dense(cb, self.normed, self.w_vocab, self.logits, rows, HIDDEN, self.vocab)

    def _split_flags(self, rows):
        """c9 of attention_decode_split_ms as the host runtime sets it: one or two lanes take
        their blocks in turn (bit 1); where the grid is larger than the chip and part of it
        holds no keys, the workgroups that do go first (bit 2)."""
        live = split_workgroups([c + 1 for c in self.context[:rows]], self.split_keys)
        grid = self.max_splits * 2 * rows
        # (bits 3..7: contiguous ranges are walked from a rotated starting block)
        return (2 if rows <= 2 else 8) | (4 if grid > live and grid > self.groups else 0)

    # ---- one token for every lane ----
    def record_token_wave(self, cb, with_head=True):
        """Records one decode step of all lanes; the lanes' inputs are rows of self.x.
        Call advance_token_wave() after the recording has been committed."""
        P, rows = self.lib.pipeline, self.lanes
        if not self._fused_wave(self.layers[0], rows):
            self._rms(cb, self.x, self.layers[0]["input_norm"], self.normed, rows)
        for index, layer in enumerate(self.layers):
            self._project_in(cb, layer, rows, block=False)
            if layer["kind"] == "G":
                cb.encode(P("gdn_decode_fused_ms"),
                          {0: self.proj, 1: layer["conv"], 2: layer["conv_w"], 3: layer["a_log"],
                           4: layer["dt_bias"], 5: layer["rec"], 6: layer["norm_w"], 7: self.mixed,
                           8: layer["table"]}, {9: GDN_PROJ, 10: 4096}, (32, rows), (512,))
            elif self.attention_form == "token":
                bind = {0: self.proj, 1: layer["q_norm"], 2: layer["k_norm"], 3: layer["keys"],
                        4: layer["values"], 5: layer["table"], 6: self.partials, 7: self.mixed}
                deepest = max(self.context[:rows])
                const = {8: self.capacity, 9: ATTN_PROJ, 10: 4096, 11: self.split_keys,
                         12: self.max_splits, 13: self._split_flags(rows),
                         14: -(-deepest // self.split_keys)}
                cb.encode(P("attention_decode_token_ms"), bind, const, (self.max_splits, 2, rows),
                          (256,))
                cb.barrier()
                cb.encode(P("attention_decode_token_finish_ms"), bind, const, (16, rows), (256,))
            else:
                cb.encode(P("attn_qk_rope_ms"),
                          {0: self.proj, 1: layer["q_norm"], 2: layer["k_norm"], 3: self.q, 4: self.gate,
                           5: layer["keys"], 6: layer["values"], 8: layer["table"]},
                          {7: self.capacity, 9: ATTN_PROJ, 10: 4096}, (18, rows), (256,))
                cb.barrier()
                cb.encode(P("attention_decode_split_ms"),
                          {0: self.q, 1: layer["keys"], 2: layer["values"], 3: layer["table"],
                           4: self.partials},
                          {5: self.capacity, 6: 4096, 7: self.split_keys, 8: self.max_splits,
                           9: self._split_flags(rows)},
                          (self.max_splits, 2, rows), (256,))
                cb.barrier()
                cb.encode(P("attention_decode_combine_ms"),
                          {0: self.partials, 1: self.gate, 2: layer["table"], 3: self.mixed},
                          {4: self.split_keys, 5: self.max_splits, 6: 4096, 7: 0, 8: self.capacity},
                          (16, rows), (256,))
            cb.barrier()
            self._project_out(cb, layer, rows, block=False)
            if not self._fused_wave(layer, rows):
                self._residual_and_norm(cb, rows, index)
            elif index + 1 == len(self.layers):
                self._rms(cb, self.x, self.final_norm, self.normed, rows)   # for the head
            elif not self._fused_wave(self.layers[index + 1], rows):
                self._rms(cb, self.x, self.layers[index + 1]["input_norm"], self.normed, rows)
        if with_head:
            self._head(cb, rows)

    def advance_token_wave(self):
        """The lanes' GDN planes swap and their contexts grow by one (decode_step.cpp:
        advance_decode_state); rewrites the state tables."""
        for lane in range(self.lanes):
            self.swapped[lane] = not self.swapped[lane]
            self.context[lane] += 1
        self._write_tables()

    # ---- a block of rows for one lane ----
    def record_prefill_block(self, cb, lane, rows, chunked=True, with_head=False):
        """Records `rows` new tokens of `lane` (inputs are rows of self.x) after its
        self.context[lane] cached ones.  Call advance_prefill_block(lane, rows) after."""
        assert 1 <= rows <= self.block_rows and self.context[lane] + rows <= self.capacity
        P = self.lib.pipeline
        base = self.context[lane]
        stripe_bytes = 2 * self.capacity * 256 * 2
        plane_in, plane_out = self._gdn_planes(lane)
        self._rms(cb, self.x, self.layers[0]["input_norm"], self.normed, rows)
        for index, layer in enumerate(self.layers):
            self._project_in(cb, layer, rows, block=True)
            if layer["kind"] == "G":
                conv_in = (layer["conv"], plane_in * CONV_ELEMS * 2)
                conv_out = (layer["conv"], plane_out * CONV_ELEMS * 2)
                rec_in = (layer["rec"], plane_in * REC_ELEMS * 4)
                rec_out = (layer["rec"], plane_out * REC_ELEMS * 4)
                cb.encode(P("gdn_conv_blk"),
                          {0: self.proj, 1: conv_in, 2: layer["conv_w"], 3: self.qk, 4: self.v,
                           5: self.z, 6: conv_out}, {7: rows}, (96, rows), (128,))
                cb.encode(P("gdn_gates_blk"),
                          {0: self.proj, 1: layer["a_log"], 2: layer["dt_bias"], 3: self.decay,
                           4: self.beta}, {5: rows}, (1, (rows + 3) // 4, 1), (32, 4, 1))
                cb.barrier()
                if chunked:
                    cb.encode(P("gdn_chunk_recurrence_blk"),
                              {0: self.qk, 1: self.v, 2: self.decay, 3: self.beta, 4: self.chunk,
                               5: rec_in, 6: self.y, 7: rec_out}, {8: rows}, (8, 32), (256,))
                else:
                    cb.encode(P("gdn_recurrence_gates_blk"),
                              {0: self.qk, 1: self.v, 2: self.decay, 3: layer["a_log"], 4: self.beta,
                               5: rec_in, 6: self.y, 7: rec_out}, {8: rows}, (1, 32, 32), (32, 4, 1))
                cb.barrier()
                cb.encode(P("gdn_gate_norm_blk"), {0: self.y, 1: self.z, 2: layer["norm_w"], 3: self.mixed},
                          {}, (32, rows), (128,))
            else:
                keys = (layer["keys"], lane * stripe_bytes)
                values = (layer["values"], lane * stripe_bytes)
                cb.encode(P("attn_qk_rope_blk"),
                          {0: self.proj, 1: layer["q_norm"], 2: layer["k_norm"], 3: self.q, 4: self.gate,
                           5: keys, 6: values}, {7: base, 8: self.capacity}, (18, rows), (256,))
                cb.barrier()
                splits = backend.flash_prefill_splits(rows, base + rows, self.groups)
                if splits > 1:
                    cb.encode(P("attention_flash_split_blk"),
                              {0: self.q, 1: keys, 2: values, 3: self.gate, 4: self.mixed,
                               9: self.flash_scratch},
                              {5: base + rows, 6: self.capacity, 7: rows, 8: base, 10: splits},
                              (16, (rows + 15) // 16), (256,))
                else:
                    cb.encode(P("attention_flash_v2_blk"),
                              {0: self.q, 1: keys, 2: values, 3: self.gate, 4: self.mixed},
                              {5: base + rows, 6: self.capacity, 7: rows, 8: base},
                              (16, (rows + 15) // 16), (256,))
            cb.barrier()
            self._project_out(cb, layer, rows, block=True)
            self._residual_and_norm(cb, rows, index)
        if with_head:
            self._head(cb, rows)

    def advance_prefill_block(self, lane, rows):
        self.swapped[lane] = not self.swapped[lane]
        self.context[lane] += rows
        self._write_tables()
