"""Stacked run of the hybrid 40-layer stub stack (3 GDN : 1 full attention,
hidden 2048, random bf16 dense projections in place of the Q4/MoE arithmetic) on
the GPU against the same stack evaluated with the CPU checker: block prefill of two
lanes with ragged lengths, then greedy decode waves of both lanes through the
pooled-state operators.  Judged by greedy argmax agreement on the final logits at
every step (where the checker's own top two are closer than two bf16 steps, the GPU may
pick the other of the two; the run continues with the checker's token).  The per-operator tolerance (max-abs 2e-2, mean-abs 2e-3) is held by
the single-layer tests; forty layers of bf16 re-rounding put the two evaluations of
the final logits (bf16, one step = 1.6e-2 at |x| in [2, 4)) a step or two apart, so
here the logits only have to stay within a loose sanity band."""
import numpy as np
import pytest

import oracle_lib as ol
from gpu_util import gpu, run

pytestmark = pytest.mark.gpu
o = ol.oracle
THREADS = 16
_WIDE = {}


class OracleLane:
    """One lane of the stack on the CPU checker."""

    def __init__(self, weights, capacity, vocab, fast_dense=False):
        """fast_dense: the stub's dense projections (which have no reference counterpart; the
        operator-level test holds the GPU kernel to tto_dense_bf16) are evaluated as a
        float32 matrix product by numpy instead of the checker's scalar loop, so that a
        stack of thousands of rows stays within a minute of CPU time."""
        self.w, self.cap, self.vocab = weights, capacity, vocab
        self.fast_dense = fast_dense
        self.context = 0
        self.state = []
        for lw in weights["layers"]:
            if lw["kind"] == "G":
                self.state.append({"conv": np.zeros(3 * 8192, np.uint16),
                                   "rec": np.zeros(32 * 128 * 128, np.float32)})
            else:
                self.state.append({"keys": np.zeros(2 * capacity * 256, np.uint16),
                                   "values": np.zeros(2 * capacity * 256, np.uint16)})

    def _dense(self, x, w, rows, k, n, out):
        if not self.fast_dense:
            o.tto_dense_bf16(x, w, rows, k, n, out, THREADS)
            return
        key = id(w)
        if key not in _WIDE:          # float32 copies of the weights, shared by the lanes
            _WIDE[key] = np.ascontiguousarray(ol.bf16_to_f32(w).reshape(n, k).T)
        out[:rows * n] = ol.f32_to_bf16((ol.bf16_to_f32(x[:rows * k]).reshape(rows, k) @
                                         _WIDE[key]).reshape(-1))

    def _project_in(self, lw, n, rows, width, p):
        if "in_q4" not in lw:
            self._dense(n, lw["w_in"], rows, 2048, width, p)
            return
        first = 0
        for words, scales, biases in lw["in_q4"]:
            out_rows = scales.size // 32
            o.tto_q4_project(n, 2048, rows, words, scales, biases, 2048, out_rows, p[first:], width,
                             THREADS)
            first += out_rows

    def block(self, x, rows):
        """Runs `rows` tokens (x: [rows*2048] bf16); returns logits of every row."""
        x = x.copy()
        for lw, st in zip(self.w["layers"], self.state):
            n = np.zeros(rows * 2048, np.uint16)
            o.tto_rms_only(x, lw["input_norm"], rows, 2048, n)
            if lw["kind"] == "G":
                p = np.zeros(rows * 12352, np.uint16)
                self._project_in(lw, n, rows, 12352, p)
                conv = np.zeros_like(st["conv"]); rec = np.zeros_like(st["rec"])
                a = np.zeros(rows * 4096, np.uint16)
                scratch = [np.zeros(rows * 4096, np.uint16) for _ in range(3)]
                o.tto_gdn_prefill(p, rows, st["conv"], lw["conv_w"], lw["a_log"], lw["dt_bias"],
                                  lw["norm_w"], st["rec"], conv, rec, a, *scratch, THREADS)
                st["conv"], st["rec"] = conv, rec
            else:
                p = np.zeros(rows * 9216, np.uint16)
                self._project_in(lw, n, rows, 9216, p)
                q = np.zeros(rows * 4096, np.uint16); g = np.zeros_like(q); a = np.zeros_like(q)
                sel = np.arange(rows, dtype=np.uint32)
                o.tto_attention_prefill(p, lw["q_norm"], lw["k_norm"], rows, self.context, self.cap,
                                        q, g, st["keys"], st["values"], sel, rows, a, THREADS)
            d = np.zeros(rows * 2048, np.uint16)
            if "out_q4" in lw:
                words, scales, biases = lw["out_q4"]
                o.tto_q4_project(a, 4096, rows, words, scales, biases, 4096, 2048, d, 2048, THREADS)
            else:
                self._dense(a, lw["w_out"], rows, 4096, 2048, d)
            o.tto_add_bf16(x, d, rows * 2048, x)
        self.context += rows
        n = np.zeros(rows * 2048, np.uint16)
        o.tto_rms_only(x, self.w["final_norm"], rows, 2048, n)
        logits = np.zeros(rows * self.vocab, np.uint16)
        self._dense(n, self.w["vocab"], rows, 2048, self.vocab, logits)
        return ol.bf16_to_f32(logits).reshape(rows, self.vocab)


def _compare(step, got, want):
    err = np.abs(got - want)
    top2 = np.sort(want)[-2:]
    print(f"[parity] {step}: logits max-abs {err.max():.3e} mean-abs {err.mean():.3e} "
          f"argmax {got.argmax()} / {want.argmax()} top-2 gap {top2[1] - top2[0]:.3e}", flush=True)
    assert np.isfinite(got).all()
    assert err.mean() <= 2e-2 * max(1.0, np.abs(want).max())
    # no single logit far off either: eight bf16 steps of the largest logit (the logits are
    # bf16 values of a 2048-term sum behind a stack of bf16 stages)
    step16 = 2.0 ** (np.floor(np.log2(max(np.abs(want).max(), 1e-30))) - 7)
    assert err.max() <= 8 * step16, f"{step}: a logit is off by {err.max():.3e} (bf16 step {step16:.3e})"
    if got.argmax() != want.argmax():
        # a tie within the noise of the run: the checker itself ranks the GPU's choice below its
        # own by no more than two bf16 steps of the winning logit, or by no more than the two
        # competing logits themselves are off (a gap smaller than their error decides nothing)
        margin = want.max() - want[got.argmax()]
        competing = err[got.argmax()] + err[want.argmax()]
        print(f"[parity] {step}: argmax differs on a margin of {margin:.3e} (bf16 step {step16:.3e}, "
              f"error of the two logits {competing:.3e})", flush=True)
        assert margin <= max(2 * step16, competing), step


@pytest.mark.parametrize("layers,quantized,fused", [(40, False, False), (12, True, False), (12, True, True)],
                         ids=["dense40", "q4x12", "q4x12-fused-steps"])
def test_stacked_prefill_and_greedy_decode_match_the_checker(layers, quantized, fused):
    """quantized: the projections are the affine 4-bit operators (block forms in the
    prefill, wave forms in the decode); fused: the decode waves take the norm in the
    prologue of the input projection and the residual sum in the output projection."""
    print(f"[case] {layers}-layer stub stack (quantized={quantized}): prefill 2 lanes + 3 greedy "
          "decode waves", flush=True)
    from tatara_amd import stack as S
    B, dev, queue, lib = gpu()
    vocab, capacity, lanes = 4096, 128, 2
    weights = S.make_weights(layers, vocab, 0x57AC, quantized=quantized)
    embed = weights["embed"].reshape(vocab, 2048)
    gpu_stack = S.StubStack(dev, lib, weights, lanes, capacity, vocab, block_rows=64, split_keys=64,
                            fused_wave_steps=fused)
    cpu_lanes = [OracleLane(weights, capacity, vocab) for _ in range(lanes)]
    rng = np.random.default_rng(5)
    prompts = [rng.integers(0, vocab, 24), rng.integers(0, vocab, 9)]
    tokens = []
    for lane, prompt in enumerate(prompts):
        rows = len(prompt)
        x = np.ascontiguousarray(embed[prompt]).reshape(-1)
        gpu_stack.x.write(x)
        cb = queue.create_command_buffer()
        cb.begin_compute_pass()
        gpu_stack.record_prefill_block(cb, lane, rows, chunked=True, with_head=True)
        cb.end_compute_pass()
        cb.commit().wait()
        gpu_stack.advance_prefill_block(lane, rows)
        got = ol.bf16_to_f32(gpu_stack.logits.read(np.uint16, rows * vocab)).reshape(rows, vocab)
        want = cpu_lanes[lane].block(x, rows)
        _compare(f"prefill lane {lane} last row", got[-1], want[-1])
        tokens.append(int(want[-1].argmax()))
    for step in range(3):
        x = np.ascontiguousarray(embed[tokens]).reshape(-1)
        gpu_stack.x.write(x)
        cb = queue.create_command_buffer()
        cb.begin_compute_pass()
        gpu_stack.record_token_wave(cb)
        cb.end_compute_pass()
        cb.commit().wait()
        gpu_stack.advance_token_wave()
        got = ol.bf16_to_f32(gpu_stack.logits.read(np.uint16, lanes * vocab)).reshape(lanes, vocab)
        for lane in range(lanes):
            want = cpu_lanes[lane].block(np.ascontiguousarray(x[lane * 2048:(lane + 1) * 2048]), 1)
            _compare(f"decode step {step} lane {lane}", got[lane], want[0])
            tokens[lane] = int(want[0].argmax())
    assert gpu_stack.context == [24 + 3, 9 + 3]


@pytest.mark.parametrize("rows,hidden", [(1, 2048), (5, 2048), (3, 256), (2, 4096)])
def test_residual_rms_operators(rows, hidden):
    """residual = bf16(a + b) and the row norm of the rounded sums, single row and
    strided rows, bit for bit against the checker (add, then rms_only)."""
    print(f"[case] residual_rms rows={rows} hidden={hidden}", flush=True)
    B, dev, queue, lib = gpu()
    a = ol.gaussian_bf16(0xA1 + rows, rows * hidden, 0.0, 2.0)
    b = ol.gaussian_bf16(0xB1 + rows, rows * hidden, 0.0, 0.5)
    w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(0xC1, hidden))
    sums = np.zeros(rows * hidden, np.uint16)
    o.tto_add_bf16(a, b, rows * hidden, sums)
    normed = np.zeros(rows * hidden, np.uint16)
    o.tto_rms_only(sums, w, rows, hidden, normed)
    b_a, b_b, b_w = dev.buffer_from(a), dev.buffer_from(b), dev.buffer_from(w)
    b_res, b_norm = dev.create_buffer(rows * hidden * 2), dev.create_buffer(rows * hidden * 2)

    def rec(cb):
        if rows == 1:
            cb.encode(lib.pipeline("residual_rms"), {0: b_a, 1: b_b, 2: b_res, 3: b_w, 4: b_norm}, {},
                      (1,), (hidden // 4,))
        else:
            cb.encode(lib.pipeline("residual_rms_ms"), {0: b_a, 1: b_b, 2: b_res, 3: b_w, 4: b_norm},
                      {5: hidden, 6: hidden, 7: hidden}, (1, rows), (hidden // 4,))
    run(rec)
    assert np.array_equal(b_res.read(np.uint16), sums)
    assert np.array_equal(b_norm.read(np.uint16), normed)
    # in place on the second operand, as the layer loop uses it
    def rec2(cb):
        cb.encode(lib.pipeline("residual_rms_ms"), {0: b_a, 1: b_b, 2: b_b, 3: b_w, 4: b_norm},
                  {5: hidden, 6: hidden, 7: hidden}, (1, rows), (hidden // 4,))
    run(rec2)
    assert np.array_equal(b_b.read(np.uint16), sums)
    assert np.array_equal(b_norm.read(np.uint16), normed)


@pytest.mark.parametrize("rows,hidden", [(1, 2048), (4, 2048), (7, 256), (2, 4096)])
def test_rms_only_operators_bit_for_bit(rows, hidden):
    """rms_only (one row) and rms_only_ms (strided rows, strides wider than the row):
    every bf16 output is the checker's bit pattern."""
    print(f"[case] rms_only rows={rows} hidden={hidden}", flush=True)
    B, dev, queue, lib = gpu()
    x = ol.gaussian_bf16(0xD1 + rows, rows * hidden, 0.0, 3.0)
    w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(0xD2, hidden))
    want = np.zeros(rows * hidden, np.uint16)
    o.tto_rms_only(x, w, rows, hidden, want)
    b_w = dev.buffer_from(w)
    if rows == 1:
        b_x, b_o = dev.buffer_from(x), dev.create_buffer(hidden * 2)
        run(lambda cb: cb.encode(lib.pipeline("rms_only"), {0: b_x, 1: b_w, 2: b_o}, {}, (1,),
                                 (hidden // 4,)))
        assert np.array_equal(b_o.read(np.uint16), want)
        return
    in_stride, out_stride = hidden + 64, hidden + 128
    slab = np.full((rows, in_stride), 0x7FC0, np.uint16)        # NaN between the rows
    slab[:, :hidden] = x.reshape(rows, hidden)
    b_x = dev.buffer_from(slab.reshape(-1))
    b_o = dev.create_buffer(rows * out_stride * 2)
    run(lambda cb: cb.encode(lib.pipeline("rms_only_ms"), {0: b_x, 1: b_w, 2: b_o},
                             {3: in_stride, 4: out_stride}, (1, rows), (hidden // 4,)))
    got = b_o.read(np.uint16).reshape(rows, out_stride)
    assert np.array_equal(got[:, :hidden].reshape(-1), want)
    assert not got[:, hidden:].any()                             # nothing written past a row


def test_norm_and_residual_sum_over_every_bf16_value():
    """rms_only_ms, residual_rms_ms and add_bf16 on all 65536 bf16 bit patterns (non-finite
    ones replaced by zero), ordered by magnitude so that a row of 2048 holds neighbouring
    binades: rows of subnormals (flushed on the way in), rows that round into and out of the
    subnormal range, rows whose squares overflow."""
    print("[case] rms_only_ms / residual_rms_ms / add_bf16 over every bf16 value", flush=True)
    B, dev, queue, lib = gpu()
    hidden, rows = 2048, 32
    patterns = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    patterns[(patterns & 0x7F80) == 0x7F80] = 0
    order = np.argsort(patterns & 0x7FFF, kind="stable")
    x = np.ascontiguousarray(patterns[order])
    # the second operand: the same magnitudes one binade away and in another order of signs
    other = np.ascontiguousarray(np.roll(x, 193) ^ np.uint16(0x8000))
    w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(0xE2, hidden))
    want_norm = np.zeros(rows * hidden, np.uint16)
    o.tto_rms_only(x, w, rows, hidden, want_norm)
    sums = np.zeros(rows * hidden, np.uint16)
    o.tto_add_bf16(x, other, rows * hidden, sums)
    want_sum_norm = np.zeros(rows * hidden, np.uint16)
    o.tto_rms_only(sums, w, rows, hidden, want_sum_norm)
    b_x, b_y, b_w = dev.buffer_from(x), dev.buffer_from(other), dev.buffer_from(w)
    b_norm, b_res, b_res_norm, b_add = (dev.create_buffer(rows * hidden * 2) for _ in range(4))

    def rec(cb):
        cb.encode(lib.pipeline("rms_only_ms"), {0: b_x, 1: b_w, 2: b_norm}, {3: hidden, 4: hidden},
                  (1, rows), (hidden // 4,))
        cb.encode(lib.pipeline("residual_rms_ms"), {0: b_x, 1: b_y, 2: b_res, 3: b_w, 4: b_res_norm},
                  {5: hidden, 6: hidden, 7: hidden}, (1, rows), (hidden // 4,))
        cb.encode(lib.pipeline("add_bf16"), {0: b_x, 1: b_y, 2: b_add}, {3: rows * hidden},
                  ((rows * hidden + 255) // 256,), (256,))
    run(rec)
    for what, got, want in (("rms_only_ms", b_norm, want_norm), ("residual", b_res, sums),
                            ("residual_rms_ms norm", b_res_norm, want_sum_norm),
                            ("add_bf16", b_add, sums)):
        g = got.read(np.uint16)
        differ = np.flatnonzero(g != want)
        assert differ.size == 0, (f"{what}: {differ.size} of 65536 differ, first at input "
                                  f"{x[differ[0]]:#06x}: got {g[differ[0]]:#06x} want "
                                  f"{want[differ[0]]:#06x}")


@pytest.mark.parametrize("rows,in_dim,out_dim", [(1, 2048, 9216), (4, 2048, 12352), (16, 4096, 2048),
                                                 (37, 2048, 4096), (3, 64, 70), (2, 2048, 70),
                                                 (13, 4096, 24)])
def test_dense_bf16_operator(rows, in_dim, out_dim):
    """The stub stack's dense projection against the checker (fp32 dot in ascending
    order, one bf16 rounding); the matrix unit sums in another order, so the bar is the
    path's output tolerance scaled to the magnitude of the sums, and most outputs are
    the checker's bit pattern."""
    print(f"[case] dense_bf16 rows={rows} in={in_dim} out={out_dim}", flush=True)
    B, dev, queue, lib = gpu()
    x = ol.gaussian_bf16(0xE1 + rows, rows * in_dim)
    w = ol.gaussian_bf16(0xE2 + rows, out_dim * in_dim, 0.0, 1.0 / np.sqrt(in_dim))
    want = np.zeros(rows * out_dim, np.uint16)
    o.tto_dense_bf16(x, w, rows, in_dim, out_dim, want, THREADS)
    b_x, b_w = dev.buffer_from(x), dev.buffer_from(w)
    b_o = dev.create_buffer(rows * out_dim * 2)
    run(lambda cb: cb.encode(lib.pipeline("dense_bf16"), {0: b_x, 1: b_w, 2: b_o},
                             {3: rows, 4: in_dim, 5: out_dim},
                             ((out_dim + 63) // 64, (rows + 15) // 16), (256,)))
    got = b_o.read(np.uint16)
    from gpu_util import check_bf16
    check_bf16(got, want, f"dense_bf16 {rows}x{in_dim}x{out_dim}", ulps=1)
    assert np.mean(got == want) > 0.97


def _dense_block_case(rows, in_dim, out_dim, sample_rows, seed):
    """dense_bf16 on a block of rows; the checker evaluates `sample_rows` of them."""
    B, dev, queue, lib = gpu()
    x = ol.gaussian_bf16(seed, rows * in_dim).reshape(rows, in_dim)
    w = ol.gaussian_bf16(seed + 1, out_dim * in_dim, 0.0, 1.0 / np.sqrt(in_dim))
    b_x, b_w = dev.buffer_from(x), dev.buffer_from(w)
    b_o = dev.create_buffer(rows * out_dim * 2)
    b_o.write(np.full(rows * out_dim, 0x7FC0, np.uint16))       # NaN wherever nothing is stored
    run(lambda cb: cb.encode(lib.pipeline("dense_bf16"), {0: b_x, 1: b_w, 2: b_o},
                             {3: rows, 4: in_dim, 5: out_dim},
                             ((out_dim + 63) // 64, (rows + 15) // 16), (256,)))
    got = b_o.read(np.uint16).reshape(rows, out_dim)
    sample = np.asarray(sorted(set(sample_rows)))
    want = np.zeros(sample.size * out_dim, np.uint16)
    o.tto_dense_bf16(np.ascontiguousarray(x[sample]).reshape(-1), w, sample.size, in_dim, out_dim,
                     want, THREADS)
    from gpu_util import check_bf16
    check_bf16(got[sample].reshape(-1), want, f"dense_bf16 block {rows}x{in_dim}x{out_dim}", ulps=1)
    assert np.mean(got[sample].reshape(-1) == want) > 0.97
    return got


@pytest.mark.parametrize("rows,in_dim,out_dim", [
    (65, 64, 70),          # the smallest block: two steps, one tile mostly padding, narrow stores
    (257, 2048, 300),      # one row and 44 outputs into a second tile either way
    (300, 4096, 2048),     # the output projection's shape
    (1000, 2048, 515),     # an odd output width: rows are not 8-byte aligned
    (513, 128, 256),       # four steps: the walk's lead-in and lead-out only
    (640, 192, 1024),      # six steps: one round of the steady loop
], ids=["65x64x70", "257x2048x300", "300x4096x2048", "1000x2048x515", "513x128x256", "640x192x1024"])
def test_dense_bf16_block_kernel(rows, in_dim, out_dim):
    """Blocks of more than 64 rows take the LDS-staged 256 x 256 kernel: every row against the
    checker, partial tiles either way, every length of the K walk's lead-in and lead-out."""
    print(f"[case] dense_bf16 block rows={rows} in={in_dim} out={out_dim}", flush=True)
    _dense_block_case(rows, in_dim, out_dim, range(rows), 0xB10C + rows)


def test_dense_bf16_block_kernel_at_the_prefill_shape():
    """16384 rows x 2048 -> 9216 (the attention input projection of a 16384-row block): 2304
    tiles on one workgroup per compute unit, nine tiles each.  The checker evaluates every
    251st row (66 rows, each at another position inside its tile) and the last rows."""
    rows, in_dim, out_dim = 16384, 2048, 9216
    print(f"[case] dense_bf16 block rows={rows} in={in_dim} out={out_dim}, sampled rows", flush=True)
    sample = list(range(0, rows, 251)) + [rows - 2, rows - 1]
    assert len({r % 256 for r in range(0, rows, 251)}) > 60
    got = _dense_block_case(rows, in_dim, out_dim, sample, 0xB16B)
    assert not np.any((got & 0x7F80) == 0x7F80), "an output was not stored"


def test_add_bf16_operator_bit_for_bit():
    print("[case] add_bf16", flush=True)
    B, dev, queue, lib = gpu()
    n = 5 * 2048 + 3
    a = ol.gaussian_bf16(0xF1, n, 0.0, 2.0); b = ol.gaussian_bf16(0xF2, n)
    want = np.zeros(n, np.uint16)
    o.tto_add_bf16(a, b, n, want)
    b_a, b_b = dev.buffer_from(a), dev.buffer_from(b)
    run(lambda cb: cb.encode(lib.pipeline("add_bf16"), {0: b_a, 1: b_b, 2: b_a}, {3: n},
                             ((n + 255) // 256,), (256,)))
    assert np.array_equal(b_a.read(np.uint16), want)


_DEPTH = {}


def _depth_reference(layers, vocab, capacity, prompts, waves):
    """The checker's side of the run at depth, evaluated once for both attention forms:
    last-row logits of every lane's prefill and every lane's logits of each greedy wave."""
    from tatara_amd import stack as S
    key = (layers, vocab, capacity, tuple(len(p) for p in prompts), waves)
    if key in _DEPTH:
        return _DEPTH[key]
    weights = S.make_weights(layers, vocab, 0xD3E9)
    embed = weights["embed"].reshape(vocab, 2048)
    lanes = [OracleLane(weights, capacity, vocab, fast_dense=True) for _ in prompts]
    prefill, tokens = [], []
    for lane, prompt in enumerate(prompts):
        print(f"[checker] prefill lane {lane}: {len(prompt)} rows", flush=True)
        want = lanes[lane].block(np.ascontiguousarray(embed[prompt]).reshape(-1), len(prompt))
        prefill.append(want[-1])
        tokens.append(int(want[-1].argmax()))
    steps = []
    for step in range(waves):
        print(f"[checker] greedy wave {step}", flush=True)
        row = [lanes[lane].block(np.ascontiguousarray(embed[tokens[lane]]), 1)[0]
               for lane in range(len(prompts))]
        steps.append((list(tokens), row))
        tokens = [int(r.argmax()) for r in row]
    _DEPTH[key] = (weights, prefill, steps)
    return _DEPTH[key]


@pytest.mark.parametrize("form", ["three", "token"])
def test_stacked_run_at_depth_four_ragged_lanes(form):
    """Config 5 at depth: 12 layers (G,G,G,A x 3), four lanes with prompts of 1024, 640,
    384 and 160 tokens prefilled in blocks of 512 rows (two blocks for the longer ones), then
    three greedy token waves of all four lanes through the pooled-state operators, with the
    split size the stack chooses for itself, as rope + split-K + combine (form "three") or
    with the rope inside the walk and the token folded in by the finishing dispatch (form
    "token").  Every greedy token must be the checker's (ties within two bf16 steps of the
    winning logit aside, as in the shallow run)."""
    print(f"[case] stacked run at depth, attention form {form}", flush=True)
    from tatara_amd import stack as S
    B, dev, queue, lib = gpu()
    layers, vocab, capacity, block_rows, waves = 12, 4096, 1280, 512, 3
    rng = np.random.default_rng(17)
    prompts = [rng.integers(0, vocab, n) for n in (1024, 640, 384, 160)]
    weights, want_prefill, want_steps = _depth_reference(layers, vocab, capacity, prompts, waves)
    embed = weights["embed"].reshape(vocab, 2048)
    stack = S.StubStack(dev, lib, weights, len(prompts), capacity, vocab, block_rows=block_rows,
                        attention_form=form)
    assert stack.split_keys == S.choose_split_keys([capacity] * len(prompts))
    for lane, prompt in enumerate(prompts):
        for first in range(0, len(prompt), block_rows):
            rows = min(block_rows, len(prompt) - first)
            stack.x.write(np.ascontiguousarray(embed[prompt[first:first + rows]]).reshape(-1))
            cb = queue.create_command_buffer()
            cb.begin_compute_pass()
            stack.record_prefill_block(cb, lane, rows, chunked=True, with_head=True)
            cb.end_compute_pass()
            cb.commit().wait()
            stack.advance_prefill_block(lane, rows)
        got = ol.bf16_to_f32(stack.logits.read(np.uint16, rows * vocab)).reshape(rows, vocab)
        _compare(f"depth prefill lane {lane} ({len(prompt)} rows) last row", got[-1],
                 want_prefill[lane])
    assert stack.context == [len(p) for p in prompts]
    for step, (tokens, want_rows) in enumerate(want_steps):
        stack.x.write(np.ascontiguousarray(embed[tokens]).reshape(-1))
        cb = queue.create_command_buffer()
        cb.begin_compute_pass()
        stack.record_token_wave(cb)
        cb.end_compute_pass()
        cb.commit().wait()
        stack.advance_token_wave()
        got = ol.bf16_to_f32(stack.logits.read(np.uint16, len(prompts) * vocab)).reshape(-1, vocab)
        for lane in range(len(prompts)):
            _compare(f"depth wave {step} lane {lane} (context {stack.context[lane] - 1})",
                     got[lane], want_rows[lane])


# ---- token waves over deep, installed state -----------------------------------------------

_DEEP = {}


def _deep_states(weights, capacity, contexts, seed):
    """Synthetic lane states as they might stand after `contexts[lane]` tokens: caches of
    N(0, 1) keys and values up to the context (NaN beyond it: a row past the context must
    never be read), conv windows N(0, 0.5), recurrent states N(0, 0.02).  A generator of
    (lane, states): the same seeds give the same arrays for the checker and for the GPU."""
    for lane, context in enumerate(contexts):
        rng = np.random.default_rng(seed + 101 * lane)
        states = []
        for lw in weights["layers"]:
            if lw["kind"] == "G":
                conv = (rng.standard_normal(3 * 8192, dtype=np.float32) * np.float32(0.5))
                rec = rng.standard_normal(32 * 128 * 128, dtype=np.float32) * np.float32(0.02)
                states.append({"conv": ol.f32_to_bf16(conv), "rec": rec})
            else:
                def cache():
                    c = np.full((2, capacity, 256), 0x7FC0, np.uint16)
                    c[:, :context] = ol.f32_to_bf16(
                        rng.standard_normal(2 * context * 256, dtype=np.float32)).reshape(2, context, 256)
                    return c.reshape(-1)
                states.append({"keys": cache(), "values": cache()})
        yield lane, states


def _deep_reference(layers, vocab, capacity, contexts, waves, seed):
    """The checker's side of greedy token waves over installed deep state, evaluated once
    for both attention forms.  Its dense projections are numpy float32 products (another
    summation order than tto_dense_bf16, which the operator-level test holds the kernel to);
    everything of the attention family is the checker's own arithmetic."""
    from tatara_amd import stack as S
    key = (layers, vocab, capacity, tuple(contexts), waves, seed)
    if key in _DEEP:
        return _DEEP[key]
    weights = S.make_weights(layers, vocab, seed)
    embed = weights["embed"].reshape(vocab, 2048)
    lanes = []
    for lane, states in _deep_states(weights, capacity, contexts, seed):
        checker = OracleLane(weights, capacity, vocab, fast_dense=True)
        checker.state = states
        checker.context = contexts[lane]
        lanes.append(checker)
    tokens = [int(t) for t in np.random.default_rng(seed ^ 0x70C).integers(0, vocab, len(contexts))]
    steps = []
    for step in range(waves):
        print(f"[checker] deep greedy wave {step}", flush=True)
        row = [lanes[lane].block(np.ascontiguousarray(embed[tokens[lane]]), 1)[0]
               for lane in range(len(contexts))]
        steps.append((list(tokens), row))
        tokens = [int(r.argmax()) for r in row]
    _DEEP[key] = (weights, steps)
    return _DEEP[key]


def _deep_waves(form, layers, capacity, contexts, seed, waves=2, vocab=4096):
    from tatara_amd import stack as S
    B, dev, queue, lib = gpu()
    weights, want_steps = _deep_reference(layers, vocab, capacity, contexts, waves, seed)
    embed = weights["embed"].reshape(vocab, 2048)
    stack = S.StubStack(dev, lib, weights, len(contexts), capacity, vocab, block_rows=64,
                        attention_form=form)
    print(f"[plan] {len(contexts)} lanes, capacity {capacity}: {stack.split_keys} keys per "
          f"workgroup, {stack.max_splits} splits", flush=True)
    assert stack.split_keys == S.choose_split_keys([capacity] * len(contexts), dev.compute_units)
    for lane, states in _deep_states(weights, capacity, contexts, seed):
        stack.install_lane_state(lane, contexts[lane], states)
    for step, (tokens, want_rows) in enumerate(want_steps):
        stack.x.write(np.ascontiguousarray(embed[tokens]).reshape(-1))
        cb = queue.create_command_buffer()
        cb.begin_compute_pass()
        stack.record_token_wave(cb)
        cb.end_compute_pass()
        cb.commit().wait()
        stack.advance_token_wave()
        got = ol.bf16_to_f32(stack.logits.read(np.uint16, len(contexts) * vocab)).reshape(-1, vocab)
        for lane in range(len(contexts)):
            _compare(f"deep wave {step} lane {lane} (context {stack.context[lane] - 1}, {form})",
                     got[lane], want_rows[lane])


@pytest.mark.parametrize("form", ["three", "token"])
def test_token_waves_at_32k_depth_forty_layers(form):
    """Config 5 where the sweep times it: all 40 layers, four ragged lanes around 32k keys
    (32767 - the last position but one of the cache -, 30000, 24576, 8191), their state
    installed directly, two greedy token waves through state table, split planner (the split
    the stack picks for the capacity, with whatever dispatch order and block order follow
    from it) and both attention forms.  Every greedy token must be the checker's."""
    print(f"[case] 40 layers, 4 ragged lanes at 32k depth, form {form}", flush=True)
    _deep_waves(form, 40, 32768 + 64, [32767, 30000, 24576, 8191], 0xDEE9)


@pytest.mark.parametrize("form", ["three", "token"])
def test_token_waves_one_lane_at_100k_depth(form):
    """One lane of 100000 cached keys through 12 layers (three attention layers): the deep
    single-lane shape of config 3 inside the stack, blocks dealt in turn."""
    print(f"[case] 12 layers, 1 lane at 100k depth, form {form}", flush=True)
    _deep_waves(form, 12, 100096, [100000], 0xDEEA)
