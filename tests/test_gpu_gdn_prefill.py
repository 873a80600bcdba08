"""Gated DeltaNet block prefill on the GPU against the CPU checker, through the
C ABI: the block operators one at a time (conv, gates, register-loop recurrence,
gate-norm) and the chunked evaluation of the recurrence (64-token chunks on
MFMA) against the token-by-token checker.

Tolerance for the chunked path: its products run in bf16 on MFMA with fp32
accumulation, so it is held to the path's stated bar (max-abs 2e-2, mean-abs
2e-3 on outputs); the recurrent state is compared in fp32 with the same
absolute bar scaled to the state's magnitude."""
import numpy as np
import pytest

import oracle_lib as ol
from gpu_util import check_bf16, check_f32, gpu, run

pytestmark = pytest.mark.gpu
o = ol.oracle
STATE = 32 * 128 * 128


def _weights():
    conv_w = ol.gaussian_bf16(0x77, 4 * 8192, 0.0, 0.5)
    a_log = ol.f32_to_bf16(ol.uniform_f32(0x78, 32, -4.0, -2.5))
    dt_bias = ol.gaussian_bf16(0x79, 32, 0.0, 0.3)
    norm_w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(0x7A, 128))
    return conv_w, a_log, dt_bias, norm_w


def _block(rows, seed):
    proj = ol.gaussian_bf16(seed, rows * 12352, 0.0, 0.5).reshape(rows, 12352)
    proj[:, 12288:12320] = ol.gaussian_bf16(seed + 1, rows * 32).reshape(rows, 32)
    conv_state = ol.gaussian_bf16(seed + 2, 3 * 8192, 0.0, 0.5)
    state = ol.gaussian_f32(seed + 3, STATE, 0.0, 0.02)
    return np.ascontiguousarray(proj), conv_state, state


def _oracle_block(proj, conv_state, state, weights, rows):
    conv_w, a_log, dt_bias, norm_w = weights
    out = {
        "conv": np.zeros(3 * 8192, np.uint16), "state": np.zeros(STATE, np.float32),
        "gated": np.zeros(rows * 4096, np.uint16), "qk": np.zeros(rows * 4096, np.uint16),
        "value": np.zeros(rows * 4096, np.uint16), "y": np.zeros(rows * 4096, np.uint16),
    }
    o.tto_gdn_prefill(proj.reshape(-1), rows, conv_state, conv_w, a_log, dt_bias, norm_w, state,
                      out["conv"], out["state"], out["gated"], out["qk"], out["value"], out["y"], 8)
    decay = np.zeros((rows, 32), np.float32); beta = np.zeros((rows, 32), np.float32)
    for r in range(rows):
        o.tto_gdn_gates(proj[r], a_log, dt_bias, decay[r], beta[r])
    out["decay"], out["beta"] = decay, beta
    return out


def _encode_front(cb, lib, bufs, rows):
    cb.encode(lib.pipeline("gdn_conv_blk"),
              {0: bufs["proj"], 1: bufs["conv_in"], 2: bufs["conv_w"], 3: bufs["qk"],
               4: bufs["value"], 5: bufs["z"], 6: bufs["conv_out"]}, {7: rows},
              (96, rows, 1), (128, 1, 1))
    cb.encode(lib.pipeline("gdn_gates_blk"),
              {0: bufs["proj"], 1: bufs["a_log"], 2: bufs["dt_bias"], 3: bufs["decay"],
               4: bufs["beta"]}, {5: rows}, (1, (rows + 3) // 4, 1), (32, 4, 1))
    cb.barrier()


def _encode_gate_norm(cb, lib, bufs, rows):
    cb.barrier()
    cb.encode(lib.pipeline("gdn_gate_norm_blk"),
              {0: bufs["y"], 1: bufs["z"], 2: bufs["norm_w"], 3: bufs["gated"]}, {},
              (32, rows, 1), (128, 1, 1))


def _buffers(dev, proj, conv_state, state, weights, rows):
    conv_w, a_log, dt_bias, norm_w = weights
    chunks = (rows + 63) // 64
    return {
        "proj": dev.buffer_from(proj.reshape(-1)), "conv_in": dev.buffer_from(conv_state),
        "conv_out": dev.create_buffer(3 * 8192 * 2), "conv_w": dev.buffer_from(conv_w),
        "a_log": dev.buffer_from(a_log), "dt_bias": dev.buffer_from(dt_bias),
        "norm_w": dev.buffer_from(norm_w), "qk": dev.create_buffer(rows * 8192),
        "value": dev.create_buffer(rows * 8192), "z": dev.create_buffer(rows * 8192),
        "y": dev.create_buffer(rows * 8192), "gated": dev.create_buffer(rows * 8192),
        "decay": dev.create_buffer(rows * 128), "beta": dev.create_buffer(rows * 128),
        "state_in": dev.buffer_from(state), "state_out": dev.create_buffer(STATE * 4),
        "chunk": dev.create_buffer(chunks * 32 * 115712),
    }


@pytest.mark.parametrize("hoisted", [True, False])
def test_block_operators_register_loop(hoisted):
    """conv / gates / register-loop recurrence / gate-norm over a 37-row block;
    every stage is compared with the checker's intermediates."""
    rows = 37
    print(f"[case] gdn block operators rows={rows} hoisted={hoisted}", flush=True)
    B, dev, queue, lib = gpu()
    weights = _weights()
    proj, conv_state, state = _block(rows, 0x5101)
    ref = _oracle_block(proj, conv_state, state, weights, rows)
    bufs = _buffers(dev, proj, conv_state, state, weights, rows)

    def rec(cb):
        _encode_front(cb, lib, bufs, rows)
        if hoisted:
            cb.encode(lib.pipeline("gdn_recurrence_gates_blk"),
                      {0: bufs["qk"], 1: bufs["value"], 2: bufs["decay"], 3: bufs["a_log"],
                       4: bufs["beta"], 5: bufs["state_in"], 6: bufs["y"], 7: bufs["state_out"]},
                      {8: rows}, (1, 32, 32), (32, 4, 1))
        else:
            cb.encode(lib.pipeline("gdn_recurrence_blk"),
                      {0: bufs["qk"], 1: bufs["value"], 2: bufs["proj"], 3: bufs["a_log"],
                       4: bufs["dt_bias"], 5: bufs["state_in"], 6: bufs["y"],
                       7: bufs["state_out"]}, {8: rows}, (1, 32, 32), (32, 4, 1))
        _encode_gate_norm(cb, lib, bufs, rows)
    run(rec)
    check_bf16(bufs["qk"].read(np.uint16), ref["qk"], "qk")
    check_bf16(bufs["value"].read(np.uint16), ref["value"], "value")
    assert np.array_equal(bufs["conv_out"].read(np.uint16), ref["conv"])
    check_f32(bufs["decay"].read(np.float32), ref["decay"].reshape(-1), "decay", 1e-5, 1e-6)
    check_f32(bufs["beta"].read(np.float32), ref["beta"].reshape(-1), "beta", 1e-5, 1e-6)
    check_bf16(bufs["y"].read(np.uint16), ref["y"], "y")
    check_f32(bufs["state_out"].read(np.float32), ref["state"], "state", 2e-3, 2e-5)
    check_bf16(bufs["gated"].read(np.uint16), ref["gated"], "gated")


@pytest.mark.parametrize("rows", [1, 15, 16, 17, 33, 130])
def test_element_wise_block_kernels_bit_for_bit(rows):
    """conv / L2 norm / z copy / conv-state shift and the gate-norm of a block, at row
    counts around the 16- and 8-row groups the block kernels walk: the vectorised
    kernels keep the checker's summation order, so every bf16 output is the same
    bit pattern.  The gate-norm is fed the checker's y so that only it is tested."""
    print(f"[case] gdn element-wise block kernels rows={rows}", flush=True)
    B, dev, queue, lib = gpu()
    weights = _weights()
    proj, conv_state, state = _block(rows, 0x5300 + rows)
    ref = _oracle_block(proj, conv_state, state, weights, rows)
    bufs = _buffers(dev, proj, conv_state, state, weights, rows)
    bufs["y"] = dev.buffer_from(ref["y"])

    def rec(cb):
        _encode_front(cb, lib, bufs, rows)
        _encode_gate_norm(cb, lib, bufs, rows)
    run(rec)
    assert np.array_equal(bufs["qk"].read(np.uint16), ref["qk"])
    assert np.array_equal(bufs["value"].read(np.uint16), ref["value"])
    assert np.array_equal(bufs["z"].read(np.uint16).reshape(rows, 4096), proj[:, 8192:12288])
    assert np.array_equal(bufs["conv_out"].read(np.uint16), ref["conv"])
    assert np.array_equal(bufs["gated"].read(np.uint16), ref["gated"])


def test_activation_of_every_bf16_value_bit_for_bit():
    """conv + SiLU of all 65536 bf16 bit patterns (the non-finite ones replaced by zero):
    16 rows whose 4096 value channels carry the patterns, taps (0, 0, 0, 1) and an empty
    window, so a channel's convolution is its input.  Pins the kernels' bf16 rounding step
    and their reciprocal-instruction sigmoid to the checker's division over the whole
    range, not only where random inputs fall."""
    rows = 16
    print("[case] gdn conv + SiLU over every bf16 value", flush=True)
    B, dev, queue, lib = gpu()
    _, a_log, dt_bias, norm_w = _weights()
    patterns = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    patterns[(patterns & 0x7F80) == 0x7F80] = 0
    proj = np.zeros((rows, 12352), np.uint16)
    proj[:, 4096:8192] = patterns.reshape(rows, 4096)
    conv_w = np.zeros((8192, 4), np.uint16)
    conv_w[:, 3] = 0x3F80
    weights = (conv_w.reshape(-1), a_log, dt_bias, norm_w)
    conv_state = np.zeros(3 * 8192, np.uint16)
    state = np.zeros(STATE, np.float32)
    ref = _oracle_block(proj, conv_state, state, weights, rows)
    bufs = _buffers(dev, proj, conv_state, state, weights, rows)
    run(lambda cb: _encode_front(cb, lib, bufs, rows))
    got = bufs["value"].read(np.uint16)
    differ = np.flatnonzero(got != ref["value"])
    assert differ.size == 0, (f"{differ.size} of 65536 activations differ, first: input "
                              f"{patterns[differ[0]]:#06x} got {got[differ[0]]:#06x} "
                              f"want {ref['value'][differ[0]]:#06x}")
    assert np.array_equal(bufs["conv_out"].read(np.uint16), ref["conv"])
    # the decode operator on the last row's window: the same activations bit for bit
    last = rows - 1
    b_qk, b_v, b_z = (dev.create_buffer(8192) for _ in range(3))
    b_conv_in = dev.buffer_from(np.concatenate([proj[last - 3 + t, :8192] for t in range(3)]))
    b_conv_out = dev.create_buffer(3 * 8192 * 2)
    b_row = dev.buffer_from(proj[last])

    def rec(cb):
        cb.encode(lib.pipeline("gdn_prepare"),
                  {0: b_row, 1: b_conv_in, 2: bufs["conv_w"], 3: b_qk, 4: b_v, 5: b_z,
                   6: b_conv_out}, {}, (96,), (128,))
    run(rec)
    assert np.array_equal(b_v.read(np.uint16), ref["value"].reshape(rows, 4096)[last])


def test_output_gate_of_every_bf16_value_bit_for_bit():
    """The gate-norm's SiLU(z) over all 65536 bf16 bit patterns of z (non-finite ones replaced
    by zero) on rows of seeded y: the fp32 sigmoid with its |z| branch, the product and the
    final rounding against the checker, for the block operator and the decode operator."""
    rows = 16
    print("[case] gdn gate-norm over every bf16 gate value", flush=True)
    B, dev, queue, lib = gpu()
    _, _, _, norm_w = _weights()
    patterns = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    patterns[(patterns & 0x7F80) == 0x7F80] = 0
    z = patterns.reshape(rows, 4096)
    y = ol.gaussian_bf16(0x6E01, rows * 4096).reshape(rows, 4096)
    want = np.zeros((rows, 4096), np.uint16)
    for r in range(rows):
        o.tto_gdn_gate_norm(y[r], z[r], norm_w, 32, want[r])
    b_y, b_z, b_w = dev.buffer_from(y), dev.buffer_from(z), dev.buffer_from(norm_w)
    b_blk, b_one = dev.create_buffer(rows * 8192), dev.create_buffer(8192)

    def rec(cb):
        cb.encode(lib.pipeline("gdn_gate_norm_blk"), {0: b_y, 1: b_z, 2: b_w, 3: b_blk}, {},
                  (32, rows, 1), (128, 1, 1))
        cb.encode(lib.pipeline("gdn_gate_norm"), {0: (b_y, 5 * 8192), 1: (b_z, 5 * 8192), 2: b_w,
                                                  3: b_one}, {}, (32,), (128,))
    run(rec)
    got = b_blk.read(np.uint16).reshape(rows, 4096)
    differ = np.argwhere(got != want)
    assert differ.size == 0, (f"{len(differ)} of 65536 gated outputs differ, first: z "
                              f"{z[tuple(differ[0])]:#06x} got {got[tuple(differ[0])]:#06x} "
                              f"want {want[tuple(differ[0])]:#06x}")
    assert np.array_equal(b_one.read(np.uint16), want[5])


def test_gates_of_every_bf16_value():
    """decay and beta (gdn_gates_blk) with the a and b rows running through all 65536 bf16
    bit patterns (non-finite ones replaced by zero).  beta is a chain of bf16 steps: the
    checker's bits.  decay = exp(y) ends in two fp32 exponentials of different libraries: within
    a few ulps of y, i.e. 4e-7 (1 + |y|) of the result."""
    rows = 2048
    print("[case] gdn gates over every bf16 value", flush=True)
    B, dev, queue, lib = gpu()
    _, a_log, dt_bias, _ = _weights()
    patterns = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    patterns[(patterns & 0x7F80) == 0x7F80] = 0
    proj = np.zeros((rows, 12352), np.uint16)
    proj[:, 12288:12320] = patterns.reshape(rows, 32)                   # b
    proj[:, 12320:12352] = np.roll(patterns, 7).reshape(rows, 32)       # a
    want_decay = np.zeros((rows, 32), np.float32); want_beta = np.zeros((rows, 32), np.float32)
    for r in range(rows):
        o.tto_gdn_gates(proj[r], a_log, dt_bias, want_decay[r], want_beta[r])
    b_proj = dev.buffer_from(proj.reshape(-1))
    b_al, b_dt = dev.buffer_from(a_log), dev.buffer_from(dt_bias)
    b_decay, b_beta = dev.create_buffer(rows * 128), dev.create_buffer(rows * 128)
    run(lambda cb: cb.encode(lib.pipeline("gdn_gates_blk"),
                             {0: b_proj, 1: b_al, 2: b_dt, 3: b_decay, 4: b_beta}, {5: rows},
                             (1, (rows + 3) // 4, 1), (32, 4, 1)))
    beta = b_beta.read(np.float32).reshape(rows, 32)
    decay = b_decay.read(np.float32).reshape(rows, 32)
    assert np.array_equal(beta.view(np.uint32), want_beta.view(np.uint32)), \
        f"{np.count_nonzero(beta.view(np.uint32) != want_beta.view(np.uint32))} betas differ"
    assert np.isfinite(decay).all()
    # decay = exp(y): an ulp of y is |y| 2^-23 of the result
    exponent = np.abs(np.log(np.maximum(want_decay.astype(np.float64), 1e-300)))
    # (a subnormal decay comes out as zero: the family's arithmetic flushes, and the checker's
    # next step, state * decay, flushes the product as well)
    bar = 4e-7 * (1.0 + np.minimum(exponent, 110.0)) * np.abs(want_decay) + 1.2e-38
    close = np.abs(decay.astype(np.float64) - want_decay) <= bar
    bad = np.argwhere(~close)
    detail = [(hex(int(proj[r, 12320 + h])), hex(int(a_log[h])), hex(int(dt_bias[h])),
               float(decay[r, h]), float(want_decay[r, h])) for r, h in bad[:6]]
    assert close.all(), (f"{len(bad)} decays differ, worst relative "
                         f"{np.max(np.abs(decay - want_decay) / np.maximum(np.abs(want_decay), 1e-30)):.3e}"
                         f" (a, A_log, dt_bias, got, want): {detail}")


def _encode_chunked(cb, lib, bufs, rows, state_in="state_in", state_out="state_out"):
    chunks = (rows + 63) // 64
    cb.encode(lib.pipeline("gdn_chunk_prepare_blk"),
              {0: bufs["qk"], 1: bufs["value"], 2: bufs["decay"], 3: bufs["beta"],
               4: bufs["chunk"]}, {5: rows}, (chunks, 32, 1), (256, 1, 1))
    cb.barrier()
    cb.encode(lib.pipeline("gdn_chunk_scan_blk"),
              {0: bufs["chunk"], 1: bufs[state_in], 2: bufs["y"], 3: bufs[state_out]},
              {4: rows}, (8, 32, 1), (256, 1, 1))


@pytest.mark.parametrize("rows", [1, 63, 64, 65, 200, 1024])
def test_chunked_recurrence_matches_token_loop(rows):
    """The chunked evaluation against the token-by-token checker, including a
    single row, exact chunk multiples and ragged tails."""
    print(f"[case] gdn chunked recurrence rows={rows}", flush=True)
    B, dev, queue, lib = gpu()
    weights = _weights()
    proj, conv_state, state = _block(rows, 0x5200 + rows)
    ref = _oracle_block(proj, conv_state, state, weights, rows)
    bufs = _buffers(dev, proj, conv_state, state, weights, rows)

    def rec(cb):
        _encode_front(cb, lib, bufs, rows)
        _encode_chunked(cb, lib, bufs, rows)
        _encode_gate_norm(cb, lib, bufs, rows)
    run(rec)
    check_bf16(bufs["y"].read(np.uint16), ref["y"], "chunked y")
    check_f32(bufs["state_out"].read(np.float32), ref["state"], "chunked state", 2e-3, 2e-4)
    check_bf16(bufs["gated"].read(np.uint16), ref["gated"], "chunked gated", ulps=4)


def test_chunked_recurrence_with_harsh_gates():
    """Gates far from the seeded tests' mild ones: exp(A_log) from 0.4 to 16 and a wide a row,
    so that decays run from 1 down to exp(-100) and underflow inside a chunk, betas from 0 to 1.
    The chunked evaluation keeps its decay products in logarithms; the token loop is the bar."""
    rows = 200
    print("[case] gdn chunked recurrence with harsh gates", flush=True)
    B, dev, queue, lib = gpu()
    conv_w, _, dt_bias, norm_w = _weights()
    a_log = ol.f32_to_bf16(ol.uniform_f32(0x7B, 32, -1.0, 2.8))
    weights = (conv_w, a_log, dt_bias, norm_w)
    proj, conv_state, state = _block(rows, 0x5400)
    proj[:, 12320:12352] = ol.gaussian_bf16(0x5401, rows * 32, 0.0, 3.0).reshape(rows, 32)   # a
    proj[:, 12288:12320] = ol.gaussian_bf16(0x5402, rows * 32, 0.0, 6.0).reshape(rows, 32)   # b
    ref = _oracle_block(proj, conv_state, state, weights, rows)
    assert ref["decay"].min() < 1e-30 and ref["decay"].max() > 0.99
    assert ref["beta"].min() < 1e-3 and ref["beta"].max() > 0.999
    bufs = _buffers(dev, proj, conv_state, state, weights, rows)

    def rec(cb):
        _encode_front(cb, lib, bufs, rows)
        _encode_chunked(cb, lib, bufs, rows)
        _encode_gate_norm(cb, lib, bufs, rows)
    run(rec)
    check_bf16(bufs["y"].read(np.uint16), ref["y"], "harsh gates: chunked y")
    check_f32(bufs["state_out"].read(np.float32), ref["state"], "harsh gates: chunked state", 2e-3, 2e-4)
    check_bf16(bufs["gated"].read(np.uint16), ref["gated"], "harsh gates: chunked gated", ulps=4)


def test_chunked_recurrence_in_place_and_chained_blocks():
    """Two consecutive blocks (130 + 70 rows) with the state plane updated in
    place equal one 200-row token loop."""
    print("[case] gdn chunked recurrence, two chained blocks", flush=True)
    B, dev, queue, lib = gpu()
    weights = _weights()
    rows = 200
    proj, conv_state, state = _block(rows, 0x5300)
    ref = _oracle_block(proj, conv_state, state, weights, rows)
    bufs = _buffers(dev, proj, conv_state, state, weights, rows)
    ys = []
    start = 0
    conv_in = conv_state
    for part in (130, 70):
        sub = _buffers(dev, proj[start:start + part], conv_in, state, weights, part)
        sub["state_in"] = bufs["state_in"]

        def rec(cb, sub=sub, part=part):
            _encode_front(cb, lib, sub, part)
            _encode_chunked(cb, lib, sub, part, "state_in", "state_in")
        run(rec)
        ys.append(sub["y"].read(np.uint16))
        conv_in = sub["conv_out"].read(np.uint16)
        start += part
    check_bf16(np.concatenate(ys), ref["y"], "chained y")
    check_f32(bufs["state_in"].read(np.float32), ref["state"], "chained state", 2e-3, 2e-4)
    assert np.array_equal(conv_in, ref["conv"])


def test_chunked_recurrence_validation():
    B, dev, queue, lib = gpu()
    rows = 100
    small = dev.create_buffer(1024)
    ok = dev.create_buffer(rows * 8192)
    gates = dev.create_buffer(rows * 128)
    scratch = dev.create_buffer(2 * 32 * 115712)
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    with pytest.raises(B.BackendError) as e:   # scratch too small for two chunks
        cb.encode(lib.pipeline("gdn_chunk_prepare_blk"),
                  {0: ok, 1: ok, 2: gates, 3: gates, 4: small}, {5: rows}, (2, 32, 1), (256, 1, 1))
    assert e.value.status == 10
    with pytest.raises(B.BackendError) as e:   # grid does not match ceil(rows/64)
        cb.encode(lib.pipeline("gdn_chunk_prepare_blk"),
                  {0: ok, 1: ok, 2: gates, 3: gates, 4: scratch}, {5: rows}, (3, 32, 1),
                  (256, 1, 1))
    assert e.value.status == 15
    assert cb.command_count == 0


def test_grouped_chunk_recurrence_equals_the_two_stages():
    """gdn_chunk_recurrence_blk (stage 1 + stage 2 per group of 2048 rows, scratch for
    one group only) against gdn_chunk_prepare_blk + gdn_chunk_scan_blk over 2300 rows
    (two groups, ragged tail): bit-identical outputs and state."""
    print("[case] gdn grouped chunk recurrence, 2300 rows", flush=True)
    B, dev, queue, lib = gpu()
    rows = 2300
    rng = np.random.default_rng(9)
    q = rng.standard_normal((rows, 16, 128)); k = rng.standard_normal((rows, 16, 128))
    q /= np.linalg.norm(q, axis=2, keepdims=True) * np.sqrt(128.0)
    k /= np.linalg.norm(k, axis=2, keepdims=True)
    qk = ol.f32_to_bf16(np.concatenate([q.reshape(rows, -1), k.reshape(rows, -1)], axis=1)
                        .astype(np.float32).reshape(-1))
    v = ol.gaussian_bf16(0x6701, rows * 4096)
    decay = np.exp(rng.uniform(-0.1, 0, (rows, 32))).astype(np.float32)
    beta = (1 / (1 + np.exp(-rng.standard_normal((rows, 32))))).astype(np.float32)
    state = ol.gaussian_f32(0x6702, STATE, 0.0, 0.02)
    bufs = {"qk": dev.buffer_from(qk), "value": dev.buffer_from(v),
            "decay": dev.buffer_from(decay.reshape(-1)), "beta": dev.buffer_from(beta.reshape(-1)),
            "state_in": dev.buffer_from(state), "state_out": dev.create_buffer(STATE * 4),
            "y": dev.create_buffer(rows * 8192),
            "chunk": dev.create_buffer(((rows + 63) // 64) * 32 * 115712)}
    state2, y2 = dev.create_buffer(STATE * 4), dev.create_buffer(rows * 8192)
    small = dev.create_buffer(32 * 32 * 115712)          # records of 2048 rows

    def rec(cb):
        _encode_chunked(cb, lib, bufs, rows)
        cb.encode(lib.pipeline("gdn_chunk_recurrence_blk"),
                  {0: bufs["qk"], 1: bufs["value"], 2: bufs["decay"], 3: bufs["beta"], 4: small,
                   5: bufs["state_in"], 6: y2, 7: state2}, {8: rows}, (8, 32, 1), (256, 1, 1))
    run(rec)
    assert np.array_equal(y2.read(np.uint16), bufs["y"].read(np.uint16))
    assert np.array_equal(state2.read(np.float32), bufs["state_out"].read(np.float32))
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    with pytest.raises(B.BackendError) as e:             # scratch below one group's records
        cb.encode(lib.pipeline("gdn_chunk_recurrence_blk"),
                  {0: bufs["qk"], 1: bufs["value"], 2: bufs["decay"], 3: bufs["beta"],
                   4: dev.create_buffer(1024), 5: bufs["state_in"], 6: y2, 7: state2}, {8: rows},
                  (8, 32, 1), (256, 1, 1))
    assert e.value.status == 10


def test_config4_gdn_prefill_16384_rows_against_token_loop():
    """Config 4, Gated DeltaNet half at full size: 16384 tokens of one lane through conv,
    gates, the chunk-64 recurrence (grouped operator, scratch for one 2048-row group as
    the benchmark binds it) and the gate-norm, against the checker's token-by-token
    scan.  The drift of y is reported per 2048-row group; the bar does not move."""
    rows, group = 16384, 2048
    print(f"[case] config 4: gdn block prefill, {rows} rows", flush=True)
    B, dev, queue, lib = gpu()
    weights = _weights()
    proj, conv_state, state = _block(rows, 0xC0F4)
    ref = _oracle_block(proj, conv_state, state, weights, rows)
    bufs = _buffers(dev, proj, conv_state, state, weights, min(rows, group))
    for name in ("qk", "value", "z", "y", "gated"):
        bufs[name] = dev.create_buffer(rows * 8192)
    bufs["decay"], bufs["beta"] = dev.create_buffer(rows * 128), dev.create_buffer(rows * 128)
    bufs["proj"] = dev.buffer_from(proj.reshape(-1))

    def rec(cb):
        _encode_front(cb, lib, bufs, rows)
        cb.encode(lib.pipeline("gdn_chunk_recurrence_blk"),
                  {0: bufs["qk"], 1: bufs["value"], 2: bufs["decay"], 3: bufs["beta"],
                   4: bufs["chunk"], 5: bufs["state_in"], 6: bufs["y"], 7: bufs["state_out"]},
                  {8: rows}, (8, 32, 1), (256, 1, 1))
        _encode_gate_norm(cb, lib, bufs, rows)
    run(rec)
    assert np.array_equal(bufs["conv_out"].read(np.uint16), ref["conv"])      # conv state: exact
    y = bufs["y"].read(np.uint16).reshape(rows, 4096)
    want_y = ref["y"].reshape(rows, 4096)
    for first in range(0, rows, group):
        g = ol.bf16_to_f32(y[first:first + group].reshape(-1))
        w = ol.bf16_to_f32(want_y[first:first + group].reshape(-1))
        err = np.abs(g - w)
        print(f"[drift] y rows {first}..{first + group - 1}: max-abs {err.max():.3e} "
              f"mean-abs {err.mean():.3e}", flush=True)
    check_bf16(y, want_y, "config 4 chunked y, 16384 rows")
    check_f32(bufs["state_out"].read(np.float32), ref["state"], "config 4 final state", 2e-3, 2e-4)
    check_bf16(bufs["gated"].read(np.uint16), ref["gated"], "config 4 gated", ulps=4)
