"""Rollback tape of a short Gated DeltaNet block on the GPU, through the C ABI:
`gdn_conv_tape_blk`, `gdn_recurrence_gates_tape_blk` and `gdn_tape_replay_blk`.

The reference holds no test for the tape, so the bars are what its definition
fixes: the taped operators change nothing the plain ones compute (bit for bit);
the conv tape holds the exact window after each row (bytes, against the CPU
checker); the recurrence tape holds the scan's own keys and gates (bit for bit)
and deltas within the fp32 noise of the checker's (5e-5); and replaying c rows
gives, bit for bit, the state the forward scan stores after exactly c rows."""
import numpy as np
import pytest

import oracle_lib as ol
from gpu_util import check_f32, gpu, run
from test_gpu_gdn_prefill import _block, _buffers, _weights

pytestmark = pytest.mark.gpu
o = ol.oracle
STATE = 32 * 128 * 128
TAPE_KEYS = 40 * 16 * 32 * 128
TAPE_GATES = TAPE_KEYS + 40 * 16 * 16 * 128
TAPE_FLOATS = 40 * 16 * (32 * 128 + 16 * 128 + 64)
CONV_TAPE = 40 * 16 * 3 * 8192
FILL = np.float32(-77.0)


def _front(cb, lib, bufs, rows, taped, layer):
    bindings = {0: bufs["proj"], 1: bufs["conv_in"], 2: bufs["conv_w"], 3: bufs["qk"],
                4: bufs["value"], 5: bufs["z"], 6: bufs["conv_out"]}
    constants = {7: rows}
    if taped:
        bindings[8] = bufs["conv_tape"]
        constants[9] = layer
    cb.encode(lib.pipeline("gdn_conv_tape_blk" if taped else "gdn_conv_blk"), bindings, constants,
              (96, rows, 1), (128, 1, 1))
    cb.encode(lib.pipeline("gdn_gates_blk"),
              {0: bufs["proj"], 1: bufs["a_log"], 2: bufs["dt_bias"], 3: bufs["decay"],
               4: bufs["beta"]}, {5: rows}, (1, (rows + 3) // 4, 1), (32, 4, 1))
    cb.barrier()


def _scan(cb, lib, bufs, steps, taped, layer, state_out="state_out"):
    bindings = {0: bufs["qk"], 1: bufs["value"], 2: bufs["decay"], 3: bufs["a_log"],
                4: bufs["beta"], 5: bufs["state_in"], 6: bufs["y"], 7: bufs[state_out]}
    constants = {8: steps}
    if taped:
        bindings[9] = bufs["tape"]
        constants[10] = layer
    cb.encode(lib.pipeline("gdn_recurrence_gates_tape_blk" if taped else
                           "gdn_recurrence_gates_blk"), bindings, constants, (1, 32, 32), (32, 4, 1))


@pytest.mark.parametrize("rows,layer", [(1, 0), (7, 22), (16, 39)])
def test_tape_and_replay(rows, layer):
    print(f"[case] gdn tape rows={rows} layer={layer}", flush=True)
    B, dev, queue, lib = gpu()
    weights = _weights()
    proj, conv_state, state = _block(rows, 0x7A00 + rows)
    bufs = _buffers(dev, proj, conv_state, state, weights, rows)
    bufs["tape"] = dev.buffer_from(np.full(TAPE_FLOATS, FILL))
    bufs["conv_tape"] = dev.buffer_from(np.full(CONV_TAPE, 0x7FC0, np.uint16))

    # plain operators first: what the taped ones must reproduce
    run(lambda cb: (_front(cb, lib, bufs, rows, False, layer), _scan(cb, lib, bufs, rows, False, layer)))
    plain = {k: bufs[k].read(np.uint16) for k in ("qk", "value", "z", "conv_out", "y")}
    plain_state = bufs["state_out"].read(np.uint32)
    for name in ("qk", "value", "z", "conv_out", "y", "state_out"):
        bufs[name].write(np.zeros(bufs[name].size_bytes // 2, np.uint16))
    run(lambda cb: (_front(cb, lib, bufs, rows, True, layer), _scan(cb, lib, bufs, rows, True, layer)))
    for name, want in plain.items():
        assert np.array_equal(bufs[name].read(np.uint16), want), name
    assert np.array_equal(bufs["state_out"].read(np.uint32), plain_state)

    # conv tape: exact windows, nothing else touched
    want_conv = np.full(CONV_TAPE, 0x7FC0, np.uint16)
    o.tto_gdn_conv_tape(proj.reshape(-1), rows, conv_state, want_conv, layer)
    assert np.array_equal(bufs["conv_tape"].read(np.uint16), want_conv)
    assert np.array_equal(want_conv.reshape(40, 16, -1)[layer, rows - 1], plain["conv_out"])

    # recurrence tape: the scan's own operands, and the checker's deltas
    tape = bufs["tape"].read(np.float32)
    deltas = tape[:TAPE_KEYS].reshape(40, 16, 32, 128)
    keys = tape[TAPE_KEYS:TAPE_GATES].reshape(40, 16, 16, 128)
    gates = tape[TAPE_GATES:].reshape(40, 16, 32, 2)
    for region in (deltas, keys, gates):
        assert np.all(np.delete(region, layer, axis=0) == FILL)
        assert np.all(region[layer, rows:] == FILL)
    qk = ol.bf16_to_f32(plain["qk"]).reshape(rows, 4096)
    assert np.array_equal(keys[layer, :rows].reshape(rows, 2048), qk[:, 2048:])
    decay = bufs["decay"].read(np.float32).reshape(rows, 32)
    beta = bufs["beta"].read(np.float32).reshape(rows, 32)
    assert np.array_equal(gates[layer, :rows, :, 0], decay)
    assert np.array_equal(gates[layer, :rows, :, 1], beta)
    want_tape = np.full(TAPE_FLOATS, FILL)
    y = np.zeros(rows * 4096, np.uint16); s1 = np.zeros(STATE, np.float32)
    o.tto_gdn_scan_tape(plain["qk"], plain["value"], decay.reshape(-1), beta.reshape(-1), rows,
                        state, y, s1, want_tape, layer, 8)
    check_f32(deltas[layer, :rows].reshape(-1),
              want_tape[:TAPE_KEYS].reshape(40, 16, 32, 128)[layer, :rows].reshape(-1),
              "tape delta", 5e-5, 5e-6)

    # replay of every prefix == forward scan of that prefix, bit for bit
    bufs["rebuilt"] = dev.create_buffer(STATE * 4)
    bufs["prefix"] = dev.create_buffer(STATE * 4)
    for committed in sorted({0, 1, rows // 2, rows - 1, rows}):
        def rec(cb):
            cb.encode(lib.pipeline("gdn_tape_replay_blk"),
                      {0: bufs["tape"], 1: bufs["state_in"], 2: bufs["rebuilt"]},
                      {3: committed, 4: layer}, (1, 32, 32), (32, 4, 1))
            if committed:
                _scan(cb, lib, bufs, committed, False, layer, "prefix")
        run(rec)
        want = bufs["prefix"].read(np.uint32) if committed else state.view(np.uint32)
        assert np.array_equal(bufs["rebuilt"].read(np.uint32), want), committed
    # and the checker's replay of the checker's tape agrees within the state bar
    replayed = np.zeros(STATE, np.float32)
    o.tto_gdn_tape_replay(want_tape, state, replayed, rows, layer, 8)
    check_f32(bufs["rebuilt"].read(np.float32), replayed, "replayed state", 2e-3, 2e-5)


def test_long_block_leaves_the_tape_alone_and_validation():
    rows = 17
    print(f"[case] gdn tape rows={rows} (beyond the tape) and validation", flush=True)
    B, dev, queue, lib = gpu()
    weights = _weights()
    proj, conv_state, state = _block(rows, 0x7B00)
    bufs = _buffers(dev, proj, conv_state, state, weights, rows)
    bufs["tape"] = dev.buffer_from(np.full(TAPE_FLOATS, FILL))
    bufs["conv_tape"] = dev.buffer_from(np.full(CONV_TAPE, 0x7FC0, np.uint16))
    run(lambda cb: (_front(cb, lib, bufs, rows, True, 3), _scan(cb, lib, bufs, rows, True, 3)))
    assert np.all(bufs["tape"].read(np.float32) == FILL)
    assert np.all(bufs["conv_tape"].read(np.uint16) == 0x7FC0)
    taped_state = bufs["state_out"].read(np.uint32)
    taped_y = bufs["y"].read(np.uint16)
    run(lambda cb: (_front(cb, lib, bufs, rows, False, 3), _scan(cb, lib, bufs, rows, False, 3)))
    assert np.array_equal(bufs["state_out"].read(np.uint32), taped_state)
    assert np.array_equal(bufs["y"].read(np.uint16), taped_y)

    small = dev.create_buffer(TAPE_FLOATS * 4 - 4)
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    replay = lib.pipeline("gdn_tape_replay_blk")
    for bindings, constants, grid, status in [
        ({0: small, 1: bufs["state_in"], 2: bufs["state_out"]}, {3: 4, 4: 0}, (1, 32, 32), 10),
        ({0: bufs["tape"], 1: bufs["state_in"], 2: bufs["state_out"]}, {3: 17, 4: 0}, (1, 32, 32), 8),
        ({0: bufs["tape"], 1: bufs["state_in"], 2: bufs["state_out"]}, {3: 4, 4: 40}, (1, 32, 32), 8),
        ({0: bufs["tape"], 1: bufs["state_in"], 2: bufs["state_out"]}, {3: 4, 4: 0}, (1, 32, 31), 15),
    ]:
        with pytest.raises(B.BackendError) as e:
            cb.encode(replay, bindings, constants, grid, (32, 4, 1))
        assert e.value.status == status
    with pytest.raises(B.BackendError) as e:   # conv tape one element short
        cb.encode(lib.pipeline("gdn_conv_tape_blk"),
                  {0: bufs["proj"], 1: bufs["conv_in"], 2: bufs["conv_w"], 3: bufs["qk"],
                   4: bufs["value"], 5: bufs["z"], 6: bufs["conv_out"],
                   8: dev.create_buffer(CONV_TAPE * 2 - 2)}, {7: rows, 9: 0}, (96, rows, 1), (128, 1, 1))
    assert e.value.status == 10
    with pytest.raises(B.BackendError) as e:   # layer beyond the tape
        cb.encode(lib.pipeline("gdn_recurrence_gates_tape_blk"),
                  {0: bufs["qk"], 1: bufs["value"], 2: bufs["decay"], 3: bufs["a_log"],
                   4: bufs["beta"], 5: bufs["state_in"], 6: bufs["y"], 7: bufs["state_out"],
                   9: bufs["tape"]}, {8: rows, 10: 40}, (1, 32, 32), (32, 4, 1))
    assert e.value.status == 8
    assert cb.command_count == 0
