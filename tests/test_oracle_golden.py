"""The CPU checker against the committed vectors produced by the unmodified
reference scalar model (tests/golden/make_golden.py).  Bit-exact."""
import os

import numpy as np
import pytest

import oracle_lib as ol
from golden import cases

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz"))
o = ol.oracle


def fill(seed, n):
    return ol.banded_bf16(seed, n)


def fill_f32(seed, n):
    out = np.empty(n, np.float32)
    o.tto_fill_banded_f32(seed, out, n)
    return out


def test_generator_and_conversion():
    assert np.array_equal(fill(cases.ATTN_SEED, 64), G["banded_first64"])
    got = np.array([o.tto_bf16_from_f32(float(x)) for x in G["bf16_probe_in"]], np.uint16)
    assert np.array_equal(got, G["bf16_probe_out"])
    assert np.array_equal(ol.f32_to_bf16(G["bf16_probe_in"]), G["bf16_probe_out"])


def test_qk_rope_chain_and_decode():
    proj, q_w, k_w = cases.attention_chain_inputs(fill)
    cap = cases.ATTN_CAPACITY
    keys = np.zeros(2 * cap * 256, np.uint16)
    values = np.zeros_like(keys)
    q = np.zeros(4096, np.uint16)
    gate = np.zeros(4096, np.uint16)
    for pos in range(cases.ATTN_CHAIN_POSITIONS):
        o.tto_attn_qk_rope(proj[pos], q_w, k_w, pos, cap, q, gate, keys, values)
    n = cases.ATTN_CHAIN_POSITIONS
    assert np.array_equal(q, G["chain_q"])
    assert np.array_equal(gate, G["chain_gate"])
    assert np.array_equal(keys.reshape(2, cap, 256)[:, :n], G["chain_keys"])
    assert np.array_equal(values.reshape(2, cap, 256)[:, :n], G["chain_values"])
    # rows past the chain are untouched: slot indexing is exact
    assert not keys.reshape(2, cap, 256)[:, n:].any()
    att = np.zeros(4096, np.uint16)
    o.tto_attention_decode(q, gate, keys, values, n - 1, cap, att, 1)
    assert np.array_equal(att, G["chain_attended"])


def test_rope_far_position():
    proj, q_w, k_w = cases.attention_chain_inputs(fill)
    far = 100000
    q = np.zeros(4096, np.uint16)
    gate = np.zeros(4096, np.uint16)
    keys = np.zeros(2 * (far + 1) * 256, np.uint16)
    values = np.zeros_like(keys)
    o.tto_attn_qk_rope(proj[0], q_w, k_w, far, far + 1, q, gate, keys, values)
    assert np.array_equal(q, G["rope_far_q"])


@pytest.mark.parametrize("ctx", cases.ATTN_CONTEXTS)
def test_decode_tiled_and_split(ctx):
    q, gate, keys, values = cases.attention_decode_inputs(fill, ctx)
    cap = cases.ATTN_CAPACITY
    tiled = np.zeros(4096, np.uint16)
    o.tto_attention_decode(q, gate, keys, values, ctx, cap, tiled, 2)
    assert np.array_equal(tiled, G[f"decode_tiled_ctx{ctx}"])
    nparts = 1 if ctx + 1 <= 256 else (ctx + 256) // 256
    split = np.zeros(4096, np.uint16)
    partials = np.zeros(16 * nparts * 258, np.float32)
    o.tto_attention_decode_split(q, gate, keys, values, ctx, cap, 256, partials, split, 2)
    assert np.array_equal(split, G[f"decode_split_ctx{ctx}"])
    got = partials.reshape(16, nparts, 258)[5]
    assert np.array_equal(got.view(np.uint32), G[f"decode_partials_ctx{ctx}_head5"].view(np.uint32))
    if nparts == 1:
        # a single partition is the single-kernel family byte for byte
        # (attention_fixture_probe.cpp:869-878)
        assert np.array_equal(split, tiled)


def test_gdn_chain():
    proj, conv_state, conv_w, a_log, dt_bias, norm_w, state = cases.gdn_inputs(fill, fill_f32)
    st_in, cs = state.copy(), conv_state.copy()
    for step in range(cases.GDN_CHAIN_STEPS):
        qk = np.zeros(4096, np.uint16); v = np.zeros(4096, np.uint16)
        z = np.zeros(4096, np.uint16); ncs = np.zeros(3 * 8192, np.uint16)
        o.tto_gdn_prepare(proj[step], cs, conv_w, qk, v, z, ncs)
        decay = np.zeros(32, np.float32); beta = np.zeros(32, np.float32)
        o.tto_gdn_gates(proj[step], a_log, dt_bias, decay, beta)
        y = np.zeros(4096, np.uint16); st_out = np.zeros_like(st_in)
        o.tto_gdn_recurrence(qk, v, decay, beta, st_in, 16, 32, y, st_out, 2)
        gated = np.zeros(4096, np.uint16)
        o.tto_gdn_gate_norm(y, z, norm_w, 32, gated)
        assert np.array_equal(qk, G[f"gdn_qk_{step}"])
        assert np.array_equal(v, G[f"gdn_v_{step}"])
        assert np.array_equal(z, proj[step][8192:12288])
        assert np.array_equal(decay.view(np.uint32), G[f"gdn_decay_{step}"].view(np.uint32))
        assert np.array_equal(beta.view(np.uint32), G[f"gdn_beta_{step}"].view(np.uint32))
        assert np.array_equal(y, G[f"gdn_y_{step}"])
        assert np.array_equal(gated, G[f"gdn_gated_{step}"])
        assert np.array_equal(st_out[::cases.STATE_SAMPLE_STRIDE].view(np.uint32),
                              G[f"gdn_state_sample_{step}"].view(np.uint32))
        st_in, cs = st_out, ncs
    assert np.array_equal(cs, G["gdn_conv_state_final"])


def test_gdn_fused_step_and_prefill_equal_chain():
    """decode_step == prepare/gates/recurrence/gate_norm, and a block of T rows
    == T decode steps (prefill_gdn.metal:198-203)."""
    proj, conv_state, conv_w, a_log, dt_bias, norm_w, state = cases.gdn_inputs(fill, fill_f32)
    T = cases.GDN_CHAIN_STEPS
    st_in, cs = state.copy(), conv_state.copy()
    gated_steps = []
    for step in range(T):
        ncs = np.zeros(3 * 8192, np.uint16); st_out = np.zeros_like(st_in)
        gated = np.zeros(4096, np.uint16)
        o.tto_gdn_decode_step(proj[step], cs, conv_w, a_log, dt_bias, norm_w, st_in, ncs, st_out,
                              gated, 2)
        assert np.array_equal(gated, G[f"gdn_gated_{step}"])
        gated_steps.append(gated)
        st_in, cs = st_out, ncs
    ncs = np.zeros(3 * 8192, np.uint16); st_blk = np.zeros_like(state)
    gated_blk = np.zeros(T * 4096, np.uint16)
    o.tto_gdn_prefill(np.ascontiguousarray(proj), T, conv_state, conv_w, a_log, dt_bias, norm_w,
                      state, ncs, st_blk, gated_blk, None, None, None, 2)
    assert np.array_equal(gated_blk.reshape(T, 4096), np.stack(gated_steps))
    assert np.array_equal(st_blk.view(np.uint32), st_in.view(np.uint32))
    assert np.array_equal(ncs, cs)


def test_residual_sum_and_row_norm():
    """bf16(a + b) and the row norm of the rounded sums (residual_rms, moe.metal:1-46)."""
    hidden = 2048
    a = fill(cases.RESIDUAL_SEED, 2 * hidden)
    b = fill(cases.RESIDUAL_SEED + 1, 2 * hidden)
    w = fill(cases.RESIDUAL_SEED + 2, hidden)
    sums = np.zeros(2 * hidden, np.uint16)
    o.tto_add_bf16(a, b, 2 * hidden, sums)
    assert np.array_equal(sums, G["residual_sums"])
    normed = np.zeros(2 * hidden, np.uint16)
    o.tto_rms_only(sums, w, 2, hidden, normed)
    assert np.array_equal(normed, G["residual_normed"])
