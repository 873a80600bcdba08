"""Known answers, closed forms and invariants that pin the CPU checker where
no stored vector exists; each is chosen so a dropped term, wrong sign or
transposed operand fails it."""
import numpy as np
import pytest

import oracle_lib as ol

o = ol.oracle
BF = ol.f32_to_bf16
F = ol.bf16_to_f32


def test_bf16_known_answers():
    # kernel_reference_test.cpp:15-35
    assert o.tto_bf16_from_f32(0.0) == 0x0000
    assert o.tto_bf16_from_f32(1.0) == 0x3F80
    assert o.tto_bf16_from_f32(-2.0) == 0xC000
    tie_even = np.array([0x3F808000], np.uint32).view(np.float32)[0]
    tie_odd = np.array([0x3F818000], np.uint32).view(np.float32)[0]
    assert o.tto_bf16_from_f32(float(tie_even)) == 0x3F80
    assert o.tto_bf16_from_f32(float(tie_odd)) == 0x3F82
    assert o.tto_bf16_from_f32(float("inf")) == 0x7F80
    assert o.tto_f32_from_bf16(0x3F80) == 1.0 and o.tto_f32_from_bf16(0xC000) == -2.0


def test_flush_to_zero_known_answers():
    # kernel_reference_test.cpp:37-54
    assert o.tto_bf16_mul(0x0001, 0x7F00) == 0x0000
    assert o.tto_bf16_mul(0x3F80, 0x8014) == 0x8000
    assert o.tto_bf16_mul(0x0080, 0x3F00) == 0x0000
    assert o.tto_bf16_mul(0x8080, 0x3F00) == 0x8000
    assert o.tto_flush_bf16(0x0080) == 0x0080 and o.tto_flush_bf16(0x8000) == 0x8000


def test_tree_shapes_are_the_pinned_ones():
    rng = np.random.default_rng(3)
    lanes = (rng.standard_normal(32) * 10.0 ** rng.integers(-3, 4, 32)).astype(np.float32)
    lvl = lanes.copy()
    while lvl.size > 1:
        lvl = (lvl[0::2] + lvl[1::2]).astype(np.float32)
    assert o.tto_tree_adjacent32(lanes) == lvl[0]
    slots = (rng.standard_normal(256) * 10.0 ** rng.integers(-3, 4, 256)).astype(np.float32)
    red = slots.copy()
    off = 128
    while off:
        red[:off] = red[:off] + red[off:2 * off]
        off //= 2
    assert o.tto_tree_halving256(slots) == red[0]
    if ol.ref is not None:
        assert ol.ref.ref_tree_sum(lanes, 32, 1) == o.tto_tree_adjacent32(lanes)   # AdjacentPairs
        assert ol.ref.ref_tree_sum(slots, 256, 0) == o.tto_tree_halving256(slots)  # Halving


def test_attention_context_zero_closed_form():
    # one key: probability 1, denominator 1 -> out = bf16(V[0] * sigmoid(gate));
    # gate 0 -> V/2 (kernel_reference_test.cpp:257-275)
    cap = 8
    q = ol.banded_bf16(37, 4096)
    keys = ol.banded_bf16(38, 2 * cap * 256)
    values = ol.banded_bf16(39, 2 * cap * 256)
    gate = np.zeros(4096, np.uint16)
    out = np.zeros(4096, np.uint16)
    o.tto_attention_decode(q, gate, keys, values, 0, cap, out, 1)
    v = F(values).reshape(2, cap, 256)
    for head in range(16):
        expect = BF(v[head // 8, 0] * np.float32(0.5))
        expect = np.where((expect & 0x7F80) == 0, expect & 0x8000, expect)
        assert np.array_equal(out[head * 256:(head + 1) * 256], expect)
    out2 = np.zeros(4096, np.uint16)
    o.tto_attention_decode_split(q, gate, keys, values, 0, cap, 256, None, out2, 1)
    assert np.array_equal(out, out2)


def test_attention_matches_textbook_softmax():
    """fp64 softmax(qK^T/16)V*sigmoid(g): catches a wrong scale, a missing
    normaliser, a kv-head mapping error (head>>3) or a gate sign error."""
    cap, ctx = 1024, 700
    q = ol.gaussian_bf16(1, 4096)
    gate = ol.gaussian_bf16(2, 4096)
    keys = ol.gaussian_bf16(3, 2 * cap * 256)
    values = ol.gaussian_bf16(4, 2 * cap * 256)
    tiled = np.zeros(4096, np.uint16)
    split = np.zeros(4096, np.uint16)
    o.tto_attention_decode(q, gate, keys, values, ctx, cap, tiled, 4)
    o.tto_attention_decode_split(q, gate, keys, values, ctx, cap, 256, None, split, 4)
    qf = F(q).astype(np.float64).reshape(16, 256)
    gf = F(gate).astype(np.float64).reshape(16, 256)
    kf = F(keys).astype(np.float64).reshape(2, cap, 256)[:, :ctx + 1]
    vf = F(values).astype(np.float64).reshape(2, cap, 256)[:, :ctx + 1]
    want = np.empty((16, 256))
    for h in range(16):
        s = kf[h // 8] @ qf[h] / 16.0
        p = np.exp(s - s.max())
        p /= p.sum()
        want[h] = (p @ vf[h // 8]) / (1.0 + np.exp(-gf[h]))
    for got in (tiled, split):
        err = np.abs(F(got).reshape(16, 256) - want)
        assert err.max() < 4e-3 and err.mean() < 3e-4
    # tiled and split differ only in rounding order
    assert np.abs(F(tiled) - F(split)).max() < 4e-3


def test_softmax_shift_invariance_and_padding():
    """Keys beyond `context` are never read, whatever they hold."""
    cap, ctx = 600, 299
    q = ol.gaussian_bf16(5, 4096)
    gate = ol.gaussian_bf16(6, 4096)
    keys = ol.gaussian_bf16(7, 2 * cap * 256)
    values = ol.gaussian_bf16(8, 2 * cap * 256)
    a = np.zeros(4096, np.uint16)
    o.tto_attention_decode_split(q, gate, keys, values, ctx, cap, 256, None, a, 2)
    k2 = keys.reshape(2, cap, 256).copy()
    v2 = values.reshape(2, cap, 256).copy()
    k2[:, ctx + 1:] = 0x7FC0  # NaN
    v2[:, ctx + 1:] = 0x7FC0
    b = np.zeros(4096, np.uint16)
    o.tto_attention_decode_split(q, gate, k2.reshape(-1), v2.reshape(-1), ctx, cap, 256, None, b, 2)
    assert np.array_equal(a, b)


def test_rope_identity_at_position_zero_and_norm_preservation():
    proj = ol.gaussian_bf16(11, 9216)
    ones = np.full(256, 0x3F80, np.uint16)
    cap = 4
    def run(pos):
        q = np.zeros(4096, np.uint16); g = np.zeros(4096, np.uint16)
        k = np.zeros(2 * cap * 256, np.uint16); v = np.zeros_like(k)
        o.tto_attn_qk_rope(proj, ones, ones, pos, cap, q, g, k, v)
        return q, g, k.reshape(2, cap, 256), v.reshape(2, cap, 256)
    q0, g0, k0, v0 = run(0)
    q3, g3, k3, v3 = run(3)
    p = F(proj)
    # position 0: cos=1, sin=0 -> the normalised vector itself; RMS-norm of a
    # head with unit weight has mean square 1
    qn = F(q0).reshape(16, 256)
    assert np.allclose((qn.astype(np.float64) ** 2).mean(axis=1), 1.0, atol=2e-2)
    for h in range(16):
        x = p[h * 512:h * 512 + 256].astype(np.float64)
        want = x / np.sqrt((x ** 2).mean() + 1e-6)
        assert np.abs(qn[h] - want).max() < 2e-2
        assert np.array_equal(g0[h * 256:(h + 1) * 256], proj[h * 512 + 256:h * 512 + 512])
    # rotation preserves each (d, d+32) pair's norm and leaves dims >= 64 alone
    a, b = F(q0).reshape(16, 256), F(q3).reshape(16, 256)
    assert np.array_equal(q0.reshape(16, 256)[:, 64:], q3.reshape(16, 256)[:, 64:])
    n0 = a[:, :32] ** 2 + a[:, 32:64] ** 2
    n3 = b[:, :32] ** 2 + b[:, 32:64] ** 2
    assert np.allclose(n0, n3, rtol=3e-2, atol=1e-3)
    # rotation direction: x' = x cos - y sin, y' = y cos + x sin, theta = pos / 1e7^(pair/32)
    theta = 3.0 / (1e7 ** (np.arange(32) / 32.0))
    xr = a[:, :32] * np.cos(theta) - a[:, 32:64] * np.sin(theta)
    yr = a[:, 32:64] * np.cos(theta) + a[:, :32] * np.sin(theta)
    assert np.abs(b[:, :32] - xr).max() < 3e-2 and np.abs(b[:, 32:64] - yr).max() < 3e-2
    # K appended at row `pos` of each kv head, V raw
    assert np.array_equal(v3[:, 3], proj[8704:9216].reshape(2, 256))
    assert not k3[:, :3].any() and k3[:, 3].any()


def test_gdn_zero_qk_beta_closed_form():
    # kernel_reference_test.cpp:198-229 with the test's 2 key / 4 value heads
    qk = np.zeros(2 * 2 * 128, np.uint16)
    value = ol.banded_bf16(41, 4 * 128)
    decay = np.ones(4, np.float32)
    beta = np.zeros(4, np.float32)
    state = F(ol.banded_bf16(42, 4 * 128 * 128)).copy()
    y = np.full(4 * 128, 0xFFFF, np.uint16)
    out = np.full_like(state, -1.0)
    o.tto_gdn_recurrence(qk, value, decay, beta, state, 2, 4, y, out, 1)
    assert np.array_equal(out.view(np.uint32), state.view(np.uint32))
    assert not y.any()


def test_gdn_recurrence_matches_fp64_delta_rule():
    """S <- a S; S += k (beta (v - S k))^T; y = S q, key head = h >> 1."""
    rng = np.random.default_rng(9)
    qk = BF(rng.standard_normal(4096).astype(np.float32) * 0.1)
    value = BF(rng.standard_normal(4096).astype(np.float32))
    decay = rng.uniform(0.9, 1.0, 32).astype(np.float32)
    beta = rng.uniform(0.0, 1.0, 32).astype(np.float32)
    state = (rng.standard_normal(32 * 128 * 128) * 0.02).astype(np.float32)
    y = np.zeros(4096, np.uint16)
    out = np.zeros_like(state)
    o.tto_gdn_recurrence(qk, value, decay, beta, state, 16, 32, y, out, 4)
    S = state.astype(np.float64).reshape(32, 128, 128)
    qf = F(qk).astype(np.float64)
    vf = F(value).astype(np.float64).reshape(32, 128)
    for h in range(32):
        q = qf[(h >> 1) * 128:(h >> 1) * 128 + 128]
        k = qf[2048 + (h >> 1) * 128:2048 + (h >> 1) * 128 + 128]
        Sh = S[h] * decay[h]
        delta = (vf[h] - Sh @ k) * beta[h]
        Sh = Sh + np.outer(delta, k)
        assert np.abs(out.reshape(32, 128, 128)[h] - Sh).max() < 1e-5
        assert np.abs(F(y).reshape(32, 128)[h] - Sh @ q).max() < 2e-3


def test_gdn_prepare_matches_plain_silu_and_l2():
    """conv taps order (tap 3 is the newest sample), SiLU, and q/k scaling:
    RMS-norm x 1/128 == L2-norm / sqrt(128) for q; x bf16(1/sqrt(128)) == L2-norm for k."""
    rng = np.random.default_rng(10)
    proj = BF(rng.standard_normal(12352).astype(np.float32) * 0.5)
    cs = BF(rng.standard_normal(3 * 8192).astype(np.float32) * 0.5)
    w = BF(rng.standard_normal(4 * 8192).astype(np.float32) * 0.5)
    qk = np.zeros(4096, np.uint16); v = np.zeros(4096, np.uint16)
    z = np.zeros(4096, np.uint16); ncs = np.zeros(3 * 8192, np.uint16)
    o.tto_gdn_prepare(proj, cs, w, qk, v, z, ncs)
    taps = np.vstack([F(cs).reshape(3, 8192), F(proj)[:8192]]).astype(np.float64)
    conv = (F(w).reshape(8192, 4).astype(np.float64).T * taps).sum(axis=0)
    act = conv / (1.0 + np.exp(-conv))
    assert np.abs(F(v) - act[4096:]).max() < 3e-2
    qh = act[:2048].reshape(16, 128)
    kh = act[2048:4096].reshape(16, 128)
    ql2 = qh / np.linalg.norm(qh, axis=1, keepdims=True) / np.sqrt(128.0)
    kl2 = kh / np.linalg.norm(kh, axis=1, keepdims=True)
    assert np.abs(F(qk)[:2048].reshape(16, 128) - ql2).max() < 2e-3
    assert np.abs(F(qk)[2048:].reshape(16, 128) - kl2).max() < 2e-2
    assert np.array_equal(z, proj[8192:12288])
    assert np.array_equal(ncs.reshape(3, 8192)[0], cs.reshape(3, 8192)[1])
    assert np.array_equal(ncs.reshape(3, 8192)[1], cs.reshape(3, 8192)[2])
    assert np.array_equal(ncs.reshape(3, 8192)[2], proj[:8192])


def test_gdn_gates_match_softplus_and_sigmoid():
    rng = np.random.default_rng(12)
    proj = BF(rng.standard_normal(12352).astype(np.float32) * 2.0)
    a_log = BF(rng.uniform(-3.0, 1.0, 32).astype(np.float32))
    dt_bias = BF(rng.standard_normal(32).astype(np.float32))
    decay = np.zeros(32, np.float32); beta = np.zeros(32, np.float32)
    o.tto_gdn_gates(proj, a_log, dt_bias, decay, beta)
    a = F(proj)[12320:12352].astype(np.float64) + F(dt_bias)
    sp = np.log1p(np.exp(-np.abs(a))) + np.maximum(a, 0)
    want = np.exp(-np.exp(F(a_log).astype(np.float64)) * sp)
    assert np.abs(decay - want).max() < 1.5e-2
    b = F(proj)[12288:12320].astype(np.float64)
    assert np.abs(beta - 1.0 / (1.0 + np.exp(-b))).max() < 8e-3


def test_gdn_gate_norm_matches_plain_formula():
    rng = np.random.default_rng(13)
    y = BF(rng.standard_normal(4096).astype(np.float32))
    z = BF(rng.standard_normal(4096).astype(np.float32))
    w = BF((1.0 + 0.1 * rng.standard_normal(128)).astype(np.float32))
    out = np.zeros(4096, np.uint16)
    o.tto_gdn_gate_norm(y, z, w, 32, out)
    yf = F(y).astype(np.float64).reshape(32, 128)
    zf = F(z).astype(np.float64).reshape(32, 128)
    n = yf / np.sqrt((yf ** 2).mean(axis=1, keepdims=True) + 1e-6) * F(w)
    want = zf / (1.0 + np.exp(-zf)) * n
    # three bf16 roundings: relative 2^-8 each
    assert (np.abs(F(out).reshape(32, 128) - want) / np.maximum(1.0, np.abs(want))).max() < 2e-2


def test_rms_closed_form_via_reference():
    # ones -> 0x3F80 for every tree shape and rsqrt order (kernel_reference_test.cpp:95-109)
    if ol.ref is None:
        pytest.skip("oracle/_ref not built")
    ones = np.full(256, 0x3F80, np.uint16)
    for shape in range(6):
        for order in range(2):
            out = np.zeros(256, np.uint16)
            ol.ref.ref_rms_only(ones, ones, 256, shape, order, out)
            assert (out == 0x3F80).all()


def test_prefill_rows_equal_decode_steps():
    """Row r of a block at context c is a decode step at context c+r over the
    same cache (prefill_attention.metal:117-119)."""
    rows, base, cap = 6, 250, 512
    proj = ol.gaussian_bf16(21, rows * 9216)
    q_w = BF((1.0 + 0.1 * ol.gaussian_f32(22, 256)).astype(np.float32))
    k_w = BF((1.0 + 0.1 * ol.gaussian_f32(23, 256)).astype(np.float32))
    keys = np.zeros(2 * cap * 256, np.uint16); values = np.zeros_like(keys)
    kc = ol.gaussian_bf16(24, 2 * cap * 256).reshape(2, cap, 256)
    vc = ol.gaussian_bf16(25, 2 * cap * 256).reshape(2, cap, 256)
    keys.reshape(2, cap, 256)[:, :base] = kc[:, :base]
    values.reshape(2, cap, 256)[:, :base] = vc[:, :base]
    k_dec, v_dec = keys.copy(), values.copy()
    query = np.zeros(rows * 4096, np.uint16); gate = np.zeros_like(query)
    att = np.zeros_like(query)
    o.tto_attention_prefill(proj, q_w, k_w, rows, base, cap, query, gate, keys, values, None, 0,
                            att, 2)
    for r in range(rows):
        q = np.zeros(4096, np.uint16); g = np.zeros(4096, np.uint16)
        o.tto_attn_qk_rope(proj[r * 9216:(r + 1) * 9216], q_w, k_w, base + r, cap, q, g, k_dec,
                           v_dec)
        out = np.zeros(4096, np.uint16)
        o.tto_attention_decode_split(q, g, k_dec, v_dec, base + r, cap, 256, None, out, 1)
        assert np.array_equal(att[r * 4096:(r + 1) * 4096], out)
        assert np.array_equal(query[r * 4096:(r + 1) * 4096], q)
    assert np.array_equal(keys, k_dec) and np.array_equal(values, v_dec)
    # row selection computes the same rows and leaves the others untouched
    sel = np.array([1, 4], np.uint32)
    att2 = np.zeros_like(att)
    o.tto_attention_prefill_rows(query, gate, keys, values, base, cap, sel, 2, att2, 1)
    a, b = att.reshape(rows, 4096), att2.reshape(rows, 4096)
    assert np.array_equal(a[[1, 4]], b[[1, 4]]) and not b[[0, 2, 3, 5]].any()


@pytest.mark.parametrize("steps,chunk", [(5, 64), (64, 64), (130, 64), (40, 8)])
def test_chunked_wy_equals_sequential_fp64(steps, chunk):
    rng = np.random.default_rng(steps)
    dk, dv = 16, 12
    q = rng.standard_normal((steps, dk)); k = rng.standard_normal((steps, dk))
    k /= np.linalg.norm(k, axis=1, keepdims=True)
    v = rng.standard_normal((steps, dv))
    decay = np.exp(rng.uniform(-0.1, 0.0, steps)); beta = rng.uniform(0, 1, steps)
    s0 = rng.standard_normal((dv, dk)) * 0.02
    sa, sb = s0.copy(), s0.copy()
    ya = np.zeros((steps, dv)); yb = np.zeros((steps, dv))
    o.tto_gdn_sequential_f64(q, k, v, decay, beta, steps, dk, dv, sa, ya)
    o.tto_gdn_chunked_f64(q, k, v, decay, beta, steps, dk, dv, chunk, sb, yb)
    assert np.abs(ya - yb).max() < 1e-10 and np.abs(sa - sb).max() < 1e-10
    # and the sequential fp64 form is the textbook matrix recurrence
    S = s0.copy()
    for t in range(steps):
        S = decay[t] * S
        S = S + np.outer(beta[t] * (v[t] - S @ k[t]), k[t])
        assert np.abs(S @ q[t] - ya[t]).max() < 1e-10
    assert np.abs(S - sa).max() < 1e-10


def test_scan_matches_fp64_sequential_within_tolerance():
    """The fp32/bf16 scan against the fp64 delta rule over 96 steps, one head pair."""
    steps = 96
    rng = np.random.default_rng(77)
    qk = np.zeros((steps, 4096), np.float32)
    qn = rng.standard_normal((steps, 16, 128)); kn = rng.standard_normal((steps, 16, 128))
    qn /= np.linalg.norm(qn, axis=2, keepdims=True) * np.sqrt(128.0)
    kn /= np.linalg.norm(kn, axis=2, keepdims=True)
    qk[:, :2048] = qn.reshape(steps, -1); qk[:, 2048:] = kn.reshape(steps, -1)
    qkb = BF(qk.reshape(-1))
    vb = BF(rng.standard_normal(steps * 4096).astype(np.float32))
    decay = np.exp(rng.uniform(-0.1, 0.0, (steps, 32))).astype(np.float32)
    beta = (1 / (1 + np.exp(-rng.standard_normal((steps, 32))))).astype(np.float32)
    s0 = (rng.standard_normal(32 * 128 * 128) * 0.02).astype(np.float32)
    y = np.zeros(steps * 4096, np.uint16); s1 = np.zeros_like(s0)
    o.tto_gdn_scan(qkb, vb, decay.reshape(-1), beta.reshape(-1), steps, s0, y, s1, 4)
    h = 5
    qf = F(qkb).reshape(steps, 4096).astype(np.float64)
    q64 = np.ascontiguousarray(qf[:, (h >> 1) * 128:(h >> 1) * 128 + 128])
    k64 = np.ascontiguousarray(qf[:, 2048 + (h >> 1) * 128:2048 + (h >> 1) * 128 + 128])
    v64 = np.ascontiguousarray(F(vb).reshape(steps, 32, 128)[:, h].astype(np.float64))
    st = s0.reshape(32, 128, 128)[h].astype(np.float64).copy()
    y64 = np.zeros((steps, 128))
    o.tto_gdn_sequential_f64(q64, k64, v64, np.ascontiguousarray(decay[:, h].astype(np.float64)),
                             np.ascontiguousarray(beta[:, h].astype(np.float64)), steps, 128, 128,
                             st, y64)
    assert np.abs(F(y).reshape(steps, 32, 128)[:, h] - y64).max() < 2e-3
    assert np.abs(s1.reshape(32, 128, 128)[h] - st).max() < 1e-4


TAPE_FLOATS = 40 * 16 * (32 * 128 + 16 * 128 + 64)
TAPE_KEYS = 40 * 16 * 32 * 128
TAPE_GATES = TAPE_KEYS + 40 * 16 * 16 * 128


def _scan_inputs(steps, seed):
    rng = np.random.default_rng(seed)
    qn = rng.standard_normal((steps, 16, 128)); kn = rng.standard_normal((steps, 16, 128))
    qn /= np.linalg.norm(qn, axis=2, keepdims=True) * np.sqrt(128.0)
    kn /= np.linalg.norm(kn, axis=2, keepdims=True)
    qk = np.concatenate([qn.reshape(steps, -1), kn.reshape(steps, -1)], axis=1).astype(np.float32)
    qkb = BF(qk.reshape(-1))
    vb = BF(rng.standard_normal(steps * 4096).astype(np.float32))
    decay = np.exp(rng.uniform(-0.1, 0.0, (steps, 32))).astype(np.float32).reshape(-1)
    beta = (1 / (1 + np.exp(-rng.standard_normal((steps, 32))))).astype(np.float32).reshape(-1)
    s0 = (rng.standard_normal(32 * 128 * 128) * 0.02).astype(np.float32)
    return qkb, vb, decay, beta, s0


def test_tape_replay_rebuilds_every_prefix_of_the_scan():
    """The tape has no reference test.  What fixes it: replaying c taped rows must give,
    bit for bit, the state a scan of exactly c rows stores; the taped scan itself must
    not differ from the plain one; and the tape rows are the scan's own operands."""
    steps, layer = 16, 29
    qkb, vb, decay, beta, s0 = _scan_inputs(steps, 4242)
    y0 = np.zeros(steps * 4096, np.uint16); s_plain = np.zeros_like(s0)
    o.tto_gdn_scan(qkb, vb, decay, beta, steps, s0, y0, s_plain, 4)
    tape = np.full(TAPE_FLOATS, np.float32(-77.0))
    y1 = np.zeros_like(y0); s_taped = np.zeros_like(s0)
    o.tto_gdn_scan_tape(qkb, vb, decay, beta, steps, s0, y1, s_taped, tape, layer, 4)
    assert np.array_equal(y0, y1) and np.array_equal(s_plain.view(np.uint32), s_taped.view(np.uint32))
    # only this layer's rows were written
    deltas = tape[:TAPE_KEYS].reshape(40, 16, 32, 128)
    keys = tape[TAPE_KEYS:TAPE_GATES].reshape(40, 16, 16, 128)
    gates = tape[TAPE_GATES:].reshape(40, 16, 32, 2)
    for region in (deltas, keys, gates):
        others = np.delete(region, layer, axis=0)
        assert np.all(others == np.float32(-77.0))
    assert np.array_equal(keys[layer].reshape(steps, 2048),
                          F(qkb).reshape(steps, 4096)[:, 2048:])
    assert np.array_equal(gates[layer, :, :, 0].reshape(-1), decay)
    assert np.array_equal(gates[layer, :, :, 1].reshape(-1), beta)
    for committed in (0, 1, 2, 7, 15, 16):
        want = np.zeros_like(s0)
        if committed:
            yc = np.zeros(committed * 4096, np.uint16)
            o.tto_gdn_scan(qkb[:committed * 4096], vb[:committed * 4096], decay[:committed * 32],
                           beta[:committed * 32], committed, s0, yc, want, 4)
        else:
            want = s0.copy()
        got = np.zeros_like(s0)
        o.tto_gdn_tape_replay(tape, s0, got, committed, layer, 4)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), committed


def test_tape_delta_closed_form_and_long_blocks():
    """From a zero state the first key-value product is zero, so delta = v * beta exactly
    and the replayed state is the outer product k (x) delta; a block longer than the tape
    records nothing."""
    qkb, vb, decay, beta, _ = _scan_inputs(1, 99)
    zero = np.zeros(32 * 128 * 128, np.float32)
    tape = np.zeros(TAPE_FLOATS, np.float32)
    y = np.zeros(4096, np.uint16); s1 = np.zeros_like(zero)
    o.tto_gdn_scan_tape(qkb, vb, decay, beta, 1, zero, y, s1, tape, 0, 2)
    v = F(vb).reshape(32, 128)
    want = v * beta.reshape(32, 1)
    assert np.array_equal(tape[:32 * 128].reshape(32, 128), want.astype(np.float32))
    k = F(qkb)[2048:].reshape(16, 128)
    outer = want[:, :, None] * np.repeat(k, 2, axis=0)[:, None, :]
    assert np.array_equal(s1.reshape(32, 128, 128), outer.astype(np.float32))
    rebuilt = np.zeros_like(zero)
    o.tto_gdn_tape_replay(tape, zero, rebuilt, 1, 0, 2)
    assert np.array_equal(rebuilt, s1)

    steps = 17
    qkb, vb, decay, beta, s0 = _scan_inputs(steps, 100)
    tape = np.full(TAPE_FLOATS, np.float32(3.0))
    y = np.zeros(steps * 4096, np.uint16); s1 = np.zeros_like(s0)
    o.tto_gdn_scan_tape(qkb, vb, decay, beta, steps, s0, y, s1, tape, 5, 4)
    assert np.all(tape == np.float32(3.0))
    y2 = np.zeros_like(y); s2 = np.zeros_like(s0)
    o.tto_gdn_scan(qkb, vb, decay, beta, steps, s0, y2, s2, 4)
    assert np.array_equal(y, y2) and np.array_equal(s1, s2)


def test_conv_tape_rows_are_the_conv_state_of_each_prefix():
    """conv_tape[row] must equal the new conv state of a block that ends at that row
    (computed by the block prefill, an independent path)."""
    rows, layer = 9, 13
    proj = np.zeros(rows * 12352, np.uint16); o.tto_fill_gaussian_bf16(51, 0.0, 0.5, proj, proj.size)
    conv = np.zeros(3 * 8192, np.uint16); o.tto_fill_gaussian_bf16(52, 0.0, 0.5, conv, conv.size)
    cw = np.zeros(4 * 8192, np.uint16); o.tto_fill_gaussian_bf16(53, 0.0, 0.3, cw, cw.size)
    small = np.zeros(32, np.uint16); nw = np.full(128, 0x3F80, np.uint16)
    s0 = np.zeros(32 * 128 * 128, np.float32)
    tape = np.full(40 * 16 * 3 * 8192, 0x7FC0, np.uint16)
    o.tto_gdn_conv_tape(proj, rows, conv, tape, layer)
    windows = tape.reshape(40, 16, 3 * 8192)
    assert np.all(np.delete(windows, layer, axis=0) == 0x7FC0)
    assert np.all(windows[layer, rows:] == 0x7FC0)
    for ending in (1, 2, 3, 4, 9):
        ncs = np.zeros_like(conv); s1 = np.zeros_like(s0)
        gated = np.zeros(ending * 4096, np.uint16)
        o.tto_gdn_prefill(proj[:ending * 12352], ending, conv, cw, small, small, nw, s0, ncs, s1,
                          gated, None, None, None, 4)
        assert np.array_equal(windows[layer, ending - 1], ncs), ending
    untouched = np.full(40 * 16 * 3 * 8192, 0x7FC0, np.uint16)
    big = np.zeros(17 * 12352, np.uint16)
    o.tto_gdn_conv_tape(big, 17, conv, untouched, 0)
    assert np.all(untouched == 0x7FC0)


def test_dense_and_add_against_float64():
    """The stand-in projection is a plain dot product rounded once to bf16 and the
    residual sum is one bf16 addition: both against float64 numpy."""
    rows, k, n = 3, 256, 40
    x = ol.gaussian_bf16(0xD0, rows * k)
    w = ol.gaussian_bf16(0xD1, n * k, 0.0, 0.05)
    out = np.zeros(rows * n, np.uint16)
    o.tto_dense_bf16(x, w, rows, k, n, out, 4)
    want = F(x).astype(np.float64).reshape(rows, k) @ F(w).astype(np.float64).reshape(n, k).T
    got = F(out).reshape(rows, n)
    assert (np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-6).all()
    a = ol.gaussian_bf16(0xD2, 1000); b = ol.gaussian_bf16(0xD3, 1000)
    s = np.zeros(1000, np.uint16)
    o.tto_add_bf16(a, b, 1000, s)
    assert np.array_equal(s, ol.f32_to_bf16(F(a) + F(b)))


def test_rms_only_closed_forms():
    # ones -> ones; uniform 2.0 over 2048 -> 2 / sqrt(4 + 1e-6) rounded twice
    ones = np.full(2048, 0x3F80, np.uint16)
    out = np.zeros(2048, np.uint16)
    o.tto_rms_only(ones, ones, 1, 2048, out)
    assert (out == 0x3F80).all()
    twos = np.full(2048, 0x4000, np.uint16)
    o.tto_rms_only(twos, ones, 1, 2048, out)
    assert (out == 0x3F80).all()


def _q4_dequantised(words, scales, biases, k_size):
    """Plain reading of the format: nibble j of word i is column 8 i + j."""
    w = np.asarray(words, np.uint32)
    nib = np.stack([(w >> (4 * j)) & 0xF for j in range(8)], axis=-1).reshape(-1).astype(np.float64)
    s = np.repeat(F(scales).astype(np.float64), 64)
    b = np.repeat(F(biases).astype(np.float64), 64)
    return s * nib + b


def test_q4_addressing_and_affine_known_answers():
    """The packed-nibble known answers of kernel_reference_test.cpp:327-345: all inputs 1.0 but
    element 1 = 2.0, nibble 10 in the high half of byte 0 (column 1): 20 with unit scale, and
    2 * 20 + 513 * 0.5 with scale 2 and bias 0.5."""
    x = np.full(512, 0x3F80, np.uint16); x[1] = 0x4000
    words = np.zeros(64, np.uint32); words[0] = 0x000000A0
    ones = np.full(8, 0x3F80, np.uint16); zeros = np.zeros(8, np.uint16)
    assert o.tto_q4_dot(x, words, ones, zeros, 512) == 20.0
    twos = np.full(8, 0x4000, np.uint16); halves = np.full(8, 0x3F00, np.uint16)
    assert o.tto_q4_dot(x, words, twos, halves, 512) == 2.0 * 20.0 + 513.0 * 0.5
    # every column in turn: only that column's nibble is set, the input is one-hot there
    for column in (0, 7, 8, 63, 64, 300, 511):
        x = np.zeros(512, np.uint16); x[column] = 0x4040           # 3.0
        words = np.zeros(64, np.uint32); words[column // 8] = np.uint32(13 << (4 * (column % 8)))
        scales = np.zeros(8, np.uint16); scales[column // 64] = 0x3F00   # 0.5 for that group only
        assert o.tto_q4_dot(x, words, scales, zeros, 512) == 0.5 * 13 * 3.0, column


def test_q4_projection_matches_fp64_dequantised_product():
    rng = np.random.default_rng(2718)
    rows, k_size, out_rows = 3, 2048, 40
    x = ol.gaussian_bf16(0x51, rows * k_size, 0.0, 1.0)
    words = rng.integers(0, 2 ** 32, out_rows * k_size // 8, dtype=np.uint64).astype(np.uint32)
    scales = BF(rng.uniform(0.002, 0.01, out_rows * k_size // 64).astype(np.float32))
    biases = BF((-7.5 * F(scales) + rng.normal(0, 1e-3, scales.size)).astype(np.float32))
    out = np.zeros(rows * 48, np.uint16)
    o.tto_q4_project(x, k_size, rows, words, scales, biases, k_size, out_rows, out, 48, 4)
    w = _q4_dequantised(words, scales, biases, k_size).reshape(out_rows, k_size)
    want = F(x).reshape(rows, k_size).astype(np.float64) @ w.T
    got = F(out).reshape(rows, 48)[:, :out_rows]
    assert np.all(out.reshape(rows, 48)[:, out_rows:] == 0)
    # bf16 output rounding dominates: half a step of the result's magnitude
    assert np.all(np.abs(got - want) <= np.maximum(np.abs(want) * 2.0 ** -8, 1e-4))
