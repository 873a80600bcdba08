"""Bit equality of the restatement with the unmodified reference scalar model
(oracle/_ref) beyond the stored vectors: Gaussian model-scale inputs and
partition-edge contexts.  Skipped where oracle/_ref is not built."""
import numpy as np
import pytest

import oracle_lib as ol

pytestmark = pytest.mark.skipif(ol.ref is None, reason="oracle/_ref not built")
o, r = ol.oracle, ol.ref


@pytest.mark.parametrize("ctx", [0, 1, 254, 255, 256, 257, 511, 512, 513, 1030])
@pytest.mark.parametrize("kind", ["banded", "gauss"])
def test_attention_decode_paths(ctx, kind):
    cap = 1100
    if kind == "banded":
        gen = lambda s, n: ol.banded_bf16(s, n)
    else:
        gen = lambda s, n: ol.gaussian_bf16(s, n)
    q = gen(100 + ctx, 4096); gate = gen(200 + ctx, 4096)
    keys = gen(300 + ctx, 2 * cap * 256); values = gen(400 + ctx, 2 * cap * 256)
    a = np.zeros(4096, np.uint16); b = np.zeros(4096, np.uint16)
    o.tto_attention_decode(q, gate, keys, values, ctx, cap, a, 4)
    r.ref_attention_decode(q, gate, keys, values, ctx, cap, b)
    assert np.array_equal(a, b)
    nparts = 1 if ctx + 1 <= 256 else (ctx + 256) // 256
    pa = np.zeros(16 * nparts * 258, np.float32); pb = np.zeros_like(pa)
    o.tto_attention_decode_split(q, gate, keys, values, ctx, cap, 256, pa, a, 4)
    r.ref_attention_decode_split(q, gate, keys, values, ctx, cap, 256, pb, b)
    assert np.array_equal(pa.view(np.uint32), pb.view(np.uint32))
    assert np.array_equal(a, b)


@pytest.mark.parametrize("pos", [0, 1, 7, 4095, 32767, 99999, 262143])
def test_qk_rope_positions(pos):
    cap = pos + 1
    proj = ol.gaussian_bf16(500 + pos, 9216)
    q_w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(1, 256))
    k_w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(2, 256))
    outs = []
    for fn in (o.tto_attn_qk_rope, r.ref_attn_qk_rope):
        q = np.zeros(4096, np.uint16); g = np.zeros(4096, np.uint16)
        k = np.zeros(2 * cap * 256, np.uint16); v = np.zeros_like(k)
        fn(proj, q_w, k_w, pos, cap, q, g, k, v)
        outs.append((q, g, k.reshape(2, cap, 256)[:, pos].copy(), v.reshape(2, cap, 256)[:, pos].copy()))
    for x, y in zip(*outs):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_gdn_stages(seed):
    proj = ol.gaussian_bf16(seed, 12352, 0.0, 0.5)
    cs = ol.gaussian_bf16(seed + 10, 3 * 8192, 0.0, 0.5)
    w = ol.gaussian_bf16(seed + 20, 4 * 8192, 0.0, 0.5)
    a_log = ol.f32_to_bf16(ol.uniform_f32(seed + 30, 32, -3.0, 1.0))
    dt_bias = ol.gaussian_bf16(seed + 40, 32)
    norm_w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(seed + 50, 128))
    state = ol.gaussian_f32(seed + 60, 32 * 128 * 128, 0.0, 0.02)
    res = []
    for lib, pre in ((o, "tto_"), (r, "ref_")):
        qk = np.zeros(4096, np.uint16); v = np.zeros(4096, np.uint16)
        z = np.zeros(4096, np.uint16); ncs = np.zeros(3 * 8192, np.uint16)
        getattr(lib, pre + "gdn_prepare")(proj, cs, w, qk, v, z, ncs)
        decay = np.zeros(32, np.float32); beta = np.zeros(32, np.float32)
        getattr(lib, pre + "gdn_gates")(proj, a_log, dt_bias, decay, beta)
        y = np.zeros(4096, np.uint16); so = np.zeros_like(state)
        if lib is o:
            lib.tto_gdn_recurrence(qk, v, decay, beta, state, 16, 32, y, so, 4)
        else:
            lib.ref_gdn_recurrence(qk, v, decay, beta, state, 16, 32, y, so)
        out = np.zeros(4096, np.uint16)
        getattr(lib, pre + "gdn_gate_norm")(y, z, norm_w, 32, out)
        res.append((qk, v, z, ncs, decay.view(np.uint32), beta.view(np.uint32), y,
                    so.view(np.uint32), out))
    for x, y in zip(*res):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("hidden", [256, 2048, 4096])
@pytest.mark.parametrize("kind", ["banded", "gauss"])
def test_rms_only_rows(hidden, kind):
    """tto_rms_only against rms_only_reference (AdjacentPairs tree = 1,
    1/sqrt = order 0), three rows at once."""
    rows = 3
    x = (ol.banded_bf16(0x515 + hidden, rows * hidden) if kind == "banded"
         else ol.gaussian_bf16(0x516 + hidden, rows * hidden, 0.0, 3.0))
    w = ol.f32_to_bf16(1.0 + 0.1 * ol.gaussian_f32(0x517, hidden))
    got = np.zeros(rows * hidden, np.uint16)
    o.tto_rms_only(x, w, rows, hidden, got)
    for row in range(rows):
        want = np.zeros(hidden, np.uint16)
        r.ref_rms_only(np.ascontiguousarray(x[row * hidden:(row + 1) * hidden]), w, hidden, 1, 0, want)
        assert np.array_equal(got[row * hidden:(row + 1) * hidden], want)


@pytest.mark.parametrize("kind", ["banded", "gauss"])
def test_residual_sums(kind):
    """tto_add_bf16 against residual_rms_rounded_sums (kernel_reference.cpp:1160-1165)."""
    n = 3 * 2048
    if kind == "banded":
        a, b = ol.banded_bf16(0x7E5, n), ol.banded_bf16(0x7E6, n)
    else:
        a, b = ol.gaussian_bf16(0x7E7, n, 0.0, 2.0), ol.gaussian_bf16(0x7E8, n, 0.0, 1e-3)
    got = np.zeros(n, np.uint16)
    want = np.zeros(n, np.uint16)
    o.tto_add_bf16(a, b, n, got)
    r.ref_residual_sums(a, b, n, want)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("k_size", [512, 2048, 4096])
def test_q4_dot(k_size):
    """tto_q4_dot against q4_dot_reference in the fused order (kernel_reference.cpp:388-443),
    with the operands of the reference's own trial loop (banded bf16, raw generator words;
    kernel_reference_test.cpp:163-183) and with realistic magnitudes."""
    rng = np.random.default_rng(k_size)
    for trial in range(40):
        if trial % 2 == 0:
            x = ol.banded_bf16(0x4D00 + trial, k_size)
            scales = ol.banded_bf16(0x4E00 + trial, k_size // 64)
            biases = ol.banded_bf16(0x4F00 + trial, k_size // 64)
        else:
            x = ol.gaussian_bf16(0x4D00 + trial, k_size, 0.0, 1.0)
            scales = ol.f32_to_bf16(rng.uniform(0.001, 0.02, k_size // 64).astype(np.float32))
            biases = ol.f32_to_bf16((-8.0 * rng.uniform(0.001, 0.02, k_size // 64)).astype(np.float32))
        words = rng.integers(0, 2 ** 32, k_size // 8, dtype=np.uint64).astype(np.uint32)
        got = np.float32(o.tto_q4_dot(x, words, scales, biases, k_size))
        want = np.float32(r.ref_q4_dot(x, words, scales, biases, k_size))
        assert got.view(np.uint32) == want.view(np.uint32) or (np.isnan(got) and np.isnan(want)), trial
