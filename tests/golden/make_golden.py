"""Writes tests/golden/*.npz by running the UNMODIFIED reference scalar model
(oracle/_ref/libtatara_ref.so, built by `make -C oracle ref` from the reference
tree's tests/native/kernel_reference.cpp) on seeded inputs.

Run in the build container only (needs the reference sources):
    python tests/golden/make_golden.py
The fixtures hold parameters and expected outputs; inputs are regenerated from
the seeds by tests/golden/cases.py."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)
import cases  # noqa: E402
import oracle_lib as ol  # noqa: E402


def ref_fill(seed, n):
    out = np.empty(n, np.uint16)
    ol.ref.ref_fill_banded_bf16(seed, out, n)
    return out


def ref_fill_f32(seed, n):
    return ol.bf16_to_f32(ref_fill(seed, n)).copy()


def main():
    assert ol.ref is not None, "oracle/_ref is not built (reference sources needed)"
    r = ol.ref
    out = {}
    # generator and conversions
    out["banded_first64"] = ref_fill(cases.ATTN_SEED, 64)
    probe = np.array([0.0, 1.0, -2.0, 3.14159, 1e-40, -1e-39, 65504.0, 1e38, 0.1, -0.3],
                     np.float32)
    out["bf16_probe_in"] = probe
    out["bf16_probe_out"] = np.array([r.ref_bf16_from_f32(float(x)) for x in probe], np.uint16)

    # attention: 5 chained positions through qk-rope, decode at context 4
    proj, q_w, k_w = cases.attention_chain_inputs(ref_fill)
    cap = cases.ATTN_CAPACITY
    keys = np.zeros(2 * cap * 256, np.uint16)
    values = np.zeros_like(keys)
    q = np.zeros(4096, np.uint16)
    gate = np.zeros(4096, np.uint16)
    for pos in range(cases.ATTN_CHAIN_POSITIONS):
        r.ref_attn_qk_rope(proj[pos], q_w, k_w, pos, cap, q, gate, keys, values)
    out["chain_q"] = q.copy()
    out["chain_gate"] = gate.copy()
    kc = keys.reshape(2, cap, 256)[:, :cases.ATTN_CHAIN_POSITIONS].copy()
    vc = values.reshape(2, cap, 256)[:, :cases.ATTN_CHAIN_POSITIONS].copy()
    out["chain_keys"] = kc
    out["chain_values"] = vc
    att = np.zeros(4096, np.uint16)
    r.ref_attention_decode(q, gate, keys, values, cases.ATTN_CHAIN_POSITIONS - 1, cap, att)
    out["chain_attended"] = att.copy()
    # rope at a large position (angle reduction matters there)
    qb = np.zeros(4096, np.uint16); gb = np.zeros(4096, np.uint16)
    far = 100000
    r.ref_attn_qk_rope(proj[0], q_w, k_w, far, far + 1, qb, gb,
                       np.zeros(2 * (far + 1) * 256, np.uint16),
                       np.zeros(2 * (far + 1) * 256, np.uint16))
    out["rope_far_q"] = qb.copy()

    for ctx in cases.ATTN_CONTEXTS:
        q, gate, keys, values = cases.attention_decode_inputs(ref_fill, ctx)
        tiled = np.zeros(4096, np.uint16)
        r.ref_attention_decode(q, gate, keys, values, ctx, cap, tiled)
        out[f"decode_tiled_ctx{ctx}"] = tiled
        nparts = 1 if ctx + 1 <= 256 else (ctx + 1 + 255) // 256
        split = np.zeros(4096, np.uint16)
        partials = np.zeros(16 * nparts * 258, np.float32)
        r.ref_attention_decode_split(q, gate, keys, values, ctx, cap, 256, partials, split)
        out[f"decode_split_ctx{ctx}"] = split
        out[f"decode_partials_ctx{ctx}_head5"] = partials.reshape(16, nparts, 258)[5].copy()

    # gated delta net: prepare, gates, 4-step recurrence chain, gate-norm
    proj, conv_state, conv_w, a_log, dt_bias, norm_w, state = cases.gdn_inputs(ref_fill,
                                                                               ref_fill_f32)
    st_in = state.copy()
    cs = conv_state.copy()
    for step in range(cases.GDN_CHAIN_STEPS):
        qk = np.zeros(4096, np.uint16); v = np.zeros(4096, np.uint16)
        z = np.zeros(4096, np.uint16); ncs = np.zeros(3 * 8192, np.uint16)
        r.ref_gdn_prepare(proj[step], cs, conv_w, qk, v, z, ncs)
        decay = np.zeros(32, np.float32); beta = np.zeros(32, np.float32)
        r.ref_gdn_gates(proj[step], a_log, dt_bias, decay, beta)
        y = np.zeros(4096, np.uint16); st_out = np.zeros_like(st_in)
        r.ref_gdn_recurrence(qk, v, decay, beta, st_in, 16, 32, y, st_out)
        gated = np.zeros(4096, np.uint16)
        r.ref_gdn_gate_norm(y, z, norm_w, 32, gated)
        out[f"gdn_qk_{step}"] = qk; out[f"gdn_v_{step}"] = v
        out[f"gdn_decay_{step}"] = decay; out[f"gdn_beta_{step}"] = beta
        out[f"gdn_y_{step}"] = y; out[f"gdn_gated_{step}"] = gated
        out[f"gdn_state_sample_{step}"] = st_out[::cases.STATE_SAMPLE_STRIDE].copy()
        if step == cases.GDN_CHAIN_STEPS - 1:
            out["gdn_conv_state_final"] = ncs.copy()
        st_in, cs = st_out, ncs
    # residual sum and row norm either side of the family (hidden 2048, two rows)
    hidden = 2048
    res_a = ref_fill(cases.RESIDUAL_SEED, 2 * hidden)
    res_b = ref_fill(cases.RESIDUAL_SEED + 1, 2 * hidden)
    norm_w = ref_fill(cases.RESIDUAL_SEED + 2, hidden)
    sums = np.zeros(2 * hidden, np.uint16)
    r.ref_residual_sums(res_a, res_b, 2 * hidden, sums)
    normed = np.zeros(2 * hidden, np.uint16)
    for row in range(2):
        part = np.zeros(hidden, np.uint16)
        r.ref_rms_only(np.ascontiguousarray(sums[row * hidden:(row + 1) * hidden]), norm_w, hidden,
                       1, 0, part)
        normed[row * hidden:(row + 1) * hidden] = part
    out["residual_sums"] = sums
    out["residual_normed"] = normed
    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
