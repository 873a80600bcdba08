"""Seeded input builders shared by the fixture generator and the tests.

Inputs are regenerated from seeds (the exponent-banded xorshift64* stream of
the reference's fixture batteries) instead of being stored, so the committed
fixtures hold only parameters and expected outputs.  Seeds, capacity, contexts
and chain lengths are the reference probes' own
(tools/native/attention_fixture_probe.cpp:27-37, gdn_fixture_probe.cpp:40-45)."""
import numpy as np

ATTN_SEED = 0xA77E1755
ATTN_CAPACITY = 512
ATTN_CHAIN_POSITIONS = 5
ATTN_CONTEXTS = (4, 300, 200)
GDN_SEED = 0x6D46EED5
RESIDUAL_SEED = 0x2E51D0A1
GDN_CHAIN_STEPS = 4
STATE_SAMPLE_STRIDE = 997


def attention_chain_inputs(fill):
    """fill(seed, n) -> uint16[n] banded stream.  One stream, sliced in order."""
    n_proj = ATTN_CHAIN_POSITIONS * 9216
    stream = fill(ATTN_SEED, n_proj + 512)
    proj = stream[:n_proj].reshape(ATTN_CHAIN_POSITIONS, 9216).copy()
    q_w = stream[n_proj:n_proj + 256].copy()
    k_w = stream[n_proj + 256:n_proj + 512].copy()
    return proj, q_w, k_w


def attention_decode_inputs(fill, context):
    cache = 2 * ATTN_CAPACITY * 256
    stream = fill(ATTN_SEED ^ (context * 0x9E3779B97F4A7C15 & 0xFFFFFFFFFFFFFFFF),
                  2 * 4096 + 2 * cache)
    q = stream[:4096].copy()
    gate = stream[4096:8192].copy()
    keys = stream[8192:8192 + cache].copy()
    values = stream[8192 + cache:].copy()
    return q, gate, keys, values


def gdn_inputs(fill, fill_f32):
    n = GDN_CHAIN_STEPS * 12352 + 3 * 8192 + 4 * 8192 + 32 + 32 + 128
    s = fill(GDN_SEED, n)
    o = 0

    def take(k):
        nonlocal o
        out = s[o:o + k].copy()
        o += k
        return out
    proj = take(GDN_CHAIN_STEPS * 12352).reshape(GDN_CHAIN_STEPS, 12352)
    conv_state = take(3 * 8192)
    conv_w = take(4 * 8192)
    a_log = take(32)
    dt_bias = take(32)
    norm_w = take(128)
    state = fill_f32(GDN_SEED + 1, 32 * 128 * 128)
    return proj, conv_state, conv_w, a_log, dt_bias, norm_w, state
