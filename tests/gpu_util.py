"""Shared pieces of the GPU parity tests: one device/queue/library per process
and the tolerance check of the path (max-abs <= 2e-2, mean-abs <= 2e-3 on bf16
outputs widened to fp32)."""
import numpy as np

import oracle_lib as ol

MAX_ABS = 2e-2
MEAN_ABS = 2e-3

_ctx = {}


def gpu():
    if not _ctx:
        from tatara_amd import backend as B
        dev = B.Device()
        _ctx["B"] = B
        _ctx["dev"] = dev
        _ctx["queue"] = dev.create_queue()
        _ctx["lib"] = dev.create_library()
    return _ctx["B"], _ctx["dev"], _ctx["queue"], _ctx["lib"]


def run(record):
    """record(cb) encodes into one compute pass; commits and waits; returns gpu ms."""
    _, _, queue, _ = gpu()
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    record(cb)
    cb.end_compute_pass()
    return cb.commit().wait()


def check_bf16(got, want, what="", max_abs=MAX_ABS, mean_abs=MEAN_ABS, ulps=0):
    """max-abs / mean-abs bar on bf16 outputs.  ulps > 0 widens the max-abs bar to
    that many bf16 steps of the expected value where a step exceeds it: above
    |x| = 4 one bf16 step (2^-5) is already larger than 2e-2, so two correctly
    rounded results of differently ordered sums can differ by more than the bar."""
    g = ol.bf16_to_f32(np.asarray(got, np.uint16).reshape(-1))
    w = ol.bf16_to_f32(np.asarray(want, np.uint16).reshape(-1))
    assert g.shape == w.shape, (what, g.shape, w.shape)
    assert np.isfinite(g).all(), f"{what}: non-finite output"
    err = np.abs(g - w)
    print(f"[parity] {what}: max-abs {err.max():.3e} mean-abs {err.mean():.3e} "
          f"exact {np.mean(np.asarray(got).reshape(-1) == np.asarray(want).reshape(-1)):.4f}",
          flush=True)
    bar = np.full(err.shape, max_abs)
    if ulps:
        step = np.exp2(np.floor(np.log2(np.maximum(np.abs(w), 1e-30))) - 7.0)
        bar = np.maximum(bar, ulps * step)
    worst = int(np.argmax(err - bar))
    assert (err <= bar).all(), f"{what}: |{g[worst]} - {w[worst]}| > {bar[worst]}"
    assert err.mean() <= mean_abs, f"{what}: mean-abs {err.mean()} > {mean_abs}"
    return err.max(), err.mean()


def check_f32(got, want, what, max_abs, mean_abs=None):
    err = np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64))
    assert np.isfinite(np.asarray(got)).all(), f"{what}: non-finite"
    print(f"[parity] {what}: max-abs {err.max():.3e} mean-abs {err.mean():.3e}", flush=True)
    assert err.max() <= max_abs, f"{what}: max-abs {err.max()} > {max_abs}"
    if mean_abs is not None:
        assert err.mean() <= mean_abs
