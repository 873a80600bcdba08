"""Context sweep of the stubbed hybrid stack on one GPU: decode waves at a list of
contexts and block prefill of a list of prompt lengths, for 1 and 4 lanes.  Only
the attention-family kernels are counted (per-command device time); the stand-in
projections, norms and residual sums run but are reported separately.  A decode
point also replays the whole wave as one compiled graph (`graph_us_per_wave`:
family, projections and norms together, without the per-command events).

    python -m tatara_amd.sweep [--layers 40] [--decode 1024,4096,...] [--prefill 4096,32768]
                               [--quantized]   (4-bit projections instead of dense bf16)
                               [--attention three]   (rope, split and combine dispatches instead
                                                      of the two-dispatch token form)
prints one JSON line per measured point and a closing summary line."""
import argparse
import json
import sys

import numpy as np

from . import backend as B
from . import stack as S

STUB_KERNELS = {"rms_only", "rms_only_ms", "residual_rms_ms", "dense_bf16", "add_bf16",
                "attn_project_ms", "gdn_project_ms", "gdn_outproj_ms", "attn_project_mfma_ms",
                "gdn_project_mfma_ms", "gdn_outproj_mfma_ms", "attn_project_blk",
                "gdn_project_blk", "outproj_blk"}


def _family_ms(times):
    family = sum(ms for name, ms in times if name not in STUB_KERNELS)
    stub = sum(ms for name, ms in times if name in STUB_KERNELS)
    return family, stub


def measure_decode(dev, queue, lib, weights, layers, lanes, context, repeats=5, attention="token"):
    capacity = ((context + 1 + 1023) // 1024) * 1024
    st = S.StubStack(dev, lib, weights, lanes, capacity, vocab=1024, block_rows=16,
                     attention_form=attention)
    st.context = [context] * lanes
    st._write_tables()
    st.x.write(np.full(lanes * S.HIDDEN, 0x3C00, np.uint16))
    best = None
    for _ in range(repeats):
        cb = queue.create_command_buffer()
        cb.set_profiling(True)
        cb.begin_compute_pass()
        st.record_token_wave(cb, with_head=False)
        cb.end_compute_pass()
        cb.commit().wait()
        fam, stub = _family_ms(cb.command_times())
        if best is None or fam < best[0]:
            best = (fam, stub)
    # the same wave as one compiled graph: device time of whole replays, launch gaps and all
    graph = queue.create_command_buffer()
    graph.begin_compute_pass()
    st.record_token_wave(graph, with_head=False)
    graph.end_compute_pass()
    graph.compile()
    replays = sorted(graph.commit().wait() for _ in range(3 + 2 * repeats))[: 2 * repeats]
    attn_layers = sum(1 for k in S.layer_kinds(layers) if k == "A")
    return {"mode": "decode", "lanes": lanes, "context": context, "layers": layers,
            "family_us_per_layer": round(best[0] * 1e3 / layers, 3),
            "family_us_per_wave": round(best[0] * 1e3, 1),
            "stub_us_per_wave": round(best[1] * 1e3, 1), "split_keys": st.split_keys,
            "graph_us_per_wave": round(replays[len(replays) // 2] * 1e3, 1),
            "kv_bytes_per_wave": attn_layers * lanes * (context + 1) * 2048}


def measure_prefill(dev, queue, lib, weights, layers, lanes, tokens, block_rows=2048):
    capacity = tokens
    st = S.StubStack(dev, lib, weights, lanes, capacity, vocab=1024, block_rows=block_rows)
    st.x.write(np.full(block_rows * S.HIDDEN, 0x3C00, np.uint16))
    family = stub = 0.0
    for lane in range(lanes):
        done = 0
        while done < tokens:
            rows = min(block_rows, tokens - done)
            cb = queue.create_command_buffer()
            cb.set_profiling(True)
            cb.begin_compute_pass()
            st.record_prefill_block(cb, lane, rows, chunked=True)
            cb.end_compute_pass()
            cb.commit().wait()
            f, s = _family_ms(cb.command_times())
            family += f
            stub += s
            st.advance_prefill_block(lane, rows)
            done += rows
    total = lanes * tokens
    return {"mode": "prefill", "lanes": lanes, "tokens": tokens, "layers": layers,
            "family_ms": round(family, 3), "stub_ms": round(stub, 3),
            "family_tok_per_s": round(total / (family * 1e-3)),
            "family_us_per_layer_token": round(family * 1e3 / (layers * total), 4)}


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=40)
    ap.add_argument("--decode", default="1024,4096,16384,32768,65536,100000")
    ap.add_argument("--prefill", default="4096,32768")
    ap.add_argument("--lanes", default="1,4")
    ap.add_argument("--quantized", action="store_true")
    ap.add_argument("--attention", choices=("token", "three"), default="token")
    args = ap.parse_args(argv)
    dev = B.Device()
    queue = dev.create_queue()
    lib = dev.create_library()
    weights = S.make_weights(args.layers, 1024, 0x5EE9, quantized=args.quantized)
    points = []
    for lanes in [int(v) for v in args.lanes.split(",") if v]:
        for context in [int(v) for v in args.decode.split(",") if v]:
            points.append(measure_decode(dev, queue, lib, weights, args.layers, lanes, context,
                                         attention=args.attention))
            print(json.dumps(points[-1]), flush=True)
        for tokens in [int(v) for v in args.prefill.split(",") if v]:
            points.append(measure_prefill(dev, queue, lib, weights, args.layers, lanes, tokens))
            print(json.dumps(points[-1]), flush=True)
    print(json.dumps({"sweep": "hybrid stub stack", "device": dev.name, "points": len(points)}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
