"""Timing of the affine 4-bit projections on one GPU: the three projections of the
attention family (attention in-projection 2048 -> 9216, Gated DeltaNet in-projection
2048 -> 12352, output projection 4096 -> 2048) at decode-wave row counts (`_ms` and
`_mfma_ms` operators) and at block row counts (`_blk` operators), random weights.

    python -m tatara_amd.q4_sweep [--decode 1,4,16] [--block 256,2048,16384] [--repeats 5]
                                  [--weight-sets 24]
prints one JSON line per point: device microseconds per dispatch (best of the repeats,
several dispatches per command buffer), MFMA-rate and weight-stream equivalents."""
import argparse
import json

import numpy as np

from . import backend as B

FAMILIES = {
    "attn_project": {"segments": [8192, 512, 512], "k": 2048, "out": 10, "threads": 128},
    "gdn_project": {"segments": [8192, 4096, 32, 32], "k": 2048, "out": 13, "threads": 128},
    "gdn_outproj": {"segments": [2048], "k": 4096, "out": 4, "threads": 64},
}
BLOCK_NAMES = {"attn_project": "attn_project_blk", "gdn_project": "gdn_project_blk",
               "gdn_outproj": "outproj_blk"}


def _bf16(values):
    bits = np.asarray(values, np.float32).view(np.uint32)
    return ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)


def _bind(dev, family, rng):
    bindings = {}
    for index, rows in enumerate(family["segments"]):
        k = family["k"]
        scales = rng.uniform(0.002, 0.01, rows * k // 64).astype(np.float32)
        slot = 1 + 3 * index
        bindings[slot] = dev.buffer_from(
            rng.integers(0, 2 ** 32, rows * k // 8, dtype=np.uint64).astype(np.uint32))
        bindings[slot + 1] = dev.buffer_from(_bf16(scales))
        bindings[slot + 2] = dev.buffer_from(_bf16(-7.5 * scales))
    return bindings


def measure(dev, queue, lib, name, rows, block, repeats, dispatches=5, matrix_unit=False,
            weight_sets=1):
    """weight_sets > 1 rotates that many distinct weight sets through the dispatches of a
    command buffer: with more than 256 MB of them (the last-level cache) every dispatch
    streams its weights from HBM, as the layers of a model do."""
    family = FAMILIES[name]
    rng = np.random.default_rng(rows)
    total, k = sum(family["segments"]), family["k"]
    weights = [_bind(dev, family, rng) for _ in range(weight_sets)]
    shared = {0: dev.buffer_from(_bf16(rng.standard_normal(rows * k))),
              family["out"]: dev.create_buffer(rows * total * 2)}
    dispatches = max(dispatches, weight_sets)
    groups = (total + family["threads"] // 32 - 1) // (family["threads"] // 32)
    slot = family["out"] + 1
    if block:
        operator = BLOCK_NAMES[name]
        constants = {slot: rows, slot + 1: k} if name == "gdn_outproj" else {slot: rows}
        grid = (groups, 1, 1)
    else:
        operator = name + ("_mfma_ms" if matrix_unit else "_ms")
        tile = 16
        constants = ({slot: rows, slot + 1: total, slot + 2: tile} if name == "gdn_outproj"
                     else {slot: rows, slot + 1: tile})
        grid = (groups, (rows + tile - 1) // tile, 1)
    pipeline = lib.pipeline(operator)
    best = None
    for _ in range(repeats + 1):
        cb = queue.create_command_buffer()
        cb.begin_compute_pass()
        for index in range(dispatches):
            cb.encode(pipeline, {**weights[index % weight_sets], **shared}, constants, grid,
                      (family["threads"], 1, 1))
            cb.barrier()
        cb.end_compute_pass()
        ms = cb.commit().wait() / dispatches
        best = ms if best is None else min(best, ms)
    weight_bytes = total * k * (0.5 + 4.0 / 64.0)
    return {"operator": operator, "rows": rows, "weight_sets": weight_sets,
            "us": round(best * 1e3, 1),
            "tflops": round(2.0 * rows * total * k / best / 1e9, 1),
            "weight_gb_per_s": round(weight_bytes / best / 1e6, 1)}


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--decode", default="1,4,16")
    parser.add_argument("--block", default="256,2048,16384")
    parser.add_argument("--repeats", type=int, default=5)
    parser.add_argument("--weight-sets", type=int, default=1,
                        help="distinct weight sets rotated through a command buffer (24 keeps "
                             "the decode forms out of the last-level cache)")
    args = parser.parse_args()
    dev = B.Device()
    queue = dev.create_queue()
    lib = dev.create_library()
    for block, rows_list in ((False, args.decode), (True, args.block)):
        for rows in [int(r) for r in rows_list.split(",") if r]:
            for name in FAMILIES:
                sets = 1 if block else args.weight_sets
                print(json.dumps(measure(dev, queue, lib, name, rows, block, args.repeats,
                                         weight_sets=sets)), flush=True)
                if not block:   # the same wave on the matrix unit
                    print(json.dumps(measure(dev, queue, lib, name, rows, block, args.repeats,
                                             matrix_unit=True, weight_sets=sets)), flush=True)


if __name__ == "__main__":
    main()
