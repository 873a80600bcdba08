"""Affine 4-bit projections either side of the attention family on the GPU, through
the C ABI, against the CPU checker (itself bit-equal to the reference's
q4_dot_reference).

Decode operators (`*_project`, `*_project_ms{,_v2}`, `gdn_outproj{,_ms,_ms_v2}`) keep the
reference's sequence of operations, so every bf16 output must be the checker's bit
pattern.  The block operators (`*_blk`) are held to the path's bar (max-abs 2e-2,
mean-abs 2e-3) with a 2-step allowance on large values: their sums run in another
order."""
import numpy as np
import pytest

import oracle_lib as ol
from gpu_util import check_bf16, gpu, run

pytestmark = pytest.mark.gpu
o = ol.oracle

ATTN = {"name": "attn_project", "segments": [8192, 512, 512], "k": 2048, "out": 10, "threads": 128}
GDN = {"name": "gdn_project", "segments": [8192, 4096, 32, 32], "k": 2048, "out": 13, "threads": 128}
OUT = {"name": "gdn_outproj", "segments": [2048], "k": 4096, "out": 4, "threads": 64}


def _matrix(seed, rows, k):
    rng = np.random.default_rng(seed)
    words = rng.integers(0, 2 ** 32, rows * k // 8, dtype=np.uint64).astype(np.uint32)
    scales = ol.f32_to_bf16(rng.uniform(0.002, 0.01, rows * k // 64).astype(np.float32))
    biases = ol.f32_to_bf16((-7.5 * ol.bf16_to_f32(scales) +
                             rng.normal(0.0, 1e-3, scales.size)).astype(np.float32))
    return words, scales, biases


def _family(dev, family, seed):
    host, device = [], {}
    for index, rows in enumerate(family["segments"]):
        w, s, b = _matrix(seed + index, rows, family["k"])
        host.append((w, s, b))
        slot = 1 + 3 * index
        device[slot], device[slot + 1], device[slot + 2] = (dev.buffer_from(w), dev.buffer_from(s),
                                                            dev.buffer_from(b))
    return host, device


def _groups(family):
    per = family["threads"] // 32
    return (sum(family["segments"]) + per - 1) // per


def _expected(family, host, x, rows, out_stride=None):
    total = sum(family["segments"])
    stride = out_stride or total
    want = np.zeros(rows * stride, np.uint16)
    first = 0
    for (w, s, b), n in zip(host, family["segments"]):
        o.tto_q4_project(x, family["k"], rows, w, s, b, family["k"], n, want[first:], stride, 8)
        first += n
    return want


@pytest.mark.parametrize("family", [ATTN, GDN, OUT], ids=lambda f: f["name"])
def test_single_row_projection_bit_for_bit(family):
    print(f"[case] {family['name']} one row", flush=True)
    B, dev, queue, lib = gpu()
    host, bindings = _family(dev, family, 0x9000)
    x = ol.gaussian_bf16(0x9100, family["k"], 0.0, 1.0)
    total = sum(family["segments"])
    out = dev.create_buffer(total * 2)
    bindings[0] = dev.buffer_from(x)
    bindings[family["out"]] = out
    ms = run(lambda cb: cb.encode(lib.pipeline(family["name"]), bindings, {}, (_groups(family), 1, 1),
                                  (family["threads"], 1, 1)))
    assert np.array_equal(out.read(np.uint16), _expected(family, host, x, 1))
    print(f"[time] {family['name']}: {ms * 1e3:.1f} us", flush=True)


@pytest.mark.parametrize("rows,tile", [(1, 16), (3, 2), (16, 16), (13, 5)])
@pytest.mark.parametrize("family,suffix", [(ATTN, "_ms"), (ATTN, "_ms_v2"), (GDN, "_ms"),
                                           (GDN, "_ms_v2"), (OUT, "_ms"), (OUT, "_ms_v2")],
                         ids=["attn", "attn_v2", "gdn", "gdn_v2", "out", "out_v2"])
def test_wave_projection_bit_for_bit(family, suffix, rows, tile):
    name = family["name"] + suffix
    print(f"[case] {name} rows={rows} tile={tile}", flush=True)
    B, dev, queue, lib = gpu()
    host, bindings = _family(dev, family, 0x9200)
    x = ol.gaussian_bf16(0x9300 + rows, rows * family["k"], 0.0, 1.0)
    total = sum(family["segments"])
    strided = family is OUT
    stride = total + 64 if strided else total
    out = dev.buffer_from(np.full(rows * stride, 0x7FC0, np.uint16))
    bindings[0] = dev.buffer_from(x)
    bindings[family["out"]] = out
    slot = family["out"] + 1
    constants = {slot: rows, slot + 1: stride, slot + 2: tile} if strided else {slot: rows, slot + 1: tile}
    tiles = (rows + tile - 1) // tile
    ms = run(lambda cb: cb.encode(lib.pipeline(name), bindings, constants, (_groups(family), tiles, 1),
                                  (family["threads"], 1, 1)))
    got = out.read(np.uint16).reshape(rows, stride)
    want = _expected(family, host, x, rows, stride).reshape(rows, stride)
    assert np.array_equal(got[:, :total], want[:, :total])
    assert np.all(got[:, total:] == 0x7FC0)
    print(f"[time] {name} rows={rows} tile={tile}: {ms * 1e3:.1f} us", flush=True)


def test_wave_projection_of_every_small_bf16_input_bit_for_bit():
    """attn_project_ms on inputs that run through every bf16 bit pattern below 2^30 in
    magnitude (the subnormals among them), ordered by magnitude so that a row of 2048 holds
    neighbouring binades: what the reference's model does with subnormal inputs, products
    and sums (q4_dot_reference), bit for bit."""
    print("[case] attn_project_ms over every bf16 input below 2^30", flush=True)
    B, dev, queue, lib = gpu()
    family = ATTN
    host, bindings = _family(dev, family, 0x9800)
    patterns = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    small = patterns[(patterns & 0x7FFF) < 0x4E80]
    small = small[np.argsort(small & 0x7FFF, kind="stable")]
    rows = 16
    x = np.resize(small, rows * family["k"])            # 32768 values: the 32768 smallest magnitudes
    assert x.size <= small.size
    total = sum(family["segments"])
    out = dev.create_buffer(rows * total * 2)
    bindings[0] = dev.buffer_from(x)
    bindings[family["out"]] = out
    slot = family["out"] + 1
    run(lambda cb: cb.encode(lib.pipeline("attn_project_ms"), bindings, {slot: rows, slot + 1: 16},
                             (_groups(family), 1, 1), (family["threads"], 1, 1)))
    got = out.read(np.uint16)
    want = _expected(family, host, x, rows)
    differ = np.flatnonzero(got != want)
    assert differ.size == 0, (f"{differ.size} of {got.size} outputs differ, first: row "
                              f"{differ[0] // total} got {got[differ[0]]:#06x} want {want[differ[0]]:#06x}")


@pytest.mark.parametrize("rows", [1, 2, 4, 13, 16])
@pytest.mark.parametrize("family", [ATTN, GDN, OUT], ids=lambda f: f["name"])
def test_wave_projection_on_the_matrix_unit(family, rows):
    """The _mfma_ms forms (no reference counterpart): the bindings and grids of the _ms forms,
    sums in another order - held to the path's bar, with the share of bit-identical outputs
    printed."""
    name = family["name"] + "_mfma_ms"
    print(f"[case] {name} rows={rows}", flush=True)
    B, dev, queue, lib = gpu()
    host, bindings = _family(dev, family, 0x9800)
    x = ol.gaussian_bf16(0x9900 + rows, rows * family["k"], 0.0, 1.0)
    total = sum(family["segments"])
    strided = family is OUT
    stride = total + 64 if strided else total
    out = dev.buffer_from(np.full(rows * stride, 0x7FC0, np.uint16))
    bindings[0] = dev.buffer_from(x)
    bindings[family["out"]] = out
    slot = family["out"] + 1
    constants = {slot: rows, slot + 1: stride, slot + 2: 16} if strided else {slot: rows, slot + 1: 16}
    ms = run(lambda cb: cb.encode(lib.pipeline(name), bindings, constants, (_groups(family), 1, 1),
                                  (family["threads"], 1, 1)))
    got = out.read(np.uint16).reshape(rows, stride)
    want = _expected(family, host, x, rows, stride).reshape(rows, stride)
    check_bf16(got[:, :total], want[:, :total], name, ulps=2)
    assert np.all(got[:, total:] == 0x7FC0)
    print(f"[time] {name} rows={rows}: {ms * 1e3:.1f} us", flush=True)


@pytest.mark.parametrize("family,name", [(ATTN, "attn_project_blk"), (GDN, "gdn_project_blk"),
                                         (OUT, "outproj_blk")], ids=["attn", "gdn", "out"])
@pytest.mark.parametrize("rows", [1, 37, 130])
def test_block_projection(family, name, rows):
    print(f"[case] {name} rows={rows}", flush=True)
    B, dev, queue, lib = gpu()
    host, bindings = _family(dev, family, 0x9400)
    x = ol.gaussian_bf16(0x9500 + rows, rows * family["k"], 0.0, 1.0)
    total = sum(family["segments"])
    out = dev.create_buffer(rows * total * 2)
    bindings[0] = dev.buffer_from(x)
    bindings[family["out"]] = out
    slot = family["out"] + 1
    constants = {slot: rows, slot + 1: family["k"]} if family is OUT else {slot: rows}
    ms = run(lambda cb: cb.encode(lib.pipeline(name), bindings, constants, (_groups(family), 1, 1),
                                  (family["threads"], 1, 1)))
    check_bf16(out.read(np.uint16), _expected(family, host, x, rows), name, ulps=2)
    print(f"[time] {name} rows={rows}: {ms * 1e3:.1f} us", flush=True)


@pytest.mark.parametrize("family,name", [(ATTN, "attn_project_blk"), (GDN, "gdn_project_blk"),
                                         (OUT, "outproj_blk")], ids=["attn", "gdn", "out"])
@pytest.mark.parametrize("rows", [256, 257, 700, 2048, 16384])
def test_block_projection_over_several_row_tiles(family, name, rows):
    """Blocks that span more than one 256-row tile of the block kernel, up to the 16384 rows
    the benchmark times, among them the reference's 2048-row block, whose last, partly filled
    round of tiles is shared between workgroups (as that of most sizes here is): every output
    row is produced, and a sample of rows - the first and last of the block, the rows either
    side of each tile boundary sampled, a few inside - is held to the checker."""
    print(f"[case] {name} rows={rows} (sampled rows)", flush=True)
    B, dev, queue, lib = gpu()
    host, bindings = _family(dev, family, 0x9600)
    k = family["k"]
    x = ol.gaussian_bf16(0x9700 + rows, rows * k, 0.0, 1.0)
    total = sum(family["segments"])
    out = dev.buffer_from(np.full(rows * total, 0x7FC0, np.uint16))      # NaN until written
    bindings[0] = dev.buffer_from(x)
    bindings[family["out"]] = out
    slot = family["out"] + 1
    constants = {slot: rows, slot + 1: k} if family is OUT else {slot: rows}
    run(lambda cb: cb.encode(lib.pipeline(name), bindings, constants, (_groups(family), 1, 1),
                             (family["threads"], 1, 1)))
    got = out.read(np.uint16).reshape(rows, total)
    assert not np.any((got & 0x7FFF) > 0x7F80), "an output row was left unwritten"
    sample = {0, rows - 1, rows // 2, rows // 3}
    for edge in range(256, rows, 256 if rows <= 1024 else 4096):
        sample.update({edge - 1, edge})
    sample = sorted(r for r in sample if 0 <= r < rows)
    xs = np.ascontiguousarray(x.reshape(rows, k)[sample]).reshape(-1)
    want = _expected(family, host, xs, len(sample)).reshape(len(sample), total)
    check_bf16(got[sample], want, f"{name} rows {sample[:4]}..{sample[-1]}", ulps=2)


@pytest.mark.parametrize("rows", [2, 4, 13, 16])
@pytest.mark.parametrize("family", [ATTN, GDN], ids=lambda f: f["name"])
def test_wave_projection_with_the_norm_in_its_prologue(family, rows):
    """`*_project_rms_mfma_ms` (no reference counterpart) on rows that have not been normed
    against `rms_only_ms` followed by `*_project_mfma_ms`: the same bits, and the norm the
    fused form applies is the checker's."""
    name = family["name"]
    print(f"[case] {name}_rms_mfma_ms rows={rows}", flush=True)
    B, dev, queue, lib = gpu()
    host, bindings = _family(dev, family, 0x9A00)
    x = ol.gaussian_bf16(0x9B00 + rows, rows * 2048, 0.0, 1.5)
    weight = ol.gaussian_bf16(0x9C00, 2048, 1.0, 0.25)
    total = sum(family["segments"])
    b_x, b_w = dev.buffer_from(x), dev.buffer_from(weight)
    b_normed = dev.create_buffer(rows * 2048 * 2)
    two_step = dev.buffer_from(np.full(rows * total, 0x7FC0, np.uint16))
    fused = dev.buffer_from(np.full(rows * total, 0x7FC0, np.uint16))
    out, slot = family["out"], family["out"] + 1
    grid = (_groups(family), 1, 1)

    def rec(cb):
        cb.encode(lib.pipeline("rms_only_ms"), {0: b_x, 1: b_w, 2: b_normed}, {3: 2048, 4: 2048},
                  (1, rows), (512,))
        cb.barrier()
        cb.encode(lib.pipeline(name + "_mfma_ms"), {**bindings, 0: b_normed, out: two_step},
                  {slot: rows, slot + 1: 16}, grid, (family["threads"], 1, 1))
        cb.encode(lib.pipeline(name + "_rms_mfma_ms"), {**bindings, 0: b_x, out: fused, out + 3: b_w},
                  {slot: rows, slot + 1: 16}, grid, (family["threads"], 1, 1))
    run(rec)
    normed = np.zeros(rows * 2048, np.uint16)
    o.tto_rms_only(x, weight, rows, 2048, normed)
    assert np.array_equal(b_normed.read(np.uint16), normed)
    assert np.array_equal(fused.read(np.uint16), two_step.read(np.uint16))
    check_bf16(fused.read(np.uint16), _expected(family, host, normed, rows), name + "_rms_mfma_ms", ulps=2)


@pytest.mark.parametrize("in_place", [False, True], ids=["apart", "in-place"])
@pytest.mark.parametrize("rows", [2, 4, 16])
def test_wave_out_projection_with_the_residual_in_its_epilogue(rows, in_place):
    """`gdn_outproj_residual_mfma_ms` (no reference counterpart) against `gdn_outproj_mfma_ms`
    followed by the residual sum of `residual_rms_ms`: the same bits, with the output in a
    buffer of its own and in the residual buffer itself."""
    print(f"[case] gdn_outproj_residual_mfma_ms rows={rows} in_place={in_place}", flush=True)
    B, dev, queue, lib = gpu()
    host, bindings = _family(dev, OUT, 0x9D00)
    mixed = ol.gaussian_bf16(0x9E00 + rows, rows * 4096, 0.0, 1.0)
    x = ol.gaussian_bf16(0x9F00 + rows, rows * 2048, 0.0, 1.0)
    weight = ol.gaussian_bf16(0xA000, 2048, 1.0, 0.25)
    b_mixed, b_x, b_w = dev.buffer_from(mixed), dev.buffer_from(x), dev.buffer_from(weight)
    b_delta = dev.create_buffer(rows * 2048 * 2)
    b_sum, b_normed = dev.create_buffer(rows * 2048 * 2), dev.create_buffer(rows * 2048 * 2)
    b_fused = dev.buffer_from(x) if in_place else dev.create_buffer(rows * 2048 * 2)
    b_before = b_fused if in_place else b_x

    def rec(cb):
        cb.encode(lib.pipeline("gdn_outproj_mfma_ms"), {**bindings, 0: b_mixed, 4: b_delta},
                  {5: rows, 6: 2048, 7: 16}, (1024, 1, 1), (64, 1, 1))
        cb.barrier()
        cb.encode(lib.pipeline("residual_rms_ms"), {0: b_x, 1: b_delta, 2: b_sum, 3: b_w, 4: b_normed},
                  {5: 2048, 6: 2048, 7: 2048}, (1, rows), (512,))
        cb.encode(lib.pipeline("gdn_outproj_residual_mfma_ms"),
                  {**bindings, 0: b_mixed, 4: b_fused, 8: b_before}, {5: rows, 6: 2048, 7: 16},
                  (1024, 1, 1), (64, 1, 1))
    run(rec)
    assert np.array_equal(b_fused.read(np.uint16), b_sum.read(np.uint16))
    delta = ol.bf16_to_f32(b_delta.read(np.uint16))
    want = ol.f32_to_bf16(ol.bf16_to_f32(x) + delta)
    assert np.array_equal(b_fused.read(np.uint16), want)


def test_projection_validation():
    B, dev, queue, lib = gpu()
    host, bindings = _family(dev, ATTN, 0x9600)
    bindings[0] = dev.create_buffer(16 * 2048 * 2)
    bindings[10] = dev.create_buffer(16 * 9216 * 2)
    cb = queue.create_command_buffer()
    cb.begin_compute_pass()
    ms = lib.pipeline("attn_project_ms")
    cases = [
        (bindings, {11: 17, 12: 16}, (2304, 2, 1), 15),     # more rows than a wave holds
        (bindings, {11: 16, 12: 17}, (2304, 1, 1), 15),     # tile beyond the batch maximum
        (bindings, {11: 16, 12: 4}, (2304, 3, 1), 15),      # tiles do not cover the rows
        (bindings, {11: 16, 12: 4}, (2303, 4, 1), 15),      # groups do not cover the output rows
        ({**bindings, 4: dev.create_buffer(512 * 256 * 4 - 4)}, {11: 4, 12: 4}, (2304, 1, 1), 10),
        ({**bindings, 10: dev.create_buffer(4 * 9216 * 2 - 2)}, {11: 4, 12: 4}, (2304, 1, 1), 10),
        ({**bindings, 0: dev.create_buffer(4 * 2048 * 2 - 2)}, {11: 4, 12: 4}, (2304, 1, 1), 10),
    ]
    for buffers, constants, grid, status in cases:
        with pytest.raises(B.BackendError) as e:
            cb.encode(ms, buffers, constants, grid, (128, 1, 1))
        assert e.value.status == status, (constants, grid)
    host, out_bindings = _family(dev, OUT, 0x9700)
    out_bindings[0] = dev.create_buffer(4 * 4096 * 2)
    out_bindings[4] = dev.create_buffer(4 * 2048 * 2)
    with pytest.raises(B.BackendError) as e:   # output stride below the hidden width
        cb.encode(lib.pipeline("gdn_outproj_ms"), out_bindings, {5: 4, 6: 2047, 7: 4}, (1024, 1, 1),
                  (64, 1, 1))
    assert e.value.status == 8
    with pytest.raises(B.BackendError) as e:   # input width not a multiple of 512
        cb.encode(lib.pipeline("outproj_blk"), out_bindings, {5: 4, 6: 4000}, (1024, 1, 1), (64, 1, 1))
    assert e.value.status == 15
    # the block form moves 16-byte pieces: an input bound 2 bytes off is refused when encoded
    blk_bindings = dict(bindings)
    blk_bindings[0] = (dev.create_buffer(64 * 2048 * 2 + 16), 2)
    blk_bindings[10] = dev.create_buffer(64 * 9216 * 2)
    with pytest.raises(B.BackendError) as e:
        cb.encode(lib.pipeline("attn_project_blk"), blk_bindings, {11: 64}, (2304, 1, 1), (128, 1, 1))
    assert e.value.status == 10
    assert cb.command_count == 0
