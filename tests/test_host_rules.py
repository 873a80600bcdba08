"""Host-side planning rules that exist twice: the C++ runtime's (checked by
tests/native/geometry_contract_test.cpp) and their Python mirror in tatara_amd.stack,
which bench.py and the stub stack use.  The same figures are pinned here, so the two
cannot drift apart unnoticed."""
import pytest

from tatara_amd import stack as S


@pytest.mark.parametrize("visible,split,live", [
    ([32768] * 4, 1024, 256),                    # the headline wave
    ([32768], 256, 256),
    ([100000], 800, 250),
    ([16384] * 4, 512, 256),
    ([1], 128, 2),
    ([262144] * 16, 32768, 256),
    ([100000] * 4, 3136, 256),
    ([32768] * 3, 800, 246),                     # 768 keys would be 258 workgroups
    ([32768, 30000, 24576, 8192], 768, 252),     # config 3's ragged lanes
    ([65536, 50001, 40001, 30001, 20001, 10001, 5001, 1001], 1792, 254),
    ([], 128, 0),
])
def test_split_keys_rule_matches_the_runtime(visible, split, live):
    assert S.choose_split_keys(visible) == split
    assert S.split_workgroups(visible, split) == live
    assert split % 32 == 0 and split >= 128
    assert live <= 256


def test_split_keys_rule_never_oversubscribes():
    """Whatever the depths, the workgroups that hold keys fit the compute units (the
    measured cost of one too many is a third of the walk), and one notch finer would not."""
    import random
    rng = random.Random(0x5EED)
    for _ in range(300):
        lanes = rng.randint(1, 16)
        visible = [rng.randint(257, 262144) for _ in range(lanes)]
        for units in (256, 304, 64):
            split = S.choose_split_keys(visible, units)
            assert S.split_workgroups(visible, split) <= units
            if split > 128:
                share = -(-2 * sum(visible) // units)
                assert split - 32 < share or S.split_workgroups(visible, split - 32) > units


@pytest.mark.parametrize("rows,units,splits,scratch", [
    (2048, 256, 2, 512 + 128 * 2 * 270336), (1024, 256, 4, 256 + 64 * 4 * 270336),
    (512, 256, 8, 256 + 32 * 8 * 270336), (256, 256, 8, 256 + 16 * 8 * 270336),
    (13, 256, 8, 256 + 2 * 8 * 270336), (4096, 256, 1, 0), (16384, 256, 1, 0),
    (2048, 304, 2, 512 + 128 * 2 * 270336), (2048, 128, 1, 0), (2049, 256, 1, 0), (0, 256, 1, 0)])
def test_flash_prefill_sharing_plan(rows, units, splits, scratch):
    """tt_flash_prefill_splits: as many workgroups per position tile (32 rows x 2 kv heads) as fit
    the compute units, between one and eight; tt_flash_prefill_scratch_bytes: a 4-byte arrival
    count per tile and kv head, padded to 256 bytes, and 270,336 bytes per sharer - 32 f32x4 of O
    and one of {reference, row sum} for each of 512 lanes."""
    from tatara_amd import backend as B
    assert B.flash_prefill_splits(rows, 32768, units) == splits
    assert B.flash_prefill_splits(rows, 480, units) == 1     # a longest walk under 16 key tiles
    assert B.flash_prefill_splits(rows, 481, units) == splits
    assert B.flash_prefill_scratch_bytes(rows, splits) == scratch
    assert B.flash_prefill_scratch_bytes(rows, 1) == 0
