"""Sliding-window ring helpers against the cases of the reference's own device-free test,
tests/integrations/vllm_plugin/test_swa_cache_utils.py, restated."""

import numpy as np
import pytest

import __graft_entry__ as entry

entry.ensure_built()

from tt_xla_amd import sliding_ring as R  # noqa: E402


def cdiv(a, b):
    return -(-a // b)


@pytest.mark.parametrize("window,block_size", [(1024, 32), (4096, 32), (512, 64), (1, 32), (8192, 128), (1023, 32)])
def test_window_blocks_alignment_and_slack(window, block_size):
    wb = R.sliding_window_blocks(window, block_size, max_model_len=1_000_000)
    assert wb % R.PAGE_TABLE_STICK_BLOCK_ALIGNMENT == 0 and wb * 4 % 32 == 0
    assert wb >= cdiv(window, block_size) + 1
    assert wb - (cdiv(window, block_size) + 1) < R.PAGE_TABLE_STICK_BLOCK_ALIGNMENT


def test_window_blocks_known_values():
    assert R.sliding_window_blocks(1024, 32, max_model_len=1_000_000) == 40
    assert R.sliding_window_blocks(1024, 32, max_model_len=128) == 8
    assert R.sliding_window_blocks(1024, 32, max_model_len=1024) == R.sliding_window_blocks(1024, 32, 1_000_000)


def test_phys_blocks_bytes_and_width():
    assert R.sliding_ring_phys_blocks(40, 32) == 40 * 32 + 1
    assert 1 + 31 * 40 + 40 == R.sliding_ring_phys_blocks(40, 32)
    assert R.sliding_ring_reserve_bytes(40, 32, 256 * 1024) == (40 * 32 + 1) * 256 * 1024
    assert R.sliding_page_table_width(40, 4096) == 40
    assert R.sliding_page_table_width(40, 8) == 8


def _slots(rows, batch, mapping, free):
    return list(R.assign_ring_slots(rows, batch, mapping, free))


def test_slots_stable_reclaimed_and_partial_pass():
    mapping, free = {}, list(range(4))
    assert _slots(["a", "b", "c"], ["a", "b", "c"], mapping, free) == [0, 1, 2]
    assert _slots(["c", "b"], ["c", "b"], mapping, free) == [2, 1]
    assert mapping["b"] == 1 and mapping["c"] == 2

    mapping, free = {}, list(range(3))
    _slots(["a", "b", "c"], ["a", "b", "c"], mapping, free)
    assert _slots(["c", "d"], ["c", "d"], mapping, free) == [2, 0]
    assert _slots(["c", "d", "e"], ["c", "d", "e"], mapping, free) == [2, 0, 1]

    mapping, free = {}, list(range(2))
    _slots(["a", "b"], ["a", "b"], mapping, free)
    assert _slots(["a"], ["a", "b"], mapping, free) == [0]
    assert mapping["b"] == 1 and 1 not in free

    mapping, free = {}, [0]
    _slots(["a"], ["a"], mapping, free)
    with pytest.raises(IndexError):
        _slots(["a", "b"], ["a", "b"], mapping, free)


def test_page_table_rows():
    wb, width = 8, 8
    slots = np.array([0, 2], dtype=np.int64)
    pt = R.build_sliding_ring_page_table(np.array([0, 3], dtype=np.int64), slots, wb, width)
    assert pt.shape == (2, width)
    for row, slot in enumerate(slots):
        lo, hi = 1 + slot * wb, 1 + (slot + 1) * wb
        assert sorted(pt[row].tolist()) == list(range(lo, hi))
    assert (pt != 0).all()
    pt = R.build_sliding_ring_page_table(np.array([0]), np.array([1]), wb, width)
    assert pt[0].tolist() == [1 + wb + i for i in range(width)]
    pt = R.build_sliding_ring_page_table(np.array([3]), np.array([0]), wb, width)
    assert pt[0].tolist() == [1 + ((3 + i) % wb) for i in range(width)]


@pytest.mark.parametrize("max_model_len,profitable", [(128, False), (512, False), (1024, False), (2048, True), (131072, True)])
def test_profitable_only_past_the_window(max_model_len, profitable):
    assert R.sliding_ring_is_profitable(1024, 32, max_model_len) is profitable


def test_profitability_agrees_with_block_counts():
    for max_model_len in (32, 128, 1024, 2048, 8192, 65536):
        for window in (256, 1024, 4096):
            want = R.sliding_window_blocks(window, 32, max_model_len) < cdiv(max_model_len, 32)
            assert R.sliding_ring_is_profitable(window, 32, max_model_len) is want


def test_pass_geometry_and_fill_guard():
    # below the window: column 0 is block 0 and the position is absolute
    start, rel = R.ring_pass_geometry(np.array([0, 40, 255]), 32, 8)
    assert start.tolist() == [0, 0, 0] and rel.tolist() == [0, 40, 255]
    # past it: the window slides by whole blocks; the relative position keeps the in-block offset
    start, rel = R.ring_pass_geometry(np.array([256, 300, 1000]), 32, 8)
    assert start.tolist() == [1, 2, 24]
    assert rel.tolist() == [256 - 32, 300 - 64, 1000 - 24 * 32]
    assert all(7 * 32 <= r < 8 * 32 for r in rel.tolist())  # always in the ring's last column
    R.check_ring_fill_supported(np.array([0, 5]), np.array([0, 900]), np.array([64, 1]))
    with pytest.raises(NotImplementedError):
        R.check_ring_fill_supported(np.array([1]), np.array([0]), np.array([64]))
    with pytest.raises(NotImplementedError):
        R.check_ring_fill_supported(np.array([0]), np.array([32]), np.array([64]))
