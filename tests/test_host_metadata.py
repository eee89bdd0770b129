"""Host-side paged metadata (tt_xla_amd.metadata) against the cases the reference's own
device-free tests hold for the same functions:
tests/integrations/vllm_plugin/test_fill_page_table_width.py and
tests/integrations/vllm_plugin/test_prepare_inputs_block_alignment.py, plus the
page-table / cache-position / prefix-offset rules of model_runner.py:1722-2016 checked
through what they must mean for the cache (which block and slot each token lands in)."""

import numpy as np
import pytest
import torch

import __graft_entry__ as entry

entry.ensure_built()

from tt_xla_amd import metadata as M  # noqa: E402

_UNCLAMPED = 1 << 20
_BOUND_CASES = [(1, 32), (32, 8), (32, 32), (128, 32), (2048, 32), (2048, 64), (2048, 128),
                (4096, 32), (131072, 32), (131072, 64)]
BLOCK = 32


# ---- fill page table width (reference test_fill_page_table_width.py) ----------------------
@pytest.mark.parametrize("max_num_tokens,block_size", _BOUND_CASES)
def test_width_covers_largest_step_and_is_aligned(max_num_tokens, block_size):
    width = M.fill_page_table_width(max_num_tokens, block_size, _UNCLAMPED)
    assert width * block_size >= max_num_tokens
    assert width > 0 and width % 8 == 0


@pytest.mark.parametrize("read_width", [64, 65, 4096, _UNCLAMPED])
def test_width_never_wider_than_read_table(read_width):
    assert M.fill_page_table_width(2048, 32, read_width) <= read_width


def test_width_clamped_when_read_table_narrower():
    assert M.fill_page_table_width(128, 32, 4) == 4


@pytest.mark.parametrize("read_width", [1, 7, 8, 63])
def test_width_rejects_short_read_table(read_width):
    with pytest.raises(AssertionError, match="cannot cover"):
        M.fill_page_table_width(2048, 32, read_width)


def test_width_follows_block_size():
    assert M.fill_page_table_width(2048, 32, _UNCLAMPED) == 64
    assert M.fill_page_table_width(2048, 128, _UNCLAMPED) == 16
    assert M.fill_page_table_width(2048, 32, 131072 // 32) == 64


def test_copy_narrow_stages_leading_columns():
    host = torch.arange(2 * 16, dtype=torch.int32).reshape(2, 16)
    dev = torch.zeros((2, 8), dtype=torch.int32)
    M.copy_narrow_fill_page_table(dev, host, block_size=32, step_tokens=8 * 32)
    assert torch.equal(dev, host[:, :8])


def test_copy_narrow_rejects_short_table():
    host = torch.zeros((2, 16), dtype=torch.int32)
    dev = torch.zeros((2, 8), dtype=torch.int32)
    with pytest.raises(AssertionError, match="cannot cover this step"):
        M.copy_narrow_fill_page_table(dev, host, block_size=32, step_tokens=8 * 32 + 1)


# ---- block alignment (reference test_prepare_inputs_block_alignment.py) -------------------
def test_row_lead_cases():
    assert M.row_lead(np.array([0, 32, 64, 256], dtype=np.int32), BLOCK).tolist() == [0, 0, 0, 0]
    assert M.row_lead(np.array([41, 44, 63, 65], dtype=np.int32), BLOCK).tolist() == [9, 12, 31, 1]
    assert M.row_lead(np.array([41], dtype=np.int64), BLOCK).dtype == np.int32


@pytest.mark.parametrize("computed,want", [
    ([33, 40, 63], 3), ([41, 20], 1), ([33, 40, 80, 41], 2), ([41], 1), ([], 0),
])
def test_same_block_run_cases(computed, want):
    assert M.same_block_run(np.array(computed, dtype=np.int32), BLOCK) == want


def test_same_block_run_never_zero_for_nonempty():
    for computed in ([0, 1], [41, 20], [63, 64], [7]):
        assert M.same_block_run(np.array(computed, dtype=np.int32), BLOCK) >= 1


def test_lead_and_run_share_one_boundary():
    computed = np.array([33, 40, 63, 80], dtype=np.int32)
    run = M.same_block_run(computed, BLOCK)
    starts = (computed - M.row_lead(computed, BLOCK))[:run]
    assert len(set(starts.tolist())) == 1


class TestPassRelativeIndexing:
    TOKENS = np.array([[10, 11, 12, 13, 14, 15, 0, 0],
                       [20, 21, 22, 23, 24, 25, 0, 0],
                       [30, 31, 32, 33, 34, 35, 0, 0]], dtype=np.int32)
    COMPUTED = np.array([0, 3, 5], dtype=np.int32)

    def _rows(self, start_index, num_scheduled, lead=None, rows=None, width=8):
        n = len(num_scheduled)
        lead = np.zeros(n, dtype=np.int32) if lead is None else np.asarray(lead)
        ids = torch.zeros((rows or n, width), dtype=torch.int32)
        pos = torch.zeros((rows or n, width), dtype=torch.int32)
        sched = np.asarray(num_scheduled, dtype=np.int32)
        M.fill_pass_input_ids(ids, torch.from_numpy(self.TOKENS), self.COMPUTED, sched, lead, start_index)
        M.fill_pass_positions(pos, self.COMPUTED, sched, lead, start_index)
        return ids, pos

    def test_first_pass(self):
        ids, pos = self._rows(0, [2, 2])
        assert ids[0, :2].tolist() == [10, 11] and pos[0, :2].tolist() == [0, 1]
        assert ids[1, :2].tolist() == [23, 24] and pos[1, :2].tolist() == [3, 4]

    def test_second_pass_reads_its_own_requests(self):
        ids, pos = self._rows(1, [2, 2])
        assert ids[0, :2].tolist() == [23, 24] and pos[0, :2].tolist() == [3, 4]
        assert ids[1, :2].tolist() == [35, 0] and pos[1, :2].tolist() == [5, 6]

    def test_last_request_alone(self):
        ids, pos = self._rows(2, [1])
        assert ids[0, 0].item() == 35 and pos[0, 0].item() == 5

    def test_row_lead_extends_backwards(self):
        ids, pos = self._rows(2, [1], lead=[2])
        assert ids[0, :3].tolist() == [33, 34, 35] and pos[0, :3].tolist() == [3, 4, 5]

    def test_padding_and_zero_rows_untouched(self):
        ids, pos = self._rows(1, [1], rows=3)
        assert ids[1].tolist() == [0] * 8 and pos[2].tolist() == [0] * 8
        ids, _ = self._rows(0, [0, 2])
        assert ids[0].tolist() == [0] * 8 and ids[1, :2].tolist() == [23, 24]


# ---- token buckets ------------------------------------------------------------------------
def test_token_paddings():
    assert M.token_paddings(16, 2048) == [1, 32, 64, 128, 256, 512, 1024, 2048]
    assert M.token_paddings(32, 100) == [1, 32, 64, 128]
    assert M.token_paddings(48, 64) == [1, 64]
    assert M.token_paddings(1, 1) == [1, 32]
    p = M.token_paddings(32, 512)
    assert [M.padded_token_len(p, x) for x in (1, 2, 32, 33, 512)] == [1, 32, 32, 64, 512]
    with pytest.raises(AssertionError):
        M.padded_token_len(p, 513)


# ---- builder ------------------------------------------------------------------------------
def _builder(**kw):
    args = dict(block_size=BLOCK, max_num_blocks_per_req=16, max_num_tokens=128)
    args.update(kw)
    return M.PagedMetadataBuilder(**args)


def _table(reqs, width=16):
    return (np.arange(reqs * width, dtype=np.int32).reshape(reqs, width) + 1)


def test_decode_pass_positions_and_padding():
    b = _builder()
    plan = b.prepare(_table(3), num_computed=[40, 0, 95], num_scheduled=[1, 1, 1], target_num_reqs=8)
    md = plan.metadata
    assert plan.is_decode and plan.padded_tokens == 1
    # cache_position = seq_len - 1 for live rows, -1 for padded rows (model_runner.py:1734-1739)
    assert md.cache_position.tolist() == [40, 0, 95, -1, -1, -1, -1, -1]
    assert md.page_table.shape == (8, 16) and md.fill_page_table.shape == (8, 8)
    assert torch.equal(md.page_table[:3], torch.from_numpy(_table(3)))
    assert not md.page_table[3:].any() and not md.fill_page_table[3:].any()
    assert md.chunk_start_idx is None
    assert md.batch_idx.tolist() == list(range(8)) and md.num_users == 8
    assert plan.positions[:3, 0].tolist() == [40, 0, 95]


def test_first_chunk_has_no_offset_and_identity_fill_table():
    b = _builder()
    plan = b.prepare(_table(2), num_computed=[0, 0], num_scheduled=[100, 128])
    md = plan.metadata
    assert plan.padded_tokens == 128 and not plan.is_decode
    assert md.chunk_start_idx is None
    assert torch.equal(md.fill_page_table, md.page_table[:, :8])
    assert md.cache_position.tolist() == [99, 127]


def test_continuation_chunk_rolls_fill_table_to_first_block_written():
    b = _builder()
    table = _table(2)
    plan = b.prepare(table, num_computed=[128, 128], num_scheduled=[64, 37])
    md = plan.metadata
    assert md.chunk_start_idx.tolist() == [128] and md.chunk_start_idx.dtype == torch.int32
    # Token t of the chunk must land in the block that holds absolute position 128 + t.
    for r in range(2):
        for t in (0, 31, 32, 63):
            assert md.fill_page_table[r, t // BLOCK].item() == table[r, (128 + t) // BLOCK]
    # The read table is not rolled.
    assert torch.equal(md.page_table, torch.from_numpy(table))


def test_mixed_stage_rows_are_refused():
    b = _builder()
    with pytest.raises(RuntimeError, match="single prefix offset"):
        b.prepare(_table(2), num_computed=[64, 128], num_scheduled=[32, 32])


def test_parked_row_points_at_null_block_and_does_not_set_offset():
    b = _builder()
    table = _table(3)
    plan = b.prepare(table, num_computed=[500, 0, 0], num_scheduled=[0, 64, 64])
    md = plan.metadata
    # The parked row's 500 computed tokens say nothing about the fresh rows.
    assert md.chunk_start_idx is None
    assert not md.page_table[0].any() and not md.fill_page_table[0].any()
    assert torch.equal(md.page_table[1:], torch.from_numpy(table[1:]))


def test_stale_rows_cleared_between_passes():
    b = _builder()
    b.prepare(_table(4), num_computed=[5, 6, 7, 8], num_scheduled=[1, 1, 1, 1], target_num_reqs=4)
    plan = b.prepare(_table(2), num_computed=[9, 10], num_scheduled=[1, 1], target_num_reqs=4)
    md = plan.metadata
    assert md.cache_position.tolist() == [9, 10, -1, -1]
    assert not md.page_table[2:].any() and not md.fill_page_table[2:].any()


def test_device_buffers_are_persistent_per_bucket():
    b = _builder()
    p1 = b.prepare(_table(2), [3, 4], [1, 1], target_num_reqs=4).metadata
    ptrs = (p1.cache_position.data_ptr(), p1.page_table.data_ptr(), p1.fill_page_table.data_ptr())
    p2 = b.prepare(_table(3), [8, 9, 10], [1, 1, 1], target_num_reqs=4).metadata
    assert ptrs == (p2.cache_position.data_ptr(), p2.page_table.data_ptr(), p2.fill_page_table.data_ptr())


def test_spec_rows_are_block_aligned():
    b = _builder(spec_prefix_rows=True)
    computed = np.array([41, 44, 80], dtype=np.int64)
    sched = np.array([4, 4, 4], dtype=np.int64)
    assert b.trim_pass(computed, sched) == 2
    plan = b.prepare(_table(2), computed[:2], sched[:2])
    md = plan.metadata
    assert plan.row_lead.tolist() == [9, 12]
    assert md.chunk_start_idx.tolist() == [32]
    assert plan.padded_tokens == 32
    assert plan.positions[0, :13].tolist() == list(range(32, 45))
    assert plan.positions[1, :16].tolist() == list(range(32, 48))
    # Column 0 of the fill table is the block holding position 32.
    assert md.fill_page_table[:, 0].tolist() == [_table(2)[0, 1], _table(2)[1, 1]]
    # A decode step is never trimmed.
    assert b.trim_pass(computed, np.ones(3, dtype=np.int64)) == 3


def test_narrow_block_table_is_zero_padded():
    b = _builder()
    plan = b.prepare(_table(2, width=5), [0, 0], [1, 1])
    assert torch.equal(plan.metadata.page_table[:, :5], torch.from_numpy(_table(2, width=5)))
    assert not plan.metadata.page_table[:, 5:].any()
