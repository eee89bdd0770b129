"""Host-side geometry of the sliding-window KV rings.

A sliding-window attention layer does not need a request's whole context in the block
pool: each batch slot owns a fixed sub-ring of ``window_blocks`` physical blocks, written
round-robin, and the page table handed to the kernels is that sub-ring rotated so that
column 0 is the oldest block still inside the window.  ``cache_position`` is then counted
from the start of column 0 and the kernels' ``sliding_window`` mask cuts the rest.

Restates ``integrations/vllm_plugin/vllm_tt/swa_cache_utils.py`` (pure integer / numpy
helpers, :23-137) and the per-pass ring metadata of the model runner
(``vllm_tt/model_runner.py:1751-1823``); pinned by the reference's own cases in
``tests/integrations/vllm_plugin/test_swa_cache_utils.py``.
"""

from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import numpy as np

# Ring widths stay multiples of 8 entries so that page tables built here can be handed to
# either implementation (the reference needs 32-byte table rows, swa_cache_utils.py:19-21).
PAGE_TABLE_STICK_BLOCK_ALIGNMENT = 8


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


def sliding_window_blocks(sliding_window: int, block_size: int, max_model_len: int) -> int:
    """Blocks per user in a ring: the window (never more than ``max_model_len``) plus one
    block for a window that straddles a block boundary, rounded up to the alignment
    (swa_cache_utils.py:23-43)."""
    window = min(sliding_window, max_model_len)
    need = _cdiv(window, block_size) + 1
    return _cdiv(need, PAGE_TABLE_STICK_BLOCK_ALIGNMENT) * PAGE_TABLE_STICK_BLOCK_ALIGNMENT


def sliding_ring_is_profitable(sliding_window: int, block_size: int, max_model_len: int) -> bool:
    """A ring only pays once it is smaller than keeping the whole context
    (swa_cache_utils.py:46-58)."""
    return sliding_window_blocks(sliding_window, block_size, max_model_len) < _cdiv(max_model_len, block_size)


def sliding_ring_phys_blocks(window_blocks: int, max_num_reqs: int) -> int:
    """One sub-ring per batch slot plus the null block 0 (swa_cache_utils.py:61-64)."""
    return window_blocks * max_num_reqs + 1


def sliding_ring_reserve_bytes(window_blocks: int, max_num_reqs: int, page_size_bytes: int) -> int:
    """Bytes of one layer's rings, in un-sharded page units (swa_cache_utils.py:67-79)."""
    return sliding_ring_phys_blocks(window_blocks, max_num_reqs) * page_size_bytes


def sliding_page_table_width(window_blocks: int, base_width: int) -> int:
    """Columns of a ring page table (swa_cache_utils.py:82-85)."""
    return min(window_blocks, base_width)


def assign_ring_slots(
    row_req_ids: Sequence[str],
    batch_req_ids: Sequence[str],
    req_ring_slot: Dict[str, int],
    free_ring_slots: List[int],
) -> np.ndarray:
    """Stable slot per request id (swa_cache_utils.py:88-126).

    Slots of requests that left ``batch_req_ids`` return to the pool first; requests in
    ``row_req_ids`` without a slot take the smallest free one.  Both containers are updated
    in place.  Raises IndexError when the pool is exhausted.
    """
    alive = set(batch_req_ids)
    for rid in [r for r in req_ring_slot if r not in alive]:
        free_ring_slots.append(req_ring_slot.pop(rid))
    free_ring_slots.sort(reverse=True)  # pop() hands out the smallest
    out = []
    for rid in row_req_ids:
        if rid not in req_ring_slot:
            req_ring_slot[rid] = free_ring_slots.pop()
        out.append(req_ring_slot[rid])
    return np.array(out, dtype=np.int64)


def build_sliding_ring_page_table(
    start_block: np.ndarray, slots: np.ndarray, window_blocks: int, width: int
) -> np.ndarray:
    """Rows x width table into each request's own sub-ring, rotated into logical order:
    column j is ring position ``(start_block + j) % window_blocks`` of sub-ring ``slot``,
    which starts at physical block ``1 + slot * window_blocks`` (swa_cache_utils.py:129-137).
    """
    cols = np.arange(width)[None, :]
    ring_pos = (np.asarray(start_block)[:, None] + cols) % window_blocks
    return ring_pos + (1 + np.asarray(slots) * window_blocks)[:, None]


def ring_pass_geometry(cur_pos_abs: np.ndarray, block_size: int, window_blocks: int) -> Tuple[np.ndarray, np.ndarray]:
    """For absolute positions of the token each row writes this step: the logical block that
    column 0 of the ring table stands for, and the position counted from the start of that
    block (model_runner.py:1759-1763, 1811-1813)."""
    cur_pos_abs = np.asarray(cur_pos_abs, dtype=np.int64)
    cur_block = cur_pos_abs // block_size
    num_win = np.minimum(cur_block + 1, window_blocks)
    start_block = cur_block - num_win + 1
    return start_block, cur_pos_abs - start_block * block_size


def check_ring_fill_supported(start_block: np.ndarray, num_computed: np.ndarray, num_scheduled: np.ndarray) -> None:
    """Multi-token rows fill ring blocks positionally from column 0, which is only right
    while the context still fits the ring and starts from nothing
    (model_runner.py:1764-1782)."""
    filling = np.asarray(num_scheduled) > 1
    bad = filling & ((np.asarray(start_block) > 0) | (np.asarray(num_computed) > 0))
    if np.any(bad):
        raise NotImplementedError(
            "sliding-window prefill for context > window or with prefix caching / chunked "
            "prefill (num_computed > 0) is not supported"
        )
