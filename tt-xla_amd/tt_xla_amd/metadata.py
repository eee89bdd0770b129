"""Host-side construction of the paged-attention metadata, free of vLLM.

The attention operators consume four small integer tensors per pass
(``cache_position``, ``page_table``, ``fill_page_table``, ``chunk_start_idx``) plus
``batch_idx``.  In tt-xla they are produced inside the vLLM model runner's
``_prepare_inputs`` (``integrations/vllm_plugin/vllm_tt/model_runner.py:1590-2016``);
this module restates that logic over plain numpy inputs so that a serving loop (or a
test) can build :class:`~tt_xla_amd.attention.TTMetadata` without a scheduler:

  * ``row_lead`` / ``same_block_run``             model_runner.py:5306-5328
  * ``token_paddings`` / ``padded_token_len``     model_runner.py:5201-5252
  * ``fill_page_table_width``                     model_runner.py:1255-1286
  * ``copy_narrow_fill_page_table``               model_runner.py:1288-1307
  * ``fill_pass_positions`` / ``fill_pass_input_ids``   model_runner.py:5255-5303
  * ``PagedMetadataBuilder.prepare``              model_runner.py:1722-1745 (cache
    position), :1840 (parked rows), :1852-1890 (single prefix offset), :1935-2016
    (page table, rolled fill table, null-block redirection)

Device buffers are allocated once per row-count bucket and refreshed with ``copy_`` each
pass, as the reference does (model_runner.py:1309-1340): addresses stay stable, which is
what lets a decode step be replayed from a HIP graph.
"""

from __future__ import annotations

import bisect
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .attention import TTMetadata

# A page-table row is padded to this many int32 entries (32 bytes), the alignment rule the
# reference applies to the fill table's width (model_runner.py:1276-1278).
PAGE_TABLE_ALIGN = 8


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


def row_lead(num_computed: np.ndarray, block_size: int) -> np.ndarray:
    """Tokens to feed again so that each row starts on its KV block boundary.

    ``paged_fill_cache`` writes from the first block of ``fill_page_table`` — position
    ``(num_computed // block_size) * block_size`` — while the chunked read offsets by an
    exact token count, so a multi-token row that starts mid-block is extended left by
    ``num_computed % block_size`` (model_runner.py:5322-5328).
    """
    return (np.asarray(num_computed) % block_size).astype(np.int32)


def same_block_run(num_computed: np.ndarray, block_size: int) -> int:
    """Length of the leading run of requests whose ``num_computed`` lies in one KV block.

    One pass carries a single ``chunk_start_idx``; callers trim a multi-token pass to this
    run and take the rest in the next pass (model_runner.py:5306-5319).  Never 0 for a
    non-empty input.
    """
    num_computed = np.asarray(num_computed)
    if num_computed.size == 0:
        return 0
    boundary = num_computed // block_size
    differs = np.flatnonzero(boundary != boundary[0])
    return int(differs[0]) if differs.size else int(num_computed.size)


def token_paddings(min_token_size: int, max_token_size: int) -> List[int]:
    """Row-length buckets: 1 (decode) then powers of two from ``max(32, pow2(min))`` up to
    the first that covers ``max_token_size`` (model_runner.py:5201-5245)."""
    num = 32
    while num < min_token_size:
        num *= 2
    paddings = [1]
    while True:
        paddings.append(num)
        if num >= max_token_size:
            break
        num *= 2
    return paddings


def padded_token_len(paddings: Sequence[int], x: int) -> int:
    """First bucket >= x (model_runner.py:5248-5252)."""
    index = bisect.bisect_left(paddings, x)
    assert index < len(paddings), f"no token bucket covers {x} (largest {paddings[-1]})"
    return paddings[index]


def fill_page_table_width(max_num_tokens: int, block_size: int, read_width: int) -> int:
    """Columns ``paged_fill_cache``'s page table needs: the blocks one step can touch,
    rounded to 8 entries and clamped to the read table's width.

    Raises AssertionError ("cannot cover") when the clamped table is too short for the
    largest step, so a misconfiguration fails at start-up on the host and never as an
    out-of-range page lookup on the device (model_runner.py:1255-1286).
    """
    width = _cdiv(_cdiv(max_num_tokens, block_size), PAGE_TABLE_ALIGN) * PAGE_TABLE_ALIGN
    fill_width = min(width, read_width)
    assert fill_width * block_size >= max_num_tokens, (
        f"fill page table ({fill_width} cols x block_size {block_size}) cannot cover a "
        f"{max_num_tokens}-token step"
    )
    return fill_width


def copy_narrow_fill_page_table(
    dev_buf: torch.Tensor, host_table: torch.Tensor, block_size: int, step_tokens: int
) -> None:
    """Stage the leading ``dev_buf.shape[1]`` columns of ``host_table`` into the narrow
    fill buffer, refusing a step the truncated table cannot span
    (model_runner.py:1288-1307)."""
    fill_width = dev_buf.shape[1]
    assert fill_width * block_size >= step_tokens, (
        f"fill page table ({fill_width} cols x block_size {block_size}) cannot cover this "
        f"step's {step_tokens} tokens"
    )
    dev_buf.copy_(host_table[:, :fill_width])


def fill_pass_positions(
    positions: torch.Tensor,
    num_computed: np.ndarray,
    num_scheduled: np.ndarray,
    lead: np.ndarray,
    start_index: int = 0,
) -> None:
    """Write one pass's position ids: row i belongs to request ``start_index + i`` and
    starts ``lead[i]`` tokens before its computed count (model_runner.py:5255-5281)."""
    for i, n in enumerate(num_scheduled):
        back = int(lead[i])
        row_len = back + int(n)
        first = int(num_computed[start_index + i]) - back
        positions[i, :row_len] = torch.arange(first, first + row_len, dtype=positions.dtype)


def fill_pass_input_ids(
    input_ids: torch.Tensor,
    token_ids: torch.Tensor,
    num_computed: np.ndarray,
    num_scheduled: np.ndarray,
    lead: np.ndarray,
    start_index: int = 0,
) -> None:
    """Gather one pass's input token ids, one row per request, with the same pass-local
    vs global indexing as :func:`fill_pass_positions` (model_runner.py:5284-5303)."""
    for i, n in enumerate(num_scheduled):
        back = int(lead[i])
        req = start_index + i
        start = int(num_computed[req]) - back
        row_len = back + int(n)
        input_ids[i, :row_len] = token_ids[req, start : start + row_len]


@dataclass
class PassPlan:
    """What one pass feeds the model besides the attention metadata."""

    metadata: TTMetadata
    row_lead: np.ndarray  # [reqs] tokens re-fed per row
    padded_tokens: int  # row length bucket of this pass
    positions: torch.Tensor  # [target_num_reqs, padded_tokens] int32 (host)
    is_decode: bool


class PagedMetadataBuilder:
    """Builds :class:`TTMetadata` for one KV-cache group from scheduler state.

    Parameters follow the model runner's attributes of the same meaning
    (model_runner.py:466-567): ``max_num_blocks_per_req`` is the read table's width
    (``cdiv(max_model_len, block_size)``), ``max_num_tokens`` the per-step token budget,
    ``chunked_sdpa`` whether continuation chunks read their prefix from the paged cache,
    ``spec_prefix_rows`` whether multi-token decode rows are block-aligned with
    :func:`row_lead`.
    """

    def __init__(
        self,
        block_size: int,
        max_num_blocks_per_req: int,
        max_num_tokens: int,
        device: torch.device | str = "cpu",
        min_num_tokens: int = 32,
        chunked_sdpa: bool = True,
        spec_prefix_rows: bool = False,
    ):
        self.block_size = int(block_size)
        self.read_width = int(max_num_blocks_per_req)
        self.max_num_tokens = int(max_num_tokens)
        self.device = torch.device(device)
        self.chunked_sdpa = chunked_sdpa
        self.spec_prefix_rows = spec_prefix_rows
        self.paddings = token_paddings(min_num_tokens, max_num_tokens)
        self.fill_width = fill_page_table_width(self.max_num_tokens, self.block_size, self.read_width)
        self._chunk_start_dev = torch.zeros(1, dtype=torch.int32, device=self.device)
        self._buffers: Dict[int, Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]] = {}

    def _device_buffers(self, rows: int):
        if rows not in self._buffers:
            dev = self.device
            self._buffers[rows] = (
                torch.full((rows,), -1, dtype=torch.int32, device=dev),  # cache_position
                torch.zeros((rows, self.read_width), dtype=torch.int32, device=dev),  # page_table
                torch.zeros((rows, self.fill_width), dtype=torch.int32, device=dev),  # fill table
                torch.arange(rows, dtype=torch.int32, device=dev),  # batch_idx
            )
        return self._buffers[rows]

    def trim_pass(self, num_computed: np.ndarray, num_scheduled: np.ndarray) -> int:
        """Requests the next pass may carry: all of them for a decode step or without
        block alignment, else the leading run that shares one KV block boundary
        (model_runner.py:1560-1588 via ``_same_block_run``)."""
        num_scheduled = np.asarray(num_scheduled)
        if num_scheduled.size == 0:
            return 0
        if self.spec_prefix_rows and int(num_scheduled.max()) > 1:
            return same_block_run(np.asarray(num_computed), self.block_size)
        return int(num_scheduled.size)

    def prepare(
        self,
        block_table: np.ndarray,
        num_computed: np.ndarray,
        num_scheduled: np.ndarray,
        target_num_reqs: Optional[int] = None,
    ) -> PassPlan:
        """One pass over requests ``0..len(num_scheduled)``.

        block_table   [reqs, <= read_width] int32 physical block ids (0 = null block)
        num_computed  [reqs] tokens already in the cache per request
        num_scheduled [reqs] tokens this step per request (0 = parked row)
        target_num_reqs  padded row count (>= reqs); defaults to reqs
        """
        num_computed = np.asarray(num_computed, dtype=np.int64)
        num_scheduled = np.asarray(num_scheduled, dtype=np.int64)
        reqs = int(num_scheduled.size)
        assert reqs > 0 and num_computed.size == reqs
        rows = reqs if target_num_reqs is None else int(target_num_reqs)
        assert rows >= reqs, f"target_num_reqs {rows} < {reqs} requests"
        block_table = np.asarray(block_table)
        assert block_table.shape[0] >= reqs
        bs = self.block_size
        max_sched = int(num_scheduled.max())
        is_decode = max_sched == 1

        lead = np.zeros(reqs, dtype=np.int32)
        if self.spec_prefix_rows and max_sched > 1:
            lead = row_lead(num_computed, bs)
            starts = (num_computed - lead)[num_scheduled > 0]
            assert len(np.unique(starts)) <= 1, (
                f"spec pass spans multiple block boundaries: {starts.tolist()}"
            )
        padded_tokens = padded_token_len(self.paddings, int((num_scheduled + lead).max()))

        positions = torch.zeros((rows, padded_tokens), dtype=torch.int32)
        fill_pass_positions(positions, num_computed, num_scheduled, lead)

        cache_position_dev, page_table_dev, fill_dev, batch_idx = self._device_buffers(rows)

        # Position of the last token of the step; padded rows carry -1, which the cache
        # write skips.
        cache_position = torch.full((rows,), -1, dtype=torch.int32)
        cache_position[:reqs] = torch.from_numpy((num_computed + num_scheduled - 1).astype(np.int32))
        cache_position_dev.copy_(cache_position)

        zero_sched_rows = np.nonzero(num_scheduled == 0)[0]

        # Single prefix offset for a continuation-chunk pass.
        active_rows = np.nonzero(num_scheduled > 0)[0]
        active_computed = num_computed[active_rows]
        prefix_chunk_step = padded_tokens > 1 and bool(np.any(active_computed > 0))
        chunk_start_idx = None
        if prefix_chunk_step and (self.chunked_sdpa or self.spec_prefix_rows):
            active_starts = active_computed - lead[active_rows]
            offsets = {int(v) for v in active_starts}
            if len(offsets) > 1:
                raise RuntimeError(
                    "chunked-prefill SDPA takes a single prefix offset for the batch, but "
                    f"active rows are at different stages: start={sorted(offsets)} for rows "
                    f"{active_rows.tolist()}. Batching mixed stages would apply one row's "
                    "offset to another."
                )
            self._chunk_start_dev.copy_(torch.tensor([int(active_starts[0])], dtype=torch.int32))
            chunk_start_idx = self._chunk_start_dev

        copy_width = min(block_table.shape[1], self.read_width)
        page_table = torch.zeros((rows, self.read_width), dtype=torch.int32)
        page_table[:reqs, :copy_width] = torch.from_numpy(
            np.ascontiguousarray(block_table[:reqs, :copy_width]).astype(np.int32)
        )

        block_offsets = num_computed // bs
        if np.any(block_offsets > 0):
            fill_page_table = page_table.clone()
            for i in range(reqs):
                if block_offsets[i] > 0:
                    fill_page_table[i] = torch.roll(page_table[i], shifts=-int(block_offsets[i]))
        else:
            fill_page_table = page_table

        # A parked row points at the null block so its write cannot land in blocks the
        # scheduler has handed to another request.
        if len(zero_sched_rows) > 0:
            page_table[zero_sched_rows, :] = 0
            if fill_page_table is not page_table:
                fill_page_table[zero_sched_rows, :] = 0

        page_table_dev.copy_(page_table)
        copy_narrow_fill_page_table(fill_dev, fill_page_table, bs, padded_tokens)

        metadata = TTMetadata(
            page_table=page_table_dev,
            cache_position=cache_position_dev,
            is_causal=True,
            attn_mask=None,
            fill_page_table=fill_dev,
            chunk_start_idx=chunk_start_idx,
            batch_idx=batch_idx,
            num_users=rows,
        )
        return PassPlan(metadata, lead, padded_tokens, positions, is_decode)
