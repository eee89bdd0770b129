"""Moving whole KV blocks between a host-side cache and the device cache (block swap for
preemption / offload).  Same call surface and no-op rules as ``copy_kv_blocks`` in tt-xla's
``integrations/vllm_plugin/vllm_tt/model_runner.py:5433-5474``: caches are dicts
``layer name -> tensor`` or ``layer name -> (k_cache, v_cache)`` with blocks on dim 0, and
block ``src_block_ids[i]`` of every source tensor lands in block ``dst_block_ids[i]`` of the
matching destination tensor.  Pure block copies: torch's gather / scatter on dim 0 plus one
transfer per tensor; nothing is computed.
"""

from __future__ import annotations

from typing import Dict, List, Literal, Sequence, Tuple, Union

import torch

Cache = Union[torch.Tensor, Sequence[torch.Tensor]]


def _device_of(value: Cache) -> torch.device:
    return value[0].device if isinstance(value, (list, tuple)) else value.device


def _move(src: torch.Tensor, dst: torch.Tensor, src_idx: torch.Tensor, dst_idx: torch.Tensor) -> None:
    picked = src.index_select(0, src_idx)
    dst.index_copy_(0, dst_idx, picked.to(dst.device, non_blocking=False))


def copy_kv_blocks(
    src_kv_caches: Dict[str, Cache],
    dst_kv_caches: Dict[str, Cache],
    src_block_ids: List[int],
    dst_block_ids: List[int],
    direction: Literal["h2d", "d2h"],
) -> None:
    if (
        not src_kv_caches
        or not dst_kv_caches
        or not src_block_ids
        or not dst_block_ids
        or len(src_block_ids) != len(dst_block_ids)
    ):
        return
    if direction not in ("h2d", "d2h"):
        raise ValueError(f"direction must be 'h2d' or 'd2h', got {direction!r}")
    src_device = _device_of(next(iter(src_kv_caches.values())))
    dst_device = _device_of(next(iter(dst_kv_caches.values())))
    src_idx = torch.tensor(src_block_ids, dtype=torch.int64, device=src_device)
    dst_idx = torch.tensor(dst_block_ids, dtype=torch.int64, device=dst_device)
    for name, src in src_kv_caches.items():
        dst = dst_kv_caches[name]
        if isinstance(src, (list, tuple)):
            for s, d in zip(src, dst):
                _move(s, d, src_idx, dst_idx)
        else:
            _move(src, dst, src_idx, dst_idx)
