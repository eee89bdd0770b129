"""``torch.ops.tt.*`` operators of the paged-attention path for HIP devices.

Names, argument order and defaults are those of tt-xla's
``python_package/tt_torch/custom_ops.py`` (:635-646, :962-971, :1016-1024,
:1198-1214, :1334-1346, and the static-cache forms :745-759, :857-867, :903-906); the implementation of each is a launch of a gfx950 kernel
through the C ABI in ``include/ttpa.h``.  As in the reference the five operators are
functional (``mutates_args=[]``): the cache writers return a fresh tensor.  Because a
functional write copies the whole cache, in-place twins ``tt::paged_update_cache_`` and
``tt::paged_fill_cache_`` are provided for callers that own the cache (the attention
backend uses them); their effect on the cache equals ``cache.copy_(functional_op(...))``.

The operators are registered for the ``cuda`` (HIP) device type only.  There is no CPU
implementation here: calling them with CPU tensors raises.
"""

from __future__ import annotations

import math
from typing import Optional

import torch

from . import _native as N

# --------------------------------------------------------------------------- #
# helpers
# --------------------------------------------------------------------------- #
_BFP8_GROUP = 16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def _rows_contiguous(t: torch.Tensor) -> torch.Tensor:
    """Last dim contiguous, every other stride a multiple of 8 elements, 16-byte base."""
    if t.stride(-1) != 1 or t.data_ptr() % 16 or any(s % 8 for s in t.stride()[:-1]):
        return t.contiguous()
    return t


def _index_tensor(t: torch.Tensor) -> torch.Tensor:
    if t.dtype not in (torch.int32, torch.int64):
        t = t.to(torch.int64)
    return t.contiguous()


def _table(t: torch.Tensor) -> torch.Tensor:
    if t.dtype != torch.int32:
        t = t.to(torch.int32)
    if t.stride(-1) != 1:
        t = t.contiguous()
    return t


def _kv_format(cache: torch.Tensor) -> int:
    if cache.dtype == torch.uint8:
        return N.KV_BFP8
    if cache.dtype in (torch.bfloat16, torch.float16):
        return N.KV_BF16  # 2-byte elements; the cache writers are pure copies
    raise ValueError(f"unsupported cache dtype {cache.dtype}")


def _cache_geometry(cache: torch.Tensor):
    """(num_blocks, kv_heads, block_size, head_size, format) of a cache tensor."""
    if cache.dim() != 4 or not cache.is_contiguous():
        raise ValueError("cache must be a contiguous [num_blocks, kv_heads, block_size, head_size] tensor")
    fmt = _kv_format(cache)
    nb, hkv, rows, d = cache.shape
    if fmt == N.KV_BFP8:
        if rows % (_BFP8_GROUP + 1):
            raise ValueError("block-float-8 cache must have block_size + block_size/16 rows")
        bs = rows // (_BFP8_GROUP + 1) * _BFP8_GROUP
    else:
        bs = rows
    return nb, hkv, bs, d, fmt


def _attention_cache_geometry(cache: torch.Tensor):
    """``_cache_geometry`` for the attention operators, which read the elements as numbers: a
    bfloat16 or block-float-8 cache (the cache writers also move float16 caches: pure copies)."""
    if cache.dtype not in (torch.bfloat16, torch.uint8):
        raise ValueError(f"attention reads bfloat16 or block-float-8 (uint8) caches, got {cache.dtype}")
    return _cache_geometry(cache)


def bfp8_cache_shape(num_blocks: int, num_kv_heads: int, block_size: int, head_size: int):
    """Shape of the uint8 tensor that stores a block-float-8 cache."""
    assert block_size % _BFP8_GROUP == 0 and head_size % _BFP8_GROUP == 0
    return (num_blocks, num_kv_heads, block_size + block_size // _BFP8_GROUP, head_size)


def bfp8_empty_cache(num_blocks: int, num_kv_heads: int, block_size: int, head_size: int, device):
    """A block-float-8 cache that decodes to zeros everywhere: element bytes 128 (offset binary
    zero), exponent bytes 0.  An all-zero tensor is a valid cache too, but its never-written
    positions decode to -2^-126 rather than 0."""
    cache = torch.zeros(bfp8_cache_shape(num_blocks, num_kv_heads, block_size, head_size),
                        dtype=torch.uint8, device=device)
    cache[:, :, :block_size, :] = 128
    return cache


# --------------------------------------------------------------------------- #
# cache writes
# --------------------------------------------------------------------------- #
def _update_inplace(cache, fill_value, update_indices, page_table):
    nb, hkv, bs, d, fmt = _cache_geometry(cache)
    if fill_value.dim() != 4 or fill_value.shape[0] != 1:
        raise ValueError("fill_value must be [1, users, heads, head_size]")
    users = update_indices.shape[0]
    if fill_value.shape[1] != users or fill_value.shape[2] < hkv or fill_value.shape[3] != d:
        raise ValueError(
            f"fill_value {tuple(fill_value.shape)} does not match users={users}, "
            f"kv_heads={hkv}, head_size={d}"
        )
    if page_table.dim() != 2 or page_table.shape[0] < users:
        raise ValueError("page_table must be [users, blocks_per_user]")
    if fill_value.dtype not in (torch.bfloat16, torch.float16) or (
        fmt == N.KV_BF16 and fill_value.dtype != cache.dtype
    ):
        raise ValueError("fill_value dtype must match the cache (bfloat16 for block-float-8)")
    fill_value = _rows_contiguous(fill_value)
    idx = _index_tensor(update_indices)
    pt = _table(page_table)
    N.call(
        "ttpa_paged_update_cache",
        cache.data_ptr(), fill_value.data_ptr(), fill_value.stride(1), fill_value.stride(2),
        idx.data_ptr(), int(idx.dtype == torch.int64), pt.data_ptr(), pt.stride(0),
        users, hkv, bs, d, pt.shape[1], nb, fmt, _stream(),
    )


@torch.library.custom_op("tt::paged_update_cache", mutates_args=[], device_types=["cuda"])
def paged_update_cache(
    cache: torch.Tensor,
    fill_value: torch.Tensor,
    update_indices: torch.Tensor,
    page_table: torch.Tensor,
    share_cache: bool = False,
) -> torch.Tensor:
    out = cache.clone()
    _update_inplace(out, fill_value, update_indices, page_table)
    return out


@paged_update_cache.register_fake
def _(cache, fill_value, update_indices, page_table, share_cache=False):
    return torch.empty_like(cache)


@torch.library.custom_op("tt::paged_update_cache_", mutates_args=["cache"], device_types=["cuda"])
def paged_update_cache_(
    cache: torch.Tensor,
    fill_value: torch.Tensor,
    update_indices: torch.Tensor,
    page_table: torch.Tensor,
    share_cache: bool = False,
) -> None:
    _update_inplace(cache, fill_value, update_indices, page_table)


@paged_update_cache_.register_fake
def _(cache, fill_value, update_indices, page_table, share_cache=False):
    return None


@torch.library.custom_op("tt::paged_update_kv_cache_", mutates_args=["k_cache", "v_cache"],
                         device_types=["cuda"])
def paged_update_kv_cache_(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_fill: torch.Tensor,
    v_fill: torch.Tensor,
    update_indices: torch.Tensor,
    page_table: torch.Tensor,
) -> None:
    """``paged_update_cache_`` on the K cache and on the V cache in one launch (the decode
    step always writes both with the same indices and table)."""
    geo = _cache_geometry(k_cache)
    if _cache_geometry(v_cache) != geo or k_fill.shape != v_fill.shape or k_fill.dtype != v_fill.dtype:
        raise ValueError("K and V caches / fills must agree in shape and dtype")
    k_fill, v_fill = _rows_contiguous(k_fill), _rows_contiguous(v_fill)
    if k_fill.stride() != v_fill.stride():
        paged_update_cache_(k_cache, k_fill, update_indices, page_table)
        paged_update_cache_(v_cache, v_fill, update_indices, page_table)
        return
    nb, hkv, bs, d, fmt = geo
    users = update_indices.shape[0]
    if (k_fill.dim() != 4 or k_fill.shape[0] != 1 or k_fill.shape[1] != users
            or k_fill.shape[2] < hkv or k_fill.shape[3] != d):
        raise ValueError(f"fill {tuple(k_fill.shape)} does not match users={users}, kv_heads={hkv}, head_size={d}")
    if page_table.dim() != 2 or page_table.shape[0] < users:
        raise ValueError("page_table must be [users, blocks_per_user]")
    idx = _index_tensor(update_indices)
    pt = _table(page_table)
    N.call(
        "ttpa_paged_update_cache_kv",
        k_cache.data_ptr(), v_cache.data_ptr(), k_fill.data_ptr(), v_fill.data_ptr(),
        k_fill.stride(1), k_fill.stride(2), idx.data_ptr(), int(idx.dtype == torch.int64),
        pt.data_ptr(), pt.stride(0), users, hkv, bs, d, pt.shape[1], nb, fmt, _stream(),
    )


@paged_update_kv_cache_.register_fake
def _(k_cache, v_cache, k_fill, v_fill, update_indices, page_table):
    return None


def _fill_inplace(cache, fill_value, page_table, batch_idx, cache2=None, fill_value2=None):
    """cache2 / fill_value2 given: the second pair is written by the same launch."""
    nb, hkv, bs, d, fmt = _cache_geometry(cache)
    if fill_value.dim() != 4:
        raise ValueError("fill_value must be [users, heads, seq_len, head_size]")
    fu, fh, s, fd = fill_value.shape
    if fh != hkv or fd != d:
        raise ValueError(
            f"fill_value {tuple(fill_value.shape)} does not match kv_heads={hkv}, head_size={d}"
        )
    if page_table.dim() != 2:
        raise ValueError("page_table must be [users, blocks_per_user]")
    if batch_idx is None:
        if fu != 1:
            raise ValueError("batch_idx is required when fill_value holds more than one user")
    else:
        if batch_idx.numel() != fu:
            raise ValueError("batch_idx must have one entry per fill_value row")
        batch_idx = _index_tensor(batch_idx.reshape(-1))
    if s > page_table.shape[1] * bs:
        raise ValueError(
            f"{s} tokens do not fit {page_table.shape[1]} page-table columns of {bs} tokens"
        )
    if fill_value.dtype not in (torch.bfloat16, torch.float16) or (
        fmt == N.KV_BF16 and fill_value.dtype != cache.dtype
    ):
        raise ValueError("fill_value dtype must match the cache (bfloat16 for block-float-8)")
    fill_value = _rows_contiguous(fill_value)
    pt = _table(page_table)
    if cache2 is not None:
        if _cache_geometry(cache2) != (nb, hkv, bs, d, fmt) or fill_value2.shape != (fu, fh, s, fd) \
                or fill_value2.dtype != fill_value.dtype:
            raise ValueError("K and V caches / fills must agree in shape and dtype")
        fill_value2 = _rows_contiguous(fill_value2)
        if fill_value2.stride() != fill_value.stride():
            _fill_inplace(cache, fill_value, page_table, batch_idx)
            _fill_inplace(cache2, fill_value2, page_table, batch_idx)
            return
        N.call(
            "ttpa_paged_fill_cache_kv",
            cache.data_ptr(), cache2.data_ptr(), fill_value.data_ptr(), fill_value2.data_ptr(),
            fill_value.stride(0), fill_value.stride(1), fill_value.stride(2), pt.data_ptr(), pt.stride(0),
            _ptr(batch_idx), int(batch_idx is not None and batch_idx.dtype == torch.int64),
            fu, pt.shape[0], hkv, s, bs, d, pt.shape[1], nb, fmt, _stream(),
        )
        return
    N.call(
        "ttpa_paged_fill_cache",
        cache.data_ptr(), fill_value.data_ptr(), fill_value.stride(0), fill_value.stride(1),
        fill_value.stride(2), pt.data_ptr(), pt.stride(0), _ptr(batch_idx),
        int(batch_idx is not None and batch_idx.dtype == torch.int64),
        fu, pt.shape[0], hkv, s, bs, d, pt.shape[1], nb, fmt, _stream(),
    )


@torch.library.custom_op("tt::paged_fill_cache", mutates_args=[], device_types=["cuda"])
def paged_fill_cache(
    cache: torch.Tensor,
    fill_value: torch.Tensor,
    page_table: torch.Tensor,
    batch_idx: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    out = cache.clone()
    _fill_inplace(out, fill_value, page_table, batch_idx)
    return out


@paged_fill_cache.register_fake
def _(cache, fill_value, page_table, batch_idx=None):
    return torch.empty_like(cache)


@torch.library.custom_op("tt::paged_fill_cache_", mutates_args=["cache"], device_types=["cuda"])
def paged_fill_cache_(
    cache: torch.Tensor,
    fill_value: torch.Tensor,
    page_table: torch.Tensor,
    batch_idx: Optional[torch.Tensor] = None,
) -> None:
    _fill_inplace(cache, fill_value, page_table, batch_idx)


@paged_fill_cache_.register_fake
def _(cache, fill_value, page_table, batch_idx=None):
    return None


@torch.library.custom_op("tt::paged_fill_kv_cache_", mutates_args=["k_cache", "v_cache"],
                         device_types=["cuda"])
def paged_fill_kv_cache_(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_fill: torch.Tensor,
    v_fill: torch.Tensor,
    page_table: torch.Tensor,
    batch_idx: Optional[torch.Tensor] = None,
) -> None:
    """``paged_fill_cache_`` on the K cache and on the V cache in one launch (a prefill pass
    always fills both through the same table and batch_idx, reference attention.py:500-511)."""
    _fill_inplace(k_cache, k_fill, page_table, batch_idx, v_cache, v_fill)


# --------------------------------------------------------------------------- #
# decode attention
# --------------------------------------------------------------------------- #
@torch.library.custom_op(
    "tt::paged_scaled_dot_product_attention_decode", mutates_args=[], device_types=["cuda"]
)
def paged_scaled_dot_product_attention_decode(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    page_table: torch.Tensor,
    is_causal: bool = False,
    attn_mask: Optional[torch.Tensor] = None,
    cur_pos_tensor: Optional[torch.Tensor] = None,
    attention_sink: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    sliding_window_size: Optional[int] = None,
) -> torch.Tensor:
    return _decode(query, key, value, page_table, is_causal, attn_mask, cur_pos_tensor, attention_sink,
                   scale, sliding_window_size, None, None)


def _check_out(out, shape, name):
    """An output tensor handed in by the caller: bfloat16, the given shape, rows contiguous and
    16-byte aligned, strides in whole 8-byte units (what the kernels' vector stores need)."""
    if out.dtype != torch.bfloat16 or tuple(out.shape) != tuple(shape):
        raise ValueError(f"{name}: out must be bfloat16 of shape {tuple(shape)}, got {out.dtype} {tuple(out.shape)}")
    if out.stride(-1) != 1 or out.data_ptr() % 16 or any(st % 4 for st in out.stride()[:-1]):
        raise ValueError(f"{name}: out needs contiguous 16-byte aligned rows and strides that are multiples of 4")
    return out


def _decode(query, key, value, page_table, is_causal, attn_mask, cur_pos_tensor, attention_sink, scale,
            sliding_window_size, k_new, v_new, out=None):
    """Checks and launch shared by the decode operator and the fused update + decode operator
    (k_new / v_new given: the step's cache update happens in the same call).  ``out``
    [1, users, heads, head_size]: written in place of a fresh tensor."""
    if is_causal:
        assert attn_mask is None, "attention_mask must be None when is_causal is True."
        assert cur_pos_tensor is not None, "cur_pos_tensor must be provided when is_causal is True."
    if attn_mask is not None:
        assert not is_causal, "attention_mask must be None when is_causal is True."
    if sliding_window_size is not None and sliding_window_size <= 0:
        raise ValueError("sliding_window_size must be positive")
    if query.dim() != 4 or query.shape[0] != 1:
        raise ValueError("query must be [1, users, heads, head_size]")
    if not is_causal:
        if k_new is not None:
            raise ValueError("the fused update + decode step is causal")
        return _decode_masked(query, key, value, page_table, attn_mask, attention_sink, scale,
                              sliding_window_size, out)
    nb, hkv, bs, d, fmt = _attention_cache_geometry(key)
    if _attention_cache_geometry(value) != (nb, hkv, bs, d, fmt):
        raise ValueError("key and value caches must have the same shape and dtype")
    _, users, hq, qd = query.shape
    if qd != d or hq % hkv:
        raise ValueError(f"query {tuple(query.shape)} does not match the cache geometry")
    if query.dtype != torch.bfloat16:
        raise ValueError("query must be bfloat16")
    if page_table.dim() != 2 or page_table.shape[0] != users or cur_pos_tensor.shape[0] != users:
        raise ValueError("page_table / cur_pos_tensor must have one row per user")
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    q = _rows_contiguous(query)
    pt = _table(page_table)
    cur = _index_tensor(cur_pos_tensor)
    if out is None:
        out = torch.empty((1, users, hq, d), dtype=query.dtype, device=query.device)
    else:
        _check_out(out, (1, users, hq, d), "decode")
    ws_bytes = N.lib().ttpa_paged_decode_workspace_bytes(users, hq, hkv, d)
    ws = _workspace(ws_bytes, query.device)
    sink = None
    if attention_sink is not None:
        if attention_sink.numel() != hq:
            raise ValueError(f"attention_sink must hold one logit per query head ({hq})")
        sink = attention_sink.reshape(hq).to(device=query.device, dtype=torch.float32).contiguous()
    if k_new is None:
        N.call(
            "ttpa_paged_sdpa_decode_windowed",
            out.data_ptr(), out.stride(1), out.stride(2), q.data_ptr(), q.stride(1), q.stride(2),
            key.data_ptr(), value.data_ptr(), pt.data_ptr(), pt.stride(0), cur.data_ptr(),
            int(cur.dtype == torch.int64), users, hq, hkv, d, bs, pt.shape[1], nb, float(scale), fmt,
            int(sliding_window_size or 0), sink.data_ptr() if sink is not None else None,
            ws.data_ptr(), ws_bytes, _stream(),
        )
        return out
    if k_new.shape != v_new.shape or k_new.dtype != torch.bfloat16 or v_new.dtype != torch.bfloat16:
        raise ValueError("k_new and v_new must be bfloat16 tensors of one shape")
    if (k_new.dim() != 4 or k_new.shape[0] != 1 or k_new.shape[1] != users or k_new.shape[2] < hkv
            or k_new.shape[3] != d):
        raise ValueError(f"k_new {tuple(k_new.shape)} does not match users={users}, kv_heads={hkv}, head_size={d}")
    k_new, v_new = _rows_contiguous(k_new), _rows_contiguous(v_new)
    if k_new.stride() != v_new.stride():
        v_new = v_new.contiguous()
        k_new = k_new.contiguous()
    N.call(
        "ttpa_paged_update_decode",
        out.data_ptr(), out.stride(1), out.stride(2), q.data_ptr(), q.stride(1), q.stride(2),
        key.data_ptr(), value.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), k_new.stride(1),
        k_new.stride(2), pt.data_ptr(), pt.stride(0), cur.data_ptr(), int(cur.dtype == torch.int64),
        users, hq, hkv, d, bs, pt.shape[1], nb, float(scale), fmt, int(sliding_window_size or 0),
        sink.data_ptr() if sink is not None else None, ws.data_ptr(), ws_bytes, _stream(),
    )
    return out


_WORKSPACES = {}


# Largest scratch a block-float-8 chunk pass may ask for (bfloat16 copies of its users' blocks).
_EXPANSION_LIMIT = 8 << 30


def _workspace(nbytes: int, device) -> torch.Tensor:
    """A per-device scratch tensor for the split-K partials of a decode launch, grown on demand and
    reused by later calls: launches of one stream run in order, so one buffer serves them all, and
    an eager serving loop pays no allocator round trip per layer and step.  Under graph capture the
    allocation has to belong to the graph's pool, and a call on another stream must not share the
    buffer, so both get a fresh tensor."""
    if torch.cuda.is_current_stream_capturing() or torch.cuda.current_stream(device) != torch.cuda.default_stream(device):
        return torch.empty(nbytes, dtype=torch.uint8, device=device)
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = ws
    return ws


def _decode_mask_rows(attn_mask, users, hq, skv):
    """The additive mask of a one-token pass as (bfloat16 tensor, user stride, head stride): anything
    that broadcasts to [users, heads, 1, skv]; a head stride of 0 shares one row between the heads."""
    m = _additive_mask(attn_mask)
    if m.dim() != 4 or m.shape[2] != 1 or m.shape[3] != skv or m.shape[0] not in (1, users) or m.shape[1] not in (1, hq):
        raise ValueError(f"attn_mask must broadcast to [{users}, {hq}, 1, {skv}], got {tuple(attn_mask.shape)}")
    if m.stride(-1) != 1:
        m = m.contiguous()
    return m, (m.stride(0) if m.shape[0] == users and users > 1 else 0), (m.stride(1) if m.shape[1] == hq and hq > 1 else 0)


def _decode_masked(query, key, value, page_table, attn_mask, attention_sink, scale, sliding_window_size, out):
    """Decode with ``is_causal=False``: every position of the user's table is attended, weighted by
    the additive ``attn_mask`` (anything that broadcasts to [users, heads, 1, table_width * block_size];
    reference CPU branch custom_ops.py:1296-1311; the one-token pass of a pooling / encoder model,
    never the generative serving path).  Up to 32 query heads per KV head (either cache format) run
    on the decode kernels with the mask as an operand; the rest is _decode_masked_gathered."""
    if attn_mask is None:
        raise ValueError("attn_mask must be provided when is_causal is False")
    if attention_sink is not None or sliding_window_size is not None:
        raise NotImplementedError("attention_sink / sliding_window_size with an explicit attn_mask are not built")
    nb, hkv, bs, d, fmt = _attention_cache_geometry(key)
    if _attention_cache_geometry(value) != (nb, hkv, bs, d, fmt):
        raise ValueError("key and value caches must have the same shape and dtype")
    _, users, hq, qd = query.shape
    if qd != d or hq % hkv or query.dtype != torch.bfloat16:
        raise ValueError(f"query {tuple(query.shape)} {query.dtype} does not match the cache geometry")
    width = page_table.shape[1]
    skv = width * bs
    mask, mask_us, mask_hs = _decode_mask_rows(attn_mask, users, hq, skv)
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    g = hq // hkv
    rows_per_load = max(1, 1024 // (d * (1 if fmt == N.KV_BFP8 else 2)))
    on_dot_kernel = fmt == N.KV_BF16 and g <= 8 and bs % 4 == 0
    on_matrix_kernel = bs % rows_per_load == 0 and ((g <= 16 and d in (64, 128, 256) and users <= 2048) or
                                                    (g <= 32 and d in (64, 128) and users <= 1024))
    if on_dot_kernel or on_matrix_kernel:
        q = _rows_contiguous(query)
        pt = _table(page_table)
        if out is None:
            out = torch.empty((1, users, hq, d), dtype=query.dtype, device=query.device)
        else:
            _check_out(out, (1, users, hq, d), "decode")
        last = torch.full((users,), skv - 1, dtype=torch.int32, device=query.device)
        ws_bytes = N.lib().ttpa_paged_decode_workspace_bytes(users, hq, hkv, d)
        ws = _workspace(ws_bytes, query.device)
        N.call(
            "ttpa_paged_sdpa_decode_masked",
            out.data_ptr(), out.stride(1), out.stride(2), q.data_ptr(), q.stride(1), q.stride(2),
            key.data_ptr(), value.data_ptr(), pt.data_ptr(), pt.stride(0), last.data_ptr(), 0,
            users, hq, hkv, d, bs, width, nb, float(scale), fmt, mask.data_ptr(), mask_us, mask_hs,
            ws.data_ptr(), ws_bytes, _stream(),
        )
        return out
    return _decode_masked_gathered(query, key, value, page_table, mask, mask_hs, scale, out)


def _decode_masked_gathered(query, key, value, page_table, mask, mask_hs, scale, out):
    """What no decode kernel takes with a mask (more than 32 query heads per KV head, head size 256 with
    more than 16, block sizes that split a 1 KiB load with more than 8 or on a block-float-8 cache):
    the user's blocks gathered in table order, then the prefill kernel's masked dense form on a query
    padded to its 32-row tile.  One mask row for all heads."""
    if mask_hs != 0:
        raise NotImplementedError(
            "a decode attn_mask that differs between heads is built for up to 32 query heads per KV head")
    nb, hkv, bs, d, fmt = _attention_cache_geometry(key)
    _, users, hq, _ = query.shape
    width = page_table.shape[1]
    skv = width * bs

    ids = page_table.reshape(-1).to(torch.int64)
    ids = torch.where((ids >= 0) & (ids < nb), ids, torch.zeros_like(ids))

    def dense(cache):
        g = torch.index_select(cache, 0, ids)
        if fmt == N.KV_BFP8:
            g = bfp8_unpack_cache(g)
        return g.view(users, width, hkv, bs, d).permute(0, 2, 1, 3, 4).reshape(users, hkv, skv, d)

    rows = 32  # the prefill kernel's query tile
    q = torch.zeros((users, hq, rows, d), dtype=torch.bfloat16, device=query.device)
    q[:, :, 0] = query[0]
    mask = mask.expand(users, 1, 1, skv).expand(users, 1, rows, skv).contiguous()
    res = _prefill(q, dense(key), dense(value), None, None, mask, False, scale)[:, :, 0]  # [users, hq, d]
    if out is None:
        return res.unsqueeze(0).contiguous()
    _check_out(out, (1, users, hq, d), "decode")
    out[0].copy_(res)
    return out


def _additive_mask(attn_mask: torch.Tensor) -> torch.Tensor:
    """The mask as the kernels add it to the scaled scores: bfloat16.  A boolean mask means
    "attend where True" (torch.nn.functional.scaled_dot_product_attention's rule)."""
    if attn_mask.dtype == torch.bool:
        return torch.zeros(attn_mask.shape, dtype=torch.bfloat16, device=attn_mask.device).masked_fill(
            ~attn_mask, float("-inf"))
    return attn_mask if attn_mask.dtype == torch.bfloat16 else attn_mask.to(torch.bfloat16)


@torch.library.custom_op("tt::paged_update_kv_decode_", mutates_args=["k_cache", "v_cache"],
                         device_types=["cuda"])
def paged_update_kv_decode_(
    query: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_new: torch.Tensor,
    v_new: torch.Tensor,
    page_table: torch.Tensor,
    cur_pos_tensor: torch.Tensor,
    attention_sink: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    sliding_window_size: Optional[int] = None,
) -> torch.Tensor:
    """The decode step of the attention backend as one operator: ``paged_update_kv_cache_`` with
    ``update_indices = cur_pos_tensor`` followed by the causal
    ``paged_scaled_dot_product_attention_decode`` on the updated caches (reference
    attention.py:473-483 and :634-668).  Same results in the caches and in the output as the
    two operators; where the 16x16x32 decode kernel serves the shape it is one launch.  (The
    equivalence assumes that no user attends a row that another user's token is written to in
    the same step.)"""
    return _decode(query, k_cache, v_cache, page_table, True, None, cur_pos_tensor, attention_sink,
                   scale, sliding_window_size, k_new, v_new)


@paged_update_kv_decode_.register_fake
def _(query, k_cache, v_cache, k_new, v_new, page_table, cur_pos_tensor, attention_sink=None,
      scale=None, sliding_window_size=None):
    return torch.empty_like(query)


@torch.library.custom_op("tt::paged_update_kv_decode_out_", mutates_args=["k_cache", "v_cache", "out"],
                         device_types=["cuda"])
def paged_update_kv_decode_out_(
    query: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_new: torch.Tensor,
    v_new: torch.Tensor,
    page_table: torch.Tensor,
    cur_pos_tensor: torch.Tensor,
    out: torch.Tensor,
    attention_sink: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    sliding_window_size: Optional[int] = None,
) -> None:
    """``paged_update_kv_decode_`` writing into ``out`` [1, users, heads, head_size] (any user /
    head strides): the attention backend hands its output buffer in, which saves the copy the
    reference makes from the operator's result (attention.py:330-336)."""
    _decode(query, k_cache, v_cache, page_table, True, None, cur_pos_tensor, attention_sink,
            scale, sliding_window_size, k_new, v_new, out=out)





@paged_scaled_dot_product_attention_decode.register_fake
def _(query, key, value, page_table, is_causal=False, attn_mask=None, cur_pos_tensor=None,
      attention_sink=None, scale=None, sliding_window_size=None):
    return torch.empty_like(query)


# --------------------------------------------------------------------------- #
# prefill attention
# --------------------------------------------------------------------------- #
def _prefill(query, key, value, page_table, chunk_start, attn_mask, is_causal, scale, window=0, out=None):
    b, hq, s, d = query.shape
    if query.dtype != torch.bfloat16:
        raise ValueError("query must be bfloat16")
    q = _rows_contiguous(query)
    if out is None:
        out = torch.empty_like(q)  # keeps q's (possibly token-major) strides
    else:
        _check_out(out, (b, hq, s, d), "prefill")
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    if not scale > 0:
        raise ValueError(f"scale must be positive, got {scale}")
    if page_table is None:
        if key.dtype != torch.bfloat16 or value.dtype != torch.bfloat16:
            raise ValueError(f"key and value must be bfloat16, got {key.dtype} and {value.dtype}")
        hkv, skv = key.shape[1], key.shape[2]
        k = _rows_contiguous(key)
        v = _rows_contiguous(value)
        if k.stride() != v.stride():
            k, v = k.contiguous(), v.contiguous()
        kv_strides = (k.stride(0), k.stride(1), k.stride(2))
        bs = w = nb = 0
        pt_ptr, pt_rs = 0, 0
        fmt = N.KV_BF16
    else:
        nb, hkv, bs, kd, fmt = _attention_cache_geometry(key)
        if _attention_cache_geometry(value) != (nb, hkv, bs, kd, fmt) or kd != d:
            raise ValueError("chunked attention needs K / V caches of one shape and format, head size as the query's")
        k, v = key, value
        pt = _table(page_table)
        w = pt.shape[1]
        skv = w * bs
        kv_strides = (0, 0, 0)
        pt_ptr, pt_rs = pt.data_ptr(), pt.stride(0)
    mask_ptr, mask_bs, mask_rs = 0, 0, 0
    if attn_mask is not None:
        m = _additive_mask(attn_mask)
        if m.dim() != 4 or m.shape[1] != 1 or m.shape[2] != s or m.shape[3] != skv:
            raise ValueError("attn_mask must be [batch, 1, q_len, kv_len]")
        if m.stride(-1) != 1:
            m = m.contiguous()
        mask_ptr, mask_bs, mask_rs = m.data_ptr(), m.stride(0), m.stride(2)
    # block-float-8 caches: scratch for bfloat16 copies of the blocks the pass reads (the library uses
    # it for the shapes its fastest loop serves and ignores it otherwise)
    ws_ptr, ws_bytes = 0, 0
    if fmt == N.KV_BFP8 and d == 128 and (hq // hkv) % 4 == 0 and bs % 64 == 0 and not window and attn_mask is None:
        need = int(N.lib().ttpa_sdpa_prefill_workspace_bytes(b, hkv, d, bs, w, fmt))
        if 0 < need <= _EXPANSION_LIMIT:
            ws = _workspace(need, q.device)
            ws_ptr, ws_bytes = ws.data_ptr(), need
    N.call(
        "ttpa_sdpa_prefill_expanded",
        out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
        q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
        k.data_ptr(), v.data_ptr(), *kv_strides, pt_ptr, pt_rs, _ptr(chunk_start),
        mask_ptr, mask_bs, mask_rs, b, hq, hkv, s, skv, d, bs, w, nb, int(is_causal),
        float(scale), int(window), fmt, ws_ptr, ws_bytes, _stream(),
    )
    return out


@torch.library.custom_op("tt::scaled_dot_product_attention", mutates_args=[], device_types=["cuda"])
def scaled_dot_product_attention(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    attn_mask: Optional[torch.Tensor] = None,
    is_causal: bool = True,
    scale: Optional[float] = None,
    sliding_window_size: Optional[int] = None,
) -> torch.Tensor:
    assert len(query.shape) == 4, "query must be a 4D tensor: [B, num_heads, query_seq_len, head_size]."
    assert len(key.shape) == 4, "key must be a 4D tensor: [B, num_kv_heads, kv_seq_len, head_size]."
    assert len(value.shape) == 4, "value must be a 4D tensor: [B, num_kv_heads, kv_seq_len, head_size]."
    assert key.shape == value.shape, "key and value must have the same shape."
    assert key.shape[-1] == query.shape[-1], "key and query must have the same head size."
    assert query.shape[1] % key.shape[1] == 0, "num_heads must be divisible by num_kv_heads."
    assert (
        query.shape[2] % 32 == 0
    ), f"query sequence length must be divisible by 32 but got {query.shape[2]}."
    assert query.shape[0] == key.shape[0], "query and key must have the same batch size."
    assert query.device == key.device == value.device, "query, key, and value must be on the same device."
    if attn_mask is not None:
        assert attn_mask.device == query.device, "attn_mask must be on the same device as query, key, and value."
        assert is_causal == False, "is_causal attribute can't be True if attn_mask is available."  # noqa: E712
        assert query.shape[0] == attn_mask.shape[0], "Attention mask batch size must match query batch size."
    if sliding_window_size is not None:
        if sliding_window_size <= 0:
            raise ValueError("sliding_window_size must be positive")
        if not is_causal:
            raise NotImplementedError("sliding_window_size is built for the causal form only")
    return _prefill(query, key, value, None, None, attn_mask, is_causal, scale,
                    window=sliding_window_size or 0)


@scaled_dot_product_attention.register_fake
def _(query, key, value, attn_mask=None, is_causal=True, scale=None, sliding_window_size=None):
    return torch.empty_like(query)


@torch.library.custom_op("tt::scaled_dot_product_attention_out", mutates_args=["out"], device_types=["cuda"])
def scaled_dot_product_attention_out(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    out: torch.Tensor,
    attn_mask: Optional[torch.Tensor] = None,
    is_causal: bool = True,
    scale: Optional[float] = None,
    sliding_window_size: Optional[int] = None,
) -> None:
    """``scaled_dot_product_attention`` writing into ``out`` [B, heads, q_len, head_size] (any
    batch / head / token strides): the attention backend hands its output buffer in, which saves
    the copy the reference makes from the operator's result (attention.py:330-336)."""
    assert query.dim() == 4 and key.dim() == 4 and key.shape == value.shape
    assert query.shape[2] % 32 == 0, f"query sequence length must be divisible by 32 but got {query.shape[2]}."
    if attn_mask is not None:
        assert is_causal == False, "is_causal attribute can't be True if attn_mask is available."  # noqa: E712
    if sliding_window_size is not None:
        if sliding_window_size <= 0:
            raise ValueError("sliding_window_size must be positive")
        if not is_causal:
            raise NotImplementedError("sliding_window_size is built for the causal form only")
    _prefill(query, key, value, None, None, attn_mask, is_causal, scale,
             window=sliding_window_size or 0, out=out)


@torch.library.custom_op(
    "tt::chunked_scaled_dot_product_attention", mutates_args=[], device_types=["cuda"]
)
def chunked_scaled_dot_product_attention(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    page_table: torch.Tensor,
    chunk_start_idx_tensor: torch.Tensor,
    scale: Optional[float] = None,
) -> torch.Tensor:
    if query.dim() != 4:
        raise ValueError("query must be [users, heads, chunk_len, head_size]")
    if page_table.dim() != 2 or page_table.shape[0] != query.shape[0]:
        raise ValueError("page_table must have one row per user")
    start = chunk_start_idx_tensor.reshape(-1)
    if start.dtype != torch.int32:
        start = start.to(torch.int32)
    return _prefill(query, key, value, page_table, start, None, True, scale)


@chunked_scaled_dot_product_attention.register_fake
def _(query, key, value, page_table, chunk_start_idx_tensor, scale=None):
    return torch.empty_like(query)


@torch.library.custom_op(
    "tt::chunked_scaled_dot_product_attention_out", mutates_args=["out"], device_types=["cuda"]
)
def chunked_scaled_dot_product_attention_out(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    page_table: torch.Tensor,
    chunk_start_idx_tensor: torch.Tensor,
    out: torch.Tensor,
    scale: Optional[float] = None,
) -> None:
    """``chunked_scaled_dot_product_attention`` writing into ``out`` (see
    ``scaled_dot_product_attention_out``)."""
    if query.dim() != 4:
        raise ValueError("query must be [users, heads, chunk_len, head_size]")
    if page_table.dim() != 2 or page_table.shape[0] != query.shape[0]:
        raise ValueError("page_table must have one row per user")
    start = chunk_start_idx_tensor.reshape(-1)
    if start.dtype != torch.int32:
        start = start.to(torch.int32)
    _prefill(query, key, value, page_table, start, None, True, scale, out=out)


@torch.library.custom_op("tt::paged_fill_kv_prefill_out_", mutates_args=["k_cache", "v_cache", "out"],
                         device_types=["cuda"])
def paged_fill_kv_prefill_out_(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    fill_page_table: torch.Tensor,
    batch_idx: Optional[torch.Tensor],
    out: torch.Tensor,
    is_causal: bool = True,
    scale: Optional[float] = None,
    sliding_window_size: Optional[int] = None,
) -> None:
    """The first-chunk prefill pass of the attention backend as one operator:
    ``paged_fill_cache_`` of ``key`` into ``k_cache`` and of ``value`` into ``v_cache`` through
    ``fill_page_table`` / ``batch_idx`` (reference attention.py:486-515) and the dense
    ``scaled_dot_product_attention_out`` on the same ``query`` / ``key`` / ``value``
    [B, heads, tokens, head_size] (:576-596).  Same results in the caches and in ``out`` as the
    three operators; one launch (the rows are copied by extra workgroups of the attention
    kernel).  bfloat16 caches only."""
    b, hq, s, d = query.shape
    nb, hkv, bs, cd, fmt = _cache_geometry(k_cache)
    if fmt != N.KV_BF16 or _cache_geometry(v_cache) != (nb, hkv, bs, cd, fmt):
        raise ValueError("prefill + fill needs matching bfloat16 K / V caches")
    if key.shape != value.shape or key.dim() != 4 or key.shape[0] != b or key.shape[1] != hkv or key.shape[3] != d or cd != d:
        raise ValueError(f"key / value {tuple(key.shape)} do not match the query and the cache geometry")
    if query.dtype != torch.bfloat16 or key.dtype != torch.bfloat16 or value.dtype != torch.bfloat16:
        raise ValueError("query / key / value must be bfloat16")
    if s % 32:
        raise ValueError(f"query sequence length must be divisible by 32 but got {s}.")
    if sliding_window_size is not None:
        if sliding_window_size <= 0:
            raise ValueError("sliding_window_size must be positive")
        if not is_causal:
            raise NotImplementedError("sliding_window_size is built for the causal form only")
    if fill_page_table.dim() != 2:
        raise ValueError("fill_page_table must be [users, blocks_per_user]")
    skv = key.shape[2]
    if skv > fill_page_table.shape[1] * bs:
        raise ValueError(f"{skv} tokens do not fit {fill_page_table.shape[1]} page-table columns of {bs} tokens")
    if batch_idx is None:
        if b != 1:
            raise ValueError("batch_idx is required when key holds more than one user")
    else:
        if batch_idx.numel() != b:
            raise ValueError("batch_idx must have one entry per key row")
        batch_idx = _index_tensor(batch_idx.reshape(-1))
    q = _rows_contiguous(query)
    k, v = _rows_contiguous(key), _rows_contiguous(value)
    if k.stride() != v.stride():
        k, v = k.contiguous(), v.contiguous()
    _check_out(out, (b, hq, s, d), "prefill + fill")
    pt = _table(fill_page_table)
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    N.call(
        "ttpa_sdpa_prefill_fill",
        out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
        q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
        k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), k.stride(2),
        b, hq, hkv, s, skv, d, int(is_causal), float(scale), int(sliding_window_size or 0),
        k_cache.data_ptr(), v_cache.data_ptr(), pt.data_ptr(), pt.stride(0), _ptr(batch_idx),
        int(batch_idx is not None and batch_idx.dtype == torch.int64), pt.shape[0], bs, pt.shape[1], nb,
        _stream(),
    )


# --------------------------------------------------------------------------- #
# latent (MLA) attention
# --------------------------------------------------------------------------- #
_MLA_MAX_USERS = 1024  # users per launch of the latent decode kernel


def _mla_decode_launch(out, q, key, value, page_table, cur, head_dim_v, scale, sink, mask=None):
    """out [users, heads, dv] / q [users, heads, dh] by strides; caches in the paged layout.
    mask: (bfloat16 tensor [users or 1, heads or 1, 1, positions], user stride, head stride) or None."""
    nb, nkv, bs, dh = key.shape
    users, hq = q.shape[0], q.shape[1]
    for u0 in range(0, users, _MLA_MAX_USERS):
        n = min(_MLA_MAX_USERS, users - u0)
        ws_bytes = N.lib().ttpa_paged_mla_decode_workspace_bytes(n, hq, nkv, head_dim_v)
        if ws_bytes == 0:
            raise NotImplementedError(
                f"latent attention with {hq} query heads over {nkv} KV heads is not built "
                "(heads per KV head: up to 32 or a multiple of 32)"
            )
        ws = _workspace(ws_bytes, q.device)
        qs, os_, pts, curs = q[u0 : u0 + n], out[u0 : u0 + n], page_table[u0 : u0 + n], cur[u0 : u0 + n]
        if mask is not None:
            m, m_us, m_hs = mask
            N.call(
                "ttpa_paged_mla_decode_masked",
                os_.data_ptr(), os_.stride(0), os_.stride(1), qs.data_ptr(), qs.stride(0), qs.stride(1),
                key.data_ptr(), _ptr(value), pts.data_ptr(), pts.stride(0), curs.data_ptr(),
                int(curs.dtype == torch.int64), n, hq, nkv, dh, head_dim_v, bs, pts.shape[1], nb,
                float(scale), m.data_ptr() + 2 * u0 * m_us, m_us, m_hs, ws.data_ptr(), ws_bytes, _stream(),
            )
            continue
        N.call(
            "ttpa_paged_mla_decode",
            os_.data_ptr(), os_.stride(0), os_.stride(1), qs.data_ptr(), qs.stride(0), qs.stride(1),
            key.data_ptr(), _ptr(value), pts.data_ptr(), pts.stride(0), curs.data_ptr(),
            int(curs.dtype == torch.int64), n, hq, nkv, dh, head_dim_v, bs, pts.shape[1], nb,
            float(scale), _ptr(sink), ws.data_ptr(), ws_bytes, _stream(),
        )


@torch.library.custom_op("tt::paged_flash_mla_decode", mutates_args=[], device_types=["cuda"])
def paged_flash_mla_decode(
    query: torch.Tensor,
    key: torch.Tensor,
    head_dim_v: int,
    page_table: torch.Tensor,
    value: Optional[torch.Tensor] = None,
    is_causal: bool = True,
    attn_mask: Optional[torch.Tensor] = None,
    cur_pos_tensor: Optional[torch.Tensor] = None,
    attention_sink: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """Paged decode over a latent KV cache (reference custom_ops.py:381-632): query
    [1, users, nqh, dh_qk], key cache [blocks, nkv, block_size, dh_qk], optional value cache
    [blocks, nkv, block_size, head_dim_v]; without it V is key[..., :head_dim_v]."""
    assert len(query.shape) == 4, "query must be a 4D tensor: [1, num_users, nqh, dh_qk]."
    assert len(key.shape) == 4, "key must be a 4D tensor: [max_num_blocks, nkv, block_size, dh_qk]."
    assert len(page_table.shape) == 2, "page_table must be a 2D tensor: [num_users, num_blocks_per_user]."
    assert query.shape[0] == 1, "query dim 0 must be 1 (decode processes one token per user)."
    assert key.shape[-1] == query.shape[-1], "key and query must have the same head size (dh_qk)."
    assert query.shape[2] % key.shape[1] == 0, "nqh must be divisible by nkv (GQA/MQA/MLA constraint)."
    assert page_table.shape[0] == query.shape[1], "page_table number of users must match query number of users."
    assert isinstance(head_dim_v, int) and head_dim_v > 0, f"head_dim_v must be a positive int, got {head_dim_v}."
    if value is not None:
        assert len(value.shape) == 4, "value must be a 4D tensor: [max_num_blocks, nkv, block_size, head_dim_v]."
        assert value.shape[:3] == key.shape[:3], "value's block/head/block_size dims must match key's."
        assert value.shape[-1] == head_dim_v, f"value's last dim ({value.shape[-1]}) must equal head_dim_v ({head_dim_v})."
    else:
        assert head_dim_v <= key.shape[-1], (
            f"head_dim_v ({head_dim_v}) cannot exceed key's head dim ({key.shape[-1]}) when value is None."
        )
    if is_causal:
        assert attn_mask is None, "attn_mask must be None when is_causal is True."
        assert cur_pos_tensor is not None, "cur_pos_tensor must be provided when is_causal is True."
    if attn_mask is not None:
        assert not is_causal, "attn_mask requires is_causal to be False."
    else:
        assert is_causal, "is_causal must be True when attn_mask is not provided"
    if is_causal:
        assert len(cur_pos_tensor.shape) == 1, "cur_pos_tensor must be a 1D tensor: [num_users]."
        assert cur_pos_tensor.shape[0] == query.shape[1], "cur_pos_tensor number of users must match query number of users."
    if query.dtype != torch.bfloat16 or key.dtype != torch.bfloat16 or not key.is_contiguous():
        raise ValueError("query and the key cache must be bfloat16, the cache contiguous")
    if value is not None and (value.dtype != torch.bfloat16 or not value.is_contiguous()):
        raise ValueError("the value cache must be contiguous bfloat16")
    users, hq, dh = query.shape[1], query.shape[2], query.shape[3]
    if scale is None:
        scale = 1.0 / math.sqrt(dh)
    q = _rows_contiguous(query)[0]
    out = torch.empty((1, users, hq, head_dim_v), dtype=query.dtype, device=query.device)
    sink = None
    if attention_sink is not None:
        if attention_sink.numel() != hq:
            raise ValueError(f"attention_sink must hold one logit per query head ({hq})")
        sink = attention_sink.reshape(hq).to(device=query.device, dtype=torch.float32).contiguous()
    if is_causal:
        _mla_decode_launch(out[0], q, key, value, _table(page_table), _index_tensor(cur_pos_tensor),
                           head_dim_v, scale, sink)
        return out
    # is_causal=False (reference custom_ops.py:590-592): every position of the table, weighted by the mask
    if sink is not None:
        raise NotImplementedError("attention_sink with an explicit attn_mask is not built")
    skv = page_table.shape[1] * key.shape[2]
    last = torch.full((users,), skv - 1, dtype=torch.int32, device=query.device)
    _mla_decode_launch(out[0], q, key, value, _table(page_table), last, head_dim_v, scale, None,
                       _decode_mask_rows(attn_mask, users, hq, skv))
    return out


@paged_flash_mla_decode.register_fake
def _(query, key, head_dim_v, page_table, value=None, is_causal=True, attn_mask=None,
      cur_pos_tensor=None, attention_sink=None, scale=None):
    return torch.empty((query.shape[0], query.shape[1], query.shape[2], head_dim_v),
                       dtype=query.dtype, device=query.device)


# (head size, value width) pairs ttpa_latent_prefill is built for
_LATENT_PREFILL_SHAPES = {(576, 512), (192, 128), (128, 128)}


@torch.library.custom_op("tt::flash_mla_prefill", mutates_args=[], device_types=["cuda"])
def flash_mla_prefill(
    query: torch.Tensor,
    key: torch.Tensor,
    head_dim_v: int,
    value: Optional[torch.Tensor] = None,
    attn_mask: Optional[torch.Tensor] = None,
    is_causal: bool = True,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """Causal prefill over freshly built latent K (reference custom_ops.py:223-378): query
    [b, nqh, s, dh_qk], key [b, nkv, s, dh_qk], optional value [b, nkv, s, head_dim_v].

    With V taken from K and a head size the prefill kernel is built for, one launch of
    ttpa_latent_prefill; otherwise the latent decode kernels, one launch per batch entry."""
    assert len(query.shape) == 4, "query must be a 4D tensor: [b, nqh, s, dh_qk]."
    assert len(key.shape) == 4, "key must be a 4D tensor: [b, nkv, s, dh_qk]."
    assert key.shape[-1] == query.shape[-1], "key and query must have the same head size (dh_qk)."
    assert query.shape[0] == key.shape[0], "query and key must have the same batch size."
    assert query.shape[2] == key.shape[2], "query and key must have the same sequence length for MLA prefill."
    assert query.shape[1] % key.shape[1] == 0, "nqh must be divisible by nkv (GQA/MQA/MLA constraint)."
    assert query.shape[2] % 32 == 0, f"query sequence length must be divisible by 32 but got {query.shape[2]}."
    assert isinstance(head_dim_v, int) and head_dim_v > 0, f"head_dim_v must be a positive int, got {head_dim_v}."
    if value is not None:
        assert len(value.shape) == 4, "value must be a 4D tensor: [b, nkv, s, head_dim_v]."
        assert value.shape[:3] == key.shape[:3], "value's batch/head/seq dims must match key's."
        assert value.shape[-1] == head_dim_v, f"value's last dim ({value.shape[-1]}) must equal head_dim_v ({head_dim_v})."
    else:
        assert head_dim_v <= key.shape[-1], (
            f"head_dim_v ({head_dim_v}) cannot exceed key's head dim ({key.shape[-1]}) when value is None."
        )
    if attn_mask is not None:
        assert is_causal == False, "is_causal cannot be True when attn_mask is provided."  # noqa: E712
        assert attn_mask.shape[0] == query.shape[0], "attention mask batch size must match query batch size."
    else:
        assert is_causal == True, "is_causal must be True if attn_mask is not provided"  # noqa: E712
    if query.dtype != torch.bfloat16 or key.dtype != torch.bfloat16:
        raise ValueError("query and key must be bfloat16")
    b, hq, s, dh = query.shape
    if scale is None:
        scale = 1.0 / math.sqrt(dh)
    q = _rows_contiguous(query)
    k = key.contiguous()
    v = value.contiguous() if value is not None else None
    out = torch.empty((b, hq, s, head_dim_v), dtype=query.dtype, device=query.device)
    if v is None and (dh, head_dim_v) in _LATENT_PREFILL_SHAPES:
        # the prefill kernel: 128 (token, head) rows share every K tile
        mask_ptr, mask_strides = 0, (0, 0, 0)
        if attn_mask is not None:
            m = _additive_mask(attn_mask)
            if m.dim() != 4 or m.shape[0] != b or m.shape[1] not in (1, hq) or m.shape[2] != s or m.shape[3] != s:
                raise ValueError(f"attn_mask must broadcast to [{b}, {hq}, {s}, {s}], got {tuple(attn_mask.shape)}")
            if m.stride(-1) != 1 or any(st % 4 for st in m.stride()[:3]) or m.data_ptr() % 8:
                m = m.contiguous()
            mask_ptr = m.data_ptr()
            mask_strides = (m.stride(0), m.stride(1) if m.shape[1] == hq and hq > 1 else 0, m.stride(2))
        N.call(
            "ttpa_latent_prefill",
            out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
            q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
            k.data_ptr(), k.stride(0), k.stride(1), k.stride(2),
            mask_ptr, *mask_strides, b, hq, key.shape[1], s, dh, head_dim_v, int(is_causal), float(scale), _stream(),
        )
        return out
    # other shapes, and a separate V: the decode kernels, query row i of a sequence being a user at
    # position i whose cache is the sequence itself (one block of s tokens, a one-column page table)
    table = torch.zeros((s, 1), dtype=torch.int32, device=query.device)
    mask = None
    if attn_mask is None:
        cur = torch.arange(s, dtype=torch.int32, device=query.device)
    else:
        # every key, weighted by the mask row of the query token (reference custom_ops.py:349-357):
        # anything that broadcasts to [b, heads, s, s]; row i of a sequence is user i
        cur = torch.full((s,), s - 1, dtype=torch.int32, device=query.device)
        mask = _additive_mask(attn_mask)
        if mask.dim() != 4 or mask.shape[1] not in (1, hq) or mask.shape[2] != s or mask.shape[3] != s:
            raise ValueError(f"attn_mask must broadcast to [{b}, {hq}, {s}, {s}], got {tuple(attn_mask.shape)}")
        if mask.stride(-1) != 1:
            mask = mask.contiguous()
    for i in range(b):
        # [s, heads, d] views: token-major "users", the sequence as a single block of s tokens
        rows = None
        if mask is not None:
            rows = (mask[i], mask.stride(2), mask.stride(1) if mask.shape[1] == hq and hq > 1 else 0)
        _mla_decode_launch(out[i].transpose(0, 1), q[i].transpose(0, 1), k[i : i + 1],
                           None if v is None else v[i : i + 1], table, cur, head_dim_v, scale, None, rows)
    return out


@flash_mla_prefill.register_fake
def _(query, key, head_dim_v, value=None, attn_mask=None, is_causal=True, scale=None):
    return torch.empty((query.shape[0], query.shape[1], query.shape[2], head_dim_v),
                       dtype=query.dtype, device=query.device)


# --------------------------------------------------------------------------- #
# non-paged (static) cache: [batch, kv_heads, max_seq_len, head_size]
# --------------------------------------------------------------------------- #
# A static cache is a paged cache whose block u is the whole sequence of user u: the same
# kernels run with block_size = max_seq_len and the one-column page table [[0], [1], ...].
def _identity_table(batch: int, device) -> torch.Tensor:
    return torch.arange(batch, dtype=torch.int32, device=device).view(batch, 1)


def _static_geometry(cache: torch.Tensor):
    if cache.dim() != 4:
        raise ValueError("cache must be a 4D tensor: [B, num_heads, max_seq_len, head_size].")
    if cache.dtype not in (torch.bfloat16, torch.float16) or not cache.is_contiguous():
        raise ValueError("static caches must be contiguous 16-bit floating point tensors")
    return cache.shape


def _static_update_inplace(cache, fill_value, cache_position, batch_offset):
    assert len(cache.shape) == 4, "cache must be a 4D tensor: [B, num_heads, max_seq_len, head_size]."
    assert len(fill_value.shape) == 4, "fill_value must be a 4D tensor: [B, num_heads, 1, head_size]."
    assert fill_value.shape[-2] == 1, (
        "fill_value must have dim -2 equal to 1 as the cache cannot be updated with more than one "
        "token at a time."
    )
    assert batch_offset is not None or cache.shape[0] == 1, "batch_offset must be provided if the batch size is not 1."
    assert cache_position.shape == (1,), "cache_position must be a 1D tensor."
    assert not batch_offset, "Only batch_offset == 0 is supported for currently."
    b = _static_geometry(cache)[0]
    if fill_value.shape[0] != b:
        raise ValueError("fill_value and cache must have the same batch size")
    _update_inplace(cache, fill_value.permute(2, 0, 1, 3), cache_position.expand(b), _identity_table(b, cache.device))


@torch.library.custom_op("tt::update_cache", mutates_args=[], device_types=["cuda"])
def update_cache(
    cache: torch.Tensor,
    fill_value: torch.Tensor,
    cache_position: torch.Tensor,
    batch_offset: Optional[int] = None,
) -> torch.Tensor:
    """cache[:, :, cache_position, :] = fill_value on a copy (reference custom_ops.py:857-900);
    one position shared by the whole batch.  Positions outside [0, max_seq_len) write nothing."""
    out = cache.clone()
    _static_update_inplace(out, fill_value, cache_position, batch_offset)
    return out


@update_cache.register_fake
def _(cache, fill_value, cache_position, batch_offset=None):
    return torch.empty_like(cache)


@torch.library.custom_op("tt::update_cache_", mutates_args=["cache"], device_types=["cuda"])
def update_cache_(
    cache: torch.Tensor,
    fill_value: torch.Tensor,
    cache_position: torch.Tensor,
    batch_offset: Optional[int] = None,
) -> None:
    _static_update_inplace(cache, fill_value, cache_position, batch_offset)


@update_cache_.register_fake
def _(cache, fill_value, cache_position, batch_offset=None):
    return None


def _static_fill_inplace(cache, fill_value, batch_offset):
    assert len(cache.shape) == 4, "cache must be a 4D tensor: [B, num_heads, max_seq_len, head_size]."
    assert len(fill_value.shape) == 4, "fill_value must be a 4D tensor: [B, num_heads, seq_len, head_size]."
    assert fill_value.shape[-2] <= cache.shape[-2], (
        "fill_value must have dim -2 less than or equal to cache.shape[-2] as the cache cannot be "
        f"filled with more tokens than the cache can hold. Recieved fill_value.shape = {fill_value.shape}, "
        f"cache.shape = {cache.shape}."
    )
    assert batch_offset is not None or cache.shape[0] == 1, "batch_offset must be provided if the batch size is not 1."
    assert not batch_offset, "Only batch_offset == 0 is supported for currently."
    b = _static_geometry(cache)[0]
    if fill_value.shape[0] != b:
        raise ValueError("fill_value and cache must have the same batch size")
    _fill_inplace(cache, fill_value, _identity_table(b, cache.device),
                  torch.arange(b, dtype=torch.int32, device=cache.device))


@torch.library.custom_op("tt::fill_cache", mutates_args=[], device_types=["cuda"])
def fill_cache(cache: torch.Tensor, fill_value: torch.Tensor, batch_offset: Optional[int] = None) -> torch.Tensor:
    """cache[:, :, :seq_len, :] = fill_value on a copy (reference custom_ops.py:903-950)."""
    out = cache.clone()
    _static_fill_inplace(out, fill_value, batch_offset)
    return out


@fill_cache.register_fake
def _(cache, fill_value, batch_offset=None):
    return torch.empty_like(cache)


@torch.library.custom_op("tt::fill_cache_", mutates_args=["cache"], device_types=["cuda"])
def fill_cache_(cache: torch.Tensor, fill_value: torch.Tensor, batch_offset: Optional[int] = None) -> None:
    _static_fill_inplace(cache, fill_value, batch_offset)


@fill_cache_.register_fake
def _(cache, fill_value, batch_offset=None):
    return None


@torch.library.custom_op("tt::scaled_dot_product_attention_decode", mutates_args=[], device_types=["cuda"])
def scaled_dot_product_attention_decode(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    cur_pos_tensor: torch.Tensor,
    attn_mask: Optional[torch.Tensor] = None,
    attention_sink: Optional[torch.Tensor] = None,
    is_causal: bool = True,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """Decode attention over static caches (reference custom_ops.py:745-842): user b attends
    positions 0 .. cur_pos_tensor[b] of key[b] / value[b]; grouped heads; optional sink."""
    assert len(query.shape) == 4, "query must be a 4D tensor: [1, B, num_heads, head_size]."
    assert len(key.shape) == 4, "key must be a 4D tensor: [B, num_kv_heads, seq_len, head_size]."
    assert len(value.shape) == 4, "value must be a 4D tensor: [B, num_kv_heads, seq_len, head_size]."
    assert len(cur_pos_tensor.shape) == 1, "cur_pos_tensor must be a 1D tensor: [B]."
    assert key.shape == value.shape, "key and value must have the same shape."
    assert key.shape[-1] == query.shape[-1], "key and query must have the same head size."
    assert query.shape[2] % key.shape[1] == 0, (
        f"num_heads must be divisible by num_kv_heads. Query shape: {query.shape}, key shape: {key.shape}."
    )
    assert query.shape[0] == 1, "query must have dim 0 equal to 1."
    assert query.shape[1] == key.shape[0], "query and key must have the same batch size."
    if is_causal:
        assert attn_mask is None, "attn_mask must be None when is_causal is True."
    _static_geometry(key), _static_geometry(value)
    if key.shape[2] % 4:
        raise NotImplementedError("static-cache decode needs max_seq_len to be a multiple of 4")
    if attn_mask is not None:
        # is_causal=False: all max_seq_len positions, weighted by the mask, one row per query head
        # ([B, 1, heads, S] reshaped to [B, heads, 1, S], reference custom_ops.py:820-821)
        assert not is_causal, "attn_mask requires is_causal to be False."
        b, heads, seq = key.shape[0], query.shape[2], key.shape[2]
        if attn_mask.numel() != b * heads * seq:
            raise ValueError(f"attn_mask must hold batch x heads x max_seq_len = {b} x {heads} x {seq} values")
        if attention_sink is not None:
            raise NotImplementedError("attention_sink with an explicit attn_mask is not built")
        return paged_scaled_dot_product_attention_decode(
            query, key, value, _identity_table(b, key.device), is_causal=False,
            attn_mask=attn_mask.reshape(b, heads, 1, seq), scale=scale,
        )
    assert is_causal, "is_causal must be True when attn_mask is not provided"
    # the cache tensor already has the paged layout [blocks = B, kv_heads, block_size = S, D]
    return paged_scaled_dot_product_attention_decode(
        query, key, value, _identity_table(key.shape[0], key.device), is_causal=True,
        cur_pos_tensor=cur_pos_tensor, attention_sink=attention_sink, scale=scale,
    )


@scaled_dot_product_attention_decode.register_fake
def _(query, key, value, cur_pos_tensor, attn_mask=None, attention_sink=None, is_causal=True, scale=None):
    return torch.empty_like(query)


# --------------------------------------------------------------------------- #
# block-float-8 helpers (cache conversion; no reference operator)
# --------------------------------------------------------------------------- #
def bfp8_pack_cache(cache: torch.Tensor) -> torch.Tensor:
    """bf16 [NB, Hkv, bs, D] -> uint8 [NB, Hkv, bs + bs/16, D] on the device."""
    nb, hkv, bs, d = cache.shape
    cache = cache.contiguous()
    out = torch.empty(bfp8_cache_shape(nb, hkv, bs, d), dtype=torch.uint8, device=cache.device)
    elem = torch.empty((nb, hkv, bs, d), dtype=torch.uint8, device=cache.device)
    exps = torch.empty((nb, hkv, bs * d // _BFP8_GROUP), dtype=torch.uint8, device=cache.device)
    N.call("ttpa_bfp8_quantize", cache.data_ptr(), elem.data_ptr(), exps.data_ptr(),
           cache.numel(), _stream())
    out[:, :, :bs, :] = elem
    out[:, :, bs:, :] = exps.view(nb, hkv, bs // _BFP8_GROUP, d)
    return out


def bfp8_unpack_cache(packed: torch.Tensor) -> torch.Tensor:
    """uint8 [NB, Hkv, bs + bs/16, D] -> bf16 [NB, Hkv, bs, D] (exact decode)."""
    nb, hkv, bs, d, fmt = _cache_geometry(packed)
    assert fmt == N.KV_BFP8
    elem = packed[:, :, :bs, :].contiguous()
    exps = packed[:, :, bs:, :].contiguous()
    out = torch.empty((nb, hkv, bs, d), dtype=torch.bfloat16, device=packed.device)
    N.call("ttpa_bfp8_dequantize", elem.data_ptr(), exps.data_ptr(), out.data_ptr(),
           out.numel(), _stream())
    return out
