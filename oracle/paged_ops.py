"""Torch (CPU) restatement of the reference's CPU semantics for the five ops on the
paged-attention path.  TEST INFRASTRUCTURE: see ``oracle/__init__.py``.

Every function names the reference lines it follows.  Shapes use
B = users, Hq / Hkv = query / KV heads, D = head size, bs = block size,
NB = physical blocks, W = page-table width.

What pins each function (see tests/test_oracle_*.py):
  paged_update_cache     brute-force per-(user, head) loop, negative index and
                         padded-head cases, the reference's own parameter grid
                         (tests/torch/ops/test_custom_ops.py:139-168)
  paged_fill_cache       brute-force per-token loop over the reference's grid
                         (test_custom_ops.py:171-203), tail block kept intact
  paged_sdpa_decode      fp32 textbook attention over the first cur_pos+1 gathered
                         tokens; GQA form against the chunked op with a 1-token chunk;
                         the masked form (is_causal=False) against the causal one with the
                         causal mask handed in, and against an fp32 loop with a random mask
  chunked_sdpa           the reference's independent oracle and cases restated
                         (tests/torch/ops/test_chunked_sdpa_op_cpu.py:27-147)
  sdpa                   library routine (F.scaled_dot_product_attention)
  update_cache / fill_cache / sdpa_decode_static
                         the non-paged forms (custom_ops.py:745-950): plain slice
                         assignments, checked element by element, and the library SDPA
                         with the reference's own additive mask, checked against the fp32
                         loop and against the paged oracle on an identity page table
  flash_mla_prefill / paged_flash_mla_decode
                         the latent-attention forms (custom_ops.py:343-357, 551-610): the
                         library SDPA on gathered K with V = key[..., :head_dim_v]; checked
                         against an fp32 loop with separate QK / V widths and against the
                         grouped decode oracle when V is given explicitly
  paged_sdpa_decode_windowed / sdpa_windowed
                         PARITY UNPINNED against the reference: its CPU branches ignore
                         `sliding_window_size` and `attention_sink`
                         (custom_ops.py:1256-1312, 717-727) and the device kernels that
                         honour them are not in the tree.  The semantics are specified
                         here (window = newest W positions, current one included; sink =
                         one value-less softmax entry per head) and pinned by mathematics:
                         a window at least as long as the context changes nothing, a
                         brute-force loop over the attended range, and the closed form
                         out_sink = out * sigmoid(logsumexp(scores) - sink).
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------- #
# cache writes
# --------------------------------------------------------------------------- #
def paged_update_cache(
    cache: torch.Tensor,
    fill_value: torch.Tensor,
    update_indices: torch.Tensor,
    page_table: torch.Tensor,
    share_cache: bool = False,
) -> torch.Tensor:
    """One-token-per-user scatter into a paged cache; functional (returns a copy).

    Follows python_package/tt_torch/custom_ops.py:981-1000.
    cache [NB, Hkv, bs, D]; fill_value [1, B, >=Hkv, D]; update_indices [B] (any int
    dtype); page_table [B, W].  Index arithmetic is torch's floor division /
    modulo, so position -1 means (column -1, offset bs-1), and column -1 is the
    last page-table column (ordinary negative indexing).
    """
    out = cache.clone()
    bs = out.shape[-2]
    hkv = out.shape[-3]
    users = update_indices.shape[0]
    col = update_indices // bs
    off = update_indices % bs
    phys = page_table[torch.arange(users), col]
    # two index tensors separated by a slice: the indexed dims move to the front,
    # so the target view is [B, Hkv, D].
    out[phys, :, off, :] = fill_value[0, :, :hkv, :]
    return out


def paged_fill_cache(
    cache: torch.Tensor,
    fill_value: torch.Tensor,
    page_table: torch.Tensor,
    batch_idx: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Block-wise prefill write for ONE user; functional.

    Follows custom_ops.py:1037-1092.  cache [NB, Hkv, bs, D]; fill_value
    [1, Hkv, S, D]; page_table [B, Wf]; batch_idx [1].  Writing always starts at
    page-table column 0; the S // bs full blocks are replaced whole and the
    S % bs remaining tokens go to the head of the next block, whose other rows keep
    their old contents.
    """
    if batch_idx is None:
        batch_idx = torch.tensor([0], dtype=torch.int32)
    out = cache.clone()
    bs = out.shape[-2]
    s = fill_value.shape[-2]
    h = fill_value.shape[-3]
    d = fill_value.shape[-1]
    row = page_table[batch_idx.item()]
    n_full, rem = divmod(s, bs)
    if n_full > 0:
        body = fill_value[:, :, : n_full * bs, :]
        # [1, H, n*bs, D] -> [n, H, bs, D]
        body = body.reshape(1, h, n_full, bs, d).transpose(0, 2).reshape(n_full, h, bs, d)
        out[row[:n_full]] = body
    if rem > 0:
        out[row[n_full : n_full + 1], :, :rem, :] = fill_value[:, :, s - rem :, :]
    return out


def paged_fill_cache_batched(
    cache: torch.Tensor,
    fill_value: torch.Tensor,
    page_table: torch.Tensor,
    batch_idx: torch.Tensor,
) -> torch.Tensor:
    """Batched prefill write: row i of fill_value [B, Hkv, S, D] goes through
    page_table[batch_idx[i]].

    The reference's CPU branch cannot run this form (``batch_idx.item()`` raises for
    more than one element, custom_ops.py:1044); the plugin nevertheless calls the
    device op this way (vllm_tt/attention_impls/attention.py:486-511).  The meaning
    is fixed BY DEFINITION as the single-user op applied row by row, which is what
    the MLA impl spells out (attention_impls/attention_mla.py:350-358).
    """
    out = cache
    for i in range(fill_value.shape[0]):
        out = paged_fill_cache(out, fill_value[i : i + 1], page_table, batch_idx[i : i + 1])
    if fill_value.shape[0] == 0:
        out = cache.clone()
    return out


def gather_paged_to_dense(cache: torch.Tensor, page_table: torch.Tensor) -> torch.Tensor:
    """[NB, Hkv, bs, D] + [B, W] -> [B, Hkv, W*bs, D]; position p of user u is
    block page_table[u, p // bs], row p % bs.

    Follows attention.py:600-632 (without the final trim) and custom_ops.py:1387-1403.
    """
    users, w = page_table.shape
    _, hkv, bs, d = cache.shape
    g = torch.index_select(cache, 0, page_table.reshape(-1).long())
    g = g.view(users, w, hkv, bs, d).permute(0, 2, 1, 3, 4).contiguous()
    return g.reshape(users, hkv, w * bs, d)


# --------------------------------------------------------------------------- #
# decode attention
# --------------------------------------------------------------------------- #
def paged_sdpa_decode_mha(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    page_table: torch.Tensor,
    cur_pos_tensor: torch.Tensor,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """The reference's causal decode branch, op by op, for Hq == Hkv.

    Follows custom_ops.py:1256-1312: dense zero-initialised K/V of W*bs positions
    per user, additive mask with -inf right of cur_pos, then
    ``(q @ K^T) * scale + mask -> softmax -> @ V`` with every intermediate in the
    query dtype.  query [1, B, H, D] -> [1, B, H, D].
    """
    bs = key.shape[-2]
    h = key.shape[-3]
    d = key.shape[-1]
    users = cur_pos_tensor.shape[0]
    w = page_table.shape[1]
    span = w * bs
    dt = query.dtype
    mask = torch.zeros(users, span, dtype=dt)
    dense_k = torch.zeros(users, h, span, d, dtype=dt)
    dense_v = torch.zeros(users, h, span, d, dtype=dt)
    for u in range(users):
        blocks = page_table[u].long()
        dense_k[u] = key[blocks].transpose(0, 1).reshape(h, span, d)
        dense_v[u] = value[blocks].transpose(0, 1).reshape(h, span, d)
        mask[u, int(cur_pos_tensor[u]) + 1 :] = float("-inf")
    q = query.reshape(users, h, 1, d)
    if scale is None:
        scale = 1 / d**0.5
    w_ = q @ dense_k.transpose(-2, -1) * scale
    w_ += mask.reshape(users, 1, 1, span)
    w_ = torch.softmax(w_, dim=-1)
    out = w_ @ dense_v
    return out.reshape(1, users, h, d)


def paged_sdpa_decode_gqa(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    page_table: torch.Tensor,
    cur_pos_tensor: torch.Tensor,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """Causal paged decode for Hq = G * Hkv (query head h reads KV head h // G).

    The reference's own decode branch cannot run with Hq != Hkv (its
    ``query.reshape(B, Hkv, 1, D)`` raises, custom_ops.py:1297).  This follows the
    reference-held equivalent that does run grouped heads: the paged MLA decode CPU
    branch with an explicit value cache, custom_ops.py:551-610 (gather, additive
    -inf mask right of cur_pos, ``F.scaled_dot_product_attention(enable_gqa=True)``).
    """
    bs = key.shape[-2]
    hkv = key.shape[-3]
    d = key.shape[-1]
    users = query.shape[1]
    hq = query.shape[2]
    span = page_table.shape[1] * bs
    idx = page_table.long()
    gk = key[idx].permute(0, 2, 1, 3, 4).reshape(users, hkv, span, d)
    gv = value[idx].permute(0, 2, 1, 3, 4).reshape(users, hkv, span, value.shape[-1])
    q = query.reshape(users, hq, 1, d)
    mask = torch.zeros(users, 1, 1, span, dtype=query.dtype)
    for u in range(users):
        mask[u, :, :, int(cur_pos_tensor[u]) + 1 :] = float("-inf")
    if scale is None:
        scale = 1.0 / d**0.5
    out = F.scaled_dot_product_attention(
        q, gk, gv, mask, is_causal=False, scale=scale, enable_gqa=True
    )
    return out.reshape(1, users, hq, value.shape[-1])


def paged_sdpa_decode(
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
    """Operator-level entry with the reference's argument list
    (custom_ops.py:1203-1223).  ``attention_sink`` and ``sliding_window_size`` are
    accepted and ignored, as on the reference's CPU branch.
    """
    if is_causal:
        assert attn_mask is None, "attention_mask must be None when is_causal is True."
        assert cur_pos_tensor is not None, "cur_pos_tensor must be provided when is_causal is True."
    else:
        return paged_sdpa_decode_masked(query, key, value, page_table, attn_mask, scale)
    if query.shape[2] == key.shape[1]:
        return paged_sdpa_decode_mha(query, key, value, page_table, cur_pos_tensor, scale)
    return paged_sdpa_decode_gqa(query, key, value, page_table, cur_pos_tensor, scale)


def paged_sdpa_decode_masked(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    page_table: torch.Tensor,
    attn_mask: torch.Tensor,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """The decode operator with ``is_causal=False``: every position of the user's table is
    attended, with the caller's additive ``attn_mask`` [B, 1, 1, W*bs] in place of the causal one.

    Hq == Hkv follows the reference's branch op by op (custom_ops.py:1263-1311: the same dense
    gather as the causal form, then ``attn_mask`` where the causal mask would go, :1299-1303, every
    intermediate in the query dtype).  Grouped heads follow the reference-held form that runs
    them, as in ``paged_sdpa_decode_gqa`` (custom_ops.py:551-610 with the caller's mask).
    """
    bs, hkv, d = key.shape[-2], key.shape[-3], key.shape[-1]
    users, hq = query.shape[1], query.shape[2]
    span = page_table.shape[1] * bs
    idx = page_table.long()
    gk = key[idx].permute(0, 2, 1, 3, 4).reshape(users, hkv, span, d)
    gv = value[idx].permute(0, 2, 1, 3, 4).reshape(users, hkv, span, value.shape[-1])
    if scale is None:
        scale = 1 / d**0.5
    if hq == hkv:
        q = query.reshape(users, hkv, 1, d)
        w_ = q @ gk.to(query.dtype).transpose(-2, -1) * scale
        w_ += attn_mask
        w_ = torch.softmax(w_, dim=-1)
        return (w_ @ gv.to(query.dtype)).reshape(1, users, hkv, d)
    out = F.scaled_dot_product_attention(
        query.reshape(users, hq, 1, d), gk, gv, attn_mask.to(query.dtype), is_causal=False, scale=scale,
        enable_gqa=True,
    )
    return out.reshape(1, users, hq, value.shape[-1])


# --------------------------------------------------------------------------- #
# prefill attention
# --------------------------------------------------------------------------- #
def chunked_sdpa(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    page_table: torch.Tensor,
    chunk_start_idx_tensor: torch.Tensor,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """Chunked-prefill attention over the paged cache.

    Follows custom_ops.py:1376-1429.  query [U, Hq, Lc, D]; row i of the chunk sits
    at absolute position chunk_start + i and may see key position j iff
    j <= chunk_start + i.  KV heads are repeated G times along the head dim; mask
    and softmax run in the dtype of the score tensor.
    """
    users, hq, lc, d = query.shape
    hkv = key.shape[1]
    start = int(chunk_start_idx_tensor.reshape(-1)[0].item())
    gk = gather_paged_to_dense(key, page_table)
    gv = gather_paged_to_dense(value, page_table)
    span = gk.shape[2]
    if hkv != hq:
        gk = gk.repeat_interleave(hq // hkv, dim=1)
        gv = gv.repeat_interleave(hq // hkv, dim=1)
    if scale is None:
        scale = 1.0 / d**0.5
    att = torch.matmul(query, gk.transpose(-2, -1)) * scale
    qpos = start + torch.arange(lc).view(lc, 1)
    kpos = torch.arange(span).view(1, span)
    neg = torch.full((), float("-inf"), dtype=att.dtype)
    zero = torch.zeros((), dtype=att.dtype)
    att = att + torch.where(kpos <= qpos, zero, neg).view(1, 1, lc, span)
    att = torch.softmax(att, dim=-1)
    return torch.matmul(att, gv)


def sdpa(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    attn_mask: Optional[torch.Tensor] = None,
    is_causal: bool = True,
    scale: Optional[float] = None,
    sliding_window_size: Optional[int] = None,
) -> torch.Tensor:
    """Dense prefill attention with grouped heads.

    Follows custom_ops.py:648-692 (argument checks) and :717-727 (the CPU branch is
    the library routine with ``enable_gqa=True``; ``sliding_window_size`` ignored).
    """
    assert query.dim() == 4 and key.dim() == 4 and value.dim() == 4
    assert key.shape == value.shape, "key and value must have the same shape."
    assert key.shape[-1] == query.shape[-1], "key and query must have the same head size."
    assert query.shape[1] % key.shape[1] == 0, "num_heads must be divisible by num_kv_heads."
    assert query.shape[2] % 32 == 0, (
        f"query sequence length must be divisible by 32 but got {query.shape[2]}."
    )
    assert query.shape[0] == key.shape[0], "query and key must have the same batch size."
    if attn_mask is not None:
        assert is_causal is False, "is_causal attribute can't be True if attn_mask is available."
        assert query.shape[0] == attn_mask.shape[0]
    return F.scaled_dot_product_attention(
        query, key, value, attn_mask, is_causal=is_causal, scale=scale, enable_gqa=True
    )


# --------------------------------------------------------------------------- #
# independent fp32 forms used by tests to pin the restatements above
# --------------------------------------------------------------------------- #
def textbook_decode_fp32(query, key, value, page_table, cur_pos, scale=None):
    """softmax(q K^T * scale) V in fp32 over exactly the first cur_pos+1 tokens of
    each user, one (user, head) at a time.  No masks, no padding: a plain loop.
    Returns fp32 [1, B, Hq, D]; rows with cur_pos < 0 are NaN.
    """
    _, users, hq, d = query.shape
    hkv, bs = key.shape[1], key.shape[2]
    g = hq // hkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.full((1, users, hq, value.shape[-1]), float("nan"), dtype=torch.float32)
    for u in range(users):
        n = int(cur_pos[u]) + 1
        if n <= 0:
            continue
        n = min(n, page_table.shape[1] * bs)
        pos = torch.arange(n)
        blk = page_table[u, pos // bs].long()
        off = pos % bs
        for h in range(hq):
            k = key[blk, h // g, off, :].float()  # [n, D]
            v = value[blk, h // g, off, :].float()
            s = (k @ query[0, u, h].float()) * scale
            p = torch.softmax(s, dim=0)
            out[0, u, h] = p @ v
    return out


# --------------------------------------------------------------------------- #
# sliding window and attention sink (semantics specified here, see module docstring)
# --------------------------------------------------------------------------- #
def paged_sdpa_decode_windowed(query, key, value, page_table, cur_pos, scale=None,
                               sliding_window=None, attention_sink=None):
    """Decode attention in fp32 over positions max(0, cur_pos - W + 1) .. cur_pos of each
    user, with an optional per-head sink logit in the softmax denominator.

    Argument meaning follows tt::paged_scaled_dot_product_attention_decode
    (custom_ops.py:1198-1214): query [1, B, Hq, D], caches [NB, Hkv, bs, D], page_table
    [B, W], cur_pos [B]; attention_sink [Hq] in the units of the scaled scores.
    Returns fp32 [1, B, Hq, D]; rows with cur_pos < 0 are NaN.
    """
    _, users, hq, d = query.shape
    hkv, bs = key.shape[1], key.shape[2]
    g = hq // hkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.full((1, users, hq, value.shape[-1]), float("nan"), dtype=torch.float32)
    for u in range(users):
        n = int(cur_pos[u]) + 1
        if n <= 0:
            continue
        n = min(n, page_table.shape[1] * bs)
        lo = max(0, n - int(sliding_window)) if sliding_window else 0
        pos = torch.arange(lo, n)
        blk = page_table[u, pos // bs].long()
        off = pos % bs
        for h in range(hq):
            k = key[blk, h // g, off, :].float()
            v = value[blk, h // g, off, :].float()
            s = (k @ query[0, u, h].float()) * scale
            if attention_sink is not None:
                s = torch.cat([s, attention_sink[h].float().reshape(1)])
                p = torch.softmax(s, dim=0)[:-1]
            else:
                p = torch.softmax(s, dim=0)
            out[0, u, h] = p @ v
    return out


def sdpa_windowed(query, key, value, scale=None, sliding_window=None):
    """Causal prefill attention in fp32 where query row i attends keys
    max(0, i - W + 1) .. i.  Argument meaning follows tt::scaled_dot_product_attention
    (custom_ops.py:635-646): query [B, Hq, S, D], key / value [B, Hkv, S, D]."""
    b, hq, sq, d = query.shape
    hkv, skv = key.shape[1], key.shape[2]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    kk = key.float().repeat_interleave(hq // hkv, dim=1)
    vv = value.float().repeat_interleave(hq // hkv, dim=1)
    scores = query.float() @ kk.transpose(-1, -2) * scale
    i = torch.arange(sq).view(sq, 1)
    j = torch.arange(skv).view(1, skv)
    banned = j > i
    if sliding_window:
        banned = banned | (j < i - int(sliding_window) + 1)
    scores = scores.masked_fill(banned, float("-inf"))
    return torch.softmax(scores, dim=-1) @ vv


# --------------------------------------------------------------------------- #
# non-paged (static) caches [B, H, max_seq_len, D]
# --------------------------------------------------------------------------- #
def update_cache(cache, fill_value, cache_position, batch_offset=None):
    """custom_ops.py:857-891: one token, one position shared by the whole batch."""
    assert fill_value.shape[-2] == 1 and cache_position.shape == (1,)
    assert not batch_offset
    out = cache.clone()
    out[:, :, cache_position, :] = fill_value
    return out


def fill_cache(cache, fill_value, batch_offset=None):
    """custom_ops.py:903-940: the first seq_len positions of every (batch, head)."""
    assert fill_value.shape[-2] <= cache.shape[-2]
    assert not batch_offset
    out = cache.clone()
    out[:, :, : fill_value.shape[-2], :] = fill_value
    return out


def sdpa_decode_static(query, key, value, cur_pos_tensor, scale=None, attn_mask=None):
    """custom_ops.py:817-842: with attn_mask=None an additive mask of -inf to the right of each
    user's position; with one (is_causal=False), the mask itself, one row per query head
    ([batch, 1, heads, max_seq] reshaped to [batch, heads, 1, max_seq], custom_ops.py:820-821).
    Then the library SDPA with grouped heads, in the query's dtype."""
    batch, heads, d = query.shape[1], query.shape[2], query.shape[3]
    max_seq = key.shape[-2]
    q = query.reshape(batch, heads, 1, d)
    if attn_mask is not None:
        mask = attn_mask.reshape(batch, heads, 1, max_seq)
    else:
        mask = torch.zeros(batch, heads, 1, max_seq, dtype=q.dtype)
        for b in range(batch):
            mask[b, ..., int(cur_pos_tensor[b]) + 1 :] = float("-inf")
    out = F.scaled_dot_product_attention(q, key, value, mask, is_causal=False, scale=scale, enable_gqa=True)
    return out.reshape(1, batch, heads, d)


# --------------------------------------------------------------------------- #
# latent (MLA) attention
# --------------------------------------------------------------------------- #
def flash_mla_prefill(query, key, head_dim_v, value=None, attn_mask=None, is_causal=True, scale=None):
    """custom_ops.py:343-357: V defaults to the leading head_dim_v features of K."""
    if value is None:
        value = key[..., :head_dim_v]
    return F.scaled_dot_product_attention(query, key, value, attn_mask, is_causal=is_causal,
                                          scale=scale, enable_gqa=True)


def paged_flash_mla_decode(query, key, head_dim_v, page_table, value=None, cur_pos_tensor=None, scale=None,
                           attn_mask=None):
    """custom_ops.py:551-610: gather each user's blocks; additive mask to the right of cur_pos
    (causal form) or attn_mask itself (is_causal=False, custom_ops.py:590-592); library SDPA
    with grouped heads, in the query's dtype."""
    block_size, nkv, dh = key.shape[-2], key.shape[-3], key.shape[-1]
    users, hq = query.shape[1], query.shape[2]
    max_seq = page_table.shape[1] * block_size
    index = page_table.long()
    gk = key[index].permute(0, 2, 1, 3, 4).reshape(users, nkv, max_seq, dh)
    if value is not None:
        gv = value[index].permute(0, 2, 1, 3, 4).reshape(users, nkv, max_seq, value.shape[-1])
    else:
        gv = gk[..., :head_dim_v]
    q = query.reshape(users, hq, 1, dh)
    if attn_mask is not None:
        mask = attn_mask
    else:
        mask = torch.zeros(users, 1, 1, max_seq, dtype=query.dtype)
        for i in range(users):
            mask[i, :, :, int(cur_pos_tensor[i]) + 1 :] = float("-inf")
    scale_val = 1.0 / (dh**0.5) if scale is None else scale
    out = F.scaled_dot_product_attention(q, gk, gv, mask, is_causal=False, scale=scale_val, enable_gqa=True)
    return out.reshape(1, users, hq, head_dim_v)
