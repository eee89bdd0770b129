"""Pins oracle.paged_ops cache writes with brute-force loops that share no code with
them, over the reference's own parameter grids
(tests/torch/ops/test_custom_ops.py:139-203, subsampled so the CPU suite stays small)
and the paged-layout invariants of
tests/integrations/vllm_plugin/oot_backends/test_mla_attention_impl.py:202-218, 317-333, 435-438.
"""

import itertools

import pytest
import torch

from oracle import paged_ops as O


def _inverse_perm_table(gen, users, blocks_per_seq):
    perm = torch.randperm(users * blocks_per_seq, generator=gen)
    return torch.argsort(perm).reshape(users, blocks_per_seq).to(torch.int32)


def _brute_update(cache, fill, idx, table):
    out = cache.clone()
    nb, h, bs, d = cache.shape
    w = table.shape[1]
    for u in range(idx.shape[0]):
        p = int(idx[u])
        col, off = p // bs, p % bs  # python floor semantics
        if col < 0:
            col += w
        blk = int(table[u, col])
        for hh in range(h):
            for dd in range(d):
                out[blk, hh, off, dd] = fill[0, u, hh, dd]
    return out


UPDATE_GRID = [
    # users, blocks/seq, heads, bs, D   (every value of the reference grid appears)
    (8, 16, 1, 32, 128),
    (16, 16, 8, 64, 128),
    (24, 16, 8, 32, 256),
    (32, 16, 1, 128, 128),
    (8, 32, 8, 32, 128),
    (8, 16, 32, 32, 128),
]


@pytest.mark.parametrize("users,bps,heads,bs,d", UPDATE_GRID)
def test_update_matches_brute_force(users, bps, heads, bs, d):
    g = torch.Generator().manual_seed(users * 131 + bps + heads + bs + d)
    cache = torch.zeros(users * bps, heads, bs, d, dtype=torch.bfloat16)
    fill = torch.randn(1, users, heads, d, generator=g).to(torch.bfloat16)
    idx = torch.randperm(bps * bs, generator=g)[:users]
    table = _inverse_perm_table(g, users, bps)
    got = O.paged_update_cache(cache, fill, idx, table)
    # brute force on a thin slice of D keeps the python loop short
    want = _brute_update(cache[..., :4], fill[..., :4], idx, table)
    assert torch.equal(got[..., :4], want)
    # and the closed form on everything: exactly users*heads*D non-zero-able slots
    for u in range(users):
        p = int(idx[u])
        assert torch.equal(got[int(table[u, p // bs]), :, p % bs, :], fill[0, u])
    touched = torch.zeros(users * bps, bs, dtype=torch.bool)
    for u in range(users):
        p = int(idx[u])
        touched[int(table[u, p // bs]), p % bs] = True
    assert torch.equal(got[~touched.unsqueeze(1).expand(-1, heads, -1)], cache[~touched.unsqueeze(1).expand(-1, heads, -1)])
    assert got.data_ptr() != cache.data_ptr() and cache.abs().sum() == 0  # functional


def test_update_int32_and_int64_indices_agree():
    g = torch.Generator().manual_seed(5)
    cache = torch.randn(12, 2, 32, 64, generator=g).to(torch.bfloat16)
    fill = torch.randn(1, 3, 2, 64, generator=g).to(torch.bfloat16)
    table = _inverse_perm_table(g, 3, 4)
    idx = torch.tensor([0, 77, 127])
    a = O.paged_update_cache(cache, fill, idx, table)
    b = O.paged_update_cache(cache, fill, idx.to(torch.int32), table)
    assert torch.equal(a, b)
    assert torch.equal(a, _brute_update(cache, fill, idx, table))


def test_update_padded_row_lands_in_last_column_last_offset():
    """cache_position -1 (padded batch rows, vllm_tt/model_runner.py:1734-1741) is
    floor-divided: column -1 = last column, offset bs-1."""
    g = torch.Generator().manual_seed(6)
    cache = torch.zeros(8, 2, 32, 64, dtype=torch.bfloat16)
    fill = torch.randn(1, 2, 2, 64, generator=g).to(torch.bfloat16)
    table = torch.tensor([[3, 4, 5, 6], [0, 0, 0, 0]], dtype=torch.int32)
    idx = torch.tensor([40, -1], dtype=torch.int32)
    got = O.paged_update_cache(cache, fill, idx, table)
    assert torch.equal(got, _brute_update(cache, fill, idx, table))
    assert torch.equal(got[0, :, 31, :], fill[0, 1])  # null block 0, last row
    assert torch.equal(got[4, :, 8, :], fill[0, 0])


def test_update_ignores_padded_fill_heads():
    g = torch.Generator().manual_seed(7)
    cache = torch.zeros(4, 2, 32, 64, dtype=torch.bfloat16)
    fill = torch.randn(1, 2, 8, 64, generator=g).to(torch.bfloat16)  # 8 > Hkv = 2
    table = torch.tensor([[0, 1], [2, 3]], dtype=torch.int32)
    idx = torch.tensor([33, 2])
    got = O.paged_update_cache(cache, fill, idx, table)
    assert torch.equal(got[1, :, 1, :], fill[0, 0, :2])
    assert torch.equal(got[2, :, 2, :], fill[0, 1, :2])


def _brute_fill(cache, fill, table, b):
    out = cache.clone()
    bs = cache.shape[2]
    for t in range(fill.shape[2]):
        blk = int(table[b, t // bs])
        out[blk, :, t % bs, :] = fill[0, :, t, :]
    return out


FILL_GRID = list(
    itertools.product([8, 16], [16], [1, 8], [32, 64], [128], [10, 20, 32, 50, 70])
) + [(8, 32, 32, 32, 128, 70), (16, 32, 8, 64, 128, 50)]


@pytest.mark.parametrize("users,bps,heads,bs,d,s", FILL_GRID)
def test_fill_matches_brute_force(users, bps, heads, bs, d, s):
    g = torch.Generator().manual_seed(s * 7 + users + heads + bs)
    cache = torch.randn(users * bps, heads, bs, d, generator=g).to(torch.bfloat16)
    fill = torch.randn(1, heads, s, d, generator=g).to(torch.bfloat16)
    table = _inverse_perm_table(g, users, bps)
    b = torch.randint(0, users, (1,), generator=g, dtype=torch.int32)
    got = O.paged_fill_cache(cache, fill, table, b)
    assert torch.equal(got, _brute_fill(cache, fill, table, int(b)))


def test_fill_default_batch_idx_is_zero_and_tail_rows_survive():
    g = torch.Generator().manual_seed(9)
    cache = torch.randn(6, 2, 32, 64, generator=g).to(torch.bfloat16)
    fill = torch.randn(1, 2, 40, 64, generator=g).to(torch.bfloat16)
    table = torch.tensor([[5, 2, 1], [0, 3, 4]], dtype=torch.int32)
    got = O.paged_fill_cache(cache, fill, table)
    assert torch.equal(got[5], fill[0, :, :32])
    assert torch.equal(got[2, :, :8], fill[0, :, 32:])
    assert torch.equal(got[2, :, 8:], cache[2, :, 8:])  # rest of the tail block
    for blk in (0, 1, 3, 4):
        assert torch.equal(got[blk], cache[blk])


def test_fill_batched_is_row_by_row():
    g = torch.Generator().manual_seed(10)
    cache = torch.zeros(12, 2, 32, 64, dtype=torch.bfloat16)
    fill = torch.randn(3, 2, 50, 64, generator=g).to(torch.bfloat16)
    table = _inverse_perm_table(g, 3, 4)
    bidx = torch.tensor([2, 0, 1], dtype=torch.int32)
    got = O.paged_fill_cache_batched(cache, fill, table, bidx)
    want = cache
    for i in range(3):
        want = _brute_fill(want, fill[i : i + 1], table, int(bidx[i]))
    assert torch.equal(got, want)


def test_gather_inverts_fill():
    """position p of user u lives in block page_table[u, p // bs] at row p % bs."""
    g = torch.Generator().manual_seed(11)
    cache = torch.zeros(8, 2, 32, 64, dtype=torch.bfloat16)
    table = _inverse_perm_table(g, 2, 4)
    fills = torch.randn(2, 2, 128, 64, generator=g).to(torch.bfloat16)
    out = O.paged_fill_cache_batched(cache, fills, table, torch.arange(2, dtype=torch.int32))
    assert torch.equal(O.gather_paged_to_dense(out, table), fills)
