"""Pins the oracle's non-paged forms (reference custom_ops.py:745-950)."""

import torch

from oracle import paged_ops as O


def test_update_cache_element_by_element():
    g = torch.Generator().manual_seed(0)
    cache = torch.randn(3, 4, 16, 8, generator=g)
    fill = torch.randn(3, 4, 1, 8, generator=g)
    for p in (0, 7, 15):
        out = O.update_cache(cache, fill, torch.tensor([p]), 0)
        for b in range(3):
            for h in range(4):
                for t in range(16):
                    want = fill[b, h, 0] if t == p else cache[b, h, t]
                    assert torch.equal(out[b, h, t], want)
    assert torch.equal(cache, cache.clone())  # functional: the input is untouched


def test_fill_cache_element_by_element():
    g = torch.Generator().manual_seed(1)
    cache = torch.randn(2, 3, 12, 4, generator=g)
    for s in (1, 5, 12):
        fill = torch.randn(2, 3, s, 4, generator=g)
        out = O.fill_cache(cache, fill, 0)
        assert torch.equal(out[:, :, :s], fill) and torch.equal(out[:, :, s:], cache[:, :, s:])


def test_static_decode_is_the_paged_decode_on_an_identity_table_and_the_fp32_loop():
    g = torch.Generator().manual_seed(2)
    b, hq, hkv, s, d = 3, 8, 2, 32, 16
    key = torch.randn(b, hkv, s, d, generator=g)
    value = torch.randn(b, hkv, s, d, generator=g)
    q = torch.randn(1, b, hq, d, generator=g)
    pos = torch.tensor([0, 13, 31])
    got = O.sdpa_decode_static(q, key, value, pos)
    table = torch.arange(b, dtype=torch.int32).view(b, 1)
    want = O.textbook_decode_fp32(q, key, value, table, pos)
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
    paged = O.paged_sdpa_decode(q, key, value, table, True, None, pos, None, None)
    torch.testing.assert_close(got, paged.float(), atol=1e-5, rtol=1e-5)


def test_static_decode_with_a_mask_per_head_against_an_fp32_loop():
    """attn_mask [B, 1, heads, S] (reference custom_ops.py:817-842 with is_causal=False): all positions,
    score + the head's mask row; cur_pos plays no part."""
    g = torch.Generator().manual_seed(4)
    b, hq, hkv, s, d = 3, 6, 2, 20, 16
    key, value = torch.randn(b, hkv, s, d, generator=g), torch.randn(b, hkv, s, d, generator=g)
    q = torch.randn(1, b, hq, d, generator=g)
    mask = torch.randn(b, 1, hq, s, generator=g)
    mask[..., 2::5] = float("-inf")
    got = O.sdpa_decode_static(q, key, value, torch.zeros(b, dtype=torch.int32), 0.25, mask)
    other = O.sdpa_decode_static(q, key, value, torch.full((b,), s - 1, dtype=torch.int32), 0.25, mask)
    assert torch.equal(got, other)
    for u in range(b):
        for h in range(hq):
            p = torch.softmax((key[u, h // 3] @ q[0, u, h]) * 0.25 + mask[u, 0, h], dim=0)
            torch.testing.assert_close(got[0, u, h], p @ value[u, h // 3], atol=1e-5, rtol=1e-5)
