"""Pins the oracle's latent-attention forms (reference custom_ops.py:343-357, 551-610)."""

import math

import torch

from oracle import paged_ops as O


def _loop_decode(q, key, value, table, pos, dv, scale):
    """fp32, one (user, head) at a time, separate QK / V widths."""
    _, users, hq, dh = q.shape
    nkv, bs = key.shape[1], key.shape[2]
    g = hq // nkv
    out = torch.zeros(1, users, hq, dv)
    for u in range(users):
        idx = torch.arange(int(pos[u]) + 1)
        blk, off = table[u, idx // bs].long(), idx % bs
        for h in range(hq):
            k = key[blk, h // g, off].float()
            v = (value[blk, h // g, off] if value is not None else key[blk, h // g, off][:, :dv]).float()
            p = torch.softmax((k @ q[0, u, h].float()) * scale, dim=0)
            out[0, u, h] = p @ v
    return out


def test_paged_mla_decode_against_the_loop_and_the_grouped_oracle():
    g = torch.Generator().manual_seed(0)
    users, hq, nkv, dh, dv, bs, width = 3, 8, 2, 48, 32, 8, 5
    nb = users * width
    table = torch.randperm(nb, generator=g).view(users, width).to(torch.int32)
    key = torch.randn(nb, nkv, bs, dh, generator=g)
    value = torch.randn(nb, nkv, bs, dv, generator=g)
    q = torch.randn(1, users, hq, dh, generator=g)
    pos = torch.tensor([0, 17, 39])
    scale = 1 / math.sqrt(dh)
    latent = O.paged_flash_mla_decode(q, key, dv, table, None, pos)
    torch.testing.assert_close(latent, _loop_decode(q, key, None, table, pos, dv, scale), atol=1e-5, rtol=1e-5)
    explicit = O.paged_flash_mla_decode(q, key, dv, table, value, pos)
    torch.testing.assert_close(explicit, _loop_decode(q, key, value, table, pos, dv, scale), atol=1e-5, rtol=1e-5)
    # V given explicitly as the leading slice of K is the latent form
    sliced = O.paged_flash_mla_decode(q, key, dv, table, key[..., :dv].contiguous(), pos)
    torch.testing.assert_close(sliced, latent, atol=1e-6, rtol=1e-6)
    # equal widths: the grouped-head decode oracle
    same = O.paged_flash_mla_decode(q, key, dh, table, torch.randn(nb, nkv, bs, dh, generator=g), pos)
    assert same.shape == (1, users, hq, dh)


def test_mla_prefill_rows_are_decodes_and_equal_widths_are_plain_attention():
    g = torch.Generator().manual_seed(1)
    b, hq, nkv, s, dh, dv = 2, 4, 1, 32, 24, 16
    q = torch.randn(b, hq, s, dh, generator=g)
    k = torch.randn(b, nkv, s, dh, generator=g)
    got = O.flash_mla_prefill(q, k, dv, scale=0.3)
    table = torch.zeros(1, 1, dtype=torch.int32)
    for bi in range(b):
        for i in (0, 7, 31):
            dec = _loop_decode(q[bi, :, i].reshape(1, 1, hq, dh), k[bi : bi + 1], None, table,
                               torch.tensor([i]), dv, 0.3)
            torch.testing.assert_close(got[bi, :, i], dec[0, 0], atol=1e-5, rtol=1e-5)
    full = O.flash_mla_prefill(q, k, dh)
    want = torch.nn.functional.scaled_dot_product_attention(q, k, k, is_causal=True, enable_gqa=True)
    torch.testing.assert_close(full, want, atol=1e-6, rtol=1e-6)


def test_masked_forms_against_an_fp32_loop():
    """attn_mask in place of the causal rule (reference custom_ops.py:343-357, 590-592): every key,
    score + mask, one (row, head) at a time; a mask row for all heads and one per head."""
    g = torch.Generator().manual_seed(2)
    users, hq, nkv, dh, dv, bs, width = 3, 6, 2, 40, 24, 8, 4
    nb, span, grp = users * width, width * bs, hq // nkv
    table = torch.randperm(nb, generator=g).view(users, width).to(torch.int32)
    key = torch.randn(nb, nkv, bs, dh, generator=g)
    q = torch.randn(1, users, hq, dh, generator=g)
    for heads in (1, hq):
        mask = torch.randn(users, heads, 1, span, generator=g)
        mask[:, :, :, 5::3] = float("-inf")
        got = O.paged_flash_mla_decode(q, key, dv, table, None, None, 0.2, mask)
        idx = torch.arange(span)
        for u in range(users):
            blk, off = table[u, idx // bs].long(), idx % bs
            for h in range(hq):
                k = key[blk, h // grp, off]
                p = torch.softmax((k @ q[0, u, h]) * 0.2 + mask[u, h % heads, 0], dim=0)
                torch.testing.assert_close(got[0, u, h], p @ k[:, :dv], atol=1e-5, rtol=1e-5)
    b, s = 2, 16
    qp = torch.randn(b, hq, s, dh, generator=g)
    kp = torch.randn(b, nkv, s, dh, generator=g)
    vp = torch.randn(b, nkv, s, dv, generator=g)
    for heads in (1, hq):
        mask = torch.randn(b, heads, s, s, generator=g)
        mask[..., 3::4] = float("-inf")
        got = O.flash_mla_prefill(qp, kp, dv, vp, mask, False, 0.3)
        for bi in range(b):
            for h in range(hq):
                for i in (0, 5, s - 1):
                    p = torch.softmax((kp[bi, h // grp] @ qp[bi, h, i]) * 0.3 + mask[bi, h % heads, i], dim=0)
                    torch.testing.assert_close(got[bi, h, i], p @ vp[bi, h // grp], atol=1e-5, rtol=1e-5)
