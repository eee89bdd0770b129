"""Pins the oracle's sliding-window and attention-sink forms.  The reference's CPU branches
ignore both arguments (custom_ops.py:1256-1312, 717-727), so nothing of the reference can
pin them: PARITY UNPINNED.  What is checked is what the mathematics fixes."""

import math

import torch

from oracle import paged_ops as O


def _setup(seed, users=3, hq=8, hkv=2, d=32, bs=8, width=6):
    g = torch.Generator().manual_seed(seed)
    nb = users * width + 1
    table = (torch.randperm(nb - 1, generator=g) + 1).view(users, width).to(torch.int32)
    k = torch.randn(nb, hkv, bs, d, generator=g)
    v = torch.randn(nb, hkv, bs, d, generator=g)
    q = torch.randn(1, users, hq, d, generator=g)
    return g, q, k, v, table


def test_window_longer_than_context_changes_nothing():
    _, q, k, v, table = _setup(0)
    pos = torch.tensor([5, 20, 47])
    want = O.textbook_decode_fp32(q, k, v, table, pos)
    for w in (48, 100, 10**6):
        got = O.paged_sdpa_decode_windowed(q, k, v, table, pos, sliding_window=w)
        torch.testing.assert_close(got, want, atol=1e-6, rtol=1e-6)


def test_window_equals_attention_over_a_rebased_cache():
    """A window of W at position p must equal full attention of the same query over a cache
    that holds only positions p-W+1 .. p (copied to the front of fresh blocks)."""
    _, q, k, v, table = _setup(1)
    bs = k.shape[2]
    pos = torch.tensor([13, 30, 47])
    w = 11
    k2, v2 = torch.zeros_like(k), torch.zeros_like(v)
    new_pos = []
    for u in range(3):
        lo = max(0, int(pos[u]) + 1 - w)
        src = torch.arange(lo, int(pos[u]) + 1)
        dst = torch.arange(len(src))
        k2[table[u, dst // bs].long(), :, dst % bs] = k[table[u, src // bs].long(), :, src % bs]
        v2[table[u, dst // bs].long(), :, dst % bs] = v[table[u, src // bs].long(), :, src % bs]
        new_pos.append(len(src) - 1)
    want = O.textbook_decode_fp32(q, k2, v2, table, torch.tensor(new_pos))
    got = O.paged_sdpa_decode_windowed(q, k, v, table, pos, sliding_window=w)
    torch.testing.assert_close(got, want, atol=1e-6, rtol=1e-6)


def test_window_of_one_returns_the_current_value_row():
    _, q, k, v, table = _setup(2)
    bs = k.shape[2]
    pos = torch.tensor([0, 9, 31])
    got = O.paged_sdpa_decode_windowed(q, k, v, table, pos, sliding_window=1)
    for u in range(3):
        p = int(pos[u])
        row = v[table[u, p // bs].long(), :, p % bs]  # [hkv, d]
        torch.testing.assert_close(got[0, u], row.repeat_interleave(4, dim=0), atol=1e-6, rtol=1e-6)


def test_sink_closed_form():
    """softmax with one extra value-less logit: out_sink = out * sigmoid(lse - sink)."""
    _, q, k, v, table = _setup(3)
    bs, d = k.shape[2], k.shape[3]
    pos = torch.tensor([7, 19, 40])
    sink = torch.tensor([-3.0, -1.0, 0.0, 0.5, 1.0, 2.0, 4.0, -20.0])
    base = O.textbook_decode_fp32(q, k, v, table, pos)
    got = O.paged_sdpa_decode_windowed(q, k, v, table, pos, attention_sink=sink)
    for u in range(3):
        n = int(pos[u]) + 1
        idx = torch.arange(n)
        for h in range(8):
            kk = k[table[u, idx // bs].long(), h // 4, idx % bs]
            lse = torch.logsumexp((kk @ q[0, u, h]) / math.sqrt(d), dim=0)
            want = base[0, u, h] * torch.sigmoid(lse - sink[h])
            torch.testing.assert_close(got[0, u, h], want, atol=1e-5, rtol=1e-5)


def test_sink_at_minus_infinity_is_no_sink_and_padded_rows_are_nan():
    _, q, k, v, table = _setup(4)
    pos = torch.tensor([7, -1, 40])
    sink = torch.full((8,), float("-inf"))
    got = O.paged_sdpa_decode_windowed(q, k, v, table, pos, attention_sink=sink)
    want = O.textbook_decode_fp32(q, k, v, table, pos)
    torch.testing.assert_close(got[0, [0, 2]], want[0, [0, 2]], atol=1e-6, rtol=1e-6)
    assert torch.isnan(got[0, 1]).all()


def test_prefill_window_rows_agree_with_the_decode_form():
    """Row i of the windowed prefill is a windowed decode at position i."""
    g = torch.Generator().manual_seed(5)
    s, hq, hkv, d, bs = 32, 4, 2, 16, 8
    q = torch.randn(1, hq, s, d, generator=g)
    k = torch.randn(1, hkv, s, d, generator=g)
    v = torch.randn(1, hkv, s, d, generator=g)
    w = 9
    got = O.sdpa_windowed(q, k, v, sliding_window=w)
    # the same K/V laid out as a paged cache with an identity table
    kc = k[0].reshape(hkv, s // bs, bs, d).transpose(0, 1).contiguous()
    vc = v[0].reshape(hkv, s // bs, bs, d).transpose(0, 1).contiguous()
    table = torch.arange(s // bs, dtype=torch.int32).view(1, -1)
    for i in (0, 5, 8, 9, 20, 31):
        dec = O.paged_sdpa_decode_windowed(q[:, :, i].unsqueeze(0), kc, vc, table, torch.tensor([i]),
                                           sliding_window=w)
        torch.testing.assert_close(got[0, :, i], dec[0, 0], atol=1e-5, rtol=1e-5)
    # and no window = the library's causal attention
    full = O.sdpa_windowed(q, k, v)
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
    torch.testing.assert_close(full, want, atol=1e-5, rtol=1e-5)
