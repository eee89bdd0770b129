"""Pins oracle.paged_ops attention restatements.

* chunked op: the reference's own CPU cases (shapes, seeds, tolerances of
  tests/torch/ops/test_chunked_sdpa_op_cpu.py:58-147) against an independent
  boolean-mask SDPA over the gathered prefix, written here from scratch.
* decode (MHA restatement of custom_ops.py:1256-1312): against a plain fp32 loop over
  the first cur_pos+1 tokens.  A dropped scale, a mask off by one or a transposed
  gather each fail it.
* decode (GQA form): against the chunked op with a one-token chunk (both are
  reference-held forms that map query head h to KV head h // G) and the fp32 loop.
* dense op: library routine; checked against a manual fp32 grouped-head softmax.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import paged_ops as O


def _cache(nb, hkv, bs, d, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(nb, hkv, bs, d, generator=g)
    v = torch.randn(nb, hkv, bs, d, generator=g)
    return k.to(dtype), v.to(dtype)


def _independent_chunked(q, key, value, table, start, scale):
    users, hq, lc, d = q.shape
    hkv, bs = key.shape[1], key.shape[2]
    out = torch.empty_like(q)
    for u in range(users):
        n = table.shape[1] * bs
        pos = torch.arange(n)
        blk = table[u, pos // bs].long()
        for h in range(hq):
            k = key[blk, h // (hq // hkv), pos % bs]
            v = value[blk, h // (hq // hkv), pos % bs]
            allowed = pos.view(1, n) <= (start + torch.arange(lc)).view(lc, 1)
            out[u, h] = F.scaled_dot_product_attention(
                q[u, h][None], k[None], v[None], attn_mask=allowed[None], scale=scale
            )[0]
    return out


@pytest.mark.parametrize("hq,hkv", [(8, 8), (8, 2), (32, 8)])
@pytest.mark.parametrize("start", [0, 64, 96])
def test_chunked_reference_cases(hq, hkv, start):
    torch.manual_seed(0)
    d, bs, nbpu, users = 64, 32, 4, 2
    lc = nbpu * bs - start
    key, value = _cache(users * nbpu, hkv, bs, d, seed=1)
    table = torch.arange(users * nbpu, dtype=torch.int32).view(users, nbpu)
    q = torch.randn(users, hq, lc, d)
    scale = 1.0 / d**0.5
    got = O.chunked_sdpa(q, key, value, table, torch.tensor([start], dtype=torch.int32), scale)
    want = _independent_chunked(q, key, value, table, start, scale)
    assert got.shape == q.shape
    torch.testing.assert_close(got, want, atol=1e-4, rtol=1e-4)


def test_chunked_single_token_remainder():
    torch.manual_seed(0)
    users, hq, hkv, d, bs, nbpu = 2, 8, 2, 64, 32, 4
    key, value = _cache(users * nbpu, hkv, bs, d, seed=3)
    table = torch.arange(users * nbpu, dtype=torch.int32).view(users, nbpu)
    q = torch.randn(users, hq, 1, d)
    scale = 1.0 / d**0.5
    got = O.chunked_sdpa(q, key, value, table, torch.tensor([64], dtype=torch.int32), scale)
    want = _independent_chunked(q, key, value, table, 64, scale)
    torch.testing.assert_close(got, want, atol=1e-4, rtol=1e-4)


def test_chunked_start0_is_plain_causal():
    torch.manual_seed(0)
    users, h, d, bs, nbpu = 1, 4, 64, 32, 2
    s = nbpu * bs
    key, value = _cache(users * nbpu, h, bs, d, seed=2)
    table = torch.arange(users * nbpu, dtype=torch.int32).view(users, nbpu)
    q = torch.randn(users, h, s, d)
    scale = 1.0 / d**0.5
    got = O.chunked_sdpa(q, key, value, table, torch.zeros(1, dtype=torch.int32), scale)
    dk = key.permute(1, 0, 2, 3).reshape(1, h, s, d)
    dv = value.permute(1, 0, 2, 3).reshape(1, h, s, d)
    want = F.scaled_dot_product_attention(q, dk, dv, is_causal=True, scale=scale)
    torch.testing.assert_close(got, want, atol=1e-4, rtol=1e-4)


def test_chunked_scrambled_table_and_default_scale():
    g = torch.Generator().manual_seed(4)
    users, hq, hkv, d, bs, nbpu = 2, 8, 2, 64, 32, 3
    key, value = _cache(16, hkv, bs, d, seed=5)
    table = torch.randperm(16, generator=g)[: users * nbpu].view(users, nbpu).to(torch.int32)
    q = torch.randn(users, hq, 32, d, generator=g)
    got = O.chunked_sdpa(q, key, value, table, torch.tensor([64], dtype=torch.int32))
    want = _independent_chunked(q, key, value, table, 64, 1 / math.sqrt(d))
    torch.testing.assert_close(got, want, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("users,h,bs,d,w", [(1, 8, 32, 64, 16), (8, 1, 64, 128, 16), (3, 8, 32, 128, 5)])
def test_decode_mha_matches_fp32_loop(dtype, tol, users, h, bs, d, w):
    g = torch.Generator().manual_seed(users * 100 + h)
    nb = users * w
    key, value = _cache(nb, h, bs, d, seed=20 + users, dtype=dtype)
    table = torch.randperm(nb, generator=g).view(users, w).to(torch.int32)
    q = torch.randn(1, users, h, d, generator=g).to(dtype)
    cur = torch.randint(0, w * bs, (users,), generator=g, dtype=torch.int32)
    cur[0] = w * bs - 1  # a full table
    scale = 0.37 if dtype == torch.float32 else None
    got = O.paged_sdpa_decode(q, key, value, table, True, None, cur, None, scale)
    want = O.textbook_decode_fp32(q, key, value, table, cur, scale)
    assert got.shape == (1, users, h, d) and got.dtype == dtype
    torch.testing.assert_close(got.float(), want, atol=tol, rtol=tol)


def test_decode_reference_op_test_case():
    """tests/torch/ops/test_custom_ops.py:206-231: page table all ones, cur_pos all ones."""
    g = torch.Generator().manual_seed(8)
    users, w, h, bs, d = 8, 16, 8, 32, 128
    key, value = _cache(users * w, h, bs, d, seed=30, dtype=torch.bfloat16)
    q = torch.randn(1, users, h, d, generator=g).to(torch.bfloat16)
    table = torch.ones(users, w, dtype=torch.int32)
    cur = torch.ones(users, dtype=torch.int32)
    got = O.paged_sdpa_decode(q, key, value, table, True, None, cur)
    want = O.textbook_decode_fp32(q, key, value, table, cur)
    torch.testing.assert_close(got.float(), want, atol=2e-2, rtol=2e-2)


def test_decode_padded_row_is_nan():
    key, value = _cache(4, 2, 32, 64, seed=31)
    q = torch.randn(1, 2, 2, 64)
    table = torch.tensor([[1, 2], [0, 0]], dtype=torch.int32)
    cur = torch.tensor([40, -1], dtype=torch.int32)
    got = O.paged_sdpa_decode(q, key, value, table, True, None, cur)
    assert torch.isfinite(got[0, 0]).all() and torch.isnan(got[0, 1]).all()


@pytest.mark.parametrize("hq,hkv", [(8, 2), (32, 8), (12, 4), (8, 1)])
def test_decode_gqa_agrees_with_one_token_chunk_and_fp32_loop(hq, hkv):
    g = torch.Generator().manual_seed(hq)
    users, bs, d, w = 3, 32, 64, 4
    key, value = _cache(users * w, hkv, bs, d, seed=40)
    table = torch.randperm(users * w, generator=g).view(users, w).to(torch.int32)
    q = torch.randn(1, users, hq, d, generator=g)
    pos = 77  # the chunked op shares one position across users
    cur = torch.full((users,), pos, dtype=torch.int32)
    got = O.paged_sdpa_decode(q, key, value, table, True, None, cur)
    via_chunk = O.chunked_sdpa(
        q[0].unsqueeze(2), key, value, table, torch.tensor([pos], dtype=torch.int32)
    )  # [U, Hq, 1, D]
    torch.testing.assert_close(got[0], via_chunk[:, :, 0], atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(got, O.textbook_decode_fp32(q, key, value, table, cur), atol=1e-5, rtol=1e-5)


def test_decode_argument_checks():
    key, value = _cache(2, 1, 32, 64, seed=41)
    q = torch.randn(1, 1, 1, 64)
    table = torch.zeros(1, 2, dtype=torch.int32)
    with pytest.raises(AssertionError):
        O.paged_sdpa_decode(q, key, value, table, True, None, None)
    with pytest.raises(AssertionError):
        O.paged_sdpa_decode(q, key, value, table, True, torch.zeros(1), torch.zeros(1, dtype=torch.int32))


@pytest.mark.parametrize("b,hq,hkv,s,skv,causal", [(1, 12, 12, 32, 32, True), (8, 12, 4, 32, 32, True), (1, 12, 4, 32, 128, False)])
def test_dense_sdpa_grouped_heads(b, hq, hkv, s, skv, causal):
    """Grid rows of tests/torch/ops/test_custom_ops.py:52-95 against a manual softmax."""
    g = torch.Generator().manual_seed(s + skv + hq)
    d = 128
    q = torch.randn(b, hq, s, d, generator=g)
    k = torch.randn(b, hkv, skv, d, generator=g)
    v = torch.randn(b, hkv, skv, d, generator=g)
    mask = None if causal else torch.randn(b, 1, s, skv, generator=g)
    got = O.sdpa(q, k, v, mask, causal, 1.0)
    kk = k.repeat_interleave(hq // hkv, 1)
    vv = v.repeat_interleave(hq // hkv, 1)
    sc = q @ kk.transpose(-1, -2)
    if causal:
        sc = sc.masked_fill(torch.ones(s, skv, dtype=torch.bool).triu(1), float("-inf"))
    else:
        sc = sc + mask
    want = torch.softmax(sc, -1) @ vv
    torch.testing.assert_close(got, want, atol=1e-4, rtol=1e-4)


def test_dense_sdpa_rejects_bad_shapes():
    q = torch.randn(1, 4, 31, 64)
    k = torch.randn(1, 4, 31, 64)
    with pytest.raises(AssertionError):
        O.sdpa(q, k, k)  # q_len % 32
    q = torch.randn(1, 6, 32, 64)
    k = torch.randn(1, 4, 32, 64)
    with pytest.raises(AssertionError):
        O.sdpa(q, k, k)  # heads not divisible
    with pytest.raises(AssertionError):
        O.sdpa(torch.randn(1, 4, 32, 64), k, k, attn_mask=torch.zeros(1, 1, 32, 32), is_causal=True)


@pytest.mark.parametrize("hq,hkv", [(8, 8), (8, 2)])
def test_decode_masked_form(hq, hkv):
    """is_causal=False with a caller mask (reference custom_ops.py:1299-1303).  With the causal
    mask handed in it is the causal operator; with a random mask of 0 / -inf / finite biases it is
    softmax(q K^T scale + mask) V over ALL positions of the table, computed here by a plain loop."""
    g = torch.Generator().manual_seed(hq + hkv)
    users, bs, d, w = 3, 32, 64, 4
    span = w * bs
    key, value = _cache(users * w, hkv, bs, d, seed=50)
    table = torch.randperm(users * w, generator=g).view(users, w).to(torch.int32)
    q = torch.randn(1, users, hq, d, generator=g)
    cur = torch.tensor([0, 77, span - 1], dtype=torch.int32)
    causal_mask = torch.zeros(users, 1, 1, span)
    for u in range(users):
        causal_mask[u, :, :, int(cur[u]) + 1:] = float("-inf")
    torch.testing.assert_close(O.paged_sdpa_decode(q, key, value, table, False, causal_mask, cur),
                               O.paged_sdpa_decode(q, key, value, table, True, None, cur), atol=1e-6, rtol=1e-6)
    mask = torch.randn(users, 1, 1, span, generator=g)
    mask[torch.rand(users, 1, 1, span, generator=g) < 0.3] = float("-inf")
    mask[:, :, :, 5] = 0.0  # no row is masked out entirely
    got = O.paged_sdpa_decode(q, key, value, table, False, mask, cur, None, 0.21)
    grp = hq // hkv
    for u in range(users):
        pos = torch.arange(span)
        blk, off = table[u, pos // bs].long(), pos % bs
        for h in range(hq):
            k, v = key[blk, h // grp, off], value[blk, h // grp, off]
            p = torch.softmax((k @ q[0, u, h]) * 0.21 + mask[u, 0, 0], dim=0)
            torch.testing.assert_close(got[0, u, h], p @ v, atol=1e-5, rtol=1e-5)
