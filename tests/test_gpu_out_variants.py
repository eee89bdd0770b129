"""GPU tests of the operators that write into a caller's buffer
(tt::scaled_dot_product_attention_out, tt::chunked_scaled_dot_product_attention_out,
tt::paged_update_kv_decode_out_): bit-identical to the operator they stand for, on the
token-major strided view the attention backend hands in; the buffer around the view stays
untouched; unusable buffers are refused; the backend falls back to the copy when its output
buffer cannot be viewed."""

import pytest
import torch

import __graft_entry__ as entry

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def _bf(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16).cuda()


@pytest.mark.parametrize("b,hq,hkv,s,d,window", [(2, 8, 2, 96, 128, 0), (1, 4, 4, 64, 64, 20), (2, 8, 4, 32, 256, 0)])
def test_dense_prefill_into_a_token_major_buffer(b, hq, hkv, s, d, window):
    print(f"prefill out-variant b{b} h{hq}x{hkv} s{s} d{d} window{window}", flush=True)
    g = torch.Generator().manual_seed(b + hq + s + d)
    q, k, v = _bf(g, b, hq, s, d), _bf(g, b, hkv, s, d), _bf(g, b, hkv, s, d)
    kw = dict(is_causal=True, sliding_window_size=window if window else None)
    want = torch.ops.tt.scaled_dot_product_attention(q, k, v, **kw)
    # the backend's buffer: [tokens, heads * head_size] with a guard row on either side
    buf = torch.full((b * s + 2, hq * d), 7.0, dtype=torch.bfloat16, device="cuda")
    view = buf[1:-1].view(b, s, hq, d).transpose(1, 2)
    torch.ops.tt.scaled_dot_product_attention_out(q, k, v, view, **kw)
    torch.cuda.synchronize()
    assert torch.equal(view, want)
    assert (buf[0] == 7).all() and (buf[-1] == 7).all()


def test_chunked_prefill_into_a_token_major_buffer():
    g = torch.Generator().manual_seed(5)
    users, hq, hkv, d, bs, nbpu, start, lc = 2, 8, 2, 128, 32, 8, 64, 96
    nb = users * nbpu + 1
    key, value = _bf(g, nb, hkv, bs, d), _bf(g, nb, hkv, bs, d)
    table = (torch.randperm(nb - 1, generator=g)[: users * nbpu] + 1).view(users, nbpu).to(torch.int32).cuda()
    q = _bf(g, users, hq, lc, d)
    st = torch.tensor([start], dtype=torch.int32, device="cuda")
    want = torch.ops.tt.chunked_scaled_dot_product_attention(q, key, value, table, st)
    buf = torch.zeros(users, lc, hq, d, dtype=torch.bfloat16, device="cuda")
    torch.ops.tt.chunked_scaled_dot_product_attention_out(q, key, value, table, st, buf.transpose(1, 2))
    torch.cuda.synchronize()
    assert torch.equal(buf.transpose(1, 2), want)


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 8, 128), (16, 8, 256)])
def test_fused_step_into_a_buffer(hq, hkv, d):
    from tt_xla_amd import workloads

    users, bs = 4, 32
    ctx = [5, 64, 200, 300]
    nb = sum((c + 1 + bs - 1) // bs for c in ctx) + 3
    wl = workloads.decode_ragged("step-out", 17, users, hq, hkv, d, bs, nb, ctx).to("cuda")
    k1, v1, k2, v2 = wl.k_cache.clone(), wl.v_cache.clone(), wl.k_cache.clone(), wl.v_cache.clone()
    want = torch.ops.tt.paged_update_kv_decode_(wl.q, k1, v1, wl.k_new, wl.v_new, wl.page_table,
                                                wl.cache_position, scale=wl.scale)
    buf = torch.zeros(users, hq * d, dtype=torch.bfloat16, device="cuda")
    torch.ops.tt.paged_update_kv_decode_out_(wl.q, k2, v2, wl.k_new, wl.v_new, wl.page_table,
                                             wl.cache_position, buf.view(users, 1, hq, d).transpose(0, 1),
                                             scale=wl.scale)
    torch.cuda.synchronize()
    assert torch.equal(buf.view(1, users, hq, d), want)
    assert torch.equal(k1, k2) and torch.equal(v1, v2)


def test_unusable_output_buffers_are_refused():
    g = torch.Generator().manual_seed(1)
    q, k, v = _bf(g, 1, 4, 32, 64), _bf(g, 1, 4, 32, 64), _bf(g, 1, 4, 32, 64)
    with pytest.raises(ValueError):  # wrong shape
        torch.ops.tt.scaled_dot_product_attention_out(q, k, v, torch.empty_like(q)[:, :2])
    with pytest.raises(ValueError):  # wrong dtype
        torch.ops.tt.scaled_dot_product_attention_out(q, k, v, torch.empty_like(q, dtype=torch.float16))
    with pytest.raises(ValueError):  # head_size not the contiguous dimension
        torch.ops.tt.scaled_dot_product_attention_out(
            q, k, v, torch.empty(1, 4, 64, 32, dtype=torch.bfloat16, device="cuda").transpose(2, 3))


def test_backend_falls_back_to_the_copy_for_a_strided_output_buffer():
    """A prefill pass and a decode pass of the backend with an output buffer that is a column
    slice of a wider tensor (not viewable as [users, tokens, heads, head_size]): same values as
    with a plain buffer."""
    from tt_xla_amd import workloads
    from tt_xla_amd.attention import TTAttentionBackendImpl, TTMetadata

    users, hq, hkv, d, bs = 4, 32, 8, 128, 64
    wl = workloads.decode_ragged("backend-out", 31, users, hq, hkv, d, bs, 24, [5, 64, 200, 300]).to("cuda")
    meta = TTMetadata(cache_position=wl.cache_position, page_table=wl.page_table, is_causal=True, num_users=users)
    q, k, v = wl.q[0].reshape(users, hq * d), wl.k_new[0].reshape(users, hkv * d), wl.v_new[0].reshape(users, hkv * d)
    impl = TTAttentionBackendImpl(hq, d, wl.scale, hkv)
    plain = torch.empty(users, hq * d, dtype=torch.bfloat16, device="cuda")
    wide = torch.zeros(users, hq * d + 64, dtype=torch.bfloat16, device="cuda")
    impl.forward(None, q, k, v, [wl.k_cache.clone(), wl.v_cache.clone()], meta, output=plain)
    impl.forward(None, q, k, v, [wl.k_cache.clone(), wl.v_cache.clone()], meta, output=wide[:, : hq * d])
    torch.cuda.synchronize()
    assert torch.equal(wide[:, : hq * d], plain)
    assert (wide[:, hq * d:] == 0).all()


@pytest.mark.parametrize("b,hq,hkv,s,d,bs,window", [
    (4, 32, 8, 256, 128, 64, 0),      # Llama-3-8B heads
    (3, 8, 4, 96, 128, 32, 0),        # two heads per wavefront group, 96 tokens (not a multiple of a tile)
    (2, 4, 4, 320, 64, 16, 50),       # one head per group, sliding window, more rows than one fill chunk
    (2, 16, 8, 64, 256, 32, 0),       # head size 256
    (1, 8, 2, 32, 128, 64, 0),        # single user without batch_idx
])
def test_prefill_pass_as_one_operator(b, hq, hkv, s, d, bs, window):
    """tt::paged_fill_kv_prefill_out_ against fill K + fill V + dense attention: caches and
    output bit for bit; table rows permuted through batch_idx, one fill row pointed outside the
    table and one block id outside the cache (both skipped by the fill)."""
    print(f"prefill pass b{b} h{hq}x{hkv} s{s} d{d} bs{bs} window{window}", flush=True)
    g = torch.Generator().manual_seed(b * 7 + hq + s + d + bs)
    q, k, v = _bf(g, b, hq, s, d), _bf(g, b, hkv, s, d), _bf(g, b, hkv, s, d)
    w = (s + bs - 1) // bs + 1
    rows = b + 2
    nb = rows * w + 1
    table = (torch.randperm(nb - 1, generator=g)[: rows * w] + 1).view(rows, w).to(torch.int32)
    if b > 1:
        table[1, 0] = nb + 5             # a block id outside the cache
    bidx = None
    if b > 1:
        bidx = torch.randperm(rows, generator=g)[:b].to(torch.int32)
        if b > 2:
            bidx[2] = rows + 3           # a fill row outside the table
        bidx = bidx.cuda()
    table = table.cuda()
    kc = torch.full((nb, hkv, bs, d), 3.0, dtype=torch.bfloat16, device="cuda")
    vc = torch.full((nb, hkv, bs, d), -3.0, dtype=torch.bfloat16, device="cuda")
    kw = dict(is_causal=True, sliding_window_size=window if window else None)

    k_ref, v_ref = kc.clone(), vc.clone()
    torch.ops.tt.paged_fill_cache_(k_ref, k, table, bidx)
    torch.ops.tt.paged_fill_cache_(v_ref, v, table, bidx)
    want = torch.ops.tt.scaled_dot_product_attention(q, k, v, **kw)

    buf = torch.zeros(b, s, hq, d, dtype=torch.bfloat16, device="cuda")
    # token-major operands, as the backend hands them in
    qt, kt, vt = (x.transpose(1, 2).contiguous().transpose(1, 2) for x in (q, k, v))
    torch.ops.tt.paged_fill_kv_prefill_out_(qt, kt, vt, kc, vc, table, bidx, buf.transpose(1, 2), **kw)
    torch.cuda.synchronize()
    assert torch.equal(kc, k_ref), "K cache differs"
    assert torch.equal(vc, v_ref), "V cache differs"
    assert not torch.equal(kc, torch.full_like(kc, 3.0))
    assert torch.equal(buf.transpose(1, 2), want)


def test_backend_prefill_pass_equals_the_reference_sequence():
    """TTAttentionBackendImpl.forward on a first-chunk prefill: the one-operator pass (default)
    and the reference's sequence (functional_cache_ops=True) leave the same caches and output."""
    from tt_xla_amd.attention import TTAttentionBackendImpl, TTMetadata

    users, s, hq, hkv, d, bs = 3, 128, 32, 8, 128, 32
    g = torch.Generator().manual_seed(11)
    w = s // bs
    nb = users * w + 1
    table = (torch.randperm(nb - 1, generator=g)[: users * w] + 1).view(users, w).to(torch.int32).cuda()
    q = _bf(g, users * s, hq * d)
    k, v = _bf(g, users * s, hkv * d), _bf(g, users * s, hkv * d)
    meta = TTMetadata(cache_position=None, page_table=table, num_users=users,
                      batch_idx=torch.arange(users, dtype=torch.int32, device="cuda"),
                      fill_page_table=table, chunk_start_idx=None)
    results = []
    for functional in (False, True):
        impl = TTAttentionBackendImpl(hq, d, d**-0.5, hkv, functional_cache_ops=functional)
        caches = [torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16, device="cuda") for _ in range(2)]
        out = torch.empty(users * s, hq * d, dtype=torch.bfloat16, device="cuda")
        impl.forward(None, q, k, v, caches, meta, output=out)
        results.append((out, caches))
    torch.cuda.synchronize()
    (o1, c1), (o2, c2) = results
    assert torch.equal(c1[0], c2[0]) and torch.equal(c1[1], c2[1])
    assert c1[0].abs().sum() > 0
    assert torch.equal(o1, o2)
