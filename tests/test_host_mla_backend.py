"""Host logic of the latent-attention backend (tt_xla_amd/attention_mla.py) on the CPU: query
absorption, latent concatenation, prefill / decode dispatch, cache writes through the fill page
table and at cache_position, output expansion and layout.  The operators are substituted by
the CPU oracle, so what is checked is the plumbing around them, the way the reference's
tests/integrations/vllm_plugin/oot_backends/test_mla_attention_impl.py checks its impl: output
against an independent dense computation, and the cache position by position ("position p of
user u lives in block page_table[u, p // BS] at offset p % BS", new token at cur_pos, prior
context untouched, untouched blocks stay zero)."""

import math
import types

import pytest
import torch

from oracle import paged_ops as O


@pytest.fixture()
def mla(monkeypatch):
    import __graft_entry__  # noqa: F401  (puts the package on sys.path)
    from tt_xla_amd import attention_mla as M

    def fill_inplace(cache, fill, table, batch_idx):
        cache.copy_(O.paged_fill_cache_batched(cache, fill, table, batch_idx))

    def update_inplace(cache, fresh, idx, table):
        cache.copy_(O.paged_update_cache(cache, fresh, idx, table))

    calls = []

    def record(name, fn):
        def wrapped(*a, **k):
            calls.append(name)
            return fn(*a, **k)
        return wrapped

    stub = types.SimpleNamespace(
        flash_mla_prefill=record("flash_mla_prefill", O.flash_mla_prefill),
        paged_flash_mla_decode=record(
            "paged_flash_mla_decode",
            lambda query, key, head_dim_v, page_table, value=None, is_causal=True, attn_mask=None,
            cur_pos_tensor=None, attention_sink=None, scale=None: O.paged_flash_mla_decode(
                query, key, head_dim_v, page_table, value, cur_pos_tensor, scale)),
        paged_fill_cache=record("paged_fill_cache", O.paged_fill_cache),
        paged_fill_cache_=record("paged_fill_cache_", fill_inplace),
        paged_update_cache=record("paged_update_cache", O.paged_update_cache),
        paged_update_cache_=record("paged_update_cache_", update_inplace),
    )
    monkeypatch.setattr(M, "_ops", stub)
    M.calls = calls
    return M


N, P, R, L, V, BS = 4, 16, 8, 32, 24, 32


def _layer(gen):
    return types.SimpleNamespace(W_UK_T=torch.randn(N, P, L, generator=gen) / math.sqrt(P),
                                 W_UV=torch.randn(N, L, V, generator=gen) / math.sqrt(L))


def _impl(M, **kw):
    return M.TTMLAAttentionBackendImpl(
        num_heads=N, head_size=L + R, scale=1.0 / math.sqrt(P + R), num_kv_heads=1,
        alibi_slopes=None, sliding_window=None, kv_cache_dtype="auto", logits_soft_cap=None,
        attn_type="decoder", kv_sharing_target_layer_name=None, kv_lora_rank=L,
        qk_nope_head_dim=P, qk_rope_head_dim=R, qk_head_dim=P + R, v_head_dim=V, **kw)


def _dense_reference(q_nope, q_pe, k_lat_ctx, layer, scale, positions):
    """softmax(q_lat . k_lat^T * scale) over the keys 0..position of each query, values = leading L
    features of the latent keys, expanded by W_UV.  q_*: [users, S, N, .]; k_lat_ctx:
    [users, T, L + R]; positions [users, S]."""
    users, s = q_nope.shape[:2]
    q_lat = torch.cat([torch.einsum("bsnp,npl->bsnl", q_nope, layer.W_UK_T), q_pe], dim=-1)
    out = torch.zeros(users, s, N, V)
    for u in range(users):
        for i in range(s):
            keys = k_lat_ctx[u, : int(positions[u, i]) + 1]              # [T', L+R]
            w = torch.softmax(q_lat[u, i] @ keys.T * scale, dim=-1)      # [N, T']
            out[u, i] = torch.einsum("nl,nlv->nv", w @ keys[:, :L], layer.W_UV)
    return out.reshape(users * s, N * V)


def _gather(cache, table, u, p):
    return cache[table[u, p // BS], 0, p % BS]


@pytest.mark.parametrize("functional", [False, True])
def test_prefill_then_decode(mla, functional):
    from tt_xla_amd.attention import TTMetadata

    gen = torch.Generator().manual_seed(0)
    users, s, nb, w = 3, 40, 16, 3
    layer, impl = _layer(gen), _impl(mla, functional_cache_ops=functional)
    table = (torch.randperm(nb - 1, generator=gen)[: users * w] + 1).view(users, w).to(torch.int32)
    cache = torch.zeros(nb, 1, BS, L + R)

    # ---- prefill: 40 tokens per user ------------------------------------------------------
    q_nope, q_pe = torch.randn(users * s, N, P, generator=gen), torch.randn(users * s, N, R, generator=gen)
    kv_c, k_pe = torch.randn(users * s, L, generator=gen), torch.randn(users * s, 1, R, generator=gen)
    meta = TTMetadata(cache_position=torch.full((users,), s - 1, dtype=torch.int32), page_table=table,
                      fill_page_table=table, attn_mask=None, is_causal=True)
    out = torch.empty(users * s, N * V)
    impl.forward((q_nope, q_pe), kv_c, k_pe, cache, meta, layer, output=out)
    assert "flash_mla_prefill" in mla.calls and "paged_flash_mla_decode" not in mla.calls
    assert ("paged_fill_cache" in mla.calls) == functional and ("paged_fill_cache_" in mla.calls) != functional

    k_lat = torch.cat([kv_c.view(users, s, L), k_pe.view(users, s, R)], dim=-1)
    pos = torch.arange(s).expand(users, s)
    want = _dense_reference(q_nope.view(users, s, N, P), q_pe.view(users, s, N, R), k_lat, layer,
                            impl.scale, pos)
    torch.testing.assert_close(out, want, atol=2e-4, rtol=2e-4)
    for u in range(users):
        for p in range(s):
            assert torch.equal(_gather(cache, table, u, p), k_lat[u, p])
    used = set(table[:, : (s + BS - 1) // BS].flatten().tolist())
    for blk in range(nb):
        if blk not in used:
            assert not cache[blk].any(), f"block {blk} was written"

    # ---- decode: one more token per user ---------------------------------------------------
    mla.calls.clear()
    before = cache.clone()
    q_nope1, q_pe1 = torch.randn(users, N, P, generator=gen), torch.randn(users, N, R, generator=gen)
    kv_c1, k_pe1 = torch.randn(users, L, generator=gen), torch.randn(users, 1, R, generator=gen)
    meta1 = TTMetadata(cache_position=torch.full((users,), s, dtype=torch.int32), page_table=table,
                       attn_mask=None, is_causal=True)
    out1 = torch.empty(users, N * V)
    impl.forward((q_nope1, q_pe1), kv_c1, k_pe1, cache, meta1, layer, output=out1)
    assert "paged_flash_mla_decode" in mla.calls and "flash_mla_prefill" not in mla.calls
    k_new = torch.cat([kv_c1, k_pe1.view(users, R)], dim=-1)
    ctx = torch.cat([k_lat, k_new.view(users, 1, L + R)], dim=1)
    want1 = _dense_reference(q_nope1.view(users, 1, N, P), q_pe1.view(users, 1, N, R), ctx, layer,
                             impl.scale, torch.full((users, 1), s))
    torch.testing.assert_close(out1, want1, atol=2e-4, rtol=2e-4)
    for u in range(users):
        assert torch.equal(_gather(cache, table, u, s), k_new[u])          # new token at cur_pos
        for p in range(s):
            assert torch.equal(_gather(cache, table, u, p), _gather(before, table, u, p))


def test_profiling_run_without_metadata_or_cache(mla):
    """No metadata: treated as prefill of one user, nothing is written (reference :283-297, :337-342)."""
    gen = torch.Generator().manual_seed(1)
    layer, impl = _layer(gen), _impl(mla)
    s = 8
    out = torch.empty(s, N * V)
    impl.forward((torch.randn(s, N, P, generator=gen), torch.randn(s, N, R, generator=gen)),
                 torch.randn(s, L, generator=gen), torch.randn(s, 1, R, generator=gen),
                 torch.tensor([]), None, layer, output=out)
    assert mla.calls == ["flash_mla_prefill"]
    assert torch.isfinite(out).all()


def test_constructor_refusals_and_backend_descriptor(mla):
    with pytest.raises(NotImplementedError):
        _impl(mla).__class__(N, L + R, 1.0, 1, [0.1], None, "auto", None, "decoder", None)
    with pytest.raises(NotImplementedError):
        mla.TTMLAAttentionBackendImpl(N, L + R, 1.0, 1, None, None, "fp8", None, "decoder", None)
    impl = _impl(mla)
    with pytest.raises(RuntimeError):
        impl.forward_mha()
    with pytest.raises(RuntimeError):
        impl.forward_mqa()
    with pytest.raises(AssertionError):
        impl.forward((torch.zeros(2, N, P), torch.zeros(2, N, R)), torch.zeros(2, L),
                     torch.zeros(2, 1, R), torch.tensor([]), None, None, output=None)
    B = mla.TTMLAAttentionBackend
    assert B.get_name() == "FLASH_ATTN_MLA" and B.get_impl_cls() is mla.TTMLAAttentionBackendImpl
    assert B.get_kv_cache_shape(10, 32, 1, 576) == (10, 1, 32, 576)
    with pytest.raises(AssertionError):
        B.get_kv_cache_shape(10, 32, 2, 576)
    assert B.get_page_size(None) == 32
    with pytest.raises(RuntimeError):
        B.swap_blocks(None, None, None)
