"""TTAttentionBackendImpl.forward on the GPU against the same dispatch spelled with the CPU
oracle's operators (composition of the reference's forward, attention.py:273-668): decode
step, first prefill, continuation chunk; in-place and functional cache-op modes agree."""

import pytest
import torch

import __graft_entry__ as entry
from oracle import paged_ops as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def _bf(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


HQ, HKV, D, BS = 32, 8, 128, 32


def _impl(**kw):
    from tt_xla_amd import TTAttentionBackendImpl

    return TTAttentionBackendImpl(HQ, D, D**-0.5, HKV, None, None, "auto", **kw)


def _setup(gen, users, width):
    nb = users * width + 1
    table = (torch.randperm(nb - 1, generator=gen) + 1).view(users, width).to(torch.int32)
    kc, vc = _bf(gen, nb, HKV, BS, D), _bf(gen, nb, HKV, BS, D)
    return table, kc, vc


@pytest.mark.parametrize("functional", [False, True])
def test_decode_step(functional):
    from tt_xla_amd import TTAttentionBackend, TTMetadata

    assert TTAttentionBackend.get_kv_cache_shape(7, BS, HKV, D) == (7, HKV, BS, D)
    assert TTAttentionBackend.get_name() == "CUSTOM"
    g = torch.Generator().manual_seed(1)
    users, width = 5, 6
    table, kc, vc = _setup(g, users, width)
    pos = torch.tensor([0, 31, 32, 100, 191], dtype=torch.int32)
    q, k, v = _bf(g, users, HQ * D), _bf(g, users, HKV * D), _bf(g, users, HKV * D)
    # oracle composition
    k_ref = O.paged_update_cache(kc, k.view(users, 1, HKV, D).transpose(0, 1), pos, table)
    v_ref = O.paged_update_cache(vc, v.view(users, 1, HKV, D).transpose(0, 1), pos, table)
    want = O.paged_sdpa_decode(q.view(users, 1, HQ, D).transpose(0, 1), k_ref, v_ref, table,
                               True, None, pos, None, D**-0.5).transpose(0, 1).reshape(users, HQ * D)
    md = TTMetadata(cache_position=pos.cuda(), page_table=table.cuda(), num_users=users)
    kv = [kc.cuda(), vc.cuda()]
    out = torch.empty(users, HQ * D, dtype=torch.bfloat16, device="cuda")
    _impl(functional_cache_ops=functional).forward(None, q.cuda(), k.cuda(), v.cuda(), kv, md, output=out)
    assert torch.equal(kv[0].cpu(), k_ref) and torch.equal(kv[1].cpu(), v_ref)
    torch.testing.assert_close(out.cpu().float(), want.float(), atol=2e-2, rtol=2e-2)


def test_prefill_then_chunk_then_decode():
    from tt_xla_amd import TTMetadata

    g = torch.Generator().manual_seed(2)
    users, width, s1, s2 = 2, 8, 128, 64
    table, kc, vc = _setup(g, users, width)
    kc.zero_(), vc.zero_()
    kv = [kc.cuda(), vc.cuda()]
    impl = _impl()
    bidx = torch.arange(users, dtype=torch.int32)

    # --- first chunk: fill from column 0, dense causal attention on the fresh K/V ----------
    q1, k1, v1 = _bf(g, users * s1, HQ * D), _bf(g, users * s1, HKV * D), _bf(g, users * s1, HKV * D)
    md = TTMetadata(cache_position=None, page_table=table.cuda(), num_users=users,
                    batch_idx=bidx.cuda())
    out1 = torch.empty(users * s1, HQ * D, dtype=torch.bfloat16, device="cuda")
    impl.forward(None, q1.cuda(), k1.cuda(), v1.cuda(), kv, md, output=out1)
    k4 = k1.view(users, s1, HKV, D).transpose(1, 2)
    v4 = v1.view(users, s1, HKV, D).transpose(1, 2)
    kc_ref = O.paged_fill_cache_batched(kc, k4, table, bidx)
    vc_ref = O.paged_fill_cache_batched(vc, v4, table, bidx)
    assert torch.equal(kv[0].cpu(), kc_ref) and torch.equal(kv[1].cpu(), vc_ref)
    want1 = O.sdpa(q1.view(users, s1, HQ, D).transpose(1, 2), k4, v4, None, True, D**-0.5)
    torch.testing.assert_close(out1.cpu().float(),
                               want1.transpose(1, 2).reshape(users * s1, HQ * D).float(),
                               atol=2e-2, rtol=2e-2)

    # --- continuation chunk: fill table rolled by the computed blocks, chunked attention ----
    q2, k2, v2 = _bf(g, users * s2, HQ * D), _bf(g, users * s2, HKV * D), _bf(g, users * s2, HKV * D)
    fill_table = torch.roll(table, -(s1 // BS), dims=1)
    start = torch.tensor([s1], dtype=torch.int32)
    md = TTMetadata(cache_position=None, page_table=table.cuda(), num_users=users,
                    batch_idx=bidx.cuda(), fill_page_table=fill_table.cuda(),
                    chunk_start_idx=start.cuda())
    out2 = torch.empty(users * s2, HQ * D, dtype=torch.bfloat16, device="cuda")
    impl.forward(None, q2.cuda(), k2.cuda(), v2.cuda(), kv, md, output=out2)
    kc_ref = O.paged_fill_cache_batched(kc_ref, k2.view(users, s2, HKV, D).transpose(1, 2), fill_table, bidx)
    vc_ref = O.paged_fill_cache_batched(vc_ref, v2.view(users, s2, HKV, D).transpose(1, 2), fill_table, bidx)
    assert torch.equal(kv[0].cpu(), kc_ref) and torch.equal(kv[1].cpu(), vc_ref)
    want2 = O.chunked_sdpa(q2.view(users, s2, HQ, D).transpose(1, 2), kc_ref, vc_ref, table, start, D**-0.5)
    torch.testing.assert_close(out2.cpu().float(),
                               want2.transpose(1, 2).reshape(users * s2, HQ * D).float(),
                               atol=2e-2, rtol=2e-2)

    # --- one decode token on top ---------------------------------------------------------------
    pos = torch.full((users,), s1 + s2, dtype=torch.int32)
    q3, k3, v3 = _bf(g, users, HQ * D), _bf(g, users, HKV * D), _bf(g, users, HKV * D)
    md = TTMetadata(cache_position=pos.cuda(), page_table=table.cuda(), num_users=users)
    out3 = torch.empty(users, HQ * D, dtype=torch.bfloat16, device="cuda")
    impl.forward(None, q3.cuda(), k3.cuda(), v3.cuda(), kv, md, output=out3)
    kc_ref = O.paged_update_cache(kc_ref, k3.view(users, 1, HKV, D).transpose(0, 1), pos, table)
    vc_ref = O.paged_update_cache(vc_ref, v3.view(users, 1, HKV, D).transpose(0, 1), pos, table)
    assert torch.equal(kv[0].cpu(), kc_ref)
    want3 = O.paged_sdpa_decode(q3.view(users, 1, HQ, D).transpose(0, 1), kc_ref, vc_ref, table,
                                True, None, pos, None, D**-0.5)
    torch.testing.assert_close(out3.cpu().float(), want3.transpose(0, 1).reshape(users, HQ * D).float(),
                               atol=2e-2, rtol=2e-2)


def test_forward_errors():
    from tt_xla_amd import TTMetadata

    impl = _impl()
    md = TTMetadata(num_users=3)
    q = torch.zeros(4, HQ * D, dtype=torch.bfloat16, device="cuda")
    k = torch.zeros(4, HKV * D, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):  # 4 tokens not divisible by 3 users
        impl.forward(None, q, k, k, None, md, output=torch.empty_like(q))
    with pytest.raises(AssertionError):
        impl.forward(None, q, k, k, None, md, output=None)
    with pytest.raises(ValueError):
        impl.forward(None, q[:, :100], k, k, None, TTMetadata(num_users=4), output=torch.empty_like(q))
    with pytest.raises(NotImplementedError):
        from tt_xla_amd import TTAttentionBackendImpl

        TTAttentionBackendImpl(HQ, D, 1.0, HKV, [0.1], None, "auto")


def test_kv_shared_layer_prefill_reads_the_target_cache():
    """A layer that shares another layer's KV cache (kv_sharing_target_layer_name set) never
    writes the cache (reference attention.py:309-314) and its prefill attends over keys / values
    gathered from it through the page table, block-major then in-block, cut to the pass's token
    count (attention.py:562-574, 600-632)."""
    from tt_xla_amd import TTMetadata

    g = torch.Generator().manual_seed(5)
    users, width, s = 2, 4, 96
    table, kc, vc = _setup(g, users, width)
    kv = [kc.cuda(), vc.cuda()]
    q = _bf(g, users * s, HQ * D)
    k, v = _bf(g, users * s, HKV * D), _bf(g, users * s, HKV * D)  # ignored: the layer owns no K / V
    md = TTMetadata(cache_position=None, page_table=table.cuda(), num_users=users,
                    batch_idx=torch.arange(users, dtype=torch.int32).cuda())
    out = torch.empty(users * s, HQ * D, dtype=torch.bfloat16, device="cuda")
    _impl(kv_sharing_target_layer_name="model.layers.0.self_attn").forward(
        None, q.cuda(), k.cuda(), v.cuda(), kv, md, output=out)
    assert torch.equal(kv[0].cpu(), kc) and torch.equal(kv[1].cpu(), vc), "a KV-shared layer wrote the cache"
    k_dense = O.gather_paged_to_dense(kc, table)[:, :, :s]
    v_dense = O.gather_paged_to_dense(vc, table)[:, :, :s]
    assert k_dense.shape == (users, HKV, s, D)
    # the gather order, spelled out: position p of user u is block table[u, p // BS], row p % BS
    for u, p in ((0, 0), (1, 33), (1, s - 1)):
        assert torch.equal(k_dense[u, :, p], kc[table[u, p // BS], :, p % BS])
    want = O.sdpa(q.view(users, s, HQ, D).transpose(1, 2), k_dense, v_dense, None, True, D**-0.5)
    torch.testing.assert_close(out.cpu().float(), want.transpose(1, 2).reshape(users * s, HQ * D).float(),
                               atol=2e-2, rtol=2e-2)


def test_kv_shared_layer_decode_reads_the_target_cache():
    """The decode pass of a KV-shared layer attends over the target layer's cache as it is: no
    update, not even of the position it is at (attention.py:309-314, 634-668)."""
    from tt_xla_amd import TTMetadata

    g = torch.Generator().manual_seed(6)
    users, width = 3, 5
    table, kc, vc = _setup(g, users, width)
    pos = torch.tensor([7, 64, 159], dtype=torch.int32)
    q, k, v = _bf(g, users, HQ * D), _bf(g, users, HKV * D), _bf(g, users, HKV * D)
    kv = [kc.cuda(), vc.cuda()]
    md = TTMetadata(cache_position=pos.cuda(), page_table=table.cuda(), num_users=users)
    out = torch.empty(users, HQ * D, dtype=torch.bfloat16, device="cuda")
    _impl(kv_sharing_target_layer_name="model.layers.0.self_attn").forward(
        None, q.cuda(), k.cuda(), v.cuda(), kv, md, output=out)
    assert torch.equal(kv[0].cpu(), kc) and torch.equal(kv[1].cpu(), vc)
    want = O.paged_sdpa_decode(q.view(users, 1, HQ, D).transpose(0, 1), kc, vc, table, True, None, pos,
                               None, D**-0.5).transpose(0, 1).reshape(users, HQ * D)
    torch.testing.assert_close(out.cpu().float(), want.float(), atol=2e-2, rtol=2e-2)
