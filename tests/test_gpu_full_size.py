"""The benchmark configurations at full size on the GPU.  Where the CPU oracle would take
minutes, correctness is checked through properties that do not depend on size (linearity of the
output in V, invariance under a permutation of users, agreement of the dense and the paged
route) plus oracle spot checks on a few rows.  Tolerance atol = rtol = 2e-2 against the oracle."""

import pytest
import torch

import __graft_entry__ as entry
from oracle import paged_ops as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def test_config3_prefill_full_size():
    """4 x 2048 causal prefill, 32 / 8 heads: fill the paged cache, then the dense operator
    on the fresh K/V and the paged operator with chunk_start = 0 must agree; batch 0 is
    checked against the oracle; the output is linear in V."""
    from tt_xla_amd import workloads

    w = workloads.prefill_config3(device="cuda").to("cuda")
    u, s, hq, hkv, d = w.users, w.seq, w.q_heads, w.kv_heads, w.head_size
    q = w.q.view(u, s, hq, d).transpose(1, 2)
    k = w.k.view(u, s, hkv, d).transpose(1, 2)
    v = w.v.view(u, s, hkv, d).transpose(1, 2)
    kc, vc = w.k_cache.clone(), w.v_cache.clone()
    torch.ops.tt.paged_fill_cache_(kc, k, w.fill_page_table, w.batch_idx)
    torch.ops.tt.paged_fill_cache_(vc, v, w.fill_page_table, w.batch_idx)
    dense = torch.ops.tt.scaled_dot_product_attention(q, k, v, is_causal=True)
    start = torch.zeros(1, dtype=torch.int32, device="cuda")
    # the paged route attends the whole table: give it exactly the 32 blocks of each prompt
    paged = torch.ops.tt.chunked_scaled_dot_product_attention(q, kc, vc, w.page_table[:, : s // 64].contiguous(), start)
    torch.testing.assert_close(paged.float(), dense.float(), atol=4e-3, rtol=4e-3)
    want = O.sdpa(q[:1].cpu(), k[:1].cpu(), v[:1].cpu(), None, True, None)
    err = (dense[:1].cpu().float() - want.float()).abs().max().item()
    print(f"{w.name}: max-abs error vs oracle (batch 0) {err:.3e}", flush=True)
    torch.testing.assert_close(dense[:1].cpu().float(), want.float(), atol=2e-2, rtol=2e-2)
    # linearity in V (the weights depend on q and k only)
    g = torch.Generator(device="cuda").manual_seed(9)
    v2 = torch.randn(v.shape, generator=g, device="cuda").to(torch.bfloat16)
    o2 = torch.ops.tt.scaled_dot_product_attention(q, k, v2, is_causal=True)
    o12 = torch.ops.tt.scaled_dot_product_attention(q, k, (v.float() + v2.float()).to(torch.bfloat16), is_causal=True)
    torch.testing.assert_close(o12.float(), dense.float() + o2.float(), atol=3e-2, rtol=3e-2)


def test_config4_decode_full_size():
    """Batch 128, 64 / 8 heads, contexts 256 .. 32768 on a fragmented pool (matrix-core decode
    kernel): oracle spot checks on the three shortest and the longest context, invariance
    under a permutation of users, linearity in V."""
    from tt_xla_amd import workloads

    wl = workloads.decode_config4(cache_device="cuda")
    g = wl.to("cuda")
    run = lambda q, vcache, table, pos: torch.ops.tt.paged_scaled_dot_product_attention_decode(  # noqa: E731
        q, g.k_cache, vcache, table, is_causal=True, cur_pos_tensor=pos, scale=wl.scale)
    out = run(g.q, g.v_cache, g.page_table, g.cache_position)
    assert torch.isfinite(out.float()).all()
    pos = wl.cache_position
    order = torch.argsort(pos)
    picks = order[:3].tolist() + [int(order[-1])]
    bs = 64
    for u in picks:
        n = int(pos[u]) + 1
        nblk = (n + bs - 1) // bs
        blocks = wl.page_table[u, :nblk].long().cuda()
        kk = g.k_cache[blocks].cpu()            # [nblk, hkv, bs, d]: this user's blocks, in order
        vv = g.v_cache[blocks].cpu()
        table = torch.arange(nblk, dtype=torch.int32).view(1, nblk)
        want = O.textbook_decode_fp32(wl.q[:, u : u + 1], kk, vv, table, pos[u : u + 1], wl.scale)
        err = (out[0, u].cpu().float() - want[0, 0]).abs().max().item()
        print(f"config4 user {u} context {n}: max-abs error {err:.3e}", flush=True)
        torch.testing.assert_close(out[0, u].cpu().float(), want[0, 0], atol=2e-2, rtol=2e-2)
    perm = torch.randperm(128, generator=torch.Generator().manual_seed(1)).cuda()
    out_p = run(g.q[:, perm], g.v_cache, g.page_table[perm], g.cache_position[perm])
    torch.testing.assert_close(out_p.float(), out[:, perm].float(), atol=4e-3, rtol=4e-3)
    # linearity in V: halving V halves the output (exact in bf16 up to the final rounding)
    half = (g.v_cache.float() * 0.5).to(torch.bfloat16)
    out_h = run(g.q, half, g.page_table, g.cache_position)
    torch.testing.assert_close(out_h.float() * 2, out.float(), atol=1e-2, rtol=1e-2)


def test_config4_chunk_pass_full_size():
    """4 x 512-token chunks on top of 4096 cached tokens, 64 / 8 heads: user 0 against the
    oracle, and the whole pass against itself with V scaled."""
    from tt_xla_amd import workloads

    w = workloads.prefill_config4_chunks(device="cuda").to("cuda")
    u, s, hq, hkv, d = w.users, w.seq, w.q_heads, w.kv_heads, w.head_size
    q = w.q.view(u, s, hq, d).transpose(1, 2)
    k = w.k.view(u, s, hkv, d).transpose(1, 2)
    v = w.v.view(u, s, hkv, d).transpose(1, 2)
    kc, vc = w.k_cache.clone(), w.v_cache.clone()
    torch.ops.tt.paged_fill_cache_(kc, k, w.fill_page_table, w.batch_idx)
    torch.ops.tt.paged_fill_cache_(vc, v, w.fill_page_table, w.batch_idx)
    out = torch.ops.tt.chunked_scaled_dot_product_attention(q, kc, vc, w.page_table, w.chunk_start)
    blocks = w.page_table[0].long()
    kk, vv = kc[blocks].cpu(), vc[blocks].cpu()
    table = torch.arange(blocks.numel(), dtype=torch.int32).view(1, -1)
    want = O.chunked_sdpa(q[:1].cpu(), kk, vv, table, w.chunk_start.cpu(), None)
    err = (out[:1].cpu().float() - want.float()).abs().max().item()
    print(f"{w.name}: max-abs error vs oracle (user 0) {err:.3e}", flush=True)
    torch.testing.assert_close(out[:1].cpu().float(), want.float(), atol=2e-2, rtol=2e-2)
    out_h = torch.ops.tt.chunked_scaled_dot_product_attention(q, kc, (vc.float() * 0.5).to(torch.bfloat16),
                                                              w.page_table, w.chunk_start)
    torch.testing.assert_close(out_h.float() * 2, out.float(), atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("hq", [16, 128])
def test_latent_decode_full_size(monkeypatch, hq):
    """The latent decode workloads of the benchmark (128 users, contexts 512 .. 8192 on a shuffled
    pool, one latent head of 576 features, 16 or 128 query heads): the oracle on the three shortest
    users and the longest, invariance under a permutation of users, and at 128 heads agreement
    with the workgroup-shared kernel, which computes the same thing another way."""
    users, dh, dv, bs, lo, hi = 128, 576, 512, 64, 512, 8192
    print(f"case: latent decode full size h{hq}", flush=True)
    g = torch.Generator().manual_seed(11)
    ctx = torch.randint(lo, hi + 1, (users,), generator=g)
    w = (hi + bs) // bs
    nb = users * w + 1
    gd = torch.Generator(device="cuda").manual_seed(12)
    key = torch.randn(nb, 1, bs, dh, generator=gd, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    table = (torch.randperm(nb - 1, generator=g)[: users * w] + 1).view(users, w).to(torch.int32)
    q = torch.randn(1, users, hq, dh, generator=g).to(torch.bfloat16)
    pos = ctx.to(torch.int32)
    run = lambda qq, tt, pp: torch.ops.tt.paged_flash_mla_decode(qq, key, dv, tt, None, True, None, pp, None, None)  # noqa: E731
    out = run(q.cuda(), table.cuda(), pos.cuda())
    assert torch.isfinite(out.float()).all()
    order = torch.argsort(pos)
    for u in order[:3].tolist() + [int(order[-1])]:
        nblk = int(pos[u]) // bs + 1
        kk = key[table[u, :nblk].long().cuda()].cpu()  # this user's blocks, in order
        t1 = torch.arange(nblk, dtype=torch.int32).view(1, nblk)
        want = O.paged_flash_mla_decode(q[:, u : u + 1], kk, dv, t1, None, pos[u : u + 1], None)
        err = (out[0, u].cpu().float() - want[0, 0].float()).abs().max().item()
        print(f"latent decode h{hq} user {u} context {int(pos[u]) + 1}: max-abs error {err:.3e}", flush=True)
        torch.testing.assert_close(out[0, u].cpu().float(), want[0, 0].float(), atol=2e-2, rtol=2e-2)
    perm = torch.randperm(users, generator=torch.Generator().manual_seed(1))
    out_p = run(q[:, perm].cuda(), table[perm].cuda(), pos[perm].cuda())
    torch.testing.assert_close(out_p.float(), out[:, perm.cuda()].float(), atol=4e-3, rtol=4e-3)
    if hq == 128:
        monkeypatch.setenv("TTPA_LATENT_KERNEL", "wide")
        out_w = run(q.cuda(), table.cuda(), pos.cuda())
        torch.testing.assert_close(out_w.float(), out.float(), atol=8e-3, rtol=8e-3)


def test_latent_prefill_full_size():
    """4 x 2048 tokens, 16 heads over one latent head (576 / 512), causal: batch 0 against the oracle,
    and a causal prefill of the first 1024 tokens must reproduce the first 1024 rows."""
    b, hq, s, dh, dv = 4, 16, 2048, 576, 512
    print("case: latent prefill full size", flush=True)
    g = torch.Generator().manual_seed(21)
    q = (torch.randn(b, hq, s, dh, generator=g) * 0.15).to(torch.bfloat16)
    k = torch.randn(b, 1, s, dh, generator=g).to(torch.bfloat16)
    scale = dh ** -0.5
    out = torch.ops.tt.flash_mla_prefill(q.cuda(), k.cuda(), dv, None, None, True, scale)
    assert out.shape == (b, hq, s, dv) and torch.isfinite(out.float()).all()
    want = O.flash_mla_prefill(q[:1].float(), k[:1].float(), dv, None, None, True, scale)
    err = (out[:1].cpu().float() - want).abs().max().item()
    print(f"latent prefill 4 x 2048, batch 0: max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(out[:1].cpu().float(), want, atol=2e-2, rtol=2e-2)
    head = torch.ops.tt.flash_mla_prefill(q[:, :, :1024].contiguous().cuda(), k[:, :, :1024].contiguous().cuda(), dv, None, None, True, scale)
    torch.testing.assert_close(head.float(), out[:, :, :1024].float(), atol=4e-3, rtol=4e-3)
