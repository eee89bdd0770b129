"""GPU tests of tt::paged_update_kv_decode_ (ttpa_paged_update_decode): the decode step's cache
update and attention in one call.  The contract is "same caches and same output as
paged_update_kv_cache_ followed by paged_scaled_dot_product_attention_decode", so every case
runs both and compares them bit for bit (caches) and within atol = rtol = 2e-2 of the fp32
oracle (output); the rows to be written are poisoned with NaN first, so an implementation
that read the token from the cache instead of the fresh activations would show."""

import pytest
import torch

import __graft_entry__ as entry
from oracle import bfp8_codec as C
from oracle import paged_ops as O

pytestmark = pytest.mark.gpu
ATOL = RTOL = 2e-2


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


CASES = [
    # users, Hq, Hkv, D, bs, contexts (position written = context), bfp8, window, sink, small grid
    (4, 32, 8, 128, 64, [5, 64, 200, 700], False, 0, False, False),     # fused: 16x16 kernel
    (4, 32, 8, 128, 64, [0, 63, 127, 128], False, 0, False, False),     # tile edges
    (3, 16, 2, 128, 16, [15, 16, 100], False, 0, False, False),         # blocks smaller than a tile
    (4, 64, 8, 128, 64, [1990, 30, 1500, 2300], False, 1000, True, True),
    (4, 32, 8, 128, 64, [5, 64, 200, 700], True, 0, False, False),      # block-float-8, fused
    (3, 12, 4, 128, 16, [15, 16, 100], True, 64, True, False),
    (4, 32, 8, 128, 64, [1990, 2047, 1500, 2300], True, 0, False, True),
    (3, 8, 8, 64, 32, [0, 62, 300], False, 0, False, False),            # not fused: two launches
    (2, 8, 4, 128, 32, [40, 333], False, 0, False, False),              # G = 2: fused as a step
    (3, 8, 8, 128, 32, [40, 333, 64], False, 0, False, False),          # G = 1: dot-product kernel, two launches
    (2, 16, 8, 256, 64, [130, 64], False, 0, False, False),             # head size 256, fused
    (4, 8, 4, 256, 16, [31, 32, 1000, 1500], False, 300, True, True),   # blocks smaller than its 32-token tiles
    (3, 16, 8, 256, 32, [31, 32, 700], True, 0, False, False),          # head size 256, block-float-8
    (4, 4, 4, 256, 16, [15, 16, 1000, 1500], True, 300, True, True),
]


@pytest.mark.parametrize("users,hq,hkv,d,bs,ctx,bfp8,window,with_sink,small_grid", CASES)
def test_fused_step_equals_update_then_decode(monkeypatch, users, hq, hkv, d, bs, ctx, bfp8, window,
                                              with_sink, small_grid):
    from tt_xla_amd import custom_ops as ops
    from tt_xla_amd import workloads

    name = f"fused step b{users} h{hq}x{hkv} d{d} bs{bs} ctx{ctx} bfp8={bfp8} window{window} sink{with_sink}"
    print(name, flush=True)
    if small_grid:
        monkeypatch.setenv("TTPA_DECODE_WAVES_PER_CU", "1")
    nb = sum((c + 1 + bs - 1) // bs for c in ctx) + 3
    wl = workloads.decode_ragged(name, hq + d + bs + len(ctx), users, hq, hkv, d, bs, nb, ctx)
    if bfp8:
        workloads.add_outlier_channels(wl, 3, fraction=0.02)
    g = torch.Generator().manual_seed(1)
    sink = (torch.randn(hq, generator=g) * 2).to(torch.bfloat16).cuda() if with_sink else None
    dev = wl.to("cuda")
    # poison the rows the step writes
    for u, c in enumerate(ctx):
        blk = int(wl.page_table[u, c // bs])
        dev.k_cache[blk, :, c % bs, :] = float("nan")
        dev.v_cache[blk, :, c % bs, :] = float("nan")
    if bfp8:
        k0, v0 = ops.bfp8_pack_cache(torch.nan_to_num(dev.k_cache, nan=777.0)), \
            ops.bfp8_pack_cache(torch.nan_to_num(dev.v_cache, nan=-777.0))
    else:
        k0, v0 = dev.k_cache, dev.v_cache
    kw = dict(scale=wl.scale, sliding_window_size=window if window else None, attention_sink=sink)

    k_fus, v_fus = k0.clone(), v0.clone()
    out_fus = torch.ops.tt.paged_update_kv_decode_(
        dev.q, k_fus, v_fus, dev.k_new, dev.v_new, dev.page_table, dev.cache_position, **kw)

    # As a step, groups of 2 and 3 heads run on the 16x16x32 kernel, which the attention alone
    # only picks from 4 up: ask for it on the reference side, so that both run the same
    # arithmetic and the outputs can be compared exactly.
    if not bfp8 and d in (64, 128) and hq // hkv in (2, 3):
        monkeypatch.setenv("TTPA_DECODE_KERNEL", "mfma16")
    k_seq, v_seq = k0.clone(), v0.clone()
    torch.ops.tt.paged_update_kv_cache_(k_seq, v_seq, dev.k_new, dev.v_new, dev.cache_position, dev.page_table)
    out_seq = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        dev.q, k_seq, v_seq, dev.page_table, is_causal=True, cur_pos_tensor=dev.cache_position, **kw)
    torch.cuda.synchronize()

    assert torch.equal(k_fus.view(torch.uint8), k_seq.view(torch.uint8)), "K cache differs"
    assert torch.equal(v_fus.view(torch.uint8), v_seq.view(torch.uint8)), "V cache differs"
    assert torch.isfinite(out_fus).all()
    torch.testing.assert_close(out_fus.float(), out_seq.float(), atol=1e-6, rtol=0)

    if bfp8:
        k_ref = C.unpack_cache(k_seq.cpu(), bs).to(torch.bfloat16)
        v_ref = C.unpack_cache(v_seq.cpu(), bs).to(torch.bfloat16)
    else:
        k_ref, v_ref = k_seq.cpu(), v_seq.cpu()
    want = O.paged_sdpa_decode_windowed(wl.q, k_ref, v_ref, wl.page_table, wl.cache_position, wl.scale,
                                        window, None if sink is None else sink.cpu())
    err = (out_fus.cpu().float() - want).abs().max().item()
    print(f"  max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(out_fus.cpu().float(), want, atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("bfp8", [False, True])
def test_fused_step_padded_rows_and_positions_outside_the_table(bfp8):
    """Position -1 (padded batch row): nothing attended (NaN row), and the write follows the
    update operator's rule for negative positions; a position beyond the table: the whole table
    is attended and nothing is written.  Both exactly as the two separate operators do."""
    from tt_xla_amd import custom_ops as ops
    from tt_xla_amd import workloads

    users, hq, hkv, d, bs = 5, 32, 8, 128, 32
    ctx = [40, 0, 100, 0, 95]
    wl = workloads.decode_ragged("fused-edges", 21, users, hq, hkv, d, bs, 16, ctx, table_width=4)
    wl.cache_position[1] = -1
    wl.cache_position[3] = -5
    wl.cache_position[4] = 500          # the table holds 128 positions
    # Padded rows write into the null block 0 that their zero table points to; the user that
    # attends its whole table gets a real last block, so that it does not read rows another
    # user writes in the same step (such aliasing is outside the operator's contract).
    wl.page_table[4, 3] = 15
    dev = wl.to("cuda")
    k0 = ops.bfp8_pack_cache(dev.k_cache) if bfp8 else dev.k_cache
    v0 = ops.bfp8_pack_cache(dev.v_cache) if bfp8 else dev.v_cache
    k_seq, v_seq, k_fus, v_fus = k0.clone(), v0.clone(), k0.clone(), v0.clone()
    torch.ops.tt.paged_update_kv_cache_(k_seq, v_seq, dev.k_new, dev.v_new, dev.cache_position, dev.page_table)
    out_seq = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        dev.q, k_seq, v_seq, dev.page_table, is_causal=True, cur_pos_tensor=dev.cache_position, scale=wl.scale)
    out_fus = torch.ops.tt.paged_update_kv_decode_(
        dev.q, k_fus, v_fus, dev.k_new, dev.v_new, dev.page_table, dev.cache_position, scale=wl.scale)
    torch.cuda.synchronize()
    assert torch.equal(k_fus.view(torch.uint8), k_seq.view(torch.uint8))
    assert torch.equal(v_fus.view(torch.uint8), v_seq.view(torch.uint8))
    assert not torch.equal(k_fus.view(torch.uint8), k0.view(torch.uint8))
    assert torch.isnan(out_fus[0, 1]).all() and torch.isnan(out_fus[0, 3]).all()
    live = [0, 2, 4]
    torch.testing.assert_close(out_fus[0, live].float(), out_seq[0, live].float(), atol=1e-6, rtol=0)


def test_backend_decode_step_uses_the_fused_operator():
    """TTAttentionBackendImpl.forward on a decode pass: same output and caches with the fused
    step (default) and with the reference's call sequence (functional_cache_ops=True)."""
    from tt_xla_amd import workloads
    from tt_xla_amd.attention import TTAttentionBackendImpl, TTMetadata

    users, hq, hkv, d, bs = 4, 32, 8, 128, 64
    wl = workloads.decode_ragged("backend-fused", 31, users, hq, hkv, d, bs, 24, [5, 64, 200, 300]).to("cuda")
    meta = TTMetadata(cache_position=wl.cache_position, page_table=wl.page_table, is_causal=True,
                      num_users=users)
    q = wl.q[0].reshape(users, hq * d)
    k = wl.k_new[0].reshape(users, hkv * d)
    v = wl.v_new[0].reshape(users, hkv * d)
    results = []
    for functional in (False, True):
        impl = TTAttentionBackendImpl(hq, d, wl.scale, hkv, functional_cache_ops=functional)
        caches = [wl.k_cache.clone(), wl.v_cache.clone()]
        out = torch.empty(users, hq * d, dtype=torch.bfloat16, device="cuda")
        impl.forward(None, q, k, v, caches, meta, output=out)
        results.append((out, caches))
    torch.cuda.synchronize()
    (o1, c1), (o2, c2) = results
    assert torch.equal(c1[0], c2[0]) and torch.equal(c1[1], c2[1])
    torch.testing.assert_close(o1.float(), o2.float(), atol=1e-6, rtol=0)
