"""GPU parity, bit-exact: tt::paged_update_cache / tt::paged_fill_cache (HIP kernels behind
the C ABI) against the CPU oracle on the same seeded inputs.  Grids follow the reference's
op tests (tests/torch/ops/test_custom_ops.py:139-203)."""

import pytest
import torch

import __graft_entry__ as entry
from oracle import paged_ops as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def _table(gen, users, bps):
    perm = torch.randperm(users * bps, generator=gen)
    return torch.argsort(perm).reshape(users, bps).to(torch.int32)


def _dev(*ts):
    return [t.cuda() if isinstance(t, torch.Tensor) else t for t in ts]


UPDATE_GRID = [
    (8, 16, 1, 32, 128), (16, 16, 8, 64, 128), (24, 16, 8, 32, 256), (32, 16, 1, 128, 128),
    (8, 32, 8, 32, 128), (8, 16, 32, 32, 128), (32, 32, 8, 64, 128), (16, 16, 8, 128, 256),
    (1, 16, 8, 32, 64), (32, 16, 32, 64, 128),
]


@pytest.mark.parametrize("users,bps,heads,bs,d", UPDATE_GRID)
@pytest.mark.parametrize("idx_dtype", [torch.int64, torch.int32])
def test_update_bit_exact(users, bps, heads, bs, d, idx_dtype):
    print(f"update users={users} bps={bps} heads={heads} bs={bs} d={d}", flush=True)
    g = torch.Generator().manual_seed(users + bps + heads + bs + d)
    cache = torch.randn(users * bps, heads, bs, d, generator=g).to(torch.bfloat16)
    fill = torch.randn(1, users, heads, d, generator=g).to(torch.bfloat16)
    idx = torch.randperm(bps * bs, generator=g)[:users].to(idx_dtype)
    table = _table(g, users, bps)
    want = O.paged_update_cache(cache, fill, idx, table)
    c, f, i, t = _dev(cache, fill, idx, table)
    got = torch.ops.tt.paged_update_cache(c, f, i, t)
    assert torch.equal(got.cpu(), want)
    assert torch.equal(c.cpu(), cache), "functional op must not touch its input"
    torch.ops.tt.paged_update_cache_(c, f, i, t)
    assert torch.equal(c.cpu(), want)


def test_update_backend_view_padded_heads_and_padded_rows():
    """fill arrives as key.transpose(0, 1) of [users, 1, heads, D] (attention.py:470-471),
    may carry more heads than the cache, and padded rows have position -1."""
    g = torch.Generator().manual_seed(3)
    users, hkv, bs, d, w = 6, 4, 32, 128, 4
    cache = torch.zeros(users * w, hkv, bs, d, dtype=torch.bfloat16)
    key = torch.randn(users, 1, 8, d, generator=g).to(torch.bfloat16)
    table = _table(g, users, w)
    table[4:] = 0
    idx = torch.tensor([0, 31, 32, 127, -1, -1], dtype=torch.int32)
    want = O.paged_update_cache(cache, key.transpose(0, 1), idx, table)
    c, k, i, t = _dev(cache, key, idx, table)
    got = torch.ops.tt.paged_update_cache(c, k.transpose(0, 1), i, t)
    # rows 4 and 5 both target block 0, row bs-1: the winner is unspecified on both sides
    mask = torch.ones_like(want, dtype=torch.bool)
    mask[0, :, bs - 1] = False
    assert torch.equal(got.cpu()[mask], want[mask])
    row = got.cpu()[0, :, bs - 1]
    assert torch.equal(row, key[4, 0, :hkv]) or torch.equal(row, key[5, 0, :hkv])


@pytest.mark.parametrize("fmt", ["bf16", "bfp8"])
def test_update_kv_single_launch_equals_two_updates(fmt):
    """tt::paged_update_kv_cache_ (one launch for K and V) against the oracle applied twice."""
    from oracle import bfp8_codec as C

    g = torch.Generator().manual_seed(21)
    users, hkv, bs, d, w = 7, 8, 32, 128, 3
    nb = users * w
    kc = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    vc = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    key = torch.randn(users, 1, hkv, d, generator=g).to(torch.bfloat16)
    val = torch.randn(users, 1, hkv, d, generator=g).to(torch.bfloat16)
    table = _table(g, users, w)
    idx = torch.randint(0, w * bs, (users,), generator=g, dtype=torch.int32)
    k_want = O.paged_update_cache(kc, key.transpose(0, 1), idx, table)
    v_want = O.paged_update_cache(vc, val.transpose(0, 1), idx, table)
    if fmt == "bfp8":
        k_dev, v_dev = C.pack_cache(kc).cuda(), C.pack_cache(vc).cuda()
        k_want, v_want = C.pack_cache(k_want), C.pack_cache(v_want)
    else:
        k_dev, v_dev = kc.cuda(), vc.cuda()
    torch.ops.tt.paged_update_kv_cache_(k_dev, v_dev, key.cuda().transpose(0, 1),
                                        val.cuda().transpose(0, 1), idx.cuda(), table.cuda())
    assert torch.equal(k_dev.cpu(), k_want) and torch.equal(v_dev.cpu(), v_want)


def test_update_out_of_table_positions_are_skipped():
    cache = torch.zeros(4, 1, 32, 64, dtype=torch.bfloat16)
    fill = torch.ones(1, 2, 1, 64, dtype=torch.bfloat16)
    table = torch.tensor([[1, 2], [3, 99]], dtype=torch.int32)
    idx = torch.tensor([64, 40], dtype=torch.int32)  # column 2 of 2; physical block 99 of 4
    c, f, i, t = _dev(cache, fill, idx, table)
    got = torch.ops.tt.paged_update_cache(c, f, i, t)
    assert got.abs().sum().item() == 0


FILL_GRID = [
    (8, 16, 1, 32, 128, 10), (8, 16, 8, 32, 128, 20), (16, 16, 8, 64, 128, 32),
    (8, 32, 32, 32, 128, 50), (16, 16, 8, 64, 128, 70), (8, 16, 8, 32, 128, 70),
    (8, 16, 8, 64, 128, 64), (4, 8, 8, 128, 256, 300), (2, 4, 2, 32, 64, 1),
    (4, 8, 4, 48, 128, 200), (4, 16, 2, 20, 64, 131), (3, 40, 2, 1, 128, 33),   # block sizes off the powers of two, and 1
    (2, 4, 2, 32, 40, 50),                                                     # head size with 5 chunks per row
]


@pytest.mark.parametrize("users,bps,heads,bs,d,s", FILL_GRID)
def test_fill_single_user_bit_exact(users, bps, heads, bs, d, s):
    print(f"fill users={users} bps={bps} heads={heads} bs={bs} d={d} s={s}", flush=True)
    g = torch.Generator().manual_seed(s + users + heads + bs)
    cache = torch.randn(users * bps, heads, bs, d, generator=g).to(torch.bfloat16)
    fill = torch.randn(1, heads, s, d, generator=g).to(torch.bfloat16)
    table = _table(g, users, bps)
    b = torch.randint(0, users, (1,), generator=g, dtype=torch.int32)
    want = O.paged_fill_cache(cache, fill, table, b)
    c, f, t, bb = _dev(cache, fill, table, b)
    got = torch.ops.tt.paged_fill_cache(c, f, t, bb)
    assert torch.equal(got.cpu(), want)
    assert torch.equal(c.cpu(), cache)
    torch.ops.tt.paged_fill_cache_(c, f, t, bb)
    assert torch.equal(c.cpu(), want)


def test_fill_default_batch_idx():
    g = torch.Generator().manual_seed(2)
    cache = torch.randn(8, 2, 32, 64, generator=g).to(torch.bfloat16)
    fill = torch.randn(1, 2, 40, 64, generator=g).to(torch.bfloat16)
    table = _table(g, 2, 4)
    want = O.paged_fill_cache(cache, fill, table)
    c, f, t = _dev(cache, fill, table)
    assert torch.equal(torch.ops.tt.paged_fill_cache(c, f, t).cpu(), want)


@pytest.mark.parametrize("s", [32, 50, 512])
def test_fill_batched_backend_view(s):
    """The plugin's call: fill = key.transpose(1, 2) of [users, S, Hkv, D], batch_idx per
    row (attention.py:486-511).  Defined as the single-user op applied row by row."""
    g = torch.Generator().manual_seed(s)
    users, hkv, bs, d = 4, 8, 32, 128
    w = (s + bs - 1) // bs + 1
    cache = torch.zeros(users * w + 1, hkv, bs, d, dtype=torch.bfloat16)
    key = torch.randn(users, s, hkv, d, generator=g).to(torch.bfloat16)
    table = (_table(g, users, w) + 1).to(torch.int32)
    bidx = torch.tensor([2, 0, 3, 1], dtype=torch.int32)
    want = O.paged_fill_cache_batched(cache, key.transpose(1, 2), table, bidx)
    c, k, t, b = _dev(cache, key, table, bidx)
    got = torch.ops.tt.paged_fill_cache(c, k.transpose(1, 2), t, batch_idx=b)
    assert torch.equal(got.cpu(), want)
    assert torch.equal(O.gather_paged_to_dense(got.cpu(), table[bidx.long()])[:, :, :s],
                       key.transpose(1, 2))


@pytest.mark.parametrize("fmt", ["bf16", "bfp8"])
@pytest.mark.parametrize("s", [32, 50, 300])
def test_fill_kv_single_launch_equals_two_fills(fmt, s):
    """tt::paged_fill_kv_cache_ (one launch for K and V) against the oracle's batched fill applied
    to each cache; one batch_idx entry points outside the table (its row is skipped)."""
    from oracle import bfp8_codec as C

    g = torch.Generator().manual_seed(100 + s)
    users, hkv, bs, d = 4, 4, 32, 128
    w = (s + bs - 1) // bs + 1
    nb = users * w + 1
    kc = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    vc = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    key = torch.randn(users, s, hkv, d, generator=g).to(torch.bfloat16)
    val = torch.randn(users, s, hkv, d, generator=g).to(torch.bfloat16)
    table = (_table(g, users, w) + 1).to(torch.int32)
    bidx = torch.tensor([2, 0, 9, 1], dtype=torch.int32)
    # the oracle takes rows inside the table: the skipped row is left out of its call
    keep = [0, 1, 3]
    k_want = O.paged_fill_cache_batched(kc, key[keep].transpose(1, 2), table, bidx[keep])
    v_want = O.paged_fill_cache_batched(vc, val[keep].transpose(1, 2), table, bidx[keep])
    if fmt == "bfp8":
        k_dev, v_dev = C.pack_cache(kc).cuda(), C.pack_cache(vc).cuda()
        k_want, v_want = C.pack_cache(k_want), C.pack_cache(v_want)
    else:
        k_dev, v_dev = kc.cuda(), vc.cuda()
    torch.ops.tt.paged_fill_kv_cache_(k_dev, v_dev, key.cuda().transpose(1, 2), val.cuda().transpose(1, 2),
                                      table.cuda(), batch_idx=bidx.cuda())
    assert torch.equal(k_dev.cpu(), k_want) and torch.equal(v_dev.cpu(), v_want)


def test_fill_rejects_sequence_longer_than_table():
    cache = torch.zeros(4, 1, 32, 64, dtype=torch.bfloat16).cuda()
    fill = torch.zeros(1, 1, 65, 64, dtype=torch.bfloat16).cuda()
    table = torch.zeros(1, 2, dtype=torch.int32).cuda()
    with pytest.raises(ValueError):
        torch.ops.tt.paged_fill_cache(cache, fill, table)


def test_update_then_gather_roundtrip_full_size():
    """Llama-3-8B cache shape: write one token per user, read it back through the table;
    every other byte of the 512 MiB cache is unchanged (checked by checksum)."""
    from tt_xla_amd import workloads

    wl = workloads.decode_config2()
    g = wl.to("cuda")
    before = g.k_cache.view(torch.int16).to(torch.int64).sum()
    torch.ops.tt.paged_update_cache_(g.k_cache, g.k_new, g.cache_position, g.page_table)
    pos = wl.cache_position.long()
    blk = wl.page_table[torch.arange(32), pos // 64].long()
    rows = g.k_cache[blk.cuda(), :, (pos % 64).cuda(), :].cpu()
    assert torch.equal(rows, wl.k_new[0])
    old_rows = wl.k_cache[blk, :, pos % 64, :]
    delta = rows.view(torch.int16).to(torch.int64).sum() - old_rows.view(torch.int16).to(torch.int64).sum()
    after = g.k_cache.view(torch.int16).to(torch.int64).sum()
    assert (after - before).item() == delta.item()
