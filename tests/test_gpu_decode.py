"""GPU parity for tt::paged_scaled_dot_product_attention_decode: HIP split-K kernel behind
the C ABI against the CPU oracle (restated reference CPU branch; grouped heads through the
reference-held MLA-form, see oracle/paged_ops.py) on the same seeded inputs.
Tolerance atol = rtol = 2e-2 on bf16 outputs; max-abs error is printed."""

import math

import pytest
import torch

import __graft_entry__ as entry
from oracle import paged_ops as O

pytestmark = pytest.mark.gpu
ATOL = RTOL = 2e-2


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def _run(wl, update=True):
    g = wl.to("cuda")
    if update:
        k = torch.ops.tt.paged_update_cache(g.k_cache, g.k_new, g.cache_position, g.page_table)
        v = torch.ops.tt.paged_update_cache(g.v_cache, g.v_new, g.cache_position, g.page_table)
    else:
        k, v = g.k_cache, g.v_cache
    out = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        g.q, k, v, g.page_table, is_causal=True, cur_pos_tensor=g.cache_position, scale=wl.scale
    )
    torch.cuda.synchronize()
    return out.cpu(), k, v


def _check(name, got, want):
    err = (got.float() - want.float()).abs().max().item()
    print(f"{name}: max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(got.float(), want.float(), atol=ATOL, rtol=RTOL)


def test_config1_reference_cpu_case():
    from tt_xla_amd import workloads

    wl = workloads.decode_config1()
    got, k, v = _run(wl)
    k_ref = O.paged_update_cache(wl.k_cache, wl.k_new, wl.cache_position, wl.page_table)
    v_ref = O.paged_update_cache(wl.v_cache, wl.v_new, wl.cache_position, wl.page_table)
    assert torch.equal(k.cpu(), k_ref) and torch.equal(v.cpu(), v_ref)
    want = O.paged_sdpa_decode(wl.q, k_ref, v_ref, wl.page_table, True, None, wl.cache_position,
                               None, wl.scale)
    _check(wl.name, got, want)
    _check(wl.name + " vs fp32", got,
           O.textbook_decode_fp32(wl.q, k_ref, v_ref, wl.page_table, wl.cache_position, wl.scale))


SHAPES = [
    # users, Hq, Hkv, D, bs, contexts
    (8, 8, 8, 128, 32, [1, 1, 1, 1, 1, 1, 1, 1]),  # reference op test: cur_pos all ones
    (3, 8, 8, 64, 32, [0, 62, 63]),
    (4, 8, 8, 128, 64, [63, 64, 65, 300]),
    (2, 1, 1, 128, 128, [127, 700]),
    (5, 8, 2, 64, 32, [10, 200, 31, 32, 33]),
    (4, 32, 8, 128, 64, [5, 64, 200, 700]),
    (3, 12, 4, 128, 32, [100, 17, 450]),
    (2, 64, 8, 128, 64, [1000, 257]),
    (2, 16, 8, 256, 64, [130, 64]),
    (2, 8, 8, 256, 128, [255, 700]),
    (3, 16, 8, 128, 16, [15, 16, 100]),
    (3, 40, 8, 128, 32, [40, 333, 64]),
    (2, 6, 1, 64, 32, [95, 96]),
    (2, 7, 1, 128, 32, [95, 96]),
]


@pytest.mark.parametrize("users,hq,hkv,d,bs,ctx", SHAPES)
def test_decode_shapes(users, hq, hkv, d, bs, ctx):
    from tt_xla_amd import workloads

    name = f"decode b{users} h{hq}x{hkv} d{d} bs{bs} ctx{ctx}"
    print(name, flush=True)
    nb = sum((c + 1 + bs - 1) // bs for c in ctx) + 3
    wl = workloads.decode_ragged(name, hq * 7 + d + bs, users, hq, hkv, d, bs, nb, ctx)
    got, k, v = _run(wl)
    want = O.paged_sdpa_decode(wl.q, k.cpu(), v.cpu(), wl.page_table, True, None,
                               wl.cache_position, None, wl.scale)
    _check(name, got, want)
    _check(name + " vs fp32", got,
           O.textbook_decode_fp32(wl.q, k.cpu(), v.cpu(), wl.page_table, wl.cache_position, wl.scale))


def test_decode_padded_rows_nan_and_default_scale_and_int64_positions():
    from tt_xla_amd import workloads

    wl = workloads.decode_ragged("padded", 11, 4, 8, 2, 128, 32, 32, [40, 0, 100, 0])
    wl.cache_position[1] = -1
    wl.cache_position[3] = -1
    wl.page_table[1] = 0
    wl.page_table[3] = 0
    g = wl.to("cuda")
    out = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        g.q, g.k_cache, g.v_cache, g.page_table, True, None, g.cache_position.long()
    ).cpu()
    want = O.paged_sdpa_decode(wl.q, wl.k_cache, wl.v_cache, wl.page_table, True, None,
                               wl.cache_position)
    # a row that attends nothing is softmax over an empty set: NaN, as on the reference's
    # decode branch (custom_ops.py:1295-1311; pinned in tests/test_oracle_attention.py).
    # The grouped-head stand-in goes through the library SDPA, which answers 0 for such
    # rows, so only live rows are compared against it.
    assert torch.isnan(out[0, 1]).all() and torch.isnan(out[0, 3]).all()
    _check("padded live rows", out[0, [0, 2]], want[0, [0, 2]])


def test_decode_position_beyond_table_attends_whole_table():
    from tt_xla_amd import workloads

    wl = workloads.decode_ragged("beyond", 12, 2, 8, 8, 64, 32, 16, [63, 95], table_width=3)
    wl.cache_position[0] = 500  # table holds 96 positions; the reference masks nothing then
    got, _, _ = _run(wl, update=False)
    want = O.paged_sdpa_decode(wl.q, wl.k_cache, wl.v_cache, wl.page_table, True, None,
                               wl.cache_position, None, wl.scale)
    _check("beyond-table", got, want)


def test_decode_query_view_from_backend_layout():
    """q arrives as query.transpose(0, 1) of [users, 1, Hq, D] (attention.py:644)."""
    from tt_xla_amd import workloads

    wl = workloads.decode_ragged("qview", 13, 3, 8, 2, 128, 32, 16, [20, 70, 33])
    g = wl.to("cuda")
    q_users_first = g.q.transpose(0, 1).contiguous()  # [users, 1, Hq, D]
    a = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        q_users_first.transpose(0, 1), g.k_cache, g.v_cache, g.page_table, True, None, g.cache_position)
    b = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        g.q, g.k_cache, g.v_cache, g.page_table, True, None, g.cache_position)
    assert torch.equal(a, b)


def test_decode_argument_errors():
    from tt_xla_amd import workloads

    g = workloads.decode_ragged("err", 14, 2, 8, 2, 128, 32, 8, [20, 33]).to("cuda")
    with pytest.raises(AssertionError):
        torch.ops.tt.paged_scaled_dot_product_attention_decode(g.q, g.k_cache, g.v_cache, g.page_table, True)
    with pytest.raises(AssertionError):
        torch.ops.tt.paged_scaled_dot_product_attention_decode(
            g.q, g.k_cache, g.v_cache, g.page_table, True, torch.zeros(1, device="cuda"), g.cache_position)


def test_config2_full_size():
    """Llama-3-8B shape at full size against the oracle (a few seconds of CPU) and the
    split-independent property: the result must not depend on how the tile list is cut,
    checked by permuting users (which moves every segment to other wavefronts)."""
    from tt_xla_amd import workloads

    wl = workloads.decode_config2()
    got, k, v = _run(wl)
    want = O.paged_sdpa_decode(wl.q, k.cpu(), v.cpu(), wl.page_table, True, None,
                               wl.cache_position, None, wl.scale)
    _check(wl.name, got, want)
    perm = torch.randperm(32, generator=torch.Generator().manual_seed(0))
    g = wl.to("cuda")
    out_p = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        g.q[:, perm.cuda()], k, v, g.page_table[perm.cuda()], True, None,
        g.cache_position[perm.cuda()], None, wl.scale).cpu()
    torch.testing.assert_close(out_p.float(), got[:, perm].float(), atol=4e-3, rtol=4e-3)


@pytest.mark.parametrize("kernel", ["valu", "mfma", "mfma16"])
@pytest.mark.parametrize("users,hq,hkv,d,bs,ctx", [
    (4, 32, 8, 128, 64, [5, 64, 200, 700]),
    (2, 64, 8, 128, 64, [1000, 257]),
    (3, 16, 8, 128, 16, [15, 16, 100]),
    (3, 12, 4, 128, 32, [100, 17, 450]),
    (3, 16, 8, 256, 32, [31, 32, 700]),          # head size 256: tiles of 32 tokens on the 16x16 kernel
    (3, 24, 2, 256, 8, [100, 17, 450]),          # blocks smaller than a tile, 12 heads per group
    (2, 16, 16, 256, 16, [63, 64]),              # one query head per KV head
    (3, 32, 8, 128, 48, [47, 48, 700]),          # block sizes that are not powers of two: quarter-tile runs
    (3, 32, 8, 128, 24, [23, 24, 700]),          # ... one run per load
    (3, 16, 4, 64, 96, [95, 96, 1000]),
    (2, 8, 2, 256, 12, [11, 300]),
])
def test_decode_every_kernel(monkeypatch, kernel, users, hq, hkv, d, bs, ctx):
    """The dot-product kernel and the two matrix-core kernels, each forced in turn on the same
    bfloat16 cache (a kernel that does not cover a shape leaves it to the default choice)."""
    from tt_xla_amd import workloads

    monkeypatch.setenv("TTPA_DECODE_KERNEL", kernel)
    name = f"decode [{kernel}] b{users} h{hq}x{hkv} d{d} bs{bs} ctx{ctx}"
    print(name, flush=True)
    nb = sum((c + 1 + bs - 1) // bs for c in ctx) + 3
    wl = workloads.decode_ragged(name, hq * 7 + d + bs, users, hq, hkv, d, bs, nb, ctx)
    got, k, v = _run(wl)
    _check(name, got,
           O.textbook_decode_fp32(wl.q, k.cpu(), v.cpu(), wl.page_table, wl.cache_position, wl.scale))


@pytest.mark.parametrize("kernel,hq,d", [("valu", 32, 128), ("mfma", 64, 128), ("mfma16", 64, 128),
                                          ("mfma16", 32, 128), ("mfma16", 32, 256), ("mfma16", 8, 256)])
def test_decode_several_tiles_per_wavefront(monkeypatch, kernel, hq, d):
    """A grid of one wavefront per CU over ~1000 tiles: every wavefront walks several tiles and
    crosses segment boundaries (running maximum, partial hand-over, Q reload)."""
    from tt_xla_amd import workloads

    monkeypatch.setenv("TTPA_DECODE_KERNEL", kernel)
    monkeypatch.setenv("TTPA_DECODE_WAVES_PER_CU", "1")
    ctx = [1990, 2047, 1500, 2300]
    name = f"decode [{kernel}] h{hq}x8 d{d} one wavefront per CU ctx{ctx}"
    print(name, flush=True)
    nb = sum((c + 1 + 63) // 64 for c in ctx) + 3
    wl = workloads.decode_ragged(name, 91, 4, hq, 8, d, 64, nb, ctx)
    got, k, v = _run(wl)
    _check(name, got,
           O.textbook_decode_fp32(wl.q, k.cpu(), v.cpu(), wl.page_table, wl.cache_position, wl.scale))


@pytest.mark.parametrize("seg_units", ["0", "1", "3"])
@pytest.mark.parametrize("waves", ["0.25", "1", "3"])
@pytest.mark.parametrize("kernel,hq", [("mfma16", 32), ("mfma", 64), ("valu", 8)])
def test_decode_ranges_weighted_by_segment_changes(monkeypatch, seg_units, waves, kernel, hq):
    """The decode kernels cut the flat list into ranges of units, with `seg_units` units in front
    of every segment's tiles (tests/test_decode_schedule_model.py holds the arithmetic): short and
    long segments, a padded user and one tile per user, on grids where a wavefront crosses many
    segments (a quarter wavefront per CU) and where most wavefronts hold a single tile."""
    from tt_xla_amd import workloads

    monkeypatch.setenv("TTPA_DECODE_KERNEL", kernel)
    monkeypatch.setenv("TTPA_DECODE_WAVES_PER_CU", waves)
    monkeypatch.setenv("TTPA_DECODE_SEG_UNITS", seg_units)
    ctx = [5, 700, 31, 32, 33, 1200, 0, 64, 95, 257]
    name = f"decode [{kernel}] h{hq}x8 d128 seg_units={seg_units} waves/CU={waves} ctx{ctx}"
    print(name, flush=True)
    nb = sum((c + 1 + 63) // 64 for c in ctx) + 3
    wl = workloads.decode_ragged(name, 93, len(ctx), hq, 8, 128, 64, nb, ctx)
    got, k, v = _run(wl)
    _check(name, got,
           O.textbook_decode_fp32(wl.q, k.cpu(), v.cpu(), wl.page_table, wl.cache_position, wl.scale))


@pytest.mark.parametrize("bfp8", [False, True])
def test_decode_more_than_1024_users_on_the_matrix_core_kernel(bfp8):
    """1300 users (the library's limit is 2048) with 4 query heads per KV head: the 16x16x32
    kernel's prefix tables hold them; contexts of 0 ... 40 tokens and a few padded rows."""
    from tt_xla_amd import custom_ops as ops
    from tt_xla_amd import workloads

    users, hq, hkv, d, bs = 1300, 8, 2, 128, 16
    import random
    r = random.Random(5)
    ctx = [r.randint(0, 40) for _ in range(users)]
    nb = sum((c + 1 + bs - 1) // bs for c in ctx) + 3
    name = f"decode b{users} h{hq}x{hkv} d{d} bs{bs} bfp8={bfp8}"
    print(name, flush=True)
    wl = workloads.decode_ragged(name, 77, users, hq, hkv, d, bs, nb, ctx)
    for u in (3, 700, 1299):
        wl.cache_position[u] = -1
    dev = wl.to("cuda")
    kc, vc, k_ref, v_ref = dev.k_cache, dev.v_cache, wl.k_cache, wl.v_cache
    if bfp8:
        from oracle import bfp8_codec as C
        kc, vc = ops.bfp8_pack_cache(kc), ops.bfp8_pack_cache(vc)
        k_ref = C.unpack_cache(kc.cpu(), bs).to(torch.bfloat16)
        v_ref = C.unpack_cache(vc.cpu(), bs).to(torch.bfloat16)
    got = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        dev.q, kc, vc, dev.page_table, is_causal=True, cur_pos_tensor=dev.cache_position, scale=wl.scale).cpu()
    want = O.textbook_decode_fp32(wl.q, k_ref, v_ref, wl.page_table, wl.cache_position, wl.scale)
    live = [u for u in range(users) if u not in (3, 700, 1299)]
    assert torch.isnan(got[0, [3, 700, 1299]]).all()
    _check(name, got[:, live], want[:, live])


@pytest.mark.parametrize("hq,hkv,d,bs,bfp8,kernel", [
    (8, 8, 64, 32, False, ""), (32, 8, 128, 64, False, ""), (16, 4, 128, 32, True, ""),
    (32, 8, 128, 64, False, "valu"),     # the dot-product kernel where the matrix-core one is the default
    (8, 8, 64, 32, False, "mfma16"),     # ... and the other way round
    (48, 4, 128, 32, False, ""),         # 12 heads per group: the matrix-core kernel only
    (16, 1, 256, 16, True, ""),          # 16 heads, head size 256, block-float-8
    (24, 2, 64, 48, True, ""),           # a block size that is no power of two
    (64, 2, 128, 32, False, ""),         # 32 heads per group: the 32x32x16 kernel
    (48, 2, 64, 32, True, ""),           # 24 heads per group, block-float-8, head size 64: the same
    (16, 4, 128, 32, False, "mfma"),     # ... forced where the 16x16x32 kernel is the default
    (80, 2, 128, 32, False, ""),         # 40 heads per group: gathered through the dense kernel, one mask row for all heads
])
def test_decode_with_explicit_mask(monkeypatch, hq, hkv, d, bs, bfp8, kernel):
    """is_causal=False with an additive attn_mask [users, 1, 1, W*bs] (reference CPU branch
    custom_ops.py:1299-1311; the one-token pass of an encoder / pooling model) against the
    oracle's masked form: every position of the table is attended, weighted by the mask.  A
    boolean mask means "attend where True"."""
    from oracle import bfp8_codec as C
    from tt_xla_amd import custom_ops as ops

    if kernel:
        monkeypatch.setenv("TTPA_DECODE_KERNEL", kernel)
    else:
        monkeypatch.delenv("TTPA_DECODE_KERNEL", raising=False)

    g = torch.Generator().manual_seed(hq + d)
    users, w = 3, 5
    span = w * bs
    nb = users * w + 1
    key = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    value = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    table = (torch.randperm(nb - 1, generator=g) + 1).view(users, w).to(torch.int32)
    q = torch.randn(1, users, hq, d, generator=g).to(torch.bfloat16)
    cur = torch.tensor([3, 40, span - 1], dtype=torch.int32)
    mask = torch.randn(users, 1, 1, span, generator=g).to(torch.bfloat16)
    keep = torch.rand(users, 1, 1, span, generator=g) > 0.4
    keep[:, :, :, 0] = True
    mask = mask.masked_fill(~keep, float("-inf"))
    name = f"masked decode h{hq}x{hkv} d{d} bs{bs} bfp8={bfp8} kernel={kernel or 'default'}"
    print(name, flush=True)
    if bfp8:
        kd, vd = ops.bfp8_pack_cache(key.cuda()), ops.bfp8_pack_cache(value.cuda())
        key, value = C.unpack_cache(kd.cpu(), bs).to(torch.bfloat16), C.unpack_cache(vd.cpu(), bs).to(torch.bfloat16)
    else:
        kd, vd = key.cuda(), value.cuda()
    got = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        q.cuda(), kd, vd, table.cuda(), is_causal=False, attn_mask=mask.cuda(), cur_pos_tensor=cur.cuda(),
        scale=0.11).cpu()
    want = O.paged_sdpa_decode(q.float(), key.float(), value.float(), table, False, mask.float(), cur, None, 0.11)
    err = (got.float() - want).abs().max().item()
    print(f"{name}: max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(got.float(), want, atol=ATOL, rtol=RTOL)
    got_b = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        q.cuda(), kd, vd, table.cuda(), is_causal=False, attn_mask=keep.cuda(), cur_pos_tensor=cur.cuda(),
        scale=0.11).cpu()
    want_b = O.paged_sdpa_decode(q.float(), key.float(), value.float(), table, False,
                                 torch.zeros(users, 1, 1, span).masked_fill(~keep, float("-inf")), cur, None, 0.11)
    torch.testing.assert_close(got_b.float(), want_b, atol=ATOL, rtol=RTOL)
    # a mask per head: on the decode kernels (up to 32 heads per group), refused on the gathered form
    mask_h = (mask + 0.5 * torch.randn(users, hq, 1, span, generator=g).to(torch.bfloat16)).to(torch.bfloat16)
    if hq // hkv > 32:
        with pytest.raises(NotImplementedError):
            torch.ops.tt.paged_scaled_dot_product_attention_decode(
                q.cuda(), kd, vd, table.cuda(), is_causal=False, attn_mask=mask_h.cuda(), cur_pos_tensor=cur.cuda())
    else:
        got_h = torch.ops.tt.paged_scaled_dot_product_attention_decode(
            q.cuda(), kd, vd, table.cuda(), is_causal=False, attn_mask=mask_h.cuda(), cur_pos_tensor=cur.cuda(),
            scale=0.11).cpu()
        want_h = O.paged_sdpa_decode(q.float(), key.float(), value.float(), table, False, mask_h.float(), cur, None, 0.11)
        err = (got_h.float() - want_h).abs().max().item()
        print(f"{name}, one mask row per head: max-abs error {err:.3e}", flush=True)
        torch.testing.assert_close(got_h.float(), want_h, atol=ATOL, rtol=RTOL)
    # table entries outside the cache (padding -1, ids past the last block) read block 0, as the
    # kernels promise; with -inf on their positions the result is that of the valid part
    bad = table.clone()
    bad[0, w - 1], bad[1, w - 2] = -1, nb + 7
    mask_b = mask.clone()
    mask_b[0, :, :, (w - 1) * bs:] = float("-inf")
    mask_b[1, :, :, (w - 2) * bs:(w - 1) * bs] = float("-inf")
    got_x = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        q.cuda(), kd, vd, bad.cuda(), is_causal=False, attn_mask=mask_b.cuda(), cur_pos_tensor=cur.cuda(),
        scale=0.11).cpu()
    want_x = O.paged_sdpa_decode(q.float(), key.float(), value.float(), table, False, mask_b.float(), cur, None, 0.11)
    torch.testing.assert_close(got_x.float(), want_x, atol=ATOL, rtol=RTOL)
