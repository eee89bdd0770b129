"""GPU parity for the block-float-8 KV variant.  The format is this build's specification
(oracle/bfp8_codec.py; PARITY UNPINNED against the reference, which holds no CPU codec):
  * codec kernels and quantising cache writes are bit-exact against the numpy codec;
  * decode attention over a block-float-8 cache is compared with the codec's round trip
    followed by fp32 attention (atol = rtol = 2e-2), K/V ~ N(0, 1) with outlier channels."""

import numpy as np
import pytest
import torch

import __graft_entry__ as entry
from oracle import bfp8_codec as C
from oracle import paged_ops as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def _bf(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


def test_empty_cache_decodes_to_zero():
    from tt_xla_amd import custom_ops as ops

    c = ops.bfp8_empty_cache(3, 2, 32, 64, "cuda")
    assert c.shape == ops.bfp8_cache_shape(3, 2, 32, 64)
    assert torch.count_nonzero(C.unpack_cache(c.cpu(), 32)) == 0
    assert torch.count_nonzero(ops.bfp8_unpack_cache(c).float()) == 0


def test_pack_unpack_kernels_bit_exact():
    from tt_xla_amd import custom_ops as ops

    g = torch.Generator().manual_seed(0)
    cache = _bf(g, 5, 3, 32, 128) * torch.logspace(-4, 4, 5).view(5, 1, 1, 1).to(torch.bfloat16)
    cache[0, 0, 3, 16:32] = 0
    cache[1, 1, 2, 5] *= 50
    want = C.pack_cache(cache)
    got = ops.bfp8_pack_cache(cache.cuda())
    assert got.shape == want.shape and torch.equal(got.cpu(), want)
    back = ops.bfp8_unpack_cache(got)
    assert torch.equal(back.cpu().float(), C.unpack_cache(want, 32))


@pytest.mark.parametrize("users,hkv,bs,d", [(8, 8, 32, 128), (5, 2, 64, 64), (16, 1, 128, 128), (6, 4, 16, 256)])
def test_update_quantises_bit_exact(users, hkv, bs, d):
    g = torch.Generator().manual_seed(users + hkv + bs)
    w = 4
    nb = users * w
    cache = _bf(g, nb, hkv, bs, d)
    fill = _bf(g, 1, users, hkv, d)
    fill[0, 0, 0, 7] *= 20
    table = torch.randperm(nb, generator=g).view(users, w).to(torch.int32)
    idx = torch.randint(0, w * bs, (users,), generator=g, dtype=torch.int32)
    want = C.pack_cache(O.paged_update_cache(cache, fill, idx, table))
    packed = C.pack_cache(cache).cuda()
    got = torch.ops.tt.paged_update_cache(packed, fill.cuda(), idx.cuda(), table.cuda())
    assert torch.equal(got.cpu(), want)
    assert torch.equal(packed.cpu(), C.pack_cache(cache))  # functional


@pytest.mark.parametrize("s", [20, 64, 150])
def test_fill_quantises_bit_exact(s):
    g = torch.Generator().manual_seed(s)
    users, hkv, bs, d = 3, 4, 32, 128
    w = (s + bs - 1) // bs + 1
    nb = users * w
    cache = _bf(g, nb, hkv, bs, d)
    key = _bf(g, users, s, hkv, d)
    table = torch.randperm(nb, generator=g).view(users, w).to(torch.int32)
    bidx = torch.tensor([1, 2, 0], dtype=torch.int32)
    want = C.pack_cache(O.paged_fill_cache_batched(cache, key.transpose(1, 2), table, bidx))
    packed = C.pack_cache(cache).cuda()
    torch.ops.tt.paged_fill_cache_(packed, key.cuda().transpose(1, 2), table.cuda(), bidx.cuda())
    assert torch.equal(packed.cpu(), want)


def _decode_vs_roundtrip(wl, name):
    from tt_xla_amd import custom_ops as ops

    g = wl.to("cuda")
    kp, vp = ops.bfp8_pack_cache(g.k_cache), ops.bfp8_pack_cache(g.v_cache)
    kp = torch.ops.tt.paged_update_cache(kp, g.k_new, g.cache_position, g.page_table)
    vp = torch.ops.tt.paged_update_cache(vp, g.v_new, g.cache_position, g.page_table)
    out = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        g.q, kp, vp, g.page_table, True, None, g.cache_position, None, wl.scale).cpu()
    bs = wl.k_cache.shape[2]
    k_rt = C.unpack_cache(kp.cpu(), bs)
    v_rt = C.unpack_cache(vp.cpu(), bs)
    want = O.textbook_decode_fp32(wl.q, k_rt, v_rt, wl.page_table, wl.cache_position, wl.scale)
    err = (out.float() - want).abs().max().item()
    print(f"{name}: max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(out.float(), want, atol=2e-2, rtol=2e-2)
    # and the quantisation itself is visible: the bf16-cache answer differs more than rounding
    return out


@pytest.mark.parametrize("users,hq,hkv,d,bs,ctx", [
    (4, 32, 8, 128, 64, [5, 64, 200, 700]),
    (3, 8, 8, 64, 32, [0, 63, 300]),
    (2, 64, 8, 128, 64, [1000, 257]),
    (3, 12, 4, 128, 16, [15, 16, 100]),
    (2, 8, 1, 128, 128, [127, 400]),
    (3, 16, 8, 256, 32, [31, 32, 700]),           # head size 256: tiles of 32 tokens
    (3, 24, 2, 256, 16, [100, 17, 450]),          # blocks smaller than a tile, 12 heads per group
    (2, 4, 4, 256, 64, [63, 500]),                # one query head per KV head
    (3, 16, 4, 64, 32, [0, 200, 2000]),           # head size 64: tiles of 128 tokens
])
def test_decode_bfp8_shapes(users, hq, hkv, d, bs, ctx):
    from tt_xla_amd import workloads

    name = f"bfp8 decode b{users} h{hq}x{hkv} d{d} bs{bs} ctx{ctx}"
    print(name, flush=True)
    nb = sum((c + 1 + bs - 1) // bs for c in ctx) + 3
    wl = workloads.decode_ragged(name, hq + d + bs, users, hq, hkv, d, bs, nb, ctx)
    workloads.add_outlier_channels(wl, 9, fraction=0.02)
    _decode_vs_roundtrip(wl, name)


def test_decode_bfp8_config5_reduced_and_property():
    """Configuration 5 at a reduced pool (the fp32 loop oracle is slow) plus the split-
    independence property on the same data."""
    from tt_xla_amd import workloads

    wl = workloads.decode_config5(users=8, num_blocks=600)
    out = _decode_vs_roundtrip(wl, wl.name + " (8 users)")
    assert torch.isfinite(out).all()


@pytest.mark.parametrize("kernel", ["valu", "mfma", "mfma16"])
@pytest.mark.parametrize("users,hq,hkv,d,bs,ctx", [
    (4, 32, 8, 128, 64, [5, 64, 200, 700]),
    (3, 12, 4, 128, 16, [15, 16, 100]),
    (3, 16, 8, 256, 32, [31, 32, 700]),           # head size 256 is built on the 16x16x32 kernel only
])
def test_decode_bfp8_every_kernel(monkeypatch, kernel, users, hq, hkv, d, bs, ctx):
    """The three main kernels that can serve a block-float-8 cache (VALU, 32x32x16 and 16x16x32
    matrix-core), each forced in turn on the same data."""
    from tt_xla_amd import workloads

    monkeypatch.setenv("TTPA_DECODE_KERNEL", kernel)
    name = f"bfp8 decode [{kernel}] b{users} h{hq}x{hkv} d{d} bs{bs} ctx{ctx}"
    print(name, flush=True)
    nb = sum((c + 1 + bs - 1) // bs for c in ctx) + 3
    wl = workloads.decode_ragged(name, hq + d + bs, users, hq, hkv, d, bs, nb, ctx)
    workloads.add_outlier_channels(wl, 9, fraction=0.02)
    _decode_vs_roundtrip(wl, name)


@pytest.mark.parametrize("kernel", ["valu", "mfma", "mfma16"])
def test_decode_bfp8_several_tiles_per_wavefront(monkeypatch, kernel):
    """A grid of one wavefront per CU over ~1000 tiles: every wavefront walks several tiles and
    crosses segment boundaries, so the running maximum, the running V exponent, the partial
    hand-over and the Q reload are all exercised."""
    from tt_xla_amd import workloads

    monkeypatch.setenv("TTPA_DECODE_KERNEL", kernel)
    monkeypatch.setenv("TTPA_DECODE_WAVES_PER_CU", "1")
    ctx = [1990, 2047, 1500, 2300]
    name = f"bfp8 decode [{kernel}] one wavefront per CU ctx{ctx}"
    print(name, flush=True)
    nb = sum((c + 1 + 63) // 64 for c in ctx) + 3
    wl = workloads.decode_ragged(name, 77, 4, 32, 8, 128, 64, nb, ctx)
    workloads.add_outlier_channels(wl, 9, fraction=0.02)
    _decode_vs_roundtrip(wl, name)


@pytest.mark.parametrize("kernel", ["mfma", "mfma16"])
def test_decode_bfp8_exponent_spread(monkeypatch, kernel):
    """K / V magnitudes that change by large powers of two from tile to tile and from group to
    group, and a large Q: the matrix-core kernels expand a tile relative to its largest
    exponent byte and carry a running exponent for the V accumulator; both have to follow."""
    from tt_xla_amd import workloads

    monkeypatch.setenv("TTPA_DECODE_KERNEL", kernel)
    monkeypatch.setenv("TTPA_DECODE_WAVES_PER_CU", "1")
    ctx = [700, 1023, 1500, 640]
    name = f"bfp8 decode [{kernel}] exponent spread ctx{ctx}"
    print(name, flush=True)
    nb = sum((c + 1 + 63) // 64 for c in ctx) + 3
    wl = workloads.decode_ragged(name, 78, 4, 32, 8, 128, 64, nb, ctx)
    g = torch.Generator().manual_seed(5)
    # per physical block (= tile) and per 16-element group a power of two
    nblk = wl.k_cache.shape[0]
    # (the 16x16x32 kernel writes a group more than 2^14 below its tile's largest as zeros, the
    # 32x32x16 kernel one more than 2^24 below: the spread inside a tile stays within 2^10 here)
    for cache, lo, hi in ((wl.k_cache, -10, -4), (wl.v_cache, -12, 2)):
        e_blk = torch.randint(lo, hi + 1, (nblk, 1, 1, 1), generator=g).float()
        e_grp = torch.randint(-10, 1, (1, cache.shape[1], 1, 8), generator=g).float()
        e_grp = e_grp.repeat_interleave(16, dim=-1)
        cache.copy_((cache.float() * torch.exp2(e_blk) * torch.exp2(e_grp)).to(torch.bfloat16))
    wl.k_cache[1] = 0  # a block of zeros
    wl.v_cache[2] = 0
    wl.q.copy_((wl.q.float() * 2.0**8).to(torch.bfloat16))
    wl.q[0, 1] *= 2.0**-30  # one user with a tiny query
    _decode_vs_roundtrip(wl, name)


def test_config5_full_size():
    """Configuration 5 at full size (32 users, 4096-block pool, block-float-8 caches), the step
    operator as bench.py runs it: every output finite; three users (the two shortest contexts and
    the longest) against the codec round trip followed by fp32 attention over just their blocks;
    the caches after the step bit for bit equal to the quantising update operator's; user
    permutation and V scaling by a power of two (which moves exponent bytes only, so it is exact in
    the cache) leave / scale the result."""
    from tt_xla_amd import custom_ops as ops
    from tt_xla_amd import workloads

    wl = workloads.decode_config5(cache_device="cuda")
    g = wl.to("cuda")
    print(wl.name, "full size", flush=True)
    kp, vp = ops.bfp8_pack_cache(g.k_cache), ops.bfp8_pack_cache(g.v_cache)
    k_ref = torch.ops.tt.paged_update_cache(kp, g.k_new, g.cache_position, g.page_table)
    v_ref = torch.ops.tt.paged_update_cache(vp, g.v_new, g.cache_position, g.page_table)

    def step(q, k_new, v_new, vcache, table, pos):
        kc, vc = kp.clone(), vcache.clone()
        out = torch.ops.tt.paged_update_kv_decode_(q, kc, vc, k_new, v_new, table, pos, scale=wl.scale)
        return out, kc, vc

    out, kc, vc = step(g.q, g.k_new, g.v_new, vp, g.page_table, g.cache_position)
    assert torch.isfinite(out.float()).all()
    assert torch.equal(kc, k_ref) and torch.equal(vc, v_ref), "caches after the step differ from the update operator's"
    bs = 64
    pos = wl.cache_position
    order = torch.argsort(pos)
    for u in order[:2].tolist() + [int(order[-1])]:
        n = int(pos[u]) + 1
        nblk = (n + bs - 1) // bs
        blocks = wl.page_table[u, :nblk].long().cuda()
        kk = C.unpack_cache(kc[blocks].cpu(), bs)    # this user's blocks, in order, dequantised
        vv = C.unpack_cache(vc[blocks].cpu(), bs)
        table = torch.arange(nblk, dtype=torch.int32).view(1, nblk)
        want = O.textbook_decode_fp32(wl.q[:, u : u + 1], kk, vv, table, pos[u : u + 1], wl.scale)
        err = (out[0, u].cpu().float() - want[0, 0]).abs().max().item()
        print(f"config5 user {u} context {n}: max-abs error {err:.3e}", flush=True)
        torch.testing.assert_close(out[0, u].cpu().float(), want[0, 0], atol=2e-2, rtol=2e-2)
    perm = torch.randperm(32, generator=torch.Generator().manual_seed(1)).cuda()
    out_p, _, _ = step(g.q[:, perm], g.k_new[:, perm], g.v_new[:, perm], vp, g.page_table[perm],
                       g.cache_position[perm])
    # another split of the work: one bfloat16 ulp (2^-7 relative; outlier channels reach 10 and more)
    torch.testing.assert_close(out_p.float(), out[:, perm].float(), atol=4e-3, rtol=8e-3)
    # V / 4: exact in the quantised cache (every exponent byte drops by 2), also for the new token
    vp_q = ops.bfp8_pack_cache((g.v_cache.float() * 0.25).to(torch.bfloat16))
    out_q, _, _ = step(g.q, g.k_new, (g.v_new.float() * 0.25).to(torch.bfloat16), vp_q, g.page_table,
                       g.cache_position)
    torch.testing.assert_close(out_q.float() * 4, out.float(), atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("users,hq,hkv,d,bs,nbpu,start,lc", [
    (2, 32, 8, 128, 32, 8, 128, 64),     # the serving default block size, a continuation chunk
    (2, 8, 8, 64, 16, 12, 0, 96),        # first chunk through the paged operator, blocks of 16
    (1, 16, 4, 128, 64, 6, 200, 128),    # a prefix that ends inside a block
    (2, 8, 2, 256, 32, 6, 64, 64),       # head size 256
    (3, 12, 4, 128, 48, 4, 100, 32),     # a block size that is no power of two
    # shapes the expansion pass serves (head size 128, four query heads per workgroup, blocks of 64 n tokens)
    (2, 32, 8, 128, 64, 6, 192, 128),
    (3, 16, 4, 128, 128, 3, 130, 200),   # a prefix that ends inside a block, rows past the last full tile
    (1, 8, 2, 128, 64, 9, 0, 300),       # first chunk: columns behind the chunk are skipped
    (2, 64, 8, 128, 64, 5, 288, 32),     # one block of rows at the end of the table
])
def test_chunked_prefill_over_a_bfp8_cache(users, hq, hkv, d, bs, nbpu, start, lc):
    """tt::chunked_scaled_dot_product_attention on block-float-8 caches (the reference's one test
    of the option is a chunked prefill, generative/test_chunked_prefill.py:86-96): against the
    oracle's chunked operator on the codec round trip of the same caches."""
    from tt_xla_amd import custom_ops as ops

    g = torch.Generator().manual_seed(users + hq + d + bs)
    nb = users * nbpu + 1
    key = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    value = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    key[:, :, :, 5] *= 20   # an outlier channel
    table = (torch.randperm(nb - 1, generator=g) + 1).view(users, nbpu).to(torch.int32)
    q = (torch.randn(users, hq, lc, d, generator=g) * 0.5).to(torch.bfloat16)
    cs = torch.tensor([start], dtype=torch.int32)
    kp, vp = ops.bfp8_pack_cache(key.cuda()), ops.bfp8_pack_cache(value.cuda())
    name = f"bfp8 chunked b{users} h{hq}x{hkv} d{d} bs{bs} start{start} lc{lc}"
    print(name, flush=True)
    got = torch.ops.tt.chunked_scaled_dot_product_attention(q.cuda(), kp, vp, table.cuda(), cs.cuda()).cpu()
    k_rt = C.unpack_cache(kp.cpu(), bs).to(torch.bfloat16)
    v_rt = C.unpack_cache(vp.cpu(), bs).to(torch.bfloat16)
    want = O.chunked_sdpa(q.float(), k_rt.float(), v_rt.float(), table, cs, None)
    err = (got.float() - want).abs().max().item()
    print(f"{name}: max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(got.float(), want, atol=2e-2, rtol=2e-2)


def test_expansion_pass_matches_tile_by_tile_expansion():
    """ttpa_sdpa_prefill_expanded with scratch (bfloat16 copies of the blocks first, then the bfloat16
    kernel) against the same entry point without (every tile expanded on its way into LDS), through
    the C ABI: the decode is exact either way, the loops round the probabilities differently.  A
    scratch one byte short is no error and takes the second route; table entries out of range read
    block 0 on both."""
    from tt_xla_amd import _native as N
    from tt_xla_amd import custom_ops as ops

    users, hq, hkv, d, bs, nbpu, start, lc = 3, 32, 8, 128, 64, 7, 256, 160
    g = torch.Generator().manual_seed(77)
    nb = users * nbpu + 1
    key = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    value = torch.randn(nb, hkv, bs, d, generator=g).to(torch.bfloat16)
    table = (torch.randperm(nb - 1, generator=g) + 1).view(users, nbpu).to(torch.int32)
    table[1, 2] = -1
    table[2, 0] = nb + 5
    q = (torch.randn(users, hq, lc, d, generator=g) * 0.5).to(torch.bfloat16).cuda()
    cs = torch.tensor([start], dtype=torch.int32).cuda()
    kp, vp = ops.bfp8_pack_cache(key.cuda()), ops.bfp8_pack_cache(value.cuda())
    tb = table.cuda()
    need = int(N.lib().ttpa_sdpa_prefill_workspace_bytes(users, hkv, d, bs, nbpu, N.KV_BFP8))
    assert need == 2 * users * nbpu * hkv * bs * d * 2 + 256
    assert N.lib().ttpa_sdpa_prefill_workspace_bytes(users, hkv, d, bs, nbpu, N.KV_BF16) == 0
    ws = torch.full((need,), 0xAB, dtype=torch.uint8, device="cuda")

    def run(ws_ptr, ws_bytes):
        out = torch.empty_like(q)
        N.call("ttpa_sdpa_prefill_expanded", out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
               q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), kp.data_ptr(), vp.data_ptr(), 0, 0, 0,
               tb.data_ptr(), tb.stride(0), cs.data_ptr(), 0, 0, 0, users, hq, hkv, lc, nbpu * bs, d, bs, nbpu, nb, 1,
               d ** -0.5, 0, N.KV_BFP8, ws_ptr, ws_bytes, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return out

    expanded = run(ws.data_ptr(), need)
    tiles = run(0, 0)
    short = run(ws.data_ptr(), need - 1)
    assert torch.equal(short, tiles)
    torch.testing.assert_close(expanded.float(), tiles.float(), atol=1e-2, rtol=1e-2)
    # the scratch holds what the pass read: the blocks of the first (start + lc) tokens of user 0, exact
    cols = (start + lc + bs - 1) // bs
    k_rt = C.unpack_cache(kp.cpu(), bs).to(torch.bfloat16)
    copies = ws[: users * nbpu * hkv * bs * d * 2].view(torch.bfloat16).view(users, nbpu, hkv, bs, d).cpu()
    for c in range(cols):
        assert torch.equal(copies[0, c], k_rt[int(table[0, c])]), f"expanded copy of column {c} differs from the codec's decode"
    assert torch.equal(copies[1, 2], k_rt[0]), "an entry out of range reads block 0"


def test_backend_flow_on_a_bfp8_cache():
    """First chunk -> continuation chunk -> decode step through TTAttentionBackendImpl.forward on
    uint8 block-float-8 caches (the flow of the reference's test of the option,
    tests/integrations/vllm_plugin/generative/test_chunked_prefill.py:69-136): the caches after
    every pass equal the quantised oracle writes bit for bit, and every output is within
    atol = rtol = 2e-2 of the oracle's operator on the codec round trip of those caches."""
    from tt_xla_amd import TTAttentionBackend, TTAttentionBackendImpl, TTMetadata
    from tt_xla_amd import custom_ops as ops

    hq, hkv, d, bs = 32, 8, 128, 32
    users, width, s1, s2 = 2, 8, 128, 64
    g = torch.Generator().manual_seed(21)
    nb = users * width + 1
    assert TTAttentionBackend.get_kv_cache_storage_shape(nb, bs, hkv, d, "bfp_bf8") == (nb, hkv, bs + bs // 16, d)
    assert TTAttentionBackend.get_kv_cache_storage_shape(nb, bs, hkv, d) == (nb, hkv, bs, d)
    table = (torch.randperm(nb - 1, generator=g) + 1).view(users, width).to(torch.int32)
    kv = [ops.bfp8_empty_cache(nb, hkv, bs, d, "cuda"), ops.bfp8_empty_cache(nb, hkv, bs, d, "cuda")]
    kc_ref = torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16)   # what the caches decode to
    vc_ref = torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16)
    impl = TTAttentionBackendImpl(hq, d, d**-0.5, hkv, None, None, "uint8")
    bidx = torch.arange(users, dtype=torch.int32)
    bf = lambda *shape: torch.randn(*shape, generator=g).to(torch.bfloat16)  # noqa: E731
    rt = lambda t: C.roundtrip(t).to(torch.bfloat16)  # noqa: E731

    def caches_match():
        assert torch.equal(kv[0].cpu(), C.pack_cache(kc_ref)) and torch.equal(kv[1].cpu(), C.pack_cache(vc_ref))

    # first chunk: quantising fills from column 0, dense causal attention on the fresh K / V
    q1, k1, v1 = bf(users * s1, hq * d), bf(users * s1, hkv * d), bf(users * s1, hkv * d)
    md = TTMetadata(cache_position=None, page_table=table.cuda(), num_users=users, batch_idx=bidx.cuda())
    out1 = torch.empty(users * s1, hq * d, dtype=torch.bfloat16, device="cuda")
    impl.forward(None, q1.cuda(), k1.cuda(), v1.cuda(), kv, md, output=out1)
    k4, v4 = k1.view(users, s1, hkv, d).transpose(1, 2), v1.view(users, s1, hkv, d).transpose(1, 2)
    kc_ref = rt(O.paged_fill_cache_batched(kc_ref, k4, table, bidx))
    vc_ref = rt(O.paged_fill_cache_batched(vc_ref, v4, table, bidx))
    caches_match()
    want1 = O.sdpa(q1.view(users, s1, hq, d).transpose(1, 2), k4, v4, None, True, d**-0.5)
    torch.testing.assert_close(out1.cpu().float(), want1.transpose(1, 2).reshape(users * s1, hq * d).float(),
                               atol=2e-2, rtol=2e-2)

    # continuation chunk: fill table rolled by the computed blocks, chunked attention over the cache
    q2, k2, v2 = bf(users * s2, hq * d), bf(users * s2, hkv * d), bf(users * s2, hkv * d)
    fill_table = torch.roll(table, -(s1 // bs), dims=1)
    start = torch.tensor([s1], dtype=torch.int32)
    md = TTMetadata(cache_position=None, page_table=table.cuda(), num_users=users, batch_idx=bidx.cuda(),
                    fill_page_table=fill_table.cuda(), chunk_start_idx=start.cuda())
    out2 = torch.empty(users * s2, hq * d, dtype=torch.bfloat16, device="cuda")
    impl.forward(None, q2.cuda(), k2.cuda(), v2.cuda(), kv, md, output=out2)
    kc_ref = rt(O.paged_fill_cache_batched(kc_ref, k2.view(users, s2, hkv, d).transpose(1, 2), fill_table, bidx))
    vc_ref = rt(O.paged_fill_cache_batched(vc_ref, v2.view(users, s2, hkv, d).transpose(1, 2), fill_table, bidx))
    caches_match()
    want2 = O.chunked_sdpa(q2.view(users, s2, hq, d).transpose(1, 2).float(), kc_ref.float(), vc_ref.float(),
                           table, start, d**-0.5)
    torch.testing.assert_close(out2.cpu().float(), want2.transpose(1, 2).reshape(users * s2, hq * d),
                               atol=2e-2, rtol=2e-2)

    # one decode token on top
    pos = torch.full((users,), s1 + s2, dtype=torch.int32)
    q3, k3, v3 = bf(users, hq * d), bf(users, hkv * d), bf(users, hkv * d)
    md = TTMetadata(cache_position=pos.cuda(), page_table=table.cuda(), num_users=users)
    out3 = torch.empty(users, hq * d, dtype=torch.bfloat16, device="cuda")
    impl.forward(None, q3.cuda(), k3.cuda(), v3.cuda(), kv, md, output=out3)
    kc_ref = rt(O.paged_update_cache(kc_ref, k3.view(users, 1, hkv, d).transpose(0, 1), pos, table))
    vc_ref = rt(O.paged_update_cache(vc_ref, v3.view(users, 1, hkv, d).transpose(0, 1), pos, table))
    caches_match()
    want3 = O.textbook_decode_fp32(q3.view(users, 1, hq, d).transpose(0, 1), kc_ref, vc_ref, table, pos, d**-0.5)
    torch.testing.assert_close(out3.cpu().float(), want3.transpose(0, 1).reshape(users, hq * d),
                               atol=2e-2, rtol=2e-2)

    # a KV-shared layer's prefill gathers (and dequantises) the same caches
    shared = TTAttentionBackendImpl(hq, d, d**-0.5, hkv, None, None, "uint8", kv_sharing_target_layer_name="l0")
    s = s1 + s2
    q4 = bf(users * 64, hq * d)
    md = TTMetadata(cache_position=None, page_table=table.cuda(), num_users=users, batch_idx=bidx.cuda())
    out4 = torch.empty(users * 64, hq * d, dtype=torch.bfloat16, device="cuda")
    shared.forward(None, q4.cuda(), k2.cuda(), v2.cuda(), kv, md, output=out4)
    caches_match()
    k_d = O.gather_paged_to_dense(kc_ref, table)[:, :, :64]
    v_d = O.gather_paged_to_dense(vc_ref, table)[:, :, :64]
    want4 = O.sdpa(q4.view(users, 64, hq, d).transpose(1, 2), k_d, v_d, None, True, d**-0.5)
    torch.testing.assert_close(out4.cpu().float(), want4.transpose(1, 2).reshape(users * 64, hq * d).float(),
                               atol=2e-2, rtol=2e-2)
