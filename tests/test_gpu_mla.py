"""GPU parity of the latent-attention operators (tt::paged_flash_mla_decode,
tt::flash_mla_prefill; reference custom_ops.py:223-632) against the oracle's restatement of
their CPU branches, on the reference's own parameter grid (tests/torch/ops/test_custom_ops.py:
233-248, 286-303) plus the 576 / 512 latent shape of the serving backend
(vllm_tt/attention_impls/attention_mla.py:184-422).  Tolerance atol = rtol = 2e-2."""

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


def _bf(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


def _check(name, got, want):
    err = (got.float() - want.float()).abs().max().item()
    print(f"{name}: max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(got.float(), want.float(), atol=ATOL, rtol=RTOL)


DECODE = [
    # users, heads, kv_heads, head_size, head_dim_v, has_value, block_size, blocks_per_seq, scale
    (8, 16, 1, 192, 128, False, 32, 16, 1.0),     # reference grid
    (8, 16, 1, 192, 128, False, 64, 16, 1.0),
    (8, 32, 1, 128, 128, False, 32, 16, 1.0),
    (8, 16, 1, 128, 64, True, 32, 16, 1.0),
    (8, 16, 4, 192, 128, False, 32, 16, 1.0),
    (8, 8, 8, 128, 128, True, 32, 16, 1.0),
    (4, 16, 1, 576, 512, False, 32, 24, None),    # latent serving shape, 16 heads per rank
    (3, 128, 1, 576, 512, False, 64, 12, None),   # all 128 heads of the layer
    (2, 64, 2, 192, 128, False, 16, 40, 0.11),
    (3, 16, 1, 576, 384, False, 32, 12, None),    # a value width that is not a power of two (merge kernel)
    (2, 48, 1, 192, 128, False, 32, 6, 0.2),      # two of the four wavefronts of the 128-head form have heads, one of them 16
    (2, 40, 2, 128, 128, False, 16, 20, 0.2),     # 20 heads per KV head: a row block with four heads
    (2, 256, 1, 576, 512, False, 64, 6, None),    # two segments of 128 heads per user
    (6, 128, 1, 576, 384, False, 128, 5, None),   # blocks of two tiles
]


@pytest.mark.parametrize("users,hq,nkv,dh,dv,has_value,bs,width,scale", DECODE)
def test_paged_flash_mla_decode(users, hq, nkv, dh, dv, has_value, bs, width, scale):
    print(f"case: mla decode u{users} h{hq}x{nkv} dh{dh} dv{dv} value={has_value} bs{bs} w{width}", flush=True)
    g = torch.Generator().manual_seed(users * dh + hq + bs)
    nb = width * users
    # unit-variance scores at scale 1.0 would make softmax one-hot; keep the reference's scale
    # but shrink q so that many positions carry weight
    q = (_bf(g, 1, users, hq, dh).float() * (0.15 if scale == 1.0 else 1.0)).to(torch.bfloat16)
    key = _bf(g, nb, nkv, bs, dh)
    value = _bf(g, nb, nkv, bs, dv) if has_value else None
    table = torch.randperm(nb, generator=g).view(users, width).to(torch.int32)
    pos = torch.randint(0, width * bs, (users,), generator=g, dtype=torch.int32)
    pos[0], pos[-1] = 0, width * bs - 1
    got = torch.ops.tt.paged_flash_mla_decode(
        q.cuda(), key.cuda(), dv, table.cuda(), value.cuda() if has_value else None, True, None,
        pos.cuda(), None, scale).cpu()
    assert got.shape == (1, users, hq, dv)
    want = O.paged_flash_mla_decode(q, key, dv, table, value, pos, scale)
    _check(f"mla decode u{users} h{hq}x{nkv} dh{dh} dv{dv} bs{bs}", got, want)


@pytest.mark.parametrize("partials", ["f32", "bf16"])
@pytest.mark.parametrize("dv", [512, 384])
def test_mla_decode_16_heads_either_partial_format(monkeypatch, partials, dv):
    """The 16-head latent kernel hands its partial outputs to the merge as bfloat16 by default and
    as floats under TTPA_LATENT_PARTIALS=f32: both against the oracle, on a small grid (a quarter
    wavefront per CU) so that every user's context is cut into several partials."""
    monkeypatch.setenv("TTPA_LATENT_PARTIALS", partials)
    monkeypatch.setenv("TTPA_DECODE_WAVES_PER_CU", "0.25")
    users, hq, dh, bs, width = 5, 16, 576, 32, 40
    print(f"case: mla decode partials={partials} u{users} h{hq} dh{dh} dv{dv} bs{bs} w{width}", flush=True)
    g = torch.Generator().manual_seed(1000 + dv)
    nb = width * users
    q = _bf(g, 1, users, hq, dh)
    key = _bf(g, nb, 1, bs, dh)
    table = torch.randperm(nb, generator=g).view(users, width).to(torch.int32)
    pos = torch.tensor([width * bs - 1, 700, 5, 1279, 64], dtype=torch.int32)
    got = torch.ops.tt.paged_flash_mla_decode(q.cuda(), key.cuda(), dv, table.cuda(), None, True, None,
                                              pos.cuda(), None, None).cpu()
    want = O.paged_flash_mla_decode(q, key, dv, table, None, pos, None)
    _check(f"mla decode partials={partials} dv{dv}", got, want)


@pytest.mark.parametrize("kernel,partials", [("", "bf16"), ("", "f32"), ("wide", "f32")])
def test_mla_decode_128_heads_every_form(monkeypatch, kernel, partials):
    """All 128 heads of a latent layer on one GPU: the form in which four wavefronts of a workgroup take
    32 heads each on shared K, with bfloat16 and with float partials, and the older form it
    replaced (TTPA_LATENT_KERNEL=wide: blocks of 32 heads, every score computed four times), which still
    serves masks and a separate V.  Contexts from one token to several tiles per workgroup range."""
    monkeypatch.setenv("TTPA_LATENT_PARTIALS", partials)
    if kernel:
        monkeypatch.setenv("TTPA_LATENT_KERNEL", kernel)
    else:
        monkeypatch.delenv("TTPA_LATENT_KERNEL", raising=False)
    users, hq, dh, dv, bs, width = 6, 128, 576, 512, 64, 400
    print(f"case: mla decode 128 heads kernel={kernel or 'default'} partials={partials}", flush=True)
    g = torch.Generator().manual_seed(4242)
    pos = torch.tensor([0, 63, 64, 1000, 25599, 12345], dtype=torch.int32)
    blocks = [int(p) // bs + 1 for p in pos]
    nb = sum(blocks) + 1
    q = _bf(g, 1, users, hq, dh)
    key = _bf(g, nb, 1, bs, dh)
    table = torch.zeros(users, width, dtype=torch.int32)
    perm = (torch.randperm(nb - 1, generator=g) + 1).to(torch.int32)
    at = 0
    for u, nblk in enumerate(blocks):
        table[u, :nblk] = perm[at : at + nblk]
        at += nblk
    got = torch.ops.tt.paged_flash_mla_decode(q.cuda(), key.cuda(), dv, table.cuda(), None, True, None,
                                              pos.cuda(), None, None).cpu()
    want = O.paged_flash_mla_decode(q, key, dv, table, None, pos, None)
    _check(f"mla decode 128 heads kernel={kernel or 'default'} partials={partials}", got, want)


@pytest.mark.parametrize("hq", [16, 128])
@pytest.mark.parametrize("pad", [8, 2, 1])
def test_mla_decode_output_rows_by_strides(monkeypatch, hq, pad):
    """The output is addressed by strides (ttpa_paged_mla_decode): rows that start on 16-byte boundaries
    take the merge with 16 bytes per thread (pad 8), rows on 4-byte boundaries the one with 4 (pad 2),
    and rows on odd element offsets the float partials (pad 1).  A small grid cuts every user's context
    into several partials."""
    from tt_xla_amd import custom_ops as C

    monkeypatch.setenv("TTPA_DECODE_WAVES_PER_CU", "0.25")
    users, dh, dv, bs, width = 3, 576, 512, 64, 24
    print(f"case: mla decode strided output h{hq} pad{pad}", flush=True)
    g = torch.Generator().manual_seed(31 * hq + pad)
    nb = users * width
    q = _bf(g, 1, users, hq, dh)
    key = _bf(g, nb, 1, bs, dh)
    table = torch.randperm(nb, generator=g).view(users, width).to(torch.int32)
    pos = torch.tensor([width * bs - 1, 130, 900], dtype=torch.int32)
    buf = torch.full((users, hq, dv + pad), 7.0, dtype=torch.bfloat16, device="cuda")
    out = buf[:, :, :dv]
    C._mla_decode_launch(out, q[0].cuda(), key.cuda(), None, table.cuda(), pos.cuda(), dv, 1.0 / math.sqrt(dh), None)
    torch.cuda.synchronize()
    want = O.paged_flash_mla_decode(q, key, dv, table, None, pos, None)
    _check(f"mla decode strided output h{hq} pad{pad}", out.cpu(), want[0])
    assert (buf[:, :, dv:] == 7.0).all(), "the columns behind a row stay as they were"


def test_mla_decode_128_heads_negative_scale():
    """scale < 0: the softmax between the matrix instructions assumes a positive scale, so every step
    must take the other one."""
    users, hq, dh, dv, bs, width = 2, 128, 576, 512, 64, 8
    g = torch.Generator().manual_seed(99)
    nb = users * width
    q = (_bf(g, 1, users, hq, dh).float() * 0.2).to(torch.bfloat16)
    key = _bf(g, nb, 1, bs, dh)
    table = torch.randperm(nb, generator=g).view(users, width).to(torch.int32)
    pos = torch.tensor([500, 77], dtype=torch.int32)
    got = torch.ops.tt.paged_flash_mla_decode(q.cuda(), key.cuda(), dv, table.cuda(), None, True, None,
                                              pos.cuda(), None, -0.5).cpu()
    want = O.paged_flash_mla_decode(q, key, dv, table, None, pos, -0.5)
    _check("mla decode 128 heads, negative scale", got, want)


def test_mla_decode_padded_row_sink_and_errors():
    g = torch.Generator().manual_seed(3)
    users, hq, dh, dv, bs, width = 3, 16, 576, 512, 32, 8
    nb = users * width
    q, key = _bf(g, 1, users, hq, dh), _bf(g, nb, 1, bs, dh)
    table = torch.randperm(nb, generator=g).view(users, width).to(torch.int32)
    pos = torch.tensor([100, -1, 255], dtype=torch.int32)
    sink = torch.linspace(-2, 2, hq)
    got = torch.ops.tt.paged_flash_mla_decode(q.cuda(), key.cuda(), dv, table.cuda(), None, True, None,
                                              pos.cuda(), sink.cuda(), None).cpu()
    assert torch.isnan(got[0, 1].float()).all()
    # sink: closed form against the sink-free oracle, out * sigmoid(logsumexp - sink)
    base = O.paged_flash_mla_decode(q, key, dv, table, None, pos.clamp(min=0), None).float()
    for u in (0, 2):
        idx = torch.arange(int(pos[u]) + 1)
        kk = key[table[u, idx // bs].long(), 0, idx % bs].float()
        lse = torch.logsumexp((q[0, u].float() @ kk.T) / math.sqrt(dh), dim=-1)  # [hq]
        want = base[0, u] * torch.sigmoid(lse - sink).unsqueeze(-1)
        torch.testing.assert_close(got[0, u].float(), want, atol=ATOL, rtol=RTOL)
    with pytest.raises(AssertionError):
        torch.ops.tt.paged_flash_mla_decode(q.cuda(), key.cuda(), 600, table.cuda(), None, True, None,
                                            pos.cuda(), None, None)


PREFILL = [
    # batch, heads, seq, head_size, kv_heads, head_dim_v, has_value
    (1, 16, 64, 192, 1, 128, False),   # reference grid (causal rows)
    (2, 16, 128, 192, 1, 128, False),
    (1, 32, 64, 128, 1, 128, False),
    (1, 16, 64, 128, 1, 64, True),
    (2, 16, 256, 576, 1, 512, False),  # latent serving shape
    (1, 8, 1184, 192, 1, 128, False),  # more query rows than one launch of the decode kernels takes
    (1, 16, 2048, 576, 1, 512, False), # a full prompt at the latent serving shape
    (1, 128, 64, 576, 1, 512, False),  # the unsharded layer: 128 heads, a workgroup per token
    (1, 12, 96, 192, 1, 128, False),   # 12 heads: a wavefront's 16 rows straddle two tokens
    (2, 8, 160, 128, 2, 128, False),   # two KV heads, a last row block of 4 heads x 8 tokens short of 128 rows
    (1, 4, 32, 576, 1, 512, False),    # 128 rows in all: one workgroup
]


@pytest.mark.parametrize("b,hq,s,dh,nkv,dv,has_value", PREFILL)
def test_flash_mla_prefill(b, hq, s, dh, nkv, dv, has_value):
    print(f"case: mla prefill b{b} h{hq} s{s} dh{dh} kv{nkv} dv{dv} value={has_value}", flush=True)
    g = torch.Generator().manual_seed(s + dh + hq)
    q = (_bf(g, b, hq, s, dh).float() * 0.15).to(torch.bfloat16)
    k = _bf(g, b, nkv, s, dh)
    v = _bf(g, b, nkv, s, dv) if has_value else None
    got = torch.ops.tt.flash_mla_prefill(q.cuda(), k.cuda(), dv, v.cuda() if has_value else None, None, True, 1.0).cpu()
    assert got.shape == (b, hq, s, dv)
    want = O.flash_mla_prefill(q.float(), k.float(), dv, None if v is None else v.float(), None, True, 1.0)
    _check(f"mla prefill b{b} h{hq} s{s} dh{dh} dv{dv}", got, want)


@pytest.mark.parametrize("b,hq,s,dh,nkv,dv,causal", [
    (1, 16, 224, 576, 1, 512, False),   # every key for every row: all steps but a wavefront's first take the softmax
    (2, 16, 96, 192, 1, 128, False),    # that sits between the matrix instructions
    (1, 32, 96, 128, 1, 128, False),
    (1, 16, 100, 576, 1, 512, False),   # a sequence that ends inside a step of 32 keys (the operator asks for multiples
    (1, 16, 100, 576, 1, 512, True),    # of 32, the library does not): rows past the end are requested as the last one
    (2, 8, 44, 192, 1, 128, True),
])
def test_flash_mla_prefill_through_the_library(b, hq, s, dh, nkv, dv, causal):
    """The operator accepts is_causal=False only together with a mask and sequence lengths that are multiples of 32
    (reference custom_ops.py:723-726, :238); the library entry point below it takes neither restriction: called
    directly.  Without a mask and without a causal limit, the masked softmax of the kernel is left to a
    wavefront's first step."""
    from tt_xla_amd import _native as N

    print(f"case: mla prefill through the library b{b} h{hq} s{s} dh{dh} dv{dv} causal={causal}", flush=True)
    g = torch.Generator().manual_seed(7 * s + dh + int(causal))
    q = (_bf(g, b, hq, s, dh).float() * 0.15).to(torch.bfloat16)
    k = _bf(g, b, nkv, s, dh)
    qd, kd = q.cuda(), k.cuda()
    out = torch.empty(b, hq, s, dv, dtype=torch.bfloat16, device="cuda")
    N.call(
        "ttpa_latent_prefill",
        out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
        qd.data_ptr(), qd.stride(0), qd.stride(1), qd.stride(2),
        kd.data_ptr(), kd.stride(0), kd.stride(1), kd.stride(2),
        0, 0, 0, 0, b, hq, nkv, s, dh, dv, int(causal), 1.0, torch.cuda.current_stream().cuda_stream,
    )
    torch.cuda.synchronize()
    want = O.flash_mla_prefill(q.float(), k.float(), dv, None, None, causal, 1.0)
    _check(f"mla prefill through the library s{s} dh{dh} dv{dv} causal={causal}", out.cpu(), want)


MASKED_PREFILL = [
    # batch, heads, seq, head_size, kv_heads, head_dim_v, has_value: the is_causal=False rows of the
    # reference grid (tests/torch/ops/test_custom_ops.py:236-248), one mask [b, 1, s, s] for all heads
    (1, 16, 64, 192, 1, 128, False),
    (2, 16, 128, 192, 1, 128, False),
    (1, 32, 64, 128, 1, 128, False),
    (2, 16, 128, 128, 1, 64, True),
    (1, 16, 96, 576, 1, 512, False),   # latent serving shape
    (1, 12, 160, 192, 1, 128, False),  # rows of two tokens in one wavefront, each with its own mask row
]


@pytest.mark.parametrize("per_head", [False, True])
@pytest.mark.parametrize("b,hq,s,dh,nkv,dv,has_value", MASKED_PREFILL)
def test_flash_mla_prefill_with_mask(b, hq, s, dh, nkv, dv, has_value, per_head):
    print(f"case: masked mla prefill b{b} h{hq} s{s} dh{dh} kv{nkv} dv{dv} value={has_value} per_head={per_head}", flush=True)
    g = torch.Generator().manual_seed(s + dh + hq + 1)
    q = (_bf(g, b, hq, s, dh).float() * 0.15).to(torch.bfloat16)
    k = _bf(g, b, nkv, s, dh)
    v = _bf(g, b, nkv, s, dv) if has_value else None
    mask = _bf(g, b, hq if per_head else 1, s, s)
    keep = torch.rand(b, 1, s, s, generator=g) > 0.3
    keep[..., 0] = True
    mask = mask.masked_fill(~keep, float("-inf"))
    got = torch.ops.tt.flash_mla_prefill(q.cuda(), k.cuda(), dv, v.cuda() if has_value else None, mask.cuda(), False, 1.0).cpu()
    assert got.shape == (b, hq, s, dv)
    want = O.flash_mla_prefill(q.float(), k.float(), dv, None if v is None else v.float(), mask.float(), False, 1.0)
    _check(f"masked mla prefill b{b} h{hq} s{s} dh{dh} dv{dv}", got, want)


@pytest.mark.parametrize("users,hq,nkv,dh,dv,has_value,bs,width,scale", [
    (8, 16, 1, 192, 128, False, 32, 16, 1.0), (8, 32, 1, 128, 128, False, 32, 16, 1.0),
    (8, 16, 1, 128, 64, True, 32, 16, 1.0), (8, 16, 4, 192, 128, False, 32, 16, 1.0),
    (4, 16, 1, 576, 512, False, 32, 24, None), (3, 128, 1, 576, 512, False, 64, 12, None),
])
def test_paged_flash_mla_decode_with_mask(users, hq, nkv, dh, dv, has_value, bs, width, scale):
    """is_causal=False (reference custom_ops.py:590-592): every position of the table, weighted by
    attn_mask; one row for all heads and one row per head."""
    g = torch.Generator().manual_seed(users * dh + hq + bs + 5)
    nb = width * users
    q = (_bf(g, 1, users, hq, dh).float() * (0.15 if scale == 1.0 else 1.0)).to(torch.bfloat16)
    key = _bf(g, nb, nkv, bs, dh)
    value = _bf(g, nb, nkv, bs, dv) if has_value else None
    table = torch.randperm(nb, generator=g).view(users, width).to(torch.int32)
    span = width * bs
    for per_head in (False, True):
        print(f"case: masked mla decode u{users} h{hq}x{nkv} dh{dh} dv{dv} bs{bs} w{width} per_head={per_head}", flush=True)
        mask = _bf(g, users, hq if per_head else 1, 1, span)
        keep = torch.rand(users, 1, 1, span, generator=g) > 0.4
        keep[..., 0] = True
        mask = mask.masked_fill(~keep, float("-inf"))
        got = torch.ops.tt.paged_flash_mla_decode(
            q.cuda(), key.cuda(), dv, table.cuda(), value.cuda() if has_value else None, False, mask.cuda(),
            None, None, scale).cpu()
        assert got.shape == (1, users, hq, dv)
        want = O.paged_flash_mla_decode(q.float(), key.float(), dv, table, None if value is None else value.float(),
                                        None, scale, mask.float())
        _check(f"masked mla decode u{users} h{hq}x{nkv} dh{dh} dv{dv} per_head={per_head}", got, want)


def test_mla_backend_prefill_then_decode():
    """The serving backend (tt_xla_amd/attention_mla.py) end to end on the device at the
    576 / 512 latent shape: prefill of 64 tokens per user (a token bucket: the operator takes multiples of 32), one decode step, output against a
    dense fp32 computation and the latent cache position by position (the checks of
    tests/integrations/vllm_plugin/oot_backends/test_mla_attention_impl.py:202-218, 317-333)."""
    import types

    from tt_xla_amd import attention_mla as M
    from tt_xla_amd.attention import TTMetadata

    n, p, r, lat, v, bs = 16, 128, 64, 512, 128, 32
    users, s, nb, w = 2, 64, 12, 3
    g = torch.Generator().manual_seed(7)
    layer = types.SimpleNamespace(W_UK_T=(_bf(g, n, p, lat) / math.sqrt(p)).cuda(),
                                  W_UV=(_bf(g, n, lat, v) / math.sqrt(lat)).cuda())
    impl = M.TTMLAAttentionBackendImpl(
        num_heads=n, head_size=lat + r, scale=1.0 / math.sqrt(p + r), num_kv_heads=1,
        alibi_slopes=None, sliding_window=None, kv_cache_dtype="auto", logits_soft_cap=None,
        attn_type="decoder", kv_sharing_target_layer_name=None, kv_lora_rank=lat,
        qk_nope_head_dim=p, qk_rope_head_dim=r, qk_head_dim=p + r, v_head_dim=v)
    table = (torch.randperm(nb - 1, generator=g)[: users * w] + 1).view(users, w).to(torch.int32)
    cache = torch.zeros(nb, 1, bs, lat + r, dtype=torch.bfloat16, device="cuda")

    def dense(q_nope, q_pe, ctx, positions):
        q_lat = torch.cat([torch.einsum("bsnp,npl->bsnl", q_nope.float(), layer.W_UK_T.cpu().float())
                           .to(torch.bfloat16).float(), q_pe.float()], dim=-1)
        out = torch.zeros(q_nope.shape[0], q_nope.shape[1], n, v)
        for u in range(q_nope.shape[0]):
            for i in range(q_nope.shape[1]):
                keys = ctx[u, : int(positions[u, i]) + 1].float()
                wts = torch.softmax(q_lat[u, i] @ keys.T * impl.scale, dim=-1)
                out[u, i] = torch.einsum("nl,nlv->nv", wts @ keys[:, :lat], layer.W_UV.cpu().float())
        return out.reshape(-1, n * v)

    q_nope, q_pe = _bf(g, users * s, n, p), _bf(g, users * s, n, r)
    kv_c, k_pe = _bf(g, users * s, lat), _bf(g, users * s, 1, r)
    meta = TTMetadata(cache_position=torch.full((users,), s - 1, dtype=torch.int32).cuda(),
                      page_table=table.cuda(), fill_page_table=table.cuda(), is_causal=True)
    out = torch.empty(users * s, n * v, dtype=torch.bfloat16, device="cuda")
    impl.forward((q_nope.cuda(), q_pe.cuda()), kv_c.cuda(), k_pe.cuda(), cache, meta, layer, output=out)
    k_lat = torch.cat([kv_c.view(users, s, lat), k_pe.view(users, s, r)], dim=-1)
    _check("mla backend prefill", out.cpu(),
           dense(q_nope.view(users, s, n, p), q_pe.view(users, s, n, r), k_lat,
                 torch.arange(s).expand(users, s)))
    host = cache.cpu()
    for u in range(users):
        for pos in range(s):
            assert torch.equal(host[table[u, pos // bs], 0, pos % bs], k_lat[u, pos])

    q1, qp1 = _bf(g, users, n, p), _bf(g, users, n, r)
    c1, kp1 = _bf(g, users, lat), _bf(g, users, 1, r)
    meta1 = TTMetadata(cache_position=torch.full((users,), s, dtype=torch.int32).cuda(),
                       page_table=table.cuda(), is_causal=True)
    out1 = torch.empty(users, n * v, dtype=torch.bfloat16, device="cuda")
    impl.forward((q1.cuda(), qp1.cuda()), c1.cuda(), kp1.cuda(), cache, meta1, layer, output=out1)
    k_new = torch.cat([c1, kp1.view(users, r)], dim=-1)
    ctx = torch.cat([k_lat, k_new.view(users, 1, lat + r)], dim=1)
    _check("mla backend decode", out1.cpu(),
           dense(q1.view(users, 1, n, p), qp1.view(users, 1, n, r), ctx, torch.full((users, 1), s)))
    host = cache.cpu()
    for u in range(users):
        assert torch.equal(host[table[u, s // bs], 0, s % bs], k_new[u])
