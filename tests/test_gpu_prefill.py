"""GPU parity for the prefill operators (bf16 MFMA kernel behind the C ABI) against the CPU
oracle on the same seeded inputs: tt::scaled_dot_product_attention (dense, grouped heads,
causal or additive mask) and tt::chunked_scaled_dot_product_attention (paged K/V with a
cached prefix).  Cases follow tests/torch/ops/test_custom_ops.py:52-95 and
tests/torch/ops/test_chunked_sdpa_op_cpu.py:58-147 (there in fp32 at 1e-4; here the inputs
are bfloat16 and the bar is atol = rtol = 2e-2)."""

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


def _check(name, got, want):
    err = (got.float() - want.float()).abs().max().item()
    print(f"{name}: max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(got.float(), want.float(), atol=ATOL, rtol=RTOL)


def _bf(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


DENSE = [
    # batch, Hq, S, D, Hkv, Skv, causal  (first eight: the reference's own grid)
    (1, 12, 32, 128, 12, 32, True), (1, 12, 32, 128, 12, 128, False),
    (8, 12, 32, 128, 12, 32, True), (8, 12, 32, 128, 12, 128, False),
    (1, 12, 32, 128, 4, 32, True), (1, 12, 32, 128, 4, 128, False),
    (8, 12, 32, 128, 4, 32, True), (8, 12, 32, 128, 4, 128, False),
    (2, 32, 512, 128, 8, 512, True), (1, 8, 256, 64, 8, 256, True),
    (1, 8, 96, 64, 2, 96, True), (1, 16, 128, 256, 8, 128, True),
    (2, 4, 64, 128, 4, 200, False), (1, 64, 160, 128, 8, 160, True),
]


@pytest.mark.parametrize("b,hq,s,d,hkv,skv,causal", DENSE)
def test_dense_sdpa(b, hq, s, d, hkv, skv, causal):
    name = f"sdpa b{b} h{hq}x{hkv} s{s} skv{skv} d{d} causal={causal}"
    print(name, flush=True)
    g = torch.Generator().manual_seed(b + hq + s + d + skv)
    q, k, v = _bf(g, b, hq, s, d), _bf(g, b, hkv, skv, d), _bf(g, b, hkv, skv, d)
    mask = None if causal else _bf(g, b, 1, s, skv)
    scale = 1.0 if s == 32 else None
    want = O.sdpa(q, k, v, mask, causal, scale)
    got = torch.ops.tt.scaled_dot_product_attention(
        q.cuda(), k.cuda(), v.cuda(), None if mask is None else mask.cuda(), causal, scale)
    assert got.shape == q.shape and got.dtype == torch.bfloat16
    _check(name, got.cpu(), want)


def test_dense_sdpa_backend_views():
    """q / k / v arrive as transpose(-3, -2) of [users, tokens, heads, D] (attention.py:575-579)."""
    g = torch.Generator().manual_seed(7)
    users, s, hq, hkv, d = 2, 128, 32, 8, 128
    q, k, v = _bf(g, users, s, hq, d), _bf(g, users, s, hkv, d), _bf(g, users, s, hkv, d)
    want = O.sdpa(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, True, None)
    got = torch.ops.tt.scaled_dot_product_attention(
        q.cuda().transpose(1, 2), k.cuda().transpose(1, 2), v.cuda().transpose(1, 2), None, True, None)
    _check("backend views", got.cpu(), want)
    # the result keeps the token-major memory of its query, so the transpose back is free
    assert got.transpose(1, 2).is_contiguous()


def test_dense_sdpa_argument_checks():
    q = torch.zeros(1, 4, 31, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(AssertionError):
        torch.ops.tt.scaled_dot_product_attention(q, q, q)
    q = torch.zeros(1, 6, 32, 64, dtype=torch.bfloat16, device="cuda")
    k = torch.zeros(1, 4, 32, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(AssertionError):
        torch.ops.tt.scaled_dot_product_attention(q, k, k)


def _paged(gen, users, nbpu, hkv, bs, d, scramble):
    nb = users * nbpu + 1
    key, value = _bf(gen, nb, hkv, bs, d), _bf(gen, nb, hkv, bs, d)
    if scramble:
        table = (torch.randperm(nb - 1, generator=gen)[: users * nbpu] + 1).view(users, nbpu)
    else:
        table = torch.arange(users * nbpu).view(users, nbpu)
    return key, value, table.to(torch.int32)


@pytest.mark.parametrize("hq,hkv", [(8, 8), (8, 2), (32, 8)])
@pytest.mark.parametrize("start", [0, 64, 96])
def test_chunked_reference_cases(hq, hkv, start):
    g = torch.Generator().manual_seed(hq * 100 + start)
    d, bs, nbpu, users = 64, 32, 4, 2
    lc = nbpu * bs - start
    key, value, table = _paged(g, users, nbpu, hkv, bs, d, False)
    q = _bf(g, users, hq, lc, d)
    st = torch.tensor([start], dtype=torch.int32)
    want = O.chunked_sdpa(q, key, value, table, st, 1.0 / d**0.5)
    got = torch.ops.tt.chunked_scaled_dot_product_attention(
        q.cuda(), key.cuda(), value.cuda(), table.cuda(), st.cuda(), 1.0 / d**0.5)
    _check(f"chunked h{hq}x{hkv} start{start}", got.cpu(), want)


@pytest.mark.parametrize("users,hq,hkv,d,bs,nbpu,start,lc", [
    (2, 8, 2, 64, 32, 4, 64, 1),          # one-token remainder
    (1, 4, 4, 64, 32, 2, 0, 64),          # start 0 == plain causal
    (2, 32, 8, 128, 64, 8, 256, 256),     # Llama-3-8B heads, block 64
    (3, 32, 8, 128, 32, 16, 128, 50),     # ragged chunk length, block 32
    (2, 64, 8, 128, 64, 6, 192, 192),
    (1, 16, 8, 256, 64, 4, 64, 96),
    (2, 12, 4, 128, 16, 12, 96, 96),
    (2, 8, 2, 64, 4, 40, 32, 100),        # block smaller than the rows of one load: per-lane lookups
    (1, 4, 4, 128, 2, 100, 64, 70),
    (2, 16, 8, 256, 8, 30, 32, 150),      # head size 256, block of 8: one lookup per load
    (2, 8, 8, 64, 8, 40, 96, 130),        # head size 64, block of exactly one load
    (2, 16, 4, 128, 48, 6, 96, 100),      # block sizes that are not powers of two (multiply-high quotients)
    (2, 8, 2, 128, 20, 12, 64, 70),
    (1, 8, 8, 64, 24, 10, 32, 150),
])
def test_chunked_shapes(users, hq, hkv, d, bs, nbpu, start, lc):
    name = f"chunked u{users} h{hq}x{hkv} d{d} bs{bs} w{nbpu} start{start} lc{lc}"
    print(name, flush=True)
    g = torch.Generator().manual_seed(users + hq + d + bs + start + lc)
    key, value, table = _paged(g, users, nbpu, hkv, bs, d, True)
    q = _bf(g, users, hq, lc, d)
    st = torch.tensor([start], dtype=torch.int32)
    want = O.chunked_sdpa(q, key, value, table, st)
    got = torch.ops.tt.chunked_scaled_dot_product_attention(
        q.cuda(), key.cuda(), value.cuda(), table.cuda(), st.cuda())
    _check(name, got.cpu(), want)


def test_chunked_start0_equals_dense_causal_on_filled_cache():
    """Fill the cache from dense K/V through the fill op, then the paged op with start 0 must
    agree with the dense op on the fresh K/V (the two prefill routes of the backend)."""
    g = torch.Generator().manual_seed(3)
    users, s, hq, hkv, d, bs = 2, 256, 32, 8, 128, 64
    q, k, v = _bf(g, users, hq, s, d), _bf(g, users, hkv, s, d), _bf(g, users, hkv, s, d)
    nb = users * (s // bs) + 1
    table = (torch.randperm(nb - 1, generator=g) + 1).view(users, s // bs).to(torch.int32).cuda()
    kc = torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros_like(kc)
    idx = torch.arange(users, dtype=torch.int32, device="cuda")
    torch.ops.tt.paged_fill_cache_(kc, k.cuda(), table, idx)
    torch.ops.tt.paged_fill_cache_(vc, v.cuda(), table, idx)
    a = torch.ops.tt.chunked_scaled_dot_product_attention(
        q.cuda(), kc, vc, table, torch.zeros(1, dtype=torch.int32, device="cuda"))
    bb = torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda())
    torch.testing.assert_close(a.float(), bb.float(), atol=4e-3, rtol=4e-3)
    _check("filled-cache vs oracle", a.cpu(), O.sdpa(q, k, v))


def test_inputs_the_kernels_cannot_take_are_refused():
    """A boolean mask means "attend where True" (the library routine's rule); float16 / float32
    keys and values, a float16 cache under attention and a scale that is not positive raise
    instead of being reinterpreted."""
    g = torch.Generator().manual_seed(9)
    b, hq, hkv, s, d = 2, 8, 4, 64, 64
    q = torch.randn(b, hq, s, d, generator=g).to(torch.bfloat16)
    k = torch.randn(b, hkv, s, d, generator=g).to(torch.bfloat16)
    v = torch.randn(b, hkv, s, d, generator=g).to(torch.bfloat16)
    keep = torch.rand(b, 1, s, s, generator=g) > 0.5
    keep[:, :, :, 0] = True
    got = torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), attn_mask=keep.cuda(),
                                                    is_causal=False).cpu()
    want = O.sdpa(q.float(), k.float(), v.float(), keep, False, None)
    torch.testing.assert_close(got.float(), want, atol=2e-2, rtol=2e-2)
    with pytest.raises(ValueError, match="bfloat16"):
        torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda().half(), v.cuda().half())
    with pytest.raises(ValueError, match="bfloat16"):
        torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda().float(), v.cuda().float())
    with pytest.raises(ValueError, match="positive"):
        torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), scale=0.0)
    with pytest.raises(ValueError, match="positive"):
        torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), scale=-0.125)
    cache = torch.zeros(4, hkv, 32, d, dtype=torch.float16, device="cuda")
    table = torch.zeros(b, 2, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError, match="bfloat16 or block-float-8"):
        torch.ops.tt.chunked_scaled_dot_product_attention(q.cuda(), cache, cache, table,
                                                          torch.zeros(1, dtype=torch.int32, device="cuda"))
    with pytest.raises(ValueError, match="bfloat16 or block-float-8"):
        torch.ops.tt.paged_scaled_dot_product_attention_decode(
            torch.zeros(1, 1, hq, d, dtype=torch.bfloat16, device="cuda"), cache, cache,
            table[:1], is_causal=True, cur_pos_tensor=torch.zeros(1, dtype=torch.int32, device="cuda"))
