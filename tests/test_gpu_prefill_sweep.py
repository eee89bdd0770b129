"""Seeded random sweep of the prefill operators (and of the one-operator prefill pass) over their shape envelope: head sizes 64 /
128 / 256, group widths that select each heads-per-wavefront variant (4, 2, 1), query lengths
from one 32-row block to several tiles, key lengths that end inside a tile, causal / additive
mask / sliding window on the dense operator; block sizes on either side of the tile size,
scrambled tables, chunk offsets and ragged chunk lengths on the paged operator.  Every case
is compared with the CPU oracle (atol = rtol = 2e-2); the case is printed before it runs."""

import random

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


def _check(got, want):
    err = (got.float() - want.float()).abs().max().item()
    print(f"  max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(got.float(), want.float(), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("seed", range(40))
def test_dense_random_case(seed):
    r = random.Random(seed)
    d = r.choice([64, 128, 128, 256])
    hkv = r.choice([1, 2, 4])
    g = r.choice([1, 2, 3, 4, 6, 8])
    b = r.randint(1, 3)
    s = 32 * r.choice([1, 1, 2, 3, 5, 8, 12])
    mode = r.choice(["causal", "causal", "mask", "window", "full"])
    skv = s if mode in ("causal", "window") else r.choice([s, 40, 64, 200, 333])
    window = r.choice([1, 20, 64, 100, 1000]) if mode == "window" else 0
    c = dict(seed=seed, b=b, hq=hkv * g, hkv=hkv, s=s, skv=skv, d=d, mode=mode, window=window)
    print("dense prefill sweep", c, flush=True)
    gen = torch.Generator().manual_seed(seed)
    q, k, v = _bf(gen, b, hkv * g, s, d), _bf(gen, b, hkv, skv, d), _bf(gen, b, hkv, skv, d)
    mask = None
    if mode == "mask":  # the pooling runner's form: 0 / -inf padding mask plus a little noise
        mask = _bf(gen, b, 1, s, skv)
        pad = torch.rand(b, 1, 1, skv, generator=gen) < 0.2
        pad[..., 0] = False
        mask = mask.masked_fill(pad, float("-inf"))
    causal = mode in ("causal", "window")
    got = torch.ops.tt.scaled_dot_product_attention(
        q.cuda(), k.cuda(), v.cuda(), None if mask is None else mask.cuda(), causal, None,
        window if window else None).cpu()
    if window:
        want = O.sdpa_windowed(q, k, v, None, window)
    else:
        want = O.sdpa(q, k, v, mask, causal, None)
    _check(got, want)


@pytest.mark.parametrize("seed", range(40))
def test_chunked_random_case(seed):
    r = random.Random(1000 + seed)
    d = r.choice([64, 128, 128, 256])
    hkv = r.choice([1, 2, 4])
    g = r.choice([1, 2, 3, 4, 8])
    users = r.randint(1, 3)
    bs = r.choice([16, 32, 64, 128])
    start = 32 * r.randint(0, 6)            # chunk offsets are multiples of the 32-token bucket
    lc = r.choice([1, 7, 32, 50, 64, 96, 130])
    nbpu = (start + lc + bs - 1) // bs + r.randint(0, 2)
    c = dict(seed=seed, users=users, hq=hkv * g, hkv=hkv, d=d, bs=bs, start=start, lc=lc, nbpu=nbpu)
    print("chunked prefill sweep", c, flush=True)
    gen = torch.Generator().manual_seed(seed)
    nb = users * nbpu + 1
    key, value = _bf(gen, nb, hkv, bs, d), _bf(gen, nb, hkv, bs, d)
    table = (torch.randperm(nb - 1, generator=gen)[: users * nbpu] + 1).view(users, nbpu).to(torch.int32)
    q = _bf(gen, users, hkv * g, lc, d)
    st = torch.tensor([start], dtype=torch.int32)
    want = O.chunked_sdpa(q, key, value, table, st)
    got = torch.ops.tt.chunked_scaled_dot_product_attention(
        q.cuda(), key.cuda(), value.cuda(), table.cuda(), st.cuda()).cpu()
    _check(got, want)


@pytest.mark.parametrize("seed", range(32))
def test_prefill_pass_random_case(seed):
    """The first-chunk prefill pass as one operator (tt::paged_fill_kv_prefill_out_) against
    fill K + fill V + dense attention, caches and output bit for bit: head sizes, group widths,
    prompt lengths from one 32-row block up, block sizes, sliding windows, permuted table rows,
    and shapes with more fill workgroups than attention workgroups (many heads, short prompts)."""
    r = random.Random(5000 + seed)
    d = r.choice([64, 128, 128, 256])
    g = r.choice([1, 1, 2, 4, 8])
    hkv = r.choice([1, 2, 8, 16] if g == 1 else [1, 2, 4])
    b = r.randint(1, 4)
    s = 32 * r.choice([1, 1, 2, 3, 5, 9, 17])
    bs = r.choice([16, 32, 64, 128])
    window = r.choice([0, 0, 0, 40, 1000])
    c = dict(seed=seed, b=b, hq=hkv * g, hkv=hkv, s=s, d=d, bs=bs, window=window)
    print("prefill pass sweep", c, flush=True)
    gen = torch.Generator().manual_seed(seed)
    q, k, v = (_bf(gen, b, h, s, d).cuda() for h in (hkv * g, hkv, hkv))
    w = (s + bs - 1) // bs + r.randint(0, 1)
    rows = b + 1
    nb = rows * w + 1
    table = (torch.randperm(nb - 1, generator=gen)[: rows * w] + 1).view(rows, w).to(torch.int32).cuda()
    bidx = torch.randperm(rows, generator=gen)[:b].to(torch.int32).cuda() if (b > 1 or r.random() < 0.5) else None
    kc = _bf(gen, nb, hkv, bs, d).cuda()
    vc = _bf(gen, nb, hkv, bs, d).cuda()
    kw = dict(is_causal=True, sliding_window_size=window if window else None)
    k_ref, v_ref = kc.clone(), vc.clone()
    torch.ops.tt.paged_fill_kv_cache_(k_ref, v_ref, k, v, table, bidx)
    want = torch.ops.tt.scaled_dot_product_attention(q, k, v, **kw)
    out = torch.zeros(b, s, hkv * g, d, dtype=torch.bfloat16, device="cuda")
    torch.ops.tt.paged_fill_kv_prefill_out_(q, k, v, kc, vc, table, bidx, out.transpose(1, 2), **kw)
    torch.cuda.synchronize()
    assert torch.equal(kc, k_ref), "K cache differs"
    assert torch.equal(vc, v_ref), "V cache differs"
    assert torch.equal(out.transpose(1, 2), want)
