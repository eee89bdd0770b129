"""Seeded random sweep of the latent-attention operators (tt::paged_flash_mla_decode, tt::flash_mla_prefill;
reference custom_ops.py:223-632) over the shapes of the kernels that share K in LDS and of the 16-head decode
kernel: every (head size, value width) pair they are built for, 1 ... 256 query heads per KV head (one head to
two segments of 128, groups that leave a wavefront or a row block partly or wholly empty), several KV heads,
block sizes from 16 to 128, scrambled page tables, contexts from one token to several tiles per workgroup range,
prefill lengths from one step to several with row blocks that end inside a token, a workgroup or a step.  Every
case is compared with the CPU oracle (atol = rtol = 2e-2); the case is printed before it runs."""

import random

import pytest
import torch

import __graft_entry__ as entry
from oracle import paged_ops as O

pytestmark = pytest.mark.gpu
ATOL = RTOL = 2e-2
SHAPES = [(576, 512), (576, 384), (192, 128), (128, 128)]
PREFILL_SHAPES = [(576, 512), (192, 128), (128, 128)]


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


@pytest.mark.parametrize("seed", range(36))
def test_latent_decode_random_case(seed):
    r = random.Random(1000 + seed)
    dh, dv = r.choice(SHAPES)
    # heads per KV head: what the 16-head form takes, what the 128-head form takes (17 ... 128, or 256)
    g = r.choice([1, 3, 8, 16, 17, 24, 31, 33, 48, 64, 65, 96, 100, 127, 128, 256])
    nkv = r.choice([1, 1, 1, 2, 3]) if g <= 64 else 1
    bs = r.choice([16, 32, 64, 128])
    users = r.randint(1, 5)
    width = r.choice([2, 5, 9, 20]) if bs >= 64 else r.choice([4, 12, 33])
    cap = width * bs
    pos = [r.choice([0, 1, bs - 1, bs, cap - 1, r.randrange(cap), r.randrange(cap)]) for _ in range(users)]
    scale = r.choice([None, None, 0.07, 0.3])
    c = dict(seed=seed, dh=dh, dv=dv, g=g, nkv=nkv, bs=bs, users=users, width=width, pos=pos, scale=scale)
    print("latent decode sweep", c, flush=True)
    gen = torch.Generator().manual_seed(seed)
    hq = g * nkv
    nb = users * width + 1
    q = _bf(gen, 1, users, hq, dh)
    key = _bf(gen, nb, nkv, bs, dh)
    table = (torch.randperm(nb - 1, generator=gen)[: users * width] + 1).view(users, width).to(torch.int32)
    cur = torch.tensor(pos, dtype=torch.int32)
    got = torch.ops.tt.paged_flash_mla_decode(q.cuda(), key.cuda(), dv, table.cuda(), None, True, None, cur.cuda(), None, scale).cpu()
    want = O.paged_flash_mla_decode(q, key, dv, table, None, cur, scale)
    _check(got, want)


@pytest.mark.parametrize("seed", range(24))
def test_latent_prefill_random_case(seed):
    r = random.Random(2000 + seed)
    dh, dv = r.choice(PREFILL_SHAPES)
    g = r.choice([1, 2, 4, 5, 8, 12, 16, 16, 24, 32, 48, 128])
    nkv = r.choice([1, 1, 2]) if g <= 32 else 1
    b = r.randint(1, 2)
    s = 32 * r.choice([1, 2, 3, 4, 5, 7, 9]) if g <= 32 else 32 * r.choice([1, 2, 3])
    masked = r.random() < 0.3
    c = dict(seed=seed, dh=dh, dv=dv, g=g, nkv=nkv, b=b, s=s, masked=masked)
    print("latent prefill sweep", c, flush=True)
    gen = torch.Generator().manual_seed(seed)
    hq = g * nkv
    q = (_bf(gen, b, hq, s, dh).float() * 0.15).to(torch.bfloat16)
    k = _bf(gen, b, nkv, s, dh)
    mask = None
    if masked:
        per_head = r.random() < 0.5
        mask = _bf(gen, b, hq if per_head else 1, s, s)
        keep = torch.rand(b, 1, s, s, generator=gen) > 0.3
        keep[..., 0] = True
        mask = mask.masked_fill(~keep, float("-inf"))
    got = torch.ops.tt.flash_mla_prefill(q.cuda(), k.cuda(), dv, None, None if mask is None else mask.cuda(), mask is None, 1.0).cpu()
    want = O.flash_mla_prefill(q.float(), k.float(), dv, None, None if mask is None else mask.float(), mask is None, 1.0)
    _check(got, want)
