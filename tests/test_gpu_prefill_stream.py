"""GPU parity for the two inner loops of the prefill kernel.  Shapes with head size 128 and a multiple
of four query heads per KV head, causal or unmasked, dense or paged bfloat16, run the hand-scheduled
loop (32-key blocks in LDS rings, written as one assembly block by csrc/gen_prefill_stream.py);
TTPA_PREFILL_STREAM=0, read on every call, sends them through the compiler-scheduled loop that serves
every other shape, and TTPA_PREFILL_WGS_PER_GROUP=n makes a workgroup of the hand-scheduled loop walk
several blocks of query rows in turn instead of one.  Every case runs under each setting.  Same
oracle, inputs and bar (atol = rtol = 2e-2) as tests/test_gpu_prefill.py, on the shapes of that file
and of tests/test_gpu_window_sink.py, plus shapes chosen for the loops' corners: an odd number of
32-key blocks, a single block, fewer blocks than the rings hold, query lengths that are not multiples
of 64, an additive mask, the ragged end of K / V inside a block, paged blocks smaller than a tile."""

import pytest
import torch

import test_gpu_prefill as P
from oracle import paged_ops as O

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["plain", "stream", "stream-2", "stream-3"])
def _loop(request, monkeypatch):
    monkeypatch.setenv("TTPA_PREFILL_STREAM", "0" if request.param == "plain" else "1")
    if "-" in request.param:
        monkeypatch.setenv("TTPA_PREFILL_WGS_PER_GROUP", request.param.split("-")[1])
    else:
        monkeypatch.delenv("TTPA_PREFILL_WGS_PER_GROUP", raising=False)


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    P.entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def _served(hq, hkv, d):
    return (hq // hkv) % 4 == 0 and d == 128


DENSE = [c for c in P.DENSE if _served(c[1], c[4], c[3])] + [
    # batch, Hq, S, D, Hkv, Skv, causal
    (1, 4, 32, 128, 1, 32, True),      # one block
    (1, 4, 96, 64, 1, 96, True),       # three blocks: the last workgroup owns 32 rows only
    (2, 8, 160, 128, 2, 160, True),    # five blocks
    (1, 8, 192, 64, 2, 192, True),     # three tiles
    (1, 8, 128, 128, 2, 77, False),    # additive mask, K / V ending inside a block
    (2, 16, 64, 128, 4, 300, False),   # more keys than rows
    (4, 32, 256, 128, 8, 256, True),
    (1, 8, 416, 128, 2, 416, True),    # thirteen row blocks: uneven shares when a workgroup takes several
    (1, 4, 64, 128, 1, 1024, False),   # long unmasked rows: the rings wrap several times
    (2, 8, 96, 128, 2, 192, False),
]


@pytest.mark.parametrize("b,hq,s,d,hkv,skv,causal", DENSE)
def test_dense_sdpa(b, hq, s, d, hkv, skv, causal):
    P.test_dense_sdpa(b, hq, s, d, hkv, skv, causal)


CHUNKED = [
    # users, Hq, Hkv, D, block, blocks per user, start, chunk length
    (2, 32, 8, 128, 64, 8, 256, 256),
    (3, 32, 8, 128, 32, 16, 128, 50),
    (2, 64, 8, 128, 64, 6, 192, 192),
    (2, 8, 2, 64, 4, 40, 32, 100),      # per-lane table lookups
    (2, 16, 4, 128, 48, 6, 96, 100),    # one lookup per load
    (2, 8, 2, 128, 20, 12, 64, 70),
    (1, 4, 1, 64, 32, 4, 96, 1),        # one query row on top of three blocks
    (2, 8, 2, 128, 16, 9, 0, 144),      # start 0: plain causal, odd number of blocks
    (1, 16, 4, 128, 64, 5, 37, 200),    # start inside a block
]


@pytest.mark.parametrize("users,hq,hkv,d,bs,nbpu,start,lc", CHUNKED)
def test_chunked_shapes(users, hq, hkv, d, bs, nbpu, start, lc):
    P.test_chunked_shapes(users, hq, hkv, d, bs, nbpu, start, lc)


@pytest.mark.parametrize("b,hq,hkv,s,d,window", [
    (1, 32, 8, 512, 128, 200), (2, 4, 1, 128, 128, 1), (1, 8, 2, 288, 64, 33), (1, 8, 2, 160, 128, 1000),
    (1, 4, 1, 384, 128, 64),
])
def test_prefill_window(b, hq, hkv, s, d, window):
    g = torch.Generator().manual_seed(s + window)
    q = torch.randn(b, hq, s, d, generator=g).to(torch.bfloat16)
    k = torch.randn(b, hkv, s, d, generator=g).to(torch.bfloat16)
    v = torch.randn(b, hkv, s, d, generator=g).to(torch.bfloat16)
    out = torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), is_causal=True,
                                                    sliding_window_size=window)
    P._check(f"prefill b{b} h{hq}x{hkv} s{s} d{d} window{window}", out.cpu(),
             O.sdpa_windowed(q, k, v, sliding_window=window))


def test_scores_that_force_a_rescale():
    """Keys whose scores grow along the sequence move the running maximum by more than the lazy
    threshold again and again: the rarely taken path that scales the output accumulators."""
    g = torch.Generator().manual_seed(5)
    b, hq, hkv, s, d = 1, 8, 2, 256, 128
    q = torch.randn(b, hq, s, d, generator=g)
    k = torch.randn(b, hkv, s, d, generator=g)
    k = k + q[:, ::4].mean(2, keepdim=True) * torch.linspace(0, 3, s).view(1, 1, s, 1)
    v = torch.randn(b, hkv, s, d, generator=g)
    q, k, v = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
    want = O.sdpa(q, k, v, None, True, None)
    got = torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), None, True, None)
    P._check("rescale", got.cpu(), want)


def test_loops_agree(monkeypatch):
    g = torch.Generator().manual_seed(9)
    q, k, v = P._bf(g, 2, 32, 320, 128), P._bf(g, 2, 8, 320, 128), P._bf(g, 2, 8, 320, 128)
    monkeypatch.setenv("TTPA_PREFILL_STREAM", "1")
    stream = torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), is_causal=True)
    monkeypatch.setenv("TTPA_PREFILL_STREAM", "0")
    plain = torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), is_causal=True)
    # the loops split a tile differently (32 keys at a time against 64), so the running maxima and the
    # bfloat16 roundings of the probabilities differ slightly
    torch.testing.assert_close(stream.float(), plain.float(), atol=1e-2, rtol=1e-2)
